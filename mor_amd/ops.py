"""`mor.ops` for MI355X: the operator layer of the reference (mor/ops.py, mor/csrc/fake_quantize.cpp) over libmor_hip.so.

The 14 operator schemas are registered verbatim under the `mor` namespace (mor/csrc/fake_quantize.cpp:12-25), their
implementations are registered for the CUDA dispatch key (which HIP tensors use under ROCm) by libmor_torch.so
(csrc/torch_binding.cpp), and the Python wrappers and straight-through autograd registrations mirror
mor/ops.py:11-156 name for name and argument for argument.

Differences from the reference, all of them relaxations:
  * launches go to torch's current stream instead of the legacy default stream;
  * any tensor shape and block shape is accepted by fake_quantize (the reference requires an even column count and
    block shapes its thread-block geometry can launch, FQ:1767, 1781-1787);
  * an all-zero tensor does not trap in the block / channel scaling ops (FQ:1047).
There is no CPU implementation, as in the reference: CPU tensors are rejected by the dispatcher.
"""
import threading
from typing import List

import torch
from torch import Tensor

from . import _cabi

__all__ = [
    "fake_quantize", "fake_quantize_no_alloc",
    "fake_quantize_block_scaling", "fake_quantize_block_scaling_inplace",
    "fake_quantize_channel_scaling", "fake_quantize_channel_scaling_inplace",
    "fake_quantize_e8mx", "fake_quantize_e8mx_inplace",
    "quant_dequant_e4m3", "quant_dequant_e5m2", "quant_dequant_e2m3", "quant_dequant_e3m2",
    "e4m3_with_e8_scale_rne", "e4m3_with_e8_scale_rz",
]

_L = _cabi.lib()          # raises ImportError when the HIP library has not been built

# Which of the reference's two behaviours the ops return: 0 = its CUDA kernel (default), 1 = its torch emulation.
# The setting is per host thread (here and in the C++ registrations), so switching it in one thread does not change
# what the ops return in another.
class _Flavour(threading.local):
    flags = _cabi.FLAG_DEFAULT


_flavour = _Flavour()


def set_flavour(name: str) -> None:
    """'kernel' (default): bit-compatible with the reference CUDA kernel.  'torch_emulation': bit-compatible with
    the PyTorch emulation in the reference's tests (nearest-even store, true zeros).  A debugging aid; it applies to
    the calling thread's later calls only."""
    _flavour.flags = {"kernel": _cabi.FLAG_DEFAULT, "torch_emulation": _cabi.FLAG_TORCH_EMULATION,
                      "software_cast": _cabi.FLAG_SOFTWARE_CAST}[name]
    _native.mor_torch_set_flags(_flavour.flags)


# ----------------------------------------------------------------------------------------------------------------------
# schemas: mor/csrc/fake_quantize.cpp:12-25
_lib = torch.library.Library("mor", "DEF")
_lib.define("fake_quantize(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float clamp_threshold, int mode, int sf_type) -> Tensor[]")
_lib.define("fake_quantize_no_alloc(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float clamp_threshold, int mode, int sf_type, Tensor result) -> Tensor")
_lib.define("quant_dequant_e4m3(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor")
_lib.define("quant_dequant_e5m2(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor")
_lib.define("quant_dequant_e3m2(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor")
_lib.define("quant_dequant_e2m3(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor")
_lib.define("e4m3_with_e8_scale_rne(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor")
_lib.define("e4m3_with_e8_scale_rz(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor")
_lib.define("fake_quantize_block_scaling(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float e4m3_threshold, int ss_mode) -> Tensor[]")
_lib.define("fake_quantize_block_scaling_inplace(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float e4m3_threshold, int ss_mode) -> Tensor[]")
_lib.define("fake_quantize_e8mx(Tensor input, int dim_x, int dim_y, int block_x, int block_y, int quantize_type, int scaling_strategy) -> Tensor")
_lib.define("fake_quantize_e8mx_inplace(Tensor input, int dim_x, int dim_y, int block_x, int block_y, int quantize_type, int scaling_strategy, Tensor result) -> ()")
_lib.define("fake_quantize_channel_scaling(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float e4m3_threshold, int ss_mode) -> Tensor[]")
_lib.define("fake_quantize_channel_scaling_inplace(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float e4m3_threshold, int ss_mode) -> Tensor[]")


# ----------------------------------------------------------------------------------------------------------------------
# Implementations for the CUDA dispatch key (which HIP tensors use under ROCm), FQ:2663-2678: the C++ registrations of
# csrc/torch_binding.cpp (libmor_torch.so) -- the checks of FQ:1841-1844, 1887-1890, 1912-1915, 2016-2021, the
# allocations, one C ABI call -- and the straight-through autograd of the four differentiable forward ops.  There is no
# second implementation: without that library the import fails, as it does without libmor_hip.so.
def _load_native():
    import ctypes
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmor_torch.so")
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`; "
                          "the mor operators have no other implementation")
    torch.ops.load_library(path)
    lib = ctypes.CDLL(path)
    lib.mor_torch_set_flags.argtypes = [ctypes.c_uint32]
    lib.mor_torch_set_flags.restype = None
    return lib


_native = _load_native()


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


# ----------------------------------------------------------------------------------------------------------------------
# Shape / dtype propagation (fake and meta tensors), so that the ops trace under torch.compile and torch.export.  The
# reference registers none; the output shapes are those of FQ:1852-1857, 2065-2078, 2256.
def _fake_meta(i, block_x, block_y, dim_x, dim_y):
    return i.new_empty((_cdiv(dim_x, block_x), _cdiv(dim_y, block_y)), dtype=torch.int32)


def _fake_scalars(i):
    return [i.new_empty((1,), dtype=torch.int32), i.new_empty((1,), dtype=torch.float32),
            i.new_empty((1,), dtype=torch.int32), i.new_empty((1,), dtype=torch.float32)]


def _fake_like(i):
    return torch.empty_like(i, memory_format=torch.contiguous_format)


torch.library.register_fake("mor::fake_quantize")(
    lambda i, x, y, bx, by, c, m, s: [_fake_like(i), _fake_meta(i, bx, by, x, y)])
for _name in ("fake_quantize_block_scaling", "fake_quantize_channel_scaling"):
    torch.library.register_fake(f"mor::{_name}")(lambda i, x, y, bx, by, t, s: [_fake_like(i)] + _fake_scalars(i))
torch.library.register_fake("mor::fake_quantize_e8mx")(lambda i, x, y, bx, by, q, s: _fake_like(i))
# The ops that write into an argument (fake_quantize_no_alloc, the *_inplace ops) get no fake kernel: their schemas,
# kept verbatim from the reference, declare no aliasing, so a tracing compiler would take them for pure functions and
# could drop or reorder the writes.  Their Python entry points below are excluded from compilation instead
# (torch.compiler.disable: a graph break, the op runs eagerly and its results are right).
for _name in ("quant_dequant_e4m3", "quant_dequant_e5m2", "quant_dequant_e3m2", "quant_dequant_e2m3",
              "e4m3_with_e8_scale_rne", "e4m3_with_e8_scale_rz"):
    torch.library.register_fake(f"mor::{_name}")(lambda i, x, y, bx, by: _fake_like(i))


# ----------------------------------------------------------------------------------------------------------------------
# Python API and straight-through autograd: mor/ops.py:11-156
def _noop_setup_context(ctx, inputs, output):
    pass


def _ste(n_none):
    def backward(ctx, *grads):
        grad = grads[0]
        if isinstance(grad, (list, tuple)):        # ops that return Tensor[]: the gradient of the first output
            grad = grad[0]
        return (grad,) + (None,) * n_none
    return backward


def fake_quantize(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int, clamp_threshold: float, mode: int, sf_type: int) -> List[Tensor]:
    """Quantize the input bf16 Tensor to the output bf16 Tensor.  Returns [output, meta]."""
    return torch.ops.mor.fake_quantize.default(a, dim_x, dim_y, block_x, block_y, clamp_threshold, mode, sf_type)


@torch.compiler.disable
def fake_quantize_no_alloc(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int, clamp_threshold: float, mode: int, sf_type: int, output: Tensor) -> Tensor:
    """Quantize the input bf16 Tensor into the given output tensor (which may be the input).  Returns meta."""
    return torch.ops.mor.fake_quantize_no_alloc.default(a, dim_x, dim_y, block_x, block_y, clamp_threshold, mode, sf_type, output)


def fake_quantize_block_scaling(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int, e4m3_threshold: float, ss_mode: int) -> List[Tensor]:
    """E4M3 block scaling with a bf16 fallback.  Returns [output, meta, global_amax, global_non_zero, global_error]."""
    return torch.ops.mor.fake_quantize_block_scaling.default(a, dim_x, dim_y, block_x, block_y, e4m3_threshold, ss_mode)


@torch.compiler.disable
def fake_quantize_block_scaling_inplace(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int, e4m3_threshold: float, ss_mode: int) -> List[Tensor]:
    """As fake_quantize_block_scaling, overwriting a.  Returns [meta, global_amax, global_non_zero, global_error]."""
    return torch.ops.mor.fake_quantize_block_scaling_inplace.default(a, dim_x, dim_y, block_x, block_y, e4m3_threshold, ss_mode)


def fake_quantize_channel_scaling(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int, e4m3_threshold: float, ss_mode: int) -> List[Tensor]:
    """E4M3 per-row (block_x == 1) or per-column (block_y == 1) scaling with a bf16 fallback."""
    return torch.ops.mor.fake_quantize_channel_scaling.default(a, dim_x, dim_y, block_x, block_y, e4m3_threshold, ss_mode)


@torch.compiler.disable
def fake_quantize_channel_scaling_inplace(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int, e4m3_threshold: float, ss_mode: int) -> List[Tensor]:
    """As fake_quantize_channel_scaling, overwriting a."""
    return torch.ops.mor.fake_quantize_channel_scaling_inplace.default(a, dim_x, dim_y, block_x, block_y, e4m3_threshold, ss_mode)


def fake_quantize_e8mx(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int, quantize_type: int, scaling_strategy: int) -> Tensor:
    """Round the bf16 mantissa to 1, 2 or 3 bits (E8M1/2/3)."""
    return torch.ops.mor.fake_quantize_e8mx.default(a, dim_x, dim_y, block_x, block_y, quantize_type, scaling_strategy)


@torch.compiler.disable
def fake_quantize_e8mx_inplace(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int, quantize_type: int, scaling_strategy: int, output: Tensor) -> None:
    """As fake_quantize_e8mx, into the given output tensor (which may be the input)."""
    return torch.ops.mor.fake_quantize_e8mx_inplace.default(a, dim_x, dim_y, block_x, block_y, quantize_type, scaling_strategy, output)


def quant_dequant_e4m3(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int) -> Tensor:
    """fp32 -> E4M3 -> fp32 with the software cast (test op)."""
    return torch.ops.mor.quant_dequant_e4m3.default(a, dim_x, dim_y, block_x, block_y)


def quant_dequant_e5m2(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int) -> Tensor:
    """fp32 -> E5M2 -> fp32 with the software cast (test op)."""
    return torch.ops.mor.quant_dequant_e5m2.default(a, dim_x, dim_y, block_x, block_y)


def quant_dequant_e2m3(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int) -> Tensor:
    """fp32 -> E2M3 -> fp32, saturating at 7.5 (test op)."""
    return torch.ops.mor.quant_dequant_e2m3.default(a, dim_x, dim_y, block_x, block_y)


def quant_dequant_e3m2(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int) -> Tensor:
    """fp32 -> E3M2 -> fp32, saturating at 28 (test op)."""
    return torch.ops.mor.quant_dequant_e3m2.default(a, dim_x, dim_y, block_x, block_y)


def e4m3_with_e8_scale_rne(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int) -> Tensor:
    """Per-element power-of-two scale of 448 / value rounded to nearest, E4M3 cast (test op)."""
    return torch.ops.mor.e4m3_with_e8_scale_rne.default(a, dim_x, dim_y, block_x, block_y)


def e4m3_with_e8_scale_rz(a: Tensor, dim_x: int, dim_y: int, block_x: int, block_y: int) -> Tensor:
    """Per-element power-of-two scale of 448 / value rounded down, E4M3 cast (test op)."""
    return torch.ops.mor.e4m3_with_e8_scale_rz.default(a, dim_x, dim_y, block_x, block_y)


# (op, number of non-tensor arguments that get a None gradient); fake_quantize_e8mx_inplace has no autograd
# registration in the reference either (mor/ops.py:104-106).  The four differentiable forward ops have their
# straight-through autograd in C++ (libmor_torch.so).
_NATIVE_AUTOGRAD = ("fake_quantize", "fake_quantize_block_scaling", "fake_quantize_channel_scaling", "fake_quantize_e8mx")
for _name, _n in (("fake_quantize", 7), ("fake_quantize_no_alloc", 8),
                  ("fake_quantize_block_scaling", 6), ("fake_quantize_block_scaling_inplace", 6),
                  ("fake_quantize_channel_scaling", 6), ("fake_quantize_channel_scaling_inplace", 6),
                  ("fake_quantize_e8mx", 6),
                  ("quant_dequant_e4m3", 4), ("quant_dequant_e5m2", 4), ("quant_dequant_e2m3", 4), ("quant_dequant_e3m2", 4),
                  ("e4m3_with_e8_scale_rne", 4), ("e4m3_with_e8_scale_rz", 4)):
    if _name not in _NATIVE_AUTOGRAD:
        torch.library.register_autograd(f"mor::{_name}", _ste(_n), setup_context=_noop_setup_context)
