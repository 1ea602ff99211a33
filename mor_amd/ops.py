"""`mor.ops` for MI355X: the operator layer of the reference (mor/ops.py, mor/csrc/fake_quantize.cpp) over libmor_hip.so.

The 14 operator schemas are registered verbatim under the `mor` namespace (mor/csrc/fake_quantize.cpp:12-25), their
implementations are registered for the CUDA dispatch key (which HIP tensors use under ROCm), and the Python wrappers
and straight-through autograd registrations mirror mor/ops.py:11-156 name for name and argument for argument.

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
    if _native is not None:
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
# host launchers: the checks of FQ:1841-1844, 1887-1890, 1912-1915, 2016-2021, then one C ABI call
def _check_input(t: Tensor, dtype, rows: int, cols: int, what: str = "input") -> None:
    if t.dtype != dtype:
        raise RuntimeError(f"mor: {what} must be {dtype}, got {t.dtype}")
    if t.dim() != 2 or t.size(0) != rows or t.size(1) != cols:
        raise RuntimeError(f"mor: {what} must have shape ({rows}, {cols}), got {tuple(t.shape)}")
    if not t.is_cuda:
        raise RuntimeError(f"mor: {what} must be a GPU tensor")


def _check_result(t: Tensor, rows: int, cols: int) -> None:
    _check_input(t, torch.bfloat16, rows, cols, "result")
    if not t.is_contiguous():
        raise RuntimeError("mor: result must be contiguous")


def _stream(t: Tensor) -> int:
    return torch._C._cuda_getCurrentRawStream(t.device.index)


class _on_device:
    """`with torch.cuda.device(d)` only when d is not already the current device (the usual case costs nothing)."""
    __slots__ = ("ctx",)

    def __init__(self, device):
        self.ctx = None if device.index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def _check_blocks(block_x: int, block_y: int) -> None:
    if block_x <= 0 or block_y <= 0:
        raise RuntimeError(f"mor: block dims must be positive, got ({block_x}, {block_y})")


def _fake_quantize_impl(input, dim_x, dim_y, block_x, block_y, clamp_threshold, mode, sf_type):
    _check_input(input, torch.bfloat16, dim_x, dim_y)
    _check_blocks(block_x, block_y)
    x = input.contiguous()
    with _on_device(x.device):
        out = torch.empty_like(x)
        meta = torch.empty((_cdiv(dim_x, block_x), _cdiv(dim_y, block_y)), dtype=torch.int32, device=x.device)
        _cabi.check(_L.mor_fake_quantize(x.data_ptr(), out.data_ptr(), meta.data_ptr(), dim_x, dim_y, block_x, block_y,
                                         clamp_threshold, mode, sf_type, _flavour.flags, _stream(x)))
    return [out, meta]


def _fake_quantize_no_alloc_impl(input, dim_x, dim_y, block_x, block_y, clamp_threshold, mode, sf_type, result):
    _check_input(input, torch.bfloat16, dim_x, dim_y)
    _check_result(result, dim_x, dim_y)
    _check_blocks(block_x, block_y)
    x = input.contiguous()
    with _on_device(x.device):
        meta = torch.empty((_cdiv(dim_x, block_x), _cdiv(dim_y, block_y)), dtype=torch.int32, device=x.device)
        _cabi.check(_L.mor_fake_quantize(x.data_ptr(), result.data_ptr(), meta.data_ptr(), dim_x, dim_y, block_x, block_y,
                                         clamp_threshold, mode, sf_type, _flavour.flags, _stream(x)))
    return meta


def _scaling_impl(input, dim_x, dim_y, block_x, block_y, e4m3_threshold, ss_mode, channel, inplace):
    _check_input(input, torch.bfloat16, dim_x, dim_y)
    _check_blocks(block_x, block_y)
    if dim_x % block_x or dim_y % block_y:
        raise RuntimeError(f"mor: block ({block_x}, {block_y}) does not divide the tensor ({dim_x}, {dim_y})")
    x = input.contiguous()
    with _on_device(x.device):
        dev = x.device
        out = x if inplace else torch.empty_like(x)
        meta = torch.empty(1, dtype=torch.int32, device=dev)
        gamax = torch.empty(1, dtype=torch.float32, device=dev)
        gnnz = torch.empty(1, dtype=torch.int32, device=dev)
        gerr = torch.empty(1, dtype=torch.float32, device=dev)
        op = _cabi.OP_CHANNEL_SCALING if channel else _cabi.OP_BLOCK_SCALING
        nbytes = _L.mor_workspace_bytes(op, dim_x, dim_y, block_x, block_y)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _cabi.check(_L.mor_block_scaling(x.data_ptr(), out.data_ptr(), meta.data_ptr(), gamax.data_ptr(), gnnz.data_ptr(),
                                         gerr.data_ptr(), dim_x, dim_y, block_x, block_y, e4m3_threshold, ss_mode,
                                         1 if channel else 0, ws.data_ptr(), nbytes, _flavour.flags, _stream(x)))
        if inplace and x.data_ptr() != input.data_ptr():
            input.copy_(x)            # a non-contiguous input was quantized through a contiguous copy
    return [meta, gamax, gnnz, gerr] if inplace else [out, meta, gamax, gnnz, gerr]


def _e8mx_impl(input, dim_x, dim_y, block_x, block_y, quantize_type, scaling_strategy, result=None):
    _check_input(input, torch.bfloat16, dim_x, dim_y)
    _check_blocks(block_x, block_y)
    if result is not None:
        _check_result(result, dim_x, dim_y)
    x = input.contiguous()
    with _on_device(x.device):
        out = torch.empty_like(x) if result is None else result
        nbytes = _L.mor_workspace_bytes(_cabi.OP_E8MX, dim_x, dim_y, block_x, block_y)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        _cabi.check(_L.mor_e8mx(x.data_ptr(), out.data_ptr(), dim_x, dim_y, block_x, block_y, quantize_type, scaling_strategy,
                                ws.data_ptr(), nbytes, _flavour.flags, _stream(x)))
    return out


def _quant_dequant_impl(input, dim_x, dim_y, fmt):
    _check_input(input, torch.float32, dim_x, dim_y)
    x = input.contiguous()
    with _on_device(x.device):
        out = torch.empty_like(x)
        _cabi.check(_L.mor_quant_dequant(x.data_ptr(), out.data_ptr(), x.numel(), fmt, _stream(x)))
    return out


def _e8_scale_impl(input, dim_x, dim_y, rne):
    _check_input(input, torch.float32, dim_x, dim_y)
    x = input.contiguous()
    with _on_device(x.device):
        out = torch.empty_like(x)
        _cabi.check(_L.mor_e4m3_with_e8_scale(x.data_ptr(), out.data_ptr(), x.numel(), rne, _stream(x)))
    return out


# registrations for the CUDA key: FQ:2663-2678.  The C++ registrations of csrc/torch_binding.cpp (libmor_torch.so)
# are used when that library has been built: the same checks, allocations and C ABI calls without the interpreter
# (about 6 instead of 14 microseconds per call).  The Python implementations below are the same path otherwise.
def _load_native():
    import ctypes
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmor_torch.so")
    if os.environ.get("MOR_PYTHON_OPS") == "1" or not os.path.exists(path):
        return None
    torch.ops.load_library(path)
    lib = ctypes.CDLL(path)
    lib.mor_torch_set_flags.argtypes = [ctypes.c_uint32]
    lib.mor_torch_set_flags.restype = None
    return lib


_native = _load_native()


class _PythonImpls:
    """Registers an implementation only when the C++ ones are not loaded."""

    @staticmethod
    def impl(name, fn, key):
        if _native is None:
            _lib.impl(name, fn, key)


_reg = _PythonImpls
_reg.impl("fake_quantize", _fake_quantize_impl, "CUDA")
_reg.impl("fake_quantize_no_alloc", _fake_quantize_no_alloc_impl, "CUDA")
_reg.impl("quant_dequant_e4m3", lambda i, x, y, bx, by: _quant_dequant_impl(i, x, y, _cabi.FMT_E4M3), "CUDA")
_reg.impl("quant_dequant_e5m2", lambda i, x, y, bx, by: _quant_dequant_impl(i, x, y, _cabi.FMT_E5M2), "CUDA")
_reg.impl("quant_dequant_e3m2", lambda i, x, y, bx, by: _quant_dequant_impl(i, x, y, _cabi.FMT_E3M2), "CUDA")
_reg.impl("quant_dequant_e2m3", lambda i, x, y, bx, by: _quant_dequant_impl(i, x, y, _cabi.FMT_E2M3), "CUDA")
_reg.impl("e4m3_with_e8_scale_rne", lambda i, x, y, bx, by: _e8_scale_impl(i, x, y, 1), "CUDA")
_reg.impl("e4m3_with_e8_scale_rz", lambda i, x, y, bx, by: _e8_scale_impl(i, x, y, 0), "CUDA")
_reg.impl("fake_quantize_block_scaling", lambda i, x, y, bx, by, t, s: _scaling_impl(i, x, y, bx, by, t, s, False, False), "CUDA")
_reg.impl("fake_quantize_block_scaling_inplace", lambda i, x, y, bx, by, t, s: _scaling_impl(i, x, y, bx, by, t, s, False, True), "CUDA")
_reg.impl("fake_quantize_channel_scaling", lambda i, x, y, bx, by, t, s: _scaling_impl(i, x, y, bx, by, t, s, True, False), "CUDA")
_reg.impl("fake_quantize_channel_scaling_inplace", lambda i, x, y, bx, by, t, s: _scaling_impl(i, x, y, bx, by, t, s, True, True), "CUDA")
_reg.impl("fake_quantize_e8mx", lambda i, x, y, bx, by, q, s: _e8mx_impl(i, x, y, bx, by, q, s), "CUDA")


def _e8mx_inplace_impl(input, dim_x, dim_y, block_x, block_y, quantize_type, scaling_strategy, result):
    _e8mx_impl(input, dim_x, dim_y, block_x, block_y, quantize_type, scaling_strategy, result)


_reg.impl("fake_quantize_e8mx_inplace", _e8mx_inplace_impl, "CUDA")


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
# straight-through autograd in C++ when libmor_torch.so is loaded.
_NATIVE_AUTOGRAD = ("fake_quantize", "fake_quantize_block_scaling", "fake_quantize_channel_scaling", "fake_quantize_e8mx")
for _name, _n in (("fake_quantize", 7), ("fake_quantize_no_alloc", 8),
                  ("fake_quantize_block_scaling", 6), ("fake_quantize_block_scaling_inplace", 6),
                  ("fake_quantize_channel_scaling", 6), ("fake_quantize_channel_scaling_inplace", 6),
                  ("fake_quantize_e8mx", 6),
                  ("quant_dequant_e4m3", 4), ("quant_dequant_e5m2", 4), ("quant_dequant_e2m3", 4), ("quant_dequant_e3m2", 4),
                  ("e4m3_with_e8_scale_rne", 4), ("e4m3_with_e8_scale_rz", 4)):
    if _native is None or _name not in _NATIVE_AUTOGRAD:
        torch.library.register_autograd(f"mor::{_name}", _ste(_n), setup_context=_noop_setup_context)
