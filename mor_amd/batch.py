"""fake_quantize over a list of tensors in one call into the library.

The reference's callers quantize their tensors one op call at a time (mor/ops.py:14-63, one kernel launch each,
mor/csrc/cuda/fake_quantize.cu:1839-1871).  For the many small tensors of a model (biases, norms, small experts) the
launch is the cost; `fake_quantize_batch` hands the whole list to `mor_fake_quantize_batch`, where small tensors share
launches, and returns what the per-tensor calls would have returned, bit for bit.
"""
import ctypes as C
from typing import List, Sequence, Tuple

import torch
from torch import Tensor

from . import _cabi
from . import ops as _ops


class TensorDesc(C.Structure):
    """MorTensorDesc of include/mor_hip.h"""
    _fields_ = [("input", C.c_void_p), ("output", C.c_void_p), ("meta", C.c_void_p),
                ("rows", C.c_int64), ("cols", C.c_int64), ("block_rows", C.c_int64), ("block_cols", C.c_int64),
                ("clamp_threshold", C.c_double), ("mode", C.c_int64), ("sf_type", C.c_int64)]


_L = _cabi.lib()


class BatchPlan:
    """The descriptor array of a fixed list of tensors, built once and launched many times (a training loop quantizes
    the same parameter tensors every step).  Holds references to the tensors it points into."""

    def __init__(self, inputs: Sequence[Tensor], outputs: Sequence[Tensor], metas: Sequence[Tensor],
                 block_shapes: Sequence[Tuple[int, int]], clamp_threshold: float, mode: int, sf_type: int):
        if not (len(inputs) == len(outputs) == len(metas) == len(block_shapes)):
            raise RuntimeError("mor: inputs, outputs, metas and block_shapes must have one entry per tensor")
        self.device = inputs[0].device if inputs else None
        self.keep = (list(inputs), list(outputs), list(metas))
        self.descs = (TensorDesc * max(len(inputs), 1))()
        self.n = len(inputs)
        for d, x, y, m, (br, bc) in zip(self.descs, inputs, outputs, metas, block_shapes):
            if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_cuda or not x.is_contiguous():
                raise RuntimeError("mor: expected contiguous 2-D bfloat16 GPU tensors")
            if x.device != self.device or y.device != self.device or m.device != self.device:
                raise RuntimeError("mor: all tensors of a batch must be on one device")
            rows, cols = x.shape
            nblocks = -(-rows // br) * -(-cols // bc)
            if y.shape != x.shape or y.dtype != x.dtype or not y.is_contiguous():
                raise RuntimeError("mor: output must match its input in shape, dtype and layout")
            if m.dtype != torch.int32 or m.numel() != nblocks or not m.is_contiguous():
                raise RuntimeError(f"mor: meta must be a contiguous int32 tensor of {nblocks} entries")
            d.input, d.output, d.meta = x.data_ptr(), y.data_ptr(), m.data_ptr()
            d.rows, d.cols, d.block_rows, d.block_cols = rows, cols, br, bc
            d.clamp_threshold, d.mode, d.sf_type = clamp_threshold, mode, sf_type

    def run(self) -> None:
        if self.n == 0:
            return
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            _cabi.check(_L.mor_fake_quantize_batch(self.descs, self.n, _ops._flavour.flags, stream))


def fake_quantize_batch(tensors: Sequence[Tensor], block_shapes: Sequence[Tuple[int, int]], clamp_threshold: float,
                        mode: int, sf_type: int, inplace: bool = False) -> List[Tuple[Tensor, Tensor]]:
    """[(output, meta)] with output, meta = mor.ops.fake_quantize(x, rows, cols, block_rows, block_cols,
    clamp_threshold, mode, sf_type) for every x (mor/ops.py:14-38); with `inplace` the outputs are the inputs
    (mor/ops.py:66-91).  `block_shapes` holds one (block_rows, block_cols) per tensor."""
    ins = [x if inplace else x.contiguous() for x in tensors]
    if not ins:
        return []
    dev = ins[0].device
    with torch.cuda.device(dev):
        outs = ins if inplace else [torch.empty_like(x) for x in ins]
        counts = [-(-x.shape[0] // br) * -(-x.shape[1] // bc) for x, (br, bc) in zip(ins, block_shapes)]
        pool = torch.empty(sum(counts), dtype=torch.int32, device=dev)          # one allocation for every meta
        metas, at = [], 0
        for x, (br, bc), c in zip(ins, block_shapes, counts):
            metas.append(pool[at:at + c].view(-(-x.shape[0] // br), -(-x.shape[1] // bc)))
            at += c
    BatchPlan(ins, outs, metas, block_shapes, clamp_threshold, mode, sf_type).run()
    return list(zip(outs, metas))
