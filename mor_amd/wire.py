"""MX wire format and dual-orientation quantization on MI355X: the quantized tensor (element codes + E8M0 scale bytes) instead of its dequantized image.

The reference's ops only return bf16 (mor/ops.py); these functions are the step next to them in a training loop: the
payload a scaled-MFMA GEMM consumes.  The quantization is the reference's MX block rule (block modes with sf_type 2,
mor/csrc/cuda/fake_quantize.cu:801-823, :251-252): blocks of 32 elements, scale 2^floor(log2(fmax / amax)), so
`dequantize_mx(*quantize_mx(x, fmt), fmt)` equals `mor.ops.fake_quantize(x, ..., 1, 32, 0.0, mode, 2)[0]` (mode 2 for
E4M3, 3 for E5M2) wherever the latter's values are not the exponent-clamp artefacts of that kernel.
"""
from typing import Tuple

import torch
from torch import Tensor

from . import _cabi

E4M3, E5M2, E3M2, E2M3 = _cabi.FMT_E4M3, _cabi.FMT_E5M2, _cabi.FMT_E3M2, _cabi.FMT_E2M3

_L = _cabi.lib()


def payload_row_bytes(cols: int, fmt: int) -> int:
    return cols if fmt in (E4M3, E5M2) else cols // 4 * 3


def _check(x: Tensor, row_multiple: int) -> Tuple[int, int]:
    if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_cuda:
        raise RuntimeError("mor: expected a 2-D bfloat16 GPU tensor")
    rows, cols = x.shape
    if cols % 32 or rows % row_multiple:
        raise RuntimeError(f"mor: MX blocks need cols % 32 == 0 and rows % {row_multiple} == 0, got {tuple(x.shape)}")
    return rows, cols


def _stream(x: Tensor) -> int:
    return torch.cuda.current_stream(x.device).cuda_stream


def quantize_mx(x: Tensor, fmt: int = E4M3) -> Tuple[Tensor, Tensor]:
    """-> (payload uint8 [rows, cols * bits / 8], scales uint8 [rows, cols / 32]); blocks of 32 along rows."""
    rows, cols = _check(x, 1)
    x = x.contiguous()
    with torch.cuda.device(x.device):
        payload = torch.empty((rows, payload_row_bytes(cols, fmt)), dtype=torch.uint8, device=x.device)
        scales = torch.empty((rows, cols // 32), dtype=torch.uint8, device=x.device)
        _cabi.check(_L.mor_mx_quantize(x.data_ptr(), payload.data_ptr(), scales.data_ptr(), rows, cols, fmt, _stream(x)))
    return payload, scales


def quantize_mx_dual(x: Tensor, fmt: int = E4M3) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """One read of x, both orientations: (payload, scales) of x as quantize_mx gives them and (payload, scales) of
    x.t() -- the operands of the dgrad and wgrad GEMMs of a linear layer."""
    rows, cols = _check(x, 32)
    x = x.contiguous()
    with torch.cuda.device(x.device):
        rp = torch.empty((rows, payload_row_bytes(cols, fmt)), dtype=torch.uint8, device=x.device)
        rs = torch.empty((rows, cols // 32), dtype=torch.uint8, device=x.device)
        cp = torch.empty((cols, payload_row_bytes(rows, fmt)), dtype=torch.uint8, device=x.device)
        cs = torch.empty((cols, rows // 32), dtype=torch.uint8, device=x.device)
        _cabi.check(_L.mor_mx_quantize_dual(x.data_ptr(), rp.data_ptr(), rs.data_ptr(), cp.data_ptr(), cs.data_ptr(),
                                            rows, cols, fmt, _stream(x)))
    return rp, rs, cp, cs


def dequantize_mx(payload: Tensor, scales: Tensor, fmt: int = E4M3) -> Tensor:
    """payload + scales -> bf16 [rows, 32 * scales.shape[1]]"""
    if payload.dtype != torch.uint8 or scales.dtype != torch.uint8 or not payload.is_cuda or scales.dim() != 2:
        raise RuntimeError("mor: expected uint8 GPU tensors")
    rows, cols = scales.shape[0], scales.shape[1] * 32
    if payload.numel() != rows * payload_row_bytes(cols, fmt):
        raise RuntimeError("mor: payload size does not match the scales")
    payload, scales = payload.contiguous(), scales.contiguous()
    with torch.cuda.device(payload.device):
        out = torch.empty((rows, cols), dtype=torch.bfloat16, device=payload.device)
        _cabi.check(_L.mor_mx_dequantize(payload.data_ptr(), scales.data_ptr(), out.data_ptr(), rows, cols, fmt, _stream(payload)))
    return out


def fake_quantize_mx_dual(x: Tensor, mode: int = 2, sf_type: int = 2) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """One read of x: (out, meta) = mor.ops.fake_quantize(x, rows, cols, 1, 32, 0.0, mode, sf_type) and
    (out_t, meta_t) = the same op on x.t().contiguous(), bit for bit, without materialising the transpose.
    mode 2 = E4M3, 3 = E5M2; sf_type 1 = fp32 scale, 2 = power-of-two scale."""
    rows, cols = _check(x, 32)
    x = x.contiguous()
    with torch.cuda.device(x.device):
        out = torch.empty_like(x)
        out_t = torch.empty((cols, rows), dtype=torch.bfloat16, device=x.device)
        meta = torch.empty((rows, cols // 32), dtype=torch.int32, device=x.device)
        meta_t = torch.empty((cols, rows // 32), dtype=torch.int32, device=x.device)
        _cabi.check(_L.mor_fake_quantize_dual(x.data_ptr(), out.data_ptr(), meta.data_ptr(), out_t.data_ptr(), meta_t.data_ptr(),
                                              rows, cols, mode, sf_type, _stream(x)))
    return out, meta, out_t, meta_t


def fake_quantize_tiles_dual(x: Tensor, clamp_threshold: float = 0.0, mode: int = 1, sf_type: int = 1) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """One read of x, 128 x 128 tiles: (out, meta) = mor.ops.fake_quantize(x, rows, cols, 128, 128, clamp_threshold,
    mode, sf_type) and (out_t, meta_t) = the same op on x.t().contiguous(), without materialising the transpose.
    mode % 10: 1 = MoR, 2 = E4M3, 3 = E5M2."""
    if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_cuda:
        raise RuntimeError("mor: expected a 2-D bfloat16 GPU tensor")
    rows, cols = x.shape
    x = x.contiguous()
    with torch.cuda.device(x.device):
        out = torch.empty_like(x)
        out_t = torch.empty((cols, rows), dtype=torch.bfloat16, device=x.device)
        meta = torch.empty((max(rows // 128, 1), max(cols // 128, 1)), dtype=torch.int32, device=x.device)
        meta_t = torch.empty((max(cols // 128, 1), max(rows // 128, 1)), dtype=torch.int32, device=x.device)
        _cabi.check(_L.mor_fake_quantize_dual_tiles(x.data_ptr(), out.data_ptr(), meta.data_ptr(), out_t.data_ptr(), meta_t.data_ptr(),
                                                    rows, cols, float(clamp_threshold), mode, sf_type, _stream(x)))
    return out, meta, out_t, meta_t


TILE_PAYLOAD_BYTES = 32768     # MOR_TILE_PAYLOAD_BYTES
TILE_STORED_BF16 = 0x100       # MOR_TILE_STORED_BF16


def quantize_mor_tiles(x: Tensor, clamp_threshold: float = 0.0, mode: int = 1) -> Tuple[Tensor, Tensor, Tensor]:
    """The MoR decision of mor.ops.fake_quantize(x, rows, cols, 128, 128, clamp_threshold, mode, 1) with each tile's
    codes as the result: (payload uint8 [tiles_y, tiles_x, 32768], tags int32 [tiles_y, tiles_x], scales float32
    [tiles_y, tiles_x]).  A tile's slot holds 128 packed rows of 128 (E4M3 / E5M2), 96 (E2M3) or 256 (BF16) bytes.
    mode % 10: 1 = MoR, 2 / 3 = every tile E4M3 / E5M2 with its own fp32 scale."""
    if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_cuda:
        raise RuntimeError("mor: expected a 2-D bfloat16 GPU tensor")
    rows, cols = x.shape
    if rows % 128 or cols % 128:
        raise RuntimeError(f"mor: tile codes need rows and cols that are multiples of 128, got {tuple(x.shape)}")
    x = x.contiguous()
    gy, gx = rows // 128, cols // 128
    with torch.cuda.device(x.device):
        payload = torch.empty((gy, gx, TILE_PAYLOAD_BYTES), dtype=torch.uint8, device=x.device)
        tags = torch.empty((gy, gx), dtype=torch.int32, device=x.device)
        scales = torch.empty((gy, gx), dtype=torch.float32, device=x.device)
        _cabi.check(_L.mor_mor_quantize(x.data_ptr(), payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), rows, cols,
                                        float(clamp_threshold), mode, _stream(x)))
    return payload, tags, scales


def dequantize_mor_tiles(payload: Tensor, tags: Tensor, scales: Tensor) -> Tensor:
    """(payload, tags, scales) of quantize_mor_tiles -> the bf16 tensor mor.ops.fake_quantize returns for the input."""
    if (payload.dtype != torch.uint8 or tags.dtype != torch.int32 or scales.dtype != torch.float32 or not payload.is_cuda
            or tags.dim() != 2 or scales.shape != tags.shape or payload.numel() != tags.numel() * TILE_PAYLOAD_BYTES):
        raise RuntimeError("mor: expected (uint8 payload, int32 tags, float32 scales) of one tile grid on the GPU")
    payload, tags, scales = payload.contiguous(), tags.contiguous(), scales.contiguous()
    rows, cols = tags.shape[0] * 128, tags.shape[1] * 128
    with torch.cuda.device(payload.device):
        out = torch.empty((rows, cols), dtype=torch.bfloat16, device=payload.device)
        _cabi.check(_L.mor_mor_dequantize(payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), out.data_ptr(), rows, cols,
                                          _stream(payload)))
    return out


def transpose_mor_tiles(payload: Tensor, tags: Tensor, scales: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """(payload, tags, scales) of a tensor -> those of its transpose (tile (i, j) becomes tile (j, i), its codes
    transposed): the operand of the GEMM that reduces over the other dimension, without quantizing x.t() again."""
    if (payload.dtype != torch.uint8 or tags.dtype != torch.int32 or scales.dtype != torch.float32 or not payload.is_cuda
            or tags.dim() != 2 or scales.shape != tags.shape or payload.numel() != tags.numel() * TILE_PAYLOAD_BYTES):
        raise RuntimeError("mor: expected (uint8 payload, int32 tags, float32 scales) of one tile grid on the GPU")
    payload, tags, scales = payload.contiguous(), tags.contiguous(), scales.contiguous()
    gy, gx = tags.shape
    with torch.cuda.device(payload.device):
        payload_t = torch.empty((gx, gy, TILE_PAYLOAD_BYTES), dtype=torch.uint8, device=payload.device)
        tags_t = torch.empty((gx, gy), dtype=torch.int32, device=payload.device)
        scales_t = torch.empty((gx, gy), dtype=torch.float32, device=payload.device)
        _cabi.check(_L.mor_mor_transpose(payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), payload_t.data_ptr(), tags_t.data_ptr(),
                                         scales_t.data_ptr(), gy, gx, _stream(payload)))
    return payload_t, tags_t, scales_t


def quantize_mor_tiles_dual(x: Tensor, clamp_threshold: float = 0.0, mode: int = 1):
    """Tile codes of x and of x.t() (the operands of the two GEMMs that reduce over either dimension of x) from one
    decision per tile: what quantize_mor_tiles(x) and transpose_mor_tiles of it return, in one call.
    -> ((payload, tags, scales), (payload_t, tags_t, scales_t))"""
    if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_cuda:
        raise RuntimeError("mor: expected a 2-D bfloat16 GPU tensor")
    rows, cols = x.shape
    if rows % 128 or cols % 128:
        raise RuntimeError(f"mor: tile codes need rows and cols that are multiples of 128, got {tuple(x.shape)}")
    x = x.contiguous()
    gy, gx = rows // 128, cols // 128
    with torch.cuda.device(x.device):
        mk = lambda a, b: (torch.empty((a, b, TILE_PAYLOAD_BYTES), dtype=torch.uint8, device=x.device),
                           torch.empty((a, b), dtype=torch.int32, device=x.device), torch.empty((a, b), dtype=torch.float32, device=x.device))
        p, t, s = mk(gy, gx)
        pt, tt, st = mk(gx, gy)
        _cabi.check(_L.mor_mor_quantize_dual(x.data_ptr(), p.data_ptr(), t.data_ptr(), s.data_ptr(), pt.data_ptr(), tt.data_ptr(), st.data_ptr(),
                                             rows, cols, float(clamp_threshold), mode, _stream(x)))
    return (p, t, s), (pt, tt, st)
