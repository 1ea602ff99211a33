"""Torch-side emulation of fake quantization, used to pin the CPU oracle.

The reference's unit tests state the intended semantics of every op as a few
lines of PyTorch around the library casts ``Tensor.to(torch.float8_e4m3fn)`` /
``torch.float8_e5m2`` (test/test_fake_quantize.py:33-143,
test/test_fake_quantize_block_scaling.py:51-98, test/test_e8mx.py:34-129).
This module restates those semantics from their description; it shares no code
with the oracle, so agreement between the two is evidence and not a tautology.
bf16 data is exchanged as numpy uint16 bit patterns.
"""
import math
import struct

import numpy as np
import torch

FP8 = {"e4m3": (torch.float8_e4m3fn, 448.0), "e5m2": (torch.float8_e5m2, 57344.0),
       # the reference tests emulate E2M3 with an E4M3 cast scaled to 7.5 (test_fake_quantize.py:38-40)
       "e2m3": (torch.float8_e4m3fn, 7.5)}


def bits_to_bf16(a_u16):
    return torch.from_numpy(np.ascontiguousarray(a_u16).view(np.int16)).view(torch.bfloat16)


def bf16_to_bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def fixture_words(rows, cols, pokes=()):
    """Deterministic matrix of the reference tests (test_fake_quantize.py:16-24): packed
    word (r, j) = (16256 << 16 | 49024) + r * 2**16 + j, i.e. bf16 pair (low = -1.0.., high = +1.0..),
    then single words overwritten by ``pokes`` = [(row, word_col, high_bits, low_bits)].
    Returns uint16 bits of shape [rows, cols]."""
    assert cols % 2 == 0
    r = np.arange(rows, dtype=np.uint64)[:, None]
    j = np.arange(cols // 2, dtype=np.uint64)[None, :]
    words = ((16256 << 16) + 49024 + (r << 16) + j).astype(np.uint32)
    for (pr, pj, hi, lo) in pokes:
        words[pr, pj] = (hi << 16) + lo
    return words.view(np.uint16).reshape(rows, cols).copy()


def f32_bits(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def bits_f32(u):
    return struct.unpack("<f", struct.pack("<I", u & 0xFFFFFFFF))[0]


def quant_dequant_scaled(block_f32, fmt, amax, e8=False):
    """scale -> cast to fp8 -> back -> descale, all on a float32 tensor; amax is a Python float."""
    dtype, fmax = FP8[fmt]
    scale = fmax / amax
    if e8:
        scale = 2.0 ** math.floor(math.log2(scale))
    return (block_f32 * scale).to(dtype).float() / scale


def abs_rel_error_sum(orig_f32, deq_f32):
    return torch.sum(torch.abs((deq_f32 - orig_f32) / orig_f32))


def mor_block(block_bf16, dynamic_range_mode, e8=False, e4m3_range=28672):
    """Per-block MoR decision + fake quantization; returns (bf16 block, chosen format name).

    e4m3_range defaults to the kernel's constant (FQ:627); the reference test file spells it 28762."""
    x = block_bf16.float()
    ax = x.abs()
    amax = ax.max().item()
    nz = ax[ax > 0]
    if nz.numel() == 0:
        return block_bf16, "zero"
    rng = amax / nz.min().item()
    if rng <= 7.5:
        return quant_dequant_scaled(x, "e2m3", amax, e8).to(torch.bfloat16), "e2m3"
    if dynamic_range_mode:
        if rng <= e4m3_range:
            return quant_dequant_scaled(x, "e4m3", amax, e8).to(torch.bfloat16), "e4m3"
        if rng <= 939524096:
            return quant_dequant_scaled(x, "e5m2", amax, e8).to(torch.bfloat16), "e5m2"
        return block_bf16, "bf16"
    if rng <= e4m3_range * 4:
        return quant_dequant_scaled(x, "e4m3", amax, e8).to(torch.bfloat16), "e4m3"
    if rng <= 939524096:
        q4 = quant_dequant_scaled(x, "e4m3", amax, e8)
        q5 = quant_dequant_scaled(x, "e5m2", amax, e8)
        m = x != 0
        e4 = abs_rel_error_sum(x[m], q4[m])
        e5 = abs_rel_error_sum(x[m], q5[m])
        if e4 <= e5:
            return q4.to(torch.bfloat16), "e4m3"
        return block_bf16, "bf16"
    return block_bf16, "bf16"


def mor_tensor(a_u16, brows, bcols, dynamic_range_mode, e8=False):
    t = bits_to_bf16(a_u16)
    out = t.clone()
    rows, cols = t.shape
    names = {}
    for r in range(0, rows, brows):
        for c in range(0, cols, bcols):
            blk, name = mor_block(t[r:r + brows, c:c + bcols], dynamic_range_mode, e8)
            out[r:r + brows, c:c + bcols] = blk
            names[(r // brows, c // bcols)] = name
    return bf16_to_bits(out), names


def block_format_tensor(a_u16, brows, bcols, fmt, e8=False):
    """Every block quantized to one format with scale fmax/amax (zero blocks pass through)."""
    t = bits_to_bf16(a_u16)
    out = t.clone()
    rows, cols = t.shape
    for r in range(0, rows, brows):
        for c in range(0, cols, bcols):
            x = t[r:r + brows, c:c + bcols].float()
            amax = x.abs().max().item()
            if amax > 0:
                out[r:r + brows, c:c + bcols] = quant_dequant_scaled(x, fmt, amax, e8).to(torch.bfloat16)
    return bf16_to_bits(out)


def block_format_fast(a_u16, brows, bcols, fmt, e8=False):
    """Vectorised version of block_format_tensor for block shapes that tile the tensor exactly.
    The scale is a correctly rounded fp32 quotient (torch.div of two fp32 tensors), which equals the
    double quotient rounded to fp32 for these operands."""
    dtype, fmax = FP8[fmt]
    t = bits_to_bf16(a_u16).float()
    rows, cols = t.shape
    assert rows % brows == 0 and cols % bcols == 0
    v = t.view(rows // brows, brows, cols // bcols, bcols)
    amax = v.abs().amax(dim=(1, 3), keepdim=True)
    safe = torch.where(amax > 0, amax, torch.ones_like(amax))
    scale = torch.div(torch.full_like(safe, fmax), safe)
    if e8:
        scale = torch.exp2(torch.floor(torch.log2(scale)))
    q = torch.div((v * scale).to(dtype).float(), scale)
    q = torch.where(amax > 0, q, v)
    return bf16_to_bits(q.reshape(rows, cols).to(torch.bfloat16))


def shared_mantissa_scale(block_amax, global_mantissa):
    """Block scale whose 23 mantissa bits are replaced by the tensor-wide ones, halved when that
    would exceed the block's own scale (test_fake_quantize_block_scaling.py:75-98)."""
    block_sf = 448.0 / block_amax
    b = f32_bits(block_sf)
    cand = bits_f32((b & 0xFF800000) | global_mantissa)
    return cand if global_mantissa <= (b & 0x7FFFFF) else cand / 2.0


def block_scaling_tensor(a_u16, brows, bcols):
    """ss_mode 1 emulation -> (quantized bits, total relative error, amax, nnz)."""
    t = bits_to_bf16(a_u16)
    out = t.clone()
    rows, cols = t.shape
    gamax = t.float().abs().max().item()
    gman = f32_bits(448.0 / gamax) & 0x7FFFFF
    total = 0.0
    for r in range(0, rows, brows):
        for c in range(0, cols, bcols):
            x = t[r:r + brows, c:c + bcols].float()
            sf = shared_mantissa_scale(x.abs().max().item(), gman)
            d = (x * sf).to(torch.float8_e4m3fn).float() / sf
            m = x != 0
            total += float(abs_rel_error_sum(x[m].double(), d[m].double()))
            out[r:r + brows, c:c + bcols] = d.to(torch.bfloat16)
    return bf16_to_bits(out), total, gamax, int(torch.count_nonzero(t))


def _e8m(value, mbits):
    """Keep mbits mantissa bits of a float whose bf16 mantissa is m (test_e8mx.py:34-129)."""
    thresholds = {1: [32, 95], 2: [16, 47, 80, 111], 3: [8, 23, 40, 55, 72, 87, 104, 119]}[mbits]
    u = f32_bits(abs(value))
    exponent, mant = (u >> 23) & 0xFF, (u >> 16) & 0x7F
    if exponent == 0:
        mant = 0
    elif exponent < 255:
        for k, th in enumerate(thresholds):
            if mant <= th:
                mant = k << (7 - mbits)
                break
        else:
            mant = 0
            exponent += 1
            if exponent == 255:
                exponent, mant = 254, ((1 << mbits) - 1) << (7 - mbits)
    r = bits_f32((exponent << 23) | (mant << 16))
    return -r if value < 0 else r


def e8mx_tensor(a_u16, mbits):
    t = bits_to_bf16(a_u16).float()
    flat = [_e8m(v, mbits) for v in t.flatten().tolist()]
    return bf16_to_bits(torch.tensor(flat, dtype=torch.float32).reshape(t.shape).to(torch.bfloat16))
