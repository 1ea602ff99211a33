"""Pins the oracle's MX wire format (codes + E8M0 scale bytes) without retyping it: decoding the payload with the
golden decode tables and multiplying by 2^(scale - 127) must give the fake-quantized tensor of the reference's torch
emulation (oracle flavour EMU, itself pinned by torch.float8 casts), and the scale bytes must be 254 minus the exponent
field of fl32(fmax / amax) (FQ:251-252)."""
import os

import numpy as np
import pytest

from oracle import mor_oracle as O
import data_gen

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "scalar_vectors.npz"))
NAMES = {O.E4M3: "e4m3", O.E5M2: "e5m2", O.E3M2: "e3m2", O.E2M3: "e2m3"}


def unpack_codes(payload, cols, fmt):
    """payload bytes -> one code per element (python-side unpacking of the 6-bit formats)"""
    if fmt in (O.E4M3, O.E5M2):
        return payload.astype(np.uint32)
    p = payload.reshape(payload.shape[0], -1, 3).astype(np.uint32)
    w = p[..., 0] | (p[..., 1] << 8) | (p[..., 2] << 16)
    codes = np.stack([(w >> (6 * k)) & 0x3F for k in range(4)], axis=-1)
    return codes.reshape(payload.shape[0], cols)


def decode_with_tables(payload, scales, cols, fmt):
    codes = unpack_codes(payload, cols, fmt)
    vals = V[f"decode_{NAMES[fmt]}"].view(np.float32)[codes].astype(np.float64)
    mult = np.exp2(scales.astype(np.float64) - 127.0).repeat(32, axis=1)
    return (vals * mult).astype(np.float32)


def fake_quant_emulation(a, fmt):
    if fmt == O.E4M3:
        return O.fake_quantize(a, 1, 32, 0.0, 2, 2, flavour=O.EMU)[0]
    if fmt == O.E5M2:
        return O.fake_quantize(a, 1, 32, 0.0, 3, 2, flavour=O.EMU)[0]
    return O.block_format(a, 1, 32, fmt, 2, flavour=O.EMU)


def inputs():
    yield "student_t", data_gen.c2_student_t(96, 512, seed=11)
    yield "normal", data_gen.c1_normal(64, 256, seed=12)
    w = data_gen.c3_weights(64, 256, seed=13)
    w[5] = 0
    w[6, :32] = 0x8000
    yield "weights_with_zero_rows", w
    rng = np.random.default_rng(14)
    wide = (rng.integers(0x0080, 0x7F00, (48, 128)) | (rng.integers(0, 2, (48, 128)) << 15)).astype(np.uint16)
    wide[:, ::7] = (wide[:, ::7] & 0x807F) | (0x3F << 7)        # keep each block's range inside |e8| <= 100
    yield "wide_exponents", np.where(((wide >> 7) & 0xFF) > 0xB0, wide & 0xBFFF, wide).astype(np.uint16)


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2, O.E3M2, O.E2M3])
def test_payload_decodes_to_the_fake_quantized_tensor(fmt):
    for name, a in inputs():
        payload, scales = O.mx_quantize(a, fmt)
        rows, cols = a.shape
        got = decode_with_tables(payload, scales, cols, fmt)
        want = (fake_quant_emulation(a, fmt).astype(np.uint32) << 16).view(np.float32)
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert len(bad) == 0, (name, bad[0], got[tuple(bad[0])], want[tuple(bad[0])])
        # the oracle's own decoder agrees with the table decoder
        assert np.array_equal(O.mx_dequantize(payload, scales, fmt), (got.view(np.uint32) >> 16).astype(np.uint16))


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2, O.E3M2, O.E2M3])
def test_scale_bytes_are_the_e8m0_of_the_decode_multiplier(fmt):
    for name, a in inputs():
        _, scales = O.mx_quantize(a, fmt)
        amax, s, e8m0 = O.block_stats(a, 1, 32, O.FMAX[fmt])
        want = np.where(amax > 0, 254 - e8m0, 127)
        assert np.array_equal(scales.astype(np.int64), want), name


def test_known_block():
    """amax 240 in E4M3: fl32(448/240) = 1.8666 -> e8 = 0 -> byte 127; 240 -> code of 240 = 0x77 (1.875 * 2^7)."""
    a = np.zeros((1, 32), np.uint16)
    a[0, 0] = 0x4370          # 240.0
    a[0, 1] = 0xC370          # -240.0
    a[0, 2] = 0x3F80          # 1.0 -> code 0x38
    a[0, 3] = 0x3A80          # 2^-10 -> below half of the smallest subnormal 2^-9 -> 0 (ties to even)
    payload, scales = O.mx_quantize(a, O.E4M3)
    assert scales[0, 0] == 127
    assert list(payload[0, :5]) == [0x77, 0xF7, 0x38, 0x00, 0x00]
    # the same block scaled by 2^-20 has the same codes and scale byte 127 - 20
    b = a.copy()
    b[0, :4] -= (20 << 7)
    p2, s2 = O.mx_quantize(b, O.E4M3)
    assert s2[0, 0] == 107 and np.array_equal(p2, payload)
    # FP6 packing: codes 1, 2, 3, 4 -> bits 000001 | 000010 << 6 | 000011 << 12 | 000100 << 18
    c = np.zeros((1, 32), np.uint16)
    c[0, 31] = 0x40F0         # 7.5 keeps e8 = 0
    c[0, :4] = [0x3E00, 0x3E80, 0x3EC0, 0x3F00]     # 0.125, 0.25, 0.375, 0.5
    p6, s6 = O.mx_quantize(c, O.E2M3)
    assert s6[0, 0] == 127 and p6.shape == (1, 24)
    w = int(p6[0, 0]) | (int(p6[0, 1]) << 8) | (int(p6[0, 2]) << 16)
    assert w == (1 | (2 << 6) | (3 << 12) | (4 << 18))
    assert (int(p6[0, 23]) >> 2) == 0x1F            # last code 7.5 = 0b011111 in the top six bits
