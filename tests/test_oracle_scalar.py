"""Pins the scalar pieces of the CPU oracle against library routines, closed forms and brute force.

What each check would catch is stated in its docstring; none of them re-types the oracle's formula.
"""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
from torch_emulation import bits_f32, f32_bits


def all_bf16_as_f32():
    bits = (np.arange(65536, dtype=np.uint32) << 16)
    return bits.view(np.float32)


def finite(x):
    return x[np.isfinite(x)]


def test_bf16_to_fp32_exhaustive():
    """All 65536 patterns against torch's bf16 -> fp32 widening (wrong shift or mask fails)."""
    L = O.lib()
    t = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float().numpy()
    got = np.array([L.mor_oracle_bf16_to_fp32(i) for i in range(65536)], dtype=np.float32)
    nan = np.isnan(t)          # a signalling NaN is quieted on its way through a Python float
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], t.view(np.uint32)[~nan])


def test_fp32_to_bf16_round_half_up_vs_rne():
    """Round-half-up equals torch's RNE except on exact ties with an even kept mantissa
    (low 16 bits == 0x8000 and bit 16 == 0), where it is one ulp larger in magnitude."""
    L = O.lib()
    rng = np.random.default_rng(7)
    u = rng.integers(0, 2 ** 32, size=200000, dtype=np.uint64).astype(np.uint32)
    ties = (rng.integers(0, 2 ** 16, size=5000, dtype=np.uint64).astype(np.uint32) << 16) | 0x8000
    u = np.concatenate([u, ties])
    f = u.view(np.float32)
    keep = np.isfinite(f) & (((u >> 23) & 0xFF) < 0xFE)
    u, f = u[keep], f[keep]
    rne = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.mor_oracle_fp32_to_bf16(float(x)) for x in f], dtype=np.uint32).astype(np.uint16)
    got_rne = np.array([L.mor_oracle_fp32_to_bf16_rne(float(x)) for x in f], dtype=np.uint32).astype(np.uint16)
    assert np.array_equal(got_rne, rne)
    tie_even = ((u & 0xFFFF) == 0x8000) & (((u >> 16) & 1) == 0)
    assert np.array_equal(got[~tie_even], rne[~tie_even])
    assert np.array_equal(got[tie_even], rne[tie_even] + 1)
    assert tie_even.sum() > 1000


def test_fp32_to_bf16_nan_pattern():
    """FQ:52-59: the NaN 0x7fffffff carries out of the exponent field and lands on 0x8000."""
    assert O.lib().mor_oracle_fp32_to_bf16(bits_f32(0x7FFFFFFF)) == 0x8000


@pytest.mark.parametrize("fmt,dtype,lim", [(O.E4M3, torch.float8_e4m3fn, 464.0), (O.E5M2, torch.float8_e5m2, 61439.0)])
def test_cast_sw_and_hw_vs_torch_in_range(fmt, dtype, lim):
    """Software cast (FQ:125-215) and hardware-cast model against torch's CPU float8 casts for every
    bf16 value and 2M random fp32 values inside the finite range (the reference checks the same thing on
    random data, test_fake_quantize.py:570-656).  Catches wrong guard/sticky bits, subnormal shifts, bias."""
    rng = np.random.default_rng(11)
    x = np.concatenate([
        finite(all_bf16_as_f32()),
        (rng.standard_normal(500000) * lim / 3).astype(np.float32),
        rng.uniform(-lim, lim, 500000).astype(np.float32),
        (rng.standard_normal(500000) * 2.0 ** rng.integers(-20, 8, 500000)).astype(np.float32),
        rng.integers(0, 2 ** 32, size=500000, dtype=np.uint64).astype(np.uint32).view(np.float32),
    ])
    x = x[np.isfinite(x) & (np.abs(x) <= lim)]
    want = torch.from_numpy(x.copy()).to(dtype).float().numpy()
    sw = O.cast_sw(x, fmt)
    hw = O.cast_hw(x, fmt)
    assert np.array_equal(hw.view(np.uint32), want.view(np.uint32))          # sign of zero included
    nz = want != 0
    assert np.array_equal(sw[nz].view(np.uint32), want[nz].view(np.uint32))
    assert np.all(sw[~nz].view(np.uint32) == 0)                               # FQ:194: a zero result is +0


def test_cast_e4m3_known_answers():
    """test_fake_quantize.py:616-635: 463 and 464 stay finite (448), 465 is NaN in the software cast;
    the hardware cast saturates instead (cuda_fp8.hpp, __NV_SATFINITE)."""
    sw = O.cast_sw(np.array([463, 464, 465, -465, 1e9], np.float32), O.E4M3)
    assert sw[0] == 448 and sw[1] == 448 and np.isnan(sw[2:]).all()
    hw = O.cast_hw(np.array([463, 464, 465, -465, 1e9, np.inf, -np.inf], np.float32), O.E4M3)
    assert np.array_equal(hw, np.array([448, 448, 448, -448, 448, 448, -448], np.float32))
    sw5 = O.cast_sw(np.array([57344, 61439, 61440, 7e4], np.float32), O.E5M2)
    assert sw5[0] == 57344 and sw5[1] == 57344 and np.isnan(sw5[2:]).all()
    hw5 = O.cast_hw(np.array([61439, 61440, 7e4, -np.inf], np.float32), O.E5M2)
    assert np.array_equal(hw5, np.array([57344, 57344, 57344, -57344], np.float32))


def grid_of(ebits, mbits, bias, max_code_is_finite):
    """All non-negative values of a tiny float format as exact rationals."""
    vals = set()
    for e in range(2 ** ebits):
        for m in range(2 ** mbits):
            if e == 0:
                vals.add(Fraction(m, 2 ** mbits) * Fraction(2) ** (1 - bias))
            else:
                vals.add((1 + Fraction(m, 2 ** mbits)) * Fraction(2) ** (e - bias))
    return sorted(vals)


def nearest_even_on_grid(x, grid):
    """Exact nearest value with ties to the even grid index, saturating at the top."""
    x = Fraction(x)
    if x >= grid[-1]:
        return grid[-1]
    best_d, best_i = None, None
    for i, g in enumerate(grid):
        d = abs(g - x)
        if best_d is None or d < best_d or (d == best_d and i % 2 == 0):
            best_d, best_i = d, i
    return grid[best_i]


@pytest.mark.parametrize("fmt,ebits,mbits,bias,top", [(O.E2M3, 2, 3, 1, 7.5), (O.E3M2, 3, 2, 3, 28.0)])
def test_cast_sw_fp6_bruteforce(fmt, ebits, mbits, bias, top):
    """E2M3 / E3M2 (FQ:88-106,168-173): every result must be the exact nearest-even grid point, with
    saturation at 7.5 / 28; inputs include all midpoints and their neighbours."""
    grid = grid_of(ebits, mbits, bias, True)
    assert float(grid[-1]) == top and len(grid) == 2 ** (ebits + mbits)
    xs = []
    for a, b in zip(grid[:-1], grid[1:]):
        mid = float((a + b) / 2)
        xs += [float(a), mid, np.nextafter(np.float32(mid), np.float32(0)), np.nextafter(np.float32(mid), np.float32(1e9))]
    xs += [float(grid[-1]), top * 1.01, top * 2, 1e6, 1e-9]
    rng = np.random.default_rng(5)
    xs += list(rng.uniform(0, top * 1.2, 3000).astype(np.float32))
    x = np.array(xs, dtype=np.float32)
    got = O.cast_sw(np.concatenate([x, -x]), fmt)
    want = np.array([float(nearest_even_on_grid(Fraction(float(v)), grid)) for v in x], dtype=np.float32)
    n = len(x)
    assert np.array_equal(got[:n], want)
    neg = got[n:]
    assert np.array_equal(neg[want != 0], -want[want != 0])
    assert np.all(neg[want == 0].view(np.uint32) == 0)


def test_cast_sw_fp6_matches_clamped_fp8_in_normal_range():
    """test_fake_quantize.py:658-689: in their normal ranges E3M2 == clamp(e5m2 cast, +-28) on [0.25, 100]
    and E2M3 == clamp(e4m3 cast, +-7.5) on [1, 20]."""
    rng = np.random.default_rng(3)
    x = rng.uniform(0.25, 100, 200000).astype(np.float32)
    want = torch.from_numpy(x).to(torch.float8_e5m2).float().clamp(-28, 28).numpy()
    assert np.array_equal(O.quant_dequant(x, O.E3M2), want)
    x = rng.uniform(1.0, 20, 200000).astype(np.float32)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).float().clamp(-7.5, 7.5).numpy()
    assert np.array_equal(O.quant_dequant(x, O.E2M3), want)


def test_fp32_scale_bits_known_answer():
    """test_fake_quantize.py:96-103: the scale 448/240 must be 0x3FEEEEEF (a reciprocal-multiply gives ...F0)."""
    amax, scale, e8 = O.block_stats(np.full((1, 2), 0x4370, np.uint16), 1, 2, 448.0)   # 0x4370 = 240.0
    assert amax[0, 0] == 240.0
    assert scale.view(np.uint32)[0, 0] == 1072623343 == 0x3FEEEEEF
    assert e8[0, 0] == 127


def test_sqdd_fp32_vs_torch():
    """scale, cast, divide by the scale in fp32 (FQ:310-316) against torch on random (x, amax) pairs."""
    L = O.lib()
    rng = np.random.default_rng(9)
    for fmt, dtype, fmax in [(O.E4M3, torch.float8_e4m3fn, 448.0), (O.E5M2, torch.float8_e5m2, 57344.0)]:
        amax = torch.from_numpy(rng.uniform(0.01, 300, 3000).astype(np.float32)).to(torch.bfloat16).float().numpy()
        x = (rng.uniform(-1, 1, 3000).astype(np.float32) * amax)
        x = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
        s = (np.float32(fmax) / amax).astype(np.float32)
        want = (torch.from_numpy(x * s).to(dtype).float().numpy() / s).astype(np.float32)
        got = np.array([L.mor_oracle_sqdd_fp32(float(a), float(b), fmt, 1) for a, b in zip(x, s)], np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_sqdd_e8_vs_torch_and_zero_artefact():
    """Exponent-field scaling (FQ:283-305) equals x * 2**floor(log2 s) arithmetic (test_fake_quantize.py:41-46,
    732-743) whenever the cast result is non-zero; a zero cast result comes back as 2**(-e8-127) when e8 < 0."""
    L = O.lib()
    rng = np.random.default_rng(10)
    amax = torch.from_numpy(rng.uniform(0.01, 5000, 4000).astype(np.float32)).to(torch.bfloat16).float().numpy()
    x = torch.from_numpy(rng.uniform(-1, 1, 4000).astype(np.float32) * amax).to(torch.bfloat16).float().numpy()
    s = (np.float32(448.0) / amax).astype(np.float32)
    p = np.exp2(np.floor(np.log2(s.astype(np.float64)))).astype(np.float32)
    q = torch.from_numpy(x * p).to(torch.float8_e4m3fn).float().numpy()
    want = (q / p).astype(np.float32)
    got = np.array([L.mor_oracle_sqdd_e8(float(a), float(b), 0, O.E4M3, 1) for a, b in zip(x, s)], np.float32)
    nz = q != 0
    assert nz.sum() > 3000
    assert np.array_equal(got[nz].view(np.uint32), want[nz].view(np.uint32))
    e8 = ((s.view(np.uint32) >> 23) & 0xFF).astype(np.int64) - 127
    z = ~nz
    exp_bits = np.where(e8[z] < 0, (-e8[z]) << 23, 0).astype(np.uint32)
    assert np.array_equal(got[z].view(np.uint32) & 0x7FFFFFFF, exp_bits)
    # explicit: amax 1000 -> s = 0.448 -> e8 = -2; x = 1e-3 scales to 2.5e-4 < 2^-10 -> cast 0 -> 2^(2-127)
    r = L.mor_oracle_sqdd_e8(1e-3, 0.448, 0, O.E4M3, 1)
    assert f32_bits(r) == (2 << 23)


def test_e4m3_with_e8_scale_vs_torch():
    """The two fp32 test ops (FQ:865-875) against the per-element emulations of test_fake_quantize.py:712-743."""
    rng = np.random.default_rng(12)
    x = rng.uniform(-1000, 1000, 200000).astype(np.float32)
    x = x[x != 0]
    t = torch.from_numpy(x)
    a = t.abs()
    s = 448.0 / a
    small = 2 ** torch.floor(torch.log2(s))
    rz = (t * small).to(torch.float8_e4m3fn).float() / small
    assert np.array_equal(O.e4m3_with_e8_scale(x, rne=False), rz.numpy())
    large = small * 2
    pick = torch.where((a - a * small) / a <= (a * large - a) / a, small, large)
    pick = torch.where(a * large <= 464, pick, small)
    rne = (t * pick).to(torch.float8_e4m3fn).float() / pick
    got = O.e4m3_with_e8_scale(x, rne=True)
    # the emulation picks the scale by distance in fp32 arithmetic, the kernel by the guard bit of s;
    # they agree except within rounding of a tie, so allow a vanishing fraction of one-step differences
    mism = got != rne.numpy()
    assert mism.mean() < 1e-3, mism.mean()


def test_shared_mantissa_scale():
    """get_scaling_factor<SS_GLOBAL_AMAX> (FQ:1066-1076) against the struct-based model of the reference test:
    mantissa of 448/global replaces the block's, halved when it is larger; result never exceeds 448/block."""
    from torch_emulation import shared_mantissa_scale
    L = O.lib()
    rng = np.random.default_rng(13)
    for _ in range(3000):
        g = float(torch.tensor(rng.uniform(1, 1e4)).to(torch.bfloat16))
        b = float(torch.tensor(rng.uniform(1e-3, 1) * g).to(torch.bfloat16))
        gman = f32_bits(448.0 / g) & 0x7FFFFF
        want = shared_mantissa_scale(b, gman)
        got = L.mor_oracle_scaling_factor(g, b, 1)
        assert f32_bits(got) == f32_bits(want)
        assert got <= np.float32(448.0) / np.float32(b)
    assert L.mor_oracle_scaling_factor(100.0, 7.0, 2) == np.float32(448.0) / np.float32(7.0)
    assert L.mor_oracle_scaling_factor(100.0, 7.0, 4) == np.float32(448.0) / np.float32(100.0)
    assert L.mor_oracle_scaling_factor(100.0, 0.0, 3) == np.float32(448.0) / np.float32(1e-35)


@pytest.mark.parametrize("mbits", [1, 2, 3])
def test_e8m_vs_scalar_model(mbits):
    """E8M1/2/3 threshold rounding (FQ:1243-1327) for every bf16 value against the scalar model restated from
    test_e8mx.py:34-129, plus the invariant that the result keeps at most mbits mantissa bits."""
    from torch_emulation import _e8m
    L = O.lib()
    x = finite(all_bf16_as_f32())
    got = np.array([L.mor_oracle_e8m(float(v), mbits) for v in x], np.float32)
    want = np.array([_e8m(float(v), mbits) for v in x], np.float32)
    nz = want != 0
    assert np.array_equal(got[nz].view(np.uint32), want[nz].view(np.uint32))
    assert np.all((got.view(np.uint32) & ((1 << (23 - mbits)) - 1)) == 0)
    assert np.all(np.abs(got[nz] / x[nz] - 1) <= 2.0 ** -(mbits + 1) + 1e-6)
