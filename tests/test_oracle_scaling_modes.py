"""Pins the scaling strategies of the block / channel scaling op that no reference test exercises.

The reference's tests call fake_quantize_block_scaling / _channel_scaling with ss_mode 1 only
(test/test_fake_quantize_block_scaling.py, test/test_fake_quantize_channel_scaling.py).  ss_mode 2, 3 and 4
(FQ:1079-1093, the E8 / FP32 selection at FQ:1138, 1149) are pinned here in two independent ways:

 * against a torch emulation built only from primitives that are pinned elsewhere (torch's float8_e4m3fn CPU cast,
   IEEE fp32 arithmetic, exact exponent arithmetic) -- output bits, error sum against a float64 sum at 1e-6, and the
   bf16-fallback decision;
 * by cross-identities inside the oracle: with a block-local scale the op must return what fake_quantize returns for
   the same blocks (mode 2 with sf_type 2 for ss_mode 2, the reference's SS_BLOCK_AMAX == SF_E8 coincidence; mode 2
   with sf_type 1 for ss_mode 3; mode 4 with clamp_threshold = 448 / amax for ss_mode 4), except that zero inputs come
   back as +0 (FQ:1130-1134).  fake_quantize is pinned by the reference's own fixtures.

Swapping ss_mode 2 and 3, dropping the +0 rule, taking the tensor amax for the block amax or a wrong error
denominator each fail at least one assertion.
"""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
import torch_emulation as E

GEOMETRIES = [(128, 128, False), (1, 256, True), (256, 1, True), (64, 64, False), (1, 32, True)]


def scaling_data(seed, rows=256, cols=256, wide=False):
    """bf16 data with zeros of both signs, a few large and tiny blocks."""
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(rows, cols, generator=g)
    if wide:
        t = t * torch.exp(2.0 * torch.randn(rows, cols, generator=g))
        t[:64, :64] *= 1e4           # blocks whose amax exceeds 448: negative power-of-two exponents
        t[64:128, 64:192] *= 1e-6
    z = torch.rand(rows, cols, generator=g)
    t = torch.where(z < 0.02, torch.zeros(()), t)
    t = torch.where((z >= 0.02) & (z < 0.03), -torch.zeros(()), t)
    t[5, :] = 0.0                    # an all-zero row block
    t[:, 9] = 0.0                    # an all-zero column block
    return E.bf16_to_bits(t.to(torch.bfloat16))


def emulate(a_u16, brows, bcols, ss_mode):
    """-> (bits of the E4M3 result with a nearest-even bf16 store, float64 error sum, fp32 dequantized values).

    The scale is the IEEE fp32 quotient 448 / amax (torch.div on fp32 tensors is correctly rounded), per block for
    ss_mode 2 / 3 and per tensor for ss_mode 4; ss_mode 2 keeps only its power of two."""
    t = E.bits_to_bf16(a_u16).float()
    rows, cols = t.shape
    v = t.view(rows // brows, brows, cols // bcols, bcols)
    if ss_mode == 4:
        amax = t.abs().max().reshape(1, 1, 1, 1)
    else:
        amax = v.abs().amax(dim=(1, 3), keepdim=True)
    amax = torch.clamp(amax, min=1e-35)                       # FQ:1063-1064
    scale = torch.div(torch.full_like(amax, 448.0), amax)
    if ss_mode == 2:
        scale = torch.exp2(torch.floor(torch.log2(scale.double()))).float()
    dq = torch.div((v * scale).to(torch.float8_e4m3fn).float(), scale)
    dq = torch.where(v == 0, v, dq)                           # zero inputs pass (the torch flavour keeps the sign of -0)
    dq = dq.reshape(rows, cols)
    nz = t != 0
    err = torch.sum(torch.abs((dq[nz].double() - t[nz].double()) / t[nz].double())).item()
    return E.bf16_to_bits(dq.to(torch.bfloat16)), err, dq


@pytest.mark.parametrize("geom", GEOMETRIES)
@pytest.mark.parametrize("ss_mode", [2, 3, 4])
@pytest.mark.parametrize("wide", [False, True])
def test_scaling_modes_vs_independent_emulation(geom, ss_mode, wide):
    br, bc, channel = geom
    a = scaling_data(100 + ss_mode, wide=wide)
    want, err64, dq = emulate(a, br, bc, ss_mode)
    nnz = int(np.count_nonzero(a & 0x7FFF))
    amax = float(E.bits_to_bf16(a).float().abs().max())
    avg = err64 / nnz
    for thr, want_meta in ((avg * 0.9, 3), (avg * 1.1, 1)):
        out, meta, gamax, gnnz, gerr = O.block_scaling(a, br, bc, thr, ss_mode, channel=channel, flavour=O.EMU)
        assert gamax[0] == amax and gnnz[0] == nnz
        assert abs(gerr[0] - err64) <= 1e-6 * err64, (gerr[0], err64)
        assert meta[0] == want_meta
        assert np.array_equal(out, want if want_meta == 1 else a)
    # what the CUDA kernel returns: the same values with the round-half-up store, so only exact ties may differ
    # (ss_mode 2 results are exact in bf16; there only the 2^(-e8-127) artefact of a zero cast result may differ)
    # and zero inputs come back as +0 (FQ:1130-1134)
    outk, metak, _, _, gerrk = O.block_scaling(a, br, bc, avg * 1.1, ss_mode, channel=channel)
    assert metak[0] == 1 and abs(gerrk[0] - err64) <= 1e-6 * err64
    zero_in = (a & 0x7FFF) == 0
    assert np.all(outk[zero_in] == 0)
    want = np.where(zero_in, 0, want).astype(np.uint16)
    d = outk != want
    if ss_mode == 2:
        assert np.all((want[d] & 0x7FFF) == 0) and np.all(a[d] & 0x7FFF)
    else:
        # exactly the fp32 results that are bf16 ties with an even kept mantissa, one ulp up
        q = dq.numpy().view(np.uint32)
        tie = ((q & 0xFFFF) == 0x8000) & (((q >> 16) & 1) == 0) & ~zero_in
        assert np.array_equal(d, tie) and np.array_equal(outk[d].astype(np.int64), want[d].astype(np.int64) + 1)


@pytest.mark.parametrize("geom", GEOMETRIES)
@pytest.mark.parametrize("wide", [False, True])
def test_block_local_strategies_equal_fake_quantize(geom, wide):
    """ss_mode 2 == mode 2 / sf_type 2 (power of two), ss_mode 3 == mode 2 / sf_type 1 (fp32 scale), bit for bit on
    non-zero inputs; zero inputs are +0."""
    br, bc, channel = geom
    a = scaling_data(200, wide=wide)
    zero_in = (a & 0x7FFF) == 0
    outs = {}
    for ss_mode, sf_type in ((2, 2), (3, 1)):
        out, meta, _, _, _ = O.block_scaling(a, br, bc, 1e30, ss_mode, channel=channel)
        fq, _ = O.fake_quantize(a, br, bc, 0.0, 2, sf_type)
        assert meta[0] == 1
        assert np.array_equal(out[~zero_in], fq[~zero_in])
        assert np.all(out[zero_in] == 0)
        outs[ss_mode] = out
    assert (outs[2] != outs[3]).mean() > 0.05          # the two strategies are not interchangeable


@pytest.mark.parametrize("geom", GEOMETRIES)
def test_tensor_amax_strategy_equals_current_scaling(geom):
    """ss_mode 4 == fake_quantize mode 4 with clamp_threshold = 448 / tensor amax (FQ:825-833, 1086-1089)."""
    br, bc, channel = geom
    a = scaling_data(300, wide=True)
    amax = np.float32(E.bits_to_bf16(a).float().abs().max().item())
    scale = np.float32(448.0) / amax
    out, meta, gamax, _, _ = O.block_scaling(a, br, bc, 1e30, 4, channel=channel)
    fq, _ = O.fake_quantize(a, br, bc, float(scale), 4, 1)
    zero_in = (a & 0x7FFF) == 0
    assert meta[0] == 1 and gamax[0] == amax
    assert np.array_equal(out[~zero_in], fq[~zero_in])
    assert np.all(out[zero_in] == 0)


def test_scale_strategies_differ_where_they_should():
    """One block of 1 x 32 with amax 3: 448 / 3 = 149.33; its power of two is 128.  The element 2.9 quantizes to
    different E4M3 grid points under the two scales, so a swap of ss_mode 2 and 3 shows."""
    x = torch.zeros(1, 32)
    x[0, 0], x[0, 1] = 3.0, 2.90625
    a = E.bf16_to_bits(x.to(torch.bfloat16))
    o3, *_ = O.block_scaling(a, 1, 32, 1e30, 3, channel=True)
    o2, *_ = O.block_scaling(a, 1, 32, 1e30, 2, channel=True)
    v3 = E.bits_to_bf16(o3).float()[0, 1].item()
    v2 = E.bits_to_bf16(o2).float()[0, 1].item()
    # fp32 scale: 2.90625 * 149.33 = 434 -> grid step 32 -> 448 -> 448 / 149.33 = 3.0
    assert v3 == 3.0
    # power of two: 2.90625 * 128 = 372 -> grid step 32 -> 384 -> 384 / 128 = 3.0; 372 is nearer 384 than 352
    assert v2 == 3.0
    x[0, 1] = 2.59375                      # * 149.33 = 387.3 -> 384 -> 2.5714 -> bf16 2.5781 (half up) ; * 128 = 332 -> 320 -> 2.5
    a = E.bf16_to_bits(x.to(torch.bfloat16))
    o3, *_ = O.block_scaling(a, 1, 32, 1e30, 3, channel=True)
    o2, *_ = O.block_scaling(a, 1, 32, 1e30, 2, channel=True)
    assert E.bits_to_bf16(o2).float()[0, 1].item() == 2.5
    assert abs(E.bits_to_bf16(o3).float()[0, 1].item() - 384.0 / (448.0 / 3.0)) < 0.01


# ---------------------------------------------------------------- e4m3_with_e8_scale, nearest-even exponent

def _rne_emulation(x):
    """test/test_fake_quantize.py:712-730 restated with torch primitives."""
    t = torch.from_numpy(x)
    a = t.abs()
    s = 448.0 / a
    small = 2 ** torch.floor(torch.log2(s))
    large = small * 2
    pick = torch.where((a - a * small) / a <= (a * large - a) / a, small, large)
    pick = torch.where(a * large <= 464, pick, small)
    return ((t * pick).to(torch.float8_e4m3fn).float() / pick).numpy()


def test_e4m3_with_e8_scale_rne_exact():
    """The nearest-even variant (FQ:259-281) equals the reference's emulation bit for bit, on random data and on the
    points where its rule acts: it raises the exponent only when |x| 2^e8 lies in (224, 232], and then 2 |x| 2^e8 in
    (448, 464] rounds to 448, whose half is the 224 that |x| 2^e8 rounds to anyway -- so the results also equal the
    round-toward-zero variant's.  A rule that raised the exponent more often (a wrong bound on the mantissa or the
    exponent sum, a missing guard-bit test) would produce NaN or a finer grid on these points."""
    rng = np.random.default_rng(12)
    x = rng.uniform(-1000, 1000, 400000).astype(np.float32)
    x = x[x != 0]
    pts = []
    for e in range(-12, 12):
        for base in (224.0, 228.0, 232.0, 240.0, 256.0, 298.6666, 448.0, 456.0, 464.0, 472.0, 480.0, 232.0, 192.0,
                     1.8125 * 128, 200.0, 208.0, 216.0):
            u = int(np.float32(base * 2.0 ** e).view(np.uint32))
            pts += [u + d for d in range(-3, 4)]
    p = np.array(pts, np.uint32).view(np.float32)
    p = p[np.abs(p) <= 1000]
    x = np.concatenate([x, p, -p])
    got = O.e4m3_with_e8_scale(x, rne=True)
    assert np.array_equal(got.view(np.uint32), _rne_emulation(x).view(np.uint32))
    assert np.array_equal(got.view(np.uint32), O.e4m3_with_e8_scale(x, rne=False).view(np.uint32))
    assert not np.isnan(got).any()


# ---------------------------------------------------------------- e8mx with the tensor-amax scale

E8M_THRESHOLDS = {1: [32, 95], 2: [16, 47, 80, 111], 3: [8, 23, 40, 55, 72, 87, 104, 119]}     # FQ:1243-1327, units of 2^16


def _e8m_numpy(v, mbits):
    """Threshold rounding of fp32 values on the full 23-bit mantissa: k = number of thresholds below the mantissa."""
    b = v.view(np.uint32).astype(np.int64)
    sign, e, m = b & 0x80000000, (b >> 23) & 0xFF, b & 0x7FFFFF
    th = np.array(E8M_THRESHOLDS[mbits], np.int64) << 16
    k = np.searchsorted(th, m, side="left")            # thresholds strictly below m
    carry = k == (1 << mbits)
    e2 = np.where(carry, e + 1, e)
    m2 = np.where(carry, 0, k << (23 - mbits))
    sat = e2 == 255
    e2 = np.where(sat, 254, e2)
    m2 = np.where(sat, ((1 << mbits) - 1) << (23 - mbits), m2)
    m2 = np.where(e == 0, 0, m2)
    e2 = np.where(e == 0, 0, e2)
    keep = e == 255
    out = np.where(keep, b, sign | (e2 << 23) | m2)
    return out.astype(np.uint32).view(np.float32)


def _e8mx_scale_closed_form(amax, mbits):
    """FQ:1335-1359 as exact arithmetic: fp_max = (2 - 2^-mbits) 2^(E+1) with E = floor(log2 amax); the quotient
    fp_max / amax, halved when it reaches 2, lies in [1, 2)."""
    from fractions import Fraction
    fa = Fraction(float(amax))
    E_ = int(np.floor(np.log2(float(amax))))
    q = (2 - Fraction(1, 1 << mbits)) * Fraction(2) ** (E_ + 1) / fa
    s = np.float32(float(q))                 # a double rounds the rational once more, far below fp32's half ulp here
    return s / np.float32(2.0) if s >= 2 else s


@pytest.mark.parametrize("mbits", [1, 2, 3])
def test_e8mx_tensor_amax_strategy(mbits):
    """scaling_strategy 1 against exact arithmetic for the scale, numpy threshold tables on the scaled fp32 values,
    IEEE division and the round-half-up store; and the special cases that reduce to the unscaled op."""
    L = O.lib()
    rng = np.random.default_rng(70 + mbits)
    for amax in list(rng.uniform(1e-3, 1e4, 200)) + [1.0, 1.5, 1.75, 1.875, 1.9921875, 3.0, 7e4]:
        amax = float(torch.tensor(amax).to(torch.bfloat16))
        assert np.float32(L.mor_oracle_e8mx_scaling_factor(amax, mbits, 1)) == _e8mx_scale_closed_form(amax, mbits)
    g = torch.Generator().manual_seed(80 + mbits)
    t = (torch.randn(64, 96, generator=g) * torch.exp(2 * torch.randn(64, 96, generator=g))).to(torch.bfloat16)
    t[3, :7] = 0.0
    a = E.bf16_to_bits(t)
    x = t.float().numpy()
    sf = _e8mx_scale_closed_form(float(np.abs(x).max()), mbits)
    v = (x * sf).astype(np.float32)
    dq = np.where(v != 0, _e8m_numpy(v, mbits), np.float32(0)).astype(np.float32) / sf
    want = ((dq.astype(np.float32).view(np.uint32).astype(np.uint64) + 0x8000) >> 16).astype(np.uint16)   # round half up
    assert np.array_equal(O.e8mx(a, 32, 32, mbits, 1), want)
    # amax = (2 - 2^-mbits) 2^k: the scale is exactly 1 and the op equals the unscaled one
    t2 = t.clone().float()
    t2 = t2 / t2.abs().max() * (2 - 2.0 ** -mbits) * 4
    t2 = t2.to(torch.bfloat16)
    t2[0, 0] = (2 - 2.0 ** -mbits) * 4
    a2 = E.bf16_to_bits(t2)
    assert float(t2.float().abs().max()) == (2 - 2.0 ** -mbits) * 4
    assert np.array_equal(O.e8mx(a2, 32, 32, mbits, 1), O.e8mx(a2, 32, 32, mbits, 3))
