"""Pins the op-level CPU oracle against the reference's own fixtures and known answers.

Fixtures are regenerated from the deterministic recipe in the reference tests; the expected results are
(a) the literal known answers those tests assert (meta grids, identities) and (b) the torch emulation in
tests/torch_emulation.py, which is what those tests compare the CUDA kernel with.
"""
import os

import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
import torch_emulation as E

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_fixtures.npz")

# pokes of test_fake_quantize.py:230-239 (dynamic-range fixture) and :317-329 (error-mode fixture)
POKES_RANGE = [(128, 1, 18200, 50968), (0, 70, 21000, 53768), (1, 1, 17262, 50030)]
POKES_ERROR = [(128, 1, 18403, 51171), (0, 70, 21000, 53768), (1, 1, 17264, 50032)]


def seeded_uniform_bf16(seed, rows, cols, lo, hi):
    g = torch.Generator().manual_seed(seed)
    t = torch.empty(rows, cols).uniform_(lo, hi, generator=g).to(torch.bfloat16)
    return E.bf16_to_bits(t)


def test_mor_dynamic_range_fixture_known_meta():
    """test_fake_quantize.py:225-283: meta [[1,3],[2,4]] and output == emulation."""
    a = E.fixture_words(256, 256, POKES_RANGE)
    out, meta = O.fake_quantize(a, 128, 128, 1e-15, 101, 1)
    assert meta.tolist() == [[1, 3], [2, 4]]
    emu, names = E.mor_tensor(a, 128, 128, True)
    assert names == {(0, 0): "e4m3", (0, 1): "bf16", (1, 0): "e5m2", (1, 1): "e2m3"}
    assert np.array_equal(out, emu)


def test_mor_error_mode_fixture_known_meta():
    """test_fake_quantize.py:312-374: meta [[1,3],[3,4]] (the E5M2-range tile goes to BF16)."""
    a = E.fixture_words(256, 256, POKES_ERROR)
    out, meta, stats = O.fake_quantize(a, 128, 128, 1e-15, 1, 1, want_stats=True)
    assert meta.tolist() == [[1, 3], [3, 4]]
    assert stats[1, 0, 2] > stats[1, 0, 3] > 0          # E4M3 error exceeds E5M2 error on that tile
    emu, _ = E.mor_tensor(a, 128, 128, False)
    assert np.array_equal(out, emu)


def test_mor_e8_fixture_known_meta():
    """test_fake_quantize.py:787-845 (sf_type=2, clamp 1e-25)."""
    a = E.fixture_words(256, 256, POKES_RANGE)
    out, meta = O.fake_quantize(a, 128, 128, 1e-25, 101, 2)
    assert meta.tolist() == [[1, 3], [2, 4]]
    emu, _ = E.mor_tensor(a, 128, 128, True, e8=True)
    assert np.array_equal(out, emu)


def test_zero_and_tiny_tensors_meta4():
    """test_fake_quantize.py:874-948: all-zero tensor and 1e-27 tensor -> meta 4; zero tensor passes through."""
    z = np.zeros((256, 256), np.uint16)
    out, meta = O.fake_quantize(z, 128, 128, 1e-25, 101, 2)
    assert (meta == 4).all() and np.array_equal(out, z)
    t = E.bf16_to_bits(torch.ones(256, 256, dtype=torch.bfloat16) * 1e-27)
    out, meta = O.fake_quantize(t, 128, 128, 1e-25, 101, 2)
    assert (meta == 4).all()
    emu, _ = E.mor_tensor(t, 128, 128, True, e8=True)
    assert np.array_equal(out, emu)


def test_mode7_identity_and_unused_modes():
    """test_fake_quantize.py:463-489: mode 7 -> meta 3 and identity; the unused mode digits behave alike (FQ:1831)."""
    a = seeded_uniform_bf16(1, 256, 256, -53768.0, 53768.0)
    for mode in (7, 0, 6, 8, 9, 17):
        out, meta = O.fake_quantize(a, 128, 128, 1e-15, mode, 1)
        assert (meta == 3).all() and np.array_equal(out, a)


@pytest.mark.parametrize("mode,fmt,fmax", [(4, "e4m3", 448.0), (5, "e5m2", 57344.0)])
def test_current_scaling_vs_emulation(mode, fmt, fmax):
    """test_fake_quantize.py:413-461: clamp_threshold carries the per-tensor scale."""
    a = seeded_uniform_bf16(2 + mode, 256, 256, -53768.0, 53768.0)
    t = E.bits_to_bf16(a).float()
    amax = t.abs().max()
    scale = float(np.float32(fmax) / np.float32(amax.item()))
    out, meta = O.fake_quantize(a, 128, 128, scale, mode, 1)
    emu = E.quant_dequant_scaled(t, fmt, amax.item())
    emu_rne = E.bf16_to_bits(emu.to(torch.bfloat16))
    assert (meta == (1 if mode == 4 else 2)).all()
    # identical except where the fp32 result is an exact bf16 tie (round-half-up vs nearest-even)
    tie = (emu.numpy().view(np.uint32) & 0xFFFF) == 0x8000
    assert np.array_equal(out[~tie], emu_rne[~tie])
    out_emu, _ = O.fake_quantize(a, 128, 128, scale, mode, 1, flavour=O.EMU)
    assert np.array_equal(out_emu, emu_rne)


@pytest.mark.parametrize("seed,dyn,e8", [(21, True, False), (22, False, False), (23, True, True), (24, False, True)])
def test_mor_random_vs_emulation(seed, dyn, e8):
    """test_fake_quantize.py:285-310, 376-411, 847-872 with a seed: uniform(-53768, 53768), 128x128 tiles."""
    a = seeded_uniform_bf16(seed, 256, 256, -53768.0, 53768.0)
    mode = 101 if dyn else 1
    out, meta = O.fake_quantize(a, 128, 128, 1e-15, mode, 2 if e8 else 1)
    emu, names = E.mor_tensor(a, 128, 128, dyn, e8=e8)
    code = {"e4m3": 1, "e5m2": 2, "bf16": 3, "e2m3": 4}
    assert meta.tolist() == [[code[names[(i, j)]] for j in range(2)] for i in range(2)]
    out_emu, meta_emu = O.fake_quantize(a, 128, 128, 1e-15, mode, 2 if e8 else 1, flavour=O.EMU)
    assert np.array_equal(meta, meta_emu)
    assert np.array_equal(out_emu, emu)
    # kernel flavour: only exact-tie roundings (fp32 scale) or zero artefacts (E8 scale) may differ
    diff = out != emu
    assert diff.mean() < 0.02


def test_kernel_vs_emulation_differences_are_exactly_the_ties():
    """128x128 E4M3 blocks with fp32 scale on N(0,1): the kernel flavour differs from the emulation exactly
    where the fp32 quotient is a bf16 tie with an even kept mantissa, and there by one ulp upwards."""
    g = torch.Generator().manual_seed(31)
    t = torch.randn(256, 256, generator=g).to(torch.bfloat16)
    a = E.bf16_to_bits(t)
    out, _ = O.fake_quantize(a, 128, 128, 0.0, 2, 1)
    emu = E.block_format_tensor(a, 128, 128, "e4m3")
    assert np.array_equal(emu, E.block_format_fast(a, 128, 128, "e4m3"))
    out_emu, _ = O.fake_quantize(a, 128, 128, 0.0, 2, 1, flavour=O.EMU)
    assert np.array_equal(out_emu, emu)
    # recompute the fp32 quotient to locate ties
    x = t.float()
    tie = np.zeros((256, 256), bool)
    for r in (0, 128):
        for c in (0, 128):
            blk = x[r:r + 128, c:c + 128]
            q = E.quant_dequant_scaled(blk, "e4m3", blk.abs().max().item()).numpy().view(np.uint32)
            tie[r:r + 128, c:c + 128] = ((q & 0xFFFF) == 0x8000) & (((q >> 16) & 1) == 0)
    diff = out != emu
    assert np.array_equal(diff, tie)
    assert np.array_equal(out[diff].astype(np.int64), emu[diff].astype(np.int64) + 1)


@pytest.mark.parametrize("fmt,mode", [("e4m3", 2), ("e5m2", 3)])
@pytest.mark.parametrize("e8", [False, True])
def test_block_modes_vs_emulation(fmt, mode, e8):
    """modes 2/3 (no reference test): by analogy with the MoR emulation, 1x32 and 64x64 blocks, Student-t data."""
    g = torch.Generator().manual_seed(41)
    z = torch.randn(4, 64, 256, generator=g)
    t = (z[0] / torch.sqrt((z[1] ** 2 + z[2] ** 2 + z[3] ** 2) / 3) * 0.02)
    t = torch.where(torch.rand(64, 256, generator=g) < 1e-2, t * 1000, t).to(torch.bfloat16)
    a = E.bf16_to_bits(t)
    for (br, bc) in ((1, 32), (64, 64)):
        out_emu, meta = O.fake_quantize(a, br, bc, 0.0, mode, 2 if e8 else 1, flavour=O.EMU)
        emu = E.block_format_fast(a, br, bc, fmt, e8=e8)
        assert (meta == (1 if mode == 2 else 2)).all()
        assert np.array_equal(out_emu, emu)
        out, _ = O.fake_quantize(a, br, bc, 0.0, mode, 2 if e8 else 1)
        if e8:
            # E8: outputs are exact in bf16, so only the zero artefact (blocks with amax > fmax) can differ
            d = out != emu
            assert np.all((emu[d] & 0x7FFF) == 0)
        else:
            assert (out != emu).mean() < 0.02


def test_block_scaling_fixture_e4m3():
    """test_fake_quantize_block_scaling.py:100-135: meta 1, amax/nnz equal torch's, error within 1e-6 of a float64 sum (the reference asserts 1e-3), output equal."""
    a = E.fixture_words(256, 256)
    out, meta, gamax, gnnz, gerr = O.block_scaling(a, 128, 128, 0.045, 1)
    emu, total, amax, nnz = E.block_scaling_tensor(a, 128, 128)
    assert meta[0] == 1 and gamax[0] == amax and gnnz[0] == nnz
    assert abs(gerr[0] - total) <= 1e-6 * total
    assert np.array_equal(out, emu)


def test_block_scaling_fixture_bf16_fallback():
    """test_fake_quantize_block_scaling.py:138-175: the 1.46e11 outlier pushes the average error over 0.045."""
    a = E.fixture_words(256, 256, [(0, 70, 21000, 53768)])
    out, meta, gamax, gnnz, gerr = O.block_scaling(a, 128, 128, 0.045, 1)
    _, total, amax, nnz = E.block_scaling_tensor(a, 128, 128)
    assert meta[0] == 3 and gamax[0] == amax and gnnz[0] == nnz
    assert abs(gerr[0] - total) <= 1e-6 * total
    assert np.array_equal(out, a)


@pytest.mark.parametrize("lo,hi,seed", [(-448.0, 448.0, 51), (-53768.0, 53768.0, 52)])
@pytest.mark.parametrize("shape", [(128, 128, False), (1, 256, True), (256, 1, True)])
def test_block_and_channel_scaling_random(lo, hi, seed, shape):
    """test_fake_quantize_block_scaling.py:177-267 and the channel file's row/col variants, seeded."""
    br, bc, channel = shape
    a = seeded_uniform_bf16(seed, 256, 256, lo, hi)
    out, meta, gamax, gnnz, gerr = O.block_scaling(a, br, bc, 0.045, 1, channel=channel, flavour=O.EMU)
    emu, total, amax, nnz = E.block_scaling_tensor(a, br, bc)
    assert gamax[0] == amax and gnnz[0] == nnz
    assert abs(gerr[0] - total) <= 1e-6 * total
    want_meta = 3 if gerr[0] / gnnz[0] > 0.045 else 1
    assert meta[0] == want_meta
    assert np.array_equal(out, emu if want_meta == 1 else a)
    outk, metak, _, _, gerrk = O.block_scaling(a, br, bc, 0.045, 1, channel=channel)
    assert metak[0] == meta[0] and gerrk[0] == gerr[0]
    assert (outk != out).mean() < 0.02


def test_block_scaling_rejects_indivisible():
    """FQ:2019-2020."""
    with pytest.raises(RuntimeError):
        O.block_scaling(np.zeros((100, 256), np.uint16), 128, 128, 0.045, 1)


@pytest.mark.parametrize("mbits", [1, 2, 3])
def test_e8mx_fixture(mbits):
    """test_e8mx.py:194-403: scaling_strategy 3 (no global scale) on the poked fixture, 64x64 corner to keep
    the scalar emulation fast."""
    a = E.fixture_words(64, 64, [(0, 30, 21000, 53768)])
    out = O.e8mx(a, 32, 32, mbits, 3)
    assert np.array_equal(out, E.e8mx_tensor(a, mbits))


def test_e8mx_global_amax_properties():
    """scaling_strategy 1 (FQ:1335-1359; the reference only checks in-place == out-of-place): the scale lies in
    [1, 2) and maps the tensor amax onto the largest value below the next power of two; results stay within
    half a step of the input."""
    L = O.lib()
    for mbits in (1, 2, 3):
        for amax in (1.0, 1.5, 1.99, 3.0, 1e-3, 7e4):
            s = L.mor_oracle_e8mx_scaling_factor(amax, mbits, 1)
            assert 1.0 <= s < 2.0
            top = amax * s
            m, e = np.frexp(np.float32(top))
            assert abs(m * 2 - (2 - 2.0 ** -mbits)) < 1e-6
    a = seeded_uniform_bf16(61, 64, 64, -100.0, 100.0)
    out = O.e8mx(a, 32, 32, 3, 1)
    x = E.bits_to_bf16(a).float().numpy()
    y = E.bits_to_bf16(out).float().numpy()
    nz = x != 0
    assert np.all(np.abs(y[nz] / x[nz] - 1) <= 2.0 ** -4 + 2.0 ** -7)


def test_ragged_and_tiny_shapes():
    """Edge shapes the reference launch code cannot run (odd columns, partial blocks, 1x32): block results must equal
    the same blocks quantized on their own."""
    a = seeded_uniform_bf16(71, 37, 45, -10.0, 10.0)
    out, meta = O.fake_quantize(a, 16, 32, 0.0, 2, 1)
    assert meta.shape == (3, 2)
    for (r0, r1) in ((0, 16), (16, 32), (32, 37)):
        for (c0, c1) in ((0, 32), (32, 45)):
            sub = np.ascontiguousarray(a[r0:r1, c0:c1])
            o2, _ = O.fake_quantize(sub, 16, 32, 0.0, 2, 1)
            assert np.array_equal(out[r0:r1, c0:c1], o2)
    one = seeded_uniform_bf16(72, 1, 32, -1.0, 1.0)
    o, m = O.fake_quantize(one, 1, 32, 0.0, 2, 2)
    assert m.shape == (1, 1) and np.array_equal(o, E.block_format_fast(one, 1, 32, "e4m3", e8=True))


def test_golden_file_matches_emulation_and_oracle():
    """The committed fixture file (inputs + torch-emulation outputs + the reference's literal meta answers)."""
    g = np.load(GOLDEN)
    for key, mode, sf, clamp in (("range", 101, 1, 1e-15), ("error", 1, 1, 1e-15), ("range_e8", 101, 2, 1e-25)):
        a = g[f"{key}_in"]
        out, meta = O.fake_quantize(a, 128, 128, clamp, mode, sf)
        assert np.array_equal(meta, g[f"{key}_meta"])
        assert np.array_equal(out, g[f"{key}_out"])
