"""GPU parity of mor_block_scaling (block and channel), mor_e8mx and the fp32 test ops against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
import data_gen
import torch_emulation as E

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def uniform_bits(seed, rows, cols, lo, hi):
    g = torch.Generator().manual_seed(seed)
    return E.bf16_to_bits(torch.empty(rows, cols).uniform_(lo, hi, generator=g).to(torch.bfloat16))


def reference_chain(shape, br, bc, channel):
    """the longest chain of sequential fp32 additions in the reference's error sum for this launch geometry
    (mor/csrc/cuda/fake_quantize.cu:1095-1201, 1633-1752; the oracle adds in the same orders)"""
    rows, cols = shape
    nb = (rows // br) * (cols // bc)
    if channel and bc == 1 and br == rows and cols % 64 == 0 and rows % 16 == 0:
        per_block = rows // 16
    elif not channel and bc % 64 == 0 and br % 32 == 0:
        per_block = (br // 32) * (bc // 64)
    elif channel and br == 1 and bc >= 128 and bc % 128 == 0:
        per_block = bc // 128
    else:
        per_block = 1                         # no working launch in the reference: the oracle adds in float64
    return max(per_block, -(-nb // 1024))


IN_WINDOW = []          # cases whose mean error is within 1e-5 (relative) of the threshold


def check_scaling(G, a, br, bc, thr, ss, channel, flags=0, inplace=False):
    print("scaling", a.shape, br, bc, thr, ss, channel, flags, inplace, flush=True)
    out, meta, gamax, gnnz, gerr = G.block_scaling(a, br, bc, thr, ss, channel=channel, flags=flags, inplace=inplace)
    want, wmeta, wamax, wnnz, werr = O.block_scaling(a, br, bc, thr, ss, channel=channel, flavour=O.EMU if flags & 1 else O.KERNEL)
    assert gamax[0] == wamax[0] and gnnz[0] == wnnz[0]
    # error sums: 1e-6 relative to the terms added in float64, and equal to the reference's fp32 sum up to what the
    # reference's own order of additions can lose (chains of n sequential fp32 additions: n * 2^-24, Higham's bound)
    if not flags & 1:
        np.testing.assert_allclose(gerr[0], O.last_exact_error(), rtol=1e-6, atol=0)
    np.testing.assert_allclose(gerr[0], werr[0], rtol=max(1e-6, reference_chain(a.shape, br, bc, channel) * 2.0 ** -24), atol=0)
    # The bf16 fallback compares sum / count with the threshold (fake_quantize.cu:1214).  The kernels' sum is within
    # 1e-6 of the reference's but not added in its order, so a mean within 1e-5 of the threshold could fall on the other
    # side; such cases are counted (IN_WINDOW) and the test at the end of this file expects none.
    avg = werr[0] / max(wnnz[0], 1)
    if abs(avg - thr) <= 1e-5 * thr:
        IN_WINDOW.append((a.shape, br, bc, thr, ss, channel, flags, inplace))
    else:
        assert meta[0] == wmeta[0]
    if meta[0] == wmeta[0]:
        bad = np.argwhere(out != want)
        assert len(bad) == 0, f"{len(bad)} differ, first {bad[0]} got {out[tuple(bad[0])]:#06x} want {want[tuple(bad[0])]:#06x}"
    return meta[0]


@pytest.mark.parametrize("ss", [1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(256, 256, 128, 128, False), (256, 256, 1, 256, True), (256, 256, 256, 1, True),
                                   (64, 512, 1, 32, True), (96, 80, 32, 16, False), (60, 36, 20, 12, False),
                                   (512, 40, 128, 1, True),
                                   # single-pass kernel (ss_mode 2 / 3): whole rows, 128 lanes, odd chunks per row,
                                   # more blocks than partial slots
                                   (64, 4096, 1, 4096, True), (32, 2048, 1, 1024, True), (64, 240, 16, 120, False),
                                   (9000, 1024, 1, 1024, True),
                                   # ... rows whose chunk count is no power of two (1792, 257, 384 chunks)
                                   (24, 14336, 1, 14336, True), (40, 2056, 1, 2056, True), (64, 3072, 1, 3072, True),
                                   # ... blocks of up to 32768 / 65536 elements (512 / 1024 threads)
                                   (12, 28672, 1, 28672, True), (256, 512, 128, 256, False), (512, 512, 256, 256, False),
                                   (6, 65536, 1, 65536, True), (5, 40000, 1, 40000, True),
                                   # ... small blocks: lane groups in the amax pass
                                   (64, 96, 8, 8, False), (48, 192, 16, 16, False), (40, 192, 1, 96, True), (64, 160, 32, 32, False),
                                   # ... and larger ones (two reads)
                                   (4, 131072, 1, 131072, True), (512, 1024, 512, 256, False)])
def test_scaling_fixture_and_random(G, ss, shape):
    rows, cols, br, bc, channel = shape
    if rows == 256 and cols == 256:
        a = E.fixture_words(256, 256)
        assert check_scaling(G, a, br, bc, 0.045, ss, channel) == 1
        a = E.fixture_words(256, 256, [(0, 70, 21000, 53768)])
        check_scaling(G, a, br, bc, 0.045, ss, channel)
    a = uniform_bits(rows + ss, rows, cols, -448.0, 448.0)
    a[1, :8] = 0
    a[3, 5] = 0x8000
    check_scaling(G, a, br, bc, 0.045, ss, channel)
    check_scaling(G, a, br, bc, 0.02, ss, channel)       # low threshold: bf16 fallback copies the input
    b = data_gen.c3_weights(rows, cols, seed=rows * 3 + ss)
    check_scaling(G, b, br, bc, 0.045, ss, channel)


@pytest.mark.parametrize("shape", [(256, 256, 128, 128, False), (128, 512, 1, 512, True), (256, 64, 256, 1, True)])
@pytest.mark.parametrize("thr", [0.045, 0.001])
def test_scaling_inplace_and_flavour(G, shape, thr):
    rows, cols, br, bc, channel = shape
    a = uniform_bits(9, rows, cols, -53768.0, 53768.0)
    for ss in (1, 3):
        check_scaling(G, a, br, bc, thr, ss, channel, inplace=True)
        check_scaling(G, a, br, bc, thr, ss, channel, flags=1)


# in place with a block-local scale: a decision pass and a gated write pass of the single-pass kernel, for blocks of
# 2, 4 and 8 vectors per lane, whole and ragged, and a width that is not a power of two (general path)
@pytest.mark.parametrize("ss", [2, 3])
@pytest.mark.parametrize("shape", [(64, 4096, 1, 4096, True), (128, 256, 64, 128, False), (256, 384, 128, 128, False),
                                   (96, 2048, 1, 2048, True), (64, 3072, 1, 3072, True), (200, 256, 100, 128, False),
                                   (24, 14336, 1, 14336, True), (40, 2056, 1, 2056, True),
                                   (12, 28672, 1, 28672, True), (512, 512, 256, 256, False), (5, 40000, 1, 40000, True)])
def test_scaling_single_pass_in_place(G, ss, shape):
    rows, cols, br, bc, channel = shape
    a = uniform_bits(rows + cols + ss, rows, cols, -300.0, 300.0)
    a[1, :8] = 0
    a[3, 5] = 0x8000
    assert check_scaling(G, a, br, bc, 0.045, ss, channel, inplace=True) == 1
    assert check_scaling(G, a, br, bc, 0.02, ss, channel, inplace=True) == 3      # fallback: the input stays as it is


@pytest.mark.parametrize("ss", [1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(256, 256, 128, 128, False), (64, 4096, 1, 4096, True), (64, 512, 1, 32, True),
                                   (512, 64, 128, 1, True), (96, 80, 32, 16, False), (24, 14336, 1, 14336, True),
                                   (12, 28672, 1, 28672, True), (512, 512, 256, 256, False)])
def test_scaling_blocks_with_nan_and_inf(G, ss, shape):
    """A NaN does not become the block's amax (the reference's float maximum skips it), an infinity does; the error sum
    is NaN either way, which is not above any threshold."""
    rows, cols, br, bc, channel = shape
    a = uniform_bits(7 + ss, rows, cols, -100.0, 100.0)
    a[5, 7] = 0x7FC0
    a[rows - 3, cols - 2] = 0xFF80
    print("scaling nan/inf", shape, ss, flush=True)
    out, meta, gamax, gnnz, gerr = G.block_scaling(a, br, bc, 0.045, ss, channel=channel)
    want, wmeta, wamax, wnnz, werr = O.block_scaling(a, br, bc, 0.045, ss, channel=channel)
    assert gnnz[0] == wnnz[0] and meta[0] == wmeta[0]
    assert (np.isnan(gamax[0]) and np.isnan(wamax[0])) or gamax[0] == wamax[0]
    assert (np.isnan(gerr[0]) and np.isnan(werr[0])) or np.isclose(gerr[0], werr[0], rtol=1e-6)
    bad = np.argwhere(out != want)
    assert len(bad) == 0, f"{len(bad)} differ, first {bad[0]} got {out[tuple(bad[0])]:#06x} want {want[tuple(bad[0])]:#06x}"


def test_scaling_reference_bf16_fallback_known_answer(G):
    """test_fake_quantize_block_scaling.py:138-175: the 1.46e11 outlier gives meta 3 and output == input."""
    a = E.fixture_words(256, 256, [(0, 70, 21000, 53768)])
    out, meta, gamax, gnnz, gerr = G.block_scaling(a, 128, 128, 0.045, 1)
    assert meta[0] == 3 and np.array_equal(out, a)
    t = E.bits_to_bf16(a)
    assert gamax[0] == t.float().abs().max().item() and gnnz[0] == int(torch.count_nonzero(t))


def test_scaling_all_zero_tensor_does_not_trap(G):
    z = np.zeros((128, 128), np.uint16)
    out, meta, gamax, gnnz, gerr = G.block_scaling(z, 64, 64, 0.045, 1)
    assert meta[0] == 1 and gamax[0] == 0 and gnnz[0] == 0 and np.array_equal(out, z)


def test_scaling_rejects_bad_arguments(G):
    a = np.zeros((100, 256), np.uint16)
    with pytest.raises(RuntimeError):
        G.block_scaling(a, 128, 128, 0.045, 1)
    with pytest.raises(RuntimeError):
        G.block_scaling(np.zeros((128, 128), np.uint16), 64, 64, 0.045, 5)
    with pytest.raises(RuntimeError):
        G.block_scaling(np.zeros((128, 128), np.uint16), 64, 64, 0.045, 1, channel=True)


@pytest.mark.parametrize("qt", [1, 2, 3])
@pytest.mark.parametrize("strategy", [1, 3])
def test_e8mx(G, qt, strategy):
    a = E.fixture_words(256, 256, [(0, 70, 21000, 53768)])
    b = data_gen.c2_student_t(67, 93, seed=qt)
    every = np.arange(0x0000, 0x10000, dtype=np.uint32).astype(np.uint16).reshape(256, 256)
    every = every[(every & 0x7F80) != 0x7F80].reshape(-1, 64)      # all finite bf16 values
    for x in (a, b, every):
        print("e8mx", qt, strategy, x.shape, flush=True)
        want = O.e8mx(x, 128, 128, qt, strategy)
        assert np.array_equal(G.e8mx(x, 128, 128, qt, strategy), want)
        assert np.array_equal(G.e8mx(x, 128, 128, qt, strategy, inplace=True), want)
    if strategy == 3:
        small = E.fixture_words(64, 64, [(0, 30, 21000, 53768)])
        assert np.array_equal(G.e8mx(small, 32, 32, qt, 3), E.e8mx_tensor(small, qt))


@pytest.mark.parametrize("qt", [1, 2, 3])
def test_e8mx_closed_form_paths(G, qt):
    """The two forms of the e8mx kernel that test nothing per element.  Scale 1: every 16-bit pattern (vectors that
    hold a NaN, an infinity or a -0 take the element-wise code, their neighbours the packed one).  Tensor amax: tensors
    the amax pass finds plain, over a range of magnitudes, and the same tensors with one tiny element, one -0, one NaN,
    which must send them back to the element-wise code; an amax of 2^96 and more, an all-zero tensor."""
    every = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    rng = np.random.default_rng(qt)
    every = np.concatenate([every, rng.permutation(every)]).reshape(-1, 512)
    print("e8mx unit, every pattern", qt, flush=True)
    want = O.e8mx(every, 32, 32, qt, 3)
    got = G.e8mx(every, 32, 32, qt, 3)
    nan = (every & 0x7FFF) > 0x7F80
    assert np.array_equal(got[~nan], want[~nan]) and ((got[nan] & 0x7FFF) > 0x7F80).all()
    for scale in (1e-20, 3e-5, 1.0, 777.0, 1e20, 5e28, 2e29, 1e33):
        x = (rng.standard_normal((384, 1024)) * scale).astype(np.float32)
        x[rng.random(x.shape) < 0.05] = 0.0
        a = ((x.view(np.uint32) + 0x8000) >> 16).astype(np.uint16)
        a[a == 0x8000] = 0
        tiny = ((a & 0x7FFF) != 0) & ((a & 0x7FFF) < (33 << 7))
        a[tiny] = 0
        print("e8mx tensor amax", qt, scale, flush=True)
        assert np.array_equal(G.e8mx(a, 32, 32, qt, 1), O.e8mx(a, 32, 32, qt, 1))
        assert np.array_equal(G.e8mx(a, 32, 32, qt, 1, inplace=True), O.e8mx(a, 32, 32, qt, 1))
        for special in (0x0001, 0x1040, 0x8000, 0x9000):            # a denormal, 2^-95, -0, a negative tiny value
            b = a.copy()
            b[7, 33] = special
            assert np.array_equal(G.e8mx(b, 32, 32, qt, 1), O.e8mx(b, 32, 32, qt, 1)), hex(special)
    z = np.zeros((64, 512), np.uint16)
    assert np.array_equal(G.e8mx(z, 32, 32, qt, 1), O.e8mx(z, 32, 32, qt, 1))


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2, O.E3M2, O.E2M3])
def test_quant_dequant_ops(G, fmt):
    rng = np.random.default_rng(fmt)
    lim = O.FMAX[fmt]
    x = np.concatenate([rng.uniform(-lim * 1.2, lim * 1.2, 200000), rng.standard_normal(100000) * lim / 50,
                        rng.standard_normal(50000) * 1e-3, [463, 464, 465, 0.0, -0.0, 1e30, -1e30]]).astype(np.float32)
    print("quant_dequant", fmt, flush=True)
    got, want = G.quant_dequant(x, fmt), O.quant_dequant(x, fmt)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    if fmt in (O.E4M3, O.E5M2):
        dt = torch.float8_e4m3fn if fmt == O.E4M3 else torch.float8_e5m2
        inr = np.abs(x) <= (448 if fmt == O.E4M3 else 57344)
        ref = torch.from_numpy(x[inr]).to(dt).float().numpy()
        assert np.array_equal(got[inr], ref)


@pytest.mark.parametrize("rne", [False, True])
def test_e4m3_with_e8_scale_ops(G, rne):
    rng = np.random.default_rng(3)
    x = rng.uniform(-1000, 1000, 300000).astype(np.float32)
    x = x[x != 0]
    print("e4m3_with_e8_scale", rne, flush=True)
    got, want = G.e4m3_with_e8_scale(x, rne), O.e4m3_with_e8_scale(x, rne)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# Column blocks N x 1 with a block-local fp32 scale.  Shapes: several row segments per block, several block rows, a
# last column group that is partial, block heights that are no multiple of the rows a workgroup takes, tall thin tensors.
COLUMN_SHAPES = [(2048, 256, 2048, 1), (1024, 384, 512, 1), (600, 200, 300, 1), (16384, 512, 16384, 1), (4096, 2048, 1024, 1),
                 (130, 136, 130, 1), (8192, 1024, 128, 1), (384, 4096, 192, 1), (76800, 8, 76800, 1), (70000, 16, 70000, 1)]


@pytest.mark.parametrize("shape", COLUMN_SHAPES)
def test_column_blocks(G, shape):
    rows, cols, br, bc = shape
    a = uniform_bits(rows + cols, rows, cols, -448.0, 448.0)
    a[1, :8] = 0
    a[3, 5] = 0x8000
    a[:, cols - 1] = 0                      # an all-zero column
    a[rows // 2:, 2] &= 0x80FF              # a column whose lower half is tiny (denormals among them)
    m_hi = check_scaling(G, a, br, bc, 0.045, 3, True)
    m_lo = check_scaling(G, a, br, bc, 0.02, 3, True)
    if cols >= 128:                         # (in a narrow tensor the tiny column alone pushes the mean error up)
        assert (m_hi, m_lo) == (1, 3)
    b = data_gen.c3_weights(rows, cols, seed=rows + 5)
    check_scaling(G, b, br, bc, 0.045, 3, True)


@pytest.mark.parametrize("shape", COLUMN_SHAPES[:6])
def test_column_blocks_in_place_and_special_values(G, shape):
    rows, cols, br, bc = shape
    a = uniform_bits(rows * 7 + cols, rows, cols, -300.0, 300.0)
    a[1, :8] = 0
    assert check_scaling(G, a, br, bc, 0.045, 3, True, inplace=True) == 1
    assert check_scaling(G, a, br, bc, 0.02, 3, True, inplace=True) == 3
    a[5, 7] = 0x7FC0                        # NaN: not a column maximum, not counted
    a[rows - 3, cols - 2] = 0xFF80          # -inf: its column's maximum
    out, meta, gamax, gnnz, gerr = G.block_scaling(a, br, bc, 0.045, 3, channel=True)
    want, wmeta, wamax, wnnz, werr = O.block_scaling(a, br, bc, 0.045, 3, channel=True)
    assert gnnz[0] == wnnz[0] and meta[0] == wmeta[0]
    assert (np.isnan(gamax[0]) and np.isnan(wamax[0])) or gamax[0] == wamax[0]
    assert (np.isnan(gerr[0]) and np.isnan(werr[0])) or np.isclose(gerr[0], werr[0], rtol=1e-6)
    assert np.array_equal(out, want)


def test_column_blocks_repeated_calls_share_a_workspace(G):
    """the per-column maxima are cleared by every call: three calls in a row on one workspace, the middle one smaller"""
    from mor_amd import _cabi
    L = _cabi.lib()
    big = uniform_bits(3, 4096, 512, -100.0, 100.0)
    small = uniform_bits(4, 512, 256, -100.0, 100.0)
    nbytes = L.mor_workspace_bytes(_cabi.OP_CHANNEL_SCALING, 4096, 512, 4096, 1)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=G.dev())
    for a in (big, small, big):
        rows, cols = a.shape
        x = G.to_dev_u16(a)
        out = torch.empty_like(x)
        meta = torch.zeros(1, dtype=torch.int32, device=G.dev())
        f = torch.zeros(3, dtype=torch.float32, device=G.dev())
        n = torch.zeros(1, dtype=torch.int32, device=G.dev())
        _cabi.check(L.mor_block_scaling(x.data_ptr(), out.data_ptr(), meta.data_ptr(), f[0:].data_ptr(), n.data_ptr(), f[1:].data_ptr(),
                                        rows, cols, rows, 1, 0.045, 3, 1, ws.data_ptr(), nbytes, 0, G.stream_ptr()))
        torch.cuda.synchronize()
        want, wmeta, wamax, wnnz, werr = O.block_scaling(a, rows, 1, 0.045, 3, channel=True)
        assert np.array_equal(G.to_host_u16(out), want) and int(n[0]) == wnnz[0] and float(f[0]) == wamax[0]


@pytest.mark.parametrize("ss", [1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(256, 256, 128, 128, False), (64, 4096, 1, 4096, True), (64, 512, 1, 32, True),
                                   (512, 64, 128, 1, True), (96, 80, 32, 16, False), (2048, 256, 2048, 1, True)])
def test_scaling_denormal_elements(G, ss, shape):
    """Non-zero elements below 2^-126 among ordinary ones: they quantize to zero and add exactly 1 each to the error sum
    (|0 - x| / x), whatever the reciprocal of such an x does."""
    rows, cols, br, bc, channel = shape
    a = uniform_bits(31 + ss, rows, cols, -100.0, 100.0)
    rng = np.random.default_rng(rows + cols + ss)
    pick = rng.random((rows, cols)) < 0.1
    a[pick] = (a[pick] & 0x8000) | rng.integers(1, 0x100, int(pick.sum())).astype(np.uint16)     # 2^-133 .. 2^-125
    check_scaling(G, a, br, bc, 0.045, ss, channel)
    check_scaling(G, a, br, bc, 0.2, ss, channel, inplace=True)


@pytest.mark.parametrize("ss", [1, 2, 3, 4])
@pytest.mark.parametrize("shape", [(256, 256, 128, 128, False), (64, 4096, 1, 4096, True), (48, 2048, 1, 1024, True), (64, 512, 1, 32, True),
                                   (512, 64, 128, 1, True), (96, 80, 32, 16, False), (2048, 256, 2048, 1, True), (1024, 4096, 512, 1, True),
                                   (256, 1024, 64, 256, False)])
def test_scaling_zeros_of_both_signs(G, ss, shape):
    """Zeros leave as +0 whatever their sign (fake_quantize.cu:1133-1134) while a negative element that quantizes to zero
    keeps its sign: a third of the elements are +0 or -0, some rows, columns and vectors hold nothing else, tiny negative
    elements sit beside them, and one column group holds a NaN next to a -0."""
    rows, cols, br, bc, channel = shape
    a = uniform_bits(77 + ss, rows, cols, -200.0, 200.0)
    rng = np.random.default_rng(rows * 3 + cols + ss)
    u = rng.random((rows, cols))
    a[u < 0.17] = 0x8000
    a[(u >= 0.17) & (u < 0.33)] = 0x0000
    tiny = (u >= 0.33) & (u < 0.40)
    a[tiny] = 0x8000 | rng.integers(0x0080, 0x3000, int(tiny.sum())).astype(np.uint16)        # -1e-38 .. -5e-10
    a[5, :] = 0x8000
    a[:, 9] = np.where(rng.random(rows) < 0.5, 0x8000, 0).astype(np.uint16)
    a[7, 16:24] = 0x8000
    assert check_scaling(G, a, br, bc, 10.0, ss, channel) == 1
    check_scaling(G, a, br, bc, 10.0, ss, channel, inplace=True)
    a[11, 40] = 0x7FC0
    a[12, 41] = 0x8000
    out, meta, gamax, gnnz, gerr = G.block_scaling(a, br, bc, 10.0, ss, channel=channel)
    want, wmeta, wamax, wnnz, werr = O.block_scaling(a, br, bc, 10.0, ss, channel=channel)
    assert gnnz[0] == wnnz[0] and np.array_equal(out, want)


@pytest.mark.parametrize("shape", [(256, 256, 128, 128, False), (64, 4096, 1, 4096, True), (96, 80, 32, 16, False), (1000, 1024, 8, 1024, False),
                                   (2048, 256, 2048, 1, True), (512, 1024, 1, 32, True)])
def test_scaling_tensor_scale_without_special_values(G, shape):
    """ss_mode 4 on tensors that hold neither a NaN nor a -0 (the quantize pass then tests no vector for them), with and
    without zeros, out of place and in place; then one -0, then one NaN, which must switch the tests back on."""
    rows, cols, br, bc, channel = shape
    a = uniform_bits(rows + 13 * cols, rows, cols, -60.0, 60.0)
    a[a == 0x8000] = 0
    check_scaling(G, a, br, bc, 0.045, 4, channel)
    a[::3, ::5] = 0
    a[2, :] = 0
    check_scaling(G, a, br, bc, 0.045, 4, channel)
    check_scaling(G, a, br, bc, 0.045, 4, channel, inplace=True)
    check_scaling(G, a, br, bc, 0.001, 4, channel)
    a[rows - 1, cols - 1] = 0x8000
    check_scaling(G, a, br, bc, 0.045, 4, channel)
    a[rows // 2, 3] = 0x7FC0
    out, meta, gamax, gnnz, gerr = G.block_scaling(a, br, bc, 0.045, 4, channel=channel)
    want, wmeta, wamax, wnnz, werr = O.block_scaling(a, br, bc, 0.045, 4, channel=channel)
    assert gnnz[0] == wnnz[0] and gamax[0] == wamax[0] and np.array_equal(out, want)


@pytest.mark.parametrize("ss", [1, 2, 3])
@pytest.mark.parametrize("shape", [(256, 512, 32, 64, False), (128, 256, 16, 64, False), (256, 256, 64, 64, False), (128, 1024, 32, 128, False),
                                   (64, 2048, 2, 512, False), (64, 1024, 4, 256, False), (96, 192, 32, 64, False), (2048, 1024, 32, 32, False),
                                   (64, 8192, 1, 4096, True), (64, 6144, 1, 2048, True), (96, 3072, 1, 1024, True), (100, 4096, 1, 4096, True),
                                   (96, 512, 32, 128, False), (160, 448, 32, 64, False)])
def test_scaling_a_wave_per_block(G, ss, shape):
    """Blocks of 1024, 2048 and 4096 elements, one row or several (32 x 64 is the smallest block the reference's launch
    geometry takes): a wave holds a block (the op takes whole blocks only)."""
    rows, cols, br, bc, channel = shape
    a = uniform_bits(rows + cols + ss, rows, cols, -100.0, 100.0)
    a[3, 5] = 0x8000
    a[rows // 2, :] = 0
    a[rows - 1, cols - 9] = 0x7F00          # a large value: its block's scale is small
    check_scaling(G, a, br, bc, 0.045, ss, channel)
    check_scaling(G, a, br, bc, 0.045, ss, channel, inplace=True)
    check_scaling(G, a, br, bc, 0.0005, ss, channel)
    a[5, 64:72] = 0x0003                    # denormals in one block
    a[9, 9] = 0x7FC0                        # a NaN in another
    out, meta, gamax, gnnz, gerr = G.block_scaling(a, br, bc, 0.045, ss, channel=channel)
    want, wmeta, wamax, wnnz, werr = O.block_scaling(a, br, bc, 0.045, ss, channel=channel)
    assert gnnz[0] == wnnz[0] and np.array_equal(out, want)


def test_zz_no_case_was_within_the_threshold_window():
    """runs last in this file: how many of the cases above had a mean error within 1e-5 of the threshold"""
    print("scaling cases inside the 1e-5 threshold window:", len(IN_WINDOW), flush=True)
    assert not IN_WINDOW, IN_WINDOW
