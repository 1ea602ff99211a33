"""Seeded random sweep over shapes, block shapes, modes and data kinds: every case goes through the C ABI and must
equal the CPU oracle bit for bit (error sums to 1e-6).  The case list is fixed by the seed, so a failure names its case."""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O

IN_WINDOW = []          # scaling cases whose mean error is within 1e-5 (relative) of the threshold

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def make_data(rng, rows, cols, kind):
    if kind == 0:      # normal
        x = rng.standard_normal((rows, cols)).astype(np.float32)
    elif kind == 1:    # heavy tails with outliers
        x = (rng.standard_t(3, (rows, cols)) * 0.02).astype(np.float32)
        x[rng.random((rows, cols)) < 1e-2] *= 1000
    elif kind == 2:    # log-normal magnitudes, random sign, sparse zeros
        x = (np.exp(3 * rng.standard_normal((rows, cols))) * rng.choice([-1.0, 1.0], (rows, cols))).astype(np.float32)
        x[rng.random((rows, cols)) < 0.05] = 0
    else:              # tiny values with a zero stripe
        x = (rng.standard_normal((rows, cols)) * 1e-4).astype(np.float32)
        x[rows // 3] = 0
    t = torch.from_numpy(x).to(torch.bfloat16)
    return t.view(torch.int16).numpy().view(np.uint16).copy()


def fq_cases_lane_groups_and_large_blocks():
    """Small blocks (a group of lanes per block) and blocks beyond what 256 threads hold in registers."""
    rng = np.random.default_rng(20253)
    blocks = [(1, 48), (1, 96), (1, 192), (1, 384), (1, 768), (1, 1536), (2, 40), (8, 16), (32, 8), (128, 8), (16, 128), (32, 64),
              (24, 24), (128, 256), (256, 256), (1, 28672), (1, 40000), (1, 131072), (129, 2048), (512, 64), (64, 1024), (300, 512)]
    cases = []
    for i in range(60):
        br, bc = blocks[rng.integers(len(blocks))]
        exact = rng.random() < 0.5
        ny, nx = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        rows = br * ny if exact else br * ny - int(rng.integers(0, br))
        cols = bc * nx if exact else bc * nx - 8 * int(rng.integers(0, max(bc // 8, 1)))     # whole vectors: the vector kernels
        rows, cols = max(rows, 1), max(cols, 8)
        mode = int(rng.choice([1, 101, 2, 3]))
        sf = int(rng.choice([1, 2]))
        cases.append((100 + i, rows, cols, br, bc, mode, sf, int(rng.integers(4))))
    return cases


def fq_cases():
    rng = np.random.default_rng(20251)
    blocks = [(1, 8), (1, 16), (1, 32), (1, 64), (1, 128), (1, 256), (1, 512), (1, 1024), (1, 2048), (2, 64), (4, 32),
              (8, 8), (16, 16), (16, 56), (32, 32), (64, 64), (128, 128), (128, 64), (64, 256), (3, 40), (5, 7), (1, 24)]
    cases = []
    for i in range(90):
        br, bc = blocks[rng.integers(len(blocks))]
        exact = rng.random() < 0.6
        ny, nx = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        rows = br * ny if exact else br * ny - int(rng.integers(0, br))
        cols = bc * nx if exact else bc * nx - int(rng.integers(0, min(bc, 9)))
        rows, cols = max(rows, 1), max(cols, 1)
        mode = int(rng.choice([1, 101, 2, 3, 4, 5, 7]))
        sf = int(rng.choice([1, 2]))
        cases.append((i, rows, cols, br, bc, mode, sf, int(rng.integers(4))))
    return cases


@pytest.mark.parametrize("case", fq_cases() + fq_cases_lane_groups_and_large_blocks(), ids=lambda c: "fq%d_%dx%d_b%dx%d_m%d_s%d_k%d" % c)
def test_fake_quantize_sweep(G, case):
    i, rows, cols, br, bc, mode, sf, kind = case
    rng = np.random.default_rng(1000 + i)
    a = make_data(rng, rows, cols, kind)
    clamp = 1e-15 if mode not in (4, 5) else float(np.float32((448.0 if mode == 4 else 57344.0) / max(np.abs((a.astype(np.uint32) << 16).view(np.float32)).max(), 1e-30)))
    print("sweep", case, flush=True)
    out, meta = G.fake_quantize(a, br, bc, clamp, mode, sf)
    want, wmeta, stats = O.fake_quantize(a, br, bc, clamp, mode, sf, want_stats=True)
    # no change in format choice in any block of any case
    flip = meta != wmeta
    assert not flip.any(), (case, int(flip.sum()), stats[..., 2][flip], stats[..., 3][flip])
    bad = np.argwhere(out != want)
    assert len(bad) == 0, (case, len(bad), tuple(bad[0]), hex(int(out[tuple(bad[0])])), hex(int(want[tuple(bad[0])])))


def scaling_cases():
    rng = np.random.default_rng(20252)
    blocks = [(1, 32), (1, 64), (1, 256), (1, 1024), (1, 2048), (128, 128), (64, 64), (32, 16), (16, 120), (20, 12),
              (64, 1), (256, 1), (8, 1)]
    cases = []
    for i in range(60):
        br, bc = blocks[rng.integers(len(blocks))]
        ny, nx = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        if bc == 1:
            nx = int(rng.choice([40, 64, 200, 520]))
        cases.append((i, br * ny, bc * nx, br, bc, int(rng.choice([1, 2, 3, 4])), int(rng.integers(3)), bool(rng.integers(2)),
                      float(rng.choice([0.02, 0.045, 0.2]))))
    return cases


def scaling_cases_small_and_large_blocks():
    rng = np.random.default_rng(20254)
    blocks = [(1, 96), (1, 768), (8, 8), (16, 16), (32, 32), (1, 14336), (1, 28672), (1, 40000), (128, 256), (256, 256), (512, 256)]
    cases = []
    for i in range(40):
        br, bc = blocks[rng.integers(len(blocks))]
        ny, nx = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        cases.append((100 + i, br * ny, bc * nx, br, bc, int(rng.choice([1, 2, 3, 4])), int(rng.integers(3)), bool(rng.integers(2)),
                      float(rng.choice([0.02, 0.045, 0.2]))))
    return cases


@pytest.mark.parametrize("case", scaling_cases() + scaling_cases_small_and_large_blocks(), ids=lambda c: "bs%d_%dx%d_b%dx%d_ss%d_k%d_%s_%g" % c)
def test_scaling_sweep(G, case):
    i, rows, cols, br, bc, ss, kind, inplace, thr = case
    rng = np.random.default_rng(2000 + i)
    a = make_data(rng, rows, cols, kind)
    channel = (br == 1 or bc == 1)
    print("sweep", case, flush=True)
    out, meta, gamax, gnnz, gerr = G.block_scaling(a, br, bc, thr, ss, channel=channel, inplace=inplace)
    want, wmeta, wamax, wnnz, werr = O.block_scaling(a, br, bc, thr, ss, channel=channel)
    assert gamax[0] == wamax[0] and gnnz[0] == wnnz[0], case
    np.testing.assert_allclose(gerr[0], werr[0], rtol=1e-6, atol=0)
    avg = werr[0] / max(wnnz[0], 1)
    if abs(avg - thr) <= 1e-5 * thr:          # the kernels' sum is not added in the reference's order: counted, none expected
        IN_WINDOW.append(case)
    else:
        assert meta[0] == wmeta[0], case
    if meta[0] == wmeta[0]:
        bad = np.argwhere(out != want)
        assert len(bad) == 0, (case, len(bad), tuple(bad[0]), hex(int(out[tuple(bad[0])])), hex(int(want[tuple(bad[0])])))


def test_scaling_sweep_no_case_within_the_threshold_window():
    """runs after the sweep above: the cases whose decision the order of the additions could have changed"""
    print("scaling sweep cases inside the 1e-5 threshold window:", len(IN_WINDOW), flush=True)
    assert not IN_WINDOW, IN_WINDOW


def wire_cases():
    rng = np.random.default_rng(20253)
    return [(i, 32 * int(rng.integers(1, 9)), 32 * int(rng.integers(1, 12)), int(rng.integers(4)), int(rng.integers(4))) for i in range(32)]


@pytest.mark.parametrize("case", wire_cases(), ids=lambda c: "mx%d_%dx%d_f%d_k%d" % c)
def test_wire_sweep(G, case):
    i, rows, cols, fmt, kind = case
    rng = np.random.default_rng(3000 + i)
    a = make_data(rng, rows, cols, kind)
    print("sweep", case, flush=True)
    wp, ws = O.mx_quantize(a, fmt)
    tp, ts = O.mx_quantize(np.ascontiguousarray(a.T), fmt)
    rp, rs, cp, cs = G.mx_quantize_dual(a, fmt)
    gp, gs = G.mx_quantize(a, fmt)
    assert np.array_equal(gp, wp) and np.array_equal(gs, ws), case
    assert np.array_equal(rp, wp) and np.array_equal(rs, ws) and np.array_equal(cp, tp) and np.array_equal(cs, ts), case
    assert np.array_equal(G.mx_dequantize(wp, ws, fmt), O.mx_dequantize(wp, ws, fmt)), case
    if fmt in (O.E4M3, O.E5M2):
        for sf in (1, 2):
            mode = 2 if fmt == O.E4M3 else 3
            o, m, ot, mt = G.fake_quantize_dual(a, mode, sf)
            w, _ = O.fake_quantize(a, 1, 32, 0.0, mode, sf)
            wt, _ = O.fake_quantize(np.ascontiguousarray(a.T), 1, 32, 0.0, mode, sf)
            assert np.array_equal(o, w) and np.array_equal(ot, wt), (case, sf)


def tile_cases():
    rng = np.random.default_rng(20257)
    return [(i, 128 * int(rng.integers(1, 7)), 128 * int(rng.integers(1, 9)), int(rng.choice([1, 101, 2, 3])), int(rng.integers(4)))
            for i in range(24)]


@pytest.mark.parametrize("case", tile_cases(), ids=lambda c: "tiles%d_%dx%d_m%d_k%d" % c)
def test_tile_entries_sweep(G, case):
    """128 x 128 tiles through the three entries that work on them besides mor_fake_quantize: the tile codes and their
    decode, both orientations from one read, and a batch call; all against the oracle."""
    import mor_amd
    i, rows, cols, mode, kind = case
    rng = np.random.default_rng(5000 + i)
    a = make_data(rng, rows, cols, kind)
    if kind == 2:
        a[:128, :128] = (a[:128, :128] & 0x8000) | 0x0080 | (a[:128, :128] & 0x007F)        # a tile of values near 2^-126: scale outside the fast range
    print("sweep", case, flush=True)
    clamp = 1e-3
    want, wmeta = O.fake_quantize(a, 128, 128, clamp, mode, 1)
    x = G.to_dev_u16(a)
    payload, tags, scales = mor_amd.wire.quantize_mor_tiles(x, clamp, mode)
    back = mor_amd.wire.dequantize_mor_tiles(payload, tags, scales)
    assert np.array_equal((tags & 0xFF).cpu().numpy(), wmeta), case
    assert np.array_equal(G.to_host_u16(back), want), case
    out, meta, out_t, meta_t = mor_amd.wire.fake_quantize_tiles_dual(x, clamp, mode, 1)
    want_t, wmeta_t = O.fake_quantize(np.ascontiguousarray(a.T), 128, 128, clamp, mode, 1)
    assert np.array_equal(meta.cpu().numpy(), wmeta) and np.array_equal(G.to_host_u16(out), want), case
    assert np.array_equal(meta_t.cpu().numpy(), wmeta_t) and np.array_equal(G.to_host_u16(out_t), want_t), case
    # the same tensor three times in a batch (large enough for the tile path when rows * cols > 2^18), next to a small one
    small = make_data(rng, 64, 96, kind)
    got = G.fake_quantize_batch([a, small, a, a], [(128, 128), (16, 32), (128, 128), (128, 128)], clamp, mode, 1)
    for k in (0, 2, 3):
        assert np.array_equal(got[k][1], wmeta) and np.array_equal(got[k][0], want), (case, k)
    ws, wsm = O.fake_quantize(small, 16, 32, clamp, mode, 1)
    assert np.array_equal(got[1][1], wsm) and np.array_equal(got[1][0], ws), case


def test_more_random_cases_on_request(G):
    """MOR_SWEEP_EXTRA=n (with MOR_SWEEP_SEED=s) runs n further random cases of fake_quantize and of the scaling ops
    against the oracle: a way to look for rare disagreements with seeds the fixed lists above do not hold."""
    import os
    n = int(os.environ.get("MOR_SWEEP_EXTRA", "0"))
    if n == 0:
        pytest.skip("set MOR_SWEEP_EXTRA to run")
    seed0 = int(os.environ.get("MOR_SWEEP_SEED", "1"))
    rng = np.random.default_rng(seed0)
    fq_blocks = [(1, 8), (1, 32), (1, 64), (1, 256), (1, 1024), (1, 4096), (2, 64), (8, 8), (16, 56), (32, 32), (64, 64), (128, 128),
                 (128, 64), (64, 256), (3, 40), (5, 7), (1, 24), (128, 256), (256, 256), (100, 127), (7, 3)]
    bs_blocks = [(1, 32), (1, 256), (1, 2048), (1, 4096), (128, 128), (64, 64), (32, 16), (16, 120), (20, 12), (64, 1), (256, 1), (8, 1),
                 (8, 8), (128, 256), (512, 1)]
    bad = []
    in_window = 0
    for i in range(n):
        data_rng = np.random.default_rng(seed0 * 100003 + i)
        kind = int(rng.integers(4))
        if i % 2 == 0:
            br, bc = fq_blocks[rng.integers(len(fq_blocks))]
            rows = max(1, br * int(rng.integers(1, 5)) - (int(rng.integers(0, br)) if rng.random() < 0.4 else 0))
            cols = max(1, bc * int(rng.integers(1, 5)) - (int(rng.integers(0, bc)) if rng.random() < 0.4 else 0))
            mode, sf, clamp = int(rng.choice([1, 101, 2, 3])), int(rng.choice([1, 2])), float(rng.choice([1e-15, 1e-3, 0.5]))
            a = make_data(data_rng, rows, cols, kind)
            out, meta = G.fake_quantize(a, br, bc, clamp, mode, sf)
            want, wmeta, stats = O.fake_quantize(a, br, bc, clamp, mode, sf, want_stats=True)
            if (meta != wmeta).any():            # (close sums are added in the reference's order: no decision may differ)
                bad.append(("decision", i, rows, cols, br, bc, mode, sf, kind))
            elif not np.array_equal(out, want):
                bad.append(("values", i, rows, cols, br, bc, mode, sf, kind))
        else:
            br, bc = bs_blocks[rng.integers(len(bs_blocks))]
            rows, cols = br * int(rng.integers(1, 5)), bc * (int(rng.choice([8, 40, 64, 200, 520])) if bc == 1 else int(rng.integers(1, 5)))
            ss, inplace, thr = int(rng.choice([1, 2, 3, 4])), bool(rng.integers(2)), float(rng.choice([0.02, 0.045, 0.2]))
            a = make_data(data_rng, rows, cols, kind % 3)
            channel = br == 1 or bc == 1
            out, meta, gamax, gnnz, gerr = G.block_scaling(a, br, bc, thr, ss, channel=channel, inplace=inplace)
            want, wmeta, wamax, wnnz, werr = O.block_scaling(a, br, bc, thr, ss, channel=channel)
            case = ("scaling", i, rows, cols, br, bc, ss, kind % 3, inplace, thr)
            if gamax[0] != wamax[0] or gnnz[0] != wnnz[0] or abs(float(gerr[0]) - float(werr[0])) > 2e-6 * abs(float(werr[0])):
                bad.append(case)
            elif abs(werr[0] / max(wnnz[0], 1) - thr) <= 1e-5 * thr:
                in_window += 1
            elif meta[0] != wmeta[0]:
                bad.append(case)
            elif not np.array_equal(out, want):
                bad.append(case)
    print("extra random cases:", n, "seed", seed0, "disagreements:", len(bad), "scaling cases inside the 1e-5 threshold window:", in_window, flush=True)
    assert not bad, bad[:10]
