"""mor_fake_quantize_dual: one read, the fake-quantized tensor (1 x 32 blocks) and the fake-quantized transpose.
Both halves must equal what the oracle (and mor_fake_quantize) give for the tensor and for its transpose."""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
import data_gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def cases():
    yield "student_t", data_gen.c2_student_t(128, 256, seed=41)
    yield "ragged_tiles", data_gen.c1_normal(160, 224, seed=42)
    w = data_gen.c3_weights(96, 160, seed=43)
    w[5] = 0
    w[:, 7] = 0x8000
    yield "zero_row_and_column", w
    rng = np.random.default_rng(44)
    yield "every_exponent", (rng.integers(0x0001, 0x7F80, (64, 96)) | (rng.integers(0, 2, (64, 96)) << 15)).astype(np.uint16)
    yield "one_block", data_gen.c1_normal(32, 32, seed=45)


@pytest.mark.parametrize("mode", [2, 3])
@pytest.mark.parametrize("sf", [1, 2])
def test_both_orientations_match_oracle(G, mode, sf):
    for name, a in cases():
        print("fq_dual", name, a.shape, mode, sf, flush=True)
        at = np.ascontiguousarray(a.T)
        want, wmeta = O.fake_quantize(a, 1, 32, 0.0, mode, sf)
        want_t, wmeta_t = O.fake_quantize(at, 1, 32, 0.0, mode, sf)
        out, meta, out_t, meta_t = G.fake_quantize_dual(a, mode, sf)
        for got, exp, what in ((out, want, "rows"), (out_t, want_t, "columns"), (meta, wmeta, "meta"), (meta_t, wmeta_t, "meta_t")):
            bad = np.argwhere(got != exp)
            assert len(bad) == 0, (name, what, len(bad), tuple(bad[0]), hex(int(got[tuple(bad[0])])), hex(int(exp[tuple(bad[0])])))
    out, meta, out_t, meta_t = G.fake_quantize_dual(a, mode, sf, want_meta=False)      # NULL meta pointers
    assert np.all(meta == -7) and np.all(meta_t == -7) and np.array_equal(out, want)


# tile grids (128 x 128 tiles) that take each of the workgroup -> tile orders the kernel chooses between
@pytest.mark.parametrize("rows,cols,mode,sf", [(1024, 512, 2, 2), (2048, 1024, 3, 1), (4096, 1024, 2, 1), (1024, 4096, 3, 2),
                                               (2048, 4096, 2, 2), (8192, 512, 3, 2), (256, 8192, 2, 1), (128, 8192, 2, 2),
                                               (1152, 1280, 3, 1)])
def test_tile_orders_match_oracle(G, rows, cols, mode, sf):
    print("fq_dual tile order", rows, cols, mode, sf, flush=True)
    a = data_gen.c2_student_t(rows, cols, seed=rows + cols)
    want, wmeta = O.fake_quantize(a, 1, 32, 0.0, mode, sf)
    want_t, wmeta_t = O.fake_quantize(np.ascontiguousarray(a.T), 1, 32, 0.0, mode, sf)
    out, meta, out_t, meta_t = G.fake_quantize_dual(a, mode, sf)
    for got, exp, what in ((out, want, "rows"), (out_t, want_t, "columns"), (meta, wmeta, "meta"), (meta_t, wmeta_t, "meta_t")):
        bad = np.argwhere(got != exp)
        assert len(bad) == 0, (what, len(bad), tuple(bad[0]))


def test_argument_checks(G):
    from mor_amd import _cabi
    L = _cabi.lib()
    x = torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda")
    o = torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda")
    t = torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda")
    assert L.mor_fake_quantize_dual(x.data_ptr(), o.data_ptr(), None, t.data_ptr(), None, 64, 48, 2, 2, None) == -1
    assert L.mor_fake_quantize_dual(x.data_ptr(), x.data_ptr(), None, t.data_ptr(), None, 64, 64, 2, 2, None) == -1   # alias
    assert L.mor_fake_quantize_dual(x.data_ptr(), o.data_ptr(), None, t.data_ptr(), None, 64, 64, 1, 2, None) == -1   # MoR mode
    assert b"mode" in L.mor_last_error()


@pytest.mark.parametrize("mode,sf", [(2, 2), (3, 1)])
def test_full_size_equals_the_single_orientation_kernels(G, mode, sf):
    from mor_amd import _cabi
    L = _cabi.lib()
    rows, cols = 8192, 4096
    x = data_gen.c2_student_t(rows, cols, seed=1002, as_tensor=True).cuda()
    xt = x.t().contiguous()
    st = torch.cuda.current_stream().cuda_stream
    o, ot = torch.empty_like(x), torch.empty_like(xt)
    m = torch.empty((rows, cols // 32), dtype=torch.int32, device="cuda")
    mt = torch.empty((cols, rows // 32), dtype=torch.int32, device="cuda")
    _cabi.check(L.mor_fake_quantize_dual(x.data_ptr(), o.data_ptr(), m.data_ptr(), ot.data_ptr(), mt.data_ptr(), rows, cols, mode, sf, st))
    w, wt = torch.empty_like(x), torch.empty_like(xt)
    wm, wmt = torch.empty_like(m), torch.empty_like(mt)
    _cabi.check(L.mor_fake_quantize(x.data_ptr(), w.data_ptr(), wm.data_ptr(), rows, cols, 1, 32, 0.0, mode, sf, 0, st))
    _cabi.check(L.mor_fake_quantize(xt.data_ptr(), wt.data_ptr(), wmt.data_ptr(), cols, rows, 1, 32, 0.0, mode, sf, 0, st))
    torch.cuda.synchronize()
    assert torch.equal(o.view(torch.int16), w.view(torch.int16)) and torch.equal(m, wm)
    assert torch.equal(ot.view(torch.int16), wt.view(torch.int16)) and torch.equal(mt, wmt)


def test_python_api(G):
    from mor_amd import wire
    import mor
    x = data_gen.c2_student_t(256, 512, seed=51, as_tensor=True).cuda()
    out, meta, out_t, meta_t = wire.fake_quantize_mx_dual(x, mode=3, sf_type=2)
    want, wmeta = mor.ops.fake_quantize(x, 256, 512, 1, 32, 0.0, 3, 2)
    want_t, wmeta_t = mor.ops.fake_quantize(x.t().contiguous(), 512, 256, 1, 32, 0.0, 3, 2)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16)) and torch.equal(meta, wmeta)
    assert torch.equal(out_t.view(torch.int16), want_t.view(torch.int16)) and torch.equal(meta_t, wmeta_t)
