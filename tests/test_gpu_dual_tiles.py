"""mor_fake_quantize_dual_tiles: both outputs equal what the CPU oracle gives for x and for its transpose, 128 x 128
tiles, MoR and the forced formats."""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
from data_gen import tile_mixture as mixture

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def dual(G, a, clamp, mode, sf):
    from mor_amd import _cabi
    L = _cabi.lib()
    rows, cols = a.shape
    x = G.to_dev_u16(a)
    out = torch.full_like(x, 7.0)
    out_t = torch.full((cols, rows), 7.0, dtype=torch.bfloat16, device=G.dev())
    meta = torch.full((rows // 128, cols // 128), -7, dtype=torch.int32, device=G.dev())
    meta_t = torch.full((cols // 128, rows // 128), -7, dtype=torch.int32, device=G.dev())
    _cabi.check(L.mor_fake_quantize_dual_tiles(x.data_ptr(), out.data_ptr(), meta.data_ptr(), out_t.data_ptr(), meta_t.data_ptr(),
                                               rows, cols, float(clamp), mode, sf, G.stream_ptr()))
    torch.cuda.synchronize()
    return G.to_host_u16(out), meta.cpu().numpy(), G.to_host_u16(out_t), meta_t.cpu().numpy()


@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (1024, 512), (2048, 2048)])
@pytest.mark.parametrize("mode,sf", [(1, 1), (1, 2), (101, 1), (2, 1), (2, 2), (3, 1), (3, 2)])
def test_both_orientations_match_the_oracle(G, shape, mode, sf):
    rows, cols = shape
    rng = np.random.default_rng(rows * 3 + cols + mode * 7 + sf)
    a = mixture(rng, rows, cols)
    a[5, 7] = 0x7FC0                # a NaN and an infinity in the first tile
    a[9, 3] = 0xFF80
    clamp = 1e-3
    print("dual tiles", shape, mode, sf, flush=True)
    out, meta, out_t, meta_t = dual(G, a, clamp, mode, sf)
    want, wmeta = O.fake_quantize(a, 128, 128, clamp, mode, sf)
    at = np.ascontiguousarray(a.T)
    want_t, wmeta_t = O.fake_quantize(at, 128, 128, clamp, mode, sf)
    assert np.array_equal(meta, wmeta), "meta differs"
    assert np.array_equal(out, want), "output differs"
    assert np.array_equal(meta_t, wmeta_t), "transposed meta differs"
    assert np.array_equal(out_t, want_t), "transposed output differs"
    assert np.array_equal(out_t, np.ascontiguousarray(out.T)) and np.array_equal(meta_t, meta.T)


def test_large_tensor_round_trip_property(G):
    """8192 x 4096 (band order, streaming stores): out_t is the transpose of out, and out is what mor_fake_quantize gives"""
    rows, cols = 8192, 4096
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(rows, cols, device="cuda", generator=g)
    x[:, :1024] *= torch.exp(3 * torch.randn(rows, 1024, device="cuda", generator=g))
    x = x.to(torch.bfloat16)
    import mor_amd
    for mode in (1, 2):
        out, meta, out_t, meta_t = mor_amd.wire.fake_quantize_tiles_dual(x, 1e-15, mode, 1)
        ref, rmeta = mor_amd.ops.fake_quantize(x, rows, cols, 128, 128, 1e-15, mode, 1)
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)) and torch.equal(meta, rmeta.view(meta.shape))
        assert torch.equal(out_t.view(torch.int16), out.t().contiguous().view(torch.int16)) and torch.equal(meta_t, meta.t())


def test_rejects_what_it_cannot_do(G):
    from mor_amd import _cabi
    L = _cabi.lib()
    x = torch.zeros((128, 256), dtype=torch.bfloat16, device=G.dev())
    o = torch.zeros_like(x)
    ot = torch.zeros((256, 128), dtype=torch.bfloat16, device=G.dev())
    m = torch.zeros(2, dtype=torch.int32, device=G.dev())
    args = lambda r, c, mode, a=x, b=o, d=ot: (a.data_ptr(), b.data_ptr(), m.data_ptr(), d.data_ptr(), m.data_ptr(), r, c, 0.0, mode, 1, G.stream_ptr())
    assert L.mor_fake_quantize_dual_tiles(*args(128, 200, 1)) != 0 and b"multiples of 128" in L.mor_last_error()
    assert L.mor_fake_quantize_dual_tiles(*args(128, 256, 4)) != 0 and b"mode" in L.mor_last_error()
    assert L.mor_fake_quantize_dual_tiles(*args(128, 256, 1, x, x, ot)) != 0 and b"different" in L.mor_last_error()
