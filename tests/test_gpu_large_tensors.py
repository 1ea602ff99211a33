"""Tensors beyond the 256 MB last-level cache (more than 2^27 elements): there the tile kernels walk the block grid in
XCD bands.  Every block is quantized on its own, so the result on the whole tensor must equal the results on its two
halves (which are small enough for the plain order), bit for bit; global sums add up."""
import pytest
import torch

from mor_amd import _cabi

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(300)]

ROWS, COLS = 16384, 9216          # 72 x 128 tiles of 128 x 128; 151 M elements


@pytest.fixture(scope="module")
def x():
    assert torch.cuda.is_available()
    g = torch.Generator(device="cuda").manual_seed(2024)
    t = torch.randn(ROWS, COLS, device="cuda", generator=g)
    t[:128, :128] *= 1e-3
    t[4096:4224, 256:384] = torch.exp(3 * t[4096:4224, 256:384])
    t[300, :] = 0
    return t.to(torch.bfloat16)


def stream():
    return torch.cuda.current_stream().cuda_stream


def fq(t, mode, sf, clamp=1e-15):
    L = _cabi.lib()
    r, c = t.shape
    out = torch.empty_like(t)
    meta = torch.full((r // 128, c // 128), -9, dtype=torch.int32, device="cuda")
    _cabi.check(L.mor_fake_quantize(t.data_ptr(), out.data_ptr(), meta.data_ptr(), r, c, 128, 128, clamp, mode, sf, 0, stream()))
    return out, meta


@pytest.mark.parametrize("mode,sf", [(1, 1), (2, 1), (3, 2)])
def test_fake_quantize_whole_equals_halves(x, mode, sf):
    print("large fake_quantize", mode, sf, flush=True)
    out, meta = fq(x, mode, sf)
    h = ROWS // 2
    for part in (slice(0, h), slice(h, ROWS)):
        o2, m2 = fq(x[part].contiguous(), mode, sf)
        assert torch.equal(out[part].view(torch.int16), o2.view(torch.int16))
        assert torch.equal(meta[part.start // 128: part.stop // 128], m2)
    assert int((meta == -9).sum()) == 0


def scaling(t, inplace=False):
    L = _cabi.lib()
    r, c = t.shape
    src = t.clone() if inplace else t
    out = src if inplace else torch.empty_like(t)
    meta = torch.empty(1, dtype=torch.int32, device="cuda")
    amax = torch.empty(1, dtype=torch.float32, device="cuda")
    nnz = torch.empty(1, dtype=torch.int32, device="cuda")
    err = torch.empty(1, dtype=torch.float32, device="cuda")
    nbytes = L.mor_workspace_bytes(_cabi.OP_BLOCK_SCALING, r, c, 128, 128)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device="cuda")
    _cabi.check(L.mor_block_scaling(src.data_ptr(), out.data_ptr(), meta.data_ptr(), amax.data_ptr(), nnz.data_ptr(), err.data_ptr(),
                                    r, c, 128, 128, 0.045, 3, 0, ws.data_ptr(), nbytes, 0, stream()))
    torch.cuda.synchronize()
    return out, int(meta.item()), float(amax.item()), int(nnz.item()), float(err.item())


@pytest.mark.parametrize("inplace", [False, True])
def test_block_scaling_whole_equals_halves(x, inplace):
    print("large block_scaling", inplace, flush=True)
    out, meta, amax, nnz, err = scaling(x, inplace)
    assert meta == 1
    h = ROWS // 2
    parts = [scaling(x[:h].contiguous(), inplace), scaling(x[h:].contiguous(), inplace)]
    assert torch.equal(out[:h].view(torch.int16), parts[0][0].view(torch.int16))
    assert torch.equal(out[h:].view(torch.int16), parts[1][0].view(torch.int16))
    assert nnz == parts[0][3] + parts[1][3] == int((x != 0).sum())
    assert amax == max(parts[0][2], parts[1][2])
    assert err == pytest.approx(parts[0][4] + parts[1][4], rel=1e-6)


@pytest.mark.parametrize("fmt", [_cabi.FMT_E4M3, _cabi.FMT_E2M3])
def test_dual_wire_whole_equals_single_orientation(x, fmt):
    print("large mx_quantize_dual", fmt, flush=True)
    L = _cabi.lib()
    n = ROWS * COLS
    pb = n if fmt == _cabi.FMT_E4M3 else n // 4 * 3
    bufs = [torch.empty(pb, dtype=torch.uint8, device="cuda") for _ in range(3)]
    scs = [torch.empty(n // 32, dtype=torch.uint8, device="cuda") for _ in range(3)]
    _cabi.check(L.mor_mx_quantize_dual(x.data_ptr(), bufs[0].data_ptr(), scs[0].data_ptr(), bufs[1].data_ptr(), scs[1].data_ptr(),
                                       ROWS, COLS, fmt, stream()))
    _cabi.check(L.mor_mx_quantize(x.data_ptr(), bufs[2].data_ptr(), scs[2].data_ptr(), ROWS, COLS, fmt, stream()))
    torch.cuda.synchronize()
    assert torch.equal(bufs[0], bufs[2]) and torch.equal(scs[0], scs[2])
    xt = x.t().contiguous()
    _cabi.check(L.mor_mx_quantize(xt.data_ptr(), bufs[2].data_ptr(), scs[2].data_ptr(), COLS, ROWS, fmt, stream()))
    torch.cuda.synchronize()
    assert torch.equal(bufs[1], bufs[2]) and torch.equal(scs[1], scs[2])


def test_fake_quantize_dual_whole_equals_single_orientation(x):
    print("large fake_quantize_dual", flush=True)
    L = _cabi.lib()
    n = ROWS * COLS
    o, ot, ref = torch.empty_like(x), torch.empty((COLS, ROWS), dtype=torch.bfloat16, device="cuda"), torch.empty_like(x)
    m, mt, mref = (torch.empty(n // 32, dtype=torch.int32, device="cuda") for _ in range(3))
    _cabi.check(L.mor_fake_quantize_dual(x.data_ptr(), o.data_ptr(), m.data_ptr(), ot.data_ptr(), mt.data_ptr(), ROWS, COLS, 2, 2, stream()))
    _cabi.check(L.mor_fake_quantize(x.data_ptr(), ref.data_ptr(), mref.data_ptr(), ROWS, COLS, 1, 32, 0.0, 2, 2, 0, stream()))
    torch.cuda.synchronize()
    assert torch.equal(o.view(torch.int16), ref.view(torch.int16)) and torch.equal(m, mref)
    xt = x.t().contiguous()
    reft = torch.empty_like(xt)
    _cabi.check(L.mor_fake_quantize(xt.data_ptr(), reft.data_ptr(), mref.data_ptr(), COLS, ROWS, 1, 32, 0.0, 2, 2, 0, stream()))
    torch.cuda.synchronize()
    assert torch.equal(ot.view(torch.int16), reft.view(torch.int16)) and torch.equal(mt, mref)


def test_linear_kernels_whole_equals_halves(x):
    """MX 1 x 32, per-tensor scale and the wire quantizer read such a tensor with streaming loads."""
    print("large linear kernels", flush=True)
    L = _cabi.lib()
    h = ROWS // 2

    def mx(t, mode, sf, br, bc, clamp=0.0):
        r, c = t.shape
        out = torch.empty_like(t)
        meta = torch.full(((r + br - 1) // br, c // bc), -9, dtype=torch.int32, device="cuda")
        _cabi.check(L.mor_fake_quantize(t.data_ptr(), out.data_ptr(), meta.data_ptr(), r, c, br, bc, clamp, mode, sf, 0, stream()))
        return out, meta

    for args in ((2, 2, 1, 32), (3, 2, 1, 32), (4, 1, 128, 128, 37.5), (2, 1, 1, 1024)):
        out, meta = mx(x, *args)
        for part in (slice(0, h), slice(h, ROWS)):
            o2, _ = mx(x[part].contiguous(), *args)
            assert torch.equal(out[part].view(torch.int16), o2.view(torch.int16)), args
        assert int((meta == -9).sum()) == 0
    n = ROWS * COLS
    p, s_ = torch.empty(n, dtype=torch.uint8, device="cuda"), torch.empty(n // 32, dtype=torch.uint8, device="cuda")
    p2, s2 = torch.empty(n // 2, dtype=torch.uint8, device="cuda"), torch.empty(n // 64, dtype=torch.uint8, device="cuda")
    _cabi.check(L.mor_mx_quantize(x.data_ptr(), p.data_ptr(), s_.data_ptr(), ROWS, COLS, _cabi.FMT_E4M3, stream()))
    for k, part in enumerate((slice(0, h), slice(h, ROWS))):
        xp = x[part].contiguous()
        _cabi.check(L.mor_mx_quantize(xp.data_ptr(), p2.data_ptr(), s2.data_ptr(), h, COLS, _cabi.FMT_E4M3, stream()))
        torch.cuda.synchronize()
        assert torch.equal(p[k * (n // 2):(k + 1) * (n // 2)], p2) and torch.equal(s_[k * (n // 64):(k + 1) * (n // 64)], s2)
