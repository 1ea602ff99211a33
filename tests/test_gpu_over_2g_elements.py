"""A tensor of more than 2^31 elements (4.3 GB of bf16; an embedding table of 128256 x 16384 is of this size): element
and chunk offsets no longer fit 32 bits.  Every block is quantized on its own, so the result on the whole tensor must
equal the results on its two parts, bit for bit, and the row-wise half of the two-orientation wire quantizer must equal
the single-orientation one.

A launch holds fewer than 2^32 threads per dimension and wraps a larger grid without an error, so kernels that take one
workgroup per block are launched in slices of 2^22 blocks: the cases here with more blocks than that check the slices
against launches that need none."""
import pytest
import torch

from mor_amd import _cabi

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(300)]

ROWS, COLS = 32384, 66560         # 253 x 520 tiles of 128 x 128: 2 155 479 040 elements
SPLIT = 126 * 128


@pytest.fixture(scope="module")
def x():
    assert torch.cuda.is_available()
    assert ROWS * COLS > 2 ** 31
    g = torch.Generator(device="cuda").manual_seed(77)
    t = torch.empty(ROWS, COLS, dtype=torch.bfloat16, device="cuda")
    for r in range(0, ROWS, 4048):                          # in slabs, so that the fp32 draw stays small
        t[r:r + 4048] = torch.randn(min(4048, ROWS - r), COLS, device="cuda", generator=g).to(torch.bfloat16)
    t[:128, :128] *= 1e-3
    t[ROWS - 128:, COLS - 128:] = torch.exp(3 * t[ROWS - 128:, COLS - 128:].float()).to(torch.bfloat16)   # the last tile: wide range
    t[ROWS - 1, :] = 0
    t[1000:1200, :] = 0                                      # so that the count of non-zero elements fits its 32-bit int
    return t


def stream():
    return torch.cuda.current_stream().cuda_stream


def fq(t, mode, sf, br, bc, clamp, flags=0):
    L = _cabi.lib()
    r, c = t.shape
    out = torch.empty_like(t)
    meta = torch.full(((r + br - 1) // br, c // bc), -9, dtype=torch.int32, device="cuda")
    _cabi.check(L.mor_fake_quantize(t.data_ptr(), out.data_ptr(), meta.data_ptr(), r, c, br, bc, clamp, mode, sf, flags, stream()))
    torch.cuda.synchronize()
    return out, meta


@pytest.mark.parametrize("args", [(1, 1, 128, 128, 1e-15), (2, 2, 1, 32, 0.0), (4, 1, 128, 128, 37.5), (3, 1, 1, 66560, 0.0)],
                         ids=["mor_tiles", "mx_1x32", "per_tensor_scale", "per_row"])
def test_fake_quantize_whole_equals_parts(x, args):
    print("over 2^31 elements: fake_quantize", args, flush=True)
    mode, sf, br, bc, clamp = args
    out, meta = fq(x, mode, sf, br, bc, clamp)
    assert int((meta == -9).sum()) == 0
    for part in (slice(0, SPLIT), slice(SPLIT, ROWS)):
        o2, m2 = fq(x[part], mode, sf, br, bc, clamp)        # a row range of a contiguous tensor is contiguous
        assert torch.equal(out[part].view(torch.int16), o2.view(torch.int16))
        assert torch.equal(meta[part.start // br: (part.stop + br - 1) // br], m2)
        del o2, m2
    if mode == 1:
        assert int(meta[-1, -1]) in (2, 3, 12)               # the wide-range tile at the far end was seen as such


def scaling(t):
    L = _cabi.lib()
    r, c = t.shape
    out = torch.empty_like(t)
    meta = torch.empty(1, dtype=torch.int32, device="cuda")
    amax = torch.empty(1, dtype=torch.float32, device="cuda")
    nnz = torch.empty(1, dtype=torch.int32, device="cuda")
    err = torch.empty(1, dtype=torch.float32, device="cuda")
    nbytes = L.mor_workspace_bytes(_cabi.OP_BLOCK_SCALING, r, c, 128, 128)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device="cuda")
    _cabi.check(L.mor_block_scaling(t.data_ptr(), out.data_ptr(), meta.data_ptr(), amax.data_ptr(), nnz.data_ptr(), err.data_ptr(),
                                    r, c, 128, 128, 0.045, 3, 0, ws.data_ptr(), nbytes, 0, stream()))
    torch.cuda.synchronize()
    return out, int(meta.item()), float(amax.item()), int(nnz.item()), float(err.item())


def test_block_scaling_whole_equals_parts(x):
    print("over 2^31 elements: block_scaling", flush=True)
    out, meta, amax, nnz, err = scaling(x)
    assert meta == 1
    a, b = scaling(x[:SPLIT]), scaling(x[SPLIT:])
    assert torch.equal(out[:SPLIT].view(torch.int16), a[0].view(torch.int16))
    assert torch.equal(out[SPLIT:].view(torch.int16), b[0].view(torch.int16))
    # the reference's count is a 32-bit int as well (mor/csrc/cuda/fake_quantize.cu:1017-1049); this tensor's fits
    assert nnz == a[3] + b[3] == ROWS * COLS - int((x == 0).sum())
    assert amax == max(a[2], b[2])
    assert err == pytest.approx(a[4] + b[4], rel=1e-6)


def test_wire_whole_equals_parts_and_round_trip(x):
    print("over 2^31 elements: wire format", flush=True)
    L = _cabi.lib()
    n = ROWS * COLS
    fmt = _cabi.FMT_E4M3
    p, s = torch.empty(n, dtype=torch.uint8, device="cuda"), torch.empty(n // 32, dtype=torch.uint8, device="cuda")
    _cabi.check(L.mor_mx_quantize(x.data_ptr(), p.data_ptr(), s.data_ptr(), ROWS, COLS, fmt, stream()))
    torch.cuda.synchronize()
    for part in (slice(0, SPLIT), slice(SPLIT, ROWS)):
        xp = x[part]
        m = xp.numel()
        p2, s2 = torch.empty(m, dtype=torch.uint8, device="cuda"), torch.empty(m // 32, dtype=torch.uint8, device="cuda")
        _cabi.check(L.mor_mx_quantize(xp.data_ptr(), p2.data_ptr(), s2.data_ptr(), xp.shape[0], COLS, fmt, stream()))
        torch.cuda.synchronize()
        lo = part.start * COLS
        assert torch.equal(p[lo:lo + m], p2) and torch.equal(s[lo // 32:(lo + m) // 32], s2)
        del p2, s2
    # decode == the fake quantizer's output (MX E4M3, E8M0 scales) in the torch-emulation flavour, which is free of the
    # exponent-field artefacts of the production arithmetic (mor/csrc/cuda/fake_quantize.cu:248-306)
    back = torch.empty_like(x)
    _cabi.check(L.mor_mx_dequantize(p.data_ptr(), s.data_ptr(), back.data_ptr(), ROWS, COLS, fmt, stream()))
    want, _ = fq(x, 2, 2, 1, 32, 0.0, _cabi.FLAG_TORCH_EMULATION)
    assert torch.equal(back.view(torch.int16), want.view(torch.int16))
    del back, want
    # both orientations in one read: its row half is the same payload; its column half is the payload of the transpose
    pc, sc = torch.empty(n, dtype=torch.uint8, device="cuda"), torch.empty(n // 32, dtype=torch.uint8, device="cuda")
    pr, sr = torch.empty(n, dtype=torch.uint8, device="cuda"), torch.empty(n // 32, dtype=torch.uint8, device="cuda")
    _cabi.check(L.mor_mx_quantize_dual(x.data_ptr(), pr.data_ptr(), sr.data_ptr(), pc.data_ptr(), sc.data_ptr(), ROWS, COLS, fmt, stream()))
    torch.cuda.synchronize()
    assert torch.equal(pr, p) and torch.equal(sr, s)
    xt = x.t().contiguous()
    _cabi.check(L.mor_mx_quantize(xt.data_ptr(), p.data_ptr(), s.data_ptr(), COLS, ROWS, fmt, stream()))
    torch.cuda.synchronize()
    assert torch.equal(pc, p) and torch.equal(sc, s)


@pytest.mark.parametrize("flags", [0, _cabi.FLAG_TORCH_EMULATION], ids=["production", "torch_emulation"])
@pytest.mark.parametrize("bc", [40, 20], ids=["1x40_vector_rows", "1x20_pairs"])
def test_more_blocks_than_one_launch(x, flags, bc):
    """53.9 M (107.8 M) blocks of 1 x 40 (1 x 20): one workgroup per block, 13 (26) launches.  Slabs of 1024 rows need one."""
    print("over 2^31 elements: one workgroup per block", flags, bc, flush=True)
    out, meta = fq(x, 2, 1, 1, bc, 0.0, flags)
    assert int((meta == -9).sum()) == 0
    for r0 in (0, 1024, 14336, 24576, ROWS - 1024):
        part = slice(r0, r0 + 1024)
        assert 1024 * (COLS // bc) < 2 ** 22
        o2, m2 = fq(x[part], 2, 1, 1, bc, 0.0, flags)
        assert torch.equal(out[part].view(torch.int16), o2.view(torch.int16))
        assert torch.equal(meta[part], m2)


def test_tensor_size_limit():
    L = _cabi.lib()
    t = torch.zeros(64, dtype=torch.bfloat16, device="cuda")
    m = torch.zeros(64, dtype=torch.int32, device="cuda")
    assert L.mor_fake_quantize(t.data_ptr(), t.data_ptr(), m.data_ptr(), 2 ** 20, 2 ** 15 + 8, 2 ** 20, 2 ** 15 + 8, 0.0, 7, 1, 0, None) == -1
    assert b"too large" in L.mor_last_error()
