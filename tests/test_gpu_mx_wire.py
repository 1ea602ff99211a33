"""GPU parity of the MX wire format (mor_mx_quantize, mor_mx_quantize_dual, mor_mx_dequantize) against the CPU oracle,
plus size-independent properties at the benchmark size."""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
import data_gen
import torch_emulation as E

pytestmark = pytest.mark.gpu

FORMATS = [O.E4M3, O.E5M2, O.E3M2, O.E2M3]


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def cases():
    yield "student_t", data_gen.c2_student_t(96, 512, seed=21)
    yield "normal_ragged_tile", data_gen.c1_normal(160, 224, seed=22)
    w = data_gen.c3_weights(64, 256, seed=23)
    w[5] = 0
    w[6, :32] = 0x8000
    yield "weights_with_zero_rows", w
    rng = np.random.default_rng(24)
    wide = (rng.integers(0x0080, 0x7F00, (64, 128)) | (rng.integers(0, 2, (64, 128)) << 15)).astype(np.uint16)
    yield "wide_exponents", wide
    yield "one_block", data_gen.c1_normal(32, 32, seed=25)


def first_diff(got, want):
    bad = np.argwhere(got != want)
    return None if len(bad) == 0 else (tuple(bad[0]), int(got[tuple(bad[0])]), int(want[tuple(bad[0])]), len(bad))


@pytest.mark.parametrize("fmt", FORMATS)
def test_quantize_matches_oracle(G, fmt):
    for name, a in cases():
        print("mx_quantize", name, a.shape, fmt, flush=True)
        wp, ws = O.mx_quantize(a, fmt)
        gp, gs = G.mx_quantize(a, fmt)
        assert first_diff(gs, ws) is None, (name, "scales", first_diff(gs, ws))
        assert first_diff(gp, wp) is None, (name, "payload", first_diff(gp, wp))


@pytest.mark.parametrize("fmt", FORMATS)
def test_dual_matches_oracle_on_the_tensor_and_its_transpose(G, fmt):
    for name, a in cases():
        print("mx_quantize_dual", name, a.shape, fmt, flush=True)
        wp, ws = O.mx_quantize(a, fmt)
        tp, ts = O.mx_quantize(np.ascontiguousarray(a.T), fmt)
        rp, rs, cp, cs = G.mx_quantize_dual(a, fmt)
        assert first_diff(rs, ws) is None and first_diff(rp, wp) is None, (name, "rows", first_diff(rs, ws), first_diff(rp, wp))
        assert first_diff(cs, ts) is None, (name, "column scales", first_diff(cs, ts))
        assert first_diff(cp, tp) is None, (name, "column payload", first_diff(cp, tp))


# tile grids (128 x 128 tiles) that take each of the workgroup -> tile orders the dual kernels choose between
TILE_ORDER_SHAPES = [(1024, 512), (2048, 1024), (1024, 2048), (4096, 1024), (1024, 4096), (2048, 4096), (8192, 512),
                     (256, 8192), (128, 8192), (1152, 1280)]


@pytest.mark.parametrize("k", range(len(TILE_ORDER_SHAPES)))
def test_dual_tile_orders_match_oracle(G, k):
    rows, cols = TILE_ORDER_SHAPES[k]
    fmt = FORMATS[k % 4]
    print("mx_quantize_dual tile order", rows, cols, fmt, flush=True)
    a = data_gen.c2_student_t(rows, cols, seed=60 + k)
    wp, ws = O.mx_quantize(a, fmt)
    tp, ts = O.mx_quantize(np.ascontiguousarray(a.T), fmt)
    rp, rs, cp, cs = G.mx_quantize_dual(a, fmt)
    assert first_diff(rs, ws) is None and first_diff(rp, wp) is None, ("rows", first_diff(rs, ws), first_diff(rp, wp))
    assert first_diff(cs, ts) is None and first_diff(cp, tp) is None, ("columns", first_diff(cs, ts), first_diff(cp, tp))


@pytest.mark.parametrize("fmt", FORMATS)
def test_dequantize_matches_oracle(G, fmt):
    for name, a in cases():
        print("mx_dequantize", name, a.shape, fmt, flush=True)
        wp, ws = O.mx_quantize(a, fmt)
        want = O.mx_dequantize(wp, ws, fmt)
        got = G.mx_dequantize(wp, ws, fmt)
        assert first_diff(got, want) is None, (name, first_diff(got, want))


def test_argument_checks(G):
    from mor_amd import _cabi
    L = _cabi.lib()
    x = torch.zeros(32, 48, dtype=torch.bfloat16, device="cuda")
    p = torch.zeros(32 * 48, dtype=torch.uint8, device="cuda")
    s = torch.zeros(64, dtype=torch.uint8, device="cuda")
    assert L.mor_mx_quantize(x.data_ptr(), p.data_ptr(), s.data_ptr(), 32, 48, 0, None) == -1       # cols % 32
    assert b"cols" in L.mor_last_error()
    assert L.mor_mx_quantize(x.data_ptr(), p.data_ptr(), s.data_ptr(), 32, 64, 7, None) == -1       # format
    assert L.mor_mx_quantize(x.data_ptr(), None, s.data_ptr(), 32, 64, 0, None) == -1
    assert L.mor_mx_quantize_dual(x.data_ptr(), p.data_ptr(), s.data_ptr(), p.data_ptr(), s.data_ptr(), 48, 64, 0, None) == -1
    assert L.mor_mx_payload_bytes(64, 128, 0) == 64 * 128 and L.mor_mx_payload_bytes(64, 128, 3) == 64 * 96


@pytest.mark.parametrize("fmt", FORMATS)
def test_full_size_properties(G, fmt):
    """8192 x 8192 (the benchmark tensor): dequantize(quantize(x)) equals the fake-quantized tensor in the
    torch-emulation flavour, quantizing that tensor again decodes to the same values, and the dual kernel's two halves equal the single
    kernel on x and on x transposed."""
    from mor_amd import _cabi
    L = _cabi.lib()
    rows = cols = 8192
    x = data_gen.c2_student_t(rows, cols, seed=1002, as_tensor=True).cuda()
    st = torch.cuda.current_stream().cuda_stream
    rb = G.mx_row_bytes(cols, fmt)

    def quantize(t):
        p = torch.empty((rows, rb), dtype=torch.uint8, device="cuda")
        s = torch.empty((rows, cols // 32), dtype=torch.uint8, device="cuda")
        _cabi.check(L.mor_mx_quantize(t.data_ptr(), p.data_ptr(), s.data_ptr(), rows, cols, fmt, st))
        return p, s

    p, s = quantize(x)
    deq = torch.empty_like(x)
    _cabi.check(L.mor_mx_dequantize(p.data_ptr(), s.data_ptr(), deq.data_ptr(), rows, cols, fmt, st))
    fq = torch.empty_like(x)
    if fmt in (O.E4M3, O.E5M2):
        meta = torch.empty((rows, cols // 32), dtype=torch.int32, device="cuda")
        _cabi.check(L.mor_fake_quantize(x.data_ptr(), fq.data_ptr(), meta.data_ptr(), rows, cols, 1, 32, 0.0,
                                        2 if fmt == O.E4M3 else 3, 2, _cabi.FLAG_TORCH_EMULATION, st))
    else:
        _cabi.check(L.mor_block_format(x.data_ptr(), fq.data_ptr(), rows, cols, 1, 32, fmt, 2, _cabi.FLAG_TORCH_EMULATION, st))
    torch.cuda.synchronize()
    assert torch.equal(deq.view(torch.int16), fq.view(torch.int16))
    p2, s2 = quantize(deq)                                 # a block's amax may round down, so codes and scale can
    deq2 = torch.empty_like(x)                             # shift by a binade together; the decoded values cannot
    _cabi.check(L.mor_mx_dequantize(p2.data_ptr(), s2.data_ptr(), deq2.data_ptr(), rows, cols, fmt, st))
    torch.cuda.synchronize()
    assert torch.equal(deq2.view(torch.int16), deq.view(torch.int16))
    rp = torch.empty_like(p); rs = torch.empty_like(s); cp = torch.empty_like(p); cs = torch.empty_like(s)
    _cabi.check(L.mor_mx_quantize_dual(x.data_ptr(), rp.data_ptr(), rs.data_ptr(), cp.data_ptr(), cs.data_ptr(), rows, cols, fmt, st))
    tp, ts = quantize(x.t().contiguous())
    torch.cuda.synchronize()
    assert torch.equal(rp, p) and torch.equal(rs, s)
    assert torch.equal(cp, tp) and torch.equal(cs, ts)


def test_python_api_round_trip():
    from mor_amd import wire
    import mor
    x = data_gen.c2_student_t(256, 512, seed=31, as_tensor=True).cuda()
    for fmt, mode in ((wire.E4M3, 2), (wire.E5M2, 3)):
        p, s = wire.quantize_mx(x, fmt)
        mor.ops.set_flavour("torch_emulation")
        try:
            want = mor.ops.fake_quantize(x, 256, 512, 1, 32, 0.0, mode, 2)[0]
        finally:
            mor.ops.set_flavour("kernel")
        assert torch.equal(wire.dequantize_mx(p, s, fmt).view(torch.int16), want.view(torch.int16))
        rp, rs, cp, cs = wire.quantize_mx_dual(x, fmt)
        tp, ts = wire.quantize_mx(x.t().contiguous(), fmt)
        assert torch.equal(rp, p) and torch.equal(rs, s) and torch.equal(cp, tp) and torch.equal(cs, ts)
    with pytest.raises(RuntimeError):
        wire.quantize_mx(x[:, :48], wire.E4M3)
    p6, s6 = wire.quantize_mx(x, wire.E2M3)
    assert p6.shape == (256, 384) and wire.dequantize_mx(p6, s6, wire.E2M3).shape == (256, 512)


def test_hw_scaled_converts_selftest(G):
    """The gfx950 scaled converts of the wire-format kernels against the software codes / values: FP6 block convert
    (65 280 finite bf16 values x 253 scale exponents), its inverse and the FP8 decode (every code x 201 exponents)."""
    from mor_amd import _cabi
    L = _cabi.lib()
    bad = torch.full((4,), -1, dtype=torch.int64, device="cuda")
    _cabi.check(L.mor_selftest_hw_wire(bad.data_ptr(), None))
    torch.cuda.synchronize()
    assert bad.tolist() == [0, 0, 0, 0]


@pytest.mark.parametrize("fmt", [0, 1, 2, 3])
def test_scaled_mfma_consumes_the_wire_format(G, fmt):
    """Payload and scale bytes of mor_mx_quantize, loaded as they lie in memory, are the operands of the gfx950 scaled
    matrix instruction: its 16 x 16 x 128 product equals the product of the dequantized tensors (exact in float64: the
    operands are small dyadic numbers) up to the fp32 accumulation of 128 terms."""
    from mor_amd import _cabi
    L = _cabi.lib()
    rng = np.random.default_rng(40 + fmt)
    for trial in range(6):
        wide = trial % 2 == 0                # blocks with scales of their own (2^-20 .. 2^20) / one scale for all
        mats = []
        for _ in range(2):
            x = rng.standard_normal((16, 128)).astype(np.float32)
            if wide:
                x *= np.exp2(rng.integers(-20, 20, (16, 4))).repeat(32, axis=1).astype(np.float32)
            if trial == 3:
                x[3, 32:64] = 0                                                                     # an all-zero block
            mats.append(torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy())
        q = [G.mx_quantize(m, fmt) for m in mats]                    # (payload, scales) as numpy uint8
        deq = [E.bits_to_bf16(G.mx_dequantize(p, s, fmt)).double().numpy() for p, s in q]
        want = deq[0] @ deq[1].T
        bound = np.abs(deq[0]) @ np.abs(deq[1]).T
        dev = [[torch.from_numpy(np.ascontiguousarray(t)).to(G.dev()) for t in ps] for ps in q]
        out = torch.zeros((16, 16), dtype=torch.float32, device=G.dev())
        _cabi.check(L.mor_selftest_mx_mfma(dev[0][0].data_ptr(), dev[0][1].data_ptr(), dev[1][0].data_ptr(), dev[1][1].data_ptr(),
                                           fmt, out.data_ptr(), G.stream_ptr()))
        torch.cuda.synchronize()
        got = out.cpu().double().numpy()
        # the instruction aligns the products of a row to the largest before it adds them, so small ones lose bits
        # (measured, as a fraction of the sum of magnitudes: 3e-5 with scales 2^40 apart, 7e-6 with one scale, 4e-8 for
        # E3M2); a wrong layout would be wrong by the sum itself
        tol = 1e-4 if wide else 2e-5
        excess = np.max(np.abs(got - want) / (bound + 1e-300))
        print(f"scaled mfma fmt {fmt} trial {trial}: max |error| / sum of magnitudes {excess:.3e}", flush=True)
        assert excess <= tol, f"fmt {fmt} trial {trial}: {excess:.3e}"
