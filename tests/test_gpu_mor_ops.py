"""The reference's own test logic (test/test_fake_quantize*.py, test/test_e8mx.py) restated against `mor.ops` on the GPU.

Each case builds the reference's input, calls the public op exactly as the reference test does (same keyword names)
and makes the reference's assertions; the expected tensors come from tests/torch_emulation.py.  Random inputs are
seeded here (the reference's are not, its seeding method is never called).  Where the CUDA kernel and the torch
emulation can differ (round-half-up vs nearest-even on exact ties) the comparison is also made in the
'torch_emulation' flavour, where it must be exact.
"""
import numpy as np
import pytest
import torch

import torch_emulation as E

pytestmark = pytest.mark.gpu

POKES_RANGE = [(128, 1, 18200, 50968), (0, 70, 21000, 53768), (1, 1, 17262, 50030)]
POKES_ERROR = [(128, 1, 18403, 51171), (0, 70, 21000, 53768), (1, 1, 17264, 50032)]


@pytest.fixture(scope="module")
def mor():
    import mor
    assert torch.cuda.is_available()
    yield mor
    mor.ops.set_flavour("kernel")


def fixture_bf16(pokes=()):
    return E.bits_to_bf16(E.fixture_words(256, 256, pokes))


def random_bf16(seed, lo, hi, rows=256, cols=256):
    g = torch.Generator().manual_seed(seed)
    return torch.empty(rows, cols).uniform_(lo, hi, generator=g).to(torch.bfloat16)


def bits(t):
    return E.bf16_to_bits(t.cpu())


def test_uint32_matrix_large_block_dynamic_range(mor):
    m = fixture_bf16(POKES_RANGE)
    out, meta = mor.ops.fake_quantize(m.to("cuda"), 256, 256, 128, 128, clamp_threshold=1e-15, mode=101, sf_type=1)
    assert meta.cpu().tolist() == [[1, 3], [2, 4]]
    want, _ = E.mor_tensor(bits(m), 128, 128, True)
    assert out.cpu().equal(E.bits_to_bf16(want))


def test_uint32_matrix_large_block(mor):
    m = fixture_bf16(POKES_ERROR)
    out, meta = mor.ops.fake_quantize(m.to("cuda"), 256, 256, 128, 128, clamp_threshold=1e-15, mode=1, sf_type=1)
    assert meta.cpu().tolist() == [[1, 3], [3, 4]]
    want, _ = E.mor_tensor(bits(m), 128, 128, False)
    assert out.cpu().equal(E.bits_to_bf16(want))


def test_uint32_matrix_large_block_dynamic_range_e8_scaling(mor):
    m = fixture_bf16(POKES_RANGE)
    out, meta = mor.ops.fake_quantize(m.to("cuda"), 256, 256, 128, 128, clamp_threshold=1e-25, mode=101, sf_type=2)
    assert meta.cpu().tolist() == [[1, 3], [2, 4]]
    want, _ = E.mor_tensor(bits(m), 128, 128, True, e8=True)
    assert out.cpu().equal(E.bits_to_bf16(want))


@pytest.mark.parametrize("seed,mode,sf", [(1, 101, 1), (2, 1, 1), (3, 101, 2)])
def test_random_matrix_large_block(mor, seed, mode, sf):
    m = random_bf16(seed, -53768.0, 53768.0)
    want, _ = E.mor_tensor(bits(m), 128, 128, mode == 101, e8=(sf == 2))
    mor.ops.set_flavour("torch_emulation")
    out, _ = mor.ops.fake_quantize(m.to("cuda"), 256, 256, 128, 128, clamp_threshold=1e-15 if sf == 1 else 1e-25, mode=mode, sf_type=sf)
    mor.ops.set_flavour("kernel")
    assert out.cpu().equal(E.bits_to_bf16(want))
    out_k, _ = mor.ops.fake_quantize(m.to("cuda"), 256, 256, 128, 128, clamp_threshold=1e-15 if sf == 1 else 1e-25, mode=mode, sf_type=sf)
    assert (bits(out_k) != want).mean() < 0.02


@pytest.mark.parametrize("mode,fmt,fmax", [(4, "e4m3", 448.0), (5, "e5m2", 57344.0)])
def test_random_matrix_large_block_current_scaling(mor, mode, fmt, fmax):
    m = random_bf16(10 + mode, -53768.0, 53768.0)
    x = m.to("cuda")
    amax = torch.max(torch.abs(x)).float()
    scaling_factor = fmax / amax                      # a 0-dim GPU tensor, as in the reference test
    mor.ops.set_flavour("torch_emulation")
    out, _ = mor.ops.fake_quantize(x, 256, 256, 128, 128, clamp_threshold=scaling_factor, mode=mode, sf_type=1)
    mor.ops.set_flavour("kernel")
    # the emulation divides by the Python-double scale; use the same fp32 scale the op received
    s = float(scaling_factor)
    want = ((m.float() * s).to(E.FP8[fmt][0]).float() / s).to(torch.bfloat16)
    assert out.cpu().equal(want)


def test_random_matrix_bf16_block(mor):
    x = random_bf16(20, -53768.0, 53768.0).to("cuda")
    out, meta = mor.ops.fake_quantize(x, 256, 256, 128, 128, clamp_threshold=1e-15, mode=7, sf_type=1)
    assert (meta.cpu() == 3).all() and x.equal(out)


def test_no_alloc_and_inplace(mor):
    m = fixture_bf16(POKES_RANGE[:2])
    x = m.to("cuda")
    output = torch.zeros(256, 256, dtype=torch.bfloat16, device="cuda")
    meta_na = mor.ops.fake_quantize_no_alloc(x, 256, 256, 128, 128, clamp_threshold=1e-15, mode=1, sf_type=1, output=output)
    out, meta = mor.ops.fake_quantize(x, 256, 256, 128, 128, clamp_threshold=1e-15, mode=1, sf_type=1)
    assert meta_na.equal(meta) and output.equal(out)
    meta_ip = mor.ops.fake_quantize_no_alloc(x, 256, 256, 128, 128, clamp_threshold=1e-15, mode=1, sf_type=1, output=x)
    assert meta_ip.equal(meta) and x.equal(out)


def test_zero_and_small_value_blocks(mor):
    z = torch.zeros(256, 256, dtype=torch.bfloat16, device="cuda")
    out, meta = mor.ops.fake_quantize(z, 256, 256, 128, 128, clamp_threshold=1e-25, mode=101, sf_type=2)
    assert (meta.cpu() == 4).all() and out.equal(z)
    t = (torch.ones(256, 256, dtype=torch.bfloat16) * 1e-27)
    out, meta = mor.ops.fake_quantize(t.to("cuda"), 256, 256, 128, 128, clamp_threshold=1e-25, mode=101, sf_type=2)
    assert (meta.cpu() == 4).all()
    want, _ = E.mor_tensor(bits(t), 128, 128, True, e8=True)
    assert out.cpu().equal(E.bits_to_bf16(want))


def test_quant_dequant_ops(mor):
    g = torch.Generator().manual_seed(30)
    x = torch.empty(256, 256).uniform_(-400.0, 400.0, generator=g)
    assert mor.ops.quant_dequant_e4m3(x.to("cuda"), 256, 256, 128, 128).cpu().equal(x.to(torch.float8_e4m3fn).float())
    x = torch.empty(256, 256).uniform_(-1.0, 1.0, generator=g)
    assert mor.ops.quant_dequant_e4m3(x.to("cuda"), 256, 256, 128, 128).cpu().equal(x.to(torch.float8_e4m3fn).float())
    x = torch.empty(256, 256).uniform_(-1000.0, 1000.0, generator=g)
    x[0, 0], x[0, 1], x[0, 2] = 463, 464, 465
    got = mor.ops.quant_dequant_e4m3(x.to("cuda"), 256, 256, 128, 128).cpu()
    ref = x.to(torch.float8_e4m3fn).float()
    assert torch.isnan(got).equal(torch.isnan(ref)) and got[~torch.isnan(ref)].equal(ref[~torch.isnan(ref)])
    x = torch.empty(256, 256).uniform_(-53768.0, 53768.0, generator=g)
    assert mor.ops.quant_dequant_e5m2(x.to("cuda"), 256, 256, 128, 128).cpu().equal(x.to(torch.float8_e5m2).float())
    x = torch.empty(256, 256).uniform_(0.25, 100.0, generator=g)
    assert mor.ops.quant_dequant_e3m2(x.to("cuda"), 256, 256, 128, 128).cpu().equal(x.to(torch.float8_e5m2).float().clamp(-28, 28))
    x = torch.empty(256, 256).uniform_(1.0, 20.0, generator=g)
    assert mor.ops.quant_dequant_e2m3(x.to("cuda"), 256, 256, 128, 128).cpu().equal(x.to(torch.float8_e4m3fn).float().clamp(-7.5, 7.5))


def test_e4m3_with_e8_scale_rz(mor):
    g = torch.Generator().manual_seed(31)
    x = torch.empty(256, 256).uniform_(-1000, 1000, generator=g)
    a = x.abs()
    p = 2 ** torch.floor(torch.log2(448.0 / a))
    want = (x * p).to(torch.float8_e4m3fn).float() / p
    assert mor.ops.e4m3_with_e8_scale_rz(x.to("cuda"), 256, 256, 128, 128).cpu().equal(want)


@pytest.mark.parametrize("bx,by,channel", [(128, 128, False), (1, 256, True), (256, 1, True)])
def test_scaling_ops_fixture(mor, bx, by, channel):
    op = mor.ops.fake_quantize_channel_scaling if channel else mor.ops.fake_quantize_block_scaling
    m = fixture_bf16()
    x = m.to("cuda")
    out, meta, gamax, gnnz, gerr = op(x, 256, 256, bx, by, e4m3_threshold=0.045, ss_mode=1)
    want, total, amax, nnz = E.block_scaling_tensor(bits(m), bx, by)
    assert meta.item() == 1 and gamax.item() == amax and gnnz.item() == nnz
    torch.testing.assert_close(torch.tensor(total, dtype=torch.float32), gerr[0].cpu(), rtol=1e-3, atol=0)
    assert out.cpu().equal(E.bits_to_bf16(want))
    m2 = fixture_bf16([(0, 70, 21000, 53768)])
    out, meta, gamax, gnnz, gerr = op(m2.to("cuda"), 256, 256, bx, by, e4m3_threshold=0.045, ss_mode=1)
    if not channel:
        assert meta.item() == 3
    assert out.cpu().equal(m2 if meta.item() == 3 else out.cpu())


@pytest.mark.parametrize("bx,by,channel", [(128, 128, False), (1, 256, True), (256, 1, True)])
@pytest.mark.parametrize("lo,hi", [(-448.0, 448.0), (-53768.0, 53768.0)])
def test_scaling_ops_random_and_inplace(mor, bx, by, channel, lo, hi):
    op = mor.ops.fake_quantize_channel_scaling if channel else mor.ops.fake_quantize_block_scaling
    op_ip = mor.ops.fake_quantize_channel_scaling_inplace if channel else mor.ops.fake_quantize_block_scaling_inplace
    m = random_bf16(40, lo, hi)
    want, total, amax, nnz = E.block_scaling_tensor(bits(m), bx, by)
    mor.ops.set_flavour("torch_emulation")
    out, meta, gamax, gnnz, gerr = op(m.to("cuda"), 256, 256, bx, by, e4m3_threshold=0.045, ss_mode=1)
    x = m.to("cuda")
    meta2, gamax2, gnnz2, gerr2 = op_ip(x, 256, 256, bx, by, 0.045, ss_mode=1)
    mor.ops.set_flavour("kernel")
    assert meta.item() == (3 if gerr.item() / gnnz.item() > 0.045 else 1)
    assert gamax.item() == amax and gnnz.item() == nnz
    torch.testing.assert_close(torch.tensor(total, dtype=torch.float32), gerr[0].cpu(), rtol=1e-2, atol=0)
    expect = E.bits_to_bf16(want) if meta.item() == 1 else m
    assert out.cpu().equal(expect)
    assert meta2.item() == meta.item() and gerr2.item() == gerr.item() and x.cpu().equal(expect)


@pytest.mark.parametrize("qt", [1, 2, 3])
def test_e8mx_ops(mor, qt):
    m = E.bits_to_bf16(E.fixture_words(64, 64, [(0, 30, 21000, 53768)]))
    want = E.bits_to_bf16(E.e8mx_tensor(bits(m), qt))
    x = m.to("cuda")
    out = mor.ops.fake_quantize_e8mx(x, 64, 64, 32, 32, quantize_type=qt, scaling_strategy=3)
    assert out.cpu().equal(want)
    mor.ops.fake_quantize_e8mx_inplace(x, 64, 64, 32, 32, qt, 3, x)
    assert x.cpu().equal(want)
    y = m.to("cuda")
    out_g = mor.ops.fake_quantize_e8mx(y, 64, 64, 32, 32, quantize_type=qt, scaling_strategy=1)
    mor.ops.fake_quantize_e8mx_inplace(y, 64, 64, 32, 32, qt, 1, y)
    assert y.equal(out_g)                                  # test_e8mx.py:406-440


def test_errors_and_autograd(mor):
    x = torch.zeros(256, 256, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError):
        mor.ops.fake_quantize(x, 256, 256, 128, 128, 1e-15, 1, 1)                       # dtype
    b = torch.zeros(256, 256, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError):
        mor.ops.fake_quantize(b, 128, 256, 128, 128, 1e-15, 1, 1)                       # size mismatch
    with pytest.raises(RuntimeError):
        mor.ops.fake_quantize_block_scaling(b, 256, 256, 100, 128, 0.045, 1)            # indivisible
    with pytest.raises(RuntimeError):
        mor.ops.quant_dequant_e4m3(b, 256, 256, 128, 128)                               # needs fp32
    # straight-through estimator: the gradient passes unchanged
    w = torch.randn(256, 256, device="cuda").to(torch.bfloat16).requires_grad_(True)
    out = mor.ops.fake_quantize_e8mx(w, 256, 256, 128, 128, 3, 3)
    out.float().sum().backward()
    assert w.grad is not None and torch.all(w.grad == 1)
    # a non-contiguous input is accepted (FQ:1845)
    t = torch.randn(256, 512, device="cuda").to(torch.bfloat16)[:, ::2]
    o1, _ = mor.ops.fake_quantize(t, 256, 256, 128, 128, 1e-15, 1, 1)
    o2, _ = mor.ops.fake_quantize(t.contiguous(), 256, 256, 128, 128, 1e-15, 1, 1)
    assert o1.equal(o2)


def test_ops_replay_in_a_hip_graph(mor):
    """The library allocates nothing and clears its workspace with kernels, so the ops can be captured: every replay,
    with eager work and synchronizations between replays and fresh input each time, equals the eager result."""
    x = torch.empty(512, 1024, dtype=torch.bfloat16, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(7)

    def body(t):
        o1, m1 = mor.ops.fake_quantize(t, 512, 1024, 128, 128, clamp_threshold=1e-15, mode=1, sf_type=1)
        o2, m2 = mor.ops.fake_quantize(t, 512, 1024, 1, 32, clamp_threshold=0.0, mode=2, sf_type=2)
        r = mor.ops.fake_quantize_channel_scaling(t, 512, 1024, 512, 1, e4m3_threshold=0.045, ss_mode=1)
        e = mor.ops.fake_quantize_e8mx(t, 512, 1024, 128, 128, quantize_type=2, scaling_strategy=1)
        return [o1, m1, o2, m2, e] + list(r)

    x.copy_(torch.randn(512, 1024, device="cuda", generator=g))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        body(x)                                            # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = body(x)
    for rep in range(4):
        x.copy_(torch.randn(512, 1024, device="cuda", generator=g) * (10.0 ** rep))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = body(x)                                     # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), rep


def test_ops_trace_under_torch_compile(mor):
    """aot_eager traces forward and backward through the fake kernels and the straight-through autograd."""
    def f(t):
        q = mor.ops.fake_quantize(t * 1.0, 256, 512, 128, 128, 1e-15, 1, 1)[0]
        return mor.ops.fake_quantize_e8mx(q, 256, 512, 128, 128, 3, 1).float().sum()

    w = torch.randn(256, 512, device="cuda").to(torch.bfloat16).requires_grad_(True)
    want = f(w)
    want.backward()
    g_eager = w.grad.clone()
    w.grad = None
    got = torch.compile(f, backend="aot_eager", fullgraph=True)(w)
    got.backward()
    assert torch.equal(got, want) and torch.equal(w.grad, g_eager) and torch.all(g_eager == 1)


def test_inplace_ops_under_torch_compile_run_eagerly_and_write(mor):
    """The ops that write into an argument are excluded from compilation (their schemas declare no aliasing): a compiled
    function that calls them breaks the graph there, the writes happen, and the values equal the eager ones."""
    def f(t, buf):
        y = t * 1.0
        mor.ops.fake_quantize_e8mx_inplace(y, 256, 512, 128, 128, 2, 1, y)
        meta = mor.ops.fake_quantize_no_alloc(y, 256, 512, 1, 32, 0.0, 2, 2, buf)
        stats = mor.ops.fake_quantize_block_scaling_inplace(buf, 256, 512, 128, 128, 0.045, 3)
        return y + 0.0, meta, stats[0]

    x = random_bf16(77, -8.0, 8.0, 256, 512).cuda()
    b1, b2 = torch.zeros_like(x), torch.zeros_like(x)
    want = f(x, b1)
    got = torch.compile(f, backend="aot_eager")(x, b2)
    torch.cuda.synchronize()
    assert torch.equal(b1, b2) and b1.abs().sum() > 0
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    e = mor.ops.fake_quantize_e8mx(x, 256, 512, 128, 128, 2, 1)
    assert torch.equal(want[0], e)


def test_flavour_is_per_thread(mor):
    """set_flavour applies to the calling thread only."""
    import threading
    # blocks of 1 x 32 with amax 1000 and a power-of-two scale: 1e-3 casts to zero, which the CUDA kernel's exponent
    # arithmetic returns as 2^(2-127) and the torch emulation as 0
    x = torch.zeros(256, 256)
    x[:, 0], x[:, 1] = 1000.0, 1e-3
    x = x.to(torch.bfloat16).cuda()
    args = (x, 256, 256, 1, 32, 0.0, 2, 2)
    base = mor.ops.fake_quantize(*args)[0]
    mor.ops.set_flavour("torch_emulation")
    emu_here = mor.ops.fake_quantize(*args)[0]
    mor.ops.set_flavour("kernel")
    assert base[0, 1].item() > 0 and emu_here[0, 1].item() == 0
    res = {}

    def other():
        mor.ops.set_flavour("torch_emulation")
        res["emu"] = mor.ops.fake_quantize(*args)[0]
        torch.cuda.synchronize()

    t = threading.Thread(target=other)
    t.start()
    t.join()
    again = mor.ops.fake_quantize(*args)[0]
    assert torch.equal(base, again)
    assert torch.equal(emu_here, res["emu"])


def test_concurrent_streams_and_host_threads(mor):
    """The library keeps no state between calls: four host threads, each on its own stream with its own tensors,
    interleave different ops and get what a single-threaded run gets."""
    import threading
    xs = [random_bf16(100 + i, -8.0, 8.0, 512, 1024).cuda() for i in range(4)]

    def work(x):
        a = mor.ops.fake_quantize(x, 512, 1024, 128, 128, clamp_threshold=1e-15, mode=1, sf_type=1)
        b = mor.ops.fake_quantize(x, 512, 1024, 1, 32, clamp_threshold=0.0, mode=2, sf_type=2)
        c = mor.ops.fake_quantize_block_scaling(x, 512, 1024, 128, 128, e4m3_threshold=0.045, ss_mode=1)
        d = mor.ops.fake_quantize_channel_scaling(x, 512, 1024, 1, 1024, e4m3_threshold=0.045, ss_mode=3)
        e = mor.ops.fake_quantize_e8mx(x, 512, 1024, 128, 128, quantize_type=2, scaling_strategy=1)
        return list(a) + list(b) + list(c) + list(d) + [e]

    want = [work(x) for x in xs]
    torch.cuda.synchronize()
    got = [None] * 4
    errors = []

    def run(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for _ in range(20):
                    got[i] = work(xs[i])
            s.synchronize()
        except Exception as exc:                      # surfaced below
            errors.append(exc)

    threads = [threading.Thread(target=run, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(4):
        for a, b in zip(got[i], want[i]):
            assert torch.equal(a, b), i
