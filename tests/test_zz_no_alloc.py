"""mor_block_scaling_static (the entry point that allocates nothing: its workspace is a static device array inside
the library) against mor_block_scaling on the same inputs, through the C ABI.

Two calls in a row share the array, the second on a smaller input, so stale contents of the first call would show;
every strategy and geometry of the op is covered, out of place and in place, and the size limit is checked."""
import numpy as np
import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(300)]


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def make(seed, rows, cols):
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(rows, cols, generator=g) * torch.exp(1.5 * torch.randn(rows, cols, generator=g))
    t = torch.where(torch.rand(rows, cols, generator=g) < 0.02, torch.zeros(()), t)
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()


def static_call(G, a, br, bc, thr, ss, channel, inplace=False):
    from mor_amd import _cabi
    L = _cabi.lib()
    rows, cols = a.shape
    x = G.to_dev_u16(a)
    out = x if inplace else torch.full_like(x, 7.0)
    meta = torch.full((1,), -7, dtype=torch.int32, device=G.dev())
    gamax = torch.zeros(1, dtype=torch.float32, device=G.dev())
    gnnz = torch.zeros(1, dtype=torch.int32, device=G.dev())
    gerr = torch.zeros(1, dtype=torch.float32, device=G.dev())
    torch.cuda.synchronize()
    # torch's allocator counts torch's own allocations only; the free bytes of the device (hipMemGetInfo) would also
    # show a hipMalloc made inside the library.  The first call on a device loads the code object with its static
    # array, so the device-level comparison starts with the second.
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    rc = L.mor_block_scaling_static(x.data_ptr(), out.data_ptr(), meta.data_ptr(), gamax.data_ptr(), gnnz.data_ptr(),
                                    gerr.data_ptr(), rows, cols, br, bc, float(thr), ss, int(channel), 0, G.stream_ptr())
    _cabi.check(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    if static_call.warm:
        assert torch.cuda.mem_get_info()[0] == free_before, "the device's free memory changed during the call"
    static_call.warm = True
    return G.to_host_u16(out), meta.cpu().numpy(), gamax.cpu().numpy(), gnnz.cpu().numpy(), gerr.cpu().numpy()


static_call.warm = False


def same(got, want, what):
    for g, w, name in zip(got, want, ("out", "meta", "amax", "nnz", "err")):
        assert np.array_equal(g.view(np.uint32) if g.dtype == np.float32 else g, w.view(np.uint32) if w.dtype == np.float32 else w), (what, name, g[:4] if g.ndim == 1 else None, w[:4] if w.ndim == 1 else None)


CASES = [
    # (block_rows, block_cols, channel, big shape, small shape)
    (128, 128, False, (1024, 2048), (256, 384)),
    (1, 32, True, (512, 4096), (64, 96)),
    (1, 2048, True, (768, 4096), (96, 2048)),
    (64, 1, True, (1024, 1536), (128, 200)),
    (1024, 1, True, (1024, 1536), (1024, 64)),
    (16, 16, False, (512, 768), (48, 32)),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "b%dx%d" % (c[0], c[1]))
@pytest.mark.parametrize("ss", [1, 2, 3, 4])
def test_static_scratch_equals_workspace_entry(G, case, ss):
    br, bc, channel, big, small = case
    for i, (rows, cols) in enumerate((big, small)):          # the second call on the smaller input reuses the array
        a = make(900 + 10 * ss + i, rows, cols)
        print("no-alloc", case, ss, rows, cols, flush=True)
        for thr in (0.02, 0.2):
            for inplace in (False, True):
                want = G.block_scaling(a, br, bc, thr, ss, channel=channel, inplace=inplace)
                got = static_call(G, a, br, bc, thr, ss, channel, inplace=inplace)
                same(got, want, (case, ss, rows, cols, thr, inplace))


def test_static_scratch_refuses_too_many_blocks(G):
    from mor_amd import _cabi
    L = _cabi.lib()
    x = torch.zeros(2048, 32 * 1024 // 2, dtype=torch.bfloat16, device=G.dev())          # 2^25 elements
    s = torch.zeros(4, dtype=torch.int32, device=G.dev())
    rows, cols = x.shape
    rc = L.mor_block_scaling_static(x.data_ptr(), x.data_ptr(), s.data_ptr(), s.data_ptr(), s.data_ptr(), s.data_ptr(),
                                    rows, cols, 1, 16, 0.045, 3, 1, 0, G.stream_ptr())      # 2^21 blocks
    assert rc == -2 and b"at most" in L.mor_last_error()
    rc = L.mor_block_scaling_static(x.data_ptr(), x.data_ptr(), s.data_ptr(), s.data_ptr(), s.data_ptr(), s.data_ptr(),
                                    rows, cols, 1, 32, 0.045, 3, 1, 0, G.stream_ptr())      # 2^20 blocks: the limit itself
    assert rc == 0
    torch.cuda.synchronize()
