"""The five benchmark configurations at their full sizes: GPU (through the C ABI) against the CPU oracle, bit for bit.

The oracle is OpenMP-parallel and needs a few seconds per configuration at these sizes.  Besides equality, each case
checks properties that do not depend on the oracle: signs are kept, no magnitude exceeds the block amax by more than
one quantization step, and the format histogram of the MoR case matches the tile mixture it was generated from.
"""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
import data_gen

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def same(got, want, what):
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        raise AssertionError(f"{what}: {len(bad)} of {got.size} differ, first at {tuple(bad[0])}: "
                             f"got {got[tuple(bad[0])]:#06x} want {want[tuple(bad[0])]:#06x}")


def sign_and_bound_ok(a, out, br, bc, slack):
    """Outputs keep the input's sign; |out| <= block amax * (1 + slack).  Values below 2^-100 are left out of the sign
    check: a software-cast zero in a block whose amax exceeds the format maximum comes back as +2^(-e8-127)."""
    x = (a.astype(np.uint32) << 16).view(np.float32)
    y = (out.astype(np.uint32) << 16).view(np.float32)
    nz = (out & 0x7F80) > (27 << 7)
    assert np.array_equal((a & 0x8000)[nz], (out & 0x8000)[nz])
    rows, cols = a.shape
    amax = np.abs(x).reshape(rows // br, br, cols // bc, bc).max(axis=(1, 3), keepdims=True)
    assert np.all(np.abs(y).reshape(rows // br, br, cols // bc, bc) <= amax * (1 + slack) + 1e-37)


def test_c1_per_tensor_e4m3_4096(G):
    a = data_gen.c1_normal()
    x = (a.astype(np.uint32) << 16).view(np.float32)
    scale = float(np.float32(448.0) / np.float32(np.abs(x).max()))
    print("C1", a.shape, scale, flush=True)
    out, meta = G.fake_quantize(a, 128, 128, scale, 4, 1)
    want, wmeta = O.fake_quantize(a, 128, 128, scale, 4, 1)
    assert (meta == 1).all() and np.array_equal(meta, wmeta)
    same(out, want, "C1")
    # the on-GPU amax variant of the same configuration: block scaling with ss_mode 4
    out2, m2, gamax, gnnz, gerr = G.block_scaling(a, 128, 128, 1.0, 4)
    w2, wm2, wamax, wnnz, werr = O.block_scaling(a, 128, 128, 1.0, 4)
    assert gamax[0] == wamax[0] == np.abs(x).max() and gnnz[0] == wnnz[0] == np.count_nonzero(a & 0x7FFF)
    np.testing.assert_allclose(gerr[0], werr[0], rtol=1e-6)
    assert m2[0] == wm2[0] == 1
    same(out2, w2, "C1 block_scaling ss4")
    # with a correct tensor scale both routes give the same tensor except for the sign of zero
    assert np.array_equal(out2 & 0x7FFF, out & 0x7FFF)


@pytest.mark.parametrize("name,fmt", [("e4m3", O.E4M3), ("e5m2", O.E5M2), ("e2m3", O.E2M3)])
def test_c2_mx_8192(G, name, fmt):
    a = data_gen.c2_student_t()
    print("C2", name, a.shape, flush=True)
    if fmt == O.E2M3:
        out = G.block_format(a, 1, 32, fmt, 2)
        want = O.block_format(a, 1, 32, fmt, 2)
    else:
        mode = 2 if fmt == O.E4M3 else 3
        out, meta = G.fake_quantize(a, 1, 32, 0.0, mode, 2)
        want, wmeta = O.fake_quantize(a, 1, 32, 0.0, mode, 2)
        assert np.array_equal(meta, wmeta) and meta.shape == (8192, 256)
    same(out, want, f"C2 {name}")
    amax, scale, e8 = G.block_stats(a, 1, 32, O.FMAX[fmt])
    wa, ws, we = O.block_stats(a, 1, 32, O.FMAX[fmt])
    assert np.array_equal(amax, wa) and np.array_equal(scale.view(np.uint32), ws.view(np.uint32)) and np.array_equal(e8, we)
    step = {O.E4M3: 2.0 ** -3, O.E5M2: 2.0 ** -2, O.E2M3: 2.0 ** -3}[fmt]
    sign_and_bound_ok(a, out, 1, 32, step)


@pytest.mark.parametrize("mode", [2, 3])
def test_c3_per_row_16384x4096(G, mode):
    a = data_gen.c3_weights()
    assert not a[7].any()
    print("C3", mode, a.shape, flush=True)
    out, meta = G.fake_quantize(a, 1, 4096, 0.0, mode, 1)
    want, wmeta = O.fake_quantize(a, 1, 4096, 0.0, mode, 1)
    assert np.array_equal(meta, wmeta)
    same(out, want, f"C3 mode {mode}")
    assert not out[7].any()                                   # the all-zero row passes through
    if mode == 2:
        o2, m2, gamax, gnnz, gerr = G.block_scaling(a, 1, 4096, 0.045, 3, channel=True)
        w2, wm2, wamax, wnnz, werr = O.block_scaling(a, 1, 4096, 0.045, 3, channel=True)
        assert gamax[0] == wamax[0] and gnnz[0] == wnnz[0] and m2[0] == wm2[0]
        np.testing.assert_allclose(gerr[0], werr[0], rtol=1e-6)
        same(o2, w2, "C3 channel scaling")


def test_c4_mor_16384x14336(G):
    a = data_gen.c4_mixture()
    print("C4", a.shape, flush=True)
    out, meta = G.fake_quantize(a, 128, 128, 1e-15, 1, 1)
    want, wmeta, stats = O.fake_quantize(a, 128, 128, 1e-15, 1, 1, want_stats=True)
    flip = meta != wmeta
    print("C4 format decisions that differ from the oracle's:", int(flip.sum()), "of", meta.size, flush=True)
    assert not flip.any(), (int(flip.sum()), stats[..., 2][flip], stats[..., 3][flip])     # no change in format choice
    same(out, want, "C4")
    hist = np.bincount(meta.ravel(), minlength=5)
    n = meta.size
    assert hist[1] + hist[3] + hist[4] == n                  # error mode never returns E5M2
    assert 0.15 * n < hist[3] < 0.30 * n                     # the log-normal tiles (20 %) and a few lost E4M3 votes
    st = G.mor_stats(a, 128, 128, 1e-15, 1, 1)
    assert np.array_equal(st[..., :2], stats[..., :2])
    np.testing.assert_allclose(st[..., 2:], stats[..., 2:], rtol=1e-6, atol=0)
    # the same decisions and values through the tile codes and their decode, and through a batch call
    import mor_amd
    x = G.to_dev_u16(a)
    payload, tags, scales = mor_amd.wire.quantize_mor_tiles(x, 1e-15, 1)
    assert np.array_equal((tags & 0xFF).cpu().numpy(), wmeta), "C4 tile codes: tags"
    same(G.to_host_u16(mor_amd.wire.dequantize_mor_tiles(payload, tags, scales)), want, "C4 tile codes decoded")
    del payload
    (bout, bmeta), = mor_amd.batch.fake_quantize_batch([x], [(128, 128)], 1e-15, 1, 1)
    assert np.array_equal(bmeta.cpu().numpy(), wmeta), "C4 batch call: meta"
    same(G.to_host_u16(bout), want, "C4 batch call")


C5_SHAPES = [
    # (rows, cols) of the tensors quantized around one Llama-3-8B layer at 16384 tokens
    (16384, 4096), (16384, 14336), (4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (16384, 1024),
]


@pytest.mark.parametrize("shape", C5_SHAPES)
def test_c5_layer_sweep(G, shape):
    rows, cols = shape
    weight = rows in (4096, 1024, 14336) and (rows, cols) != (16384, 1024)
    g = torch.Generator().manual_seed(1005 + rows + cols)
    t = torch.randn(rows, cols, generator=g) * (0.02 if weight else 1.0)
    a = t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()
    del t
    print("C5", shape, flush=True)
    out, meta = G.fake_quantize(a, 128, 128, 1e-15, 1, 1)                       # MoR
    want, wmeta, stats = O.fake_quantize(a, 128, 128, 1e-15, 1, 1, want_stats=True)
    flip = meta != wmeta
    print("C5", shape, "format decisions that differ from the oracle's:", int(flip.sum()), "of", meta.size, flush=True)
    assert not flip.any(), (int(flip.sum()), stats[..., 2][flip], stats[..., 3][flip])     # no change in format choice
    same(out, want, f"C5 MoR {shape}")
    for mode in (2, 3):                                                          # block 128x128
        out, meta = G.fake_quantize(a, 128, 128, 0.0, mode, 1)
        want, wmeta = O.fake_quantize(a, 128, 128, 0.0, mode, 1)
        assert np.array_equal(meta, wmeta)
        same(out, want, f"C5 block mode {mode} {shape}")
    for (br, bc) in ((1, cols), (rows, 1)):                                      # per-channel rows (dgrad) and columns (wgrad)
        o2, m2, gamax, gnnz, gerr = G.block_scaling(a, br, bc, 0.045, 3, channel=True)
        w2, wm2, wamax, wnnz, werr = O.block_scaling(a, br, bc, 0.045, 3, channel=True)
        assert gamax[0] == wamax[0] and gnnz[0] == wnnz[0] and m2[0] == wm2[0]
        np.testing.assert_allclose(gerr[0], werr[0], rtol=1e-6)
        same(o2, w2, f"C5 channel {br}x{bc} {shape}")


def test_c5_ragged_and_tiny(G):
    g = torch.Generator().manual_seed(1005)
    t = torch.randn(4097, 4095, generator=g)
    a = t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()
    print("C5 ragged", a.shape, flush=True)
    for mode, sf in ((1, 1), (2, 1), (3, 2)):
        out, meta = G.fake_quantize(a, 128, 128, 1e-15, mode, sf)
        want, wmeta = O.fake_quantize(a, 128, 128, 1e-15, mode, sf)
        assert meta.shape == (33, 32) and np.array_equal(meta, wmeta)
        same(out, want, f"ragged mode {mode}")
    one = torch.randn(1, 32, generator=g).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()
    for mode, sf in ((1, 1), (2, 2), (3, 1)):
        out, meta = G.fake_quantize(one, 1, 32, 1e-15, mode, sf)
        want, wmeta = O.fake_quantize(one, 1, 32, 1e-15, mode, sf)
        assert np.array_equal(meta, wmeta)
        same(out, want, f"1x32 mode {mode}")
