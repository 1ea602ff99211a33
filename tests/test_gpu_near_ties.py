"""MoR decisions on blocks whose two error sums meet (GPU against the CPU oracle).

The reference decides e4 <= e5 on two fp32 sums added in the order of its thread layout
(/root/reference/mor/csrc/cuda/fake_quantize.cu:491-583, 661).  The blocks here are constructed so that the sums agree
to a few units in the last place (near_ties.mine_block), where any other order of the additions takes the other
decision for about half of them.  The HIP kernels must return the reference's decision for every one of them, and
their error sums must be the oracle's bit for bit."""
import numpy as np
import pytest
import torch

from mor_amd import _cabi
from oracle import mor_oracle as O
import near_ties as NT

pytestmark = pytest.mark.gpu

CLAMP = 1e-15


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def bits_equal(a, b):
    return np.array_equal(np.asarray(a, np.float32).view(np.uint32), np.asarray(b, np.float32).view(np.uint32))


def check_tensor(G, t, bh, bw, sf, flags=0, flavour=O.KERNEL, min_close=0):
    want, wmeta, wst = O.fake_quantize(t, bh, bw, CLAMP, 1, sf, flavour, want_stats=True)
    e4, e5 = wst[..., 2], wst[..., 3]
    close = (np.maximum(e4, e5) > 0) & (np.abs(e4 - e5) <= 1e-6 * np.maximum(e4, e5))
    assert close.sum() >= min_close, f"only {close.sum()} blocks with sums within 1e-6"
    out, meta = G.fake_quantize(t, bh, bw, CLAMP, 1, sf, flags)
    flips = int((meta != wmeta).sum())
    assert flips == 0, f"{flips} of {meta.size} decisions differ from the reference's"
    assert np.array_equal(out, want)
    if flavour == O.KERNEL:
        st = G.mor_stats(t, bh, bw, CLAMP, 1, sf, flags)
        # sums within 1e-5 of each other are recomputed in the reference's order: the oracle's bits
        assert bits_equal(st[..., 2][close], e4[close]) and bits_equal(st[..., 3][close], e5[close])
        assert bits_equal(st[..., 0], wst[..., 0]) and bits_equal(st[..., 1], wst[..., 1])
    return int(close.sum()), np.unique(wmeta, return_counts=True)


@pytest.mark.parametrize("sf", [1, 2])
def test_256_tiles_whose_sums_meet(G, sf):
    """the headline block shape: 256 tiles of 128 x 128, each within 1e-6 (most within 2 ulp), both decisions present"""
    t = NT.mine_tensor(100 + sf, 16, 16, 128, 128, sf)
    print("near ties 128x128 sf", sf, flush=True)
    n, (vals, counts) = check_tensor(G, t, 128, 128, sf, min_close=200)
    print("  blocks within 1e-6:", n, "decisions", dict(zip(vals.tolist(), counts.tolist())), flush=True)
    assert set(vals.tolist()) == {1, 3} and counts.min() >= 20


# block shape -> the kernel it reaches (aligned tensors, default flavour): lane groups with the workgroup fallback,
# register-resident blocks of 2 / 16 vectors per lane, the block that is swept from memory
@pytest.mark.parametrize("bh,bw,gy,gx", [(32, 32, 12, 12), (64, 64, 8, 8), (32, 128, 8, 4), (256, 256, 3, 3), (512, 512, 1, 2)])
@pytest.mark.parametrize("sf", [1, 2])
def test_other_block_shapes(G, bh, bw, gy, gx, sf):
    t = NT.mine_tensor(bh * 7 + bw + sf, gy, gx, bh, bw, sf)
    print("near ties", bh, bw, "sf", sf, flush=True)
    n, _ = check_tensor(G, t, bh, bw, sf, min_close=(gy * gx * 3) // 4)
    print("  blocks within 1e-6:", n, flush=True)


@pytest.mark.parametrize("sf", [1, 2])
def test_rows_that_are_not_vectors(G, sf):
    """128 x 128 blocks on a tensor whose width is not a multiple of 8 (pair-wise accesses): the mined tiles plus a
    ragged last block column"""
    t = NT.mine_tensor(300 + sf, 3, 3, 128, 128, sf)
    rng = np.random.default_rng(5)
    edge = NT.f32_to_bf16_bits(rng.standard_normal((t.shape[0], 6)).astype(np.float32))
    t = np.ascontiguousarray(np.concatenate([t, edge], axis=1))
    print("near ties ragged", t.shape, "sf", sf, flush=True)
    check_tensor(G, t, 128, 128, sf, min_close=7)


@pytest.mark.parametrize("sf", [1, 2])
def test_torch_emulation_flavour(G, sf):
    """the other flavour runs the exact arithmetic throughout (one workgroup per block straight from memory)"""
    t = NT.mine_tensor(400 + sf, 4, 4, 128, 128, sf, flavour=O.EMU)
    print("near ties emulation flavour sf", sf, flush=True)
    want, wmeta, wst = O.fake_quantize(t, 128, 128, CLAMP, 1, sf, O.EMU, want_stats=True)
    out, meta = G.fake_quantize(t, 128, 128, CLAMP, 1, sf, _cabi.FLAG_TORCH_EMULATION)
    assert np.array_equal(meta, wmeta) and np.array_equal(out, want)
    st = G.mor_stats(t, 128, 128, CLAMP, 1, sf, _cabi.FLAG_TORCH_EMULATION)
    assert bits_equal(st[..., 2], wst[..., 2]) and bits_equal(st[..., 3], wst[..., 3])


@pytest.mark.parametrize("sf", [1, 2])
def test_both_orientations_decide_for_themselves(G, sf):
    """mor_fake_quantize_dual_tiles: the transposed tile holds the same terms, the reference adds them in another order"""
    from test_gpu_dual_tiles import dual
    t = NT.mine_tensor(500 + sf, 12, 12, 128, 128, sf)
    tt = np.ascontiguousarray(t.T)
    want, wmeta = O.fake_quantize(t, 128, 128, CLAMP, 1, sf)
    want_t, wmeta_t = O.fake_quantize(tt, 128, 128, CLAMP, 1, sf)
    differ = int((wmeta_t != wmeta.T).sum())
    print("near ties, two orientations, sf", sf, ":", differ, "of", wmeta.size, "tiles decide differently when transposed", flush=True)
    out, meta, out_t, meta_t = dual(G, t, CLAMP, 1, sf)
    assert np.array_equal(meta, wmeta) and np.array_equal(out, want)
    assert np.array_equal(meta_t, wmeta_t), f"{int((meta_t != wmeta_t).sum())} transposed decisions differ"
    assert np.array_equal(out_t, want_t)
    assert differ > 0, "no tile of this tensor tells the two orders apart"


def test_tile_codes_take_the_same_decisions(G):
    from test_gpu_mor_wire import quantize, dequantize
    t = NT.mine_tensor(600, 8, 8, 128, 128, 1)
    want, wmeta = O.fake_quantize(t, 128, 128, CLAMP, 1, 1)
    payload, tags, scales = quantize(G, t, CLAMP, 1)
    assert np.array_equal(tags.cpu().numpy(), wmeta)
    assert np.array_equal(dequantize(G, payload, tags, scales), want)


@pytest.mark.parametrize("sf", [1, 2])
def test_batch_entry(G, sf):
    """small tensors (one workgroup per block from memory) and large ones (the register-resident kernel) in one call"""
    arrays = [NT.mine_tensor(700 + i + sf, gy, gx, bh, bw, sf) for i, (gy, gx, bh, bw) in
              enumerate([(2, 2, 128, 128), (4, 4, 32, 32), (8, 8, 128, 128), (1, 3, 64, 64), (6, 4, 128, 128)])]
    blocks = [(128, 128), (32, 32), (128, 128), (64, 64), (128, 128)]
    got = G.fake_quantize_batch(arrays, blocks, CLAMP, 1, sf)
    for a, (bh, bw), (out, meta) in zip(arrays, blocks, got):
        want, wmeta = O.fake_quantize(a, bh, bw, CLAMP, 1, sf)
        assert np.array_equal(meta, wmeta), (a.shape, bh, bw)
        assert np.array_equal(out, want)


@pytest.mark.parametrize("bh,bw", [(128, 128), (32, 32), (64, 256), (256, 256), (16, 64), (1024, 128)])
@pytest.mark.parametrize("sf", [1, 2])
def test_every_sum_in_the_reference_order_on_request(G, bh, bw, sf):
    """MOR_FLAG_REFERENCE_ORDER_SUMS on ordinary data: every block's sums are the oracle's bits, the results do not change"""
    from data_gen import tile_mixture
    rng = np.random.default_rng(bh + bw + sf)
    rows, cols = max(1024, bh), max(1024, 2 * bw)
    t = tile_mixture(rng, rows, cols)
    want, wmeta, wst = O.fake_quantize(t, bh, bw, 1e-3, 1, sf, want_stats=True)
    print("reference-order sums on request", bh, bw, "sf", sf, "blocks with sums:", int((wst[..., 2] > 0).sum()), flush=True)
    out, meta = G.fake_quantize(t, bh, bw, 1e-3, 1, sf, _cabi.FLAG_REFERENCE_ORDER_SUMS)
    assert np.array_equal(meta, wmeta) and np.array_equal(out, want)
    st = G.mor_stats(t, bh, bw, 1e-3, 1, sf, _cabi.FLAG_REFERENCE_ORDER_SUMS)
    assert bits_equal(st, wst)
    out0, meta0 = G.fake_quantize(t, bh, bw, 1e-3, 1, sf)
    assert np.array_equal(meta0, meta) and np.array_equal(out0, out)
