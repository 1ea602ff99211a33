"""The order of the additions in the oracle's MoR error sums (CPU).

The reference adds the terms |q / x - 1| of a block in the order its thread layout and shuffle trees give
(/root/reference/mor/csrc/cuda/fake_quantize.cu:491-583, launch geometry :1770-1789).  The order only shows in the last
bits of the sums, so it is pinned here on blocks whose two sums meet (near_ties.mine_block): the oracle's sums have
to equal, bit for bit, a restatement of that order with numpy slices (near_ties.reference_order_sum) that shares no
code with the oracle's loops, and the restatement must differ from plainer orders on those blocks (else the test
would pin nothing)."""
import numpy as np
import pytest

from oracle import mor_oracle as O
import near_ties as NT


def thread_terms(block, sf_type, bh, bw):
    """float32 [tby, tbx, k, 2] per format: the words each reference thread meets, in its order (rows outer, words inner)"""
    amax = float(NT.bf16_bits_to_f32(block & 0x7FFF).max())
    e4, e5 = O.mor_error_terms(block, amax, sf_type)
    if bh * bw > 1024:
        tbx, tby = 16, 32
    else:
        tbx, tby = bw // 2, bh
    out = []
    for e in (e4, e5):
        t = e.reshape(bh, bw // 2, 2)                     # [row, word, (even column, odd column)]
        t = t[:, :, ::-1]                                 # the reference adds (odd column's term + even column's term)
        # row r = ty + tby * a, word w = tx + tbx * b  ->  [a, ty, b, tx, 2] -> [ty, tx, a, b, 2]
        t = t.reshape(bh // tby, tby, (bw // 2) // tbx, tbx, 2).transpose(1, 3, 0, 2, 4)
        out.append(np.ascontiguousarray(t).reshape(tby, tbx, -1, 2))
    return out


@pytest.mark.parametrize("bh,bw", [(128, 128), (32, 32), (64, 64), (8, 8), (32, 64), (256, 256)])
@pytest.mark.parametrize("sf_type", [1, 2])
def test_oracle_adds_in_the_reference_order(bh, bw, sf_type):
    rng = np.random.default_rng(bh * 1000 + bw + sf_type)
    differs_from_row_major = 0
    for _ in range(6 if bh * bw <= 16384 else 2):
        block = NT.mine_block(rng, bh, bw, sf_type) if bh * bw >= 1024 else NT.f32_to_bf16_bits(
            np.exp(4 * rng.standard_normal((bh, bw))).astype(np.float32))
        _, _, st = O.fake_quantize(block, bh, bw, 1e-15, 1, sf_type, want_stats=True)
        t4, t5 = thread_terms(block, sf_type, bh, bw)
        if st[0, 0, 2] == 0 and st[0, 0, 3] == 0:
            continue                                       # (an 8 x 8 block that was decided by its range)
        want4, want5 = NT.reference_order_sum(t4), NT.reference_order_sum(t5)
        assert st[0, 0, 2].view(np.uint32) == want4.view(np.uint32), (st[0, 0, 2], want4)
        assert st[0, 0, 3].view(np.uint32) == want5.view(np.uint32), (st[0, 0, 3], want5)
        amax = float(NT.bf16_bits_to_f32(block & 0x7FFF).max())
        e4, _ = O.mor_error_terms(block, amax, sf_type)
        seq = np.float32(0)
        for v in e4:
            seq = np.float32(seq + v)
        differs_from_row_major += int(seq.view(np.uint32) != want4.view(np.uint32))
    if bh * bw >= 4096:
        assert differs_from_row_major > 0, "the order of additions does not show on these blocks"


def test_mined_blocks_meet():
    """the construction itself: sums within 1e-6 of each other, both decisions occur"""
    t = NT.mine_tensor(7, 6, 6, 128, 128, 1)
    _, meta, st = O.fake_quantize(t, 128, 128, 1e-15, 1, 1, want_stats=True)
    e4, e5 = st[..., 2], st[..., 3]
    assert (np.abs(e4 - e5) <= 1e-6 * np.maximum(e4, e5)).all()
    assert set(np.unique(meta)) == {1, 3}
    # the decision is the comparison of the two sums (fake_quantize.cu:661)
    assert np.array_equal(meta == 1, e4 <= e5)
