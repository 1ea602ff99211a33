"""Constructs quantization blocks whose two MoR error sums meet (test helper, CPU only).

The MoR decision of a block in the error band compares two fp32 sums, e4 <= e5
(/root/reference/mor/csrc/cuda/fake_quantize.cu:661).  On ordinary data the sums are far apart and the order of the
additions cannot matter.  The blocks made here are tuned, element by element, until the two sums agree to about their
last bits, so that only an implementation that adds the same terms in the same order takes the same decision.

Recipe for one block: normal data with one element as amax; elements of about amax * 2^-20 (they quantize to zero in
E4M3, term 1, and are representable in E5M2, small term) are added until the difference of the sums changes sign;
then single elements, and at the end a pair of elements, are moved to the bf16 values that bring the float64
difference of the terms closest to zero.  The oracle's sums in the reference's order are the judge of the result.
"""
import numpy as np

from oracle import mor_oracle as O


def f32_to_bf16_bits(x):
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(h):
    return (np.asarray(h, dtype=np.uint32) << 16).view(np.float32)


def _diff(e4, e5):
    return e4.astype(np.float64) - e5.astype(np.float64)


def mine_block(rng, bh, bw, sf_type, flavour=O.KERNEL, tol=2e-7):
    """-> uint16 [bh, bw] whose error sums differ by at most about `tol` relative (in float64 over the fp32 terms)."""
    n = bh * bw
    x = f32_to_bf16_bits(rng.standard_normal(n).astype(np.float32))
    # amax: one element above everything else, with a random mantissa (so that the scales differ from block to block)
    amax_bits = np.uint16(0x4080 | int(rng.integers(0, 128)))          # 4.0 .. 7.97
    amax = float(bf16_bits_to_f32(amax_bits))
    mag = x & 0x7FFF
    x = np.where(mag >= 0x4080, (x & 0x8000) | 0x407F, x).astype(np.uint16)       # everything else below 4.0
    order = rng.permutation(n)
    i_amax = order[0]
    x[i_amax] = amax_bits | (np.uint16(0x8000) if rng.integers(0, 2) else np.uint16(0))
    x[order[1:4]] = np.array([0x0000, 0x8000, 0x0000], np.uint16)[: max(0, min(3, n - 1))]      # a few zeros of both signs
    free = order[4:]
    e4, e5 = O.mor_error_terms(x, amax, sf_type, flavour)
    d = _diff(e4, e5)
    D = float(d.sum())
    # tiny elements: amax * 2^-21 .. 2^-19, i.e. exponent field of amax minus 19 .. 21
    amax_e = (int(amax_bits) >> 7) & 0xFF
    used = 0

    def tiny():
        e = amax_e - int(rng.integers(19, 22))
        return np.uint16((int(rng.integers(0, 2)) << 15) | (e << 7) | int(rng.integers(0, 128)))
    while D < 0.0 and used < free.size - 8:
        i = free[used]
        used += 1
        x[i] = tiny()
        t4, t5 = O.mor_error_terms(x[i:i + 1], amax, sf_type, flavour)
        nd = float(t4[0]) - float(t5[0])
        D += nd - d[i]
        d[i] = nd
    assert used > 0 and D >= 0.0, "the block never reached the point where the sums meet"
    rest = free[used:]
    # candidate values for the fine tuning: every bf16 magnitude from amax / 64 up to (not including) 4.0
    cand = np.array([(e << 7) | m for e in range(amax_e - 6, 0x81) for m in range(128)], np.uint16)
    cand = cand[cand < 0x4080]
    c4, c5 = O.mor_error_terms(cand, amax, sf_type, flavour)
    cd = _diff(c4, c5)
    srt = np.argsort(cd)
    cds = cd[srt]
    scale = float(e4.astype(np.float64).sum()) + 1.0
    k = 0
    # single elements: the candidate that brings D closest to zero
    while abs(D) > 1e-4 and k < rest.size - 2:
        i = rest[k]
        k += 1
        target = d[i] - D
        j = int(np.clip(np.searchsorted(cds, target), 1, cds.size - 1))
        j = j if abs(cds[j] - target) < abs(cds[j - 1] - target) else j - 1
        x[i] = cand[srt[j]] | (x[i] & 0x8000)
        D += cds[j] - d[i]
        d[i] = cds[j]
    # a pair of elements: for every value of the first, the best value of the second
    while abs(D) > tol * scale and k < rest.size - 1:
        i, i2 = rest[k], rest[k + 1]
        k += 2
        target = d[i] + d[i2] - D                       # wanted: cd[a] + cd[b] == target
        want_b = target - cds
        jb = np.clip(np.searchsorted(cds, want_b), 1, cds.size - 1)
        jb = np.where(np.abs(cds[jb] - want_b) < np.abs(cds[jb - 1] - want_b), jb, jb - 1)
        err = np.abs(cds + cds[jb] - target)
        a = int(np.argmin(err))
        b = int(jb[a])
        x[i] = cand[srt[a]] | (x[i] & 0x8000)
        x[i2] = cand[srt[b]] | (x[i2] & 0x8000)
        D += cds[a] + cds[b] - d[i] - d[i2]
        d[i], d[i2] = cds[a], cds[b]
    return x.reshape(bh, bw)


def mine_tensor(seed, gy, gx, bh, bw, sf_type, flavour=O.KERNEL):
    """-> uint16 [gy * bh, gx * bw]: every block tuned so that its error sums meet."""
    rng = np.random.default_rng(seed)
    t = np.empty((gy * bh, gx * bw), np.uint16)
    for by in range(gy):
        for bx in range(gx):
            t[by * bh:(by + 1) * bh, bx * bw:(bx + 1) * bw] = mine_block(rng, bh, bw, sf_type, flavour)
    return t


def reference_order_sum(terms_hi_lo):
    """The reference's order of additions (fake_quantize.cu:491-583) restated with numpy slices, independently of the
    oracle's loops: `terms_hi_lo` is float32 [tby, tbx, k, 2] -- for every thread (ty, tx) its k words in the order it
    meets them, each with the term of the odd and of the even column.  Returns the float32 block sum."""
    t = np.asarray(terms_hi_lo, np.float32)
    tby, tbx, k, _ = t.shape
    acc = np.zeros((tby, tbx), np.float32)
    for j in range(k):
        acc = acc + (t[:, :, j, 0] + t[:, :, j, 1])                # one float32 addition per word and thread
    v = acc.reshape(-1, 32)                                          # warps of 32 consecutive threads
    for off in (16, 8, 4, 2, 1):
        v = v[:, :off] + v[:, off:2 * off]
    w = np.zeros(32, np.float32)
    w[: v.shape[0]] = v[:, 0]
    for off in (16, 8, 4, 2, 1):
        w = w[:off] + w[off:2 * off]
    return np.float32(w[0])
