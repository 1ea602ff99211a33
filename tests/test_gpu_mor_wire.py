"""mor_mor_quantize / mor_mor_dequantize (MoR or a forced FP8 format per 128 x 128 tile, codes + tag + fp32 scale): the tags are the oracle's
meta values, the decoded tensor is the oracle's fake-quantized output, and the payload is decoded a second time on the
host from the documented layout alone (float8 views, a table for E2M3, an IEEE division, a round-half-up bf16 store)."""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
from data_gen import tile_mixture as mixture

pytestmark = pytest.mark.gpu

TILE_BYTES = 32768
STORED_BF16 = 0x100


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def quantize(G, a, clamp, mode):
    from mor_amd import _cabi
    L = _cabi.lib()
    rows, cols = a.shape
    gy, gx = rows // 128, cols // 128
    x = G.to_dev_u16(a)
    payload = torch.full((gy, gx, TILE_BYTES), 0xA5, dtype=torch.uint8, device=G.dev())
    tags = torch.full((gy, gx), -7, dtype=torch.int32, device=G.dev())
    scales = torch.full((gy, gx), -7.0, dtype=torch.float32, device=G.dev())
    _cabi.check(L.mor_mor_quantize(x.data_ptr(), payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), rows, cols, float(clamp), mode,
                                   G.stream_ptr()))
    torch.cuda.synchronize()
    return payload, tags, scales


def dequantize(G, payload, tags, scales):
    from mor_amd import _cabi
    L = _cabi.lib()
    rows, cols = tags.shape[0] * 128, tags.shape[1] * 128
    out = torch.full((rows, cols), 7.0, dtype=torch.bfloat16, device=G.dev())
    _cabi.check(L.mor_mor_dequantize(payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), out.data_ptr(), rows, cols, G.stream_ptr()))
    torch.cuda.synchronize()
    return G.to_host_u16(out)


E2M3_VALUES = np.array([m / 8.0 for m in range(8)] + [(1 + m / 8.0) * 2.0 ** (e - 1) for e in range(1, 4) for m in range(8)], dtype=np.float32)


def host_code_values(slot, tag):
    """one payload slot of an FP8 / FP6 tile -> (magnitudes float32 [128, 128], sign bits uint16 [128, 128])"""
    if tag in (1, 11, 2, 12):
        codes = slot[:128 * 128].reshape(128, 128)
        dt = torch.float8_e4m3fn if tag in (1, 11) else torch.float8_e5m2
        mag = torch.from_numpy((codes & 0x7F).copy()).view(dt).to(torch.float32).numpy()
        return mag, (codes >> 7).astype(np.uint16)
    assert tag == 4, tag
    b = slot[:128 * 96].reshape(128, 32, 3).astype(np.uint32)
    w = b[..., 0] | (b[..., 1] << 8) | (b[..., 2] << 16)                      # 4 codes per 3 bytes, code k at bits 6k
    codes = np.stack([(w >> (6 * k)) & 0x3F for k in range(4)], axis=-1).reshape(128, 128)
    return E2M3_VALUES[codes & 0x1F], (codes >> 5).astype(np.uint16)


def host_decode_tile(slot, tag, scale):
    """one payload slot (uint8[32768]) -> uint16[128, 128] bf16 bits, from the documented layout"""
    if tag & STORED_BF16 or tag == 3:
        return slot[:128 * 256].view(np.uint16).reshape(128, 128).copy()
    mag, sign = host_code_values(slot, tag)
    q = (mag / np.float32(scale)).astype(np.float32)                               # IEEE division
    bits = ((q.view(np.uint32).astype(np.uint64) + 0x8000) >> 16).astype(np.uint16)  # bf16, half rounded up
    return bits | (sign << 15)


def tile_amax(a, by, bx):
    t = a[by * 128:(by + 1) * 128, bx * 128:(bx + 1) * 128]
    return (t & 0x7FFF).max()


def bf16_bits_to_f32(b):
    return np.array([int(b) << 16], dtype=np.uint32).view(np.float32)[0]


@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (1024, 512), (2048, 2048)])
@pytest.mark.parametrize("mode", [1, 101, 2, 3])
def test_tags_round_trip_and_host_decode(G, shape, mode):
    rows, cols = shape
    rng = np.random.default_rng(rows * 5 + cols + mode)
    a = mixture(rng, rows, cols)
    if rows > 128:
        a[133, 7] = 0x7FC0              # a NaN and an infinity in tiles of their own
        a[9, 131] = 0xFF80
        a[128:256, 128:256] = np.where(rng.random((128, 128)) < 0.5, 0x8000, 0).astype(np.uint16)    # zeros of both signs
    clamp = 1e-3
    print("mor wire", shape, mode, flush=True)
    payload, tags, scales = quantize(G, a, clamp, mode)
    got = dequantize(G, payload, tags, scales)
    want, wmeta = O.fake_quantize(a, 128, 128, clamp, mode, 1)
    t, s, p = tags.cpu().numpy(), scales.cpu().numpy(), payload.cpu().numpy()
    assert np.array_equal(t & 0xFF, wmeta.reshape(t.shape)), "tags differ from the oracle's meta"
    assert np.array_equal(got, want), "decoded tensor differs from the oracle's output"
    seen = set()
    for by in range(rows // 128):
        for bx in range(cols // 128):
            tag, amax_bits = int(t[by, bx]), int(tile_amax(a, by, bx))
            amax = bf16_bits_to_f32(amax_bits)
            # tiles stored as bf16 images: those with a NaN, and those whose scale 448 / amax leaves 2^-90 .. 2^90
            with np.errstate(divide="ignore", over="ignore"):
                s4 = np.float32(448.0) / amax if amax_bits <= 0x7F80 and amax_bits != 0 else np.float32(1.0)
            s4_bits = int(np.array([s4], dtype=np.float32).view(np.uint32)[0])
            expo = ((s4_bits >> 23) & 0xFF) - 127
            outside = amax_bits > 0x7F80 or (amax_bits != 0 and (not (-90 <= expo <= 90) or s4_bits & 0x7FFFFF == 0x7FFFFF))
            assert bool(tag & STORED_BF16) == bool(outside), (by, bx, tag, amax_bits)
            fmax = {1: 448.0, 11: 448.0, 2: 57344.0, 12: 57344.0, 4: 7.5}.get(tag)
            if fmax is not None and amax_bits != 0:
                assert s[by, bx] == np.float32(fmax) / amax, (by, bx, tag, s[by, bx])
            else:
                assert s[by, bx] == 1.0, (by, bx, tag, s[by, bx])
            dec = host_decode_tile(p[by, bx], tag, s[by, bx])
            assert np.array_equal(dec, want[by * 128:(by + 1) * 128, bx * 128:(bx + 1) * 128]), ("host decode", by, bx, tag)
            seen.add(tag)
    if rows * cols >= 2048 * 2048 and mode % 10 == 1:
        assert len({x & 0xFF for x in seen}) >= 4 and any(x & STORED_BF16 for x in seen), seen


def test_slot_bytes_beyond_the_tile_are_left_alone(G):
    rng = np.random.default_rng(3)
    a = mixture(rng, 512, 512)
    payload, tags, scales = quantize(G, a, 1e-3, 1)
    p, t = payload.cpu().numpy(), tags.cpu().numpy()
    for by in range(4):
        for bx in range(4):
            tag = int(t[by, bx])
            used = 128 * (256 if (tag & STORED_BF16 or tag == 3) else 96 if tag == 4 else 128)
            assert (p[by, bx, used:] == 0xA5).all(), (by, bx, tag)


def test_large_tensor_round_trip_equals_fake_quantize(G):
    """8192 x 8192 (band order, streaming loads and stores): decode(encode(x)) is mor_fake_quantize's output, the tags its meta"""
    import mor_amd
    rows, cols = 8192, 8192
    g = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn(rows, cols, device="cuda", generator=g)
    x[:, :2048] *= torch.exp(3 * torch.randn(rows, 2048, device="cuda", generator=g))
    x[:, 2048:3072] = 1.0 + 0.3 * torch.rand(rows, 1024, device="cuda", generator=g)
    x[:1024, 4096:] *= 1e-34
    x = x.to(torch.bfloat16)
    for mode in (1, 101, 2):
        payload, tags, scales = mor_amd.wire.quantize_mor_tiles(x, 1e-15, mode)
        back = mor_amd.wire.dequantize_mor_tiles(payload, tags, scales)
        ref, rmeta = mor_amd.ops.fake_quantize(x, rows, cols, 128, 128, 1e-15, mode, 1)
        assert torch.equal(tags & 0xFF, rmeta.view(tags.shape))
        assert torch.equal(back.view(torch.int16), ref.view(torch.int16))
        kinds = set((tags & 0xFF).unique().tolist())
        assert (len(kinds) >= 3 or mode == 2) and bool((tags & STORED_BF16).any()), kinds


def test_rejects_what_it_cannot_do(G):
    from mor_amd import _cabi
    L = _cabi.lib()
    x = torch.zeros((128, 256), dtype=torch.bfloat16, device=G.dev())
    p = torch.zeros(2 * TILE_BYTES, dtype=torch.uint8, device=G.dev())
    t = torch.zeros(2, dtype=torch.int32, device=G.dev())
    s = torch.zeros(2, dtype=torch.float32, device=G.dev())
    q = lambda r, c, mode, a=x, b=p: L.mor_mor_quantize(a.data_ptr(), b.data_ptr(), t.data_ptr(), s.data_ptr(), r, c, 0.0, mode, G.stream_ptr())
    assert q(128, 200, 1) != 0 and b"multiples of 128" in L.mor_last_error()
    assert q(128, 256, 4) != 0 and b"mode" in L.mor_last_error()
    assert q(128, 256, 1, x, x) != 0 and b"different" in L.mor_last_error()
    assert L.mor_mor_quantize(x.data_ptr(), p.data_ptr(), 0, s.data_ptr(), 128, 256, 0.0, 1, G.stream_ptr()) != 0
    assert L.mor_mor_dequantize(p.data_ptr(), t.data_ptr(), s.data_ptr(), x.data_ptr(), 100, 256, G.stream_ptr()) != 0
    assert q(128, 256, 1) == 0
    torch.cuda.synchronize()


def test_matrix_instruction_consumes_tile_rows(G):
    """Rows of a tile's payload are operands of the gfx950 scaled matrix instruction as they lie in the slot (128 code
    bytes per row for E4M3 / E5M2, 96 for E2M3: the row layout of the MX payload): 16 rows of one tile times 16 rows of
    another with unit block scales, divided by the two tile scales, is the product of the decoded rows."""
    from mor_amd import _cabi
    L = _cabi.lib()
    rng = np.random.default_rng(77)
    x = rng.standard_normal((128, 768)).astype(np.float32)
    x[:, 128:256] *= 37.0                                                          # another scale, E4M3 as well
    x[:, 256:384] = 1.0 + 0.3 * rng.random((128, 128))                             # E2M3
    x[:, 384:512] = -(2.0 + 0.5 * rng.random((128, 128)))                          # E2M3
    x[:, 512:768] = np.exp2(rng.uniform(-12.0, 8.0, (128, 256))) * rng.choice([-1.0, 1.0], (128, 256))   # range 2^20: E5M2 by the dynamic-range rule
    a = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()
    payload, tags, scales = quantize(G, a, 1e-3, 101)
    t, s, p = tags.cpu().numpy()[0], scales.cpu().numpy()[0], payload.cpu().numpy()[0]
    print("tile tags", t, flush=True)
    assert t[0] in (1, 11) and t[1] in (1, 11) and t[2] == 4 and t[3] == 4 and t[4] in (2, 12) and t[5] in (2, 12), t
    unit = torch.full((16, 4), 127, dtype=torch.uint8, device=G.dev())             # E8M0 bytes of 2^0
    for ta, tb, fmt in ((0, 1, 0), (4, 5, 1), (2, 3, 3)):
        out = torch.zeros((16, 16), dtype=torch.float32, device=G.dev())
        pa, pb = payload[0, ta], payload[0, tb]                                     # rows 0..15 of each slot
        _cabi.check(L.mor_selftest_mx_mfma(pa.data_ptr(), unit.data_ptr(), pb.data_ptr(), unit.data_ptr(), fmt, out.data_ptr(), G.stream_ptr()))
        torch.cuda.synchronize()
        got = out.cpu().double().numpy() / (float(s[ta]) * float(s[tb]))
        rows = []
        for k in (ta, tb):                                                          # value(code) / scale, from the documented layout
            mag, sign = host_code_values(p[k], int(t[k]))
            rows.append((mag[:16].astype(np.float64) * np.where(sign[:16] != 0, -1.0, 1.0)) / float(s[k]))
        want = rows[0] @ rows[1].T
        bound = np.abs(rows[0]) @ np.abs(rows[1]).T
        excess = np.max(np.abs(got - want) / bound)
        print(f"tile rows through the matrix instruction, format {fmt}: max |difference| / sum of magnitudes {excess:.3e}", flush=True)
        # the instruction aligns the 128 products of a row to the largest before it adds them: 1e-5 of the sum of magnitudes
        # for the narrow tiles, 1.3e-4 for the E5M2 rows whose products span 2^40; a wrong layout is wrong by the sum itself
        assert excess <= (5e-4 if fmt == 1 else 2e-5), (fmt, excess)


def test_tile_entries_replay_in_a_hip_graph(G):
    """The tile-code, dual-orientation and batch entries allocate nothing and clear nothing with memsets, so they can be
    captured: every replay, with eager work and synchronizations in between and fresh input each time, equals the eager
    result.  (Buffers are allocated before the capture; the calls go through the C ABI.)"""
    import ctypes as C
    from mor_amd import _cabi
    from mor_amd.batch import TensorDesc
    L = _cabi.lib()
    rows, cols = 512, 1024
    dev = G.dev()
    x = torch.empty(rows, cols, dtype=torch.bfloat16, device=dev)
    gy, gx = rows // 128, cols // 128

    def buffers():
        return dict(payload=torch.zeros((gy, gx, TILE_BYTES), dtype=torch.uint8, device=dev),
                    tags=torch.zeros((gy, gx), dtype=torch.int32, device=dev), scales=torch.zeros((gy, gx), dtype=torch.float32, device=dev),
                    back=torch.zeros_like(x), out=torch.zeros_like(x), out_t=torch.zeros((cols, rows), dtype=torch.bfloat16, device=dev),
                    meta=torch.zeros((gy, gx), dtype=torch.int32, device=dev), meta_t=torch.zeros((gx, gy), dtype=torch.int32, device=dev),
                    bout=torch.zeros_like(x), bmeta=torch.zeros((gy, gx), dtype=torch.int32, device=dev))

    def body(b):
        st = torch.cuda.current_stream().cuda_stream
        _cabi.check(L.mor_mor_quantize(x.data_ptr(), b["payload"].data_ptr(), b["tags"].data_ptr(), b["scales"].data_ptr(), rows, cols, 1e-3, 1, st))
        _cabi.check(L.mor_mor_dequantize(b["payload"].data_ptr(), b["tags"].data_ptr(), b["scales"].data_ptr(), b["back"].data_ptr(), rows, cols, st))
        _cabi.check(L.mor_fake_quantize_dual_tiles(x.data_ptr(), b["out"].data_ptr(), b["meta"].data_ptr(), b["out_t"].data_ptr(),
                                                   b["meta_t"].data_ptr(), rows, cols, 1e-3, 1, 1, st))
        d = (TensorDesc * 1)()
        d[0].input, d[0].output, d[0].meta = x.data_ptr(), b["bout"].data_ptr(), b["bmeta"].data_ptr()
        d[0].rows, d[0].cols, d[0].block_rows, d[0].block_cols = rows, cols, 128, 128
        d[0].clamp_threshold, d[0].mode, d[0].sf_type = 1e-3, 1, 1
        _cabi.check(L.mor_fake_quantize_batch(d, 1, 0, st))

    g = torch.Generator(device="cuda").manual_seed(19)
    x.copy_(torch.randn(rows, cols, device=dev, generator=g))
    cap, eager = buffers(), buffers()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        body(eager)                                        # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        body(cap)
    for rep in range(4):
        x.copy_(torch.randn(rows, cols, device=dev, generator=g) * (30.0 ** rep))
        if rep == 2:
            x[:128, :128] *= 1e-30                         # a tile outside the fast range
        graph.replay()
        torch.cuda.synchronize()
        body(eager)                                        # eager work between the replays
        torch.cuda.synchronize()
        ref, rmeta = G.fake_quantize(G.to_host_u16(x), 128, 128, 1e-3, 1, 1)
        for k in cap:
            if k == "payload":
                continue                                   # (slot tails are never written: compared through `back`)
            assert torch.equal(cap[k].view(torch.int32) if cap[k].dtype == torch.float32 else cap[k], eager[k].view(torch.int32) if eager[k].dtype == torch.float32 else eager[k]), (rep, k)
        assert np.array_equal(G.to_host_u16(cap["back"]), ref) and np.array_equal(G.to_host_u16(cap["bout"]), ref), rep
        assert np.array_equal(cap["bmeta"].cpu().numpy(), rmeta), rep


def host_transpose_slot(slot, tag):
    """the slot of the transposed tile, from the documented layout"""
    out = np.full(TILE_BYTES, 0xA5, dtype=np.uint8)
    if tag & STORED_BF16 or tag == 3:
        out[:128 * 256] = np.ascontiguousarray(slot[:128 * 256].view(np.uint16).reshape(128, 128).T).view(np.uint8).ravel()
    elif tag in (1, 11, 2, 12):
        out[:128 * 128] = np.ascontiguousarray(slot[:128 * 128].reshape(128, 128).T).ravel()
    else:
        b = slot[:128 * 96].reshape(128, 32, 3).astype(np.uint32)
        w = b[..., 0] | (b[..., 1] << 8) | (b[..., 2] << 16)
        codes = np.stack([(w >> (6 * k)) & 0x3F for k in range(4)], axis=-1).reshape(128, 128).T.reshape(128, 32, 4)
        w = codes[..., 0] | (codes[..., 1] << 6) | (codes[..., 2] << 12) | (codes[..., 3] << 18)
        out[:128 * 96] = np.stack([w & 0xFF, (w >> 8) & 0xFF, (w >> 16) & 0xFF], axis=-1).astype(np.uint8).ravel()
    return out


@pytest.mark.parametrize("shape", [(128, 128), (256, 640), (1024, 512), (384, 2048)])
def test_transposed_tile_codes(G, shape):
    """mor_mor_transpose: every slot is the transposed tile in the same packing, tags and scales move with their tiles,
    and the result decodes to the transpose of what the source decodes to."""
    import mor_amd
    rows, cols = shape
    rng = np.random.default_rng(rows * 11 + cols)
    a = mixture(rng, rows, cols)
    if rows > 128:
        a[133, 7] = 0x7FC0
    payload, tags, scales = quantize(G, a, 1e-3, 1)
    gy, gx = tags.shape
    payload_t = torch.full((gx, gy, TILE_BYTES), 0xA5, dtype=torch.uint8, device=G.dev())
    tags_t = torch.full((gx, gy), -7, dtype=torch.int32, device=G.dev())
    scales_t = torch.full((gx, gy), -7.0, dtype=torch.float32, device=G.dev())
    from mor_amd import _cabi
    L = _cabi.lib()
    _cabi.check(L.mor_mor_transpose(payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), payload_t.data_ptr(), tags_t.data_ptr(),
                                    scales_t.data_ptr(), gy, gx, G.stream_ptr()))
    torch.cuda.synchronize()
    assert torch.equal(tags_t, tags.t()) and torch.equal(scales_t, scales.t())
    p, pt, t = payload.cpu().numpy(), payload_t.cpu().numpy(), tags.cpu().numpy()
    seen = set()
    for by in range(gy):
        for bx in range(gx):
            assert np.array_equal(pt[bx, by], host_transpose_slot(p[by, bx], int(t[by, bx]))), (by, bx, int(t[by, bx]))
            seen.add(int(t[by, bx]))
    back = dequantize(G, payload, tags, scales)
    back_t = dequantize(G, payload_t, tags_t, scales_t)
    assert np.array_equal(back_t, np.ascontiguousarray(back.T))
    if rows * cols >= 1024 * 512:
        assert len({x & 0xFF for x in seen}) >= 3 and any(x & STORED_BF16 for x in seen), seen
    # the Python helpers
    (p3, t3, s3), (pt3, tt3, st3) = mor_amd.wire.quantize_mor_tiles_dual(G.to_dev_u16(a), 1e-3, 1)
    assert torch.equal(t3, tags) and torch.equal(tt3, tags_t) and torch.equal(st3, scales_t)
    assert np.array_equal(G.to_host_u16(mor_amd.wire.dequantize_mor_tiles(pt3, tt3, st3)), back_t)
    pt2, tt2, st2 = mor_amd.wire.transpose_mor_tiles(payload, tags, scales)
    assert torch.equal(tt2, tags_t) and torch.equal(st2, scales_t)
    assert np.array_equal(G.to_host_u16(mor_amd.wire.dequantize_mor_tiles(pt2, tt2, st2)), back_t)


def test_transposed_tile_codes_equal_the_codes_of_the_transpose(G):
    """On tiles whose decision does not hang on the order of the error sums, transposing the codes equals quantizing the
    transposed tensor (the same elements, the same amax, scale and format)."""
    import mor_amd
    rows, cols = 1024, 768
    g = torch.Generator(device="cuda").manual_seed(23)
    x = torch.randn(rows, cols, device="cuda", generator=g)
    x[:, :256] = 1.0 + 0.3 * torch.rand(rows, 256, device="cuda", generator=g)
    x = x.to(torch.bfloat16)
    for mode in (101, 2):                                        # (dynamic-range rule and a forced format: no error sums)
        p, t, s = mor_amd.wire.quantize_mor_tiles(x, 1e-3, mode)
        pt, tt, st = mor_amd.wire.transpose_mor_tiles(p, t, s)
        q, u, v = mor_amd.wire.quantize_mor_tiles(x.t().contiguous(), 1e-3, mode)
        assert torch.equal(tt, u) and torch.equal(st, v)
        used = torch.where((u == 4)[..., None], torch.arange(TILE_BYTES, device="cuda") < 128 * 96, torch.arange(TILE_BYTES, device="cuda") < 128 * 128)
        assert torch.equal(pt[used], q[used])


@pytest.mark.parametrize("shape", [(128, 128), (256, 640), (1024, 512), (2048, 2048)])
@pytest.mark.parametrize("mode", [1, 101, 2])
def test_both_orientations_in_one_call(G, shape, mode):
    """mor_mor_quantize_dual writes, byte for byte (slot tails untouched), what mor_mor_quantize and mor_mor_transpose
    of its result write."""
    from mor_amd import _cabi
    L = _cabi.lib()
    rows, cols = shape
    rng = np.random.default_rng(rows * 13 + cols + mode)
    a = mixture(rng, rows, cols)
    if rows > 128:
        a[133, 7] = 0x7FC0
        a[128:256, 128:256] = np.where(rng.random((128, 128)) < 0.5, 0x8000, 0).astype(np.uint16)
    print("tile codes, both orientations", shape, mode, flush=True)
    payload, tags, scales = quantize(G, a, 1e-3, mode)
    gy, gx = tags.shape

    def fresh(y, x):
        return (torch.full((y, x, TILE_BYTES), 0xA5, dtype=torch.uint8, device=G.dev()), torch.full((y, x), -7, dtype=torch.int32, device=G.dev()),
                torch.full((y, x), -7.0, dtype=torch.float32, device=G.dev()))

    pt, tt, st = fresh(gx, gy)
    _cabi.check(L.mor_mor_transpose(payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), pt.data_ptr(), tt.data_ptr(), st.data_ptr(), gy, gx, G.stream_ptr()))
    p2, t2, s2 = fresh(gy, gx)
    pt2, tt2, st2 = fresh(gx, gy)
    x = G.to_dev_u16(a)
    _cabi.check(L.mor_mor_quantize_dual(x.data_ptr(), p2.data_ptr(), t2.data_ptr(), s2.data_ptr(), pt2.data_ptr(), tt2.data_ptr(), st2.data_ptr(),
                                        rows, cols, 1e-3, mode, G.stream_ptr()))
    torch.cuda.synchronize()
    assert torch.equal(t2, tags) and torch.equal(s2.view(torch.int32), scales.view(torch.int32)) and torch.equal(p2, payload)
    assert torch.equal(tt2, tt) and torch.equal(st2.view(torch.int32), st.view(torch.int32)) and torch.equal(pt2, pt)
    assert L.mor_mor_quantize_dual(x.data_ptr(), p2.data_ptr(), t2.data_ptr(), s2.data_ptr(), p2.data_ptr(), tt2.data_ptr(), st2.data_ptr(),
                                   rows, cols, 1e-3, mode, G.stream_ptr()) != 0 and b"different" in L.mor_last_error()
