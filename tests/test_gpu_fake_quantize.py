"""GPU parity of mor_fake_quantize / mor_block_format (C ABI) against the CPU oracle: bit-exact outputs and meta."""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O
import data_gen
import torch_emulation as E

pytestmark = pytest.mark.gpu

POKES_RANGE = [(128, 1, 18200, 50968), (0, 70, 21000, 53768), (1, 1, 17262, 50030)]
POKES_ERROR = [(128, 1, 18403, 51171), (0, 70, 21000, 53768), (1, 1, 17264, 50032)]


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def uniform_bits(seed, rows, cols, lo, hi):
    g = torch.Generator().manual_seed(seed)
    return E.bf16_to_bits(torch.empty(rows, cols).uniform_(lo, hi, generator=g).to(torch.bfloat16))


def assert_same(got, want, what):
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        r, c = bad[0]
        raise AssertionError(f"{what}: {len(bad)} of {got.size} differ; first at ({r},{c}): got {got[r, c]:#06x} want {want[r, c]:#06x}")


def test_hw_cast_selftest(G):
    """All 2^32 fp32 inputs in range: the gfx950 converts equal the software model of the reference's cast."""
    from mor_amd import _cabi
    m = torch.full((3,), -1, dtype=torch.int64, device="cuda")
    print("selftest hw cast", flush=True)
    _cabi.check(_cabi.lib().mor_selftest_hw_cast(m.data_ptr(), G.stream_ptr()))
    torch.cuda.synchronize()
    assert m.tolist() == [0, 0, 0], m.tolist()       # E4M3, E5M2, scaled pair converts against the plain ones


@pytest.mark.parametrize("pokes,mode,sf,clamp,want_meta", [
    (POKES_RANGE, 101, 1, 1e-15, [[1, 3], [2, 4]]),
    (POKES_ERROR, 1, 1, 1e-15, [[1, 3], [3, 4]]),
    (POKES_RANGE, 101, 2, 1e-25, [[1, 3], [2, 4]]),
    (POKES_ERROR, 1, 2, 1e-25, None),
])
def test_reference_fixtures(G, pokes, mode, sf, clamp, want_meta):
    a = E.fixture_words(256, 256, pokes)
    print("fixture", mode, sf, flush=True)
    out, meta = G.fake_quantize(a, 128, 128, clamp, mode, sf)
    want, wmeta = O.fake_quantize(a, 128, 128, clamp, mode, sf)
    if want_meta is not None:
        assert meta.tolist() == want_meta
    assert np.array_equal(meta, wmeta)
    assert_same(out, want, "fixture")


def test_golden_file(G):
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_fixtures.npz"))
    for key, mode, sf, clamp in (("range", 101, 1, 1e-15), ("error", 1, 1, 1e-15), ("range_e8", 101, 2, 1e-25)):
        out, meta = G.fake_quantize(g[f"{key}_in"], 128, 128, clamp, mode, sf)
        assert np.array_equal(meta, g[f"{key}_meta"])
        assert_same(out, g[f"{key}_out"], key)


def test_zero_tiny_and_bf16_modes(G):
    z = np.zeros((256, 256), np.uint16)
    out, meta = G.fake_quantize(z, 128, 128, 1e-25, 101, 2)
    assert (meta == 4).all() and np.array_equal(out, z)
    t = E.bf16_to_bits(torch.ones(256, 256, dtype=torch.bfloat16) * 1e-27)
    out, meta = G.fake_quantize(t, 128, 128, 1e-25, 101, 2)
    want, wmeta = O.fake_quantize(t, 128, 128, 1e-25, 101, 2)
    assert (meta == 4).all() and np.array_equal(out, want)
    a = uniform_bits(1, 256, 256, -53768.0, 53768.0)
    for mode in (7, 0, 6, 8, 9):
        out, meta = G.fake_quantize(a, 128, 128, 1e-15, mode, 1)
        assert (meta == 3).all() and np.array_equal(out, a)


SHAPES = [
    # rows, cols, brows, bcols        kernel that serves it
    (64, 256, 1, 32),                 # row groups of 4 lanes (MX)
    (16, 1024, 1, 8),                 # 1 lane per block
    (8, 2048, 1, 512),                # 64 lanes per block
    (7, 2048, 1, 1024),               # 128 lanes per block: two waves meet in LDS; 7 rows leave a partial workgroup
    (5, 2048, 1, 2048),               # 256 lanes per block: the whole workgroup
    (8200, 1024, 1, 1024),            # 128 lanes, 16 MiB output (streaming stores)
    (32, 4096, 1, 4096),              # workgroup per row
    (256, 384, 128, 128),             # workgroup per tile
    (200, 256, 128, 128),             # partial tile rows
    (64, 192, 64, 64),
    (48, 112, 16, 56),                # odd chunk count per block row
    (37, 45, 16, 32),                 # odd columns: generic kernel
    (1, 32, 1, 32),
    (130, 260, 128, 128),             # ragged, cols not a multiple of 8
    (12, 14336, 1, 14336),            # one long row per workgroup of 512 threads, last vector partly filled
    (6, 16384, 1, 16384),             # the same, every vector full
    (9, 10000, 1, 10000),             # ... and a chunk count per row that is not a power of two
    (16, 40000, 1, 40000),            # block larger than the register-resident limit
    (300, 7, 64, 1),                  # blocks one column wide: every pair of the element-wise kernel is half empty
    (257, 33, 128, 3),                # odd block width, partial last block row and column
    (500, 129, 100, 127),             # odd width close to the pair capacity of a workgroup
    (9000, 5, 8192, 1),               # 8192 single-element pairs: the capacity itself
    (9000, 5, 8193, 1),               # ... and one more: the generic kernel
    (40, 96, 8, 8),                   # lane groups: 8 lanes per tile, 32 tiles per workgroup
    (50, 200, 16, 16),                # ... 32 lanes, partial last tile row and column
    (96, 160, 32, 32),                # ... a wave per tile, two vectors per lane
    (30, 192, 1, 24),                 # ... 3 vectors per block in groups of 4 lanes
    (20, 1536, 1, 1536),              # ... 192 vectors per block: 3 of 4 vector slots per lane
    (70, 120, 2, 40),                 # ... 10 vectors per block in groups of 16 lanes
    (6, 32768, 1, 32768),             # 32768 elements: in the registers of 512 threads
    (512, 768, 256, 256),             # blocks of 65536 elements: in the registers of 1024 threads
    (300, 1032, 256, 1024),           # larger blocks: the large-block kernel (a pass over the block per step)
    (300, 520, 256, 512),             # ... with partial last block rows and a last block column 8 elements wide
    (5, 28672, 1, 28672),             # ... one long row per block
    (3, 131072, 1, 131072),
    (131, 2056, 129, 2048),           # ... an odd row count per block
    # blocks 128 columns wide on rows that do not start on 16-byte boundaries
    (259, 383, 128, 128),             # odd width: every shift 0 .. 7, last block column 127 wide, last block row 3 rows
    (140, 644, 128, 128),             # rows 8-byte aligned (shifts 0 and 4), last block column 4 wide
    (70, 1026, 64, 128),              # rows 4-byte aligned, 4 vectors per lane, last block column 2 wide
    (40, 301, 16, 128),               # one vector per lane, last block column 45 wide (a partial vector in the middle of the row)
    (33, 129, 1, 128),                # one-row blocks, last block column 1 wide
    (129, 127, 128, 128),             # a tensor narrower than the block
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("mode", [1, 101, 2, 3])
@pytest.mark.parametrize("sf", [1, 2])
def test_shapes_modes_vs_oracle(G, shape, mode, sf):
    rows, cols, br, bc = shape
    a = data_gen.c2_student_t(rows, cols, seed=rows * 7 + cols)
    a[0, : min(32, cols)] = 0                      # a zero block / zero elements
    if rows > 2:
        a[2, 0] = 0x8000                            # negative zero
    print("shape", shape, mode, sf, flush=True)
    out, meta = G.fake_quantize(a, br, bc, 1e-15, mode, sf)
    want, wmeta, stats = O.fake_quantize(a, br, bc, 1e-15, mode, sf, want_stats=True)
    # no change in format choice: the decisions are the oracle's in every block (none of these seeded cases holds a
    # block whose two error sums tie to within their own summation noise)
    assert np.array_equal(meta, wmeta), (int((meta != wmeta).sum()), stats[..., 2][meta != wmeta], stats[..., 3][meta != wmeta])
    assert_same(out, want, f"{shape} mode {mode} sf {sf}")


@pytest.mark.parametrize("mode,fmax", [(4, 448.0), (5, 57344.0)])
@pytest.mark.parametrize("sf", [1, 2])
@pytest.mark.parametrize("shape", [(256, 256), (33, 77)])
def test_current_scaling(G, mode, fmax, sf, shape):
    a = uniform_bits(5 + mode, shape[0], shape[1], -53768.0, 53768.0)
    amax = float(E.bits_to_bf16(a).float().abs().max())
    for scale in (float(np.float32(fmax) / np.float32(amax)), float(np.float32(fmax) / np.float32(amax)) * 3.7):
        print("current scaling", mode, sf, shape, scale, flush=True)
        out, meta = G.fake_quantize(a, 128, 128, scale, mode, sf)
        want, wmeta = O.fake_quantize(a, 128, 128, scale, mode, sf)
        assert np.array_equal(meta, wmeta)
        assert_same(out, want, "current scaling")


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2, O.E3M2, O.E2M3])
@pytest.mark.parametrize("sf", [1, 2])
@pytest.mark.parametrize("shape", [(64, 512, 1, 32), (256, 256, 128, 128), (37, 45, 16, 32)])
def test_block_format(G, fmt, sf, shape):
    rows, cols, br, bc = shape
    a = data_gen.c2_student_t(rows, cols, seed=fmt * 13 + sf)
    print("block_format", fmt, sf, shape, flush=True)
    out = G.block_format(a, br, bc, fmt, sf)
    assert_same(out, O.block_format(a, br, bc, fmt, sf), "block_format")


@pytest.mark.parametrize("flags", [1, 2])
@pytest.mark.parametrize("mode,sf,shape", [(1, 1, (256, 256, 128, 128)), (2, 2, (64, 512, 1, 32)), (3, 1, (32, 4096, 1, 4096)),
                                           (1, 2, (256, 256, 128, 128)), (2, 1, (37, 45, 16, 32))])
def test_flavours(G, flags, mode, sf, shape):
    """flag 1: torch-emulation flavour == oracle EMU flavour; flag 2: software casts == hardware casts."""
    rows, cols, br, bc = shape
    a = data_gen.c4_mixture(rows, cols, seed=mode * 5 + sf, tile=64)
    print("flavour", flags, mode, sf, shape, flush=True)
    out, meta = G.fake_quantize(a, br, bc, 1e-15, mode, sf, flags=flags)
    want, wmeta = O.fake_quantize(a, br, bc, 1e-15, mode, sf, flavour=O.EMU if flags == 1 else O.KERNEL)
    assert np.array_equal(meta, wmeta)
    assert_same(out, want, "flavour")


def test_inplace_and_stats(G):
    a = data_gen.c4_mixture(512, 512, seed=77)
    x = G.to_dev_u16(a)
    out, meta = G.fake_quantize(a, 128, 128, 1e-15, 1, 1)
    out2, meta2 = G.fake_quantize(a, 128, 128, 1e-15, 1, 1, inplace=True, x_dev=x)
    assert np.array_equal(meta, meta2) and np.array_equal(out, out2)
    st = G.mor_stats(a, 128, 128, 1e-15, 1, 1)
    _, _, want = O.fake_quantize(a, 128, 128, 1e-15, 1, 1, want_stats=True)
    assert np.array_equal(st[..., 0], want[..., 0]) and np.array_equal(st[..., 1], want[..., 1])
    np.testing.assert_allclose(st[..., 2:], want[..., 2:], rtol=1e-6, atol=0)
    amax, scale, e8 = G.block_stats(a, 1, 32, 448.0)
    wa, ws, we = O.block_stats(a, 1, 32, 448.0)
    assert np.array_equal(amax, wa) and np.array_equal(scale.view(np.uint32), ws.view(np.uint32)) and np.array_equal(e8, we)


def test_large_blocks_inplace_and_stats(G):
    a = data_gen.c4_mixture(512, 1024, seed=78)
    x = G.to_dev_u16(a)
    out, meta = G.fake_quantize(a, 256, 256, 1e-15, 1, 1)
    want, wmeta, wstats = O.fake_quantize(a, 256, 256, 1e-15, 1, 1, want_stats=True)
    assert np.array_equal(meta, wmeta)
    assert_same(out, want, "large blocks")
    out2, meta2 = G.fake_quantize(a, 256, 256, 1e-15, 1, 1, inplace=True, x_dev=x)
    assert np.array_equal(meta, meta2) and np.array_equal(out, out2)
    st = G.mor_stats(a, 256, 256, 1e-15, 1, 1)
    assert np.array_equal(st[..., 0], wstats[..., 0]) and np.array_equal(st[..., 1], wstats[..., 1])
    np.testing.assert_allclose(st[..., 2:], wstats[..., 2:], rtol=1e-6, atol=0)


def test_extreme_exponents(G):
    """Blocks whose scale exponent is outside the fast-path range, bf16 denormals and the largest finite values."""
    rng = np.random.default_rng(5)
    a = np.zeros((8, 256), np.uint16)
    a[0] = rng.integers(0x0001, 0x0080, 256)            # denormals only
    a[1] = rng.integers(0x0001, 0x0400, 256)            # denormals and tiny normals
    a[2] = rng.integers(0x7E00, 0x7F80, 256)            # near the top of the range
    a[3] = rng.integers(0x0000, 0x7F80, 256)            # everything finite, positive
    a[4] = rng.integers(0x8000, 0xFF80, 256)            # everything finite, negative
    a[5] = rng.integers(0x0080, 0x1000, 256)
    a[6] = rng.integers(0x7000, 0x7F80, 256)
    a[7, ::2] = rng.integers(0x0001, 0x7F80, 128)
    wide = np.zeros((8, 2048), np.uint16)                # rows of 1024 / 2048 elements: blocks spanning 2 / 4 waves
    for r in range(8):
        wide[r] = np.tile(a[r], 8)
    for (br, bc) in ((1, 1024), (1, 2048)):
        for mode, sf in ((2, 1), (2, 2), (3, 1), (3, 2)):
            print("extreme wide", br, bc, mode, sf, flush=True)
            out, meta = G.fake_quantize(wide, br, bc, 1e-15, mode, sf)
            want, wmeta = O.fake_quantize(wide, br, bc, 1e-15, mode, sf)
            assert np.array_equal(meta, wmeta), (br, bc, mode, sf)
            assert_same(out, want, f"extreme wide {br}x{bc} mode {mode} sf {sf}")
    huge = np.zeros((16, 32768), np.uint16)              # rows of 32768 elements, and two of them per block
    for r in range(16):
        huge[r] = np.tile(a[r % 8], 128)
    for (br, bc) in ((1, 32768), (2, 32768)):
        for mode, sf in ((2, 1), (2, 2), (3, 1), (3, 2), (1, 1), (1, 2), (101, 2)):
            print("extreme huge", br, bc, mode, sf, flush=True)
            out, meta = G.fake_quantize(huge, br, bc, 1e-15, mode, sf)
            want, wmeta = O.fake_quantize(huge, br, bc, 1e-15, mode, sf)
            assert np.array_equal(meta, wmeta), (br, bc, mode, sf)
            assert_same(out, want, f"extreme huge {br}x{bc} mode {mode} sf {sf}")
    for (br, bc) in ((1, 32), (1, 256), (8, 256)):
        for mode, sf in ((2, 1), (2, 2), (3, 1), (3, 2), (1, 1), (1, 2), (101, 2)):
            print("extreme", br, bc, mode, sf, flush=True)
            out, meta = G.fake_quantize(a, br, bc, 1e-15, mode, sf)
            want, wmeta = O.fake_quantize(a, br, bc, 1e-15, mode, sf)
            assert np.array_equal(meta, wmeta), (br, bc, mode, sf)
            assert_same(out, want, f"extreme {br}x{bc} mode {mode} sf {sf}")


@pytest.mark.parametrize("br,bc", [(1, 32), (128, 128), (1, 512), (128, 256)])
@pytest.mark.parametrize("mode,sf", [(1, 1), (2, 2), (3, 1)])
def test_nan_and_inf_elements_stay_inside_their_block(G, br, bc, mode, sf):
    """NaN / Inf inputs have no pinned reference result; what is asserted: the call completes and every block without
    such an element is bit-equal to the oracle's."""
    a = data_gen.c1_normal(256, 512, seed=91)
    special = [(3, 5, 0x7FC0), (3, 6, 0xFFC0), (140, 300, 0x7F80), (200, 40, 0xFF80), (17, 490, 0x7FFF)]
    for r, c, bits in special:
        a[r, c] = bits
    out, meta = G.fake_quantize(a, br, bc, 1e-15, mode, sf)
    want, wmeta = O.fake_quantize(a, br, bc, 1e-15, mode, sf)
    clean = np.ones((256 // br, 512 // bc), bool)
    for r, c, _ in special:
        clean[r // br, c // bc] = False
    mask = np.repeat(np.repeat(clean, br, 0), bc, 1)
    assert np.array_equal(out[mask], want[mask])
    assert np.array_equal(meta[clean], wmeta[clean])


@pytest.mark.parametrize("offset", [1, 3, 4, 7])
@pytest.mark.parametrize("inplace", [False, True])
def test_tensor_that_does_not_start_on_a_vector_boundary(G, offset, inplace):
    """A tensor `offset` elements into an allocation (128-wide blocks, column count a multiple of 8): input and output
    rows start `offset` elements past 16-byte boundaries; what lies before and after the tensor stays as it was."""
    from mor_amd import _cabi
    L = _cabi.lib()
    rows, cols = 150, 264
    a = data_gen.c2_student_t(rows, cols, seed=90 + offset)
    a[3, 5] = 0x7FC0                                           # a NaN: its block takes the exact path
    pad = 24
    buf = torch.full((offset + rows * cols + pad,), 3.0, dtype=torch.bfloat16, device=G.dev())
    x = buf[offset:offset + rows * cols]
    x.copy_(G.to_dev_u16(a).flatten())
    obuf = buf if inplace else torch.full_like(buf, 5.0)
    o = obuf[offset:offset + rows * cols]
    meta = torch.full((2, 3), -7, dtype=torch.int32, device=G.dev())
    for mode in (1, 2):
        if inplace:
            x.copy_(G.to_dev_u16(a).flatten())
        print("offset tensor", offset, inplace, mode, flush=True)
        _cabi.check(L.mor_fake_quantize(x.data_ptr(), o.data_ptr(), meta.data_ptr(), rows, cols, 128, 128, 1e-15, mode, 1, 0, G.stream_ptr()))
        torch.cuda.synchronize()
        want, wmeta = O.fake_quantize(a, 128, 128, 1e-15, mode, 1)
        assert np.array_equal(meta.cpu().numpy(), wmeta)
        assert_same(G.to_host_u16(o).reshape(rows, cols), want, f"offset {offset} mode {mode}")
        fill = 3.0 if inplace else 5.0
        assert bool((obuf[:offset] == fill).all()) and bool((obuf[offset + rows * cols:] == fill).all()), "wrote outside the tensor"
