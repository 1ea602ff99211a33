"""mor_fake_quantize_batch: a list of tensors in one call must give, tensor by tensor, the bits of the CPU oracle
(and so of mor_fake_quantize), whatever mix of shapes, block shapes and sizes the list holds."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import mor_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def bits(rng, rows, cols, kind):
    if kind == 0:
        x = rng.standard_normal((rows, cols)).astype(np.float32)
    elif kind == 1:
        x = (rng.standard_t(3, (rows, cols)) * 0.02).astype(np.float32)
        x[rng.random((rows, cols)) < 1e-2] *= 1000
    elif kind == 2:
        x = (np.exp(3 * rng.standard_normal((rows, cols))) * rng.choice([-1.0, 1.0], (rows, cols))).astype(np.float32)
        x[rng.random((rows, cols)) < 0.05] = 0
    else:
        x = np.zeros((rows, cols), dtype=np.float32)
    return torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()


def run_batch(G, arrays, blocks, clamp, mode, sf, flags=0, inplace=False):
    return G.fake_quantize_batch(arrays, blocks, clamp, mode, sf, flags, inplace)


def check_against_oracle(arrays, blocks, clamp, mode, sf, got, flavour=O.KERNEL):
    for i, (a, (br, bc), (out, meta)) in enumerate(zip(arrays, blocks, got)):
        want_out, want_meta = O.fake_quantize(a, br, bc, clamp, mode, sf, flavour)
        assert np.array_equal(meta, want_meta), f"tensor {i} {a.shape} blocks {br}x{bc} mode {mode} sf {sf}: meta differs"
        assert np.array_equal(out, want_out), f"tensor {i} {a.shape} blocks {br}x{bc} mode {mode} sf {sf}: output differs"


@pytest.mark.parametrize("mode,sf", [(1, 1), (1, 2), (101, 1), (2, 1), (2, 2), (3, 1), (3, 2), (4, 1), (5, 2), (7, 1)])
def test_hundred_tiny_tensors(G, mode, sf):
    """100 tensors of one 1 x 32 block each: two launches instead of a hundred"""
    rng = np.random.default_rng(400 + mode * 3 + sf)
    arrays = [bits(rng, 1, 32, i % 4) for i in range(100)]
    blocks = [(1, 32)] * 100
    clamp = 0.37 if mode in (4, 5) else 1e-3
    check_against_oracle(arrays, blocks, clamp, mode, sf, run_batch(G, arrays, blocks, clamp, mode, sf))


SHAPES = [((1, 32), (1, 32)), ((33, 17), (5, 7)), ((64, 64), (16, 16)), ((7, 129), (1, 32)), ((128, 128), (128, 128)),
          ((300, 200), (128, 128)), ((1, 1), (1, 1)), ((17, 40), (32, 64)), ((512, 512), (1, 32)), ((256, 1024), (64, 64)),
          ((1024, 1024), (128, 128)), ((3, 5), (1000000000000, 3)), ((96, 100), (1, 100)), ((2048, 1024), (1, 32))]


@pytest.mark.parametrize("mode,sf", [(1, 1), (1, 2), (101, 2), (2, 1), (3, 2), (4, 2), (5, 1), (6, 1)])
def test_mixed_list(G, mode, sf):
    """small and large tensors, ragged edges, blocks larger than the tensor, in one list (more than one launch's worth)"""
    rng = np.random.default_rng(900 + mode * 3 + sf)
    arrays, blocks = [], []
    for rep in range(5):
        for (shape, blk) in SHAPES:
            if rep and shape[0] * shape[1] > 1 << 18:
                continue                      # the large ones once
            arrays.append(bits(rng, shape[0], shape[1], int(rng.integers(3))))
            blocks.append(blk)
    clamp = 2.5 if mode in (4, 5) else 0.05
    check_against_oracle(arrays, blocks, clamp, mode, sf, run_batch(G, arrays, blocks, clamp, mode, sf))


def test_emulation_flavour_and_inplace(G):
    from mor_amd import _cabi
    rng = np.random.default_rng(77)
    arrays = [bits(rng, r, c, k % 3) for k, (r, c) in enumerate([(4, 64), (33, 17), (1, 32), (64, 96)] * 8)]
    blocks = [(1, 32), (5, 7), (1, 32), (16, 32)] * 8
    got = run_batch(G, arrays, blocks, 1e-3, 1, 2, flags=_cabi.FLAG_TORCH_EMULATION)
    check_against_oracle(arrays, blocks, 1e-3, 1, 2, got, flavour=O.EMU)
    got = run_batch(G, arrays, blocks, 1e-3, 2, 1, inplace=True)
    check_against_oracle(arrays, blocks, 1e-3, 2, 1, got)


def test_list_helper_matches_the_op(G):
    """mor_amd.batch.fake_quantize_batch == [mor.ops.fake_quantize(x, ...) for x in xs]"""
    import mor_amd
    rng = np.random.default_rng(5)
    shapes = [(1, 32), (8, 64), (33, 48), (256, 256), (1024, 512)] * 3
    blocks = [(1, 32), (1, 32), (4, 16), (128, 128), (1, 64)] * 3
    xs = [G.to_dev_u16(bits(rng, r, c, 1)) for r, c in shapes]
    for mode, sf in [(1, 1), (2, 2)]:
        got = mor_amd.batch.fake_quantize_batch(xs, blocks, 1e-3, mode, sf)
        assert len(got) == len(xs)
        for x, (br, bc), (out, meta) in zip(xs, blocks, got):
            want_out, want_meta = mor_amd.ops.fake_quantize(x, x.shape[0], x.shape[1], br, bc, 1e-3, mode, sf)
            assert torch.equal(out.view(torch.int16), want_out.view(torch.int16))
            assert torch.equal(meta, want_meta.view(meta.shape))
    ys = [x.clone() for x in xs]
    got = mor_amd.batch.fake_quantize_batch(ys, blocks, 1e-3, 3, 1, inplace=True)
    for x, y, (br, bc), (out, meta) in zip(xs, ys, blocks, got):
        assert out.data_ptr() == y.data_ptr()
        want_out, _ = mor_amd.ops.fake_quantize(x, x.shape[0], x.shape[1], br, bc, 1e-3, 3, 1)
        assert torch.equal(y.view(torch.int16), want_out.view(torch.int16))
    assert mor_amd.batch.fake_quantize_batch([], [], 0.0, 1, 1) == []


def test_a_bad_descriptor_stops_the_call_before_any_launch(G):
    from mor_amd import _cabi
    from mor_amd.batch import TensorDesc
    L = _cabi.lib()
    x = torch.ones((4, 32), dtype=torch.bfloat16, device=G.dev())
    y = torch.zeros_like(x)
    m = torch.full((4, 1), -7, dtype=torch.int32, device=G.dev())
    descs = (TensorDesc * 2)()
    for d in descs:
        d.input, d.output, d.meta = x.data_ptr(), y.data_ptr(), m.data_ptr()
        d.rows, d.cols, d.block_rows, d.block_cols = 4, 32, 1, 32
        d.clamp_threshold, d.mode, d.sf_type = 0.0, 2, 1
    descs[1].block_cols = 0
    assert L.mor_fake_quantize_batch(descs, 2, 0, G.stream_ptr()) != 0
    assert b"block dims" in L.mor_last_error()
    torch.cuda.synchronize()
    assert (m.cpu().numpy() == -7).all() and float(y.float().abs().sum()) == 0.0


@pytest.mark.parametrize("mode,sf", [(1, 1), (1, 2), (101, 1), (2, 1), (2, 2), (3, 1)])
@pytest.mark.parametrize("inplace", [False, True])
def test_tensors_in_whole_tiles_share_launches(G, mode, sf, inplace):
    """Tensors in whole 128 x 128 tiles beyond the small-tensor limit: their tiles run as one grid of the tile kernel
    (several streaming classes, grids with and without the band order, a tensor that is not in whole tiles and a small
    one in between); every tensor must come out as the oracle gives it."""
    rng = np.random.default_rng(1300 + mode * 3 + sf)
    shapes = [(512, 1024), (1024, 256), (2048, 1024), (640, 896), (4096, 1024), (384, 768), (1000, 520), (128, 128),
              (1024, 2048), (2304, 2176)]
    arrays = [bits(rng, r, c, i % 3) for i, (r, c) in enumerate(shapes)]
    arrays[2][:128, :128] = 0                                      # a zero tile
    arrays[4][130, 5] = 0x7FC0                                     # a NaN: its tile takes the exact path
    arrays[0][:128, 128:256] = bits(rng, 128, 128, 0) & 0x807F     # a tile of tiny values: scale outside the fast range
    blocks = [(128, 128)] * len(shapes)
    got = run_batch(G, arrays, blocks, 1e-3, mode, sf, inplace=inplace)
    check_against_oracle(arrays, blocks, 1e-3, mode, sf, got)


def test_fifty_tile_tensors_take_two_launches(G):
    """more tensors than one launch of the tile kernel holds (48), every one as from a call of its own"""
    rng = np.random.default_rng(77)
    shapes = [(512, 640)] * 25 + [(768, 512)] * 25
    arrays = [bits(rng, r, c, i % 3) for i, (r, c) in enumerate(shapes)]
    blocks = [(128, 128)] * len(shapes)
    got = run_batch(G, arrays, blocks, 1e-3, 1, 1)
    singles = [G.fake_quantize(a, 128, 128, 1e-3, 1, 1) for a in arrays]
    for i, ((out, meta), (want, wmeta)) in enumerate(zip(got, singles)):
        assert np.array_equal(meta, wmeta) and np.array_equal(out, want), i
    check_against_oracle(arrays[:4], blocks[:4], 1e-3, 1, 1, got[:4])


@pytest.mark.parametrize("mode,sf", [(2, 1), (3, 2), (1, 1), (101, 2)])
def test_register_resident_blocks_of_every_size_share_launches(G, mode, sf):
    """Tensors beyond the small-tensor limit in whole blocks of 2048, 4096, 8192 and 16384 elements (rows, tiles of
    several shapes): a launch per size class, every tensor as the oracle gives it.  (MoR shares launches for blocks of
    16384 elements only; the other MoR tensors go through calls of their own.)"""
    rng = np.random.default_rng(1700 + mode * 3 + sf)
    cases = [((512, 4096), (1, 4096)), ((1024, 2048), (1, 2048)), ((768, 4096), (1, 4096)), ((512, 1024), (64, 64)),
             ((640, 768), (32, 64)), ((96, 16384), (1, 16384)), ((1024, 1024), (128, 128)), ((512, 2048), (64, 256)),
             ((300, 8192), (1, 8192)), ((1024, 512), (256, 64)), ((2048, 4096), (1, 4096)), ((512, 1024), (128, 64))]
    arrays = [bits(rng, r, c, i % 3) for i, ((r, c), _) in enumerate(cases)]
    arrays[0][3] = 0                                               # a zero row
    arrays[2][5, 7] = 0x7FC0                                       # a NaN
    blocks = [b for _, b in cases]
    got = run_batch(G, arrays, blocks, 1e-3, mode, sf)
    check_against_oracle(arrays, blocks, 1e-3, mode, sf, got)


@pytest.mark.parametrize("flags,flavour", [(1, "EMU"), (2, "KERNEL")])
def test_other_flavours_do_not_take_the_shared_launches(G, flags, flavour):
    """With the torch-emulation flavour or the software casts, large tensors in whole tiles are forwarded to calls of
    their own (the shared launches run the default arithmetic only); the results are the flavour's."""
    rng = np.random.default_rng(2100 + flags)
    shapes = [(1024, 1024), (512, 640), (64, 64)]
    arrays = [bits(rng, r, c, i % 3) for i, (r, c) in enumerate(shapes)]
    blocks = [(128, 128), (128, 128), (16, 32)]
    for mode, sf in ((1, 1), (2, 2)):
        got = run_batch(G, arrays, blocks, 1e-3, mode, sf, flags=flags)
        check_against_oracle(arrays, blocks, 1e-3, mode, sf, got, flavour=getattr(O, flavour))
