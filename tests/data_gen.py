"""Seeded synthetic inputs of the benchmark configurations (bf16 bit patterns as numpy uint16).

Shapes can be scaled down for tests; the distributions are those of the configurations:
C1 N(0,1); C2 Student-t(3) * 0.02 with 0.1 % outliers x1000; C3 N(0, 0.02) rows with 1 % rows x100 and a zero row;
C4 per-128x128-tile mixture (70 % N(0,1), 20 % +-exp(3 N(0,1)), 10 % N(0,1) * 1e-4).
"""
import numpy as np
import torch


def _bits(t):
    return t.to(torch.bfloat16).contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def c1_normal(rows=4096, cols=4096, seed=1001, as_tensor=False):
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(rows, cols, generator=g)
    return t.to(torch.bfloat16) if as_tensor else _bits(t)


def c2_student_t(rows=8192, cols=8192, seed=1002, as_tensor=False):
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(rows, cols, generator=g)
    d = torch.zeros(rows, cols)
    for _ in range(3):
        d += torch.randn(rows, cols, generator=g) ** 2
    t = z / torch.sqrt(d / 3) * 0.02
    del z, d
    mask = torch.rand(rows, cols, generator=g) < 1e-3
    t = torch.where(mask, t * 1000, t)
    return t.to(torch.bfloat16) if as_tensor else _bits(t)


def c3_weights(rows=16384, cols=4096, seed=1003, as_tensor=False):
    g = torch.Generator().manual_seed(seed)
    t = torch.randn(rows, cols, generator=g) * 0.02
    hot = torch.randperm(rows, generator=g)[: max(1, rows // 100)]
    t[hot] *= 100
    t[min(7, rows - 1)] = 0
    return t.to(torch.bfloat16) if as_tensor else _bits(t)


def c4_mixture(rows=16384, cols=14336, seed=1004, tile=128, as_tensor=False):
    g = torch.Generator().manual_seed(seed)
    gy, gx = (rows + tile - 1) // tile, (cols + tile - 1) // tile
    u = torch.rand(gy, gx, generator=g)
    t = torch.randn(rows, cols, generator=g)
    kind = torch.where(u < 0.7, 0, torch.where(u < 0.9, 1, 2))
    kind_e = kind.repeat_interleave(tile, 0).repeat_interleave(tile, 1)[:rows, :cols]
    sign = torch.where(torch.rand(rows, cols, generator=g) < 0.5, -1.0, 1.0)
    t = torch.where(kind_e == 1, torch.exp(3 * t) * sign, torch.where(kind_e == 2, t * 1e-4, t))
    return t.to(torch.bfloat16) if as_tensor else _bits(t)


def tile_mixture(rng, rows, cols):
    """tiles of every kind MoR tells apart: narrow range, moderate, wide, outliers, tiny, zero, out of the fast range"""
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    kinds = rng.integers(0, 8, (rows // 128, cols // 128))
    for by in range(rows // 128):
        for bx in range(cols // 128):
            t = x[by * 128:(by + 1) * 128, bx * 128:(bx + 1) * 128]
            k = kinds[by, bx]
            if k == 0:
                t[:] = 1.0 + 0.3 * rng.random((128, 128))                       # range <= 7.5: E2M3
            elif k == 1:
                t *= np.exp(4 * rng.standard_normal((128, 128)))               # wide: the error sums decide
            elif k == 2:
                t[rng.random((128, 128)) < 0.01] *= 3000                      # outliers
            elif k == 3:
                t *= 1e-5
            elif k == 4:
                t[:] = 0
            elif k == 5:
                t *= 1e-33                                                    # scale outside the fast range
            elif k == 6:
                t[rng.random((128, 128)) < 0.3] = 0
    return torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()
