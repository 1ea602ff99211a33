"""Writes tests/golden/reference_fixtures.npz.

Inputs: the deterministic 256x256 matrices of the reference tests (test_fake_quantize.py:16-24 with the pokes of
:230-239, :317-329, :792-801).  Expected outputs: the torch emulation in tests/torch_emulation.py (what the reference
tests compare the CUDA kernel with) and the meta grids the reference tests assert literally (:254-269, :344-359,
:816-831).  Nothing here runs reference code or the oracle.
Usage: python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import torch_emulation as E  # noqa: E402

POKES_RANGE = [(128, 1, 18200, 50968), (0, 70, 21000, 53768), (1, 1, 17262, 50030)]
POKES_ERROR = [(128, 1, 18403, 51171), (0, 70, 21000, 53768), (1, 1, 17264, 50032)]


def main():
    out = {}
    for key, pokes, dyn, e8, meta in (
        ("range", POKES_RANGE, True, False, [[1, 3], [2, 4]]),
        ("error", POKES_ERROR, False, False, [[1, 3], [3, 4]]),
        ("range_e8", POKES_RANGE, True, True, [[1, 3], [2, 4]]),
    ):
        a = E.fixture_words(256, 256, pokes)
        emu, _ = E.mor_tensor(a, 128, 128, dyn, e8=e8)
        out[f"{key}_in"] = a
        out[f"{key}_out"] = emu
        out[f"{key}_meta"] = np.array(meta, np.int32)
    np.savez_compressed(os.path.join(HERE, "reference_fixtures.npz"), **out)


if __name__ == "__main__":
    main()
