"""The known answers of tests/golden/scalar_vectors.npz (exact-rational / integer models of the formats and of the
reference's bit rules, made by tests/golden/make_scalar_vectors.py) against the CPU oracle and, on the GPU, against the
HIP library through the C ABI."""
import os

import numpy as np
import pytest
import torch

from oracle import mor_oracle as O

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "scalar_vectors.npz"))
FMT = {"e4m3": O.E4M3, "e5m2": O.E5M2, "e3m2": O.E3M2, "e2m3": O.E2M3}
NAN_BITS = 0x7FFFFFFF


def same_bits(got_f32, want_bits):
    got = np.ascontiguousarray(got_f32, np.float32).view(np.uint32)
    nan = want_bits == NAN_BITS
    assert np.all(np.isnan(got_f32[nan]))
    assert np.array_equal(got[~nan], want_bits[~nan])


def test_decode_tables_are_the_torch_float8_values():
    """The tables themselves against a library routine: torch's float8 decode of every code."""
    for name, dtype in (("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)):
        want = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(dtype).float().numpy()
        got = V[f"decode_{name}"].view(np.float32)
        fin = np.isfinite(want)
        assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32))
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))
    assert V["decode_e2m3"].view(np.float32)[31] == 7.5 and V["decode_e3m2"].view(np.float32)[31] == 28.0
    assert V["decode_e2m3"].view(np.float32)[1] == 0.125 and V["decode_e3m2"].view(np.float32)[1] == 0.0625


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e3m2", "e2m3"])
def test_oracle_software_cast(fmt):
    same_bits(O.cast_sw(V["cast_x"].view(np.float32), FMT[fmt]), V[f"cast_sw_{fmt}"])


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_oracle_hardware_cast_model(fmt):
    same_bits(O.cast_hw(V["cast_x"].view(np.float32), FMT[fmt]), V[f"cast_hw_{fmt}"])


def scale_groups():
    x, s = V["sqdd_x"], V["sqdd_s"]
    for sb in np.unique(s):
        sel = s == sb
        yield float(np.array([sb], np.uint32).view(np.float32)[0]), x[sel].reshape(1, -1), sel


@pytest.mark.parametrize("fmt,mode", [("e4m3", 4), ("e5m2", 5)])
@pytest.mark.parametrize("sf,key", [(1, "fp32"), (2, "e8")])
def test_oracle_scale_cast_descale(fmt, mode, sf, key):
    """Current-scaling modes take the scale from clamp_threshold (FQ:825-842): scale -> cast -> descale per element."""
    for scale, x, sel in scale_groups():
        got, _ = O.fake_quantize(x, 1, x.shape[1], scale, mode, sf)
        assert np.array_equal(got.ravel(), V[f"sqdd_{key}_{fmt}"][sel]), (scale, fmt, key)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,mode", [("e4m3", 4), ("e5m2", 5)])
@pytest.mark.parametrize("sf,key", [(1, "fp32"), (2, "e8")])
def test_gpu_scale_cast_descale(fmt, mode, sf, key):
    import gpu_util as G
    for scale, x, sel in scale_groups():
        got, _ = G.fake_quantize(x, 1, x.shape[1], scale, mode, sf)
        want = V[f"sqdd_{key}_{fmt}"][sel]
        bad = np.flatnonzero(got.ravel() != want)
        assert len(bad) == 0, (scale, fmt, key, hex(x.ravel()[bad[0]]), hex(got.ravel()[bad[0]]), hex(want[bad[0]]))


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e3m2", "e2m3"])
def test_gpu_software_cast_ops(fmt):
    import gpu_util as G
    same_bits(G.quant_dequant(V["cast_x"].view(np.float32), FMT[fmt]), V[f"cast_sw_{fmt}"])
