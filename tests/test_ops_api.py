"""The drop-in boundary without a GPU: `import mor` works, the 14 schemas match the reference text, argument checks raise."""
import inspect

import pytest
import torch

import mor

# mor/csrc/fake_quantize.cpp:12-25, verbatim
SCHEMAS = {
    "fake_quantize": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float clamp_threshold, int mode, int sf_type) -> Tensor[]",
    "fake_quantize_no_alloc": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float clamp_threshold, int mode, int sf_type, Tensor result) -> Tensor",
    "quant_dequant_e4m3": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor",
    "quant_dequant_e5m2": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor",
    "quant_dequant_e3m2": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor",
    "quant_dequant_e2m3": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor",
    "e4m3_with_e8_scale_rne": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor",
    "e4m3_with_e8_scale_rz": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y) -> Tensor",
    "fake_quantize_block_scaling": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float e4m3_threshold, int ss_mode) -> Tensor[]",
    "fake_quantize_block_scaling_inplace": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float e4m3_threshold, int ss_mode) -> Tensor[]",
    "fake_quantize_e8mx": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y, int quantize_type, int scaling_strategy) -> Tensor",
    "fake_quantize_e8mx_inplace": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y, int quantize_type, int scaling_strategy, Tensor result) -> ()",
    "fake_quantize_channel_scaling": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float e4m3_threshold, int ss_mode) -> Tensor[]",
    "fake_quantize_channel_scaling_inplace": "(Tensor input, int dim_x, int dim_y, int block_x, int block_y, float e4m3_threshold, int ss_mode) -> Tensor[]",
}

# positional / keyword names of mor/ops.py
PY_ARGS = {
    "fake_quantize": ["a", "dim_x", "dim_y", "block_x", "block_y", "clamp_threshold", "mode", "sf_type"],
    "fake_quantize_no_alloc": ["a", "dim_x", "dim_y", "block_x", "block_y", "clamp_threshold", "mode", "sf_type", "output"],
    "fake_quantize_block_scaling": ["a", "dim_x", "dim_y", "block_x", "block_y", "e4m3_threshold", "ss_mode"],
    "fake_quantize_block_scaling_inplace": ["a", "dim_x", "dim_y", "block_x", "block_y", "e4m3_threshold", "ss_mode"],
    "fake_quantize_channel_scaling": ["a", "dim_x", "dim_y", "block_x", "block_y", "e4m3_threshold", "ss_mode"],
    "fake_quantize_channel_scaling_inplace": ["a", "dim_x", "dim_y", "block_x", "block_y", "e4m3_threshold", "ss_mode"],
    "fake_quantize_e8mx": ["a", "dim_x", "dim_y", "block_x", "block_y", "quantize_type", "scaling_strategy"],
    "fake_quantize_e8mx_inplace": ["a", "dim_x", "dim_y", "block_x", "block_y", "quantize_type", "scaling_strategy", "output"],
    "quant_dequant_e4m3": ["a", "dim_x", "dim_y", "block_x", "block_y"],
    "quant_dequant_e5m2": ["a", "dim_x", "dim_y", "block_x", "block_y"],
    "quant_dequant_e2m3": ["a", "dim_x", "dim_y", "block_x", "block_y"],
    "quant_dequant_e3m2": ["a", "dim_x", "dim_y", "block_x", "block_y"],
    "e4m3_with_e8_scale_rne": ["a", "dim_x", "dim_y", "block_x", "block_y"],
    "e4m3_with_e8_scale_rz": ["a", "dim_x", "dim_y", "block_x", "block_y"],
}


def test_schemas_match_reference_text():
    for name, sig in SCHEMAS.items():
        op = getattr(torch.ops.mor, name).default
        assert str(op._schema) == f"mor::{name}{sig}", str(op._schema)


def test_python_api_names_and_arguments():
    assert hasattr(mor, "ops") and hasattr(mor, "_C")
    for name, args in PY_ARGS.items():
        fn = getattr(mor.ops, name)
        assert list(inspect.signature(fn).parameters) == args, name


def test_cpu_tensors_are_rejected_as_in_the_reference():
    x = torch.zeros(4, 8, dtype=torch.bfloat16)
    with pytest.raises((NotImplementedError, RuntimeError)):
        mor.ops.fake_quantize(x, 4, 8, 4, 8, 0.0, 2, 1)


def test_fake_tensor_shapes_without_a_gpu():
    """Shape propagation (what torch.compile / export trace through) needs no device: meta and fake tensors."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    x = torch.empty(300, 520, dtype=torch.bfloat16, device="meta")
    out, meta = mor.ops.fake_quantize(x, 300, 520, 128, 128, clamp_threshold=1e-15, mode=1, sf_type=1)
    assert out.shape == x.shape and out.dtype == torch.bfloat16
    assert meta.shape == (3, 5) and meta.dtype == torch.int32
    for op in (mor.ops.fake_quantize_block_scaling, mor.ops.fake_quantize_channel_scaling):
        res = op(x, 300, 520, 1, 520, e4m3_threshold=0.045, ss_mode=3)
        assert [tuple(t.shape) for t in res] == [(300, 520), (1,), (1,), (1,), (1,)]
        assert [t.dtype for t in res] == [torch.bfloat16, torch.int32, torch.float32, torch.int32, torch.float32]
    assert mor.ops.fake_quantize_e8mx(x, 300, 520, 128, 128, quantize_type=2, scaling_strategy=1).shape == x.shape
    f = torch.empty(16, 32, dtype=torch.float32, device="meta")
    for name in ("quant_dequant_e4m3", "quant_dequant_e5m2", "quant_dequant_e2m3", "quant_dequant_e3m2",
                 "e4m3_with_e8_scale_rne", "e4m3_with_e8_scale_rz"):
        r = getattr(mor.ops, name)(f, 16, 32, 16, 32)
        assert r.shape == f.shape and r.dtype == torch.float32
    with FakeTensorMode():
        y = torch.empty(256, 256, dtype=torch.bfloat16, device="cuda")
        out, meta = mor.ops.fake_quantize(y, 256, 256, 128, 128, 1e-15, 1, 1)
        assert out.device.type == "cuda" and meta.shape == (2, 2)


def test_mutating_ops_have_no_fake_kernel():
    """The ops that write into an argument keep the reference's schemas, which declare no aliasing: a fake kernel would
    let a tracing compiler treat them as pure and drop the writes, so there is none and tracing them fails loudly
    (their Python entry points are excluded from compilation and run eagerly instead)."""
    x = torch.empty(64, 64, dtype=torch.bfloat16, device="meta")
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.mor.fake_quantize_no_alloc.default(x, 64, 64, 1, 32, 0.0, 2, 2, x)
    for op in (torch.ops.mor.fake_quantize_block_scaling_inplace, torch.ops.mor.fake_quantize_channel_scaling_inplace):
        with pytest.raises((NotImplementedError, RuntimeError)):
            op.default(x, 64, 64, 1, 64, 0.045, 3)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.mor.fake_quantize_e8mx_inplace.default(x, 64, 64, 32, 32, 2, 1, x)


def test_import_fails_loudly_without_the_host_library():
    """libmor_torch.so is the only implementation behind the operators: when it is absent the import raises instead of
    registering anything else (run in a child process that hides the file from os.path.exists)."""
    import subprocess
    import sys
    code = (
        "import os, sys\n"
        "real = os.path.exists\n"
        "os.path.exists = lambda p: False if str(p).endswith('libmor_torch.so') else real(p)\n"
        "try:\n"
        "    import mor\n"
        "except ImportError as e:\n"
        "    assert 'libmor_torch.so' in str(e), e\n"
        "    sys.exit(42)\n"
        "sys.exit(0)\n"
    )
    root = __import__("os").path.dirname(__import__("os").path.dirname(__import__("os").path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 42, (r.returncode, r.stderr[-400:])
