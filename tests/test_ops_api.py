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
