"""The statistics log line: the reference's processor (train_logs/process_example_logs.py:38-72) must find every field."""
import pytest
import torch

import log_line_fields
from mor_amd import stats


def reference_style_parse(line):
    p = log_line_fields.parse(line)
    assert p["tensor_dimension"] is not None, line
    return (p["node_id"], p["tensor_name"], p["counter"], p["step"], p["tensor_dimension"], p["global_non_zero"],
            p["global_error"], p["relative_error"], p["histogram"])


def test_line_has_every_field_the_processor_searches_for():
    hist = [3, 0, 7] + [0] * 13
    line = stats.format_log_line(5, "decoder.layers.3.mlp.linear_fc1.weight", 1200, 37, 14336, 4096, 58720256, 1512345.25, hist)
    got = reference_style_parse(line)
    assert got[:6] == (5, "decoder.layers.3.mlp.linear_fc1.weight", 1200, 37, "14336x4096", 58720256)
    assert got[6] == pytest.approx(1512345.25) and got[7] == pytest.approx(1512345.25 / 58720256, rel=1e-6) and got[8] == hist
    assert "Tensor" in line and "at counter" in line          # the filter of process_log_file (:79)


def test_all_zero_tensor_and_bad_lines():
    line = stats.format_log_line(0, "w", 1, 1, 2, 2, 0, 0.0, [0] * 16)
    assert reference_style_parse(line)[7] == 0.0
    with pytest.raises(ValueError):
        log_line_fields.parse("3: Tensor w at counter 1 step 2 global_non_zero: 4")


def test_block_error_histogram_by_hand():
    # 2 x 2 blocks of 2 x 2: mean relative errors 0.0, 0.0125 (bin 2), 0.5 (last bin), and one all-zero block (not counted)
    x = torch.tensor([[1.0, 2.0, 4.0, 4.0],
                      [4.0, 8.0, 4.0, 0.0],
                      [2.0, 2.0, 0.0, 0.0],
                      [2.0, 2.0, 0.0, 0.0]])
    q = x.clone()
    q[0, 2] = 4.1          # 0.025
    q[1, 2] = 4.05         # 0.0125 -> block mean over 3 non-zero elements = 0.0125
    q[2, 0] = 3.0          # 0.5
    q[3, 1] = 3.0          # 0.5; block mean (0.5 + 0.5) / 4 = 0.25 -> bin 15 (everything above 0.075)
    h = stats.block_error_histogram(x, q, 2, 2)
    assert len(h) == 16 and sum(h) == 3
    assert h[0] == 1 and h[2] == 1 and h[15] == 1
