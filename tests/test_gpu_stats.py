"""The statistics line of a GPU tensor: scalars from the block-scaling op (HIP), histogram over its blocks."""
import numpy as np
import pytest
import torch

from oracle import mor_oracle as O

pytestmark = pytest.mark.gpu


def test_tensor_log_line_matches_oracle_scalars():
    from mor_amd import stats
    g = torch.Generator().manual_seed(77)
    x = torch.randn(512, 768, generator=g)
    x[:128, :128] *= 50.0
    x[5, :40] = 0
    xb = x.to(torch.bfloat16)
    a = xb.view(torch.int16).numpy().view(np.uint16).copy()
    print("stats line 512x768", flush=True)
    line = stats.tensor_log_line(3, "layers.0.attn.qkv.weight", 10, 2, xb.cuda())
    import log_line_fields
    p = log_line_fields.parse(line)
    _, _, _, wnnz, werr = O.block_scaling(a, 128, 128, 1.0e30, 3)
    assert p["node_id"] == 3 and p["tensor_name"] == "layers.0.attn.qkv.weight" and p["counter"] == 10 and p["step"] == 2
    assert p["tensor_dimension"] == "512x768" and p["global_non_zero"] == int(wnnz[0]) == int((xb != 0).sum())
    assert p["global_error"] == pytest.approx(float(werr[0]), rel=1e-6)
    assert p["relative_error"] == pytest.approx(float(werr[0]) / int(wnnz[0]), rel=1e-5)
    assert sum(p["histogram"]) == 4 * 6 and len(p["histogram"]) == stats.NUM_BINS
    # E4M3 relative error is at most 2^-4 in its normal range and about 0.03 on average: nothing in the last bin here
    assert p["histogram"][-1] == 0 and sum(p["histogram"][3:9]) == 24
