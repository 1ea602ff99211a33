"""Per-tensor quantization statistics in the log-line format the reference's log processor reads.

The reference ships only the consumer, train_logs/process_example_logs.py: its parser (parse_log_entry, :38-72) fixes
the fields of a line,

    <node>: Tensor <name> at counter <c> step <s> tensor dimension: <rows>x<cols> global_non_zero: <n>
    global_error: <e> relative_error: <e / n> histogram [h0, h1, ...]

(one line), and its plots label histogram bin i as (i + 1) * 0.005 (:196, :244, :301) and use the first 12 bins.  The
producer is not part of the reference, so what is counted into the histogram is inferred from those labels: the number
of quantization blocks whose mean relative error lies in [i * 0.005, (i + 1) * 0.005), the last bin also taking
everything above.  The scalars are those of the block-scaling op (mor/csrc/cuda/fake_quantize.cu:1178-1241): the count
of non-zero elements, the sum of |q / x - 1| over them, and their quotient.
"""
from typing import List, Sequence

import torch
from torch import Tensor

BIN_WIDTH = 0.005
NUM_BINS = 16


def format_log_line(node_id: int, tensor_name: str, counter: int, step: int, rows: int, cols: int, global_non_zero: int,
                    global_error: float, histogram: Sequence[int]) -> str:
    rel = global_error / global_non_zero if global_non_zero else 0.0
    return (f"{node_id}: Tensor {tensor_name} at counter {counter} step {step} tensor dimension: {rows}x{cols} "
            f"global_non_zero: {global_non_zero} global_error: {global_error:.6f} relative_error: {rel:.8f} "
            f"histogram [{', '.join(str(int(h)) for h in histogram)}]")


def block_error_histogram(x: Tensor, q: Tensor, block_rows: int, block_cols: int, bin_width: float = BIN_WIDTH,
                          num_bins: int = NUM_BINS) -> List[int]:
    """Blocks per bin of their mean relative error sum(|q / x - 1| over x != 0) / count(x != 0); blocks without a
    non-zero element are not counted.  Plain torch on the tensors' device (observability, not the hot path)."""
    rows, cols = x.shape
    if rows % block_rows or cols % block_cols:
        raise RuntimeError("mor: the histogram needs whole blocks")
    xf, qf = x.float(), q.float()
    nz = xf != 0
    rel = torch.where(nz, ((qf - xf) / torch.where(nz, xf, torch.ones_like(xf))).abs(), torch.zeros_like(xf))
    gy, gx = rows // block_rows, cols // block_cols
    per_block = lambda t: t.view(gy, block_rows, gx, block_cols).sum(dim=(1, 3))
    err, cnt = per_block(rel), per_block(nz.float())
    mean = (err / cnt.clamp(min=1.0))[cnt > 0]
    bins = torch.clamp((mean / bin_width).floor().long(), 0, num_bins - 1)
    return torch.bincount(bins, minlength=num_bins).tolist()


def tensor_log_line(node_id: int, tensor_name: str, counter: int, step: int, x: Tensor, block_rows: int = 128,
                    block_cols: int = 128, ss_mode: int = 3, e4m3_threshold: float = 1.0e30) -> str:
    """One statistics line for the bf16 GPU tensor x under E4M3 block scaling (through mor.ops, i.e. the HIP library)."""
    from . import ops
    rows, cols = x.shape
    out, _meta, _amax, nnz, err = ops.fake_quantize_block_scaling(x, rows, cols, block_rows, block_cols, e4m3_threshold, ss_mode)
    hist = block_error_histogram(x, out, block_rows, block_cols)
    return format_log_line(node_id, tensor_name, counter, step, rows, cols, int(nnz.item()), float(err.item()), hist)
