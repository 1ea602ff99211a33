"""Helpers for the GPU parity tests: device buffers are torch tensors, calls go through the C ABI."""
import numpy as np
import torch

from mor_amd import _cabi


def dev():
    return torch.device("cuda:0")


def to_dev_u16(a_u16):
    """numpy uint16 bits -> bf16 tensor on the GPU"""
    t = torch.from_numpy(np.ascontiguousarray(a_u16).view(np.int16)).view(torch.bfloat16)
    return t.to(dev())


def to_host_u16(t):
    return t.contiguous().cpu().view(torch.int16).numpy().view(np.uint16).copy()


def stream_ptr():
    return torch.cuda.current_stream().cuda_stream


def cdiv(a, b):
    return (a + b - 1) // b


def fake_quantize(a_u16, block_x, block_y, clamp, mode, sf_type, flags=0, inplace=False, x_dev=None):
    """-> (out bits, meta) through mor_fake_quantize"""
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16) if x_dev is None else x_dev
    out = x if inplace else torch.empty_like(x)
    meta = torch.full((cdiv(rows, block_x), cdiv(cols, block_y)), -7, dtype=torch.int32, device=dev())
    _cabi.check(L.mor_fake_quantize(x.data_ptr(), out.data_ptr(), meta.data_ptr(), rows, cols, block_x, block_y,
                                    float(clamp), mode, sf_type, flags, stream_ptr()))
    torch.cuda.synchronize()
    return to_host_u16(out), meta.cpu().numpy()


def block_format(a_u16, block_x, block_y, fmt, sf_type, flags=0):
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16)
    out = torch.empty_like(x)
    _cabi.check(L.mor_block_format(x.data_ptr(), out.data_ptr(), rows, cols, block_x, block_y, fmt, sf_type, flags, stream_ptr()))
    torch.cuda.synchronize()
    return to_host_u16(out)


def mor_stats(a_u16, block_x, block_y, clamp, mode, sf_type, flags=0):
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16)
    st = torch.zeros((cdiv(rows, block_x), cdiv(cols, block_y), 4), dtype=torch.float32, device=dev())
    _cabi.check(L.mor_mor_stats(x.data_ptr(), rows, cols, block_x, block_y, float(clamp), mode, sf_type, st.data_ptr(), flags, stream_ptr()))
    torch.cuda.synchronize()
    return st.cpu().numpy()


def block_stats(a_u16, block_x, block_y, fmax):
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16)
    shape = (cdiv(rows, block_x), cdiv(cols, block_y))
    amax = torch.zeros(shape, dtype=torch.float32, device=dev())
    scale = torch.zeros(shape, dtype=torch.float32, device=dev())
    e8 = torch.zeros(shape, dtype=torch.int32, device=dev())
    _cabi.check(L.mor_block_stats(x.data_ptr(), rows, cols, block_x, block_y, float(fmax), amax.data_ptr(), scale.data_ptr(), e8.data_ptr(), stream_ptr()))
    torch.cuda.synchronize()
    return amax.cpu().numpy(), scale.cpu().numpy(), e8.cpu().numpy()


def block_scaling(a_u16, block_x, block_y, threshold, ss_mode, channel=False, flags=0, inplace=False):
    """-> (out bits, meta, global_amax, global_non_zero, global_error) through mor_block_scaling"""
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16)
    out = x if inplace else torch.full_like(x, 7.0)
    meta = torch.full((1,), -7, dtype=torch.int32, device=dev())
    gamax = torch.zeros(1, dtype=torch.float32, device=dev())
    gnnz = torch.zeros(1, dtype=torch.int32, device=dev())
    gerr = torch.zeros(1, dtype=torch.float32, device=dev())
    op = _cabi.OP_CHANNEL_SCALING if channel else _cabi.OP_BLOCK_SCALING
    nbytes = L.mor_workspace_bytes(op, rows, cols, block_x, block_y)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=dev())
    _cabi.check(L.mor_block_scaling(x.data_ptr(), out.data_ptr(), meta.data_ptr(), gamax.data_ptr(), gnnz.data_ptr(),
                                    gerr.data_ptr(), rows, cols, block_x, block_y, float(threshold), ss_mode,
                                    int(channel), ws.data_ptr(), nbytes, flags, stream_ptr()))
    torch.cuda.synchronize()
    return to_host_u16(out), meta.cpu().numpy(), gamax.cpu().numpy(), gnnz.cpu().numpy(), gerr.cpu().numpy()


def e8mx(a_u16, block_x, block_y, quantize_type, scaling_strategy, flags=0, inplace=False):
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16)
    out = x if inplace else torch.empty_like(x)
    nbytes = L.mor_workspace_bytes(_cabi.OP_E8MX, rows, cols, block_x, block_y)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=dev())
    _cabi.check(L.mor_e8mx(x.data_ptr(), out.data_ptr(), rows, cols, block_x, block_y, quantize_type, scaling_strategy,
                           ws.data_ptr(), nbytes, flags, stream_ptr()))
    torch.cuda.synchronize()
    return to_host_u16(out)


def quant_dequant(x_f32, fmt):
    L = _cabi.lib()
    x = torch.from_numpy(np.ascontiguousarray(x_f32, dtype=np.float32)).to(dev())
    out = torch.empty_like(x)
    _cabi.check(L.mor_quant_dequant(x.data_ptr(), out.data_ptr(), x.numel(), fmt, stream_ptr()))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def e4m3_with_e8_scale(x_f32, rne):
    L = _cabi.lib()
    x = torch.from_numpy(np.ascontiguousarray(x_f32, dtype=np.float32)).to(dev())
    out = torch.empty_like(x)
    _cabi.check(L.mor_e4m3_with_e8_scale(x.data_ptr(), out.data_ptr(), x.numel(), int(rne), stream_ptr()))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def mx_row_bytes(cols, fmt):
    return cols if fmt in (_cabi.FMT_E4M3, _cabi.FMT_E5M2) else cols // 4 * 3


def mx_quantize(a_u16, fmt, x_dev=None):
    """-> (payload uint8 [rows, row_bytes], scales uint8 [rows, cols // 32]) through mor_mx_quantize"""
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16) if x_dev is None else x_dev
    payload = torch.full((rows, mx_row_bytes(cols, fmt)), 0xA5, dtype=torch.uint8, device=dev())
    scales = torch.full((rows, cols // 32), 0xA5, dtype=torch.uint8, device=dev())
    _cabi.check(L.mor_mx_quantize(x.data_ptr(), payload.data_ptr(), scales.data_ptr(), rows, cols, fmt, stream_ptr()))
    torch.cuda.synchronize()
    return payload.cpu().numpy(), scales.cpu().numpy()


def mx_quantize_dual(a_u16, fmt):
    """-> (row payload, row scales, column payload [cols, ...], column scales [cols, rows // 32])"""
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16)
    rp = torch.full((rows, mx_row_bytes(cols, fmt)), 0xA5, dtype=torch.uint8, device=dev())
    rs = torch.full((rows, cols // 32), 0xA5, dtype=torch.uint8, device=dev())
    cp = torch.full((cols, mx_row_bytes(rows, fmt)), 0xA5, dtype=torch.uint8, device=dev())
    cs = torch.full((cols, rows // 32), 0xA5, dtype=torch.uint8, device=dev())
    _cabi.check(L.mor_mx_quantize_dual(x.data_ptr(), rp.data_ptr(), rs.data_ptr(), cp.data_ptr(), cs.data_ptr(),
                                       rows, cols, fmt, stream_ptr()))
    torch.cuda.synchronize()
    return rp.cpu().numpy(), rs.cpu().numpy(), cp.cpu().numpy(), cs.cpu().numpy()


def mx_dequantize(payload, scales, fmt):
    L = _cabi.lib()
    rows, cols = scales.shape[0], scales.shape[1] * 32
    p = torch.from_numpy(np.ascontiguousarray(payload)).to(dev())
    s = torch.from_numpy(np.ascontiguousarray(scales)).to(dev())
    out = torch.empty((rows, cols), dtype=torch.bfloat16, device=dev())
    _cabi.check(L.mor_mx_dequantize(p.data_ptr(), s.data_ptr(), out.data_ptr(), rows, cols, fmt, stream_ptr()))
    torch.cuda.synchronize()
    return to_host_u16(out)


def fake_quantize_dual(a_u16, mode, sf_type, want_meta=True):
    """-> (out [rows, cols], meta [rows, cols/32], out_t [cols, rows], meta_t [cols, rows/32]) through mor_fake_quantize_dual"""
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16)
    o = torch.full((rows, cols), 7.0, dtype=torch.bfloat16, device=dev())
    ot = torch.full((cols, rows), 7.0, dtype=torch.bfloat16, device=dev())
    m = torch.full((rows, cols // 32), -7, dtype=torch.int32, device=dev())
    mt = torch.full((cols, rows // 32), -7, dtype=torch.int32, device=dev())
    _cabi.check(L.mor_fake_quantize_dual(x.data_ptr(), o.data_ptr(), m.data_ptr() if want_meta else None, ot.data_ptr(),
                                         mt.data_ptr() if want_meta else None, rows, cols, mode, sf_type, stream_ptr()))
    torch.cuda.synchronize()
    return to_host_u16(o), m.cpu().numpy(), to_host_u16(ot), mt.cpu().numpy()


def fake_quantize_batch(arrays, blocks, clamp, mode, sf, flags=0, inplace=False):
    """-> [(out bits, meta)] through mor_fake_quantize_batch, every tensor with the same clamp / mode / sf_type"""
    from mor_amd.batch import TensorDesc
    L = _cabi.lib()
    xs = [to_dev_u16(a) for a in arrays]
    outs = xs if inplace else [torch.full_like(x, 7.0) for x in xs]
    metas = [torch.full((cdiv(a.shape[0], br), cdiv(a.shape[1], bc)), -7, dtype=torch.int32, device=dev())
             for a, (br, bc) in zip(arrays, blocks)]
    descs = (TensorDesc * len(xs))()
    for d, x, y, m, (br, bc) in zip(descs, xs, outs, metas, blocks):
        d.input, d.output, d.meta = x.data_ptr(), y.data_ptr(), m.data_ptr()
        d.rows, d.cols, d.block_rows, d.block_cols = x.shape[0], x.shape[1], br, bc
        d.clamp_threshold, d.mode, d.sf_type = clamp, mode, sf
    _cabi.check(L.mor_fake_quantize_batch(descs, len(xs), flags, stream_ptr()))
    torch.cuda.synchronize()
    return [(to_host_u16(y), m.cpu().numpy()) for y, m in zip(outs, metas)]
