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


def mor_stats(a_u16, block_x, block_y, clamp, mode, sf_type):
    L = _cabi.lib()
    rows, cols = a_u16.shape
    x = to_dev_u16(a_u16)
    st = torch.zeros((cdiv(rows, block_x), cdiv(cols, block_y), 4), dtype=torch.float32, device=dev())
    _cabi.check(L.mor_mor_stats(x.data_ptr(), rows, cols, block_x, block_y, float(clamp), mode, sf_type, st.data_ptr(), stream_ptr()))
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
