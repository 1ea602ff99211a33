"""ctypes/numpy binding of the CPU oracle (libmor_oracle.so) -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the cpu_baseline leg of the benchmark may
import this module.  bf16 tensors travel as numpy uint16 arrays (raw bits).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmor_oracle.so")

E4M3, E5M2, E3M2, E2M3 = 0, 1, 2, 3
KERNEL, EMU = 0, 1
FMAX = {E4M3: 448.0, E5M2: 57344.0, E3M2: 28.0, E2M3: 7.5}


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        f32, u32, i32, i64, vp, sz = C.c_float, C.c_uint32, C.c_int32, C.c_int64, C.c_void_p, C.c_size_t
        sig = {
            "mor_oracle_bf16_to_fp32": (f32, [u32]),
            "mor_oracle_fp32_to_bf16": (u32, [f32]),
            "mor_oracle_fp32_to_bf16_rne": (u32, [f32]),
            "mor_oracle_cast_sw": (f32, [f32, C.c_int]),
            "mor_oracle_cast_hw": (f32, [f32, C.c_int]),
            "mor_oracle_sqdd_e8": (f32, [f32, f32, C.c_int, C.c_int, C.c_int]),
            "mor_oracle_sqdd_fp32": (f32, [f32, f32, C.c_int, C.c_int]),
            "mor_oracle_scaling_factor": (f32, [f32, f32, C.c_int]),
            "mor_oracle_e8m": (f32, [f32, C.c_int]),
            "mor_oracle_e8mx_scaling_factor": (f32, [f32, C.c_int, C.c_int]),
            "mor_oracle_mor_error_terms": (None, [vp, sz, f32, C.c_int, C.c_int, vp, vp]),
            "mor_oracle_cast_sw_n": (None, [vp, vp, sz, C.c_int]),
            "mor_oracle_cast_hw_n": (None, [vp, vp, sz, C.c_int]),
            "mor_oracle_fake_quantize": (C.c_int, [vp, vp, vp, i64, i64, i64, i64, f32, i64, i64, C.c_int, vp]),
            "mor_oracle_block_format": (C.c_int, [vp, vp, i64, i64, i64, i64, C.c_int, i64, C.c_int]),
            "mor_oracle_block_scaling": (C.c_int, [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, f32, i64, C.c_int, C.c_int]),
            "mor_oracle_last_exact_error": (C.c_double, []),
            "mor_oracle_e8mx": (C.c_int, [vp, vp, i64, i64, i64, i64, i64, i64, C.c_int]),
            "mor_oracle_quant_dequant": (None, [vp, vp, sz, C.c_int]),
            "mor_oracle_e4m3_with_e8_scale": (None, [vp, vp, sz, C.c_int]),
            "mor_oracle_block_stats": (C.c_int, [vp, i64, i64, i64, i64, f32, vp, vp, vp]),
            "mor_oracle_mx_quantize": (C.c_int, [vp, vp, vp, i64, i64, C.c_int]),
            "mor_oracle_mx_dequantize": (C.c_int, [vp, vp, vp, i64, i64, C.c_int]),
            "mor_oracle_num_threads": (C.c_int, []),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _u16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16 and a.ndim == 2, (a.dtype, a.shape)
    return a


def cdiv(a, b):
    return (a + b - 1) // b


def num_threads():
    return lib().mor_oracle_num_threads()


def cast_sw(x, fmt):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().mor_oracle_cast_sw_n(_p(x), _p(out), x.size, fmt)
    return out


def cast_hw(x, fmt):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().mor_oracle_cast_hw_n(_p(x), _p(out), x.size, fmt)
    return out


def mor_error_terms(x_u16, amax, sf_type, flavour=KERNEL):
    """The E4M3 and E5M2 terms |q / x - 1| of the MoR error sums for the elements x (bf16 bits) of a block with that amax."""
    x = np.ascontiguousarray(x_u16, dtype=np.uint16).ravel()
    e4 = np.empty(x.size, np.float32)
    e5 = np.empty(x.size, np.float32)
    lib().mor_oracle_mor_error_terms(_p(x), x.size, float(amax), int(sf_type == 2), flavour, _p(e4), _p(e5))
    return e4, e5


def fake_quantize(a, block_x, block_y, clamp_threshold, mode, sf_type, flavour=KERNEL, want_stats=False):
    """-> (out uint16 [rows, cols], meta int32 [gy, gx][, stats float32 [gy, gx, 4]])"""
    a = _u16(a)
    rows, cols = a.shape
    gy, gx = cdiv(rows, block_x), cdiv(cols, block_y)
    out = np.empty_like(a)
    meta = np.empty((gy, gx), dtype=np.int32)
    stats = np.zeros((gy, gx, 4), dtype=np.float32) if want_stats else None
    rc = lib().mor_oracle_fake_quantize(_p(a), _p(out), _p(meta), rows, cols, block_x, block_y,
                                        float(clamp_threshold), mode, sf_type, flavour,
                                        _p(stats) if want_stats else None)
    if rc:
        raise RuntimeError(f"mor_oracle_fake_quantize failed: {rc}")
    return (out, meta, stats) if want_stats else (out, meta)


def block_format(a, block_x, block_y, fmt, sf_type, flavour=KERNEL):
    a = _u16(a)
    rows, cols = a.shape
    out = np.empty_like(a)
    rc = lib().mor_oracle_block_format(_p(a), _p(out), rows, cols, block_x, block_y, fmt, sf_type, flavour)
    if rc:
        raise RuntimeError(f"mor_oracle_block_format failed: {rc}")
    return out


def block_scaling(a, block_x, block_y, e4m3_threshold, ss_mode, channel=False, flavour=KERNEL):
    """-> (out, meta[1], global_amax[1], global_non_zero[1], global_error[1])"""
    a = _u16(a)
    rows, cols = a.shape
    out = np.empty_like(a)
    meta = np.zeros(1, np.int32)
    gamax = np.zeros(1, np.float32)
    gnnz = np.zeros(1, np.int32)
    gerr = np.zeros(1, np.float32)
    rc = lib().mor_oracle_block_scaling(_p(a), _p(out), _p(meta), _p(gamax), _p(gnnz), _p(gerr), rows, cols,
                                        block_x, block_y, float(e4m3_threshold), ss_mode, int(channel), flavour)
    if rc:
        raise RuntimeError(f"mor_oracle_block_scaling failed: {rc}")
    return out, meta, gamax, gnnz, gerr


def last_exact_error():
    """The error terms of this thread's last block_scaling call added in float64 (global_error is the reference's fp32
    sum in the reference's order of additions, rounding included)."""
    return float(lib().mor_oracle_last_exact_error())


def e8mx(a, block_x, block_y, quantize_type, scaling_strategy, flavour=KERNEL):
    a = _u16(a)
    rows, cols = a.shape
    out = np.empty_like(a)
    rc = lib().mor_oracle_e8mx(_p(a), _p(out), rows, cols, block_x, block_y, quantize_type, scaling_strategy, flavour)
    if rc:
        raise RuntimeError(f"mor_oracle_e8mx failed: {rc}")
    return out


def quant_dequant(x, fmt):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().mor_oracle_quant_dequant(_p(x), _p(out), x.size, fmt)
    return out


def e4m3_with_e8_scale(x, rne):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().mor_oracle_e4m3_with_e8_scale(_p(x), _p(out), x.size, int(rne))
    return out


def block_stats(a, block_x, block_y, fmax):
    """-> (amax f32 [gy,gx], scale f32 [gy,gx], biased E8M0 exponent i32 [gy,gx])"""
    a = _u16(a)
    rows, cols = a.shape
    gy, gx = cdiv(rows, block_x), cdiv(cols, block_y)
    amax = np.empty((gy, gx), np.float32)
    scale = np.empty((gy, gx), np.float32)
    e8 = np.empty((gy, gx), np.int32)
    rc = lib().mor_oracle_block_stats(_p(a), rows, cols, block_x, block_y, float(fmax), _p(amax), _p(scale), _p(e8))
    if rc:
        raise RuntimeError(f"mor_oracle_block_stats failed: {rc}")
    return amax, scale, e8


def mx_row_bytes(cols, fmt):
    return cols if fmt in (E4M3, E5M2) else cols // 4 * 3


def mx_quantize(a, fmt):
    """bf16 bits [rows, cols] -> (payload uint8 [rows, row_bytes], scales uint8 [rows, cols // 32])"""
    a = _u16(a)
    rows, cols = a.shape
    payload = np.empty((rows, mx_row_bytes(cols, fmt)), np.uint8)
    scales = np.empty((rows, cols // 32), np.uint8)
    if lib().mor_oracle_mx_quantize(_p(a), _p(payload), _p(scales), rows, cols, fmt):
        raise RuntimeError("mor_oracle_mx_quantize: invalid argument")
    return payload, scales


def mx_dequantize(payload, scales, fmt):
    payload = np.ascontiguousarray(payload, np.uint8)
    scales = np.ascontiguousarray(scales, np.uint8)
    rows, cols = scales.shape[0], scales.shape[1] * 32
    out = np.empty((rows, cols), np.uint16)
    if lib().mor_oracle_mx_dequantize(_p(payload), _p(scales), _p(out), rows, cols, fmt):
        raise RuntimeError("mor_oracle_mx_dequantize: invalid argument")
    return out
