"""ctypes binding of libmor_hip.so (the C ABI declared in include/mor_hip.h).

There is no CPU fallback: if the library has not been built, importing this module raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmor_hip.so")

FLAG_DEFAULT = 0
FLAG_TORCH_EMULATION = 1
FLAG_SOFTWARE_CAST = 2
FLAG_REFERENCE_ORDER_SUMS = 4
FMT_E4M3, FMT_E5M2, FMT_E3M2, FMT_E2M3 = 0, 1, 2, 3
FMT_COPY = -1          # mor_block_format only: the block kernels' access pattern without the arithmetic
OP_FAKE_QUANTIZE, OP_BLOCK_SCALING, OP_CHANNEL_SCALING, OP_E8MX = 0, 1, 2, 3

_vp, _i64, _i32p, _f64, _u32, _int, _sz = C.c_void_p, C.c_int64, C.c_void_p, C.c_double, C.c_uint32, C.c_int, C.c_size_t

# name -> (restype, argtypes); kept in step with include/mor_hip.h
SIGNATURES = {
    "mor_last_error": (C.c_char_p, []),
    "mor_version": (C.c_char_p, []),
    "mor_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64]),
    "mor_fake_quantize": (_int, [_vp, _vp, _i32p, _i64, _i64, _i64, _i64, _f64, _i64, _i64, _u32, _vp]),
    "mor_fake_quantize_batch": (_int, [_vp, _i64, _u32, _vp]),
    "mor_block_format": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _int, _i64, _u32, _vp]),
    "mor_block_scaling": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f64, _i64, _int, _vp, _sz, _u32, _vp]),
    "mor_block_scaling_static": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f64, _i64, _int, _u32, _vp]),
    "mor_e8mx": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _sz, _u32, _vp]),
    "mor_quant_dequant": (_int, [_vp, _vp, _i64, _int, _vp]),
    "mor_e4m3_with_e8_scale": (_int, [_vp, _vp, _i64, _int, _vp]),
    "mor_block_stats": (_int, [_vp, _i64, _i64, _i64, _i64, C.c_float, _vp, _vp, _vp, _vp]),
    "mor_mor_stats": (_int, [_vp, _i64, _i64, _i64, _i64, _f64, _i64, _i64, _vp, _u32, _vp]),
    "mor_selftest_hw_cast": (_int, [_vp, _vp]),
    "mor_selftest_hw_wire": (_int, [_vp, _vp]),
    "mor_selftest_mx_mfma": (_int, [_vp, _vp, _vp, _vp, _int, _vp, _vp]),
    "mor_mx_payload_bytes": (_sz, [_i64, _i64, _int]),
    "mor_mx_quantize": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _vp]),
    "mor_mx_quantize_dual": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _vp]),
    "mor_mx_dequantize": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _vp]),
    "mor_fake_quantize_dual": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "mor_fake_quantize_dual_tiles": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _f64, _i64, _i64, _vp]),
    "mor_mor_quantize": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _f64, _i64, _vp]),
    "mor_mor_dequantize": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "mor_mor_transpose": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "mor_mor_quantize_dual": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f64, _i64, _vp]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc --offload-arch=gfx950); there is no CPU fallback")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        # a library built from other sources than the ones next to it must not be run silently
        from . import build as _build
        if os.path.exists(_build.VERSION_SRC):
            want, have = _build.source_hash(), L.mor_version().decode()
            if not have.endswith("src " + want):
                raise ImportError(f"{LIB_PATH} reports '{have}' but the sources in {_build._CSRC} hash to {want}: "
                                  "rebuild it (python -c 'import __graft_entry__ as g; g.build()')")
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise RuntimeError(f"mor_hip error {rc}: {lib().mor_last_error().decode()}")
