// Device-side numerics of the fake-quantization path for gfx950 (wave64).
//
// Two implementations of every per-element step live here:
//   *_exact : integer/float software that follows the reference arithmetic step by step
//             (mor/csrc/cuda/fake_quantize.cu, "FQ") for every fp32 bit pattern;
//   *_fast  : a few VALU instructions (hardware FP8 converts, ldexp, integer exponent
//             arithmetic) that give the same bits whenever the block's scale exponent is
//             in a safe range; kernels pick per block.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mor {

enum : int { FMT_E4M3 = 0, FMT_E5M2 = 1, FMT_E3M2 = 2, FMT_E2M3 = 3 };

__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }

template <int F> struct Fmt;
template <> struct Fmt<FMT_E4M3> { static constexpr float fmax = 448.0f;   static constexpr int mbits = 3; static constexpr int emin = -6;  static constexpr bool hw = true; };
template <> struct Fmt<FMT_E5M2> { static constexpr float fmax = 57344.0f; static constexpr int mbits = 2; static constexpr int emin = -14; static constexpr bool hw = true; };
template <> struct Fmt<FMT_E3M2> { static constexpr float fmax = 28.0f;    static constexpr int mbits = 2; static constexpr int emin = -2;  static constexpr bool hw = false; };
template <> struct Fmt<FMT_E2M3> { static constexpr float fmax = 7.5f;     static constexpr int mbits = 3; static constexpr int emin = 0;   static constexpr bool hw = false; };

__host__ __device__ __forceinline__ float fmax_of(int fmt) {
    return fmt == FMT_E4M3 ? 448.0f : fmt == FMT_E5M2 ? 57344.0f : fmt == FMT_E3M2 ? 28.0f : 7.5f;
}

// ---------------------------------------------------------------- 16-byte global accesses
// NT = streaming (non-temporal) access for tensors far larger than the last-level cache.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <bool NT> __device__ __forceinline__ uint4 load16(const uint4* p) {
    if constexpr (NT) {
        u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        return make_uint4(t.x, t.y, t.z, t.w);
    } else {
        return *p;
    }
}
template <bool NT> __device__ __forceinline__ void store16(uint4* p, uint4 v) {
    if constexpr (NT) {
        u32x4 t = {v.x, v.y, v.z, v.w};
        __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
    } else {
        *p = v;
    }
}

// Run-time choice (uniform over the grid).  Outputs of 4 MiB and more do not fit an L2 and are not read back by
// the kernel that writes them: streaming stores keep them from evicting the input and the caller's data.
__device__ __forceinline__ bool streams_out(int64_t bf16_elements) { return bf16_elements >= ((int64_t)2 << 20); }
__device__ __forceinline__ void store16_rt(uint4* p, uint4 v, bool nt) {
    if (nt) store16<true>(p, v);
    else store16<false>(p, v);
}

// Inputs stream too once a kernel's traffic (2 bytes read + 2 written per element) exceeds twice the 256 MB last-level
// cache: nothing of such a tensor is found there again (MX 1 x 32 on 16384 x 14336: 160 -> 150 us; at 8192^2 streaming
// loads cost 39 -> 44 us).
__device__ __forceinline__ bool streams_in(int64_t bf16_elements) { return bf16_elements > ((int64_t)128 << 20); }
// The last (or only) read a kernel makes of a tensor of 64 MiB or more streams as well: nothing reads those lines again,
// and with streaming loads a tensor that comes from HBM does not push the caller's data out of the caches on its way
// (8192^2 from HBM, 1 x 32 blocks: 45.5 -> 43 us; repeated launches on one buffer pair, which find part of their input in
// the last-level cache only because the previous launch left it there, lose that: 39 -> 44 us).
// A tensor of 32 MiB and its image fit the 256 MB last-level cache with room to spare and keep the allocating loads
// (4096^2 with the caller's scale: 10.0 against 12.5 us).
__device__ __forceinline__ bool streams_last_read(int64_t bf16_elements) { return bf16_elements >= ((int64_t)32 << 20); }
__device__ __forceinline__ uint4 load16_rt(const uint4* p, bool nt) { return nt ? load16<true>(p) : load16<false>(p); }
// N loads under one run-time choice of the policy.  Chosen load by load (load16_rt in an unrolled loop) every load
// sits in a branch of its own, and the registers the two arms share are merged behind it: the compiler then waits for
// each load before it issues the next one, and a wave has one request in flight instead of N.
template <int N, class At> __device__ __forceinline__ void load16_group(uint4 (&v)[N], bool nt, At&& at) {
    if (nt) {
#pragma unroll
        for (int k = 0; k < N; ++k) v[k] = load16<true>(at(k));
    } else {
#pragma unroll
        for (int k = 0; k < N; ++k) v[k] = load16<false>(at(k));
    }
}

// ---------------------------------------------------------------- bf16 <-> fp32
// FQ:38-44: a bf16 is the upper half of an fp32.
__device__ __forceinline__ float bf16_lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return u2f(w & 0xFFFF0000u); }
__device__ __forceinline__ float bf16_one(uint16_t h) { return u2f((uint32_t)h << 16); }

// FQ:46-60: round half up on the magnitude.  Adding 0x8000 to the word does that, the carry
// running into the exponent exactly as the reference's mantissa/exponent increments do.
__device__ __forceinline__ uint32_t rhu_bits(float v) { return f2u(v) + 0x8000u; }
// torch's nearest-even store (NaN kept as a quiet NaN)
__device__ __forceinline__ uint32_t rne_bits(float v) {
    uint32_t b = f2u(v);
    uint32_t r = b + 0x7FFFu + ((b >> 16) & 1u);
    return (v != v) ? ((b & 0x80000000u) | 0x7FC00000u) : r;
}
template <bool EMU> __device__ __forceinline__ uint32_t store_bits(float v) { return EMU ? rne_bits(v) : rhu_bits(v); }
template <bool EMU> __device__ __forceinline__ uint16_t store_bf16(float v) { return (uint16_t)(store_bits<EMU>(v) >> 16); }
// two results -> one packed word: bytes 3:2 of each rounded word
template <bool EMU> __device__ __forceinline__ uint32_t store_pair(float lo, float hi) {
    return __builtin_amdgcn_perm(store_bits<EMU>(hi), store_bits<EMU>(lo), 0x07060302u);
}

// ---------------------------------------------------------------- casts
// Exact nearest-even rounding of |v| onto the grid of format F, saturating at fmax.
// (a + M) - M with M = 2^(23 - mbits) * 2^max(exponent, emin) rounds a to that quantum in hardware.
template <int F> __device__ __forceinline__ float round_mag_sat(float a) {
    a = fminf(a, Fmt<F>::fmax);
    int e = (int)(f2u(a) >> 23);
    e = max(e, Fmt<F>::emin + 127);
    float M = u2f((uint32_t)(e + 23 - Fmt<F>::mbits) << 23);
    return (a + M) - M;
}

// Software model of the reference's hardware cast (FQ:223-227, cuda_fp8.hpp with SATFINITE):
// nearest even, saturate to +-fmax, sign of a zero kept, NaN -> the canonical NaN 0x7fffffff.
template <int F> __device__ __forceinline__ float cast_hwmodel_exact(float v) {
    if (v != v) return u2f(0x7FFFFFFFu);
    return u2f(f2u(round_mag_sat<F>(fabsf(v))) | (f2u(v) & 0x80000000u));
}

// The reference's software cast (FQ:125-215): nearest even; E3M2/E2M3 saturate, E4M3/E5M2 give
// NaN 0x7fffffff above their range; a zero result is +0.
template <int F> __device__ __forceinline__ float cast_sw_exact(float v) {
    float a = fabsf(v);
    if constexpr (F == FMT_E4M3) { if (!(a <= 464.0f)) return u2f(0x7FFFFFFFu); }
    if constexpr (F == FMT_E5M2) { if (!(a < 61440.0f)) return u2f(0x7FFFFFFFu); }
    if constexpr (F == FMT_E3M2 || F == FMT_E2M3) { if (v != v) return u2f(f2u(Fmt<F>::fmax) | (f2u(v) & 0x80000000u)); }
    float r = round_mag_sat<F>(a);
    uint32_t rb = f2u(r);
    // sign only on a non-zero result
    return u2f(rb | ((rb + 0x7FFFFFFFu) & f2u(v) & 0x80000000u));
}

// torch's CPU cast to float8_e4m3fn / float8_e5m2 and back
template <int F> __device__ __forceinline__ float cast_torch_exact(float v) {
    uint32_t s = f2u(v) & 0x80000000u;
    if (v != v) return u2f(0x7FC00000u | s);
    float a = fabsf(v);
    bool over = (F == FMT_E4M3) ? (a > 464.0f) : (a >= 61440.0f);
    if (over) return u2f(((F == FMT_E4M3) ? 0x7FC00000u : 0x7F800000u) | s);
    return u2f(f2u(round_mag_sat<F>(a)) | s);
}

// which cast a production path uses (FQ:338-379): hardware for E4M3/E5M2, software for E2M3/E3M2
template <int F, bool EMU> __device__ __forceinline__ float cast_exact(float v) {
    if constexpr (EMU) {
        if constexpr (Fmt<F>::hw) return cast_torch_exact<F>(v);
        else {
            float r = cast_sw_exact<F>(v);
            return (r == 0.0f) ? u2f(f2u(v) & 0x80000000u) : r;
        }
    } else {
        if constexpr (Fmt<F>::hw) return cast_hwmodel_exact<F>(v);
        else return cast_sw_exact<F>(v);
    }
}

// gfx950 converts.  In range (|v| <= fmax) they are nearest-even with the sign of zero kept.
template <int F> __device__ __forceinline__ uint32_t hw_pack2(float a, float b) {
    if constexpr (F == FMT_E4M3) return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    else return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
}
template <int F, int BYTE> __device__ __forceinline__ float hw_unpack(uint32_t p) {
    if constexpr (F == FMT_E4M3) return __builtin_amdgcn_cvt_f32_fp8((int)p, BYTE);
    else return __builtin_amdgcn_cvt_f32_bf8((int)p, BYTE);
}

// gfx950 scaled converts on fp32 pairs: both fp8 codes of a pair of values in one register, E4M3 codes of (a, b) in
// the low word and E5M2 codes of (128 a, 128 b) in the high word (the scale operand of the convert divides by 2^-7),
// and both values of a word decoded by one instruction.  mor_selftest_hw_cast compares them with the plain converts
// over every fp32 value in range.
typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t hw_pack2_both(float a, float b, uint32_t old) {
    s16x2 p = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(__builtin_bit_cast(s16x2, old), a, b, 1.0f, false);
    p = __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(p, a, b, 0x1p-7f, true);
    return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ f32x2 hw_unpack2_e4m3_low(uint32_t p) { return __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(p, 1.0f, false); }
__device__ __forceinline__ f32x2 hw_unpack2_e5m2_high_div128(uint32_t p) { return __builtin_amdgcn_cvt_scalef32_pk_f32_bf8(p, 0x1p-7f, true); }
template <int F> __device__ __forceinline__ uint32_t hw_pack2_low(float a, float b) {
    const s16x2 z = {0, 0};
    if constexpr (F == FMT_E4M3) return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(z, a, b, 1.0f, false));
    else return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(z, a, b, 1.0f, false));
}
// the same with the other half of the result register taken from `old` (its contents do not matter to the caller)
template <int F> __device__ __forceinline__ uint32_t hw_pack2_low_keep(float a, float b, uint32_t old) {
    const s16x2 o = __builtin_bit_cast(s16x2, old);
    if constexpr (F == FMT_E4M3) return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, a, b, 1.0f, false));
    else return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf8_f32(o, a, b, 1.0f, false));
}
template <int F> __device__ __forceinline__ f32x2 hw_unpack2_low(uint32_t p) {
    if constexpr (F == FMT_E4M3) return __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(p, 1.0f, false);
    else return __builtin_amdgcn_cvt_scalef32_pk_f32_bf8(p, 1.0f, false);
}

// ---------------------------------------------------------------- scale-quantize-dequantize-descale
// FQ:248-306 with E8_RZ: the power of two is taken from the exponent field of the fp32 scale and
// added to / subtracted from exponent fields, clamping at 0 and keeping the mantissa.
template <int F, bool EMU> __device__ __forceinline__ float sqdd_e8_exact(float x, int e8) {
    if constexpr (EMU) {
        float p = ldexpf(1.0f, e8);
        return cast_exact<F, true>(x * p) / p;
    } else {
        uint32_t xb = f2u(x);
        int ve = (int)((xb >> 23) & 0xFF) + e8;
        if (ve < 0) ve = 0;
        float scaled = u2f((xb & 0x80000000u) | ((uint32_t)ve << 23) | (xb & 0x7FFFFFu));
        uint32_t db = f2u(cast_exact<F, false>(scaled));
        int de = (int)((db >> 23) & 0xFF) - e8;
        if (de < 0) de = 0;
        return u2f((db & 0x80000000u) | ((uint32_t)de << 23) | (db & 0x7FFFFFu));
    }
}

// FQ:310-316.  NVIDIA arithmetic returns 0x7fffffff for a NaN result.
template <int F, bool EMU> __device__ __forceinline__ float sqdd_fp32_exact(float x, float s) {
    float r = cast_exact<F, EMU>(x * s) / s;
    if constexpr (!EMU) { if (r != r) r = u2f(0x7FFFFFFFu); }
    return r;
}

// Per-block scale state shared by the fast and exact paths.
struct Scale {
    float s;      // fp32 scale (fmax / amax, or the caller's)
    float r;      // RN(1 / s) for div_by_scale (fp32-scale paths only)
    int e8;       // exponent field of s minus 127
    bool fast;    // the fast path reproduces the exact one for every finite bf16 element
};

__device__ __forceinline__ Scale make_scale(float s) {
    Scale sc;
    sc.s = s;
    sc.e8 = (int)((f2u(s) >> 23) & 0xFF) - 127;
    // |e8| <= 100 keeps every scaled / descaled exponent inside the normal range, so exponent-field
    // arithmetic, ldexp and IEEE multiply/divide agree (see the fast paths below); a significand of all ones is
    // the one case in which div_by_scale may differ from the IEEE quotient.
    sc.r = 1.0f / s;
    sc.fast = (sc.e8 >= -100) && (sc.e8 <= 100) && ((f2u(s) & 0x7FFFFFu) != 0x7FFFFFu);
    return sc;
}

// Exponent of the power-of-two scale without the division: for amax = m * 2^ea (1 <= m < 2, a normal bf16)
// and fmax = f * 2^eb, floor(log2(fl(fmax / amax))) = eb - ea - (m > f).  The fp32 quotient cannot round up to a
// power of two because m has 8 significant bits.  Returns the Scale of FQ:251-252 with s left unset (E8 paths only
// use e8); `fast` additionally requires a normal amax.
template <int F> __device__ __forceinline__ Scale make_scale_e8(float amax) {
    constexpr int eb = (F == FMT_E4M3) ? 8 : (F == FMT_E5M2) ? 15 : (F == FMT_E3M2) ? 4 : 2;
    constexpr uint32_t mth = (F == FMT_E2M3) ? 0x70u : 0x60u;       // mantissa field of 1.875 / 1.75
    const uint32_t b = f2u(amax);
    const int ea = (int)(b >> 23);
    Scale sc;
    sc.s = 0.0f;
    sc.r = 0.0f;
    sc.e8 = (127 + eb) - ea - (((b >> 16) & 0x7Fu) > mth ? 1 : 0);
    sc.fast = (ea != 0) && (sc.e8 >= -100) && (sc.e8 <= 100);
    return sc;
}

// Fast E8 path on a pair (lo, hi) of one packed word, result packed.  For E4M3/E5M2:
//   |x| * 2^e8 (exact), hardware convert and back, then integer exponent subtraction clamped at 0,
//   which also yields the reference's 2^(-e8-127) for a zero cast result when e8 < 0.  The sign
//   comes from the input word (the hardware cast keeps the sign, including on zeros).
// (E4M3 / E5M2: this is the reference form of the arithmetic; kernels run e8_pair_fast_scaled below, which the
// library's selftest compares with it for every finite bf16 value and every e8 of the fast range)
template <int F, bool CLAMP> __device__ __forceinline__ uint32_t e8_pair_fast_scaled(uint32_t w, int e8);
template <int F, bool CLAMP> __device__ __forceinline__ uint32_t e8_pair_fast_ref(uint32_t w, int e8) {
    const int e8s = e8 << 23;
    if constexpr (Fmt<F>::hw) {
        float a = ldexpf(fabsf(bf16_lo(w)), e8);
        float b = ldexpf(fabsf(bf16_hi(w)), e8);
        if constexpr (CLAMP) { a = fminf(a, Fmt<F>::fmax); b = fminf(b, Fmt<F>::fmax); }
        uint32_t p = hw_pack2<F>(a, b);
        int ma = max((int)f2u(hw_unpack<F, 0>(p)) - e8s, 0);
        int mb = max((int)f2u(hw_unpack<F, 1>(p)) - e8s, 0);
        uint32_t mag = __builtin_amdgcn_perm((uint32_t)mb, (uint32_t)ma, 0x07060302u);
        return mag | (w & 0x80008000u);
    } else {
        // software saturating cast: a zero result is +0, so the sign is applied to non-zero results only
        float a = round_mag_sat<F>(ldexpf(fabsf(bf16_lo(w)), e8));
        float b = round_mag_sat<F>(ldexpf(fabsf(bf16_hi(w)), e8));
        uint32_t ra = f2u(a), rb = f2u(b);
        uint32_t sa = (ra + 0x7FFFFFFFu) & (w << 16) & 0x80000000u;
        uint32_t sb = (rb + 0x7FFFFFFFu) & w & 0x80000000u;
        uint32_t ma = (uint32_t)max((int)ra - e8s, 0) | sa;
        uint32_t mb = (uint32_t)max((int)rb - e8s, 0) | sb;
        return __builtin_amdgcn_perm(mb, ma, 0x07060302u);
    }
}
template <int F, bool CLAMP> __device__ __forceinline__ uint32_t e8_pair_fast(uint32_t w, int e8) {
    if constexpr (Fmt<F>::hw) return e8_pair_fast_scaled<F, CLAMP>(w, e8);
    else return e8_pair_fast_ref<F, CLAMP>(w, e8);
}

// Division by the block scale without a divide per element: with r = RN(1 / s) (one IEEE division per block),
// t = c * r; q = fma(fma(-t, s, c), r, t) is the correctly rounded quotient c / s (Markstein) as long as nothing
// over- or underflows (the fast range) and the significand of s is not all ones (make_scale clears `fast` then).
__device__ __forceinline__ float div_by_scale(float c, float s, float r) {
    const float t = c * r;
    return fmaf(fmaf(-t, s, c), r, t);
}

// Fast fp32-scale path on a pair: multiply, convert, divide by the scale, round-half-up store.  Works on
// magnitudes; the hardware cast keeps the sign (also of a zero result), the software cast returns +0.
template <int F, bool CLAMP> __device__ __forceinline__ uint32_t fp32_pair_fast(uint32_t w, float s, float r) {
    const float a = fabsf(bf16_lo(w)) * s, b = fabsf(bf16_hi(w)) * s;
    if constexpr (Fmt<F>::hw) {
        float v0 = a, v1 = b;
        if constexpr (CLAMP) {   // the reference's hardware cast saturates (user-supplied scales only)
            v0 = fminf(v0, Fmt<F>::fmax);
            v1 = fminf(v1, Fmt<F>::fmax);
        }
        const f32x2 c = hw_unpack2_low<F>(hw_pack2_low<F>(v0, v1));
        return store_pair<false>(div_by_scale(c.x, s, r), div_by_scale(c.y, s, r)) | (w & 0x80008000u);
    } else {
        const float d0 = cast_sw_exact<F>(a), d1 = cast_sw_exact<F>(b);
        const uint32_t sign = ((d0 != 0.0f) ? (w & 0x8000u) : 0u) | ((d1 != 0.0f) ? (w & 0x80000000u) : 0u);
        return store_pair<false>(div_by_scale(d0, s, r), div_by_scale(d1, s, r)) | sign;
    }
}

// One element, exact path, any flavour -> fp32 result before the bf16 store.
template <int F, bool E8, bool EMU> __device__ __forceinline__ float sqdd_exact(float x, const Scale& sc) {
    if constexpr (E8) return sqdd_e8_exact<F, EMU>(x, sc.e8);
    else return sqdd_fp32_exact<F, EMU>(x, sc.s);
}

// One packed word -> one packed word, fast path only (the caller has checked sc.fast).
template <int F, bool E8, bool CLAMP = false>
__device__ __forceinline__ uint32_t fq_pair_fast(uint32_t w, const Scale& sc) {
    if constexpr (E8) return e8_pair_fast<F, CLAMP>(w, sc.e8);
    else return fp32_pair_fast<F, CLAMP>(w, sc.s, sc.r);
}
template <int F, bool E8, bool CLAMP = false>
__device__ __forceinline__ uint4 fq_vec_fast(uint4 v, const Scale& sc) {
    uint4 r;
    r.x = fq_pair_fast<F, E8, CLAMP>(v.x, sc);
    r.y = fq_pair_fast<F, E8, CLAMP>(v.y, sc);
    r.z = fq_pair_fast<F, E8, CLAMP>(v.z, sc);
    r.w = fq_pair_fast<F, E8, CLAMP>(v.w, sc);
    return r;
}
// One packed word -> one packed word, exact path.
template <int F, bool E8, bool EMU>
__device__ __forceinline__ uint32_t fq_pair_exact(uint32_t w, const Scale& sc) {
    return store_pair<EMU>(sqdd_exact<F, E8, EMU>(bf16_lo(w), sc), sqdd_exact<F, E8, EMU>(bf16_hi(w), sc));
}

// ---------------------------------------------------------------- wave64 reductions
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL> __device__ __forceinline__ uint32_t dpp_u(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
constexpr int DPP_XOR1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int DPP_XOR2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141; // lane i <-> 7 - i inside each 8 lanes
constexpr int DPP_MIRROR = 0x140;      // lane i <-> 15 - i inside each 16 lanes

// all-reduce max over aligned groups of G lanes (G power of two, 1..64); inputs are non-negative
__device__ __forceinline__ float group_max(float v, int G) {
    if (G >= 2) v = fmaxf(v, dpp_f<DPP_XOR1>(v));
    if (G >= 4) v = fmaxf(v, dpp_f<DPP_XOR2>(v));
    if (G >= 8) v = fmaxf(v, dpp_f<DPP_HALF_MIRROR>(v));
    if (G >= 16) v = fmaxf(v, dpp_f<DPP_MIRROR>(v));
    if (G >= 32) v = fmaxf(v, __shfl_xor(v, 16));
    if (G >= 64) v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}
// same with the group size known at compile time (GT > 0), else the run-time G
template <int GT> __device__ __forceinline__ float group_max_t(float v, int G) {
    if constexpr (GT == 0) return group_max(v, G);
    else {
        if constexpr (GT >= 2) v = fmaxf(v, dpp_f<DPP_XOR1>(v));
        if constexpr (GT >= 4) v = fmaxf(v, dpp_f<DPP_XOR2>(v));
        if constexpr (GT >= 8) v = fmaxf(v, dpp_f<DPP_HALF_MIRROR>(v));
        if constexpr (GT >= 16) v = fmaxf(v, dpp_f<DPP_MIRROR>(v));
        if constexpr (GT >= 32) v = fmaxf(v, __shfl_xor(v, 16));
        if constexpr (GT >= 64) v = fmaxf(v, __shfl_xor(v, 32));
        return v;
    }
}
__device__ __forceinline__ uint32_t group_umax(uint32_t v, int G) {
    if (G >= 2) v = max(v, dpp_u<DPP_XOR1>(v));
    if (G >= 4) v = max(v, dpp_u<DPP_XOR2>(v));
    if (G >= 8) v = max(v, dpp_u<DPP_HALF_MIRROR>(v));
    if (G >= 16) v = max(v, dpp_u<DPP_MIRROR>(v));
    if (G >= 32) v = max(v, (uint32_t)__shfl_xor((int)v, 16));
    if (G >= 64) v = max(v, (uint32_t)__shfl_xor((int)v, 32));
    return v;
}
__device__ __forceinline__ uint32_t group_umin(uint32_t v, int G) {
    if (G >= 2) v = min(v, dpp_u<DPP_XOR1>(v));
    if (G >= 4) v = min(v, dpp_u<DPP_XOR2>(v));
    if (G >= 8) v = min(v, dpp_u<DPP_HALF_MIRROR>(v));
    if (G >= 16) v = min(v, dpp_u<DPP_MIRROR>(v));
    if (G >= 32) v = min(v, (uint32_t)__shfl_xor((int)v, 16));
    if (G >= 64) v = min(v, (uint32_t)__shfl_xor((int)v, 32));
    return v;
}
// Sum over groups of G = 1, 2, 4, ... 64 consecutive lanes (every lane of a group gets the group's sum).
__device__ __forceinline__ float group_sum(float v, int G) {
    if (G >= 2) v += dpp_f<DPP_XOR1>(v);
    if (G >= 4) v += dpp_f<DPP_XOR2>(v);
    if (G >= 8) v += dpp_f<DPP_HALF_MIRROR>(v);
    if (G >= 16) v += dpp_f<DPP_MIRROR>(v);
    if (G >= 32) v += __shfl_xor(v, 16);
    if (G >= 64) v += __shfl_xor(v, 32);
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<DPP_XOR1>(v);
    v += dpp_f<DPP_XOR2>(v);
    v += dpp_f<DPP_HALF_MIRROR>(v);
    v += dpp_f<DPP_MIRROR>(v);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
    v += (int)dpp_u<DPP_XOR1>((uint32_t)v);
    v += (int)dpp_u<DPP_XOR2>((uint32_t)v);
    v += (int)dpp_u<DPP_HALF_MIRROR>((uint32_t)v);
    v += (int)dpp_u<DPP_MIRROR>((uint32_t)v);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

// amax / min-nonzero accumulation over one packed word (FQ:431-441).
// The minimum over non-zero magnitudes is taken on (bits - 1) as unsigned, which sends 0 to the top.
__device__ __forceinline__ void acc_amax(float& amax, uint32_t w) {
    amax = fmaxf(fmaxf(amax, fabsf(bf16_lo(w))), fabsf(bf16_hi(w)));
}
__device__ __forceinline__ void acc_amin(uint32_t& amin_m1, uint32_t w) {
    uint32_t a = ((w << 16) & 0x7FFFFFFFu) - 1u;
    uint32_t b = (w & 0x7FFF0000u) - 1u;
    amin_m1 = min(min(amin_m1, a), b);
}
constexpr uint32_t AMIN_INIT_M1 = 0x7F7F0000u - 1u;   // bf16 max, FQ:409-412

// The same on both halves of a word at once with packed 16-bit integer instructions: bf16 magnitudes order as their
// bit patterns do.  amax2 holds two running maxima of magnitudes, amin2_m1 two running minima of (magnitude - 1),
// where zero wraps to 0xFFFF and so never wins.  A NaN (magnitude above 0x7F80) would win the maximum, which the
// float maximum of the reference (FQ:430) does not allow: callers send such blocks to the exact path.
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}
// (the instruction itself: written as an elementwise minimum, min(x, 1) on 16-bit halves is turned into a compare and a
// select per half, eight instructions where the uses below count on two)
__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_min_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// Read as signed 16-bit integers the halves of a packed bf16 word have one smallest value, 0x8000: the bf16 -0.  A
// running signed minimum over words therefore ends with a half of 0x8000 exactly when a -0 was among them: one
// instruction per word to learn whether the sign bits of a group of words may be copied as they are.
__device__ __forceinline__ uint32_t pk_min_i16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_min_i16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
constexpr uint32_t NEGZERO_INIT = 0x7FFF7FFFu;
__device__ __forceinline__ void acc_negzero_pk(uint32_t& m, uint32_t w) { m = pk_min_i16(m, w); }
__device__ __forceinline__ bool saw_negzero(uint32_t m) { return (m & 0xFFFFu) == 0x8000u || (m >> 16) == 0x8000u; }
__device__ __forceinline__ uint32_t pk_lshr_u16(uint32_t a, int n) {          // both halves shifted right, nothing crosses
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, a) >> (unsigned short)n);
}
__device__ __forceinline__ uint32_t pk_mul_lo_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, a) * __builtin_bit_cast(u16x2, b));
}
__device__ __forceinline__ uint32_t pk_sub_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, a) - __builtin_bit_cast(u16x2, b));
}
// a packed word with its -0 halves set to +0
__device__ __forceinline__ uint32_t drop_negzero_pk(uint32_t w) {
    const uint32_t nonzero = pk_min_u16(w & 0x7FFF7FFFu, 0x00010001u);        // 1 in each half that is not +-0
    return w & ((nonzero << 15) | 0x7FFF7FFFu);
}
__device__ __forceinline__ uint4 drop_negzero_vec(uint4 v) {
    return make_uint4(drop_negzero_pk(v.x), drop_negzero_pk(v.y), drop_negzero_pk(v.z), drop_negzero_pk(v.w));
}
__device__ __forceinline__ void acc_amax_pk(uint32_t& amax2, uint32_t w) { amax2 = pk_max_u16(amax2, w & 0x7FFF7FFFu); }
__device__ __forceinline__ void acc_amin_pk(uint32_t& amin2_m1, uint32_t w) {
    amin2_m1 = pk_min_u16(amin2_m1, pk_sub_u16(w & 0x7FFF7FFFu, 0x00010001u));
}
constexpr uint32_t AMIN2_INIT_M1 = 0x7F7E7F7Eu;
// two running counts of non-zero magnitudes (each half adds 1 when its magnitude is not 0); at most 65535 words per lane
__device__ __forceinline__ void acc_nnz_pk(uint32_t& nnz2, uint32_t w) {
    nnz2 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, nnz2) + __builtin_bit_cast(u16x2, pk_min_u16(w & 0x7FFF7FFFu, 0x00010001u)));
}
// fp32 bit pattern of the larger half / (magnitude - 1) of the smaller half in the 32-bit form acc_amin keeps
__device__ __forceinline__ uint32_t amax_bits_of(uint32_t amax2) { return max(amax2 << 16, amax2 & 0xFFFF0000u); }
__device__ __forceinline__ uint32_t amin_m1_of(uint32_t amin2_m1) { return (min(amin2_m1 & 0xFFFFu, amin2_m1 >> 16) << 16) | 0xFFFFu; }
// whether one of the 8 values of a vector is a NaN (the fast arithmetic is only exact for finite values; an infinity
// shows in the block's scale instead)
__device__ __forceinline__ bool vec_has_nan(uint4 v) {
    uint32_t m = 0;
    acc_amax_pk(m, v.x); acc_amax_pk(m, v.y); acc_amax_pk(m, v.z); acc_amax_pk(m, v.w);
    return amax_bits_of(m) > 0x7F800000u;
}
// The same pair function for E4M3 / E5M2 through the gfx950 scaled converts, straight from the packed bf16 word:
// v_cvt_scalef32_pk_fp8/bf8_bf16 gives the codes of |x| / 2^-e8 and v_cvt_scalef32_pk_bf16_fp8/bf8 the packed bf16
// values of code * 2^-e8 (exact: a code has at most 4 significant bits), 5 instructions for the pair instead of 18.
// A zero code comes back as 0, where the reference's exponent subtraction leaves 2^(-e8-127) for e8 < 0: the packed
// maximum with that value puts it back (every non-zero result is far above it).  |e8| <= 126 (callers: |e8| <= 100).
// mor_selftest_hw_cast compares it with e8_pair_fast_ref for every finite bf16 value and every e8 in [-100, 100].
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
template <int F, bool CLAMP> __device__ __forceinline__ uint32_t e8_pair_fast_scaled(uint32_t w, int e8) {
    static_assert(Fmt<F>::hw, "E4M3 / E5M2 only");
    const float scale = u2f((uint32_t)(127 - e8) << 23);                      // 2^-e8
    uint32_t mag = w & 0x7FFF7FFFu;
    if constexpr (CLAMP) {          // the reference's hardware cast saturates; the scaled convert returns NaN above fmax
        const uint32_t lim = (F == FMT_E4M3 ? 0x43E0u : 0x4760u) - ((uint32_t)e8 << 7);      // bf16 bits of fmax * 2^-e8
        mag = pk_min_u16(mag, lim | (lim << 16));
    }
    const s16x2 z = {0, 0};
    uint32_t res;
    if constexpr (F == FMT_E4M3) {
        const s16x2 codes = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(z, __builtin_bit_cast(bf16x2v, mag), scale, false);
        res = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(__builtin_bit_cast(uint32_t, codes), scale, false));
    } else {
        const s16x2 codes = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(z, __builtin_bit_cast(bf16x2v, mag), scale, false);
        res = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(__builtin_bit_cast(uint32_t, codes), scale, false));
    }
    const uint32_t art = e8 < 0 ? (uint32_t)(-e8) << 7 : 0u;                  // bf16 bits of 2^(-e8-127)
    res = pk_max_u16(res, art | (art << 16));
    return res | (w & 0x80008000u);
}

// E4M3 / E5M2 values of both halves of a packed bf16 word under a power-of-two scale, as two floats: |x| * 2^e8 to
// codes and code * 2^-e8 back, both by the scaled converts (true arithmetic: a zero code gives 0).  |e8| <= 126.
template <int F> __device__ __forceinline__ f32x2 e8_pair_values(uint32_t mag2, int e8) {
    const float scale = u2f((uint32_t)(127 - e8) << 23);
    const s16x2 z = {0, 0};
    if constexpr (F == FMT_E4M3) {
        const s16x2 codes = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(z, __builtin_bit_cast(bf16x2v, mag2), scale, false);
        return __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(__builtin_bit_cast(uint32_t, codes), scale, false);
    } else {
        const s16x2 codes = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(z, __builtin_bit_cast(bf16x2v, mag2), scale, false);
        return __builtin_amdgcn_cvt_scalef32_pk_f32_bf8(__builtin_bit_cast(uint32_t, codes), scale, false);
    }
}

// keeps the compiler from carrying unpacked copies of a data register from one pass over the block to the next
__device__ __forceinline__ void opaque(uint4& v) { asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }


// ---------------------------------------------------------------- gfx950 block converts (32 values per lane)
// FP6 by the gfx950 block convert: v_cvt_scalef32_pk32_{fp6,bf6}_bf16 turns 32 bf16 values into 32 packed 6-bit codes
// of RNE(x / 2^floor(log2(scale))), saturating, sign kept (E2M3 = "fp6", E3M2 = "bf6"); the library's selftest compares
// it with the software codes over every bf16 value and every scale exponent.  Used when 2^-e8 is a normal float.
typedef __bf16 bf16x32 __attribute__((ext_vector_type(32)));
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x6 __attribute__((ext_vector_type(6)));
__device__ __forceinline__ bool fp6_hw_ok(int e8) { return e8 >= -126 && e8 <= 126; }
template <int F> __device__ __forceinline__ u32x6 fp6_block_hw(const uint32_t (&words)[16], int e8) {
    const float scale = u2f((uint32_t)(127 - e8) << 23);
    u32x16 t;
#pragma unroll
    for (int i = 0; i < 16; ++i) t[i] = words[i];
    const bf16x32 x = __builtin_bit_cast(bf16x32, t);
    if constexpr (F == FMT_E2M3) return __builtin_bit_cast(u32x6, __builtin_amdgcn_cvt_scalef32_pk32_fp6_bf16(x, scale));
    else return __builtin_bit_cast(u32x6, __builtin_amdgcn_cvt_scalef32_pk32_bf6_bf16(x, scale));
}
// The inverse block convert, v_cvt_scalef32_pk32_bf16_{fp6,bf6}: 32 packed codes -> 32 bf16 of decode(code) * 2^de.
// Used for |de| <= 100, where every product is a normal bf16 value.
__device__ __forceinline__ bool fp6_decode_hw_ok(int de) { return de >= -100 && de <= 100; }
template <int F> __device__ __forceinline__ u32x16 fp6_block_decode_hw(u32x6 codes, int de) {
    const float scale = u2f((uint32_t)(127 + de) << 23);
    if constexpr (F == FMT_E2M3) return __builtin_bit_cast(u32x16, __builtin_amdgcn_cvt_scalef32_pk32_bf16_fp6(codes, scale));
    else return __builtin_bit_cast(u32x16, __builtin_amdgcn_cvt_scalef32_pk32_bf16_bf6(codes, scale));
}
// quad_perm [J,J,J,J]: every lane of a quad reads lane J of its quad
template <int J> __device__ __forceinline__ uint32_t quad_bcast(uint32_t v) { return dpp_u<J * 0x55>(v); }
// the 4 chunks (16 words) of a quad's block in every lane of the quad
__device__ __forceinline__ void quad_gather(uint4 v, uint32_t (&w)[16]) {
    w[0] = quad_bcast<0>(v.x); w[1] = quad_bcast<0>(v.y); w[2] = quad_bcast<0>(v.z); w[3] = quad_bcast<0>(v.w);
    w[4] = quad_bcast<1>(v.x); w[5] = quad_bcast<1>(v.y); w[6] = quad_bcast<1>(v.z); w[7] = quad_bcast<1>(v.w);
    w[8] = quad_bcast<2>(v.x); w[9] = quad_bcast<2>(v.y); w[10] = quad_bcast<2>(v.z); w[11] = quad_bcast<2>(v.w);
    w[12] = quad_bcast<3>(v.x); w[13] = quad_bcast<3>(v.y); w[14] = quad_bcast<3>(v.z); w[15] = quad_bcast<3>(v.w);
}

}  // namespace mor
