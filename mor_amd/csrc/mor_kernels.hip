// HIP kernels and C ABI of the MoR fake-quantization path for MI355X (gfx950, wave64).
//
// One pass over HBM wherever a quantization block fits in registers:
//   k_rowgroup   blocks 1 x 8G elements (G = 1..256 lanes, 16-byte loads; the MX 1x32 case is G = 4):
//                amax by DPP inside the lane group, quantize from registers, 16-byte stores.
//   k_wgblock    one workgroup per block of up to 65536 elements (128x128 tiles, 1x4096 rows: 256 threads; up to
//                32768 / 65536 elements: 512 / 1024 threads): the block lives in registers as 16-byte vectors;
//                amax / min-nonzero / MoR error sums by DPP + LDS; the MoR decision and the quantization reuse the
//                registers.  A variant reads and writes pairs of elements where rows cannot be read as vectors.
//   k_subblock   blocks of fewer than 256 vectors (8x8 ... 32x32 tiles, short rows): a group of 1 ... 64 lanes per
//                block, several blocks per wave, reductions inside the lane group.
//   k_bigblock   larger blocks of whole vectors: one 512-thread workgroup per block, a pass over the block per step
//                (the repeated reads come from cache).
//   k_elementwise  current-scaling modes (the scale is an argument): flat 16-byte vectors + scalar tail.
//   k_generic    any block shape and alignment (odd columns, partial blocks, huge blocks) and the other flavours:
//                scalar loads, the block is re-read from cache for each pass.
// "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <string.h>
#include <algorithm>

#include "mor_device.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

namespace mor {

constexpr int WG = 256;
constexpr int WAVES = WG / 64;

// MorQuantType, FQ:600-608 (the values written to meta)
enum : int { Q_UNKNOWN = 0, Q_E4M3 = 1, Q_E5M2 = 2, Q_BF16 = 3, Q_E2M3 = 4, Q_E4M3_SMALL = 11, Q_E5M2_SMALL = 12 };

struct Shape {
    int64_t rows, cols, brows, bcols, gy, gx;
};

struct QuantArgs {
    int qmode;        // 1 MoR, 2 fixed format (fmt), 4 current scaling (fmt, scale = clamp)
    int fmt;          // forced format for qmode 2 / 4
    int meta_val;     // value written to meta for qmode 2 / 4; < 0: leave meta alone
    int dyn_range;    // MoR decision by dynamic range instead of quantization error
    float clamp;      // clamp_threshold
};

// ------------------------------------------------------------------------------------------------
// exact one-element quantization with run-time format / scale type (only used inside non-unrolled loops)
template <bool EMU>
__device__ __forceinline__ uint16_t fq_one_exact(uint16_t h, int fmt, bool e8, const Scale& sc) {
    float x = bf16_one(h);
    float r;
    if (e8) {
        switch (fmt) {
            case FMT_E4M3: r = sqdd_exact<FMT_E4M3, true, EMU>(x, sc); break;
            case FMT_E5M2: r = sqdd_exact<FMT_E5M2, true, EMU>(x, sc); break;
            case FMT_E3M2: r = sqdd_exact<FMT_E3M2, true, EMU>(x, sc); break;
            default:       r = sqdd_exact<FMT_E2M3, true, EMU>(x, sc); break;
        }
    } else {
        switch (fmt) {
            case FMT_E4M3: r = sqdd_exact<FMT_E4M3, false, EMU>(x, sc); break;
            case FMT_E5M2: r = sqdd_exact<FMT_E5M2, false, EMU>(x, sc); break;
            case FMT_E3M2: r = sqdd_exact<FMT_E3M2, false, EMU>(x, sc); break;
            default:       r = sqdd_exact<FMT_E2M3, false, EMU>(x, sc); break;
        }
    }
    return store_bf16<EMU>(r);
}

// FQ:610-682 without the error pass: returns Q_UNKNOWN when the error sums are needed.
__device__ __forceinline__ int mor_decide_range(float amax, float amin, float clamp, int dyn_range) {
    float range = 0.0f;
    if (amax == 0.0f) { amax = clamp; range = 1.0f; }
    if (range == 0.0f) range = amax / amin;
    const float e4m3_range = dyn_range ? 28672.0f : 114688.0f;
    if (range <= 7.5f) return Q_E2M3;
    if (range <= e4m3_range) return (amax <= clamp) ? Q_E4M3_SMALL : Q_E4M3;
    if (range <= 939524096.0f) {
        if (dyn_range) return (amax <= clamp) ? Q_E5M2_SMALL : Q_E5M2;
        return Q_UNKNOWN;
    }
    return Q_BF16;
}
__device__ __forceinline__ int mor_decide_error(float amax, float clamp, float e4, float e5) {
    if (e4 <= e5) return (amax <= clamp) ? Q_E4M3_SMALL : Q_E4M3;
    return Q_BF16;
}
__device__ __forceinline__ int mor_fmt_of(int qt) {
    switch (qt) {
        case Q_E2M3: return FMT_E2M3;
        case Q_E4M3: case Q_E4M3_SMALL: return FMT_E4M3;
        case Q_E5M2: case Q_E5M2_SMALL: return FMT_E5M2;
        default: return -1;
    }
}

// One element's two error terms with IEEE divisions, FQ:504-542.
template <bool EMU>
__device__ __forceinline__ void err_terms_exact(float x, bool e8, const Scale& s4, const Scale& s5, float& e4, float& e5) {
    if (x != 0.0f) {
        float q4 = e8 ? sqdd_exact<FMT_E4M3, true, EMU>(x, s4) : sqdd_exact<FMT_E4M3, false, EMU>(x, s4);
        float q5 = e8 ? sqdd_exact<FMT_E5M2, true, EMU>(x, s5) : sqdd_exact<FMT_E5M2, false, EMU>(x, s5);
        e4 += fabsf(q4 / x - 1.0f);
        e5 += fabsf(q5 / x - 1.0f);
    }
}

// ------------------------------------------------------------------------------------------------
// quantize one packed word with an fp32 scale: |x| * s, hardware convert, divide by s, round-half-up store, sign
template <int F> __device__ __forceinline__ uint32_t fq_pair_div(uint32_t w, float s, float r) {
    const f32x2 c = hw_unpack2_low<F>(hw_pack2_low<F>(fabsf(bf16_lo(w)) * s, fabsf(bf16_hi(w)) * s));
    return store_pair<false>(div_by_scale(c.x, s, r), div_by_scale(c.y, s, r)) | (w & 0x80008000u);
}
template <int F> __device__ __forceinline__ uint4 fq_vec_div(uint4 v, float s, float r) {
    uint4 o;
    o.x = fq_pair_div<F>(v.x, s, r);
    o.y = fq_pair_div<F>(v.y, s, r);
    o.z = fq_pair_div<F>(v.z, s, r);
    o.w = fq_pair_div<F>(v.w, s, r);
    return o;
}

// The two error terms of one packed word (FQ:504-542) on magnitudes; s5 = 128 * s4 exactly.
// The reference computes |q / x - 1| with q = c / s.  E8 scale: |q - x| * (1 / x), q - x exact.  FP32 scale:
// with y = x * s the same quantity is |c - y| / y (c - y is exact: c is within a factor 2 of y, or 0), which needs
// neither q nor a division; for E5M2 c5 / 128 - y is one exact fma.  Each term differs from the reference's by
// rounding errors of 1e-7 relative, of either sign, far inside the 1e-6 tolerance on the sums; decisions that would
// depend on less than 1e-5 are recomputed with the reference's divisions by the caller.  The sums are only wanted
// for blocks with amax / min non-zero |x| <= 939524096 (FQ:637), so a non-zero element scales to at least
// 448 / 939524096 and no reciprocal overflows.
// `codes` carries the register of the fp8 codes from one word to the next (the converts write half of it).
template <bool E8>
__device__ __forceinline__ void err_pair_fast(uint32_t w, const Scale& s4, float& e4, float& e5, uint32_t& codes) {
    float a = fabsf(bf16_lo(w)), b = fabsf(bf16_hi(w));
    if constexpr (E8) {
        // q = cast(x 2^e8) 2^-e8 by the scaled converts from the packed word (a zero code gives 0 where the reference's
        // exponent arithmetic leaves 2^(-e8-127): a difference far below the terms' rounding errors); a zero element has
        // q = 0, so its term is 0 * min(1 / 0, FLT_MAX) = 0
        const uint32_t mag2 = w & 0x7FFF7FFFu;
        const f32x2 q4 = e8_pair_values<FMT_E4M3>(mag2, s4.e8), q5 = e8_pair_values<FMT_E5M2>(mag2, s4.e8 + 7);
        const float ya = fminf(__builtin_amdgcn_rcpf(a), 0x1.fffffep127f), yb = fminf(__builtin_amdgcn_rcpf(b), 0x1.fffffep127f);
        e4 = fmaf(fabsf(q4.x - a), ya, e4);
        e5 = fmaf(fabsf(q5.x - a), ya, e5);
        e4 = fmaf(fabsf(q4.y - b), yb, e4);
        e5 = fmaf(fabsf(q5.y - b), yb, e5);
    } else {
        // y + 2^-100 is y for every non-zero element of such a block and keeps the reciprocal of a zero element
        // finite: its codes are 0 and c - x s = 0 (one fma, x s not rounded), so its term is 0 without a select
        const float va = fmaf(a, s4.s, 0x1p-100f), vb = fmaf(b, s4.s, 0x1p-100f);
        codes = hw_pack2_both(va, vb, codes);
        const f32x2 c4 = hw_unpack2_e4m3_low(codes), c5 = hw_unpack2_e5m2_high_div128(codes);
        const float ya = __builtin_amdgcn_rcpf(va), yb = __builtin_amdgcn_rcpf(vb);
        e4 = fmaf(fabsf(fmaf(-a, s4.s, c4.x)), ya, e4);
        e5 = fmaf(fabsf(fmaf(-a, s4.s, c5.x)), ya, e5);
        e4 = fmaf(fabsf(fmaf(-b, s4.s, c4.y)), yb, e4);
        e5 = fmaf(fabsf(fmaf(-b, s4.s, c5.y)), yb, e5);
    }
}

// One element through the fast pair functions (the other half of the word is zero and contributes nothing).
__device__ __forceinline__ uint16_t fq_one_fast(uint16_t h, int fmt, bool e8, const Scale& sc) {
    const uint32_t w = h;
    uint32_t r;
    if (e8) {
        switch (fmt) {
            case FMT_E4M3: r = fq_pair_fast<FMT_E4M3, true>(w, sc); break;
            case FMT_E5M2: r = fq_pair_fast<FMT_E5M2, true>(w, sc); break;
            case FMT_E3M2: r = fq_pair_fast<FMT_E3M2, true>(w, sc); break;
            default:       r = fq_pair_fast<FMT_E2M3, true>(w, sc); break;
        }
    } else {
        switch (fmt) {
            case FMT_E4M3: r = fq_pair_fast<FMT_E4M3, false>(w, sc); break;
            case FMT_E5M2: r = fq_pair_fast<FMT_E5M2, false>(w, sc); break;
            case FMT_E3M2: r = fq_pair_fast<FMT_E3M2, false>(w, sc); break;
            default:       r = fq_pair_fast<FMT_E2M3, false>(w, sc); break;
        }
    }
    return (uint16_t)r;
}

// Walks the elements tid, tid + 256, ... of a bh x bw block in row-major order and calls f(offset of the element
// from the block's first element) without a division per element: (r, c) advance by (256 / bw, 256 % bw) with one
// carry.
// per-wave partial results in LDS -> the workgroup's result, for NW = 4 or 8 waves (sums in a fixed pairwise order)
template <int NW> __device__ __forceinline__ float lds_fmax(const float* s) {
    float m = s[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) m = fmaxf(m, s[w]);
    return m;
}
template <int NW> __device__ __forceinline__ float lds_umaxf(const float* s) {      // maximum of the bit patterns (NaN wins)
    uint32_t m = f2u(s[0]);
#pragma unroll
    for (int w = 1; w < NW; ++w) m = max(m, f2u(s[w]));
    return u2f(m);
}
template <int NW> __device__ __forceinline__ uint32_t lds_umin(const uint32_t* s) {
    uint32_t m = s[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) m = min(m, s[w]);
    return m;
}
template <int NW> __device__ __forceinline__ float lds_sum(const float* s) {
    static_assert(NW == 4 || NW == 8 || NW == 16, "4, 8 or 16 waves");
    float a = (s[0] + s[1]) + (s[2] + s[3]);
    if constexpr (NW >= 8) a += (s[4] + s[5]) + (s[6] + s[7]);
    if constexpr (NW == 16) a += ((s[8] + s[9]) + (s[10] + s[11])) + ((s[12] + s[13]) + (s[14] + s[15]));
    return a;
}

template <int WGS = WG, class F>
__device__ __forceinline__ void for_block_elements(int64_t bh, int64_t bw, int64_t row_pitch, int tid, F&& f) {
    const int64_t step_r = WGS / bw, step_c = WGS % bw;
    int64_t r = tid / bw, c = tid % bw;
#pragma unroll 1
    while (r < bh) {
        f(r * row_pitch + c);
        r += step_r;
        c += step_c;
        if (c >= bw) { c -= bw; ++r; }
    }
}

// generic_block: one workgroup quantizes one block of any shape straight from memory with the exact arithmetic.
// It is the body of k_generic and the fallback of k_wgblock for blocks outside the fast range.  FAST (k_generic, default
// flavour): blocks whose scale is in the fast range use the few-instruction arithmetic, with the same safeguard on
// close MoR decisions as k_wgblock.
template <bool EMU, bool FAST = false, int WGS = WG>
__device__ __forceinline__ void generic_block(const uint16_t* in, uint16_t* out, int32_t* meta, float* stats,
                                              const Shape& sh, const QuantArgs& qa, bool e8, int64_t bid,
                                              float (*s_f)[WGS / 64], uint32_t* s_u, bool allow_fast = false) {
    constexpr int NW = WGS / 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t by = bid / sh.gx, bx = bid - by * sh.gx;
    const int64_t r0 = by * sh.brows, c0 = bx * sh.bcols;
    const int64_t bh = min(sh.brows, sh.rows - r0), bw = min(sh.bcols, sh.cols - c0);
    float amax = 0.0f;
    uint32_t amin_m1 = AMIN_INIT_M1;
    const uint16_t* bin = in + r0 * sh.cols + c0;
    for_block_elements<WGS>(bh, bw, sh.cols, tid, [&](int64_t at) {
        uint32_t a = ((uint32_t)bin[at] << 16) & 0x7FFFFFFFu;
        amax = fmaxf(amax, u2f(a));
        amin_m1 = min(amin_m1, a - 1u);
    });
    amax = group_max(amax, 64);
    amin_m1 = group_umin(amin_m1, 64);
    __syncthreads();
    if (lane == 0) { s_f[0][wave] = amax; s_u[wave] = amin_m1; }
    __syncthreads();
    amax = lds_fmax<NW>(s_f[0]);
    amin_m1 = lds_umin<NW>(s_u);
    const float amin = u2f(amin_m1 + 1u);

    int fmt = qa.fmt;
    int meta_val = qa.meta_val;
    float e4 = 0.0f, e5 = 0.0f;
    if (qa.qmode == 1) {
        int qt = mor_decide_range(amax, amin, qa.clamp, qa.dyn_range);
        if (qt == Q_UNKNOWN) {
            const Scale s4 = make_scale(448.0f / amax), s5 = make_scale(57344.0f / amax);
            bool exact = true;
            if constexpr (FAST && !EMU) {
                if (allow_fast && s4.fast && s4.e8 >= -90 && s4.e8 <= 90) {
                    uint32_t codes = 0;
                    if (e8) for_block_elements<WGS>(bh, bw, sh.cols, tid, [&](int64_t at) { err_pair_fast<true>((uint32_t)bin[at], s4, e4, e5, codes); });
                    else for_block_elements<WGS>(bh, bw, sh.cols, tid, [&](int64_t at) { err_pair_fast<false>((uint32_t)bin[at], s4, e4, e5, codes); });
                    e4 = wave_sum(e4);
                    e5 = wave_sum(e5);
                    __syncthreads();
                    if (lane == 0) { s_f[0][wave] = e4; s_f[1][wave] = e5; }
                    __syncthreads();
                    e4 = lds_sum<NW>(s_f[0]);
                    e5 = lds_sum<NW>(s_f[1]);
                    exact = !(fabsf(e4 - e5) > 1e-5f * fmaxf(e4, e5));       // too close: repeat with the reference's divisions
                    if (exact) { e4 = 0.0f; e5 = 0.0f; }
                }
            }
            if (exact) {
                for_block_elements<WGS>(bh, bw, sh.cols, tid, [&](int64_t at) { err_terms_exact<EMU>(bf16_one(bin[at]), e8, s4, s5, e4, e5); });
                e4 = wave_sum(e4);
                e5 = wave_sum(e5);
                __syncthreads();
                if (lane == 0) { s_f[0][wave] = e4; s_f[1][wave] = e5; }
                __syncthreads();
                e4 = lds_sum<NW>(s_f[0]);
                e5 = lds_sum<NW>(s_f[1]);
            }
            qt = mor_decide_error(amax, qa.clamp, e4, e5);
        }
        meta_val = qt;
        fmt = mor_fmt_of(qt);
    }
    if (tid == 0) {
        if (meta && meta_val >= 0) meta[bid] = meta_val;
        if (stats) { float* s = stats + 4 * bid; s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5; }
    }
    if (!out) return;
    const bool copy = (fmt < 0) || !(amax > 0.0f);
    if (copy && out == in) return;
    const Scale sc = make_scale(copy ? 1.0f : fmax_of(fmt) / amax);
    uint16_t* bout = out + r0 * sh.cols + c0;
    bool fast = false;
    if constexpr (FAST && !EMU) fast = allow_fast && !copy && sc.fast && sc.e8 >= -90 && sc.e8 <= 90;
    if (fast) {
        for_block_elements<WGS>(bh, bw, sh.cols, tid, [&](int64_t at) { bout[at] = fq_one_fast(bin[at], fmt, e8, sc); });
    } else {
        for_block_elements<WGS>(bh, bw, sh.cols, tid, [&](int64_t at) {
            uint16_t h = bin[at];
            if (!copy) h = fq_one_exact<EMU>(h, fmt, e8, sc);
            bout[at] = h;
        });
    }
}

template <bool EMU>
__global__ __launch_bounds__(WG) void k_generic(const uint16_t* in, uint16_t* out, int32_t* __restrict__ meta,
                                                float* __restrict__ stats, Shape sh, QuantArgs qa, int e8, int64_t first) {
    __shared__ float s_f[2][WAVES];
    __shared__ uint32_t s_u[WAVES];
    generic_block<EMU, true>(in, out, meta, stats, sh, qa, (e8 & 1) != 0, first + blockIdx.x, s_f, s_u, (e8 & 2) != 0);
}

// ------------------------------------------------------------------------------------------------
// k_elementwise: modes 4 / 5 (FQ:825-842): every element uses the caller's scale; meta is a constant.
// The host picks the fast kernel when the scale is in the fast range, else (or for the other flavours) the exact one.
// EW_NV = 16-byte vectors per thread of the flat kernels (fewer for small tensors, so that every CU gets work)
template <bool E8, int EW_NV>
__global__ __launch_bounds__(WG) void k_elementwise_fast(const uint16_t* in, uint16_t* out, int32_t* __restrict__ meta,
                                                         int64_t n, int64_t nvec, int64_t nmeta, int fmt, float scale, int meta_val) {
    const Scale sc = make_scale(scale);
    const int64_t stride = (int64_t)gridDim.x * WG;
    const int64_t gtid = (int64_t)blockIdx.x * WG + threadIdx.x;
    if (meta) for (int64_t i = gtid; i < nmeta; i += stride) meta[i] = meta_val;
    const uint4* in4 = reinterpret_cast<const uint4*>(in);
    uint4* out4 = reinterpret_cast<uint4*>(out);
    const int64_t base = (int64_t)blockIdx.x * (EW_NV * WG) + threadIdx.x;
    uint4 v[EW_NV];
#pragma unroll
    for (int k = 0; k < EW_NV; ++k) { int64_t c = base + k * WG; v[k] = make_uint4(0, 0, 0, 0); if (c < nvec) v[k] = load16_rt(in4 + c, streams_in(n)); }
    const bool nt = streams_out(n);
    if (fmt == FMT_E4M3) {
#pragma unroll
        for (int k = 0; k < EW_NV; ++k) { int64_t c = base + k * WG; if (c < nvec) store16_rt(out4 + c, fq_vec_fast<FMT_E4M3, E8, true>(v[k], sc), nt); }
    } else {
#pragma unroll
        for (int k = 0; k < EW_NV; ++k) { int64_t c = base + k * WG; if (c < nvec) store16_rt(out4 + c, fq_vec_fast<FMT_E5M2, E8, true>(v[k], sc), nt); }
    }
#pragma unroll 1
    for (int64_t i = nvec * 8 + gtid; i < n; i += stride) out[i] = fq_one_exact<false>(in[i], fmt, E8, sc);
}

template <bool EMU>
__global__ __launch_bounds__(WG) void k_elementwise_exact(const uint16_t* in, uint16_t* out, int32_t* __restrict__ meta,
                                                          int64_t n, int64_t nmeta, int fmt, int e8, float scale, int meta_val) {
    const Scale sc = make_scale(scale);
    const int64_t stride = (int64_t)gridDim.x * WG;
    const int64_t gtid = (int64_t)blockIdx.x * WG + threadIdx.x;
    if (meta) for (int64_t i = gtid; i < nmeta; i += stride) meta[i] = meta_val;
#pragma unroll 1
    for (int64_t i = gtid; i < n; i += stride) out[i] = fq_one_exact<EMU>(in[i], fmt, e8 != 0, sc);
}

__global__ __launch_bounds__(WG) void k_fill_i32(int32_t* p, int64_t n, int32_t v) {
    for (int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x; i < n; i += (int64_t)gridDim.x * WG) p[i] = v;
}

// bf16 copy (mode 7 and the unused mode digits, FQ:1831-1833): 16-byte vectors and a scalar tail
template <int EW_NV>
__global__ __launch_bounds__(WG) void k_copy(const uint16_t* in, uint16_t* out, int64_t n, int64_t nvec) {
    const int64_t stride = (int64_t)gridDim.x * WG;
    const int64_t gtid = (int64_t)blockIdx.x * WG + threadIdx.x;
    const uint4* in4 = reinterpret_cast<const uint4*>(in);
    uint4* out4 = reinterpret_cast<uint4*>(out);
    const int64_t base = (int64_t)blockIdx.x * (EW_NV * WG) + threadIdx.x;
    uint4 v[EW_NV];
#pragma unroll
    for (int k = 0; k < EW_NV; ++k) { int64_t c = base + k * WG; v[k] = make_uint4(0, 0, 0, 0); if (c < nvec) v[k] = load16_rt(in4 + c, streams_in(n)); }
#pragma unroll
    for (int k = 0; k < EW_NV; ++k) { int64_t c = base + k * WG; if (c < nvec) store16_rt(out4 + c, v[k], streams_out(n)); }
    for (int64_t i = nvec * 8 + gtid; i < n; i += stride) out[i] = in[i];
}

// ------------------------------------------------------------------------------------------------
// k_rowgroup: blocks of 1 x 8G elements; the tensor is a flat array of 16-byte chunks and a block is G
// consecutive chunks held by G consecutive lanes.  A workgroup owns NV * 256 consecutive chunks and issues all of
// its loads before it computes.  The main path is branch-free: the fast result is computed for every chunk and
// replaced by the input for all-zero groups (FQ:802, 814) and for groups whose scale is outside the fast range; the
// latter are redone by a second, non-unrolled exact loop.  GT > 0 fixes the group size at compile time (GT = 128 / 256:
// a block spans 2 / 4 waves, whose maxima meet in LDS); FULL means nchunks is a multiple of NV * 256.
template <int F, bool E8, int NV, int GT, bool FULL, bool SNT = false>
__global__ __launch_bounds__(WG) void k_rowgroup(const uint4* in, uint4* out, int32_t* __restrict__ meta,
                                                 int64_t nchunks, int G, int logG, int meta_val) {
    if constexpr (GT > 0) { G = GT; }
    const int64_t base = (int64_t)blockIdx.x * (NV * WG) + threadIdx.x;
    const bool lnt = streams_in(nchunks * 8);
    uint4 v[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        int64_t c = base + k * WG;
        v[k] = make_uint4(0, 0, 0, 0);
        if (FULL || c < nchunks) v[k] = load16_rt(in + c, lnt);
    }
    // groups wider than a wave (GT = 128 / 256 lanes): the waves' maxima meet in LDS, once for all NV chunks
    float wide_amax[NV];
    if constexpr (GT > 64) {
        __shared__ float s_am[NV][WAVES];
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            float a = 0.0f;
            acc_amax(a, v[k].x); acc_amax(a, v[k].y); acc_amax(a, v[k].z); acc_amax(a, v[k].w);
            a = group_max_t<64>(a, 64);
            if (lane == 0) s_am[k][wave] = a;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < NV; ++k)
            wide_amax[k] = (GT == 256) ? fmaxf(fmaxf(s_am[k][0], s_am[k][1]), fmaxf(s_am[k][2], s_am[k][3]))
                                       : fmaxf(s_am[k][wave & 2], s_am[k][(wave & 2) + 1]);
    }
    const bool snt = SNT || (GT > 64 && streams_out(nchunks * 8));
    uint32_t slow = 0;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        int64_t c = base + k * WG;
        float amax = 0.0f;
        if constexpr (GT > 64) amax = wide_amax[k];
        else {
            acc_amax(amax, v[k].x); acc_amax(amax, v[k].y); acc_amax(amax, v[k].z); acc_amax(amax, v[k].w);
            amax = group_max_t<GT>(amax, G);
        }
        Scale sc;
        if constexpr (E8) sc = make_scale_e8<F>(amax);
        else sc = make_scale(Fmt<F>::fmax / amax);
        const bool quant = (amax > 0.0f) && sc.fast;
        const uint4 q = fq_vec_fast<F, E8>(v[k], sc);
        uint4 r;
        r.x = quant ? q.x : v[k].x;
        r.y = quant ? q.y : v[k].y;
        r.z = quant ? q.z : v[k].z;
        r.w = quant ? q.w : v[k].w;
        if ((amax > 0.0f) && !sc.fast) slow |= 1u << k;
        if (FULL || c < nchunks) {
            if constexpr (GT > 64) store16_rt(out + c, r, snt);
            else store16<SNT>(out + c, r);
            if (meta_val >= 0 && (c & (G - 1)) == 0) meta[c >> logG] = meta_val;
        }
    }
    if (slow) {
        if constexpr (GT > 64) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                int64_t c = base + k * WG;
                if (!((slow >> k) & 1u) || !(FULL || c < nchunks)) continue;
                const Scale sc = make_scale(Fmt<F>::fmax / wide_amax[k]);
                uint4 r;
                r.x = fq_pair_exact<F, E8, false>(v[k].x, sc);
                r.y = fq_pair_exact<F, E8, false>(v[k].y, sc);
                r.z = fq_pair_exact<F, E8, false>(v[k].z, sc);
                r.w = fq_pair_exact<F, E8, false>(v[k].w, sc);
                out[c] = r;
            }
        } else {
#pragma unroll 1
            for (int k = 0; k < NV; ++k) {
                if (!((slow >> k) & 1u)) continue;
                int64_t c = base + k * WG;
                uint4 x = in[c];                    // when out == in this is the input again: it was stored back above
                float amax = 0.0f;
                acc_amax(amax, x.x); acc_amax(amax, x.y); acc_amax(amax, x.z); acc_amax(amax, x.w);
                amax = group_max_t<GT>(amax, G);
                const Scale sc = make_scale(Fmt<F>::fmax / amax);
                uint4 r;
                r.x = fq_pair_exact<F, E8, false>(x.x, sc);
                r.y = fq_pair_exact<F, E8, false>(x.y, sc);
                r.z = fq_pair_exact<F, E8, false>(x.z, sc);
                r.w = fq_pair_exact<F, E8, false>(x.w, sc);
                out[c] = r;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// ------------------------------------------------------------------------------------------------
// k_wgblock: one workgroup per quantization block, the block held in registers (NV 16-byte vectors per lane).
// Chunk ch = k * 256 + tid of the block sits at block row ch / cpr, chunk column ch % cpr.
// MOR: per-block format selection (FQ:610-682), else one forced format.  FULL: every block is complete and has
// exactly NV * 256 chunks, so no predicates.  NT: streaming loads and stores.  Blocks outside the fast range go
// through generic_block.  WGS threads per workgroup: 256, or 512 for one-row blocks of more than 8192 elements.
// GATHER: the block's elements are read and written pair by pair (odd column counts, pointers or block widths that are
// not multiples of 16 bytes): a lane's words are pairs of neighbouring elements of a row; every later step is
// elementwise, so nothing else changes.
template <bool MOR, bool E8, int NV, bool FULL, int NT, int WGS = WG, bool GATHER = false>
__global__ __launch_bounds__(WGS) void k_wgblock(const uint4* in, uint4* out, int32_t* __restrict__ meta,
                                                 float* __restrict__ stats, Shape sh, QuantArgs qa, int cpr, int cpr_shift,
                                                 int64_t first) {
    constexpr int NW = WGS / 64;
    __shared__ float s_f[2][NW];
    __shared__ uint32_t s_u[NW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Workgroup -> block.  cpr_shift bit 8 (large tensors whose block grid is a multiple of 8 wide): consecutive
    // workgroup ids go round the 8 XCDs, and each XCD takes a band of gx / 8 block columns, walking it row by row.
    int64_t bid = first + blockIdx.x;       // (a launch holds a slice of the blocks, see for_slices)
    if (cpr_shift >= 256) {            // (a negative cpr_shift means a chunk count per row that is not a power of two)
        const int64_t xcd = bid & 7, j = bid >> 3, per = sh.gx >> 3, byb = j / per;
        bid = byb * sh.gx + xcd * per + (j - byb * per);
        cpr_shift &= 255;
        if (cpr_shift == 255) cpr_shift = -1;
    }
    const int64_t by = bid / sh.gx, bx = bid - by * sh.gx;
    const int64_t r0 = by * sh.brows, c0 = bx * sh.bcols;
    const uint32_t row_stride = (uint32_t)(sh.cols >> 3);          // chunks per tensor row
    const uint4* bin = in + (r0 * row_stride + (c0 >> 3));
    uint4* bout = out ? out + (r0 * row_stride + (c0 >> 3)) : nullptr;
    const int rows_valid = (int)min(sh.brows, sh.rows - r0);
    const int cols_valid = (int)min((int64_t)cpr, (sh.cols - c0) >> 3);
    const int nch = (int)sh.brows * cpr;

    uint4 v[NV];
    uint32_t off[NV];
    bool ok[NV];
    // GATHER: word s of a lane is pair s * WGS + tid of the block's valid part, pairs counted row by row (the last pair of
    // a row of odd width has one element); the walk advances by WGS pairs per word, without a division per word.  A pair
    // is one 4-byte access at a 2-byte-aligned address.
    typedef uint32_t u32_a2 __attribute__((aligned(2)));
    const int g_bw = (int)min(sh.bcols, sh.cols - c0);
    const int g_pr = (g_bw + 1) >> 1;                                   // pairs per row
    const int g_step_r = WGS / g_pr, g_step_c = WGS % g_pr;
    const uint32_t g_cols = (uint32_t)sh.cols;
    if constexpr (GATHER) {
        const uint16_t* src = reinterpret_cast<const uint16_t*>(in) + (r0 * sh.cols + c0);
        int r = tid / g_pr, cp = tid - r * g_pr;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            ok[k] = true;
            off[k] = 0;
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                w[j] = 0;
                if (r < rows_valid) {
                    const uint16_t* p = src + ((uint32_t)r * g_cols + 2u * (uint32_t)cp);
                    w[j] = (2 * cp + 1 < g_bw) ? *reinterpret_cast<const u32_a2*>(p) : (uint32_t)*p;
                }
                r += g_step_r; cp += g_step_c;
                if (cp >= g_pr) { cp -= g_pr; ++r; }
            }
            v[k] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    } else {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        int ch = k * WGS + tid;
        int r = cpr_shift >= 0 ? (ch >> cpr_shift) : (ch / cpr);
        int cc = ch - r * cpr;
        ok[k] = FULL || ((ch < nch) && (r < rows_valid) && (cc < cols_valid));
        off[k] = (uint32_t)r * row_stride + (uint32_t)cc;
        if (ok[k]) v[k] = load16<(NT == 1)>(bin + off[k]);
    }
    }
    // the store of one result vector (GATHER: pair by pair along the same walk, which `put` is called in order of)
    int g_r = tid / g_pr, g_cp = tid - g_r * g_pr;
    auto put = [&](int k, uint4 q) {
        if constexpr (GATHER) {
            uint16_t* dst = reinterpret_cast<uint16_t*>(out) + (r0 * sh.cols + c0);
            const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (g_r < rows_valid) {
                    uint16_t* p = dst + ((uint32_t)g_r * g_cols + 2u * (uint32_t)g_cp);
                    if (2 * g_cp + 1 < g_bw) *reinterpret_cast<u32_a2*>(p) = w[j];
                    else *p = (uint16_t)w[j];
                }
                g_r += g_step_r; g_cp += g_step_c;
                if (g_cp >= g_pr) { g_cp -= g_pr; ++g_r; }
            }
        } else {
            store16<(NT != 0)>(bout + off[k], q);
        }
    };

    // pass 1 (registers): amax and min over non-zero magnitudes, FQ:407-485
    // (packed 16-bit integer maxima / minima of both halves of a word; the data stays packed in its registers)
    uint32_t amax2 = 0, amin2_m1 = AMIN2_INIT_M1;
#pragma unroll
    for (int k = 0; k < NV; ++k)
        if (ok[k]) {
            acc_amax_pk(amax2, v[k].x); acc_amax_pk(amax2, v[k].y); acc_amax_pk(amax2, v[k].z); acc_amax_pk(amax2, v[k].w);
            if constexpr (MOR) { acc_amin_pk(amin2_m1, v[k].x); acc_amin_pk(amin2_m1, v[k].y); acc_amin_pk(amin2_m1, v[k].z); acc_amin_pk(amin2_m1, v[k].w); }
            opaque(v[k]);
        }
    uint32_t amax_b = group_umax(amax_bits_of(amax2), 64);
    uint32_t amin_m1 = AMIN_INIT_M1;
    if constexpr (MOR) amin_m1 = group_umin(amin_m1_of(amin2_m1), 64);
    if (lane == 0) { s_f[0][wave] = u2f(amax_b); s_u[wave] = amin_m1; }
    __syncthreads();
    amax_b = f2u(lds_umaxf<NW>(s_f[0]));
    amin_m1 = lds_umin<NW>(s_u);
    const float amax = u2f(amax_b);
    const float amin = u2f(amin_m1 + 1u);

    // scales of the two fp8 formats; the fp6 scales differ from s4 by 2^4 / 2^6, inside the margin of `fast`
    const Scale s4 = make_scale(448.0f / amax), s5 = make_scale(57344.0f / amax);
    // (a NaN in the block shows as amax_b above the bits of infinity: the exact path takes its maximum as the reference does)
    if (amax_b > 0x7F800000u || (amax > 0.0f && !(s4.e8 >= -90 && s4.e8 <= 90 && s4.fast))) {           // uniform over the workgroup
        generic_block<false, false, WGS>(reinterpret_cast<const uint16_t*>(in), reinterpret_cast<uint16_t*>(out), meta, stats,
                             sh, qa, E8, bid, s_f, s_u);
        return;
    }

    int fmt = qa.fmt;
    int meta_val = qa.meta_val;
    float e4 = 0.0f, e5 = 0.0f;
    if constexpr (MOR) {
        int qt = mor_decide_range(amax, amin, qa.clamp, qa.dyn_range);
        if (qt == Q_UNKNOWN) {
            // pass 2 (registers): the two error sums, FQ:487-584.  amax > 0 here.
            __syncthreads();                     // s_f[0] has been read by every wave
            uint32_t codes = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k)
                if (ok[k]) {
                    err_pair_fast<E8>(v[k].x, s4, e4, e5, codes);
                    err_pair_fast<E8>(v[k].y, s4, e4, e5, codes);
                    err_pair_fast<E8>(v[k].z, s4, e4, e5, codes);
                    err_pair_fast<E8>(v[k].w, s4, e4, e5, codes);
                }
#pragma unroll
            for (int k = 0; k < NV; ++k) if (ok[k]) opaque(v[k]);
            e4 = wave_sum(e4);
            e5 = wave_sum(e5);
            if (lane == 0) { s_f[0][wave] = e4; s_f[1][wave] = e5; }
            __syncthreads();
            e4 = lds_sum<NW>(s_f[0]);
            e5 = lds_sum<NW>(s_f[1]);
            if (!(fabsf(e4 - e5) > 1e-5f * fmaxf(e4, e5))) {
                // The sums above divide with a Newton step.  When they are too close for that to be trusted with
                // the decision, repeat them with IEEE divisions (from memory, non-unrolled: this is rare).
                const uint16_t* in16 = reinterpret_cast<const uint16_t*>(in);
                const int64_t bh = min(sh.brows, sh.rows - r0), bw = min(sh.bcols, sh.cols - c0);
                e4 = 0.0f; e5 = 0.0f;
#pragma unroll 1
                for (int64_t i = tid; i < bh * bw; i += WGS) {
                    int64_t r = i / bw, c = i - r * bw;
                    err_terms_exact<false>(bf16_one(in16[(r0 + r) * sh.cols + c0 + c]), E8, s4, s5, e4, e5);
                }
                e4 = wave_sum(e4);
                e5 = wave_sum(e5);
                __syncthreads();
                if (lane == 0) { s_f[0][wave] = e4; s_f[1][wave] = e5; }
                __syncthreads();
                e4 = lds_sum<NW>(s_f[0]);
                e5 = lds_sum<NW>(s_f[1]);
            }
            qt = mor_decide_error(amax, qa.clamp, e4, e5);
        }
        meta_val = qt;
        fmt = mor_fmt_of(qt);
    }
    if (tid == 0) {
        if (meta && meta_val >= 0) meta[bid] = meta_val;
        if (stats) { float* s = stats + 4 * bid; s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5; }
    }
    if (!out) return;

    // pass 3 (registers): quantize and store, FQ:733-851
    if ((fmt < 0) || !(amax > 0.0f)) {
        if (out != in) {
#pragma unroll
            for (int k = 0; k < NV; ++k) if (ok[k]) put(k, v[k]);
        }
        return;
    }
    if constexpr (!E8) {
        if (fmt == FMT_E4M3 || fmt == FMT_E5M2) {
            const float r4 = 1.0f / s4.s;            // 1 / s5 = r4 / 128 exactly
            if (fmt == FMT_E4M3) {
#pragma unroll
                for (int k = 0; k < NV; ++k) if (ok[k]) put(k, fq_vec_div<FMT_E4M3>(v[k], s4.s, r4));
            } else {
#pragma unroll
                for (int k = 0; k < NV; ++k) if (ok[k]) put(k, fq_vec_div<FMT_E5M2>(v[k], s5.s, r4 * 0.0078125f));
            }
            return;
        }
    }
    const Scale sc = make_scale(fmax_of(fmt) / amax);
    switch (fmt) {
        case FMT_E4M3:
#pragma unroll
            for (int k = 0; k < NV; ++k) if (ok[k]) put(k, fq_vec_fast<FMT_E4M3, E8>(v[k], sc));
            break;
        case FMT_E5M2:
#pragma unroll
            for (int k = 0; k < NV; ++k) if (ok[k]) put(k, fq_vec_fast<FMT_E5M2, E8>(v[k], sc));
            break;
        case FMT_E3M2:
            if constexpr (!MOR) {
#pragma unroll
                for (int k = 0; k < NV; ++k) if (ok[k]) put(k, fq_vec_fast<FMT_E3M2, E8>(v[k], sc));
            }
            break;
        default:
#pragma unroll
            for (int k = 0; k < NV; ++k) if (ok[k]) put(k, fq_vec_fast<FMT_E2M3, E8>(v[k], sc));
            break;
    }
}

struct DivU32 {   // x / d for 32-bit x by multiply-shift (d >= 1)
    uint32_t d, mul, shift;
};
static DivU32 make_div(uint32_t d) {
    DivU32 r{d, 0, 0};
    if (d <= 1) { r.mul = 0; r.shift = 0; return r; }
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;                       // ceil(log2 d)
    r.mul = (uint32_t)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
    r.shift = l;
    return r;
}
__device__ __forceinline__ uint32_t div_u32(uint32_t x, const DivU32& d) {
    if (d.d <= 1) return x;
    uint32_t t = __umulhi(x, d.mul);
    return (t + ((x - t) >> 1)) >> (d.shift - 1);
}

// ------------------------------------------------------------------------------------------------
// k_subblock: blocks of fewer than 256 vectors (8 x 8 ... 32 x 32 tiles, rows of 24 ... 1536 elements, MoR on 1 x 32):
// a group of L = 1, 2, 4 ... 64 consecutive lanes holds one block, NV <= 4 vectors per lane, so a wave works on 64 / L
// blocks at once and a workgroup on 256 / L (one workgroup per such block would leave most of its lanes idle: 8 x 8
// tiles of a 4096 x 6144 tensor took 354 us, now 17.4 us, the time of a copy).  Reductions stay inside the group (DPP and shuffles, no LDS); the steps
// are those of k_wgblock, lane groups of a wave diverging where their blocks choose different formats.  Blocks that
// need the exact arithmetic (a NaN, a scale outside the fast range, MoR error sums too close to call) are flagged and
// done afterwards by the whole workgroup through generic_block.
template <bool MOR, bool E8, int NV>
__global__ __launch_bounds__(WG) void k_subblock(const uint4* in, uint4* out, int32_t* __restrict__ meta,
                                                 float* __restrict__ stats, Shape sh, QuantArgs qa, int cpr, int L, int logL,
                                                 int64_t first, DivU32 d_gx, DivU32 d_cpr) {
    __shared__ float s_f[2][WAVES];
    __shared__ uint32_t s_u[WAVES];
    __shared__ uint32_t s_hard[WG];
    const int tid = threadIdx.x;
    const int g = tid >> logL, l = tid & (L - 1), groups = WG >> logL;
    const int64_t nblocks = sh.gy * sh.gx;
    const int64_t bid0 = (first + blockIdx.x) * groups;
    const int64_t bid = bid0 + g;
    const bool valid = bid < nblocks;
    s_hard[tid] = 0;
    __syncthreads();

    const int64_t by = valid ? (int64_t)div_u32((uint32_t)bid, d_gx) : 0, bx = valid ? bid - by * sh.gx : 0;   // (fewer than 2^31 blocks)
    const int64_t r0 = by * sh.brows, c0 = bx * sh.bcols;
    const uint32_t row_stride = (uint32_t)(sh.cols >> 3);
    const uint4* bin = in + (r0 * row_stride + (c0 >> 3));
    uint4* bout = out ? out + (r0 * row_stride + (c0 >> 3)) : nullptr;
    const int rows_valid = (int)min(sh.brows, sh.rows - r0);
    const int cols_valid = (int)min((int64_t)cpr, (sh.cols - c0) >> 3);
    const int nchb = (int)sh.brows * cpr;
    const bool nt_in = streams_in(sh.rows * sh.cols), nt_out = streams_out(sh.rows * sh.cols);

    uint4 v[NV];
    uint32_t off[NV];
    bool ok[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int j = l + k * L, r = (int)div_u32((uint32_t)j, d_cpr), cc = j - r * cpr;
        ok[k] = valid && j < nchb && r < rows_valid && cc < cols_valid;
        off[k] = (uint32_t)r * row_stride + (uint32_t)cc;
        v[k] = make_uint4(0, 0, 0, 0);
        if (ok[k]) v[k] = load16_rt(bin + off[k], nt_in);
    }
    // pass 1: amax and min over non-zero magnitudes, FQ:407-485 (zeros of idle lanes change neither)
    uint32_t amax2 = 0, amin2_m1 = AMIN2_INIT_M1;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        acc_amax_pk(amax2, v[k].x); acc_amax_pk(amax2, v[k].y); acc_amax_pk(amax2, v[k].z); acc_amax_pk(amax2, v[k].w);
        if constexpr (MOR) { acc_amin_pk(amin2_m1, v[k].x); acc_amin_pk(amin2_m1, v[k].y); acc_amin_pk(amin2_m1, v[k].z); acc_amin_pk(amin2_m1, v[k].w); }
    }
    const uint32_t amax_b = group_umax(amax_bits_of(amax2), L);
    uint32_t amin_m1 = AMIN_INIT_M1;
    if constexpr (MOR) amin_m1 = group_umin(amin_m1_of(amin2_m1), L);
    const float amax = u2f(amax_b);
    const float amin = u2f(amin_m1 + 1u);
    const Scale s4 = make_scale(448.0f / amax), s5 = make_scale(57344.0f / amax);
    bool hard = amax_b > 0x7F800000u || (amax > 0.0f && !(s4.e8 >= -90 && s4.e8 <= 90 && s4.fast));

    int fmt = qa.fmt;
    int meta_val = qa.meta_val;
    float e4 = 0.0f, e5 = 0.0f;
    if constexpr (MOR) {
        int qt = Q_UNKNOWN;
        if (!hard) qt = mor_decide_range(amax, amin, qa.clamp, qa.dyn_range);
        // (the group sums use shuffles: every lane of the wave takes part, with zeros where its block needs no sums)
        const bool want = valid && !hard && qt == Q_UNKNOWN;
        uint32_t codes = 0;
        if (want) {
#pragma unroll
            for (int k = 0; k < NV; ++k)
                if (ok[k]) {
                    err_pair_fast<E8>(v[k].x, s4, e4, e5, codes);
                    err_pair_fast<E8>(v[k].y, s4, e4, e5, codes);
                    err_pair_fast<E8>(v[k].z, s4, e4, e5, codes);
                    err_pair_fast<E8>(v[k].w, s4, e4, e5, codes);
                }
        }
        e4 = group_sum(e4, L);
        e5 = group_sum(e5, L);
        if (want) {
            if (!(fabsf(e4 - e5) > 1e-5f * fmaxf(e4, e5))) hard = true;        // too close for the reciprocal-based sums
            else qt = mor_decide_error(amax, qa.clamp, e4, e5);
        }
        meta_val = qt;
        fmt = mor_fmt_of(qt);
    }
    if (valid && hard && l == 0) s_hard[g] = 1;
    if (valid && !hard) {
        if (l == 0) {
            if (meta && meta_val >= 0) meta[bid] = meta_val;
            if (stats) { float* s = stats + 4 * bid; s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5; }
        }
        // pass 3: quantize and store, FQ:733-851
        if (out) {
            if ((fmt < 0) || !(amax > 0.0f)) {
                if (out != in) {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], v[k], nt_out);
                }
            } else if (!E8 && (fmt == FMT_E4M3 || fmt == FMT_E5M2)) {
                const float r4 = 1.0f / s4.s;            // 1 / s5 = r4 / 128 exactly
                if (fmt == FMT_E4M3) {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], fq_vec_div<FMT_E4M3>(v[k], s4.s, r4), nt_out);
                } else {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], fq_vec_div<FMT_E5M2>(v[k], s5.s, r4 * 0.0078125f), nt_out);
                }
            } else {
                const Scale sc = make_scale(fmax_of(fmt) / amax);
                // (one branch per format around the loop over the vectors, not one per vector)
                if (fmt == FMT_E4M3) {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], fq_vec_fast<FMT_E4M3, E8>(v[k], sc), nt_out);
                } else if (fmt == FMT_E5M2) {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], fq_vec_fast<FMT_E5M2, E8>(v[k], sc), nt_out);
                } else if (!MOR && fmt == FMT_E3M2) {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], fq_vec_fast<FMT_E3M2, E8>(v[k], sc), nt_out);
                } else {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], fq_vec_fast<FMT_E2M3, E8>(v[k], sc), nt_out);
                }
            }
        }
    }
    // the flagged blocks, one after the other, by the whole workgroup (their inputs are untouched: blocks are disjoint)
    // (most workgroups have none: one vote instead of a walk over up to 256 flags, each an LDS round trip)
    if (!__syncthreads_or(valid && hard ? 1 : 0)) return;
#pragma unroll 1
    for (int g2 = 0; g2 < groups; ++g2) {
        if (!s_hard[g2]) continue;                 // uniform over the workgroup
        __syncthreads();
        generic_block<false, false, WG>(reinterpret_cast<const uint16_t*>(in), reinterpret_cast<uint16_t*>(out), meta, stats,
                                        sh, qa, E8, bid0 + g2, s_f, s_u);
    }
}

// ------------------------------------------------------------------------------------------------
// k_bigblock: blocks of more than 16384 elements whose rows can be read as 16-byte vectors (rows of 28672 or 131072
// elements, 256 x 256 tiles, ...).  One 512-thread workgroup per block, as the reference's one thread block per block
// (FQ:1782-1790).  The block does not fit the registers, so every pass reads it again, four vectors in flight per
// lane; the second and third read come from L2 / the last-level cache, HBM still sees one read and one write.
// The steps are those of k_wgblock.
constexpr int BIG_WG = 512;
template <bool MOR, bool E8>
__global__ __launch_bounds__(BIG_WG) void k_bigblock(const uint4* in, uint4* out, int32_t* __restrict__ meta,
                                                     float* __restrict__ stats, Shape sh, QuantArgs qa, int64_t first) {
    constexpr int WGS = BIG_WG, NW = WGS / 64, UN = 4;
    __shared__ float s_f[2][NW];
    __shared__ uint32_t s_u[NW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t bid = first + blockIdx.x;
    const int64_t by = bid / sh.gx, bx = bid - by * sh.gx;
    const int64_t r0 = by * sh.brows, c0 = bx * sh.bcols;
    const uint32_t row_stride = (uint32_t)(sh.cols >> 3);          // chunks per tensor row
    const uint4* bin = in + (r0 * row_stride + (c0 >> 3));
    uint4* bout = out ? out + (r0 * row_stride + (c0 >> 3)) : nullptr;
    const int rows_valid = (int)min(sh.brows, sh.rows - r0);
    const int cpr = (int)(min(sh.bcols, sh.cols - c0) >> 3);       // chunks per row of the block's valid part
    const int nch = rows_valid * cpr;                              // (the host checks brows * cols / 8 < 2^31)
    const int step_r = WGS / cpr, step_c = WGS % cpr;
    // chunk tid + j * WGS of the valid part, j = 0, 1, ...: the walk advances by WGS chunks without a division
    auto sweep = [&](bool nt, auto&& f) {
        int r = tid / cpr, cc = tid - r * cpr;
        for (int64_t i = tid; i < nch; i += UN * WGS) {        // (64-bit: i + u * WGS may pass 2^31)
            uint4 v[UN];
            uint32_t off[UN];
            bool ok[UN];
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                ok[u] = i + u * WGS < nch;
                off[u] = (uint32_t)r * row_stride + (uint32_t)cc;
                r += step_r; cc += step_c;
                if (cc >= cpr) { cc -= cpr; ++r; }
                if (ok[u]) v[u] = load16_rt(bin + off[u], nt);
            }
#pragma unroll
            for (int u = 0; u < UN; ++u) if (ok[u]) f(v[u], off[u]);
        }
    };

    // pass 1: amax and min over non-zero magnitudes, FQ:407-485 (packed 16-bit integer maxima / minima)
    uint32_t amax2 = 0, amin2_m1 = AMIN2_INIT_M1;
    sweep(false, [&](uint4 v, uint32_t) {
        acc_amax_pk(amax2, v.x); acc_amax_pk(amax2, v.y); acc_amax_pk(amax2, v.z); acc_amax_pk(amax2, v.w);
        if constexpr (MOR) { acc_amin_pk(amin2_m1, v.x); acc_amin_pk(amin2_m1, v.y); acc_amin_pk(amin2_m1, v.z); acc_amin_pk(amin2_m1, v.w); }
    });
    uint32_t amax_b = group_umax(amax_bits_of(amax2), 64);
    uint32_t amin_m1 = AMIN_INIT_M1;
    if constexpr (MOR) amin_m1 = group_umin(amin_m1_of(amin2_m1), 64);
    if (lane == 0) { s_f[0][wave] = u2f(amax_b); s_u[wave] = amin_m1; }
    __syncthreads();
    amax_b = f2u(lds_umaxf<NW>(s_f[0]));
    amin_m1 = lds_umin<NW>(s_u);
    const float amax = u2f(amax_b);
    const float amin = u2f(amin_m1 + 1u);

    const Scale s4 = make_scale(448.0f / amax), s5 = make_scale(57344.0f / amax);
    // a NaN in the block, or a scale outside the range of the few-instruction arithmetic: the exact path
    if (amax_b > 0x7F800000u || (amax > 0.0f && !(s4.e8 >= -90 && s4.e8 <= 90 && s4.fast))) {           // uniform over the workgroup
        generic_block<false, false, WGS>(reinterpret_cast<const uint16_t*>(in), reinterpret_cast<uint16_t*>(out), meta, stats,
                                         sh, qa, E8, bid, s_f, s_u);
        return;
    }

    int fmt = qa.fmt;
    int meta_val = qa.meta_val;
    float e4 = 0.0f, e5 = 0.0f;
    if constexpr (MOR) {
        int qt = mor_decide_range(amax, amin, qa.clamp, qa.dyn_range);
        if (qt == Q_UNKNOWN) {
            // pass 2: the two error sums, FQ:487-584.  amax > 0 here.
            __syncthreads();                     // s_f[0] has been read by every wave
            uint32_t codes = 0;
            sweep(false, [&](uint4 v, uint32_t) {
                err_pair_fast<E8>(v.x, s4, e4, e5, codes);
                err_pair_fast<E8>(v.y, s4, e4, e5, codes);
                err_pair_fast<E8>(v.z, s4, e4, e5, codes);
                err_pair_fast<E8>(v.w, s4, e4, e5, codes);
            });
            e4 = wave_sum(e4);
            e5 = wave_sum(e5);
            if (lane == 0) { s_f[0][wave] = e4; s_f[1][wave] = e5; }
            __syncthreads();
            e4 = lds_sum<NW>(s_f[0]);
            e5 = lds_sum<NW>(s_f[1]);
            if (!(fabsf(e4 - e5) > 1e-5f * fmaxf(e4, e5))) {
                // too close for the reciprocal-based sums to be trusted with the decision: IEEE divisions (rare)
                const uint16_t* in16 = reinterpret_cast<const uint16_t*>(in);
                const int64_t bh = rows_valid, bw = min(sh.bcols, sh.cols - c0);
                e4 = 0.0f; e5 = 0.0f;
#pragma unroll 1
                for (int64_t i = tid; i < bh * bw; i += WGS) {
                    int64_t r = i / bw, c = i - r * bw;
                    err_terms_exact<false>(bf16_one(in16[(r0 + r) * sh.cols + c0 + c]), E8, s4, s5, e4, e5);
                }
                e4 = wave_sum(e4);
                e5 = wave_sum(e5);
                __syncthreads();
                if (lane == 0) { s_f[0][wave] = e4; s_f[1][wave] = e5; }
                __syncthreads();
                e4 = lds_sum<NW>(s_f[0]);
                e5 = lds_sum<NW>(s_f[1]);
            }
            qt = mor_decide_error(amax, qa.clamp, e4, e5);
        }
        meta_val = qt;
        fmt = mor_fmt_of(qt);
    }
    if (tid == 0) {
        if (meta && meta_val >= 0) meta[bid] = meta_val;
        if (stats) { float* s = stats + 4 * bid; s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5; }
    }
    if (!out) return;

    // pass 3: quantize and store, FQ:733-851 (the last read of the block: streamed when the tensor streams)
    const bool nt_in = streams_in(sh.rows * sh.cols), nt_out = streams_out(sh.rows * sh.cols);
    if ((fmt < 0) || !(amax > 0.0f)) {
        if (out != in) sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, v, nt_out); });
        return;
    }
    if constexpr (!E8) {
        if (fmt == FMT_E4M3 || fmt == FMT_E5M2) {
            const float r4 = 1.0f / s4.s;            // 1 / s5 = r4 / 128 exactly
            if (fmt == FMT_E4M3) sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, fq_vec_div<FMT_E4M3>(v, s4.s, r4), nt_out); });
            else sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, fq_vec_div<FMT_E5M2>(v, s5.s, r4 * 0.0078125f), nt_out); });
            return;
        }
    }
    const Scale sc = make_scale(fmax_of(fmt) / amax);
    switch (fmt) {
        case FMT_E4M3: sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, fq_vec_fast<FMT_E4M3, E8>(v, sc), nt_out); }); break;
        case FMT_E5M2: sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, fq_vec_fast<FMT_E5M2, E8>(v, sc), nt_out); }); break;
        case FMT_E3M2:
            if constexpr (!MOR) sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, fq_vec_fast<FMT_E3M2, E8>(v, sc), nt_out); });
            break;
        default: sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, fq_vec_fast<FMT_E2M3, E8>(v, sc), nt_out); }); break;
    }
}

// ------------------------------------------------------------------------------------------------
// Debug view: per block amax, fp32 scale, biased exponent of the scale.
__global__ __launch_bounds__(WG) void k_block_stats(const uint16_t* __restrict__ in, Shape sh, float fmax,
                                                    float* __restrict__ amax_o, float* __restrict__ scale_o,
                                                    int32_t* __restrict__ e8m0_o, int64_t first) {
    __shared__ float s_f[WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t bid = first + blockIdx.x;
    const int64_t by = bid / sh.gx, bx = bid - by * sh.gx;
    const int64_t r0 = by * sh.brows, c0 = bx * sh.bcols;
    const int64_t bh = min(sh.brows, sh.rows - r0), bw = min(sh.bcols, sh.cols - c0);
    float amax = 0.0f;
    for (int64_t i = tid; i < bh * bw; i += WG) {
        int64_t r = i / bw, c = i - r * bw;
        amax = fmaxf(amax, fabsf(bf16_one(in[(r0 + r) * sh.cols + c0 + c])));
    }
    amax = group_max(amax, 64);
    if (lane == 0) s_f[wave] = amax;
    __syncthreads();
    if (tid == 0) {
        amax = fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3]));
        float s = amax > 0.0f ? fmax / amax : 1.0f;
        amax_o[bid] = amax;
        scale_o[bid] = s;
        e8m0_o[bid] = (int32_t)((f2u(s) >> 23) & 0xFF);
    }
}

// ------------------------------------------------------------------------------------------------
// Exhaustive check of the hardware converts against the software model, in range.
__global__ __launch_bounds__(WG) void k_selftest_hw_cast(unsigned long long* mism) {
    unsigned long long bad4 = 0, bad5 = 0, bad_scaled = 0;
    const uint64_t stride = (uint64_t)gridDim.x * WG;
    for (uint64_t i = (uint64_t)blockIdx.x * WG + threadIdx.x; i < (1ull << 32); i += stride) {
        float v = u2f((uint32_t)i);
        float a = fabsf(v);
        if (a <= 448.0f) {
            uint32_t hw = f2u(hw_unpack<FMT_E4M3, 0>(hw_pack2<FMT_E4M3>(v, 0.0f)));
            bad4 += (hw != f2u(cast_hwmodel_exact<FMT_E4M3>(v)));
        }
        if (a <= 57344.0f) {
            uint32_t hw = f2u(hw_unpack<FMT_E5M2, 1>(hw_pack2<FMT_E5M2>(0.0f, v)));
            bad5 += (hw != f2u(cast_hwmodel_exact<FMT_E5M2>(v)));
        }
        // the scaled converts against the plain ones: codes and decoded values, both lanes of the pair
        if (a <= 448.0f) {
            const float o = u2f((uint32_t)i ^ 0x00400000u);              // the other value of the pair (same exponent)
            const uint32_t both = hw_pack2_both(v, o, 0xA5A5A5A5u);
            const uint32_t p4 = hw_pack2<FMT_E4M3>(v, o), p5 = hw_pack2<FMT_E5M2>(v * 128.0f, o * 128.0f);
            const f32x2 c4 = hw_unpack2_e4m3_low(both), c5 = hw_unpack2_e5m2_high_div128(both);
            bool ok = ((both & 0xFFFFu) == (p4 & 0xFFFFu)) && ((both >> 16) == (p5 & 0xFFFFu));
            ok = ok && f2u(c4.x) == f2u(hw_unpack<FMT_E4M3, 0>(p4)) && f2u(c4.y) == f2u(hw_unpack<FMT_E4M3, 1>(p4));
            ok = ok && f2u(c5.x) == f2u(hw_unpack<FMT_E5M2, 0>(p5) * 0.0078125f) && f2u(c5.y) == f2u(hw_unpack<FMT_E5M2, 1>(p5) * 0.0078125f);
            const uint32_t l4 = hw_pack2_low<FMT_E4M3>(v, o);
            const f32x2 d4 = hw_unpack2_low<FMT_E4M3>(l4);
            ok = ok && ((l4 & 0xFFFFu) == (p4 & 0xFFFFu)) && f2u(d4.x) == f2u(c4.x) && f2u(d4.y) == f2u(c4.y);
            bad_scaled += !ok;
        }
        if (a <= 57344.0f) {
            const float o = u2f((uint32_t)i ^ 0x00400000u);
            const uint32_t p5 = hw_pack2<FMT_E5M2>(v, o), l5 = hw_pack2_low<FMT_E5M2>(v, o);
            const f32x2 d5 = hw_unpack2_low<FMT_E5M2>(l5);
            bad_scaled += !(((l5 & 0xFFFFu) == (p5 & 0xFFFFu)) && f2u(d5.x) == f2u(hw_unpack<FMT_E5M2, 0>(p5)) && f2u(d5.y) == f2u(hw_unpack<FMT_E5M2, 1>(p5)));
        }
    }
    // the power-of-two pair function through the scaled converts against the one through ldexp and exponent
    // arithmetic: every bf16 pattern (finite or not counted alike: only finite ones reach it) and every e8 in [-100, 100]
    for (uint64_t i = (uint64_t)blockIdx.x * WG + threadIdx.x; i < 65536ull * 201ull; i += stride) {
        const uint32_t h = (uint32_t)(i & 0xFFFFu);
        const int e8 = (int)(i >> 16) - 100;
        if ((h & 0x7F80u) == 0x7F80u) continue;                    // Inf / NaN: such blocks do not take the fast path
        const uint32_t w = h | ((h ^ 0x8055u) << 16);               // the other half: another finite value or the same class
        if ((w & 0x7F800000u) == 0x7F800000u) continue;
        // (without the clamp the pair function is only used on blocks scaled by their own amax: nothing above fmax)
        const float big = ldexpf(fmaxf(fabsf(bf16_lo(w)), fabsf(bf16_hi(w))), e8);
        bool ok = big > 448.0f || e8_pair_fast_scaled<FMT_E4M3, false>(w, e8) == e8_pair_fast_ref<FMT_E4M3, false>(w, e8);
        ok = ok && (big > 57344.0f || e8_pair_fast_scaled<FMT_E5M2, false>(w, e8) == e8_pair_fast_ref<FMT_E5M2, false>(w, e8));
        ok = ok && e8_pair_fast_scaled<FMT_E4M3, true>(w, e8) == e8_pair_fast_ref<FMT_E4M3, true>(w, e8);
        ok = ok && e8_pair_fast_scaled<FMT_E5M2, true>(w, e8) == e8_pair_fast_ref<FMT_E5M2, true>(w, e8);
        bad_scaled += !ok;
    }
    if (bad4) atomicAdd(&mism[0], bad4);
    if (bad5) atomicAdd(&mism[1], bad5);
    if (bad_scaled) atomicAdd(&mism[2], bad_scaled);
}

// ------------------------------------------------------------------------------------------------
// fp32 elementwise test ops, FQ:854-875
__global__ __launch_bounds__(WG) void k_quant_dequant(const float* __restrict__ in, float* __restrict__ out, int64_t n, int fmt) {
    for (int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x; i < n; i += (int64_t)gridDim.x * WG) {
        float v = in[i], r;
        switch (fmt) {
            case FMT_E4M3: r = cast_sw_exact<FMT_E4M3>(v); break;
            case FMT_E5M2: r = cast_sw_exact<FMT_E5M2>(v); break;
            case FMT_E3M2: r = cast_sw_exact<FMT_E3M2>(v); break;
            default:       r = cast_sw_exact<FMT_E2M3>(v); break;
        }
        out[i] = r;
    }
}

// FQ:865-875 + FQ:259-281: per-element power-of-two scale of 448 / value, software E4M3 cast.
__global__ __launch_bounds__(WG) void k_e4m3_e8_scale(const float* __restrict__ in, float* __restrict__ out, int64_t n, int rne) {
    for (int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x; i < n; i += (int64_t)gridDim.x * WG) {
        float v = in[i];
        float sf = 448.0f / v;
        uint32_t sb = f2u(sf), vb = f2u(v);
        int e8 = (int)((sb >> 23) & 0xFF) - 127;
        int ve = (int)((vb >> 23) & 0xFF);
        uint32_t vman = vb & 0x7FFFFFu;
        if (rne) {
            uint32_t sman = sb & 0x7FFFFFu;
            uint32_t guard = (sman >> 22) & 1u;
            uint32_t sticky = (sman & ((1u << 22) - 1u)) != 0;
            if (guard == 1 && vman <= 6815744u && ve + e8 < 135) {
                if (sticky == 1 || (e8 & 1)) e8++;
            }
        }
        ve += e8;
        if (ve < 0) ve = 0;
        float scaled = u2f((vb & 0x80000000u) | ((uint32_t)ve << 23) | vman);
        uint32_t db = f2u(cast_sw_exact<FMT_E4M3>(scaled));
        int de = (int)((db >> 23) & 0xFF) - e8;
        if (de < 0) de = 0;
        out[i] = u2f((db & 0x80000000u) | ((uint32_t)de << 23) | (db & 0x7FFFFFu));
    }
}

}  // namespace mor

// ================================================================================================
// host side
using namespace mor;

static thread_local char g_err[512] = "";

int mor_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int mor_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return mor_fail(MOR_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MOR_OK;
}

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }
static inline int ilog2(int64_t x) { int l = 0; while ((1ll << l) < x) ++l; return l; }

static int grid_for(int64_t work_items, int per_cu = 8) {
    // enough workgroups to fill 256 CUs several times over, capped so grid-stride loops stay short
    int64_t want = cdiv(work_items, WG);
    int64_t cap = 256ll * per_cu;
    if (want < 1) want = 1;
    return (int)(want < cap ? want : cap);
}

// A launch holds fewer than 2^32 threads per dimension (a larger grid wraps without an error): kernels that take one
// workgroup per block are launched slice by slice, f(first block, blocks of the slice).
constexpr int64_t LAUNCH_SLICE = (int64_t)1 << 22;
template <class Fn> static void for_slices(int64_t nblocks, Fn&& f) {
    for (int64_t first = 0; first < nblocks; first += LAUNCH_SLICE) f(first, (int)std::min(LAUNCH_SLICE, nblocks - first));
}

extern "C" const char* mor_last_error(void) { return g_err; }
extern "C" const char* mor_version(void) { return "mor_hip 0.1 (gfx950)"; }

static int validate_shape(const void* input, int64_t rows, int64_t cols, int64_t brows, int64_t bcols) {
    if (!input) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "input is NULL");
    if (rows <= 0 || cols <= 0) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "rows and cols must be positive (got %lld x %lld)", (long long)rows, (long long)cols);
    if (brows <= 0 || bcols <= 0) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "block dims must be positive (got %lld x %lld)", (long long)brows, (long long)bcols);
    if (cdiv(rows, brows) * cdiv(cols, bcols) > 0x7FFFFFFFll) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "too many blocks");
    // 2^35 elements (64 GiB of bf16): the flat kernels' grids, one workgroup per 512 vectors, stay below 2^24 workgroups
    if (rows > MOR_MAX_ELEMENTS / cols) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "tensor too large (more than 2^35 elements)");
    return MOR_OK;
}

template <int F, bool E8>
static void launch_rowgroup_f(const uint4* i4, uint4* o4, int32_t* meta, int64_t nchunks, int G, int meta_val, hipStream_t st) {
    // small tensors take fewer chunks per workgroup so that every CU still gets several workgroups; outputs of 4 MiB
    // and more are written with streaming stores, which keeps the input and whatever the caller has in
    // the last-level cache from being evicted by data nobody reads back soon (measured: 45.6 -> 41.9 us at 8192^2)
    const int lg = ilog2(G);
    if (G > 64) {                         // 128 or 256 lanes per block: rows of 1024 / 2048 elements
        constexpr int NV = 2;
        const int grid = (int)cdiv(nchunks, (int64_t)NV * WG);
        if (G == 128) k_rowgroup<F, E8, NV, 128, false><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val);
        else k_rowgroup<F, E8, NV, 256, false><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val);
        return;
    }
    // Two vectors per lane: many small workgroups interleave their loads and stores more finely than few large ones
    // (measured at 8192^2 with 8 / 4 / 2 / 1 vectors per lane: E4M3 41.3 / 40.6 / 39.3 / 42.4 us, E2M3 41.8 / 40.1 /
    // 37.9 / 38.6 us).
    constexpr int NV = 2;
    if (nchunks * 16 >= ((int64_t)4 << 20) && nchunks % ((int64_t)NV * WG) == 0 && (G == 4 || G == 16)) {
        const int64_t grid64 = nchunks / ((int64_t)NV * WG);
        if (grid64 <= 0x7FFFFFFFll) {
            const int grid = (int)grid64;
            if (G == 4) k_rowgroup<F, E8, NV, 4, true, true><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val);
            else k_rowgroup<F, E8, NV, 16, true, true><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val);
            return;
        }
    }
    {
        const int grid = (int)cdiv(nchunks, (int64_t)NV * WG);
        if (nchunks * 16 >= ((int64_t)4 << 20)) k_rowgroup<F, E8, NV, 0, false, true><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val);
        else k_rowgroup<F, E8, NV, 0, false><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val);
    }
}

template <bool E8>
static void launch_rowgroup(int fmt, const void* in, void* out, int32_t* meta, int64_t nchunks, int G, int meta_val, hipStream_t st) {
    const uint4* i4 = static_cast<const uint4*>(in);
    uint4* o4 = static_cast<uint4*>(out);
    switch (fmt) {
        case FMT_E4M3: launch_rowgroup_f<FMT_E4M3, E8>(i4, o4, meta, nchunks, G, meta_val, st); break;
        case FMT_E5M2: launch_rowgroup_f<FMT_E5M2, E8>(i4, o4, meta, nchunks, G, meta_val, st); break;
        case FMT_E3M2: launch_rowgroup_f<FMT_E3M2, E8>(i4, o4, meta, nchunks, G, meta_val, st); break;
        default:       launch_rowgroup_f<FMT_E2M3, E8>(i4, o4, meta, nchunks, G, meta_val, st); break;
    }
}

template <bool MOR, bool E8, int NV, int WGS = WG>
static void launch_wgblock_nv(bool full, int grid, const uint4* i4, uint4* o4, int32_t* meta, float* stats,
                              const Shape& sh, const QuantArgs& qa, int cpr, int shift, hipStream_t st) {
    // Streaming stores for outputs that do not fit an L2 anyway (>= 4 MiB): the quantized tensor then does not evict
    // the input or the caller's data from the caches (measured at 8192^2: 42.7 -> 40.4 us, at 4096^2: 13.3 -> 10.3 us).
    // Tensors whose traffic exceeds twice the 256 MB last-level cache stream their loads as well.
    const int64_t out_bytes = sh.rows * sh.cols * 2;
    const int ntm = (2 * out_bytes > ((int64_t)512 << 20)) ? 1 : (out_bytes >= ((int64_t)4 << 20)) ? 2 : 0;
    // Large grids run 3 workgroups per CU (unused dynamic LDS caps the occupancy the registers would allow at 5):
    // fewer tiles in flight keep the memory system on fewer DRAM pages at a time (16384 x 14336 MoR: 176.8 -> 170.8 us,
    // 8192^2 block E4M3: 41.4 -> 40.1 us), while a grid that fits the chip at once wants every slot (4096^2: 9.2
    // against 10.8 us).
    const size_t dyn_lds = (NV == 8 && WGS == WG && grid >= 4096) ? 53000 : 0;
    // Tensors beyond the last-level cache: each XCD takes a band of gx / 8 block columns and walks it row by row, so
    // that the blocks sharing a DRAM page are in flight on one XCD at about the same time (16384 x 14336, 128 x 128
    // blocks: MoR 170 -> 157 us, block E4M3 166.6 -> 153.8 us; no difference at 8192^2 and below).
    const int shift_arg = (ntm == 1 && sh.gx % 8 == 0) ? ((shift & 255) | 256) : shift;
#define MOR_WGBLOCK(FULL, NT) for_slices(grid, [&](int64_t first, int count) { \
        k_wgblock<MOR, E8, NV, FULL, NT, WGS><<<count, WGS, dyn_lds, st>>>(i4, o4, meta, stats, sh, qa, cpr, shift_arg, first); })
    if (full) {
        if (ntm == 1) MOR_WGBLOCK(true, 1); else if (ntm == 2) MOR_WGBLOCK(true, 2); else MOR_WGBLOCK(true, 0);
    } else {
        if (ntm == 1) MOR_WGBLOCK(false, 1); else if (ntm == 2) MOR_WGBLOCK(false, 2); else MOR_WGBLOCK(false, 0);
    }
#undef MOR_WGBLOCK
}

template <bool MOR, bool E8>
static void launch_wgblock(const void* in, void* out, int32_t* meta, float* stats, const Shape& sh, const QuantArgs& qa, hipStream_t st) {
    int cpr = (int)(sh.bcols / 8);
    int nch = (int)sh.brows * cpr;
    int nv = (int)cdiv(nch, WG);
    int shift = is_pow2(cpr) ? ilog2(cpr) : -1;
    int grid = (int)(sh.gy * sh.gx);
    const uint4* i4 = static_cast<const uint4*>(in);
    uint4* o4 = static_cast<uint4*>(out);
    int NVc = nv <= 1 ? 1 : nv <= 2 ? 2 : nv <= 4 ? 4 : 8;
    bool full = (sh.rows % sh.brows == 0) && (sh.cols % sh.bcols == 0) && (nch == NVc * WG);
    if (nch > 8 * WG) {
        // up to 32768 / 65536 elements (rows of 28672 elements, 256 x 256 tiles): still in registers, 8 vectors per lane
        // of 512 / 1024 threads (8192^2 in 256 x 256 tiles: block E4M3 59.5 us with a pass over the block per step)
        const bool w512 = nch <= 8 * 512;
        full = (sh.rows % sh.brows == 0) && (sh.cols % sh.bcols == 0) && (nch == 8 * (w512 ? 512 : 1024));
        if (w512) launch_wgblock_nv<MOR, E8, 8, 512>(full, grid, i4, o4, meta, stats, sh, qa, cpr, shift, st);
        // (tiles of several rows: 16 vectors per lane of 512 threads; 256 x 256 tiles at 8192^2 take 47 against 52 us with
        // 1024 threads, MoR 64 against 68 us; one row of 65536 elements 44 against 43 us)
        else if (sh.brows > 1) launch_wgblock_nv<MOR, E8, 16, 512>(full, grid, i4, o4, meta, stats, sh, qa, cpr, shift, st);
        else launch_wgblock_nv<MOR, E8, 8, 1024>(full, grid, i4, o4, meta, stats, sh, qa, cpr, shift, st);
        return;
    }
    switch (NVc) {
        case 1: launch_wgblock_nv<MOR, E8, 1>(full, grid, i4, o4, meta, stats, sh, qa, cpr, shift, st); break;
        case 2: launch_wgblock_nv<MOR, E8, 2>(full, grid, i4, o4, meta, stats, sh, qa, cpr, shift, st); break;
        case 4: launch_wgblock_nv<MOR, E8, 4>(full, grid, i4, o4, meta, stats, sh, qa, cpr, shift, st); break;
        default:
            // a contiguous block (one long row) is faster with 512 threads and 4 vectors per lane (rows of 14336 elements:
            // 167 -> 157 us at 16384 rows, 38.7 -> 36.2 us at 4096 rows); a 128 x 128 tile is not
            if (sh.brows == 1) launch_wgblock_nv<MOR, E8, 4, 512>(full, grid, i4, o4, meta, stats, sh, qa, cpr, shift, st);
            else launch_wgblock_nv<MOR, E8, 8>(full, grid, i4, o4, meta, stats, sh, qa, cpr, shift, st);
            break;
    }
}

// Blocks of up to 16384 elements whose rows cannot be read as 16-byte vectors: the same kernel with element-wise
// loads and stores (4097 x 4095 MoR 128 x 128: 84 us through k_generic).
template <bool MOR, bool E8>
static void launch_wgblock_gather(const void* in, void* out, int32_t* meta, float* stats, const Shape& sh, const QuantArgs& qa, hipStream_t st) {
    const int grid = (int)(sh.gy * sh.gx);
    const int nv = (int)cdiv(sh.brows * ((sh.bcols + 1) / 2), 4 * WG);        // a lane's word is one pair of a row
    const uint4* i4 = static_cast<const uint4*>(in);
    uint4* o4 = static_cast<uint4*>(out);
#define MOR_GATHER(NV) for_slices(grid, [&](int64_t first, int count) { \
        k_wgblock<MOR, E8, NV, false, 0, WG, true><<<count, WG, 0, st>>>(i4, o4, meta, stats, sh, qa, 1, 0, first); })
    if (nv <= 1) MOR_GATHER(1); else if (nv <= 2) MOR_GATHER(2); else if (nv <= 4) MOR_GATHER(4); else MOR_GATHER(8);
#undef MOR_GATHER
}

// Blocks of fewer than 256 vectors: lane groups (k_subblock).
template <bool MOR, bool E8>
static void launch_subblock(const void* in, void* out, int32_t* meta, float* stats, const Shape& sh, const QuantArgs& qa, hipStream_t st) {
    const int cpr = (int)(sh.bcols / 8);
    const int nchb = (int)sh.brows * cpr;
    int logL = 0;
    // vectors per lane: 4 where the group still has 8 lanes or so, else 2 (a 4096 x 6144 tensor in rows of 192 elements:
    // 29.8 / 18.9 / 17.2 us with 1 / 2 / 4 vectors per lane, in 8 x 8 tiles 21.9 / 17.4 / 18.8 us, the plain copy 17 us)
    const int pref = nchb >= 24 ? 4 : 2;
    while ((1 << logL) * pref < nchb && logL < 6) ++logL;
    const int L = 1 << logL, nv = (int)cdiv(nchb, L), groups = WG >> logL;
    const uint4* i4 = static_cast<const uint4*>(in);
    uint4* o4 = static_cast<uint4*>(out);
    const DivU32 d_gx = make_div((uint32_t)sh.gx), d_cpr = make_div((uint32_t)cpr);
    for_slices(cdiv(sh.gy * sh.gx, groups), [&](int64_t first, int count) {
        if (nv <= 1) k_subblock<MOR, E8, 1><<<count, WG, 0, st>>>(i4, o4, meta, stats, sh, qa, cpr, L, logL, first, d_gx, d_cpr);
        else if (nv <= 2) k_subblock<MOR, E8, 2><<<count, WG, 0, st>>>(i4, o4, meta, stats, sh, qa, cpr, L, logL, first, d_gx, d_cpr);
        else k_subblock<MOR, E8, 4><<<count, WG, 0, st>>>(i4, o4, meta, stats, sh, qa, cpr, L, logL, first, d_gx, d_cpr);
    });
}

// Common driver of mor_fake_quantize / mor_block_format / mor_mor_stats.
static int run_quantize(const void* input, void* output, int32_t* meta, float* stats,
                        int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                        const QuantArgs& qa, bool e8, uint32_t flags, hipStream_t st) {
    Shape sh{rows, cols, brows, bcols, cdiv(rows, brows), cdiv(cols, bcols)};
    const bool emu = flags & MOR_FLAG_TORCH_EMULATION;
    const bool fast_ok = !emu && !(flags & MOR_FLAG_SOFTWARE_CAST);
    const int64_t nblocks = sh.gy * sh.gx;
    const uint16_t* in16 = static_cast<const uint16_t*>(input);
    uint16_t* out16 = static_cast<uint16_t*>(output);

    if (qa.qmode == 4) {
        const int64_t n = rows * cols;
        uint32_t sbits;
        memcpy(&sbits, &qa.clamp, 4);
        const int e8v = (int)((sbits >> 23) & 0xFF) - 127;
        if (fast_ok && e8v >= -100 && e8v <= 100) {
            int64_t nvec = (aligned16(input) && aligned16(output)) ? n / 8 : 0;
            {       // two vectors per lane at every size (as k_rowgroup)
                int grid = nvec > 0 ? (int)cdiv(nvec, 2ll * WG) : grid_for(n, 16);
                if (e8) k_elementwise_fast<true, 2><<<grid, WG, 0, st>>>(in16, out16, meta, n, nvec, nblocks, qa.fmt, qa.clamp, qa.meta_val);
                else k_elementwise_fast<false, 2><<<grid, WG, 0, st>>>(in16, out16, meta, n, nvec, nblocks, qa.fmt, qa.clamp, qa.meta_val);
            }
        } else {
            int grid = grid_for(n, 16);
            if (emu) k_elementwise_exact<true><<<grid, WG, 0, st>>>(in16, out16, meta, n, nblocks, qa.fmt, e8, qa.clamp, qa.meta_val);
            else k_elementwise_exact<false><<<grid, WG, 0, st>>>(in16, out16, meta, n, nblocks, qa.fmt, e8, qa.clamp, qa.meta_val);
        }
        return mor_check_launch("k_elementwise");
    }
    const bool vec_ok = fast_ok && aligned16(input) && (!output || aligned16(output)) && cols % 8 == 0 && bcols % 8 == 0
                        && brows * (cols / 8) < 0x7FFFFFFFll;
    const int64_t G = bcols / 8;
    if (qa.qmode == 2 && !stats && output && vec_ok && brows == 1 && cols % bcols == 0 && is_pow2(G) && G <= 256) {
        if (e8) launch_rowgroup<true>(qa.fmt, input, output, meta, rows * cols / 8, (int)G, meta ? qa.meta_val : -1, st);
        else launch_rowgroup<false>(qa.fmt, input, output, meta, rows * cols / 8, (int)G, meta ? qa.meta_val : -1, st);
        return mor_check_launch("k_rowgroup");
    }
    if (vec_ok && brows * (bcols / 8) < WG) {
        if (qa.qmode == 1) {
            if (e8) launch_subblock<true, true>(input, output, meta, stats, sh, qa, st);
            else launch_subblock<true, false>(input, output, meta, stats, sh, qa, st);
        } else {
            if (e8) launch_subblock<false, true>(input, output, meta, stats, sh, qa, st);
            else launch_subblock<false, false>(input, output, meta, stats, sh, qa, st);
        }
        return mor_check_launch("k_subblock");
    }
    if (vec_ok && brows * (bcols / 8) <= 8 * 1024) {
        if (qa.qmode == 1) {
            if (e8) launch_wgblock<true, true>(input, output, meta, stats, sh, qa, st);
            else launch_wgblock<true, false>(input, output, meta, stats, sh, qa, st);
        } else {
            if (e8) launch_wgblock<false, true>(input, output, meta, stats, sh, qa, st);
            else launch_wgblock<false, false>(input, output, meta, stats, sh, qa, st);
        }
        return mor_check_launch("k_wgblock");
    }
    if (vec_ok) {                                   // larger blocks of whole vectors
        const uint4* i4 = static_cast<const uint4*>(input);
        uint4* o4 = static_cast<uint4*>(output);
        for_slices(nblocks, [&](int64_t first, int count) {
            if (qa.qmode == 1) {
                if (e8) k_bigblock<true, true><<<count, BIG_WG, 0, st>>>(i4, o4, meta, stats, sh, qa, first);
                else k_bigblock<true, false><<<count, BIG_WG, 0, st>>>(i4, o4, meta, stats, sh, qa, first);
            } else {
                if (e8) k_bigblock<false, true><<<count, BIG_WG, 0, st>>>(i4, o4, meta, stats, sh, qa, first);
                else k_bigblock<false, false><<<count, BIG_WG, 0, st>>>(i4, o4, meta, stats, sh, qa, first);
            }
        });
        return mor_check_launch("k_bigblock");
    }
    if (fast_ok && brows * ((bcols + 1) / 2) <= 32 * WG && brows * cols < 0x7FFFFFFFll && nblocks <= 0x7FFFFFFFll) {
        if (qa.qmode == 1) {
            if (e8) launch_wgblock_gather<true, true>(input, output, meta, stats, sh, qa, st);
            else launch_wgblock_gather<true, false>(input, output, meta, stats, sh, qa, st);
        } else {
            if (e8) launch_wgblock_gather<false, true>(input, output, meta, stats, sh, qa, st);
            else launch_wgblock_gather<false, false>(input, output, meta, stats, sh, qa, st);
        }
        return mor_check_launch("k_wgblock (element-wise)");
    }
    // bit 0: power-of-two scale; bit 1: the few-instruction arithmetic (hardware converts) is allowed
    const int gflags = (e8 ? 1 : 0) | (fast_ok ? 2 : 0);
    for_slices(nblocks, [&](int64_t first, int count) {
        if (emu) k_generic<true><<<count, WG, 0, st>>>(in16, out16, meta, stats, sh, qa, gflags, first);
        else k_generic<false><<<count, WG, 0, st>>>(in16, out16, meta, stats, sh, qa, gflags, first);
    });
    return mor_check_launch("k_generic");
}

extern "C" int mor_fake_quantize(const void* input, void* output, int32_t* meta,
                                 int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                                 double clamp_threshold, int64_t mode, int64_t sf_type,
                                 uint32_t flags, void* stream) {
    if (int rc = validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!output || !meta) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output / meta is NULL");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int qmode = (int)(mode % 10);                 // FQ:1774
    QuantArgs qa{};
    qa.clamp = (float)clamp_threshold;
    qa.dyn_range = (mode / 100 > 0) ? 1 : 0;            // FQ:1776-1779
    const bool e8 = (sf_type == 2);                     // FQ:1792, 1797
    switch (qmode) {
        case 1: qa.qmode = 1; qa.fmt = -1; qa.meta_val = -1; break;
        case 2: qa.qmode = 2; qa.fmt = FMT_E4M3; qa.meta_val = 1; break;
        case 3: qa.qmode = 2; qa.fmt = FMT_E5M2; qa.meta_val = 2; break;
        case 4: qa.qmode = 4; qa.fmt = FMT_E4M3; qa.meta_val = 1; break;
        case 5: qa.qmode = 4; qa.fmt = FMT_E5M2; qa.meta_val = 2; break;
        default: {
            // FQ:1831-1833, 727-729, 843: bf16 copy, meta 3
            const int64_t nblocks = cdiv(rows, brows) * cdiv(cols, bcols);
            if (output != input) {
                const int64_t n = rows * cols;
                const int64_t nvec = (aligned16(input) && aligned16(output)) ? n / 8 : 0;
                k_copy<2><<<nvec > 0 ? (int)cdiv(nvec, 2ll * WG) : grid_for(n, 16), WG, 0, st>>>(static_cast<const uint16_t*>(input), static_cast<uint16_t*>(output), n, nvec);
            }
            k_fill_i32<<<grid_for(nblocks), WG, 0, st>>>(meta, nblocks, 3);
            return mor_check_launch("k_copy / k_fill_i32");
        }
    }
    return run_quantize(input, output, meta, nullptr, rows, cols, brows, bcols, qa, e8, flags, st);
}

extern "C" int mor_block_format(const void* input, void* output,
                                int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                                int fmt, int64_t sf_type, uint32_t flags, void* stream) {
    if (int rc = validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!output) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output is NULL");
    if (fmt < 0 || fmt > 3) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "unknown format %d", fmt);
    QuantArgs qa{};
    qa.qmode = 2; qa.fmt = fmt; qa.meta_val = -1;
    return run_quantize(input, output, nullptr, nullptr, rows, cols, brows, bcols, qa, sf_type == 2, flags, static_cast<hipStream_t>(stream));
}

extern "C" int mor_mor_stats(const void* input, int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                             double clamp_threshold, int64_t mode, int64_t sf_type, float* stats, void* stream) {
    if (int rc = validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!stats) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "stats is NULL");
    QuantArgs qa{};
    qa.qmode = 1; qa.fmt = -1; qa.meta_val = -1;
    qa.clamp = (float)clamp_threshold;
    qa.dyn_range = (mode / 100 > 0) ? 1 : 0;
    return run_quantize(input, nullptr, nullptr, stats, rows, cols, brows, bcols, qa, sf_type == 2, MOR_FLAG_DEFAULT, static_cast<hipStream_t>(stream));
}

extern "C" int mor_block_stats(const void* input, int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                               float fmax, float* amax, float* scale, int32_t* e8m0, void* stream) {
    if (int rc = validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!amax || !scale || !e8m0) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output pointer is NULL");
    Shape sh{rows, cols, brows, bcols, cdiv(rows, brows), cdiv(cols, bcols)};
    for_slices(sh.gy * sh.gx, [&](int64_t first, int count) {
        k_block_stats<<<count, WG, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const uint16_t*>(input), sh, fmax, amax, scale, e8m0, first);
    });
    return mor_check_launch("k_block_stats");
}

extern "C" int mor_quant_dequant(const float* input, float* output, int64_t n, int fmt, void* stream) {
    if (!input || !output || n < 0) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "bad pointer or size");
    if (fmt < 0 || fmt > 3) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "unknown format %d", fmt);
    if (n == 0) return MOR_OK;
    k_quant_dequant<<<grid_for(n, 16), WG, 0, static_cast<hipStream_t>(stream)>>>(input, output, n, fmt);
    return mor_check_launch("k_quant_dequant");
}

extern "C" int mor_e4m3_with_e8_scale(const float* input, float* output, int64_t n, int rne, void* stream) {
    if (!input || !output || n < 0) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "bad pointer or size");
    if (n == 0) return MOR_OK;
    k_e4m3_e8_scale<<<grid_for(n, 16), WG, 0, static_cast<hipStream_t>(stream)>>>(input, output, n, rne);
    return mor_check_launch("k_e4m3_e8_scale");
}

extern "C" int mor_selftest_hw_cast(uint64_t* mismatches, void* stream) {
    if (!mismatches) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "mismatches is NULL");
    hipStream_t st = static_cast<hipStream_t>(stream);
    k_fill_i32<<<1, WG, 0, st>>>(reinterpret_cast<int32_t*>(mismatches), 6, 0);
    k_selftest_hw_cast<<<256 * 16, WG, 0, st>>>(reinterpret_cast<unsigned long long*>(mismatches));
    return mor_check_launch("k_selftest_hw_cast");
}


// ================================================================================================
// Block / channel scaling (FQ:951-1241, 1459-1752, host FQ:2013-2230, 2431-2660) and e8mx (FQ:1243-1428).
//
// Workspace layout (32-bit words): [0] tensor amax bits, [1] non-zero count, [2..3] spare, then three arrays of
// MAX_PARTIALS per-workgroup partials (error sums of pass 2; amax and non-zero counts of pass 1), then one float
// per block (amax, turned into the block's scale in place).  Nothing is accumulated with atomics except the
// per-column maxima of the column kernel, so all results are independent of scheduling.
namespace mor {

constexpr int WS_HEADER = 4;
constexpr int MAX_PARTIALS = 8192;
constexpr int WS_ERR = WS_HEADER;
constexpr int WS_PAMAX = WS_HEADER + MAX_PARTIALS;
constexpr int WS_PNNZ = WS_HEADER + 2 * MAX_PARTIALS;
constexpr int WS_BLOCKS = WS_HEADER + 3 * MAX_PARTIALS;

__global__ void k_zero_f32(float* p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x; i < n; i += (int64_t)gridDim.x * WG) p[i] = 0.0f;
}

// FQ:998-999: an element counts when |x| > 0 as floats, so a NaN does not
__device__ __forceinline__ int nnz_word(uint32_t w) {
    return (fabsf(bf16_lo(w)) > 0.0f) + (fabsf(bf16_hi(w)) > 0.0f);
}
__device__ __forceinline__ int nan_word(uint32_t w) { return ((w & 0x7FFFu) > 0x7F80u) + ((w & 0x7FFF0000u) > 0x7F800000u); }
__device__ __forceinline__ void acc_amax_nnz(float& amax, int& nnz, uint4 v) {
    acc_amax(amax, v.x); acc_amax(amax, v.y); acc_amax(amax, v.z); acc_amax(amax, v.w);
    nnz += nnz_word(v.x) + nnz_word(v.y) + nnz_word(v.z) + nnz_word(v.w);
}

// one workgroup's amax / nnz -> its slot of the partial arrays; returns the workgroup amax to every thread
__device__ __forceinline__ float publish_partial(uint32_t* ws, float amax, int nnz, float* s_f, int* s_i) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    amax = group_max(amax, 64);
    nnz = wave_sum_i(nnz);
    __syncthreads();
    if (lane == 0) { s_f[wave] = amax; s_i[wave] = nnz; }
    __syncthreads();
    const float a = fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3]));
    if (threadIdx.x == 0) {
        reinterpret_cast<float*>(ws)[WS_PAMAX + blockIdx.x] = a;
        reinterpret_cast<int*>(ws)[WS_PNNZ + blockIdx.x] = s_i[0] + s_i[1] + s_i[2] + s_i[3];
    }
    return a;
}

// tensor amax from the pass-1 partials (every thread of the workgroup gets it)
__device__ __forceinline__ float reduce_partial_amax(const uint32_t* ws, int npart, float* s_f) {
    const float* pa = reinterpret_cast<const float*>(ws) + WS_PAMAX;
    float a = 0.0f;
#pragma unroll 8
    for (int i = threadIdx.x; i < npart; i += WG) a = fmaxf(a, pa[i]);
    a = group_max(a, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s_f[threadIdx.x >> 6] = a;
    __syncthreads();
    return fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3]));
}

// pass 1, blocks 1 x 8G as lane groups over the flat chunk array (FQ:1430-1457, 1611-1629).  A workgroup takes
// tiles of 8 * 256 consecutive chunks, all loads of a tile in flight at once.  block_amax may be NULL (e8mx).
__global__ __launch_bounds__(WG) void k_bs_amax_flat(const uint4* in, uint32_t* ws, float* block_amax,
                                                     int64_t nchunks, int G, int logG) {
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    constexpr int NV = 8;
    float gmax = 0.0f;
    int nnz = 0;
    const int64_t ntiles = (nchunks + NV * WG - 1) / (NV * WG);
    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int64_t base = tile * (NV * WG) + threadIdx.x;
        uint4 v[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            v[k] = make_uint4(0, 0, 0, 0);
            if (base + k * WG < nchunks) v[k] = load16_rt(in + base + k * WG, streams_in(nchunks * 8));
        }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int64_t c = base + k * WG;
            float amax = 0.0f;
            acc_amax_nnz(amax, nnz, v[k]);
            gmax = fmaxf(gmax, amax);
            if (block_amax) {
                amax = group_max(amax, G);
                if (c < nchunks && (c & (G - 1)) == 0) block_amax[c >> logG] = amax;
            }
        }
    }
    publish_partial(ws, gmax, nnz, s_f, s_i);
}

// tensor amax of an unaligned or odd-sized buffer, element by element (e8mx only needs the tensor amax)
__global__ __launch_bounds__(WG) void k_amax_scalar(const uint16_t* in, uint32_t* ws, int64_t n) {
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    float amax = 0.0f;
    for (int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x; i < n; i += (int64_t)gridDim.x * WG)
        amax = fmaxf(amax, fabsf(bf16_one(in[i])));
    publish_partial(ws, amax, 0, s_f, s_i);
}

// pass 1, one workgroup per block of any shape (FQ:951-1015), blocks taken grid-stride;
// vec: 16-byte loads (cols and bcols multiples of 8, aligned base)
__global__ __launch_bounds__(WG) void k_bs_amax_block(const uint16_t* in, uint32_t* ws, float* block_amax, Shape sh, int vec,
                                                      DivU32 d_gx, DivU32 d_cpr) {
    __shared__ float s_f[WAVES];
    __shared__ float s_b[WAVES];
    __shared__ int s_i[WAVES];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t nb = (uint32_t)(sh.gy * sh.gx);
    float gmax = 0.0f;
    int nnz = 0;
    for (uint32_t bid = blockIdx.x; bid < nb; bid += gridDim.x) {
        const uint32_t by = div_u32(bid, d_gx), bx = bid - by * (uint32_t)sh.gx;
        const int64_t r0 = (int64_t)by * sh.brows, c0 = (int64_t)bx * sh.bcols;
        float amax = 0.0f;
        if (vec) {
            const uint32_t row_stride = (uint32_t)(sh.cols >> 3), cpr = (uint32_t)(sh.bcols >> 3);
            const uint4* bin = reinterpret_cast<const uint4*>(in) + (r0 * row_stride + (c0 >> 3));
            const uint32_t nch = (uint32_t)sh.brows * cpr;
#pragma unroll 4
            for (uint32_t i = threadIdx.x; i < nch; i += WG) {
                const uint32_t r = div_u32(i, d_cpr), cc = i - r * cpr;
                acc_amax_nnz(amax, nnz, load16_rt(bin + r * row_stride + cc, streams_in(sh.rows * sh.cols)));
            }
        } else {
            for (int64_t i = threadIdx.x; i < sh.brows * sh.bcols; i += WG) {
                int64_t r = i / sh.bcols, c = i - r * sh.bcols;
                uint32_t a = ((uint32_t)in[(r0 + r) * sh.cols + c0 + c] << 16) & 0x7FFFFFFFu;
                amax = fmaxf(amax, u2f(a));
                nnz += (u2f(a) > 0.0f);
            }
        }
        amax = group_max(amax, 64);
        __syncthreads();
        if (lane == 0) s_b[wave] = amax;
        __syncthreads();
        amax = fmaxf(fmaxf(s_b[0], s_b[1]), fmaxf(s_b[2], s_b[3]));
        if (threadIdx.x == 0) block_amax[bid] = amax;
        gmax = fmaxf(gmax, amax);
    }
    publish_partial(ws, gmax, nnz, s_f, s_i);
}

// The same for blocks of fewer than 256 vectors (8 x 8 ... 32 x 32 tiles, rows of 96 or 768 elements): a group of
// L = 1 ... 64 consecutive lanes per block, as in k_subblock, 256 / L blocks per workgroup and step; the block maximum
// by DPP / shuffles inside the group.  (One workgroup per block: 4096 x 6144 in 8 x 8 tiles 242 us for the whole op.)
__global__ __launch_bounds__(WG) void k_bs_amax_sub(const uint4* in, uint32_t* ws, float* block_amax, Shape sh, int L, int logL,
                                                    DivU32 d_gx, DivU32 d_cpr) {
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    const int tid = threadIdx.x;
    const uint32_t g = (uint32_t)(tid >> logL), l = (uint32_t)(tid & (L - 1)), groups = (uint32_t)(WG >> logL);
    const uint32_t nb = (uint32_t)(sh.gy * sh.gx);                       // (fewer than 2^31 blocks)
    const uint32_t row_stride = (uint32_t)(sh.cols >> 3), cpr = (uint32_t)(sh.bcols >> 3), nchb = (uint32_t)sh.brows * cpr;
    const bool nt = streams_in(sh.rows * sh.cols);
    float gmax = 0.0f;
    int nnz = 0;
    for (uint32_t b0 = blockIdx.x * groups; b0 < nb; b0 += gridDim.x * groups) {
        const uint32_t bid = b0 + g;
        float amax = 0.0f;
        if (bid < nb) {
            const uint32_t by = div_u32(bid, d_gx), bx = bid - by * (uint32_t)sh.gx;
            const uint4* bin = in + ((int64_t)by * sh.brows * row_stride + (((int64_t)bx * sh.bcols) >> 3));
#pragma unroll 4
            for (uint32_t j = l; j < nchb; j += (uint32_t)L) {
                const uint32_t r = div_u32(j, d_cpr), cc = j - r * cpr;
                acc_amax_nnz(amax, nnz, load16_rt(bin + r * row_stride + cc, nt));
            }
        }
        amax = group_max(amax, L);                   // (shuffles: every lane of the wave takes part)
        if (bid < nb && l == 0) block_amax[bid] = amax;
        gmax = fmaxf(gmax, amax);
    }
    publish_partial(ws, gmax, nnz, s_f, s_i);
}


// pass 1, column blocks N x 1 (FQ:1538-1610): a workgroup covers 256 adjacent columns (32 groups of 8) with 8 row
// lanes; a thread takes every 8th row of a row segment, the 8 row lanes meet in LDS and one thread per column merges
// into the (zero-initialised) per-block maxima with atomicMax on the bit patterns of non-negative floats.
__global__ __launch_bounds__(WG) void k_bs_amax_col(const uint16_t* in, uint32_t* ws, float* block_amax, Shape sh,
                                                    int rows_per_wg, int vec) {
    __shared__ float s_m[8][32 * 8 + 8];
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    const int cg = threadIdx.x & 31, rl = threadIdx.x >> 5;
    const int64_t col0 = ((int64_t)blockIdx.x * 32 + cg) * 8;
    const int64_t segs_per_block = (sh.brows + rows_per_wg - 1) / rows_per_wg;
    const int ncol = (int)max((int64_t)0, min((int64_t)8, sh.cols - col0));
    float gmax = 0.0f;
    int nnz = 0;
    // row segments of all block rows, taken grid-stride along y
    for (int64_t seg = blockIdx.y; seg < sh.gy * segs_per_block; seg += gridDim.y) {
        const int64_t by = seg / segs_per_block;
        const int64_t r_begin = by * sh.brows + (seg - by * segs_per_block) * rows_per_wg;
        const int64_t r_end = min(r_begin + rows_per_wg, (by + 1) * sh.brows);
        float m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (vec && ncol == 8) {
            const uint4* in4 = reinterpret_cast<const uint4*>(in);
#pragma unroll 8
            for (int64_t r = r_begin + rl; r < r_end; r += 8) {
                const uint4 v = load16_rt(in4 + ((r * sh.cols + col0) >> 3), streams_in(sh.rows * sh.cols));
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    m[2 * j] = fmaxf(m[2 * j], fabsf(bf16_lo(w[j])));
                    m[2 * j + 1] = fmaxf(m[2 * j + 1], fabsf(bf16_hi(w[j])));
                    nnz += nnz_word(w[j]);
                }
            }
        } else {
            for (int64_t r = r_begin + rl; r < r_end; r += 8)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (j < ncol) {
                        const uint32_t a = ((uint32_t)in[r * sh.cols + col0 + j] << 16) & 0x7FFFFFFFu;
                        m[j] = fmaxf(m[j], u2f(a));
                        nnz += (a != 0);
                    }
        }
        __syncthreads();                       // the previous segment's readers are done
#pragma unroll
        for (int j = 0; j < 8; ++j) s_m[rl][cg * 8 + j] = m[j];
        __syncthreads();
        float cm = s_m[0][threadIdx.x];
#pragma unroll
        for (int k = 1; k < 8; ++k) cm = fmaxf(cm, s_m[k][threadIdx.x]);
        const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
        if (c < sh.cols && cm > 0.0f) atomicMax(reinterpret_cast<uint32_t*>(&block_amax[by * sh.cols + c]), f2u(cm));
        gmax = fmaxf(gmax, cm);
    }
    const uint32_t slot = blockIdx.x + gridDim.x * blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    gmax = group_max(gmax, 64);
    nnz = wave_sum_i(nnz);
    if (lane == 0) { s_f[wave] = gmax; s_i[wave] = nnz; }
    __syncthreads();
    if (threadIdx.x == 0) {
        reinterpret_cast<float*>(ws)[WS_PAMAX + slot] = fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3]));
        reinterpret_cast<int*>(ws)[WS_PNNZ + slot] = s_i[0] + s_i[1] + s_i[2] + s_i[3];
    }
}

// FQ:1059-1093
__device__ __forceinline__ float scaling_factor(float global_amax, float block_amax, int ss_mode) {
    float sf = 1.0f;
    const float fmax = 448.0f;
    if (block_amax < 1e-35f) block_amax = 1e-35f;
    switch (ss_mode) {
        case 1: {
            float ratio = fmax / global_amax;
            uint32_t gman = f2u(ratio) & 0x007FFFFFu;
            float bsf = fmax / block_amax;
            uint32_t bb = f2u(bsf);
            float adj = u2f((bb & 0xFF800000u) | gman);
            sf = (gman <= (bb & 0x007FFFFFu)) ? adj : adj / 2.0f;
            break;
        }
        case 2:
        case 3: sf = fmax / block_amax; break;
        case 4: if (global_amax > 0.0f) sf = fmax / global_amax; break;
        default: break;
    }
    return sf;
}

// pass 1.5 (FQ:1017-1049 + the scale of every block): tensor amax and non-zero count from the partials into the
// header, block amax -> block scale in place
__global__ __launch_bounds__(WG) void k_bs_scales(uint32_t* ws, float* block_amax, int64_t nb, int ss_mode, int npart) {
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    const float gamax = reduce_partial_amax(ws, npart, s_f);
    if (blockIdx.x == 0) {
        const int* pn = reinterpret_cast<const int*>(ws) + WS_PNNZ;
        int n = 0;
#pragma unroll 8
        for (int i = threadIdx.x; i < npart; i += WG) n += pn[i];
        n = wave_sum_i(n);
        if ((threadIdx.x & 63) == 0) s_i[threadIdx.x >> 6] = n;
        __syncthreads();
        if (threadIdx.x == 0) { ws[0] = f2u(gamax); ws[1] = (uint32_t)(s_i[0] + s_i[1] + s_i[2] + s_i[3]); }
    }
    for (int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x; i < nb; i += (int64_t)gridDim.x * WG)
        block_amax[i] = scaling_factor(gamax, block_amax[i], ss_mode);
}

// One element of FQ:1133-1162: zeros give +0 and no error; others E4M3 through the hardware-cast model.
// The power-of-two path is taken for ss_mode 2 (the reference tests the strategy against SF_E8 = 2, FQ:1138).
template <bool E8, bool EMU>
__device__ __forceinline__ float bs_element(float x, const Scale& sc, float& err) {
    if (x == 0.0f) return EMU ? x : 0.0f;
    float dq = sqdd_exact<FMT_E4M3, E8, EMU>(x, sc);
    err += fabsf((dq - x) / x);
    return dq;
}
// Fast version on magnitudes for scales in the fast range: hardware convert; q = c / s by a reciprocal-multiply
// with one exact-residual correction (r = 1 / s correctly rounded, the result is then the rounded quotient);
// error term |q - x| / x through the hardware reciprocal (relative 1e-7, tolerance on the sum 1e-6).
// No selects: a zero element has q = 0, so its term is 0 * min(1 / 0, FLT_MAX) = 0 and its magnitude bits are 0;
// the sign of the input is kept for non-zero halves only (zero inputs come back as +0, FQ:1133-1134), through a
// packed 16-bit mask.
// ERR / OUT: whether the error terms / the output word are wanted (the in-place phases need one of them each).
template <bool E8, bool ERR = true, bool OUT = true>
__device__ __forceinline__ uint32_t bs_pair_fast(uint32_t w, const Scale& sc, float rs, float& err) {
    const float a = fabsf(bf16_lo(w)), b = fabsf(bf16_hi(w));
    float qa, qb;
    if constexpr (E8) {
        // scaled converts from the packed word; a zero code of a non-zero element is the reference's 2^(-e8-127) for
        // e8 < 0 (its exponent subtraction, FQ:296-303), zero inputs are skipped by the reference (FQ:1133) and stay 0
        const f32x2 q = e8_pair_values<FMT_E4M3>(w & 0x7FFF7FFFu, sc.e8);
        const float art = u2f(sc.e8 < 0 ? (uint32_t)(-sc.e8) << 23 : 0u);
        qa = (a == 0.0f) ? 0.0f : fmaxf(q.x, art);
        qb = (b == 0.0f) ? 0.0f : fmaxf(q.y, art);
    } else {
        const f32x2 c = hw_unpack2_low<FMT_E4M3>(hw_pack2_low<FMT_E4M3>(a * sc.s, b * sc.s));
        qa = div_by_scale(c.x, sc.s, rs);
        qb = div_by_scale(c.y, sc.s, rs);
    }
    if constexpr (ERR) {
        const float ya = fminf(__builtin_amdgcn_rcpf(a), 0x1.fffffep127f), yb = fminf(__builtin_amdgcn_rcpf(b), 0x1.fffffep127f);
        err = fmaf(fabsf(qa - a), ya, err);
        err = fmaf(fabsf(qb - b), yb, err);
    }
    if constexpr (!OUT) return 0u;
    const uint32_t nonzero = pk_min_u16(w & 0x7FFF7FFFu, 0x00010001u);        // 1 in each half that is not +-0
    return store_pair<false>(qa, qb) | (w & (nonzero << 15));
}
template <bool E8, bool ERR, bool OUT>
__device__ __forceinline__ uint4 bs_vec_fast(uint4 v, const Scale& sc, float& err) {
    uint4 q;
    q.x = bs_pair_fast<E8, ERR, OUT>(v.x, sc, sc.r, err);
    q.y = bs_pair_fast<E8, ERR, OUT>(v.y, sc, sc.r, err);
    q.z = bs_pair_fast<E8, ERR, OUT>(v.z, sc, sc.r, err);
    q.w = bs_pair_fast<E8, ERR, OUT>(v.w, sc, sc.r, err);
    return q;
}

// pass 2 / pass 4: quantize every element with its block's scale (looked up per chunk, or per column in column
// mode), accumulate the relative error, optionally write.  GATE > 0: run only if meta[0] == GATE.
template <bool E8, bool EMU, bool COL, bool WRITE, bool ERR>
__global__ __launch_bounds__(WG) void k_bs_quant(const uint16_t* in, uint16_t* out, uint32_t* ws, const float* scales,
                                                 const int32_t* meta, int gate, Shape sh, int vec, DivU32 d_rowchunks,
                                                 DivU32 d_brows, DivU32 d_bchunks, DivU32 d_bcols) {
    __shared__ float s_f[WAVES];
    if (gate > 0 && meta[0] != gate) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float err = 0.0f;
    if (vec) {
        const uint32_t row_chunks = (uint32_t)(sh.cols >> 3);
        const uint32_t nchunks = (uint32_t)sh.rows * row_chunks;
        const uint4* in4 = reinterpret_cast<const uint4*>(in);
        uint4* out4 = reinterpret_cast<uint4*>(out);
        for (uint32_t c = blockIdx.x * WG + threadIdx.x; c < nchunks; c += gridDim.x * WG) {
            const uint32_t row = div_u32(c, d_rowchunks), cc = c - row * row_chunks;
            const uint32_t by = div_u32(row, d_brows);
            uint4 v = load16_rt(in4 + c, streams_in(sh.rows * sh.cols));
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
            if constexpr (COL) {
                const float* sp = scales + (int64_t)by * sh.cols + (int64_t)cc * 8;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const Scale s0 = make_scale(sp[2 * j]), s1 = make_scale(sp[2 * j + 1]);
                    float q0 = bs_element<E8, EMU>(bf16_lo(w[j]), s0, err);
                    float q1 = bs_element<E8, EMU>(bf16_hi(w[j]), s1, err);
                    w[j] = store_pair<EMU>(q0, q1);
                }
            } else {
                const uint32_t bx = div_u32(cc, d_bchunks);
                const Scale sc = make_scale(scales[(int64_t)by * sh.gx + bx]);
                if (!EMU && sc.fast && !vec_has_nan(v)) {
                    const float rs = 1.0f / sc.s;
#pragma unroll
                    for (int j = 0; j < 4; ++j) w[j] = bs_pair_fast<E8, ERR, WRITE>(w[j], sc, rs, err);
                } else {
#pragma unroll 1
                    for (int j = 0; j < 4; ++j) {
                        float q0 = bs_element<E8, EMU>(bf16_lo(w[j]), sc, err);
                        float q1 = bs_element<E8, EMU>(bf16_hi(w[j]), sc, err);
                        w[j] = store_pair<EMU>(q0, q1);
                    }
                }
            }
            if constexpr (WRITE) store16_rt(out4 + c, make_uint4(w[0], w[1], w[2], w[3]), streams_out(sh.rows * sh.cols));
        }
    } else {
        const int64_t n = sh.rows * sh.cols;
        for (int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x; i < n; i += (int64_t)gridDim.x * WG) {
            const int64_t row = i / sh.cols, col = i - row * sh.cols;
            const int64_t by = row / sh.brows, bx = col / sh.bcols;
            const Scale sc = make_scale(scales[by * sh.gx + bx]);
            float q = bs_element<E8, EMU>(bf16_one(in[i]), sc, err);
            if constexpr (WRITE) out[i] = store_bf16<EMU>(q);
        }
    }
    if constexpr (ERR) {
        err = wave_sum(err);
        if (lane == 0) s_f[wave] = err;
        __syncthreads();
        if (threadIdx.x == 0) {
            reinterpret_cast<float*>(ws)[WS_ERR + blockIdx.x] = (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]);
        }
    }
}

// pass 2 / pass 4 for column blocks N x 1 with aligned rows (the geometry of k_bs_amax_col): a thread owns 8 adjacent
// columns over a segment of rows, so its 8 scales and their reciprocals are computed once.  Threads whose scales are
// not all in the fast range use the exact arithmetic.
template <bool WRITE, bool ERR>
__global__ __launch_bounds__(WG) void k_bs_quant_col(const uint16_t* in, uint16_t* out, uint32_t* ws, const float* scales,
                                                     const int32_t* meta, int gate, Shape sh, int rows_per_wg) {
    __shared__ float s_f[WAVES];
    if (gate > 0 && meta[0] != gate) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t col0 = ((int64_t)blockIdx.x * WG + threadIdx.x) * 8;
    const int64_t segs_per_block = (sh.brows + rows_per_wg - 1) / rows_per_wg;
    const int64_t row_stride = sh.cols >> 3;
    const uint4* in4 = reinterpret_cast<const uint4*>(in);
    uint4* out4 = reinterpret_cast<uint4*>(out);
    float err = 0.0f;
    const bool nt = streams_out(sh.rows * sh.cols);
    if (col0 < sh.cols) {
        for (int64_t seg = blockIdx.y; seg < sh.gy * segs_per_block; seg += gridDim.y) {
            const int64_t by = seg / segs_per_block;
            const int64_t r_begin = by * sh.brows + (seg - by * segs_per_block) * rows_per_wg;
            const int64_t r_end = min(r_begin + rows_per_wg, (by + 1) * sh.brows);
            const float* sp = scales + by * sh.cols + col0;
            Scale sc[8];
            float rs[8];
            bool fast = true;
#pragma unroll
            for (int j = 0; j < 8; ++j) { sc[j] = make_scale(sp[j]); rs[j] = 1.0f / sc[j].s; fast = fast && sc[j].fast; }
            if (fast) {
#pragma unroll 1
                for (int64_t r = r_begin; r < r_end; r += 4) {
                    uint4 v[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        v[k] = make_uint4(0, 0, 0, 0);
                        if (r + k < r_end) v[k] = load16_rt(in4 + (r + k) * row_stride + (col0 >> 3), streams_in(sh.rows * sh.cols));
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        uint32_t w[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
                        float row_err = 0.0f;
                        if (vec_has_nan(v[k])) {          // a NaN among the 8 values: the exact arithmetic for this vector (rare)
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                float q0 = bs_element<false, false>(bf16_lo(w[j]), sc[2 * j], row_err);
                                float q1 = bs_element<false, false>(bf16_hi(w[j]), sc[2 * j + 1], row_err);
                                w[j] = store_pair<false>(q0, q1);
                            }
                        } else
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            // as bs_pair_fast, with a scale of its own for each of the two columns of the word
                            const float a = fabsf(bf16_lo(w[j])), b = fabsf(bf16_hi(w[j]));
                            const f32x2 c = hw_unpack2_low<FMT_E4M3>(hw_pack2_low<FMT_E4M3>(a * sc[2 * j].s, b * sc[2 * j + 1].s));
                            const float qa = div_by_scale(c.x, sc[2 * j].s, rs[2 * j]);
                            const float qb = div_by_scale(c.y, sc[2 * j + 1].s, rs[2 * j + 1]);
                            if constexpr (ERR) {
                                row_err = fmaf(fabsf(qa - a), fminf(__builtin_amdgcn_rcpf(a), 0x1.fffffep127f), row_err);
                                row_err = fmaf(fabsf(qb - b), fminf(__builtin_amdgcn_rcpf(b), 0x1.fffffep127f), row_err);
                            }
                            if constexpr (WRITE) {
                                const uint32_t nonzero = pk_min_u16(w[j] & 0x7FFF7FFFu, 0x00010001u);
                                w[j] = store_pair<false>(qa, qb) | (w[j] & (nonzero << 15));
                            }
                        }
                        err += row_err;
                        if constexpr (WRITE) {
                            if (r + k < r_end) store16_rt(out4 + (r + k) * row_stride + (col0 >> 3), make_uint4(w[0], w[1], w[2], w[3]), nt);
                        }
                    }
                }
            } else {
#pragma unroll 1
                for (int64_t r = r_begin; r < r_end; ++r) {
                    const uint4 v = in4[r * row_stride + (col0 >> 3)];
                    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float s0 = sp[2 * j], s1 = sp[2 * j + 1];
                        float q0 = bs_element<false, false>(bf16_lo(w[j]), make_scale(s0), err);
                        float q1 = bs_element<false, false>(bf16_hi(w[j]), make_scale(s1), err);
                        w[j] = store_pair<false>(q0, q1);
                    }
                    if constexpr (WRITE) out4[r * row_stride + (col0 >> 3)] = make_uint4(w[0], w[1], w[2], w[3]);
                }
            }
        }
    }
    if constexpr (ERR) {
        err = wave_sum(err);
        if (lane == 0) s_f[wave] = err;
        __syncthreads();
        if (threadIdx.x == 0)
            reinterpret_cast<float*>(ws)[WS_ERR + blockIdx.x + gridDim.x * blockIdx.y] = (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]);
    }
}

// pass 3 (FQ:1178-1241): total error (fixed summation order), the bf16 decision, the scalar outputs.
// npart_stats > 0: the tensor amax and the non-zero count are still per-workgroup partials (single-pass kernel)
// and are reduced here; otherwise they are in the header words.
__global__ __launch_bounds__(WG) void k_bs_finalize(const uint32_t* ws, int npartials, int npart_stats, float threshold,
                                                    int32_t* meta, float* gamax_o, int32_t* gnnz_o, float* gerr_o) {
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    const float* part = reinterpret_cast<const float*>(ws) + WS_ERR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float gamax = u2f(ws[0]);
    int gnnz = (int)ws[1];
    float acc = 0.0f;
    if (npart_stats > 0 && npart_stats == npartials) {
        // the three partial arrays in one sweep, all loads of a batch in flight (three sweeps in a row were 6.4 us
        // of one workgroup's load latency); every sum keeps the order of the separate sweeps
        const float* pa = reinterpret_cast<const float*>(ws) + WS_PAMAX;
        const int* pn = reinterpret_cast<const int*>(ws) + WS_PNNZ;
        float a = 0.0f;
        int n = 0;
#pragma unroll 8
        for (int i = threadIdx.x; i < npartials; i += WG) {
            a = fmaxf(a, pa[i]);
            n += pn[i];
            acc += part[i];
        }
        a = group_max(a, 64);
        n = wave_sum_i(n);
        if (lane == 0) { s_f[wave] = a; s_i[wave] = n; }
        __syncthreads();
        gamax = fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3]));
        gnnz = s_i[0] + s_i[1] + s_i[2] + s_i[3];
    } else {
        if (npart_stats > 0) {
            gamax = reduce_partial_amax(ws, npart_stats, s_f);
            const int* pn = reinterpret_cast<const int*>(ws) + WS_PNNZ;
            int n = 0;
#pragma unroll 8
            for (int i = threadIdx.x; i < npart_stats; i += WG) n += pn[i];
            n = wave_sum_i(n);
            if (lane == 0) s_i[wave] = n;
            __syncthreads();
            gnnz = s_i[0] + s_i[1] + s_i[2] + s_i[3];
        }
#pragma unroll 8
        for (int i = threadIdx.x; i < npartials; i += WG) acc += part[i];
    }
    acc = wave_sum(acc);
    __syncthreads();
    if (lane == 0) s_f[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        const float gerr = (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]);
        const float avg = gerr / (float)gnnz;        // 0 / 0 = NaN on an all-zero tensor: not above the threshold
        meta[0] = (avg > threshold) ? 3 : 1;
        gamax_o[0] = gamax;
        gnnz_o[0] = gnnz;
        gerr_o[0] = gerr;
    }
}

// Single pass for the strategies whose scale depends on the block alone (ss_mode 2 and 3, FQ:1079-1088), out of
// place: one workgroup per block of up to 16384 elements holds it in registers (as k_wgblock does), finds amax and
// the non-zero count, quantizes, accumulates the relative error and stores -- one read and one write of the tensor
// instead of two reads.  Workgroups walk the blocks grid-stride and publish one partial each of the tensor amax, the
// non-zero count and the error sum.  A block whose scale is outside the fast range is redone from memory with the
// exact arithmetic.
template <bool E8, int NV, bool FULL, int WGS = WG>
__global__ __launch_bounds__(WGS) void k_bs_fused(const uint4* in, uint4* out, uint32_t* ws, Shape sh, int ss_mode,
                                                 int cpr, int cpr_shift, int64_t nblocks, const int32_t* meta, int phase) {
    constexpr int NW = WGS / 64, LG = WGS == 256 ? 8 : WGS == 512 ? 9 : 10;       // waves; log2 of the workgroup size
    __shared__ float s_f[NW];
    __shared__ int s_i[NW];
    // sums and maxima over the waves' LDS slots (four waves: pairwise, the order the sums have always had)
    auto red_fsum = [&]() { if constexpr (NW == 4) return (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]); else return lds_sum<NW>(s_f); };
    auto red_fmax = [&]() { if constexpr (NW == 4) return fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3])); else return lds_fmax<NW>(s_f); };
    // phase 0: out of place (write and publish the partials); in place the input must survive until the decision:
    // phase 1 publishes the partials without writing, phase 2 writes if the decision was E4M3 (meta[0] == 1)
    if (phase == 2 && meta[0] != 1) return;
    const bool write = phase != 1;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t row_stride = (uint32_t)(sh.cols >> 3);
    const int nch = (int)sh.brows * cpr;
    const bool nt = streams_out(sh.rows * sh.cols);
    const bool bands = (cpr_shift & 256) != 0;      // XCD bands of block columns, as in k_wgblock (gx and the grid multiples of 8)
    cpr_shift &= 255;
    // chunk k * 256 + tid of a block is at off_k(k) + off_tid; cpr is a power of two, so off_k is uniform (no per-lane
    // index arithmetic is carried through the loop over blocks)
    const uint32_t off_tid = cpr_shift <= LG ? (uint32_t)(tid >> cpr_shift) * row_stride + (uint32_t)(tid & (cpr - 1)) : (uint32_t)tid;
    auto off_k = [&](int k) -> uint32_t {
        return cpr_shift <= LG ? (uint32_t)(k << (LG - cpr_shift)) * row_stride
                               : (uint32_t)(k >> (cpr_shift - LG)) * row_stride + (uint32_t)((k & ((1 << (cpr_shift - LG)) - 1)) << LG);
    };
    float gmax = 0.0f, err = 0.0f;
    int nnz_total = 0;
    for (int64_t t = blockIdx.x; t < nblocks; t += gridDim.x) {
        int64_t bid = t;
        if (bands) {
            const int64_t xcd = t & 7, j = t >> 3, per = sh.gx >> 3, byb = j / per;
            bid = byb * sh.gx + xcd * per + (j - byb * per);
        }
        const int64_t by = bid / sh.gx, bx = bid - by * sh.gx;
        const int64_t base = by * sh.brows * row_stride + ((bx * sh.bcols) >> 3);
        uint4 v[NV];
        bool ok[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            ok[k] = FULL || (k * WGS + tid < nch);
            v[k] = make_uint4(0, 0, 0, 0);
            if (ok[k]) v[k] = in[base + off_k(k) + off_tid];
        }
        // amax and the non-zero count.  Large blocks: on packed 16-bit magnitudes, the data staying packed in its
        // registers from pass to pass (NV = 8: 100 registers instead of 220).  Small blocks: float maxima, whose
        // unpacked magnitudes the quantize pass then uses again (measured faster for NV <= 2).
        constexpr bool PACKED = NV > 2;
        uint32_t amax_b, nnz2 = 0;
        if constexpr (PACKED) {
            uint32_t amax2 = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                acc_amax_pk(amax2, v[k].x); acc_amax_pk(amax2, v[k].y); acc_amax_pk(amax2, v[k].z); acc_amax_pk(amax2, v[k].w);
                acc_nnz_pk(nnz2, v[k].x); acc_nnz_pk(nnz2, v[k].y); acc_nnz_pk(nnz2, v[k].z); acc_nnz_pk(nnz2, v[k].w);
                opaque(v[k]);
            }
            amax_b = group_umax(amax_bits_of(amax2), 64);
        } else {
            uint32_t amax2 = 0;
            int nnzf = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                acc_amax_pk(amax2, v[k].x); acc_amax_pk(amax2, v[k].y); acc_amax_pk(amax2, v[k].z); acc_amax_pk(amax2, v[k].w);
                nnzf += nnz_word(v[k].x) + nnz_word(v[k].y) + nnz_word(v[k].z) + nnz_word(v[k].w);
            }
            nnz2 = (uint32_t)nnzf;
            amax_b = group_umax(amax_bits_of(amax2), 64);
        }
        __syncthreads();                          // the previous block's readers of s_f are done
        if (lane == 0) s_f[wave] = u2f(amax_b);
        __syncthreads();
        amax_b = f2u(lds_umaxf<NW>(s_f));
        float amax = u2f(amax_b);
        const bool has_nan = amax_b > 0x7F800000u;
        if (has_nan) {                            // the float maximum and the count of the reference skip a NaN (rare)
            amax = 0.0f;
            int nans = 0;
#pragma unroll 1
            for (int ch = tid; ch < nch; ch += WGS) {              // from memory again: no second use of the registers
                const int r = cpr_shift >= 0 ? (ch >> cpr_shift) : (ch / cpr);
                const uint4 x = in[base + (uint32_t)r * row_stride + (uint32_t)(ch - r * cpr)];
                acc_amax(amax, x.x); acc_amax(amax, x.y); acc_amax(amax, x.z); acc_amax(amax, x.w);
                if constexpr (PACKED) nans += nan_word(x.x) + nan_word(x.y) + nan_word(x.z) + nan_word(x.w);
            }
            nnz_total -= nans;                    // the packed count took them for non-zero values
            amax = group_max(amax, 64);
            __syncthreads();
            if (lane == 0) s_f[wave] = amax;
            __syncthreads();
            amax = red_fmax();
        }
        gmax = fmaxf(gmax, amax);
        nnz_total += (int)((nnz2 & 0xFFFFu) + (nnz2 >> 16));
        const Scale sc = make_scale(scaling_factor(0.0f, amax, ss_mode));
        if (!has_nan && (sc.fast || !(amax > 0.0f))) {          // an all-zero block gives +0 whatever its (clamped) scale is
            // For large blocks every vector is finished before the next begins (register barriers): otherwise the
            // compiler hoists work from all of them, and sinks the whole chain of error terms below the last store
            // with every magnitude and quotient alive, which doubles the registers.
            if (phase == 1) {                      // decision pass of the in-place variant: error terms only
#pragma unroll
                for (int k = 0; k < NV; ++k) {
                    if constexpr (PACKED) opaque(v[k]);
                    bs_vec_fast<E8, true, false>(v[k], sc, err);
                    if constexpr (PACKED) asm volatile("" : "+v"(err));
                }
            } else if (phase == 2) {               // write pass of the in-place variant: no error terms
#pragma unroll
                for (int k = 0; k < NV; ++k) {
                    if constexpr (PACKED) opaque(v[k]);
                    uint4 q = bs_vec_fast<E8, false, true>(v[k], sc, err);
                    if constexpr (PACKED) opaque(q);
                    if (ok[k]) store16_rt(out + base + off_k(k) + off_tid, q, nt);
                }
            } else {
#pragma unroll
                for (int k = 0; k < NV; ++k) {
                    if constexpr (PACKED) opaque(v[k]);
                    uint4 q = bs_vec_fast<E8, true, true>(v[k], sc, err);
                    if constexpr (PACKED) { opaque(q); asm volatile("" : "+v"(err)); }
                    if (ok[k]) store16_rt(out + base + off_k(k) + off_tid, q, nt);
                }
            }
        } else {
            const uint16_t* in16 = reinterpret_cast<const uint16_t*>(in);
            uint16_t* out16 = reinterpret_cast<uint16_t*>(out);
            const int64_t e0 = by * sh.brows * sh.cols + bx * sh.bcols;
#pragma unroll 1
            for (int64_t i = tid; i < sh.brows * sh.bcols; i += WGS) {
                const int64_t r = i / sh.bcols, c = i - r * sh.bcols;
                const float q = bs_element<E8, false>(bf16_one(in16[e0 + r * sh.cols + c]), sc, err);
                if (write) out16[e0 + r * sh.cols + c] = store_bf16<false>(q);
            }
        }
    }
    err = wave_sum(err);
    nnz_total = wave_sum_i(nnz_total);
    gmax = group_max(gmax, 64);
    __syncthreads();
    if (lane == 0) { s_f[wave] = err; s_i[wave] = nnz_total; }
    __syncthreads();
    const float e = red_fsum();
    int n = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) n += s_i[w];
    __syncthreads();
    if (lane == 0) s_f[wave] = gmax;
    __syncthreads();
    if (tid == 0 && phase != 2) {
        reinterpret_cast<float*>(ws)[WS_ERR + blockIdx.x] = e;
        reinterpret_cast<int*>(ws)[WS_PNNZ + blockIdx.x] = n;
        reinterpret_cast<float*>(ws)[WS_PAMAX + blockIdx.x] = red_fmax();
    }
}

// The same single pass for row blocks of 1 x 8G elements, G <= 64 lanes (MX 1 x 32 through the channel op is G = 4):
// the flat chunk array in tiles of 4 * 256 chunks, a block is G consecutive lanes (amax by DPP), as in k_rowgroup.
// Groups whose scale is outside the fast range are redone from memory by a second, non-unrolled loop.
constexpr int BS_ROWS_NV = 4;         // vectors per lane and tile (2 is not faster here: 55.9 against 54.5 us)
template <bool E8>
__global__ __launch_bounds__(WG) void k_bs_fused_rows(const uint4* in, uint4* out, uint32_t* ws, int64_t nchunks, int G, int ss_mode,
                                                      const int32_t* meta, int phase) {
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    if (phase == 2 && meta[0] != 1) return;          // phases as in k_bs_fused
    const bool write = phase != 1;
    constexpr int NV = BS_ROWS_NV;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool nt = streams_out(nchunks * 8);
    float gmax = 0.0f, err = 0.0f;
    int nnz = 0;
    const int64_t ntiles = (nchunks + NV * WG - 1) / (NV * WG);
    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int64_t base = tile * (NV * WG) + tid;
        uint4 v[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            v[k] = make_uint4(0, 0, 0, 0);
            if (base + k * WG < nchunks) v[k] = load16_rt(in + base + k * WG, streams_in(nchunks * 8));
        }
        uint32_t slow = 0;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int64_t c = base + k * WG;
            float amax = 0.0f;
            acc_amax_nnz(amax, nnz, v[k]);
            amax = group_max(amax, G);
            gmax = fmaxf(gmax, amax);
            const Scale sc = make_scale(scaling_factor(0.0f, amax, ss_mode));
            float e = 0.0f;
            uint4 q;
            if (phase == 1) q = bs_vec_fast<E8, true, false>(v[k], sc, e);          // in place: decision pass,
            else if (phase == 2) q = bs_vec_fast<E8, false, true>(v[k], sc, e);     // write pass
            else q = bs_vec_fast<E8, true, true>(v[k], sc, e);
            const bool has_nan = group_umax(vec_has_nan(v[k]) ? 1u : 0u, G) != 0u;          // exact arithmetic for such a block
            if (!has_nan && (sc.fast || !(amax > 0.0f))) {      // an all-zero block gives +0 whatever its (clamped) scale is
                err += e;
                if (c < nchunks && write) store16_rt(out + c, q, nt);
            } else if (c < nchunks) slow |= 1u << k;
        }
        if (slow) {
#pragma unroll 1
            for (int k = 0; k < NV; ++k) {
                if (!((slow >> k) & 1u)) continue;              // uniform over the lanes of a group
                const int64_t c = base + k * WG;
                const uint4 x = in[c];
                float amax = 0.0f;
                acc_amax(amax, x.x); acc_amax(amax, x.y); acc_amax(amax, x.z); acc_amax(amax, x.w);
                amax = group_max(amax, G);
                const Scale sc = make_scale(scaling_factor(0.0f, amax, ss_mode));
                uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    w[j] = store_pair<false>(bs_element<E8, false>(bf16_lo(w[j]), sc, err), bs_element<E8, false>(bf16_hi(w[j]), sc, err));
                if (write) out[c] = make_uint4(w[0], w[1], w[2], w[3]);
            }
        }
    }
    err = wave_sum(err);
    nnz = wave_sum_i(nnz);
    gmax = group_max(gmax, 64);
    if (lane == 0) { s_f[wave] = err; s_i[wave] = nnz; }
    __syncthreads();
    const float e = (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]);
    const int n = s_i[0] + s_i[1] + s_i[2] + s_i[3];
    __syncthreads();
    if (lane == 0) s_f[wave] = gmax;
    __syncthreads();
    if (tid == 0 && phase != 2) {
        reinterpret_cast<float*>(ws)[WS_ERR + blockIdx.x] = e;
        reinterpret_cast<int*>(ws)[WS_PNNZ + blockIdx.x] = n;
        reinterpret_cast<float*>(ws)[WS_PAMAX + blockIdx.x] = fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3]));
    }
}

// pass 4 for the out-of-place ops (FQ:1217-1235): copy the input over the quantized output when meta[0] == 3
__global__ __launch_bounds__(WG) void k_copy_if(const uint16_t* in, uint16_t* out, const int32_t* meta, int gate, int64_t n, int64_t nvec) {
    if (meta[0] != gate) return;
    const int64_t stride = (int64_t)gridDim.x * WG;
    const int64_t gtid = (int64_t)blockIdx.x * WG + threadIdx.x;
    const uint4* in4 = reinterpret_cast<const uint4*>(in);
    uint4* out4 = reinterpret_cast<uint4*>(out);
    for (int64_t c = gtid; c < nvec; c += stride) out4[c] = in4[c];
    for (int64_t i = nvec * 8 + gtid; i < n; i += stride) out[i] = in[i];
}

// FQ:1243-1327: keep MB mantissa bits by comparing the 23-bit mantissa with the reference's threshold tables
// (on bf16 inputs they are the midpoints with ties to even; on scaled inputs, whose low 16 bits are not zero,
// they are what they are).  Exponent 0 loses its mantissa, exponent 255 is left alone, a carry out of exponent
// 254 saturates.
template <int MB> __device__ __forceinline__ float quant_e8m(float v) {
    uint32_t b = f2u(v);
    uint32_t sign = b & 0x80000000u;
    uint32_t e = (b >> 23) & 0xFF, m = b & 0x7FFFFFu;
    if (e == 0) m = 0;
    else if (e != 255) {
        // The reference's thresholds, in units of 2^16: even j -> j*S + S/2, odd j -> j*S + S/2 - 1 with S = 2^(7-MB);
        // k = number of thresholds below the mantissa.  With h = mantissa >> 16 plus one if any lower bit is set and
        // u = h - S/2 this count is floor(u / S) plus one if that quotient is odd or the division leaves a remainder
        // (nearest even on bf16 inputs, the same tables on inputs with low bits).
        constexpr int S = 1 << (7 - MB);
        const int u = (int)(m >> 16) + ((m & 0xFFFFu) != 0 ? 1 : 0) - S / 2;
        const uint32_t q = (uint32_t)max(u, 0) >> (7 - MB);
        const uint32_t k = (u < 0) ? 0u : q + (((q & 1u) | (((uint32_t)u & (S - 1)) != 0 ? 1u : 0u)));
        if (k == (1u << MB)) {
            m = 0; e++;
            if (e == 255) { e = 254; m = ((1u << MB) - 1u) << (23 - MB); }
        } else m = k << (23 - MB);
    }
    return u2f(sign | (e << 23) | m);
}

// FQ:1335-1359
template <int MB> __device__ __forceinline__ float e8mx_scale(float gamax, int strategy) {
    if (strategy != 1) return 1.0f;
    uint32_t y = f2u(gamax);
    uint32_t e = (y >> 23) + 1;
    float fp_max = u2f((e << 23) | (((1u << MB) - 1u) << (23 - MB)));
    float sf = fp_max / gamax;
    if (sf >= 2.0f) sf /= 2.0f;
    return sf;
}

// One element of FQ:1399-1419.  UNIT: the scale is 1 (no tensor-amax strategy), so the multiply and the divide are
// exact no-ops.  Otherwise dq / sf is a reciprocal-multiply with one exact-residual correction (rs = 1 / sf correctly
// rounded), which gives the rounded quotient when the operands are well inside the exponent range and the
// significand of sf is not all ones; the IEEE division covers the rest.
template <int MB, bool UNIT> __device__ __forceinline__ float e8mx_element(float x, float sf, float rs, bool markstein_ok) {
    if constexpr (UNIT) {
        return (x != 0.0f) ? quant_e8m<MB>(x) : 0.0f;
    } else {
        float v = x * sf;
        float dq = 0.0f;
        if (v != 0.0f) dq = quant_e8m<MB>(v);
        const uint32_t e = (f2u(dq) >> 23) & 0xFF;
        if (markstein_ok && e > 30 && e < 225) {
            float t = dq * rs;
            return fmaf(fmaf(-t, sf, dq), rs, t);
        }
        return dq / sf;
    }
}

// FQ:1361-1428
template <int MB, bool EMU, bool UNIT>
__global__ __launch_bounds__(WG) void k_e8mx(const uint16_t* in, uint16_t* out, const uint32_t* ws, int npart, int strategy, int64_t n, int64_t nvec) {
    __shared__ float s_f[WAVES];
    const float gamax = (!UNIT && strategy == 1) ? reduce_partial_amax(ws, npart, s_f) : 0.0f;
    const float sf = UNIT ? 1.0f : e8mx_scale<MB>(gamax, strategy);
    const float rs = 1.0f / sf;
    const bool mk = (f2u(sf) & 0x7FFFFFu) != 0x7FFFFFu;
    const int64_t stride = (int64_t)gridDim.x * WG;
    const int64_t gtid = (int64_t)blockIdx.x * WG + threadIdx.x;
    const uint4* in4 = reinterpret_cast<const uint4*>(in);
    uint4* out4 = reinterpret_cast<uint4*>(out);
    constexpr int NV = 2;                       // a workgroup takes tiles of NV * 256 consecutive 16-byte chunks
    const int64_t ntiles = (nvec + NV * WG - 1) / (NV * WG);
    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int64_t c0 = tile * (NV * WG) + threadIdx.x;
        uint4 v[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) { v[k] = make_uint4(0, 0, 0, 0); if (c0 + k * WG < nvec) v[k] = load16_rt(in4 + c0 + k * WG, streams_in(n)); }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            uint32_t w[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = store_pair<EMU>(e8mx_element<MB, UNIT>(bf16_lo(w[j]), sf, rs, mk), e8mx_element<MB, UNIT>(bf16_hi(w[j]), sf, rs, mk));
            if (c0 + k * WG < nvec) store16_rt(out4 + c0 + k * WG, make_uint4(w[0], w[1], w[2], w[3]), streams_out(n));
        }
    }
    for (int64_t i = nvec * 8 + gtid; i < n; i += stride) out[i] = store_bf16<EMU>(e8mx_element<MB, UNIT>(bf16_one(in[i]), sf, rs, mk));
}

}  // namespace mor

extern "C" size_t mor_workspace_bytes(int op, int64_t rows, int64_t cols, int64_t brows, int64_t bcols) {
    if (rows <= 0 || cols <= 0 || brows <= 0 || bcols <= 0) return 0;
    switch (op) {
        case MOR_OP_BLOCK_SCALING:
        case MOR_OP_CHANNEL_SCALING:
            return (size_t)(WS_BLOCKS + cdiv(rows, brows) * cdiv(cols, bcols)) * 4;
        case MOR_OP_E8MX:
            return (size_t)WS_BLOCKS * 4;
        default:
            return 0;
    }
}

template <bool E8, bool EMU, bool COL>
static void launch_bs_quant(bool write, bool err, int grid, hipStream_t st, const uint16_t* in, uint16_t* out, uint32_t* ws,
                            const float* scales, const int32_t* meta, int gate, const Shape& sh, int vec,
                            DivU32 d0, DivU32 d1, DivU32 d2, DivU32 d3) {
    if (write && err) k_bs_quant<E8, EMU, COL, true, true><<<grid, WG, 0, st>>>(in, out, ws, scales, meta, gate, sh, vec, d0, d1, d2, d3);
    else if (write) k_bs_quant<E8, EMU, COL, true, false><<<grid, WG, 0, st>>>(in, out, ws, scales, meta, gate, sh, vec, d0, d1, d2, d3);
    else k_bs_quant<E8, EMU, COL, false, true><<<grid, WG, 0, st>>>(in, out, ws, scales, meta, gate, sh, vec, d0, d1, d2, d3);
}

static void dispatch_bs_quant(bool e8, bool emu, bool col, bool write, bool err, int grid, hipStream_t st, const uint16_t* in,
                              uint16_t* out, uint32_t* ws, const float* scales, const int32_t* meta, int gate, const Shape& sh,
                              int vec, DivU32 d0, DivU32 d1, DivU32 d2, DivU32 d3) {
#define BSQ(E8, EMU, COL) launch_bs_quant<E8, EMU, COL>(write, err, grid, st, in, out, ws, scales, meta, gate, sh, vec, d0, d1, d2, d3)
    if (e8) {
        if (emu) { if (col) BSQ(true, true, true); else BSQ(true, true, false); }
        else { if (col) BSQ(true, false, true); else BSQ(true, false, false); }
    } else {
        if (emu) { if (col) BSQ(false, true, true); else BSQ(false, true, false); }
        else { if (col) BSQ(false, false, true); else BSQ(false, false, false); }
    }
#undef BSQ
}

extern "C" int mor_block_scaling(const void* input, void* output, int32_t* meta,
                                 float* global_amax, int32_t* global_non_zero, float* global_error,
                                 int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                                 double e4m3_threshold, int64_t ss_mode, int channel,
                                 void* workspace, size_t workspace_bytes, uint32_t flags, void* stream) {
    if (int rc = validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!output || !meta || !global_amax || !global_non_zero || !global_error) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output pointer is NULL");
    if (rows % brows != 0 || cols % bcols != 0)      // FQ:2019-2020, 2437-2438
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "block dims %lld x %lld do not divide the tensor %lld x %lld", (long long)brows, (long long)bcols, (long long)rows, (long long)cols);
    if (ss_mode < 1 || ss_mode > 4) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "ss_mode must be 1..4 (got %lld)", (long long)ss_mode);
    if (channel && brows != 1 && bcols != 1)         // FQ:2501
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "channel scaling needs block_rows == 1 or block_cols == 1");
    if (rows * cols >= (1ll << 34)) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "tensor too large");
    const size_t need = mor_workspace_bytes(MOR_OP_BLOCK_SCALING, rows, cols, brows, bcols);
    if (!workspace || workspace_bytes < need) return mor_fail(MOR_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool emu = flags & MOR_FLAG_TORCH_EMULATION;
    Shape sh{rows, cols, brows, bcols, rows / brows, cols / bcols};
    const int64_t nb = sh.gy * sh.gx;
    uint32_t* ws = static_cast<uint32_t*>(workspace);
    float* blocks = reinterpret_cast<float*>(ws + WS_BLOCKS);
    const uint16_t* in16 = static_cast<const uint16_t*>(input);
    uint16_t* out16 = static_cast<uint16_t*>(output);
    const bool inplace = (input == output);
    const int vec = (aligned16(input) && aligned16(output) && cols % 8 == 0) ? 1 : 0;
    const bool col = (bcols == 1 && brows > 1);

    // block-local scales: one pass out of place; in place one pass for the decision and one gated pass that writes
    const int64_t blk_chunks = (bcols % 8 == 0) ? brows * (bcols / 8) : 0;
    // (a decision pass that computes no output words and a write pass that computes no error terms; 128 x 128 blocks
    // in place at 8192^2: 83 us against 99 through the general three-pass path; blocks that fill less than a workgroup
    // take the general path)
    if (!emu && vec && !col && (ss_mode == 2 || ss_mode == 3) && blk_chunks >= WG && blk_chunks <= 8 * 1024
        && brows * (cols / 8) < 0x7FFFFFFFll && (is_pow2(bcols / 8) || brows == 1)) {
        const int cpr = (int)(bcols / 8);
        const int nv = (int)cdiv(blk_chunks, WG);
        const int NVc = nv <= 1 ? 1 : nv <= 2 ? 2 : nv <= 4 ? 4 : 8;
        // up to 8 * 256 chunks: 256 threads; up to 32768 / 65536 elements: 8 vectors per lane of 512 / 1024 threads
        const int wgs = blk_chunks <= 8 * WG ? WG : blk_chunks <= 8 * 512 ? 512 : 1024;
        const bool full = blk_chunks == (int64_t)(wgs == WG ? NVc : 8) * wgs;
        const int grid = (int)std::min<int64_t>(nb, 4096);      // partials: one per workgroup (the finalize kernel reads them all)
        // tensors beyond the last-level cache: XCD bands of block columns (16384 x 14336, 128 x 128 blocks: 193 -> 185 us)
        const bool bands = rows * cols > ((int64_t)128 << 20) && sh.gx % 8 == 0 && grid % 8 == 0 && nb % 8 == 0;
        // a one-row block is contiguous whatever its width: chunk k * 256 + tid is at that offset (shift 20: row 0 always)
        const int shift = (brows == 1 ? 20 : ilog2(cpr)) | (bands ? 256 : 0);
        const uint4* i4 = static_cast<const uint4*>(input);
        uint4* o4 = static_cast<uint4*>(output);
#define MOR_BS_FUSED(E8, NV, PHASE) do { \
        if (full) k_bs_fused<E8, NV, true><<<grid, WG, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, cpr, shift, nb, meta, PHASE); \
        else k_bs_fused<E8, NV, false><<<grid, WG, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, cpr, shift, nb, meta, PHASE); } while (0)
#define MOR_BS_FUSED_W(E8, WGS_, PHASE) do { \
        if (full) k_bs_fused<E8, 8, true, WGS_><<<grid, WGS_, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, cpr, shift, nb, meta, PHASE); \
        else k_bs_fused<E8, 8, false, WGS_><<<grid, WGS_, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, cpr, shift, nb, meta, PHASE); } while (0)
#define MOR_BS_FUSED_ALL(PHASE) do { \
        if (wgs == 512) { if (ss_mode == 2) MOR_BS_FUSED_W(true, 512, PHASE); else MOR_BS_FUSED_W(false, 512, PHASE); } \
        else if (wgs == 1024) { if (ss_mode == 2) MOR_BS_FUSED_W(true, 1024, PHASE); else MOR_BS_FUSED_W(false, 1024, PHASE); } \
        else if (ss_mode == 2) { switch (NVc) { case 1: MOR_BS_FUSED(true, 1, PHASE); break; case 2: MOR_BS_FUSED(true, 2, PHASE); break; case 4: MOR_BS_FUSED(true, 4, PHASE); break; default: MOR_BS_FUSED(true, 8, PHASE); break; } } \
        else { switch (NVc) { case 1: MOR_BS_FUSED(false, 1, PHASE); break; case 2: MOR_BS_FUSED(false, 2, PHASE); break; case 4: MOR_BS_FUSED(false, 4, PHASE); break; default: MOR_BS_FUSED(false, 8, PHASE); break; } } } while (0)
        MOR_BS_FUSED_ALL(inplace ? 1 : 0);
        k_bs_finalize<<<1, WG, 0, st>>>(ws, grid, grid, (float)e4m3_threshold, meta, global_amax, global_non_zero, global_error);
        if (inplace) MOR_BS_FUSED_ALL(2);
        else {
            const int64_t n_all = rows * cols;
            k_copy_if<<<grid_for(n_all / 8, 4), WG, 0, st>>>(in16, out16, meta, 3, n_all, n_all / 8);
        }
#undef MOR_BS_FUSED_ALL
#undef MOR_BS_FUSED_W
#undef MOR_BS_FUSED
        return mor_check_launch("mor_block_scaling (single pass)");
    }

    if (!emu && vec && !col && (ss_mode == 2 || ss_mode == 3) && brows == 1 && bcols % 8 == 0 && is_pow2(bcols / 8)
        && bcols / 8 <= 64) {
        const int64_t nchunks = rows * cols / 8;
        const int grid = (int)std::min<int64_t>(cdiv(nchunks, BS_ROWS_NV * WG), MAX_PARTIALS);
        const uint4* i4 = static_cast<const uint4*>(input);
        uint4* o4 = static_cast<uint4*>(output);
        const int G = (int)(bcols / 8);
        for (int phase = inplace ? 1 : 0; phase <= (inplace ? 2 : 0); ++phase) {
            if (ss_mode == 2) k_bs_fused_rows<true><<<grid, WG, 0, st>>>(i4, o4, ws, nchunks, G, (int)ss_mode, meta, phase);
            else k_bs_fused_rows<false><<<grid, WG, 0, st>>>(i4, o4, ws, nchunks, G, (int)ss_mode, meta, phase);
            if (phase != 2) k_bs_finalize<<<1, WG, 0, st>>>(ws, grid, grid, (float)e4m3_threshold, meta, global_amax, global_non_zero, global_error);
        }
        if (!inplace) k_copy_if<<<grid_for(nchunks, 4), WG, 0, st>>>(in16, out16, meta, 3, rows * cols, nchunks);
        return mor_check_launch("mor_block_scaling (single pass, row blocks)");
    }

    // pass 1: per-block amax, per-workgroup partials of the tensor amax and the non-zero count
    const int64_t G = bcols / 8;
    int npart;
    if (col) {
        k_zero_f32<<<grid_for(nb), WG, 0, st>>>(blocks, nb);
        const int rows_per_wg = (int)std::min<int64_t>(brows, 256);
        const unsigned gx = (unsigned)cdiv(cols, 256);
        const int64_t segs = sh.gy * cdiv(brows, rows_per_wg);
        if ((int64_t)gx > MAX_PARTIALS) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "too many columns (%lld)", (long long)cols);
        const unsigned gy = (unsigned)std::min<int64_t>(segs, std::max<int64_t>(MAX_PARTIALS / gx, 1));
        npart = (int)(gx * gy);
        k_bs_amax_col<<<dim3(gx, gy), WG, 0, st>>>(in16, ws, blocks, sh, rows_per_wg, vec);
    } else if (vec && brows == 1 && bcols % 8 == 0 && is_pow2(G) && G <= 64) {
        const int64_t nchunks = rows * cols / 8;
        npart = (int)std::min<int64_t>(cdiv(nchunks, 8 * WG), MAX_PARTIALS);
        k_bs_amax_flat<<<npart, WG, 0, st>>>(static_cast<const uint4*>(input), ws, blocks, nchunks, (int)G, ilog2(G));
    } else if (vec && bcols % 8 == 0 && brows * (bcols / 8) < WG && brows * (cols / 8) < 0x7FFFFFFFll) {
        const int nchb = (int)(brows * (bcols / 8));
        int logL = 0;
        while ((4 << logL) < nchb && logL < 6) ++logL;               // about four vectors per lane
        const int groups = WG >> logL;
        npart = (int)std::min<int64_t>(cdiv(nb, groups), MAX_PARTIALS);
        k_bs_amax_sub<<<npart, WG, 0, st>>>(static_cast<const uint4*>(input), ws, blocks, sh, 1 << logL, logL, make_div((uint32_t)sh.gx),
                                            make_div((uint32_t)(bcols / 8)));
    } else {
        const int v1 = (vec && bcols % 8 == 0 && brows * (cols / 8) < 0x7FFFFFFFll) ? 1 : 0;
        npart = (int)std::min<int64_t>(nb, MAX_PARTIALS);
        k_bs_amax_block<<<npart, WG, 0, st>>>(in16, ws, blocks, sh, v1, make_div((uint32_t)sh.gx),
                                              make_div((uint32_t)std::max<int64_t>(bcols / 8, 1)));
    }
    // pass 1.5: tensor amax and non-zero count into the header, block scales
    k_bs_scales<<<(int)std::min<int64_t>(cdiv(nb, WG), 256), WG, 0, st>>>(ws, blocks, nb, (int)ss_mode, npart);
    // pass 2: quantize (out of place: write now; in place: error only), error partials
    // pass 3: decision and scalars
    // pass 4: bf16 fallback (out of place: copy if meta == 3) or the quantized write (in place: only if meta == 1)
    const bool e8 = (ss_mode == 2);
    const int64_t n = rows * cols;
    if (col && vec && !emu && !e8) {
        const int rows_per_wg = (int)std::min<int64_t>(brows, 16);
        const unsigned gx = (unsigned)cdiv(cdiv(cols, 8), WG);
        const int64_t segs = sh.gy * cdiv(brows, rows_per_wg);
        const dim3 grid(gx, (unsigned)std::min<int64_t>(segs, std::max<int64_t>(MAX_PARTIALS / gx, 1)));
        if (inplace) k_bs_quant_col<false, true><<<grid, WG, 0, st>>>(in16, out16, ws, blocks, meta, 0, sh, rows_per_wg);
        else k_bs_quant_col<true, true><<<grid, WG, 0, st>>>(in16, out16, ws, blocks, meta, 0, sh, rows_per_wg);
        k_bs_finalize<<<1, WG, 0, st>>>(ws, (int)(grid.x * grid.y), 0, (float)e4m3_threshold, meta, global_amax, global_non_zero, global_error);
        if (inplace) k_bs_quant_col<true, false><<<grid, WG, 0, st>>>(in16, out16, ws, blocks, meta, 1, sh, rows_per_wg);
    } else {
        const bool vec2 = vec && (col || bcols % 8 == 0) && n / 8 < 0xFFFFFFFFll;
        const int64_t work = vec2 ? n / 8 : n;
        const int grid2 = (int)std::min<int64_t>(std::max<int64_t>(cdiv(work, WG), 1), MAX_PARTIALS);
        DivU32 d0 = make_div((uint32_t)std::max<int64_t>(cols / 8, 1)), d1 = make_div((uint32_t)brows),
               d2 = make_div((uint32_t)std::max<int64_t>(bcols / 8, 1)), d3 = make_div((uint32_t)bcols);
        dispatch_bs_quant(e8, emu, col, !inplace, true, grid2, st, in16, out16, ws, blocks, meta, 0, sh, vec2 ? 1 : 0, d0, d1, d2, d3);
        k_bs_finalize<<<1, WG, 0, st>>>(ws, grid2, 0, (float)e4m3_threshold, meta, global_amax, global_non_zero, global_error);
        if (inplace) dispatch_bs_quant(e8, emu, col, true, false, grid2, st, in16, out16, ws, blocks, meta, 1, sh, vec2 ? 1 : 0, d0, d1, d2, d3);
    }
    if (!inplace) {
        const int64_t nvec = vec ? n / 8 : 0;
        k_copy_if<<<grid_for(nvec > 0 ? nvec : n, 4), WG, 0, st>>>(in16, out16, meta, 3, n, nvec);
    }
    return mor_check_launch("mor_block_scaling");
}

extern "C" int mor_e8mx(const void* input, void* output, int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                        int64_t quantize_type, int64_t scaling_strategy, void* workspace, size_t workspace_bytes,
                        uint32_t flags, void* stream) {
    if (int rc = validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!output) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output is NULL");
    if (quantize_type < 1 || quantize_type > 3) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "quantize_type must be 1..3 (got %lld)", (long long)quantize_type);
    const size_t need = mor_workspace_bytes(MOR_OP_E8MX, rows, cols, brows, bcols);
    if (!workspace || workspace_bytes < need) return mor_fail(MOR_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool emu = flags & MOR_FLAG_TORCH_EMULATION;
    uint32_t* ws = static_cast<uint32_t*>(workspace);
    const uint16_t* in16 = static_cast<const uint16_t*>(input);
    uint16_t* out16 = static_cast<uint16_t*>(output);
    const int64_t n = rows * cols;
    const int64_t nvec = (aligned16(input) && aligned16(output)) ? n / 8 : 0;
    const int grid = nvec > 0 ? (int)std::min<int64_t>(cdiv(nvec, 2 * WG), 1 << 20) : grid_for(n, 16);
    const int strategy = (int)scaling_strategy;
    int npart = 0;
    if (strategy == 1) {
        if (nvec > 0 && nvec * 8 == n) {
            npart = (int)std::min<int64_t>(cdiv(nvec, 8 * WG), 1024);
            k_bs_amax_flat<<<npart, WG, 0, st>>>(static_cast<const uint4*>(input), ws, nullptr, nvec, 1, 0);
        } else {
            npart = (int)std::min<int64_t>(cdiv(n, WG), 1024);
            k_amax_scalar<<<npart, WG, 0, st>>>(in16, ws, n);
        }
    }
#define E8MX(MB) do { \
        if (strategy != 1) { if (emu) k_e8mx<MB, true, true><<<grid, WG, 0, st>>>(in16, out16, ws, npart, strategy, n, nvec); \
                             else k_e8mx<MB, false, true><<<grid, WG, 0, st>>>(in16, out16, ws, npart, strategy, n, nvec); } \
        else { if (emu) k_e8mx<MB, true, false><<<grid, WG, 0, st>>>(in16, out16, ws, npart, strategy, n, nvec); \
               else k_e8mx<MB, false, false><<<grid, WG, 0, st>>>(in16, out16, ws, npart, strategy, n, nvec); } } while (0)
    if (quantize_type == 1) E8MX(1); else if (quantize_type == 2) E8MX(2); else E8MX(3);
#undef E8MX
    return mor_check_launch("mor_e8mx");
}
