// Device-side pieces shared by the fake-quantization kernels: the MoR decision, the error terms, the generic
// one-workgroup-per-block path, and the declarations of the launchers each kernel file exports to the driver.
// "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.
#pragma once

#include <algorithm>

#include "mor_common.h"

namespace mor {



// MorQuantType, FQ:600-608 (the values written to meta)
enum : int { Q_UNKNOWN = 0, Q_E4M3 = 1, Q_E5M2 = 2, Q_BF16 = 3, Q_E2M3 = 4, Q_E4M3_SMALL = 11, Q_E5M2_SMALL = 12 };


struct QuantArgs {
    int qmode;        // 1 MoR, 2 fixed format (fmt), 4 current scaling (fmt, scale = clamp)
    int fmt;          // forced format for qmode 2 / 4
    int meta_val;     // value written to meta for qmode 2 / 4; < 0: leave meta alone
    int dyn_range;    // MoR decision by dynamic range instead of quantization error
    float clamp;      // clamp_threshold
    int ref_sums;     // MoR: every error sum with the reference's divisions in the reference's order (else only the close ones)
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

// The two MoR error sums of one block as the reference computes them (FQ:487-584): its arithmetic (err_terms_exact)
// and the order of its additions.  The reference runs tbx x tby threads on a block: 16 x 32 on blocks of more than
// 1024 elements, (block_cols / 2) x block_rows otherwise (FQ:1770-1789).  Thread (tx, ty) walks the rows ty, ty + tby,
// ... and in each the packed words tx, tx + tbx, ..., adding (term of the odd column + term of the even column) of
// every word to its own sum; 32 consecutive threads (in row-major order of (ty, tx)) then add their sums in a
// shuffle-down tree (lane i += lane i + 16, 8, 4, 2, 1) and the warps' sums meet in one more such tree over 32 slots,
// the unused ones zero.  Here the workgroup's threads take the reference's threads ("virtual threads") in turn, the
// sums go through LDS and the trees are made of the same additions.  Shapes the reference cannot launch (odd widths,
// thread counts that are not whole warps) have no such order: their terms are added in double and rounded once.
// Called by all WGS threads of the workgroup with the same arguments; ld(r, c) returns the bf16 bits of element (r, c)
// of the block's valid part bh x bw; every thread gets the sums.
// This is the rare path (error sums too close to call) and the exact path: its cost does not matter.
// Its LDS: one copy per kernel, however many call sites the kernel has.
constexpr int REF_SUMS_MAXVT = 1024;                  // the reference's largest thread block
struct RefSumsLds { float p4[REF_SUMS_MAXVT], p5[REF_SUMS_MAXVT], w4[32], w5[32]; double d[2][16]; };
constexpr int REF_SUMS_LDS_BYTES = (int)sizeof(RefSumsLds);
__device__ __forceinline__ RefSumsLds& ref_sums_lds() {
    __shared__ RefSumsLds s;
    return s;
}
template <bool EMU, int WGS, class Ld>
__device__ __forceinline__ void err_sums_reference_order(Ld&& ld, int bh, int bw, int64_t brows, int64_t bcols, bool even_cols,
                                                         bool e8, const Scale& s4, const Scale& s5, float& e4, float& e5) {
    static_assert(WGS / 64 <= 16, "at most 16 waves");
    constexpr int MAXVT = REF_SUMS_MAXVT;
    RefSumsLds& L = ref_sums_lds();
    float* s_p4 = L.p4; float* s_p5 = L.p5; float* s_w4 = L.w4; float* s_w5 = L.w5;
    double (*s_d)[16] = L.d;
    const int tid = threadIdx.x;
    int tbx = 16, tby = 32;
    bool geom = even_cols && (bcols % 2 == 0);
    if (brows * bcols > 1024) {
        if (bcols < 32 || brows < 32) geom = false;
    } else {
        tbx = (int)(bcols / 2); tby = (int)brows;
    }
    const int nvt = tbx * tby;
    if (nvt <= 0 || nvt % 32 != 0 || nvt > MAXVT) geom = false;
    __syncthreads();                                   // earlier readers of the LDS arrays are done
    if (!geom) {
        double d4 = 0.0, d5 = 0.0;
#pragma unroll 1
        for (int i = tid; i < bh * bw; i += WGS) {
            const int r = i / bw, c = i - r * bw;
            float t4 = 0.0f, t5 = 0.0f;
            err_terms_exact<EMU>(bf16_one(ld(r, c)), e8, s4, s5, t4, t5);
            d4 += (double)t4; d5 += (double)t5;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) { d4 += __shfl_xor(d4, off); d5 += __shfl_xor(d5, off); }
        if ((tid & 63) == 0) { s_d[0][tid >> 6] = d4; s_d[1][tid >> 6] = d5; }
        __syncthreads();
        d4 = 0.0; d5 = 0.0;
#pragma unroll
        for (int w = 0; w < WGS / 64; ++w) { d4 += s_d[0][w]; d5 += s_d[1][w]; }
        e4 = (float)d4; e5 = (float)d5;
        return;
    }
    const int pw = bw >> 1;                            // packed words per row of the valid part
#pragma unroll 1
    for (int vt = tid; vt < nvt; vt += WGS) {
        const int ty = vt / tbx, tx = vt - ty * tbx;
        float a4 = 0.0f, a5 = 0.0f;
#pragma unroll 1
        for (int r = ty; r < bh; r += tby)
#pragma unroll 1
            for (int pc = tx; pc < pw; pc += tbx) {
                float h4 = 0.0f, h5 = 0.0f, l4 = 0.0f, l5 = 0.0f;
                err_terms_exact<EMU>(bf16_one(ld(r, 2 * pc + 1)), e8, s4, s5, h4, h5);
                err_terms_exact<EMU>(bf16_one(ld(r, 2 * pc)), e8, s4, s5, l4, l5);
                a4 += (h4 + l4);
                a5 += (h5 + l5);
            }
        s_p4[vt] = a4; s_p5[vt] = a5;
    }
    __syncthreads();
    // the shuffle-down tree of every warp: in a step only lanes below `off` matter, and they read lanes they do not write
#pragma unroll 1
    for (int off = 16; off > 0; off >>= 1) {
#pragma unroll 1
        for (int vt = tid; vt < nvt; vt += WGS)
            if ((vt & 31) < off) { s_p4[vt] += s_p4[vt + off]; s_p5[vt] += s_p5[vt + off]; }
        __syncthreads();
    }
    // the warps' sums in the first warp's tree
    if (tid < 32) {
        const int nw = nvt >> 5;
        s_w4[tid] = tid < nw ? s_p4[32 * tid] : 0.0f;
        s_w5[tid] = tid < nw ? s_p5[32 * tid] : 0.0f;
    }
    __syncthreads();
#pragma unroll 1
    for (int off = 16; off > 0; off >>= 1) {
        if (tid < off) { s_w4[tid] += s_w4[tid + off]; s_w5[tid] += s_w5[tid + off]; }
        __syncthreads();
    }
    e4 = s_w4[0]; e5 = s_w5[0];
}

// ------------------------------------------------------------------------------------------------
// quantize one packed word with an fp32 scale: |x| * s, hardware convert, divide by s, round-half-up store, sign
// (`codes`: the register the converts write half of, carried from word to word so that no fresh zero is needed)
template <int F> __device__ __forceinline__ uint32_t fq_pair_div(uint32_t w, float s, float r, uint32_t& codes) {
    codes = hw_pack2_low_keep<F>(fabsf(bf16_lo(w)) * s, fabsf(bf16_hi(w)) * s, codes);
    const f32x2 c = hw_unpack2_low<F>(codes);
    return store_pair<false>(div_by_scale(c.x, s, r), div_by_scale(c.y, s, r)) | (w & 0x80008000u);
}
template <int F> __device__ __forceinline__ uint4 fq_vec_div(uint4 v, float s, float r, uint32_t& codes) {
    uint4 o;
    o.x = fq_pair_div<F>(v.x, s, r, codes);
    o.y = fq_pair_div<F>(v.y, s, r, codes);
    o.z = fq_pair_div<F>(v.z, s, r, codes);
    o.w = fq_pair_div<F>(v.w, s, r, codes);
    return o;
}

// the same through a table of the block's 128 dequantized magnitudes (bf16 bits of code / s, in LDS): |x| * s, hardware
// convert, two lookups, sign
template <int F> __device__ __forceinline__ uint32_t fq_pair_tab(uint32_t w, float s, const uint16_t* tab, uint32_t& codes) {
    codes = hw_pack2_low_keep<F>(fabsf(bf16_lo(w)) * s, fabsf(bf16_hi(w)) * s, codes);
    const uint32_t qa = tab[codes & 0xFFu], qb = tab[(codes >> 8) & 0xFFu];
    return qa | (qb << 16) | (w & 0x80008000u);
}
// the same from codes the error pass left (err_pair_fast: E4M3 codes of the pair in the low half, E5M2 codes in the high half)
template <int F> __device__ __forceinline__ uint32_t fq_pair_tab_codes(uint32_t w, uint32_t codes, const uint16_t* tab) {
    const uint32_t c = F == FMT_E4M3 ? codes : codes >> 16;
    const uint32_t qa = tab[c & 0xFFu], qb = tab[(c >> 8) & 0xFFu];
    return qa | (qb << 16) | (w & 0x80008000u);
}
template <int F> __device__ __forceinline__ uint4 fq_vec_tab_codes(uint4 v, const uint32_t (&codes)[4], const uint16_t* tab) {
    uint4 o;
    o.x = fq_pair_tab_codes<F>(v.x, codes[0], tab);
    o.y = fq_pair_tab_codes<F>(v.y, codes[1], tab);
    o.z = fq_pair_tab_codes<F>(v.z, codes[2], tab);
    o.w = fq_pair_tab_codes<F>(v.w, codes[3], tab);
    return o;
}
template <int F> __device__ __forceinline__ uint4 fq_vec_tab(uint4 v, float s, const uint16_t* tab, uint32_t& codes) {
    uint4 o;
    o.x = fq_pair_tab<F>(v.x, s, tab, codes);
    o.y = fq_pair_tab<F>(v.y, s, tab, codes);
    o.z = fq_pair_tab<F>(v.z, s, tab, codes);
    o.w = fq_pair_tab<F>(v.w, s, tab, codes);
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
// close MoR decisions as k_wgblock.  The exact MoR error sums are the reference's, addition by addition
// (err_sums_reference_order).
// MORP: whether the caller can be in MoR mode at all (a kernel that never is leaves the decision's code and LDS out).
template <bool EMU, bool FAST = false, int WGS = WG, bool MORP = true>
__device__ __forceinline__ void generic_block(const uint16_t* in, uint16_t* out, int32_t* meta, float* stats,
                                              const Shape& sh, const QuantArgs& qa, bool e8, int64_t bid,
                                              float (*s_f)[WGS / 64], uint32_t* s_u, bool allow_fast = false,
                                              uint16_t* packed_out = nullptr) {
    // packed_out: the block's result goes there with the rows bh x bw packed (row pitch sh.bcols) instead of into `out`
    constexpr int NW = WGS / 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t by32, bx32;
    block_of(sh, (uint32_t)bid, by32, bx32);                  // (fewer than 2^31 blocks)
    const int64_t by = by32, bx = bx32;
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
    if constexpr (MORP) if (qa.qmode == 1) {
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
                    // too close to call (or asked for): the reference's divisions in the reference's order
                    exact = qa.ref_sums || !(fabsf(e4 - e5) > 1e-5f * fmaxf(e4, e5));
                }
            }
            if (exact)
                err_sums_reference_order<EMU, WGS>([&](int r, int c) { return bin[(int64_t)r * sh.cols + c]; },
                                                   (int)bh, (int)bw, sh.brows, sh.bcols, sh.cols % 2 == 0, e8, s4, s5, e4, e5);
            qt = mor_decide_error(amax, qa.clamp, e4, e5);
        }
        meta_val = qt;
        fmt = mor_fmt_of(qt);
    }
    if (tid == 0) {
        if (meta && meta_val >= 0) meta[bid] = meta_val;
        if (stats) { float* s = stats + 4 * (int64_t)bid; s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5; }
    }
    if (!out && !packed_out) return;
    const bool copy = (fmt < 0) || !(amax > 0.0f);
    if (copy && out == in && !packed_out) return;
    const Scale sc = make_scale(copy ? 1.0f : fmax_of(fmt) / amax);
    uint16_t* bout = out + r0 * sh.cols + c0;
    // where the element at offset `at` of the block (row pitch sh.cols) goes
    auto dst = [&](int64_t at) -> uint16_t* {
        if (!packed_out) return bout + at;
        const int64_t r = at / sh.cols;                 // (rare path: a division per element does not matter)
        return packed_out + r * sh.bcols + (at - r * sh.cols);
    };
    bool fast = false;
    if constexpr (FAST && !EMU) fast = allow_fast && !copy && sc.fast && sc.e8 >= -90 && sc.e8 <= 90;
    if (fast) {
        for_block_elements<WGS>(bh, bw, sh.cols, tid, [&](int64_t at) { *dst(at) = fq_one_fast(bin[at], fmt, e8, sc); });
    } else {
        for_block_elements<WGS>(bh, bw, sh.cols, tid, [&](int64_t at) {
            uint16_t h = bin[at];
            if (!copy) h = fq_one_exact<EMU>(h, fmt, e8, sc);
            *dst(at) = h;
        });
    }
}

}  // namespace mor

// mode / clamp_threshold of the fake_quantize ops -> what the kernels take (FQ:1773-1779, 1792-1834).  Returns false
// for the mode digits that copy the tensor (meta 3).
static inline bool mor_decode_mode(int64_t mode, double clamp_threshold, mor::QuantArgs& qa) {
    qa = mor::QuantArgs{};
    qa.clamp = (float)clamp_threshold;
    qa.dyn_range = (mode / 100 > 0) ? 1 : 0;
    switch ((int)(mode % 10)) {
        case 1: qa.qmode = 1; qa.fmt = -1; qa.meta_val = -1; return true;
        case 2: qa.qmode = 2; qa.fmt = mor::FMT_E4M3; qa.meta_val = 1; return true;
        case 3: qa.qmode = 2; qa.fmt = mor::FMT_E5M2; qa.meta_val = 2; return true;
        case 4: qa.qmode = 4; qa.fmt = mor::FMT_E4M3; qa.meta_val = 1; return true;
        case 5: qa.qmode = 4; qa.fmt = mor::FMT_E5M2; qa.meta_val = 2; return true;
        default: return false;
    }
}


// A launch holds fewer than 2^32 threads per dimension (a larger grid wraps without an error): kernels that take one
// workgroup per block are launched slice by slice, f(first block, blocks of the slice).
constexpr int64_t LAUNCH_SLICE = (int64_t)1 << 22;
template <class Fn> static void for_slices(int64_t nblocks, Fn&& f) {
    for (int64_t first = 0; first < nblocks; first += LAUNCH_SLICE) f(first, (int)std::min(LAUNCH_SLICE, nblocks - first));
}

// Launchers of the kernels that live in files of their own (mor_wgblock.hip, mor_subblock.hip); `mor` selects the
// per-block format decision, `e8` the power-of-two scale.
__attribute__((visibility("hidden"))) void mor_launch_wgblock(bool mor, bool e8, bool gather, const void* in, void* out, int32_t* meta, float* stats,
                                                              const mor::Shape& sh, const mor::QuantArgs& qa, hipStream_t st);
__attribute__((visibility("hidden"))) void mor_launch_subblock(bool mor, bool e8, const void* in, void* out, int32_t* meta, float* stats,
                                                               const mor::Shape& sh, const mor::QuantArgs& qa, hipStream_t st);
__attribute__((visibility("hidden"))) void mor_launch_bigblock(bool mor, bool e8, const void* in, void* out, int32_t* meta, float* stats,
                                                               const mor::Shape& sh, const mor::QuantArgs& qa, hipStream_t st);
