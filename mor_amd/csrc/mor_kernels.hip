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

#include "mor_quant.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

namespace mor {

template <bool EMU>
__global__ __launch_bounds__(WG) void k_generic(const uint16_t* in, uint16_t* out, int32_t* __restrict__ meta,
                                                float* __restrict__ stats, Shape sh, QuantArgs qa, int e8, int64_t first) {
    __shared__ float s_f[2][WAVES];
    __shared__ uint32_t s_u[WAVES];
    generic_block<EMU, true>(in, out, meta, stats, sh, qa, (e8 & 1) != 0, first + blockIdx.x, s_f, s_u, (e8 & 2) != 0);
}

// Small blocks (up to 512 elements) that no vector kernel serves, e.g. 1 x 32 blocks on a tensor with an odd column
// count: a workgroup is one wave and takes `per_wave` consecutive blocks, so that 32 blocks are in flight per CU
// instead of 8 and a workgroup's start-up is shared (4097 x 4095 in 1 x 32 blocks: 0.5 ms with a 256-thread
// workgroup per block).
template <bool EMU>
__global__ __launch_bounds__(64) void k_generic_wave(const uint16_t* in, uint16_t* out, int32_t* __restrict__ meta,
                                                     float* __restrict__ stats, Shape sh, QuantArgs qa, int e8, int64_t first,
                                                     int64_t nblocks, int per_wave) {
    __shared__ float s_f[2][1];
    __shared__ uint32_t s_u[1];
    const int64_t b0 = first + (int64_t)blockIdx.x * per_wave;
    for (int i = 0; i < per_wave && b0 + i < nblocks; ++i)
        generic_block<EMU, true, 64>(in, out, meta, stats, sh, qa, (e8 & 1) != 0, b0 + i, s_f, s_u, (e8 & 2) != 0);
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
    for (int k = 0; k < EW_NV; ++k) { int64_t c = base + k * WG; v[k] = make_uint4(0, 0, 0, 0); if (c < nvec) v[k] = load16_rt(in4 + c, streams_last_read(n)); }
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
// (meta: the blocks' entries, all 3, written by the same launch; may be NULL)
template <int EW_NV>
__global__ __launch_bounds__(WG) void k_copy(const uint16_t* in, uint16_t* out, int64_t n, int64_t nvec, int32_t* meta, int64_t nblocks) {
    const int64_t stride = (int64_t)gridDim.x * WG;
    const int64_t gtid = (int64_t)blockIdx.x * WG + threadIdx.x;
    if (meta) for (int64_t i = gtid; i < nblocks; i += stride) meta[i] = 3;
    const uint4* in4 = reinterpret_cast<const uint4*>(in);
    uint4* out4 = reinterpret_cast<uint4*>(out);
    const int64_t base = (int64_t)blockIdx.x * (EW_NV * WG) + threadIdx.x;
    uint4 v[EW_NV];
#pragma unroll
    for (int k = 0; k < EW_NV; ++k) { int64_t c = base + k * WG; v[k] = make_uint4(0, 0, 0, 0); if (c < nvec) v[k] = load16_rt(in4 + c, streams_last_read(n)); }
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
    const bool lnt = streams_last_read(nchunks * 8);
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
// Debug view: per block amax, fp32 scale, biased exponent of the scale.
__global__ __launch_bounds__(WG) void k_block_stats(const uint16_t* __restrict__ in, Shape sh, float fmax,
                                                    float* __restrict__ amax_o, float* __restrict__ scale_o,
                                                    int32_t* __restrict__ e8m0_o, int64_t first) {
    __shared__ float s_f[WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t bid = first + blockIdx.x;
    uint32_t by32, bx32;
    block_of(sh, (uint32_t)bid, by32, bx32);                  // (fewer than 2^31 blocks)
    const int64_t by = by32, bx = bx32;
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



extern "C" const char* mor_last_error(void) { return g_err; }

int mor_validate_shape(const void* input, int64_t rows, int64_t cols, int64_t brows, int64_t bcols) {
    if (!input) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "input is NULL");
    if (rows <= 0 || cols <= 0) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "rows and cols must be positive (got %lld x %lld)", (long long)rows, (long long)cols);
    if (brows <= 0 || bcols <= 0) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "block dims must be positive (got %lld x %lld)", (long long)brows, (long long)bcols);
    // 2^35 elements (64 GiB of bf16): the flat kernels' grids, one workgroup per 512 vectors, stay below 2^24 workgroups
    // (checked first: with rows * cols bounded, the block count below cannot overflow)
    if (rows > MOR_MAX_ELEMENTS / cols) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "tensor too large (more than 2^35 elements)");
    if (cdiv(rows, brows) * cdiv(cols, bcols) > 0x7FFFFFFFll) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "too many blocks");
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
    // Few vectors per lane: many small workgroups interleave their loads and stores more finely than few large ones.
    // Tensors of 64 MiB and more (they come from HBM) take one vector per lane: a plain copy of 8192^2 from HBM runs at
    // 0.79 of the peak rate with one, 0.76 with two, 0.73 with eight vectors per lane; at 16384 x 14336: 0.82 / 0.76 /
    // 0.73.  Smaller tensors take two (fewer workgroups to launch).
    // (the software casts of E2M3 / E3M2 cost more instructions per element and are better off with two: 49.6 -> 45.4 us)
    const bool big = nchunks * 16 >= ((int64_t)64 << 20) && Fmt<F>::hw;
    const bool nt_out = nchunks * 16 >= ((int64_t)4 << 20);
#define MOR_ROWGROUP(NV) do { \
        if (nt_out && nchunks % ((int64_t)NV * WG) == 0 && (G == 4 || G == 16) && nchunks / ((int64_t)NV * WG) <= 0x7FFFFFFFll) { \
            const int grid = (int)(nchunks / ((int64_t)NV * WG)); \
            if (G == 4) k_rowgroup<F, E8, NV, 4, true, true><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val); \
            else k_rowgroup<F, E8, NV, 16, true, true><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val); \
        } else { \
            const int grid = (int)cdiv(nchunks, (int64_t)NV * WG); \
            if (nt_out) k_rowgroup<F, E8, NV, 0, false, true><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val); \
            else k_rowgroup<F, E8, NV, 0, false><<<grid, WG, 0, st>>>(i4, o4, meta, nchunks, G, lg, meta_val); \
        } } while (0)
    if (big) MOR_ROWGROUP(1); else MOR_ROWGROUP(2);
#undef MOR_ROWGROUP
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

// Common driver of mor_fake_quantize / mor_block_format / mor_mor_stats.
static int run_quantize(const void* input, void* output, int32_t* meta, float* stats,
                        int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                        const QuantArgs& qa, bool e8, uint32_t flags, hipStream_t st) {
    const Shape sh = make_shape(rows, cols, brows, bcols);
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
    if (qa.qmode == 2 && qa.fmt >= 0 && !stats && output && vec_ok && brows == 1 && cols % bcols == 0 && is_pow2(G) && G <= 256) {
        if (e8) launch_rowgroup<true>(qa.fmt, input, output, meta, rows * cols / 8, (int)G, meta ? qa.meta_val : -1, st);
        else launch_rowgroup<false>(qa.fmt, input, output, meta, rows * cols / 8, (int)G, meta ? qa.meta_val : -1, st);
        return mor_check_launch("k_rowgroup");
    }
    const bool mor_mode = qa.qmode == 1;
    if (vec_ok && brows * (bcols / 8) < WG) {
        mor_launch_subblock(mor_mode, e8, input, output, meta, stats, sh, qa, st);
        return mor_check_launch("k_subblock");
    }
    if (vec_ok && brows * (bcols / 8) <= 8 * 1024) {
        mor_launch_wgblock(mor_mode, e8, false, input, output, meta, stats, sh, qa, st);
        return mor_check_launch("k_wgblock");
    }
    if (vec_ok) {                                   // larger blocks of whole vectors
        mor_launch_bigblock(mor_mode, e8, input, output, meta, stats, sh, qa, st);
        return mor_check_launch("k_bigblock");
    }
    // bit 0: power-of-two scale; bit 1: the few-instruction arithmetic (hardware converts) is allowed
    const int gflags = (e8 ? 1 : 0) | (fast_ok ? 2 : 0);
    if (brows * bcols <= 512) {
        constexpr int PER_WAVE = 8;
        for_slices(cdiv(nblocks, PER_WAVE), [&](int64_t first, int count) {
            if (emu) k_generic_wave<true><<<count, 64, 0, st>>>(in16, out16, meta, stats, sh, qa, gflags, first * PER_WAVE, nblocks, PER_WAVE);
            else k_generic_wave<false><<<count, 64, 0, st>>>(in16, out16, meta, stats, sh, qa, gflags, first * PER_WAVE, nblocks, PER_WAVE);
        });
        return mor_check_launch("k_generic_wave");
    }
    if (fast_ok && brows * ((bcols + 1) / 2) <= 32 * WG && brows * cols < 0x7FFFFFFFll && nblocks <= 0x7FFFFFFFll) {
        mor_launch_wgblock(mor_mode, e8, true, input, output, meta, stats, sh, qa, st);
        return mor_check_launch("k_wgblock (element-wise)");
    }
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
    if (int rc = mor_validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!output || !meta) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output / meta is NULL");
    hipStream_t st = static_cast<hipStream_t>(stream);
    QuantArgs qa;
    const bool e8 = (sf_type == 2);                     // FQ:1792, 1797
    if (!mor_decode_mode(mode, clamp_threshold, qa)) {
        // FQ:1831-1833, 727-729, 843: bf16 copy, meta 3
        const int64_t nblocks = cdiv(rows, brows) * cdiv(cols, bcols);
        if (output != input) {
            const int64_t n = rows * cols;
            const int64_t nvec = (aligned16(input) && aligned16(output)) ? n / 8 : 0;
            const uint16_t* i16 = static_cast<const uint16_t*>(input);
            uint16_t* o16 = static_cast<uint16_t*>(output);
            // (from HBM one vector per lane copies fastest, as in k_rowgroup)
            // (the meta entries leave with the same launch: a launch of their own costs 2 us of the 45 at 8192^2)
            if (nvec >= ((int64_t)4 << 20)) k_copy<1><<<(int)cdiv(nvec, (int64_t)WG), WG, 0, st>>>(i16, o16, n, nvec, meta, nblocks);
            else k_copy<2><<<nvec > 0 ? (int)cdiv(nvec, 2ll * WG) : grid_for(n, 16), WG, 0, st>>>(i16, o16, n, nvec, meta, nblocks);
        } else {
            k_fill_i32<<<grid_for(nblocks), WG, 0, st>>>(meta, nblocks, 3);
        }
        return mor_check_launch("k_copy / k_fill_i32");
    }
    qa.ref_sums = (flags & MOR_FLAG_REFERENCE_ORDER_SUMS) ? 1 : 0;
    return run_quantize(input, output, meta, nullptr, rows, cols, brows, bcols, qa, e8, flags, st);
}

extern "C" int mor_block_format(const void* input, void* output,
                                int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                                int fmt, int64_t sf_type, uint32_t flags, void* stream) {
    if (int rc = mor_validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!output) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output is NULL");
    if (fmt < MOR_FMT_COPY || fmt > 3) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "unknown format %d", fmt);
    QuantArgs qa{};
    qa.qmode = 2; qa.fmt = fmt; qa.meta_val = -1;
    return run_quantize(input, output, nullptr, nullptr, rows, cols, brows, bcols, qa, sf_type == 2, flags, static_cast<hipStream_t>(stream));
}

extern "C" int mor_mor_stats(const void* input, int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                             double clamp_threshold, int64_t mode, int64_t sf_type, float* stats, uint32_t flags, void* stream) {
    if (int rc = mor_validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!stats) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "stats is NULL");
    QuantArgs qa{};
    qa.qmode = 1; qa.fmt = -1; qa.meta_val = -1;
    qa.clamp = (float)clamp_threshold;
    qa.dyn_range = (mode / 100 > 0) ? 1 : 0;
    qa.ref_sums = (flags & MOR_FLAG_REFERENCE_ORDER_SUMS) ? 1 : 0;
    return run_quantize(input, nullptr, nullptr, stats, rows, cols, brows, bcols, qa, sf_type == 2, flags, static_cast<hipStream_t>(stream));
}

extern "C" int mor_block_stats(const void* input, int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                               float fmax, float* amax, float* scale, int32_t* e8m0, void* stream) {
    if (int rc = mor_validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!amax || !scale || !e8m0) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output pointer is NULL");
    const Shape sh = make_shape(rows, cols, brows, bcols);
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
