// k_subblock (a lane group per small block) and k_bigblock (one workgroup sweeping a block that exceeds the registers).
// "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>

#include "mor_quant.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

namespace mor {

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
    const bool nt_in = streams_last_read(sh.rows * sh.cols), nt_out = streams_out(sh.rows * sh.cols);

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
            if (qa.ref_sums || !(fabsf(e4 - e5) > 1e-5f * fmaxf(e4, e5))) hard = true;        // too close for the reciprocal-based sums (or the reference's order is asked for)
            else qt = mor_decide_error(amax, qa.clamp, e4, e5);
        }
        meta_val = qt;
        fmt = mor_fmt_of(qt);
    }
    if (valid && hard && l == 0) s_hard[g] = 1;
    if (valid && !hard) {
        if (l == 0) {
            if (meta && meta_val >= 0) meta[bid] = meta_val;
            if (stats) { float* s = stats + 4 * (int64_t)bid; s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5; }
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
                uint32_t qcodes = 0;
                if (fmt == FMT_E4M3) {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], fq_vec_div<FMT_E4M3>(v[k], s4.s, r4, qcodes), nt_out);
                } else {
#pragma unroll
                    for (int k = 0; k < NV; ++k) if (ok[k]) store16_rt(bout + off[k], fq_vec_div<FMT_E5M2>(v[k], s5.s, r4 * 0.0078125f, qcodes), nt_out);
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
        generic_block<false, false, WG, MOR>(reinterpret_cast<const uint16_t*>(in), reinterpret_cast<uint16_t*>(out), meta, stats,
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
    uint32_t by32, bx32;
    block_of(sh, (uint32_t)bid, by32, bx32);                  // (fewer than 2^31 blocks)
    const int64_t by = by32, bx = bx32;
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
        generic_block<false, false, WGS, MOR>(reinterpret_cast<const uint16_t*>(in), reinterpret_cast<uint16_t*>(out), meta, stats,
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
            if (qa.ref_sums || !(fabsf(e4 - e5) > 1e-5f * fmaxf(e4, e5))) {
                // too close for the reciprocal-based sums and this kernel's order of additions to be trusted with the
                // decision (or asked for): the reference's divisions in the reference's order (rare)
                const uint16_t* b16 = reinterpret_cast<const uint16_t*>(in) + (r0 * sh.cols + c0);
                err_sums_reference_order<false, WGS>([&](int r, int c) { return b16[(int64_t)r * sh.cols + c]; },
                                                     rows_valid, (int)min(sh.bcols, sh.cols - c0), sh.brows, sh.bcols, sh.cols % 2 == 0,
                                                     E8, s4, s5, e4, e5);
            }
            qt = mor_decide_error(amax, qa.clamp, e4, e5);
        }
        meta_val = qt;
        fmt = mor_fmt_of(qt);
    }
    if (tid == 0) {
        if (meta && meta_val >= 0) meta[bid] = meta_val;
        if (stats) { float* s = stats + 4 * (int64_t)bid; s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5; }
    }
    if (!out) return;

    // pass 3: quantize and store, FQ:733-851 (the last read of the block: streamed when the tensor streams)
    const bool nt_in = streams_last_read(sh.rows * sh.cols), nt_out = streams_out(sh.rows * sh.cols);
    if ((fmt < 0) || !(amax > 0.0f)) {
        if (out != in) sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, v, nt_out); });
        return;
    }
    if constexpr (!E8) {
        if (fmt == FMT_E4M3 || fmt == FMT_E5M2) {
            const float r4 = 1.0f / s4.s;            // 1 / s5 = r4 / 128 exactly
            uint32_t qcodes = 0;
            if (fmt == FMT_E4M3) sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, fq_vec_div<FMT_E4M3>(v, s4.s, r4, qcodes), nt_out); });
            else sweep(nt_in, [&](uint4 v, uint32_t off) { store16_rt(bout + off, fq_vec_div<FMT_E5M2>(v, s5.s, r4 * 0.0078125f, qcodes), nt_out); });
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

}  // namespace mor

using namespace mor;

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
void mor_launch_subblock(bool mor, bool e8, const void* in, void* out, int32_t* meta, float* stats,
                         const Shape& sh, const QuantArgs& qa, hipStream_t st) {
    if (mor) { if (e8) launch_subblock<true, true>(in, out, meta, stats, sh, qa, st); else launch_subblock<true, false>(in, out, meta, stats, sh, qa, st); }
    else { if (e8) launch_subblock<false, true>(in, out, meta, stats, sh, qa, st); else launch_subblock<false, false>(in, out, meta, stats, sh, qa, st); }
}

void mor_launch_bigblock(bool mor, bool e8, const void* in, void* out, int32_t* meta, float* stats,
                         const Shape& sh, const QuantArgs& qa, hipStream_t st) {
    const uint4* i4 = static_cast<const uint4*>(in);
    uint4* o4 = static_cast<uint4*>(out);
    for_slices(sh.gy * sh.gx, [&](int64_t first, int count) {
        if (mor) {
            if (e8) k_bigblock<true, true><<<count, BIG_WG, 0, st>>>(i4, o4, meta, stats, sh, qa, first);
            else k_bigblock<true, false><<<count, BIG_WG, 0, st>>>(i4, o4, meta, stats, sh, qa, first);
        } else {
            if (e8) k_bigblock<false, true><<<count, BIG_WG, 0, st>>>(i4, o4, meta, stats, sh, qa, first);
            else k_bigblock<false, false><<<count, BIG_WG, 0, st>>>(i4, o4, meta, stats, sh, qa, first);
        }
    });
}
