// Block / channel scaling and e8mx kernels and their C ABI entry points for MI355X (gfx950, wave64).
// "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.

#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>
#include <algorithm>
#include <atomic>

#include "mor_common.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

// ================================================================================================
// Block / channel scaling (FQ:951-1241, 1459-1752, host FQ:2013-2230, 2431-2660) and e8mx (FQ:1243-1428).
//
// Workspace layout (32-bit words): [0] tensor amax bits, [1] non-zero count, [2..3] spare, then three arrays of
// MAX_PARTIALS per-workgroup partials (error sums of pass 2; amax and non-zero counts of pass 1), then one float
// per block (amax, turned into the block's scale in place).  Nothing is accumulated with atomics except the
// per-column maxima of the column kernel, so all results are independent of scheduling.
namespace mor {

constexpr int WS_HEADER = 4;
constexpr int MAX_PARTIALS = 8192;     // slots of each partial array in the workspace
constexpr int PASS1_MAX = 1024;        // workgroups (= partials) of a pass-1 kernel: every pass-2 workgroup reduces them again
constexpr int PASS2_MAX = 2048;        // workgroups (= error partials) of a pass-2 kernel: every workgroup of the last kernel adds them
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

// one workgroup's amax / nnz -> its slot of the partial arrays; returns the workgroup amax to every thread.
// An amax of bf16 values has 16 low zero bits as a float: two of them carry what the workgroup saw besides
// (PART_SPECIAL: a NaN or a -0; PART_TINY: a non-zero magnitude below 2^-94, denormals included).  Every reader masks
// them off; k_bs_amax_flat sets them, the other producers leave them 0 and their consumers do not ask.
constexpr uint32_t PART_SPECIAL = 1u, PART_TINY = 2u, PART_FLAGS = 0xFFFFu;
__device__ __forceinline__ float publish_partial(uint32_t* ws, float amax, int nnz, float* s_f, int* s_i, uint32_t flags = 0u) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    amax = group_max(amax, 64);
    nnz = wave_sum_i(nnz);
    const uint32_t wave_flags = (__builtin_amdgcn_ballot_w64((flags & PART_SPECIAL) != 0) != 0 ? PART_SPECIAL : 0u)
                              | (__builtin_amdgcn_ballot_w64((flags & PART_TINY) != 0) != 0 ? PART_TINY : 0u);
    __syncthreads();
    if (lane == 0) { s_f[wave] = u2f((f2u(amax) & ~PART_FLAGS) | wave_flags); s_i[wave] = nnz; }
    __syncthreads();
    const uint32_t b0 = f2u(s_f[0]), b1 = f2u(s_f[1]), b2 = f2u(s_f[2]), b3 = f2u(s_f[3]);
    const uint32_t a = max(max(b0 & ~PART_FLAGS, b1 & ~PART_FLAGS), max(b2 & ~PART_FLAGS, b3 & ~PART_FLAGS));       // (non-negative floats order as integers)
    if (threadIdx.x == 0) {
        ws[WS_PAMAX + blockIdx.x] = a | ((b0 | b1 | b2 | b3) & PART_FLAGS);
        reinterpret_cast<int*>(ws)[WS_PNNZ + blockIdx.x] = s_i[0] + s_i[1] + s_i[2] + s_i[3];
    }
    return u2f(a);
}

// tensor amax from the pass-1 partials (every thread of the workgroup gets it); `flags`: the OR of the partials' flags
__device__ __forceinline__ float reduce_partial_amax(const uint32_t* ws, int npart, float* s_f, uint32_t* flags = nullptr) {
    const uint32_t* pa = ws + WS_PAMAX;
    uint32_t a = 0, fl = 0;
#pragma unroll 8
    for (int i = threadIdx.x; i < npart; i += WG) { const uint32_t b = pa[i]; a = max(a, b & ~PART_FLAGS); fl |= b; }
    a = group_umax(a, 64);
    fl = (__builtin_amdgcn_ballot_w64((fl & PART_SPECIAL) != 0) != 0 ? PART_SPECIAL : 0u) | (__builtin_amdgcn_ballot_w64((fl & PART_TINY) != 0) != 0 ? PART_TINY : 0u);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s_f[threadIdx.x >> 6] = u2f(a | fl);
    __syncthreads();
    const uint32_t b0 = f2u(s_f[0]), b1 = f2u(s_f[1]), b2 = f2u(s_f[2]), b3 = f2u(s_f[3]);
    if (flags) *flags = (b0 | b1 | b2 | b3) & PART_FLAGS;
    return u2f(max(max(b0 & ~PART_FLAGS, b1 & ~PART_FLAGS), max(b2 & ~PART_FLAGS, b3 & ~PART_FLAGS)));
}

// pass 1, blocks 1 x 8G as lane groups over the flat chunk array (FQ:1430-1457, 1611-1629).  A workgroup takes
// tiles of 8 * 256 consecutive chunks, all loads of a tile in flight at once.  block_amax may be NULL (e8mx).
// Without block maxima (the tensor-amax strategies that keep no per-block array, e8mx) the maxima and the count are
// taken on packed 16-bit magnitudes, and the partial carries a flag when the workgroup saw a NaN or a -0, so that the
// quantize pass of a tensor without either need not look for them again.
__global__ __launch_bounds__(WG) void k_bs_amax_flat(const uint4* in, uint32_t* ws, float* block_amax,
                                                     int64_t nchunks, int G, int logG) {
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    constexpr int NV = 8;
    float gmax = 0.0f;
    int nnz = 0;
    const int64_t ntiles = (nchunks + NV * WG - 1) / (NV * WG);
    if (!block_amax) {
        uint32_t negz2 = NEGZERO_INIT, amin2 = AMIN2_INIT_M1;
        bool special = false;
        const bool nt = streams_in(nchunks * 8);
        for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
            const int64_t base = tile * (NV * WG) + threadIdx.x;
            uint4 v[NV];
            if (base + (NV - 1) * WG < nchunks) {          // a whole tile for this lane: eight loads in a row
                load16_group(v, nt, [&](int k) { return in + base + k * WG; });
            } else {
#pragma unroll
                for (int k = 0; k < NV; ++k) {
                    v[k] = make_uint4(0, 0, 0, 0);
                    if (base + k * WG < nchunks) v[k] = load16_rt(in + base + k * WG, nt);
                }
            }
            uint32_t amax2 = 0, nnz2 = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                acc_amax_pk(amax2, v[k].x); acc_amax_pk(amax2, v[k].y); acc_amax_pk(amax2, v[k].z); acc_amax_pk(amax2, v[k].w);
                acc_nnz_pk(nnz2, v[k].x); acc_nnz_pk(nnz2, v[k].y); acc_nnz_pk(nnz2, v[k].z); acc_nnz_pk(nnz2, v[k].w);
                acc_negzero_pk(negz2, v[k].x); acc_negzero_pk(negz2, v[k].y); acc_negzero_pk(negz2, v[k].z); acc_negzero_pk(negz2, v[k].w);
                acc_amin_pk(amin2, v[k].x); acc_amin_pk(amin2, v[k].y); acc_amin_pk(amin2, v[k].z); acc_amin_pk(amin2, v[k].w);
            }
            if (amax_bits_of(amax2) > 0x7F800000u) {      // a NaN among the lane's 64 values (rare): the float maximum and count skip it
                special = true;
                float amax = 0.0f;
                int n = 0;
#pragma unroll
                for (int k = 0; k < NV; ++k) acc_amax_nnz(amax, n, v[k]);
                gmax = fmaxf(gmax, amax);
                nnz += n;
            } else {
                gmax = fmaxf(gmax, u2f(amax_bits_of(amax2)));
                nnz += (int)((nnz2 & 0xFFFFu) + (nnz2 >> 16));
            }
        }
        // (amin_m1_of: fp32 bits of the smallest non-zero magnitude minus one bf16 step, low half ones)
        const bool tiny = amin_m1_of(amin2) < ((33u << 23) - 1u);
        publish_partial(ws, gmax, nnz, s_f, s_i, ((special || saw_negzero(negz2)) ? PART_SPECIAL : 0u) | (tiny ? PART_TINY : 0u));
        return;
    }
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
    publish_partial(ws, amax, 0, s_f, s_i, PART_SPECIAL | PART_TINY);          // (nothing was looked for: consumers assume the worst)
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
            // Four loads at a time, unconditional (a chunk beyond the block reads the lane's first chunk again and counts
            // as zeros), under one choice of the cache policy: loads chosen or bounded one by one are each waited for
            // before the next is issued.
            auto scan = [&](auto streaming) {
#pragma unroll 1
                for (uint32_t j = l; j < nchb; j += 4u * (uint32_t)L) {
                    uint4 v[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const uint32_t jj = j + (uint32_t)u * (uint32_t)L, js = jj < nchb ? jj : l;
                        const uint32_t r = div_u32(js, d_cpr), cc = js - r * cpr;
                        v[u] = load16<decltype(streaming)::value>(bin + r * row_stride + cc);
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (j + (uint32_t)u * (uint32_t)L >= nchb) v[u] = make_uint4(0, 0, 0, 0);
                        acc_amax_nnz(amax, nnz, v[u]);
                    }
                }
            };
            if (nt) scan(std::true_type{}); else scan(std::false_type{});
        }
        amax = group_max(amax, L);                   // (shuffles: every lane of the wave takes part)
        if (bid < nb && l == 0) block_amax[bid] = amax;
        gmax = fmaxf(gmax, amax);
    }
    publish_partial(ws, gmax, nnz, s_f, s_i);
}


// pass 1, column blocks N x 1 (FQ:1538-1610) for the tensors k_bs_colmax does not take (other flavour, power-of-two
// scale, unaligned rows): a workgroup covers 256 adjacent columns (32 groups of 8) with 8 row
// lanes; a thread takes every 8th row of a row segment, the 8 row lanes meet in LDS and one thread per column merges
// into the (zero-initialised) per-block maxima with atomicMax on the bit patterns of non-negative floats.
__global__ __launch_bounds__(WG) void k_bs_amax_col(const uint16_t* in, uint32_t* ws, float* block_amax, Shape sh,
                                                    int rows_per_wg, int vec) {
    __shared__ float s_m[8][32 * 8 + 8];
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    const int cg = threadIdx.x & 31, rl = threadIdx.x >> 5;
    const int64_t segs_per_block = (sh.brows + rows_per_wg - 1) / rows_per_wg;
    float gmax = 0.0f;
    int nnz = 0;
    // groups of 256 columns grid-stride along x, row segments of all block rows grid-stride along y
    for (int64_t bx = blockIdx.x; bx * 256 < sh.cols; bx += gridDim.x) {
    const int64_t col0 = (bx * 32 + cg) * 8;
    const int ncol = (int)max((int64_t)0, min((int64_t)8, sh.cols - col0));
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
        const int64_t c = bx * 256 + threadIdx.x;
        if (c < sh.cols && cm > 0.0f) atomicMax(reinterpret_cast<uint32_t*>(&block_amax[by * sh.cols + c]), f2u(cm));
        gmax = fmaxf(gmax, cm);
    }
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

// Column blocks N x 1 with aligned rows, default flavour, fp32 scale: three kernels and the plan they share.
//   k_bs_colmax   reads the tensor in the order it lies in memory (a workgroup owns whole rows, or NG * 4 KiB of each
//                 of its rows): every lane meets the same few column groups again and again and keeps their packed
//                 16-bit maxima; a block's rows are cut into P segments, one row of partial maxima per segment (bf16
//                 bits, no atomics, nothing to clear);
//   k_bs_colfold  folds the P partial rows of every block and column and leaves the column's scale and its reciprocal;
//   k_bs_quant_col quantizes, a lane holding 8 rows of its 8 columns, strips as wide as a row allows.
// W = lanes a row (or a slab of it) is wide in pass 1: min(256, column groups), a power of two; a row of more than 256
// groups is NG * 256 groups (or slabs of that width).  Tensors whose group count fits neither form take the general
// kernels.
constexpr int COL_PASS1_WGS = 512;
struct ColPlan {
    int w_log;                  // pass 1: log2 of the lanes per row sweep (256 groups and more: 8)
    int ng;                     // pass 1: column groups per lane (1 when a sweep holds one or several whole rows)
    int64_t slabs;              // pass 1: slabs of ng * 256 groups a row is cut into
    int r1, P;                  // pass 1: rows per batch, workgroups (and partial rows) per block and slab
    int64_t items1;             // (slab, block row, segment) triples, slabs fastest
    int cg_log;                 // pass 2: log2 of the lanes a strip is wide
    int64_t strips, items2;     // pass 2: strips per row; (strip, block row, workgroup) triples
    int Q;                      // pass 2: workgroups per block and strip
};
static bool col_plan(int64_t rows, int64_t cols, int64_t brows, ColPlan& p) {
    p = ColPlan{};
    if (cols % 8 != 0 || brows <= 0 || rows % brows != 0) return false;
    const int64_t groups = cols / 8, gyb = rows / brows;
    if (groups <= WG) {
        if (!is_pow2(groups)) return false;
        p.w_log = ilog2(groups); p.ng = 1; p.slabs = 1;
    } else {
        if (groups % WG != 0) return false;
        const int64_t q = groups / WG;
        p.w_log = 8;
        p.ng = 1;
        for (int g = 8; g >= 1; --g) if (q % g == 0) { p.ng = g; break; }
        p.slabs = q / p.ng;
    }
    // pass 1: a block's rows in batches of whole sweeps (8 loads in flight per lane where the rows allow), dealt out in
    // turn to the P workgroups of the block and slab; about COL_PASS1_WGS workgroups (more read no faster and leave more
    // partial rows to fold: 16384 x 14336 takes 76 + 10 us with 512, 90 + 17 us with 1024), never more than PASS1_MAX (each
    // publishes a partial of the tensor amax and of the non-zero count)
    const int64_t rows_per_sweep = (int64_t)WG >> p.w_log;                 // (1 for 256 groups and more)
    p.r1 = (int)(rows_per_sweep * (p.ng >= 6 ? 1 : p.ng >= 3 ? 2 : 8 / p.ng));          // rows of a batch (UN sweeps of k_bs_colmax)
    const int64_t nb1 = cdiv(brows, p.r1);
    p.P = (int)std::max<int64_t>(1, std::min<int64_t>(nb1, COL_PASS1_WGS / std::max<int64_t>(1, gyb * p.slabs)));
    p.items1 = p.slabs * gyb * p.P;
    // pass 2: strips of up to 256 lanes; a block's rows in batches of 4 per row lane, dealt out in turn to the Q workgroups
    // of the block and strip; about PASS2_MAX workgroups (each publishes a partial of the error sum)
    p.cg_log = (int)std::min<int64_t>(8, ilog2(groups + 1) - 1);          // floor(log2(groups))
    p.strips = cdiv(groups, (int64_t)1 << p.cg_log);
    const int64_t nb2 = cdiv(brows, 4 * ((int64_t)WG >> p.cg_log));
    p.Q = (int)std::max<int64_t>(1, std::min<int64_t>(cdiv(nb2, 2), PASS2_MAX / std::max<int64_t>(1, gyb * p.strips)));
    p.items2 = p.strips * gyb * p.Q;
    return true;
}
// 32-bit words of the workspace this path takes behind the header: the partial maxima ([block row][segment][column]
// 16-bit) and the columns' scales ([block row][column] pairs of floats)
static int64_t col_words(int64_t rows, int64_t cols, int64_t brows) {
    ColPlan p;
    if (!col_plan(rows, cols, brows, p)) return 0;
    return (rows / brows) * cols * 2 + (rows / brows) * p.P * cols / 2;
}

// Magnitudes leave bit 15 of each half of a partial word free.  In the first word of a column group those two bits
// say what the group's 8 columns held in the rows the partial covers: a NaN, a -0.
constexpr uint32_t COL_FLAG_NAN = 0x00008000u, COL_FLAG_NEGZERO = 0x80000000u, COL_FLAGS = COL_FLAG_NAN | COL_FLAG_NEGZERO;
// a packed word with the halves that hold a NaN set to +0
__device__ __forceinline__ uint32_t drop_nan_pk(uint32_t w) {
    const uint32_t lo = ((w & 0x7FFFu) > 0x7F80u) ? 0u : (w & 0xFFFFu), hi = ((w & 0x7FFF0000u) > 0x7F800000u) ? 0u : (w & 0xFFFF0000u);
    return lo | hi;
}
// pass 1 (FQ:1538-1610 without the atomics).  item = (slab, block row, workgroup of the P that share them), slabs fastest.
template <int NG>
__global__ __launch_bounds__(WG) void k_bs_colmax(const uint4* in, uint32_t* ws, uint16_t* partial, Shape sh, ColPlan p) {
    __shared__ uint4 s_m[WG];
    __shared__ float s_f[WAVES];
    __shared__ int s_i[WAVES];
    constexpr int UN = NG >= 6 ? 1 : NG >= 3 ? 2 : 8 / NG;               // sweeps of a batch: NG * UN = 6 to 8 loads in flight per lane
    const int tid = threadIdx.x, W = 1 << p.w_log, cl = tid & (W - 1), rsub = tid >> p.w_log, rps = WG >> p.w_log;
    const int64_t row_stride = sh.cols >> 3, groups = row_stride;
    const bool nt = streams_in(sh.rows * sh.cols);
    uint32_t gmax2 = 0;
    int nnz = 0;
    for (int64_t item = blockIdx.x; item < p.items1; item += gridDim.x) {
        const int64_t seg = item / p.slabs, slab = item - seg * p.slabs;
        const int64_t by = seg / p.P, sg = seg - by * p.P;
        // the block's batches sg, sg + P, ...: workgroups that run side by side read neighbouring rows
        const int64_t b_rows = by * sh.brows, r_end = (by + 1) * sh.brows, step = p.r1, stride = step * p.P;
        const int64_t r_first = b_rows + sg * step + rsub;
        const uint4* col = in + (slab * NG * WG + cl);                    // this lane's first column group
        uint32_t m[NG][4];
#pragma unroll
        for (int g = 0; g < NG; ++g) { m[g][0] = 0; m[g][1] = 0; m[g][2] = 0; m[g][3] = 0; }
        // what pass 2 wants to know about this lane's columns besides their maxima: whether one of them holds a NaN (then
        // they take the exact arithmetic) or a -0 (then the sign bits are not copied blindly)
        uint32_t negz2 = NEGZERO_INIT, flags = 0;
#pragma unroll 1
        for (int64_t r = r_first; r < r_end; r += stride) {
            uint4 v[UN][NG];
#pragma unroll
            for (int u = 0; u < UN; ++u)
#pragma unroll
                for (int g = 0; g < NG; ++g) {
                    v[u][g] = make_uint4(0, 0, 0, 0);
                    if (r + u * rps < r_end) v[u][g] = load16_rt(col + (r + u * rps) * row_stride + g * WG, nt);
                }
            // the batch's maxima and count; a NaN wins a packed maximum and counts as non-zero where the reference's float
            // maximum and its count (FQ:998-999) skip it: a batch that holds one is folded again with its NaNs set to zero
            uint32_t t[NG][4], nz2 = 0;
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                t[g][0] = 0; t[g][1] = 0; t[g][2] = 0; t[g][3] = 0;
#pragma unroll
                for (int u = 0; u < UN; ++u) {
                    acc_amax_pk(t[g][0], v[u][g].x); acc_amax_pk(t[g][1], v[u][g].y); acc_amax_pk(t[g][2], v[u][g].z); acc_amax_pk(t[g][3], v[u][g].w);
                    acc_nnz_pk(nz2, v[u][g].x); acc_nnz_pk(nz2, v[u][g].y); acc_nnz_pk(nz2, v[u][g].z); acc_nnz_pk(nz2, v[u][g].w);
                    acc_negzero_pk(negz2, v[u][g].x); acc_negzero_pk(negz2, v[u][g].y); acc_negzero_pk(negz2, v[u][g].z); acc_negzero_pk(negz2, v[u][g].w);
                }
            }
            uint32_t any = 0;
#pragma unroll
            for (int g = 0; g < NG; ++g) any = pk_max_u16(any, pk_max_u16(pk_max_u16(t[g][0], t[g][1]), pk_max_u16(t[g][2], t[g][3])));
            if (amax_bits_of(any) > 0x7F800000u) {          // (rare)
                flags |= COL_FLAG_NAN;
                nz2 = 0;
#pragma unroll
                for (int g = 0; g < NG; ++g) {
                    t[g][0] = 0; t[g][1] = 0; t[g][2] = 0; t[g][3] = 0;
#pragma unroll
                    for (int u = 0; u < UN; ++u) {
                        const uint32_t w[4] = {drop_nan_pk(v[u][g].x), drop_nan_pk(v[u][g].y), drop_nan_pk(v[u][g].z), drop_nan_pk(v[u][g].w)};
#pragma unroll
                        for (int j = 0; j < 4; ++j) { acc_amax_pk(t[g][j], w[j]); acc_nnz_pk(nz2, w[j]); }
                    }
                }
            }
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                m[g][0] = pk_max_u16(m[g][0], t[g][0]); m[g][1] = pk_max_u16(m[g][1], t[g][1]);
                m[g][2] = pk_max_u16(m[g][2], t[g][2]); m[g][3] = pk_max_u16(m[g][3], t[g][3]);
            }
            nnz += (int)((nz2 & 0xFFFFu) + (nz2 >> 16));          // (at most 8 * UN * NG <= 128 per batch: the 16-bit counts cannot wrap)
        }
        // several rows per sweep (fewer than 256 groups): the lanes of one column group meet in LDS
        if (saw_negzero(negz2)) flags |= COL_FLAG_NEGZERO;
        if (rps > 1) {
            __syncthreads();                       // the previous item's readers are done
            s_m[tid] = make_uint4(m[0][0] | flags, m[0][1], m[0][2], m[0][3]);
            __syncthreads();
            if (rsub == 0) {
#pragma unroll 1
                for (int k = 1; k < rps; ++k) {
                    const uint4 o = s_m[(k << p.w_log) + cl];
                    flags |= o.x & COL_FLAGS;
                    m[0][0] = pk_max_u16(m[0][0], o.x & ~COL_FLAGS); m[0][1] = pk_max_u16(m[0][1], o.y); m[0][2] = pk_max_u16(m[0][2], o.z); m[0][3] = pk_max_u16(m[0][3], o.w);
                }
            }
        }
        if (rsub == 0) {
            // (the flags are the lane's: they ride in the two free top bits of the first word of each of its column groups)
            uint4* prow = reinterpret_cast<uint4*>(partial) + (seg * groups + slab * NG * WG + cl);
#pragma unroll
            for (int g = 0; g < NG; ++g) prow[g * WG] = make_uint4(m[g][0] | flags, m[g][1], m[g][2], m[g][3]);
        }
#pragma unroll
        for (int g = 0; g < NG; ++g) gmax2 = pk_max_u16(gmax2, pk_max_u16(pk_max_u16(m[g][0], m[g][1]), pk_max_u16(m[g][2], m[g][3])));
    }
    publish_partial(ws, u2f(amax_bits_of(gmax2)), nnz, s_f, s_i);
}

__device__ __forceinline__ float scaling_factor(float global_amax, float block_amax, int ss_mode);

// pass 1b: for every block row and column the maximum over the P partial rows, turned into the column's scale and its
// reciprocal (0 for a scale outside the fast range).  A workgroup takes 8 column groups (64 columns, whole cache lines of the partial rows) of one block row,
// 32 lanes of partial rows each: the 8 of a wave meet by shuffles, the waves in LDS.
constexpr int FOLD_G = 8;
__global__ __launch_bounds__(WG) void k_bs_colfold(const uint16_t* partial, float2* scales, uint32_t* ws, int npart1, int ss_mode,
                                                   Shape sh, ColPlan p) {
    __shared__ float s_f[WAVES];
    __shared__ uint4 s_m[WAVES][FOLD_G];
    __shared__ uint32_t s_flags[WAVES][FOLD_G];
    const float gamax = reduce_partial_amax(ws, npart1, s_f);
    const int tid = threadIdx.x, c = tid & (FOLD_G - 1), pl = tid / FOLD_G, lane = tid & 63, wave = tid >> 6;
    const int64_t groups = sh.cols >> 3, gw = (groups + FOLD_G - 1) / FOLD_G;
    const int64_t by = blockIdx.x / gw, cg0 = (blockIdx.x - by * gw) * FOLD_G, cg = cg0 + c;
    const uint4* prow = reinterpret_cast<const uint4*>(partial) + by * p.P * groups;
    uint32_t m[4] = {0, 0, 0, 0}, flags = 0;
    if (cg < groups) {
#pragma unroll 8
        for (int k = pl; k < p.P; k += WG / FOLD_G) {
            const uint4 o = prow[k * groups + cg];
            flags |= o.x & COL_FLAGS;
            m[0] = pk_max_u16(m[0], o.x & ~COL_FLAGS); m[1] = pk_max_u16(m[1], o.y); m[2] = pk_max_u16(m[2], o.z); m[3] = pk_max_u16(m[3], o.w);
        }
    }
#pragma unroll
    for (int off = FOLD_G; off < 64; off <<= 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j) m[j] = pk_max_u16(m[j], (uint32_t)__shfl_xor((int)m[j], off));
        flags |= (uint32_t)__shfl_xor((int)flags, off);
    }
    if (lane < FOLD_G) { s_m[wave][lane] = make_uint4(m[0], m[1], m[2], m[3]); s_flags[wave][lane] = flags; }
    __syncthreads();
    if (tid < 8 * FOLD_G) {                    // one thread per column
        const int g = tid >> 3, j = tid & 7;
        uint32_t mb = 0, fl = 0;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            mb = max(mb, (uint32_t)reinterpret_cast<const uint16_t*>(&s_m[w][g])[j]);
            fl |= s_flags[w][g];
        }
        const float amax = u2f(mb << 16);
        Scale sc = make_scale(scaling_factor(gamax, amax, ss_mode));
        // a column of zeros (FQ:1063-1064: its scale is 448 / 1e-35, outside the fast range) gives +0 with any scale
        if (!(amax > 0.0f)) { sc.s = 1.0f; sc.r = 1.0f; sc.fast = true; }
        // second word: the reciprocal; 0 = the column takes the exact arithmetic (scale outside the fast range, a NaN
        // in the column group); negative = a -0 in the column group
        float r = (sc.fast && !(fl & COL_FLAG_NAN)) ? sc.r : 0.0f;
        if (fl & COL_FLAG_NEGZERO) r = -r;
        const int64_t col = (cg0 + g) * 8 + j;
        if (col < sh.cols) scales[by * sh.cols + col] = make_float2(sc.s, r);
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

// The scale of one block (FQ:1059-1093) from the tensor amax and the block's amax, computed where it is used: the
// quantize kernels reduce the pass-1 partials to the tensor amax themselves (every workgroup, a few loads per thread)
// instead of waiting for a kernel of its own to do that and to turn every block amax into a scale.  ss_mode 4 takes
// the tensor amax alone; no per-block amax is kept for it.
__device__ __forceinline__ float block_scale(float gamax, const float* block_amax, int64_t idx, int ss_mode) {
    return scaling_factor(gamax, ss_mode == 4 ? 1.0f : block_amax[idx], ss_mode);
}

// The end of the op (FQ:1178-1241), evaluated by every workgroup of the kernel that acts on the decision (the gated
// copy or the gated write) instead of by a one-workgroup kernel of its own: the error partials are added in a fixed
// order (the same in every workgroup), the tensor amax and the non-zero count are reduced from the pass-1 partials,
// workgroup 0 writes the scalar outputs.  Returns meta: 3 (bf16 fallback) or 1 (E4M3).
struct Finish {
    const uint32_t* ws;
    int nerr, nstat;                  // error partials (pass 2), amax / non-zero partials (pass 1)
    float threshold;
    int32_t* meta;
    float* gamax_o;
    int32_t* gnnz_o;
    float* gerr_o;
};
// (WGS: threads of the calling workgroup; the first 256 do the sums, so that the order of the additions does not depend
// on the workgroup size; s_f: 8 floats, s_i: 4 ints of LDS)
template <int WGS = WG>
__device__ __forceinline__ int finish_decision(const Finish& f, float* s_f, int* s_i) {
    const float* part = reinterpret_cast<const float*>(f.ws) + WS_ERR;
    const float* pa = reinterpret_cast<const float*>(f.ws) + WS_PAMAX;
    const int* pn = reinterpret_cast<const int*>(f.ws) + WS_PNNZ;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float acc = 0.0f, a = 0.0f;
    int n = 0;
    if (WGS == WG || threadIdx.x < WG) {
#pragma unroll 4
        for (int i = threadIdx.x; i < f.nerr; i += WG) acc += part[i];
#pragma unroll 4
        for (int i = threadIdx.x; i < f.nstat; i += WG) { a = fmaxf(a, u2f(f2u(pa[i]) & ~PART_FLAGS)); n += pn[i]; }          // (low bits: publish_partial's flags)
    }
    acc = wave_sum(acc);
    a = group_max(a, 64);
    n = wave_sum_i(n);
    __syncthreads();
    if (lane == 0 && wave < WAVES) { s_f[wave] = acc; s_f[4 + wave] = a; s_i[wave] = n; }
    __syncthreads();
    const float gerr = (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]);
    const float gamax = fmaxf(fmaxf(s_f[4], s_f[5]), fmaxf(s_f[6], s_f[7]));
    const int gnnz = s_i[0] + s_i[1] + s_i[2] + s_i[3];
    const float avg = gerr / (float)gnnz;        // 0 / 0 = NaN on an all-zero tensor: not above the threshold
    const int m = (avg > f.threshold) ? 3 : 1;
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
        f.meta[0] = m;
        f.gamax_o[0] = gamax;
        f.gnnz_o[0] = gnnz;
        f.gerr_o[0] = gerr;
    }
    __syncthreads();
    return m;
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
// acc + |q - a| / a for magnitudes a of a block whose scale is in the fast range, through the hardware reciprocal.
// Both operands are taken times 2^16 first: the smallest bf16 denormal (2^-133) then has a reciprocal that fits the
// format, and the largest element such a block can hold (448 * 2^100) does not overflow, so the term is right for
// every finite element.  No selects: a zero element has q = 0 and its term is 0 * min(1 / 0, FLT_MAX) = 0.
__device__ __forceinline__ float rel_err_fast(float q, float a, float acc) {
    const float ac = a * 0x1p16f;
    return fmaf(fabsf(fmaf(q, 0x1p16f, -ac)), fminf(__builtin_amdgcn_rcpf(ac), 0x1.fffffep127f), acc);
}
// Fast version on magnitudes for scales in the fast range: hardware convert; q = c / s by a reciprocal-multiply
// with one exact-residual correction (r = 1 / s correctly rounded, the result is then the rounded quotient);
// error term |q - x| / x through the hardware reciprocal (relative 1e-7, tolerance on the sum 1e-6).
// No selects: a zero element's magnitude bits are 0; the sign of the input is kept for non-zero halves only (zero inputs come back as +0, FQ:1133-1134), through a
// packed 16-bit mask.
// ERR / OUT: whether the error terms / the output word are wanted (the in-place phases need one of them each).
// NZ: whether the word may hold a -0.  Callers that know it does not (acc_negzero_pk over the words they hold, -0
// halves cleared by drop_negzero_pk in the rare case) pass false, and the sign bits are copied as they are.
// (`codes`: the register the convert writes half of, carried from word to word so that no fresh zero is needed)
template <bool E8, bool ERR = true, bool OUT = true, bool NZ = true>
__device__ __forceinline__ uint32_t bs_pair_fast(uint32_t w, const Scale& sc, float rs, float& err, uint32_t& codes) {
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
        codes = hw_pack2_low_keep<FMT_E4M3>(a * sc.s, b * sc.s, codes);
        const f32x2 c = hw_unpack2_low<FMT_E4M3>(codes);
        qa = div_by_scale(c.x, sc.s, rs);
        qb = div_by_scale(c.y, sc.s, rs);
    }
    if constexpr (ERR) {
        err = rel_err_fast(qa, a, err);
        err = rel_err_fast(qb, b, err);
    }
    if constexpr (!OUT) return 0u;
    if constexpr (!NZ) return store_pair<false>(qa, qb) | (w & 0x80008000u);
    const uint32_t nonzero = pk_min_u16(w & 0x7FFF7FFFu, 0x00010001u);        // 1 in each half that is not +-0
    return store_pair<false>(qa, qb) | (w & (nonzero << 15));
}
template <bool E8, bool ERR, bool OUT, bool NZ = true>
__device__ __forceinline__ uint4 bs_vec_fast(uint4 v, const Scale& sc, float& err) {
    uint4 q;
    uint32_t codes = 0;
    q.x = bs_pair_fast<E8, ERR, OUT, NZ>(v.x, sc, sc.r, err, codes);
    q.y = bs_pair_fast<E8, ERR, OUT, NZ>(v.y, sc, sc.r, err, codes);
    q.z = bs_pair_fast<E8, ERR, OUT, NZ>(v.z, sc, sc.r, err, codes);
    q.w = bs_pair_fast<E8, ERR, OUT, NZ>(v.w, sc, sc.r, err, codes);
    return q;
}
// whether one of a vector's 8 values is a -0 (4 instructions and a test)
__device__ __forceinline__ bool vec_has_negzero(uint4 v) {
    return saw_negzero(pk_min_i16(pk_min_i16(v.x, v.y), pk_min_i16(v.z, v.w)));
}

// pass 2 / pass 4: quantize every element with its block's scale (from the block's amax, per chunk, or per column in
// column mode), accumulate the relative error, optionally write.  gate > 0: the gated write of the in-place op: the
// decision is evaluated first (finish_decision) and the pass runs only if it is `gate`.
template <bool E8, bool EMU, bool COL, bool WRITE, bool ERR>
__global__ __launch_bounds__(WG) void k_bs_quant(const uint16_t* in, uint16_t* out, uint32_t* ws, const float* scales,
                                                 Finish fin, int gate, int ss_mode, int npart1, Shape sh, int vec, DivU32 d_rowchunks,
                                                 DivU32 d_brows, DivU32 d_bchunks, DivU32 d_bcols) {
    __shared__ float s_f[2 * WAVES];
    __shared__ int s_i[WAVES];
    if (gate > 0 && finish_decision(fin, s_f, s_i) != gate) return;
    const float gamax = reduce_partial_amax(ws, npart1, s_f);
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
            uint4 v = load16_rt(in4 + c, WRITE && streams_last_read(sh.rows * sh.cols));
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
            if constexpr (COL) {
                const int64_t sp = (int64_t)by * sh.cols + (int64_t)cc * 8;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const Scale s0 = make_scale(block_scale(gamax, scales, sp + 2 * j, ss_mode)), s1 = make_scale(block_scale(gamax, scales, sp + 2 * j + 1, ss_mode));
                    float q0 = bs_element<E8, EMU>(bf16_lo(w[j]), s0, err);
                    float q1 = bs_element<E8, EMU>(bf16_hi(w[j]), s1, err);
                    w[j] = store_pair<EMU>(q0, q1);
                }
            } else {
                const uint32_t bx = div_u32(cc, d_bchunks);
                const Scale sc = make_scale(block_scale(gamax, scales, (int64_t)by * sh.gx + bx, ss_mode));
                if (!EMU && sc.fast && !vec_has_nan(v)) {
                    const float rs = 1.0f / sc.s;
                    uint32_t codes = 0;
                    if (WRITE && vec_has_negzero(v)) {          // (rare)
#pragma unroll
                        for (int j = 0; j < 4; ++j) w[j] = drop_negzero_pk(w[j]);
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) w[j] = bs_pair_fast<E8, ERR, WRITE, false>(w[j], sc, rs, err, codes);
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
            const Scale sc = make_scale(block_scale(gamax, scales, by * sh.gx + bx, ss_mode));
            float q = bs_element<E8, EMU>(bf16_one(in[i]), sc, err);
            if constexpr (WRITE) out[i] = store_bf16<EMU>(q);
        }
    }
    if constexpr (ERR) {
        err = wave_sum(err);
        __syncthreads();                   // every wave has read the tensor amax from these slots
        if (lane == 0) s_f[wave] = err;
        __syncthreads();
        if (threadIdx.x == 0) {
            reinterpret_cast<float*>(ws)[WS_ERR + blockIdx.x] = (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]);
        }
    }
}

// One vector of 8 adjacent columns, each with the scale cs[j] of its own column block and its reciprocal cr[j] (all in
// the fast range): the arithmetic of bs_pair_fast with a scale per half of a word; a vector that holds a NaN takes the
// exact arithmetic.
__device__ __forceinline__ Scale scale_only(float s) {
    Scale sc;
    sc.s = s; sc.r = 0.0f; sc.e8 = 0; sc.fast = false;
    return sc;
}
// the same vector with the exact arithmetic (a scale outside the fast range, a NaN)
__device__ __forceinline__ uint4 bs_cols_vec_exact(uint4 v, const float (&cs)[8], float& err) {
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float q0 = bs_element<false, false>(bf16_lo(w[j]), scale_only(cs[2 * j]), err);
        float q1 = bs_element<false, false>(bf16_hi(w[j]), scale_only(cs[2 * j + 1]), err);
        w[j] = store_pair<false>(q0, q1);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}
// (no NaN among the values: the columns that hold one are marked by k_bs_colfold and take the exact arithmetic;
// NZ: whether a -0 may be among them, as in bs_pair_fast)
template <bool WRITE, bool ERR, bool NZ>
__device__ __forceinline__ uint4 bs_cols_vec_fast(uint4 v, const float (&cs)[8], const float (&cr)[8], float& err) {
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float row_err = 0.0f;
    uint32_t codes = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = fabsf(bf16_lo(w[j])), b = fabsf(bf16_hi(w[j]));
        codes = hw_pack2_low_keep<FMT_E4M3>(a * cs[2 * j], b * cs[2 * j + 1], codes);
        const f32x2 c = hw_unpack2_low<FMT_E4M3>(codes);
        const float qa = div_by_scale(c.x, cs[2 * j], cr[2 * j]);
        const float qb = div_by_scale(c.y, cs[2 * j + 1], cr[2 * j + 1]);
        if constexpr (ERR) {
            row_err = rel_err_fast(qa, a, row_err);
            row_err = rel_err_fast(qb, b, row_err);
        }
        if constexpr (WRITE) {
            if constexpr (NZ) {
                const uint32_t nonzero = pk_min_u16(w[j] & 0x7FFF7FFFu, 0x00010001u);
                w[j] = store_pair<false>(qa, qb) | (w[j] & (nonzero << 15));
            } else {
                w[j] = store_pair<false>(qa, qb) | (w[j] & 0x80008000u);
            }
        }
    }
    err += row_err;
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// pass 2 / pass 4 for column blocks N x 1 with aligned rows: item = (strip, block row, workgroup of the Q that share
// them), strips fastest.  A lane owns 8 adjacent columns: it loads their scales and reciprocals (k_bs_colfold) once and
// takes every Q-th batch of 4 rows per row lane of the block, two register buffers in turn (workgroups that run side
// by side work on neighbouring rows).  Lanes whose scales are not all in the fast range use the exact
// arithmetic.
// (The loads of a batch sit in a branch -- the run-time cache policy, the bounds test of the last batch -- and are
// waited for where it ends, so the two buffers do not in fact overlap loads with arithmetic.  With the policy fixed at
// compile time and every load unconditional they do, and the kernel is slower: 47.9 against 45.3 us at 16384 x 4096.)
template <bool WRITE, bool ERR>
__global__ __launch_bounds__(WG) void k_bs_quant_col(const uint4* in, uint4* out, uint32_t* ws, const float2* scales,
                                                     Finish fin, int gate, Shape sh, ColPlan p) {
    __shared__ float s_f[2 * WAVES];
    __shared__ int s_i[WAVES];
    if (gate > 0 && finish_decision(fin, s_f, s_i) != gate) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = tid & ((1 << p.cg_log) - 1), rl = tid >> p.cg_log, row_lanes = WG >> p.cg_log;
    const int64_t row_stride = sh.cols >> 3, groups = row_stride;
    // (the decision pass of the in-place op is not the last read: its loads allocate, and the write pass finds what
    // the last-level cache kept of the tensor)
    const bool nt_in = WRITE && streams_last_read(sh.rows * sh.cols), nt_out = streams_out(sh.rows * sh.cols);
    float err = 0.0f;
    for (int64_t item = blockIdx.x; item < p.items2; item += gridDim.x) {
        const int64_t pid = item / p.strips, strip = item - pid * p.strips;
        const int64_t by = pid / p.Q, pc = pid - by * p.Q;
        const int64_t cg = (strip << p.cg_log) + cl;
        if (cg >= groups) continue;
        // the block's batches pc, pc + Q, ... of 4 rows per row lane (neighbouring workgroups on neighbouring rows)
        const int64_t step = 4 * (int64_t)row_lanes, stride = step * p.Q;
        const int64_t r_first = by * sh.brows + pc * step + rl, r_end = (by + 1) * sh.brows;
        const uint4* sp = reinterpret_cast<const uint4*>(scales + by * sh.cols + cg * 8);
        const uint4 t0 = sp[0], t1 = sp[1], t2 = sp[2], t3 = sp[3];
        const uint4* cin = in + cg;
        uint4* cout = out + cg;
        auto load_batch = [&](uint4 (&v)[4], int64_t r) {
            if ((r - rl) + step <= r_end) {        // a whole batch (uniform over the workgroup): four loads in a row
                load16_group(v, nt_in, [&](int k) { return cin + (r + k * row_lanes) * row_stride; });
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v[k] = make_uint4(0, 0, 0, 0);
                    if (r + k * row_lanes < r_end) v[k] = load16_rt(cin + (r + k * row_lanes) * row_stride, nt_in);
                }
            }
        };
        uint4 va[4], vb[4];
        load_batch(va, r_first);
        const float cs[8] = {u2f(t0.x), u2f(t0.z), u2f(t1.x), u2f(t1.z), u2f(t2.x), u2f(t2.z), u2f(t3.x), u2f(t3.z)};
        const uint32_t crb[8] = {t0.y, t0.w, t1.y, t1.w, t2.y, t2.w, t3.y, t3.w};
        bool fast = true, negz_lane = false;
#pragma unroll
        for (int j = 0; j < 8; ++j) { fast = fast && ((crb[j] & 0x7FFFFFFFu) != 0u); negz_lane = negz_lane || (crb[j] >> 31); }
        const float cr[8] = {u2f(crb[0] & 0x7FFFFFFFu), u2f(crb[1] & 0x7FFFFFFFu), u2f(crb[2] & 0x7FFFFFFFu), u2f(crb[3] & 0x7FFFFFFFu),
                             u2f(crb[4] & 0x7FFFFFFFu), u2f(crb[5] & 0x7FFFFFFFu), u2f(crb[6] & 0x7FFFFFFFu), u2f(crb[7] & 0x7FFFFFFFu)};
        const bool negz = WRITE && __builtin_amdgcn_ballot_w64(negz_lane) != 0;            // uniform over the wave
        auto do_batch = [&](uint4 (&v)[4], int64_t r) {
            if (fast) {
                if (negz) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        opaque(v[k]);                  // one vector at a time: interleaved, the four take 165 registers
                        uint4 q = bs_cols_vec_fast<WRITE, ERR, true>(v[k], cs, cr, err);
                        opaque(q);
                        if constexpr (ERR) asm volatile("" : "+v"(err));
                        if constexpr (WRITE) {
                            if (r + k * row_lanes < r_end) store16_rt(cout + (r + k * row_lanes) * row_stride, q, nt_out);
                        }
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        opaque(v[k]);                  // one vector at a time: interleaved, the four take 165 registers
                        uint4 q = bs_cols_vec_fast<WRITE, ERR, false>(v[k], cs, cr, err);
                        opaque(q);
                        if constexpr (ERR) asm volatile("" : "+v"(err));
                        if constexpr (WRITE) {
                            if (r + k * row_lanes < r_end) store16_rt(cout + (r + k * row_lanes) * row_stride, q, nt_out);
                        }
                    }
                }
            } else {
                // (from memory again, non-unrolled: indexing the register arrays with a run-time k would move them to
                // scratch memory for the fast path as well)
#pragma unroll 1
                for (int k = 0; k < 4; ++k) {
                    if (r + k * row_lanes >= r_end) break;
                    const uint4 q = bs_cols_vec_exact(cin[(r + k * row_lanes) * row_stride], cs, err);
                    if constexpr (WRITE) cout[(r + k * row_lanes) * row_stride] = q;
                }
            }
        };
#pragma unroll 1
        for (int64_t r = r_first; r < r_end; r += 2 * stride) {
            load_batch(vb, r + stride);
            asm volatile("" ::: "memory");         // (the loads stay ahead of the arithmetic they are meant to overlap)
            do_batch(va, r);
            load_batch(va, r + 2 * stride);
            asm volatile("" ::: "memory");
            do_batch(vb, r + stride);
        }
    }
    if constexpr (ERR) {
        err = wave_sum(err);
        __syncthreads();
        if (lane == 0) s_f[wave] = err;
        __syncthreads();
        if (threadIdx.x == 0) reinterpret_cast<float*>(ws)[WS_ERR + blockIdx.x] = (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]);
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
                                                 int cpr, int cpr_shift, int64_t nblocks, Finish fin, int phase, int npart1) {
    constexpr int NW = WGS / 64, LG = WGS == 256 ? 8 : WGS == 512 ? 9 : 10;       // waves; log2 of the workgroup size
    __shared__ float s_f[NW];
    __shared__ int s_i[NW];
    // sums and maxima over the waves' LDS slots (four waves: pairwise, the order the sums have always had)
    auto red_fsum = [&]() { if constexpr (NW == 4) return (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]); else return lds_sum<NW>(s_f); };
    auto red_fmax = [&]() { if constexpr (NW == 4) return fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3])); else return lds_fmax<NW>(s_f); };
    // phase 0: out of place (write and publish the partials); in place the input must survive until the decision:
    // phase 1 publishes the partials without writing, phase 2 evaluates the decision and writes if it was E4M3
    if (phase == 2) {
        __shared__ float s_d[2 * WAVES];
        __shared__ int s_di[WAVES];
        if (finish_decision<WGS>(fin, s_d, s_di) != 1) return;
    }
    // npart1 > 0: the strategies that take the tensor amax (ss_mode 1 and 4) after a pass that found it; the amax and
    // non-zero partials of that pass stand, this kernel then publishes error partials only
    const float gamax = npart1 > 0 ? reduce_partial_amax(ws, npart1, s_f) : 0.0f;
    __syncthreads();
    const bool write = phase != 1;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t row_stride = (uint32_t)(sh.cols >> 3);
    const int nch = (int)sh.brows * cpr;
    const bool nt = streams_out(sh.rows * sh.cols);
    const bool nt_in = phase != 1 && streams_last_read(sh.rows * sh.cols);          // (the decision pass of the in-place op is not the last read)
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
        const uint32_t bid = bands ? band_order(sh, (uint32_t)t) : (uint32_t)t;          // (fewer than 2^31 blocks)
        uint32_t by32, bx32;
        block_of(sh, bid, by32, bx32);
        const int64_t by = by32, bx = bx32;
        const int64_t base = by * sh.brows * row_stride + ((bx * sh.bcols) >> 3);
        uint4 v[NV];
        bool ok[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) ok[k] = FULL || (k * WGS + tid < nch);
        // every lane loads: a lane beyond the block reads the block's first chunk and drops it (a load under a
        // condition is waited for before the next one is issued: the registers of its two outcomes are merged behind it)
        load16_group(v, nt_in, [&](int k) { return in + base + (ok[k] ? off_k(k) + off_tid : 0u); });
        if constexpr (!FULL) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                v[k].x = ok[k] ? v[k].x : 0u; v[k].y = ok[k] ? v[k].y : 0u; v[k].z = ok[k] ? v[k].z : 0u; v[k].w = ok[k] ? v[k].w : 0u;
            }
        }
        // amax and the non-zero count.  Large blocks: on packed 16-bit magnitudes, the data staying packed in its
        // registers from pass to pass (NV = 8: 100 registers instead of 220).  Small blocks: float maxima, whose
        // unpacked magnitudes the quantize pass then uses again (measured faster for NV <= 2).
        constexpr bool PACKED = NV > 2;
        uint32_t amax_b, nnz2 = 0;
        uint32_t negz2 = NEGZERO_INIT;            // whether this lane holds a -0 (its sign must not reach the output)
        if constexpr (PACKED) {
            uint32_t amax2 = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                acc_amax_pk(amax2, v[k].x); acc_amax_pk(amax2, v[k].y); acc_amax_pk(amax2, v[k].z); acc_amax_pk(amax2, v[k].w);
                acc_nnz_pk(nnz2, v[k].x); acc_nnz_pk(nnz2, v[k].y); acc_nnz_pk(nnz2, v[k].z); acc_nnz_pk(nnz2, v[k].w);
                acc_negzero_pk(negz2, v[k].x); acc_negzero_pk(negz2, v[k].y); acc_negzero_pk(negz2, v[k].z); acc_negzero_pk(negz2, v[k].w);
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
                acc_negzero_pk(negz2, v[k].x); acc_negzero_pk(negz2, v[k].y); acc_negzero_pk(negz2, v[k].z); acc_negzero_pk(negz2, v[k].w);
            }
            nnz2 = (uint32_t)nnzf;
            amax_b = group_umax(amax_bits_of(amax2), 64);
        }
        const bool negz = saw_negzero(negz2);     // (rare) zeros leave as +0 (FQ:1133-1134): the lane clears its -0 first
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
        const Scale sc = make_scale(scaling_factor(gamax, amax, ss_mode));
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
                    if (negz) v[k] = drop_negzero_vec(v[k]);
                    uint4 q = bs_vec_fast<E8, false, true, false>(v[k], sc, err);
                    if constexpr (PACKED) opaque(q);
                    if (ok[k]) store16_rt(out + base + off_k(k) + off_tid, q, nt);
                }
            } else {
#pragma unroll
                for (int k = 0; k < NV; ++k) {
                    if constexpr (PACKED) opaque(v[k]);
                    if (negz) v[k] = drop_negzero_vec(v[k]);
                    uint4 q = bs_vec_fast<E8, true, true, false>(v[k], sc, err);
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
        if (npart1 == 0) {
            reinterpret_cast<int*>(ws)[WS_PNNZ + blockIdx.x] = n;
            reinterpret_cast<float*>(ws)[WS_PAMAX + blockIdx.x] = red_fmax();
        }
    }
}

// The same single pass for row blocks of 512 * NVW elements, NVW = 2, 4 or 8 (rows of 4096 elements: per-channel
// scaling of a weight matrix): a wave per block.  A lane holds NVW vectors of its row, the block's amax and non-zero
// count meet by DPP and two shuffles inside the wave, so a workgroup works on four rows at once without a barrier or an
// LDS exchange between them, every wave's loads in flight while the others quantize (one workgroup per row: 58 us for
// 16384 rows of 4096 elements from HBM, the plain quantization of the same rows 43).  Rows are dealt out to the waves in
// turn, so that the waves that run side by side work on neighbouring rows.  Phases and npart1 as in k_bs_fused.
// TILE: blocks of several rows (512 * NVW elements in rows of 8 << cpr_log, e.g. 32 x 64: the smallest block the
// reference's own launch geometry takes, FQ:2080-2094): chunk 64 k + lane of a block lies at row (64 k + lane) >> cpr_log
// of the block; blocks in row-major order, so the four waves of a workgroup hold four neighbours.
template <bool E8, int NVW, bool TILE>
__global__ __launch_bounds__(WG) void k_bs_fused_wave(const uint4* in, uint4* out, uint32_t* ws, Shape sh, int ss_mode,
                                                      int64_t nrows, Finish fin, int phase, int npart1, int cpr_log) {
    __shared__ float s_f[2 * WAVES];
    __shared__ int s_i[WAVES];
    if (phase == 2 && finish_decision(fin, s_f, s_i) != 1) return;
    const float gamax = npart1 > 0 ? reduce_partial_amax(ws, npart1, s_f) : 0.0f;
    __syncthreads();
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool write = phase != 1;
    const bool nt_out = streams_out(sh.rows * sh.cols), nt_in = phase != 1 && streams_last_read(sh.rows * sh.cols);       // (phase 1 is not the last read)
    constexpr int ROW = 64 * NVW;                                   // chunks of a block
    float gmax = 0.0f, err = 0.0f;
    int nnz_total = 0;
    const uint32_t row_stride = (uint32_t)(sh.cols >> 3);
    uint32_t off[NVW];                                              // where the lane's chunks lie in a block
#pragma unroll
    for (int k = 0; k < NVW; ++k) {
        const uint32_t j = (uint32_t)(64 * k + lane);
        off[k] = TILE ? (j >> cpr_log) * row_stride + (j & ((1u << cpr_log) - 1u)) : j;
    }
    // (Issuing a wave's next row before the arithmetic of the row it holds -- two register buffers in turn -- was measured
    // slower: 56.3 against 52.5 us for 16384 rows of 4096 elements, at 168 registers.)
    for (int64_t row = (int64_t)blockIdx.x * WAVES + wave; row < nrows; row += (int64_t)gridDim.x * WAVES) {
        int64_t base = row * ROW;                                  // (one-row blocks in whole rows lie one after the other)
        uint32_t by32 = 0, bx32 = 0;
        if constexpr (TILE) {
            block_of(sh, (uint32_t)row, by32, bx32);               // (fewer than 2^31 blocks)
            base = (int64_t)by32 * sh.brows * row_stride + (((int64_t)bx32 * sh.bcols) >> 3);
        }
        const uint4* bin = in + base;
        uint4* bout = out + base;
        uint4 v[NVW];
        load16_group(v, nt_in, [&](int k) { return bin + (TILE ? off[k] : (uint32_t)(64 * k + lane)); });
        uint32_t amax2 = 0, nnz2 = 0, negz2 = NEGZERO_INIT;
#pragma unroll
        for (int k = 0; k < NVW; ++k) {
            acc_amax_pk(amax2, v[k].x); acc_amax_pk(amax2, v[k].y); acc_amax_pk(amax2, v[k].z); acc_amax_pk(amax2, v[k].w);
            acc_nnz_pk(nnz2, v[k].x); acc_nnz_pk(nnz2, v[k].y); acc_nnz_pk(nnz2, v[k].z); acc_nnz_pk(nnz2, v[k].w);
            acc_negzero_pk(negz2, v[k].x); acc_negzero_pk(negz2, v[k].y); acc_negzero_pk(negz2, v[k].z); acc_negzero_pk(negz2, v[k].w);
            opaque(v[k]);
        }
        const bool negz = saw_negzero(negz2);     // (rare) zeros leave as +0 (FQ:1133-1134): the lane clears its -0 first
        const uint32_t amax_b = group_umax(amax_bits_of(amax2), 64);
        const bool has_nan = amax_b > 0x7F800000u;                  // uniform over the wave
        float amax = u2f(amax_b);
        int nnz_row = (int)((nnz2 & 0xFFFFu) + (nnz2 >> 16));
        if (has_nan) {                            // the float maximum and the count of the reference skip a NaN (rare)
            amax = 0.0f;
#pragma unroll
            for (int k = 0; k < NVW; ++k) {
                acc_amax(amax, v[k].x); acc_amax(amax, v[k].y); acc_amax(amax, v[k].z); acc_amax(amax, v[k].w);
                nnz_row -= nan_word(v[k].x) + nan_word(v[k].y) + nan_word(v[k].z) + nan_word(v[k].w);
            }
            amax = group_max(amax, 64);
        }
        gmax = fmaxf(gmax, amax);
        nnz_total += nnz_row;
        const Scale sc = make_scale(scaling_factor(gamax, amax, ss_mode));
        if (!has_nan && (sc.fast || !(amax > 0.0f))) {          // an all-zero block gives +0 whatever its (clamped) scale is
            if (phase == 1) {                      // decision pass of the in-place variant: error terms only
#pragma unroll
                for (int k = 0; k < NVW; ++k) { opaque(v[k]); bs_vec_fast<E8, true, false>(v[k], sc, err); asm volatile("" : "+v"(err)); }
            } else if (phase == 2) {               // write pass of the in-place variant: no error terms
#pragma unroll
                for (int k = 0; k < NVW; ++k) {
                    opaque(v[k]);
                    if (negz) v[k] = drop_negzero_vec(v[k]);
                    uint4 q = bs_vec_fast<E8, false, true, false>(v[k], sc, err);
                    opaque(q);
                    store16_rt(bout + (TILE ? off[k] : (uint32_t)(64 * k + lane)), q, nt_out);
                }
            } else {
#pragma unroll
                for (int k = 0; k < NVW; ++k) {
                    opaque(v[k]);
                    if (negz) v[k] = drop_negzero_vec(v[k]);
                    uint4 q = bs_vec_fast<E8, true, true, false>(v[k], sc, err);
                    opaque(q);
                    asm volatile("" : "+v"(err));
                    store16_rt(bout + (TILE ? off[k] : (uint32_t)(64 * k + lane)), q, nt_out);
                }
            }
        } else {
            // the exact arithmetic, from memory again (non-unrolled: no run-time index into the register array)
            const uint16_t* in16 = reinterpret_cast<const uint16_t*>(in) + base * 8;
            uint16_t* out16 = reinterpret_cast<uint16_t*>(out) + base * 8;
#pragma unroll 1
            for (int i = lane; i < ROW * 8; i += 64) {
                const int64_t e = TILE ? (int64_t)(i >> (cpr_log + 3)) * sh.cols + (i & ((8 << cpr_log) - 1)) : i;
                const float q = bs_element<E8, false>(bf16_one(in16[e]), sc, err);
                if (write) out16[e] = store_bf16<false>(q);
            }
        }
        }
    err = wave_sum(err);
    nnz_total = wave_sum_i(nnz_total);
    gmax = group_max(gmax, 64);
    __syncthreads();
    if (lane == 0) { s_f[wave] = err; s_f[4 + wave] = gmax; s_i[wave] = nnz_total; }
    __syncthreads();
    if (tid == 0 && phase != 2) {
        reinterpret_cast<float*>(ws)[WS_ERR + blockIdx.x] = (s_f[0] + s_f[1]) + (s_f[2] + s_f[3]);
        if (npart1 == 0) {
            reinterpret_cast<int*>(ws)[WS_PNNZ + blockIdx.x] = s_i[0] + s_i[1] + s_i[2] + s_i[3];
            reinterpret_cast<float*>(ws)[WS_PAMAX + blockIdx.x] = fmaxf(fmaxf(s_f[4], s_f[5]), fmaxf(s_f[6], s_f[7]));
        }
    }
}

// The same single pass for row blocks of 1 x 8G elements, G <= 64 lanes (MX 1 x 32 through the channel op is G = 4):
// the flat chunk array in tiles of 4 * 256 chunks, a block is G consecutive lanes (amax by DPP), as in k_rowgroup.
// Groups whose scale is outside the fast range are redone from memory by a second, non-unrolled loop.
constexpr int BS_ROWS_NV = 4;         // vectors per lane and tile (2 is not faster here: 55.9 against 54.5 us)
// GM: 0 = the scale depends on the block alone (ss_mode 2 / 3; this kernel also publishes the amax and non-zero partials),
// 1 = tensor-amax mantissa shared by the blocks (ss_mode 1), 2 = one scale for the tensor (ss_mode 4: G is 1 whatever
// the block shape is); for 1 and 2 a pass over the tensor has left its amax and non-zero partials (npart1 of them).
template <bool E8, int GM>
__global__ __launch_bounds__(WG) void k_bs_fused_rows(const uint4* in, uint4* out, uint32_t* ws, int64_t nchunks, int G, int ss_mode,
                                                      Finish fin, int phase, int npart1) {
    __shared__ float s_f[2 * WAVES];
    __shared__ int s_i[WAVES];
    if (phase == 2 && finish_decision(fin, s_f, s_i) != 1) return;          // phases as in k_bs_fused
    constexpr int NV = BS_ROWS_NV;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t ntiles = (nchunks + NV * WG - 1) / (NV * WG);
    auto load_tile = [&](uint4 (&v)[NV], int64_t tile) {
        const int64_t base = tile * (NV * WG) + tid;
        if (base + (NV - 1) * WG < nchunks) {
            load16_group(v, phase != 1 && streams_last_read(nchunks * 8), [&](int k) { return in + base + k * WG; });
        } else {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                v[k] = make_uint4(0, 0, 0, 0);
                if (base + k * WG < nchunks) v[k] = load16_rt(in + base + k * WG, phase != 1 && streams_last_read(nchunks * 8));
            }
        }
    };
    // One scale for the tensor: the first tile's loads go out before the partials of the pass that found the amax are
    // reduced (about 2 us that every workgroup spends before it knows the scale)
    uint4 v0[NV];
    if (GM == 2 && (int64_t)blockIdx.x < ntiles) load_tile(v0, blockIdx.x);
    uint32_t pflags = 0;
    const float gamax = GM != 0 ? reduce_partial_amax(ws, npart1, s_f, &pflags) : 0.0f;
    const bool special = (pflags & PART_SPECIAL) != 0;          // a NaN or a -0 somewhere in the tensor, as the pass that found its amax saw it
    __syncthreads();
    const Scale scu = make_scale(scaling_factor(gamax, 1.0f, 4));           // (GM == 2)
    const bool write = phase != 1;
    const bool nt = streams_out(nchunks * 8);
    float gmax = 0.0f, err = 0.0f;
    int nnz = 0;
    // ... in the fast range, and neither a NaN nor a -0 in the tensor: nothing to test per vector
    const bool plain = GM == 2 && !special && scu.fast;
    for (int64_t tile = blockIdx.x; plain && tile < ntiles; tile += gridDim.x) {
        const int64_t base = tile * (NV * WG) + tid;
        const bool whole = base + (NV - 1) * WG < nchunks;
        uint4 v[NV];
        if (tile == (int64_t)blockIdx.x) {
#pragma unroll
            for (int k = 0; k < NV; ++k) v[k] = v0[k];
        } else {
            load_tile(v, tile);
        }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int64_t c = base + k * WG;
            opaque(v[k]);
            uint4 q;
            if (phase == 1) q = bs_vec_fast<E8, true, false, false>(v[k], scu, err);
            else if (phase == 2) q = bs_vec_fast<E8, false, true, false>(v[k], scu, err);
            else q = bs_vec_fast<E8, true, true, false>(v[k], scu, err);
            opaque(q);
            asm volatile("" : "+v"(err));
            if (write && (whole || c < nchunks)) store16_rt(out + c, q, nt);
        }
    }
    for (int64_t tile = blockIdx.x; !plain && tile < ntiles; tile += gridDim.x) {
        const int64_t base = tile * (NV * WG) + tid;
        uint4 v[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            v[k] = make_uint4(0, 0, 0, 0);
            if (base + k * WG < nchunks) v[k] = load16_rt(in + base + k * WG, phase != 1 && streams_last_read(nchunks * 8));
        }
        uint32_t slow = 0, nnz2 = 0;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int64_t c = base + k * WG;
            // the block maximum on packed 16-bit magnitudes; a NaN wins it and sends the block to the exact arithmetic
            uint32_t amax2 = 0;
            acc_amax_pk(amax2, v[k].x); acc_amax_pk(amax2, v[k].y); acc_amax_pk(amax2, v[k].z); acc_amax_pk(amax2, v[k].w);
            if constexpr (GM == 0) { acc_nnz_pk(nnz2, v[k].x); acc_nnz_pk(nnz2, v[k].y); acc_nnz_pk(nnz2, v[k].z); acc_nnz_pk(nnz2, v[k].w); }
            const uint32_t amax_b = group_umax(amax_bits_of(amax2), G);
            const bool has_nan = amax_b > 0x7F800000u;
            const float amax = u2f(amax_b);
            if constexpr (GM == 0) { if (!has_nan) gmax = fmaxf(gmax, amax); }
            const Scale sc = GM == 2 ? scu : make_scale(scaling_factor(gamax, amax, ss_mode));
            float e = 0.0f;
            uint4 q;
            if (phase != 1 && vec_has_negzero(v[k])) v[k] = drop_negzero_vec(v[k]);       // (rare) zeros leave as +0 (FQ:1133-1134)
            if (phase == 1) q = bs_vec_fast<E8, true, false>(v[k], sc, e);          // in place: decision pass,
            else if (phase == 2) q = bs_vec_fast<E8, false, true, false>(v[k], sc, e);     // write pass
            else q = bs_vec_fast<E8, true, true, false>(v[k], sc, e);
            if (!has_nan && (sc.fast || !(amax > 0.0f))) {      // an all-zero block gives +0 whatever its (clamped) scale is
                err += e;
                if (c < nchunks && write) store16_rt(out + c, q, nt);
            } else if (c < nchunks) slow |= 1u << k;
        }
        nnz += (int)((nnz2 & 0xFFFFu) + (nnz2 >> 16));
        if (slow) {
#pragma unroll 1
            for (int k = 0; k < NV; ++k) {
                if (!((slow >> k) & 1u)) continue;              // uniform over the lanes of a group
                const int64_t c = base + k * WG;
                const uint4 x = in[c];
                float amax = 0.0f;                               // the float maximum skips a NaN, as the reference's does
                acc_amax(amax, x.x); acc_amax(amax, x.y); acc_amax(amax, x.z); acc_amax(amax, x.w);
                amax = group_max(amax, G);
                if constexpr (GM == 0) {
                    gmax = fmaxf(gmax, amax);
                    nnz -= nan_word(x.x) + nan_word(x.y) + nan_word(x.z) + nan_word(x.w);      // the packed count took them for non-zero values
                }
                const Scale sc = make_scale(scaling_factor(gamax, amax, ss_mode));
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
        if constexpr (GM == 0) {
            reinterpret_cast<int*>(ws)[WS_PNNZ + blockIdx.x] = n;
            reinterpret_cast<float*>(ws)[WS_PAMAX + blockIdx.x] = fmaxf(fmaxf(s_f[0], s_f[1]), fmaxf(s_f[2], s_f[3]));
        }
    }
}

// The end of the out-of-place ops (FQ:1178-1241): the decision, and the input copied over the quantized output when it
// is the bf16 fallback
__global__ __launch_bounds__(WG) void k_copy_if(const uint16_t* in, uint16_t* out, Finish fin, int64_t n, int64_t nvec) {
    __shared__ float s_f[2 * WAVES];
    __shared__ int s_i[WAVES];
    if (finish_decision(fin, s_f, s_i) != 3) return;
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

// The rounding of quant_e8m in closed form.  With h = the mantissa in bf16 steps, rounded up (the threshold tables look at
// nothing finer), the count of thresholds below the mantissa is h / S rounded to nearest, ties to even, S = 2^(7-MB); a
// carry out of the mantissa is the exponent's increment.  So on hb = (e << 7) + h, the value's bf16 bit pattern rounded
// up: (hb + S/2 - 1 + bit LS of hb) with the low LS bits cleared.  Holds for 0 < e < 255 and for zero; e = 0 gives 0 in
// the reference (the callers see to that), a result of e = 255 is the reference's clamp to the largest finite value.
//
// Scale 1 (no tensor-amax strategy): the input is bf16, so hb is its magnitude and the result is again a bf16 pattern --
// both halves of a packed word at once, no conversion to float.  Vectors with a NaN, an infinity (passed through by
// the reference, FQ:1243-1327) or a -0 (zeros leave as +0, FQ:1399-1419) take the element-wise code.
template <int MB> __device__ __forceinline__ uint32_t e8mx_pair_unit(uint32_t w) {
    constexpr int LS = 7 - MB;
    constexpr uint32_t S = 1u << LS, MAXF = (254u << 7) | (((1u << MB) - 1u) << LS);
    const uint32_t mag = w & 0x7FFF7FFFu;
    const uint32_t odd = (mag >> LS) & 0x00010001u;                       // (bits that cross from the upper half are masked off)
    uint32_t r = (mag + (S / 2 - 1) * 0x00010001u + odd) & ~((S - 1) * 0x00010001u);          // (no carry out of a half: 0x7F7F + 32)
    r = pk_min_u16(r, MAXF * 0x00010001u);
    const uint32_t normal = pk_min_u16(pk_lshr_u16(mag, 7), 0x00010001u);                       // 1 where the exponent field is not 0
    r = pk_mul_lo_u16(r, normal);                                           // denormals give 0 (the sign stays: FQ keeps it)
    return r | (w & 0x80008000u);
}
// whether a vector holds a value the packed form does not cover: a magnitude of 0x7F80 or more (infinity, NaN), a -0
__device__ __forceinline__ bool e8mx_vec_special(uint4 v) {
    uint32_t m = 0;
    acc_amax_pk(m, v.x); acc_amax_pk(m, v.y); acc_amax_pk(m, v.z); acc_amax_pk(m, v.w);
    return amax_bits_of(m) >= 0x7F800000u || vec_has_negzero(v);
}
// Tensor-amax strategy on a tensor the amax pass found plain (no NaN, no -0, no non-zero magnitude below 2^-94, amax below
// 2^96, Markstein's condition on the scale): |x| * sf, the closed form on its bits, the exact quotient by sf, half-up
// store; the sign bits are copied.  Nothing is tested per element.
template <int MB> __device__ __forceinline__ uint32_t e8mx_pair_plain(uint32_t w, float sf, float rs) {
    constexpr int LS = 7 - MB;
    constexpr uint32_t S = 1u << LS;
    const uint32_t b0 = f2u(fabsf(bf16_lo(w)) * sf), b1 = f2u(fabsf(bf16_hi(w)) * sf);
    const uint32_t h0 = (b0 + 0xFFFFu) >> 16, h1 = (b1 + 0xFFFFu) >> 16;
    const float d0 = u2f(((h0 + (S / 2 - 1) + ((h0 >> LS) & 1u)) & ~(S - 1)) << 16);
    const float d1 = u2f(((h1 + (S / 2 - 1) + ((h1 >> LS) & 1u)) & ~(S - 1)) << 16);
    return store_pair<false>(div_by_scale(d0, sf, rs), div_by_scale(d1, sf, rs)) | (w & 0x80008000u);
}

// FQ:1361-1428
template <int MB, bool EMU, bool UNIT>
__global__ __launch_bounds__(WG) void k_e8mx(const uint16_t* in, uint16_t* out, const uint32_t* ws, int npart, int strategy, int64_t n, int64_t nvec) {
    __shared__ float s_f[WAVES];
    uint32_t pflags = PART_SPECIAL | PART_TINY;
    const float gamax = (!UNIT && strategy == 1) ? reduce_partial_amax(ws, npart, s_f, &pflags) : 0.0f;
    const float sf = UNIT ? 1.0f : e8mx_scale<MB>(gamax, strategy);
    const float rs = 1.0f / sf;
    const bool mk = (f2u(sf) & 0x7FFFFFu) != 0x7FFFFFu;
    // (amax at least 2^-60: the scaled values of a tensor without tiny elements are then nowhere near the denormals either)
    const bool plain = !UNIT && !EMU && strategy == 1 && pflags == 0 && mk && gamax < 0x1p96f && gamax >= 0x1p-60f;
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
        for (int k = 0; k < NV; ++k) { v[k] = make_uint4(0, 0, 0, 0); if (c0 + k * WG < nvec) v[k] = load16_rt(in4 + c0 + k * WG, streams_last_read(n)); }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            uint32_t w[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
            if (UNIT && !EMU && !e8mx_vec_special(v[k])) {
#pragma unroll
                for (int j = 0; j < 4; ++j) w[j] = e8mx_pair_unit<MB>(w[j]);
            } else if (plain) {
#pragma unroll
                for (int j = 0; j < 4; ++j) w[j] = e8mx_pair_plain<MB>(w[j], sf, rs);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    w[j] = store_pair<EMU>(e8mx_element<MB, UNIT>(bf16_lo(w[j]), sf, rs, mk), e8mx_element<MB, UNIT>(bf16_hi(w[j]), sf, rs, mk));
            }
            if (c0 + k * WG < nvec) store16_rt(out4 + c0 + k * WG, make_uint4(w[0], w[1], w[2], w[3]), streams_out(n));
        }
    }
    for (int64_t i = nvec * 8 + gtid; i < n; i += stride) out[i] = store_bf16<EMU>(e8mx_element<MB, UNIT>(bf16_one(in[i]), sf, rs, mk));
}

}  // namespace mor

using namespace mor;

// 32-bit words of the workspace behind the header and the partial arrays: one float per block, or, for column blocks
// N x 1, the scales and the partial maxima of the column kernels where they take more
static int64_t block_words(int64_t rows, int64_t cols, int64_t brows, int64_t bcols) {
    int64_t words = cdiv(rows, brows) * cdiv(cols, bcols);
    if (bcols == 1 && brows > 1) words = std::max(words, col_words(rows, cols, brows));
    return words;
}

extern "C" size_t mor_workspace_bytes(int op, int64_t rows, int64_t cols, int64_t brows, int64_t bcols) {
    if (rows <= 0 || cols <= 0 || brows <= 0 || bcols <= 0) return 0;
    switch (op) {
        case MOR_OP_BLOCK_SCALING:
        case MOR_OP_CHANNEL_SCALING:
            return (size_t)(WS_BLOCKS + block_words(rows, cols, brows, bcols)) * 4;
        case MOR_OP_E8MX:
            return (size_t)WS_BLOCKS * 4;
        default:
            return 0;
    }
}

template <bool E8, bool EMU, bool COL>
static void launch_bs_quant(bool write, bool err, int grid, hipStream_t st, const uint16_t* in, uint16_t* out, uint32_t* ws,
                            const float* scales, const Finish& fin, int gate, int ss_mode, int npart1, const Shape& sh, int vec,
                            DivU32 d0, DivU32 d1, DivU32 d2, DivU32 d3) {
    if (write && err) k_bs_quant<E8, EMU, COL, true, true><<<grid, WG, 0, st>>>(in, out, ws, scales, fin, gate, ss_mode, npart1, sh, vec, d0, d1, d2, d3);
    else if (write) k_bs_quant<E8, EMU, COL, true, false><<<grid, WG, 0, st>>>(in, out, ws, scales, fin, gate, ss_mode, npart1, sh, vec, d0, d1, d2, d3);
    else k_bs_quant<E8, EMU, COL, false, true><<<grid, WG, 0, st>>>(in, out, ws, scales, fin, gate, ss_mode, npart1, sh, vec, d0, d1, d2, d3);
}

static void dispatch_bs_quant(bool e8, bool emu, bool col, bool write, bool err, int grid, hipStream_t st, const uint16_t* in,
                              uint16_t* out, uint32_t* ws, const float* scales, const Finish& fin, int gate, int ss_mode, int npart1,
                              const Shape& sh, int vec, DivU32 d0, DivU32 d1, DivU32 d2, DivU32 d3) {
#define BSQ(E8, EMU, COL) launch_bs_quant<E8, EMU, COL>(write, err, grid, st, in, out, ws, scales, fin, gate, ss_mode, npart1, sh, vec, d0, d1, d2, d3)
    if (e8) {
        if (emu) { if (col) BSQ(true, true, true); else BSQ(true, true, false); }
        else { if (col) BSQ(true, false, true); else BSQ(true, false, false); }
    } else {
        if (emu) { if (col) BSQ(false, true, true); else BSQ(false, true, false); }
        else { if (col) BSQ(false, false, true); else BSQ(false, false, false); }
    }
#undef BSQ
}

// Argument checks of the block / channel scaling entry points (FQ:2019-2020, 2437-2438, 2501).
static int block_scaling_check(const void* input, void* output, int32_t* meta, float* global_amax, int32_t* global_non_zero,
                               float* global_error, int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                               int64_t ss_mode, int channel) {
    if (int rc = mor_validate_shape(input, rows, cols, brows, bcols)) return rc;
    if (!output || !meta || !global_amax || !global_non_zero || !global_error) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output pointer is NULL");
    if (rows % brows != 0 || cols % bcols != 0)      // FQ:2019-2020, 2437-2438
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "block dims %lld x %lld do not divide the tensor %lld x %lld", (long long)brows, (long long)bcols, (long long)rows, (long long)cols);
    if (ss_mode < 1 || ss_mode > 4) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "ss_mode must be 1..4 (got %lld)", (long long)ss_mode);
    if (channel && brows != 1 && bcols != 1)         // FQ:2501
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "channel scaling needs block_rows == 1 or block_cols == 1");
    if (rows * cols >= (1ll << 34)) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "tensor too large");
    return MOR_OK;
}

static int block_scaling_run(const void* input, void* output, int32_t* meta,
                             float* global_amax, int32_t* global_non_zero, float* global_error,
                             int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                             double e4m3_threshold, int64_t ss_mode, void* workspace, uint32_t flags, void* stream);

extern "C" int mor_block_scaling(const void* input, void* output, int32_t* meta,
                                 float* global_amax, int32_t* global_non_zero, float* global_error,
                                 int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                                 double e4m3_threshold, int64_t ss_mode, int channel,
                                 void* workspace, size_t workspace_bytes, uint32_t flags, void* stream) {
    if (int rc = block_scaling_check(input, output, meta, global_amax, global_non_zero, global_error, rows, cols, brows, bcols, ss_mode, channel)) return rc;
    const size_t need = mor_workspace_bytes(MOR_OP_BLOCK_SCALING, rows, cols, brows, bcols);
    if (!workspace || workspace_bytes < need) return mor_fail(MOR_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    return block_scaling_run(input, output, meta, global_amax, global_non_zero, global_error, rows, cols, brows, bcols,
                             e4m3_threshold, ss_mode, workspace, flags, stream);
}

// The launches of mor_block_scaling; `workspace` holds at least mor_workspace_bytes(MOR_OP_BLOCK_SCALING, ...) bytes.
static int block_scaling_run(const void* input, void* output, int32_t* meta,
                             float* global_amax, int32_t* global_non_zero, float* global_error,
                             int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                             double e4m3_threshold, int64_t ss_mode, void* workspace, uint32_t flags, void* stream) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool emu = flags & MOR_FLAG_TORCH_EMULATION;
    const Shape sh = make_shape(rows, cols, brows, bcols);
    const int64_t nb = sh.gy * sh.gx;
    uint32_t* ws = static_cast<uint32_t*>(workspace);
    float* blocks = reinterpret_cast<float*>(ws + WS_BLOCKS);
    const uint16_t* in16 = static_cast<const uint16_t*>(input);
    uint16_t* out16 = static_cast<uint16_t*>(output);
    const bool inplace = (input == output);
    const int vec = (aligned16(input) && aligned16(output) && cols % 8 == 0) ? 1 : 0;
    const bool col = (bcols == 1 && brows > 1);

    // The launches: pass 1 (amax / non-zero partials, block amax), pass 2 (quantize, error partials), and the end of the
    // op in the workgroups of the kernel that acts on the decision (out of place: the gated copy; in place: the gated
    // write).  The grids of pass 1 and pass 2 are capped (PASS1_MAX / PASS2_MAX workgroups, grid-stride): every
    // workgroup of the following kernel reduces their partials again.
    Finish fin{ws, 0, 0, (float)e4m3_threshold, meta, global_amax, global_non_zero, global_error};
    const int64_t n = rows * cols;
    const int64_t nvec_all = vec ? n / 8 : 0;
    auto gated_copy = [&]() { k_copy_if<<<grid_for(nvec_all > 0 ? nvec_all : n, 4), WG, 0, st>>>(in16, out16, fin, n, nvec_all); };

    // block-local scales: one pass out of place; in place one pass for the decision and one gated pass that writes
    const int64_t blk_chunks = (bcols % 8 == 0) ? brows * (bcols / 8) : 0;
    // (a decision pass that computes no output words and a write pass that computes no error terms; 128 x 128 blocks
    // in place at 8192^2: 83 us against 99 through the general three-pass path; blocks that fill less than a workgroup
    // take the general path)
    // The strategies that take the tensor amax (ss_mode 1 and 4) run the same kernels after a pass over the flat tensor
    // that finds it: the blocks' own maxima come from the registers of the quantize pass, no per-block array is kept.
    // ss_mode 4 needs no block maxima at all and takes the flat row kernel whatever the block shape is.
    const bool global = (ss_mode == 1 || ss_mode == 4);
    int npart1 = 0;
    auto tensor_amax_pass = [&]() {
        npart1 = (int)std::min<int64_t>(cdiv(n / 8, 8 * WG), 512);
        k_bs_amax_flat<<<npart1, WG, 0, st>>>(static_cast<const uint4*>(input), ws, nullptr, n / 8, 1, 0);
    };
    const bool flat_ok = !emu && vec && n % 8 == 0;
    const bool wave_rows = brows == 1 && cols % bcols == 0;
    // (rows of a block of at least 128 bytes: with 64-byte pieces a load instruction touches 16 rows and the kernel is no
    // faster than the two-read path, 76 us for 32 x 32 blocks at 8192^2)
    const bool wave_tiles = brows > 1 && rows % brows == 0 && cols % bcols == 0 && is_pow2(bcols / 8) && bcols / 8 >= 8 && bcols / 8 <= 64 && nb < ((int64_t)1 << 31);
    if (flat_ok && (wave_rows || wave_tiles) && ss_mode != 4 && (blk_chunks == 128 || blk_chunks == 256 || blk_chunks == 512)) {
        // row blocks of 1024, 2048 or 4096 elements, tiles of as many elements in rows of up to 512: a wave per block
        if (global) tensor_amax_pass();
        // (four workgroups per CU: 16384 rows of 4096 elements from HBM take 52.6 us with 1024 workgroups, 55.7 with 768,
        // 55.1 with 1536, 54.9 with 2048, 53.4 with 4096)
        const int grid = (int)std::min<int64_t>(cdiv(nb, WAVES), 1024);
        fin.nerr = grid;
        fin.nstat = global ? npart1 : grid;
        const uint4* i4 = static_cast<const uint4*>(input);
        uint4* o4 = static_cast<uint4*>(output);
        const int nvw = (int)(blk_chunks / 64);
        for (int phase = inplace ? 1 : 0; phase <= (inplace ? 2 : 0); ++phase) {
        const int cpr_log = wave_tiles ? ilog2(bcols / 8) : 0;
#define MOR_BS_WAVE(E8, NVW) do { \
            if (wave_tiles) k_bs_fused_wave<E8, NVW, true><<<grid, WG, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, nb, fin, phase, npart1, cpr_log); \
            else k_bs_fused_wave<E8, NVW, false><<<grid, WG, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, nb, fin, phase, npart1, cpr_log); } while (0)
            if (ss_mode == 2) { if (nvw == 2) MOR_BS_WAVE(true, 2); else if (nvw == 4) MOR_BS_WAVE(true, 4); else MOR_BS_WAVE(true, 8); }
            else { if (nvw == 2) MOR_BS_WAVE(false, 2); else if (nvw == 4) MOR_BS_WAVE(false, 4); else MOR_BS_WAVE(false, 8); }
#undef MOR_BS_WAVE
        }
        if (!inplace) gated_copy();
        return mor_check_launch("mor_block_scaling (single pass, a wave per row block)");
    }
    if (flat_ok && !col && ss_mode != 4 && blk_chunks >= WG && blk_chunks <= 8 * 1024
        && brows * (cols / 8) < 0x7FFFFFFFll && (is_pow2(bcols / 8) || brows == 1)) {
        if (global) tensor_amax_pass();
        const int cpr = (int)(bcols / 8);
        const int nv = (int)cdiv(blk_chunks, WG);
        const int NVc = nv <= 1 ? 1 : nv <= 2 ? 2 : nv <= 4 ? 4 : 8;
        // up to 8 * 256 chunks: 256 threads; up to 32768 / 65536 elements: 8 vectors per lane of 512 / 1024 threads
        const int wgs = blk_chunks <= 8 * WG ? WG : blk_chunks <= 8 * 512 ? 512 : 1024;
        const bool full = blk_chunks == (int64_t)(wgs == WG ? NVc : 8) * wgs;
        int grid = (int)std::min<int64_t>(nb, PASS2_MAX);      // partials: one per workgroup
        // tensors that come from HBM: XCD bands of block columns (16384 x 14336, 128 x 128 blocks: 193 -> 185 us)
        const bool bands = rows * cols >= ((int64_t)16 << 20) && sh.gx % 8 == 0 && nb % 8 == 0;
        if (bands) grid &= ~7;
        fin.nerr = grid;
        fin.nstat = global ? npart1 : grid;
        // a one-row block is contiguous whatever its width: chunk k * 256 + tid is at that offset (shift 20: row 0 always)
        const int shift = (brows == 1 ? 20 : ilog2(cpr)) | (bands ? 256 : 0);
        const uint4* i4 = static_cast<const uint4*>(input);
        uint4* o4 = static_cast<uint4*>(output);
#define MOR_BS_FUSED(E8, NV, PHASE) do { \
        if (full) k_bs_fused<E8, NV, true><<<grid, WG, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, cpr, shift, nb, fin, PHASE, npart1); \
        else k_bs_fused<E8, NV, false><<<grid, WG, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, cpr, shift, nb, fin, PHASE, npart1); } while (0)
#define MOR_BS_FUSED_W(E8, WGS_, PHASE) do { \
        if (full) k_bs_fused<E8, 8, true, WGS_><<<grid, WGS_, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, cpr, shift, nb, fin, PHASE, npart1); \
        else k_bs_fused<E8, 8, false, WGS_><<<grid, WGS_, 0, st>>>(i4, o4, ws, sh, (int)ss_mode, cpr, shift, nb, fin, PHASE, npart1); } while (0)
#define MOR_BS_FUSED_ALL(PHASE) do { \
        if (wgs == 512) { if (ss_mode == 2) MOR_BS_FUSED_W(true, 512, PHASE); else MOR_BS_FUSED_W(false, 512, PHASE); } \
        else if (wgs == 1024) { if (ss_mode == 2) MOR_BS_FUSED_W(true, 1024, PHASE); else MOR_BS_FUSED_W(false, 1024, PHASE); } \
        else if (ss_mode == 2) { switch (NVc) { case 1: MOR_BS_FUSED(true, 1, PHASE); break; case 2: MOR_BS_FUSED(true, 2, PHASE); break; case 4: MOR_BS_FUSED(true, 4, PHASE); break; default: MOR_BS_FUSED(true, 8, PHASE); break; } } \
        else { switch (NVc) { case 1: MOR_BS_FUSED(false, 1, PHASE); break; case 2: MOR_BS_FUSED(false, 2, PHASE); break; case 4: MOR_BS_FUSED(false, 4, PHASE); break; default: MOR_BS_FUSED(false, 8, PHASE); break; } } } while (0)
        MOR_BS_FUSED_ALL(inplace ? 1 : 0);
        if (inplace) MOR_BS_FUSED_ALL(2);
        else gated_copy();
#undef MOR_BS_FUSED_ALL
#undef MOR_BS_FUSED_W
#undef MOR_BS_FUSED
        return mor_check_launch("mor_block_scaling (single pass)");
    }

    if (flat_ok && (ss_mode == 4 || (!col && brows == 1 && bcols % 8 == 0 && is_pow2(bcols / 8) && bcols / 8 <= 64))) {
        if (global) tensor_amax_pass();
        const int64_t nchunks = rows * cols / 8;
        // (after a tensor-amax pass every workgroup starts by reducing that pass's partials, and the last kernel reduces this
        // one's: 512 and 1024 of them instead of 1024 and 2048 take 1 us off the three launches at 4096^2, 2 us at 8192^2)
        const int grid = (int)std::min<int64_t>(cdiv(nchunks, BS_ROWS_NV * WG), global ? 1024 : PASS2_MAX);
        fin.nerr = grid;
        fin.nstat = global ? npart1 : grid;
        const uint4* i4 = static_cast<const uint4*>(input);
        uint4* o4 = static_cast<uint4*>(output);
        const int G = ss_mode == 4 ? 1 : (int)(bcols / 8);
        for (int phase = inplace ? 1 : 0; phase <= (inplace ? 2 : 0); ++phase) {
            if (ss_mode == 2) k_bs_fused_rows<true, 0><<<grid, WG, 0, st>>>(i4, o4, ws, nchunks, G, (int)ss_mode, fin, phase, npart1);
            else if (ss_mode == 3) k_bs_fused_rows<false, 0><<<grid, WG, 0, st>>>(i4, o4, ws, nchunks, G, (int)ss_mode, fin, phase, npart1);
            else if (ss_mode == 1) k_bs_fused_rows<false, 1><<<grid, WG, 0, st>>>(i4, o4, ws, nchunks, G, (int)ss_mode, fin, phase, npart1);
            else k_bs_fused_rows<false, 2><<<grid, WG, 0, st>>>(i4, o4, ws, nchunks, G, (int)ss_mode, fin, phase, npart1);
        }
        if (!inplace) gated_copy();
        return mor_check_launch("mor_block_scaling (single pass, row blocks)");
    }

    // pass 1: per-block amax (not for ss_mode 4, which only takes the tensor amax), per-workgroup partials of the tensor
    // amax and the non-zero count
    const int64_t G = bcols / 8;
    int npart;
    // column blocks with aligned rows, default flavour, fp32 scale: k_bs_colmax / k_bs_quant_col (16-byte accesses to the
    // partial maxima in the workspace)
    ColPlan cp;
    const bool col_fast = col && vec && !emu && ss_mode != 2 && aligned16(blocks) && col_plan(rows, cols, brows, cp);
    float2* col_scales = reinterpret_cast<float2*>(blocks);                                   // [block row][column]
    uint16_t* col_partial = reinterpret_cast<uint16_t*>(blocks + sh.gy * cols * 2);           // [block row][segment][column]
    if (ss_mode == 4 && !col && vec && n % 8 == 0) {
        npart = (int)std::min<int64_t>(cdiv(n / 8, 8 * WG), PASS1_MAX);
        k_bs_amax_flat<<<npart, WG, 0, st>>>(static_cast<const uint4*>(input), ws, nullptr, n / 8, 1, 0);
    } else if (col_fast) {
        // column blocks, the fast path: rows of partial maxima (no atomics, nothing to clear), folded into the columns' scales
        npart = (int)std::min<int64_t>(cp.items1, PASS1_MAX);
        const uint4* i4 = static_cast<const uint4*>(input);
        switch (cp.ng) {
#define MOR_COLMAX(NG) case NG: k_bs_colmax<NG><<<npart, WG, 0, st>>>(i4, ws, col_partial, sh, cp); break
            MOR_COLMAX(1); MOR_COLMAX(2); MOR_COLMAX(3); MOR_COLMAX(4); MOR_COLMAX(5); MOR_COLMAX(6); MOR_COLMAX(7); MOR_COLMAX(8);
#undef MOR_COLMAX
        }
        k_bs_colfold<<<(unsigned)(sh.gy * cdiv(cols / 8, FOLD_G)), WG, 0, st>>>(col_partial, col_scales, ws, npart, (int)ss_mode, sh, cp);
    } else if (col) {
        k_zero_f32<<<grid_for(nb), WG, 0, st>>>(blocks, nb);
        const int rows_per_wg = (int)std::min<int64_t>(brows, 256);
        const unsigned gx = (unsigned)std::min<int64_t>(cdiv(cols, 256), PASS1_MAX);
        const int64_t segs = sh.gy * cdiv(brows, rows_per_wg);
        const unsigned gy = (unsigned)std::min<int64_t>(segs, std::max<int64_t>(PASS1_MAX / gx, 1));
        npart = (int)(gx * gy);
        k_bs_amax_col<<<dim3(gx, gy), WG, 0, st>>>(in16, ws, blocks, sh, rows_per_wg, vec);
    } else if (vec && brows == 1 && bcols % 8 == 0 && is_pow2(G) && G <= 64) {
        const int64_t nchunks = rows * cols / 8;
        npart = (int)std::min<int64_t>(cdiv(nchunks, 8 * WG), PASS1_MAX);
        k_bs_amax_flat<<<npart, WG, 0, st>>>(static_cast<const uint4*>(input), ws, blocks, nchunks, (int)G, ilog2(G));
    } else if (vec && bcols % 8 == 0 && brows * (bcols / 8) < WG && brows * (cols / 8) < 0x7FFFFFFFll) {
        const int nchb = (int)(brows * (bcols / 8));
        int logL = 0;
        while ((4 << logL) < nchb && logL < 6) ++logL;               // about four vectors per lane
        const int groups = WG >> logL;
        npart = (int)std::min<int64_t>(cdiv(nb, groups), PASS1_MAX);
        k_bs_amax_sub<<<npart, WG, 0, st>>>(static_cast<const uint4*>(input), ws, blocks, sh, 1 << logL, logL, make_div((uint32_t)sh.gx),
                                            make_div((uint32_t)(bcols / 8)));
    } else {
        const int v1 = (vec && bcols % 8 == 0 && brows * (cols / 8) < 0x7FFFFFFFll) ? 1 : 0;
        npart = (int)std::min<int64_t>(nb, PASS1_MAX);
        k_bs_amax_block<<<npart, WG, 0, st>>>(in16, ws, blocks, sh, v1, make_div((uint32_t)sh.gx),
                                              make_div((uint32_t)std::max<int64_t>(bcols / 8, 1)));
    }
    fin.nstat = npart;
    // pass 2: quantize (out of place: write now; in place: error only), error partials; every workgroup first reduces
    // the pass-1 partials to the tensor amax and computes its blocks' scales from it
    // end: bf16 fallback (out of place: copy if meta == 3) or the quantized write (in place: only if meta == 1)
    const bool e8 = (ss_mode == 2);
    if (col_fast) {
        const int grid = (int)std::min<int64_t>(cp.items2, PASS2_MAX);
        fin.nerr = grid;
        const uint4* i4 = static_cast<const uint4*>(input);
        uint4* o4 = static_cast<uint4*>(output);
        if (inplace) k_bs_quant_col<false, true><<<grid, WG, 0, st>>>(i4, o4, ws, col_scales, fin, 0, sh, cp);
        else k_bs_quant_col<true, true><<<grid, WG, 0, st>>>(i4, o4, ws, col_scales, fin, 0, sh, cp);
        if (inplace) k_bs_quant_col<true, false><<<grid, WG, 0, st>>>(i4, o4, ws, col_scales, fin, 1, sh, cp);
    } else {
        const bool vec2 = vec && (col || bcols % 8 == 0) && n / 8 < 0xFFFFFFFFll;
        const int64_t work = vec2 ? n / 8 : n;
        const int grid2 = (int)std::min<int64_t>(std::max<int64_t>(cdiv(work, WG), 1), PASS2_MAX);
        fin.nerr = grid2;
        DivU32 d0 = make_div((uint32_t)std::max<int64_t>(cols / 8, 1)), d1 = make_div((uint32_t)brows),
               d2 = make_div((uint32_t)std::max<int64_t>(bcols / 8, 1)), d3 = make_div((uint32_t)bcols);
        dispatch_bs_quant(e8, emu, col, !inplace, true, grid2, st, in16, out16, ws, blocks, fin, 0, (int)ss_mode, npart, sh, vec2 ? 1 : 0, d0, d1, d2, d3);
        if (inplace) dispatch_bs_quant(e8, emu, col, true, false, grid2, st, in16, out16, ws, blocks, fin, 1, (int)ss_mode, npart, sh, vec2 ? 1 : 0, d0, d1, d2, d3);
    }
    if (!inplace) gated_copy();
    return mor_check_launch("mor_block_scaling");
}

// ------------------------------------------------------------------------------------------------
// mor_block_scaling_static: the same op for callers that cannot allocate (and so cannot bring a workspace).  The
// workspace is this file-scope device array, one copy per GPU, held until the process ends: the header, the three
// partial arrays and one float for each of up to MOR_STATIC_MAX_BLOCKS blocks.  Calls on one GPU share it, so calls that
// overlap on one GPU race; every word a call reads was written by a kernel of that call (the general path clears the
// per-column maxima with a fill kernel), so stale contents of an earlier call are never read.
constexpr size_t STATIC_SCRATCH_WORDS = (size_t)WS_BLOCKS + (size_t)MOR_STATIC_MAX_BLOCKS;
static __device__ __align__(256) uint32_t scratch[STATIC_SCRATCH_WORDS];

// The device address of `scratch` on the current GPU.  In host code the array's name is only a handle: the address a
// kernel can use comes from hipGetSymbolAddress, once per device with that device current, and is kept per device.
constexpr int STATIC_MAX_DEVICES = 64;
static std::atomic<void*> g_scratch_ptr[STATIC_MAX_DEVICES];
static int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return mor_fail(MOR_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "device %d out of range", dev);
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return mor_fail(MOR_ERR_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
        g_scratch_ptr[dev].store(p, std::memory_order_release);      // (two threads racing here store the same address)
    }
    *out = p;
    return MOR_OK;
}

extern "C" int mor_block_scaling_static(const void* input, void* output, int32_t* meta,
                                        float* global_amax, int32_t* global_non_zero, float* global_error,
                                        int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                                        double e4m3_threshold, int64_t ss_mode, int channel,
                                        uint32_t flags, void* stream) {
    if (int rc = block_scaling_check(input, output, meta, global_amax, global_non_zero, global_error, rows, cols, brows, bcols, ss_mode, channel)) return rc;
    const int64_t nb = (rows / brows) * (cols / bcols);
    if (nb > (int64_t)MOR_STATIC_MAX_BLOCKS || block_words(rows, cols, brows, bcols) > (int64_t)MOR_STATIC_MAX_BLOCKS)
        return mor_fail(MOR_ERR_WORKSPACE, "mor_block_scaling_static takes at most %lld blocks (got %lld; column blocks take up to 32 "
                        "workspace words each): use mor_block_scaling with a workspace", (long long)MOR_STATIC_MAX_BLOCKS, (long long)nb);
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return block_scaling_run(input, output, meta, global_amax, global_non_zero, global_error, rows, cols, brows, bcols,
                             e4m3_threshold, ss_mode, ws, flags, stream);
}

extern "C" int mor_e8mx(const void* input, void* output, int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                        int64_t quantize_type, int64_t scaling_strategy, void* workspace, size_t workspace_bytes,
                        uint32_t flags, void* stream) {
    if (int rc = mor_validate_shape(input, rows, cols, brows, bcols)) return rc;
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
