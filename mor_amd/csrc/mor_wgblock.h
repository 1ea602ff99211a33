// k_wgblock: one workgroup per quantization block held in registers (the kernel template; its launchers are in
// mor_wgblock.hip).  "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.
#pragma once

#include "mor_quant.h"
#include "mor_wirefmt.h"

namespace mor {

// k_wgblock: one workgroup per quantization block, the block held in registers (NV 16-byte vectors per lane).
// Chunk ch = k * 256 + tid of the block sits at block row ch / cpr, chunk column ch % cpr.
// MOR: per-block format selection (FQ:610-682), else one forced format.  FULL: every block is complete and has
// exactly NV * 256 chunks, so no predicates.  NT: streaming loads and stores.  Blocks outside the fast range go
// through generic_block.  WGS threads per workgroup: 256, or 512 for one-row blocks of more than 8192 elements.
// GATHER: the block's elements are read and written pair by pair (odd column counts, pointers or block widths that are
// not multiples of 16 bytes): a lane's words are pairs of neighbouring elements of a row; every later step is
// elementwise, so nothing else changes.
// DUAL (whole 128 x 128 tiles, 256 threads): the quantized tile is also written transposed, to out_t [cols, rows]
// (with its meta entry at meta_t [cols / 128, rows / 128]): every result vector goes to LDS as well as to `out`, and
// the tile is read back from LDS column by column.  LDS layout: row r of the tile is 64 words (two columns each) at
// r * 64, and the word of columns (2w, 2w + 1) sits at position w ^ ((r >> 3) << 1) of its row.  A vector of 8 columns
// stays one aligned group of 4 words (in another order), so the writes are 16-byte writes; the 16 lanes that store one
// transposed row read, for rows 8j .. 8j + 7 (j = 0 .. 15) of one column, words in 16 different banks, and the four
// columns a wave handles at a time fill the other 16.
template <class V> __device__ __forceinline__ void dual_tile_put(uint32_t* s_t, int r, int cc, V q) {
    const int R = r >> 3;
    const uint4 p = (R & 1) ? make_uint4(q.z, q.w, q.x, q.y) : make_uint4(q.x, q.y, q.z, q.w);
    *reinterpret_cast<uint4*>(s_t + r * 64 + ((cc ^ (R >> 1)) << 2)) = p;
}
// WIRE (whole 128 x 128 tiles, 256 threads, fp32 scale; MoR or a forced format): instead of the fake-quantized bf16 tile the kernel writes
// the tile's codes: `out` is the payload, MOR_TILE_PAYLOAD_BYTES (32768) per tile, tile after tile in block order, rows
// packed (128 rows of 128 one-byte codes, of 96 bytes of 6-bit codes, or of 256 bytes of bf16); `meta` takes the
// storage format of each tile and `stats` one float per tile, its scale.  A tile whose scale is outside the fast range
// (or that holds a NaN) is stored as the bf16 image of its fake-quantized values, its format ORed with TILE_STORED_BF16.
constexpr int TILE_PAYLOAD_BYTES = 32768;
constexpr int TILE_STORED_BF16 = 0x100;
// The work of one workgroup on block `bid` (k_wgblock below is its kernel; the batch entry runs it on the blocks of
// several tensors in one launch).  cpr_shift: log2 of the chunk count per block row, negative when that is not a power
// of two.
template <bool MOR, bool E8, int NV, bool FULL, int NT, int WGS = WG, bool GATHER = false, bool DUAL = false, bool WIRE = false>
__device__ __forceinline__ void wgblock_body(const uint4* in, uint4* out, int32_t* __restrict__ meta, float* __restrict__ stats,
                                             const Shape& sh, const QuantArgs& qa, int cpr, int cpr_shift, uint32_t bid,
                                             uint4* out_t, int32_t* __restrict__ meta_t) {
    static_assert(!DUAL || (FULL && NV == 8 && WGS == 256 && !GATHER), "DUAL: whole 128 x 128 tiles");
    static_assert(!WIRE || (!E8 && FULL && NV == 8 && WGS == 256 && !GATHER && !DUAL), "WIRE: whole 128 x 128 tiles, fp32 scale");
    constexpr int NW = WGS / 64;
    __shared__ __attribute__((aligned(16))) uint32_t s_t[DUAL ? 128 * 64 : 4];
    __shared__ float s_f[2][NW];
    __shared__ uint32_t s_u[NW];
    __shared__ float s_e[2][NW];           // the error sums have slots of their own: no barrier between pass 1's readers and pass 2's writers
    __shared__ uint16_t s_q[128];          // pass 3, fp32 scale: the dequantized bf16 value of every 7-bit magnitude code
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t by32, bx32;
    block_of(sh, bid, by32, bx32);
    const int64_t by = by32, bx = bx32;
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
    // the store of one result vector (GATHER: pair by pair along the same walk, which `put` is called in order of;
    // DUAL: to `out` and to the LDS copy of the tile that out_t is written from -- both, unless the transposed tile
    // decided on another format, see below)
    int g_r = tid / g_pr, g_cp = tid - g_r * g_pr;
    bool to_out = true, to_lds = true;
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
        } else if constexpr (DUAL) {
            if (to_out) store16<(NT != 0)>(bout + off[k], q);
            if (to_lds) dual_tile_put(s_t, (k * WGS + tid) >> 4, tid & 15, q);
        } else {
            store16<(NT != 0)>(bout + off[k], q);
        }
    };
    // DUAL: the tile in LDS -> out_t, a lane per 8 consecutive rows of one column; the tile's entry of meta_t
    auto write_transposed = [&](int meta_val) {
        if constexpr (DUAL) {
            __syncthreads();
            const uint16_t* s16 = reinterpret_cast<const uint16_t*>(s_t);
            const uint32_t row_stride_t = (uint32_t)(sh.rows >> 3);
            uint4* tb = out_t + (c0 * row_stride_t + (r0 >> 3));
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int ch = k * WGS + tid, c = ch >> 4, j = ch & 15;
                uint32_t w[4];
                const int at = 2 * ((c >> 1) ^ (j << 1)) + (c & 1);            // (rows 8j .. 8j + 7: the same position in each)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t lo = s16[(8 * j + 2 * i) * 128 + at], hi = s16[(8 * j + 2 * i + 1) * 128 + at];
                    w[i] = lo | (hi << 16);
                }
                store16<(NT != 0)>(tb + (int64_t)c * row_stride_t + j, make_uint4(w[0], w[1], w[2], w[3]));
            }
            if (tid == 0 && meta_t && meta_val >= 0) meta_t[bx * sh.gy + by] = meta_val;
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
    // (57344 / amax is 128 * (448 / amax) exactly: one division for both)
    const Scale s4 = make_scale(448.0f / amax);
    Scale s5 = s4;
    s5.s = s4.s * 128.0f;
    s5.e8 = s4.e8 + 7;
    // (a NaN in the block shows as amax_b above the bits of infinity: the exact path takes its maximum as the reference does)
    if (amax_b > 0x7F800000u || (amax > 0.0f && !(s4.e8 >= -90 && s4.e8 <= 90 && s4.fast))) {           // uniform over the workgroup
        if constexpr (WIRE) {
            // the exact path's decision and values; the tile is stored as their bf16 image
            generic_block<false, false, WGS, MOR>(reinterpret_cast<const uint16_t*>(in), nullptr, meta, nullptr, sh, qa, E8, bid, s_f, s_u, false,
                                             reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(out) + (int64_t)bid * TILE_PAYLOAD_BYTES));
            if (tid == 0) { meta[bid] |= TILE_STORED_BF16; stats[bid] = 1.0f; }      // (thread 0 wrote the decision there)
            return;
        }
        generic_block<false, false, WGS, MOR>(reinterpret_cast<const uint16_t*>(in), reinterpret_cast<uint16_t*>(out), meta, stats,
                                  sh, qa, E8, bid, s_f, s_u);
        if constexpr (DUAL) {
            // the tile as generic_block has just written it (this workgroup's own stores), through LDS to out_t
            __syncthreads();
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                dual_tile_put(s_t, (k * WGS + tid) >> 4, tid & 15, bout[off[k]]);
            }
            int mv = qa.meta_val;
            if constexpr (MOR) mv = meta[bid];                        // (thread 0 wrote it before the barrier above)
            write_transposed(mv);
        }
        return;
    }

    int fmt = qa.fmt;
    int meta_val = qa.meta_val;
    int qt_t = Q_UNKNOWN;                  // DUAL: the decision of the transposed tile where it has sums of its own
    float e4 = 0.0f, e5 = 0.0f;
    // The error pass converts every pair to its E4M3 and its E5M2 codes; pass 3 looks the winner's codes up again instead
    // of multiplying and converting a second time (a register per pair: whole blocks of up to 8 vectors per lane).
    // (256 threads only: with 512 threads the 132 registers this takes leave one workgroup per CU, 128 x 256 tiles 48 -> 57 us)
    constexpr bool KEEP = MOR && !E8 && FULL && NV <= 8 && WGS == 256 && !GATHER && !WIRE;
    uint32_t kc[KEEP ? NV : 1][4];
    bool have_codes = false;
    if constexpr (MOR) {
        int qt = mor_decide_range(amax, amin, qa.clamp, qa.dyn_range);
        if (qt == Q_UNKNOWN) {
            // pass 2 (registers): the two error sums, FQ:487-584.  amax > 0 here.
            uint32_t codes = 0;
#pragma unroll
            for (int k = 0; k < NV; ++k)
                if (ok[k]) {
                    if constexpr (KEEP) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) asm volatile("" : "=v"(kc[k][j]));          // (any register: the converts write both halves)
                        err_pair_fast<E8>(v[k].x, s4, e4, e5, kc[k][0]);
                        err_pair_fast<E8>(v[k].y, s4, e4, e5, kc[k][1]);
                        err_pair_fast<E8>(v[k].z, s4, e4, e5, kc[k][2]);
                        err_pair_fast<E8>(v[k].w, s4, e4, e5, kc[k][3]);
                    } else {
                        err_pair_fast<E8>(v[k].x, s4, e4, e5, codes);
                        err_pair_fast<E8>(v[k].y, s4, e4, e5, codes);
                        err_pair_fast<E8>(v[k].z, s4, e4, e5, codes);
                        err_pair_fast<E8>(v[k].w, s4, e4, e5, codes);
                    }
                }
            have_codes = KEEP;
#pragma unroll
            for (int k = 0; k < NV; ++k) if (ok[k]) opaque(v[k]);
            e4 = wave_sum(e4);
            e5 = wave_sum(e5);
            if (lane == 0) { s_e[0][wave] = e4; s_e[1][wave] = e5; }
            __syncthreads();
            e4 = lds_sum<NW>(s_e[0]);
            e5 = lds_sum<NW>(s_e[1]);
            if (qa.ref_sums || !(fabsf(e4 - e5) > 1e-5f * fmaxf(e4, e5))) {
                // The sums above use reciprocals and this kernel's own order of additions.  When they are too close for
                // that to be trusted with the decision (or the caller asks for it), they are replaced by the reference's:
                // its divisions, its order of additions (from memory, non-unrolled: this is rare).  A tile and its
                // transpose hold the same terms, but the reference adds them in another order on the transposed
                // tensor: there the transposed tile gets sums, and a decision, of its own.
                const uint16_t* b16 = reinterpret_cast<const uint16_t*>(in) + (r0 * sh.cols + c0);
                const int bh = (int)min(sh.brows, sh.rows - r0), bw = (int)min(sh.bcols, sh.cols - c0);
#pragma unroll 1
                for (int o = 0; o < (DUAL ? 2 : 1); ++o) {
                    float t4, t5;
                    err_sums_reference_order<false, WGS>([&](int r, int c) { return o ? b16[(int64_t)c * sh.cols + r] : b16[(int64_t)r * sh.cols + c]; },
                                                         o ? bw : bh, o ? bh : bw, o ? sh.bcols : sh.brows, o ? sh.brows : sh.bcols,
                                                         (o ? sh.rows : sh.cols) % 2 == 0, E8, s4, s5, t4, t5);
                    if (o == 0) { e4 = t4; e5 = t5; }
                    else qt_t = mor_decide_error(amax, qa.clamp, t4, t5);
                }
            }
            qt = mor_decide_error(amax, qa.clamp, e4, e5);
        }
        meta_val = qt;
        fmt = mor_fmt_of(qt);
    }
    if constexpr (WIRE) {
        // codes instead of values: tile `bid` of the payload, rows packed; lane (row r, chunk cc) writes its 8 codes
        uint8_t* tile = reinterpret_cast<uint8_t*>(out) + (int64_t)bid * TILE_PAYLOAD_BYTES;
        const bool zero_tile = !(amax > 0.0f);               // (decided as E2M3, FQ:620-627: all codes are signed zeros)
        const Scale sc = make_scale((fmt < 0 || zero_tile) ? 1.0f : fmax_of(fmt) / amax);
        if (tid == 0) { meta[bid] = meta_val; stats[bid] = sc.s; }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int ch = k * WGS + tid, r = ch >> 4, cc = ch & 15;
            const uint32_t w[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
            if (fmt < 0) {
                *reinterpret_cast<uint4*>(tile + r * 256 + cc * 16) = v[k];
            } else if (fmt == FMT_E4M3 || fmt == FMT_E5M2) {
                // the magnitudes' codes as pass 3 of the bf16 kernel computes them, the sign of the input on top
                uint32_t c2[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float a = fabsf(bf16_lo(w[j])) * sc.s, b = fabsf(bf16_hi(w[j])) * sc.s;
                    const uint32_t p = (fmt == FMT_E4M3) ? hw_pack2_low<FMT_E4M3>(a, b) : hw_pack2_low<FMT_E5M2>(a, b);
                    c2[j] = (p & 0xFFFFu) | ((w[j] >> 8) & 0x80u) | ((w[j] >> 16) & 0x8000u);
                }
                *reinterpret_cast<uint2*>(tile + r * 128 + cc * 8) = make_uint2(c2[0] | (c2[1] << 16), c2[2] | (c2[3] << 16));
            } else {
                // E2M3 (the reference's software cast: a zero result is +0): 8 codes of 6 bits = 3 half-words
                uint64_t bits = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t ca = 0, cb = 0;
                    if (!zero_tile) {
                        const float a = fminf(fabsf(bf16_lo(w[j])) * sc.s, Fmt<FMT_E2M3>::fmax), b = fminf(fabsf(bf16_hi(w[j])) * sc.s, Fmt<FMT_E2M3>::fmax);
                        fp6_mag_codes<FMT_E2M3>(a, b, ca, cb);
                        if (ca) ca |= (w[j] >> 10) & 0x20u;
                        if (cb) cb |= (w[j] >> 26) & 0x20u;
                    } else {
                        ca = (w[j] >> 10) & 0x20u;           // (a zero tile is copied: its zeros keep their signs)
                        cb = (w[j] >> 26) & 0x20u;
                    }
                    bits |= (uint64_t)(ca | (cb << 6)) << (12 * j);
                }
                uint16_t* d = reinterpret_cast<uint16_t*>(tile + r * 96 + cc * 6);
                d[0] = (uint16_t)bits; d[1] = (uint16_t)(bits >> 16); d[2] = (uint16_t)(bits >> 32);
            }
        }
        return;
    }
    if (tid == 0) {
        if (meta && meta_val >= 0) meta[bid] = meta_val;
        if (stats) { float* s = stats + 4 * (int64_t)bid; s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5; }
    }
    if (!out) return;

    // pass 3 (registers): quantize and store, FQ:733-851
    auto pass3 = [&]() {
    if ((fmt < 0) || !(amax > 0.0f)) {
        if (out != in) {
#pragma unroll
            for (int k = 0; k < NV; ++k) if (ok[k]) put(k, v[k]);
        }
        return;
    }
    if constexpr (!E8) {
        if (fmt == FMT_E4M3 || fmt == FMT_E5M2) {
            // An FP8 format has 127 magnitudes, a block one scale: code / scale, rounded to bf16, is computed once per
            // code (a thread each) and looked up per element, which leaves a multiply, the convert and the sign per element.
            const float r4 = s4.r;                    // 1 / s5 = r4 / 128 exactly
            if (tid < 128) {
                const float c = (fmt == FMT_E4M3) ? hw_unpack2_low<FMT_E4M3>((uint32_t)tid).x : hw_unpack2_low<FMT_E5M2>((uint32_t)tid).x;
                s_q[tid] = store_bf16<false>((fmt == FMT_E4M3) ? div_by_scale(c, s4.s, r4) : div_by_scale(c, s5.s, r4 * 0.0078125f));
            }
            __syncthreads();
            uint32_t codes = 0;                       // (the converts write half of this register: carried from word to word)
            if constexpr (KEEP) {
                if (have_codes) {                     // uniform over the workgroup
                    if (fmt == FMT_E4M3) {
#pragma unroll
                        for (int k = 0; k < NV; ++k) put(k, fq_vec_tab_codes<FMT_E4M3>(v[k], kc[k], s_q));
                    } else {
#pragma unroll
                        for (int k = 0; k < NV; ++k) put(k, fq_vec_tab_codes<FMT_E5M2>(v[k], kc[k], s_q));
                    }
                    return;
                }
            }
            if (fmt == FMT_E4M3) {
#pragma unroll
                for (int k = 0; k < NV; ++k) if (ok[k]) put(k, fq_vec_tab<FMT_E4M3>(v[k], s4.s, s_q, codes));
            } else {
#pragma unroll
                for (int k = 0; k < NV; ++k) if (ok[k]) put(k, fq_vec_tab<FMT_E5M2>(v[k], s5.s, s_q, codes));
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
    };
    if constexpr (DUAL && MOR) {
        if (qt_t != Q_UNKNOWN && mor_fmt_of(qt_t) != fmt) {
            // the transposed tile decided on the other format (sums that agree to their last bits, added in two orders):
            // the tile is quantized twice, for `out` and then for the LDS copy that out_t is written from
            to_lds = false;
            pass3();
            __syncthreads();               // the readers of the first table are done
            fmt = mor_fmt_of(qt_t);
            meta_val = qt_t;
            to_out = false; to_lds = true;
        }
    }
    pass3();
    write_transposed(meta_val);
}

// (MoR on blocks of 16 vectors per lane -- 256 x 256 tiles in 512 threads -- is held to 128 registers: at the 136 it takes
// otherwise one workgroup fills a CU and nothing overlaps its phases; 8192^2: 60.6 -> 56.7 us)
template <bool MOR, bool E8, int NV, bool FULL, int NT, int WGS = WG, bool GATHER = false, bool DUAL = false, bool WIRE = false>
__global__ __launch_bounds__(WGS) __attribute__((amdgpu_waves_per_eu((MOR && NV == 16) ? 4 : 1, 8))) void k_wgblock(const uint4* in, uint4* out, int32_t* __restrict__ meta,
                                                 float* __restrict__ stats, Shape sh, QuantArgs qa, int cpr, int cpr_shift,
                                                 int64_t first, uint4* out_t, int32_t* __restrict__ meta_t) {
    // Workgroup -> block.  cpr_shift bit 8 (large tensors whose block grid is a multiple of 8 wide): consecutive
    // workgroup ids go round the 8 XCDs, and each XCD takes a band of gx / 8 block columns, walking it row by row.
    uint32_t bid = (uint32_t)(first + blockIdx.x);       // (a launch holds a slice of the blocks, see for_slices; fewer than 2^31 blocks)
    if (cpr_shift >= 256) {            // (a negative cpr_shift means a chunk count per row that is not a power of two)
        bid = band_order(sh, bid);
        cpr_shift &= 255;
        if (cpr_shift == 255) cpr_shift = -1;
    }
    wgblock_body<MOR, E8, NV, FULL, NT, WGS, GATHER, DUAL, WIRE>(in, out, meta, stats, sh, qa, cpr, cpr_shift, bid, out_t, meta_t);
}


}  // namespace mor
