// mor_mor_quantize / mor_mor_dequantize: the MoR decision (or a forced FP8 format) per 128 x 128 tile with the tile's
// codes as the result (format tag + fp32 scale + payload) instead of the fake-quantized bf16 values, and the way back.
// The encoder is k_wgblock in its WIRE form (same passes 1 and 2, codes stored in pass 3); the decoder below repeats
// the second half of the bf16 kernel's pass 3 (code -> value, division by the scale, bf16 store), so that
// decode(encode(x)) is the output of mor_fake_quantize bit for bit.
// "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mor_wgblock.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

using namespace mor;

static_assert(TILE_PAYLOAD_BYTES == MOR_TILE_PAYLOAD_BYTES && TILE_STORED_BF16 == MOR_TILE_STORED_BF16, "header constants");

namespace mor {

// One workgroup per tile; lane (row r, chunk cc) of step k decodes 8 codes into one 16-byte vector of the output,
// the mapping the encoder wrote them with.  The reads of a tile are one linear run of 16 / 12 / 32 KiB.
template <int NT>
__global__ __launch_bounds__(WG) void k_mor_decode(const uint8_t* __restrict__ payload, const int32_t* __restrict__ tags,
                                                   const float* __restrict__ scales, uint4* __restrict__ out, Shape sh,
                                                   int band, int64_t first) {
    const int tid = threadIdx.x;
    uint32_t bid = (uint32_t)(first + blockIdx.x);
    if (band) bid = band_order(sh, bid);
    uint32_t by, bx;
    block_of(sh, bid, by, bx);
    const uint32_t row_stride = (uint32_t)(sh.cols >> 3);
    uint4* bout = out + ((int64_t)by * 128 * row_stride + (int64_t)bx * 16);
    const uint8_t* tile = payload + (int64_t)bid * TILE_PAYLOAD_BYTES;
    const int tag = tags[bid];
    const int fmt = (tag & TILE_STORED_BF16) ? -1 : mor_fmt_of(tag);
    const float s = scales[bid];
    const float r = 1.0f / s;
    // (the format is uniform over the workgroup: each case loads its 8 vectors first, then converts and stores)
    auto put = [&](int k, uint4 q) {
        const int ch = k * WG + tid;
        store16<(NT != 0)>(bout + (uint32_t)(ch >> 4) * row_stride + (uint32_t)(ch & 15), q);
    };
    if (fmt < 0) {
        uint4 c[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) c[k] = reinterpret_cast<const uint4*>(tile)[k * WG + tid];
#pragma unroll
        for (int k = 0; k < 8; ++k) put(k, c[k]);
    } else if (fmt == FMT_E4M3 || fmt == FMT_E5M2) {
        uint2 c[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) c[k] = reinterpret_cast<const uint2*>(tile)[k * WG + tid];
        auto decode = [&](auto unpack) {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const uint32_t c2[4] = {c[k].x & 0xFFFFu, c[k].x >> 16, c[k].y & 0xFFFFu, c[k].y >> 16};
                uint32_t w[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const f32x2 d = unpack(c2[j] & 0x7F7Fu);
                    const uint32_t sign = ((c2[j] & 0x80u) << 8) | ((c2[j] & 0x8000u) << 16);
                    w[j] = store_pair<false>(div_by_scale(d.x, s, r), div_by_scale(d.y, s, r)) | sign;
                }
                put(k, make_uint4(w[0], w[1], w[2], w[3]));
            }
        };
        if (fmt == FMT_E4M3) decode([](uint32_t m) { return hw_unpack2_low<FMT_E4M3>(m); });
        else decode([](uint32_t m) { return hw_unpack2_low<FMT_E5M2>(m); });
    } else {
        uint16_t c[8][3];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint16_t* p = reinterpret_cast<const uint16_t*>(tile) + 3 * (k * WG + tid);
            c[k][0] = p[0]; c[k][1] = p[1]; c[k][2] = p[2];
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint64_t bits = (uint64_t)c[k][0] | ((uint64_t)c[k][1] << 16) | ((uint64_t)c[k][2] << 32);
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t ca = (uint32_t)(bits >> (12 * j)) & 0x3Fu, cb = (uint32_t)(bits >> (12 * j + 6)) & 0x3Fu;
                const float da = fp6_value<FMT_E2M3>(ca & 0x1Fu), db = fp6_value<FMT_E2M3>(cb & 0x1Fu);
                const uint32_t sign = ((ca & 0x20u) << 10) | ((cb & 0x20u) << 26);
                w[j] = store_pair<false>(div_by_scale(da, s, r), div_by_scale(db, s, r)) | sign;
            }
            put(k, make_uint4(w[0], w[1], w[2], w[3]));
        }
    }
}

// The codes of a tile, transposed: one workgroup per tile reads its slot, turns the tile through LDS and writes the
// slot of the transposed tensor's tile (the same format, scale and tag: a tile and its transpose hold the same
// elements).  8-bit codes travel as a 128 x 128 byte tile, 6-bit codes are unpacked to bytes on the way in and packed on
// the way out, bf16 tiles go in two halves through the word layout of the two-output kernel.  Byte tile in LDS: row r
// is 32 words, and word w of row r sits at position w ^ (r >> 3): the 16 lanes that collect, for one column, the bytes
// of rows 8 j .. 8 j + 7 (j = 0 .. 15) read 16 different banks, and the four columns a wave handles at a time share
// their words.
__global__ __launch_bounds__(WG) void k_mor_transpose(const uint8_t* __restrict__ payload, const int32_t* __restrict__ tags,
                                                      const float* __restrict__ scales, uint8_t* __restrict__ payload_t,
                                                      int32_t* __restrict__ tags_t, float* __restrict__ scales_t, int gy, int gx,
                                                      int64_t first) {
    __shared__ __attribute__((aligned(16))) uint32_t s_t[128 * 32];            // 16 KiB: a byte tile, or half a bf16 tile
    const int tid = threadIdx.x;
    const int64_t bid = first + blockIdx.x;
    const int by = (int)(bid / gx), bx = (int)(bid - (int64_t)by * gx);
    const int64_t tid_t = (int64_t)bx * gy + by;
    const uint8_t* slot = payload + bid * TILE_PAYLOAD_BYTES;
    uint8_t* slot_t = payload_t + tid_t * TILE_PAYLOAD_BYTES;
    const int tag = tags[bid];
    const int fmt = (tag & TILE_STORED_BF16) ? -1 : mor_fmt_of(tag);
    if (tid == 0) { tags_t[tid_t] = tag; scales_t[tid_t] = scales[bid]; }
    if (fmt < 0) {
        // bf16, the left and the right half of the tile in turn (64 columns = 32 words per row): vectors of 8 columns in,
        // vectors of 8 rows out.  The word of columns (2 w, 2 w + 1) of row r sits at position w ^ ((r >> 3) << 1) of its
        // row, as in the two-output kernel: a vector stays one aligned group of 4 words, in another order.
        const uint16_t* s16 = reinterpret_cast<const uint16_t*>(s_t);
#pragma unroll 1
        for (int h = 0; h < 2; ++h) {
            if (h) __syncthreads();                                            // the first half has been read out
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int ch = k * WG + tid, r = ch >> 3, c8 = ch & 7, R = r >> 3;
                const uint4 q = reinterpret_cast<const uint4*>(slot)[r * 16 + h * 8 + c8];
                const uint4 p = (R & 1) ? make_uint4(q.z, q.w, q.x, q.y) : q;
                *reinterpret_cast<uint4*>(s_t + r * 32 + ((c8 ^ (R >> 1)) << 2)) = p;
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int ch = k * WG + tid, c = ch >> 4, j = ch & 15;       // column c of the half, rows 8 j .. 8 j + 7
                const int at = 2 * ((c >> 1) ^ (j << 1)) + (c & 1);
                uint32_t w[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t lo = s16[(8 * j + 2 * i) * 64 + at], hi = s16[(8 * j + 2 * i + 1) * 64 + at];
                    w[i] = lo | (hi << 16);
                }
                reinterpret_cast<uint4*>(slot_t)[(h * 64 + c) * 16 + j] = make_uint4(w[0], w[1], w[2], w[3]);
            }
        }
        return;
    }
    const bool six = fmt == FMT_E2M3;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int ch = k * WG + tid, r = ch >> 4, cc = ch & 15, j = r >> 3;
        uint2 v;
        if (six) {
            const uint16_t* p = reinterpret_cast<const uint16_t*>(slot) + 3 * ch;
            const uint64_t bits = (uint64_t)p[0] | ((uint64_t)p[1] << 16) | ((uint64_t)p[2] << 32);
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                lo |= ((uint32_t)(bits >> (6 * i)) & 0x3Fu) << (8 * i);
                hi |= ((uint32_t)(bits >> (6 * (i + 4))) & 0x3Fu) << (8 * i);
            }
            v = make_uint2(lo, hi);
        } else {
            v = reinterpret_cast<const uint2*>(slot)[ch];
        }
        // words 2 cc, 2 cc + 1 of row r at positions (2 cc) ^ j, (2 cc + 1) ^ j: one aligned pair, halves swapped for odd j
        *reinterpret_cast<uint2*>(s_t + r * 32 + 2 * (cc ^ (j >> 1))) = (j & 1) ? make_uint2(v.y, v.x) : v;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int ch = k * WG + tid, c = ch >> 4, j = ch & 15;             // column c of the tile, rows 8 j .. 8 j + 7
        const int at = (c >> 2) ^ j, sh8 = 8 * (c & 3);
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lo |= ((s_t[(8 * j + i) * 32 + at] >> sh8) & 0xFFu) << (8 * i);
            hi |= ((s_t[(8 * j + 4 + i) * 32 + at] >> sh8) & 0xFFu) << (8 * i);
        }
        if (six) {
            uint64_t bits = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                bits |= (uint64_t)((lo >> (8 * i)) & 0x3Fu) << (6 * i);
                bits |= (uint64_t)((hi >> (8 * i)) & 0x3Fu) << (6 * (i + 4));
            }
            uint16_t* d = reinterpret_cast<uint16_t*>(slot_t) + 3 * ch;
            d[0] = (uint16_t)bits; d[1] = (uint16_t)(bits >> 16); d[2] = (uint16_t)(bits >> 32);
        } else {
            reinterpret_cast<uint2*>(slot_t)[ch] = make_uint2(lo, hi);
        }
    }
}

}  // namespace mor

static int check_tiles(const void* a, const void* b, const void* tags, const void* scales, int64_t rows, int64_t cols) {
    if (int rc = mor_validate_shape(a, rows, cols, 128, 128)) return rc;
    if (!b || !tags || !scales) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "NULL payload, tags or scales pointer");
    if (rows % 128 || cols % 128)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "rows and cols must be multiples of 128 (got %lld x %lld)", (long long)rows, (long long)cols);
    if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "tensor and payload must be 16-byte aligned");
    if (a == b) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "tensor and payload must be different buffers");
    // (a tile row's chunk offsets are 32-bit; mor_mor_transpose takes tile grids of up to 2^20 x 2^20 and 2^30 tiles)
    if (cols >= ((int64_t)1 << 27) || rows >= ((int64_t)1 << 27) || (rows / 128) * (cols / 128) > ((int64_t)1 << 30))
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "more than 2^27 rows or columns, or more than 2^30 tiles (%lld x %lld)", (long long)rows, (long long)cols);
    return MOR_OK;
}

extern "C" int mor_mor_quantize(const void* input, void* payload, int32_t* tags, float* scales, int64_t rows, int64_t cols,
                                double clamp_threshold, int64_t mode, void* stream) {
    if (int rc = check_tiles(input, payload, tags, scales, rows, cols)) return rc;
    QuantArgs qa;
    if (!mor_decode_mode(mode, clamp_threshold, qa) || qa.qmode == 4)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "mode %% 10 must be 1 (MoR), 2 (E4M3) or 3 (E5M2), got %lld", (long long)mode);
    const Shape sh = make_shape(rows, cols, 128, 128);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t nblocks = sh.gy * sh.gx;
    // loads and XCD bands as for the bf16 kernel (launch_wgblock_nv)
    const bool stream_loads = rows * cols * 2 >= ((int64_t)64 << 20);
    const int shift = (nblocks >= 2048 && sh.gx % 8 == 0 && nblocks % 8 == 0) ? (4 | 256) : 4;
    // four workgroups per CU on large grids (the bf16 kernel runs three: half the bytes are written here; 8192^2 from HBM:
    // 42.0 us with three, 39.3 with four, 39.1 - 40.0 without a cap)
    const bool mor = qa.qmode == 1;
    const size_t dl = nblocks >= 4096 ? 36000 - (mor ? REF_SUMS_LDS_BYTES : 0) : 0;
    const uint4* in = static_cast<const uint4*>(input);
    uint4* out = static_cast<uint4*>(payload);
    for_slices(nblocks, [&](int64_t first, int count) {
#define MOR_TILE_CODES(MOR_, NT_) k_wgblock<MOR_, false, 8, true, NT_, WG, false, false, true><<<count, WG, dl, st>>>(in, out, tags, scales, sh, qa, 16, shift, first, nullptr, nullptr)
        if (mor) { if (stream_loads) MOR_TILE_CODES(true, 1); else MOR_TILE_CODES(true, 0); }
        else { if (stream_loads) MOR_TILE_CODES(false, 1); else MOR_TILE_CODES(false, 0); }
#undef MOR_TILE_CODES
    });
    return mor_check_launch("k_wgblock (tile codes)");
}

extern "C" int mor_mor_dequantize(const void* payload, const int32_t* tags, const float* scales, void* output, int64_t rows,
                                  int64_t cols, void* stream) {
    if (int rc = check_tiles(output, payload, tags, scales, rows, cols)) return rc;
    const Shape sh = make_shape(rows, cols, 128, 128);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t nblocks = sh.gy * sh.gx;
    const int band = (nblocks >= 2048 && sh.gx % 8 == 0 && nblocks % 8 == 0) ? 1 : 0;
    const bool nt = rows * cols * 2 >= ((int64_t)4 << 20);
    const uint8_t* p = static_cast<const uint8_t*>(payload);
    uint4* out = static_cast<uint4*>(output);
    for_slices(nblocks, [&](int64_t first, int count) {
        // (full occupancy: 8192^2 from HBM 37.4 us; capped at 4 / 3 workgroups per CU 43 / 53 us)
        if (nt) k_mor_decode<1><<<count, WG, 0, st>>>(p, tags, scales, out, sh, band, first);
        else k_mor_decode<0><<<count, WG, 0, st>>>(p, tags, scales, out, sh, band, first);
    });
    return mor_check_launch("k_mor_decode");
}

extern "C" int mor_mor_transpose(const void* payload, const int32_t* tags, const float* scales, void* payload_t, int32_t* tags_t,
                                 float* scales_t, int64_t tile_rows, int64_t tile_cols, void* stream) {
    if (tile_rows <= 0 || tile_cols <= 0 || tile_rows > (1 << 20) || tile_cols > (1 << 20) || tile_rows * tile_cols > ((int64_t)1 << 30))
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "bad tile grid %lld x %lld", (long long)tile_rows, (long long)tile_cols);
    if (!payload || !tags || !scales || !payload_t || !tags_t || !scales_t) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "NULL pointer");
    if ((reinterpret_cast<uintptr_t>(payload) | reinterpret_cast<uintptr_t>(payload_t)) & 15u)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "payloads must be 16-byte aligned");
    if (payload == payload_t || tags == tags_t || scales == scales_t)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "source and destination must be different buffers");
    hipStream_t st = static_cast<hipStream_t>(stream);
    for_slices(tile_rows * tile_cols, [&](int64_t first, int count) {
        k_mor_transpose<<<count, WG, 0, st>>>(static_cast<const uint8_t*>(payload), tags, scales, static_cast<uint8_t*>(payload_t), tags_t, scales_t,
                                              (int)tile_rows, (int)tile_cols, first);
    });
    return mor_check_launch("k_mor_transpose");
}

// Both orientations in one call: the codes of the tensor, then the codes of its transpose from them (two launches; a
// kernel that wrote both from one read of the tensor was built and measured no faster: 63.4 against 61.6 us at 8192^2 from
// HBM, the transposition through LDS and the second slot lengthen every workgroup by what the second launch costs).
extern "C" int mor_mor_quantize_dual(const void* input, void* payload, int32_t* tags, float* scales, void* payload_t, int32_t* tags_t,
                                     float* scales_t, int64_t rows, int64_t cols, double clamp_threshold, int64_t mode, void* stream) {
    if (!payload_t || !tags_t || !scales_t) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "NULL pointer of the transposed tensor");
    if (payload_t == input || payload_t == payload || tags_t == tags || scales_t == scales)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "the outputs of the two orientations must be different buffers");
    if (reinterpret_cast<uintptr_t>(payload_t) & 15u) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "payloads must be 16-byte aligned");
    if (int rc = mor_mor_quantize(input, payload, tags, scales, rows, cols, clamp_threshold, mode, stream)) return rc;
    return mor_mor_transpose(payload, tags, scales, payload_t, tags_t, scales_t, rows / 128, cols / 128, stream);
}
