// Small pieces shared by the source files of libmor_hip.so: workgroup size, the tensor / block shape record,
// per-wave LDS combines, division by multiply-shift, host-side integer helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>

#include "mor_device.h"

namespace mor {

constexpr int WG = 256;
constexpr int WAVES = WG / 64;

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

// A tensor of rows x cols elements in blocks of brows x bcols: gy x gx blocks (fewer than 2^31, so block ids are
// 32-bit), with the multiply-shift constants that turn a block id into (block row, block column) without a division.
struct Shape {
    int64_t rows, cols, brows, bcols, gy, gx;
    DivU32 d_gx;        // / gx
    DivU32 d_band;      // / (gx / 8): the width of the band of block columns one XCD walks (gx a multiple of 8)
};
// block id -> (block row, block column)
__device__ __forceinline__ void block_of(const Shape& sh, uint32_t bid, uint32_t& by, uint32_t& bx) {
    by = div_u32(bid, sh.d_gx);
    bx = bid - by * (uint32_t)sh.gx;
}
// Consecutive workgroup ids go round the 8 XCDs.  Band order: XCD x takes the band of gx / 8 block columns starting at
// x * gx / 8 and walks it row by row, so that the blocks in flight on one XCD are neighbours in memory (gx and the
// number of workgroups multiples of 8).  Returns the block id workgroup `wid` works on.
__device__ __forceinline__ uint32_t band_order(const Shape& sh, uint32_t wid) {
    const uint32_t xcd = wid & 7u, j = wid >> 3, per = (uint32_t)sh.gx >> 3, byb = div_u32(j, sh.d_band);
    return byb * (uint32_t)sh.gx + xcd * per + (j - byb * per);
}

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
    static_assert(NW == 1 || NW == 4 || NW == 8 || NW == 16, "1, 4, 8 or 16 waves");
    if constexpr (NW == 1) return s[0];
    float a = (s[0] + s[1]) + (s[2] + s[3]);
    if constexpr (NW >= 8) a += (s[4] + s[5]) + (s[6] + s[7]);
    if constexpr (NW == 16) a += ((s[8] + s[9]) + (s[10] + s[11])) + ((s[12] + s[13]) + (s[14] + s[15]));
    return a;
}

}  // namespace mor

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline bool is_pow2(int64_t x) { return x > 0 && (x & (x - 1)) == 0; }
static inline int ilog2(int64_t x) { int l = 0; while ((1ll << l) < x) ++l; return l; }

static inline mor::Shape make_shape(int64_t rows, int64_t cols, int64_t brows, int64_t bcols) {
    mor::Shape sh{rows, cols, brows, bcols, cdiv(rows, brows), cdiv(cols, bcols), {}, {}};
    sh.d_gx = mor::make_div((uint32_t)sh.gx);
    sh.d_band = mor::make_div((uint32_t)std::max<int64_t>(sh.gx >> 3, 1));
    return sh;
}

static inline int grid_for(int64_t work_items, int per_cu = 8) {
    // enough workgroups to fill 256 CUs several times over, capped so grid-stride loops stay short
    int64_t want = cdiv(work_items, mor::WG);
    int64_t cap = 256ll * per_cu;
    if (want < 1) want = 1;
    return (int)(want < cap ? want : cap);
}
