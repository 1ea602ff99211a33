// k_wgblock: one workgroup per quantization block held in registers (128 x 128 tiles, rows of 4096 elements, ...).
// "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>

#include "mor_wgblock.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

using namespace mor;

template <bool MOR, bool E8, int NV, int WGS = WG>
static void launch_wgblock_nv(bool full, int grid, const uint4* i4, uint4* o4, int32_t* meta, float* stats,
                              const Shape& sh, const QuantArgs& qa, int cpr, int shift, hipStream_t st) {
    // Streaming stores for outputs that do not fit an L2 anyway (>= 4 MiB): the quantized tensor then does not evict
    // the input or the caller's data from the caches (measured at 8192^2: 42.7 -> 40.4 us, at 4096^2: 13.3 -> 10.3 us).
    // Tensors of 64 MiB and more stream their loads as well (the block is read once; a smaller tensor is likely to sit
    // in the last-level cache, where its producer left it).
    const int64_t out_bytes = sh.rows * sh.cols * 2;
    const int ntm = (out_bytes >= ((int64_t)64 << 20)) ? 1 : (out_bytes >= ((int64_t)4 << 20)) ? 2 : 0;
    // Large grids run 3 workgroups per CU (unused dynamic LDS caps the occupancy the registers would allow at 5):
    // fewer tiles in flight keep the memory system on fewer DRAM pages at a time (8192^2 from HBM, MoR 128 x 128:
    // 49.4 -> 47.5 us; 16384 x 14336: 161 -> 156 us), while a grid that fits the chip at once wants every slot
    // (4096^2: 9.2 against 10.8 us).
    // (the MoR kernels hold REF_SUMS_LDS_BYTES of static LDS for the reference-order sums)
    const size_t dyn_lds = ((NV == 8 && WGS == WG) || (NV == 4 && WGS == 512)) && grid >= 4096 ? 53000 - (MOR ? REF_SUMS_LDS_BYTES : 0) : 0;
    // Consecutive workgroup ids go round the 8 XCDs.  In band order each XCD takes a band of gx / 8 block columns and
    // walks it row by row, so that the blocks sharing a DRAM page are in flight on one XCD at about the same time
    // (from HBM, 128 x 128 blocks: 8192^2 MoR 50.4 -> 47.5 us, 16384 x 14336 170 -> 156 us; a tensor that sits in the
    // last-level cache does not care).
    const int shift_arg = (grid >= 2048 && sh.gx % 8 == 0 && grid % 8 == 0) ? ((shift & 255) | 256) : shift;
#define MOR_WGBLOCK(FULL, NT) for_slices(grid, [&](int64_t first, int count) { \
        k_wgblock<MOR, E8, NV, FULL, NT, WGS><<<count, WGS, dyn_lds, st>>>(i4, o4, meta, stats, sh, qa, cpr, shift_arg, first, nullptr, nullptr); })
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
        k_wgblock<MOR, E8, NV, false, 0, WG, true><<<count, WG, 0, st>>>(i4, o4, meta, stats, sh, qa, 1, 0, first, nullptr, nullptr); })
    if (nv <= 1) MOR_GATHER(1); else if (nv <= 2) MOR_GATHER(2); else if (nv <= 4) MOR_GATHER(4); else MOR_GATHER(8);
#undef MOR_GATHER
}
void mor_launch_wgblock(bool mor, bool e8, bool gather, const void* in, void* out, int32_t* meta, float* stats,
                        const Shape& sh, const QuantArgs& qa, hipStream_t st) {
    if (gather) {
        if (mor) { if (e8) launch_wgblock_gather<true, true>(in, out, meta, stats, sh, qa, st); else launch_wgblock_gather<true, false>(in, out, meta, stats, sh, qa, st); }
        else { if (e8) launch_wgblock_gather<false, true>(in, out, meta, stats, sh, qa, st); else launch_wgblock_gather<false, false>(in, out, meta, stats, sh, qa, st); }
    } else {
        if (mor) { if (e8) launch_wgblock<true, true>(in, out, meta, stats, sh, qa, st); else launch_wgblock<true, false>(in, out, meta, stats, sh, qa, st); }
        else { if (e8) launch_wgblock<false, true>(in, out, meta, stats, sh, qa, st); else launch_wgblock<false, false>(in, out, meta, stats, sh, qa, st); }
    }
}
