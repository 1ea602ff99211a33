// mor_fake_quantize_batch: many tensors in one call.  Tensors of a few hundred thousand elements cost one launch
// each through mor_fake_quantize (7 us of launch for well under a microsecond of work); here up to 56 of them share
// a launch: one workgroup per quantization block, the workgroup id telling the tensor and the block.  The tensors'
// records travel in the kernel argument (no device table to fill, nothing to allocate).  Larger tensors go to
// mor_fake_quantize, whose kernels fill the chip by themselves.
// "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>

#include "mor_wgblock.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

namespace mor {

constexpr int BATCH_MAX = 56;                       // tensors per launch: 56 records of 64 bytes fit the 4 KiB of kernel arguments
constexpr int64_t BATCH_SMALL = (int64_t)1 << 18;   // elements: larger tensors are launched on their own

enum : int { B_BLOCKS = 0, B_ELEMENTWISE = 1, B_COPY = 2 };
struct BatchItem {                                   // 64 bytes
    const uint16_t* in;
    uint16_t* out;
    int32_t* meta;
    int32_t rows, cols, brows, bcols;                // (block dims clipped to the tensor's: the same blocks)
    DivU32 d_gx;                                     // d = blocks per block row
    float clamp;
    int8_t kind;       // B_BLOCKS: modes 1 / 2 / 3 (generic_block); B_ELEMENTWISE: modes 4 / 5; B_COPY: every other mode
    int8_t e8, qmode, fmt;
    int8_t meta_val, dyn_range, pad[2];
};
static_assert(sizeof(BatchItem) == 64, "record size");
struct BatchArgs {
    int n;
    uint32_t first[BATCH_MAX + 1];       // workgroups [first[t], first[t + 1]) work on tensor t
    BatchItem item[BATCH_MAX];
};
static_assert(sizeof(BatchArgs) <= 4096 - 16, "kernel argument size");

// One block of a tensor in the current-scaling modes (FQ:825-842: the caller's scale for every element) or of a copy.
template <bool EMU>
__device__ __forceinline__ void elementwise_block(const BatchItem& it, const Shape& sh, const QuantArgs& qa, int64_t bid) {
    uint32_t by, bx;
    block_of(sh, (uint32_t)bid, by, bx);
    const int64_t r0 = (int64_t)by * sh.brows, c0 = (int64_t)bx * sh.bcols;
    const int64_t bh = min(sh.brows, sh.rows - r0), bw = min(sh.bcols, sh.cols - c0);
    const uint16_t* bin = it.in + r0 * sh.cols + c0;
    uint16_t* bout = it.out + r0 * sh.cols + c0;
    if (it.kind == B_COPY) {
        if (it.out != it.in) for_block_elements(bh, bw, sh.cols, threadIdx.x, [&](int64_t at) { bout[at] = bin[at]; });
        if (threadIdx.x == 0) it.meta[bid] = 3;
        return;
    }
    const Scale sc = make_scale(qa.clamp);
    const bool e8 = it.e8 != 0;
    for_block_elements(bh, bw, sh.cols, threadIdx.x, [&](int64_t at) { bout[at] = fq_one_exact<EMU>(bin[at], qa.fmt, e8, sc); });
    if (threadIdx.x == 0) it.meta[bid] = qa.meta_val;
}

template <bool EMU>
__global__ __launch_bounds__(WG) void k_batch(BatchArgs a, int fast_ok) {
    __shared__ float s_f[2][WAVES];
    __shared__ uint32_t s_u[WAVES];
    int lo = 0, hi = a.n - 1;                                         // the tensor of this workgroup (uniform over it)
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (blockIdx.x >= a.first[mid]) lo = mid; else hi = mid - 1;
    }
    const BatchItem& it = a.item[lo];
    const int64_t bid = blockIdx.x - a.first[lo];
    Shape sh{};
    sh.rows = it.rows; sh.cols = it.cols; sh.brows = it.brows; sh.bcols = it.bcols;
    sh.gx = it.d_gx.d; sh.gy = (it.rows + it.brows - 1) / it.brows;
    sh.d_gx = it.d_gx;
    QuantArgs qa{};
    qa.qmode = it.qmode; qa.fmt = it.fmt; qa.meta_val = it.meta_val; qa.dyn_range = it.dyn_range; qa.clamp = it.clamp;
    if (it.kind == B_BLOCKS) generic_block<EMU, true>(it.in, it.out, it.meta, nullptr, sh, qa, it.e8 != 0, bid, s_f, s_u, fast_ok != 0);
    else elementwise_block<EMU>(it, sh, qa, bid);
}

// Tensors that are too large for the records above and whose blocks a workgroup holds in registers: whole blocks of
// 2048 x NV elements, NV = 1, 2, 4 or 8 (128 x 128 tiles, rows of 4096 elements, ...), MoR for NV = 8 or a forced
// format.  The blocks of up to 48 such tensors run as one grid of the register-resident block kernel (wgblock_body), so
// that a tensor of a few MiB does not pay a launch of its own and the tail of one tensor's grid overlaps the head of the
// next.  A tensor's workgroups start at a multiple of 8 (the XCD band order counts on workgroup id mod 8); the padding
// workgroups leave at once.
constexpr int BLOCK_BATCH_MAX = 48;
struct BlockItem {                                   // 80 bytes
    const uint4* in;
    uint4* out;
    int32_t* meta;
    int32_t rows, cols, brows, bcols;
    DivU32 d_gx, d_band;
    float clamp;
    int8_t qmode, fmt, meta_val, dyn_range;
    int8_t band, shift, pad[6];                      // shift: log2 of the chunks per block row (20 for one-row blocks: row 0 always)
};
static_assert(sizeof(BlockItem) == 80, "record size");
struct BlockArgs {
    int n;
    uint32_t first[BLOCK_BATCH_MAX + 1];
    BlockItem item[BLOCK_BATCH_MAX];
};
static_assert(sizeof(BlockArgs) <= 4096 - 16, "kernel argument size");

template <bool MOR, bool E8, int NV, int NT>
__global__ __launch_bounds__(WG) void k_batch_blocks(BlockArgs a) {
    int lo = 0, hi = a.n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (blockIdx.x >= a.first[mid]) lo = mid; else hi = mid - 1;
    }
    const BlockItem& it = a.item[lo];
    const uint32_t local = blockIdx.x - a.first[lo];
    Shape sh{};
    sh.rows = it.rows; sh.cols = it.cols; sh.brows = it.brows; sh.bcols = it.bcols;
    sh.gx = it.d_gx.d; sh.gy = it.rows / it.brows;
    sh.d_gx = it.d_gx; sh.d_band = it.d_band;
    if (local >= (uint32_t)(sh.gy * sh.gx)) return;                  // padding up to the next multiple of 8
    QuantArgs qa{};
    qa.qmode = it.qmode; qa.fmt = it.fmt; qa.meta_val = it.meta_val; qa.dyn_range = it.dyn_range; qa.clamp = it.clamp;
    const uint32_t bid = it.band ? band_order(sh, local) : local;
    wgblock_body<MOR, E8, NV, true, NT>(it.in, it.out, it.meta, nullptr, sh, qa, it.bcols >> 3, it.shift, bid, nullptr, nullptr);
}

}  // namespace mor

using namespace mor;

// streaming class of a tensor's loads and stores, as launch_wgblock_nv chooses it
static int block_nt_class(int64_t bytes) { return bytes >= ((int64_t)64 << 20) ? 1 : bytes >= ((int64_t)4 << 20) ? 2 : 0; }

template <bool MOR, bool E8, int NV>
static void launch_batch_blocks_nv(const BlockArgs& a, int nt, hipStream_t st) {
    const uint32_t grid = a.first[a.n];
    const size_t dyn_lds = (NV == 8 && grid >= 4096) ? 53000 - (MOR ? REF_SUMS_LDS_BYTES : 0) : 0;    // three workgroups per CU on large grids (launch_wgblock_nv)
    if (nt == 1) k_batch_blocks<MOR, E8, NV, 1><<<grid, WG, dyn_lds, st>>>(a);
    else if (nt == 2) k_batch_blocks<MOR, E8, NV, 2><<<grid, WG, dyn_lds, st>>>(a);
    else k_batch_blocks<MOR, E8, NV, 0><<<grid, WG, dyn_lds, st>>>(a);
}
// (MoR only with NV = 8: the caller sends other MoR tensors to mor_fake_quantize)
template <bool E8>
static void launch_batch_blocks(const BlockArgs& a, bool mor, int nv, int nt, hipStream_t st) {
    if (mor) { launch_batch_blocks_nv<true, E8, 8>(a, nt, st); return; }
    switch (nv) {
        case 1: launch_batch_blocks_nv<false, E8, 1>(a, nt, st); break;
        case 2: launch_batch_blocks_nv<false, E8, 2>(a, nt, st); break;
        case 4: launch_batch_blocks_nv<false, E8, 4>(a, nt, st); break;
        default: launch_batch_blocks_nv<false, E8, 8>(a, nt, st); break;
    }
}

extern "C" int mor_fake_quantize_batch(const MorTensorDesc* descs, int64_t n, uint32_t flags, void* stream) {
    if (n < 0 || (n > 0 && !descs)) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "bad descriptor array");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool emu = flags & MOR_FLAG_TORCH_EMULATION;
    const int fast_ok = (!emu && !(flags & MOR_FLAG_SOFTWARE_CAST)) ? 1 : 0;
    // every descriptor is checked before anything is launched
    for (int64_t i = 0; i < n; ++i) {
        const MorTensorDesc& d = descs[i];
        if (int rc = mor_validate_shape(d.input, d.rows, d.cols, d.block_rows, d.block_cols)) return rc;
        if (!d.output || !d.meta) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "output / meta of tensor %lld is NULL", (long long)i);
    }
    // tensors in whole register-resident blocks share launches of the block kernel (same mode class, scale type, block
    // size class and streaming class)
    BlockArgs ta{};
    int ta_mor = 0, ta_e8 = 0, ta_nv = 0, ta_nt = 0;
    auto flush_blocks = [&]() -> int {
        if (ta.n == 0) return MOR_OK;
        if (ta_e8) launch_batch_blocks<true>(ta, ta_mor != 0, ta_nv, ta_nt, st);
        else launch_batch_blocks<false>(ta, ta_mor != 0, ta_nv, ta_nt, st);
        ta.n = 0;
        return mor_check_launch("k_batch_blocks");
    };
    BatchArgs a{};
    auto flush = [&]() -> int {
        if (a.n == 0) return MOR_OK;
        if (emu) k_batch<true><<<a.first[a.n], WG, 0, st>>>(a, fast_ok);
        else k_batch<false><<<a.first[a.n], WG, 0, st>>>(a, fast_ok);
        a.n = 0;
        return mor_check_launch("k_batch");
    };
    for (int64_t i = 0; i < n; ++i) {
        const MorTensorDesc& d = descs[i];
        const int64_t nblocks = cdiv(d.rows, d.block_rows) * cdiv(d.cols, d.block_cols);
        if (d.rows * d.cols > BATCH_SMALL || nblocks > (1 << 16)) {
            QuantArgs tq;
            // 16-byte chunks per block (block dims beyond the tensor's, which may be anything, never make whole blocks:
            // left out before the product, which they could overflow)
            const bool dims_ok = d.block_rows <= d.rows && d.block_cols <= d.cols;
            const int64_t nch = (dims_ok && d.block_cols % 8 == 0) ? d.block_rows * (d.block_cols / 8) : 0;
            const int64_t cpr = d.block_cols / 8;
            bool blocks = fast_ok && (nch == WG || nch == 2 * WG || nch == 4 * WG || nch == 8 * WG)
                          && d.rows % d.block_rows == 0 && d.cols % d.block_cols == 0 && (d.block_rows == 1 || is_pow2(cpr))
                          && nblocks <= (1 << 20) && d.rows <= 0x7FFFFFFFll && d.cols <= 0x7FFFFFFFll && d.block_rows * (d.cols / 8) < 0x7FFFFFFFll
                          && ((reinterpret_cast<uintptr_t>(d.input) | reinterpret_cast<uintptr_t>(d.output)) & 15u) == 0
                          && (d.sf_type == 1 || d.sf_type == 2) && mor_decode_mode(d.mode, d.clamp_threshold, tq) && tq.qmode != 4;
            if (blocks && tq.qmode == 1 && nch != 8 * WG) blocks = false;
            if (blocks) {
                const int is_mor = tq.qmode == 1, is_e8 = d.sf_type == 2, nv = (int)(nch / WG), nt = block_nt_class(d.rows * d.cols * 2);
                if (ta.n && (is_mor != ta_mor || is_e8 != ta_e8 || nv != ta_nv || nt != ta_nt || ta.n == BLOCK_BATCH_MAX
                             || (uint64_t)ta.first[ta.n] + (uint64_t)nblocks + 8 > (1u << 22))) {
                    if (int rc = flush_blocks()) return rc;
                }
                ta_mor = is_mor; ta_e8 = is_e8; ta_nv = nv; ta_nt = nt;
                BlockItem& it = ta.item[ta.n];
                it = BlockItem{};
                it.in = static_cast<const uint4*>(d.input);
                it.out = static_cast<uint4*>(d.output);
                it.meta = d.meta;
                it.rows = (int32_t)d.rows;
                it.cols = (int32_t)d.cols;
                it.brows = (int32_t)d.block_rows;
                it.bcols = (int32_t)d.block_cols;
                const int64_t gx = d.cols / d.block_cols;
                it.d_gx = make_div((uint32_t)gx);
                it.d_band = make_div((uint32_t)std::max<int64_t>(gx >> 3, 1));
                it.clamp = tq.clamp;
                it.qmode = (int8_t)tq.qmode; it.fmt = (int8_t)tq.fmt; it.meta_val = (int8_t)tq.meta_val; it.dyn_range = (int8_t)tq.dyn_range;
                it.band = (nblocks >= 2048 && gx % 8 == 0 && nblocks % 8 == 0) ? 1 : 0;
                it.shift = (int8_t)(d.block_rows == 1 ? 20 : ilog2((int)cpr));
                ta.first[ta.n + 1] = ta.first[ta.n] + (uint32_t)((nblocks + 7) & ~(int64_t)7);
                ++ta.n;
                continue;
            }
            if (int rc = mor_fake_quantize(d.input, d.output, d.meta, d.rows, d.cols, d.block_rows, d.block_cols,
                                           d.clamp_threshold, d.mode, d.sf_type, flags, stream)) return rc;
            continue;
        }
        BatchItem& it = a.item[a.n];
        QuantArgs qa;
        const bool quantizes = mor_decode_mode(d.mode, d.clamp_threshold, qa);
        it = BatchItem{};
        it.in = static_cast<const uint16_t*>(d.input);
        it.out = static_cast<uint16_t*>(d.output);
        it.meta = d.meta;
        it.rows = (int32_t)d.rows;
        it.cols = (int32_t)d.cols;
        it.brows = (int32_t)std::min(d.block_rows, d.rows);
        it.bcols = (int32_t)std::min(d.block_cols, d.cols);
        it.d_gx = make_div((uint32_t)cdiv(d.cols, d.block_cols));
        it.clamp = qa.clamp;
        it.kind = (int8_t)(!quantizes ? B_COPY : qa.qmode == 4 ? B_ELEMENTWISE : B_BLOCKS);
        it.e8 = d.sf_type == 2 ? 1 : 0;
        it.qmode = (int8_t)qa.qmode; it.fmt = (int8_t)qa.fmt; it.meta_val = (int8_t)qa.meta_val; it.dyn_range = (int8_t)qa.dyn_range;
        a.first[a.n + 1] = a.first[a.n] + (uint32_t)nblocks;
        if (++a.n == BATCH_MAX) { if (int rc = flush()) return rc; }
    }
    if (int rc = flush_blocks()) return rc;
    return flush();
}
