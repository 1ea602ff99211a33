// mor_fake_quantize_dual_tiles: fake quantization in 128 x 128 tiles of a tensor and of its transpose from one read.
// The kernel is k_wgblock with its second, transposed output.
// "FQ" below is the reference file mor/csrc/cuda/fake_quantize.cu.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mor_wgblock.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

using namespace mor;

template <bool MOR, bool E8>
static void launch_dual(const uint4* in, uint4* out, int32_t* meta, uint4* out_t, int32_t* meta_t, const Shape& sh,
                        const QuantArgs& qa, hipStream_t st) {
    const int64_t nblocks = sh.gy * sh.gx;
    const int64_t out_bytes = sh.rows * sh.cols * 2;
    // streaming stores / loads and the XCD bands of tile columns as for the one-output kernel (launch_wgblock_nv)
    const int ntm = (out_bytes >= ((int64_t)64 << 20)) ? 1 : (out_bytes >= ((int64_t)4 << 20)) ? 2 : 0;
    const int shift = (nblocks >= 2048 && sh.gx % 8 == 0 && nblocks % 8 == 0) ? (4 | 256) : 4;
    // large grids: three workgroups per CU, as for the one-output kernel (unused dynamic LDS on top of the tile's 32 KiB;
    // 8192^2: 83 -> 81 us)
    const size_t dl = nblocks >= 4096 ? 20000 - (MOR ? REF_SUMS_LDS_BYTES : 0) : 0;
    for_slices(nblocks, [&](int64_t first, int count) {
        if (ntm == 1) k_wgblock<MOR, E8, 8, true, 1, WG, false, true><<<count, WG, dl, st>>>(in, out, meta, nullptr, sh, qa, 16, shift, first, out_t, meta_t);
        else if (ntm == 2) k_wgblock<MOR, E8, 8, true, 2, WG, false, true><<<count, WG, 0, st>>>(in, out, meta, nullptr, sh, qa, 16, shift, first, out_t, meta_t);
        else k_wgblock<MOR, E8, 8, true, 0, WG, false, true><<<count, WG, 0, st>>>(in, out, meta, nullptr, sh, qa, 16, shift, first, out_t, meta_t);
    });
}

extern "C" int mor_fake_quantize_dual_tiles(const void* input, void* output, int32_t* meta, void* output_t, int32_t* meta_t,
                                            int64_t rows, int64_t cols, double clamp_threshold, int64_t mode, int64_t sf_type,
                                            void* stream) {
    if (int rc = mor_validate_shape(input, rows, cols, 128, 128)) return rc;
    if (!output || !output_t || !meta || !meta_t) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "NULL output or meta pointer");
    if (rows % 128 || cols % 128)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "rows and cols must be multiples of 128 (got %lld x %lld)", (long long)rows, (long long)cols);
    if ((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(output) | reinterpret_cast<uintptr_t>(output_t)) & 15u)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "tensors must be 16-byte aligned");
    if (cols >= ((int64_t)1 << 27) || rows >= ((int64_t)1 << 27))              // (a tile row's chunk offsets are 32-bit, in both tensors)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "more than 2^27 rows or columns (%lld x %lld)", (long long)rows, (long long)cols);
    if (input == output || input == output_t || output == output_t)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "input and the two outputs must be three different tensors");
    QuantArgs qa;
    if (!mor_decode_mode(mode, clamp_threshold, qa) || qa.qmode == 4)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "mode %% 10 must be 1 (MoR), 2 (E4M3) or 3 (E5M2), got %lld", (long long)mode);
    const Shape sh = make_shape(rows, cols, 128, 128);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint4* in = static_cast<const uint4*>(input);
    uint4* out = static_cast<uint4*>(output);
    uint4* out_t = static_cast<uint4*>(output_t);
    const bool mor = qa.qmode == 1, e8 = sf_type == 2;
    if (mor) { if (e8) launch_dual<true, true>(in, out, meta, out_t, meta_t, sh, qa, st); else launch_dual<true, false>(in, out, meta, out_t, meta_t, sh, qa, st); }
    else { if (e8) launch_dual<false, true>(in, out, meta, out_t, meta_t, sh, qa, st); else launch_dual<false, false>(in, out, meta, out_t, meta_t, sh, qa, st); }
    return mor_check_launch("k_wgblock (two outputs)");
}
