/*
 * C ABI of libmor_hip.so: MI355X (gfx950) fake quantization of bf16 tensors.
 *
 * These entry points are what a binding of the reference's operator layer needs:
 * each one stands in for one host launcher of the reference file
 * mor/csrc/cuda/fake_quantize.cu ("FQ").  All pointers are device pointers unless
 * stated otherwise, tensors are row-major and contiguous, bf16 is passed as raw
 * 16-bit patterns.  Calls are asynchronous on `stream` (a hipStream_t passed as
 * void*; NULL = the null stream), allocate nothing, keep no state between calls
 * and may be issued from several host threads.
 *
 * Return value: 0 on success, a negative MOR_ERR_* code otherwise; the message of
 * the calling thread's last error is available from mor_last_error().
 */
#ifndef MOR_HIP_H_
#define MOR_HIP_H_

#include <stddef.h>
#include <stdint.h>

/* the library is built with hidden visibility: only these entry points are exported */
#define MOR_API __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

#define MOR_OK 0
#define MOR_ERR_INVALID_ARGUMENT (-1)   /* a TORCH_CHECK of the reference would have failed */
#define MOR_ERR_WORKSPACE (-2)          /* workspace missing or too small */
#define MOR_ERR_LAUNCH (-3)             /* hipGetLastError() after a launch */

/* The largest tensor an entry point takes: 2^35 elements (64 GiB of bf16).  Larger ones are refused with
 * MOR_ERR_INVALID_ARGUMENT (the scaling ops, whose element counts are 32-bit as in the reference, stop at 2^34). */
#define MOR_MAX_ELEMENTS (1ll << 35)

/* flags */
#define MOR_FLAG_DEFAULT 0u
/* Return what the reference's torch emulation returns instead of what its CUDA
 * kernel returns: nearest-even bf16 store, arithmetic power-of-two scaling (true
 * zeros), sign-preserving zeros.  The two differ only on exact rounding ties and
 * on values that quantize to zero in blocks whose amax exceeds the format maximum. */
#define MOR_FLAG_TORCH_EMULATION 1u
/* Do not use the gfx950 FP8 convert instructions; cast in integer/float software. */
#define MOR_FLAG_SOFTWARE_CAST 2u
/* MoR (FQ:487-584, 661): compute the two error sums of every block that needs them with the reference's
 * divisions and in the order of the reference's additions (its thread layout and shuffle trees), which
 * is what the kernels otherwise do only for blocks whose two sums are within 1e-5 of each other.  The
 * results are the same either way; the flag exists so that tests can compare the sums bit for bit. */
#define MOR_FLAG_REFERENCE_ORDER_SUMS 4u

/* element formats for mor_block_format / mor_quant_dequant */
#define MOR_FMT_E4M3 0
#define MOR_FMT_E5M2 1
#define MOR_FMT_E3M2 2
#define MOR_FMT_E2M3 3
/* mor_block_format only: no quantization.  The kernel that would quantize blocks of this shape reads every block,
 * finds its amax and writes the block back unchanged: what the memory system gives that kernel's access pattern
 * (a measurement aid; blocks of one row and up to 2048 elements go through the general block kernels for it). */
#define MOR_FMT_COPY (-1)

/* op ids for mor_workspace_bytes */
#define MOR_OP_FAKE_QUANTIZE 0
#define MOR_OP_BLOCK_SCALING 1
#define MOR_OP_CHANNEL_SCALING 2
#define MOR_OP_E8MX 3

MOR_API const char* mor_last_error(void);

/* Library version and the offload architecture it was built for. */
MOR_API const char* mor_version(void);

/* Bytes of device workspace an op needs for this shape (0 for ops that need none). */
MOR_API size_t mor_workspace_bytes(int op, int64_t rows, int64_t cols, int64_t block_rows, int64_t block_cols);

/*
 * fake_quantize / fake_quantize_no_alloc: FQ:1839-1907 (launch decoding FQ:1763-1835,
 * device code FQ:684-852).  mode % 10: 1 MoR, 2 block E4M3, 3 block E5M2, 4/5 current
 * scaling E4M3/E5M2 with clamp_threshold as the scale, anything else bf16 copy;
 * mode / 100 > 0 selects the dynamic-range MoR decision; sf_type 1 = fp32 scale,
 * 2 = power-of-two (E8) scale.  meta has ceil(rows/block_rows) x ceil(cols/block_cols)
 * int32 entries.  output may alias input.  Any shape is accepted (the reference
 * requires even cols and launchable block shapes).
 */
MOR_API int mor_fake_quantize(const void* input, void* output, int32_t* meta,
                      int64_t rows, int64_t cols, int64_t block_rows, int64_t block_cols,
                      double clamp_threshold, int64_t mode, int64_t sf_type,
                      uint32_t flags, void* stream);

/*
 * fake_quantize on many tensors in one call: descs[i] holds the arguments of one mor_fake_quantize
 * call (FQ:1839-1871; the reference's callers loop over their tensors, one launch each), and the
 * result of every tensor is bit for bit that call's.  descs is host memory, read before the call
 * returns.  Tensors of up to 2^18 elements share launches, 56 to a launch, one workgroup per block;
 * larger ones in whole blocks of 2048, 4096, 8192 or 16384 elements (128 x 128 tiles, rows of 4096
 * elements, ...; a forced format, or MoR on blocks of 16384 elements; default flavour, 16-byte
 * aligned) share launches of the kernel that holds a block in registers, 48 tensors to a launch; the
 * rest are forwarded to mor_fake_quantize.
 * Every descriptor is validated before anything is launched; no device memory is allocated.
 */
typedef struct MorTensorDesc {
    const void* input;
    void* output;             /* may alias input */
    int32_t* meta;
    int64_t rows, cols, block_rows, block_cols;
    double clamp_threshold;
    int64_t mode, sf_type;
} MorTensorDesc;
MOR_API int mor_fake_quantize_batch(const MorTensorDesc* descs, int64_t n, uint32_t flags, void* stream);

/*
 * Block fake quantization to one forced element format, scale fmax/amax per block as in
 * the block modes of FQ:801-823; MOR_FMT_E2M3 follows the E2M3 branch FQ:758-770
 * (software saturating cast).  The reference has no public op for a forced E2M3; this
 * entry exists for the MX E2M3 benchmark configuration and for tests.
 */
MOR_API int mor_block_format(const void* input, void* output,
                     int64_t rows, int64_t cols, int64_t block_rows, int64_t block_cols,
                     int fmt, int64_t sf_type, uint32_t flags, void* stream);

/*
 * fake_quantize_block_scaling(_inplace): FQ:2013-2230; fake_quantize_channel_scaling(_inplace):
 * FQ:2431-2660 (channel != 0; block_rows == 1 or block_cols == 1).  E4M3 with the scale
 * rule ss_mode (1 tensor-amax mantissa shared by all blocks, 2 block amax with E8 scale,
 * 3 block amax with fp32 scale, 4 tensor amax), falling back to a bf16 copy of the input
 * when the mean relative error exceeds e4m3_threshold.  Scalars meta / global_amax /
 * global_non_zero / global_error are device pointers to one element each.  output may
 * alias input (the in-place ops).  rows % block_rows == 0 and cols % block_cols == 0.
 */
MOR_API int mor_block_scaling(const void* input, void* output, int32_t* meta,
                      float* global_amax, int32_t* global_non_zero, float* global_error,
                      int64_t rows, int64_t cols, int64_t block_rows, int64_t block_cols,
                      double e4m3_threshold, int64_t ss_mode, int channel,
                      void* workspace, size_t workspace_bytes, uint32_t flags, void* stream);

/*
 * mor_block_scaling without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose
 * launchers allocate three temporaries per call (FQ:2069-2078).  The workspace is a static device array inside the
 * library, MOR_STATIC_MAX_BLOCKS * 4 + 98320 bytes on each GPU the library runs on, kept until the process ends; the
 * entry point calls no allocating routine.  Tensors of more than MOR_STATIC_MAX_BLOCKS blocks are refused with
 * MOR_ERR_WORKSPACE.  All calls on one GPU share the array: calls that overlap on one GPU (two streams, two host
 * threads) race.  The first call on a GPU looks the array's address up (hipGetSymbolAddress); make that call outside a
 * graph capture.  Results are those of mor_block_scaling, bit for bit.
 */
#define MOR_STATIC_MAX_BLOCKS (1 << 20)
MOR_API int mor_block_scaling_static(const void* input, void* output, int32_t* meta,
                             float* global_amax, int32_t* global_non_zero, float* global_error,
                             int64_t rows, int64_t cols, int64_t block_rows, int64_t block_cols,
                             double e4m3_threshold, int64_t ss_mode, int channel,
                             uint32_t flags, void* stream);

/* fake_quantize_e8mx(_inplace): FQ:2232-2397.  quantize_type 1/2/3 = E8M1/2/3;
 * scaling_strategy 1 = scale by the tensor amax, else no scale.  output may alias input. */
MOR_API int mor_e8mx(const void* input, void* output, int64_t rows, int64_t cols,
             int64_t block_rows, int64_t block_cols, int64_t quantize_type, int64_t scaling_strategy,
             void* workspace, size_t workspace_bytes, uint32_t flags, void* stream);

/* quant_dequant_e4m3/e5m2/e3m2/e2m3: FQ:1909-1964 (fp32 in, fp32 out, n elements). */
MOR_API int mor_quant_dequant(const float* input, float* output, int64_t n, int fmt, void* stream);

/* e4m3_with_e8_scale_rne / _rz: FQ:1966-2011 (fp32 in, fp32 out, n elements). */
MOR_API int mor_e4m3_with_e8_scale(const float* input, float* output, int64_t n, int rne, void* stream);

/*
 * Debug view that the public ops never return: per block amax, the fp32 scale fmax/amax
 * and its biased exponent field (the E8M0 shared exponent of the power-of-two scale,
 * FQ:251-252).  Arrays have ceil(rows/block_rows) x ceil(cols/block_cols) entries.
 */
MOR_API int mor_block_stats(const void* input, int64_t rows, int64_t cols, int64_t block_rows, int64_t block_cols,
                    float fmax, float* amax, float* scale, int32_t* e8m0, void* stream);

/* Per block {amax, min non-zero |x|, E4M3 error sum, E5M2 error sum} of the MoR decision
 * (FQ:407-584); error sums are 0 for blocks that did not need them.  4 floats per block.  The sums of a
 * block are the reference's bit for bit when they are within 1e-5 of each other, and for every block with
 * MOR_FLAG_REFERENCE_ORDER_SUMS; otherwise they agree with the reference's within 1e-6 relative. */
MOR_API int mor_mor_stats(const void* input, int64_t rows, int64_t cols, int64_t block_rows, int64_t block_cols,
                  double clamp_threshold, int64_t mode, int64_t sf_type, float* stats, uint32_t flags, void* stream);

/*
 * Exhaustive on-device comparison of the gfx950 FP8 convert instructions with the software
 * cast over all 2^32 fp32 inputs whose magnitude does not exceed the format maximum.
 * mismatches[0] = E4M3 count, mismatches[1] = E5M2 count, mismatches[2] = count of inputs for which
 * the scaled converts differ from the plain ones: the fp32 pair converts (codes of both formats in
 * one register, two values decoded at once) on the same inputs, and the power-of-two quantize step
 * through the scaled bf16 converts against its ldexp / exponent-arithmetic form for every finite bf16
 * value and every scale exponent in [-100, 100] (device pointer, 3 x uint64).
 */
MOR_API int mor_selftest_hw_cast(uint64_t* mismatches, void* stream);

/*
 * The same for the gfx950 scaled converts the MX wire format uses: the block convert of 32 bf16
 * values to packed FP6 (every finite bf16 value with every scale exponent, against the software
 * codes), its inverse, and the FP8 -> bf16 scaled convert of the dequantizer (every finite code
 * with every scale exponent it is used with).  mismatches[MOR_FMT_*] = count per element format
 * (device pointer, 4 x uint64).
 */
MOR_API int mor_selftest_hw_wire(uint64_t* mismatches, void* stream);

/*
 * The MX wire format as operands of the gfx950 scaled matrix instruction (no counterpart in the
 * reference): out [16, 16] fp32 = A x B^T for two [16, 128] tensors given as mor_mx_quantize gives
 * them (payload: 16 rows x 4 blocks of 32 codes, scales: 16 x 4 E8M0 bytes), computed by one
 * V_MFMA_SCALE_F32_16X16X128_F8F6F4 whose lanes load a block of codes and its scale byte each, with
 * no conversion in between.  Equals the product of the dequantized tensors up to the fp32
 * accumulation.  fmt = MOR_FMT_*, the same for both operands; payloads 4-byte aligned.
 */
MOR_API int mor_selftest_mx_mfma(const void* payload_a, const void* scales_a, const void* payload_b,
                                 const void* scales_b, int fmt, float* out, void* stream);

/*
 * MX wire format: the quantized tensor itself instead of its dequantized bf16 image.
 *
 * No counterpart in the reference, whose ops all return bf16 (FQ:1839-1871).  For blocks of 32
 * elements these entries emit what its MX block quantization (block modes with sf_type 2,
 * FQ:801-823; E2M3 branch FQ:758-770) computes between "quantize" and "dequantize":
 *   e8      = exponent field of fl32(fmax / amax) - 127 (FQ:251-252), limited to [-127, 127]
 *   code    = cast(x * 2^e8) in the element format, nearest even, sign of x kept
 *   scale   = one byte per block, 127 - e8: the E8M0 encoding of the multiplier 2^-e8
 * so that decode(code) * 2^(scale - 127) equals the tensor mor_fake_quantize / mor_block_format
 * return with MOR_FLAG_TORCH_EMULATION for 1 x 32 blocks and sf_type 2.  A zero block has scale
 * byte 127.  FP8 payload: one byte per element (OCP E4M3 / E5M2 encodings).  FP6 payload (E2M3 /
 * E3M2): 32 codes packed little-endian into 24 bytes, element i in bits [6i, 6i + 6) of its block.
 * cols must be a multiple of 32; tensors and payloads 16-byte aligned, scales 4-byte aligned.
 */
MOR_API size_t mor_mx_payload_bytes(int64_t rows, int64_t cols, int fmt);

/* Blocks of 32 along rows.  payload: [rows, cols * bits / 8] bytes, scales: [rows, cols / 32]. */
MOR_API int mor_mx_quantize(const void* input, void* payload, void* scales, int64_t rows, int64_t cols,
                    int fmt, void* stream);

/* Both orientations from one read of the tensor (rows and cols multiples of 32): the row-wise
 * result as above and the column-wise one (blocks of 32 along columns) stored transposed, i.e. what
 * mor_mx_quantize returns for the transposed tensor: col_payload [cols, rows * bits / 8],
 * col_scales [cols, rows / 32].  This is the pair a linear layer needs for dgrad and wgrad. */
MOR_API int mor_mx_quantize_dual(const void* input, void* row_payload, void* row_scales, void* col_payload,
                         void* col_scales, int64_t rows, int64_t cols, int fmt, void* stream);

/* payload + scales -> bf16 [rows, cols] (blocks of 32 along rows). */
MOR_API int mor_mx_dequantize(const void* payload, const void* scales, void* output, int64_t rows,
                      int64_t cols, int fmt, void* stream);

/*
 * Fake quantization of a tensor and of its transpose from one read (no counterpart in the
 * reference, whose callers run fake_quantize on x and on x.t().contiguous(), FQ:1839-1871 twice):
 *   output_rows [rows, cols], meta_rows [rows, cols / 32]  == mor_fake_quantize(x,   rows, cols, 1, 32, 0, mode, sf_type)
 *   output_cols [cols, rows], meta_cols [cols, rows / 32]  == mor_fake_quantize(x^T, cols, rows, 1, 32, 0, mode, sf_type)
 * bit for bit, for mode 2 (E4M3) or 3 (E5M2), sf_type 1 (fp32 scale) or 2 (power-of-two scale), default
 * flavour.  rows and cols multiples of 32, 16-byte aligned tensors, outputs distinct from the
 * input; either meta pointer may be NULL.
 */
MOR_API int mor_fake_quantize_dual(const void* input, void* output_rows, int32_t* meta_rows,
                                   void* output_cols, int32_t* meta_cols, int64_t rows, int64_t cols,
                                   int64_t mode, int64_t sf_type, void* stream);

/*
 * The same for 128 x 128 tiles, with MoR (no counterpart in the reference either: its callers
 * quantize x and x.t().contiguous() in two calls of fake_quantize, FQ:1839-1871):
 *   output   [rows, cols], meta   [rows / 128, cols / 128] == mor_fake_quantize(x,   rows, cols, 128, 128, clamp, mode, sf_type)
 *   output_t [cols, rows], meta_t [cols / 128, rows / 128] == mor_fake_quantize(x^T, cols, rows, 128, 128, clamp, mode, sf_type)
 * for mode % 10 in 1 (MoR), 2 (E4M3), 3 (E5M2), mode / 100 as in mor_fake_quantize, default flavour.
 * A tile and its transpose hold the same elements, so they share amax, scale and format: the tile is
 * quantized once and stored twice.  (MoR compares two fp32 error sums; the call on x^T adds the same
 * terms in another order, so a tile whose two sums agree to the last bits could come out in the other
 * format there: for tiles whose sums are that close both are added again in the reference's two
 * orders, and each orientation gets the decision, and the values, of its own call.  The one exception
 * is a tile whose scale is outside 2^+-90: there the decision of the call on x stands for both.)
 * rows and cols multiples of 128 and below 2^27; three different 16-byte aligned tensors.
 */
MOR_API int mor_fake_quantize_dual_tiles(const void* input, void* output, int32_t* meta, void* output_t,
                                         int32_t* meta_t, int64_t rows, int64_t cols, double clamp_threshold,
                                         int64_t mode, int64_t sf_type, void* stream);

/*
 * The MoR decision per 128 x 128 tile with the tile's codes as the result, and the way back (no
 * counterpart in the reference, which only ever materialises the fake-quantized bf16 values,
 * FQ:733-851; this is what a real low-precision GEMM after the MoR decision would read):
 *   tags   [rows / 128, cols / 128] int32: the meta value mor_fake_quantize(input, rows, cols, 128, 128,
 *          clamp_threshold, mode, 1) gives the tile (1 / 11 E4M3, 2 / 12 E5M2, 3 BF16, 4 E2M3).  A tile
 *          whose scale is outside 2^-90 .. 2^90 or that holds a NaN has MOR_TILE_STORED_BF16 ORed in.
 *   scales [rows / 128, cols / 128] float: the tile's fp32 scale fmax / amax (FQ:297-304); 1 for a
 *          BF16 tile, a tile stored as bf16 and an all-zero tile.
 *   payload: MOR_TILE_PAYLOAD_BYTES per tile, tile after tile in row-major tile order.  A tile
 *          holds its 128 rows packed: E4M3 / E5M2 128 bytes per row (one code per element: the
 *          OCP code of |x| * scale, the sign of x in bit 7); E2M3 96 bytes per row (6-bit codes,
 *          dense little-endian, code k at bits 6k; a zero result has no sign, as the reference's
 *          software cast gives +0 -- except in an all-zero tile, which the reference copies: its
 *          zeros keep their signs); BF16 (and MOR_TILE_STORED_BF16) 256 bytes per row: the bf16
 *          values mor_fake_quantize writes for the tile.  The rest of a tile's slot is not written.
 * mor_mor_dequantize gives the output of that mor_fake_quantize call bit for bit: value of the code,
 * divided by the scale (IEEE), rounded to bf16 half-up (FQ:312-316).
 * mode % 10: 1 (MoR), or 2 / 3: every tile E4M3 / E5M2 with its own fp32 scale (block scaling in 128 x 128
 * tiles: tags 1 / 2); mode / 100 as in mor_fake_quantize; default flavour, fp32 scales.
 * rows and cols multiples of 128 and below 2^27, at most 2^30 tiles; tensor and payload 16-byte aligned,
 * different buffers.
 */
#define MOR_TILE_PAYLOAD_BYTES 32768
#define MOR_TILE_STORED_BF16 0x100
MOR_API int mor_mor_quantize(const void* input, void* payload, int32_t* tags, float* scales, int64_t rows,
                             int64_t cols, double clamp_threshold, int64_t mode, void* stream);
MOR_API int mor_mor_dequantize(const void* payload, const int32_t* tags, const float* scales, void* output,
                               int64_t rows, int64_t cols, void* stream);

/*
 * The tile codes of the transposed tensor from the tile codes of the tensor (no counterpart in the
 * reference, whose callers quantize x.t().contiguous() in a call of its own): tile (i, j) of
 * [tile_rows, tile_cols] tiles becomes tile (j, i) of [tile_cols, tile_rows] tiles with its codes
 * transposed; tags and scales move with it (a tile and its transpose hold the same elements, so they
 * share format and scale; only for a MoR tile whose two error sums agree to their last bits can
 * mor_mor_quantize of the transposed tensor, which adds them in another order, choose the other format).
 * mor_mor_dequantize of the result is the transpose of mor_mor_dequantize of the source, bit for bit.  Source and destination are different buffers; payloads 16-byte aligned;
 * tile_rows and tile_cols at most 2^20, their product at most 2^30.
 */
MOR_API int mor_mor_transpose(const void* payload, const int32_t* tags, const float* scales, void* payload_t,
                              int32_t* tags_t, float* scales_t, int64_t tile_rows, int64_t tile_cols, void* stream);

/*
 * mor_mor_quantize and mor_mor_transpose of its result in one call (no counterpart in the
 * reference): payload / tags / scales as mor_mor_quantize writes them, payload_t / tags_t / scales_t
 * as mor_mor_transpose writes them.  Every output its own buffer.
 */
MOR_API int mor_mor_quantize_dual(const void* input, void* payload, int32_t* tags, float* scales, void* payload_t,
                                  int32_t* tags_t, float* scales_t, int64_t rows, int64_t cols,
                                  double clamp_threshold, int64_t mode, void* stream);

#ifdef __cplusplus
}
#endif
#endif
