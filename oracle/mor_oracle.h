/*
 * CPU oracle for the MoR fake-quantization hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the arithmetic of the reference CUDA file
 * mor/csrc/cuda/fake_quantize.cu (abbreviated FQ below).  It exists so that the
 * HIP kernels can be checked bit for bit on a CPU.  Nothing in the shipped
 * library links, imports or calls it; only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may.
 *
 * Every function names the reference lines it follows.  Parity status:
 *   - bf16<->fp32, software casts, E8/FP32 scale-quantize-dequantize-descale,
 *     amax / min-nonzero / nnz, MoR selection, block/channel scaling, e8mx:
 *     pinned by the reference's own fixtures and by torch.float8 CPU casts
 *     (see tests/test_oracle_*.py).
 *   - mor_oracle_cast_hw outside the finite range (saturation, NaN payloads,
 *     sign of an underflowed zero): follows the text of NVIDIA's cuda_fp8.hpp
 *     (__nv_cvt_double_to_fp8, __NV_SATFINITE), a third-party header that the
 *     reference includes but does not vendor.  PARITY UNPINNED for those inputs.
 *   - NaN / Inf tensor elements: the reference result depends on NVIDIA NaN
 *     payloads and on device asserts.  PARITY UNPINNED.
 */
#ifndef MOR_ORACLE_H_
#define MOR_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element formats of the software cast, FQ:72-122 */
enum { MOR_O_E4M3 = 0, MOR_O_E5M2 = 1, MOR_O_E3M2 = 2, MOR_O_E2M3 = 3 };

/* flavour: 0 = what the CUDA kernel returns (round-half-up bf16 store,
 * exponent-field E8 scaling, +0 from the software cast); 1 = what the
 * reference's torch emulation in test/ returns (round-to-nearest-even store,
 * arithmetic E8 scaling, torch float8 overflow rules). */
enum { MOR_O_KERNEL = 0, MOR_O_EMU = 1 };

/* scalar pieces (exported so tests can pin them one by one) */
float    mor_oracle_bf16_to_fp32(uint32_t v);                 /* FQ:38-44  */
uint32_t mor_oracle_fp32_to_bf16(float v);                    /* FQ:46-60  */
uint32_t mor_oracle_fp32_to_bf16_rne(float v);                /* torch .type(bfloat16) */
float    mor_oracle_cast_sw(float v, int fmt);                /* FQ:125-215 */
float    mor_oracle_cast_hw(float v, int fmt);                /* FQ:223-227 + cuda_fp8.hpp */
float    mor_oracle_sqdd_e8(float v, float sf, int rne, int fmt, int use_hw);   /* FQ:248-306 */
float    mor_oracle_sqdd_fp32(float v, float sf, int fmt, int use_hw);          /* FQ:310-316 */
float    mor_oracle_scaling_factor(float global_amax, float block_amax, int ss_mode); /* FQ:1059-1093 */
float    mor_oracle_e8m(float v, int mbits);                  /* FQ:1243-1327 */
float    mor_oracle_e8mx_scaling_factor(float global_amax, int mbits, int strategy); /* FQ:1335-1359 */

/* the two per-element terms |q / x - 1| of the MoR error sums (FQ:504-542) for n elements of a block with the
 * given amax; e8: power-of-two scale */
void mor_oracle_mor_error_terms(const uint16_t* x, size_t n, float amax, int e8, int flavour, float* e4, float* e5);

/* vectorised scalar pieces */
void mor_oracle_cast_sw_n(const float* in, float* out, size_t n, int fmt);
void mor_oracle_cast_hw_n(const float* in, float* out, size_t n, int fmt);

/* FQ:684-852 + FQ:1763-1871.  meta has ceil(rows/brows) x ceil(cols/bcols)
 * entries.  stats (optional, may be NULL) receives 4 floats per block: amax,
 * amin, e4m3 error sum, e5m2 error sum (error sums are 0 when not computed). */
int mor_oracle_fake_quantize(const uint16_t* in, uint16_t* out, int32_t* meta,
                             int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                             float clamp_threshold, int64_t mode, int64_t sf_type,
                             int flavour, float* stats);

/* Block fake-quant with a forced element format (E2M3 included), the scale
 * rule of quantize_kernel's block modes (FQ:801-823, and FQ:758-770 for E2M3):
 * fmax/amax per block, E8 or FP32.  meta is not written. */
int mor_oracle_block_format(const uint16_t* in, uint16_t* out,
                            int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                            int fmt, int64_t sf_type, int flavour);

/* FQ:951-1241 + FQ:2013-2120 (block) and FQ:1459-1752 + FQ:2431-2544 (channel):
 * the arithmetic is the same, only the reduction geometry differs.  channel != 0
 * selects the channel geometry for the order of the error sum.  out may alias in. */
int mor_oracle_block_scaling(const uint16_t* in, uint16_t* out, int32_t* meta,
                             float* global_amax, int32_t* global_non_zero, float* global_error,
                             int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                             float e4m3_threshold, int64_t ss_mode, int channel, int flavour);

/* FQ:1361-1428 + FQ:2232-2313.  out may alias in. */
int mor_oracle_e8mx(const uint16_t* in, uint16_t* out, int64_t rows, int64_t cols,
                    int64_t brows, int64_t bcols, int64_t quantize_type, int64_t scaling_strategy,
                    int flavour);

/* FQ:854-875: fp32 elementwise test ops */
void mor_oracle_quant_dequant(const float* in, float* out, size_t n, int fmt);
void mor_oracle_e4m3_with_e8_scale(const float* in, float* out, size_t n, int rne);

/* per-block debug view: amax, fp32 scale (fmax/amax) and biased E8M0 exponent */
int mor_oracle_block_stats(const uint16_t* in, int64_t rows, int64_t cols, int64_t brows,
                           int64_t bcols, float fmax, float* amax, float* scale, int32_t* e8m0);

/* MX wire format (no counterpart in the reference, which returns only the dequantized tensor):
 * blocks of 32 elements along a row, payload = element codes (FP8: one byte each, FP6: 4 codes in
 * 3 bytes, little-endian), scales = one E8M0 byte per block (127 - e8, the decode multiplier). */
int mor_oracle_mx_quantize(const uint16_t* in, uint8_t* payload, uint8_t* scales,
                           int64_t rows, int64_t cols, int fmt);
int mor_oracle_mx_dequantize(const uint8_t* payload, const uint8_t* scales, uint16_t* out,
                             int64_t rows, int64_t cols, int fmt);

int mor_oracle_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
