// mor_selftest_mx_mfma: the MX wire format (mor_mx_quantize) as the operands of the gfx950 scaled matrix instruction.
// One wave multiplies A [16, 128] by B^T (B [16, 128]) with V_MFMA_SCALE_F32_16X16X128_F8F6F4 straight from the
// payload and scale bytes.  The instruction's operand layout (found by probing it: single non-zero codes and single
// changed scales), for lane l = 16 g + r and row r:
//   8-bit codes: the 16 codes of columns 16 g .. 16 g + 15 and the 16 codes of columns 64 + 16 g ..., as the two
//                halves of the lane's 8 registers;
//   6-bit codes: the 32 codes of columns 32 g .. 32 g + 31, 24 bytes packed as the wire format packs them;
//   the scale of the 32 columns 32 b .. 32 b + 31 of row r is taken from lane 16 b + r.
// All of these are plain loads from the wire format: half an MX block twice or a whole one, and one E8M0 byte.
// A test of the format, not a GEMM.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mor_common.h"
#include "mor_host.h"
#include "../../include/mor_hip.h"

namespace mor {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

// HWF: the instruction's format code (0 E4M3, 1 E5M2, 2 E2M3, 3 E3M2); BYTES per block of 32 codes (32 or 24)
template <int HWF, int BYTES>
__global__ __launch_bounds__(64) void k_mx_mfma_16x16x128(const uint8_t* pa, const uint8_t* sa, const uint8_t* pb,
                                                          const uint8_t* sb, float* out) {
    const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    v8i a = {0, 0, 0, 0, 0, 0, 0, 0}, b = {0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (BYTES == 32) {
        // columns 16 g ...: block g / 2, half g % 2; columns 64 + 16 g ...: block 2 + g / 2, the same half
        const int first = (r * 4 + (g >> 1)) * 32 + (g & 1) * 16, second = first + 64;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[i] = (int)*reinterpret_cast<const uint32_t*>(pa + first + 4 * i);
            a[4 + i] = (int)*reinterpret_cast<const uint32_t*>(pa + second + 4 * i);
            b[i] = (int)*reinterpret_cast<const uint32_t*>(pb + first + 4 * i);
            b[4 + i] = (int)*reinterpret_cast<const uint32_t*>(pb + second + 4 * i);
        }
    } else {
        const int at = (r * 4 + g) * 24;
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            a[i] = (int)*reinterpret_cast<const uint32_t*>(pa + at + 4 * i);
            b[i] = (int)*reinterpret_cast<const uint32_t*>(pb + at + 4 * i);
        }
    }
    const int scale_a = sa[r * 4 + g], scale_b = sb[r * 4 + g];          // lane 16 b + r: the scale of block b of row r
    v4f c = {0.0f, 0.0f, 0.0f, 0.0f};
    c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, HWF, HWF, 0, scale_a, 0, scale_b);
    // lane l holds rows 4 * (l / 16) .. + 3 of column l % 16
#pragma unroll
    for (int j = 0; j < 4; ++j) out[(4 * g + j) * 16 + r] = c[j];
}

}  // namespace mor

using namespace mor;

extern "C" int mor_selftest_mx_mfma(const void* payload_a, const void* scales_a, const void* payload_b, const void* scales_b,
                                    int fmt, float* out, void* stream) {
    if (!payload_a || !scales_a || !payload_b || !scales_b || !out) return mor_fail(MOR_ERR_INVALID_ARGUMENT, "NULL pointer");
    if ((reinterpret_cast<uintptr_t>(payload_a) | reinterpret_cast<uintptr_t>(payload_b)) & 3u)
        return mor_fail(MOR_ERR_INVALID_ARGUMENT, "payloads must be 4-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint8_t* pa = static_cast<const uint8_t*>(payload_a);
    const uint8_t* sa = static_cast<const uint8_t*>(scales_a);
    const uint8_t* pb = static_cast<const uint8_t*>(payload_b);
    const uint8_t* sb = static_cast<const uint8_t*>(scales_b);
    switch (fmt) {
        case MOR_FMT_E4M3: k_mx_mfma_16x16x128<0, 32><<<1, 64, 0, st>>>(pa, sa, pb, sb, out); break;
        case MOR_FMT_E5M2: k_mx_mfma_16x16x128<1, 32><<<1, 64, 0, st>>>(pa, sa, pb, sb, out); break;
        case MOR_FMT_E2M3: k_mx_mfma_16x16x128<2, 24><<<1, 64, 0, st>>>(pa, sa, pb, sb, out); break;
        case MOR_FMT_E3M2: k_mx_mfma_16x16x128<3, 24><<<1, 64, 0, st>>>(pa, sa, pb, sb, out); break;
        default: return mor_fail(MOR_ERR_INVALID_ARGUMENT, "unknown format %d", fmt);
    }
    return mor_check_launch("k_mx_mfma_16x16x128");
}
