// The code formats of the wire kernels (MX blocks, MoR tiles): code widths and biases, the value of a 6-bit code,
// and the 6-bit magnitude codes of scaled magnitudes through the FP8 converts.
#pragma once

#include "mor_device.h"

namespace mor {

template <int F> struct Wire {
    static constexpr int bits = Fmt<F>::hw ? 8 : 6;
    static constexpr int bias = (F == FMT_E4M3) ? 7 : (F == FMT_E5M2) ? 15 : (F == FMT_E3M2) ? 3 : 1;
};

// value of a 5-bit magnitude code of F
template <int F> __device__ __forceinline__ float fp6_value(uint32_t mag) {
    constexpr int mb = Fmt<F>::mbits, bias = Wire<F>::bias;
    const uint32_t e = mag >> mb, m = mag & ((1u << mb) - 1u);
    const float sub = (float)m * (1.0f / (float)(1 << (mb + bias - 1)));
    const float normal = u2f(((e + 127u - bias) << 23) | (m << (23 - mb)));
    return e == 0 ? sub : normal;
}

// 5-bit magnitude codes of two scaled magnitudes a, b (not above fmax) in the 6-bit format F, through the FP8 converts:
// E2M3 / E3M2 have the mantissa width of E4M3 / E5M2, so for a magnitude in the normal range of the 6-bit format the
// 8-bit code differs from the 6-bit one by the bias difference only; below that range the 6-bit grid is uniform (step
// = its subnormal step), which is the 8-bit grid of the binade [norm_min, 2 norm_min): convert a + norm_min instead
// (the sum is exact whenever the rounding can depend on it).
template <int F> __device__ __forceinline__ void fp6_mag_codes(float a, float b, uint32_t& ca, uint32_t& cb) {
    static_assert(!Fmt<F>::hw, "6-bit formats");
    constexpr int F8 = (F == FMT_E2M3) ? FMT_E4M3 : FMT_E5M2;
    constexpr int mb = Fmt<F>::mbits;
    constexpr float norm_min = (F == FMT_E2M3) ? 1.0f : 0.25f;
    constexpr uint32_t off_normal = (uint32_t)(Wire<F8>::bias - Wire<F>::bias) << mb;
    constexpr uint32_t off_sub = (uint32_t)(1 - Wire<F>::bias + Wire<F8>::bias) << mb;
    const bool na = a >= norm_min, nb = b >= norm_min;
    const uint32_t p = hw_pack2<F8>(na ? a : a + norm_min, nb ? b : b + norm_min);
    ca = (p & 0xFFu) - (na ? off_normal : off_sub);
    cb = ((p >> 8) & 0xFFu) - (nb ? off_normal : off_sub);
}

}  // namespace mor
