/*
 * CPU oracle for the MoR fake-quantization hot path -- TEST INFRASTRUCTURE ONLY.
 * See mor_oracle.h for scope and parity status.  "FQ" = the reference file
 * mor/csrc/cuda/fake_quantize.cu.
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off -fopenmp -shared -fPIC
 * (x86-64 SSE float arithmetic is IEEE single: the divisions below are the
 * correctly rounded fp32 divisions the CUDA kernel performs).
 */
#include "mor_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* NVIDIA GPUs return this pattern for an fp32 NaN produced by arithmetic. */
#define NV_CANONICAL_NAN 0x7fffffffu
static inline float nv_canon(float r) { return (r != r) ? u2f(NV_CANONICAL_NAN) : r; }
/* fmaxf/fminf of CUDA: a NaN operand is ignored. */
static inline float max_nn(float a, float b) { return (a != a) ? b : (b != b) ? a : (a > b ? a : b); }
static inline float min_nn(float a, float b) { return (a != a) ? b : (b != b) ? a : (a < b ? a : b); }

int mor_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ */
/* FQ:38-44 */
float mor_oracle_bf16_to_fp32(uint32_t value) {
    uint32_t sign = (value >> 15) & 0x1;
    uint32_t exponent = (value >> 7) & 0xFF;
    uint32_t mantissa = value & 0x7F;
    return u2f((sign << 31) | (exponent << 23) | (mantissa << 16));
}

/* FQ:46-60: round half up on the magnitude; the exponent may reach 256, in
 * which case the shifted field lands on bit 15 (NaN 0x7fffffff -> 0x8000). */
uint32_t mor_oracle_fp32_to_bf16(float value) {
    uint32_t bits = f2u(value);
    uint32_t sign = (bits >> 31) & 0x1;
    uint32_t exponent = (bits >> 23) & 0xFF;
    uint32_t mantissa = (bits >> 16) & 0x7F;
    uint32_t extra = (bits >> 15) & 0x1;
    if (extra == 1) {
        mantissa++;
        if (mantissa == 128) { exponent++; mantissa = 0; }
    }
    return ((sign << 15) | (exponent << 7) | mantissa) & 0xFFFFu;
}

/* torch's fp32 -> bfloat16 (round to nearest even, NaN -> quiet NaN) */
uint32_t mor_oracle_fp32_to_bf16_rne(float value) {
    uint32_t bits = f2u(value);
    if (value != value) return ((bits >> 16) & 0x8000u) | 0x7FC0u;
    uint32_t lsb = (bits >> 16) & 1u;
    bits += 0x7FFFu + lsb;
    return bits >> 16;
}

static inline uint32_t store_bf16(float v, int flavour) {
    return flavour == MOR_O_EMU ? mor_oracle_fp32_to_bf16_rne(v) : mor_oracle_fp32_to_bf16(v);
}

/* ------------------------------------------------------------------ */
/* format traits, FQ:72-122 */
typedef struct { uint32_t ebits, bias, before_overflow, mbits, shift, carry; int saturating; } fmt_t;
static const fmt_t FMT[4] = {
    /* E4M3 */ {4, 7, 15, 3, 20, 8, 0},
    /* E5M2 */ {5, 15, 30, 2, 21, 4, 0},
    /* E3M2 */ {3, 3, 7, 2, 21, 4, 1},
    /* E2M3 */ {2, 1, 3, 3, 20, 8, 1},
};

/* FQ:125-215: software cast fp32 -> {E4M3,E5M2,E3M2,E2M3} -> fp32 */
float mor_oracle_cast_sw(float fp32_value, int fmt) {
    const fmt_t* F = &FMT[fmt];
    uint32_t bits = f2u(fp32_value);
    uint32_t sign = (bits >> 31) & 0x1;
    int32_t exponent = (int32_t)((bits >> 23) & 0xFF) - 127 + (int32_t)F->bias;
    uint32_t mantissa = 0;
    uint32_t guard = 0, sticky = 0;
    const uint32_t mmask = (1u << F->mbits) - 1u;

    if (exponent > 0) {
        mantissa = (bits >> F->shift) & mmask;
        guard = (bits >> (F->shift - 1)) & 0x1;
        sticky = (bits & ((1u << (F->shift - 1)) - 1u)) != 0;
    } else {
        uint32_t rshift = (uint32_t)(1 - exponent);
        exponent = 0;
        if (rshift <= F->mbits + 1) {
            mantissa = (bits & 0x7fffffu) | (1u << 23);
            sticky = (mantissa & ((1u << (rshift + F->shift - 1)) - 1u)) != 0;
            mantissa >>= rshift;
            guard = (mantissa >> (F->shift - 1)) & 0x1;
            mantissa = (mantissa >> F->shift) & mmask;
        } else {
            mantissa = 0;
        }
    }
    if (guard == 1) {
        if (sticky == 1 || (mantissa & 1u)) {
            mantissa++;
            if (mantissa == F->carry) { mantissa = 0; exponent++; }
        }
    }
    if (F->saturating) {
        if (exponent > (int32_t)F->before_overflow) {
            exponent = (int32_t)((1u << F->ebits) - 1u);
            mantissa = mmask;
        }
    } else {
        if (exponent > (int32_t)F->before_overflow) return u2f(NV_CANONICAL_NAN);
        if (exponent == (int32_t)F->before_overflow && fmt == MOR_O_E4M3 && mantissa == F->carry - 1)
            return u2f(NV_CANONICAL_NAN);
    }
    uint32_t new_bits = 0;
    if (exponent > 0) {
        exponent += 127 - (int32_t)F->bias;
        new_bits = (sign << 31) | ((uint32_t)exponent << 23) | (mantissa << F->shift);
    } else if (mantissa) {
        exponent += 127 - (int32_t)F->bias + 1;
        const uint32_t top = 1u << F->mbits;
        while ((mantissa & top) == 0) { mantissa <<= 1; exponent--; }
        mantissa &= mmask;
        new_bits = (sign << 31) | ((uint32_t)exponent << 23) | (mantissa << F->shift);
    }
    return u2f(new_bits);
}

/* Exact round-to-nearest-even onto the grid of a small float format, written
 * independently of mor_oracle_cast_sw (value-based, not field-based) so that the
 * two can pin each other.  Returns the magnitude; *over is set when the rounded
 * magnitude exceeds max_finite. */
static float rne_to_grid(float mag, int mbits, int emin, float max_finite, int* over) {
    *over = 0;
    if (mag == 0.0f) return 0.0f;
    int e;
    (void)frexpf(mag, &e);            /* mag = m * 2^e, m in [0.5,1) */
    int ex = e - 1;                   /* mag in [2^ex, 2^(ex+1)) */
    if (ex < emin) ex = emin;
    float quantum = ldexpf(1.0f, ex - mbits);
    /* mag / quantum is exact (power of two) and < 2^24 for every caller */
    float scaled = mag / quantum;
    float r = nearbyintf(scaled);     /* default rounding mode: nearest even */
    float q = r * quantum;
    if (q > max_finite) *over = 1;
    return q;
}

/* Model of static_cast<__nv_fp8_e4m3/e5m2>(float) -> float, FQ:223-227, after
 * the text of __nv_cvt_double_to_fp8 (cuda_fp8.hpp) with __NV_SATFINITE. */
float mor_oracle_cast_hw(float v, int fmt) {
    uint32_t bits = f2u(v);
    uint32_t sign = bits & 0x80000000u;
    if (v != v) return u2f(NV_CANONICAL_NAN);
    float mag = fabsf(v);
    float max_finite = (fmt == MOR_O_E4M3) ? 448.0f : 57344.0f;
    int over;
    float q;
    if (isinf(mag)) { q = max_finite; }
    else {
        q = rne_to_grid(mag, fmt == MOR_O_E4M3 ? 3 : 2, fmt == MOR_O_E4M3 ? -6 : -14, max_finite, &over);
        if (over) q = max_finite;
    }
    return u2f(f2u(q) | sign);
}

/* torch's float -> float8_e4m3fn / float8_e5m2 -> float on the CPU */
static float cast_torch(float v, int fmt) {
    uint32_t sign = f2u(v) & 0x80000000u;
    if (v != v) return u2f(0x7fc00000u | sign);
    float mag = fabsf(v);
    float max_finite = (fmt == MOR_O_E4M3) ? 448.0f : 57344.0f;
    int over = 0;
    float q;
    if (isinf(mag)) over = 1;
    else q = rne_to_grid(mag, fmt == MOR_O_E4M3 ? 3 : 2, fmt == MOR_O_E4M3 ? -6 : -14, max_finite, &over);
    if (over) q = (fmt == MOR_O_E4M3) ? u2f(0x7fc00000u) : INFINITY;
    return u2f(f2u(q) | sign);
}

/* FQ:218-245 dispatch */
static float cast_any(float v, int fmt, int use_hw, int flavour) {
    if (flavour == MOR_O_EMU) {
        if (fmt == MOR_O_E4M3 || fmt == MOR_O_E5M2) return cast_torch(v, fmt);
        float r = mor_oracle_cast_sw(v, fmt);
        if (r == 0.0f) r = u2f(f2u(v) & 0x80000000u);
        return r;
    }
    if (use_hw) return mor_oracle_cast_hw(v, fmt);
    return mor_oracle_cast_sw(v, fmt);
}

void mor_oracle_cast_sw_n(const float* in, float* out, size_t n, int fmt) {
    for (size_t i = 0; i < n; ++i) out[i] = mor_oracle_cast_sw(in[i], fmt);
}
void mor_oracle_cast_hw_n(const float* in, float* out, size_t n, int fmt) {
    for (size_t i = 0; i < n; ++i) out[i] = mor_oracle_cast_hw(in[i], fmt);
}

/* ------------------------------------------------------------------ */
/* FQ:248-306 */
static float sqdd_e8(float value, float sf, int rne, int fmt, int use_hw, int flavour) {
    uint32_t sf_bits = f2u(sf);
    int32_t e8 = (int32_t)((sf_bits >> 23) & 0xFF) - 127;
    uint32_t vb = f2u(value);
    uint32_t vsign = (vb >> 31) & 0x1;
    int32_t vexp = (int32_t)((vb >> 23) & 0xFF);
    uint32_t vman = vb & 0x7fffffu;

    if (rne) {
        uint32_t sman = sf_bits & 0x7fffffu;
        uint32_t guard = (sman >> 22) & 0x1;
        uint32_t sticky = (sman & ((1u << 22) - 1u)) != 0;
        if (guard == 1 && vman <= 6815744u && vexp + e8 < 135) {
            uint32_t lsb = (uint32_t)e8 & 0x1;
            if (sticky == 1 || lsb == 1) e8++;
        }
    }
    if (flavour == MOR_O_EMU) {
        /* x * 2^e8, cast, / 2^e8 in fp32 arithmetic (test_fake_quantize.py:41-46) */
        float p = ldexpf(1.0f, e8);
        float scaled = value * p;
        float dq = cast_any(scaled, fmt, use_hw, flavour);
        return dq / p;
    }
    vexp += e8;
    if (vexp < 0) vexp = 0;
    float scaled = u2f((vsign << 31) | ((uint32_t)vexp << 23) | vman);
    float dq = cast_any(scaled, fmt, use_hw, flavour);
    uint32_t db = f2u(dq);
    uint32_t dsign = (db >> 31) & 0x1;
    int32_t dexp = (int32_t)((db >> 23) & 0xFF);
    uint32_t dman = db & 0x7fffffu;
    dexp -= e8;
    if (dexp < 0) dexp = 0;
    return u2f((dsign << 31) | ((uint32_t)dexp << 23) | dman);
}

float mor_oracle_sqdd_e8(float v, float sf, int rne, int fmt, int use_hw) {
    return sqdd_e8(v, sf, rne, fmt, use_hw, MOR_O_KERNEL);
}

/* FQ:310-316 */
static float sqdd_fp32(float value, float sf, int fmt, int use_hw, int flavour) {
    float scaled = value * sf;
    float dq = cast_any(scaled, fmt, use_hw, flavour);
    float r = dq / sf;
    return flavour == MOR_O_EMU ? r : nv_canon(r);
}

float mor_oracle_sqdd_fp32(float v, float sf, int fmt, int use_hw) {
    return sqdd_fp32(v, sf, fmt, use_hw, MOR_O_KERNEL);
}

/* FQ:319-379: production wrappers.  E4M3/E5M2 use the hardware cast and E8_RZ,
 * E2M3 uses the software cast. */
static float sqdd(float v, float sf, int fmt, int e8, int flavour) {
    int use_hw = (fmt == MOR_O_E4M3 || fmt == MOR_O_E5M2);
    return e8 ? sqdd_e8(v, sf, 0, fmt, use_hw, flavour) : sqdd_fp32(v, sf, fmt, use_hw, flavour);
}

static const float FMAX_OF[4] = {448.0f, 57344.0f, 28.0f, 7.5f};

/* ------------------------------------------------------------------ */
/* Reduction-order helpers: the reference sums per-thread partials with a
 * 32-lane shuffle-down tree, then the per-warp results with the same tree
 * (FQ:399-405, 546-583, 917-948).  partial[] is indexed by flattened thread id. */
static float warp_tree(const float* v32) {
    float v[32];
    memcpy(v, v32, sizeof v);
    for (int off = 16; off > 0; off >>= 1)
        for (int i = 0; i < 32; ++i) {
            /* lanes past the end read their own value, as __shfl_down_sync does */
            float other = (i + off < 32) ? v[i + off] : v[i];
            v[i] = v[i] + other;
        }
    return v[0];
}

/* valid only when nthreads is a multiple of 32 and nthreads/32 <= 32 */
static float block_tree_sum(const float* partial, int nthreads) {
    int nw = nthreads / 32;
    float w[32];
    for (int i = 0; i < 32; ++i) w[i] = 0.0f;
    for (int i = 0; i < nw; ++i) w[i] = warp_tree(partial + 32 * i);
    return warp_tree(w);
}

/* ------------------------------------------------------------------ */
typedef struct {
    const uint16_t* in;
    int64_t rows, cols, brows, bcols;
    int64_t r0, r1, c0, c1;   /* element bounds of this block */
} blk_t;

static inline float ld(const blk_t* b, int64_t r, int64_t c) {
    return mor_oracle_bf16_to_fp32(b->in[r * b->cols + c]);
}

/* FQ:407-485 */
static void block_amax_amin(const blk_t* b, float* amax_o, float* amin_o) {
    float bf16_max = mor_oracle_bf16_to_fp32(0x7F7F);
    float amax = 0.0f, amin = bf16_max;
    for (int64_t r = b->r0; r < b->r1; ++r)
        for (int64_t c = b->c0; c < b->c1; ++c) {
            float a = fabsf(ld(b, r, c));
            amax = max_nn(amax, a);
            if (a > 0) amin = min_nn(amin, a);
        }
    *amax_o = amax;
    *amin_o = amin;
}

/* one element's contribution to FQ:504-542 */
static inline void err_terms(float x, float amax, int e8, int flavour, float* e4, float* e5) {
    float s4 = 448.0f / amax;
    float s5 = 57344.0f / amax;
    float q4 = sqdd(x, s4, MOR_O_E4M3, e8, flavour);
    float q5 = sqdd(x, s5, MOR_O_E5M2, e8, flavour);
    *e4 = 0.0f; *e5 = 0.0f;
    if (x != 0.0f) { *e4 = fabsf((q4 / x) - 1.0f); *e5 = fabsf((q5 / x) - 1.0f); }
}

/* FQ:487-584.  When the reference launch geometry exists for this block shape
 * (even cols and block cols, thread block a multiple of 32, FQ:1770-1789) the
 * float additions are made in its order; otherwise row-major sequential. */
static void block_error(const blk_t* b, float amax, int e8, int flavour, float* e4_o, float* e5_o) {
    int64_t tbx = 16, tby = 32;
    int geom = (b->cols % 2 == 0) && (b->bcols % 2 == 0);
    if (b->brows * b->bcols > 1024) {
        if (b->bcols < 32 || b->brows < 32) geom = 0;
    } else {
        tbx = b->bcols / 2; tby = b->brows;
    }
    int64_t nthreads = tbx * tby;
    if (nthreads <= 0 || nthreads % 32 != 0 || nthreads > 1024) geom = 0;
    if (!geom) {
        /* no reference launch geometry exists for this shape, hence no reference order: the fp32 terms are
         * added in double and rounded once */
        double s4 = 0.0, s5 = 0.0;
        for (int64_t r = b->r0; r < b->r1; ++r)
            for (int64_t c = b->c0; c < b->c1; ++c) {
                float e4, e5;
                err_terms(ld(b, r, c), amax, e8, flavour, &e4, &e5);
                s4 += e4; s5 += e5;
            }
        *e4_o = (float)s4; *e5_o = (float)s5;
        return;
    }
    float p4[1024], p5[1024];
    int64_t pc0 = b->c0 / 2, pc1 = b->c1 / 2;   /* packed column bounds */
    for (int64_t ty = 0; ty < tby; ++ty)
        for (int64_t tx = 0; tx < tbx; ++tx) {
            float s4 = 0.0f, s5 = 0.0f;
            for (int64_t r = b->r0 + ty; r < b->r1; r += tby)
                for (int64_t pc = pc0 + tx; pc < pc1; pc += tbx) {
                    float a4, a5, b4, b5;
                    /* value1 = high half = odd column, value2 = low half */
                    err_terms(ld(b, r, 2 * pc + 1), amax, e8, flavour, &a4, &a5);
                    err_terms(ld(b, r, 2 * pc), amax, e8, flavour, &b4, &b5);
                    s4 += (a4 + b4);
                    s5 += (a5 + b5);
                }
            p4[ty * tbx + tx] = s4;
            p5[ty * tbx + tx] = s5;
        }
    *e4_o = block_tree_sum(p4, (int)nthreads);
    *e5_o = block_tree_sum(p5, (int)nthreads);
}

/* The per-element terms of FQ:504-542 for n elements of a block whose amax is given (what block_error adds up):
 * exported so that tests can construct blocks whose two sums meet. */
void mor_oracle_mor_error_terms(const uint16_t* x, size_t n, float amax, int e8, int flavour, float* e4, float* e5) {
    for (size_t i = 0; i < n; ++i) err_terms(mor_oracle_bf16_to_fp32(x[i]), amax, e8, flavour, &e4[i], &e5[i]);
}

/* MorQuantType, FQ:600-608 */
enum { Q_UNKNOWN = 0, Q_E4M3 = 1, Q_E5M2 = 2, Q_BF16 = 3, Q_E2M3 = 4, Q_E4M3_SMALL = 11, Q_E5M2_SMALL = 12 };

/* FQ:610-682 */
static int choose_mor(const blk_t* b, float clamp, int dynamic_range_mode, int e8, int flavour,
                      float amax, float amin, float* e4_o, float* e5_o) {
    float range = 0.0f;
    *e4_o = 0.0f; *e5_o = 0.0f;
    if (amax == 0.0f) { amax = clamp; range = 1.0f; }
    if (range == 0.0f) range = amax / amin;
    uint32_t e4m3_range = 28672u;
    if (!dynamic_range_mode) e4m3_range *= 4u;
    uint32_t e5m2_range = 939524096u;
    float e2m3_range = 7.5f;
    if (range <= e2m3_range) return Q_E2M3;
    if (range <= (float)e4m3_range) return (amax <= clamp) ? Q_E4M3_SMALL : Q_E4M3;
    if (range <= (float)e5m2_range) {
        if (dynamic_range_mode) return (amax <= clamp) ? Q_E5M2_SMALL : Q_E5M2;
        block_error(b, amax, e8, flavour, e4_o, e5_o);
        if (*e4_o <= *e5_o) return (amax <= clamp) ? Q_E4M3_SMALL : Q_E4M3;
        return Q_BF16;
    }
    return Q_BF16;
}

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

/* FQ:684-852, launch decoding FQ:1763-1835 */
int mor_oracle_fake_quantize(const uint16_t* in, uint16_t* out, int32_t* meta,
                             int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                             float clamp, int64_t mode, int64_t sf_type, int flavour, float* stats) {
    if (rows <= 0 || cols <= 0 || brows <= 0 || bcols <= 0) return -1;
    int qmode = (int)(mode % 10);
    int dynamic_range_mode = (mode / 100 > 0);
    int e8 = (sf_type == 2);
    int64_t gy = cdiv(rows, brows), gx = cdiv(cols, bcols);
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t by = 0; by < gy; ++by)
        for (int64_t bx = 0; bx < gx; ++bx) {
            blk_t b = {in, rows, cols, brows, bcols, by * brows, 0, bx * bcols, 0};
            b.r1 = b.r0 + brows < rows ? b.r0 + brows : rows;
            b.c1 = b.c0 + bcols < cols ? b.c0 + bcols : cols;
            float amax = 0.0f, amin = 0.0f, e4 = 0.0f, e5 = 0.0f;
            if (qmode != 4 && qmode != 5) block_amax_amin(&b, &amax, &amin);
            int qt = Q_UNKNOWN, m;
            if (qmode == 1) qt = choose_mor(&b, clamp, dynamic_range_mode, e8, flavour, amax, amin, &e4, &e5);
            switch (qmode) {
                case 1: m = qt; break;
                case 2: m = 1; break;
                case 3: m = 2; break;
                case 4: m = 1; break;
                case 5: m = 2; break;
                default: m = 3; break;
            }
            meta[by * gx + bx] = m;
            if (stats) {
                float* s = stats + 4 * (by * gx + bx);
                s[0] = amax; s[1] = amin; s[2] = e4; s[3] = e5;
            }
            int fmt = -1;           /* -1: copy */
            float sf = 1.0f;
            switch (qmode) {
                case 1:
                    if (amax > 0) {
                        if (qt == Q_E2M3) fmt = MOR_O_E2M3;
                        else if (qt == Q_E4M3 || qt == Q_E4M3_SMALL) fmt = MOR_O_E4M3;
                        else if (qt == Q_E5M2 || qt == Q_E5M2_SMALL) fmt = MOR_O_E5M2;
                        if (fmt >= 0) sf = FMAX_OF[fmt] / amax;
                    }
                    break;
                case 2: if (amax > 0) { fmt = MOR_O_E4M3; sf = 448.0f / amax; } break;
                case 3: if (amax > 0) { fmt = MOR_O_E5M2; sf = 57344.0f / amax; } break;
                case 4: fmt = MOR_O_E4M3; sf = clamp; break;
                case 5: fmt = MOR_O_E5M2; sf = clamp; break;
                default: break;
            }
            for (int64_t r = b.r0; r < b.r1; ++r)
                for (int64_t c = b.c0; c < b.c1; ++c) {
                    uint16_t raw = in[r * cols + c];
                    if (fmt < 0) { out[r * cols + c] = raw; continue; }
                    float v = mor_oracle_bf16_to_fp32(raw);
                    out[r * cols + c] = (uint16_t)store_bf16(sqdd(v, sf, fmt, e8, flavour), flavour);
                }
        }
    return 0;
}

int mor_oracle_block_format(const uint16_t* in, uint16_t* out,
                            int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                            int fmt, int64_t sf_type, int flavour) {
    if (rows <= 0 || cols <= 0 || brows <= 0 || bcols <= 0 || fmt < 0 || fmt > 3) return -1;
    int e8 = (sf_type == 2);
    int64_t gy = cdiv(rows, brows), gx = cdiv(cols, bcols);
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t by = 0; by < gy; ++by)
        for (int64_t bx = 0; bx < gx; ++bx) {
            blk_t b = {in, rows, cols, brows, bcols, by * brows, 0, bx * bcols, 0};
            b.r1 = b.r0 + brows < rows ? b.r0 + brows : rows;
            b.c1 = b.c0 + bcols < cols ? b.c0 + bcols : cols;
            float amax, amin;
            block_amax_amin(&b, &amax, &amin);
            float sf = amax > 0 ? FMAX_OF[fmt] / amax : 1.0f;
            for (int64_t r = b.r0; r < b.r1; ++r)
                for (int64_t c = b.c0; c < b.c1; ++c) {
                    uint16_t raw = in[r * cols + c];
                    if (!(amax > 0)) { out[r * cols + c] = raw; continue; }
                    float v = mor_oracle_bf16_to_fp32(raw);
                    out[r * cols + c] = (uint16_t)store_bf16(sqdd(v, sf, fmt, e8, flavour), flavour);
                }
        }
    return 0;
}

int mor_oracle_block_stats(const uint16_t* in, int64_t rows, int64_t cols, int64_t brows,
                           int64_t bcols, float fmax, float* amax_o, float* scale_o, int32_t* e8m0_o) {
    if (rows <= 0 || cols <= 0 || brows <= 0 || bcols <= 0) return -1;
    int64_t gy = cdiv(rows, brows), gx = cdiv(cols, bcols);
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t by = 0; by < gy; ++by)
        for (int64_t bx = 0; bx < gx; ++bx) {
            blk_t b = {in, rows, cols, brows, bcols, by * brows, 0, bx * bcols, 0};
            b.r1 = b.r0 + brows < rows ? b.r0 + brows : rows;
            b.c1 = b.c0 + bcols < cols ? b.c0 + bcols : cols;
            float amax, amin;
            block_amax_amin(&b, &amax, &amin);
            float s = amax > 0 ? fmax / amax : 1.0f;
            amax_o[by * gx + bx] = amax;
            scale_o[by * gx + bx] = s;
            e8m0_o[by * gx + bx] = (int32_t)((f2u(s) >> 23) & 0xFF);
        }
    return 0;
}

/* ------------------------------------------------------------------ */
/* FQ:1059-1093.  ss_mode: 1 global-amax mantissa, 2 block amax, 3 E8, 4 current. */
float mor_oracle_scaling_factor(float global_amax, float block_amax, int ss_mode) {
    float sf = 1.0f;
    const float fmax = 448.0f;
    const float epsilon = 1e-35f;
    if (block_amax < epsilon) block_amax = epsilon;
    switch (ss_mode) {
        case 1: {
            float ratio = fmax / global_amax;
            uint32_t gman = f2u(ratio) & 0x007FFFFFu;
            if (block_amax > 0) {
                float bsf = fmax / block_amax;
                uint32_t bb = f2u(bsf);
                uint32_t bman = bb & 0x007FFFFFu;
                float adj = u2f((bb & 0xFF800000u) | gman);
                sf = (gman <= bman) ? adj : adj / 2.0f;
            }
            break;
        }
        case 2:
        case 3:
            if (block_amax > 0) sf = fmax / block_amax;
            break;
        case 4:
            if (global_amax > 0) sf = fmax / global_amax;
            break;
        default: break;
    }
    return sf;
}

/* One element of FQ:1133-1162 / FQ:1712-1740.  The template test at FQ:1138
 * compares the ScalingStrategy with ScalingFactorType::SF_E8 (= 2), so it is
 * ss_mode 2 that takes the power-of-two path. */
static inline float bs_element(float x, float sf, int64_t ss_mode, int flavour, float* err) {
    float dq = 0.0f;
    *err = 0.0f;
    if (x != 0.0f) {
        dq = sqdd(x, sf, MOR_O_E4M3, ss_mode == 2, flavour);
        *err = fabsf((dq - x) / x);
    } else if (flavour == MOR_O_EMU) {
        dq = x;
    }
    return dq;
}

/* The sum of the per-element error terms of the last mor_oracle_block_scaling call of this thread, added in double:
 * the value the fp32 sums of the reference approach, whatever order they are added in.  (The reference's own result,
 * global_error, carries the rounding of its order of additions: about sqrt(n) * 2^-24 relative for chains of n
 * terms.) */
static _Thread_local double g_last_exact_error;
double mor_oracle_last_exact_error(void) { return g_last_exact_error; }

int mor_oracle_block_scaling(const uint16_t* in, uint16_t* out, int32_t* meta,
                             float* global_amax_o, int32_t* global_nnz_o, float* global_error_o,
                             int64_t rows, int64_t cols, int64_t brows, int64_t bcols,
                             float threshold, int64_t ss_mode, int channel, int flavour) {
    if (rows <= 0 || cols <= 0 || brows <= 0 || bcols <= 0) return -1;
    if (rows % brows || cols % bcols) return -2;            /* FQ:2019-2020 */
    if (ss_mode < 1 || ss_mode > 4) return -3;
    int64_t gy = rows / brows, gx = cols / bcols, nb = gy * gx;
    float* bamax = (float*)malloc(sizeof(float) * (size_t)nb);
    float* berr = (float*)malloc(sizeof(float) * (size_t)nb);
    int32_t* bnnz = (int32_t*)malloc(sizeof(int32_t) * (size_t)nb);
    uint16_t* tmp = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(rows * cols));
    if (!bamax || !berr || !bnnz || !tmp) { free(bamax); free(berr); free(bnnz); free(tmp); return -4; }

    /* FQ:951-1015 / FQ:1459-1631 */
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < nb; ++k) {
        int64_t by = k / gx, bx = k % gx;
        float amax = channel ? 0.0f : -INFINITY;
        int32_t nnz = 0;
        for (int64_t r = by * brows; r < (by + 1) * brows; ++r)
            for (int64_t c = bx * bcols; c < (bx + 1) * bcols; ++c) {
                float a = fabsf(mor_oracle_bf16_to_fp32(in[r * cols + c]));
                if (a > 0) nnz++;
                amax = max_nn(amax, a);
            }
        bamax[k] = amax; bnnz[k] = nnz;
    }
    /* FQ:1017-1049 (no trap on an all-zero tensor) */
    float gamax = -3.402823466e+38f;
    int32_t gnnz = 0;
    for (int64_t k = 0; k < nb; ++k) { gamax = max_nn(gamax, bamax[k]); gnnz += bnnz[k]; }

    /* FQ:1095-1176 / FQ:1633-1752.  The per-element arithmetic does not depend on the launch geometry; the
     * order of the fp32 additions of the error sum does.  Three geometries of the reference are reproduced:
     *   block op, 32x32 threads per block (needs bcols % 64 == 0, brows % 32 == 0);
     *   channel op, row blocks 1 x N with N >= 128, N % 128 == 0: 64 threads per block (FQ:2502, 2399-2415);
     *   channel op, column blocks rows x 1 (one block row) with cols % 64 == 0: 32x16 threads per 64 columns,
     *     the sum of a thread block goes to its first column, the other 63 get 0 (FQ:2503, 1750-1751).
     * For any other shape the reference has no working launch, hence no order: terms are added in double. */
    const int geom_block = !channel && (bcols % 64 == 0) && (brows % 32 == 0);
    const int geom_row = channel && brows == 1 && bcols >= 128 && (bcols % 128 == 0);
    const int geom_col = channel && bcols == 1 && brows == rows && (cols % 64 == 0) && (rows % 16 == 0);
    double exact = 0.0;
    if (geom_col) {
        for (int64_t k = 0; k < nb; ++k) berr[k] = 0.0f;
#pragma omp parallel for schedule(static) reduction(+:exact)
        for (int64_t tb = 0; tb < cols / 64; ++tb) {
            float partial[512];
            for (int ty = 0; ty < 16; ++ty)
                for (int tx = 0; tx < 32; ++tx) {
                    int64_t c1 = tb * 64 + 2 * tx + 1, c2 = c1 - 1;       /* high half = odd column */
                    float sf1 = mor_oracle_scaling_factor(gamax, bamax[c1], (int)ss_mode);
                    float sf2 = mor_oracle_scaling_factor(gamax, bamax[c2], (int)ss_mode);
                    float e1 = 0.0f, e2 = 0.0f;
                    for (int64_t r = ty; r < rows; r += 16) {
                        float t1, t2;
                        float x1 = mor_oracle_bf16_to_fp32(in[r * cols + c1]), x2 = mor_oracle_bf16_to_fp32(in[r * cols + c2]);
                        float q1 = bs_element(x1, sf1, ss_mode, flavour, &t1);
                        float q2 = bs_element(x2, sf2, ss_mode, flavour, &t2);
                        if (x1 != 0.0f) { e1 += t1; exact += (double)t1; }
                        if (x2 != 0.0f) { e2 += t2; exact += (double)t2; }
                        tmp[r * cols + c1] = (uint16_t)store_bf16(q1, flavour);
                        tmp[r * cols + c2] = (uint16_t)store_bf16(q2, flavour);
                    }
                    partial[ty * 32 + tx] = e1 + e2;
                }
            berr[tb * 64] = block_tree_sum(partial, 512);
        }
    } else {
#pragma omp parallel for schedule(static) reduction(+:exact)
    for (int64_t k = 0; k < nb; ++k) {
        int64_t by = k / gx, bx = k % gx;
        float sf = mor_oracle_scaling_factor(gamax, bamax[k], (int)ss_mode);
        int64_t r0 = by * brows, c0 = bx * bcols;
        float partial[1024];
        if (geom_block) {
            /* 32x32 threads over packed columns, r outer / c inner, high half first */
            for (int ty = 0; ty < 32; ++ty)
                for (int tx = 0; tx < 32; ++tx) {
                    float acc = 0.0f;
                    for (int64_t r = ty; r < brows; r += 32)
                        for (int64_t pc = tx; pc < bcols / 2; pc += 32) {
                            float e1, e2;
                            int64_t i1 = (r0 + r) * cols + c0 + 2 * pc + 1, i2 = i1 - 1;
                            float x1 = mor_oracle_bf16_to_fp32(in[i1]), x2 = mor_oracle_bf16_to_fp32(in[i2]);
                            float q1 = bs_element(x1, sf, ss_mode, flavour, &e1);
                            float q2 = bs_element(x2, sf, ss_mode, flavour, &e2);
                            if (x1 != 0.0f) { acc += e1; exact += (double)e1; }
                            if (x2 != 0.0f) { acc += e2; exact += (double)e2; }
                            tmp[i1] = (uint16_t)store_bf16(q1, flavour);
                            tmp[i2] = (uint16_t)store_bf16(q2, flavour);
                        }
                    partial[ty * 32 + tx] = acc;
                }
            berr[k] = block_tree_sum(partial, 1024);
        } else if (geom_row) {
            /* 64 threads along the row, one packed column each per step; odd and even columns summed apart */
            for (int tx = 0; tx < 64; ++tx) {
                float e1 = 0.0f, e2 = 0.0f;
                for (int64_t pc = tx; pc < bcols / 2; pc += 64) {
                    float t1, t2;
                    int64_t i1 = r0 * cols + c0 + 2 * pc + 1, i2 = i1 - 1;
                    float x1 = mor_oracle_bf16_to_fp32(in[i1]), x2 = mor_oracle_bf16_to_fp32(in[i2]);
                    float q1 = bs_element(x1, sf, ss_mode, flavour, &t1);
                    float q2 = bs_element(x2, sf, ss_mode, flavour, &t2);
                    if (x1 != 0.0f) { e1 += t1; exact += (double)t1; }
                    if (x2 != 0.0f) { e2 += t2; exact += (double)t2; }
                    tmp[i1] = (uint16_t)store_bf16(q1, flavour);
                    tmp[i2] = (uint16_t)store_bf16(q2, flavour);
                }
                partial[tx] = e1 + e2;
            }
            berr[k] = block_tree_sum(partial, 64);
        } else {
            double seq = 0.0;
            for (int64_t r = r0; r < r0 + brows; ++r)
                for (int64_t c = c0; c < c0 + bcols; ++c) {
                    float e;
                    float x = mor_oracle_bf16_to_fp32(in[r * cols + c]);
                    float q = bs_element(x, sf, ss_mode, flavour, &e);
                    if (x != 0.0f) seq += e;
                    tmp[r * cols + c] = (uint16_t)store_bf16(q, flavour);
                }
            berr[k] = (float)seq;
            exact += seq;
        }
    }
    }
    /* FQ:1178-1201: 1024 threads stride over the block errors, then the tree */
    float gerr;
    {
        float partial[1024];
        for (int t = 0; t < 1024; ++t) {
            float acc = 0.0f;
            for (int64_t i = t; i < nb; i += 1024) acc += berr[i];
            partial[t] = acc;
        }
        gerr = block_tree_sum(partial, 1024);
    }
    /* FQ:1203-1241 */
    float avg = gerr / (float)gnnz;
    int use_bf16 = (avg > threshold);
    meta[0] = use_bf16 ? 3 : 1;
    *global_amax_o = gamax;
    *global_nnz_o = gnnz;
    *global_error_o = gerr;
    g_last_exact_error = exact;
    if (use_bf16) {
        if (out != in) memcpy(out, in, sizeof(uint16_t) * (size_t)(rows * cols));
    } else {
        memcpy(out, tmp, sizeof(uint16_t) * (size_t)(rows * cols));
    }
    free(bamax); free(berr); free(bnnz); free(tmp);
    return 0;
}

/* ------------------------------------------------------------------ */
/* FQ:1243-1327: keep mbits (1..3) mantissa bits of an fp32 whose low 16 bits
 * are zero, thresholds on the 7-bit bf16 mantissa. */
float mor_oracle_e8m(float value, int mbits) {
    uint32_t bits = f2u(value);
    uint32_t sign = (bits >> 31) & 0x1;
    int32_t exponent = (int32_t)((bits >> 23) & 0xFF);
    uint32_t mantissa = bits & 0x7FFFFFu;
    if (exponent == 0) mantissa = 0;
    else if (exponent != 255) {
        /* thresholds: E8M1 {32,95}; E8M2 {16,47,80,111}; E8M3 {8,23,40,55,72,87,104,119} */
        static const uint32_t T1[] = {32, 95};
        static const uint32_t T2[] = {16, 47, 80, 111};
        static const uint32_t T3[] = {8, 23, 40, 55, 72, 87, 104, 119};
        const uint32_t* T = mbits == 1 ? T1 : mbits == 2 ? T2 : T3;
        int n = 1 << mbits;
        int k = 0;
        while (k < n && mantissa > (T[k] << 16)) ++k;
        if (k < n) mantissa = (uint32_t)k << (23 - mbits);
        else {
            mantissa = 0;
            exponent++;
            if (exponent == 255) { exponent = 254; mantissa = (uint32_t)(n - 1) << (23 - mbits); }
        }
    }
    return u2f((sign << 31) | ((uint32_t)exponent << 23) | mantissa);
}

/* FQ:1335-1359 */
float mor_oracle_e8mx_scaling_factor(float global_amax, int mbits, int strategy) {
    float sf = 1.0f;
    if (strategy == 1) {
        uint32_t y = f2u(global_amax);
        uint32_t exponent = (y >> 23) + 1;
        uint32_t y2 = (exponent << 23) | (((1u << mbits) - 1u) << (23 - mbits));
        float fp_max = u2f(y2);
        sf = fp_max / global_amax;
        if (sf >= 2) sf /= 2;
    }
    return sf;
}

int mor_oracle_e8mx(const uint16_t* in, uint16_t* out, int64_t rows, int64_t cols,
                    int64_t brows, int64_t bcols, int64_t qtype, int64_t strategy, int flavour) {
    (void)brows; (void)bcols;
    if (rows <= 0 || cols <= 0) return -1;
    if (qtype < 1 || qtype > 3) return -3;
    float gamax = -3.402823466e+38f;
    for (int64_t i = 0; i < rows * cols; ++i)
        gamax = max_nn(gamax, fabsf(mor_oracle_bf16_to_fp32(in[i])));
    float sf = mor_oracle_e8mx_scaling_factor(gamax, (int)qtype, (int)strategy);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows * cols; ++i) {
        float v = mor_oracle_bf16_to_fp32(in[i]);
        float dq = 0.0f;
        v *= sf;
        if (v != 0.0f) dq = mor_oracle_e8m(v, (int)qtype);
        dq /= sf;
        out[i] = (uint16_t)store_bf16(dq, flavour);
    }
    return 0;
}

/* ------------------------------------------------------------------ */
/* FQ:854-863 with T_USE_CUDA_CAST = false (FQ:1945) */
void mor_oracle_quant_dequant(const float* in, float* out, size_t n, int fmt) {
    for (size_t i = 0; i < n; ++i) out[i] = mor_oracle_cast_sw(in[i], fmt);
}

/* FQ:865-875: sf = 448.0 / value (double division rounded to float == the
 * correctly rounded fp32 quotient), software E4M3 cast. */
void mor_oracle_e4m3_with_e8_scale(const float* in, float* out, size_t n, int rne) {
    for (size_t i = 0; i < n; ++i) {
        float v = in[i];
        float sf = (float)(448.0 / (double)v);
        out[i] = sqdd_e8(v, sf, rne, MOR_O_E4M3, 0, MOR_O_KERNEL);
    }
}

/* ------------------------------------------------------------------ */
/* MX wire format: element codes + one E8M0 scale byte per block of 32 elements along a row.
 *
 * The reference only returns the dequantized bf16 tensor; these two functions state what its MX
 * block quantization (quantize_kernel block modes with SF_E8, FQ:801-823, and the E2M3 branch
 * FQ:758-770) stores before dequantizing: per block, e8 = exponent field of fl32(fmax / amax) - 127
 * (FQ:251-252), code = cast(x * 2^e8) with the block format's cast (nearest even; the scaled value
 * never exceeds fmax), scale byte = 127 - e8, i.e. the E8M0 encoding of the multiplier 2^-e8 that
 * decodes the block.  Scaling is arithmetic (what the reference's torch emulation does,
 * test_fake_quantize.py:41-46), so a zero code decodes to zero; the sign of the input is kept on
 * every code.  A zero block has scale byte 127.  e8 is limited to [-127, 127] so that the byte
 * stays a finite E8M0 value.  FP6 codes are packed little-endian, 4 codes in 3 bytes.
 * Pinned by: decode(code) * 2^-e8 == mor_oracle_fake_quantize / mor_oracle_block_format in the
 * torch-emulation flavour (itself pinned by torch), with the decode tables of
 * tests/golden/scalar_vectors.npz; scale bytes == 254 - mor_oracle_block_stats exponents. */
static uint32_t encode_mag(float r, int fmt) {          /* r >= 0 on the grid of fmt */
    const fmt_t* f = &FMT[fmt];
    if (r == 0.0f) return 0;
    uint32_t b = f2u(r);
    int e = (int)(b >> 23) - 127;
    int emin = 1 - (int)f->bias;
    if (e < emin) return (uint32_t)ldexpf(r, (int)f->mbits - emin);       /* subnormal: r / 2^(emin - mbits) */
    return ((uint32_t)(e + (int)f->bias) << f->mbits) | ((b & 0x7FFFFFu) >> (23 - f->mbits));
}

static float decode_mag(uint32_t code, int fmt) {
    const fmt_t* f = &FMT[fmt];
    uint32_t e = code >> f->mbits, m = code & ((1u << f->mbits) - 1u);
    if (e == 0) return ldexpf((float)m, 1 - (int)f->bias - (int)f->mbits);
    return ldexpf(1.0f + (float)m / (float)(1u << f->mbits), (int)e - (int)f->bias);
}

static int mx_block_e8(const uint16_t* x, int n, int fmt, float* amax_o) {
    float amax = 0.0f;
    for (int i = 0; i < n; ++i) amax = max_nn(amax, fabsf(mor_oracle_bf16_to_fp32(x[i])));
    *amax_o = amax;
    if (!(amax > 0)) return 0;
    int e8 = (int)((f2u(FMAX_OF[fmt] / amax) >> 23) & 0xFF) - 127;
    return e8 > 127 ? 127 : e8 < -127 ? -127 : e8;
}

static size_t mx_row_bytes(int64_t cols, int fmt) { return (fmt <= MOR_O_E5M2) ? (size_t)cols : (size_t)cols / 4 * 3; }

int mor_oracle_mx_quantize(const uint16_t* in, uint8_t* payload, uint8_t* scales, int64_t rows, int64_t cols, int fmt) {
    if (rows <= 0 || cols <= 0 || cols % 32 || fmt < 0 || fmt > 3) return -1;
    const int nbits = (fmt <= MOR_O_E5M2) ? 8 : 6;
    const size_t rb = mx_row_bytes(cols, fmt);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t b = 0; b < cols / 32; ++b) {
            const uint16_t* x = in + r * cols + b * 32;
            float amax;
            int e8 = mx_block_e8(x, 32, fmt, &amax);
            scales[r * (cols / 32) + b] = (uint8_t)(127 - e8);
            uint8_t* dst = payload + r * rb + b * (32 * nbits / 8);
            uint32_t codes[32];
            for (int i = 0; i < 32; ++i) {
                float v = mor_oracle_bf16_to_fp32(x[i]);
                float scaled = (float)ldexp((double)fabsf(v), e8);      /* exact or below every grid's half step */
                int over;
                float q = rne_to_grid(scaled, (int)FMT[fmt].mbits, 1 - (int)FMT[fmt].bias, FMAX_OF[fmt], &over);
                if (over) q = FMAX_OF[fmt];
                codes[i] = encode_mag(q, fmt) | ((uint32_t)(x[i] >> 15) << (nbits - 1));
            }
            if (nbits == 8) for (int i = 0; i < 32; ++i) dst[i] = (uint8_t)codes[i];
            else
                for (int g = 0; g < 8; ++g) {                            /* 4 codes -> 24 bits, little-endian */
                    uint32_t w = codes[4 * g] | (codes[4 * g + 1] << 6) | (codes[4 * g + 2] << 12) | (codes[4 * g + 3] << 18);
                    dst[3 * g] = (uint8_t)w; dst[3 * g + 1] = (uint8_t)(w >> 8); dst[3 * g + 2] = (uint8_t)(w >> 16);
                }
        }
    return 0;
}

int mor_oracle_mx_dequantize(const uint8_t* payload, const uint8_t* scales, uint16_t* out, int64_t rows, int64_t cols, int fmt) {
    if (rows <= 0 || cols <= 0 || cols % 32 || fmt < 0 || fmt > 3) return -1;
    const int nbits = (fmt <= MOR_O_E5M2) ? 8 : 6;
    const size_t rb = mx_row_bytes(cols, fmt);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t b = 0; b < cols / 32; ++b) {
            const uint8_t* src = payload + r * rb + b * (32 * nbits / 8);
            int de = (int)scales[r * (cols / 32) + b] - 127;
            for (int i = 0; i < 32; ++i) {
                uint32_t code;
                if (nbits == 8) code = src[i];
                else {
                    const uint8_t* p = src + 3 * (i / 4);
                    uint32_t w = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
                    code = (w >> (6 * (i % 4))) & 0x3Fu;
                }
                uint32_t sign = code >> (nbits - 1), mag = code & ((1u << (nbits - 1)) - 1u);
                float v = (float)ldexp((double)decode_mag(mag, fmt), de);
                out[r * cols + b * 32 + i] = (uint16_t)(mor_oracle_fp32_to_bf16_rne(v) | (sign << 15));
            }
        }
    return 0;
}
