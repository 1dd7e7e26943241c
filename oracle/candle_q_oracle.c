/*
 * CPU oracle for candle's quantized matmul path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the reference's CPU algorithm
 * (candle-core/src/quantized/{k_quants.rs,utils.rs,mod.rs}).  It exists so
 * that tests, the smoke check and the bench's CPU-baseline leg have something
 * to compare the HIP kernels with.  Nothing in the shipped library links,
 * loads or calls it.
 *
 * Build: gcc -O2 -ffp-contract=off -fPIC -shared (see oracle/Makefile).
 * -ffp-contract=off matters: Rust never fuses a*b+c, GCC would by default.
 *
 * Parity status of each function (what pins it besides reading the source):
 *   q4_0 / q8_0 quantize + dot + matmul driver : reference goldens
 *        quantized_tests.rs:58-64, :123-129, :235-250      (exact)
 *   q8k quantize, q8k x q8k dot                 : :694-698, :1147
 *   q4k quantize (make_qkx1_quants, packing), dequant, q4k x q8k dot
 *                                               : :553-557, :546, :572, :1069, :786-861
 *   q5k quantize (make_qkx1_quants with 31 levels), dequant, q5k x q8k dot
 *                                               : :578-625 (spot values, < 0.009, < 2.5), :792, :1077-1098
 *   q6k quantize (make_qx_quants), dequant, q6k x q8k dot
 *                                               : :647-651, :640, :666, :1122, :786-861
 *   f16 conversion                              : exhaustive comparison with numpy.float16
 *   softmax / silu / top-k MoE combine          : brute-force dense-masked MoE on tiny sizes
 *   rms_norm (candle-nn/src/ops.rs:482-495)     : reference golden candle-nn/tests/ops.rs:55-66
 *        (4 decimals) and the closed form x / sqrt(mean(x^2) + eps) * alpha in float64
 *   silu_mul (op.rs:607-609, quantized_llama.rs:60-62) : closed form in float64 (no reference
 *        golden prints silu of known inputs on this path; PARITY UNPINNED beyond that: the last
 *        bits depend on the platform's expf)
 *   q5_0 quantize, dequant, q5_0 x q8_0 dot (k_quants.rs:352-452) : :289-319 (128 round-trip values), :317
 *        (RMSE bound), :795-805 (dot-product error <= 0.001353), numpy brute force from unpacked blocks
 *   q2k quantize (make_qkx1_quants with 3 levels over 16 elements), dequant, q2k x q8k dot (k_quants.rs:698-872)
 *                                               : :437-482 (spot values, < 0.1, < 6.0, RMSE <= 0.0075),
 *        :795-805 (dot-product error <= 0.004086), numpy brute force from unpacked blocks
 *   q3k quantize (make_q3_quants, utils.rs:261-326), dequant, q3k x q8k dot (k_quants.rs:874-1148)
 *                                               : :484-529 (spot values, < 0.03, < 3.5, RMSE <= 0.004),
 *        :795-805 (dot-product error <= 0.016148), numpy brute force from unpacked blocks
 *   q5_1 quantize, dequant, q5_1 x q8_1 dot (k_quants.rs:454-560) : :321-351 (128 round-trip values), :349
 *        (RMSE bound), :795-805 (dot-product error <= 0.00149), numpy brute force from unpacked blocks
 *   q4_1 quantize, dequant, q4_1 x q8_1 dot (k_quants.rs:257-350)            : :256-287 (128 round-trip values), :393-434
 *        (RMSE bound), :795 + :866 (dot-product error <= 0.008 on cos vectors, x2 on ramps)
 *   q8_1 quantize (k_quants.rs:665-691)         : d and qs by the q8_0 goldens (same
 *        arithmetic); the `s` field by the reference's q4_1 x q8_1 dot-product bounds above
 *        (the result is sum_i*d*d8 + m*s, so a dropped, mis-signed or unscaled s leaves the
 *        bound by orders of magnitude: tests/test_oracle_golden.py shows each such mutant
 *        failing) and by the invariant |s - d*sum(q)| <= one f16 ulp of s.
 *   q4k x q8_1 and q6k x q8_1 dot formulas      : PARITY UNPINNED on CPU (they
 *        exist only in the reference's CUDA kernels, quantized.cu:2141-2166,
 *        :2258-2281); checked by float64 brute force on dequantized operands.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK_K 256
#define K_SCALE_SIZE 12

/* GgmlDType ids, candle-core/src/quantized/mod.rs:173-190 */
enum {
    ORC_F32 = 0, ORC_F16 = 1, ORC_Q4_0 = 2, ORC_Q4_1 = 3, ORC_Q5_0 = 6, ORC_Q5_1 = 7,
    ORC_Q8_0 = 8, ORC_Q8_1 = 9, ORC_Q2K = 10, ORC_Q3K = 11, ORC_Q4K = 12, ORC_Q5K = 13,
    ORC_Q6K = 14, ORC_Q8K = 15
};

/* Block layouts, k_quants.rs:42-155 (#[repr(C)], little endian). */
#pragma pack(push, 1)
typedef struct { uint16_t d; uint8_t qs[16]; } block_q4_0;                      /* 18  */
typedef struct { uint16_t d; uint16_t m; uint8_t qs[16]; } block_q4_1;          /* 20  */
typedef struct { uint16_t d; int8_t qs[32]; } block_q8_0;                       /* 34  */
typedef struct { uint16_t d; uint16_t s; int8_t qs[32]; } block_q8_1;           /* 36  */
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[K_SCALE_SIZE]; uint8_t qs[QK_K / 2]; } block_q4k; /* 144 */
typedef struct { uint8_t ql[QK_K / 2]; uint8_t qh[QK_K / 4]; int8_t scales[QK_K / 16]; uint16_t d; } block_q6k; /* 210 */
typedef struct { float d; int8_t qs[QK_K]; int16_t bsums[QK_K / 16]; } block_q8k; /* 292 */
#pragma pack(pop)

typedef struct { uint16_t d; uint8_t qh[4]; uint8_t qs[16]; } block_q5_0;       /* 22, k_quants.rs:61-67 */
typedef struct { uint16_t d; uint16_t m; uint8_t qh[4]; uint8_t qs[16]; } block_q5_1; /* 24, k_quants.rs:69-76 */
_Static_assert(sizeof(block_q5_1) == 24, "q5_1");
typedef struct { uint8_t hmask[QK_K / 8]; uint8_t qs[QK_K / 4]; uint8_t scales[12]; uint16_t d; } block_q3k; /* 110, k_quants.rs:107-114 */
typedef struct { uint8_t scales[QK_K / 16]; uint8_t qs[QK_K / 4]; uint16_t d; uint16_t dmin; } block_q2k;    /* 84, k_quants.rs:96-103 */
_Static_assert(sizeof(block_q2k) == 84, "q2k");
_Static_assert(sizeof(block_q5_0) == 22, "q5_0");
_Static_assert(sizeof(block_q3k) == 110, "q3k");
_Static_assert(sizeof(block_q4_0) == 18, "q4_0");
_Static_assert(sizeof(block_q4_1) == 20, "q4_1");
_Static_assert(sizeof(block_q8_0) == 34, "q8_0");
_Static_assert(sizeof(block_q8_1) == 36, "q8_1");
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[K_SCALE_SIZE]; uint8_t qh[QK_K / 8]; uint8_t qs[QK_K / 2]; } block_q5k; /* 176, k_quants.rs:119-127 */
_Static_assert(sizeof(block_q4k) == 144, "q4k");
_Static_assert(sizeof(block_q5k) == 176, "q5k");
_Static_assert(sizeof(block_q6k) == 210, "q6k");
_Static_assert(sizeof(block_q8k) == 292, "q8k");

/* ---------------------------------------------------------------- f16 ---- */
/* IEEE binary16 <-> binary32, round-to-nearest-even; what crate `half`
 * (Cargo.toml:50) does in f16::from_f32 / f16::to_f32. */
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do { e++; man <<= 1; } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xff;
    uint32_t man = x & 0x7fffffu;
    if (exp == 255) { /* inf / nan */
        uint32_t nan_bit = man ? 0x0200u : 0;
        return (uint16_t)(sign | 0x7c00u | nan_bit | (man >> 13));
    }
    int32_t unbiased = (int32_t)exp - 127;
    if (unbiased > 15) return (uint16_t)(sign | 0x7c00u);        /* overflow -> inf */
    if (unbiased >= -14) {                                        /* normal */
        uint32_t half_exp = (uint32_t)(unbiased + 15) << 10;
        uint32_t half_man = man >> 13;
        uint32_t round_bit = 0x1000u;
        uint32_t r = sign | half_exp | half_man;
        if ((man & round_bit) && (man & (3 * round_bit - 1))) r += 1; /* RNE; carry may bump exp */
        return (uint16_t)r;
    }
    if (unbiased < -25) return (uint16_t)sign;                    /* underflow -> 0 */
    /* subnormal */
    man |= 0x800000u;
    uint32_t shift = (uint32_t)(-unbiased - 14 + 13);             /* 14..24 */
    uint32_t half_man = man >> shift;
    uint32_t round_bit = 1u << (shift - 1);
    if ((man & round_bit) && (man & (3 * round_bit - 1))) half_man += 1;
    return (uint16_t)(sign | half_man);
}

/* ------------------------------------------------- Rust cast semantics ---- */
/* `v as u8` / `as i8` / `as i32` on f32: truncate toward zero, saturate, NaN -> 0. */
static inline uint8_t as_u8(float v) {
    if (!(v == v)) return 0;
    if (v <= 0.0f) return 0;
    if (v >= 255.0f) return 255;
    return (uint8_t)v;
}
static inline int8_t as_i8(float v) {
    if (!(v == v)) return 0;
    if (v <= -128.0f) return -128;
    if (v >= 127.0f) return 127;
    return (int8_t)v;
}
static inline int32_t as_i32(float v) {
    if (!(v == v)) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}
/* utils.rs:3-5 */
static inline int32_t nearest_int(float v) { return as_i32(roundf(v)); }
static inline int32_t clampi(int32_t v, int32_t lo, int32_t hi) { return v < lo ? lo : (v > hi ? hi : v); }
/* f32::max / f32::min ignore a NaN operand, like fmaxf/fminf. */

/* --------------------------------------------------------------- Q4_0 ---- */
/* k_quants.rs:185-220 */
int orc_quantize_q4_0(const float *xs, void *out, int64_t k) {
    if (k % 32 != 0) return -1;
    block_q4_0 *ys = (block_q4_0 *)out;
    int64_t nb = k / 32;
    for (int64_t i = 0; i < nb; i++) {
        const float *x = xs + i * 32;
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < 32; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        }
        float d = max / -8.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = orc_f32_to_f16(d);
        for (int j = 0; j < 16; j++) {
            float x0 = x[j] * id;
            float x1 = x[16 + j] * id;
            uint8_t xi0 = as_u8(x0 + 8.5f); if (xi0 > 15) xi0 = 15;
            uint8_t xi1 = as_u8(x1 + 8.5f); if (xi1 > 15) xi1 = 15;
            ys[i].qs[j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
    return 0;
}

/* k_quants.rs:163-183 */
int orc_dequantize_q4_0(const void *in, float *ys, int64_t k) {
    if (k % 32 != 0) return -1;
    const block_q4_0 *xs = (const block_q4_0 *)in;
    for (int64_t i = 0; i < k / 32; i++) {
        float d = orc_f16_to_f32(xs[i].d);
        for (int j = 0; j < 16; j++) {
            int x0 = (xs[i].qs[j] & 0x0F) - 8;
            int x1 = (xs[i].qs[j] >> 4) - 8;
            ys[i * 32 + j] = (float)x0 * d;
            ys[i * 32 + j + 16] = (float)x1 * d;
        }
    }
    return 0;
}

static inline int32_t sumi_q4_0_q8_0(const block_q4_0 *x, const block_q8_0 *y) {
    int32_t sum_i = 0;
    for (int j = 0; j < 16; j++) {
        int32_t v0 = (x->qs[j] & 0x0F) - 8;
        int32_t v1 = (x->qs[j] >> 4) - 8;
        sum_i += v0 * y->qs[j] + v1 * y->qs[j + 16];
    }
    return sum_i;
}

/* k_quants.rs:237-254 (vec_dot_unopt) */
static float vec_dot_q4_0_q8_0(int64_t n, const block_q4_0 *xs, const block_q8_0 *ys) {
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / 32; i++) {
        int32_t sum_i = sumi_q4_0_q8_0(&xs[i], &ys[i]);
        sumf += (float)sum_i * orc_f16_to_f32(xs[i].d) * orc_f16_to_f32(ys[i].d);
    }
    return sumf;
}

/* --------------------------------------------------------------- Q5_0 ---- */
/* k_quants.rs:393-425 (from_float) */
int orc_quantize_q5_0(const float *xs, void *out, int64_t k) {
    if (k % 32 != 0) return -1;
    block_q5_0 *ys = (block_q5_0 *)out;
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < 32; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        }
        float d = max / -16.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = orc_f32_to_f16(d);
        uint32_t qh = 0;
        for (int j = 0; j < 16; j++) {
            float x0 = x[j] * id, x1 = x[j + 16] * id;
            int8_t s0 = as_i8(x0 + 16.5f), s1 = as_i8(x1 + 16.5f);
            uint8_t xi0 = (uint8_t)(s0 < 31 ? s0 : 31), xi1 = (uint8_t)(s1 < 31 ? s1 : 31);
            ys[i].qs[j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= (((uint32_t)xi0 & 0x10u) >> 4) << j;
            qh |= (((uint32_t)xi1 & 0x10u) >> 4) << (j + 16);
        }
        ys[i].qh[0] = (uint8_t)qh; ys[i].qh[1] = (uint8_t)(qh >> 8);
        ys[i].qh[2] = (uint8_t)(qh >> 16); ys[i].qh[3] = (uint8_t)(qh >> 24);
    }
    return 0;
}

static inline uint32_t q5_0_qh(const block_q5_0 *x) {
    return (uint32_t)x->qh[0] | ((uint32_t)x->qh[1] << 8) | ((uint32_t)x->qh[2] << 16) | ((uint32_t)x->qh[3] << 24);
}

/* k_quants.rs:428-451 (to_float) */
int orc_dequantize_q5_0(const void *in, float *ys, int64_t k) {
    if (k % 32 != 0) return -1;
    const block_q5_0 *xs = (const block_q5_0 *)in;
    for (int64_t i = 0; i < k / 32; i++) {
        float d = orc_f16_to_f32(xs[i].d);
        uint32_t qh = q5_0_qh(&xs[i]);
        for (int j = 0; j < 16; j++) {
            uint8_t xh_0 = (uint8_t)(((qh >> j) << 4) & 0x10);
            uint8_t xh_1 = (uint8_t)((qh >> (j + 12)) & 0x10);
            int32_t x0 = (int32_t)((xs[i].qs[j] & 0x0F) | xh_0) - 16;
            int32_t x1 = (int32_t)((xs[i].qs[j] >> 4) | xh_1) - 16;
            ys[i * 32 + j] = (float)x0 * d;
            ys[i * 32 + j + 16] = (float)x1 * d;
        }
    }
    return 0;
}

/* k_quants.rs:371-391 (vec_dot_unopt of Q5_0 x Q8_0) */
static int32_t sumi_q5_0_q8_0(const block_q5_0 *x, const block_q8_0 *y) {
    uint32_t qh = q5_0_qh(x);
    int32_t sumi = 0;
    for (int j = 0; j < 16; j++) {
        uint8_t xh_0 = (uint8_t)(((qh & (1u << j)) >> j) << 4);
        uint8_t xh_1 = (uint8_t)((qh & (1u << (j + 16))) >> (j + 12));
        int32_t x0 = ((int32_t)(x->qs[j] & 0x0F) | (int32_t)xh_0) - 16;
        int32_t x1 = ((int32_t)(x->qs[j] >> 4) | (int32_t)xh_1) - 16;
        sumi += x0 * (int32_t)y->qs[j] + x1 * (int32_t)y->qs[j + 16];
    }
    return sumi;
}
static float vec_dot_q5_0_q8_0(int64_t n, const block_q5_0 *xs, const block_q8_0 *ys) {
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / 32; i++) {
        int32_t sumi = sumi_q5_0_q8_0(&xs[i], &ys[i]);
        sumf += (float)sumi * orc_f16_to_f32(xs[i].d) * orc_f16_to_f32(ys[i].d);
    }
    return sumf;
}

/* --------------------------------------------------------------- Q4_1 ---- */
/* Oracle only: the reference's own Q4_1 vectors are what pins BlockQ8_1::from_float's `s`.
 * k_quants.rs:296-326 (from_float; f32::min / f32::max ignore a NaN operand like fminf / fmaxf) */
int orc_quantize_q4_1(const float *xs, void *out, int64_t k) {
    if (k % 32 != 0) return -1;
    block_q4_1 *ys = (block_q4_1 *)out;
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float min = INFINITY, max = -INFINITY;
        for (int j = 0; j < 32; j++) {
            min = fminf(x[j], min);
            max = fmaxf(x[j], max);
        }
        float d = (max - min) / 15.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = orc_f32_to_f16(d);
        ys[i].m = orc_f32_to_f16(min);
        for (int j = 0; j < 16; j++) {
            float x0 = (x[j] - min) * id;
            float x1 = (x[16 + j] - min) * id;
            uint8_t xi0 = as_u8(x0 + 0.5f); if (xi0 > 15) xi0 = 15;
            uint8_t xi1 = as_u8(x1 + 0.5f); if (xi1 > 15) xi1 = 15;
            ys[i].qs[j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
    return 0;
}

/* k_quants.rs:329-349 */
int orc_dequantize_q4_1(const void *in, float *ys, int64_t k) {
    if (k % 32 != 0) return -1;
    const block_q4_1 *xs = (const block_q4_1 *)in;
    for (int64_t i = 0; i < k / 32; i++) {
        float d = orc_f16_to_f32(xs[i].d), m = orc_f16_to_f32(xs[i].m);
        for (int j = 0; j < 16; j++) {
            ys[i * 32 + j] = (float)(xs[i].qs[j] & 0x0F) * d + m;
            ys[i * 32 + j + 16] = (float)(xs[i].qs[j] >> 4) * d + m;
        }
    }
    return 0;
}

/* --------------------------------------------------------------- Q8_0 ---- */
/* k_quants.rs:586-615 */
int orc_quantize_q8_0(const float *xs, void *out, int64_t k) {
    if (k % 32 != 0) return -1;
    block_q8_0 *ys = (block_q8_0 *)out;
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(x[j]));
        float d = amax / 127.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = orc_f32_to_f16(d);
        for (int j = 0; j < 32; j++) ys[i].qs[j] = as_i8(roundf(x[j] * id));
    }
    return 0;
}

/* k_quants.rs:568-584 */
int orc_dequantize_q8_0(const void *in, float *ys, int64_t k) {
    if (k % 32 != 0) return -1;
    const block_q8_0 *xs = (const block_q8_0 *)in;
    for (int64_t i = 0; i < k / 32; i++) {
        float d = orc_f16_to_f32(xs[i].d);
        for (int j = 0; j < 32; j++) ys[i * 32 + j] = (float)xs[i].qs[j] * d;
    }
    return 0;
}

static inline int32_t sumi_q8_0_q8_0(const block_q8_0 *x, const block_q8_0 *y) {
    int32_t s = 0;
    for (int j = 0; j < 32; j++) s += (int32_t)x->qs[j] * (int32_t)y->qs[j];
    return s;
}

/* k_quants.rs:631-649 */
static float vec_dot_q8_0_q8_0(int64_t n, const block_q8_0 *xs, const block_q8_0 *ys) {
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / 32; i++) {
        int32_t sum_i = sumi_q8_0_q8_0(&xs[i], &ys[i]);
        sumf += (float)sum_i * orc_f16_to_f32(xs[i].d) * orc_f16_to_f32(ys[i].d);
    }
    return sumf;
}

/* --------------------------------------------------------------- Q8_1 ---- */
/* k_quants.rs:665-691.  `f16 * f16` in crate half = f16(f32(a) * f32(b)). */
int orc_quantize_q8_1(const float *xs, void *out, int64_t k) {
    if (k % 32 != 0) return -1;
    block_q8_1 *ys = (block_q8_1 *)out;
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(x[j]));
        float d = amax / 127.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = orc_f32_to_f16(d);
        int32_t sum = 0;
        for (int j = 0; j < 16; j++) {
            float v0 = x[j] * id;
            float v1 = x[j + 16] * id;
            ys[i].qs[j] = as_i8(roundf(v0));
            ys[i].qs[j + 16] = as_i8(roundf(v1));
            sum += (int32_t)ys[i].qs[j] + (int32_t)ys[i].qs[j + 16];
        }
        uint16_t hs = orc_f32_to_f16((float)sum);
        ys[i].s = orc_f32_to_f16(orc_f16_to_f32(hs) * orc_f16_to_f32(ys[i].d));
    }
    return 0;
}

/* k_quants.rs:267-294 (vec_dot_unopt of Q4_1 x Q8_1; the block count must be even) */
static int vec_dot_q4_1_q8_1(int64_t n, const block_q4_1 *xs, const block_q8_1 *ys, float *out) {
    int64_t nb = n / 32;
    if (nb % 2 != 0) return -1;
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) {
            int32_t v0 = xs[i].qs[j] & 0x0F;
            int32_t v1 = xs[i].qs[j] >> 4;
            sumi += v0 * (int32_t)ys[i].qs[j] + v1 * (int32_t)ys[i].qs[j + 16];
        }
        sumf += (float)sumi * orc_f16_to_f32(xs[i].d) * orc_f16_to_f32(ys[i].d) +
                orc_f16_to_f32(xs[i].m) * orc_f16_to_f32(ys[i].s);
    }
    *out = sumf;
    return 0;
}

/* --------------------------------------------------------------- Q5_1 ---- */
/* k_quants.rs:496-530 (from_float) */
int orc_quantize_q5_1(const float *xs, void *out, int64_t k) {
    if (k % 32 != 0) return -1;
    block_q5_1 *ys = (block_q5_1 *)out;
    for (int64_t i = 0; i < k / 32; i++) {
        const float *x = xs + i * 32;
        float min = INFINITY, max = -INFINITY;
        for (int j = 0; j < 32; j++) {
            min = fminf(x[j], min);
            max = fmaxf(x[j], max);
        }
        float d = (max - min) / 31.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        ys[i].d = orc_f32_to_f16(d);
        ys[i].m = orc_f32_to_f16(min);
        uint32_t qh = 0;
        for (int j = 0; j < 16; j++) {
            float x0 = (x[j] - min) * id;
            float x1 = (x[16 + j] - min) * id;
            uint8_t xi0 = as_u8(x0 + 0.5f), xi1 = as_u8(x1 + 0.5f);
            ys[i].qs[j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= (((uint32_t)xi0 & 0x10u) >> 4) << j;
            qh |= (((uint32_t)xi1 & 0x10u) >> 4) << (j + 16);
        }
        ys[i].qh[0] = (uint8_t)qh; ys[i].qh[1] = (uint8_t)(qh >> 8);
        ys[i].qh[2] = (uint8_t)(qh >> 16); ys[i].qh[3] = (uint8_t)(qh >> 24);
    }
    return 0;
}

static inline uint32_t q5_1_qh(const block_q5_1 *x) {
    return (uint32_t)x->qh[0] | ((uint32_t)x->qh[1] << 8) | ((uint32_t)x->qh[2] << 16) | ((uint32_t)x->qh[3] << 24);
}
/* the five-bit quant of element e (0..31) */
static inline int32_t q5_1_quant(const block_q5_1 *x, int e) {
    uint32_t qh = q5_1_qh(x);
    int j = e & 15;
    int32_t lo = e < 16 ? (x->qs[j] & 0x0F) : (x->qs[j] >> 4);
    return lo | (int32_t)(((qh >> e) & 1u) << 4);
}

/* k_quants.rs:533-558 (to_float) */
int orc_dequantize_q5_1(const void *in, float *ys, int64_t k) {
    if (k % 32 != 0) return -1;
    const block_q5_1 *xs = (const block_q5_1 *)in;
    for (int64_t i = 0; i < k / 32; i++) {
        float d = orc_f16_to_f32(xs[i].d), m = orc_f16_to_f32(xs[i].m);
        for (int e = 0; e < 32; e++) ys[i * 32 + e] = (float)q5_1_quant(&xs[i], e) * d + m;
    }
    return 0;
}

/* k_quants.rs:463-494 (vec_dot_unopt of Q5_1 x Q8_1; the block count must be even) */
static int32_t sumi_q5_1_q8_1(const block_q5_1 *x, const block_q8_1 *y) {
    int32_t sumi = 0;
    for (int j = 0; j < 16; j++)
        sumi += q5_1_quant(x, j) * (int32_t)y->qs[j] + q5_1_quant(x, j + 16) * (int32_t)y->qs[j + 16];
    return sumi;
}
static int32_t sumi_q4_1_q8_1(const block_q4_1 *x, const block_q8_1 *y) {
    int32_t sumi = 0;
    for (int j = 0; j < 16; j++)
        sumi += (int32_t)(x->qs[j] & 0x0F) * (int32_t)y->qs[j] + (int32_t)(x->qs[j] >> 4) * (int32_t)y->qs[j + 16];
    return sumi;
}
static int vec_dot_q5_1_q8_1(int64_t n, const block_q5_1 *xs, const block_q8_1 *ys, float *out) {
    int64_t nb = n / 32;
    if (nb % 2 != 0) return -1;
    float sumf = 0.0f;
    for (int64_t i = 0; i < nb; i++) {
        int32_t sumi = sumi_q5_1_q8_1(&xs[i], &ys[i]);
        sumf += (float)sumi * orc_f16_to_f32(xs[i].d) * orc_f16_to_f32(ys[i].d) +
                orc_f16_to_f32(xs[i].m) * orc_f16_to_f32(ys[i].s);
    }
    *out = sumf;
    return 0;
}

/* ---------------------------------------------------------------- Q8K ---- */
/* k_quants.rs:1788-1825.  `ys` must start zeroed (the reference allocates with
 * zeros(), k_quants.rs:1857), bsums are left untouched for an all-zero block. */
int orc_quantize_q8k(const float *xs, void *out, int64_t k) {
    if (k % QK_K != 0) return -1;
    block_q8k *ys = (block_q8k *)out;
    for (int64_t i = 0; i < k / QK_K; i++) {
        const float *x = xs + i * QK_K;
        float max = 0.0f, amax = 0.0f;
        for (int j = 0; j < QK_K; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        }
        if (amax == 0.0f) {
            ys[i].d = 0.0f;
            memset(ys[i].qs, 0, QK_K);
        } else {
            float iscale = -128.0f / max;
            for (int j = 0; j < QK_K; j++) {
                float v = roundf(iscale * x[j]);
                ys[i].qs[j] = as_i8(fminf(v, 127.0f));
            }
            for (int j = 0; j < QK_K / 16; j++) {
                int32_t sum = 0;
                for (int ii = 0; ii < 16; ii++) sum += ys[i].qs[j * 16 + ii];
                ys[i].bsums[j] = (int16_t)sum;
            }
            ys[i].d = 1.0f / iscale;
        }
    }
    return 0;
}

/* k_quants.rs:1827-1838 */
int orc_dequantize_q8k(const void *in, float *ys, int64_t k) {
    if (k % QK_K != 0) return -1;
    const block_q8k *xs = (const block_q8k *)in;
    for (int64_t i = 0; i < k / QK_K; i++)
        for (int j = 0; j < QK_K; j++) ys[i * QK_K + j] = xs[i].d * (float)xs[i].qs[j];
    return 0;
}

static inline int32_t sumi_q8k_q8k(const block_q8k *x, const block_q8k *y) {
    int32_t s = 0;
    for (int j = 0; j < QK_K; j++) s += (int32_t)x->qs[j] * (int32_t)y->qs[j];
    return s;
}

/* k_quants.rs:1768-1786 */
static float vec_dot_q8k_q8k(int64_t n, const block_q8k *xs, const block_q8k *ys) {
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / QK_K; i++) {
        int32_t sum_i = sumi_q8k_q8k(&xs[i], &ys[i]);
        sumf += (float)sum_i * xs[i].d * ys[i].d;
    }
    return sumf;
}

/* ---------------------------------------------------------------- Q4K ---- */
/* utils.rs:49-59 */
static inline void get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* utils.rs:201-258 */
static void make_qkx1_quants(int32_t nmax, int ntry, const float *x, int n, float *out_scale,
                             float *out_min) {
    uint8_t l[64];
    memset(l, 0, sizeof(l));
    float min = x[0], max = x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
    }
    if (max == min) { *out_scale = 0.0f; *out_min = 0.0f; return; }
    min = fminf(min, 0.0f);
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    for (int t = 0; t < ntry; t++) {
        float sumlx = 0.0f;
        int32_t suml2 = 0;
        int did_change = 0;
        for (int i = 0; i < n; i++) {
            int32_t li = clampi(nearest_int(iscale * (x[i] - min)), 0, nmax);
            uint8_t cl = (uint8_t)li;
            if (cl != l[i]) { l[i] = cl; did_change = 1; }
            sumlx += (x[i] - min) * (float)li;
            suml2 += li * li;
        }
        scale = sumlx / (float)suml2;
        float sum = 0.0f;
        for (int i = 0; i < n; i++) sum += x[i] - scale * (float)l[i];
        min = sum / (float)n;
        if (min > 0.0f) min = 0.0f;
        iscale = 1.0f / scale;
        if (!did_change) break;
    }
    *out_scale = scale;
    *out_min = -min;
}

/* k_quants.rs:1252-1311 */
int orc_quantize_q4k(const float *xs, void *out, int64_t k) {
    if (k % QK_K != 0) return -1;
    block_q4k *ys = (block_q4k *)out;
    for (int64_t ib = 0; ib < k / QK_K; ib++) {
        const float *x = xs + ib * QK_K;
        block_q4k *block = &ys[ib];
        memset(block->scales, 0, K_SCALE_SIZE); /* blocks come from zeros() in the reference */
        float mins[8], scales[8];
        for (int j = 0; j < 8; j++) make_qkx1_quants(15, 5, x + 32 * j, 32, &scales[j], &mins[j]);
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) max_scale = fmaxf(scales[j], max_scale);
        for (int j = 0; j < 8; j++) max_min = fmaxf(mins[j], max_min);
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        for (int j = 0; j < 8; j++) {
            int32_t lsi = nearest_int(inv_scale * scales[j]); if (lsi > 63) lsi = 63;
            int32_t lmi = nearest_int(inv_min * mins[j]); if (lmi > 63) lmi = 63;
            uint8_t ls = (uint8_t)lsi, lm = (uint8_t)lmi;
            if (j < 4) {
                block->scales[j] = ls;
                block->scales[j + 4] = lm;
            } else {
                block->scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                block->scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                block->scales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        block->d = orc_f32_to_f16(max_scale / 63.0f);
        block->dmin = orc_f32_to_f16(max_min / 63.0f);
        uint8_t l[QK_K];
        memset(l, 0, sizeof(l));
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            get_scale_min_k4(j, block->scales, &sc, &m);
            float d = orc_f16_to_f32(block->d) * (float)sc;
            if (d != 0.0f) {
                float dm = orc_f16_to_f32(block->dmin) * (float)m;
                for (int ii = 0; ii < 32; ii++) {
                    int32_t lv = nearest_int((x[32 * j + ii] + dm) / d);
                    l[32 * j + ii] = (uint8_t)clampi(lv, 0, 15);
                }
            }
        }
        for (int j = 0; j < QK_K; j += 64)
            for (int lv = 0; lv < 32; lv++)
                block->qs[(j / 64) * 32 + lv] = (uint8_t)(l[j + lv] | (l[j + lv + 32] << 4));
    }
    return 0;
}

/* k_quants.rs:1313-1341 */
int orc_dequantize_q4k(const void *in, float *ys, int64_t k) {
    if (k % QK_K != 0) return -1;
    const block_q4k *xs = (const block_q4k *)in;
    for (int64_t ib = 0; ib < k / QK_K; ib++) {
        const block_q4k *b = &xs[ib];
        float d = orc_f16_to_f32(b->d), min = orc_f16_to_f32(b->dmin);
        float *y = ys + ib * QK_K;
        int is = 0, yi = 0;
        for (int j = 0; j < QK_K; j += 64) {
            const uint8_t *q = b->qs + j / 2;
            uint8_t sc, m;
            get_scale_min_k4(is, b->scales, &sc, &m);
            float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, b->scales, &sc, &m);
            float d2 = d * (float)sc, m2 = min * (float)m;
            for (int l = 0; l < 32; l++) y[yi++] = d1 * (float)(q[l] & 0xF) - m1;
            for (int l = 0; l < 32; l++) y[yi++] = d2 * (float)(q[l] >> 4) - m2;
            is += 2;
        }
    }
    return 0;
}

/* Per-block integer parts of Q4K x Q8K (k_quants.rs:1190-1241):
 * aux32[l] = sum_j sc_j * sum_{elements = l mod 8 in sub-block j} q4*q8 ; sumi = sum_j bsums_j * m_{j/2} */
static inline void ints_q4k_q8k(const block_q4k *x, const block_q8k *y, int32_t aux32[8], int32_t *sumi) {
    int8_t aux8[QK_K];
    for (int g = 0; g < 4; g++) {
        for (int l = 0; l < 32; l++) aux8[64 * g + l] = (int8_t)(x->qs[32 * g + l] & 0xF);
        for (int l = 0; l < 32; l++) aux8[64 * g + 32 + l] = (int8_t)(x->qs[32 * g + l] >> 4);
    }
    uint8_t scales[8], mins[8];
    for (int j = 0; j < 8; j++) get_scale_min_k4(j, x->scales, &scales[j], &mins[j]);
    int32_t s = 0;
    for (int j = 0; j < 16; j++) s += (int32_t)y->bsums[j] * (int32_t)mins[j / 2];
    *sumi = s;
    for (int l = 0; l < 8; l++) aux32[l] = 0;
    const int8_t *a = aux8, *q8 = y->qs;
    for (int j = 0; j < 8; j++) {
        int32_t scale = scales[j];
        for (int r = 0; r < 4; r++) {
            for (int l = 0; l < 8; l++) {
                int16_t p = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
                aux32[l] += scale * (int32_t)p;
            }
            q8 += 8; a += 8;
        }
    }
}

/* k_quants.rs:1171-1250 (vec_dot_unopt) */
static float vec_dot_q4k_q8k(int64_t n, const block_q4k *xs, const block_q8k *ys) {
    float sums[8] = {0};
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / QK_K; i++) {
        int32_t aux32[8], sumi;
        ints_q4k_q8k(&xs[i], &ys[i], aux32, &sumi);
        float d = orc_f16_to_f32(xs[i].d) * ys[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
        float dmin = orc_f16_to_f32(xs[i].dmin) * ys[i].d;
        sumf -= dmin * (float)sumi;
    }
    float t = 0.0f;
    for (int l = 0; l < 8; l++) t += sums[l];
    return sumf + t;
}

/* ---------------------------------------------------------------- Q5K ---- */
/* k_quants.rs:1450-1525 */
int orc_quantize_q5k(const float *xs, void *out, int64_t k) {
    if (k % QK_K != 0) return -1;
    block_q5k *ys = (block_q5k *)out;
    for (int64_t ib = 0; ib < k / QK_K; ib++) {
        const float *x = xs + ib * QK_K;
        block_q5k *block = &ys[ib];
        memset(block->scales, 0, K_SCALE_SIZE); /* blocks come from zeros() in the reference */
        float mins[8], scales[8];
        for (int j = 0; j < 8; j++) make_qkx1_quants(31, 5, x + 32 * j, 32, &scales[j], &mins[j]);
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) max_scale = fmaxf(scales[j], max_scale);
        for (int j = 0; j < 8; j++) max_min = fmaxf(mins[j], max_min);
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        for (int j = 0; j < 8; j++) {
            int32_t lsi = nearest_int(inv_scale * scales[j]); if (lsi > 63) lsi = 63;
            int32_t lmi = nearest_int(inv_min * mins[j]); if (lmi > 63) lmi = 63;
            uint8_t ls = (uint8_t)lsi, lm = (uint8_t)lmi;
            if (j < 4) {
                block->scales[j] = ls;
                block->scales[j + 4] = lm;
            } else {
                block->scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                block->scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                block->scales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        block->d = orc_f32_to_f16(max_scale / 63.0f);
        block->dmin = orc_f32_to_f16(max_min / 63.0f);
        uint8_t l[QK_K];
        memset(l, 0, sizeof(l));
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            get_scale_min_k4(j, block->scales, &sc, &m);
            float d = orc_f16_to_f32(block->d) * (float)sc;
            if (d != 0.0f) {
                float dm = orc_f16_to_f32(block->dmin) * (float)m;
                for (int ii = 0; ii < 32; ii++) {
                    int32_t lv = nearest_int((x[32 * j + ii] + dm) / d);
                    l[32 * j + ii] = (uint8_t)clampi(lv, 0, 31);
                }
            }
        }
        memset(block->qh, 0, sizeof(block->qh));
        uint8_t m1 = 1, m2 = 2;
        for (int n = 0; n < QK_K; n += 64) {
            int offset = (n / 64) * 32;
            for (int j = 0; j < 32; j++) {
                uint8_t l1 = l[n + j], l2 = l[n + j + 32];
                if (l1 > 15) { l1 -= 16; block->qh[j] |= m1; }
                if (l2 > 15) { l2 -= 16; block->qh[j] |= m2; }
                block->qs[offset + j] = (uint8_t)(l1 | (l2 << 4));
            }
            m1 <<= 2;
            m2 <<= 2;
        }
    }
    return 0;
}

/* k_quants.rs:1527-1564 */
int orc_dequantize_q5k(const void *in, float *ys, int64_t k) {
    if (k % QK_K != 0) return -1;
    const block_q5k *xs = (const block_q5k *)in;
    for (int64_t ib = 0; ib < k / QK_K; ib++) {
        const block_q5k *b = &xs[ib];
        float d = orc_f16_to_f32(b->d), min = orc_f16_to_f32(b->dmin);
        float *y = ys + ib * QK_K;
        int is = 0, yi = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < QK_K; j += 64) {
            const uint8_t *ql = b->qs + j / 2;
            uint8_t sc, m;
            get_scale_min_k4(is, b->scales, &sc, &m);
            float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, b->scales, &sc, &m);
            float d2 = d * (float)sc, m2 = min * (float)m;
            for (int l = 0; l < 32; l++) y[yi++] = d1 * (float)((ql[l] & 0xF) + ((b->qh[l] & u1) ? 16 : 0)) - m1;
            for (int l = 0; l < 32; l++) y[yi++] = d2 * (float)((ql[l] >> 4) + ((b->qh[l] & u2) ? 16 : 0)) - m2;
            is += 2;
            u1 <<= 2;
            u2 <<= 2;
        }
    }
    return 0;
}

/* Per-block integer parts of Q5K x Q8K (k_quants.rs:1380-1438), as for Q4K with the fifth bit of
 * each quant taken from qh: bit 2g of qh[l] for element 64g + l, bit 2g+1 for element 64g + 32 + l. */
static inline void ints_q5k_q8k(const block_q5k *x, const block_q8k *y, int32_t aux32[8], int32_t *sumi) {
    int8_t aux8[QK_K];
    uint8_t m = 1;
    for (int g = 0; g < 4; g++) {
        for (int l = 0; l < 32; l++) aux8[64 * g + l] = (int8_t)((x->qs[32 * g + l] & 0xF) + ((x->qh[l] & m) ? 16 : 0));
        m <<= 1;
        for (int l = 0; l < 32; l++) aux8[64 * g + 32 + l] = (int8_t)((x->qs[32 * g + l] >> 4) + ((x->qh[l] & m) ? 16 : 0));
        m <<= 1;
    }
    uint8_t scales[8], mins[8];
    for (int j = 0; j < 8; j++) get_scale_min_k4(j, x->scales, &scales[j], &mins[j]);
    int32_t s = 0;
    for (int j = 0; j < 16; j++) s += (int32_t)y->bsums[j] * (int32_t)mins[j / 2];
    *sumi = s;
    for (int l = 0; l < 8; l++) aux32[l] = 0;
    const int8_t *a = aux8, *q8 = y->qs;
    for (int j = 0; j < 8; j++) {
        int32_t scale = scales[j];
        for (int r = 0; r < 4; r++) {
            for (int l = 0; l < 8; l++) {
                int16_t p = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
                aux32[l] += scale * (int32_t)p;
            }
            q8 += 8; a += 8;
        }
    }
}

/* k_quants.rs:1361-1447 (vec_dot_unopt) */
static float vec_dot_q5k_q8k(int64_t n, const block_q5k *xs, const block_q8k *ys) {
    float sums[8] = {0};
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / QK_K; i++) {
        int32_t aux32[8], sumi;
        ints_q5k_q8k(&xs[i], &ys[i], aux32, &sumi);
        float d = orc_f16_to_f32(xs[i].d) * ys[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
        float dmin = orc_f16_to_f32(xs[i].dmin) * ys[i].d;
        sumf -= dmin * (float)sumi;
    }
    float t = 0.0f;
    for (int l = 0; l < 8; l++) t += sums[l];
    return sumf + t;
}

/* ---------------------------------------------------------------- Q6K ---- */
/* utils.rs:61-198 */
static float make_qx_quants(int n, int32_t nmax, const float *x, int8_t *ls, int rmse_type) {
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.0f) {
        for (int i = 0; i < n; i++) ls[i] = 0;
        return 0.0f;
    }
    float iscale = -(float)nmax / max;
    if (rmse_type == 0) {
        for (int i = 0; i < n; i++) {
            int32_t l = nearest_int(iscale * x[i]);
            ls[i] = (int8_t)(nmax + clampi(l, -nmax, nmax - 1));
        }
        return 1.0f / iscale;
    }
    int weight_type = rmse_type % 2;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int32_t l = clampi(nearest_int(iscale * x[i]), -nmax, nmax - 1);
        ls[i] = (int8_t)(l + nmax);
        float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
        float lf = (float)l;
        sumlx += w * x[i] * lf;
        suml2 += w * lf * lf;
    }
    float scale = sumlx / suml2;
    float best = scale * sumlx;
    for (int itry = 0; itry < 3; itry++) {
        float is2 = 1.0f / scale;
        float slx = 0.0f, sl2 = 0.0f;
        int changed = 0;
        for (int i = 0; i < n; i++) {
            int32_t l = clampi(nearest_int(is2 * x[i]), -nmax, nmax - 1);
            if (l + nmax != (int32_t)ls[i]) changed = 1;
            float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
            float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;
        for (int i = 0; i < n; i++) {
            int32_t l = nearest_int(is2 * x[i]);
            ls[i] = (int8_t)(nmax + clampi(l, -nmax, nmax - 1));
        }
        sumlx = slx;
        suml2 = sl2;
        scale = sumlx / suml2;
        best = scale * sumlx;
    }
    for (int itry = 0; itry < 5; itry++) {
        int n_changed = 0;
        for (int i = 0; i < n; i++) {
            float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
            int32_t l = (int32_t)ls[i] - nmax;
            float slx = sumlx - w * x[i] * (float)l;
            if (slx > 0.0f) {
                float sl2 = suml2 - w * (float)l * (float)l;
                int32_t new_l = clampi(nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1);
                if (new_l != l) {
                    slx += w * x[i] * (float)new_l;
                    sl2 += w * (float)new_l * (float)new_l;
                    if (sl2 > 0.0f && slx * slx * suml2 > sumlx * sumlx * sl2) {
                        ls[i] = (int8_t)(nmax + new_l);
                        sumlx = slx;
                        suml2 = sl2;
                        scale = sumlx / suml2;
                        best = scale * sumlx;
                        n_changed++;
                    }
                }
            }
        }
        if (n_changed == 0) break;
    }
    if (rmse_type < 3) return scale;
    for (int is = -4; is < 4; is++) {
        if (is == 0) continue;
        iscale = -((float)nmax + 0.1f * (float)is) / max;
        float slx = 0.0f, sl2 = 0.0f;
        for (int i = 0; i < n; i++) {
            int32_t l = clampi(nearest_int(iscale * x[i]), -nmax, nmax - 1);
            float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
            float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (sl2 > 0.0f && slx * slx > best * sl2) {
            for (int i = 0; i < n; i++) {
                int32_t l = nearest_int(iscale * x[i]);
                ls[i] = (int8_t)(nmax + clampi(l, -nmax, nmax - 1));
            }
            scale = slx / sl2;
            best = scale * slx;
        }
    }
    return scale;
}

/* k_quants.rs:1643-1713 */
int orc_quantize_q6k(const float *xs, void *out, int64_t k) {
    if (k % QK_K != 0) return -1;
    block_q6k *ys = (block_q6k *)out;
    int8_t l[QK_K];
    memset(l, 0, sizeof(l));
    float scales[QK_K / 16];
    for (int64_t ib = 0; ib < k / QK_K; ib++) {
        const float *x = xs + ib * QK_K;
        block_q6k *y = &ys[ib];
        float max_scale = 0.0f, max_abs_scale = 0.0f;
        for (int j = 0; j < 16; j++) {
            float scale = make_qx_quants(16, 32, x + 16 * j, l + 16 * j, 1);
            scales[j] = scale;
            float a = fabsf(scale);
            if (a > max_abs_scale) { max_abs_scale = a; max_scale = scale; }
        }
        float iscale = -128.0f / max_scale;
        y->d = orc_f32_to_f16(1.0f / iscale);
        for (int j = 0; j < 16; j++) {
            int32_t v = nearest_int(iscale * scales[j]);
            if (v > 127) v = 127;
            y->scales[j] = (int8_t)v;
        }
        for (int j = 0; j < 16; j++) {
            float d = orc_f16_to_f32(y->d) * (float)y->scales[j];
            if (d == 0.0f) continue;
            for (int ii = 0; ii < 16; ii++) {
                int32_t ll = clampi(nearest_int(x[16 * j + ii] / d), -32, 31);
                l[16 * j + ii] = (int8_t)(ll + 32);
            }
        }
        uint8_t *ql = y->ql, *qh = y->qh;
        for (int j = 0; j < QK_K; j += 128) {
            for (int li = 0; li < 32; li++) {
                int8_t q1 = l[j + li] & 0xF;
                int8_t q2 = l[j + li + 32] & 0xF;
                int8_t q3 = l[j + li + 64] & 0xF;
                int8_t q4 = l[j + li + 96] & 0xF;
                ql[li] = (uint8_t)(q1 | (q3 << 4));
                ql[li + 32] = (uint8_t)(q2 | (q4 << 4));
                qh[li] = (uint8_t)((l[j + li] >> 4) | ((l[j + li + 32] >> 4) << 2) |
                                   ((l[j + li + 64] >> 4) << 4) | ((l[j + li + 96] >> 4) << 6));
            }
            ql += 64;
            qh += 32;
        }
    }
    return 0;
}

/* k_quants.rs:1716-1746 */
int orc_dequantize_q6k(const void *in, float *ys, int64_t k) {
    if (k % QK_K != 0) return -1;
    const block_q6k *xs = (const block_q6k *)in;
    for (int64_t ib = 0; ib < k / QK_K; ib++) {
        const block_q6k *x = &xs[ib];
        float d = orc_f16_to_f32(x->d);
        for (int n = 0; n < QK_K; n += 128) {
            int idx = n / 128;
            float *y = ys + ib * QK_K + n;
            const int8_t *sc = x->scales + 8 * idx;
            const uint8_t *ql = x->ql + 64 * idx;
            const uint8_t *qh = x->qh + 32 * idx;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int8_t q1 = (int8_t)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32;
                int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int8_t q3 = (int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l] = d * (float)sc[is] * (float)q1;
                y[l + 32] = d * (float)sc[is + 2] * (float)q2;
                y[l + 64] = d * (float)sc[is + 4] * (float)q3;
                y[l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
        }
    }
    return 0;
}

static inline void unpack_q6k(const block_q6k *x, int8_t aux8[QK_K]) {
    for (int j = 0; j < QK_K; j += 128) {
        int8_t *a = aux8 + j;
        const uint8_t *q4 = x->ql + j / 2;
        const uint8_t *qh = x->qh + j / 4;
        for (int l = 0; l < 32; l++) {
            a[l] = (int8_t)((int32_t)((q4[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
            a[l + 32] = (int8_t)((int32_t)((q4[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
            a[l + 64] = (int8_t)((int32_t)((q4[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            a[l + 96] = (int8_t)((int32_t)((q4[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
        }
    }
}

/* k_quants.rs:1585-1641 (vec_dot_unopt); aux32 is f32 in the reference. */
static float vec_dot_q6k_q8k(int64_t n, const block_q6k *xs, const block_q8k *ys) {
    int8_t aux8[QK_K];
    float sums[8] = {0};
    for (int64_t i = 0; i < n / QK_K; i++) {
        const block_q6k *x = &xs[i];
        const block_q8k *y = &ys[i];
        float aux32[8] = {0};
        unpack_q6k(x, aux8);
        for (int j = 0; j < 16; j++) {
            float scale = (float)x->scales[j];
            const int8_t *q8 = y->qs + 16 * j;
            const int8_t *a = aux8 + 16 * j;
            for (int l = 0; l < 8; l++) aux32[l] += scale * (float)(int16_t)((int16_t)q8[l] * (int16_t)a[l]);
            for (int l = 0; l < 8; l++) aux32[l] += scale * (float)(int16_t)((int16_t)q8[l + 8] * (int16_t)a[l + 8]);
        }
        float d = orc_f16_to_f32(x->d) * y->d;
        for (int l = 0; l < 8; l++) sums[l] += aux32[l] * d;
    }
    float t = 0.0f;
    for (int l = 0; l < 8; l++) t += sums[l];
    return t;
}

/* Integer I_b = sum_j sc_j * sum_16 (q6-32)*q8 for one block (exact int32). */
static inline int32_t int_q6k_q8k(const block_q6k *x, const block_q8k *y) {
    int8_t aux8[QK_K];
    unpack_q6k(x, aux8);
    int32_t total = 0;
    for (int j = 0; j < 16; j++) {
        int32_t s = 0;
        for (int l = 0; l < 16; l++) s += (int32_t)aux8[16 * j + l] * (int32_t)y->qs[16 * j + l];
        total += (int32_t)x->scales[j] * s;
    }
    return total;
}

/* ---------------------------------------------------------------- Q2K ---- */
/* the two-bit quant of element e */
static inline int32_t q2k_quant(const block_q2k *b, int e) {
    return (b->qs[32 * (e / 128) + e % 32] >> (2 * ((e % 128) / 32))) & 3;
}

/* k_quants.rs:770-839 (from_float; make_qkx1_quants(3, 5, 16 elements), utils.rs:201-258) */
int orc_quantize_q2k(const float *xs, void *out, int64_t k) {
    if (k % QK_K != 0) return -1;
    block_q2k *ys = (block_q2k *)out;
    const float Q4SCALE = 15.0f;
    for (int64_t i = 0; i < k / QK_K; i++) {
        const float *x = xs + i * QK_K;
        block_q2k *block = &ys[i];
        float mins[QK_K / 16], scales[QK_K / 16];
        for (int j = 0; j < QK_K / 16; j++) make_qkx1_quants(3, 5, x + 16 * j, 16, &scales[j], &mins[j]);
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < QK_K / 16; j++) {
            max_scale = fmaxf(scales[j], max_scale);
            max_min = fmaxf(mins[j], max_min);
        }
        if (max_scale > 0.0f) {
            float iscale = Q4SCALE / max_scale;
            for (int j = 0; j < QK_K / 16; j++) block->scales[j] = (uint8_t)nearest_int(iscale * scales[j]);
            block->d = orc_f32_to_f16(max_scale / Q4SCALE);
        } else {
            for (int j = 0; j < QK_K / 16; j++) block->scales[j] = 0;
            block->d = orc_f32_to_f16(0.0f);
        }
        if (max_min > 0.0f) {
            float iscale = Q4SCALE / max_min;
            for (int j = 0; j < QK_K / 16; j++) {
                uint8_t l = (uint8_t)nearest_int(iscale * mins[j]);
                block->scales[j] |= (uint8_t)(l << 4);
            }
            block->dmin = orc_f32_to_f16(max_min / Q4SCALE);
        } else {
            block->dmin = orc_f32_to_f16(0.0f);
        }
        uint8_t big_l[QK_K];
        memset(big_l, 0, sizeof big_l);
        for (int j = 0; j < QK_K / 16; j++) {
            float d = orc_f16_to_f32(block->d) * (float)(block->scales[j] & 0xF);
            if (d == 0.0f) continue;
            float dm = orc_f16_to_f32(block->dmin) * (float)(block->scales[j] >> 4);
            for (int ii = 0; ii < 16; ii++)
                big_l[16 * j + ii] = (uint8_t)clampi(nearest_int((x[16 * j + ii] + dm) / d), 0, 3);
        }
        for (int j = 0; j < QK_K; j += 128)
            for (int ll = 0; ll < 32; ll++)
                block->qs[j / 4 + ll] = (uint8_t)(big_l[j + ll] | (big_l[j + ll + 32] << 2) | (big_l[j + ll + 64] << 4) | (big_l[j + ll + 96] << 6));
    }
    return 0;
}

/* k_quants.rs:841-872 (to_float): y = (d * sc) * q - (dmin * m) */
int orc_dequantize_q2k(const void *in, float *ys, int64_t k) {
    if (k % QK_K != 0) return -1;
    const block_q2k *xs = (const block_q2k *)in;
    for (int64_t i = 0; i < k / QK_K; i++) {
        float d = orc_f16_to_f32(xs[i].d), min = orc_f16_to_f32(xs[i].dmin);
        for (int e = 0; e < QK_K; e++) {
            uint8_t sc = xs[i].scales[e / 16];
            float dl = d * (float)(sc & 0xF), ml = min * (float)(sc >> 4);
            ys[i * QK_K + e] = dl * (float)q2k_quant(&xs[i], e) - ml;
        }
    }
    return 0;
}

/* k_quants.rs:717-767 (vec_dot_unopt of Q2K x Q8K): per block dall * isum - dmin * summs */
static void ints_q2k_q8k(const block_q2k *x, const block_q8k *y, int32_t *isum, int32_t *summs) {
    int32_t s = 0, t = 0;
    for (int j = 0; j < QK_K / 16; j++) {
        s += (int32_t)y->bsums[j] * (int32_t)(x->scales[j] >> 4);
        int32_t isuml = 0;
        for (int l = 0; l < 16; l++) isuml += (int32_t)y->qs[16 * j + l] * q2k_quant(x, 16 * j + l);
        t += (int32_t)(x->scales[j] & 0xF) * isuml;
    }
    *isum = t;
    *summs = s;
}
static float vec_dot_q2k_q8k(int64_t n, const block_q2k *xs, const block_q8k *ys) {
    float sumf = 0.0f;
    for (int64_t i = 0; i < n / QK_K; i++) {
        int32_t isum, summs;
        ints_q2k_q8k(&xs[i], &ys[i], &isum, &summs);
        float dall = ys[i].d * orc_f16_to_f32(xs[i].d);
        float dmin = ys[i].d * orc_f16_to_f32(xs[i].dmin);
        sumf += dall * (float)isum - dmin * (float)summs;
    }
    return sumf;
}

/* ---------------------------------------------------------------- Q3K ---- */
/* utils.rs:261-326 (make_q3_quants; from_float calls it with nmax = 4, do_rmse = true and uses the returned
 * scale only) */
static float make_q3_quants(const float *x, int n, int32_t nmax, int do_rmse) {
    int8_t l[32];
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.0f) return 0.0f;
    float iscale = -(float)nmax / max;
    if (do_rmse) {
        float sumlx = 0.0f, suml2 = 0.0f;
        for (int i = 0; i < n; i++) {
            int32_t li = clampi(nearest_int(iscale * x[i]), -nmax, nmax - 1);
            l[i] = (int8_t)li;
            float w = x[i] * x[i];
            sumlx += w * x[i] * (float)li;
            suml2 += w * (float)(li * li);
        }
        for (int t = 0; t < 5; t++) {
            int n_changed = 0;
            for (int i = 0; i < n; i++) {
                float w = x[i] * x[i];
                float slx = sumlx - w * x[i] * (float)l[i];
                if (slx > 0.0f) {
                    float sl2 = suml2 - w * (float)((int32_t)l[i] * (int32_t)l[i]);
                    int32_t new_l = clampi(nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1);
                    if (new_l != (int32_t)l[i]) {
                        slx += w * x[i] * (float)new_l;
                        sl2 += w * (float)(new_l * new_l);
                        if (sl2 > 0.0f && slx * slx * suml2 > sumlx * sumlx * sl2) {
                            l[i] = (int8_t)new_l;
                            sumlx = slx;
                            suml2 = sl2;
                            n_changed++;
                        }
                    }
                }
            }
            if (n_changed == 0) break;
        }
        return sumlx / suml2;
    }
    return 1.0f / iscale;
}

/* the 6-bit scale of 16-element group j, k_quants.rs:1055-1061 */
static inline int32_t q3k_scale(const block_q3k *b, int j) {
    int32_t sc = j < 8 ? (b->scales[j] & 0xF) : (b->scales[j - 8] >> 4);
    return sc | (((b->scales[8 + j % 4] >> (2 * (j / 4))) & 3) << 4);
}
/* the signed 3-bit quant of element e: two low bits from qs, minus 4 unless its hmask bit is set */
static inline int32_t q3k_quant(const block_q3k *b, int e) {
    int half = e / 128, r = e % 128;
    int32_t low = (b->qs[32 * half + r % 32] >> (2 * (r / 32))) & 3;
    return low - ((b->hmask[e % 32] >> (e / 32)) & 1 ? 0 : 4);
}

/* k_quants.rs:1011-1090 (from_float) */
int orc_quantize_q3k(const float *xs, void *out, int64_t k) {
    if (k % QK_K != 0) return -1;
    block_q3k *ys = (block_q3k *)out;
    for (int64_t i = 0; i < k / QK_K; i++) {
        const float *x = xs + i * QK_K;
        block_q3k *block = &ys[i];
        float scales[QK_K / 16];
        for (int j = 0; j < QK_K / 16; j++) scales[j] = make_q3_quants(x + 16 * j, 16, 4, 1);
        float max_scale = 0.0f;
        for (int j = 0; j < QK_K / 16; j++)
            if (fabsf(scales[j]) > fabsf(max_scale)) max_scale = scales[j];
        memset(block->scales, 0, 12);
        if (max_scale != 0.0f) {
            float iscale = -32.0f / max_scale;
            for (int j = 0; j < QK_K / 16; j++) {
                int32_t l_val = clampi(nearest_int(iscale * scales[j]), -32, 31) + 32;
                if (j < 8) block->scales[j] = (uint8_t)(l_val & 0xF);
                else block->scales[j - 8] |= (uint8_t)((l_val & 0xF) << 4);
                l_val >>= 4;
                block->scales[j % 4 + 8] |= (uint8_t)(l_val << (2 * (j / 4)));
            }
            block->d = orc_f32_to_f16(1.0f / iscale);
        } else {
            block->d = orc_f32_to_f16(0.0f);
        }
        int8_t l[QK_K];
        memset(l, 0, sizeof l);
        for (int j = 0; j < QK_K / 16; j++) {
            int32_t sc = q3k_scale(block, j) - 32;
            float d = orc_f16_to_f32(block->d) * (float)sc;
            if (d != 0.0f) {
                for (int ii = 0; ii < 16; ii++) {
                    int32_t l_val = nearest_int(x[16 * j + ii] / d);
                    l[16 * j + ii] = (int8_t)(clampi(l_val, -4, 3) + 4);
                }
            }
        }
        memset(block->hmask, 0, QK_K / 8);
        int m = 0;
        uint8_t hm = 1;
        for (int e = 0; e < QK_K; e++) {
            if (l[e] > 3) { block->hmask[m] |= hm; l[e] -= 4; }
            if (++m == QK_K / 8) { m = 0; hm = (uint8_t)(hm << 1); }
        }
        for (int j = 0; j < QK_K; j += 128)
            for (int lv = 0; lv < 32; lv++)
                block->qs[j / 4 + lv] = (uint8_t)(l[j + lv] | (l[j + lv + 32] << 2) | (l[j + lv + 64] << 4) | (l[j + lv + 96] << 6));
    }
    return 0;
}

/* k_quants.rs:1094-1146 (to_float): y = (d_all * (scale - 32)) * q */
int orc_dequantize_q3k(const void *in, float *ys, int64_t k) {
    if (k % QK_K != 0) return -1;
    const block_q3k *xs = (const block_q3k *)in;
    for (int64_t i = 0; i < k / QK_K; i++) {
        float d_all = orc_f16_to_f32(xs[i].d);
        for (int e = 0; e < QK_K; e++) {
            float dl = d_all * ((float)(int8_t)q3k_scale(&xs[i], e / 16) - 32.0f);
            ys[i * QK_K + e] = dl * (float)(int8_t)q3k_quant(&xs[i], e);
        }
    }
    return 0;
}

/* k_quants.rs:890-1009 (vec_dot_unopt of Q3K x Q8K): eight integer lanes (element index mod 8) per block,
 * sums[l] += (d * d8) * aux32[l], the eight sums added at the end. */
static void ints_q3k_q8k(const block_q3k *x, const block_q8k *y, int32_t aux32[8]) {
    for (int l = 0; l < 8; l++) aux32[l] = 0;
    for (int j = 0; j < QK_K / 16; j++) {
        int32_t scale = q3k_scale(x, j) - 32;
        for (int h = 0; h < 2; h++)
            for (int l = 0; l < 8; l++) {
                int e = 16 * j + 8 * h + l;
                int16_t p = (int16_t)((int16_t)y->qs[e] * (int16_t)q3k_quant(x, e));
                aux32[l] += scale * (int32_t)p;
            }
    }
}
static float vec_dot_q3k_q8k(int64_t n, const block_q3k *xs, const block_q8k *ys) {
    float sums[8] = {0};
    for (int64_t i = 0; i < n / QK_K; i++) {
        int32_t aux32[8];
        ints_q3k_q8k(&xs[i], &ys[i], aux32);
        float d = orc_f16_to_f32(xs[i].d) * ys[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
    }
    float total = 0.0f;
    for (int l = 0; l < 8; l++) total += sums[l];
    return total;
}

/* -------------------------------------------------------- type dispatch ---- */
int64_t orc_block_size(int dtype) {
    switch (dtype) {
    case ORC_Q4_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: case ORC_Q8_0: case ORC_Q8_1: return 32;
    case ORC_Q2K: case ORC_Q3K: case ORC_Q4K: case ORC_Q5K: case ORC_Q6K: case ORC_Q8K: return QK_K;
    default: return 0;
    }
}
int64_t orc_type_size(int dtype) {
    switch (dtype) {
    case ORC_Q4_0: return 18; case ORC_Q4_1: return 20; case ORC_Q5_0: return 22; case ORC_Q5_1: return 24; case ORC_Q8_0: return 34; case ORC_Q8_1: return 36;
    case ORC_Q2K: return 84; case ORC_Q3K: return 110; case ORC_Q4K: return 144; case ORC_Q5K: return 176; case ORC_Q6K: return 210; case ORC_Q8K: return 292;
    default: return 0;
    }
}
/* The activation type each weight type is contracted with (VecDotType,
 * k_quants.rs:160, :565, :1155, :1569, :1752). */
int orc_vec_dot_type(int dtype) {
    switch (dtype) {
    case ORC_Q4_0: case ORC_Q5_0: case ORC_Q8_0: return ORC_Q8_0;   /* Q5_0: k_quants.rs:356 */
    case ORC_Q4_1: case ORC_Q5_1: return ORC_Q8_1;   /* k_quants.rs:260, :457 */
    case ORC_Q2K: case ORC_Q3K: case ORC_Q4K: case ORC_Q5K: case ORC_Q6K: case ORC_Q8K: return ORC_Q8K;   /* Q2K: k_quants.rs:701, Q3K: :877 */
    default: return -1;
    }
}

int orc_quantize(int dtype, const float *xs, void *out, int64_t k) {
    switch (dtype) {
    case ORC_Q4_0: return orc_quantize_q4_0(xs, out, k);
    case ORC_Q4_1: return orc_quantize_q4_1(xs, out, k);
    case ORC_Q5_0: return orc_quantize_q5_0(xs, out, k);
    case ORC_Q5_1: return orc_quantize_q5_1(xs, out, k);
    case ORC_Q2K: return orc_quantize_q2k(xs, out, k);
    case ORC_Q3K: return orc_quantize_q3k(xs, out, k);
    case ORC_Q8_0: return orc_quantize_q8_0(xs, out, k);
    case ORC_Q8_1: return orc_quantize_q8_1(xs, out, k);
    case ORC_Q4K: return orc_quantize_q4k(xs, out, k);
    case ORC_Q5K: return orc_quantize_q5k(xs, out, k);
    case ORC_Q6K: return orc_quantize_q6k(xs, out, k);
    case ORC_Q8K: memset(out, 0, (size_t)(k / QK_K) * 292); return orc_quantize_q8k(xs, out, k);
    default: return -2;
    }
}

int orc_dequantize(int dtype, const void *in, float *ys, int64_t k) {
    switch (dtype) {
    case ORC_Q4_0: return orc_dequantize_q4_0(in, ys, k);
    case ORC_Q4_1: return orc_dequantize_q4_1(in, ys, k);
    case ORC_Q5_0: return orc_dequantize_q5_0(in, ys, k);
    case ORC_Q5_1: return orc_dequantize_q5_1(in, ys, k);
    case ORC_Q2K: return orc_dequantize_q2k(in, ys, k);
    case ORC_Q3K: return orc_dequantize_q3k(in, ys, k);
    case ORC_Q8_0: return orc_dequantize_q8_0(in, ys, k);
    case ORC_Q4K: return orc_dequantize_q4k(in, ys, k);
    case ORC_Q5K: return orc_dequantize_q5k(in, ys, k);
    case ORC_Q6K: return orc_dequantize_q6k(in, ys, k);
    case ORC_Q8K: return orc_dequantize_q8k(in, ys, k);
    default: return -2;
    }
}

/* T::vec_dot_unopt(n, xs, ys) for weight type `dtype`; ys is its VecDotType. */
int orc_vec_dot(int dtype, int64_t n, const void *xs, const void *ys, float *out) {
    int64_t bs = orc_block_size(dtype);
    if (bs == 0 || n % bs != 0) return -1;
    switch (dtype) {
    case ORC_Q4_0: *out = vec_dot_q4_0_q8_0(n, xs, ys); return 0;
    case ORC_Q4_1: return vec_dot_q4_1_q8_1(n, xs, ys, out);
    case ORC_Q5_0:
        if ((n / 32) % 2 != 0) return -1;   /* k_quants.rs:363: nb is not divisible by 2 */
        *out = vec_dot_q5_0_q8_0(n, xs, ys);
        return 0;
    case ORC_Q5_1: return vec_dot_q5_1_q8_1(n, xs, ys, out);
    case ORC_Q2K: *out = vec_dot_q2k_q8k(n, xs, ys); return 0;
    case ORC_Q3K: *out = vec_dot_q3k_q8k(n, xs, ys); return 0;
    case ORC_Q8_0: *out = vec_dot_q8_0_q8_0(n, xs, ys); return 0;
    case ORC_Q4K: *out = vec_dot_q4k_q8k(n, xs, ys); return 0;
    case ORC_Q5K: *out = vec_dot_q5k_q8k(n, xs, ys); return 0;
    case ORC_Q6K: *out = vec_dot_q6k_q8k(n, xs, ys); return 0;
    case ORC_Q8K: *out = vec_dot_q8k_q8k(n, xs, ys); return 0;
    default: return -2;
    }
}

/* k_quants.rs:1842-1883: quantize every lhs row to the VecDotType, then
 * dst[row*n + col] = vec_dot(k, rhs_t[col], lhs_b[row]).  (rayon only changes
 * scheduling: one task computes one element.) */
int orc_matmul(int dtype, int64_t m, int64_t k, int64_t n, const float *lhs, const void *rhs_t,
               float *dst) {
    int64_t bs = orc_block_size(dtype);
    int adt = orc_vec_dot_type(dtype);
    if (bs == 0 || adt < 0 || k % bs != 0) return -1;
    int64_t abs_ = orc_block_size(adt), ats = orc_type_size(adt), wts = orc_type_size(dtype);
    int64_t a_row_bytes = k / abs_ * ats, w_row_bytes = k / bs * wts;
    uint8_t *lhs_b = (uint8_t *)calloc((size_t)(m * a_row_bytes) + 1, 1);
    if (!lhs_b) return -3;
    for (int64_t r = 0; r < m; r++) {
        int rc = orc_quantize(adt, lhs + r * k, lhs_b + r * a_row_bytes, k);
        if (rc) { free(lhs_b); return rc; }
    }
    for (int64_t r = 0; r < m; r++) {
        for (int64_t c = 0; c < n; c++) {
            float v;
            int rc = orc_vec_dot(dtype, k, (const uint8_t *)rhs_t + c * w_row_bytes, lhs_b + r * a_row_bytes, &v);
            if (rc) { free(lhs_b); return rc; }   /* vec_dot's Err ends the matmul (k_quants.rs:1876-1880) */
            dst[r * n + c] = v;
        }
    }
    free(lhs_b);
    return 0;
}

/* Per-block integer dot products, the quantities that must be bit-exact on
 * the GPU.  `acts` are already-quantized activation rows (VecDotType blocks),
 * out_i[(r*n + c)*kb + b] = I_b, out_mn likewise = Mn_b (Q4K only; may be NULL
 * for other types).  Q4_0/Q8_0/Q8K: I_b = sumi of the block. */
int orc_block_int_dots(int dtype, int64_t m, int64_t k, int64_t n, const void *acts,
                       const void *rhs_t, int32_t *out_i, int32_t *out_mn) {
    int64_t bs = orc_block_size(dtype);
    int adt = orc_vec_dot_type(dtype);
    if (bs == 0 || adt < 0 || k % bs != 0) return -1;
    int64_t kb = k / bs;
    int64_t ats = orc_type_size(adt), wts = orc_type_size(dtype);
    for (int64_t r = 0; r < m; r++) {
        for (int64_t c = 0; c < n; c++) {
            const uint8_t *w = (const uint8_t *)rhs_t + c * kb * wts;
            const uint8_t *a = (const uint8_t *)acts + r * kb * ats;
            for (int64_t b = 0; b < kb; b++) {
                int64_t o = (r * n + c) * kb + b;
                switch (dtype) {
                case ORC_Q4_0:
                    out_i[o] = sumi_q4_0_q8_0((const block_q4_0 *)w + b, (const block_q8_0 *)a + b);
                    break;
                case ORC_Q8_0:
                    out_i[o] = sumi_q8_0_q8_0((const block_q8_0 *)w + b, (const block_q8_0 *)a + b);
                    break;
                case ORC_Q5_0:
                    out_i[o] = sumi_q5_0_q8_0((const block_q5_0 *)w + b, (const block_q8_0 *)a + b);
                    break;
                case ORC_Q4_1:
                    out_i[o] = sumi_q4_1_q8_1((const block_q4_1 *)w + b, (const block_q8_1 *)a + b);
                    break;
                case ORC_Q5_1:
                    out_i[o] = sumi_q5_1_q8_1((const block_q5_1 *)w + b, (const block_q8_1 *)a + b);
                    break;
                case ORC_Q2K: {
                    int32_t isum, summs;
                    ints_q2k_q8k((const block_q2k *)w + b, (const block_q8k *)a + b, &isum, &summs);
                    out_i[o] = isum;
                    if (out_mn) out_mn[o] = summs;
                    break;
                }
                case ORC_Q3K: {
                    int32_t aux32[8], t = 0;
                    ints_q3k_q8k((const block_q3k *)w + b, (const block_q8k *)a + b, aux32);
                    for (int l = 0; l < 8; l++) t += aux32[l];
                    out_i[o] = t;
                    break;
                }
                case ORC_Q8K:
                    out_i[o] = sumi_q8k_q8k((const block_q8k *)w + b, (const block_q8k *)a + b);
                    break;
                case ORC_Q4K: {
                    int32_t aux32[8], sumi, t = 0;
                    ints_q4k_q8k((const block_q4k *)w + b, (const block_q8k *)a + b, aux32, &sumi);
                    for (int l = 0; l < 8; l++) t += aux32[l];
                    out_i[o] = t;
                    if (out_mn) out_mn[o] = sumi;
                    break;
                }
                case ORC_Q5K: {
                    int32_t aux32[8], sumi, t = 0;
                    ints_q5k_q8k((const block_q5k *)w + b, (const block_q8k *)a + b, aux32, &sumi);
                    for (int l = 0; l < 8; l++) t += aux32[l];
                    out_i[o] = t;
                    if (out_mn) out_mn[o] = sumi;
                    break;
                }
                case ORC_Q6K:
                    out_i[o] = int_q6k_q8k((const block_q6k *)w + b, (const block_q8k *)a + b);
                    break;
                default: return -2;
                }
            }
        }
    }
    return 0;
}

/* ------------------------------------------------ Q8_1-activation variant ---- */
/* The reference's CUDA prefill path contracts K-quant weights with Q8_1
 * activation blocks (quantized.cu:2141-2166 for Q4K, :2258-2281 for Q6K):
 *   Q4K: sum over 32-wide sub-blocks j of  d*sc_j*d8_j*dot(q4,q8) - dmin*m_j*s8_j
 *        where s8_j is the Q8_1 block's `s` field (d8 * sum q8),
 *   Q6K: sum over 16-wide groups of d*sc*d8*dot(q6-32, q8) (d8 of the enclosing 32-block).
 * Here the activations are produced with the CPU rounding rule of
 * BlockQ8_1::from_float, not the CUDA kernel's.  PARITY UNPINNED (see header). */
int orc_matmul_q8_1(int dtype, int64_t m, int64_t k, int64_t n, const float *lhs, const void *rhs_t,
                    float *dst) {
    if ((dtype != ORC_Q4K && dtype != ORC_Q6K) || k % QK_K != 0) return -1;
    int64_t kb = k / QK_K, nb32 = k / 32;
    block_q8_1 *acts = (block_q8_1 *)calloc((size_t)(m * nb32), sizeof(block_q8_1));
    if (!acts) return -3;
    for (int64_t r = 0; r < m; r++) orc_quantize_q8_1(lhs + r * k, acts + r * nb32, k);
    for (int64_t r = 0; r < m; r++) {
        for (int64_t c = 0; c < n; c++) {
            float sumf = 0.0f;
            for (int64_t b = 0; b < kb; b++) {
                const block_q8_1 *a = acts + r * nb32 + b * 8;
                if (dtype == ORC_Q4K) {
                    const block_q4k *w = (const block_q4k *)rhs_t + c * kb + b;
                    float d = orc_f16_to_f32(w->d), dmin = orc_f16_to_f32(w->dmin);
                    float sumf_d = 0.0f, sumf_m = 0.0f;
                    for (int j = 0; j < 8; j++) {
                        uint8_t sc, mn;
                        get_scale_min_k4(j, w->scales, &sc, &mn);
                        int32_t dot = 0;
                        for (int l = 0; l < 32; l++) {
                            uint8_t q = w->qs[32 * (j / 2) + l];
                            int32_t v = (j & 1) ? (q >> 4) : (q & 0xF);
                            dot += v * (int32_t)a[j].qs[l];
                        }
                        float d8 = orc_f16_to_f32(a[j].d);
                        sumf_d += d8 * (float)(dot * (int32_t)sc);
                        sumf_m += orc_f16_to_f32(a[j].s) * (float)mn;
                    }
                    sumf += d * sumf_d - dmin * sumf_m;
                } else {
                    const block_q6k *w = (const block_q6k *)rhs_t + c * kb + b;
                    int8_t aux8[QK_K];
                    unpack_q6k(w, aux8);
                    float d = orc_f16_to_f32(w->d);
                    float acc = 0.0f;
                    for (int j = 0; j < 16; j++) {
                        int32_t dot = 0;
                        for (int l = 0; l < 16; l++)
                            dot += (int32_t)aux8[16 * j + l] * (int32_t)a[j / 2].qs[(j & 1) * 16 + l];
                        acc += (float)w->scales[j] * (orc_f16_to_f32(a[j / 2].d) * (float)dot);
                    }
                    sumf += d * acc;
                }
            }
            dst[r * n + c] = sumf;
        }
    }
    free(acts);
    return 0;
}

/* -------------------------------------------------------------- MoE FFN ---- */
/* candle-nn/src/ops.rs:296-325 (softmax over the last dim, f32) */
void orc_softmax_last_dim(const float *src, float *dst, int64_t rows, int64_t dim) {
    for (int64_t r = 0; r < rows; r++) {
        const float *s = src + r * dim;
        float *d = dst + r * dim;
        float max = -INFINITY;
        for (int64_t i = 0; i < dim; i++) max = fmaxf(max, s[i]);
        for (int64_t i = 0; i < dim; i++) d[i] = expf(s[i] - max);
        float sum = 0.0f;
        for (int64_t i = 0; i < dim; i++) sum += d[i];
        for (int64_t i = 0; i < dim; i++) d[i] /= sum;
    }
}

/* quantized_llama.rs:94-111: per token, experts sorted by descending routing
 * weight (stable), the first top_k kept, weights renormalised by their sum.
 * Output is CSR over experts: rows of expert e are row_ids[offsets[e]..offsets[e+1]],
 * in increasing token order, with weights in the same positions. */
int orc_moe_route(const float *routing_weights, int64_t tokens, int n_experts, int top_k,
                  int32_t *offsets, int32_t *row_ids, float *weights) {
    if (n_experts > 64 || top_k > n_experts) return -1;
    int32_t *count = (int32_t *)calloc((size_t)n_experts + 1, sizeof(int32_t));
    int32_t *sel = (int32_t *)malloc(sizeof(int32_t) * (size_t)(tokens * top_k));
    float *selw = (float *)malloc(sizeof(float) * (size_t)(tokens * top_k));
    for (int64_t t = 0; t < tokens; t++) {
        const float *rw = routing_weights + t * n_experts;
        int idx[64];
        for (int i = 0; i < n_experts; i++) idx[i] = i;
        /* stable insertion sort, descending by rw (sort_by(|i,j| rw[j].total_cmp(rw[i]))) */
        for (int i = 1; i < n_experts; i++) {
            int v = idx[i], j = i - 1;
            while (j >= 0 && rw[idx[j]] < rw[v]) { idx[j + 1] = idx[j]; j--; }
            idx[j + 1] = v;
        }
        float sum = 0.0f;
        for (int i = 0; i < top_k; i++) sum += rw[idx[i]];
        for (int i = 0; i < top_k; i++) {
            sel[t * top_k + i] = idx[i];
            selw[t * top_k + i] = rw[idx[i]] / sum;
            count[idx[i]]++;
        }
    }
    offsets[0] = 0;
    for (int e = 0; e < n_experts; e++) offsets[e + 1] = offsets[e] + count[e];
    memset(count, 0, sizeof(int32_t) * (size_t)n_experts);
    for (int64_t t = 0; t < tokens; t++)
        for (int i = 0; i < top_k; i++) {
            int e = sel[t * top_k + i];
            int32_t p = offsets[e] + count[e]++;
            row_ids[p] = (int32_t)t;
            weights[p] = selw[t * top_k + i];
        }
    free(count); free(sel); free(selw);
    return 0;
}

/* quantized_llama.rs:56-63 and :116-135: for each expert in increasing index
 * with at least one token: gather rows, y_e = W2(silu(W1 x) * W3 x), scale each
 * row by its routing weight, index_add into ys (sequential +=,
 * cpu_backend/mod.rs:619-653).  silu = v / (1 + exp(-v)) (op.rs:607-609).
 * w1/w3: [ffn, hidden] of dtype13; w2: [hidden, ffn] of dtype2. */
int orc_moe_ffn(int n_experts, int dtype13, int dtype2, const void *const *w1, const void *const *w2,
                const void *const *w3, int64_t hidden, int64_t ffn, const float *xs, int64_t tokens,
                const int32_t *offsets, const int32_t *row_ids, const float *weights, float *ys) {
    memset(ys, 0, sizeof(float) * (size_t)(tokens * hidden));
    for (int e = 0; e < n_experts; e++) {
        int64_t te = offsets[e + 1] - offsets[e];
        if (te == 0) continue;
        float *cur = (float *)malloc(sizeof(float) * (size_t)(te * hidden));
        float *h1 = (float *)malloc(sizeof(float) * (size_t)(te * ffn));
        float *h3 = (float *)malloc(sizeof(float) * (size_t)(te * ffn));
        float *out = (float *)malloc(sizeof(float) * (size_t)(te * hidden));
        for (int64_t i = 0; i < te; i++)
            memcpy(cur + i * hidden, xs + (int64_t)row_ids[offsets[e] + i] * hidden, sizeof(float) * (size_t)hidden);
        int rc = orc_matmul(dtype13, te, hidden, ffn, cur, w1[e], h1);
        if (!rc) rc = orc_matmul(dtype13, te, hidden, ffn, cur, w3[e], h3);
        if (!rc) {
            for (int64_t i = 0; i < te * ffn; i++) {
                float v = h1[i];
                float s = v / (1.0f + expf(-v));
                h1[i] = s * h3[i];
            }
            rc = orc_matmul(dtype2, te, ffn, hidden, h1, w2[e], out);
        }
        if (!rc) {
            for (int64_t i = 0; i < te; i++) {
                float w = weights[offsets[e] + i];
                float *dst = ys + (int64_t)row_ids[offsets[e] + i] * hidden;
                for (int64_t j = 0; j < hidden; j++) dst[j] += out[i * hidden + j] * w;
            }
        }
        free(cur); free(h1); free(h3); free(out);
        if (rc) return rc;
    }
    return 0;
}

/* candle-nn/src/ops.rs:482-495 (RmsNorm::cpu_fwd, f32): per row of `dim` elements the squares are
 * added one by one in f32, m = sqrt(sum / dim + eps), then dst = src / m * alpha. */
void orc_rms_norm(const float *x, const float *alpha, float eps, int64_t rows, int64_t dim, float *out) {
    for (int64_t r = 0; r < rows; r++) {
        const float *src = x + r * dim;
        float *dst = out + r * dim;
        float sum2 = 0.0f;
        for (int64_t i = 0; i < dim; i++) sum2 += src[i] * src[i];
        float m = sqrtf(sum2 / (float)dim + eps);
        for (int64_t i = 0; i < dim; i++) dst[i] = src[i] / m * alpha[i];
    }
}

/* quantized_llama.rs:60-62: silu(w1) * w3 with silu(v) = v / (1 + exp(-v)) (op.rs:607-609). */
void orc_silu_mul(const float *a, const float *b, int64_t count, float *out) {
    for (int64_t i = 0; i < count; i++) {
        float v = a[i];
        float s = v / (1.0f + expf(-v));
        out[i] = s * b[i];
    }
}
