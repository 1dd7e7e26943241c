// Timed CPU baseline: the reference's CPU QMatMul restated for AVX2 + threads.
// TEST / BENCH INFRASTRUCTURE ONLY - never linked into the product.
//
// Work decomposition of k_quants::matmul (candle-core/src/quantized/k_quants.rs:1842-1883):
// every activation row is quantized to the weight type's VecDotType serially, then for each
// activation row the output columns are split over threads (rayon chunks of 128..512 columns
// there; OpenMP dynamic chunks of 256 here) and each output is one vec_dot over K.
// Inner loops follow the AVX2 formulation of candle-core/src/quantized/avx.rs
// (q4_0 :51-69, q8_0 :72-88, q6k :132-217, q4k :442-523): maddubs/madd integer dots, one f32
// fused multiply-add per block into eight lanes, horizontal sum at the end.
// Checked against the scalar oracle to <= 1e-6 * K absolute (the reference's own criterion for
// its SIMD paths, candle-core/tests/quantized_tests.rs:836).
#include <immintrin.h>
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

namespace {

#pragma pack(push, 1)
struct BQ4_0 { uint16_t d; uint8_t qs[16]; };
struct BQ8_0 { uint16_t d; int8_t qs[32]; };
struct BQ4K { uint16_t d, dmin; uint8_t scales[12]; uint8_t qs[128]; };
struct BQ6K { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; };
struct BQ8K { float d; int8_t qs[256]; int16_t bsums[16]; };
#pragma pack(pop)

inline float h2f(uint16_t h) { return _cvtsh_ss(h); }
inline uint16_t f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }

inline int8_t sat_i8(float v) {
    if (!(v == v)) return 0;
    if (v <= -128.f) return -128;
    if (v >= 127.f) return 127;
    return (int8_t)v;
}

// k_quants.rs:586-615
void quantize_q8_0(const float *x, BQ8_0 *y, int64_t k) {
    for (int64_t i = 0; i < k / 32; i++) {
        float amax = 0.f;
        for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(x[i * 32 + j]));
        const float d = amax / 127.f;
        const float id = d != 0.f ? 1.f / d : 0.f;
        y[i].d = f2h(d);
        for (int j = 0; j < 32; j++) y[i].qs[j] = sat_i8(roundf(x[i * 32 + j] * id));
    }
}

// k_quants.rs:1788-1825
void quantize_q8k(const float *x, BQ8K *y, int64_t k) {
    for (int64_t i = 0; i < k / 256; i++) {
        const float *xb = x + i * 256;
        float max = 0.f, amax = 0.f;
        for (int j = 0; j < 256; j++)
            if (amax < fabsf(xb[j])) { amax = fabsf(xb[j]); max = xb[j]; }
        if (amax == 0.f) {
            memset(&y[i], 0, sizeof(BQ8K));
            continue;
        }
        const float iscale = -128.f / max;
        for (int j = 0; j < 256; j++) y[i].qs[j] = sat_i8(fminf(roundf(iscale * xb[j]), 127.f));
        for (int j = 0; j < 16; j++) {
            int s = 0;
            for (int t = 0; t < 16; t++) s += y[i].qs[16 * j + t];
            y[i].bsums[j] = (int16_t)s;
        }
        y[i].d = 1.f / iscale;
    }
}

inline float hsum8(__m256 x) {
    __m128 r = _mm_add_ps(_mm256_extractf128_ps(x, 1), _mm256_castps256_ps128(x));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_movehdup_ps(r));
    return _mm_cvtss_f32(r);
}

// signed i8 x signed i8 -> 8 x f32 partial sums
inline __m256 dot_i8_f32(__m256i x, __m256i y) {
    const __m256i ax = _mm256_sign_epi8(x, x);
    const __m256i sy = _mm256_sign_epi8(y, x);
    const __m256i p16 = _mm256_maddubs_epi16(ax, sy);
    return _mm256_cvtepi32_ps(_mm256_madd_epi16(_mm256_set1_epi16(1), p16));
}

float dot_q4_0(int64_t k, const BQ4_0 *x, const BQ8_0 *y) {
    __m256 acc = _mm256_setzero_ps();
    for (int64_t i = 0; i < k / 32; i++) {
        const __m256 d = _mm256_set1_ps(h2f(x[i].d) * h2f(y[i].d));
        const __m128i raw = _mm_loadu_si128((const __m128i *)x[i].qs);
        __m256i bx = _mm256_set_m128i(_mm_srli_epi16(raw, 4), raw);
        bx = _mm256_sub_epi8(_mm256_and_si256(bx, _mm256_set1_epi8(0xF)), _mm256_set1_epi8(8));
        const __m256i by = _mm256_loadu_si256((const __m256i *)y[i].qs);
        acc = _mm256_fmadd_ps(d, dot_i8_f32(bx, by), acc);
    }
    return hsum8(acc);
}

float dot_q8_0(int64_t k, const BQ8_0 *x, const BQ8_0 *y) {
    __m256 acc = _mm256_setzero_ps();
    for (int64_t i = 0; i < k / 32; i++) {
        const __m256 d = _mm256_set1_ps(h2f(x[i].d) * h2f(y[i].d));
        const __m256i bx = _mm256_loadu_si256((const __m256i *)x[i].qs);
        const __m256i by = _mm256_loadu_si256((const __m256i *)y[i].qs);
        acc = _mm256_fmadd_ps(d, dot_i8_f32(bx, by), acc);
    }
    return hsum8(acc);
}

// broadcast 16-bit scale j of `s16` (8 x i16 in the low half, repeated) to a whole vector pair pattern
inline __m256i bcast_scale16(__m128i s16, int j) {
    const __m128i idx = _mm_set1_epi16((short)((2 * j) | ((2 * j + 1) << 8)));
    const __m128i v = _mm_shuffle_epi8(s16, idx);
    return _mm256_set_m128i(v, v);
}

float dot_q4k(int64_t k, const BQ4K *x, const BQ8K *y) {
    const uint32_t m1 = 0x3f3f3f3f, m2 = 0x0f0f0f0f, m3 = 0x03030303;
    __m256 acc = _mm256_setzero_ps();
    __m128 acc_m = _mm_setzero_ps();
    for (int64_t i = 0; i < k / 256; i++) {
        const float d = y[i].d * h2f(x[i].d);
        const float dmin = -y[i].d * h2f(x[i].dmin);
        uint32_t u[4];
        memcpy(u, x[i].scales, 12);
        u[3] = ((u[2] >> 4) & m2) | (((u[1] >> 6) & m3) << 4);
        const uint32_t t = u[1] & m1;
        u[1] = (u[2] & m2) | (((u[0] >> 6) & m3) << 4);
        u[2] = t;
        u[0] &= m1;
        // u[0..1]: the eight 6-bit scales as bytes, u[2..3]: the eight mins
        const __m256i sm = _mm256_cvtepu8_epi16(_mm_set_epi32((int)u[3], (int)u[2], (int)u[1], (int)u[0]));
        const __m256i bs = _mm256_loadu_si256((const __m256i *)y[i].bsums);
        const __m128i bs2 = _mm_hadd_epi16(_mm256_extracti128_si256(bs, 0), _mm256_extracti128_si256(bs, 1));
        const __m128i pm = _mm_madd_epi16(_mm256_extracti128_si256(sm, 1), bs2);
        acc_m = _mm_fmadd_ps(_mm_set1_ps(dmin), _mm_cvtepi32_ps(pm), acc_m);
        const __m128i sc16 = _mm256_extracti128_si256(sm, 0);
        __m256i sumi = _mm256_setzero_si256();
        const uint8_t *q4 = x[i].qs;
        const int8_t *q8 = y[i].qs;
        for (int g = 0; g < 4; g++) {
            const __m256i bits = _mm256_loadu_si256((const __m256i *)(q4 + 32 * g));
            const __m256i lo = _mm256_and_si256(bits, _mm256_set1_epi8(0xF));
            const __m256i hi = _mm256_and_si256(_mm256_srli_epi16(bits, 4), _mm256_set1_epi8(0xF));
            const __m256i a0 = _mm256_loadu_si256((const __m256i *)(q8 + 64 * g));
            const __m256i a1 = _mm256_loadu_si256((const __m256i *)(q8 + 64 * g + 32));
            sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(bcast_scale16(sc16, 2 * g), _mm256_maddubs_epi16(lo, a0)));
            sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(bcast_scale16(sc16, 2 * g + 1), _mm256_maddubs_epi16(hi, a1)));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    acc_m = _mm_add_ps(acc_m, _mm_movehl_ps(acc_m, acc_m));
    acc_m = _mm_add_ss(acc_m, _mm_movehdup_ps(acc_m));
    return hsum8(acc) + _mm_cvtss_f32(acc_m);
}

// sign-extended 8-bit scale j broadcast over 8 x i16 lanes of both halves: lanes of the first
// 16 products take scale js, the next 16 take js + 1
inline __m256i q6_scales(const int8_t *sc, int js) {
    const __m128i a = _mm_set1_epi16((short)sc[js]);
    const __m128i b = _mm_set1_epi16((short)sc[js + 1]);
    return _mm256_set_m128i(b, a);
}

float dot_q6k(int64_t k, const BQ6K *x, const BQ8K *y) {
    const __m256i m4 = _mm256_set1_epi8(0xF), m2 = _mm256_set1_epi8(3), m32 = _mm256_set1_epi8(32);
    __m256 acc = _mm256_setzero_ps();
    for (int64_t i = 0; i < k / 256; i++) {
        const float d = y[i].d * h2f(x[i].d);
        __m256i sumi = _mm256_setzero_si256();
        for (int h = 0; h < 2; h++) {
            const __m256i l0 = _mm256_loadu_si256((const __m256i *)(x[i].ql + 64 * h));
            const __m256i l1 = _mm256_loadu_si256((const __m256i *)(x[i].ql + 64 * h + 32));
            const __m256i hb = _mm256_loadu_si256((const __m256i *)(x[i].qh + 32 * h));
            const __m256i q[4] = {
                _mm256_or_si256(_mm256_and_si256(l0, m4), _mm256_slli_epi16(_mm256_and_si256(hb, m2), 4)),
                _mm256_or_si256(_mm256_and_si256(l1, m4), _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(hb, 2), m2), 4)),
                _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(l0, 4), m4), _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(hb, 4), m2), 4)),
                _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(l1, 4), m4), _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(hb, 6), m2), 4)),
            };
            for (int t = 0; t < 4; t++) {
                const __m256i a = _mm256_loadu_si256((const __m256i *)(y[i].qs + 128 * h + 32 * t));
                // (q - 32) * a = q * a - 32 * a, both as unsigned x signed maddubs
                __m256i p = _mm256_sub_epi16(_mm256_maddubs_epi16(q[t], a), _mm256_maddubs_epi16(m32, a));
                sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(q6_scales(x[i].scales, 8 * h + 2 * t), p));
            }
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum8(acc);
}

template <typename W, typename A, float (*DOT)(int64_t, const W *, const A *), void (*QUANT)(const float *, A *, int64_t)>
void matmul_t(int64_t m, int64_t k, int64_t n, const float *lhs, const void *rhs, float *dst, int64_t wblk,
              int64_t ablk) {
    const int64_t kb_w = k / wblk, kb_a = k / ablk;
    std::vector<A> acts((size_t)(m * kb_a));
    for (int64_t r = 0; r < m; r++) QUANT(lhs + r * k, acts.data() + r * kb_a, k);  // serial, as the reference
    const W *w = (const W *)rhs;
    for (int64_t r = 0; r < m; r++) {
        const A *a = acts.data() + r * kb_a;
        float *out = dst + r * n;
#pragma omp parallel for schedule(dynamic, 256)
        for (int64_t c = 0; c < n; c++) out[c] = DOT(k, w + c * kb_w, a);
    }
}

}  // namespace

extern "C" int cpub_num_threads(void) { return omp_get_max_threads(); }
extern "C" void cpub_set_num_threads(int n) { omp_set_num_threads(n); }

// dst[m, n] = lhs[m, k] . rhs_t[n, k]^T ; dtype ids as GgmlDType::to_u32
extern "C" int cpub_matmul(int dtype, int64_t m, int64_t k, int64_t n, const float *lhs, const void *rhs_t,
                           float *dst) {
    switch (dtype) {
    case 2:
        if (k % 32) return -1;
        matmul_t<BQ4_0, BQ8_0, dot_q4_0, quantize_q8_0>(m, k, n, lhs, rhs_t, dst, 32, 32);
        return 0;
    case 8:
        if (k % 32) return -1;
        matmul_t<BQ8_0, BQ8_0, dot_q8_0, quantize_q8_0>(m, k, n, lhs, rhs_t, dst, 32, 32);
        return 0;
    case 12:
        if (k % 256) return -1;
        matmul_t<BQ4K, BQ8K, dot_q4k, quantize_q8k>(m, k, n, lhs, rhs_t, dst, 256, 256);
        return 0;
    case 14:
        if (k % 256) return -1;
        matmul_t<BQ6K, BQ8K, dot_q6k, quantize_q8k>(m, k, n, lhs, rhs_t, dst, 256, 256);
        return 0;
    default:
        return -2;
    }
}
