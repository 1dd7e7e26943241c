// Weight quantizers on the device: f32 -> GGML blocks (array-of-blocks bytes), the
// arithmetic of T::from_float in candle-core/src/quantized/k_quants.rs and utils.rs,
// one thread per block, every f32 operation a single IEEE operation in the reference's
// order (compiled with -ffp-contract=off).  The reference's CUDA arm copies the tensor to
// the host and quantizes there (cuda.rs:448-472); the bytes produced here are the same.
//   Q4_0 k_quants.rs:185-220      Q8_0 :586-615
//   Q4K  :1252-1311 + utils.rs:201-258 (make_qkx1_quants) + :49-59 (get_scale_min_k4)
//   Q5K  :1450-1525, the same with 32 levels
//   Q6K  :1643-1713 + utils.rs:61-198  (make_qx_quants, n=16, nmax=32, rmse_type=1)
//   Q2K  :770-839 (make_qkx1_quants over 16 elements, 3 levels)
//   Q4_1 :296-326   Q5_1 :496-530   Q5_0 :393-425   Q3K  :1011-1090 + utils.rs:261-326 (make_q3_quants, nmax=4, do_rmse)
#include "qhip_internal.h"

namespace {

__device__ void store_u16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)(v & 0xff); p[1] = (uint8_t)(v >> 8); }

__global__ void quantize_q4_0(const float *__restrict__ src, int64_t nblocks, uint8_t *__restrict__ out) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *x = src + b * 32;
    float amax = 0.0f, max = 0.0f;
    for (int j = 0; j < 32; j++) {
        const float v = x[j];
        if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
    }
    const float d = max / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t *y = out + b * 18;
    store_u16(y, cq_f2h(d));
    for (int j = 0; j < 16; j++) {
        const float x0 = x[j] * id;
        const float x1 = x[16 + j] * id;
        uint8_t xi0 = cq_as_u8(x0 + 8.5f);
        uint8_t xi1 = cq_as_u8(x1 + 8.5f);
        if (xi0 > 15) xi0 = 15;
        if (xi1 > 15) xi1 = 15;
        y[2 + j] = (uint8_t)(xi0 | (xi1 << 4));
    }
}

__global__ void quantize_q8_0(const float *__restrict__ src, int64_t nblocks, uint8_t *__restrict__ out) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *x = src + b * 32;
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(x[j]));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t *y = out + b * 34;
    store_u16(y, cq_f2h(d));
    for (int j = 0; j < 32; j++) y[2 + j] = (uint8_t)cq_as_i8(roundf(x[j] * id));
}

// utils.rs:201-258
template <int N = 32>
__device__ void make_qkx1_quants(const float *x, int nmax, float &out_scale, float &out_min) {
    const int n = N, ntry = 5;
    uint8_t l[N];
    for (int i = 0; i < n; i++) l[i] = 0;
    float min = x[0], max = x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
    }
    if (max == min) { out_scale = 0.0f; out_min = 0.0f; return; }
    min = fminf(min, 0.0f);
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    for (int t = 0; t < ntry; t++) {
        float sumlx = 0.0f;
        int32_t suml2 = 0;
        bool did_change = false;
        for (int i = 0; i < n; i++) {
            const int32_t li = cq_clampi(cq_nearest_int(iscale * (x[i] - min)), 0, nmax);
            if ((uint8_t)li != l[i]) { l[i] = (uint8_t)li; did_change = true; }
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
    out_scale = scale;
    out_min = -min;
}

// LEVELS = 16: Q4K (144-byte blocks).  LEVELS = 32: Q5K (k_quants.rs:1450-1525), the same scale search
// with 31 as the top level, the quants' fifth bits in qh[32] between the scales and the nibbles.
template <int LEVELS>
__global__ void quantize_q4k(const float *__restrict__ src, int64_t nblocks, uint8_t *__restrict__ out) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *x = src + b * QK_K;
    constexpr int kQs = LEVELS == 16 ? 16 : 48;   // offset of the nibbles in the block
    uint8_t *y = out + b * (LEVELS == 16 ? 144 : 176);
    uint8_t qh[32];
    for (int l = 0; l < 32; l++) qh[l] = 0;
    float mins[8], scales[8];
    for (int j = 0; j < 8; j++) make_qkx1_quants(x + 32 * j, LEVELS - 1, scales[j], mins[j]);
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 8; j++) max_scale = fmaxf(scales[j], max_scale);
    for (int j = 0; j < 8; j++) max_min = fmaxf(mins[j], max_min);
    const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    uint8_t sc12[12];
    for (int j = 0; j < 12; j++) sc12[j] = 0;
    for (int j = 0; j < 8; j++) {
        int32_t lsi = cq_nearest_int(inv_scale * scales[j]);
        int32_t lmi = cq_nearest_int(inv_min * mins[j]);
        if (lsi > 63) lsi = 63;
        if (lmi > 63) lmi = 63;
        const uint8_t ls = (uint8_t)lsi, lm = (uint8_t)lmi;
        if (j < 4) {
            sc12[j] = ls;
            sc12[j + 4] = lm;
        } else {
            sc12[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            sc12[j - 4] |= (uint8_t)((ls >> 4) << 6);
            sc12[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    const uint16_t dh = cq_f2h(max_scale / 63.0f);
    const uint16_t dminh = cq_f2h(max_min / 63.0f);
    store_u16(y, dh);
    store_u16(y + 2, dminh);
    for (int j = 0; j < 12; j++) y[4 + j] = sc12[j];
    const uint32_t u0 = sc12[0] | (sc12[1] << 8) | (sc12[2] << 16) | ((uint32_t)sc12[3] << 24);
    const uint32_t u1 = sc12[4] | (sc12[5] << 8) | (sc12[6] << 16) | ((uint32_t)sc12[7] << 24);
    const uint32_t u2 = sc12[8] | (sc12[9] << 8) | (sc12[10] << 16) | ((uint32_t)sc12[11] << 24);
    // two 32-element sub-blocks share the 32 output bytes of their 64-element group
    for (int g = 0; g < 4; g++) {
        uint8_t lo[32], hi[32];
        for (int half = 0; half < 2; half++) {
            const int j = 2 * g + half;
            int sc, m;
            cq_scale_min_k4(j, u0, u1, u2, sc, m);
            const float d = cq_h2f(dh) * (float)sc;
            uint8_t *dst = half ? hi : lo;
            if (d != 0.0f) {
                const float dm = cq_h2f(dminh) * (float)m;
                for (int ii = 0; ii < 32; ii++)
                    dst[ii] = (uint8_t)cq_clampi(cq_nearest_int((x[32 * j + ii] + dm) / d), 0, LEVELS - 1);
            } else {
                for (int ii = 0; ii < 32; ii++) dst[ii] = 0;
            }
        }
        for (int l = 0; l < 32; l++) {
            if (LEVELS == 32) qh[l] |= (uint8_t)(((lo[l] >> 4) << (2 * g)) | ((hi[l] >> 4) << (2 * g + 1)));
            y[kQs + 32 * g + l] = (uint8_t)((lo[l] & 15) | ((hi[l] & 15) << 4));
        }
    }
    if (LEVELS == 32)
        for (int l = 0; l < 32; l++) y[16 + l] = qh[l];
}

// utils.rs:61-198 specialised to n = 16, nmax = 32, rmse_type = 1 (weights w = x*x; returns after
// the five refinement passes, utils.rs:168-170).
__device__ float make_qx_quants_16_32(const float *x, int8_t *ls) {
    const int n = 16, nmax = 32;
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        const float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.0f) {
        for (int i = 0; i < n; i++) ls[i] = 0;
        return 0.0f;
    }
    const float iscale = -(float)nmax / max;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        const int32_t l = cq_clampi(cq_nearest_int(iscale * x[i]), -nmax, nmax - 1);
        ls[i] = (int8_t)(l + nmax);
        const float w = x[i] * x[i];
        const float lf = (float)l;
        sumlx += w * x[i] * lf;
        suml2 += w * lf * lf;
    }
    float scale = sumlx / suml2;
    float best = scale * sumlx;
    for (int itry = 0; itry < 3; itry++) {
        const float is2 = 1.0f / scale;
        float slx = 0.0f, sl2 = 0.0f;
        bool changed = false;
        for (int i = 0; i < n; i++) {
            const int32_t l = cq_clampi(cq_nearest_int(is2 * x[i]), -nmax, nmax - 1);
            if (l + nmax != (int32_t)ls[i]) changed = true;
            const float w = x[i] * x[i];
            const float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;
        for (int i = 0; i < n; i++) {
            const int32_t l = cq_nearest_int(is2 * x[i]);
            ls[i] = (int8_t)(nmax + cq_clampi(l, -nmax, nmax - 1));
        }
        sumlx = slx;
        suml2 = sl2;
        scale = sumlx / suml2;
        best = scale * sumlx;
    }
    for (int itry = 0; itry < 5; itry++) {
        int n_changed = 0;
        for (int i = 0; i < n; i++) {
            const float w = x[i] * x[i];
            const int32_t l = (int32_t)ls[i] - nmax;
            float slx = sumlx - w * x[i] * (float)l;
            if (slx > 0.0f) {
                float sl2 = suml2 - w * (float)l * (float)l;
                const int32_t new_l = cq_clampi(cq_nearest_int(x[i] * sl2 / slx), -nmax, nmax - 1);
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
    (void)best;
    return scale;
}

__global__ void quantize_q6k(const float *__restrict__ src, int64_t nblocks, uint8_t *__restrict__ out) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *x = src + b * QK_K;
    uint8_t *y = out + b * 210;
    int8_t l[QK_K];
    float scales[16];
    float max_scale = 0.0f, max_abs_scale = 0.0f;
    for (int j = 0; j < 16; j++) {
        const float scale = make_qx_quants_16_32(x + 16 * j, l + 16 * j);
        scales[j] = scale;
        const float a = fabsf(scale);
        if (a > max_abs_scale) { max_abs_scale = a; max_scale = scale; }
    }
    const float iscale = -128.0f / max_scale;
    const uint16_t dh = cq_f2h(1.0f / iscale);
    int8_t sc8[16];
    for (int j = 0; j < 16; j++) {
        int32_t v = cq_nearest_int(iscale * scales[j]);
        if (v > 127) v = 127;
        sc8[j] = (int8_t)v;
    }
    for (int j = 0; j < 16; j++) {
        const float d = cq_h2f(dh) * (float)sc8[j];
        if (d == 0.0f) continue;
        for (int ii = 0; ii < 16; ii++) {
            const int32_t ll = cq_clampi(cq_nearest_int(x[16 * j + ii] / d), -32, 31);
            l[16 * j + ii] = (int8_t)(ll + 32);
        }
    }
    for (int h = 0; h < 2; h++) {
        const int j = 128 * h;
        for (int li = 0; li < 32; li++) {
            const int8_t q1 = l[j + li] & 0xF, q2 = l[j + li + 32] & 0xF, q3 = l[j + li + 64] & 0xF,
                         q4 = l[j + li + 96] & 0xF;
            y[64 * h + li] = (uint8_t)(q1 | (q3 << 4));
            y[64 * h + li + 32] = (uint8_t)(q2 | (q4 << 4));
            y[128 + 32 * h + li] = (uint8_t)((l[j + li] >> 4) | ((l[j + li + 32] >> 4) << 2) |
                                             ((l[j + li + 64] >> 4) << 4) | ((l[j + li + 96] >> 4) << 6));
        }
    }
    for (int j = 0; j < 16; j++) y[192 + j] = (uint8_t)sc8[j];
    store_u16(y + 208, dh);
}

__global__ void quantize_q5_0(const float *__restrict__ src, int64_t nblocks, uint8_t *__restrict__ out) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *x = src + b * 32;
    float amax = 0.0f, max = 0.0f;
    for (int j = 0; j < 32; j++) {
        const float v = x[j];
        if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
    }
    const float d = max / -16.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t *y = out + b * 22;
    store_u16(y, cq_f2h(d));
    uint32_t qh = 0;
    for (int j = 0; j < 16; j++) {
        const float x0 = x[j] * id, x1 = x[j + 16] * id;
        const int8_t s0 = cq_as_i8(x0 + 16.5f), s1 = cq_as_i8(x1 + 16.5f);
        const uint8_t xi0 = (uint8_t)(s0 < 31 ? s0 : 31), xi1 = (uint8_t)(s1 < 31 ? s1 : 31);
        y[6 + j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
        qh |= (((uint32_t)xi0 & 0x10u) >> 4) << j;
        qh |= (((uint32_t)xi1 & 0x10u) >> 4) << (j + 16);
    }
    y[2] = (uint8_t)qh; y[3] = (uint8_t)(qh >> 8); y[4] = (uint8_t)(qh >> 16); y[5] = (uint8_t)(qh >> 24);
}

// Q2K (k_quants.rs:770-839): sixteen groups of sixteen, make_qkx1_quants with three levels, 4-bit scales and minima
__global__ void quantize_q2k(const float *__restrict__ src, int64_t nblocks, uint8_t *__restrict__ out) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *x = src + b * 256;
    uint8_t *y = out + b * 84;
    uint8_t *sc = y, *qs = y + 16;
    const float Q4SCALE = 15.0f;
    float mins[16], scales[16];
    for (int j = 0; j < 16; j++) make_qkx1_quants<16>(x + 16 * j, 3, scales[j], mins[j]);
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 16; j++) {
        max_scale = fmaxf(scales[j], max_scale);
        max_min = fmaxf(mins[j], max_min);
    }
    uint16_t dh = cq_f2h(0.0f), dmh = cq_f2h(0.0f);
    if (max_scale > 0.0f) {
        const float iscale = Q4SCALE / max_scale;
        for (int j = 0; j < 16; j++) sc[j] = (uint8_t)cq_nearest_int(iscale * scales[j]);
        dh = cq_f2h(max_scale / Q4SCALE);
    } else {
        for (int j = 0; j < 16; j++) sc[j] = 0;
    }
    if (max_min > 0.0f) {
        const float iscale = Q4SCALE / max_min;
        for (int j = 0; j < 16; j++) sc[j] |= (uint8_t)((uint8_t)cq_nearest_int(iscale * mins[j]) << 4);
        dmh = cq_f2h(max_min / Q4SCALE);
    }
    store_u16(y + 80, dh);
    store_u16(y + 82, dmh);
    for (int i = 0; i < 64; i++) qs[i] = 0;
    const float dall = cq_h2f(dh), dmin = cq_h2f(dmh);
    for (int j = 0; j < 16; j++) {
        const float d = dall * (float)(sc[j] & 0xF);
        if (d == 0.0f) continue;
        const float dm = dmin * (float)(sc[j] >> 4);
        for (int ii = 0; ii < 16; ii++) {
            const int e = 16 * j + ii;
            const int ll = cq_clampi(cq_nearest_int((x[e] + dm) / d), 0, 3);
            qs[32 * (e / 128) + e % 32] |= (uint8_t)(ll << (2 * ((e % 128) / 32)));
        }
    }
}

// Q4_1 (k_quants.rs:296-326) and, FIVE, Q5_1 (:496-530): d = (max - min) / levels, quants round((x - min) / d)
template <bool FIVE>
__global__ void quantize_q4_1(const float *__restrict__ src, int64_t nblocks, uint8_t *__restrict__ out) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *x = src + b * 32;
    float min = INFINITY, max = -INFINITY;
    for (int j = 0; j < 32; j++) {
        min = fminf(x[j], min);   // f32::min / f32::max: a NaN operand loses
        max = fmaxf(x[j], max);
    }
    const float d = (max - min) / (FIVE ? 31.0f : 15.0f);
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t *y = out + b * (FIVE ? 24 : 20);
    store_u16(y, cq_f2h(d));
    store_u16(y + 2, cq_f2h(min));
    uint32_t qh = 0;
    for (int j = 0; j < 16; j++) {
        const float x0 = (x[j] - min) * id;
        const float x1 = (x[16 + j] - min) * id;
        uint8_t xi0 = cq_as_u8(x0 + 0.5f), xi1 = cq_as_u8(x1 + 0.5f);
        if (!FIVE) {
            if (xi0 > 15) xi0 = 15;
            if (xi1 > 15) xi1 = 15;
        }
        y[(FIVE ? 8 : 4) + j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
        qh |= (((uint32_t)xi0 & 0x10u) >> 4) << j;
        qh |= (((uint32_t)xi1 & 0x10u) >> 4) << (j + 16);
    }
    if (FIVE) { y[4] = (uint8_t)qh; y[5] = (uint8_t)(qh >> 8); y[6] = (uint8_t)(qh >> 16); y[7] = (uint8_t)(qh >> 24); }
}

// utils.rs:261-326 with nmax = 4, do_rmse = true, n = 16: only the returned scale is used
__device__ float make_q3_quants_16(const float *x) {
    const int n = 16, nmax = 4;
    int8_t l[16];
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        const float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.0f) return 0.0f;
    const float iscale = -(float)nmax / max;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int li = cq_nearest_int(iscale * x[i]);
        li = li < -nmax ? -nmax : (li > nmax - 1 ? nmax - 1 : li);
        l[i] = (int8_t)li;
        const float w = x[i] * x[i];
        sumlx += w * x[i] * (float)li;
        suml2 += w * (float)(li * li);
    }
    for (int t = 0; t < 5; t++) {
        int n_changed = 0;
        for (int i = 0; i < n; i++) {
            const float w = x[i] * x[i];
            float slx = sumlx - w * x[i] * (float)l[i];
            if (slx > 0.0f) {
                float sl2 = suml2 - w * (float)((int)l[i] * (int)l[i]);
                int new_l = cq_nearest_int(x[i] * sl2 / slx);
                new_l = new_l < -nmax ? -nmax : (new_l > nmax - 1 ? nmax - 1 : new_l);
                if (new_l != (int)l[i]) {
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

__global__ void quantize_q3k(const float *__restrict__ src, int64_t nblocks, uint8_t *__restrict__ out) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float *x = src + b * 256;
    uint8_t *y = out + b * 110;
    uint8_t *hmask = y, *qs = y + 32, *sc = y + 96;
    float scales[16];
    for (int j = 0; j < 16; j++) scales[j] = make_q3_quants_16(x + 16 * j);
    float max_scale = 0.0f;
    for (int j = 0; j < 16; j++)
        if (fabsf(scales[j]) > fabsf(max_scale)) max_scale = scales[j];
    for (int i = 0; i < 108; i++) y[i] = 0;
    uint16_t dh = cq_f2h(0.0f);
    if (max_scale != 0.0f) {
        const float iscale = -32.0f / max_scale;
        for (int j = 0; j < 16; j++) {
            int lv = cq_nearest_int(iscale * scales[j]);
            lv = (lv < -32 ? -32 : (lv > 31 ? 31 : lv)) + 32;
            if (j < 8) sc[j] = (uint8_t)(lv & 0xF);
            else sc[j - 8] |= (uint8_t)((lv & 0xF) << 4);
            lv >>= 4;
            sc[j % 4 + 8] |= (uint8_t)(lv << (2 * (j / 4)));
        }
        dh = cq_f2h(1.0f / iscale);
    }
    store_u16(y + 108, dh);
    const float dall = cq_h2f(dh);
    // element e: two low bits into qs[32 * (e / 128) + e % 32] at 2 * ((e % 128) / 32), the third into hmask[e % 32] bit e / 32
    for (int j = 0; j < 16; j++) {
        const int low = j < 8 ? (sc[j] & 0xF) : (sc[j - 8] >> 4);
        const int s6 = (low | (((sc[8 + j % 4] >> (2 * (j / 4))) & 3) << 4)) - 32;
        const float d = dall * (float)s6;
        for (int ii = 0; ii < 16; ii++) {
            const int e = 16 * j + ii;
            int lv = 0;
            if (d != 0.0f) {
                lv = cq_nearest_int(x[e] / d);
                lv = (lv < -4 ? -4 : (lv > 3 ? 3 : lv)) + 4;
            }
            if (lv > 3) { hmask[e % 32] |= (uint8_t)(1u << (e / 32)); lv -= 4; }
            qs[32 * (e / 128) + e % 32] |= (uint8_t)(lv << (2 * ((e % 128) / 32)));
        }
    }
}

}  // namespace

hipError_t cq_launch_quantize_weight(int dtype, const float *src, int64_t nblocks, uint8_t *aos_dev, hipStream_t s) {
    if (nblocks == 0) return hipSuccess;
    const int threads = 64;
    const unsigned grid = (unsigned)((nblocks + threads - 1) / threads);
    switch (dtype) {
    case CQ_DTYPE_Q4_0: quantize_q4_0<<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    case CQ_DTYPE_Q8_0: quantize_q8_0<<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    case CQ_DTYPE_Q5_0: quantize_q5_0<<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    case CQ_DTYPE_Q4_1: quantize_q4_1<false><<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    case CQ_DTYPE_Q5_1: quantize_q4_1<true><<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    case CQ_DTYPE_Q3K: quantize_q3k<<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    case CQ_DTYPE_Q2K: quantize_q2k<<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    // Q8K (k_quants.rs:1788-1825): the activation quantizer writing GGML blocks, one 256-element row per block
    case CQ_DTYPE_Q8K: return cq_launch_quantize_act_aos(CQ_DTYPE_Q8K, src, nblocks, 256, cq_no_pre(), aos_dev, s);
    case CQ_DTYPE_Q4K: quantize_q4k<16><<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    case CQ_DTYPE_Q5K: quantize_q4k<32><<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    case CQ_DTYPE_Q6K: quantize_q6k<<<grid, threads, 0, s>>>(src, nblocks, aos_dev); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
