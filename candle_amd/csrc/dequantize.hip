// Device planes -> f32 / f16 (QTensor::dequantize, dequantize_f16;
// candle-core/src/quantized/mod.rs:361-382, CUDA precedent cuda.rs:69-181).
// The f32 values are those of T::to_float (k_quants.rs:163-183, :329-349, :533-558, :568-584, :841-872, :1094-1146, :1313-1341,
// :1527-1564, :1716-1746): same products in the same order, no contraction.  The f16 output is the
// f32 output rounded to nearest-even, as the reference's tests require
// (candle-core/tests/quantized_tests.rs:229-234).
// One thread per 16-byte lane of the main plane; a wave covers 1 KiB of it.
#include "qhip_internal.h"

namespace {

// Sixteen consecutive results starting at element i (a multiple of 16): 64 or 32 bytes in
// 16-byte stores.
template <bool F16>
__device__ __forceinline__ void put16(float *d32, uint16_t *d16, int64_t i, const float (&v)[16]) {
    if (F16) {
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; j++) w[j] = (uint32_t)cq_f2h(v[2 * j]) | ((uint32_t)cq_f2h(v[2 * j + 1]) << 16);
        uint4 *dst = (uint4 *)(d16 + i);
        dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
        dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
    } else {
        float4 *dst = (float4 *)(d32 + i);
#pragma unroll
        for (int j = 0; j < 4; j++) dst[j] = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
    }
}

template <bool F16>
__global__ void dequant_q4_0(const uint8_t *__restrict__ qs, const uint16_t *__restrict__ dpl, int64_t nblocks,
                             float *d32, uint16_t *d16) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const uint4 q = *(const uint4 *)(qs + b * 16);
    const float d = cq_h2f(dpl[b]);
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    float lo[16], hi[16];
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const uint32_t byte = (w[j >> 2] >> (8 * (j & 3))) & 0xff;
        const int x0 = (int)(byte & 0xF) - 8, x1 = (int)(byte >> 4) - 8;
        lo[j] = (float)x0 * d;
        hi[j] = (float)x1 * d;
    }
    put16<F16>(d32, d16, b * 32, lo);
    put16<F16>(d32, d16, b * 32 + 16, hi);
}

// MIN: Q4_1 / Q5_1 held as Q8_0 planes plus the plane of block minima: q * d + m (k_quants.rs:329-349, :533-558)
template <bool F16, bool MIN>
__global__ void dequant_q8_0(const uint8_t *__restrict__ qs, const uint16_t *__restrict__ dpl,
                             const uint16_t *__restrict__ mpl, int64_t nunits, float *d32, uint16_t *d16) {
    const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // 16 elements each
    if (u >= nunits) return;
    const uint4 q = *(const uint4 *)(qs + u * 16);
    const float d = cq_h2f(dpl[u >> 1]);
    const float mn = MIN ? cq_h2f(mpl[u >> 1]) : 0.0f;
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    float out[16];
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const int8_t v = (int8_t)((w[j >> 2] >> (8 * (j & 3))) & 0xff);
        out[j] = (float)v * d;
        if (MIN) out[j] = out[j] + mn;
    }
    put16<F16>(d32, d16, u * 16, out);
}

// Q5 (Q5K, to_float k_quants.rs:1527-1564): the fifth bits come from the re-ordered qh plane, words
// {L, H} per 32 qs bytes, bit 8c + i for byte c of qs word i.
template <bool F16, bool Q5>
__global__ void dequant_q4k(const uint8_t *__restrict__ qs, const uint8_t *__restrict__ hd,
                            const uint8_t *__restrict__ qh, int64_t nunits, float *d32, uint16_t *d16) {
    const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // 16 bytes of qs = 32 elements
    if (u >= nunits) return;
    const int64_t b = u >> 3;
    const int p = (int)(u & 7), g = p >> 1, half = p & 1;
    const uint4 q = *(const uint4 *)(qs + u * 16);
    const uint32_t *h = (const uint32_t *)(hd + b * CQ_Q4K_HDR);
    const uint32_t dd = h[0], rec = h[1 + g];
    const float d = cq_h2f((uint16_t)(dd & 0xffff)), dmin = cq_h2f((uint16_t)(dd >> 16));
    const int sc1 = (int)(rec & 0xff), sc2 = (int)((rec >> 8) & 0xff);
    const int m1 = (int)((rec >> 16) & 0xff), m2 = (int)(rec >> 24);
    const float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
    const float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    const int64_t base = b * 256 + 64 * g + 16 * half;
    uint2 fifth = make_uint2(0u, 0u);
    if (Q5) fifth = *(const uint2 *)(qh + (b * 4 + g) * 8);
    float lo[16], hi[16];
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const uint32_t byte = (w[j >> 2] >> (8 * (j & 3))) & 0xff;
        const int bit = 8 * (j & 3) + 4 * half + (j >> 2);
        lo[j] = d1 * (float)((byte & 0xF) + (((fifth.x >> bit) & 1u) << 4)) - mm1;
        hi[j] = d2 * (float)((byte >> 4) + (((fifth.y >> bit) & 1u) << 4)) - mm2;
    }
    put16<F16>(d32, d16, base, lo);
    put16<F16>(d32, d16, base + 32, hi);
}

// MIN: Q2K held as Q6K planes plus the groups' minima and dmin: (d * sc) * q - dmin * m (k_quants.rs:841-872)
template <bool F16, bool MIN>
__global__ void dequant_q6k(const uint8_t *__restrict__ ql, const uint8_t *__restrict__ qh,
                            const int8_t *__restrict__ sc, const uint16_t *__restrict__ dpl,
                            const uint8_t *__restrict__ mins, const uint16_t *__restrict__ dmins, int64_t nunits,
                            float *d32, uint16_t *d16) {
    const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // 16 bytes of ql = 32 elements
    if (u >= nunits) return;
    const int64_t b = u >> 3;
    const int p = (int)(u & 7), h = p >> 2, t = (p >> 1) & 1, i0 = (p & 1) * 16;
    const uint4 q = *(const uint4 *)(ql + u * 16);
    const uint2 hh = *(const uint2 *)(qh + u * 8);
    const float d = cq_h2f(dpl[b]);
    // low nibbles: elements 128h + 32t + i0 + e, one 16-element scale group; high nibbles: +64
    const float s_lo = (float)sc[u * 2], s_hi = (float)sc[u * 2 + 1];  // re-packed: the lane's two scales
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    const uint32_t hw[2] = {hh.x, hh.y};
    const int64_t base = b * 256 + 128 * h + 32 * t + i0;
    float lo[16], hi[16];
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const int wi = e >> 2, c = e & 3;
        const uint32_t byte = (w[wi] >> (8 * c)) & 0xff;
        const uint32_t hb = (hw[wi >> 1] >> (8 * c)) & 0xff;
        const int sh = (wi & 1) * 4;
        const int q_lo = (int)((byte & 0xF) | (((hb >> sh) & 3) << 4)) - 32;
        const int q_hi = (int)((byte >> 4) | (((hb >> (sh + 2)) & 3) << 4)) - 32;
        lo[e] = d * s_lo * (float)q_lo;
        hi[e] = d * s_hi * (float)q_hi;
    }
    if (MIN) {
        // the lane's low-nibble elements are group 8h + 2t + p%2 of the block, the high-nibble ones four groups on
        const int j = 8 * h + 2 * t + (p & 1);
        const float dmin = cq_h2f(dmins[b]);
        const float ml_lo = dmin * (float)mins[b * 16 + j], ml_hi = dmin * (float)mins[b * 16 + j + 4];
#pragma unroll
        for (int e = 0; e < 16; e++) {
            lo[e] = lo[e] - ml_lo;
            hi[e] = hi[e] - ml_hi;
        }
    }
    put16<F16>(d32, d16, base, lo);
    put16<F16>(d32, d16, base + 64, hi);
}

template <bool F16>
hipError_t launch(const cq_weight *w, float *d32, uint16_t *d16, hipStream_t s) {
    const int threads = 256;
    const int64_t total = w->n * w->k;
    if (total == 0) return hipSuccess;
    auto grid = [&](int64_t n) { return (unsigned)((n + threads - 1) / threads); };
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0:
        dequant_q4_0<F16><<<grid(total / 32), threads, 0, s>>>(w->p0, (const uint16_t *)w->p1, total / 32, d32, d16);
        break;
    case CQ_DTYPE_Q8_0:
        if (cq_has_min32(w->ggml_dtype))
            dequant_q8_0<F16, true><<<grid(total / 16), threads, 0, s>>>(w->p0, (const uint16_t *)w->p1, (const uint16_t *)w->p2,
                                                                         total / 16, d32, d16);
        else
            dequant_q8_0<F16, false><<<grid(total / 16), threads, 0, s>>>(w->p0, (const uint16_t *)w->p1, nullptr, total / 16, d32, d16);
        break;
    case CQ_DTYPE_Q4K:
        dequant_q4k<F16, false><<<grid(total / 32), threads, 0, s>>>(w->p0, w->p1, nullptr, total / 32, d32, d16);
        break;
    case CQ_DTYPE_Q5K:
        dequant_q4k<F16, true><<<grid(total / 32), threads, 0, s>>>(w->p0, w->p1, w->p2, total / 32, d32, d16);
        break;
    case CQ_DTYPE_Q6K:
        if (cq_has_min16(w->ggml_dtype))
            dequant_q6k<F16, true><<<grid(total / 32), threads, 0, s>>>(w->p0, w->p1, (const int8_t *)w->p2, (const uint16_t *)w->p3,
                                                                        w->p4, (const uint16_t *)w->p5, total / 32, d32, d16);
        else
            dequant_q6k<F16, false><<<grid(total / 32), threads, 0, s>>>(w->p0, w->p1, (const int8_t *)w->p2, (const uint16_t *)w->p3,
                                                                         nullptr, nullptr, total / 32, d32, d16);
        break;
    case CQ_DTYPE_Q8K: return cq_launch_dequantize_q8k(w, d32, d16, s);
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

hipError_t cq_launch_dequantize(const cq_weight *w, float *dst32, uint16_t *dst16, hipStream_t s) {
    return dst16 ? launch<true>(w, nullptr, dst16, s) : launch<false>(w, dst32, nullptr, s);
}
