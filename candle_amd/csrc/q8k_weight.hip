// Q8K as a weight type (BlockQ8K as GgmlType, candle-core/src/quantized/k_quants.rs:1749-1839): blocks
// {f32 d; i8 qs[256]; i16 bsums[16]}, contracted with Q8K activations block by block,
//   sumf += (float)(sum_256 qw * qa) * dw * d8                                   (vec_dot_unopt, :1768-1786)
// No checkpoint stores weights in this type; the reference offers it (QTensor::quantize, QMatMul) and tests it
// (candle-core/tests/quantized_tests.rs:672-717, :1124-1150), so the boundary takes it too, through one plain
// dot-product kernel for every row count.  Planes: qs [blocks][256] i8, d [blocks] f32, bsums [blocks][16] i16 (kept for
// the way back to GGML bytes only: the dot product does not use them).
#include "qhip_internal.h"

namespace {

__global__ void repack_q8k(uint8_t *__restrict__ aos, uint8_t *__restrict__ qs, float *__restrict__ d, int16_t *__restrict__ bsums,
                           int64_t nblocks, bool inverse) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // one thread per 16 bytes of qs
    const int64_t b = t >> 4;
    const int p = (int)(t & 15);
    if (b >= nblocks) return;
    uint8_t *blk = aos + b * 292;   // 292 = 4 * 73: words are aligned, 16-byte vectors are not
    uint32_t *aq = (uint32_t *)(blk + 4 + p * 16), *pq = (uint32_t *)(qs + b * 256 + p * 16);
    if (!inverse) {
        for (int i = 0; i < 4; i++) pq[i] = aq[i];
        if (p == 0) d[b] = *(const float *)blk;
        bsums[b * 16 + p] = *(const int16_t *)(blk + 260 + 2 * p);
    } else {
        for (int i = 0; i < 4; i++) aq[i] = pq[i];
        if (p == 0) *(float *)blk = d[b];
        *(int16_t *)(blk + 260 + 2 * p) = bsums[b * 16 + p];
    }
}

// k_quants.rs:1827-1838: y = d * q
template <bool F16>
__global__ void dequant_q8k(const uint8_t *__restrict__ qs, const float *__restrict__ dpl, int64_t npieces, float *d32, uint16_t *d16) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // 16 elements each
    if (t >= npieces) return;
    const uint4 q = *(const uint4 *)(qs + t * 16);
    const float d = dpl[t >> 4];
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    for (int j = 0; j < 16; j += 4) {
        float v[4];
#pragma unroll
        for (int c = 0; c < 4; c++) v[c] = d * (float)(int8_t)((w[j >> 2] >> (8 * c)) & 0xff);
        if (F16) {
            uint2 h;
            h.x = (uint32_t)cq_f2h(v[0]) | ((uint32_t)cq_f2h(v[1]) << 16);
            h.y = (uint32_t)cq_f2h(v[2]) | ((uint32_t)cq_f2h(v[3]) << 16);
            *(uint2 *)(d16 + t * 16 + j) = h;
        } else {
            *(float4 *)(d32 + t * 16 + j) = make_float4(v[0], v[1], v[2], v[3]);
        }
    }
}

// One wave per weight row, lanes over the 16-byte pieces of the row (sixteen consecutive lanes = one block); per
// activation row the block integers are summed over those sixteen lanes, scaled like the reference and added up per
// lane group, then over the wave.  A row's result does not depend on the rows beside it.
__global__ void __launch_bounds__(256) q8k_weight_kernel(cq_weight w, cq_act_view a, int64_t m, float *__restrict__ y) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= w.n) return;
    const int64_t k = w.k, kb = k >> 8, pieces = k >> 4;
    const uint8_t *wq = w.p0 + row * k;
    const float *wd = (const float *)w.p1 + row * kb;
    for (int64_t r = 0; r < m; r++) {
        const int8_t *aq = a.qs + r * k;
        float acc = 0.0f;
        for (int64_t p0 = 0; p0 < pieces; p0 += 64) {
            const int64_t p = p0 + lane;
            int I = 0;
            if (p < pieces) {
                const uint4 wv = *(const uint4 *)(wq + p * 16);
                const int4 av = *(const int4 *)(aq + p * 16);
                I = __builtin_amdgcn_sdot4((int)wv.x, av.x, 0, false);
                I = __builtin_amdgcn_sdot4((int)wv.y, av.y, I, false);
                I = __builtin_amdgcn_sdot4((int)wv.z, av.z, I, false);
                I = __builtin_amdgcn_sdot4((int)wv.w, av.w, I, false);
            }
            // the block's integer in every lane of its sixteen
            I += dpp_i<kQuadSwap1>(I);
            I += dpp_i<kQuadSwap2>(I);
            I += dpp_i<kHalfMirror>(I);
            I += dpp_i<kRowMirror>(I);
            if ((lane & 15) == 0 && p < pieces) {
                const int64_t b = p >> 4;
                acc += ((float)I * wd[b]) * a.d[r * kb + b];
            }
        }
        acc = wave_sum(acc);
        if (lane == 0) y[r * w.n + row] = acc;
    }
}

}  // namespace

hipError_t cq_launch_repack_q8k(const cq_weight *w, uint8_t *aos, bool inverse, hipStream_t s) {
    const int64_t nblocks = w->n * (w->k / 256);
    if (nblocks == 0) return hipSuccess;
    repack_q8k<<<(unsigned)((nblocks * 16 + 255) / 256), 256, 0, s>>>(aos, w->p0, (float *)w->p1, (int16_t *)w->p2, nblocks, inverse);
    return hipGetLastError();
}

hipError_t cq_launch_dequantize_q8k(const cq_weight *w, float *d32, uint16_t *d16, hipStream_t s) {
    const int64_t npieces = w->n * w->k / 16;
    if (npieces == 0) return hipSuccess;
    const unsigned grid = (unsigned)((npieces + 255) / 256);
    if (d16) dequant_q8k<true><<<grid, 256, 0, s>>>(w->p0, (const float *)w->p1, npieces, nullptr, d16);
    else dequant_q8k<false><<<grid, 256, 0, s>>>(w->p0, (const float *)w->p1, npieces, d32, nullptr);
    return hipGetLastError();
}

hipError_t cq_launch_q8k_weight_matmul(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    if (w->dtype != CQ_DTYPE_Q8K) return hipErrorInvalidValue;
    if (m == 0 || w->n == 0) return hipSuccess;
    CQ_LAUNCH(q8k_weight_kernel, dim3((unsigned)((w->n + 3) / 4)), 256, 0, s, *w, a, m, y);
    return hipGetLastError();
}
