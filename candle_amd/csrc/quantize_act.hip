// Activation quantizers: f32 rows -> Q8_0 / Q8_1 / Q8K blocks, bit-identical to
// the reference's CPU code (candle-core/src/quantized/k_quants.rs):
//   BlockQ8_0::from_float :586-615     d = amax/127, id = 1/d, q = round(x*id) as i8
//   BlockQ8_1::from_float :665-691     as Q8_0 plus s = f16(f16(sum q) * d)
//   BlockQ8K::from_float  :1788-1825   signed max of the first largest |x|, iscale = -128/max,
//                                      q = min(127, round(iscale*x)) as i8, bsums, d = 1/iscale
// One wave (64 lanes) handles 256 consecutive elements of one row: lane l owns elements
// 4l..4l+3 (one float4 load, a whole 1 KiB line per wave).  Reductions are wave shuffles.
// Every f32 operation is a single IEEE operation in the reference's order (this file is
// compiled with -ffp-contract=off; `/` is correctly rounded).
#include "qhip_internal.h"

namespace {

struct Sink {
    // GGML struct layout (AOS) or the workspace layout (qhip_internal.h)
    uint8_t *aos;
    cq_act_view v;
};

__device__ __forceinline__ int8_t round_to_i8(float v) { return cq_as_i8(roundf(v)); }

// Q8_0 / Q8_1: eight 32-element blocks per wave, 8 lanes per block.
template <bool AOS, bool Q8_1>
__global__ void __launch_bounds__(256) quantize_q8_0_kernel(const float *__restrict__ x,
                                                            const int32_t *__restrict__ row_ids, int64_t m,
                                                            int64_t k, Sink out) {
    const int lane = threadIdx.x & 63;
    const int64_t chunks_per_row = (k + 255) / 256;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (wave >= m * chunks_per_row) return;
    const int64_t row = wave / chunks_per_row;
    const int64_t e0 = (wave - row * chunks_per_row) * 256 + 4 * lane;
    const bool active = e0 < k;  // k % 32 == 0, so a lane is either fully inside or fully outside
    const int64_t src_row = row_ids ? (int64_t)row_ids[row] : row;
    float4 f = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) f = *(const float4 *)(x + src_row * k + e0);

    float amax = fmaxf(fmaxf(fmaxf(fmaxf(0.0f, fabsf(f.x)), fabsf(f.y)), fabsf(f.z)), fabsf(f.w));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    amax = fmaxf(amax, __shfl_xor(amax, 4));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int8_t q0 = round_to_i8(f.x * id), q1 = round_to_i8(f.y * id), q2 = round_to_i8(f.z * id),
                 q3 = round_to_i8(f.w * id);
    int sum = (int)q0 + (int)q1 + (int)q2 + (int)q3;
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    sum += __shfl_xor(sum, 4);
    if (!active) return;
    const uint32_t packed = (uint32_t)(uint8_t)q0 | ((uint32_t)(uint8_t)q1 << 8) | ((uint32_t)(uint8_t)q2 << 16) |
                            ((uint32_t)(uint8_t)q3 << 24);
    const uint16_t dh = cq_f2h(d);
    const int64_t blk = row * (k / 32) + e0 / 32;
    const int within = (int)(e0 & 31);
    uint16_t sh = 0;
    if (Q8_1) sh = cq_f2h(cq_h2f(cq_f2h((float)sum)) * cq_h2f(dh));
    if (AOS) {
        const int ts = Q8_1 ? 36 : 34;
        uint8_t *b = out.aos + blk * ts;
        uint16_t *b16 = (uint16_t *)b;  // block offsets are even
        if (within == 0) {
            b16[0] = dh;
            if (Q8_1) b16[1] = sh;
        }
        uint16_t *q16 = (uint16_t *)(b + (Q8_1 ? 4 : 2) + within);
        q16[0] = (uint16_t)(packed & 0xffff);
        q16[1] = (uint16_t)(packed >> 16);
    } else {
        *(uint32_t *)(out.v.qs + row * k + e0) = packed;
        if (within == 0) {
            out.v.d[blk] = cq_h2f(dh);
            out.v.bsum32[blk] = sum;
            if (Q8_1) out.v.s16[blk] = sh;
        }
    }
}

// Q8K: one 256-element block per wave.
template <bool AOS>
__global__ void __launch_bounds__(256) quantize_q8k_kernel(const float *__restrict__ x,
                                                           const int32_t *__restrict__ row_ids, int64_t m, int64_t k,
                                                           Sink out) {
    const int lane = threadIdx.x & 63;
    const int64_t kb = k / 256;
    const int64_t blk = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (blk >= m * kb) return;
    const int64_t row = blk / kb;
    const int64_t b_in_row = blk - row * kb;
    const int64_t src_row = row_ids ? (int64_t)row_ids[row] : row;
    const float4 f = *(const float4 *)(x + src_row * k + b_in_row * 256 + 4 * lane);

    // first index with the largest |x| (strict `<` in the reference keeps the earliest)
    float amax = 0.0f, max = 0.0f;
    int idx = 0x7fffffff;
    {
        const float v[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (amax < fabsf(v[i])) { amax = fabsf(v[i]); max = v[i]; idx = 4 * lane + i; }
        }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float oa = __shfl_xor(amax, off);
        const float om = __shfl_xor(max, off);
        const int oi = __shfl_xor(idx, off);
        if (oa > amax || (oa == amax && oi < idx)) { amax = oa; max = om; idx = oi; }
    }

    uint32_t packed = 0;
    int sum = 0;
    float d = 0.0f;
    if (amax != 0.0f) {
        const float iscale = -128.0f / max;
        const int8_t q0 = cq_as_i8(fminf(roundf(iscale * f.x), 127.0f));
        const int8_t q1 = cq_as_i8(fminf(roundf(iscale * f.y), 127.0f));
        const int8_t q2 = cq_as_i8(fminf(roundf(iscale * f.z), 127.0f));
        const int8_t q3 = cq_as_i8(fminf(roundf(iscale * f.w), 127.0f));
        packed = (uint32_t)(uint8_t)q0 | ((uint32_t)(uint8_t)q1 << 8) | ((uint32_t)(uint8_t)q2 << 16) |
                 ((uint32_t)(uint8_t)q3 << 24);
        sum = (int)q0 + (int)q1 + (int)q2 + (int)q3;
        d = 1.0f / iscale;
    }
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);  // lanes 4j..4j+3 now hold bsums[j]
    if (AOS) {
        uint8_t *b = out.aos + blk * 292;  // 292 = 4 * 73: 4-byte aligned
        if (lane == 0) *(float *)b = d;
        *(uint32_t *)(b + 4 + 4 * lane) = packed;
        if ((lane & 3) == 0) *(int16_t *)(b + 260 + 2 * (lane >> 2)) = (int16_t)sum;
    } else {
        *(uint32_t *)(out.v.qs + row * k + b_in_row * 256 + 4 * lane) = packed;
        if (lane == 0) out.v.d[blk] = d;
        if ((lane & 3) == 0) out.v.bsums[blk * 16 + (lane >> 2)] = (int16_t)sum;
        // For the GEMM (block-major copies): d again, and for the min term d * (sum of the 32
        // quants of sub-block j) as two f16 pieces p1 + p2 (22 significant bits), [p1[8] | p2[8]].
        const int64_t tb = b_in_row * out.v.m_stride + row;
        if (lane == 0) out.v.dT[tb] = d;
        const int sum32 = sum + __shfl_xor(sum, 4);
        if ((lane & 7) == 0) {
            const float v = d * (float)sum32;
            const _Float16 p1 = (_Float16)v;
            const _Float16 p2 = (_Float16)(v - (float)p1);
            _Float16 *mp = (_Float16 *)out.v.minp + tb * 16;
            mp[lane >> 3] = p1;
            mp[8 + (lane >> 3)] = p2;
        }
    }
}

template <bool AOS>
hipError_t launch(int act_dtype, const float *x, const int32_t *row_ids, int64_t m, int64_t k, Sink out,
                  hipStream_t s) {
    if (m == 0 || k == 0) return hipSuccess;
    const int threads = 256, waves = threads / 64;
    if (act_dtype == CQ_DTYPE_Q8K) {
        const int64_t nw = m * (k / 256);
        quantize_q8k_kernel<AOS><<<(unsigned)((nw + waves - 1) / waves), threads, 0, s>>>(x, row_ids, m, k, out);
    } else if (act_dtype == CQ_DTYPE_Q8_0) {
        const int64_t nw = m * ((k + 255) / 256);
        quantize_q8_0_kernel<AOS, false><<<(unsigned)((nw + waves - 1) / waves), threads, 0, s>>>(x, row_ids, m, k, out);
    } else if (act_dtype == CQ_DTYPE_Q8_1) {
        const int64_t nw = m * ((k + 255) / 256);
        quantize_q8_0_kernel<AOS, true><<<(unsigned)((nw + waves - 1) / waves), threads, 0, s>>>(x, row_ids, m, k, out);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

hipError_t cq_launch_quantize_act_aos(int act_dtype, const float *x, int64_t m, int64_t k, void *dst, hipStream_t s) {
    Sink out{};
    out.aos = (uint8_t *)dst;
    return launch<true>(act_dtype, x, nullptr, m, k, out, s);
}

hipError_t cq_launch_quantize_act_ws(int act_dtype, const float *x, const int32_t *row_ids, int64_t m, int64_t k,
                                     cq_act_view v, hipStream_t s) {
    Sink out{};
    out.v = v;
    return launch<false>(act_dtype, x, row_ids, m, k, out, s);
}
