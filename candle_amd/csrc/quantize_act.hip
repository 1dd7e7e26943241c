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
//
// A step of the caller's model can run in front of the quantizer (cq_pre): silu(x) * x2 between the
// feed-forward projections (candle-transformers/src/models/quantized_llama.rs:56-63, silu as in
// candle-core/src/op.rs:607-609) is elementwise and goes into the kernels above; rms_norm
// (candle-nn/src/ops.rs:482-495: x / sqrt(mean(x^2) + eps) * alpha) needs the whole row first and
// has a kernel of its own with one workgroup per row.
#include "qhip_internal.h"

namespace {

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float4 silu_mul4(float4 f, float4 a) {
    return make_float4(silu_f(f.x) * a.x, silu_f(f.y) * a.y, silu_f(f.z) * a.z, silu_f(f.w) * a.w);
}
__device__ __forceinline__ float4 rms_scale4(float4 f, float scale, float4 a) {
    return make_float4(scale * f.x * a.x, scale * f.y * a.y, scale * f.z * a.z, scale * f.w * a.w);
}

struct Sink {
    // GGML struct layout (AOS) or the workspace layout (qhip_internal.h)
    uint8_t *aos;
    cq_act_view v;
    cq_clear clear;
};

// The launch's threads share the floats to be cleared, four at a time (clear.p is 16-byte aligned).
__device__ __forceinline__ void clear_floats(const cq_clear &c) {
    if (!c.p) return;
    const int64_t step = (int64_t)gridDim.x * blockDim.x * 4;
    for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < c.count; i += step) {
        if (i + 4 <= c.count) {
            *(float4 *)(c.p + i) = make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
            for (int64_t j = i; j < c.count; j++) c.p[j] = 0.0f;
        }
    }
}

__device__ __forceinline__ int8_t round_to_i8(float v) { return cq_as_i8(roundf(v)); }

// Q8_0 / Q8_1: eight 32-element blocks per wave, 8 lanes per block.  `f` = the lane's four values
// at element e0 of `row` (zeros in a lane past the end of the row); called by all 64 lanes.
template <bool AOS, bool Q8_1>
__device__ __forceinline__ void q8_0_chunk(const float4 f, bool active, int64_t row, int64_t e0, int64_t k, const Sink &out) {
    float amax = fmaxf(fmaxf(fmaxf(fmaxf(0.0f, fabsf(f.x)), fabsf(f.y)), fabsf(f.z)), fabsf(f.w));
    amax = fmaxf(amax, dpp_f<kQuadSwap1>(amax));
    amax = fmaxf(amax, dpp_f<kQuadSwap2>(amax));
    amax = fmaxf(amax, dpp_f<kHalfMirror>(amax));  // quads hold one value each: the mirror pairs them
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int8_t q0 = round_to_i8(f.x * id), q1 = round_to_i8(f.y * id), q2 = round_to_i8(f.z * id),
                 q3 = round_to_i8(f.w * id);
    int sum = (int)q0 + (int)q1 + (int)q2 + (int)q3;
    sum += dpp_i<kQuadSwap1>(sum);
    sum += dpp_i<kQuadSwap2>(sum);
    sum += dpp_i<kHalfMirror>(sum);
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

template <bool AOS, bool Q8_1, bool SILU>
__global__ void __launch_bounds__(256) quantize_q8_0_kernel(const float *__restrict__ x,
                                                            const int32_t *__restrict__ row_ids, int64_t m,
                                                            int64_t k, const float *__restrict__ x2, Sink out) {
    const int lane = threadIdx.x & 63;
    const int64_t chunks_per_row = (k + 255) / 256;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    clear_floats(out.clear);
    if (wave >= m * chunks_per_row) return;
    const int64_t row = wave / chunks_per_row;
    const int64_t e0 = (wave - row * chunks_per_row) * 256 + 4 * lane;
    const bool active = e0 < k;  // k % 32 == 0, so a lane is either fully inside or fully outside
    const int64_t src_row = row_ids ? (int64_t)row_ids[row] : row;
    float4 f = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) {
        f = *(const float4 *)(x + src_row * k + e0);
        if (SILU) f = silu_mul4(f, *(const float4 *)(x2 + src_row * k + e0));
    }
    q8_0_chunk<AOS, Q8_1>(f, active, row, e0, k, out);
}

// Q8K: one 256-element block per wave.
// `f` = the lane's four values of block b_in_row of `row`; called by all 64 lanes.  SCALED: the
// block's scale is multiplied by `dscale` on the way out (the block then stands for dscale * f).
template <bool AOS, bool SCALED = false>
__device__ __forceinline__ void q8k_chunk(const float4 f, int64_t row, int64_t b_in_row, int64_t k, const Sink &out,
                                          float dscale = 1.0f) {
    const int lane = threadIdx.x & 63;
    const int64_t blk = row * (k / 256) + b_in_row;

    // The first element whose |x| equals the block maximum decides the sign of the scale (strict
    // `<` in the reference keeps the earliest).  Reductions run on DPP operands, not through LDS.
    const float a0 = fabsf(f.x), a1 = fabsf(f.y), a2 = fabsf(f.z), a3 = fabsf(f.w);
    const float amax = wave_max(fmaxf(fmaxf(fmaxf(fmaxf(0.0f, a0), a1), a2), a3));
    int idx = 0x7fffffff;
    if (a3 == amax) idx = 4 * lane + 3;
    if (a2 == amax) idx = 4 * lane + 2;
    if (a1 == amax) idx = 4 * lane + 1;
    if (a0 == amax) idx = 4 * lane;
    idx = wave_min_i(idx);
    const int sel = idx & 3;
    const float cand = sel == 0 ? f.x : (sel == 1 ? f.y : (sel == 2 ? f.z : f.w));
    const float max = readlane_f(cand, __builtin_amdgcn_readfirstlane(idx >> 2));

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
        if (SCALED) d *= dscale;
    }
    sum += dpp_i<kQuadSwap1>(sum);
    sum += dpp_i<kQuadSwap2>(sum);  // lanes 4j..4j+3 now hold bsums[j]
    if (AOS) {
        uint8_t *b = out.aos + blk * 292;  // 292 = 4 * 73: 4-byte aligned
        if (lane == 0) *(float *)b = d;
        *(uint32_t *)(b + 4 + 4 * lane) = packed;
        if ((lane & 3) == 0) *(int16_t *)(b + 260 + 2 * (lane >> 2)) = (int16_t)sum;
    } else {
        *(uint32_t *)(out.v.qs + row * k + b_in_row * 256 + 4 * lane) = packed;
        if (lane == 0) out.v.d[blk] = d;
        if ((lane & 3) == 0) out.v.bsums[blk * 16 + (lane >> 2)] = (int16_t)sum;
        // For the matrix-core kernels (block-major copies): d again, and for their min term the sixteen sums once more
        // as f16 (at most 16 * 128 in magnitude: exact), the operand of its contraction.
        const int64_t tb = b_in_row * out.v.m_stride + row;
        if (lane == 0) out.v.dT[tb] = d;
        if ((lane & 3) == 0) ((_Float16 *)out.v.bsh)[tb * 16 + (lane >> 2)] = (_Float16)(float)sum;
    }
}

template <bool AOS, bool SILU>
__global__ void __launch_bounds__(256) quantize_q8k_kernel(const float *__restrict__ x,
                                                           const int32_t *__restrict__ row_ids, int64_t m, int64_t k,
                                                           const float *__restrict__ x2, Sink out) {
    const int lane = threadIdx.x & 63;
    const int64_t kb = k / 256;
    const int64_t blk = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    clear_floats(out.clear);
    if (blk >= m * kb) return;
    const int64_t row = blk / kb;
    const int64_t b_in_row = blk - row * kb;
    const int64_t src_row = row_ids ? (int64_t)row_ids[row] : row;
    float4 f = *(const float4 *)(x + src_row * k + b_in_row * 256 + 4 * lane);
    if (SILU) f = silu_mul4(f, *(const float4 *)(x2 + src_row * k + b_in_row * 256 + 4 * lane));
    q8k_chunk<AOS>(f, row, b_in_row, k, out);
}

// rms_norm in front of the quantizer: one workgroup of four waves per row.  The squares are added
// in a fixed order that does not depend on the kernel (the decode matvec's prologue follows it
// too, so a row gives the same bits whatever the batch): groups of 8 consecutive elements as two
// sequential sums of 4, added; a binary tree over the 32 groups of a 256-element chunk (group j
// with j^1, then ^2, ^4, ^8, ^16); then the chunks one after the other.  The reference's CPU code
// adds all squares one after the other: the two sums agree to rounding, not to the bit.
// scale = 1 / sqrt(mean + eps) multiplies the elements as in the reference's device kernel
// (candle-kernels/src/reduce.cu:161-172; its CPU code divides every element by the root).  The
// second pass reads the row again (from L2):
//   Q8_0 / Q8_1: quantizes scale * x * alpha chunk by chunk;
//   Q8K: quantizes z = x * alpha and multiplies the block scales by `scale`: the quants of
//        scale * z are those of z, and the decode matvec uses the same form.
// ACT: 0 = Q8K, 1 = Q8_0, 2 = Q8_1.  Dynamic LDS: one float per chunk.
template <bool AOS, int ACT>
__global__ void __launch_bounds__(256) quantize_rms_rows_kernel(const float *__restrict__ x,
                                                                const int32_t *__restrict__ row_ids, int64_t k,
                                                                const float *__restrict__ alpha, float eps, Sink out) {
    extern __shared__ float chunk_sums[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row = blockIdx.x;
    const int64_t src_row = row_ids ? (int64_t)row_ids[row] : row;
    const float *xr = x + src_row * k;
    const int64_t chunks = (k + 255) / 256;
    clear_floats(out.clear);
    for (int64_t c = wave; c < chunks; c += 4) {
        const int64_t e0 = c * 256 + 4 * lane;
        float t = 0.0f;
        if (e0 < k) {
            const float4 f = *(const float4 *)(xr + e0);
            t = f.x * f.x;
            t += f.y * f.y;
            t += f.z * f.z;
            t += f.w * f.w;
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) t += __shfl_xor(t, off);
        if (lane == 0) chunk_sums[c] = t;
    }
    __syncthreads();
    float sum2 = chunk_sums[0];
    for (int64_t c = 1; c < chunks; c++) sum2 += chunk_sums[c];
    const float scale = 1.0f / sqrtf(sum2 / (float)k + eps);
    // Q8K: a row whose scale is NaN, infinite or zero (NaN or infinities among its elements, squares that overflow) is
    // all NaN or all zero after the reference's normalisation and quantizes to zero blocks; z alone would not
    const float keep = scale > 0.0f && scale < __builtin_inff() ? 1.0f : __builtin_nanf("");
    for (int64_t c = wave; c < chunks; c += 4) {
        const int64_t e0 = c * 256 + 4 * lane;
        const bool active = e0 < k;
        float4 f = make_float4(0.f, 0.f, 0.f, 0.f), a = f;
        if (active) { f = *(const float4 *)(xr + e0); a = *(const float4 *)(alpha + e0); }
        if (ACT == 0) q8k_chunk<AOS, true>(make_float4(f.x * a.x * keep, f.y * a.y * keep, f.z * a.z * keep, f.w * a.w * keep), row, c, k, out, keep == keep ? scale : 0.0f);
        else q8_0_chunk<AOS, ACT == 2>(rms_scale4(f, scale, a), active, row, e0, k, out);
    }
}

template <bool AOS>
hipError_t launch(int act_dtype, const float *x, const int32_t *row_ids, int64_t m, int64_t k, cq_pre pre, Sink out,
                  hipStream_t s) {
    if (m == 0 || k == 0) return hipSuccess;
    if (act_dtype != CQ_DTYPE_Q8K && act_dtype != CQ_DTYPE_Q8_0 && act_dtype != CQ_DTYPE_Q8_1) return hipErrorInvalidValue;
    const int threads = 256, waves = threads / 64;
    if (pre.kind == CQ_PRE_RMS_NORM) {
        const unsigned grid = (unsigned)m;
        const size_t lds = (size_t)((k + 255) / 256) * 4;
        if (lds > 48 * 1024) return hipErrorInvalidValue;   // rows of more than 3 million elements
        if (act_dtype == CQ_DTYPE_Q8K) quantize_rms_rows_kernel<AOS, 0><<<grid, threads, lds, s>>>(x, row_ids, k, pre.aux, pre.eps, out);
        else if (act_dtype == CQ_DTYPE_Q8_0) quantize_rms_rows_kernel<AOS, 1><<<grid, threads, lds, s>>>(x, row_ids, k, pre.aux, pre.eps, out);
        else quantize_rms_rows_kernel<AOS, 2><<<grid, threads, lds, s>>>(x, row_ids, k, pre.aux, pre.eps, out);
        return hipGetLastError();
    }
    const bool silu = pre.kind == CQ_PRE_SILU_MUL;
    const int64_t nw = act_dtype == CQ_DTYPE_Q8K ? m * (k / 256) : m * ((k + 255) / 256);
    const unsigned grid = (unsigned)((nw + waves - 1) / waves);
    if (act_dtype == CQ_DTYPE_Q8K) {
        if (silu) quantize_q8k_kernel<AOS, true><<<grid, threads, 0, s>>>(x, row_ids, m, k, pre.aux, out);
        else quantize_q8k_kernel<AOS, false><<<grid, threads, 0, s>>>(x, row_ids, m, k, nullptr, out);
    } else if (act_dtype == CQ_DTYPE_Q8_0) {
        if (silu) quantize_q8_0_kernel<AOS, false, true><<<grid, threads, 0, s>>>(x, row_ids, m, k, pre.aux, out);
        else quantize_q8_0_kernel<AOS, false, false><<<grid, threads, 0, s>>>(x, row_ids, m, k, nullptr, out);
    } else {
        if (silu) quantize_q8_0_kernel<AOS, true, true><<<grid, threads, 0, s>>>(x, row_ids, m, k, pre.aux, out);
        else quantize_q8_0_kernel<AOS, true, false><<<grid, threads, 0, s>>>(x, row_ids, m, k, nullptr, out);
    }
    return hipGetLastError();
}

}  // namespace

hipError_t cq_launch_quantize_act_aos(int act_dtype, const float *x, int64_t m, int64_t k, cq_pre pre, void *dst,
                                      hipStream_t s) {
    Sink out{};
    out.aos = (uint8_t *)dst;
    return launch<true>(act_dtype, x, nullptr, m, k, pre, out, s);
}

hipError_t cq_launch_quantize_act_ws(int act_dtype, const float *x, const int32_t *row_ids, int64_t m, int64_t k,
                                     cq_pre pre, cq_act_view v, cq_clear clear, hipStream_t s) {
    Sink out{};
    out.v = v;
    out.clear = clear;
    return launch<false>(act_dtype, x, row_ids, m, k, pre, out, s);
}
