// Decode matvec: y[m, n] = sum_k W[n, k] * x[m, k] for a few activation rows, weights streamed
// once from HBM.  Replaces the reference's MMVQ kernels (candle-kernels/src/quantized.cu:2626-2698,
// launched from quantized/cuda.rs:227-295) with the CPU formulation's arithmetic
// (k_quants.rs:237-254, :631-649, :1171-1250, :1585-1641): integer block dots against Q8_0 / Q8K
// activations, then f32 scales.
//
// Work split: a "unit" is what one lane takes of a row's main plane per step: 16 bytes (32 elements
// for Q4_0 and Q6K, 16 for Q8_0), or 32 bytes for Q4K (64 elements = two whole sub-blocks, so the
// lane's scale/min record is decoded once for them).  A wave walks one row 64 units at a time;
// nibbles are split in registers and contracted with v_dot4_i32_i8; the lane sums are reduced
// with DPP.  Quantized activations sit in LDS, permuted so that lane l of a chunk reads its
// operands at l * 16 bytes (no bank conflicts).
//
// Kernels:
//   fused_kernel   (m == 1): one launch per QMatMul call.  Each wave first issues the loads of its
//       first weight rows, then the workgroup quantizes the f32 activation row into LDS
//       (BlockQ8K / BlockQ8_0::from_float, bit-identical to quantize_act.hip), then rows are
//       processed with the next row's loads in flight (register double buffering).
//   batched_kernel (2..8 rows per pass): the same persistent structure with the quantized rows
//       copied from the workspace of the stand-alone quantizer; a weight unit is unpacked once for
//       all rows.
//   staged_kernel  (up to 4 rows per launch): the simple fallback for rows too long for the LDS
//       budget of the above.
//   int_dots_kernel: the per-block integers of the dot products, for the bit-exactness test.
#include "qhip_internal.h"

namespace {

template <int DT> struct Geo;
template <> struct Geo<CQ_DTYPE_Q4_0> { static constexpr int kElems = 32;  static constexpr int kUnitsPerBlock = 1; static constexpr bool kActK = false; };
template <> struct Geo<CQ_DTYPE_Q8_0> { static constexpr int kElems = 16;  static constexpr int kUnitsPerBlock = 2; static constexpr bool kActK = false; };
template <> struct Geo<CQ_DTYPE_Q4K>  { static constexpr int kElems = 64;  static constexpr int kUnitsPerBlock = 4; static constexpr bool kActK = true; };
template <> struct Geo<CQ_DTYPE_Q5K>  { static constexpr int kElems = 64;  static constexpr int kUnitsPerBlock = 4; static constexpr bool kActK = true; };
template <> struct Geo<CQ_DTYPE_Q6K>  { static constexpr int kElems = 32;  static constexpr int kUnitsPerBlock = 8; static constexpr bool kActK = true; };

// Q5K is Q4K with a fifth bit per quant from a plane of its own: same units, same LDS image, same
// scale / min records.
constexpr bool is_k4(int dt) { return dt == CQ_DTYPE_Q4K || dt == CQ_DTYPE_Q5K; }

// ---------------------------------------------------------------------------------------------
// LDS image of one quantized activation row:
//   lo [units] int4, hi [units] int4 (nibble types), d [blocks] f32,
//   bs: Q6K: bsums [blocks][16] i16 ; Q8_0 activations: sum of the 32 quants [blocks] i32
//   Q4K: four planes [units] int4 (elements 64u + 16j + [0,16) in plane j), d [blocks] f32,
//        bs [units] {i16 sum of elements 64u..64u+31, i16 sum of elements 64u+32..64u+63}
// ---------------------------------------------------------------------------------------------
template <int DT> __host__ __device__ constexpr int64_t act_blocks(int64_t k) { return Geo<DT>::kActK ? k / 256 : k / 32; }
template <int DT> __host__ __device__ constexpr size_t lds_row_bytes(int64_t k) {
    return (size_t)k + (size_t)act_blocks<DT>(k) * (is_k4(DT) ? 4 + 16 : (Geo<DT>::kActK ? 4 + 32 : 4 + 4));
}

// Byte offsets from the start of dynamic LDS (plain integers: every access below is then a
// ds_read / ds_write on the one LDS base pointer, never a generic-address access).
struct LdsRow {
    uint32_t lo, hi, d, bs;
};

template <int DT> __device__ __forceinline__ LdsRow lds_row(int64_t k, int m) {
    const uint32_t units = (uint32_t)(k / Geo<DT>::kElems);
    uint32_t p = (uint32_t)m * (uint32_t)lds_row_bytes<DT>(k);
    LdsRow r;
    r.lo = p;
    r.hi = p + units * 16;
    p += (uint32_t)k;
    r.d = p; p += (uint32_t)act_blocks<DT>(k) * 4;
    r.bs = p;
    return r;
}

template <typename T> __device__ __forceinline__ T lds_get(const uint8_t *smem, uint32_t off) { return *(const T *)(smem + off); }
template <typename T> __device__ __forceinline__ void lds_put(uint8_t *smem, uint32_t off, T v) { *(T *)(smem + off) = v; }

// Byte offset in LDS of the 16 consecutive activation elements [16*piece, 16*piece+16) of a row.
template <int DT> __device__ __forceinline__ uint32_t piece_off(const LdsRow r, int64_t piece, uint32_t units) {
    if (DT == CQ_DTYPE_Q8_0) return r.lo + (uint32_t)piece * 16;
    if (DT == CQ_DTYPE_Q4_0) return ((piece & 1) ? r.hi : r.lo) + (uint32_t)(piece >> 1) * 16;
    if (is_k4(DT)) return r.lo + (uint32_t)(piece & 3) * units * 16 + (uint32_t)(piece >> 2) * 16;
    // Q6K: unit p = 4h + 2t + i covers 128h + 32t + 16i + [0,16) (low) and + 64 (high)
    const int64_t b = piece >> 4;
    const int w = (int)(piece & 15);
    const int h = w >> 3, o = w & 7;
    return (o >= 4 ? r.hi : r.lo) + (uint32_t)(8 * b + 4 * h + (o & 3)) * 16;
}

// ------------------------------------------------ activation quantizer inside the matvec ----
__device__ __forceinline__ uint32_t pack4(int8_t a, int8_t b, int8_t c, int8_t d) {
    return (uint32_t)(uint8_t)a | ((uint32_t)(uint8_t)b << 8) | ((uint32_t)(uint8_t)c << 16) | ((uint32_t)(uint8_t)d << 24);
}

// The workgroup's waves quantize x[0, k) into the LDS image of row 0.  Same arithmetic, operation
// for operation, as quantize_act.hip (BlockQ8K::from_float k_quants.rs:1788-1825,
// BlockQ8_0::from_float :586-615).
// One 256-element chunk (chunk index c, this lane's four elements f at e0 = 256c + 4*lane).
template <int DT>
__device__ __forceinline__ void quantize_chunk_to_lds(uint8_t *smem, const float4 fin, int c, int e0, bool active,
                                                      bool chunk_ok, const LdsRow r, uint32_t units) {
    const int lane = threadIdx.x & 63;
    const float4 f = active ? fin : make_float4(0.f, 0.f, 0.f, 0.f);
    {
        uint32_t packed = 0;
        int sum4 = 0;
        if (Geo<DT>::kActK) {
            const float a0 = fabsf(f.x), a1 = fabsf(f.y), a2 = fabsf(f.z), a3 = fabsf(f.w);
            const float amax = wave_max(fmaxf(fmaxf(fmaxf(fmaxf(0.0f, a0), a1), a2), a3));
            // the first element whose |x| equals the block maximum decides the sign of the scale
            int idx = 0x7fffffff;
            if (a3 == amax) idx = 4 * lane + 3;
            if (a2 == amax) idx = 4 * lane + 2;
            if (a1 == amax) idx = 4 * lane + 1;
            if (a0 == amax) idx = 4 * lane;
            idx = wave_min_i(idx);
            const int sel = idx & 3;
            const float cand = sel == 0 ? f.x : (sel == 1 ? f.y : (sel == 2 ? f.z : f.w));
            const float max = readlane_f(cand, __builtin_amdgcn_readfirstlane(idx >> 2));
            float d = 0.0f;
            if (amax != 0.0f) {
                const float iscale = -128.0f / max;
                const int8_t q0 = cq_as_i8(fminf(roundf(iscale * f.x), 127.0f));
                const int8_t q1 = cq_as_i8(fminf(roundf(iscale * f.y), 127.0f));
                const int8_t q2 = cq_as_i8(fminf(roundf(iscale * f.z), 127.0f));
                const int8_t q3 = cq_as_i8(fminf(roundf(iscale * f.w), 127.0f));
                packed = pack4(q0, q1, q2, q3);
                sum4 = (int)q0 + (int)q1 + (int)q2 + (int)q3;
                d = 1.0f / iscale;
            }
            sum4 += dpp_i<kQuadSwap1>(sum4);
            sum4 += dpp_i<kQuadSwap2>(sum4);  // the four lanes of a 16-element group hold its sum
            if (chunk_ok && lane == 0) lds_put<float>(smem, r.d + 4 * c, d);
            if (is_k4(DT)) {
                sum4 += dpp_i<kHalfMirror>(sum4);   // eight lanes = one 32-element sub-block
                if (chunk_ok && (lane & 7) == 0) lds_put<int16_t>(smem, r.bs + 2 * (c * 8 + (lane >> 3)), (int16_t)sum4);
            } else if (chunk_ok && (lane & 3) == 0) {
                lds_put<int16_t>(smem, r.bs + 2 * (c * 16 + (lane >> 2)), (int16_t)sum4);
            }
        } else {
            float amax = fmaxf(fmaxf(fmaxf(fmaxf(0.0f, fabsf(f.x)), fabsf(f.y)), fabsf(f.z)), fabsf(f.w));
            amax = fmaxf(amax, dpp_f<kQuadSwap1>(amax));
            amax = fmaxf(amax, dpp_f<kQuadSwap2>(amax));
            amax = fmaxf(amax, dpp_f<kHalfMirror>(amax));  // 8 lanes = one 32-element block
            const float d = amax / 127.0f;
            const float id = d != 0.0f ? 1.0f / d : 0.0f;
            const int8_t q0 = cq_as_i8(roundf(f.x * id)), q1 = cq_as_i8(roundf(f.y * id)),
                         q2 = cq_as_i8(roundf(f.z * id)), q3 = cq_as_i8(roundf(f.w * id));
            packed = pack4(q0, q1, q2, q3);
            sum4 = (int)q0 + (int)q1 + (int)q2 + (int)q3;
            sum4 += dpp_i<kQuadSwap1>(sum4);
            sum4 += dpp_i<kQuadSwap2>(sum4);
            sum4 += dpp_i<kHalfMirror>(sum4);
            if (active && (lane & 7) == 0) {
                lds_put<float>(smem, r.d + 4 * (e0 >> 5), cq_h2f(cq_f2h(d)));
                lds_put<int32_t>(smem, r.bs + 4 * (e0 >> 5), sum4);
            }
        }
        if (active) lds_put<uint32_t>(smem, piece_off<DT>(r, e0 >> 4, units) + 4 * (lane & 3), packed);
    }
}

__device__ __forceinline__ float4 load_x_chunk(const float *x, int64_t k, int c, int chunks) {
    // Unconditional load from a clamped address (a masked load would make the compiler wait for it
    // at once); lanes past the end of the row are zeroed where the values are used.
    const int e0 = c * 256 + 4 * (int)(threadIdx.x & 63);
    (void)chunks;
    return *(const float4 *)(x + (e0 < k ? e0 : 0));
}

// A wave of an NW-wave workgroup owns chunks wave, wave + NW, ...: at most XCH of them.  All are
// loaded up front (before the weight rows) and quantized in straight-line code, so every wait is
// an exact count and the weight loads behind them stay in flight.
template <int XCH, int NW>
__device__ __forceinline__ void load_x_chunks(const float *x, int64_t k, int wave, float4 (&fx)[XCH]) {
#pragma unroll
    for (int i = 0; i < XCH; i++) fx[i] = load_x_chunk(x, k, wave + i * NW, 0);
}

template <int DT, int XCH, int NW>
__device__ __forceinline__ void quantize_row_to_lds(uint8_t *smem, int64_t k, int wave, const LdsRow r,
                                                    const float4 (&fx)[XCH]) {
    const int lane = threadIdx.x & 63;
    const int chunks = (int)((k + 255) / 256);
#pragma unroll
    for (int i = 0; i < XCH; i++) {
        const int c = wave + i * NW;
        const int e0 = c * 256 + 4 * lane;
        quantize_chunk_to_lds<DT>(smem, fx[i], c, e0, c < chunks && e0 < k, c < chunks, r, (uint32_t)(k / Geo<DT>::kElems));
    }
}

// ---- model steps in front of the quantizer (cq_pre) --------------------------------------------
// silu(v) = v / (1 + exp(-v)) (candle-core/src/op.rs:607-609), every operation single and in the
// reference's order; rms_norm as the reference's device kernel writes it, scale * x * alpha
// (candle-kernels/src/reduce.cu:161-172), with scale = 1 / sqrt(mean + eps) from two correctly
// rounded operations (the CPU code divides each element by sqrt(mean + eps) instead,
// candle-nn/src/ops.rs:491-494: a difference of a unit in the last place of some elements).
__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float4 silu_mul4(float4 f, float4 a) {
    return make_float4(silu_f(f.x) * a.x, silu_f(f.y) * a.y, silu_f(f.z) * a.z, silu_f(f.w) * a.w);
}
__device__ __forceinline__ float4 rms_scale4(float4 f, float scale, float4 a) {
    return make_float4(scale * f.x * a.x, scale * f.y * a.y, scale * f.z * a.z, scale * f.w * a.w);
}
__device__ __forceinline__ float4 mul4(float4 f, float4 a) { return make_float4(f.x * a.x, f.y * a.y, f.z * a.z, f.w * a.w); }
__device__ __forceinline__ float sum_sq4(float4 f) {
    float t = f.x * f.x;
    t += f.y * f.y;
    t += f.z * f.z;
    t += f.w * f.w;
    return t;
}
// LDS offset of the per-chunk sums of squares: behind the activation image
template <int DT> __host__ __device__ constexpr size_t fused_red_offset(int64_t k) { return (lds_row_bytes<DT>(k) + 15) / 16 * 16; }

// ---- Q8K activations, two chunks per wave ------------------------------------------------------
// Lane l takes the eight consecutive elements 8*(l%32) + [0,8) of chunk 2*pair + l/32, so a wave
// covers two 256-element chunks and the per-chunk work (maximum search, the two divisions) is
// paid once per eight elements instead of once per four.  Same arithmetic as above.
struct X8 {
    float4 a, b;
};

template <int XP, int NW>
__device__ __forceinline__ void load_x_pairs(const float *x, int64_t k, int wave, X8 (&fx)[XP]) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i < XP; i++) {
        const int e0 = (2 * (wave + i * NW) + (lane >> 5)) * 256 + 8 * (lane & 31);
        const float *p = x + (e0 < k ? e0 : 0);   // k is a multiple of 256: a chunk is inside or outside as a whole
        fx[i].a = *(const float4 *)p;
        fx[i].b = *(const float4 *)(p + 4);
    }
}

// Maxima over the two halves of the wave (lanes 0..31 and 32..63) of non-negative floats, as two
// wave-uniform values.  Non-negative floats order like their bit patterns, so the steps are single
// integer max instructions with a DPP operand.
__device__ __forceinline__ void half_max_bits(uint32_t v, uint32_t &lo, uint32_t &hi) {
    v = max(v, (uint32_t)dpp_i<kQuadSwap1>((int)v));
    v = max(v, (uint32_t)dpp_i<kQuadSwap2>((int)v));
    v = max(v, (uint32_t)dpp_i<kHalfMirror>((int)v));
    v = max(v, (uint32_t)dpp_i<kRowMirror>((int)v));
    lo = max((uint32_t)__builtin_amdgcn_readlane((int)v, 0), (uint32_t)__builtin_amdgcn_readlane((int)v, 16));
    hi = max((uint32_t)__builtin_amdgcn_readlane((int)v, 32), (uint32_t)__builtin_amdgcn_readlane((int)v, 48));
}
// max / min of three floats in one instruction (NaN operands lose against numbers)
__device__ __forceinline__ float max3f(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float min3f(float a, float b, float c) {
    float r;
    asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
// the same against 0.0 as the third operand: never NaN, never below / above zero
__device__ __forceinline__ float max3f_zero(float a, float b) {
    float r;
    asm("v_max3_f32 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float min3f_zero(float a, float b) {
    float r;
    asm("v_min3_f32 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ int half_min_i(int v) {
    v = min(v, dpp_i<kQuadSwap1>(v));
    v = min(v, dpp_i<kQuadSwap2>(v));
    v = min(v, dpp_i<kHalfMirror>(v));
    v = min(v, dpp_i<kRowMirror>(v));
    const int lo = min(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16));
    const int hi = min(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48));
    return (threadIdx.x & 32) ? hi : lo;
}

// Low bytes of four integers as one word.
__device__ __forceinline__ uint32_t pack4i(int a, int b, int c, int d) {
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

template <int DT>
__device__ __forceinline__ void quantize_pair_to_lds(uint8_t *smem, const X8 &fin, int c, bool chunk_ok,
                                                     const LdsRow r, uint32_t units) {
    const int lane = threadIdx.x & 63, hl = lane & 31;
    const float v[8] = {fin.a.x, fin.a.y, fin.a.z, fin.a.w, fin.b.x, fin.b.y, fin.b.z, fin.b.w};
    // magnitude of the lane's largest positive and largest negative value (zero if it has none), then
    // of the chunk (an out-of-range chunk goes through the arithmetic on the bytes of chunk 0; nothing
    // of it is stored)
    // (0.0 as one operand: a lane whose eight values are all NaN ends with zero, as the reference's search, whose
    // comparisons with a NaN are false, passes over them)
    const float vmax = max3f(max3f(v[0], v[1], v[2]), max3f(v[3], v[4], v[5]), max3f_zero(v[6], v[7]));
    const float vmin = min3f(min3f(v[0], v[1], v[2]), min3f(v[3], v[4], v[5]), min3f_zero(v[6], v[7]));
    const uint32_t pbits = (uint32_t)max(__builtin_bit_cast(int, vmax), 0);
    const uint32_t nbits = (uint32_t)max(__builtin_bit_cast(int, vmin) ^ (int)0x80000000, 0);
    uint32_t a_lo, a_hi;
    half_max_bits(max(pbits, nbits), a_lo, a_hi);
    const bool upper = (lane & 32) != 0;
    const uint32_t abits = upper ? a_hi : a_lo;
    // The first element of the chunk whose |x| equals the maximum decides the sign of the scale.
    // Unless the maximum occurs with both signs that is simply the sign it occurs with; all of this
    // is wave-uniform (scalar) work on the two lane masks.
    const uint64_t pos_hit = __builtin_amdgcn_ballot_w64(pbits == abits);
    const uint64_t neg_hit = __builtin_amdgcn_ballot_w64(nbits == abits);
    const bool pos_lo = (uint32_t)pos_hit != 0, pos_hi = (uint32_t)(pos_hit >> 32) != 0;
    const bool neg_lo = (uint32_t)neg_hit != 0, neg_hi = (uint32_t)(neg_hit >> 32) != 0;
    const uint32_t m_lo = a_lo | (neg_lo ? 0x80000000u : 0u), m_hi = a_hi | (neg_hi ? 0x80000000u : 0u);
    uint32_t mbits = upper ? m_hi : m_lo;
    if ((pos_lo && neg_lo && a_lo != 0) || (pos_hi && neg_hi && a_hi != 0)) {
        // both signs in one of the chunks: search the first index the long way
        int idx = 0x7fffffff;
        float cand = 0.0f;
#pragma unroll
        for (int i = 7; i >= 0; i--) {
            if ((__builtin_bit_cast(uint32_t, v[i]) & 0x7fffffffu) == abits) { idx = 8 * hl + i; cand = v[i]; }
        }
        idx = half_min_i(idx);
        const int src_lo = (__builtin_amdgcn_readlane(idx, 0) >> 3) & 31;
        const int src_hi = 32 + ((__builtin_amdgcn_readlane(idx, 32) >> 3) & 31);
        const float max_lo = readlane_f(cand, src_lo), max_hi = readlane_f(cand, src_hi);
        mbits = __builtin_bit_cast(uint32_t, upper ? max_hi : max_lo);
    }
    const float max = __builtin_bit_cast(float, mbits);
    uint32_t w0 = 0, w1 = 0;
    int sum = 0;
    float d = 0.0f;
    if (abits != 0) {
        const float iscale = -128.0f / max;
        int q[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            q[i] = min(cq_round_away_i32(iscale * v[i]), 127);
            sum += q[i];
        }
        w0 = pack4i(q[0], q[1], q[2], q[3]);
        w1 = pack4i(q[4], q[5], q[6], q[7]);
        d = 1.0f / iscale;
    }
    sum += dpp_i<kQuadSwap1>(sum);   // two lanes = one 16-element group
    if (is_k4(DT)) {
        sum += dpp_i<kQuadSwap2>(sum);   // four lanes = one 32-element sub-block
        if (chunk_ok && (hl & 3) == 0) lds_put<int16_t>(smem, r.bs + 2 * (c * 8 + (hl >> 2)), (int16_t)sum);
    } else if (chunk_ok && (hl & 1) == 0) {
        lds_put<int16_t>(smem, r.bs + 2 * (c * 16 + (hl >> 1)), (int16_t)sum);
    }
    if (chunk_ok) {
        if (hl == 0) lds_put<float>(smem, r.d + 4 * c, d);
        lds_put<uint2>(smem, piece_off<DT>(r, c * 16 + (hl >> 1), units) + 8 * (hl & 1), make_uint2(w0, w1));
    }
}

template <int DT, int XP, int NW>
__device__ __forceinline__ void quantize_pairs_to_lds(uint8_t *smem, int64_t k, int wave, const LdsRow r,
                                                      const X8 (&fx)[XP]) {
    const int lane = threadIdx.x & 63;
    const int chunks = (int)(k / 256);
#pragma unroll
    for (int i = 0; i < XP; i++) {
        const int c = 2 * (wave + i * NW) + (lane >> 5);
        quantize_pair_to_lds<DT>(smem, fx[i], c, c < chunks, r, (uint32_t)(k / Geo<DT>::kElems));
    }
}

// Copy an already-quantized activation row from the workspace into its LDS image.
template <int DT, int NT>
__device__ __forceinline__ void stage_row(uint8_t *smem, const LdsRow r, const cq_act_view &a, int64_t row, int64_t k) {
    const int4 *src = (const int4 *)(a.qs + row * k);
    const uint32_t units = (uint32_t)(k / Geo<DT>::kElems);
    for (int piece = threadIdx.x; piece < (int)(k / 16); piece += NT)
        lds_put<int4>(smem, piece_off<DT>(r, piece, units), src[piece]);
    const int nb = (int)act_blocks<DT>(k);
    for (int b = threadIdx.x; b < nb; b += NT) {
        lds_put<float>(smem, r.d + 4 * b, a.d[row * nb + b]);
        if (!Geo<DT>::kActK) lds_put<int32_t>(smem, r.bs + 4 * b, a.bsum32[row * nb + b]);
    }
    if (Geo<DT>::kActK) {
        const int32_t *bs = (const int32_t *)(a.bsums + row * nb * 16);  // 8 words per block
        for (int i = threadIdx.x; i < nb * 8; i += NT) {
            const int32_t two = bs[i];   // bsums 2i and 2i+1: the two halves of 32-element sub-block i
            if (is_k4(DT)) lds_put<int16_t>(smem, r.bs + 2 * i, (int16_t)((int16_t)(two & 0xffff) + (int16_t)(two >> 16)));
            else lds_put<int32_t>(smem, r.bs + 4 * i, two);
        }
    }
}

// The same for the part [k0, k0 + kc) of a row of k elements (k0 a multiple of 256): the LDS image is that of a row of
// kc elements.
template <int DT, int NT>
__device__ __forceinline__ void stage_row_part(uint8_t *smem, const LdsRow r, const cq_act_view &a, int64_t row, int64_t k,
                                               int64_t k0, int64_t kc) {
    const int4 *src = (const int4 *)(a.qs + row * k + k0);
    const uint32_t units = (uint32_t)(kc / Geo<DT>::kElems);
    for (int piece = threadIdx.x; piece < (int)(kc / 16); piece += NT)
        lds_put<int4>(smem, piece_off<DT>(r, piece, units), src[piece]);
    const int64_t nb = act_blocks<DT>(k), b0 = act_blocks<DT>(k0);
    const int nbc = (int)act_blocks<DT>(kc);
    for (int b = threadIdx.x; b < nbc; b += NT) {
        lds_put<float>(smem, r.d + 4 * b, a.d[row * nb + b0 + b]);
        if (!Geo<DT>::kActK) lds_put<int32_t>(smem, r.bs + 4 * b, a.bsum32[row * nb + b0 + b]);
    }
    if (Geo<DT>::kActK) {
        const int32_t *bs = (const int32_t *)(a.bsums + (row * nb + b0) * 16);  // 8 words per block
        for (int i = threadIdx.x; i < nbc * 8; i += NT) {
            const int32_t two = bs[i];
            if (is_k4(DT)) lds_put<int16_t>(smem, r.bs + 2 * i, (int16_t)((int16_t)(two & 0xffff) + (int16_t)(two >> 16)));
            else lds_put<int32_t>(smem, r.bs + 4 * i, two);
        }
    }
}

// ------------------------------------------------------------------------ weight units ----
// Raw bytes of one unit as loaded from the planes (decoded later, so loads can run ahead).
template <int DT> struct UnitRaw {
    uint4 q;       // main plane lane
    uint4 q2;      // Q4K: the second 16 bytes of the lane's 32
    uint2 h;       // Q4K: {d | dmin << 16, record {sc[2g], sc[2g+1], mn[2g], mn[2g+1]}}
    uint2 hh;      // Q6K: high bits of the lane's 32 elements; Q5K: fifth bits {L, H} of the lane's 64
    uint16_t sc2;  // Q6K: the lane's two group scales
    uint16_t d;    // Q4_0 / Q8_0 / Q6K: f16 scale
};

// Plane pointers of one weight row (wave-uniform: they stay in scalar registers and the loads take
// them as scalar base plus a 32-bit lane offset, without 64-bit vector address arithmetic).
struct RowPtr {
    const uint8_t *p0, *p1, *p2, *p3;
};
template <int DT> __device__ __forceinline__ RowPtr row_ptr(const cq_weight &w, int64_t row, uint32_t units) {
    constexpr int kB = Geo<DT>::kUnitsPerBlock;
    const int64_t g0 = row * units;   // units per row is a multiple of the units per block
    RowPtr rp;
    rp.p0 = w.p0 + g0 * (is_k4(DT) ? 32 : 16);
    rp.p1 = w.p1 + (is_k4(DT) ? (g0 / kB) * CQ_Q4K_HDR : DT == CQ_DTYPE_Q6K ? g0 * 8 : DT == CQ_DTYPE_Q4_0 ? g0 * 2 : g0);
    rp.p2 = DT == CQ_DTYPE_Q6K ? w.p2 + g0 * 2 : DT == CQ_DTYPE_Q5K ? w.p2 + g0 * 8 : nullptr;
    rp.p3 = DT == CQ_DTYPE_Q6K ? w.p3 + (g0 / kB) * 2 : nullptr;
    return rp;
}

template <int DT> __device__ __forceinline__ void load_unit(const RowPtr &rp, uint32_t u, UnitRaw<DT> &o) {
    // streaming (non-temporal) loads: every weight byte is read once per launch
    if (is_k4(DT)) {
        o.q = cq_ld_stream16(rp.p0 + u * 32u);
        o.q2 = cq_ld_stream16(rp.p0 + u * 32u + 16u);
        const uint8_t *h = rp.p1 + (u >> 2) * (uint32_t)CQ_Q4K_HDR;
        o.h.x = cq_ld_stream4(h);
        o.h.y = cq_ld_stream4(h + 4u + (u & 3u) * 4u);
        if (DT == CQ_DTYPE_Q5K) o.hh = cq_ld_stream8(rp.p2 + u * 8u);
        return;
    }
    o.q = cq_ld_stream16(rp.p0 + u * 16u);
    if (DT == CQ_DTYPE_Q4_0) o.d = cq_ld_stream2(rp.p1 + u * 2u);
    if (DT == CQ_DTYPE_Q8_0) o.d = cq_ld_stream2(rp.p1 + (u >> 1) * 2u);
    if (DT == CQ_DTYPE_Q6K) {
        o.hh = cq_ld_stream8(rp.p1 + u * 8u);
        o.sc2 = cq_ld_stream2(rp.p2 + u * 2u);
        o.d = cq_ld_stream2(rp.p3 + (u >> 3) * 2u);
    }
}

template <int DT>
__device__ __forceinline__ void load_unit(const cq_weight &w, int64_t row, int64_t units, int64_t u, UnitRaw<DT> &o) {
    load_unit<DT>(row_ptr<DT>(w, row, (uint32_t)units), (uint32_t)u, o);
}

__device__ __forceinline__ int dot16(const uint32_t w[4], const int4 &a) {
    int s = __builtin_amdgcn_sdot4((int)w[0], a.x, 0, false);
    s = __builtin_amdgcn_sdot4((int)w[1], a.y, s, false);
    s = __builtin_amdgcn_sdot4((int)w[2], a.z, s, false);
    s = __builtin_amdgcn_sdot4((int)w[3], a.w, s, false);
    return s;
}

// Decoded weight side of a unit, reused for every activation row.
template <int DT> struct UnitW {
    uint32_t lo[8], hi[8];   // Q4K uses all eight words (32 bytes of nibbles), the others four
    float dw, dmin;
    int sc_lo, sc_hi, mn_lo, mn_hi;
};

template <int DT> __device__ __forceinline__ void decode_unit(const UnitRaw<DT> &r, int p, UnitW<DT> &o) {
    const uint32_t qw[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    if (DT == CQ_DTYPE_Q8_0) {
        o.dw = cq_h2f(r.d);
#pragma unroll
        for (int i = 0; i < 4; i++) o.lo[i] = qw[i];
    } else if (DT == CQ_DTYPE_Q4_0) {
        o.dw = cq_h2f(r.d);
#pragma unroll
        for (int i = 0; i < 4; i++) { o.lo[i] = qw[i] & 0x0F0F0F0Fu; o.hi[i] = (qw[i] >> 4) & 0x0F0F0F0Fu; }
    } else if (is_k4(DT)) {
        (void)p;
        o.dw = cq_h2f((uint16_t)(r.h.x & 0xffff));
        o.dmin = cq_h2f((uint16_t)(r.h.x >> 16));
        o.sc_lo = (int)(r.h.y & 0xff); o.sc_hi = (int)((r.h.y >> 8) & 0xff);
        o.mn_lo = (int)((r.h.y >> 16) & 0xff); o.mn_hi = (int)(r.h.y >> 24);
        const uint32_t q2[4] = {r.q2.x, r.q2.y, r.q2.z, r.q2.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            o.lo[i] = qw[i] & 0x0F0F0F0Fu; o.hi[i] = (qw[i] >> 4) & 0x0F0F0F0Fu;
            o.lo[4 + i] = q2[i] & 0x0F0F0F0Fu; o.hi[4 + i] = (q2[i] >> 4) & 0x0F0F0F0Fu;
        }
        if (DT == CQ_DTYPE_Q5K) {
            // bit 8c + i of L (H) is the fifth bit of the low (high) nibble in byte c of qs word i
#pragma unroll
            for (int i = 0; i < 8; i++) {
                o.lo[i] |= ((r.hh.x >> i) & 0x01010101u) << 4;
                o.hi[i] |= ((r.hh.y >> i) & 0x01010101u) << 4;
            }
        }
    } else {
        o.sc_lo = (int)(int8_t)(r.sc2 & 0xff);
        o.sc_hi = (int)(int8_t)(r.sc2 >> 8);
        o.dw = cq_h2f(r.d);
        const uint32_t hw[2] = {r.hh.x, r.hh.y};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t H = hw[i >> 1];
            const int sh = (i & 1) * 4;
            o.lo[i] = (qw[i] & 0x0F0F0F0Fu) | (((H >> sh) & 0x03030303u) << 4);
            o.hi[i] = ((qw[i] >> 4) & 0x0F0F0F0Fu) | (((H >> (sh + 2)) & 0x03030303u) << 4);
        }
    }
}

// Integer parts of unit u (p = u mod 8) against one activation row.
//   Q4_0: I = sum (q-8)*a over the block.            Q8_0: I = sum q*a over half a block.
//   Q4K : I = sc_2g*dot_lo + sc_2g+1*dot_hi over sub-blocks 2g and 2g+1;
//         Mn = min_2g * S_lo + min_2g+1 * S_hi with S = sum of the sub-block's activation quants
//         (over the four lanes of a block: sum_j bsums_j * min_{j/2}).
//   Q6K : I = sc_lo*(dot_lo - 32*bsums_lo) + sc_hi*(dot_hi - 32*bsums_hi).
template <int DT>
__device__ __forceinline__ void unit_ints(const uint8_t *smem, const UnitW<DT> &w, const LdsRow r, uint32_t u,
                                          uint32_t units, int &I, int &Mn) {
    if (is_k4(DT)) {
        // unit u = 32 qs bytes: low nibbles are elements 64u + [0,32) (sub-block 2g, planes 0 and 1),
        // high nibbles elements 64u + 32 + [0,32) (sub-block 2g+1, planes 2 and 3)
        const uint32_t plane = units * 16, at = r.lo + u * 16;
        const int4 a0 = lds_get<int4>(smem, at), a1 = lds_get<int4>(smem, at + plane);
        const int4 a2 = lds_get<int4>(smem, at + 2 * plane), a3 = lds_get<int4>(smem, at + 3 * plane);
        const int dlo = dot16(w.lo, a0) + dot16(w.lo + 4, a1);
        const int dhi = dot16(w.hi, a2) + dot16(w.hi + 4, a3);
        I = __mul24(w.sc_lo, dlo) + __mul24(w.sc_hi, dhi);
        const uint32_t ss = lds_get<uint32_t>(smem, r.bs + 4 * u);   // {sum of sub-block 2g, sum of 2g+1} as i16
        Mn = __mul24(w.mn_lo, (int)(int16_t)(ss & 0xffff)) + __mul24(w.mn_hi, (int)ss >> 16);
        return;
    }
    const int4 alo = lds_get<int4>(smem, r.lo + u * 16);
    Mn = 0;
    if (DT == CQ_DTYPE_Q8_0) {
        I = dot16(w.lo, alo);
        return;
    }
    const int4 ahi = lds_get<int4>(smem, r.hi + u * 16);
    const int dlo = dot16(w.lo, alo), dhi = dot16(w.hi, ahi);
    if (DT == CQ_DTYPE_Q4_0) {
        I = dlo + dhi - 8 * lds_get<int32_t>(smem, r.bs + 4 * u);
    } else {
        // unit p = 4h + 2t + i: low nibbles are group 8h + 2t + i, high nibbles that + 4
        const uint32_t p = u & 7;
        const uint32_t js = p + 4 * (p >> 2);
        const uint32_t bs = r.bs + 32 * (u >> 3);
        I = __mul24(w.sc_lo, dlo - 32 * (int)lds_get<int16_t>(smem, bs + 2 * js)) +
            __mul24(w.sc_hi, dhi - 32 * (int)lds_get<int16_t>(smem, bs + 2 * (js + 4)));
    }
}

template <int DT>
__device__ __forceinline__ float unit_value(const uint8_t *smem, const UnitW<DT> &w, const LdsRow r, uint32_t u,
                                            uint32_t units) {
    int I, Mn;
    unit_ints<DT>(smem, w, r, u, units, I, Mn);
    const float ad = lds_get<float>(smem, r.d + 4 * (u / Geo<DT>::kUnitsPerBlock));
    if (is_k4(DT)) return ad * (w.dw * (float)I - w.dmin * (float)Mn);
    return ((float)I * w.dw) * ad;
}

// ---- offset terms of the types held in another type's planes ------------------------------------
// Q4_1 / Q5_1 (Q8_0 planes plus the plane p2 of block minima) add sum_b m_b * s8_b, Q2K (Q6K planes plus p4, p5)
// subtracts sum_b (d8_b * dmin_b) * sum_j bsums_j * m_j: the sums of the kernels in min_term.hip, formed from the
// quantized row in LDS with the same operations in the same order (chunk and block sums per lane, added lane after
// lane), so that the one-launch decode gives the bits of the launches that go through the workspace.  Called by whole
// waves; `lr` = the weight row.  Returns the value to add to the row's result.
// The rows of the one-launch kernels have at most 16 384 elements: one lane per group of eight 32-element blocks
// (Q4_1 / Q5_1, whole groups only) or per 256-element block (Q2K) covers a row, so the weight side of a row's term
// is one unconditional request per lane, made together with the row's units (a request behind a branch or in a loop
// would make the compiler wait for everything in flight, the next row's units included).
template <int DT> struct OffsetRow {
    uint4 mw;        // Q4_1 / Q5_1: the lane's eight block minima (f16); Q2K: the sixteen group minima of the lane's block
    uint16_t dmin;   // Q2K: the block's dmin
};
template <int DT> __device__ __forceinline__ void offset_load(const cq_weight &ws, int64_t lr, OffsetRow<DT> &o) {
    const uint32_t lane = threadIdx.x & 63;
    if constexpr (DT == CQ_DTYPE_Q8_0) {
        const uint32_t nb = (uint32_t)(ws.k / 32), b = lane * 8;   // lanes past the row re-read its last group
        o.mw = *(const uint4 *)((const uint16_t *)ws.p2 + lr * nb + (b < nb ? b : nb - 8));
    } else {
        const uint32_t kb = (uint32_t)(ws.k / 256), b = lane < kb ? lane : kb - 1;
        o.mw = *(const uint4 *)(ws.p4 + (lr * kb + b) * 16);
        o.dmin = ((const uint16_t *)ws.p5)[lr * kb + b];
    }
}
template <int DT>
__device__ __forceinline__ float offset_term(const uint8_t *smem, const LdsRow r, const cq_weight &ws, const OffsetRow<DT> &o) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t mw[4] = {o.mw.x, o.mw.y, o.mw.z, o.mw.w};
    float acc = 0.0f;
    if constexpr (DT == CQ_DTYPE_Q8_0) {
        const uint32_t nb = (uint32_t)(ws.k / 32), b = lane * 8, bc = b < nb ? b : nb - 8;
        // the blocks' scaled sums, left in place of the integer sums by the kernel's prologue
        const float4 s0 = lds_get<float4>(smem, r.bs + 4 * bc), s1 = lds_get<float4>(smem, r.bs + 4 * bc + 16);
        const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        float t = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) t += cq_h2f((uint16_t)(mw[i >> 1] >> (16 * (i & 1)))) * sv[i];
        t = b < nb ? t : 0.0f;
        for (uint32_t jj = 0; jj * 8 < nb; jj++) acc += readlane_f(t, jj);
        return acc;
    } else {
        const uint32_t kb = (uint32_t)(ws.k / 256), b = lane < kb ? lane : kb - 1;
        int summs = 0;
#pragma unroll
        for (int g = 0; g < 16; g++)
            summs += (int)lds_get<int16_t>(smem, r.bs + 32 * b + 2 * g) * (int)((mw[g >> 2] >> (8 * (g & 3))) & 0xff);
        float term = (lds_get<float>(smem, r.d + 4 * b) * cq_h2f(o.dmin)) * (float)summs;
        term = lane < kb ? term : 0.0f;
        for (uint32_t jj = 0; jj < kb; jj++) acc += readlane_f(term, jj);
        return -acc;
    }
}

// --------------------------------------------------------------------- fused kernel (m = 1) ----
// Loads of one weight row for this lane: units lane, lane + 64, ...  Lanes past the end of the row
// re-read its last unit (same cache line as a neighbour, no extra traffic) and are masked when
// accumulating, so the loads are unconditional and nothing waits on them early.
template <int DT, int UPL, bool ORDERED = false>
__device__ __forceinline__ void load_row(const cq_weight &w, int64_t row, uint32_t units, UnitRaw<DT> (&buf)[UPL]) {
    const uint32_t lane = threadIdx.x & 63;
    constexpr uint32_t kB = Geo<DT>::kUnitsPerBlock;
    const RowPtr rp = row_ptr<DT>(w, row, units);
#pragma unroll
    for (int c = 0; c < UPL; c++) {
        const uint32_t u = c * 64 + lane;
        // keep the lane's position in its block when clamping (rows hold whole blocks)
        const uint32_t uc = u < units ? u : (units - kB + (lane & (kB - 1)));
        load_unit<DT>(rp, uc, buf[c]);
        // ORDERED: keep the requests in unit order (the optimizer otherwise groups them by plane, and the first
        // unit's quants, which the arithmetic wants first, come back behind every other plane's bytes)
        if constexpr (ORDERED) asm volatile("" ::: "memory");
    }
}

template <int DT, int UPL>
__device__ __forceinline__ float row_dot(const uint8_t *smem, const LdsRow r, uint32_t units,
                                         const UnitRaw<DT> (&buf)[UPL]) {
    const uint32_t lane = threadIdx.x & 63;
    constexpr uint32_t kB = Geo<DT>::kUnitsPerBlock;
    float acc = 0.0f;
#pragma unroll
    for (int c = 0; c < UPL; c++) {
        const uint32_t u = c * 64 + lane;
        const uint32_t uc = u < units ? u : (units - kB + (lane & (kB - 1)));
        UnitW<DT> uw;
        decode_unit<DT>(buf[c], lane & 7, uw);
        const float v = unit_value<DT>(smem, uw, r, uc, units);
        acc += u < units ? v : 0.0f;
    }
    return wave_sum(acc);
}

// The same for MB activation rows in LDS: the unit is unpacked once, every row's sum is added up in the
// order of the single-row function.
template <int MB> struct Sums {
    float v[MB];
};
template <int DT, int UPL, int MB>
__device__ __forceinline__ Sums<MB> row_dot_rows(const uint8_t *smem, const LdsRow (&r)[MB], uint32_t units,
                                               const UnitRaw<DT> (&buf)[UPL]) {
    const uint32_t lane = threadIdx.x & 63;
    constexpr uint32_t kB = Geo<DT>::kUnitsPerBlock;
    Sums<MB> acc;
#pragma unroll
    for (int m = 0; m < MB; m++) acc.v[m] = 0.0f;
#pragma unroll
    for (int c = 0; c < UPL; c++) {
        const uint32_t u = c * 64 + lane;
        const uint32_t uc = u < units ? u : (units - kB + (lane & (kB - 1)));
        UnitW<DT> uw;
        decode_unit<DT>(buf[c], lane & 7, uw);
#pragma unroll
        for (int m = 0; m < MB; m++) {
            const float v = unit_value<DT>(smem, uw, r[m], uc, units);
            acc.v[m] += u < units ? v : 0.0f;
        }
    }
#pragma unroll
    for (int m = 0; m < MB; m++) acc.v[m] = wave_sum(acc.v[m]);
    return acc;
}

// Wave g of `total_waves` handles rows g, g + total_waves, ...  The launcher guarantees that every
// wave has at least DEPTH rows, so the prologue loads are unconditional: the compiler can then
// count outstanding loads exactly and waits for the activation chunk only (issued first; loads
// return in order), not for the weight rows behind it.
//   DEPTH 2 (short rows): two static register buffers, each refilled right after it is consumed.
//   DEPTH 1 (long rows) : one buffer; a row is several KiB in flight per wave already.
//
// PRE: the model step computed on the loaded activations before they are quantized (cq_pre):
// silu(x) * x2 elementwise, or rms_norm, for which the waves first add up the squares of their
// chunks and exchange the chunk sums through LDS, at the price of one more workgroup barrier.
// The weights behind the first of a launch over several weights: planes, output, first row of the launch.
template <int NWT> struct FusedMore {
    uint8_t *p[NWT - 1][4];
    float *y[NWT - 1];
    int64_t first[NWT - 1];
    int64_t n[NWT - 1];   // rows of the weight (the stride between the output rows of two activation rows)
};
template <> struct FusedMore<1> {};

// NWT > 1: up to NWT weights of the same type and row length take the same activations in one launch
// (q, k, v of an attention block).  The launch's rows are the weights' rows one after the other;
// `more` names the planes, outputs and row ranges of the weights behind the first.
// MB > 1 (with PRE none and one weight): MB activation rows x[MB][k], outputs y[MB][n]; every weight row is
// unpacked once and contracted with each of them.
template <int DT, int UPL, int NW, int DEPTH, int PRE, int NWT = 1, int MB = 1, bool OFFSETS = false>
__global__ void __launch_bounds__(NW * 64) fused_kernel(cq_weight w, const float *x, cq_pre pre,
                                                        float *__restrict__ y, int64_t total_waves,
                                                        int64_t rows_per_wave, int64_t rows_extra, FusedMore<NWT> more) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: scalar loops and branches
    const uint32_t units = (uint32_t)(w.k / Geo<DT>::kElems);
    const int64_t row0 = (int64_t)blockIdx.x * NW + wave;
    const int64_t T = total_waves;
    // weight, output and local row of a row of the launch (wave-uniform: scalar selects)
    auto pick = [&](int64_t row, cq_weight &ws, float *&ys) -> int64_t {
        ws = w;
        ys = y;
        int64_t first = 0;
        if constexpr (NWT > 1) {
#pragma unroll
            for (int t = 0; t < NWT - 1; t++) {
                if (row >= more.first[t]) {
                    ws.p0 = more.p[t][0]; ws.p1 = more.p[t][1]; ws.p2 = more.p[t][2]; ws.p3 = more.p[t][3];
                    ws.n = more.n[t];
                    ys = more.y[t];
                    first = more.first[t];
                }
            }
        }
        return row - first;
    };
    // OFFSETS: Q4_1 / Q5_1 / Q2K weights (instances of their own, so that the kernels of the plain Q8_0 and Q6K
    // weights carry nothing for them): the minima of a row travel with the row's units, requested when they are and
    // summed when the row's result is stored.
    static_assert(!OFFSETS || (PRE == CQ_PRE_NONE && NWT == 1 && (DT == CQ_DTYPE_Q8_0 || DT == CQ_DTYPE_Q6K)), "offset terms: Q8_0 / Q6K planes, one weight, no fused step");
    constexpr bool kOffsets = OFFSETS;
    auto load_launch_row = [&](int64_t row, UnitRaw<DT> (&buf)[UPL], OffsetRow<DT> &o) {
        cq_weight ws;
        float *ys;
        const int64_t lr = pick(row, ws, ys);
        // one activation row, longer weight rows of the types with one main plane: requests in unit order (measured:
        // Q8_0 4096 x 4096 5.9 -> 5.7 us, Q4K K = 14336 10.5 -> 10.3; Q6K, with three planes a unit, gains nothing at
        // one row and loses 11 % at two)
        constexpr bool kOrdered = MB == 1 && UPL >= 3 && DT != CQ_DTYPE_Q6K;
        load_row<DT, UPL, kOrdered>(ws, lr, units, buf);
        if constexpr (kOffsets) offset_load<DT>(ws, lr, o);
    };
    // rows of this wave (>= DEPTH): n / T, plus one for the first n % T waves (both from the host)
    const int64_t cnt = rows_per_wave + (row0 < rows_extra ? 1 : 0);

    // chunks of 256 activations: at most 64 * UPL units * kElems / 256; a wave quantizes one chunk
    // per step for Q8_0 activations, two for Q8K
    constexpr bool kPairs = Geo<DT>::kActK;
    constexpr int XCH = (UPL * Geo<DT>::kElems / (kPairs ? 8 : 4) + NW - 1) / NW;
    float4 fxa[MB][kPairs ? 1 : XCH];
    X8 fx8a[MB][kPairs ? XCH : 1];
#pragma unroll
    for (int m = 0; m < MB; m++) {
        if constexpr (kPairs) load_x_pairs<XCH, NW>(x + m * w.k, w.k, wave, fx8a[m]);
        else load_x_chunks<XCH, NW>(x + m * w.k, w.k, wave, fxa[m]);
    }
    auto &fx = fxa[0];
    auto &fx8 = fx8a[0];
    float4 gx[(PRE != CQ_PRE_NONE && !kPairs) ? XCH : 1];   // the second operand, at the same elements
    X8 gx8[(PRE != CQ_PRE_NONE && kPairs) ? XCH : 1];
    if constexpr (PRE != CQ_PRE_NONE) {
        if constexpr (kPairs) load_x_pairs<XCH, NW>(pre.aux, w.k, wave, gx8);
        else load_x_chunks<XCH, NW>(pre.aux, w.k, wave, gx);
    }
    // Pin the issue order: activation loads, then weight loads, then the quantizer arithmetic.
    // (The empty asm stops the optimizer from sinking loads past it, the scheduling barrier stops
    // the instruction scheduler.)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    UnitRaw<DT> a[UPL], b[DEPTH == 2 ? UPL : 1];
    OffsetRow<DT> oa = {}, ob = {};
    load_launch_row(row0, a, oa);
    if constexpr (DEPTH == 2) load_launch_row(row0 + T, b, ob);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    const LdsRow r = lds_row<DT>(w.k, 0);
    if constexpr (PRE == CQ_PRE_SILU_MUL) {
#pragma unroll
        for (int i = 0; i < XCH; i++) {
            if constexpr (kPairs) { fx8[i].a = silu_mul4(fx8[i].a, gx8[i].a); fx8[i].b = silu_mul4(fx8[i].b, gx8[i].b); }
            else fx[i] = silu_mul4(fx[i], gx[i]);
        }
    }
    // rms_norm.  Sum of squares in the order every rms_norm kernel of this library uses, so that a
    // row gives the same bits whatever the batch: groups of 8 consecutive elements (two sequential
    // sums of 4, added), a binary tree over the 32 groups of a 256-element chunk (group j with
    // j^1, then ^2, ^4, ^8, ^16), then the chunks one after the other.
    // Q8K activations: quantizing scale * z gives the quants of z and the block scales of z times
    // `scale` (up to rounding), so the waves quantize z = x * alpha at once, leave their chunk sums
    // in LDS for after the barrier that follows anyway, and multiply the row results by `scale`.
    // Q8_0 activations round their block scale to f16, which does not commute with the scaling:
    // there the elements are scaled before they are quantized, behind a barrier of its own.
    constexpr bool kRms = PRE == CQ_PRE_RMS_NORM;
    constexpr int kSlots = (kPairs ? 2 : 1) * XCH * NW;   // chunk slots of the workgroup (a multiple of 8)
    const uint32_t red = (uint32_t)fused_red_offset<DT>(w.k);
    auto row_scale = [&]() {
        // all slots are read at once and added in order; the zeros behind the last chunk change nothing
        float4 ps[kSlots / 4];
#pragma unroll
        for (int c = 0; c < kSlots / 4; c++) ps[c] = lds_get<float4>(smem, red + 16 * c);
        float sum2 = ps[0].x;
        sum2 += ps[0].y; sum2 += ps[0].z; sum2 += ps[0].w;
#pragma unroll
        for (int c = 1; c < kSlots / 4; c++) { sum2 += ps[c].x; sum2 += ps[c].y; sum2 += ps[c].z; sum2 += ps[c].w; }
        return 1.0f / sqrtf(sum2 / (float)w.k + pre.eps);
    };
    if constexpr (kRms) {
        const int chunks = (int)((w.k + 255) / 256);
#pragma unroll
        for (int i = 0; i < XCH; i++) {
            if constexpr (kPairs) {
                float t = sum_sq4(fx8[i].a) + sum_sq4(fx8[i].b);   // lane = group; 32 lanes = chunk
                t += dpp_f<kQuadSwap1>(t);
                t += dpp_f<kQuadSwap2>(t);
                t += dpp_f<kHalfMirror>(t);
                t += dpp_f<kRowMirror>(t);
                const float p_lo = readlane_f(t, 0) + readlane_f(t, 16), p_hi = readlane_f(t, 32) + readlane_f(t, 48);
                const int c = 2 * (wave + i * NW) + lane;   // every slot below kSlots is written: zero past the row
                if (lane < 2) lds_put<float>(smem, red + 4 * c, c < chunks ? (lane ? p_hi : p_lo) : 0.0f);
                fx8[i].a = mul4(fx8[i].a, gx8[i].a);
                fx8[i].b = mul4(fx8[i].b, gx8[i].b);
            } else {
                const int c = wave + i * NW;
                float t = c * 256 + 4 * lane < w.k ? sum_sq4(fx[i]) : 0.0f;   // two lanes = group
                t += dpp_f<kQuadSwap1>(t);
                t += dpp_f<kQuadSwap2>(t);
                t += dpp_f<kHalfMirror>(t);
                t += dpp_f<kRowMirror>(t);
                const float p = (readlane_f(t, 0) + readlane_f(t, 16)) + (readlane_f(t, 32) + readlane_f(t, 48));
                if (lane == 0) lds_put<float>(smem, red + 4 * c, c < chunks ? p : 0.0f);
            }
        }
        if constexpr (!kPairs) {
            __syncthreads();
            const float scale = row_scale();
#pragma unroll
            for (int i = 0; i < XCH; i++) fx[i] = rms_scale4(fx[i], scale, gx[i]);
        }
    }
    if constexpr (kPairs) quantize_pairs_to_lds<DT, XCH, NW>(smem, w.k, wave, r, fx8);
    else quantize_row_to_lds<DT, XCH, NW>(smem, w.k, wave, r, fx);
    LdsRow rm[MB];
    rm[0] = r;
#pragma unroll
    for (int m = 1; m < MB; m++) {
        rm[m] = lds_row<DT>(w.k, m);
        if constexpr (kPairs) quantize_pairs_to_lds<DT, XCH, NW>(smem, w.k, wave, rm[m], fx8a[m]);
        else quantize_row_to_lds<DT, XCH, NW>(smem, w.k, wave, rm[m], fxa[m]);
    }
    __syncthreads();
    if constexpr (OFFSETS && DT == CQ_DTYPE_Q8_0) {
        // Q4_1 / Q5_1: the activation blocks' scaled sums s = f16(f16(sum) * d) of the Q8_1 format are the same for
        // every weight row: computed once per workgroup, in place of the integer sums (which Q8_0 planes do not use)
        const uint32_t nb = (uint32_t)(w.k / 32);
#pragma unroll
        for (int m = 0; m < MB; m++) {
            for (uint32_t b = threadIdx.x; b < nb; b += NW * 64) {
                const float hs = cq_h2f(cq_f2h((float)lds_get<int32_t>(smem, rm[m].bs + 4 * b)));
                lds_put<float>(smem, rm[m].bs + 4 * b, cq_h2f(cq_f2h(hs * lds_get<float>(smem, rm[m].d + 4 * b))));
            }
        }
        __syncthreads();
    }
    float yscale = 1.0f;
    bool yscale_ok = true;   // (a NaN, infinite or zero scale: the reference's normalised row quantizes to zero blocks)
    if constexpr (kRms && kPairs) {
        yscale = row_scale();
        yscale_ok = yscale > 0.0f && yscale < __builtin_inff();
    }
    auto put = [&](int64_t row, Sums<MB> v, const OffsetRow<DT> &o) {
        cq_weight ws;
        float *ys;
        const int64_t lr = pick(row, ws, ys);
#pragma unroll
        for (int m = 0; m < MB; m++) {
            float t = v.v[m];
            if constexpr (kRms && kPairs) t = yscale_ok ? t * yscale : 0.0f;
            if constexpr (kOffsets) {
                t += offset_term<DT>(smem, rm[m], ws, o);   // the f32 addition the workspace path's second launch makes
            }
            if (lane == 0) ys[m * ws.n + lr] = t;
        }
    };

    if constexpr (DEPTH == 1) {
        for (int64_t i = 0; i < cnt; i++) {
            const Sums<MB> s = row_dot_rows<DT, UPL, MB>(smem, rm, units, a);
            const OffsetRow<DT> o = oa;
            if (i + 1 < cnt) load_launch_row(row0 + (i + 1) * T, a, oa);
            put(row0 + i * T, s, o);
        }
    } else {
        int64_t i = 0;
        // steady state: rows i and i+1 are in a and b, rows i+2 and i+3 exist
        for (; i + 3 < cnt; i += 2) {
            // the refill of a buffer is issued before the arithmetic on its old contents (which move
            // to other registers), so a wave keeps up to three rows in flight
            Sums<MB> s0, s1;
            const OffsetRow<DT> o0 = oa, o1 = ob;
            if constexpr (UPL <= 2) {
                UnitRaw<DT> ta[UPL], tb[UPL];
#pragma unroll
                for (int c = 0; c < UPL; c++) ta[c] = a[c];
                load_launch_row(row0 + (i + 2) * T, a, oa);
                __builtin_amdgcn_sched_barrier(0);
                s0 = row_dot_rows<DT, UPL, MB>(smem, rm, units, ta);
#pragma unroll
                for (int c = 0; c < UPL; c++) tb[c] = b[c];
                load_launch_row(row0 + (i + 3) * T, b, ob);
                __builtin_amdgcn_sched_barrier(0);
                s1 = row_dot_rows<DT, UPL, MB>(smem, rm, units, tb);
            } else {
                s0 = row_dot_rows<DT, UPL, MB>(smem, rm, units, a);
                load_launch_row(row0 + (i + 2) * T, a, oa);
                s1 = row_dot_rows<DT, UPL, MB>(smem, rm, units, b);
                load_launch_row(row0 + (i + 3) * T, b, ob);
            }
            put(row0 + i * T, s0, o0);
            put(row0 + (i + 1) * T, s1, o1);
        }
        // tail: two or three rows left (a = row i, b = row i+1, maybe row i+2 still to load)
        const bool third = i + 2 < cnt;
        if (!third) {
            // two rows in one stretch of straight-line code: their dependent chains (dot products,
            // wave reductions) interleave
            const Sums<MB> s0 = row_dot_rows<DT, UPL, MB>(smem, rm, units, a);
            const Sums<MB> s1 = row_dot_rows<DT, UPL, MB>(smem, rm, units, b);
            put(row0 + i * T, s0, oa);
            put(row0 + (i + 1) * T, s1, ob);
        } else {
            const Sums<MB> s0 = row_dot_rows<DT, UPL, MB>(smem, rm, units, a);
            const OffsetRow<DT> o0 = oa;
            load_launch_row(row0 + (i + 2) * T, a, oa);
            const Sums<MB> s1 = row_dot_rows<DT, UPL, MB>(smem, rm, units, b);
            put(row0 + i * T, s0, o0);
            put(row0 + (i + 1) * T, s1, ob);
            const Sums<MB> s2 = row_dot_rows<DT, UPL, MB>(smem, rm, units, a);
            put(row0 + (i + 2) * T, s2, oa);
        }
    }
}

// ------------------------------------------------------ batched kernel (2 <= m <= 8 rows) ----
// The same persistent structure as fused_kernel for a few activation rows: one workgroup per CU
// copies the MB quantized rows from the workspace into LDS once, then every wave streams its weight
// rows (next row's loads in flight) and contracts each decoded unit against all MB rows, so the
// weights are read and unpacked once.  Rows m0 + MB and beyond of the call are masked (their LDS
// image is a copy of the last valid row).
template <int DT, int UPL, int MB>
__device__ __forceinline__ void row_dot_mb(const uint8_t *smem, const LdsRow (&rows)[MB], uint32_t units,
                                           const UnitRaw<DT> (&buf)[UPL], float (&out)[MB]) {
    const uint32_t lane = threadIdx.x & 63;
    constexpr uint32_t kB = Geo<DT>::kUnitsPerBlock;
    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; m++) acc[m] = 0.0f;
#pragma unroll
    for (int c = 0; c < UPL; c++) {
        const uint32_t u = c * 64 + lane;
        const uint32_t uc = u < units ? u : (units - kB + (lane & (kB - 1)));
        UnitW<DT> uw;
        decode_unit<DT>(buf[c], lane & 7, uw);
#pragma unroll
        for (int m = 0; m < MB; m++) {
            const float v = unit_value<DT>(smem, uw, rows[m], uc, units);
            acc[m] += u < units ? v : 0.0f;
        }
    }
#pragma unroll
    for (int m = 0; m < MB; m++) out[m] = wave_sum(acc[m]);
}

template <int DT, int UPL, int NW, int MB>
__global__ void __launch_bounds__(NW * 64) batched_kernel(cq_weight w, cq_act_view a, int64_t m0, int64_t m,
                                                          float *__restrict__ y, int64_t total_waves,
                                                          int64_t rows_per_wave, int64_t rows_extra) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t units = (uint32_t)(w.k / Geo<DT>::kElems);
    const int64_t row0 = (int64_t)blockIdx.x * NW + wave;
    const int64_t T = total_waves;
    const int64_t cnt = rows_per_wave + (row0 < rows_extra ? 1 : 0);   // >= 1

    UnitRaw<DT> cur[UPL], nxt[UPL];
    load_row<DT, UPL>(w, row0, units, cur);
    LdsRow rows[MB];
#pragma unroll
    for (int i = 0; i < MB; i++) {
        rows[i] = lds_row<DT>(w.k, i);
        const int64_t src = m0 + i < m ? m0 + i : m - 1;
        stage_row<DT, NW * 64>(smem, rows[i], a, src, w.k);
    }
    __syncthreads();
    for (int64_t i = 0; i < cnt; i++) {
        const int64_t row = row0 + i * T;
        const bool more = i + 1 < cnt;
        load_row<DT, UPL>(w, more ? row + T : row, units, nxt);   // unconditional: the last one re-reads its own row
        float out[MB];
        row_dot_mb<DT, UPL, MB>(smem, rows, units, cur, out);
        if (lane == 0) {
#pragma unroll
            for (int j = 0; j < MB; j++)
                if (m0 + j < m) y[(m0 + j) * w.n + row] = out[j];
        }
#pragma unroll
        for (int c = 0; c < UPL; c++) cur[c] = nxt[c];
    }
}

// ------------------------------------------------------------ staged kernel (m <= 4 rows) ----
constexpr int kStagedThreads = 256;
// The dot-product kernels keep one whole quantized activation row in LDS: a workgroup can have 160 KiB.
constexpr size_t kMaxRowLds = 160 * 1024;

template <int DT, int MB>
__global__ void __launch_bounds__(kStagedThreads) staged_kernel(cq_weight w, cq_act_view a, int64_t m0,
                                                                int rows_per_wg, float *__restrict__ y) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int64_t units = w.k / Geo<DT>::kElems;
    LdsRow rows[MB];
#pragma unroll
    for (int m = 0; m < MB; m++) {
        rows[m] = lds_row<DT>(w.k, m);
        stage_row<DT, kStagedThreads>(smem, rows[m], a, m0 + m, w.k);
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row_begin = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t row_end = row_begin + rows_per_wg < w.n ? row_begin + rows_per_wg : w.n;
    for (int64_t row = row_begin + wave; row < row_end; row += kStagedThreads / 64) {
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; m++) acc[m] = 0.0f;
#pragma unroll 2
        for (int64_t u = lane; u < units; u += 64) {
            UnitRaw<DT> raw;
            load_unit<DT>(w, row, units, u, raw);
            UnitW<DT> uw;
            decode_unit<DT>(raw, lane & 7, uw);
#pragma unroll
            for (int m = 0; m < MB; m++) acc[m] += unit_value<DT>(smem, uw, rows[m], (uint32_t)u, (uint32_t)units);
        }
#pragma unroll
        for (int m = 0; m < MB; m++) {
            const float s = wave_sum(acc[m]);
            if (lane == 0) y[(m0 + m) * w.n + row] = s;
        }
    }
}

// ----------------------------------------------------- rows of any length (m <= 4 rows per launch) ----
// staged_kernel for rows whose quantized image does not fit the LDS (k_quants::matmul, k_quants.rs:1842-1883, has no
// limit on k): the workgroup walks the row in chunks of kChunkElems elements, one chunk of the MB activation rows in
// LDS at a time, and every wave keeps the partial sums of its weight rows in registers across the chunks.  A lane adds
// its units in the order of staged_kernel (a chunk is a whole number of 64-unit steps), so the two kernels give the
// same bits.
constexpr int64_t kChunkElems = 16384;
constexpr int kChunkRowsPerWave = 4;   // rows_per_wg <= 16, four waves
template <int DT, int MB>
__global__ void __launch_bounds__(kStagedThreads) chunked_kernel(cq_weight w, cq_act_view a, int64_t m0,
                                                                 int rows_per_wg, float *__restrict__ y) {
    extern __shared__ __align__(16) uint8_t smem[];
    static_assert(kChunkElems % (64 * Geo<DT>::kElems) == 0, "whole 64-unit steps per chunk");
    const int64_t units = w.k / Geo<DT>::kElems;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row_begin = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t row_end = row_begin + rows_per_wg < w.n ? row_begin + rows_per_wg : w.n;
    float acc[kChunkRowsPerWave][MB];
#pragma unroll
    for (int ri = 0; ri < kChunkRowsPerWave; ri++)
#pragma unroll
        for (int m = 0; m < MB; m++) acc[ri][m] = 0.0f;
    for (int64_t k0 = 0; k0 < w.k; k0 += kChunkElems) {
        const int64_t kc = w.k - k0 < kChunkElems ? w.k - k0 : kChunkElems;
        __syncthreads();   // every wave is done with the chunk before
        LdsRow rows[MB];
#pragma unroll
        for (int m = 0; m < MB; m++) {
            rows[m] = lds_row<DT>(kc, m);
            stage_row_part<DT, kStagedThreads>(smem, rows[m], a, m0 + m, w.k, k0, kc);
        }
        __syncthreads();
        const int64_t u0 = k0 / Geo<DT>::kElems, uc = kc / Geo<DT>::kElems;
#pragma unroll
        for (int ri = 0; ri < kChunkRowsPerWave; ri++) {
            const int64_t row = row_begin + wave + ri * (kStagedThreads / 64);
            if (row >= row_end) continue;
#pragma unroll 2
            for (int64_t u = lane; u < uc; u += 64) {
                UnitRaw<DT> raw;
                load_unit<DT>(w, row, units, u0 + u, raw);
                UnitW<DT> uw;
                decode_unit<DT>(raw, lane & 7, uw);
#pragma unroll
                for (int m = 0; m < MB; m++) acc[ri][m] += unit_value<DT>(smem, uw, rows[m], (uint32_t)u, (uint32_t)uc);
            }
        }
    }
#pragma unroll
    for (int ri = 0; ri < kChunkRowsPerWave; ri++) {
        const int64_t row = row_begin + wave + ri * (kStagedThreads / 64);
#pragma unroll
        for (int m = 0; m < MB; m++) {
            const float t = wave_sum(acc[ri][m]);
            if (lane == 0 && row < row_end) y[(m0 + m) * w.n + row] = t;
        }
    }
}

// ------------------------------------------------- K-quant weights x Q8_1 activations ----
// The formulation of the reference's CUDA arm (mul_mat_via_q8_1, quantized/cuda.rs:298-365; dot bodies
// candle-kernels/src/quantized.cu:2141-2166 for Q4K and :2258-2281 for Q6K) with the activations quantized by the CPU
// rule of BlockQ8_1::from_float (k_quants.rs:665-691):
//   Q4K: per block  d * sum_j d8_j * float(sc_j * dot_j)  -  dmin * sum_j s8_j * float(m_j)      (j: 32-element sub-blocks)
//   Q6K: per block  d * sum_j float(sc_j) * (d8_{j/2} * float(dot_j))                            (j: 16-element groups)
// with d8 / s8 the scale and the `s` field of the activation's 32-element Q8_1 block.  The integers (dot_j, sc_j * dot_j)
// are exact; the f32 sums run per lane and then over the wave, not in the reference's block order.
// LDS image of one activation row: the int8 planes of the Q8K image (piece_off), then per unit the two block
// scales {d8, d8'} and, for Q4K, the two `s` values, as f32.
template <int DT> __host__ __device__ constexpr size_t q81_row_bytes(int64_t k) {
    return (size_t)k + (size_t)(k / Geo<DT>::kElems) * (DT == CQ_DTYPE_Q4K ? 16 : 8);
}

template <int DT, int MB>
__global__ void __launch_bounds__(kStagedThreads) q81_kernel(cq_weight w, cq_act_view a, int64_t m0, int64_t m,
                                                             int rows_per_wg, float *__restrict__ y) {
    static_assert(DT == CQ_DTYPE_Q4K || DT == CQ_DTYPE_Q6K, "Q4K and Q6K only");
    extern __shared__ __align__(16) uint8_t smem[];
    const int64_t k = w.k;
    const uint32_t units = (uint32_t)(k / Geo<DT>::kElems);
    const uint32_t row_bytes = (uint32_t)q81_row_bytes<DT>(k);
    const int64_t nb32 = k / 32;
    // ---- stage MB quantized rows (rows past the last one repeat it; their results are not stored)
    for (int i = 0; i < MB; i++) {
        const int64_t src = m0 + i < m ? m0 + i : m - 1;
        LdsRow r;
        r.lo = i * row_bytes;
        r.hi = r.lo + units * 16;
        const int4 *q = (const int4 *)(a.qs + src * k);
        for (int piece = threadIdx.x; piece < (int)(k / 16); piece += kStagedThreads)
            lds_put<int4>(smem, piece_off<DT>(r, piece, units), q[piece]);
        const uint32_t sc_off = i * row_bytes + (uint32_t)k;
        for (uint32_t u = threadIdx.x; u < units; u += kStagedThreads) {
            if (DT == CQ_DTYPE_Q4K) {
                // unit u = sub-blocks 2u and 2u + 1 = Q8_1 blocks 2u, 2u + 1
                const float2 d = *(const float2 *)(a.d + src * nb32 + 2 * u);
                const uint32_t s2 = *(const uint32_t *)(a.s16 + src * nb32 + 2 * u);
                lds_put<float4>(smem, sc_off + 16 * u, make_float4(d.x, d.y, cq_h2f((uint16_t)(s2 & 0xffff)), cq_h2f((uint16_t)(s2 >> 16))));
            } else {
                // unit p = 4h + 2t + i of a weight block: the low nibbles are elements 128h + 32t + 16i + [0, 16) of the
                // block, the high nibbles those 64 further on: Q8_1 blocks 4h + t and 4h + t + 2 of the block's eight
                const uint32_t blk = u >> 3, p = u & 7, q = 4 * (p >> 2) + ((p >> 1) & 1);
                const float *d = a.d + src * nb32 + 8 * blk + q;
                lds_put<float2>(smem, sc_off + 8 * u, make_float2(d[0], d[2]));
            }
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row_begin = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t row_end = row_begin + rows_per_wg < w.n ? row_begin + rows_per_wg : w.n;
    for (int64_t row = row_begin + wave; row < row_end; row += kStagedThreads / 64) {
        float acc[MB];
#pragma unroll
        for (int i = 0; i < MB; i++) acc[i] = 0.0f;
        for (uint32_t u = lane; u < units; u += 64) {
            UnitRaw<DT> raw;
            load_unit<DT>(w, row, units, u, raw);
            UnitW<DT> uw;
            decode_unit<DT>(raw, lane & 7, uw);
            if (DT == CQ_DTYPE_Q6K) {
                // quants 0..63 -> q - 32 as int8, byte-wise (no carry between bytes: q + 0x60 < 0x100)
#pragma unroll
                for (int x = 0; x < 4; x++) {
                    uw.lo[x] = (uw.lo[x] + 0x60606060u) ^ 0x80808080u;
                    uw.hi[x] = (uw.hi[x] + 0x60606060u) ^ 0x80808080u;
                }
            }
#pragma unroll
            for (int i = 0; i < MB; i++) {
                const uint32_t base = i * row_bytes;
                if (DT == CQ_DTYPE_Q4K) {
                    const uint32_t plane = units * 16, at = base + u * 16;
                    const int4 a0 = lds_get<int4>(smem, at), a1 = lds_get<int4>(smem, at + plane);
                    const int4 a2 = lds_get<int4>(smem, at + 2 * plane), a3 = lds_get<int4>(smem, at + 3 * plane);
                    const int dlo = dot16(uw.lo, a0) + dot16(uw.lo + 4, a1);
                    const int dhi = dot16(uw.hi, a2) + dot16(uw.hi + 4, a3);
                    const float4 sc = lds_get<float4>(smem, base + (uint32_t)k + 16 * u);   // {d8, d8', s8, s8'}
                    float sd = sc.x * (float)(dlo * uw.sc_lo);
                    sd += sc.y * (float)(dhi * uw.sc_hi);
                    float sm = sc.z * (float)uw.mn_lo;
                    sm += sc.w * (float)uw.mn_hi;
                    acc[i] += uw.dw * sd - uw.dmin * sm;
                } else {
                    const int4 alo = lds_get<int4>(smem, base + u * 16);
                    const int4 ahi = lds_get<int4>(smem, base + units * 16 + u * 16);
                    const int dlo = dot16(uw.lo, alo), dhi = dot16(uw.hi, ahi);
                    const float2 d8 = lds_get<float2>(smem, base + (uint32_t)k + 8 * u);
                    float sd = (float)uw.sc_lo * (d8.x * (float)dlo);
                    sd += (float)uw.sc_hi * (d8.y * (float)dhi);
                    acc[i] += uw.dw * sd;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MB; i++) {
            const float sum = wave_sum(acc[i]);
            if (lane == 0 && m0 + i < m) y[(m0 + i) * w.n + row] = sum;
        }
    }
}

// Per-block integer dots for verification: same unit arithmetic as the kernels above.
template <int DT>
__global__ void __launch_bounds__(kStagedThreads) int_dots_kernel(cq_weight w, cq_act_view a, int64_t m0,
                                                                  int rows_per_wg, int32_t *__restrict__ out_i,
                                                                  int32_t *__restrict__ out_mn) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int64_t units = w.k / Geo<DT>::kElems;
    const LdsRow r = lds_row<DT>(w.k, 0);
    stage_row<DT, kStagedThreads>(smem, r, a, m0, w.k);
    __syncthreads();
    constexpr int kUPB = Geo<DT>::kUnitsPerBlock;
    const int64_t kb = units / kUPB;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row_begin = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t row_end = row_begin + rows_per_wg < w.n ? row_begin + rows_per_wg : w.n;
    for (int64_t row = row_begin + wave; row < row_end; row += kStagedThreads / 64) {
        for (int64_t u0 = 0; u0 < units; u0 += 64) {
            const int64_t u = u0 + lane;
            int I = 0, Mn = 0;
            if (u < units) {
                UnitRaw<DT> raw;
                load_unit<DT>(w, row, units, u, raw);
                UnitW<DT> uw;
                decode_unit<DT>(raw, lane & 7, uw);
                unit_ints<DT>(smem, uw, r, (uint32_t)u, (uint32_t)units, I, Mn);
            }
#pragma unroll
            for (int off = 1; off < kUPB; off <<= 1) {
                I += __shfl_xor(I, off);
                Mn += __shfl_xor(Mn, off);
            }
            if (u < units && (u % kUPB) == 0) {
                const int64_t o = (m0 * w.n + row) * kb + u / kUPB;
                out_i[o] = I;
                if (out_mn) out_mn[o] = Mn;
            }
        }
    }
}

// ------------------------------------------------------------------------------- launch ----
int g_num_cus = 0;
int num_cus() {
    if (g_num_cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            g_num_cus = n;
        else
            g_num_cus = 256;
    }
    return g_num_cus;
}

// Eight waves per workgroup, one workgroup per CU.  Whole workgroups only, and every wave
// gets at least `depth` rows: wgs * 8 * depth <= n.
template <int DT, int UPL, int PRE, int NWT = 1, int MB = 1>
hipError_t launch_fused_upl(const cq_weight *w, int64_t n, FusedMore<NWT> more, const float *x, cq_pre pre, float *y,
                            hipStream_t s) {
    constexpr int NW = 8;
    constexpr int kXch = (UPL * Geo<DT>::kElems / (Geo<DT>::kActK ? 8 : 4) + NW - 1) / NW;   // as in the kernel
    const size_t lds = PRE == CQ_PRE_RMS_NORM ? fused_red_offset<DT>(w->k) + 4 * (size_t)((Geo<DT>::kActK ? 2 : 1) * kXch * NW)
                                              : lds_row_bytes<DT>(w->k) * MB;
    // every workgroup quantizes the whole activation row, so fewer, longer-lived workgroups win: one
    // per CU measured faster than two on every decode shape (11008 x 4096 Q4K: 7.0 us against 7.6 us)
    const int64_t max_wgs = num_cus();
    int depth = UPL <= 2 ? 2 : 1;
    if (n < NW * 2) depth = 1;
    if (n < NW) {  // fewer rows than one workgroup's waves: the two-launch path handles it
        return hipErrorInvalidConfiguration;
    }
    int64_t wgs = n / (NW * depth);
    if (wgs > max_wgs) wgs = max_wgs;
    const int64_t tw = wgs * NW, rpw = n / tw, extra = n % tw;
    // weights with an offset term (Q4_1 / Q5_1 in Q8_0 planes, Q2K in Q6K planes) take the instances that add it
    constexpr bool kCanOffset = PRE == CQ_PRE_NONE && NWT == 1 && (DT == CQ_DTYPE_Q8_0 || DT == CQ_DTYPE_Q6K);
    const bool offsets = w->ggml_dtype != w->dtype && (cq_has_min32(w->ggml_dtype) || cq_has_min16(w->ggml_dtype));
    if (offsets && !kCanOffset) return hipErrorInvalidValue;
    if constexpr (UPL <= 2) {   // (longer rows never run two deep: no instance of that)
        if (depth == 2) {
            if constexpr (kCanOffset) {
                if (offsets) {
                    CQ_LAUNCH((fused_kernel<DT, UPL, NW, 2, PRE, NWT, MB, true>), (unsigned)wgs, NW * 64, lds, s, *w, x, pre, y, tw, rpw, extra, more);
                    return hipGetLastError();
                }
            }
            CQ_LAUNCH((fused_kernel<DT, UPL, NW, 2, PRE, NWT, MB>), (unsigned)wgs, NW * 64, lds, s, *w, x, pre, y, tw, rpw, extra, more);
            return hipGetLastError();
        }
    }
    if constexpr (kCanOffset) {
        if (offsets) {
            CQ_LAUNCH((fused_kernel<DT, UPL, NW, 1, PRE, NWT, MB, true>), (unsigned)wgs, NW * 64, lds, s, *w, x, pre, y, tw, rpw, extra, more);
            return hipGetLastError();
        }
    }
    CQ_LAUNCH((fused_kernel<DT, UPL, NW, 1, PRE, NWT, MB>), (unsigned)wgs, NW * 64, lds, s, *w, x, pre, y, tw, rpw, extra, more);
    return hipGetLastError();
}
template <int DT, int UPL, int PRE>
hipError_t launch_fused_upl(const cq_weight *w, const float *x, cq_pre pre, float *y, hipStream_t s) {
    return launch_fused_upl<DT, UPL, PRE, 1>(w, w->n, FusedMore<1>{}, x, pre, y, s);
}

template <int DT>
bool fused_ok(const cq_weight *w) {
    // Every workgroup re-quantizes the whole activation row in its prologue, which pays off against a
    // separate quantizer launch up to the row lengths measured (K = 11008: 12.0 us against 11.6 + 3.1 us).
    // The launcher instantiates up to eight units per lane (512 units per row).
    return w->k <= 16384 && w->k / Geo<DT>::kElems <= 512 && w->n >= 8 && lds_row_bytes<DT>(w->k) <= 64 * 1024 - 1024;
}

template <int DT, int PRE>
hipError_t launch_fused_pre(const cq_weight *w, const float *x, cq_pre pre, float *y, hipStream_t s) {
    const int64_t units = w->k / Geo<DT>::kElems;
    const int upl = (int)((units + 63) / 64);
    if (upl <= 1) return launch_fused_upl<DT, 1, PRE>(w, x, pre, y, s);
    if (upl <= 2) return launch_fused_upl<DT, 2, PRE>(w, x, pre, y, s);
    if (upl <= 3) return launch_fused_upl<DT, 3, PRE>(w, x, pre, y, s);
    if (upl <= 4) return launch_fused_upl<DT, 4, PRE>(w, x, pre, y, s);
    if (upl <= 6) return launch_fused_upl<DT, 6, PRE>(w, x, pre, y, s);
    return launch_fused_upl<DT, 8, PRE>(w, x, pre, y, s);
}

template <int DT>
hipError_t launch_fused(const cq_weight *w, const float *x, cq_pre pre, float *y, hipStream_t s) {
    switch (pre.kind) {
    case CQ_PRE_NONE: return launch_fused_pre<DT, CQ_PRE_NONE>(w, x, pre, y, s);
    case CQ_PRE_RMS_NORM: return launch_fused_pre<DT, CQ_PRE_RMS_NORM>(w, x, pre, y, s);
    case CQ_PRE_SILU_MUL: return launch_fused_pre<DT, CQ_PRE_SILU_MUL>(w, x, pre, y, s);
    default: return hipErrorInvalidValue;
    }
}

int pick_rows_per_wg(int64_t n) {
    int r = 16;
    while (r > 4 && (n + r - 1) / r < 2048) r >>= 1;
    return r;
}

template <int DT, int UPL, int MB>
hipError_t launch_batched_upl(const cq_weight *w, cq_act_view a, int64_t m0, int64_t m, float *y, hipStream_t s) {
    constexpr int NW = 8;
    const size_t lds = lds_row_bytes<DT>(w->k) * MB;
    if (hipError_t e = cq_ensure_lds<batched_kernel<DT, UPL, NW, MB>>(w->dev, lds); e != hipSuccess) return e;
    int64_t wgs = w->n / NW;
    if (wgs > num_cus()) wgs = num_cus();
    const int64_t tw = wgs * NW, rpw = w->n / tw, extra = w->n % tw;
    CQ_LAUNCH((batched_kernel<DT, UPL, NW, MB>), (unsigned)wgs, NW * 64, lds, s, *w, a, m0, m, y, tw, rpw, extra);
    return hipGetLastError();
}

template <int DT, int MB>
hipError_t launch_batched(const cq_weight *w, cq_act_view a, int64_t m0, int64_t m, float *y, hipStream_t s) {
    const int64_t units = w->k / Geo<DT>::kElems;
    const int upl = (int)((units + 63) / 64);
    if (upl <= 1) return launch_batched_upl<DT, 1, MB>(w, a, m0, m, y, s);
    if (upl <= 2) return launch_batched_upl<DT, 2, MB>(w, a, m0, m, y, s);
    if (upl <= 3) return launch_batched_upl<DT, 3, MB>(w, a, m0, m, y, s);
    if (upl <= 4) return launch_batched_upl<DT, 4, MB>(w, a, m0, m, y, s);
    if (upl <= 6) return launch_batched_upl<DT, 6, MB>(w, a, m0, m, y, s);
    return launch_batched_upl<DT, 8, MB>(w, a, m0, m, y, s);
}

// Rows of eight (or four) per launch on the persistent kernel when the row fits its unit and LDS
// budget, else the simple kernel below.
template <int DT>
bool batched_ok(const cq_weight *w, int mb) {
    return w->k / Geo<DT>::kElems <= 512 && w->n >= 8 && lds_row_bytes<DT>(w->k) * mb <= 128 * 1024;
}

template <int DT>
hipError_t launch_chunked(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    const int rpw = pick_rows_per_wg(w->n);   // at most 16: four rows per wave
    const unsigned grid = (unsigned)((w->n + rpw - 1) / rpw);
    const int64_t kc = w->k < kChunkElems ? w->k : kChunkElems;
    int64_t m0 = 0;
    while (m0 < m) {
        const int64_t left = m - m0;
        const int mb = left >= 4 ? 4 : (left >= 2 ? 2 : 1);
        const size_t lds = lds_row_bytes<DT>(kc) * mb;
        if (mb == 4) {
            if (hipError_t e = cq_ensure_lds<chunked_kernel<DT, 4>>(w->dev, lds); e != hipSuccess) return e;
            CQ_LAUNCH((chunked_kernel<DT, 4>), grid, kStagedThreads, lds, s, *w, a, m0, rpw, y);
        } else if (mb == 2) {
            if (hipError_t e = cq_ensure_lds<chunked_kernel<DT, 2>>(w->dev, lds); e != hipSuccess) return e;
            CQ_LAUNCH((chunked_kernel<DT, 2>), grid, kStagedThreads, lds, s, *w, a, m0, rpw, y);
        } else {
            if (hipError_t e = cq_ensure_lds<chunked_kernel<DT, 1>>(w->dev, lds); e != hipSuccess) return e;
            CQ_LAUNCH((chunked_kernel<DT, 1>), grid, kStagedThreads, lds, s, *w, a, m0, rpw, y);
        }
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
        m0 += mb;
    }
    return hipSuccess;
}

template <int DT>
hipError_t launch_staged(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    // rows whose quantized image does not fit the LDS: walked in chunks
    if (lds_row_bytes<DT>(w->k) > kMaxRowLds) return launch_chunked<DT>(w, a, m, y, s);
    if (m >= 2) {
        int64_t m0 = 0;
        bool done = true;
        while (m0 < m) {
            const int64_t left = m - m0;
            hipError_t e;
            if (left > 4 && batched_ok<DT>(w, 8)) e = launch_batched<DT, 8>(w, a, m0, m, y, s), m0 += 8;
            else if (batched_ok<DT>(w, 4)) e = launch_batched<DT, 4>(w, a, m0, m, y, s), m0 += 4;
            else { done = false; break; }
            if (e != hipSuccess) return e;
        }
        if (done) return hipSuccess;
        if (m0 != 0) return hipErrorInvalidValue;   // unreachable: the checks above do not depend on m0
    }
    const int rpw = pick_rows_per_wg(w->n);
    const unsigned grid = (unsigned)((w->n + rpw - 1) / rpw);
    int64_t m0 = 0;
    while (m0 < m) {
        const int64_t left = m - m0;
        int mb = left >= 4 ? 4 : (left >= 2 ? 2 : 1);
        while (mb > 1 && lds_row_bytes<DT>(w->k) * mb > 64 * 1024) mb >>= 1;
        const size_t lds = lds_row_bytes<DT>(w->k) * mb;
        if (lds > kMaxRowLds) return hipErrorInvalidValue;   // (cq_matvec_row_fits tells beforehand)
        if (mb == 4) {
            if (hipError_t e = cq_ensure_lds<staged_kernel<DT, 4>>(w->dev, lds); e != hipSuccess) return e;
            CQ_LAUNCH((staged_kernel<DT, 4>), grid, kStagedThreads, lds, s, *w, a, m0, rpw, y);
        } else if (mb == 2) {
            if (hipError_t e = cq_ensure_lds<staged_kernel<DT, 2>>(w->dev, lds); e != hipSuccess) return e;
            CQ_LAUNCH((staged_kernel<DT, 2>), grid, kStagedThreads, lds, s, *w, a, m0, rpw, y);
        } else {
            if (hipError_t e = cq_ensure_lds<staged_kernel<DT, 1>>(w->dev, lds); e != hipSuccess) return e;
            CQ_LAUNCH((staged_kernel<DT, 1>), grid, kStagedThreads, lds, s, *w, a, m0, rpw, y);
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        m0 += mb;
    }
    return hipSuccess;
}

template <int DT>
hipError_t launch_ints(const cq_weight *w, cq_act_view a, int64_t m, int32_t *oi, int32_t *omn, hipStream_t s) {
    const size_t lds = lds_row_bytes<DT>(w->k);
    if (lds > kMaxRowLds) return hipErrorInvalidValue;
    if (hipError_t e = cq_ensure_lds<int_dots_kernel<DT>>(w->dev, lds); e != hipSuccess) return e;
    const int rpw = 8;
    const unsigned grid = (unsigned)((w->n + rpw - 1) / rpw);
    for (int64_t m0 = 0; m0 < m; m0++) {
        int_dots_kernel<DT><<<grid, kStagedThreads, lds, s>>>(*w, a, m0, rpw, oi, omn);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// Two to four activation rows in the one-launch kernel (rows of at most 256 units; 384 for two rows).
template <int DT, int MB>
hipError_t launch_fused_rows_mb(const cq_weight *w, const float *x, float *y, hipStream_t s) {
    const int upl = (int)((w->k / Geo<DT>::kElems + 63) / 64);
    if (upl <= 1) return launch_fused_upl<DT, 1, CQ_PRE_NONE, 1, MB>(w, w->n, FusedMore<1>{}, x, cq_no_pre(), y, s);
    if (upl <= 2) return launch_fused_upl<DT, 2, CQ_PRE_NONE, 1, MB>(w, w->n, FusedMore<1>{}, x, cq_no_pre(), y, s);
    if (upl <= 3) return launch_fused_upl<DT, 3, CQ_PRE_NONE, 1, MB>(w, w->n, FusedMore<1>{}, x, cq_no_pre(), y, s);
    if (upl <= 4) return launch_fused_upl<DT, 4, CQ_PRE_NONE, 1, MB>(w, w->n, FusedMore<1>{}, x, cq_no_pre(), y, s);
    if constexpr (MB == 2) return launch_fused_upl<DT, 6, CQ_PRE_NONE, 1, MB>(w, w->n, FusedMore<1>{}, x, cq_no_pre(), y, s);
    return hipErrorInvalidConfiguration;
}
template <int DT>
hipError_t launch_fused_rows(const cq_weight *w, const float *x, int64_t m, float *y, hipStream_t s) {
    if (m == 2) return launch_fused_rows_mb<DT, 2>(w, x, y, s);
    if (m == 3) return launch_fused_rows_mb<DT, 3>(w, x, y, s);
    return launch_fused_rows_mb<DT, 4>(w, x, y, s);
}

// Two or three weights on the same activations (same type, row length and device; rows of at most 256
// units): one launch over all their rows.
constexpr int kMultiMax = 3;
template <int DT, int PRE, int MB = 1>
hipError_t launch_fused_multi_pre(const cq_weight *const *ws, int count, const float *x, cq_pre pre, float *const *ys,
                                  hipStream_t s) {
    FusedMore<kMultiMax> more;
    int64_t n = ws[0]->n;
    for (int t = 0; t < kMultiMax - 1; t++) {
        const int j = t + 1 < count ? t + 1 : count - 1;   // unused slots repeat the last weight with no rows
        more.p[t][0] = ws[j]->p0; more.p[t][1] = ws[j]->p1; more.p[t][2] = ws[j]->p2; more.p[t][3] = ws[j]->p3;
        more.y[t] = ys[j];
        more.n[t] = ws[j]->n;
        more.first[t] = n;
        if (t + 1 < count) n += ws[j]->n;
    }
    // (a slot that repeats the last weight starts at the end of the launch: no row reaches it)
    const cq_weight *w = ws[0];
    const int upl = (int)((w->k / Geo<DT>::kElems + 63) / 64);
    if (upl <= 1) return launch_fused_upl<DT, 1, PRE, kMultiMax, MB>(w, n, more, x, pre, ys[0], s);
    if (upl <= 2) return launch_fused_upl<DT, 2, PRE, kMultiMax, MB>(w, n, more, x, pre, ys[0], s);
    if (upl <= 3) return launch_fused_upl<DT, 3, PRE, kMultiMax, MB>(w, n, more, x, pre, ys[0], s);
    return launch_fused_upl<DT, 4, PRE, kMultiMax, MB>(w, n, more, x, pre, ys[0], s);
}
template <int DT>
hipError_t launch_fused_multi(const cq_weight *const *ws, int count, const float *x, cq_pre pre, int64_t m,
                              float *const *ys, hipStream_t s) {
    if (m == 2) return launch_fused_multi_pre<DT, CQ_PRE_NONE, 2>(ws, count, x, pre, ys, s);
    if (m == 3) return launch_fused_multi_pre<DT, CQ_PRE_NONE, 3>(ws, count, x, pre, ys, s);
    if (m == 4) return launch_fused_multi_pre<DT, CQ_PRE_NONE, 4>(ws, count, x, pre, ys, s);
    switch (pre.kind) {
    case CQ_PRE_NONE: return launch_fused_multi_pre<DT, CQ_PRE_NONE>(ws, count, x, pre, ys, s);
    case CQ_PRE_RMS_NORM: return launch_fused_multi_pre<DT, CQ_PRE_RMS_NORM>(ws, count, x, pre, ys, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

// Measured against the quantizer launch + split-K MFMA kernel (us per call, 2 / 3 / 4 rows): Q4K 4096 x 4096
// 5.0 / 6.2 / 7.2 against 8.9; 11008 x 4096 8.4 / 10.1 / 11.7 against 13.5; Q8_0 4096 x 4096 6.8 / 7.7 / 8.9
// against 10.5.  Every further row costs the dot products of one more row per unpacked unit, so the longer
// the rows (elements per lane), the fewer rows pay off: K = 8192 Q4K 8.7 / 10.5 / 13.9 against 12.5,
// K = 14336 Q4K 13.8 / 43 (registers spill) against 17.6.
bool cq_matvec_fused_rows_supported(const cq_weight *w, int64_t m) {
    if (m < 2 || m > 4 || !cq_matvec_fused_supported(w)) return false;
    int64_t units = 0, elems = 0;
    size_t row_bytes = 0;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: elems = Geo<CQ_DTYPE_Q4_0>::kElems; row_bytes = lds_row_bytes<CQ_DTYPE_Q4_0>(w->k); break;
    case CQ_DTYPE_Q8_0: elems = Geo<CQ_DTYPE_Q8_0>::kElems; row_bytes = lds_row_bytes<CQ_DTYPE_Q8_0>(w->k); break;
    case CQ_DTYPE_Q4K: elems = Geo<CQ_DTYPE_Q4K>::kElems; row_bytes = lds_row_bytes<CQ_DTYPE_Q4K>(w->k); break;
    case CQ_DTYPE_Q5K: elems = Geo<CQ_DTYPE_Q5K>::kElems; row_bytes = lds_row_bytes<CQ_DTYPE_Q5K>(w->k); break;
    case CQ_DTYPE_Q6K: elems = Geo<CQ_DTYPE_Q6K>::kElems; row_bytes = lds_row_bytes<CQ_DTYPE_Q6K>(w->k); break;
    default: return false;
    }
    units = w->k / elems;
    if (units > (m == 2 ? 384 : 256) || row_bytes * (size_t)m > 64 * 1024 - 1024) return false;
    const int64_t per_lane = (units + 63) / 64 * elems;   // elements of a row per lane
    return per_lane <= 64 ? true : per_lane <= 128 ? m <= 3 : m <= 2;
}

hipError_t cq_launch_matvec_fused_rows(const cq_weight *w, const float *x, int64_t m, float *y, hipStream_t s) {
    if (w->n == 0) return hipSuccess;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: return launch_fused_rows<CQ_DTYPE_Q4_0>(w, x, m, y, s);
    case CQ_DTYPE_Q8_0: return launch_fused_rows<CQ_DTYPE_Q8_0>(w, x, m, y, s);
    case CQ_DTYPE_Q4K: return launch_fused_rows<CQ_DTYPE_Q4K>(w, x, m, y, s);
    case CQ_DTYPE_Q5K: return launch_fused_rows<CQ_DTYPE_Q5K>(w, x, m, y, s);
    case CQ_DTYPE_Q6K: return launch_fused_rows<CQ_DTYPE_Q6K>(w, x, m, y, s);
    default: return hipErrorInvalidValue;
    }
}

bool cq_matvec_fused_multi_supported(const cq_weight *const *ws, int count, int pre_kind, int64_t m) {
    if (count < 2 || count > kMultiMax || (pre_kind != CQ_PRE_NONE && pre_kind != CQ_PRE_RMS_NORM)) return false;
    if (m != 1 && (pre_kind != CQ_PRE_NONE || !cq_matvec_fused_rows_supported(ws[0], m))) return false;
    for (int i = 0; i < count; i++) {
        if (ws[i]->dtype != ws[0]->dtype || ws[i]->k != ws[0]->k || ws[i]->dev != ws[0]->dev || ws[i]->n == 0) return false;
        if (!cq_matvec_fused_supported(ws[i])) return false;
    }
    int64_t units = 0;
    switch (ws[0]->dtype) {
    case CQ_DTYPE_Q4_0: units = ws[0]->k / Geo<CQ_DTYPE_Q4_0>::kElems; break;
    case CQ_DTYPE_Q8_0: units = ws[0]->k / Geo<CQ_DTYPE_Q8_0>::kElems; break;
    case CQ_DTYPE_Q4K: units = ws[0]->k / Geo<CQ_DTYPE_Q4K>::kElems; break;
    case CQ_DTYPE_Q5K: units = ws[0]->k / Geo<CQ_DTYPE_Q5K>::kElems; break;
    case CQ_DTYPE_Q6K: units = ws[0]->k / Geo<CQ_DTYPE_Q6K>::kElems; break;
    default: return false;
    }
    return units <= 256;
}

hipError_t cq_launch_matvec_fused_multi(const cq_weight *const *ws, int count, const float *x, cq_pre pre, int64_t m,
                                        float *const *ys, hipStream_t s) {
    switch (ws[0]->dtype) {
    case CQ_DTYPE_Q4_0: return launch_fused_multi<CQ_DTYPE_Q4_0>(ws, count, x, pre, m, ys, s);
    case CQ_DTYPE_Q8_0: return launch_fused_multi<CQ_DTYPE_Q8_0>(ws, count, x, pre, m, ys, s);
    case CQ_DTYPE_Q4K: return launch_fused_multi<CQ_DTYPE_Q4K>(ws, count, x, pre, m, ys, s);
    case CQ_DTYPE_Q5K: return launch_fused_multi<CQ_DTYPE_Q5K>(ws, count, x, pre, m, ys, s);
    case CQ_DTYPE_Q6K: return launch_fused_multi<CQ_DTYPE_Q6K>(ws, count, x, pre, m, ys, s);
    default: return hipErrorInvalidValue;
    }
}

// Whether one quantized activation row of this weight's K fits the LDS of a workgroup, which every
// dot-product kernel needs (K up to about 150 000 for the K-quants, 139 000 for Q8_0 / Q4_0).
bool cq_matvec_row_fits(const cq_weight *w) {
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: return lds_row_bytes<CQ_DTYPE_Q4_0>(w->k) <= kMaxRowLds;
    case CQ_DTYPE_Q8_0: return lds_row_bytes<CQ_DTYPE_Q8_0>(w->k) <= kMaxRowLds;
    case CQ_DTYPE_Q4K: return lds_row_bytes<CQ_DTYPE_Q4K>(w->k) <= kMaxRowLds;
    case CQ_DTYPE_Q5K: return lds_row_bytes<CQ_DTYPE_Q5K>(w->k) <= kMaxRowLds;
    case CQ_DTYPE_Q6K: return lds_row_bytes<CQ_DTYPE_Q6K>(w->k) <= kMaxRowLds;
    default: return false;
    }
}

bool cq_matvec_fused_supported(const cq_weight *w) {
    // Q4_1 / Q5_1: the kernels that add the offset term take a row's minima in whole groups of eight blocks
    if (cq_has_min32(w->ggml_dtype) && w->k % 256 != 0) return false;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: return fused_ok<CQ_DTYPE_Q4_0>(w);
    case CQ_DTYPE_Q8_0: return fused_ok<CQ_DTYPE_Q8_0>(w);
    case CQ_DTYPE_Q4K: return fused_ok<CQ_DTYPE_Q4K>(w);
    case CQ_DTYPE_Q5K: return fused_ok<CQ_DTYPE_Q5K>(w);
    case CQ_DTYPE_Q6K: return fused_ok<CQ_DTYPE_Q6K>(w);
    default: return false;
    }
}

hipError_t cq_launch_matvec_fused(const cq_weight *w, const float *x, cq_pre pre, float *y, hipStream_t s) {
    if (w->n == 0) return hipSuccess;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: return launch_fused<CQ_DTYPE_Q4_0>(w, x, pre, y, s);
    case CQ_DTYPE_Q8_0: return launch_fused<CQ_DTYPE_Q8_0>(w, x, pre, y, s);
    case CQ_DTYPE_Q4K: return launch_fused<CQ_DTYPE_Q4K>(w, x, pre, y, s);
    case CQ_DTYPE_Q5K: return launch_fused<CQ_DTYPE_Q5K>(w, x, pre, y, s);
    case CQ_DTYPE_Q6K: return launch_fused<CQ_DTYPE_Q6K>(w, x, pre, y, s);
    default: return hipErrorInvalidValue;
    }
}

hipError_t cq_launch_matvec(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, hipStream_t s) {
    (void)act_dtype;
    if (m == 0 || w->n == 0) return hipSuccess;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: return launch_staged<CQ_DTYPE_Q4_0>(w, a, m, y, s);
    case CQ_DTYPE_Q8_0: return launch_staged<CQ_DTYPE_Q8_0>(w, a, m, y, s);
    case CQ_DTYPE_Q4K: return launch_staged<CQ_DTYPE_Q4K>(w, a, m, y, s);
    case CQ_DTYPE_Q5K: return launch_staged<CQ_DTYPE_Q5K>(w, a, m, y, s);
    case CQ_DTYPE_Q6K: return launch_staged<CQ_DTYPE_Q6K>(w, a, m, y, s);
    default: return hipErrorInvalidValue;
    }
}

namespace {
template <int DT, int MB>
hipError_t launch_q81_mb(const cq_weight *w, cq_act_view a, int64_t m0, int64_t m, float *y, hipStream_t s) {
    const size_t lds = q81_row_bytes<DT>(w->k) * MB;
    if (hipError_t e = cq_ensure_lds<q81_kernel<DT, MB>>(w->dev, lds); e != hipSuccess) return e;
    const int rpw = pick_rows_per_wg(w->n);
    const unsigned grid = (unsigned)((w->n + rpw - 1) / rpw);
    CQ_LAUNCH((q81_kernel<DT, MB>), grid, kStagedThreads, lds, s, *w, a, m0, m, rpw, y);
    return hipGetLastError();
}
template <int DT> hipError_t launch_q81(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    // eight activation rows per pass over the weights when their images fit the LDS, else four, two, one
    int mb = 8;
    while (mb > 1 && q81_row_bytes<DT>(w->k) * mb > kMaxRowLds) mb >>= 1;
    if (q81_row_bytes<DT>(w->k) > kMaxRowLds) return hipErrorInvalidValue;
    for (int64_t m0 = 0; m0 < m; m0 += mb) {
        const int64_t left = m - m0;
        hipError_t e;
        if (mb == 8 && left > 4) e = launch_q81_mb<DT, 8>(w, a, m0, m, y, s);
        else if (mb >= 4 && left > 2) e = launch_q81_mb<DT, 4>(w, a, m0, m, y, s);
        else if (mb >= 2 && left > 1) e = launch_q81_mb<DT, 2>(w, a, m0, m, y, s);
        else e = launch_q81_mb<DT, 1>(w, a, m0, m, y, s);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}
}  // namespace

bool cq_matmul_q8_1_supported(const cq_weight *w) {
    if (w->dtype == CQ_DTYPE_Q4K) return q81_row_bytes<CQ_DTYPE_Q4K>(w->k) <= kMaxRowLds;
    if (w->dtype == CQ_DTYPE_Q6K) return q81_row_bytes<CQ_DTYPE_Q6K>(w->k) <= kMaxRowLds;
    return false;
}

hipError_t cq_launch_matmul_q8_1(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    if (m == 0 || w->n == 0) return hipSuccess;
    if (w->dtype == CQ_DTYPE_Q4K) return launch_q81<CQ_DTYPE_Q4K>(w, a, m, y, s);
    if (w->dtype == CQ_DTYPE_Q6K) return launch_q81<CQ_DTYPE_Q6K>(w, a, m, y, s);
    return hipErrorInvalidValue;
}

hipError_t cq_launch_int_dots(const cq_weight *w, cq_act_view a, int64_t m, int32_t *out_i, int32_t *out_mn,
                              hipStream_t s) {
    if (m == 0 || w->n == 0) return hipSuccess;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: return launch_ints<CQ_DTYPE_Q4_0>(w, a, m, out_i, out_mn, s);
    case CQ_DTYPE_Q8_0: return launch_ints<CQ_DTYPE_Q8_0>(w, a, m, out_i, out_mn, s);
    case CQ_DTYPE_Q4K: return launch_ints<CQ_DTYPE_Q4K>(w, a, m, out_i, out_mn, s);
    case CQ_DTYPE_Q5K: return launch_ints<CQ_DTYPE_Q5K>(w, a, m, out_i, out_mn, s);
    case CQ_DTYPE_Q6K: return launch_ints<CQ_DTYPE_Q6K>(w, a, m, out_i, out_mn, s);
    default: return hipErrorInvalidValue;
    }
}
