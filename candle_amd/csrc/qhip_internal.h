// Internal declarations shared by the HIP sources of libcandle_qhip.
// Device layouts here are private to the library (see include/candle_qhip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/candle_qhip.h"

#define QK_K 256

// ---------------------------------------------------------------------------
// Device weight storage: GGML blocks split into planes so that every wave-wide
// load is a run of 16-byte lanes over whole 128-byte lines.
//
//   Q4_0 : qs [n][k/32][16]  u8   (nibbles, element j low / j+16 high)
//          d  [n][k/32]      f16
//   Q8_0 : qs [n][k/32][32]  i8
//          d  [n][k/32]      f16
//   Q4K  : qs [n][k/256][128] u8  (GGML order: byte 32g+l = elem 64g+l | elem 64g+32+l << 4)
//          hd [n][k/256][20]      (d f16, dmin f16, then four records {sc[2g], sc[2g+1], mn[2g], mn[2g+1]}:
//                                  the 6-bit scales and mins of the GGML scales[12] unpacked to bytes,
//                                  grouped by the 32 qs bytes g they belong to)
//   Q5K  : qs and hd as Q4K (the low four bits of every quant)
//          qh [n][k/256][32]  u8  (re-ordered, see repack.hip: per 32 qs bytes g two words {L, H} with the
//                                  fifth bits of their low-nibble and high-nibble elements, bit 8c+i of a
//                                  word belonging to byte c of qs word i)
//   Q6K  : ql [n][k/256][128] u8  (GGML order)
//          qh [n][k/256][64]  u8  (re-ordered, see repack.hip: 8 bytes per 16-byte ql lane)
//          sc [n][k/256][16]  i8  (re-ordered: two scales per 16-byte ql lane, see repack.hip)
//          d  [n][k/256]      f16
// All planes live in one allocation; each plane starts 256-byte aligned and the
// allocation carries CQ_TAIL_PAD spare bytes so that a partial tail tile can be
// read with full-width loads.
// ---------------------------------------------------------------------------
#define CQ_TAIL_PAD 4096
#define CQ_Q4K_HDR 20   // bytes per block in the Q4K header plane

struct cq_weight {
    int dev;
    int dtype;           // the type whose planes hold the blocks: what every kernel dispatches on
    int ggml_dtype;      // the type the caller sees; differs from dtype for Q5_0, Q4_1, Q5_1 (held as Q8_0), Q3K and Q2K (as Q6K)
    int64_t n, k;
    size_t ggml_bytes;   // n * k/block * type_size of ggml_dtype
    void *base;          // the single device allocation
    size_t alloc_bytes;
    uint8_t *p0;         // qs / ql
    uint8_t *p1;         // d (Q4_0,Q8_0) / hd (Q4K) / qh (Q6K)
    uint8_t *p2;         // sc (Q6K) / qh (Q5K) / m (Q4_1, Q5_1: f16 block minima beside the Q8_0 planes)
    uint8_t *p3;         // d  (Q6K)
    uint8_t *p4;         // Q2K (held as Q6K): the sixteen group minima of a block, one byte each
    uint8_t *p5;         // Q2K: dmin (f16)
};

// ---------------------------------------------------------------------------
// Device activation storage used between the quantizer and the matmul kernels
// (workspace layout).  Same numbers as the GGML activation blocks, split so
// that int8 values are 16-byte aligned:
//   Q8K : qs [m_stride][k] i8 ; d [m][k/256] f32 ; bsums [m][k/256][16] i16
//   Q8_0: qs [m][k] i8 ; d [m][k/32]  f32 (the f16-rounded scale widened) ;
//         bsum [m][k/32] i32 (sum of the 32 quants, for the Q4_0 "-8" term)
// ---------------------------------------------------------------------------
struct cq_act_view {
    int8_t *qs;
    float *d;
    int16_t *bsums;  // Q8K
    // Q8K, for the matrix-core kernels (block-major so that a tile of rows is contiguous per block):
    float *dT;         // [k/256][m_stride] f32, the same values as d
    uint16_t *bsh;     // [k/256][m_stride][16] f16: the block's sixteen bsums as f16 (exact), the min term's operand
    int64_t m_stride;  // rows allocated: at least 256 more than the rows quantized, so that the GEMM
                       // may read (and ignore) whole 128-row tiles past the last row
    int32_t *bsum32; // Q8_0 / Q8_1
    uint16_t *s16;   // Q8_1: the block's `s` field (f16 bits)
};

static inline size_t cq_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// error plumbing (api.cpp)
int cq_set_error(int code, const char *fmt, ...);
#define CQ_HIP_CHECK(expr)                                                                       \
    do {                                                                                         \
        hipError_t _e = (expr);                                                                  \
        if (_e != hipSuccess)                                                                    \
            return cq_set_error(CQ_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                                __FILE__, __LINE__);                                             \
    } while (0)

// CQ_FLAG_DETERMINISTIC (api.hip): true while the calling thread runs a call with the flag; the tile kernels' launchers
// then never split K (no partial sums added atomically in arrival order).
bool cq_no_split_k();

// Kernel timing hook (api.hip): true when the calling thread armed the timer; the launch then goes
// through CQ_LAUNCH below with the two events.  Disarms.
bool cq_timing_take(hipEvent_t *start, hipEvent_t *stop);

// ---- launchers implemented in the .hip files -------------------------------
// repack.hip
hipError_t cq_launch_repack(const cq_weight *w, const uint8_t *aos_dev, hipStream_t s);   // GGML AoS -> planes
hipError_t cq_launch_unpack(const cq_weight *w, uint8_t *aos_dev, hipStream_t s);         // planes -> GGML AoS
// Types held in another type's planes (same values, same arithmetic): Q5_0 as Q8_0, Q3K as Q6K.
// Q4_1 and Q5_1 (value d * q + m) are Q8_0 planes with qs = q plus the plane p2 of the blocks' minima m (f16): the
// holding type's kernels give the sum_i * d * d8 part of their dot product, cq_launch_min32_term adds sum_b m_b * s8_b.
__host__ __device__ inline bool cq_has_min32(int ggml_dtype) { return ggml_dtype == CQ_DTYPE_Q4_1 || ggml_dtype == CQ_DTYPE_Q5_1; }
// Q2K (value d * sc_j * q - dmin * m_j, sixteen groups of sixteen) is a Q6K block with scales sc_j and six-bit quants
// q + 32, plus the planes p4 / p5 of the groups' minima and dmin: the Q6K kernels give sum_b d * d8 * I_b of its dot
// product with Q8K activations, cq_launch_min16_term subtracts sum_b dmin * d8 * sum_j bsums_j * m_j.
__host__ __device__ inline bool cq_has_min16(int ggml_dtype) { return ggml_dtype == CQ_DTYPE_Q2K; }
inline int cq_storage_dtype(int ggml_dtype) {
    if (ggml_dtype == CQ_DTYPE_Q5_0 || cq_has_min32(ggml_dtype)) return CQ_DTYPE_Q8_0;
    return ggml_dtype == CQ_DTYPE_Q3K || ggml_dtype == CQ_DTYPE_Q2K ? CQ_DTYPE_Q6K : ggml_dtype;
}
// `w` supplies the planes beside the holding type's blocks: the minima of Q4_1 / Q5_1 (p2), of Q2K (p4, p5)
hipError_t cq_launch_transcode(const cq_weight *w, uint8_t *ggml_aos_dev, uint8_t *storage_aos_dev, int64_t nblocks, bool inverse,
                               hipStream_t s);
// y[r, c] -= sum_b (d8[r, b] * dmin[c, b]) * sum_j bsums[r, b, j] * m[c, b, j] for Q2K weights (k_quants.rs:727-733, :762)
hipError_t cq_launch_min16_term(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s);
// Q8K as a weight type (q8k_weight.hip): planes p0 qs, p1 d (f32), p2 bsums
hipError_t cq_launch_repack_q8k(const cq_weight *w, uint8_t *aos, bool inverse, hipStream_t s);
hipError_t cq_launch_dequantize_q8k(const cq_weight *w, float *d32, uint16_t *d16, hipStream_t s);
hipError_t cq_launch_q8k_weight_matmul(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s);
// y[r, c] += sum_b m[c, b] * s8[r, b] for Q4_1 / Q5_1 weights, s8 the `s` field of the activation's Q8_1 block
// (k_quants.rs:665-691) recomputed from the workspace's block sums and scales.
hipError_t cq_launch_min32_term(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s);
// A step of the caller's model computed on the way into the activation quantizer (CQ_PRE_*):
// rms_norm: x / sqrt(mean(x^2) + eps) * aux[k]; silu_mul: silu(x) * aux[m][k] (aux indexed like x).
struct cq_pre {
    int kind;
    const float *aux;
    float eps;
};
static inline cq_pre cq_no_pre() { return cq_pre{CQ_PRE_NONE, nullptr, 0.0f}; }
// Floats the activation quantizer sets to zero on its way: the output of a matmul that splits K and adds
// its partial sums atomically (the launch it saves costs as much as the clearing).  p == nullptr: nothing.
struct cq_clear {
    float *p;
    int64_t count;
};
static inline cq_clear cq_no_clear() { return cq_clear{nullptr, 0}; }

// quantize_act.hip
hipError_t cq_launch_quantize_act_aos(int act_dtype, const float *x, int64_t m, int64_t k, cq_pre pre, void *dst,
                                      hipStream_t s);
hipError_t cq_launch_quantize_act_ws(int act_dtype, const float *x, const int32_t *row_ids, int64_t m, int64_t k,
                                     cq_pre pre, cq_act_view v, cq_clear clear, hipStream_t s);
// quantize_weight.hip
hipError_t cq_launch_quantize_weight(int dtype, const float *src, int64_t nblocks, uint8_t *aos_dev, hipStream_t s);
// dequantize.hip
hipError_t cq_launch_dequantize(const cq_weight *w, float *dst32, uint16_t *dst16, hipStream_t s);
// matvec.hip
hipError_t cq_launch_matvec(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, hipStream_t s);
hipError_t cq_launch_int_dots(const cq_weight *w, cq_act_view a, int64_t m, int32_t *out_i, int32_t *out_mn,
                              hipStream_t s);
bool cq_matvec_row_fits(const cq_weight *w);          // K small enough for the dot-product kernels (one quantized row in LDS)
// Q4K / Q6K weights with Q8_1 activations (the reference's CUDA formulation), any number of rows
bool cq_matmul_q8_1_supported(const cq_weight *w);
hipError_t cq_launch_matmul_q8_1(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s);
// the same on the matrix cores, for more than 32 rows (gemm.hip)
bool cq_gemm_q81_supported(const cq_weight *w, int64_t m);
hipError_t cq_launch_gemm_q81(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s);
bool cq_matvec_fused_supported(const cq_weight *w);   // m == 1: quantizer fused into the matvec launch
hipError_t cq_launch_matvec_fused(const cq_weight *w, const float *x, cq_pre pre, float *y, hipStream_t s);
// 2 <= m <= 4 rows in the one-launch kernel (short rows only)
bool cq_matvec_fused_rows_supported(const cq_weight *w, int64_t m);
hipError_t cq_launch_matvec_fused_rows(const cq_weight *w, const float *x, int64_t m, float *y, hipStream_t s);
// several weights on the same activations in one launch (same dtype, k, device; 2 or 3 of them): one row, or
// as many rows as cq_matvec_fused_rows_supported allows (then without a fused step)
bool cq_matvec_fused_multi_supported(const cq_weight *const *ws, int count, int pre_kind, int64_t m);
hipError_t cq_launch_matvec_fused_multi(const cq_weight *const *ws, int count, const float *x, cq_pre pre, int64_t m,
                                        float *const *ys, hipStream_t s);
// Verification output of the MFMA kernels (gemm.hip, gemm_blk32.hip, skinny.hip): what the f32 result is combined
// from, per activation row r, weight row c and block b, at [(r*n + c)*blocks + b].
//   i  : the block's integer dot product, the number the dot-product kernels and the CPU form
//   mn : types with a min term (Q4K, Q5K; else null): -(dmin*d8) * sum_j min_j*bsum32_j as the f16 MFMA delivers
//        it from a zero accumulator - a float, the kernels never hold this term as an integer
struct cq_mfma_dump {
    int32_t *i;
    float *mn;
    int int_min;   // store the integer Mn_b = sum_j min_j * bsum32_j (exact in f32) instead of the float min term
};
hipError_t cq_launch_gemm_dump(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, cq_mfma_dump d, hipStream_t s);
hipError_t cq_launch_gemm32_dump(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, cq_mfma_dump d, hipStream_t s);
hipError_t cq_launch_skinny_dump(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, cq_mfma_dump d, hipStream_t s);
// gemm.hip
bool cq_gemm_supported(const cq_weight *w, int64_t m, int act_dtype);
// `y_cleared`: y is already zero (a launch that splits K otherwise clears it first); *_splits_k tell
// beforehand whether the launch will add its results atomically
hipError_t cq_launch_gemm(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, bool y_cleared,
                          hipStream_t s);
bool cq_gemm_splits_k(const cq_weight *w, int64_t m);
// all experts of a mixture-of-experts projection in one launch; `a` and `y` cover all routed rows
bool cq_gemm_grouped_supported(const cq_weight *const *experts, int n_experts, const int32_t *offsets, int act_dtype);
hipError_t cq_launch_gemm_grouped(const cq_weight *const *experts, int n_experts, const int32_t *offsets, cq_act_view a,
                                  float *y, bool y_cleared, hipStream_t s);
bool cq_gemm_grouped_splits_k(const cq_weight *const *experts, int n_experts, const int32_t *offsets);
// gemm_blk32.hip: the tile kernel for Q8_0 / Q4_0 weights with Q8_0 activations (K a multiple of 256)
bool cq_gemm32_supported(const cq_weight *w, int act_dtype);
hipError_t cq_launch_gemm32(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, bool y_cleared,
                            hipStream_t s);
bool cq_gemm32_splits_k(const cq_weight *w, int64_t m);
// skinny.hip: a few activation rows (32 per pass) on the int8 MFMA, K split over the waves of a workgroup
bool cq_skinny_supported(const cq_weight *w, int act_dtype);
hipError_t cq_launch_skinny(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, hipStream_t s);
// moe.hip
hipError_t cq_launch_silu_mul(const float *a, const float *b, float *h, int64_t count, hipStream_t s);
hipError_t cq_launch_scatter_add(const float *y, const int32_t *row_ids, const float *weights, int64_t total_rows,
                                 int64_t hidden, float *ys, int64_t tokens, hipStream_t s);

hipError_t cq_launch_fill_zero(float *p, int64_t count, hipStream_t s);

// no_alloc.hip: device address of the static scratch array of cq_qmatmul_static on `dev` (the current
// device); looked up once per device.  Weight creation calls it so that the first matmul on a device finds
// the address cached.
uint8_t *cq_static_scratch_ptr(int dev);

#if defined(__HIPCC__)
#include <hip/hip_ext.h>
#include <atomic>
// Kernel launch that honours the timing hook.  `kernel` in parentheses when it contains commas.
#define CQ_LAUNCH(kernel, grid, block, lds, stream, ...)                                                  \
    do {                                                                                                  \
        hipEvent_t _ea, _eb;                                                                              \
        if (cq_timing_take(&_ea, &_eb))                                                                   \
            hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), (uint32_t)(lds), stream, _ea, _eb, 0,  \
                                  __VA_ARGS__);                                                           \
        else                                                                                              \
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), (uint32_t)(lds), stream, __VA_ARGS__);    \
    } while (0)

// Raises the dynamic-LDS limit of `Kernel` on device `dev` when a launch needs more than the
// default 48 KiB; remembers, per kernel and device, the largest size already granted.
template <auto Kernel> hipError_t cq_ensure_lds(int dev, size_t lds) {
    constexpr int kMaxDev = 32;
    static std::atomic<size_t> granted[kMaxDev];
    if (lds <= 48 * 1024) return hipSuccess;
    const int slot = dev >= 0 && dev < kMaxDev ? dev : -1;
    if (slot >= 0 && granted[slot].load(std::memory_order_relaxed) >= lds) return hipSuccess;
    hipError_t e = hipFuncSetAttribute((const void *)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess && slot >= 0) granted[slot].store(lds, std::memory_order_relaxed);
    return e;
}
#endif

// ---- small device helpers ---------------------------------------------------
#if defined(__HIPCC__)
__device__ __forceinline__ float cq_h2f(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}
__device__ __forceinline__ uint16_t cq_f2h(float f) {  // round-to-nearest-even
    // Keep the f32 value in a register of its own: otherwise the compiler folds a preceding
    // multiply into one mixed-precision fma (x*c + 0 -> f16), which skips the f32 rounding step
    // and turns a -0.0 product into +0.0.
    asm volatile("" : "+v"(f));
    _Float16 v = (_Float16)f;
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}
// ---- streaming loads ------------------------------------------------------------------------
// Weight bytes are read once per launch: loads marked non-temporal (the `nt` bit of the load) do not displace what
// the caches hold for later use, and on this part a launch that only reads runs 5-12 % faster with it
// (9.4 MB: 3.13 -> 2.78 us, 25 MB: 5.45 -> 5.04 us, 107 MB: 19.6 -> 18.6 us per graph node).
typedef uint32_t cq_u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t cq_u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 cq_ld_stream16(const void *p) {
    const cq_u32x4_t v = __builtin_nontemporal_load((const cq_u32x4_t *)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 cq_ld_stream8(const void *p) {
    const cq_u32x2_t v = __builtin_nontemporal_load((const cq_u32x2_t *)p);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t cq_ld_stream4(const void *p) { return __builtin_nontemporal_load((const uint32_t *)p); }
__device__ __forceinline__ uint16_t cq_ld_stream2(const void *p) { return __builtin_nontemporal_load((const uint16_t *)p); }

// ------------------------------------------------------------------ wave reductions (DPP) ----
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL> __device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
constexpr int kQuadSwap1 = 0xB1;   // quad_perm [1,0,3,2]
constexpr int kQuadSwap2 = 0x4E;   // quad_perm [2,3,0,1]
constexpr int kHalfMirror = 0x141; // lanes i <-> 7-i inside each 8
constexpr int kRowMirror = 0x140;  // lanes i <-> 15-i inside each 16

__device__ __forceinline__ float readlane_f(float v, int l) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
// Sum over the 64 lanes, valid in every lane.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<kQuadSwap1>(v);
    v += dpp_f<kQuadSwap2>(v);
    v += dpp_f<kHalfMirror>(v);
    v += dpp_f<kRowMirror>(v);
    return readlane_f(v, 0) + readlane_f(v, 16) + readlane_f(v, 32) + readlane_f(v, 48);
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<kQuadSwap1>(v));
    v = fmaxf(v, dpp_f<kQuadSwap2>(v));
    v = fmaxf(v, dpp_f<kHalfMirror>(v));
    v = fmaxf(v, dpp_f<kRowMirror>(v));
    return fmaxf(fmaxf(readlane_f(v, 0), readlane_f(v, 16)), fmaxf(readlane_f(v, 32), readlane_f(v, 48)));
}
__device__ __forceinline__ int wave_min_i(int v) {
    v = min(v, dpp_i<kQuadSwap1>(v));
    v = min(v, dpp_i<kQuadSwap2>(v));
    v = min(v, dpp_i<kHalfMirror>(v));
    v = min(v, dpp_i<kRowMirror>(v));
    return min(min(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
               min(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

// Q5K / Q6K on the int8 matrix core: the four byte-sized quants of word `q`, each times the group scale (plus an
// offset), as two int8 digit words.  In 16-bit lanes T = q * s + c with c = 128 + offset (mod 2^16), so that
// P = q * s + offset = T - 128 = 256 * hi + lo with hi = the high byte of T (signed) and lo = its low byte ^ 0x80 in
// [-128, 127]; needs |P| <= 2^15 - 256.  Q6K: s = the group scale, offset = -32 * s; Q5K: s = the sub-block
// scale, offset = 0.  Output bytes are in the order of q's.
typedef unsigned short cq_us2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void cq_scaled_digits(uint32_t q, unsigned short s16, unsigned short c16, int &lo, int &hi) {
    const cq_us2 s = {s16, s16}, c = {c16, c16};   // splats: the packed instruction takes one half twice
    const cq_us2 e02 = __builtin_bit_cast(cq_us2, __builtin_amdgcn_perm(q, 0u, 0x0c060c04u));   // bytes 0, 2 as 16-bit lanes
    const cq_us2 e13 = __builtin_bit_cast(cq_us2, __builtin_amdgcn_perm(q, 0u, 0x0c070c05u));   // bytes 1, 3
    const uint32_t t02 = __builtin_bit_cast(uint32_t, (cq_us2)(e02 * s + c));
    const uint32_t t13 = __builtin_bit_cast(uint32_t, (cq_us2)(e13 * s + c));
    lo = (int)(__builtin_amdgcn_perm(t13, t02, 0x06020400u) ^ 0x80808080u);
    hi = (int)__builtin_amdgcn_perm(t13, t02, 0x07030501u);
}

// Operand of the Q4K / Q5K min term on the f16 matrix core: the eight values -dmin * min_j of a block, each split in
// two f16 pieces p1 = f16(v), p2 = f16(v - p1) (v has 17 significant bits; p1 + p2 == v).  Done in packed f16
// arithmetic: the f16 product IS p1 (correctly rounded), and the f16 fma dmin * min - p1 is the product's rounding
// error, exactly.  `dd` = d | dmin << 16 (f16 bits), `rec` = the block's four records {sc, sc, mn[2g], mn[2g+1]};
// `second` picks the piece this lane carries.  Returns the eight halves as four words.
typedef _Float16 cq_half2 __attribute__((ext_vector_type(2)));
typedef uint32_t cq_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ cq_u32x4 cq_min_term_operand(uint32_t dd, const uint32_t (&rec)[4], bool second) {
    const uint32_t nd = (dd >> 16) ^ 0x8000u;   // -dmin
    const cq_half2 ndmin = __builtin_bit_cast(cq_half2, nd | (nd << 16));
    const cq_half2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    cq_u32x4 out;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        // the two min bytes as f16: 0x6400 | n is 1024 + n
        const uint32_t n2 = __builtin_amdgcn_perm(rec[g], 0u, 0x0c070c06u) | 0x64006400u;
        const cq_half2 mn = __builtin_bit_cast(cq_half2, n2) - k1024;
        const cq_half2 p1 = ndmin * mn;
        const cq_half2 p2 = __builtin_elementwise_fma(ndmin, mn, -p1);
        out[g] = second ? __builtin_bit_cast(uint32_t, p2) : __builtin_bit_cast(uint32_t, p1);
    }
    return out;
}

// The same term with its range taken out of the operands (the Q8K matrix-core kernels): the activation side of the
// contraction is the block's sixteen 16-element sums bsums_j as f16 (|bsums_j| <= 2048: exact, whatever the activations'
// magnitude), the block scale d8 multiplies the result afterwards.  Weight side per group j: -dmin * min_{j/2} in two
// f16 pieces as above.  `half` picks the groups 8*half .. 8*half+7 (sub-blocks 4*half .. 4*half+3, each value twice in a
// row), `second` the piece.
__device__ __forceinline__ cq_u32x4 cq_min_term_groups(uint32_t dd, const uint32_t (&rec)[4], bool half, bool second) {
    const uint32_t nd = (dd >> 16) ^ 0x8000u;   // -dmin
    const cq_half2 ndmin = __builtin_bit_cast(cq_half2, nd | (nd << 16));
    const cq_half2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    cq_u32x4 out;
#pragma unroll
    for (int g = 0; g < 2; g++) {
        const uint32_t rg = half ? rec[2 + g] : rec[g];
        const uint32_t n2 = __builtin_amdgcn_perm(rg, 0u, 0x0c070c06u) | 0x64006400u;   // the two min bytes as 1024 + n
        const cq_half2 mn = __builtin_bit_cast(cq_half2, n2) - k1024;
        const cq_half2 p1 = ndmin * mn;
        const cq_half2 p2 = __builtin_elementwise_fma(ndmin, mn, -p1);
        const uint32_t u = second ? __builtin_bit_cast(uint32_t, p2) : __builtin_bit_cast(uint32_t, p1);
        out[2 * g] = __builtin_amdgcn_perm(u, u, 0x01000100u);       // sub-block 2g' twice
        out[2 * g + 1] = __builtin_amdgcn_perm(u, u, 0x03020302u);   // sub-block 2g'+1 twice
    }
    return out;
}

// Verification form of the operand above: the group minima themselves (first piece; the second is zero), so that the
// same MFMAs deliver the integer sum_j bsums_j * min_{j/2} = Mn_b (at most 16 * 2048 * 63: exact in f32).
__device__ __forceinline__ cq_u32x4 cq_min_term_groups_int(const uint32_t (&rec)[4], bool half, bool second) {
    const cq_half2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    cq_u32x4 out;
#pragma unroll
    for (int g = 0; g < 2; g++) {
        const uint32_t rg = half ? rec[2 + g] : rec[g];
        const uint32_t n2 = __builtin_amdgcn_perm(rg, 0u, 0x0c070c06u) | 0x64006400u;   // the two min bytes as 1024 + n
        const cq_half2 mn = __builtin_bit_cast(cq_half2, n2) - k1024;
        const uint32_t u = second ? 0u : __builtin_bit_cast(uint32_t, mn);
        out[2 * g] = __builtin_amdgcn_perm(u, u, 0x01000100u);
        out[2 * g + 1] = __builtin_amdgcn_perm(u, u, 0x03020302u);
    }
    return out;
}

// Rust `as i8` / `as u8` / `as i32` on f32: truncate toward zero, saturate, NaN -> 0.  That is
// what the hardware conversions do for the 32-bit range (v_cvt_i32_f32 / v_cvt_u32_f32 round toward
// zero, clamp, and turn NaN into 0), so the narrow types only add an integer clamp; no branches.
__device__ __forceinline__ int32_t cq_as_i32(float v) {
    int32_t r;
    asm("v_cvt_i32_f32_e32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}
__device__ __forceinline__ int8_t cq_as_i8(float v) {
    const int32_t r = cq_as_i32(v);
    return (int8_t)(r < -128 ? -128 : (r > 127 ? 127 : r));
}
// round(t) (half away from zero) as an integer, for |t| <= 130: v_cvt_rpi_i32_f32 is floor(|t| + 0.5)
// computed exactly (no rounded intermediate sum; checked against the exact value for every float
// in [0, 130] by cq_selfcheck_round), the sign goes back on in integers.
__device__ __forceinline__ int cq_round_away_i32(float t) {
    int m;
    asm("v_cvt_rpi_i32_f32_e64 %0, |%1|" : "=v"(m) : "v"(t));
    const int sgn = __builtin_bit_cast(int, t) >> 31;
    return (m ^ sgn) - sgn;
}

__device__ __forceinline__ uint8_t cq_as_u8(float v) {
    uint32_t r;
    asm("v_cvt_u32_f32_e32 %0, %1" : "=v"(r) : "v"(v));
    return (uint8_t)(r > 255u ? 255u : r);
}
// utils.rs:3-5 nearest_int = v.round() as i32 (round half away from zero)
__device__ __forceinline__ int32_t cq_nearest_int(float v) { return cq_as_i32(roundf(v)); }
__device__ __forceinline__ int32_t cq_clampi(int32_t v, int32_t lo, int32_t hi) { return v < lo ? lo : (v > hi ? hi : v); }

// utils.rs:49-59 on the 12 scale bytes held as three little-endian words
__device__ __forceinline__ void cq_scale_min_k4(int j, uint32_t u0, uint32_t u1, uint32_t u2, int &sc, int &mn) {
    // Branch-free (lanes of one wave differ in j): for j < 4 the value is one 6-bit field; for
    // j >= 4 it is a 4-bit field of u2 plus the two top bits of byte j-4 of u0 / u1.
    const bool first = j < 4;
    const uint32_t sh = 8u * (uint32_t)(j & 3);
    const uint32_t wlo = first ? 6u : 4u, whi = first ? 0u : 2u;   // a zero-width field reads as 0
    sc = (int)(__builtin_amdgcn_ubfe(first ? u0 : u2, sh, wlo) | (__builtin_amdgcn_ubfe(u0, sh + 6, whi) << 4));
    mn = (int)(__builtin_amdgcn_ubfe(first ? u1 : u2, first ? sh : sh + 4, wlo) |
               (__builtin_amdgcn_ubfe(u1, sh + 6, whi) << 4));
}
#endif
