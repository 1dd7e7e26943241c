// Decode matvec: y[m, n] = sum_k W[n, k] * x[m, k] for a few activation rows (m <= 4 per
// launch), weights streamed once from HBM.  Replaces the reference's MMVQ kernels
// (candle-kernels/src/quantized.cu:2626-2698, launched from quantized/cuda.rs:227-295) with the
// CPU formulation's arithmetic (k_quants.rs:237-254, :631-649, :1171-1250, :1585-1641):
// integer block dots against Q8_0 / Q8K activations, then f32 scales.
//
// Work split: a "unit" is one 16-byte lane of a row's main plane (32 elements for Q4_0, Q4K and
// Q6K, 16 for Q8_0).  A wave walks one row 64 units (1 KiB, eight 128-byte lines) at a time;
// nibbles are split in registers and contracted with v_dot4_i32_i8; the lane sums are reduced
// with DPP.  Activations are staged once per workgroup in LDS, permuted so that lane l of a
// chunk reads its operands at l * 16 bytes (no bank conflicts).
#include "qhip_internal.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

template <int DT> struct Geo;
template <> struct Geo<CQ_DTYPE_Q4_0> { static constexpr int kElems = 32; static constexpr bool kHi = true;  static constexpr int kAux = 1; };
template <> struct Geo<CQ_DTYPE_Q8_0> { static constexpr int kElems = 16; static constexpr bool kHi = false; static constexpr int kAux = 0; };
template <> struct Geo<CQ_DTYPE_Q4K>  { static constexpr int kElems = 32; static constexpr bool kHi = true;  static constexpr int kAux = 1; };
template <> struct Geo<CQ_DTYPE_Q6K>  { static constexpr int kElems = 32; static constexpr bool kHi = true;  static constexpr int kAux = 2; };

// LDS bytes of one staged activation row with `units` units.
template <int DT> __host__ __device__ constexpr size_t lds_row_bytes(int64_t units) {
    return (size_t)units * (16 + (Geo<DT>::kHi ? 16 : 0) + 4 + 4 * Geo<DT>::kAux);
}

struct LdsRow {
    const int4 *lo;   // [units]
    const int4 *hi;   // [units]   (types with two nibble planes)
    const float *ad;  // [units]   activation scale of the unit's block
    const int *s0;    // [units]   Q4_0: sum of the block's quants; Q4K: bsums of the lane's sub-block pair;
                      //           Q6K: bsums of the low-nibble group
    const int *s1;    // [units]   Q6K: bsums of the high-nibble group
};

template <int DT> __device__ __forceinline__ LdsRow lds_row(uint8_t *smem, int64_t units, int m) {
    uint8_t *p = smem + (size_t)m * lds_row_bytes<DT>(units);
    LdsRow r;
    r.lo = (const int4 *)p; p += units * 16;
    r.hi = (const int4 *)p; if (Geo<DT>::kHi) p += units * 16;
    r.ad = (const float *)p; p += units * 4;
    r.s0 = (const int *)p; if (Geo<DT>::kAux >= 1) p += units * 4;
    r.s1 = (const int *)p;
    return r;
}

// Where the 16 consecutive activation elements [16*piece, 16*piece+16) of a row go.
template <int DT> __device__ __forceinline__ void piece_slot(int64_t piece, int64_t &unit, bool &hi) {
    if (DT == CQ_DTYPE_Q8_0) { unit = piece; hi = false; return; }
    if (DT == CQ_DTYPE_Q4_0) { unit = piece >> 1; hi = piece & 1; return; }
    const int64_t b = piece >> 4;
    const int w = (int)(piece & 15);
    if (DT == CQ_DTYPE_Q4K) {
        // unit p = 2g + r covers elements 64g + 16r + [0,16) (low nibbles) and + 32 (high nibbles)
        const int g = w >> 2, r = w & 3;
        unit = 8 * b + 2 * g + (r & 1);
        hi = r >= 2;
    } else {
        // Q6K: unit p = 4h + 2t + i covers 128h + 32t + 16i + [0,16) (low) and + 64 (high)
        const int h = w >> 3, o = w & 7;
        unit = 8 * b + 4 * h + (o & 3);
        hi = o >= 4;
    }
}

template <int DT>
__device__ void stage_row(uint8_t *smem, int64_t units, int m, const cq_act_view &a, int64_t row, int64_t k) {
    LdsRow r = lds_row<DT>(smem, units, m);
    const int4 *src = (const int4 *)(a.qs + row * k);
    for (int64_t piece = threadIdx.x; piece < k / 16; piece += kThreads) {
        int64_t unit; bool hi;
        piece_slot<DT>(piece, unit, hi);
        ((int4 *)(hi ? r.hi : r.lo))[unit] = src[piece];
    }
    for (int64_t u = threadIdx.x; u < units; u += kThreads) {
        if (DT == CQ_DTYPE_Q4_0) {
            ((float *)r.ad)[u] = a.d[row * units + u];
            ((int *)r.s0)[u] = a.bsum32[row * units + u];
        } else if (DT == CQ_DTYPE_Q8_0) {
            ((float *)r.ad)[u] = a.d[row * (units >> 1) + (u >> 1)];
        } else {
            const int64_t blk = row * (units >> 3) + (u >> 3);
            const int p = (int)(u & 7);
            ((float *)r.ad)[u] = a.d[blk];
            const int16_t *bs = a.bsums + blk * 16;
            if (DT == CQ_DTYPE_Q4K) {
                ((int *)r.s0)[u] = (int)bs[2 * p] + (int)bs[2 * p + 1];
            } else {
                const int js = 8 * (p >> 2) + 2 * ((p >> 1) & 1) + (p & 1);
                ((int *)r.s0)[u] = bs[js];
                ((int *)r.s1)[u] = bs[js + 4];
            }
        }
    }
}

__device__ __forceinline__ int dot16(const uint32_t w[4], const int4 &a) {
    int s = __builtin_amdgcn_sdot4((int)w[0], a.x, 0, false);
    s = __builtin_amdgcn_sdot4((int)w[1], a.y, s, false);
    s = __builtin_amdgcn_sdot4((int)w[2], a.z, s, false);
    s = __builtin_amdgcn_sdot4((int)w[3], a.w, s, false);
    return s;
}

// The weight side of one unit, decoded once and reused for every activation row.
template <int DT> struct UnitW {
    uint32_t lo[4], hi[4];
    float dw, dmin;
    int sc_lo, sc_hi, mn;
};

template <int DT>
__device__ __forceinline__ void load_unit(const cq_weight &w, int64_t row, int64_t units, int64_t u, UnitW<DT> &o) {
    const uint4 q = *(const uint4 *)(w.p0 + (row * units + u) * 16);
    const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
    if (DT == CQ_DTYPE_Q4_0) {
        o.dw = cq_h2f(((const uint16_t *)w.p1)[row * units + u]);
#pragma unroll
        for (int i = 0; i < 4; i++) { o.lo[i] = qw[i] & 0x0F0F0F0Fu; o.hi[i] = (qw[i] >> 4) & 0x0F0F0F0Fu; }
    } else if (DT == CQ_DTYPE_Q8_0) {
        o.dw = cq_h2f(((const uint16_t *)w.p1)[row * (units >> 1) + (u >> 1)]);
#pragma unroll
        for (int i = 0; i < 4; i++) o.lo[i] = qw[i];
    } else if (DT == CQ_DTYPE_Q4K) {
        const uint4 h = *(const uint4 *)(w.p1 + (row * (units >> 3) + (u >> 3)) * 16);
        const int p = (int)(u & 7), g = p >> 1;
        o.dw = cq_h2f((uint16_t)(h.x & 0xffff));
        o.dmin = cq_h2f((uint16_t)(h.x >> 16));
        int m0, m1;
        cq_scale_min_k4(2 * g, h.y, h.z, h.w, o.sc_lo, m0);
        cq_scale_min_k4(2 * g + 1, h.y, h.z, h.w, o.sc_hi, m1);
        int scp;
        cq_scale_min_k4(p, h.y, h.z, h.w, scp, o.mn);   // lane p owns the min of sub-block p
#pragma unroll
        for (int i = 0; i < 4; i++) { o.lo[i] = qw[i] & 0x0F0F0F0Fu; o.hi[i] = (qw[i] >> 4) & 0x0F0F0F0Fu; }
    } else {  // Q6K
        const int64_t blk = row * (units >> 3) + (u >> 3);
        const uint2 hh = *(const uint2 *)(w.p1 + (row * units + u) * 8);
        const int p = (int)(u & 7);
        const int js = 8 * (p >> 2) + 2 * ((p >> 1) & 1) + (p & 1);
        const int8_t *sc = (const int8_t *)w.p2 + blk * 16;
        o.sc_lo = sc[js];
        o.sc_hi = sc[js + 4];
        o.dw = cq_h2f(((const uint16_t *)w.p3)[blk]);
        const uint32_t hw[2] = {hh.x, hh.y};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t H = hw[i >> 1];
            const int sh = (i & 1) * 4;
            o.lo[i] = (qw[i] & 0x0F0F0F0Fu) | (((H >> sh) & 0x03030303u) << 4);
            o.hi[i] = ((qw[i] >> 4) & 0x0F0F0F0Fu) | (((H >> (sh + 2)) & 0x03030303u) << 4);
        }
    }
}

// Integer parts of one unit against one staged activation row.
//   Q4_0: I = sum (q-8)*a over the block.            Q8_0: I = sum q*a over half a block.
//   Q4K : I = sc_lo*dot_lo + sc_hi*dot_hi, Mn = min_p * (bsums[2p] + bsums[2p+1]).
//   Q6K : I = sc_lo*(dot_lo - 32*bsums_lo) + sc_hi*(dot_hi - 32*bsums_hi).
template <int DT>
__device__ __forceinline__ void unit_ints(const UnitW<DT> &w, const LdsRow &r, int64_t u, int &I, int &Mn) {
    const int4 alo = r.lo[u];
    Mn = 0;
    if (DT == CQ_DTYPE_Q8_0) {
        I = dot16(w.lo, alo);
        return;
    }
    const int4 ahi = r.hi[u];
    const int dlo = dot16(w.lo, alo), dhi = dot16(w.hi, ahi);
    if (DT == CQ_DTYPE_Q4_0) {
        I = dlo + dhi - 8 * r.s0[u];
    } else if (DT == CQ_DTYPE_Q4K) {
        I = w.sc_lo * dlo + w.sc_hi * dhi;
        Mn = w.mn * r.s0[u];
    } else {
        I = w.sc_lo * (dlo - 32 * r.s0[u]) + w.sc_hi * (dhi - 32 * r.s1[u]);
    }
}

template <int DT>
__device__ __forceinline__ float unit_value(const UnitW<DT> &w, const LdsRow &r, int64_t u) {
    int I, Mn;
    unit_ints<DT>(w, r, u, I, Mn);
    const float ad = r.ad[u];
    if (DT == CQ_DTYPE_Q4K) return ad * (w.dw * (float)I - w.dmin * (float)Mn);
    return ((float)I * w.dw) * ad;
}

// Sum over the 64 lanes of a wave, result valid in every lane.
__device__ __forceinline__ float wave_sum(float v) {
#define CQ_DPP_ADD(ctrl)                                                                                   \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))
    CQ_DPP_ADD(0xB1);   // quad_perm [1,0,3,2]
    CQ_DPP_ADD(0x4E);   // quad_perm [2,3,0,1]
    CQ_DPP_ADD(0x141);  // row_half_mirror
    CQ_DPP_ADD(0x140);  // row_mirror
#undef CQ_DPP_ADD
    // every lane of a 16-lane row now holds the row's sum
    const int iv = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
}

template <int DT, int MB>
__global__ void __launch_bounds__(kThreads) matvec_kernel(cq_weight w, cq_act_view a, int64_t m0, int rows_per_wg,
                                                          float *__restrict__ y) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int64_t units = w.k / Geo<DT>::kElems;
#pragma unroll
    for (int m = 0; m < MB; m++) stage_row<DT>(smem, units, m, a, m0 + m, w.k);
    __syncthreads();
    LdsRow rows[MB];
#pragma unroll
    for (int m = 0; m < MB; m++) rows[m] = lds_row<DT>(smem, units, m);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row_begin = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t row_end = row_begin + rows_per_wg < w.n ? row_begin + rows_per_wg : w.n;
    for (int64_t row = row_begin + wave; row < row_end; row += kWaves) {
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; m++) acc[m] = 0.0f;
#pragma unroll 2
        for (int64_t u = lane; u < units; u += 64) {
            UnitW<DT> uw;
            load_unit<DT>(w, row, units, u, uw);
#pragma unroll
            for (int m = 0; m < MB; m++) acc[m] += unit_value<DT>(uw, rows[m], u);
        }
#pragma unroll
        for (int m = 0; m < MB; m++) {
            const float s = wave_sum(acc[m]);
            if (lane == 0) y[(m0 + m) * w.n + row] = s;
        }
    }
}

// Per-block integer dots for verification: one wave per (activation row, weight row).
template <int DT>
__global__ void __launch_bounds__(kThreads) int_dots_kernel(cq_weight w, cq_act_view a, int64_t m0, int rows_per_wg,
                                                            int32_t *__restrict__ out_i, int32_t *__restrict__ out_mn) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int64_t units = w.k / Geo<DT>::kElems;
    stage_row<DT>(smem, units, 0, a, m0, w.k);
    __syncthreads();
    const LdsRow r = lds_row<DT>(smem, units, 0);
    constexpr int kUnitsPerBlock = DT == CQ_DTYPE_Q4_0 ? 1 : (DT == CQ_DTYPE_Q8_0 ? 2 : 8);
    const int64_t kb = units / kUnitsPerBlock;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row_begin = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t row_end = row_begin + rows_per_wg < w.n ? row_begin + rows_per_wg : w.n;
    for (int64_t row = row_begin + wave; row < row_end; row += kWaves) {
        for (int64_t u0 = 0; u0 < units; u0 += 64) {
            const int64_t u = u0 + lane;
            int I = 0, Mn = 0;
            if (u < units) {
                UnitW<DT> uw;
                load_unit<DT>(w, row, units, u, uw);
                unit_ints<DT>(uw, r, u, I, Mn);
            }
#pragma unroll
            for (int off = 1; off < kUnitsPerBlock; off <<= 1) {
                I += __shfl_xor(I, off);
                Mn += __shfl_xor(Mn, off);
            }
            if (u < units && (u % kUnitsPerBlock) == 0) {
                const int64_t o = (m0 * w.n + row) * kb + u / kUnitsPerBlock;
                out_i[o] = I;
                if (out_mn) out_mn[o] = Mn;
            }
        }
    }
}

int pick_rows_per_wg(int64_t n) {
    // Enough workgroups to fill 256 CUs several times over, few enough that the activation
    // staging is amortised over several rows per wave.
    int r = 16;
    while (r > 4 && (n + r - 1) / r < 2048) r >>= 1;
    return r;
}

template <int DT>
hipError_t launch_dt(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    const int64_t units = w->k / Geo<DT>::kElems;
    const int rpw = pick_rows_per_wg(w->n);
    const unsigned grid = (unsigned)((w->n + rpw - 1) / rpw);
    int64_t m0 = 0;
    while (m0 < m) {
        const int64_t left = m - m0;
        // keep the staged rows within 64 KiB of LDS
        int mb = left >= 4 ? 4 : (left >= 2 ? 2 : 1);
        while (mb > 1 && lds_row_bytes<DT>(units) * mb > 64 * 1024) mb >>= 1;
        const size_t lds = lds_row_bytes<DT>(units) * mb;
        if (lds > 150 * 1024) return hipErrorInvalidValue;
        if (mb == 4) matvec_kernel<DT, 4><<<grid, kThreads, lds, s>>>(*w, a, m0, rpw, y);
        else if (mb == 2) matvec_kernel<DT, 2><<<grid, kThreads, lds, s>>>(*w, a, m0, rpw, y);
        else matvec_kernel<DT, 1><<<grid, kThreads, lds, s>>>(*w, a, m0, rpw, y);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        m0 += mb;
    }
    return hipSuccess;
}

template <int DT>
hipError_t launch_ints(const cq_weight *w, cq_act_view a, int64_t m, int32_t *oi, int32_t *omn, hipStream_t s) {
    const int64_t units = w->k / Geo<DT>::kElems;
    const size_t lds = lds_row_bytes<DT>(units);
    if (lds > 150 * 1024) return hipErrorInvalidValue;
    const int rpw = 8;
    const unsigned grid = (unsigned)((w->n + rpw - 1) / rpw);
    for (int64_t m0 = 0; m0 < m; m0++) {
        int_dots_kernel<DT><<<grid, kThreads, lds, s>>>(*w, a, m0, rpw, oi, omn);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace

hipError_t cq_launch_matvec(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, hipStream_t s) {
    (void)act_dtype;
    if (m == 0 || w->n == 0) return hipSuccess;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: return launch_dt<CQ_DTYPE_Q4_0>(w, a, m, y, s);
    case CQ_DTYPE_Q8_0: return launch_dt<CQ_DTYPE_Q8_0>(w, a, m, y, s);
    case CQ_DTYPE_Q4K: return launch_dt<CQ_DTYPE_Q4K>(w, a, m, y, s);
    case CQ_DTYPE_Q6K: return launch_dt<CQ_DTYPE_Q6K>(w, a, m, y, s);
    default: return hipErrorInvalidValue;
    }
}

hipError_t cq_launch_int_dots(const cq_weight *w, cq_act_view a, int64_t m, int32_t *out_i, int32_t *out_mn,
                              hipStream_t s) {
    if (m == 0 || w->n == 0) return hipSuccess;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: return launch_ints<CQ_DTYPE_Q4_0>(w, a, m, out_i, out_mn, s);
    case CQ_DTYPE_Q8_0: return launch_ints<CQ_DTYPE_Q8_0>(w, a, m, out_i, out_mn, s);
    case CQ_DTYPE_Q4K: return launch_ints<CQ_DTYPE_Q4K>(w, a, m, out_i, out_mn, s);
    case CQ_DTYPE_Q6K: return launch_ints<CQ_DTYPE_Q6K>(w, a, m, out_i, out_mn, s);
    default: return hipErrorInvalidValue;
    }
}
