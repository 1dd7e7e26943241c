// Prefill GEMM on int8 MFMA: y[m, n] = x[m, k] . W[n, k]^T for K-quant weights and Q8K activations,
// the arithmetic of the reference's CPU matmul (k_quants.rs:1842-1883 with vec_dot :1171-1250 for
// Q4K, :1585-1641 for Q6K); replaces the MMQ kernels (candle-kernels/src/quantized.cu:436-544,
// launched from quantized/cuda.rs:298-365), which use dp4a and no matrix cores.
//
// Per 256-element block b the reference computes, for weight row n and activation row m,
//   Q4K:  d[n,b]*d8[m,b] * I  -  dmin[n,b]*d8[m,b] * Mn,   I = sum_j sc_j * sum_32 q4*q8,
//                                                          Mn = sum_j min_j * bsum32[m,j]
//   Q6K:  d[n,b]*d8[m,b] * I,                              I = sum_16-groups sc_g * sum_16 (q6-32)*q8
// The sub-block scales sit between the int8 contraction and the accumulator, so they are folded
// into the int8 weights as two digits and the block is contracted with two MFMAs per K-slice:
//   Q4K:  sc = 8*sh + sl (3-bit digits): operands sh*q4, sl*q4 <= 105;  I = 8*acc_hi + acc_lo
//   Q6K:  P = sc*(q6-32) (13 bits signed): operands P >> 7, P & 127;    I = 128*acc_hi + acc_lo
// I is the same integer as on the CPU.  The Q4K min term is a small f32 contraction over the
// eight sub-blocks; it runs on the f16 MFMA with both factors split in two f16 pieces (products
// exact to ~2^-22) and accumulates straight into the f32 result.
//
// Work split: a workgroup of four waves covers BM = 32*MT activation rows x 128 weight rows; each
// wave owns 32 weight rows (MFMA B operand: lane l holds row l%32, k = 16*(l/32)+[0,16) of a
// 32-wide K-slice) and unpacks them from HBM straight into registers - no LDS for weights; the
// next block's weight bytes are loaded one block ahead.  The activation tile of a block (MFMA A
// operands, already in fragment order) goes from global memory straight into LDS with
// global_load_lds_dwordx4, double buffered, and is shared by the four waves.  With few workgroups
// (small n) K is split over blockIdx.z and the partial results are added atomically.
#include "qhip_internal.h"
#include <stdlib.h>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short us2 __attribute__((ext_vector_type(2)));
typedef short ss2 __attribute__((ext_vector_type(2)));
typedef const void __attribute__((address_space(1))) *gptr_t;
typedef void __attribute__((address_space(3))) *lptr_t;

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;

// LDS image of one block's activation tile (BM = 32*MT rows):
//   frag : [MT][8 slices][64 lanes][16 B]   A operands, lane l = row l%32, k = 32*slice + 16*(l/32) + [0,16)
//   d8   : [BM] f32
//   minp : [BM][2 pieces][8] f16            d8 * bsum32_j split in two f16 pieces (Q4K)
template <int MT> struct Tile {
    static constexpr int kFrag = MT * 8 * 1024;
    static constexpr int kD8 = (MT * 32 < 64 ? 64 : MT * 32) * 4;   // filled by whole-wave copies of 64 floats
    static constexpr int kMin = MT * 32 * 32;
    static constexpr int kBytes = kFrag + kD8 + kMin;
};

__device__ __forceinline__ uint32_t pk_mul_u16(uint32_t a, uint32_t b) {
    const us2 r = __builtin_bit_cast(us2, a) * __builtin_bit_cast(us2, b);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pk_sub_u16(uint32_t a, uint32_t b) {
    const us2 r = __builtin_bit_cast(us2, a) - __builtin_bit_cast(us2, b);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pk_ashr7_i16(uint32_t a) {
    const ss2 r = __builtin_bit_cast(ss2, a) >> (ss2){7, 7};
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t dup16(uint32_t v) { return (v & 0xffffu) | (v << 16); }

// Asynchronous global -> LDS copies of one block's activation tile, issued by every wave for its
// share of the 1 KiB fragments.  Lane l of a wave-wide copy lands at dst + 16*l (or 4*l), whatever
// global address it reads from, so the fragment order is produced by the address computation
// alone.  Rows past m read a clamped row; their outputs are never stored.
template <int MT, bool MINS>
__device__ __forceinline__ void stage_issue(uint8_t *buf, const cq_act_view &a, int64_t m, int64_t k, int64_t m0,
                                            int64_t b, int wave, int lane) {
    const int64_t kb = k >> 8;
    const int64_t last = m - 1;
    for (int f = wave; f < MT * 8; f += kWaves) {
        const int mt = f >> 3, s = f & 7;
        int64_t row = m0 + mt * 32 + (lane & 31);
        row = row < last ? row : last;
        const int8_t *src = a.qs + row * k + b * 256 + s * 32 + (lane >> 5) * 16;
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(buf + f * 1024), 16, 0, 0);
    }
    for (int c = wave; c < (MT * 32 + 63) / 64; c += kWaves) {
        int64_t row = m0 + c * 64 + lane;
        row = row < last ? row : last;
        __builtin_amdgcn_global_load_lds((gptr_t)(a.d + row * kb + b), (lptr_t)(buf + Tile<MT>::kFrag + c * 256), 4, 0, 0);
    }
    if (MINS) {
        for (int c = wave; c < MT; c += kWaves) {
            int64_t row = m0 + c * 32 + (lane >> 1);
            row = row < last ? row : last;
            const uint16_t *src = a.minp + (row * kb + b) * 16 + (lane & 1) * 8;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(buf + Tile<MT>::kFrag + Tile<MT>::kD8 + c * 1024), 16,
                                             0, 0);
        }
    }
}

// One block of one weight row as this lane needs it (row n, k-half h = lane / 32).
template <int DT> struct WBlk;
template <> struct WBlk<CQ_DTYPE_Q4K> {
    uint4 q[4];   // qs bytes 32g + 16h + [0,16): low nibbles = K-slice 2g, high nibbles = slice 2g+1
    uint4 hd;     // d, dmin, scales[12]
};
template <> struct WBlk<CQ_DTYPE_Q6K> {
    uint4 q[4];   // ql lanes of the four units of this k-half: u = 4*(x/2) + 2*(x%2) + h
    uint2 qh[4];  // their re-packed high bits
    uint4 sc;     // re-packed scales: bytes 2u, 2u+1 = scale of the unit's low / high nibble group
    uint32_t d;
};

__device__ __forceinline__ void load_w(const cq_weight &w, int64_t blk, int h, WBlk<CQ_DTYPE_Q4K> &r) {
    r.hd = *(const uint4 *)(w.p1 + blk * 16);
#pragma unroll
    for (int g = 0; g < 4; g++) r.q[g] = *(const uint4 *)(w.p0 + blk * 128 + 32 * g + 16 * h);
}
__device__ __forceinline__ void load_w(const cq_weight &w, int64_t blk, int h, WBlk<CQ_DTYPE_Q6K> &r) {
    r.sc = *(const uint4 *)(w.p2 + blk * 16);
    r.d = ((const uint16_t *)w.p3)[blk];
#pragma unroll
    for (int x = 0; x < 4; x++) {
        const int u = 4 * (x >> 1) + 2 * (x & 1) + h;
        r.q[x] = *(const uint4 *)(w.p0 + blk * 128 + 16 * u);
        r.qh[x] = *(const uint2 *)(w.p1 + blk * 64 + 8 * u);
    }
}

// One block for this wave's 32 weight rows against the MT activation tiles in `cur`, as a
// hand-laid software pipeline of 8*(MT+1) steps.  Step (t, s) issues the two int8 MFMAs of tile t,
// K-slice s, and, in their shadow, the scaling of two of the sixteen integers of tile t-1 (VALU);
// LDS reads run two steps ahead.  The accumulator pair alternates between two register sets.  A
// scheduling barrier after every step keeps the compiler from hoisting all MFMAs to the front,
// which would need MT accumulator sets at once.
template <int MT, bool MINS, int SHIFT>
__device__ __forceinline__ void tiles_mac(const uint8_t *cur, const v4i (&bl)[8], const v4i (&bh)[8], float dw,
                                          v8h wmin, int lane, v16f (&out)[MT]) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    const int h = lane >> 5, col = lane & 31;
    const uint8_t *afrag = cur + lane * 16;
    const uint8_t *d8p = cur + Tile<MT>::kFrag + h * 16;                    // rows 8j + 4h + [0,4) of a tile
    const uint8_t *mnp = cur + Tile<MT>::kFrag + Tile<MT>::kD8 + col * 32;   // this lane's row of min pieces
    v16i acc_lo[2], acc_hi[2];
    v4i a[3];
    v4f dsc[2][4];
    v8h ma1, ma2;
    a[0] = *(const v4i *)(afrag);
    a[1] = *(const v4i *)(afrag + 1024);
    if (MINS) {
        ma1 = *(const v8h *)(mnp);
        ma2 = *(const v8h *)(mnp + 16);
    }
#pragma unroll
    for (int q = 0; q < (MT + 1) * 8; q++) {
        const int t = q >> 3, s = q & 7;
        if (q + 2 < MT * 8) a[(q + 2) % 3] = *(const v4i *)(afrag + (q + 2) * 1024);
        if (t < MT) {
            if (s == 0) {
                if (MINS) {
                    // min term: out -= sum_j (dmin*min_j) * (d8*bsum32_j).  K-slots 0..7 carry piece 1
                    // of the weight factor, slots 8..15 piece 2; the activation operand carries one of
                    // its pieces in both halves.
                    out[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma1, wmin, out[t], 0, 0, 0);
                    out[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma2, wmin, out[t], 0, 0, 0);
                }
                const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                acc_lo[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q % 3], bl[0], zero, 0, 0, 0);
                acc_hi[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q % 3], bh[0], zero, 0, 0, 0);
            } else {
                acc_lo[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q % 3], bl[s], acc_lo[t & 1], 0, 0, 0);
                acc_hi[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q % 3], bh[s], acc_hi[t & 1], 0, 0, 0);
            }
            if (s == 4) {
#pragma unroll
                for (int j = 0; j < 4; j++) dsc[t & 1][j] = *(const v4f *)(d8p + (t * 32 + 8 * j) * 4);
            }
            if (s == 6 && MINS && t + 1 < MT) {
                ma1 = *(const v8h *)(mnp + (t + 1) * 1024);
                ma2 = *(const v8h *)(mnp + (t + 1) * 1024 + 16);
            }
        }
        if (t > 0) {
            const int p = (t - 1) & 1;
#pragma unroll
#ifdef EXP_NO_EPI
            for (int i = 2 * s; i < 2 * s + (s == 0 ? 1 : 0); i++) {
#else
            for (int i = 2 * s; i < 2 * s + 2; i++) {
#endif
                const int I = (acc_hi[p][i] << SHIFT) + acc_lo[p][i];
                float o = __builtin_fmaf((float)I * dw, dsc[p][i >> 2][i & 3], out[t - 1][i]);
                asm volatile("" : "+v"(o));   // pins the scaling to this step (pure ops float otherwise)
                out[t - 1][i] = o;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int MT>
__device__ __forceinline__ void block_mac(const uint8_t *cur, const WBlk<CQ_DTYPE_Q4K> &wb, int lane, v16f (&out)[MT]) {
    const int h = lane >> 5;
    const uint4 hd = wb.hd;
    const float dw = cq_h2f((uint16_t)(hd.x & 0xffff));
    const float dmin = cq_h2f((uint16_t)(hd.x >> 16));
    // all eight scales and mins as bytes (k_quants.rs:1209-1219)
    const uint32_t sc03 = hd.y & 0x3f3f3f3fu;
    const uint32_t sc47 = (hd.w & 0x0f0f0f0fu) | (((hd.y >> 6) & 0x03030303u) << 4);
    const uint32_t mn03 = hd.z & 0x3f3f3f3fu;
    const uint32_t mn47 = ((hd.w >> 4) & 0x0f0f0f0fu) | (((hd.z >> 6) & 0x03030303u) << 4);
    v4i bl[8], bh[8];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const uint32_t scw = g < 2 ? sc03 : sc47;
        const uint32_t s0 = (scw >> (16 * (g & 1))) & 0xff, s1 = (scw >> (16 * (g & 1) + 8)) & 0xff;
        const uint32_t sl0 = dup16(s0 & 7), sh0 = dup16(s0 >> 3), sl1 = dup16(s1 & 7), sh1 = dup16(s1 >> 3);
        const uint32_t qw[4] = {wb.q[g].x, wb.q[g].y, wb.q[g].z, wb.q[g].w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t lo4 = qw[i] & 0x0F0F0F0Fu, hi4 = (qw[i] >> 4) & 0x0F0F0F0Fu;
            bl[2 * g][i] = (int)pk_mul_u16(lo4, sl0);       // sub-block 2g, low digit of the scale
            bh[2 * g][i] = (int)pk_mul_u16(lo4, sh0);
            bl[2 * g + 1][i] = (int)pk_mul_u16(hi4, sl1);   // sub-block 2g+1
            bh[2 * g + 1][i] = (int)pk_mul_u16(hi4, sh1);
        }
    }
    v8h wmin;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t mw = j < 4 ? mn03 : mn47;
        const float v = -dmin * (float)((mw >> (8 * (j & 3))) & 0xff);
        const _Float16 p1 = (_Float16)v;
        wmin[j] = h == 0 ? p1 : (_Float16)(v - (float)p1);
    }
    tiles_mac<MT, true, 3>(cur, bl, bh, dw, wmin, lane, out);
}

template <int MT>
__device__ __forceinline__ void block_mac(const uint8_t *cur, const WBlk<CQ_DTYPE_Q6K> &wb, int lane, v16f (&out)[MT]) {
    const int h = lane >> 5;
    const float dw = cq_h2f((uint16_t)wb.d);
    const uint32_t scw[4] = {wb.sc.x, wb.sc.y, wb.sc.z, wb.sc.w};
    v4i bl[8], bh[8];
#pragma unroll
    for (int s = 0; s < 8; s++) {
        // K-slice s: this lane's 16 elements are the group G = 2s + h, i.e. unit
        // u = 4*(s/4) + 2*(s%2) + h, low nibbles when (s%4) < 2 else high nibbles
        const int x = 2 * (s >> 2) + (s & 1), nib = (s & 3) >> 1;
        const int sb = 2 * (4 * (x >> 1) + 2 * (x & 1)) + nib;   // scale byte index for h = 0; h adds 2
        const uint32_t sw = scw[sb >> 2];                         // bytes sb and sb + 2 are in the same word
        const int sc = (int)(int8_t)((sw >> (8 * (sb & 3) + 16 * h)) & 0xff);
        const uint32_t sc16 = dup16((uint32_t)sc);
        const uint32_t qw[4] = {wb.q[x].x, wb.q[x].y, wb.q[x].z, wb.q[x].w};
        const uint32_t hw[2] = {wb.qh[x].x, wb.qh[x].y};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t H = hw[i >> 1];
            const int sh = (i & 1) * 4 + 2 * nib;
            const uint32_t q6 = ((qw[i] >> (4 * nib)) & 0x0F0F0F0Fu) | (((H >> sh) & 0x03030303u) << 4);
            // the four elements as 16-bit lanes, minus 32, times the group scale (low 16 bits kept)
            const uint32_t e02 = pk_sub_u16(q6 & 0x00FF00FFu, 0x00200020u);
            const uint32_t e13 = pk_sub_u16((q6 >> 8) & 0x00FF00FFu, 0x00200020u);
            const uint32_t p02 = pk_mul_u16(e02, sc16), p13 = pk_mul_u16(e13, sc16);
            // gather bytes [p02.0, p13.0, p02.2, p13.2]
            bl[s][i] = (int)(__builtin_amdgcn_perm(p13, p02, 0x06020400u) & 0x7F7F7F7Fu);
            bh[s][i] = (int)__builtin_amdgcn_perm(pk_ashr7_i16(p13), pk_ashr7_i16(p02), 0x06020400u);
        }
    }
    v8h wmin = {};
    tiles_mac<MT, false, 7>(cur, bl, bh, dw, wmin, lane, out);
}

// ------------------------------------------------------------------ kernel ----
template <int DT, int MT>
__global__ void __launch_bounds__(kThreads) gemm_kernel(cq_weight w, cq_act_view a, int64_t m, float *__restrict__ y,
                                                        int ksplit) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr bool MINS = DT == CQ_DTYPE_Q4K;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, col = lane & 31;
    const int64_t kb = w.k >> 8;
    const int64_t m0 = (int64_t)blockIdx.y * (MT * 32);
    const int64_t n_tile = ((int64_t)blockIdx.x * kWaves + wave) * 32;
    const int64_t n = n_tile + col;
    const int64_t nc = n < w.n ? n : w.n - 1;   // clamped row for loads; stores are masked
    // this workgroup's range of K blocks
    const int64_t b0 = kb * blockIdx.z / ksplit, b1 = kb * (blockIdx.z + 1) / ksplit;

    v16f out[MT];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) out[t][i] = 0.0f;

    WBlk<DT> wcur, wnxt;
    stage_issue<MT, MINS>(smem, a, m, w.k, m0, b0, wave, lane);
    load_w(w, nc * kb + b0, h, wcur);
    __builtin_amdgcn_s_waitcnt(0);   // the LDS copies above (and everything else outstanding)
    __syncthreads();

    for (int64_t b = b0; b < b1; b++) {
        const int par = (int)((b - b0) & 1);
        uint8_t *cur = smem + par * Tile<MT>::kBytes;
        uint8_t *nxt = smem + (par ^ 1) * Tile<MT>::kBytes;
        const bool more = b + 1 < b1;
        if (more) {
#ifndef EXP_NO_STAGE
            stage_issue<MT, MINS>(nxt, a, m, w.k, m0, b + 1, wave, lane);
#endif
#ifndef EXP_NO_WLOAD
            load_w(w, nc * kb + b + 1, h, wnxt);
#else
            wnxt = wcur;
#endif
        }
        block_mac<MT>(cur, wcur, lane, out);
        if (more) wcur = wnxt;
        __builtin_amdgcn_s_waitcnt(0);   // next tile has landed in LDS
        __syncthreads();
    }

    if (n < w.n) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t row = m0 + t * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                if (row < m) {
                    if (ksplit == 1) y[row * w.n + n] = out[t][i];
                    else unsafeAtomicAdd(&y[row * w.n + n], out[t][i]);
                }
            }
        }
    }
}

int g_cus = 0;
int num_cus() {
    if (g_cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            g_cus = n;
        else
            g_cus = 256;
    }
    return g_cus;
}

template <int DT, int MT>
hipError_t launch_mt(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    const size_t lds = 2 * Tile<MT>::kBytes;
    static bool attr_set = false;
    if (!attr_set && lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_kernel<DT, MT>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int64_t gx = (w->n + kWaves * 32 - 1) / (kWaves * 32), gy = (m + MT * 32 - 1) / (MT * 32);
    // too few workgroups for the machine: split K (at least four blocks per part)
    int ksplit = 1;
    const int64_t kb = w->k >> 8;
    while (gx * gy * ksplit * 2 <= num_cus() && kb / (ksplit * 2) >= 4 && ksplit < 16) ksplit *= 2;
    if (ksplit > 1) {
        hipError_t e = cq_launch_fill_zero(y, m * w->n, s);
        if (e != hipSuccess) return e;
    }
    dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)ksplit);
    gemm_kernel<DT, MT><<<grid, kThreads, lds, s>>>(*w, a, m, y, ksplit);
    return hipGetLastError();
}

template <int DT>
hipError_t launch_dt(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    if (m <= 32) return launch_mt<DT, 1>(w, a, m, y, s);
    if (m <= 64) return launch_mt<DT, 2>(w, a, m, y, s);
    static const char *force8 = getenv("CQ_GEMM_MT8");
    if (m <= 128 || !force8) return launch_mt<DT, 4>(w, a, m, y, s);
    return launch_mt<DT, 8>(w, a, m, y, s);
}

}  // namespace

bool cq_gemm_supported(const cq_weight *w, int64_t m, int act_dtype) {
    (void)m;
    return (w->dtype == CQ_DTYPE_Q4K || w->dtype == CQ_DTYPE_Q6K) && act_dtype == CQ_DTYPE_Q8K && w->k >= 256;
}

hipError_t cq_launch_gemm(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, hipStream_t s) {
    if (!cq_gemm_supported(w, m, act_dtype)) return hipErrorNotSupported;
    if (m == 0 || w->n == 0) return hipSuccess;
    if (w->dtype == CQ_DTYPE_Q4K) return launch_dt<CQ_DTYPE_Q4K>(w, a, m, y, s);
    return launch_dt<CQ_DTYPE_Q6K>(w, a, m, y, s);
}
