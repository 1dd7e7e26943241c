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
// Work split: a workgroup of eight waves (two per SIMD, so that one wave's scaling arithmetic runs
// under the other's MFMAs) covers BM = 32*MT activation rows x 128 weight rows.  Each wave owns 16
// weight rows and works with the 16x16x64 MFMA: operand lane l holds row l%16 and the 16
// consecutive k of quarter l/16 of a 64-wide K-slice; result lane l holds column l%16, rows
// 4*(l/16)+[0,4).  The wave unpacks its weight operands in registers once per block and reuses
// them for all BM rows.  Activations (shared by the waves) and each wave's packed weight bytes go
// from global memory straight into LDS (global_load_lds_dwordx4), double buffered, one block
// ahead.  Every such copy instruction reads eight whole 128-byte lines (8 rows x 128 B) - the
// texture path pays per line touched - and the 16-byte chunks of a row are XOR-swizzled by the
// row number on the way in, so that the operand reads (lanes = rows, one chunk column) spread
// over all LDS banks.  With few workgroups (small n) K is split over blockIdx.z and the partial
// results are added atomically.
#include "qhip_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short us2 __attribute__((ext_vector_type(2)));
typedef short ss2 __attribute__((ext_vector_type(2)));
typedef const void __attribute__((address_space(1))) *gptr_t;
typedef void __attribute__((address_space(3))) *lptr_t;

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kRowsPerWave = 16;
constexpr int kBN = kWaves * kRowsPerWave;

// LDS image of one pipeline stage:
//   act  : [MT][2 K-halves][4 row groups][8 rows][8 chunks of 16 B]   chunk c of row r sits at c ^ (r%8)
//   d8   : [BM] f32
//   minp : [BM][2 pieces][8] f16            d8 * bsum32_j split in two f16 pieces (Q4K)
//   wgt  : per wave: [2 row groups][8 rows][8 chunks] of the 128-byte qs / ql plane (same swizzle),
//          Q6K also [16 rows][4 chunks] of the 64-byte qh plane (chunk c at c ^ ((r/2)%4))
template <int DT, int MT> struct Tile {
    static constexpr int kAct = MT * 8 * 1024;
    static constexpr int kD8 = (MT * 32 < 64 ? 64 : MT * 32) * 4;   // filled by whole-wave copies of 64 floats
    static constexpr int kMin = DT == CQ_DTYPE_Q4K ? MT * 32 * 32 : 0;
    static constexpr int kWgtWave = DT == CQ_DTYPE_Q4K ? 2048 : 3072;
    static constexpr int oD8 = kAct, oMin = oD8 + kD8, oWgt = oMin + kMin;
    static constexpr int kBytes = oWgt + kWaves * kWgtWave;
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

// Asynchronous copy of 64 x 16 (or 64 x 4) bytes: lane l reads base + off and the data lands at
// lds + 16*l (4*l).  `base` and `lds` are wave-uniform.
__device__ __forceinline__ void dma16(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_global_load_lds((gptr_t)((const uint8_t *)base + off), (lptr_t)lds, 16, 0, 0);
}
__device__ __forceinline__ void dma4(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_global_load_lds((gptr_t)((const uint8_t *)base + off), (lptr_t)lds, 4, 0, 0);
}

// Per-lane constants of the copies and of the operand reads (r = l%16: row, kq = l/16: k quarter).
struct LaneGeo {
    uint32_t act_off;    // copy of 8 rows x 128 B of activations: (l/8)*k + ((l%8) ^ (l/8))*16
    uint32_t wq_off;     // the same over the weights' 128-byte plane: (l/8)*kb*128 + ...
    uint32_t wh_off;     // Q6K qh plane, 16 rows x 64 B: (l/4)*kb*64 + ((l%4) ^ ((l/8)%4))*16
    uint32_t a_col[2];   // activation operand of K-slice S: chunk 4*(S%2) + kq of K-half S/2, row r
    uint32_t w_col4[4];  // Q4K weight chunk 2g + kq%2 of row r
    uint32_t w_col6[2];  // Q6K ql chunk (unit) 4*hf + kq of row r
    uint32_t qh_col[2];  // Q6K: the 8 bytes of high bits of unit 4*hf + kq of row r
};

__device__ __forceinline__ uint32_t swz_col(uint32_t r, uint32_t c) {
    return (r >> 3) * 1024u + (r & 7) * 128u + ((c ^ (r & 7)) << 4);
}

__device__ __forceinline__ LaneGeo lane_geo(int lane, int64_t k) {
    LaneGeo g;
    const uint32_t kb = (uint32_t)(k >> 8);
    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    g.act_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    g.wq_off = r8 * kb * 128u + ((c8 ^ r8) << 4);
    const uint32_t r16 = lane >> 2, c4 = lane & 3;
    g.wh_off = r16 * kb * 64u + ((c4 ^ ((r16 >> 1) & 3)) << 4);
    const uint32_t r = lane & 15, kq = lane >> 4;
#pragma unroll
    for (uint32_t e = 0; e < 2; e++) {
        g.a_col[e] = swz_col(r, 4 * e + kq);
        g.w_col6[e] = swz_col(r, 4 * e + kq);
        g.qh_col[e] = r * 64u + (((2 * e + (kq >> 1)) ^ ((r >> 1) & 3)) << 4) + (kq & 1) * 8u;
    }
#pragma unroll
    for (uint32_t gi = 0; gi < 4; gi++) g.w_col4[gi] = swz_col(r, 2 * gi + (kq & 1));
    return g;
}

// Issues this wave's share of the copies for block b into stage `buf`.
template <int DT, int MT>
__device__ __forceinline__ void stage_issue(uint8_t *buf, const cq_weight &w, const cq_act_view &a, const LaneGeo &g,
                                            int64_t m0, int64_t n_tile, bool n_ok, int64_t b, int wave, int lane) {
    typedef Tile<DT, MT> T;
    const int64_t k = w.k, kb = w.k >> 8;
    // activations: MT*8 copies of 8 rows x 128 B, dealt round-robin to the waves
#pragma unroll
    for (int j = 0; j < MT * 8 / kWaves; j++) {
        const int idx = wave + kWaves * j;           // = (t*2 + kh)*4 + rg
        const int rg = idx & 3, kh = (idx >> 2) & 1, t = idx >> 3;
        const int8_t *base = a.qs + (m0 + t * 32 + rg * 8) * k + b * 256 + kh * 128;
        dma16(base, g.act_off, buf + idx * 1024);
    }
#pragma unroll
    for (int j = 0; j < (MT * 32 + 63) / 64; j++) {
        if (j == wave) dma4(a.dT + b * a.m_stride + m0 + j * 64, lane * 4u, buf + T::oD8 + j * 256);
    }
    if (DT == CQ_DTYPE_Q4K) {
#pragma unroll
        for (int j = 0; j < MT; j++) {
            if (j + 4 == wave)
                dma16(a.minp + (b * a.m_stride + m0 + j * 32) * 16, lane * 16u, buf + T::oMin + j * 1024);
        }
    }
    // this wave's 16 weight rows
    if (n_ok) {
        uint8_t *wl = buf + T::oWgt + wave * T::kWgtWave;
#pragma unroll
        for (int rg = 0; rg < 2; rg++) dma16(w.p0 + ((n_tile + rg * 8) * kb + b) * 128, g.wq_off, wl + rg * 1024);
        if (DT == CQ_DTYPE_Q6K) dma16(w.p1 + (n_tile * kb + b) * 64, g.wh_off, wl + 2048);
    }
}

// The small per-block weight fields, loaded straight into registers one block ahead.
template <int DT> struct WHead;
template <> struct WHead<CQ_DTYPE_Q4K> { uint32_t dd; uint4 rec; };   // d | dmin << 16; records {sc, sc, mn, mn} per 32 qs bytes
template <> struct WHead<CQ_DTYPE_Q6K> { uint4 sc; uint32_t d; };   // re-packed scales (two per unit); d
__device__ __forceinline__ void load_head(const cq_weight &w, int64_t blk, WHead<CQ_DTYPE_Q4K> &r) {
    const uint32_t *h = (const uint32_t *)(w.p1 + blk * CQ_Q4K_HDR);
    r.dd = h[0];
    r.rec = make_uint4(h[1], h[2], h[3], h[4]);
}
__device__ __forceinline__ void load_head(const cq_weight &w, int64_t blk, WHead<CQ_DTYPE_Q6K> &r) {
    r.sc = *(const uint4 *)(w.p2 + blk * 16);
    r.d = ((const uint16_t *)w.p3)[blk];
}

// One block for this wave's 16 weight rows against the 2*MT sixteen-row activation tiles in `cur`,
// as a software pipeline: step t issues the MFMAs of tile t (four K-slices x two digits, plus the
// min term), the scaling of the four integers of tile t-2 (VALU) and the LDS reads of tile t+1.
// The accumulator pair rotates through three register sets.  A scheduling barrier after every
// step keeps the compiler from hoisting all MFMAs to the front.
template <int DT, int MT, int SHIFT>
__device__ __forceinline__ void tiles_mac(const uint8_t *cur, const LaneGeo &g, const v4i (&bl)[4], const v4i (&bh)[4],
                                          float dw, v8h wmin, int lane, v4f (&out)[2 * MT]) {
    typedef Tile<DT, MT> T;
    constexpr bool MINS = DT == CQ_DTYPE_Q4K;
    constexpr int NT = 2 * MT;
    const int r = lane & 15, kq = lane >> 4;
    const uint8_t *d8p = cur + T::oD8 + kq * 16;                     // rows 4*kq + [0,4) of a tile
    const uint8_t *mnp = cur + T::oMin + r * 32 + (kq >> 1) * 16;    // piece 1 for kq < 2, piece 2 above
    v4i a[2][4];
    v4f dsc[4];   // read one step ahead, used two steps behind
    v8h ma[2];
    v4i acc_lo[3], acc_hi[3];   // written in step t, read in step t+2, when the MFMAs are long done
    auto load_tile = [&](int t) {
        const uint8_t *base = cur + (t >> 1) * 8192 + (t & 1) * 2048;
#pragma unroll
        for (int s = 0; s < 4; s++) a[t & 1][s] = *(const v4i *)(base + (s >> 1) * 4096 + g.a_col[s & 1]);
        dsc[t % 4] = *(const v4f *)(d8p + t * 64);
        if (MINS) ma[t & 1] = *(const v8h *)(mnp + t * 512);
    };
    load_tile(0);
#pragma unroll
    for (int t = 0; t <= NT + 1; t++) {
        if (t + 1 < NT) load_tile(t + 1);
        if (t < NT) {
            const int p = t & 1, c = t % 3;
            // min term: out -= sum_j (dmin*min_j) * (d8*bsum32_j); the 32 K-slots are the four
            // products of pieces: activation pieces [1,1,2,2] against weight pieces [1,2,1,2]
            if (MINS) out[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ma[p], wmin, out[t], 0, 0, 0);
            const v4i zero = {0, 0, 0, 0};
            acc_lo[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[p][0], bl[0], zero, 0, 0, 0);
            acc_hi[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[p][0], bh[0], zero, 0, 0, 0);
#pragma unroll
            for (int s = 1; s < 4; s++) {
                acc_lo[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[p][s], bl[s], acc_lo[c], 0, 0, 0);
                acc_hi[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[p][s], bh[s], acc_hi[c], 0, 0, 0);
            }
        }
        if (t > 1) {
            const int c = (t - 2) % 3;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int I = (acc_hi[c][i] << SHIFT) + acc_lo[c][i];
                float o = __builtin_fmaf((float)I * dw, dsc[(t - 2) % 4][i], out[t - 2][i]);
                asm volatile("" : "+v"(o));   // pins the scaling to this step (pure ops float otherwise)
                out[t - 2][i] = o;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int MT>
__device__ __forceinline__ void block_mac(const uint8_t *cur, const uint8_t *wl, const LaneGeo &g,
                                          const WHead<CQ_DTYPE_Q4K> &wb, int lane, v4f (&out)[2 * MT]) {
    const uint32_t kq = lane >> 4;
    const float dw = cq_h2f((uint16_t)(wb.dd & 0xffff));
    const float dmin = cq_h2f((uint16_t)(wb.dd >> 16));
    const uint32_t rec[4] = {wb.rec.x, wb.rec.y, wb.rec.z, wb.rec.w};
    // K-slice g = elements 64g..64g+63 = qs bytes 32g..32g+31, low nibbles for the first 32 elements
    // (quarters 0,1: sub-block 2g), high nibbles for the last 32 (quarters 2,3: sub-block 2g+1)
    const uint32_t hi = kq >> 1, nsh = hi * 4;
    v4i bl[4], bh[4];
#pragma unroll
    for (int gi = 0; gi < 4; gi++) {
        const uint4 q = *(const uint4 *)(wl + g.w_col4[gi]);
        const uint32_t sj = (rec[gi] >> (8 * hi)) & 0xff;   // scale of sub-block 2g + hi
        const uint32_t sl = dup16(sj & 7), sh = dup16(sj >> 3);
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t v = (qw[i] >> nsh) & 0x0F0F0F0Fu;
            bl[gi][i] = (int)pk_mul_u16(v, sl);   // low digit of the scale
            bh[gi][i] = (int)pk_mul_u16(v, sh);
        }
    }
    v8h wmin;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float v = -dmin * (float)((rec[j >> 1] >> (16 + 8 * (j & 1))) & 0xff);
        const _Float16 p1 = (_Float16)v;
        wmin[j] = (kq & 1) == 0 ? p1 : (_Float16)(v - (float)p1);
    }
    tiles_mac<CQ_DTYPE_Q4K, MT, 3>(cur, g, bl, bh, dw, wmin, lane, out);
}

template <int MT>
__device__ __forceinline__ void block_mac(const uint8_t *cur, const uint8_t *wl, const LaneGeo &g,
                                          const WHead<CQ_DTYPE_Q6K> &wb, int lane, v4f (&out)[2 * MT]) {
    const uint32_t kq = lane >> 4;
    const float dw = cq_h2f((uint16_t)wb.d);
    v4i bl[4], bh[4];
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
        // K-slices 2hf (low nibbles) and 2hf+1 (high nibbles) of unit u = 4hf + kq: 16 bytes of ql,
        // 8 bytes of re-packed high bits, scale bytes 2u and 2u+1
        const uint4 ql = *(const uint4 *)(wl + g.w_col6[hf]);
        const uint2 qh = *(const uint2 *)(wl + 2048 + g.qh_col[hf]);
        const uint32_t s_even = hf ? wb.sc.z : wb.sc.x, s_odd = hf ? wb.sc.w : wb.sc.y;
        const uint32_t sw = s_even ^ ((s_even ^ s_odd) & (0u - (kq >> 1)));   // word 2hf + kq/2, branch-free
        const uint32_t qw[4] = {ql.x, ql.y, ql.z, ql.w};
        const uint32_t hw[2] = {qh.x, qh.y};
#pragma unroll
        for (int nib = 0; nib < 2; nib++) {
            const int s = 2 * hf + nib;
            const int sc = (int)(int8_t)((sw >> (16 * (kq & 1) + 8 * nib)) & 0xff);
            const uint32_t sc16 = dup16((uint32_t)sc);
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
    }
    v8h wmin = {};
    tiles_mac<CQ_DTYPE_Q6K, MT, 7>(cur, g, bl, bh, dw, wmin, lane, out);
}

// Copies for block b+1 into `nxt`, then the arithmetic of block b out of `cur`.  The two stages
// are distinct (`__restrict__`): without that knowledge the compiler makes every LDS read wait for
// all copies in flight, which would serialise the pipeline.
template <int DT, int MT>
__device__ __forceinline__ void block_step(const uint8_t *__restrict__ cur, uint8_t *__restrict__ nxt,
                                           const cq_weight &w, const cq_act_view &a, const LaneGeo &g, int64_t m0,
                                           int64_t n_tile, bool n_ok, bool more, int64_t b, int wave, int lane,
                                           const WHead<DT> &hcur, v4f (&out)[2 * MT]) {
    typedef Tile<DT, MT> T;
    if (more) stage_issue<DT, MT>(nxt, w, a, g, m0, n_tile, n_ok, b + 1, wave, lane);
    if (n_ok) block_mac<MT>(cur, cur + T::oWgt + wave * T::kWgtWave, g, hcur, lane, out);
}

// ------------------------------------------------------------------ kernel ----
// Requires n % 16 == 0 and an activation workspace with padded rows (cq_act_view::m_stride).
template <int DT, int MT>
__global__ void __launch_bounds__(kThreads) gemm_kernel(cq_weight w, cq_act_view a, int64_t m, float *__restrict__ y,
                                                        int ksplit) {
    typedef Tile<DT, MT> T;
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, kq = lane >> 4;
    const int64_t kb = w.k >> 8;
    const int64_t m0 = (int64_t)blockIdx.y * (MT * 32);
    const int64_t n_tile = ((int64_t)blockIdx.x * kWaves + wave) * kRowsPerWave;
    const bool n_ok = n_tile < w.n;   // wave-uniform; a wave past the last row only helps with the copies
    const int64_t n = n_tile + r;
    const int64_t nc = n_ok ? n : 0;
    // this workgroup's range of K blocks
    const int64_t b0 = kb * blockIdx.z / ksplit, b1 = kb * (blockIdx.z + 1) / ksplit;
    const LaneGeo g = lane_geo(lane, w.k);

    v4f out[2 * MT];
#pragma unroll
    for (int t = 0; t < 2 * MT; t++) out[t] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};

    WHead<DT> hcur, hnxt;
    stage_issue<DT, MT>(smem, w, a, g, m0, n_tile, n_ok, b0, wave, lane);
    load_head(w, nc * kb + b0, hcur);
    hnxt = hcur;
    __builtin_amdgcn_s_waitcnt(0);   // the LDS copies above (and everything else outstanding)
    __syncthreads();

    for (int64_t b = b0; b < b1; b++) {
        const int par = (int)((b - b0) & 1);
        uint8_t *cur = smem + par * T::kBytes;
        uint8_t *nxt = smem + (par ^ 1) * T::kBytes;
        const bool more = b + 1 < b1;
        if (more) load_head(w, nc * kb + b + 1, hnxt);
        block_step<DT, MT>(cur, nxt, w, a, g, m0, n_tile, n_ok, more, b, wave, lane, hcur, out);
        hcur = hnxt;
        __builtin_amdgcn_s_waitcnt(0);   // the next stage has landed in LDS
        __syncthreads();
    }

    if (n_ok) {
#pragma unroll
        for (int t = 0; t < 2 * MT; t++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int64_t row = m0 + t * 16 + kq * 4 + i;
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
    const size_t lds = 2 * Tile<DT, MT>::kBytes;
    static bool attr_set = false;
    if (!attr_set && lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_kernel<DT, MT>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int64_t gx = (w->n + kBN - 1) / kBN, gy = (m + MT * 32 - 1) / (MT * 32);
    // too few workgroups for the machine: split K (at least four blocks per part)
    int ksplit = 1;
    const int64_t kb = w->k >> 8;
    while (gx * gy * ksplit * 2 <= num_cus() && kb / (ksplit * 2) >= 4 && ksplit < 16) ksplit *= 2;
    if (ksplit > 1) {
        hipError_t e = cq_launch_fill_zero(y, m * w->n, s);
        if (e != hipSuccess) return e;
    }
    dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)ksplit);
    CQ_LAUNCH((gemm_kernel<DT, MT>), grid, kThreads, lds, s, *w, a, m, y, ksplit);
    return hipGetLastError();
}

template <int DT>
hipError_t launch_dt(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    if (m <= 32) return launch_mt<DT, 1>(w, a, m, y, s);
    if (m <= 64) return launch_mt<DT, 2>(w, a, m, y, s);
    return launch_mt<DT, 4>(w, a, m, y, s);
}

}  // namespace


bool cq_gemm_supported(const cq_weight *w, int64_t m, int act_dtype) {
    (void)m;
    // the copies address rows with 32-bit offsets: 8 rows of activations, 16 rows of a weight plane
    return (w->dtype == CQ_DTYPE_Q4K || w->dtype == CQ_DTYPE_Q6K) && act_dtype == CQ_DTYPE_Q8K && w->k >= 256 &&
           w->k <= (1 << 24) && w->n % kRowsPerWave == 0;
}

hipError_t cq_launch_gemm(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, hipStream_t s) {
    if (!cq_gemm_supported(w, m, act_dtype)) return hipErrorNotSupported;
    if (m == 0 || w->n == 0) return hipSuccess;
    if (a.m_stride < (m + 127) / 128 * 128) return hipErrorInvalidValue;   // rows the last tile may read
    if (w->dtype == CQ_DTYPE_Q4K) return launch_dt<CQ_DTYPE_Q4K>(w, a, m, y, s);
    return launch_dt<CQ_DTYPE_Q6K>(w, a, m, y, s);
}
