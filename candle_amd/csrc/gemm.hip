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
//   Q6K:  P = sc*(q6-32) (13 bits signed) = 256*ph + pl, pl in [-128, 127];  I = 256*acc_hi + acc_lo
//   Q5K:  as Q4K with 5-bit quants (k_quants.rs:1361-1447): P = sc*q5 (11 bits), split like Q6K's
// I is the same integer as on the CPU.  The Q4K min term is a small f32 contraction over the
// eight sub-blocks; it runs on the f16 MFMA with both factors split in two f16 pieces (products
// exact to ~2^-22) and accumulates straight into the f32 result.
//
// Work split: a workgroup of eight waves (two per SIMD: one wave's scaling arithmetic and LDS
// reads run under the other's MFMAs) covers BM = 32*MT activation rows x 256 weight rows; each wave
// owns 32 weight rows (32x32x32 MFMA, B operand: lane l holds row l%32, k = 16*(l/32)+[0,16) of a
// 32-wide K-slice), unpacks them in registers once per block and reuses them for all BM rows.
// Activations (shared by the waves) and each wave's packed weight bytes go from global memory
// straight into LDS (buffer_load_dwordx4 ... lds), double buffered, one block ahead.  Every such copy
// instruction reads eight whole 128-byte lines (8 rows x 128 B) - the texture path pays per line
// touched - and the 16-byte chunks of a row are XOR-swizzled by the row number on the way in, so
// that the MFMA operand reads (lanes = rows, one chunk column) spread over all LDS banks.  With few
// workgroups (small n) K is split over blockIdx.z and the partial results are added atomically.
#include <type_traits>

#include "qhip_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short us2 __attribute__((ext_vector_type(2)));
typedef short ss2 __attribute__((ext_vector_type(2)));
typedef const void __attribute__((address_space(1))) *gptr_t;
typedef void __attribute__((address_space(3))) *lptr_t;

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;

// LDS image of one pipeline stage:
//   act  : [MT tiles][2 K-halves][4 row groups][8 rows][8 chunks of 16 B]   chunk c of row r sits at c ^ (r%8)
//   d8   : [BM] f32
//   bsh  : [BM][16] f16                      the block's sixteen bsums as f16 (Q4K / Q5K min term)
//   wgt  : per wave: [4 row groups][8 rows][8 chunks] of the 128-byte qs / ql plane (same swizzle),
//          Q6K also [2 row groups][16 rows][4 chunks] of the 64-byte qh plane (chunk c at c ^ ((r/2)%4)),
//          Q5K also [32 rows][32 B] of the fifth-bit plane
constexpr bool is_k4(int dt) { return dt == CQ_DTYPE_Q4K || dt == CQ_DTYPE_Q5K; }   // types with a min term

template <int DT, int MT> struct Tile {
    static constexpr int kAct = MT * 8 * 1024;
    static constexpr int kD8 = (MT * 32 < 64 ? 64 : MT * 32) * 4;   // filled by whole-wave copies of 64 floats
    static constexpr int kMin = is_k4(DT) ? MT * 32 * 32 : 0;
    static constexpr int kWgtWave = DT == CQ_DTYPE_Q4K ? 4096 : DT == CQ_DTYPE_Q5K ? 5120 : 6144;
    static constexpr int oD8 = kAct, oMin = oD8 + kD8;
    static constexpr int kBytes = oMin + kMin;                                  // one activation stage (three of them)
    static constexpr int oWgt = 3 * kBytes;                                     // weights: one buffer per wave
    static constexpr int kTotal = oWgt + kWaves * kWgtWave;
    // two buffers per wave (WBUF == 2): each also takes the 32 rows' block headers (bytes 0..15 at kWgtWave + 16 r,
    // bytes 16..19 at kWgtWave + 512 + 4 r)
    // ... and a fourth activation stage: the copies of block b+2 are issued while block b is contracted
    static constexpr int oHdr = kWgtWave, kSlot2 = kWgtWave + 640;
    static constexpr int oWgt2 = 4 * kBytes;
    static constexpr int kTotal2 = oWgt2 + kWaves * 2 * kSlot2;
};

// both 16-bit halves of `a` times `b` (a splat: the packed instruction takes one half of its operand twice)
__device__ __forceinline__ uint32_t pk_mul_u16(uint32_t a, unsigned short b) {
    const us2 r = __builtin_bit_cast(us2, a) * (us2){b, b};
    return __builtin_bit_cast(uint32_t, r);
}

// Buffer descriptor over `base` (wave-uniform): raw bytes, no stride, no bounds.  The copies below
// are buffer loads rather than global loads on purpose: with a global (FLAT-encoded) LDS copy in
// flight the compiler treats the LDS counter as out of order and turns every wait on an operand
// read into a wait for all of them, which serialises the software-pipelined LDS reads; a buffer
// load leaves the LDS counter alone and takes its per-lane offset without 64-bit vector adds.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_rsrc(const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, -1, 0x00020000);
}

// Asynchronous copy of 64 x 16 (or 64 x 4) bytes: lane l reads base + off and the data lands at
// lds + 16*l (4*l).  `base` and `lds` are wave-uniform.
__device__ __forceinline__ void dma16(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wave_rsrc(base), (lptr_t)lds, 16, (int)off, 0, 0, 0);
}
__device__ __forceinline__ void dma4(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wave_rsrc(base), (lptr_t)lds, 4, (int)off, 0, 0, 0);
}
// the same marked non-temporal: bytes that the launch reads once (a pure read of such a plane runs 10-16 % faster so)
__device__ __forceinline__ void dma16_once(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wave_rsrc(base), (lptr_t)lds, 16, (int)off, 0, 0, 2);
}
// the same 16 bytes further on in both memories (the instruction's immediate offset moves both addresses)
__device__ __forceinline__ void dma4_at16(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wave_rsrc(base), (lptr_t)lds, 4, (int)off, 0, 16, 0);
}

// Per-lane constants of the copies and of the operand reads.
// Q4K / Q5K min term: tiles of up to 64 rows keep it in an accumulator of its own until the integers are scaled; the
// 128-row tiles have no registers for that and let its MFMAs add to the scaled integers themselves (see tiles_mac).
template <int MT> __device__ __host__ constexpr bool min_term_folded() { return MT > 2; }

struct LaneGeo {
    uint32_t act_off;   // copy of 8 rows x 128 B of activations: (l/8)*k + ((l%8) ^ (l/8))*16
    uint32_t wq_off;    // the same over the weights' 128-byte plane: (l/8)*kb*128 + ...
    uint32_t wh_off;    // Q6K qh plane, 16 rows x 64 B: (l/4)*kb*64 + ((l%4) ^ ((l/8)%4))*16
    uint32_t w5_off;    // Q5K fifth-bit plane, 32 rows x 32 B: (l/2)*kb*32 + (l%2)*16
    uint32_t hd_off;    // Q4K / Q5K header plane, the 20 bytes of row l%32: (l%32)*kb*20
    uint32_t col[4];    // operand read: byte offset of chunk 2j+h of row l%32 inside a [4][8][8] x 16 B image
    uint32_t qh_col[4]; // Q6K: byte offset of the 8 bytes of unit 2x+h of row l%32 inside the qh image
};

__device__ __forceinline__ LaneGeo lane_geo(int lane, int64_t k) {
    LaneGeo g;
    const uint32_t kb = (uint32_t)(k >> 8);
    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    g.act_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    g.wq_off = r8 * kb * 128u + ((c8 ^ r8) << 4);
    const uint32_t r16 = lane >> 2, c4 = lane & 3;
    g.wh_off = r16 * kb * 64u + ((c4 ^ ((r16 >> 1) & 3)) << 4);
    g.w5_off = (uint32_t)(lane >> 1) * kb * 32u + (uint32_t)(lane & 1) * 16u;
    g.hd_off = (uint32_t)(lane & 31) * kb * (uint32_t)CQ_Q4K_HDR;
    const uint32_t r = lane & 31, h = lane >> 5;
#pragma unroll
    for (uint32_t j = 0; j < 4; j++) {
        g.col[j] = (r >> 3) * 1024u + (r & 7) * 128u + (((2 * j + h) ^ (r & 7)) << 4);
        g.qh_col[j] = (r >> 4) * 1024u + (r & 15) * 64u + ((j ^ ((r >> 1) & 3)) << 4) + h * 8u;
    }
    return g;
}

// Issues this wave's share of the activation copies for block b into stage `buf`.
template <int DT, int MT>
__device__ __forceinline__ void stage_issue(uint8_t *buf, const cq_weight &w, const cq_act_view &a, const LaneGeo &g,
                                            int64_t m0, int64_t b, int wave, int lane) {
    typedef Tile<DT, MT> T;
    const int64_t k = w.k;
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
    if (is_k4(DT)) {
#pragma unroll
        for (int j = 0; j < MT; j++) {
            if (j + 4 == wave)
                dma16(a.bsh + (b * a.m_stride + m0 + j * 32) * 16, lane * 16u, buf + T::oMin + j * 1024);
        }
    }
}

// This wave's 32 weight rows of block b into its own buffer `wl`.
template <int DT, bool ONCE = false>
__device__ __forceinline__ void stage_weights(uint8_t *wl, const cq_weight &w, const LaneGeo &g, int64_t n_tile,
                                              int64_t b) {
    const int64_t kb = w.k >> 8;
    if (ONCE) {
#pragma unroll
        for (int rg = 0; rg < 4; rg++) dma16_once(w.p0 + ((n_tile + rg * 8) * kb + b) * 128, g.wq_off, wl + rg * 1024);
        if (DT == CQ_DTYPE_Q6K) {
#pragma unroll
            for (int rg = 0; rg < 2; rg++)
                dma16_once(w.p1 + ((n_tile + rg * 16) * kb + b) * 64, g.wh_off, wl + 4096 + rg * 1024);
        }
        if (DT == CQ_DTYPE_Q5K) dma16_once(w.p2 + (n_tile * kb + b) * 32, g.w5_off, wl + 4096);
    } else {
#pragma unroll
        for (int rg = 0; rg < 4; rg++) dma16(w.p0 + ((n_tile + rg * 8) * kb + b) * 128, g.wq_off, wl + rg * 1024);
        if (DT == CQ_DTYPE_Q6K) {
#pragma unroll
            for (int rg = 0; rg < 2; rg++)
                dma16(w.p1 + ((n_tile + rg * 16) * kb + b) * 64, g.wh_off, wl + 4096 + rg * 1024);
        }
        if (DT == CQ_DTYPE_Q5K) dma16(w.p2 + (n_tile * kb + b) * 32, g.w5_off, wl + 4096);
    }
}
// s_waitcnt vmcnt(n) lgkmcnt(0) for a wave-uniform n <= 15 (the instruction takes the count as an immediate).
__device__ __forceinline__ void wait_all_but(int n) {
    switch (n) {
    case 0: __builtin_amdgcn_s_waitcnt(0x0070); break;
    case 1: __builtin_amdgcn_s_waitcnt(0x0071); break;
    case 2: __builtin_amdgcn_s_waitcnt(0x0072); break;
    case 3: __builtin_amdgcn_s_waitcnt(0x0073); break;
    case 4: __builtin_amdgcn_s_waitcnt(0x0074); break;
    case 5: __builtin_amdgcn_s_waitcnt(0x0075); break;
    case 6: __builtin_amdgcn_s_waitcnt(0x0076); break;
    case 7: __builtin_amdgcn_s_waitcnt(0x0077); break;
    case 8: __builtin_amdgcn_s_waitcnt(0x0078); break;
    case 9: __builtin_amdgcn_s_waitcnt(0x0079); break;
    case 10: __builtin_amdgcn_s_waitcnt(0x007A); break;
    case 11: __builtin_amdgcn_s_waitcnt(0x007B); break;
    case 12: __builtin_amdgcn_s_waitcnt(0x007C); break;
    default: __builtin_amdgcn_s_waitcnt(0x0070); break;
    }
}
// Copy instructions one wave issues in stage_issue.
template <int DT, int MT> __device__ __forceinline__ int stage_copies(int wave) {
    return MT * 8 / kWaves + (wave < (MT * 32 + 63) / 64 ? 1 : 0) + (is_k4(DT) && wave >= 4 && wave < 4 + MT ? 1 : 0);
}
// Copy instructions of stage_weights_hdr (the count of its s_waitcnt).
template <int DT> constexpr int weight_copies_hdr() { return 4 + (DT == CQ_DTYPE_Q5K ? 1 : 0) + 2; }
// The same plus the 32 rows' block headers behind the weights (Q4K / Q5K; lanes 0..31).
template <int DT, int MT>
__device__ __forceinline__ void stage_weights_hdr(uint8_t *wl, const cq_weight &w, const LaneGeo &g, int64_t n_tile, int64_t b,
                                                  int lane) {
    typedef Tile<DT, MT> T;
    stage_weights<DT, true>(wl, w, g, n_tile, b);   // (the launches that copy two blocks ahead read their weights once)
    const int64_t kb = w.k >> 8;
    if (lane < 32) {
        const uint8_t *h = w.p1 + (n_tile * kb + b) * CQ_Q4K_HDR;
        dma16(h, g.hd_off, wl + T::oHdr);
        dma4_at16(h, g.hd_off, wl + T::oHdr + 512 - 16);
    }
}

// The small per-block weight fields, loaded straight into registers one block ahead.
template <int DT> struct WHead;
template <> struct WHead<CQ_DTYPE_Q4K> { uint32_t dd; uint4 rec; };   // d | dmin << 16; records {sc, sc, mn, mn} per 32 qs bytes
template <> struct WHead<CQ_DTYPE_Q5K> : WHead<CQ_DTYPE_Q4K> {};     // the same header plane
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
// The header of row l%32 out of the copy stage_weights_hdr made.
__device__ __forceinline__ void head_from_lds(const uint8_t *hd, int lane, WHead<CQ_DTYPE_Q4K> &r) {
    const uint32_t row = lane & 31;
    const uint4 v = *(const uint4 *)(hd + row * 16u);
    r.dd = v.x;
    r.rec = make_uint4(v.y, v.z, v.w, *(const uint32_t *)(hd + 512 + row * 4u));
}
__device__ __forceinline__ void head_from_lds(const uint8_t *, int, WHead<CQ_DTYPE_Q6K> &) {}   // (not used: Q6K keeps one buffer)

// Verification build (DUMP): where a lane's integers of the current block go, and how many of the tile rows exist.
struct DumpLane {
    int32_t *i;     // element (row m0, the lane's weight row, block b) of cq_mfma_dump::i
    float *mn;      // the same of cq_mfma_dump::mn, or null
    int64_t rs;     // elements between two activation rows
    int64_t rows;   // rows m0 .. m0 + rows - 1 exist
    bool int_min;   // mn receives the integer Mn_b (the operands are then the minima themselves), without the activation scale
};

// The weight operand of the Q4K / Q5K min term in its two f16 pieces (cq_min_term_groups): -dmin * min_{j/2} per
// 16-element group j, contracted with the block's sixteen integer sums as f16.  No operand depends on the activations'
// magnitude; the activation block's scale multiplies the sum of main and min term afterwards.
struct MinW {
    v8h p1, p2;
};
// One block for this wave's 32 weight rows against the MT activation tiles in `cur`, as a
// hand-laid software pipeline of 8*(MT+1) steps.  Step (t, s) issues the two int8 MFMAs of tile t,
// K-slice s, and, in their shadow, the scaling of integers of tile t-1 (VALU); LDS reads run ahead.
// The accumulator pair alternates between two register sets.  A scheduling barrier after every step
// keeps the compiler from hoisting all MFMAs to the front, which would need MT accumulator sets at
// once.  Q6K: out += d8 * (I * dw), two elements a step.  Q4K / Q5K: out += d8 * (I * dw - dmin * Mn_b) with the min
// term from two f16 MFMAs (the block's sums against -dmin * min in two pieces, all products exact) -
//   tiles of up to 64 rows: behind the tile's last int8 MFMAs into an accumulator of its own, added where the
//   integers are scaled (steps 1..6 of the next tile);
//   128-row tiles (no registers for that accumulator): step 1 of the next tile turns the integers into I * dw in
//   place - the registers of the high digits are free from then on - and the two MFMAs add to them; steps 2..7
//   multiply by d8.
// DUMP: instead of scaling them into `out`, the block integers I (and the min term as the f16 MFMAs deliver
// it, times d8) are stored through `dl`.
template <int DT, int MT, int T0, int T1, int SHIFT, bool HALF, bool DUMP>
__device__ __forceinline__ void tiles_mac(const uint8_t *cur, const LaneGeo &g, const v4i (&bl)[8], const v4i (&bh)[8],
                                          float dw, const MinW &wmin, int lane, v16f (&out)[MT], const DumpLane &dl) {
    typedef Tile<DT, MT> T;
    if constexpr (T0 >= T1) return;
    constexpr bool MINS = is_k4(DT);
    constexpr bool FOLD = MINS && min_term_folded<MT>();
    constexpr bool UNSCALED = MINS && !FOLD;
    const int h = lane >> 5, col = lane & 31;
    const uint8_t *d8p = cur + T::oD8 + h * 16;        // rows 8j + 4h + [0,4) of a tile
    const uint8_t *mnp = cur + T::oMin + col * 32;     // this lane's row of sums (the min term's activation operand)
    // operand of tile t, K-slice s: chunk 2*(s%4) + h of K-half s/4
    auto afrag = [&](int q) -> v4i {
        const int t = q >> 3, s = q & 7;
        return *(const v4i *)(cur + g.col[s & 3] + (t * 2 + (s >> 2)) * 4096);
    };
    v16i acc_lo[2], acc_hi[2];
    // up to 64 rows: -dmin * Mn_b of the tile being scaled; 128 rows: its I * dw - dmin * Mn_b
    v16f mn = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    v4i a[3];
    v4f dreg[2];   // d8 of four rows each, read two steps before the scaling that needs them
    v8h ma1 = {};   // the block's sums of the tile whose min term comes next (lanes h: sums 8h .. 8h+7)
    a[(T0 * 8) % 3] = afrag(T0 * 8);
    a[(T0 * 8 + 1) % 3] = afrag(T0 * 8 + 1);
#pragma unroll
    for (int q = T0 * 8; q < (T1 + 1) * 8; q++) {
        const int t = q >> 3, s = q & 7;
        if (q + 2 < T1 * 8) a[(q + 2) % 3] = afrag(q + 2);
        if (t < T1) {
            if (s == 0) {
                const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                acc_lo[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q % 3], bl[0], zero, 0, 0, 0);
                acc_hi[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q % 3], bh[0], zero, 0, 0, 0);
            } else {
                acc_lo[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q % 3], bl[s], acc_lo[t & 1], 0, 0, 0);
                acc_hi[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[q % 3], bh[s], acc_hi[t & 1], 0, 0, 0);
            }
            if (s == 6) dreg[0] = *(const v4f *)(d8p + (t * 32) * 4);
            // UNSCALED: this tile's own min term, -dmin * sum_j bsums_j * min_{j/2} from a zero accumulator (lanes h:
            // sums 8h .. 8h+7), behind its last MFMAs; it is added where the integers are scaled, one tile later
            if (s == 6 && UNSCALED) ma1 = *(const v8h *)(mnp + t * 1024 + h * 16);
            if (s == 7 && UNSCALED && (!DUMP || dl.mn)) {
                const v16f zf = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                mn = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma1, wmin.p1, zf, 0, 0, 0);
                mn = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma1, wmin.p2, mn, 0, 0, 0);
            }
        }
        if (t > T0 && !MINS) {
            // scaling of two of the sixteen integers of tile t-1 per step (element i: rows 8*(i/4) + 4h + i%4)
            const int p = (t - 1) & 1;
            if ((s & 1) == 0 && s < 6) dreg[((s >> 1) + 1) & 1] = *(const v4f *)(d8p + ((t - 1) * 32 + 8 * ((s >> 1) + 1)) * 4);
#pragma unroll
            for (int i = 2 * s; i < 2 * s + 2; i++) {
                if (HALF && i >= 8) continue;   // rows 16..31 of the tile are not wanted
                const int I = (acc_hi[p][i] << SHIFT) + acc_lo[p][i];
                if (DUMP) {
                    const int64_t row = (t - 1) * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                    if (row < dl.rows) dl.i[row * dl.rs] = I;
                    continue;
                }
                float o = __builtin_fmaf((float)I * dw, dreg[(i >> 2) & 1][i & 3], out[t - 1][i]);
                asm volatile("" : "+v"(o));   // pins the scaling to this step (pure ops float otherwise)
                out[t - 1][i] = o;
            }
        }
        if (t < T1 && s == 7 && FOLD) ma1 = *(const v8h *)(mnp + t * 1024 + h * 16);   // this tile's sums, for step 1 of the next
        if (t > T0 && FOLD) {
            // 128-row tiles: step 1 turns the sixteen integers of tile t-1 into I * dw in place (the registers of the high
            // digits are free from then on) and lets the min term's two MFMAs add to them; steps 2..7 multiply by d8
            const int p = (t - 1) & 1;
            if (s == 1) {
                if (DUMP) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int64_t row = (t - 1) * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                        if (row < dl.rows && !(HALF && i >= 8)) dl.i[row * dl.rs] = (acc_hi[p][i] << SHIFT) + acc_lo[p][i];
                    }
                    if (dl.mn) {
                        v16f m0 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                        m0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma1, wmin.p1, m0, 0, 0, 0);
                        m0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma1, wmin.p2, m0, 0, 0, 0);
#pragma unroll
                        for (int i = 0; i < 16; i++) {
                            const int64_t row = (t - 1) * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                            if (row < dl.rows) dl.mn[row * dl.rs] = dl.int_min ? m0[i] : m0[i] * *(const float *)(d8p + ((t - 1) * 32 + 8 * (i >> 2) + (i & 3)) * 4);
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 16; i++) mn[i] = (float)((acc_hi[p][i] << SHIFT) + acc_lo[p][i]) * dw;
                    __builtin_amdgcn_sched_barrier(0);
                    mn = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma1, wmin.p1, mn, 0, 0, 0);
                    mn = __builtin_amdgcn_mfma_f32_32x32x16_f16(ma1, wmin.p2, mn, 0, 0, 0);
                }
                dreg[1] = *(const v4f *)(d8p + ((t - 1) * 32 + 8) * 4);
            }
            if (s >= 2 && !DUMP) {
                const int i0 = s < 6 ? 3 * (s - 2) : 12 + 2 * (s - 6), i1 = s < 6 ? i0 + 3 : i0 + 2;
#pragma unroll
                for (int i = i0; i < i1; i++) {
                    if (!(HALF && i >= 8)) {
                        float o = __builtin_fmaf(mn[i], dreg[(i >> 2) & 1][i & 3], out[t - 1][i]);
                        asm volatile("" : "+v"(o));   // pins the scaling to this step (pure ops float otherwise)
                        out[t - 1][i] = o;
                    }
                    if (i == 3) dreg[0] = *(const v4f *)(d8p + ((t - 1) * 32 + 16) * 4);
                    if (i == 7) dreg[1] = *(const v4f *)(d8p + ((t - 1) * 32 + 24) * 4);
                }
            }
        }
        if (t > T0 && UNSCALED) {
            // the same in steps 1..6 (the min term's MFMAs were the last of tile t-1, and this tile's follow in step 7
            // into the same registers): three elements a step, then two; out += d8 * (I * dw + min term)
            const int p = (t - 1) & 1;
            if (s == 0) {
                dreg[1] = *(const v4f *)(d8p + ((t - 1) * 32 + 8) * 4);
                if (DUMP && dl.mn) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int64_t row = (t - 1) * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                        // (stored with the activation scale, like the 128-row tiles' term)
                        if (row < dl.rows) dl.mn[row * dl.rs] = dl.int_min ? mn[i] : mn[i] * *(const float *)(d8p + ((t - 1) * 32 + 8 * (i >> 2) + (i & 3)) * 4);
                    }
                }
            }
            if (s >= 1 && s <= 6) {
                const int i0 = s < 5 ? 3 * (s - 1) : 12 + 2 * (s - 5), i1 = s < 5 ? i0 + 3 : i0 + 2;
#pragma unroll
                for (int i = i0; i < i1; i++) {
                    if (!(HALF && i >= 8)) {   // (HALF: rows 16..31 of the tile are not wanted)
                        const int I = (acc_hi[p][i] << SHIFT) + acc_lo[p][i];
                        if (DUMP) {
                            const int64_t row = (t - 1) * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                            if (row < dl.rows) dl.i[row * dl.rs] = I;
                        } else {
                            float o = __builtin_fmaf(__builtin_fmaf((float)I, dw, mn[i]), dreg[(i >> 2) & 1][i & 3], out[t - 1][i]);
                            asm volatile("" : "+v"(o));   // pins the scaling to this step (pure ops float otherwise)
                            out[t - 1][i] = o;
                        }
                    }
                    // the d8 of rows 16.. and 24.. follow their buffers' last use (elements 3 and 7)
                    if (i == 3) dreg[0] = *(const v4f *)(d8p + ((t - 1) * 32 + 16) * 4);
                    if (i == 7) dreg[1] = *(const v4f *)(d8p + ((t - 1) * 32 + 24) * 4);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Weight operands of one block: unpacks the wave's 32 rows from `wl` into the two digit operands
// of the eight K-slices, and returns the block scale (and the Q4K min-term operand).
__device__ __forceinline__ void block_unpack(const uint8_t *wl, const LaneGeo &g, const WHead<CQ_DTYPE_Q4K> &wb,
                                             int lane, v4i (&bl)[8], v4i (&bh)[8], float &dw, MinW &wmin) {
    const int h = lane >> 5;
    dw = cq_h2f((uint16_t)(wb.dd & 0xffff));
    const uint32_t rec[4] = {wb.rec.x, wb.rec.y, wb.rec.z, wb.rec.w};   // {sc[2g], sc[2g+1], mn[2g], mn[2g+1]}
#pragma unroll
    for (int gi = 0; gi < 4; gi++) {
        // qs bytes 32g + 16h + [0,16): low nibbles = K-slice 2g, high nibbles = slice 2g+1
        const uint4 q = *(const uint4 *)(wl + g.col[gi]);
        const unsigned short sl0 = (unsigned short)(rec[gi] & 7), sh0 = (unsigned short)((rec[gi] >> 3) & 31);
        const unsigned short sl1 = (unsigned short)((rec[gi] >> 8) & 7), sh1 = (unsigned short)((rec[gi] >> 11) & 31);
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t lo4 = qw[i] & 0x0F0F0F0Fu, hi4 = (qw[i] >> 4) & 0x0F0F0F0Fu;
            bl[2 * gi][i] = (int)pk_mul_u16(lo4, sl0);       // sub-block 2g, low digit of the scale
            bh[2 * gi][i] = (int)pk_mul_u16(lo4, sh0);
            bl[2 * gi + 1][i] = (int)pk_mul_u16(hi4, sl1);   // sub-block 2g+1
            bh[2 * gi + 1][i] = (int)pk_mul_u16(hi4, sh1);
        }
    }
    wmin.p1 = __builtin_bit_cast(v8h, cq_min_term_groups(wb.dd, rec, h != 0, false));
    wmin.p2 = __builtin_bit_cast(v8h, cq_min_term_groups(wb.dd, rec, h != 0, true));
}

// Q5K: the Q4K nibbles plus a fifth bit per quant (words {L, H} per 32 qs bytes, bit 8c + i for byte c
// of qs word i); scale times quant has up to 11 bits and is split as Q6K's products are.
__device__ __forceinline__ void block_unpack(const uint8_t *wl, const LaneGeo &g, const WHead<CQ_DTYPE_Q5K> &wb,
                                             int lane, v4i (&bl)[8], v4i (&bh)[8], float &dw, MinW &wmin) {
    const int h = lane >> 5;
    const uint32_t row = lane & 31;
    dw = cq_h2f((uint16_t)(wb.dd & 0xffff));
    const uint32_t rec[4] = {wb.rec.x, wb.rec.y, wb.rec.z, wb.rec.w};   // {sc[2g], sc[2g+1], mn[2g], mn[2g+1]}
    const uint4 f0 = *(const uint4 *)(wl + 4096 + row * 32u), f1 = *(const uint4 *)(wl + 4096 + row * 32u + 16u);
    const uint32_t fl[4] = {f0.x, f0.z, f1.x, f1.z}, fh[4] = {f0.y, f0.w, f1.y, f1.w};
#pragma unroll
    for (int gi = 0; gi < 4; gi++) {
        // qs bytes 32g + 16h + [0,16) = qs words 4h .. 4h+3: low nibbles = K-slice 2g, high nibbles = slice 2g+1
        const uint4 q = *(const uint4 *)(wl + g.col[gi]);
        const unsigned short s0 = (unsigned short)(rec[gi] & 0xff), s1 = (unsigned short)((rec[gi] >> 8) & 0xff);
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t lo5 = (qw[i] & 0x0F0F0F0Fu) | (((fl[gi] >> (4 * h + i)) & 0x01010101u) << 4);
            const uint32_t hi5 = ((qw[i] >> 4) & 0x0F0F0F0Fu) | (((fh[gi] >> (4 * h + i)) & 0x01010101u) << 4);
            int lo, hi;
            cq_scaled_digits(lo5, s0, (unsigned short)128, lo, hi);   // digits of sc * q5, sub-block 2g
            bl[2 * gi][i] = lo;
            bh[2 * gi][i] = hi;
            cq_scaled_digits(hi5, s1, (unsigned short)128, lo, hi);   // sub-block 2g+1
            bl[2 * gi + 1][i] = lo;
            bh[2 * gi + 1][i] = hi;
        }
    }
    wmin.p1 = __builtin_bit_cast(v8h, cq_min_term_groups(wb.dd, rec, h != 0, false));
    wmin.p2 = __builtin_bit_cast(v8h, cq_min_term_groups(wb.dd, rec, h != 0, true));
}

__device__ __forceinline__ void block_unpack(const uint8_t *wl, const LaneGeo &g, const WHead<CQ_DTYPE_Q6K> &wb,
                                             int lane, v4i (&bl)[8], v4i (&bh)[8], float &dw, MinW &wmin) {
    const int h = lane >> 5;
    dw = cq_h2f((uint16_t)wb.d);
    const uint32_t scw[4] = {wb.sc.x, wb.sc.y, wb.sc.z, wb.sc.w};
    uint4 ql[4];
    uint2 qhv[4];
#pragma unroll
    for (int x = 0; x < 4; x++) {
        // ql lane of unit u = 2x + h and its re-packed high bits
        ql[x] = *(const uint4 *)(wl + g.col[x]);
        qhv[x] = *(const uint2 *)(wl + 4096 + g.qh_col[x]);
    }
#pragma unroll
    for (int s = 0; s < 8; s++) {
        // K-slice s: this lane's 16 elements are the group G = 2s + h, i.e. unit u = 2x + h with
        // x = 2*(s/4) + s%2, low nibbles when (s%4) < 2 else high nibbles
        const int x = 2 * (s >> 2) + (s & 1), nib = (s & 3) >> 1;
        const int sb = 4 * x + nib;                  // scale byte index for h = 0; h adds 2 (same word)
        const uint32_t sw = scw[sb >> 2];
        const int sc = (int)(int8_t)((sw >> (8 * (sb & 3) + 16 * h)) & 0xff);
        const unsigned short sc16 = (unsigned short)sc, c16 = (unsigned short)(128 - 32 * sc);
        const uint32_t qw[4] = {ql[x].x, ql[x].y, ql[x].z, ql[x].w};
        const uint32_t hw[2] = {qhv[x].x, qhv[x].y};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t H = hw[i >> 1];
            const int sh = (i & 1) * 4 + 2 * nib;   // where the two high bits sit in H's bytes; wanted at bit 4
            const uint32_t hb = sh < 4 ? H << (4 - sh) : H >> (sh - 4);
            const uint32_t q6 = ((qw[i] >> (4 * nib)) & 0x0F0F0F0Fu) | (hb & 0x30303030u);
            int lo, hi;
            cq_scaled_digits(q6, sc16, c16, lo, hi);   // digits of sc * (q6 - 32)
            bl[s][i] = lo;
            bh[s][i] = hi;
        }
    }
    wmin = MinW{};
}

// One K block of one wave.  The two waves of a SIMD (waves w and w + 4 of the workgroup) run half a
// block apart: a leading wave unpacks block b, contracts all of its tiles and meets the others at
// the block barrier; a trailing wave goes through the barrier after the lower half of the tiles and
// contracts the upper half behind it, while the leading waves already unpack block b+1.  The
// unpacking is pure VALU work and the contraction mostly MFMA, so one wave's unpacking runs under
// the other's MFMAs instead of both alternating between the two in lockstep.  Activations
// therefore live in three stages: block b+1 lands in `nxt` while block b is read from `cur` and the
// trailing waves may still read block b-1.  The wave's weight bytes of block b come out of `wl`,
// which is refilled for block b+1 as soon as they are in registers.  The LDS regions are distinct
// (`__restrict__`): without that knowledge the compiler makes every LDS read wait for all copies in
// flight, which would serialise the pipeline.
// `more`: the block whose copies this step issues exists (b+1; b+2 when WBUF == 2).
// WBUF == 2 (a launch whose weights come cold from HBM, a few activation rows per weight row: a block takes less time
// than a copy): everything is copied two blocks ahead.  Two weight buffers per wave - the buffer block b has just been
// unpacked from takes block b+2 - and four activation stages; the copies of block b+2 stay in flight across the barrier
// (the waits are written out: everything but those copies).  The block headers then come through the same copies -
// a load into registers would be tracked by the compiler, which on joining the paths "copies issued" / "no block left"
// waits as the stricter of the two demands, i.e. for the copies just issued.
template <int DT, int MT, bool TRAIL, bool HALF, bool DUMP, int WBUF, bool ONCE>
__device__ __forceinline__ void block_step(const uint8_t *__restrict__ cur, uint8_t *__restrict__ nxt,
                                           uint8_t *__restrict__ wl, const cq_weight &w, const cq_act_view &a,
                                           const LaneGeo &g, int64_t m0, int64_t n_tile, bool n_ok, bool more, int64_t b,
                                           int wave, int lane, const WHead<DT> &hreg, v16f (&out)[MT], const DumpLane &dl) {
    constexpr int SHIFT = DT == CQ_DTYPE_Q4K ? 3 : 8;
    constexpr int SPLIT = TRAIL ? MT / 2 : MT;   // tiles [SPLIT, MT) follow the barrier
    v4i bl[8], bh[8];
    float dw = 0.0f;
    MinW wmin = {};
    if (more) stage_issue<DT, MT>(nxt, w, a, g, m0, b + (WBUF == 2 ? 2 : 1), wave, lane);
    if (n_ok) {
        WHead<DT> hcur = hreg;
        if (WBUF == 2) head_from_lds(wl + Tile<DT, MT>::oHdr, lane, hcur);
        block_unpack(wl, g, hcur, lane, bl, bh, dw, wmin);
        if constexpr (DUMP && is_k4(DT)) {
            if (dl.int_min) {   // verification: the minima themselves as the operand, so the MFMAs deliver the integer Mn_b
                const uint32_t rec[4] = {hcur.rec.x, hcur.rec.y, hcur.rec.z, hcur.rec.w};
                wmin.p1 = __builtin_bit_cast(v8h, cq_min_term_groups_int(rec, (lane >> 5) != 0, false));
                wmin.p2 = __builtin_bit_cast(v8h, cq_min_term_groups_int(rec, (lane >> 5) != 0, true));
            }
        }
        if (WBUF == 2) {
            if (more) {
                __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the reads above are done with the buffer
                stage_weights_hdr<DT, MT>(wl, w, g, n_tile, b + 2, lane);
            }
        } else if (more) {
            stage_weights<DT, ONCE>(wl, w, g, n_tile, b + 1);
        }
        tiles_mac<DT, MT, 0, SPLIT, SHIFT, HALF, DUMP>(cur, g, bl, bh, dw, wmin, lane, out, dl);
    }
    if (WBUF == 2) {
        // the next stage and the weights of block b+1 have landed; the copies of block b+2 may still be in flight
        // (the empty statements keep the compiler from moving LDS reads and copies across the barrier, which by itself
        // orders nothing for it)
        wait_all_but(more ? stage_copies<DT, MT>(wave) + (n_ok ? weight_copies_hdr<DT>() : 0) : 0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    } else {
        __builtin_amdgcn_s_waitcnt(0);   // the next stage and the wave's next weights have landed in LDS
        __syncthreads();
    }
    if (TRAIL && n_ok) tiles_mac<DT, MT, SPLIT, MT, SHIFT, HALF, DUMP>(cur, g, bl, bh, dw, wmin, lane, out, dl);
}

// ------------------------------------------------------------------ kernel ----
// Requires n % 32 == 0 and an activation workspace with padded rows (cq_act_view::m_stride).
// One workgroup: activation rows [m0, m0 + 32*MT) (stored up to row m - 1) x the 256 weight rows of
// blockIdx.x, K blocks of part blockIdx.z.
template <int DT, int MT, bool DUMP = false, int WBUF = 1, bool ONCE = false>
__device__ __forceinline__ void gemm_body(const cq_weight &w, const cq_act_view &a, int64_t m0, int64_t m,
                                          float *__restrict__ y, int ksplit, cq_mfma_dump dump = cq_mfma_dump{nullptr, nullptr, 0}) {
    static_assert(WBUF == 1 || DT == CQ_DTYPE_Q4K || DT == CQ_DTYPE_Q5K, "block headers of 20 bytes");
    typedef Tile<DT, MT> T;
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, col = lane & 31;
    const int64_t kb = w.k >> 8;
    const int64_t n_tile = ((int64_t)blockIdx.x * kWaves + wave) * 32;
    const bool n_ok = n_tile < w.n;   // wave-uniform; a wave past the last row only helps with the copies
    const int64_t n = n_tile + col;
    const int64_t nc = n_ok ? n : 0;
    // this workgroup's range of K blocks
    const int64_t b0 = kb * blockIdx.z / ksplit, b1 = kb * (blockIdx.z + 1) / ksplit;
    const LaneGeo g = lane_geo(lane, w.k);

    v16f out[MT];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) out[t][i] = 0.0f;

    WHead<DT> hcur = {}, hnxt = {};
    uint8_t *wl = WBUF == 2 ? smem + T::oWgt2 + wave * 2 * T::kSlot2 : smem + T::oWgt + wave * T::kWgtWave;
    stage_issue<DT, MT>(smem, w, a, g, m0, b0, wave, lane);
    if (WBUF == 2) {
        if (b0 + 1 < b1) stage_issue<DT, MT>(smem + T::kBytes, w, a, g, m0, b0 + 1, wave, lane);
        if (n_ok) {
            stage_weights_hdr<DT, MT>(wl, w, g, n_tile, b0, lane);
            if (b0 + 1 < b1) stage_weights_hdr<DT, MT>(wl + T::kSlot2, w, g, n_tile, b0 + 1, lane);
        }
    } else {
        if (n_ok) stage_weights<DT, ONCE>(wl, w, g, n_tile, b0);
        load_head(w, nc * kb + b0, hcur);
        hnxt = hcur;
    }
    __builtin_amdgcn_s_waitcnt(0);   // the LDS copies above (and everything else outstanding)
    __syncthreads();

    // Stage of block b: (b - b0) % 3 (% 4 when WBUF == 2); `in` is the stage this step's copies go to.  Both loops pass
    // the same number of barriers.
    int ic = 0, in = WBUF == 2 ? 2 : 1, ifree = WBUF == 2 ? 3 : 2, imid = 1;
    auto rotate = [&]() {
        const int t = ic;
        if (WBUF == 2) {
            ic = imid;
            imid = in;
        } else {
            ic = in;
        }
        in = ifree;
        ifree = t;
    };
    auto run = [&](auto trail, auto half) {
        for (int64_t b = b0; b < b1; b++) {
            const bool more = b + (WBUF == 2 ? 2 : 1) < b1;
            if (WBUF == 1 && more) load_head(w, nc * kb + b + 1, hnxt);
            DumpLane dl{nullptr, nullptr, 0, 0, false};
            if (DUMP) {
                const int64_t at = (m0 * w.n + nc) * kb + b;
                dl = DumpLane{dump.i + at, dump.mn ? dump.mn + at : nullptr, w.n * kb, m - m0, dump.int_min != 0};
            }
            uint8_t *wb = WBUF == 2 ? wl + ((b - b0) & 1) * T::kSlot2 : wl;   // the buffer that holds block b
            block_step<DT, MT, decltype(trail)::value, decltype(half)::value, DUMP, WBUF, ONCE>(smem + ic * T::kBytes, smem + in * T::kBytes,
                                                                                          wb, w, a, g, m0, n_tile, n_ok, more, b,
                                                                                          wave, lane, hcur, out, dl);
            hcur = hnxt;
            rotate();
        }
    };
    // a single 32-row tile of which at most 16 rows exist (an expert with few tokens): the scaling of
    // the other half of the accumulators is skipped
    const bool half = MT == 1 && m - m0 <= 16;
    using T_ = std::true_type;
    using F_ = std::false_type;
    if (wave < kWaves / 2) {
        if (MT == 1 && half) run(F_{}, std::integral_constant<bool, MT == 1>{});
        else run(F_{}, F_{});
    } else {
        if (MT == 1 && half) run(T_{}, std::integral_constant<bool, MT == 1>{});
        else run(T_{}, F_{});
    }

    if (n_ok && !DUMP) {
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

template <int DT, int MT>
__global__ void __launch_bounds__(kThreads) gemm_kernel(cq_weight w, cq_act_view a, int64_t m, float *__restrict__ y,
                                                        int ksplit) {
    gemm_body<DT, MT>(w, a, (int64_t)blockIdx.y * (MT * 32), m, y, ksplit);
}

// Up to 32 activation rows (one row tile): every weight byte is read once by the launch, cold - the form of the grouped
// expert launches (copies marked non-temporal; Q4K / Q5K: everything two blocks ahead).
template <int DT> constexpr int once_wbuf() { return DT == CQ_DTYPE_Q4K || DT == CQ_DTYPE_Q5K ? 2 : 1; }
template <int DT>
__global__ void __launch_bounds__(kThreads) gemm_once_kernel(cq_weight w, cq_act_view a, int64_t m, float *__restrict__ y,
                                                             int ksplit) {
    gemm_body<DT, 1, false, once_wbuf<DT>(), true>(w, a, 0, m, y, ksplit);
}

// The same launch with the block integers stored instead of the result (verification).
template <int DT, int MT>
__global__ void __launch_bounds__(kThreads) gemm_dump_kernel(cq_weight w, cq_act_view a, int64_t m, int ksplit,
                                                             cq_mfma_dump dump) {
    gemm_body<DT, MT, true>(w, a, (int64_t)blockIdx.y * (MT * 32), m, nullptr, ksplit, dump);
}

// ------------------------------------------------------ few weight rows, long K: K halved inside the workgroup ----
// With few 256-row column tiles (n = 4096: sixteen) the launches above fill the machine either with 32-row tiles, which
// unpack every weight block once per 32 activation rows, or by splitting K over workgroups, whose parts are added to
// the output atomically (about 1.1 TB/s, and the order of the sum is not fixed).  Here a workgroup covers 128 weight
// rows x 32*MT activation rows and halves K between its waves: waves 0..3 (one per SIMD) take the first half of the K
// blocks for their 32 weight rows, waves 4..7 the second half for the same rows - a SIMD's two waves are again half a
// step apart in what they do, the leading and trailing roles of gemm_body - and the two partial tiles meet in LDS at
// the end, first half + second half: twice the workgroups at the same tile height, no atomics, a fixed order.
// Stage layout: two activation parts per stage (the block of each half), Tile::kBytes each.
template <int DT, int MT> struct TileKH {
    typedef Tile<DT, MT> T;
    static constexpr int kStage = 2 * T::kBytes;
    static constexpr int oWgt = 3 * kStage;
    static constexpr int kTotal = oWgt + kWaves * T::kWgtWave;
    static_assert(MT * 16 * 256 * (kWaves / 2) <= oWgt, "the partial tiles of the second half fit the stages");
};

template <int DT, int MT, bool TRAIL>
__device__ __forceinline__ void block_step_kh(const uint8_t *__restrict__ cur, uint8_t *__restrict__ nxt, uint8_t *__restrict__ wl,
                                              const cq_weight &w, const cq_act_view &a, const LaneGeo &g, int64_t m0, int64_t n_tile,
                                              bool work, int64_t next0, int64_t next1, int64_t mine_next, int wave, int lane,
                                              const WHead<DT> &hcur, v16f (&out)[MT]) {
    typedef Tile<DT, MT> T;
    constexpr int SHIFT = DT == CQ_DTYPE_Q4K ? 3 : 8;
    constexpr int SPLIT = TRAIL ? MT / 2 : MT;   // tiles [SPLIT, MT) follow the barrier
    const DumpLane dl{nullptr, nullptr, 0, 0, false};
    v4i bl[8], bh[8];
    float dw = 0.0f;
    MinW wmin = {};
    if (next0 >= 0) stage_issue<DT, MT>(nxt, w, a, g, m0, next0, wave, lane);
    if (next1 >= 0) stage_issue<DT, MT>(nxt + T::kBytes, w, a, g, m0, next1, wave, lane);
    if (work) {
        block_unpack(wl, g, hcur, lane, bl, bh, dw, wmin);
        if (mine_next >= 0) stage_weights<DT>(wl, w, g, n_tile, mine_next);
        tiles_mac<DT, MT, 0, SPLIT, SHIFT, false, false>(cur, g, bl, bh, dw, wmin, lane, out, dl);
    }
    __builtin_amdgcn_s_waitcnt(0);   // the next stage and the wave's next weights have landed in LDS
    __syncthreads();
    if (TRAIL && work) tiles_mac<DT, MT, SPLIT, MT, SHIFT, false, false>(cur, g, bl, bh, dw, wmin, lane, out, dl);
}

// Requires n % 32 == 0.  One workgroup: activation rows [m0, m0 + 32*MT) x the 128 weight rows of blockIdx.x, all K.
template <int DT, int MT>
__global__ void __launch_bounds__(kThreads) gemm_kh_kernel(cq_weight w, cq_act_view a, int64_t m, float *__restrict__ y) {
    typedef Tile<DT, MT> T;
    typedef TileKH<DT, MT> TK;
    extern __shared__ __align__(16) uint8_t smem[];
    const int64_t m0 = (int64_t)blockIdx.y * (MT * 32);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int colw = wave & 3, half = wave >> 2;
    const int h = lane >> 5, col = lane & 31;
    const int64_t kb = w.k >> 8;
    const int64_t n_tile = ((int64_t)blockIdx.x * (kWaves / 2) + colw) * 32;
    const bool n_ok = n_tile < w.n;
    const int64_t n = n_tile + col;
    const int64_t nc = n_ok ? n : 0;
    const int64_t nh = (kb + 1) / 2;                        // steps; the first half has nh blocks, the second kb - nh
    const int64_t first = half ? nh : 0, count = half ? kb - nh : nh;
    const LaneGeo g = lane_geo(lane, w.k);

    v16f out[MT];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) out[t][i] = 0.0f;

    WHead<DT> hcur = {}, hnxt = {};
    uint8_t *wl = smem + TK::oWgt + wave * T::kWgtWave;
    stage_issue<DT, MT>(smem, w, a, g, m0, 0, wave, lane);
    if (kb - nh > 0) stage_issue<DT, MT>(smem + T::kBytes, w, a, g, m0, nh, wave, lane);
    if (n_ok && count > 0) {
        stage_weights<DT>(wl, w, g, n_tile, first);
        load_head(w, nc * kb + first, hcur);
    }
    hnxt = hcur;
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    int ic = 0, in = 1, ifree = 2;
    for (int64_t it = 0; it < nh; it++) {
        const bool work = n_ok && it < count;
        const int64_t next0 = it + 1 < nh ? it + 1 : -1, next1 = it + 1 < kb - nh ? nh + it + 1 : -1;
        const int64_t mine_next = it + 1 < count ? first + it + 1 : -1;
        if (n_ok && mine_next >= 0) load_head(w, nc * kb + mine_next, hnxt);
        const uint8_t *cur = smem + ic * TK::kStage + half * T::kBytes;
        uint8_t *nxt = smem + in * TK::kStage;
        if (half == 0) block_step_kh<DT, MT, false>(cur, nxt, wl, w, a, g, m0, n_tile, work, next0, next1, mine_next, wave, lane, hcur, out);
        else block_step_kh<DT, MT, true>(cur, nxt, wl, w, a, g, m0, n_tile, work, next0, next1, mine_next, wave, lane, hcur, out);
        hcur = hnxt;
        const int t = ic;
        ic = in;
        in = ifree;
        ifree = t;
    }

    // ---- first half + second half through LDS (the stages are free: every wave is past its last read)
    __syncthreads();
    float *part = (float *)smem + (size_t)colw * (MT * 16 * 64);
    if (half == 1) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) part[(t * 16 + i) * 64 + lane] = out[t][i];
    }
    __syncthreads();
    if (half == 0 && n_ok) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t row = m0 + t * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                if (row < m) y[row * w.n + n] = out[t][i] + part[(t * 16 + i) * 64 + lane];
            }
        }
    }
}

// Grouped (mixture-of-experts) variant: one launch for every expert.  blockIdx.y walks a table of
// 32-row tiles of the expert-sorted activation rows; each tile names its expert's weights.
constexpr int kMaxGroupExperts = 16, kMaxGroupTiles = 96;
struct GroupArgs {
    cq_weight w[kMaxGroupExperts];
    int32_t row0[kMaxGroupTiles];      // first activation row of the tile
    int32_t row_end[kMaxGroupTiles];   // end of its expert's rows
    int8_t expert[kMaxGroupTiles];
};

// Expert weights are read once per launch, cold: the types whose headers can come through the copies take two buffers.
template <int DT> constexpr int grouped_wbuf() { return DT == CQ_DTYPE_Q4K || DT == CQ_DTYPE_Q5K ? 2 : 1; }
template <int DT>
__global__ void __launch_bounds__(kThreads) gemm_grouped_kernel(GroupArgs ga, cq_act_view a, float *__restrict__ y,
                                                                int ksplit) {
    const int tile = blockIdx.y;
    const cq_weight w = ga.w[ga.expert[tile]];
    gemm_body<DT, 1, false, grouped_wbuf<DT>(), true>(w, a, ga.row0[tile], ga.row_end[tile], y, ksplit);
}

// ------------------------------------------------ K-quant weights x Q8_1 activations (tile kernel) ----
// The formulation of the reference's CUDA arm (mul_mat_via_q8_1, quantized/cuda.rs:298-365; dot bodies
// candle-kernels/src/quantized.cu:2141-2166 for Q4K, :2258-2281 for Q6K) on the matrix cores, activations quantized
// by the CPU rule of BlockQ8_1::from_float (k_quants.rs:665-691).  Per 32-element Q8_1 block j of a weight block
//   Q4K:  (d * sc_j) * d8_j * dot_j  -  (dmin * m_j) * s8_j          dot_j = sum_32 q4 * q8
//   Q6K:  d * d8_j * (sc_g * dot_g + sc_g' * dot_g')                 g, g' the two 16-element groups of block j
// A Q8_1 block is one K-slice of the 32x32x32 int8 MFMA, so dot_j is one result element (Q6K: the two-digit operands
// of the Q8K kernel above give sc_g * dot_g + sc_g' * dot_g' as 256 * hi + lo).  Its scale is an outer product
// (weight row factor x activation row factor): a bf16 MFMA lays it out in the accumulator layout, the weight factor
// (17 significant bits) as three bf16 pieces, the activation factor (an f16 value) as two, all six products exact.
// The Q4K min term is one f16 MFMA per tile and weight block: s8 is an f16, dmin * m_j goes in as two f16 pieces.
// Work split, LDS images and copies as in the Q8K kernel; two activation stages, the waves in step.
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

template <int DT, int MT> struct Tile81 {
    static constexpr int kAct = MT * 8 * 1024;
    static constexpr int kD8 = MT * 32 * 32;                                 // [32*MT rows][8 blocks] f32
    static constexpr int kS8 = DT == CQ_DTYPE_Q4K ? (MT < 2 ? 2 : MT) * 32 * 16 : 0;   // [32*MT rows][8 blocks] f16, whole 64-row copies
    static constexpr int oD8 = kAct, oS8 = oD8 + kD8;
    static constexpr int kStage = oS8 + kS8;
    static constexpr int kWgtWave = DT == CQ_DTYPE_Q4K ? 4096 : 6144;
    static constexpr int oWgt = 2 * kStage;
    static constexpr int kTotal = oWgt + kWaves * kWgtWave;
};

template <int DT, int MT>
__device__ __forceinline__ void stage_acts81(uint8_t *buf, const cq_act_view &a, const LaneGeo &g, int64_t k, int64_t m0,
                                             int64_t b, int wave, int lane) {
    typedef Tile81<DT, MT> T;
#pragma unroll
    for (int j = 0; j < MT * 8 / kWaves; j++) {
        const int idx = wave + kWaves * j;           // = (t*2 + kh)*4 + rg
        const int rg = idx & 3, kh = (idx >> 2) & 1, t = idx >> 3;
        dma16(a.qs + (m0 + t * 32 + rg * 8) * k + b * 256 + kh * 128, g.act_off, buf + idx * 1024);
    }
    const uint32_t nb = (uint32_t)(k >> 5);
    // block scales: 32 rows x 8 floats per copy (lane l: row l/2, half l%2)
#pragma unroll
    for (int t = 0; t < MT; t++) {
        if (t + 4 == wave)
            dma16((const uint8_t *)(a.d + (m0 + t * 32) * (int64_t)nb + b * 8), (uint32_t)(lane >> 1) * nb * 4u + (uint32_t)(lane & 1) * 16u,
                  buf + T::oD8 + t * 1024);
    }
    // the blocks' `s` fields: 64 rows x 8 halves per copy (lane l: row l)
    if (DT == CQ_DTYPE_Q4K) {
#pragma unroll
        for (int j = 0; j < (MT + 1) / 2; j++) {
            if (j == wave && (MT > 1 || lane < 32))
                dma16((const uint8_t *)(a.s16 + (m0 + j * 64) * (int64_t)nb + b * 8), (uint32_t)lane * nb * 2u, buf + T::oS8 + j * 1024);
        }
    }
}

// v (at most 24 significant bits) as bf16 pieces b1 + b2 + b3, each the leading eight bits of what the pieces before
// it leave: lanes 0..31 carry [b1, b1, b2, b2] in K-slots 0..3, lanes 32..63 carry [b3, b3] in K-slots 8, 9.
__device__ __forceinline__ v8bf weight_scale_operand(float v, int h) {
    const uint32_t vb = __float_as_uint(v);
    const float r1 = v - __uint_as_float(vb & 0xffff0000u);
    const uint32_t rb = __float_as_uint(r1);
    const float r2 = r1 - __uint_as_float(rb & 0xffff0000u);
    const uint32_t tb = __float_as_uint(r2);
    const uint32_t b11 = __builtin_amdgcn_perm(vb, vb, 0x07060706u), b22 = __builtin_amdgcn_perm(rb, rb, 0x07060706u);
    const uint32_t b33 = __builtin_amdgcn_perm(tb, tb, 0x07060706u);
    const v4u pk = {h ? b33 : b11, h ? 0u : b22, 0u, 0u};
    return __builtin_bit_cast(v8bf, pk);
}
// The activation block scale (an f16 value: two bf16 pieces a1 + a2, exact) as [a1, a2, a1, a2] in K-slots 0..3 of
// both lane halves: with the operand above the products sum to (a1 + a2) * (b1 + b2 + b3).
__device__ __forceinline__ v8bf act_scale_operand(float v) {
    const uint32_t vb = __float_as_uint(v);
    const float r1 = v - __uint_as_float(vb & 0xffff0000u);
    const uint32_t a12 = __builtin_amdgcn_perm(__float_as_uint(r1), vb, 0x07060302u);
    const v4u pk = {a12, a12, 0u, 0u};
    return __builtin_bit_cast(v8bf, pk);
}

template <int DT, int MT>
__global__ void __launch_bounds__(kThreads) gemm_q81_kernel(cq_weight w, cq_act_view a, int64_t m, float *__restrict__ y) {
    static_assert(DT == CQ_DTYPE_Q4K || DT == CQ_DTYPE_Q6K, "Q4K and Q6K only");
    typedef Tile81<DT, MT> T;
    constexpr bool K4 = DT == CQ_DTYPE_Q4K;
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, col = lane & 31;
    const int64_t k = w.k, kb = k >> 8;
    const int64_t m0 = (int64_t)blockIdx.y * (MT * 32);
    const int64_t n_tile = ((int64_t)blockIdx.x * kWaves + wave) * 32;
    const bool n_ok = n_tile < w.n;   // wave-uniform; a wave past the last row only helps with the copies
    const int64_t n = n_tile + col;
    const int64_t nc = n_ok ? n : 0;
    const LaneGeo g = lane_geo(lane, k);
    uint8_t *__restrict__ wl = smem + T::oWgt + wave * T::kWgtWave;

    v16f out[MT];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) out[t][i] = 0.0f;

    WHead<DT> hcur, hnxt;
    stage_acts81<DT, MT>(smem, a, g, k, m0, 0, wave, lane);
    if (n_ok) stage_weights<DT>(wl, w, g, n_tile, 0);
    load_head(w, nc * kb, hcur);
    hnxt = hcur;
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    for (int64_t b = 0; b < kb; b++) {
        const uint8_t *__restrict__ cur = smem + (b & 1) * T::kStage;
        uint8_t *__restrict__ nxt = smem + ((b & 1) ^ 1) * T::kStage;
        const bool more = b + 1 < kb;
        if (more) {
            stage_acts81<DT, MT>(nxt, a, g, k, m0, b + 1, wave, lane);
            load_head(w, nc * kb + b + 1, hnxt);
        }
        if (n_ok) {
            // weight operands of the eight Q8_1 blocks, their scale operands, the min-term operand
            v4i bl[8], bh[8];
            v8bf ws[K4 ? 8 : 1];
            v8h wmin = {};
            if constexpr (K4) {
                const float dw = cq_h2f((uint16_t)(hcur.dd & 0xffff));
                const uint32_t rec[4] = {hcur.rec.x, hcur.rec.y, hcur.rec.z, hcur.rec.w};   // {sc[2g], sc[2g+1], mn[2g], mn[2g+1]}
#pragma unroll
                for (int gi = 0; gi < 4; gi++) {
                    // qs bytes 32g + 16h + [0,16): low nibbles = block 2g, high nibbles = block 2g+1
                    const uint4 q = *(const uint4 *)(wl + g.col[gi]);
                    const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        bl[2 * gi][i] = (int)(qw[i] & 0x0F0F0F0Fu);
                        bl[2 * gi + 1][i] = (int)((qw[i] >> 4) & 0x0F0F0F0Fu);
                    }
                    ws[2 * gi] = weight_scale_operand(dw * (float)(rec[gi] & 0xff), h);          // d * sc_j: exact in f32
                    ws[2 * gi + 1] = weight_scale_operand(dw * (float)((rec[gi] >> 8) & 0xff), h);
                }
                wmin = __builtin_bit_cast(v8h, cq_min_term_operand(hcur.dd, rec, h != 0));
            } else {
                float dw;
                MinW none;
                block_unpack(wl, g, hcur, lane, bl, bh, dw, none);
                ws[0] = weight_scale_operand(dw, h);
            }
            if (more) stage_weights<DT>(wl, w, g, n_tile, b + 1);

            // steps q = (tile t, block s): the MFMAs of step q, and in their shadow the scaling of step q-1
            auto afrag = [&](int q) -> v4i {
                const int t = q >> 3, s = q & 7;
                return *(const v4i *)(cur + g.col[s & 3] + (t * 2 + (s >> 2)) * 4096);
            };
            auto d8raw = [&](int q) -> float {
                const int t = q >> 3, s = q & 7;
                return *(const float *)(cur + T::oD8 + (t * 32 + col) * 32 + s * 4);
            };
            v16i acc[2], acch[2];
            v16f sc[2];
            v4i av[3];
            float dv[3];
            av[0] = afrag(0); av[1] = afrag(1);
            dv[0] = d8raw(0); dv[1] = d8raw(1);
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v16f zerof = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q <= MT * 8; q++) {
                if (q + 2 < MT * 8) { av[(q + 2) % 3] = afrag(q + 2); dv[(q + 2) % 3] = d8raw(q + 2); }
                if (q < MT * 8) {
                    if (K4 && (q & 7) == 0) {
                        // min term of tile t: out -= sum_j (dmin * m_j) * s8_j
                        const v8h s8 = *(const v8h *)(cur + T::oS8 + ((q >> 3) * 32 + col) * 16);
                        out[q >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(s8, wmin, out[q >> 3], 0, 0, 0);
                    }
                    acc[q & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[q % 3], bl[q & 7], zero, 0, 0, 0);
                    if (!K4) acch[q & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[q % 3], bh[q & 7], zero, 0, 0, 0);
                    sc[q & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(act_scale_operand(dv[q % 3]), ws[K4 ? (q & 7) : 0], zerof, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);   // the MFMAs stay in front of the scaling of the step before
                if (q > 0) {
                    const int p = (q - 1) & 1, t = (q - 1) >> 3;
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int I = K4 ? acc[p][i] : (acch[p][i] << 8) + acc[p][i];
                        out[t][i] = __builtin_fmaf((float)I, sc[p][i], out[t][i]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        hcur = hnxt;
        __builtin_amdgcn_s_waitcnt(0);   // the next stage and the wave's next weights have landed in LDS
        __syncthreads();
    }

    if (n_ok) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t row = m0 + t * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                if (row < m) y[row * w.n + n] = out[t][i];
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

// Too few workgroups for `slots` of them at once: K is split (at least four blocks per part).
int pick_ksplit(int64_t tiles, int64_t kb, int64_t slots) {
    int ksplit = 1;
    if (cq_no_split_k()) return 1;   // CQ_FLAG_DETERMINISTIC
    while (tiles * ksplit * 2 <= slots && kb / (ksplit * 2) >= 4 && ksplit < 16) ksplit *= 2;
    return ksplit;
}

int64_t n_tiles(const cq_weight *w) { return (w->n + kWaves * 32 - 1) / (kWaves * 32); }

// Tile height (MT x 32 activation rows per workgroup) and K split of a launch, from a cost model fitted to
// measurements (Q4K, 256 CUs; unit 1/16 us): a workgroup spends 22 units per K block unpacking its weights
// and 13.5 per 32-row tile on it, 24 on starting and finishing; workgroups run one per CU, in rounds; a split
// launch adds every part to the output atomically, which moves about 1.1 TB/s.  Tall tiles amortise
// the unpacking, short ones fill the machine without splitting K: 4096 x 4096 at 512 rows takes 54 us as
// 64 tiles of 128 rows split four ways and 42 us as 256 tiles of 32 rows.
struct Plan {
    int mt, ksplit;
    int kh = 1;   // 2: gemm_kh_kernel (K halved inside the workgroup, 128 weight rows per workgroup)
};
Plan pick_plan(const cq_weight *w, int64_t m) {
    const int64_t gx = n_tiles(w), kb = w->k >> 8, cus = num_cus();
    // unpacking one K block of a wave's 32 rows: 152 vector instructions for Q4K, about 370 for Q6K
    const double unpack = w->dtype == CQ_DTYPE_Q4K ? 22.0 : w->dtype == CQ_DTYPE_Q5K ? 32.0 : 50.0;
    const double atomic_pass = (double)m * (double)w->n * 4.0 / 1.1e6 * 16.0;   // bytes / (1.1e6 bytes per us) in units
    Plan best{1, 1};
    double best_cost = 0.0;
    bool first = true;
    for (int mt = 4; mt >= 1; mt >>= 1) {
        if (mt > 1 && m <= 16 * mt) continue;   // half the height holds all rows
        const int64_t tiles = gx * ((m + mt * 32 - 1) / (mt * 32));
        for (int ks = 1; ks <= 16; ks *= 2) {
            if (ks > 1 && kb / ks < 4) break;
            if (ks > 1 && cq_no_split_k()) break;   // CQ_FLAG_DETERMINISTIC
            const int64_t rounds = (tiles * ks + cus - 1) / cus;
            const double cost = (double)rounds * ((double)((kb + ks - 1) / ks) * (unpack + 13.5 * mt) + 24.0) +
                                (ks > 1 ? ks * atomic_pass : 0.0);
            if (first || cost < best_cost) {
                best = Plan{mt, ks};
                best_cost = cost;
                first = false;
            }
        }
    }
    // K halved inside the workgroup: twice the column tiles, half the blocks per wave, 8 units for the meeting at the end
    const int64_t gx128 = (w->n + 127) / 128;
    for (int mt = 2; mt >= 1; mt >>= 1) {
        if (mt > 1 && m <= 16 * mt) continue;
        if (kb < 2) break;
        const int64_t tiles = gx128 * ((m + mt * 32 - 1) / (mt * 32));
        // (only where one round of workgroups does it: over several rounds the taller tiles of the launches above won
        // in every measured case, 5120 / 11008 x 14336 at 512-1024 rows by 10-16 %)
        if (tiles > cus) continue;
        const int64_t rounds = 1;
        const double cost = (double)rounds * ((double)((kb + 1) / 2) * (unpack + 13.5 * mt) + 24.0 + 8.0);
        if (cost < best_cost) {
            best = Plan{mt, 1, 2};
            best_cost = cost;
        }
    }
    return best;
}

template <int DT, int MT>
hipError_t launch_mt(const cq_weight *w, cq_act_view a, int64_t m, float *y, int ksplit, bool y_cleared, hipStream_t s) {
    const size_t lds = Tile<DT, MT>::kTotal;
    if (hipError_t e = cq_ensure_lds<gemm_kernel<DT, MT>>(w->dev, lds); e != hipSuccess) return e;
    const int64_t gx = n_tiles(w), gy = (m + MT * 32 - 1) / (MT * 32);
    if (ksplit > 1 && !y_cleared) {
        hipError_t e = cq_launch_fill_zero(y, m * w->n, s);
        if (e != hipSuccess) return e;
    }
    dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)ksplit);
    if constexpr (MT == 1) {
        if (gy == 1) {
            const size_t lds1 = once_wbuf<DT>() == 2 ? Tile<DT, 1>::kTotal2 : Tile<DT, 1>::kTotal;
            if (hipError_t e = cq_ensure_lds<gemm_once_kernel<DT>>(w->dev, lds1); e != hipSuccess) return e;
            CQ_LAUNCH((gemm_once_kernel<DT>), grid, kThreads, lds1, s, *w, a, m, y, ksplit);
            return hipGetLastError();
        }
    }
    CQ_LAUNCH((gemm_kernel<DT, MT>), grid, kThreads, lds, s, *w, a, m, y, ksplit);
    return hipGetLastError();
}

template <int DT, int MT>
hipError_t launch_kh(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    const size_t lds = TileKH<DT, MT>::kTotal;
    if (hipError_t e = cq_ensure_lds<gemm_kh_kernel<DT, MT>>(w->dev, lds); e != hipSuccess) return e;
    dim3 grid((unsigned)((w->n + 127) / 128), (unsigned)((m + MT * 32 - 1) / (MT * 32)), 1);
    CQ_LAUNCH((gemm_kh_kernel<DT, MT>), grid, kThreads, lds, s, *w, a, m, y);
    return hipGetLastError();
}

template <int DT>
hipError_t launch_dt(const cq_weight *w, cq_act_view a, int64_t m, float *y, bool y_cleared, hipStream_t s) {
    const Plan p = pick_plan(w, m);
    if (p.kh == 2) return p.mt == 1 ? launch_kh<DT, 1>(w, a, m, y, s) : launch_kh<DT, 2>(w, a, m, y, s);
    if (p.mt == 1) return launch_mt<DT, 1>(w, a, m, y, p.ksplit, y_cleared, s);
    if (p.mt == 2) return launch_mt<DT, 2>(w, a, m, y, p.ksplit, y_cleared, s);
    return launch_mt<DT, 4>(w, a, m, y, p.ksplit, y_cleared, s);
}

// The launch cq_launch_gemm would make (same tile height, same K split), storing the block integers.
template <int DT, int MT>
hipError_t launch_dump_mt(const cq_weight *w, cq_act_view a, int64_t m, int ksplit, cq_mfma_dump d, hipStream_t s) {
    const size_t lds = Tile<DT, MT>::kTotal;
    if (hipError_t e = cq_ensure_lds<gemm_dump_kernel<DT, MT>>(w->dev, lds); e != hipSuccess) return e;
    dim3 grid((unsigned)n_tiles(w), (unsigned)((m + MT * 32 - 1) / (MT * 32)), (unsigned)ksplit);
    CQ_LAUNCH((gemm_dump_kernel<DT, MT>), grid, kThreads, lds, s, *w, a, m, ksplit, d);
    return hipGetLastError();
}
template <int DT>
hipError_t launch_dump_dt(const cq_weight *w, cq_act_view a, int64_t m, cq_mfma_dump d, hipStream_t s) {
    const Plan p = pick_plan(w, m);
    if (p.mt == 1) return launch_dump_mt<DT, 1>(w, a, m, p.ksplit, d, s);
    if (p.mt == 2) return launch_dump_mt<DT, 2>(w, a, m, p.ksplit, d, s);
    return launch_dump_mt<DT, 4>(w, a, m, p.ksplit, d, s);
}

template <int DT>
hipError_t launch_grouped(const cq_weight *const *experts, int n_experts, const int32_t *offsets, cq_act_view a,
                          float *y, bool y_cleared, hipStream_t s) {
    GroupArgs ga;
    int ntiles = 0;
    for (int e = 0; e < n_experts; e++) {
        ga.w[e] = *experts[e];
        for (int32_t r = offsets[e]; r < offsets[e + 1]; r += 32) {
            if (ntiles == kMaxGroupTiles) return hipErrorInvalidConfiguration;
            ga.row0[ntiles] = r;
            ga.row_end[ntiles] = offsets[e + 1];
            ga.expert[ntiles] = (int8_t)e;
            ntiles++;
        }
    }
    if (ntiles == 0) return hipSuccess;
    const cq_weight *w = experts[0];
    const size_t lds = grouped_wbuf<DT>() == 2 ? Tile<DT, 1>::kTotal2 : Tile<DT, 1>::kTotal;
    if (hipError_t e = cq_ensure_lds<gemm_grouped_kernel<DT>>(w->dev, lds); e != hipSuccess) return e;
    const int64_t gx = n_tiles(w);
    const int ksplit = pick_ksplit(gx * ntiles, w->k >> 8, 2 * num_cus());   // two single-tile workgroups per CU
    if (ksplit > 1 && !y_cleared) {
        hipError_t e = cq_launch_fill_zero(y, (int64_t)offsets[n_experts] * w->n, s);
        if (e != hipSuccess) return e;
    }
    dim3 grid((unsigned)gx, (unsigned)ntiles, (unsigned)ksplit);
    CQ_LAUNCH((gemm_grouped_kernel<DT>), grid, kThreads, lds, s, ga, a, y, ksplit);
    return hipGetLastError();
}

template <int DT, int MT>
hipError_t launch_q81_mt(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    const size_t lds = Tile81<DT, MT>::kTotal;
    if (hipError_t e = cq_ensure_lds<gemm_q81_kernel<DT, MT>>(w->dev, lds); e != hipSuccess) return e;
    dim3 grid((unsigned)n_tiles(w), (unsigned)((m + MT * 32 - 1) / (MT * 32)), 1);
    CQ_LAUNCH((gemm_q81_kernel<DT, MT>), grid, kThreads, lds, s, *w, a, m, y);
    return hipGetLastError();
}
template <int DT>
hipError_t launch_q81_dt(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    // the tallest tile that still gives every CU a workgroup
    int mt = 4;
    while (mt > 1 && (m <= 16 * mt || n_tiles(w) * ((m + mt * 32 - 1) / (mt * 32)) < num_cus())) mt >>= 1;
    if (mt == 1) return launch_q81_mt<DT, 1>(w, a, m, y, s);
    if (mt == 2) return launch_q81_mt<DT, 2>(w, a, m, y, s);
    return launch_q81_mt<DT, 4>(w, a, m, y, s);
}

}  // namespace

bool cq_gemm_grouped_supported(const cq_weight *const *experts, int n_experts, const int32_t *offsets, int act_dtype) {
    if (n_experts > kMaxGroupExperts || !cq_gemm_supported(experts[0], 0, act_dtype)) return false;
    int64_t tiles = 0;
    for (int e = 0; e < n_experts; e++) tiles += (offsets[e + 1] - offsets[e] + 31) / 32;
    return tiles <= kMaxGroupTiles;
}

hipError_t cq_launch_gemm_grouped(const cq_weight *const *experts, int n_experts, const int32_t *offsets, cq_act_view a,
                                  float *y, bool y_cleared, hipStream_t s) {
    if (a.m_stride < ((int64_t)offsets[n_experts] + 31) / 32 * 32) return hipErrorInvalidValue;
    if (experts[0]->dtype == CQ_DTYPE_Q4K) return launch_grouped<CQ_DTYPE_Q4K>(experts, n_experts, offsets, a, y, y_cleared, s);
    if (experts[0]->dtype == CQ_DTYPE_Q5K) return launch_grouped<CQ_DTYPE_Q5K>(experts, n_experts, offsets, a, y, y_cleared, s);
    return launch_grouped<CQ_DTYPE_Q6K>(experts, n_experts, offsets, a, y, y_cleared, s);
}

hipError_t cq_launch_gemm_dump(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, cq_mfma_dump d, hipStream_t s) {
    if (!cq_gemm_supported(w, m, act_dtype)) return hipErrorNotSupported;
    if (m == 0 || w->n == 0) return hipSuccess;
    if (a.m_stride < (m + 127) / 128 * 128) return hipErrorInvalidValue;
    if (w->dtype == CQ_DTYPE_Q4K) return launch_dump_dt<CQ_DTYPE_Q4K>(w, a, m, d, s);
    if (w->dtype == CQ_DTYPE_Q5K) return launch_dump_dt<CQ_DTYPE_Q5K>(w, a, m, d, s);
    return launch_dump_dt<CQ_DTYPE_Q6K>(w, a, m, d, s);
}

bool cq_gemm_grouped_splits_k(const cq_weight *const *experts, int n_experts, const int32_t *offsets) {
    int64_t tiles = 0;
    for (int e = 0; e < n_experts; e++) tiles += (offsets[e + 1] - offsets[e] + 31) / 32;
    return tiles > 0 && pick_ksplit(n_tiles(experts[0]) * tiles, experts[0]->k >> 8, 2 * num_cus()) > 1;
}

bool cq_gemm_splits_k(const cq_weight *w, int64_t m) { return m > 0 && pick_plan(w, m).ksplit > 1; }

bool cq_gemm_supported(const cq_weight *w, int64_t m, int act_dtype) {
    (void)m;
    // the copies address rows with 32-bit offsets: 8 rows of activations, 16 rows of a weight plane
    return (w->dtype == CQ_DTYPE_Q4K || w->dtype == CQ_DTYPE_Q5K || w->dtype == CQ_DTYPE_Q6K) && act_dtype == CQ_DTYPE_Q8K && w->k >= 256 &&
           w->k <= (1 << 24) && w->n % 32 == 0;
}

hipError_t cq_launch_gemm(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, bool y_cleared,
                          hipStream_t s) {
    if (!cq_gemm_supported(w, m, act_dtype)) return hipErrorNotSupported;
    if (m == 0 || w->n == 0) return hipSuccess;
    if (a.m_stride < (m + 127) / 128 * 128) return hipErrorInvalidValue;   // rows the last tile may read
    if (w->dtype == CQ_DTYPE_Q4K) return launch_dt<CQ_DTYPE_Q4K>(w, a, m, y, y_cleared, s);
    if (w->dtype == CQ_DTYPE_Q5K) return launch_dt<CQ_DTYPE_Q5K>(w, a, m, y, y_cleared, s);
    return launch_dt<CQ_DTYPE_Q6K>(w, a, m, y, y_cleared, s);
}

// K-quant weights x Q8_1 activations on the matrix cores (see gemm_q81_kernel).  The workspace rows are padded to whole
// 128-row tiles beyond 32 rows, scales and `s` fields included.
bool cq_gemm_q81_supported(const cq_weight *w, int64_t m) {
    return (w->dtype == CQ_DTYPE_Q4K || w->dtype == CQ_DTYPE_Q6K) && m > 32 && w->k >= 256 && w->k <= (1 << 24) && w->n % 32 == 0;
}

hipError_t cq_launch_gemm_q81(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    if (!cq_gemm_q81_supported(w, m)) return hipErrorNotSupported;
    if (w->n == 0) return hipSuccess;
    if (a.m_stride < (m + 127) / 128 * 128) return hipErrorInvalidValue;   // rows the last tile may read
    if (w->dtype == CQ_DTYPE_Q4K) return launch_q81_dt<CQ_DTYPE_Q4K>(w, a, m, y, s);
    return launch_q81_dt<CQ_DTYPE_Q6K>(w, a, m, y, s);
}
