// Skinny matmul on int8 MFMA for a few activation rows (32 per pass over the weights; cq_qmatmul sends it 2..16 rows,
// more where the weight has few rows): y[m, n] = x[m, k] . W[n, k]^T with K-quant
// weights and Q8K activations (Q8_0 weights with Q8_0 activations: second kernel below) (k_quants.rs:1842-1883 with vec_dot :1171-1250 for Q4K, :1585-1641
// for Q6K) - the small-batch decode and the per-expert shapes of a mixture-of-experts layer, where
// the weights are still read once and the job stays bound by HBM.  The arithmetic is that of the
// prefill GEMM (gemm.hip): sub-block scales folded into the int8 weight operands as two digits,
// exact block integers I = 8*hi + lo (Q4K) / 128*hi + lo (Q5K, Q6K), the Q4K / Q5K min term on the f16 MFMA.
//
// Work split: with so few activation rows there is no tile to reuse weights over, so the K
// dimension is split instead.  A workgroup owns 16 weight rows (one 16x16x64 MFMA operand); its
// eight waves take the 256-element K blocks round-robin (wave w: blocks w, w+8, ...).  Per block a
// wave copies its 16 x 144 (210) weight bytes and the block's activation slice from global memory
// straight into its own LDS buffer (buffer_load ... lds, whole 128-byte lines, XOR-swizzled as in
// gemm.hip), unpacks, and issues eight MFMAs per 16 activation rows.  The waves' partial 16 x 16
// results are summed through LDS in wave order (deterministic; no atomics).  Many small workgroups
// (n / 16) and one block in flight per wave keep enough bytes outstanding per CU.
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
constexpr int kMaxLds = 160 * 1024;   // LDS of a CU, which a single workgroup may take

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

__device__ __forceinline__ void dma16(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wave_rsrc(base), (lptr_t)lds, 16, (int)off, 0, 0, 0);
}
__device__ __forceinline__ void dma4(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wave_rsrc(base), (lptr_t)lds, 4, (int)off, 0, 0, 0);
}

// Per-wave LDS buffer for RT groups of eight activation rows:
//   wgt : [2 row groups][8 rows][8 chunks of 16 B] of the 128-byte qs / ql plane, chunk c of row r at c ^ (r%8);
//         Q6K also [16 rows][4 chunks] of the 64-byte qh plane (chunk c at c ^ ((r/2)%4)),
//         Q5K also [16 rows][32 B] of the fifth-bit plane
//   act : [RT row groups][2 K-halves][8 rows][8 chunks], same swizzle
//   d8  : [8*RT] f32         bsh : [8*RT][16] f16: the rows' bsums (Q4K / Q5K)
constexpr bool is_k4(int dt) { return dt == CQ_DTYPE_Q4K || dt == CQ_DTYPE_Q5K; }   // types with a min term

template <int DT, int RT> struct Buf {
    static constexpr int kWgt = DT == CQ_DTYPE_Q4K ? 2048 : DT == CQ_DTYPE_Q5K ? 2560 : 3072;
    static constexpr int oAct = kWgt, kAct = RT * 2048;
    static constexpr int oD8 = oAct + kAct, kD8 = RT * 32;
    static constexpr int oMin = oD8 + kD8, kMin = is_k4(DT) ? RT * 256 : 0;
    static constexpr int kRaw = oMin + kMin;
    // the buffer also carries the wave's partial results at the end: 1 KiB per 16 activation rows
    static constexpr int kBytes = kRaw < 2048 ? 2048 : kRaw;
};

__device__ __forceinline__ uint32_t swz_col(uint32_t r, uint32_t c) {
    return (r >> 3) * 1024u + (r & 7) * 128u + ((c ^ (r & 7)) << 4);
}

template <int DT> struct WHead;
template <> struct WHead<CQ_DTYPE_Q4K> { uint32_t dd; uint4 rec; };   // d | dmin << 16; records {sc, sc, mn, mn} per 32 qs bytes
template <> struct WHead<CQ_DTYPE_Q5K> : WHead<CQ_DTYPE_Q4K> {};       // the same header plane
template <> struct WHead<CQ_DTYPE_Q6K> { uint4 sc; uint32_t d; };     // re-packed scales (two per unit); d
__device__ __forceinline__ void load_head(const cq_weight &w, int64_t blk, WHead<CQ_DTYPE_Q4K> &r) {
    // two loads (16 + 4 bytes; the 20-byte records are 4-byte aligned, which is all a global load needs)
    typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
    const uint8_t *h = w.p1 + blk * CQ_Q4K_HDR;
    const u32x4_a4 v = *(const u32x4_a4 *)h;
    r.dd = v.x;
    r.rec = make_uint4(v.y, v.z, v.w, *(const uint32_t *)(h + 16));
}
__device__ __forceinline__ void load_head(const cq_weight &w, int64_t blk, WHead<CQ_DTYPE_Q6K> &r) {
    r.sc = *(const uint4 *)(w.p2 + blk * 16);
    r.d = ((const uint16_t *)w.p3)[blk];
}

// Weight operands of one block for lane (row r = l%16, k quarter kq = l/16): the two digit operands
// of the four 64-wide K-slices, the block scale and the Q4K min-term operand.
__device__ __forceinline__ void block_unpack(const uint8_t *wl, int lane, const WHead<CQ_DTYPE_Q4K> &wb, v4i (&bl)[4],
                                             v4i (&bh)[4], float &dw, v8h &wmin) {
    const uint32_t r = lane & 15, kq = lane >> 4;
    dw = cq_h2f((uint16_t)(wb.dd & 0xffff));
    const uint32_t rec[4] = {wb.rec.x, wb.rec.y, wb.rec.z, wb.rec.w};
    // K-slice g = elements 64g..64g+63 = qs bytes 32g..32g+31, low nibbles for the first 32 elements
    // (quarters 0,1: sub-block 2g), high nibbles for the last 32 (quarters 2,3: sub-block 2g+1)
    const uint32_t hi = kq >> 1, nsh = hi * 4;
#pragma unroll
    for (int gi = 0; gi < 4; gi++) {
        const uint4 q = *(const uint4 *)(wl + swz_col(r, 2 * gi + (kq & 1)));
        const uint32_t sj = (rec[gi] >> (8 * hi)) & 0xff;   // scale of sub-block 2g + hi
        const unsigned short sl = (unsigned short)(sj & 7), sh = (unsigned short)(sj >> 3);
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t v = (qw[i] >> nsh) & 0x0F0F0F0Fu;
            bl[gi][i] = (int)pk_mul_u16(v, sl);   // low digit of the scale
            bh[gi][i] = (int)pk_mul_u16(v, sh);
        }
    }
    // min term operand: 32 K-slots = activation pieces [1,1,2,2] x weight pieces [1,2,1,2] of the
    // eight sub-block values -dmin*min_j
    wmin = __builtin_bit_cast(v8h, cq_min_term_groups(wb.dd, rec, (kq & 1) != 0, (kq >> 1) != 0));   // K-slots 8kq..: groups 8(kq%2).., piece kq/2
}

// Q5K: the quants are the Q4K nibbles plus a fifth bit (words {L, H} per 32 qs bytes, bit 8c + i for
// byte c of qs word i); scale times quant has up to 11 bits and is split as Q6K's products are.
__device__ __forceinline__ void block_unpack(const uint8_t *wl, int lane, const WHead<CQ_DTYPE_Q5K> &wb, v4i (&bl)[4],
                                             v4i (&bh)[4], float &dw, v8h &wmin) {
    const uint32_t r = lane & 15, kq = lane >> 4;
    dw = cq_h2f((uint16_t)(wb.dd & 0xffff));
    const uint32_t rec[4] = {wb.rec.x, wb.rec.y, wb.rec.z, wb.rec.w};
    const uint32_t hi = kq >> 1, nsh = hi * 4, w0 = 4 * (kq & 1);   // first qs word of the lane's 16 bytes
    const uint4 f0 = *(const uint4 *)(wl + 2048 + r * 32u), f1 = *(const uint4 *)(wl + 2048 + r * 32u + 16u);
    const uint32_t fifth[4] = {hi ? f0.y : f0.x, hi ? f0.w : f0.z, hi ? f1.y : f1.x, hi ? f1.w : f1.z};
#pragma unroll
    for (int gi = 0; gi < 4; gi++) {
        const uint4 q = *(const uint4 *)(wl + swz_col(r, 2 * gi + (kq & 1)));
        const unsigned short sc16 = (unsigned short)((rec[gi] >> (8 * hi)) & 0xff);   // scale of sub-block 2g + hi
        const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t q5 = ((qw[i] >> nsh) & 0x0F0F0F0Fu) | (((fifth[gi] >> (w0 + i)) & 0x01010101u) << 4);
            int lo, hi;
            cq_scaled_digits(q5, sc16, (unsigned short)128, lo, hi);   // digits of sc * q5
            bl[gi][i] = lo;
            bh[gi][i] = hi;
        }
    }
    wmin = __builtin_bit_cast(v8h, cq_min_term_groups(wb.dd, rec, (kq & 1) != 0, (kq >> 1) != 0));   // K-slots 8kq..: groups 8(kq%2).., piece kq/2
}

__device__ __forceinline__ void block_unpack(const uint8_t *wl, int lane, const WHead<CQ_DTYPE_Q6K> &wb, v4i (&bl)[4],
                                             v4i (&bh)[4], float &dw, v8h &wmin) {
    const uint32_t r = lane & 15, kq = lane >> 4;
    dw = cq_h2f((uint16_t)wb.d);
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
        // K-slices 2hf (low nibbles) and 2hf+1 (high nibbles) of unit u = 4hf + kq: 16 bytes of ql,
        // 8 bytes of re-packed high bits, scale bytes 2u and 2u+1
        const uint4 ql = *(const uint4 *)(wl + swz_col(r, 4 * hf + kq));
        const uint2 qh = *(const uint2 *)(wl + 2048 + r * 64u + (((2 * hf + (kq >> 1)) ^ ((r >> 1) & 3)) << 4) + (kq & 1) * 8u);
        const uint32_t s_even = hf ? wb.sc.z : wb.sc.x, s_odd = hf ? wb.sc.w : wb.sc.y;
        const uint32_t sw = s_even ^ ((s_even ^ s_odd) & (0u - (kq >> 1)));   // word 2hf + kq/2, branch-free
        const uint32_t qw[4] = {ql.x, ql.y, ql.z, ql.w};
        const uint32_t hw[2] = {qh.x, qh.y};
#pragma unroll
        for (int nib = 0; nib < 2; nib++) {
            const int s = 2 * hf + nib;
            const int sc = (int)(int8_t)((sw >> (16 * (kq & 1) + 8 * nib)) & 0xff);
            const unsigned short sc16 = (unsigned short)sc, c16 = (unsigned short)(128 - 32 * sc);
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
    }
    wmin = v8h{};
}

// RT = groups of eight activation rows held (rows m0 .. m0 + 8*RT - 1; the workspace pads rows, so
// whole groups can be copied); results are stored for rows < m.  Requires n % 16 == 0.
// DUMP (verification): the block integers, and the min term as the f16 MFMA delivers it from a zero accumulator,
// are stored through `dump` instead of the result through `y`.
template <int DT, int RT, bool DUMP>
__global__ void __launch_bounds__(kThreads) skinny_kernel(cq_weight w, cq_act_view a, int64_t m0, int64_t m,
                                                          float *__restrict__ y, cq_mfma_dump dump) {
    typedef Buf<DT, RT> B;
    constexpr bool MINS = is_k4(DT);
    constexpr int NT = (RT + 1) / 2;   // 16-row tiles
    constexpr int SHIFT = DT == CQ_DTYPE_Q4K ? 3 : 8;
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15, kq = lane >> 4;
    const int64_t k = w.k, kb = w.k >> 8;
    const int64_t n_tile = (int64_t)blockIdx.x * 16;
    uint8_t *buf = smem + wave * B::kBytes;

    // copy offsets: 8 rows x 128 B per instruction, chunks swizzled by the row
    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    const uint32_t act_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    const uint32_t wq_off = r8 * (uint32_t)kb * 128u + ((c8 ^ r8) << 4);
    const uint32_t r16 = lane >> 2, c4 = lane & 3;
    const uint32_t wh_off = r16 * (uint32_t)kb * 64u + ((c4 ^ ((r16 >> 1) & 3)) << 4);
    const uint32_t w5_off = (lane >> 1) * (uint32_t)kb * 32u + (lane & 1) * 16u;   // Q5K: 16 rows x 32 B, lanes 0..31
    // activation operand reads: row of tile t clamped to the rows held
    uint32_t a_col[NT][2];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const uint32_t row = t * 16 + r < 8u * RT ? t * 16 + r : 8u * RT - 1;
#pragma unroll
        for (uint32_t e = 0; e < 2; e++)
            a_col[t][e] = B::oAct + (row >> 3) * 2048u + (row & 7) * 128u + (((4 * e + kq) ^ (row & 7)) << 4);
    }

    v4f out[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) out[t] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};

    for (int64_t b = wave; b < kb; b += kWaves) {
        // ---- copies of block b: weights of the 16 rows, activation rows, their scales
#pragma unroll
        for (int rg = 0; rg < 2; rg++) dma16(w.p0 + ((n_tile + rg * 8) * kb + b) * 128, wq_off, buf + rg * 1024);
        if (DT == CQ_DTYPE_Q6K) dma16(w.p1 + (n_tile * kb + b) * 64, wh_off, buf + 2048);
        if (DT == CQ_DTYPE_Q5K && lane < 32) dma16(w.p2 + (n_tile * kb + b) * 32, w5_off, buf + 2048);
#pragma unroll
        for (int i = 0; i < 2 * RT; i++) {
            const int rg = i >> 1, kh = i & 1;
            dma16(a.qs + (m0 + rg * 8) * k + b * 256 + kh * 128, act_off, buf + B::oAct + i * 1024);
        }
        if (lane < 8 * RT) dma4(a.dT + b * a.m_stride + m0, lane * 4u, buf + B::oD8);
        if (MINS && lane < 16 * RT) dma16(a.bsh + (b * a.m_stride + m0) * 16, lane * 16u, buf + B::oMin);
        WHead<DT> head;
        load_head(w, (n_tile + r) * kb + b, head);
        __builtin_amdgcn_s_waitcnt(0);   // everything above has landed

        // ---- arithmetic of block b
        v4i bl[4], bh[4];
        float dw;
        v8h wmin;
        block_unpack(buf, lane, head, bl, bh, dw, wmin);
        if constexpr (DUMP && is_k4(DT)) {
            if (dump.int_min) {   // verification: the minima themselves as the operand: the MFMA delivers the integer Mn_b
                const uint32_t rec[4] = {head.rec.x, head.rec.y, head.rec.z, head.rec.w};
                wmin = __builtin_bit_cast(v8h, cq_min_term_groups_int(rec, (kq & 1) != 0, (kq >> 1) != 0));
            }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const v4f d8 = *(const v4f *)(buf + B::oD8 + (t * 16 + 4 * kq < 8u * RT ? t * 16 + 4 * kq : 0) * 4);
            // min term: sum_j bsums_j * (-dmin * min_{j/2}), the sums exact in f16 whatever the activations' magnitude
            // (their scale d8 multiplies afterwards, with the main term)
            v4f mn = {0.0f, 0.0f, 0.0f, 0.0f};
            if (MINS) {
                const uint32_t row = t * 16 + r < 8u * RT ? t * 16 + r : 8u * RT - 1;
                const v8h ma = *(const v8h *)(buf + B::oMin + row * 32 + (kq & 1) * 16);
                mn = __builtin_amdgcn_mfma_f32_16x16x32_f16(ma, wmin, mn, 0, 0, 0);
                if (DUMP && dump.mn) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int64_t orow = m0 + t * 16 + kq * 4 + i;
                        if (orow < m) dump.mn[(orow * w.n + n_tile + r) * kb + b] = mn[i];
                    }
                }
            }
            v4i acc_lo = {0, 0, 0, 0}, acc_hi = {0, 0, 0, 0};
#pragma unroll
            for (int s = 0; s < 4; s++) {
                const v4i av = *(const v4i *)(buf + a_col[t][s & 1] + (s >> 1) * 1024);
                acc_lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bl[s], acc_lo, 0, 0, 0);
                acc_hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bh[s], acc_hi, 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int I = (acc_hi[i] << SHIFT) + acc_lo[i];
                if (DUMP) {
                    const int64_t orow = m0 + t * 16 + kq * 4 + i;
                    if (orow < m) dump.i[(orow * w.n + n_tile + r) * kb + b] = I;
                } else {
                    const float v = MINS ? __builtin_fmaf((float)I, dw, mn[i]) : (float)I * dw;
                    out[t][i] = __builtin_fmaf(v, d8[i], out[t][i]);
                }
            }
        }
    }
    if (DUMP) return;

    // ---- sum the eight waves' partial tiles in wave order
#pragma unroll
    for (int t = 0; t < NT; t++) *(v4f *)(buf + t * 1024 + lane * 16) = out[t];
    __syncthreads();
    if (wave < NT) {
        v4f s = *(const v4f *)(smem + wave * 1024 + lane * 16);
#pragma unroll
        for (int o = 1; o < kWaves; o++) {
            const v4f p = *(const v4f *)(smem + o * B::kBytes + wave * 1024 + lane * 16);
            s += p;
        }
        const int64_t col = n_tile + r;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t row = m0 + wave * 16 + kq * 4 + i;
            if (row < m) y[row * w.n + col] = s[i];
        }
    }
}

// ------------------------------------------------------------ resident-activation variant ----
// The kernel above re-reads the activations once per 16 weight rows: with 16 activation rows that is more
// bytes (from L2) than the weights themselves (16 K against 9 K per workgroup for Q4K), and the launch is bound
// by it.  When the quantized activations of the call fit the LDS beside the weight buffers (4096 columns x 16
// rows: 75 KiB) a launch of at most one workgroup per CU copies them once, each wave the K blocks it owns (sixteen
// waves: one block each for 4096 columns, a single memory round trip), and then walks its share of the 16-row
// weight tiles (tile t of workgroup g: g + t * G) streaming weights only.  The launcher takes it where every
// workgroup has one tile (n <= 16 x the number of CUs); with more tiles per workgroup it measured no faster than
// the kernel above, also with the next tile's weights copied ahead into a second buffer (NBUF == 2).
//   per K block b  : act [RT][2 K-halves][8 rows][8 chunks] | d8 [8*RT] f32 | bsh [8*RT][16] f16 (k4 types)
//   per wave, block: weights of one tile (kWgt bytes), twice when NBUF == 2; a wave's first buffer of a tile also
//                    carries its partial results of that tile (1 KiB per 16 activation rows)
template <int DT, int RT> struct Res {
    static constexpr int kWgt = Buf<DT, RT>::kWgt;
    static constexpr int kActBlk = RT * 2048 + RT * 32 + (is_k4(DT) ? RT * 256 : 0);
    static constexpr int oD8 = RT * 2048, oMin = oD8 + RT * 32;
    static size_t bytes(int64_t kb, int nbuf) { return (size_t)kb * kActBlk + (size_t)kb * nbuf * kWgt; }
};

// Copies with one descriptor per plane, built once, and the position inside the plane as a 32-bit scalar offset
// (the planes of a tensor this kernel takes are far below 4 GiB): two scalar instructions per copy instead of
// rebuilding a descriptor from a 64-bit address for each.
struct ResPlanes {
    __amdgpu_buffer_rsrc_t wq, wh, w5, aq, ad, am;
};
__device__ __forceinline__ void dma16s(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)lds, 16, (int)voff, (int)soff, 0, 0);
}
__device__ __forceinline__ void dma4s(__amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)lds, 4, (int)voff, (int)soff, 0, 0);
}

// Issues the copies of the weights of the tile starting at row n_tile for K block b into `wl`.
template <int DT>
__device__ __forceinline__ void res_issue_weights(uint8_t *__restrict__ wl, const ResPlanes &pl, uint32_t n_tile, uint32_t b,
                                                  uint32_t kb, uint32_t wq_off, uint32_t wh_off, uint32_t w5_off, int lane) {
    const uint32_t blk = n_tile * kb + b;
    dma16s(pl.wq, wq_off, blk * 128u, wl);
    dma16s(pl.wq, wq_off, blk * 128u + kb * 1024u, wl + 1024);
    if (DT == CQ_DTYPE_Q6K) dma16s(pl.wh, wh_off, blk * 64u, wl + 2048);
    if (DT == CQ_DTYPE_Q5K && lane < 32) dma16s(pl.w5, w5_off, blk * 32u, wl + 2048);
}

// Weight operands of one K block of one tile, unpacked into registers.
struct ResOps {
    v4i bl[4], bh[4];
    float dw;
    v8h wmin;
};
template <int DT, bool DUMP>
__device__ __forceinline__ void res_unpack(const uint8_t *__restrict__ wl, int lane, const WHead<DT> &head, const cq_mfma_dump &dump,
                                           ResOps &o) {
    block_unpack(wl, lane, head, o.bl, o.bh, o.dw, o.wmin);
    if constexpr (DUMP && is_k4(DT)) {
        if (dump.int_min) {   // verification: the minima themselves as the operand: the MFMA delivers the integer Mn_b
            const uint32_t kq = lane >> 4;
            const uint32_t rec[4] = {head.rec.x, head.rec.y, head.rec.z, head.rec.w};
            o.wmin = __builtin_bit_cast(v8h, cq_min_term_groups_int(rec, (kq & 1) != 0, (kq >> 1) != 0));
        }
    }
}

// The unpacked operands `o` contracted with the resident activation slice `act` of the same K block.
// DUMP: the integers go to dump.i / dump.mn at `at` + row * `rs` (rows < m) instead of into `out`.
template <int DT, int RT, int NT, bool DUMP>
__device__ __forceinline__ void res_mac(const uint8_t *__restrict__ act, int lane, const ResOps &o, const uint32_t (&a_col)[NT][2],
                                        v4f (&out)[NT], const cq_mfma_dump &dump, int64_t at, int64_t rs, int64_t m) {
    typedef Res<DT, RT> R;
    constexpr bool MINS = is_k4(DT);
    constexpr int SHIFT = DT == CQ_DTYPE_Q4K ? 3 : 8;
    const uint32_t r = lane & 15, kq = lane >> 4;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const v4f d8 = *(const v4f *)(act + R::oD8 + (t * 16 + 4 * kq < 8u * RT ? t * 16 + 4 * kq : 0) * 4);
        v4f mn = {0.0f, 0.0f, 0.0f, 0.0f};   // min term without the activation scale (see skinny_kernel)
        if (MINS) {
            const uint32_t row = t * 16 + r < 8u * RT ? t * 16 + r : 8u * RT - 1;
            const v8h ma = *(const v8h *)(act + R::oMin + row * 32 + (kq & 1) * 16);
            mn = __builtin_amdgcn_mfma_f32_16x16x32_f16(ma, o.wmin, mn, 0, 0, 0);
            if (DUMP && dump.mn) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int64_t orow = t * 16 + kq * 4 + i;
                    if (orow < m) dump.mn[at + orow * rs] = mn[i];
                }
            }
        }
        v4i acc_lo = {0, 0, 0, 0}, acc_hi = {0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const v4i av = *(const v4i *)(act + a_col[t][s & 1] + (s >> 1) * 1024);
            acc_lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, o.bl[s], acc_lo, 0, 0, 0);
            acc_hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, o.bh[s], acc_hi, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int I = (acc_hi[i] << SHIFT) + acc_lo[i];
            if (DUMP) {
                const int64_t orow = t * 16 + kq * 4 + i;
                if (orow < m) dump.i[at + orow * rs] = I;
            } else {
                const float v = MINS ? __builtin_fmaf((float)I, o.dw, mn[i]) : (float)I * o.dw;
                out[t][i] = __builtin_fmaf(v, d8[i], out[t][i]);
            }
        }
    }
}

// One K block of one tile: unpack the weights in `wl`, contract with the resident activation slice `act`.
template <int DT, int RT, int NT, bool DUMP>
__device__ __forceinline__ void res_block(const uint8_t *__restrict__ wl, const uint8_t *__restrict__ act, int lane,
                                          const WHead<DT> &head, const uint32_t (&a_col)[NT][2], v4f (&out)[NT],
                                          const cq_mfma_dump &dump, int64_t at, int64_t rs, int64_t m) {
    ResOps o;
    res_unpack<DT, DUMP>(wl, lane, head, dump, o);
    res_mac<DT, RT, NT, DUMP>(act, lane, o, a_col, out, dump, at, rs, m);
}

// m <= 8 * RT activation rows (the workspace pads rows, so whole groups are copied); n % 16 == 0; at most
// kMaxBpw K blocks per wave.  `tiles` = n / 16, dealt to the gridDim.x workgroups in turn.
constexpr int kMaxBpw = 4;
template <int DT, int RT, int kWaves, int NBUF, bool DUMP>
__global__ void __launch_bounds__(kWaves * 64) skinny_resident_kernel(cq_weight w, cq_act_view a, int64_t m,
                                                                      float *__restrict__ y, cq_mfma_dump dump) {
    typedef Res<DT, RT> R;
    constexpr bool MINS = is_k4(DT);
    constexpr int NT = (RT + 1) / 2;   // 16-row tiles of activation rows
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15, kq = lane >> 4;
    const int64_t k = w.k, kb = w.k >> 8;
    const int64_t tiles = w.n / 16;
    uint8_t *wgt_base = smem + kb * R::kActBlk;

    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    const uint32_t act_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    const uint32_t wq_off = r8 * (uint32_t)kb * 128u + ((c8 ^ r8) << 4);
    const uint32_t r16 = lane >> 2, c4 = lane & 3;
    const uint32_t wh_off = r16 * (uint32_t)kb * 64u + ((c4 ^ ((r16 >> 1) & 3)) << 4);
    const uint32_t w5_off = (lane >> 1) * (uint32_t)kb * 32u + (lane & 1) * 16u;
    uint32_t a_col[NT][2];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const uint32_t row = t * 16 + r < 8u * RT ? t * 16 + r : 8u * RT - 1;
#pragma unroll
        for (uint32_t e = 0; e < 2; e++)
            a_col[t][e] = (row >> 3) * 2048u + (row & 7) * 128u + (((4 * e + kq) ^ (row & 7)) << 4);
    }
    ResPlanes pl;
    pl.wq = wave_rsrc(w.p0);
    pl.wh = wave_rsrc(w.p1);
    pl.w5 = wave_rsrc(w.p2);
    pl.aq = wave_rsrc(a.qs);
    pl.ad = wave_rsrc(a.dT);
    pl.am = wave_rsrc(a.bsh);
    const uint32_t kb32 = (uint32_t)kb, k32 = (uint32_t)k, mstr = (uint32_t)a.m_stride;
    // ---- the wave's K blocks: the small fields of the first tile's weights (registers; requested first, they are
    // what the unpacking starts with), activation slices once, weights of the first tile
    int64_t tile = blockIdx.x;
    WHead<DT> head[kMaxBpw];
#pragma unroll
    for (int j = 0; j < kMaxBpw; j++) {
        const int64_t b = wave + (int64_t)j * kWaves;
        if (b < kb && tile < tiles) load_head(w, (tile * 16 + r) * kb + b, head[j]);
    }
#pragma unroll
    for (int j = 0; j < kMaxBpw; j++) {
        const uint32_t b = (uint32_t)wave + (uint32_t)j * kWaves;
        if (b < kb32) {
            uint8_t *act = smem + b * R::kActBlk;
#pragma unroll
            for (int i = 0; i < 2 * RT; i++) {
                const uint32_t rg = i >> 1, kh = i & 1;
                dma16s(pl.aq, act_off, rg * 8u * k32 + b * 256u + kh * 128u, act + i * 1024);
            }
            if (lane < 8 * RT) dma4s(pl.ad, lane * 4u, b * mstr * 4u, act + R::oD8);
            if (MINS && lane < 16 * RT) dma16s(pl.am, lane * 16u, b * mstr * 32u, act + R::oMin);
            if (tile < tiles)
                res_issue_weights<DT>(wgt_base + (b * NBUF) * R::kWgt, pl, (uint32_t)tile * 16u, b, kb32, wq_off, wh_off, w5_off, lane);
        }
    }
    int par = 0;
    for (; tile < tiles; tile += gridDim.x) {
        const int64_t n_tile = tile * 16, next = tile + gridDim.x;
        __builtin_amdgcn_s_waitcnt(0);   // this tile's weights (and, the first time, the activations) have landed
        if (NBUF == 2 && next < tiles) {
#pragma unroll
            for (int j = 0; j < kMaxBpw; j++) {
                const int64_t b = wave + (int64_t)j * kWaves;
                if (b < kb)
                    res_issue_weights<DT>(wgt_base + (b * NBUF + (par ^ 1)) * R::kWgt, pl, (uint32_t)next * 16u, (uint32_t)b, kb32,
                                          wq_off, wh_off, w5_off, lane);
            }
        }
        v4f out[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) out[t] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < kMaxBpw; j++) {
            const int64_t b = wave + (int64_t)j * kWaves;
            if (b < kb)
                res_block<DT, RT, NT, DUMP>(wgt_base + (b * NBUF + (NBUF == 2 ? par : 0)) * R::kWgt, smem + b * R::kActBlk, lane,
                                            head[j], a_col, out, dump, (n_tile + r) * kb + b, w.n * kb, m);
        }
        // ---- sum the waves' partial tiles in wave order (through the wave's first weight buffer of this tile)
        uint8_t *part = wgt_base + ((int64_t)wave * NBUF + (NBUF == 2 ? par : 0)) * R::kWgt;
        if (wave < kb) {   // (a wave without a K block has no buffer and nothing to add)
#pragma unroll
            for (int t = 0; t < NT; t++) *(v4f *)(part + t * 1024 + lane * 16) = out[t];
        }
        __syncthreads();
        if (wave < NT && !DUMP) {
            v4f s = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
            const int64_t nw = kb < kWaves ? kb : kWaves;   // waves that own a block
            for (int64_t o = 0; o < nw; o++) {
                const v4f p = *(const v4f *)(wgt_base + (o * NBUF + (NBUF == 2 ? par : 0)) * R::kWgt + wave * 1024 + lane * 16);
                s += p;
            }
            const int64_t col = n_tile + r;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int64_t row = wave * 16 + kq * 4 + i;
                if (row < m) y[row * w.n + col] = s[i];
            }
        }
        if (NBUF == 1 && next < tiles) {
            __syncthreads();   // the partial results have been read: the buffers take the next tile's weights
#pragma unroll
            for (int j = 0; j < kMaxBpw; j++) {
                const int64_t b = wave + (int64_t)j * kWaves;
                if (b < kb)
                    res_issue_weights<DT>(wgt_base + b * R::kWgt, pl, (uint32_t)next * 16u, (uint32_t)b, kb32, wq_off, wh_off, w5_off, lane);
            }
        } else if (NBUF == 2) {
            __syncthreads();   // ... before the tile after the next one is copied over them
        }
        if (next < tiles) {
#pragma unroll
            for (int j = 0; j < kMaxBpw; j++) {
                const int64_t b = wave + (int64_t)j * kWaves;
                if (b < kb) load_head(w, (next * 16 + r) * kb + b, head[j]);
            }
        }
        par ^= 1;
    }
}

// ------------------------------------------- resident activations, several tiles per workgroup ----
// More weight rows than 16 x the number of CUs: every workgroup walks several 16-row tiles.  With one K block per
// wave (k <= 256 x waves) a wave keeps its partial result of each tile in registers and the workgroup meets once per
// round of up to four tiles, not once per tile: between two tiles of a round there is no barrier and no wait for
// the slowest wave, so the copies of the tile after the next one (issued into the buffer the current tile has just
// been unpacked from) really are in flight under the arithmetic.  Everything a tile needs comes through LDS copies,
// the 20-byte block headers included: a load into registers would be tracked by the compiler, which on joining the
// paths "copies issued" and "no tile left to copy" waits as the stricter of the two demands, i.e. for everything.
// The waits are written out by hand instead (s_waitcnt vmcnt(copies of one tile) while a next tile is in flight).
// The partial tiles of a round are summed in wave order as in the kernels above.  Q4K and Q5K (one header layout).
//   LDS: activation slices as skinny_resident_kernel | per wave two slots {weights kWgt | headers 16 x 16 B, 16 x 4 B},
//        which take the wave's partial results (1 KiB per tile) at the end of a round
constexpr int kTilesPerRound = 4;
template <int DT, int RT> struct ResMulti {
    static constexpr int kWgt = Res<DT, RT>::kWgt;
    static constexpr int oHdr = kWgt, kSlot = kWgt + 320;
    static constexpr int kCopies = (DT == CQ_DTYPE_Q4K ? 2 : 3) + 2;   // copy instructions per tile (multi_issue)
    static size_t bytes(int64_t kb) { return (size_t)kb * Res<DT, RT>::kActBlk + (size_t)kb * 2 * kSlot; }
};

// The copies of one tile's K block b into `slot`: weights as res_issue_weights, then the 16 rows' headers
// (bytes 0..15 of row r at oHdr + 16 r, bytes 16..19 at oHdr + 256 + 4 r; lanes 0..15).
template <int DT, int RT>
__device__ __forceinline__ void multi_issue(uint8_t *__restrict__ slot, const ResPlanes &pl, __amdgpu_buffer_rsrc_t hdr, uint32_t n_tile,
                                            uint32_t b, uint32_t kb, uint32_t wq_off, uint32_t w5_off, uint32_t hd_off, int lane) {
    typedef ResMulti<DT, RT> M;
    res_issue_weights<DT>(slot, pl, n_tile, b, kb, wq_off, 0, w5_off, lane);
    const uint32_t blk = n_tile * kb + b;
    if (lane < 16) {
        dma16s(hdr, hd_off, blk * (uint32_t)CQ_Q4K_HDR, slot + M::oHdr);
        // (the instruction's immediate offset moves both addresses: bytes 16.. of the header, and 16 bytes on in LDS)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(hdr, (lptr_t)(slot + M::oHdr + 256 - 16), 4, (int)hd_off, (int)(blk * (uint32_t)CQ_Q4K_HDR), 16, 0);
    }
}

// One tile of one wave: operands out of `slot`, then (the slot is free) the copies of the tile two ahead, then the MFMAs.
template <int DT, int RT, bool DUMP>
__device__ __forceinline__ void multi_step(uint8_t *__restrict__ slot, const uint8_t *__restrict__ act, int lane, const ResPlanes &pl,
                                           __amdgpu_buffer_rsrc_t hdr, bool ahead, uint32_t tile_ahead, uint32_t b, uint32_t kb32,
                                           uint32_t wq_off, uint32_t w5_off, uint32_t hd_off, const uint32_t (&a_col)[1][2],
                                           v4f (&out)[1], const cq_mfma_dump &dump, int64_t at, int64_t rs, int64_t m) {
    typedef ResMulti<DT, RT> M;
    const uint32_t r = lane & 15;
    WHead<DT> head;
    const uint4 h4 = *(const uint4 *)(slot + M::oHdr + r * 16u);
    head.dd = h4.x;
    head.rec = make_uint4(h4.y, h4.z, h4.w, *(const uint32_t *)(slot + M::oHdr + 256 + r * 4u));
    ResOps o;
    res_unpack<DT, DUMP>(slot, lane, head, dump, o);
    if (ahead) {
        __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the reads above are done with the slot
        multi_issue<DT, RT>(slot, pl, hdr, tile_ahead * 16u, b, kb32, wq_off, w5_off, hd_off, lane);
    }
    res_mac<DT, RT, 1, DUMP>(act, lane, o, a_col, out, dump, at, rs, m);
}

// m <= 8 * RT <= 16 activation rows; n % 16 == 0; k / 256 <= kWaves.
template <int DT, int RT, int kWaves, bool DUMP>
__global__ void __launch_bounds__(kWaves * 64) skinny_resident_multi_kernel(cq_weight w, cq_act_view a, int64_t m,
                                                                            float *__restrict__ y, cq_mfma_dump dump) {
    typedef Res<DT, RT> R;
    typedef ResMulti<DT, RT> M;
    static_assert(DT == CQ_DTYPE_Q4K || DT == CQ_DTYPE_Q5K, "block headers of 20 bytes");
    static_assert(RT <= 2, "one 16-row tile of activation rows");
    static_assert(2 * M::kSlot >= kTilesPerRound * 1024, "a round's partial tiles fit the wave's two slots");
    constexpr bool MINS = is_k4(DT);
    constexpr int kAhead = 0x0F70 | M::kCopies;   // s_waitcnt vmcnt(copies of one tile)
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15, kq = lane >> 4;
    const int64_t k = w.k, kb = w.k >> 8;
    const int64_t tiles = w.n / 16, G = gridDim.x;
    uint8_t *wgt_base = smem + kb * R::kActBlk;
    const bool has = wave < kb;   // this wave owns K block `wave`
    const uint32_t b = (uint32_t)wave;

    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    const uint32_t act_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    const uint32_t wq_off = r8 * (uint32_t)kb * 128u + ((c8 ^ r8) << 4);
    const uint32_t w5_off = (lane >> 1) * (uint32_t)kb * 32u + (lane & 1) * 16u;
    const uint32_t hd_off = (uint32_t)lane * (uint32_t)kb * (uint32_t)CQ_Q4K_HDR;   // lanes 0..15: the header of row `lane`
    uint32_t a_col[1][2];
    {
        const uint32_t row = r < 8u * RT ? r : 8u * RT - 1;
#pragma unroll
        for (uint32_t e = 0; e < 2; e++) a_col[0][e] = (row >> 3) * 2048u + (row & 7) * 128u + (((4 * e + kq) ^ (row & 7)) << 4);
    }
    ResPlanes pl;
    pl.wq = wave_rsrc(w.p0);
    pl.wh = wave_rsrc(w.p1);
    pl.w5 = wave_rsrc(w.p2);
    pl.aq = wave_rsrc(a.qs);
    pl.ad = wave_rsrc(a.dT);
    pl.am = wave_rsrc(a.bsh);
    const __amdgpu_buffer_rsrc_t hdr = wave_rsrc(w.p1);
    const uint32_t kb32 = (uint32_t)kb, k32 = (uint32_t)k, mstr = (uint32_t)a.m_stride;
    uint8_t *act = smem + b * R::kActBlk;
    uint8_t *ring = wgt_base + (size_t)b * 2 * M::kSlot;

    // ---- the wave's activation slice, once
    if (has) {
#pragma unroll
        for (int i = 0; i < 2 * RT; i++) {
            const uint32_t rg = i >> 1, kh = i & 1;
            dma16s(pl.aq, act_off, rg * 8u * k32 + b * 256u + kh * 128u, act + i * 1024);
        }
        if (lane < 8 * RT) dma4s(pl.ad, lane * 4u, b * mstr * 4u, act + R::oD8);
        if (MINS && lane < 16 * RT) dma16s(pl.am, lane * 16u, b * mstr * 32u, act + R::oMin);
    }
    for (int64_t t0 = blockIdx.x; t0 < tiles; t0 += kTilesPerRound * G) {
        // tiles of this round: t0, t0 + G, ... (cnt of them)
        int cnt = (int)((tiles - t0 + G - 1) / G);
        cnt = cnt < kTilesPerRound ? cnt : kTilesPerRound;
        if (has) {
            v4f o0 = {0.0f, 0.0f, 0.0f, 0.0f}, o1 = o0, o2 = o0, o3 = o0;
            multi_issue<DT, RT>(ring, pl, hdr, (uint32_t)t0 * 16u, b, kb32, wq_off, w5_off, hd_off, lane);
            if (cnt > 1) multi_issue<DT, RT>(ring + M::kSlot, pl, hdr, (uint32_t)(t0 + G) * 16u, b, kb32, wq_off, w5_off, hd_off, lane);
#pragma nounroll
            for (int i = 0; i < cnt; i++) {
                // everything but the copies of the next tile has landed
                if (i + 1 < cnt) __builtin_amdgcn_s_waitcnt(kAhead);
                else __builtin_amdgcn_s_waitcnt(0x0F70);
                const int64_t tile = t0 + i * G;
                v4f acc[1] = {{0.0f, 0.0f, 0.0f, 0.0f}};
                multi_step<DT, RT, DUMP>(ring + (i & 1) * M::kSlot, act, lane, pl, hdr, i + 2 < cnt, (uint32_t)(tile + 2 * G), b, kb32,
                                         wq_off, w5_off, hd_off, a_col, acc, dump, (tile * 16 + r) * kb + b, w.n * kb, m);
                // (i is wave-uniform: real branches, four moves, instead of sixteen selects - the empty statements keep them)
                if (i == 0) { o0 = acc[0]; asm volatile(""); }
                else if (i == 1) { o1 = acc[0]; asm volatile(""); }
                else if (i == 2) { o2 = acc[0]; asm volatile(""); }
                else { o3 = acc[0]; asm volatile(""); }
            }
            // ---- the round's partial tiles into the wave's slots (every copy into them has landed and been unpacked)
            *(v4f *)(ring + lane * 16) = o0;
            *(v4f *)(ring + 1024 + lane * 16) = o1;
            *(v4f *)(ring + 2048 + lane * 16) = o2;
            *(v4f *)(ring + 3072 + lane * 16) = o3;
        }
        __syncthreads();
        if (wave < cnt && !DUMP) {   // wave i sums tile i of the round, in wave order
            v4f s = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
            const int64_t nw = kb < kWaves ? kb : kWaves;   // waves that own a block
            for (int64_t o = 0; o < nw; o++) {
                const v4f p = *(const v4f *)(wgt_base + (size_t)o * 2 * M::kSlot + wave * 1024 + lane * 16);
                s += p;
            }
            const int64_t col = (t0 + wave * G) * 16 + r;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int64_t row = kq * 4 + i;
                if (row < m) y[row * w.n + col] = s[i];
            }
        }
        if (t0 + kTilesPerRound * G < tiles) __syncthreads();   // the sums have been read: the slots take the next round's copies
    }
}

// ---------------------------------------------------- Q8_0 / Q4_0 weights x Q8_0 activations ----
// The same work split for 32-element blocks (k_quants.rs:618-649, :224-254: sumf += sumi * d_w *
// d_x per block).  Q8_0 weights are int8 already and Q4_0 weights are one mask away from it, so the
// operands go from LDS (almost) straight into the 16x16x32 MFMA, one per block, and each block's
// 16 x 16 integers are scaled by the two block scales on the way into the f32 result.  Q4_0 holds
// q - 8; the MFMA contracts q and 8 * (sum of the block's activations) comes off afterwards.  A wave
// takes 256 elements (eight blocks) per step.
//   wgt : Q8_0 [2 row groups][2 K-halves][8 rows][8 chunks of 16 B], Q4_0 [2 row groups][8 rows][8 chunks
//         = blocks]; chunk c of row r at c ^ (r%8)
//   act : [RT row groups][2 K-halves][8 rows][8 chunks], same swizzle
template <int RT> struct BufQ8 {
    static constexpr int oAct = 4096, kRaw = oAct + RT * 2048;
    static constexpr int kBytes = kRaw;   // >= 2 KiB of partial results
};

template <int DT, int RT, bool DUMP>
__global__ void __launch_bounds__(kThreads) skinny_blk32_kernel(cq_weight w, cq_act_view a, int64_t m0, int64_t m,
                                                                float *__restrict__ y, cq_mfma_dump dump) {
    typedef BufQ8<RT> B;
    constexpr bool Q4 = DT == CQ_DTYPE_Q4_0;
    constexpr int NT = (RT + 1) / 2;   // 16-row tiles
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15, kq = lane >> 4;
    const int64_t k = w.k, kg = w.k >> 8, kb = w.k >> 5;
    const int64_t n_tile = (int64_t)blockIdx.x * 16;
    uint8_t *buf = smem + wave * B::kBytes;

    // copy offsets: 8 rows x 128 B per instruction, chunks swizzled by the row
    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    const uint32_t row_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    const uint32_t q4_off = r8 * (uint32_t)(k >> 1) + ((c8 ^ r8) << 4);   // Q4_0: 128 bytes per row and step
    // operand reads: 8 bytes [32b + 8kq, +8) of a row = half b/4, chunk 2(b%4) + kq/2, byte 8(kq%2);
    // Q4_0 weights: chunk b, bytes 8(kq%2) .. +8, low nibbles for kq < 2, high nibbles above
    const uint32_t w4_col = (r >> 3) * 1024u + (r & 7) * 128u + (kq & 1) * 8u, w4_shift = 4 * (kq >> 1);
    uint32_t w_col[4], a_col[NT][4];
    int64_t a_row[NT][4];   // rows whose scales this lane applies (results rows 4kq + i of tile t)
#pragma unroll
    for (uint32_t c = 0; c < 4; c++) w_col[c] = (r >> 3) * 2048u + (r & 7) * 128u + (((2 * c + (kq >> 1)) ^ (r & 7)) << 4) + (kq & 1) * 8u;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const uint32_t row = t * 16 + r < 8u * RT ? t * 16 + r : 8u * RT - 1;
#pragma unroll
        for (uint32_t c = 0; c < 4; c++)
            a_col[t][c] = B::oAct + (row >> 3) * 2048u + (row & 7) * 128u + (((2 * c + (kq >> 1)) ^ (row & 7)) << 4) + (kq & 1) * 8u;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t row_i = m0 + t * 16 + 4 * kq + i;
            a_row[t][i] = row_i < m ? row_i : m - 1;
        }
    }

    v4f out[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) out[t] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};

    for (int64_t g = wave; g < kg; g += kWaves) {
        if (Q4) {
#pragma unroll
            for (int rg = 0; rg < 2; rg++) dma16(w.p0 + (n_tile + rg * 8) * (k >> 1) + g * 128, q4_off, buf + rg * 1024);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int rg = i >> 1, kh = i & 1;
                dma16(w.p0 + (n_tile + rg * 8) * k + g * 256 + kh * 128, row_off, buf + i * 1024);
            }
        }
#pragma unroll
        for (int i = 0; i < 2 * RT; i++) {
            const int rg = i >> 1, kh = i & 1;
            dma16(a.qs + (m0 + rg * 8) * k + g * 256 + kh * 128, row_off, buf + B::oAct + i * 1024);
        }
        // the eight block scales of this lane's weight row, and of the activation rows it scales
        const uint4 dwv = *(const uint4 *)(w.p1 + ((n_tile + r) * kb + g * 8) * 2);
        v4f da[NT][4][2];
        v4i bs[Q4 ? NT : 1][4][2];   // Q4_0: the sums of the activation blocks
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const v4f *p = (const v4f *)(a.d + a_row[t][i] * kb + g * 8);
                da[t][i][0] = p[0];
                da[t][i][1] = p[1];
                if (Q4) {
                    const v4i *q = (const v4i *)(a.bsum32 + a_row[t][i] * kb + g * 8);
                    bs[t][i][0] = q[0];
                    bs[t][i][1] = q[1];
                }
            }
        __builtin_amdgcn_s_waitcnt(0);   // everything above has landed

        const uint32_t dww[4] = {dwv.x, dwv.y, dwv.z, dwv.w};
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const float dw = cq_h2f((uint16_t)(dww[b >> 1] >> (16 * (b & 1))));
            long wv;
            if (Q4) {
                const uint2 raw = *(const uint2 *)(buf + w4_col + (((uint32_t)b ^ (r & 7)) << 4));
                const uint32_t lo = (raw.x >> w4_shift) & 0x0F0F0F0Fu, hi = (raw.y >> w4_shift) & 0x0F0F0F0Fu;
                wv = (long)(((uint64_t)hi << 32) | lo);
            } else {
                wv = *(const long *)(buf + w_col[b & 3] + (b >> 2) * 1024);
            }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const long av = *(const long *)(buf + a_col[t][b & 3] + (b >> 2) * 1024);
                const v4i acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(av, wv, (v4i){0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int I = Q4 ? acc[i] - 8 * bs[Q4 ? t : 0][i][b >> 2][b & 3] : acc[i];
                    if (DUMP) {
                        const int64_t orow = m0 + t * 16 + kq * 4 + i;
                        if (orow < m) dump.i[(orow * w.n + n_tile + r) * kb + g * 8 + b] = I;
                    } else {
                        out[t][i] = __builtin_fmaf((float)I * dw, da[t][i][b >> 2][b & 3], out[t][i]);
                    }
                }
            }
        }
    }
    if (DUMP) return;

    // ---- sum the eight waves' partial tiles in wave order
#pragma unroll
    for (int t = 0; t < NT; t++) *(v4f *)(buf + t * 1024 + lane * 16) = out[t];
    __syncthreads();
    if (wave < NT) {
        v4f s = *(const v4f *)(smem + wave * 1024 + lane * 16);
#pragma unroll
        for (int o = 1; o < kWaves; o++) {
            const v4f p = *(const v4f *)(smem + o * B::kBytes + wave * 1024 + lane * 16);
            s += p;
        }
        const int64_t col = n_tile + r;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t row = m0 + wave * 16 + kq * 4 + i;
            if (row < m) y[row * w.n + col] = s[i];
        }
    }
}

// ------------------------------------------- the same with everything of a workgroup in flight at once ----
// The kernel above has one 256-element step per wave in flight and spends most of its life waiting (56 % at
// s_waitcnt, the vector units 18 % busy).  Where every workgroup has one 16-row weight tile (n <= 16 x the number of
// compute units) and the call's quantized rows fit the LDS beside the weights, every wave requests all it will need -
// the activation slices, scales and weights of the K groups it owns (wave w: groups w, w + kWaves, ...) - right away,
// a single memory round trip, and the arithmetic follows as the data lands.
//   per K group g : act [RT][2 K-halves][8 rows][8 chunks], swizzled as above | d [8*RT rows][8] f32 |
//                   Q4_0: bs [8*RT rows][8] i32 (sums of the activation blocks)
//   then, per group: the 16 weight rows (Q8_0 4 KiB, Q4_0 2 KiB); a wave's first weight buffer also carries its
//                   partial results (1 KiB per 16 activation rows)
template <int DT, int RT> struct ResQ8 {
    static constexpr bool Q4 = DT == CQ_DTYPE_Q4_0;
    static constexpr int kWgt = Q4 ? 2048 : 4096;
    static constexpr int oD = RT * 2048, oBs = oD + RT * 256;
    static constexpr int kActGrp = oBs + (Q4 ? RT * 256 : 0);
    static size_t bytes(int64_t kg) { return (size_t)kg * (kActGrp + kWgt); }
};

// m <= 8 * RT rows; n % 16 == 0, one tile per workgroup (gridDim.x == n / 16); at most kMaxBpw K groups per wave.
template <int DT, int RT, int kWaves, bool DUMP>
__global__ void __launch_bounds__(kWaves * 64) skinny_blk32_resident_kernel(cq_weight w, cq_act_view a, int64_t m,
                                                                            float *__restrict__ y, cq_mfma_dump dump) {
    typedef ResQ8<DT, RT> R;
    constexpr bool Q4 = R::Q4;
    constexpr int NT = (RT + 1) / 2;   // 16-row tiles
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15, kq = lane >> 4;
    const int64_t k = w.k, kg = w.k >> 8, kb = w.k >> 5;
    const int64_t n_tile = (int64_t)blockIdx.x * 16;
    uint8_t *wgt_base = smem + kg * R::kActGrp;

    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    const uint32_t row_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    const uint32_t q4_off = r8 * (uint32_t)(k >> 1) + ((c8 ^ r8) << 4);
    // the scales (and block sums) of row l / 2, half l % 2 of its eight blocks; rows past the last one repeat it
    // (their planes are not padded)
    const int64_t srow = (int64_t)(lane >> 1) < m ? (lane >> 1) : m - 1;
    const uint32_t sc_off = (uint32_t)(srow * kb * 4) + (lane & 1) * 16u;
    const uint32_t w4_col = (r >> 3) * 1024u + (r & 7) * 128u + (kq & 1) * 8u, w4_shift = 4 * (kq >> 1);
    uint32_t w_col[4], a_col[NT][4];
#pragma unroll
    for (uint32_t c = 0; c < 4; c++) w_col[c] = (r >> 3) * 2048u + (r & 7) * 128u + (((2 * c + (kq >> 1)) ^ (r & 7)) << 4) + (kq & 1) * 8u;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const uint32_t row = t * 16 + r < 8u * RT ? t * 16 + r : 8u * RT - 1;
#pragma unroll
        for (uint32_t c = 0; c < 4; c++)
            a_col[t][c] = (row >> 3) * 2048u + (row & 7) * 128u + (((2 * c + (kq >> 1)) ^ (row & 7)) << 4) + (kq & 1) * 8u;
    }

    // ---- everything this wave will need, requested at once
    uint4 dwv[kMaxBpw];
#pragma unroll
    for (int j = 0; j < kMaxBpw; j++) {
        const int64_t g = wave + (int64_t)j * kWaves;
        if (g < kg) dwv[j] = *(const uint4 *)(w.p1 + ((n_tile + r) * kb + g * 8) * 2);
    }
#pragma unroll
    for (int j = 0; j < kMaxBpw; j++) {
        const int64_t g = wave + (int64_t)j * kWaves;
        if (g < kg) {
            uint8_t *act = smem + g * R::kActGrp, *wl = wgt_base + g * R::kWgt;
#pragma unroll
            for (int i = 0; i < 2 * RT; i++) {
                const int rg = i >> 1, kh = i & 1;
                dma16(a.qs + (int64_t)(rg * 8) * k + g * 256 + kh * 128, row_off, act + i * 1024);
            }
            if (lane < 16 * RT) dma16((const uint8_t *)(a.d + g * 8), sc_off, act + R::oD);
            if (Q4 && lane < 16 * RT) dma16((const uint8_t *)(a.bsum32 + g * 8), sc_off, act + R::oBs);
            if (Q4) {
#pragma unroll
                for (int rg = 0; rg < 2; rg++) dma16(w.p0 + (n_tile + rg * 8) * (k >> 1) + g * 128, q4_off, wl + rg * 1024);
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int rg = i >> 1, kh = i & 1;
                    dma16(w.p0 + (n_tile + rg * 8) * k + g * 256 + kh * 128, row_off, wl + i * 1024);
                }
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0);   // everything above has landed

    v4f out[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) out[t] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < kMaxBpw; j++) {
        const int64_t g = wave + (int64_t)j * kWaves;
        if (g < kg) {
            const uint8_t *act = smem + g * R::kActGrp, *wl = wgt_base + g * R::kWgt;
            const uint32_t dww[4] = {dwv[j].x, dwv[j].y, dwv[j].z, dwv[j].w};
#pragma unroll
            for (int b = 0; b < 8; b++) {
                const float dw = cq_h2f((uint16_t)(dww[b >> 1] >> (16 * (b & 1))));
                long wv;
                if (Q4) {
                    const uint2 raw = *(const uint2 *)(wl + w4_col + (((uint32_t)b ^ (r & 7)) << 4));
                    const uint32_t lo = (raw.x >> w4_shift) & 0x0F0F0F0Fu, hi = (raw.y >> w4_shift) & 0x0F0F0F0Fu;
                    wv = (long)(((uint64_t)hi << 32) | lo);
                } else {
                    wv = *(const long *)(wl + w_col[b & 3] + (b >> 2) * 1024);
                }
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const long av = *(const long *)(act + a_col[t][b & 3] + (b >> 2) * 1024);
                    const v4i acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(av, wv, (v4i){0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        // scales of result row 4kq + i of tile t (rows past the held groups: the last one, not stored)
                        const uint32_t srow_i = t * 16 + 4 * kq + i < 8u * RT ? t * 16 + 4 * kq + i : 8u * RT - 1;
                        const float da = *(const float *)(act + R::oD + srow_i * 32 + b * 4);
                        const int I = Q4 ? acc[i] - 8 * *(const int32_t *)(act + R::oBs + srow_i * 32 + b * 4) : acc[i];
                        if (DUMP) {
                            const int64_t orow = t * 16 + kq * 4 + i;
                            if (orow < m) dump.i[(orow * w.n + n_tile + r) * kb + g * 8 + b] = I;
                        } else {
                            out[t][i] = __builtin_fmaf((float)I * dw, da, out[t][i]);
                        }
                    }
                }
            }
        }
    }
    if (DUMP) return;

    // ---- sum the waves' partial tiles in wave order (through each wave's first weight buffer)
    if (wave < kg) {
#pragma unroll
        for (int t = 0; t < NT; t++) *(v4f *)(wgt_base + (int64_t)wave * R::kWgt + t * 1024 + lane * 16) = out[t];
    }
    __syncthreads();
    if (wave < NT) {
        v4f s = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
        const int64_t nw = kg < kWaves ? kg : kWaves;   // waves that own a group
        for (int64_t o = 0; o < nw; o++) {
            const v4f p = *(const v4f *)(wgt_base + o * R::kWgt + wave * 1024 + lane * 16);
            s += p;
        }
        const int64_t col = n_tile + r;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t row = wave * 16 + kq * 4 + i;
            if (row < m) y[row * w.n + col] = s[i];
        }
    }
}

// ------------------------------------- Q8_0 / Q4_0: resident activations, several tiles per workgroup ----
// The counterpart of skinny_resident_multi_kernel for the 32-element block types: one K group of 256 elements per wave
// (k <= 256 x waves), rounds of up to four 16-row tiles with one meeting per round, the weight scales through an LDS
// copy like the weights.  Q8_0 tiles are 4 KiB per wave and the LDS has room for one slot each: a tile's operands
// are read into registers first and the next tile's copies go out right behind them, under the MFMAs and the
// scaling.  Q4_0 (2 KiB) has two slots and keeps the tile after the next in flight.
//   LDS: activation groups as skinny_blk32_resident_kernel | per wave kSlots x {weights kWgt | scales 16 rows x 16 B};
//        the slots take the wave's partial results (1 KiB per tile) at the end of a round
template <int DT, int RT> struct ResQ8Multi {
    typedef ResQ8<DT, RT> R;
    static constexpr int kSlots = R::Q4 ? 2 : 1;
    static constexpr int oSc = R::kWgt, kSlot = R::kWgt + 256;
    static constexpr int kCopies = (R::Q4 ? 2 : 4) + 1;   // copy instructions per tile (blk32_multi_issue)
    static size_t bytes(int64_t kg) { return (size_t)kg * R::kActGrp + (size_t)kg * kSlots * kSlot; }
};

template <int DT, int RT>
__device__ __forceinline__ void blk32_multi_issue(uint8_t *__restrict__ slot, const cq_weight &w, int64_t n_tile, int64_t g, uint32_t row_off,
                                                  uint32_t q4_off, uint32_t ws_off, int lane) {
    typedef ResQ8Multi<DT, RT> M;
    const int64_t k = w.k, kb = w.k >> 5;
    if (M::R::Q4) {
#pragma unroll
        for (int rg = 0; rg < 2; rg++) dma16(w.p0 + (n_tile + rg * 8) * (k >> 1) + g * 128, q4_off, slot + rg * 1024);
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int rg = i >> 1, kh = i & 1;
            dma16(w.p0 + (n_tile + rg * 8) * k + g * 256 + kh * 128, row_off, slot + i * 1024);
        }
    }
    if (lane < 16) dma16(w.p1 + (n_tile * kb + g * 8) * 2, ws_off, slot + M::oSc);   // eight f16 scales of row `lane`
}

// One tile of one wave: operands out of `slot` into registers, the copies of a tile ahead into the free slot, MFMAs.
template <int DT, int RT, bool DUMP>
__device__ __forceinline__ void blk32_multi_step(uint8_t *__restrict__ slot, const uint8_t *__restrict__ act, int lane, const cq_weight &w,
                                                 bool ahead, int64_t tile_ahead, int64_t g, uint32_t row_off, uint32_t q4_off,
                                                 uint32_t ws_off, uint32_t w4_col, uint32_t w4_shift, const uint32_t (&w_col)[4],
                                                 const uint32_t (&a_col)[4], v4f &out, const cq_mfma_dump &dump, int64_t at, int64_t rs,
                                                 int64_t m) {
    typedef ResQ8Multi<DT, RT> M;
    typedef ResQ8<DT, RT> R;
    constexpr bool Q4 = R::Q4;
    const uint32_t r = lane & 15, kq = lane >> 4;
    const uint4 dwv = *(const uint4 *)(slot + M::oSc + r * 16u);
    long wv[8];
#pragma unroll
    for (int b = 0; b < 8; b++) {
        if (Q4) {
            const uint2 raw = *(const uint2 *)(slot + w4_col + (((uint32_t)b ^ (r & 7)) << 4));
            const uint32_t lo = (raw.x >> w4_shift) & 0x0F0F0F0Fu, hi = (raw.y >> w4_shift) & 0x0F0F0F0Fu;
            wv[b] = (long)(((uint64_t)hi << 32) | lo);
        } else {
            wv[b] = *(const long *)(slot + w_col[b & 3] + (b >> 2) * 1024);
        }
    }
    if (ahead) {
        __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the reads above are done with the slot
        blk32_multi_issue<DT, RT>(slot, w, tile_ahead * 16, g, row_off, q4_off, ws_off, lane);
    }
    const uint32_t dww[4] = {dwv.x, dwv.y, dwv.z, dwv.w};
#pragma unroll
    for (int b = 0; b < 8; b++) {
        const float dw = cq_h2f((uint16_t)(dww[b >> 1] >> (16 * (b & 1))));
        const long av = *(const long *)(act + a_col[b & 3] + (b >> 2) * 1024);
        const v4i acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(av, wv[b], (v4i){0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // scales of result row 4kq + i (rows past the held groups: the last one, not stored)
            const uint32_t srow_i = 4 * kq + i < 8u * RT ? 4 * kq + i : 8u * RT - 1;
            const float da = *(const float *)(act + R::oD + srow_i * 32 + b * 4);
            const int I = Q4 ? acc[i] - 8 * *(const int32_t *)(act + R::oBs + srow_i * 32 + b * 4) : acc[i];
            if (DUMP) {
                const int64_t orow = kq * 4 + i;
                if (orow < m) dump.i[at + orow * rs + b] = I;
            } else {
                out[i] = __builtin_fmaf((float)I * dw, da, out[i]);
            }
        }
    }
}

// m <= 8 * RT <= 16 rows; n % 16 == 0; k / 256 <= kWaves.
template <int DT, int RT, int kWaves, bool DUMP>
__global__ void __launch_bounds__(kWaves * 64) skinny_blk32_multi_kernel(cq_weight w, cq_act_view a, int64_t m,
                                                                         float *__restrict__ y, cq_mfma_dump dump) {
    typedef ResQ8<DT, RT> R;
    typedef ResQ8Multi<DT, RT> M;
    constexpr bool Q4 = R::Q4;
    static_assert(RT <= 2, "one 16-row tile of activation rows");
    static_assert(M::kSlots * M::kSlot >= kTilesPerRound * 1024, "a round's partial tiles fit the wave's slots");
    constexpr int kAhead = 0x0F70 | M::kCopies;   // s_waitcnt vmcnt(copies of one tile)
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15, kq = lane >> 4;
    const int64_t k = w.k, kg = w.k >> 8, kb = w.k >> 5;
    const int64_t tiles = w.n / 16, G = gridDim.x;
    uint8_t *wgt_base = smem + kg * R::kActGrp;
    const bool has = wave < kg;   // this wave owns K group `wave`
    const int64_t g = wave;

    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    const uint32_t row_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    const uint32_t q4_off = r8 * (uint32_t)(k >> 1) + ((c8 ^ r8) << 4);
    const uint32_t ws_off = (uint32_t)lane * (uint32_t)kb * 2u;   // lanes 0..15: the scales of row `lane`
    const int64_t srow = (int64_t)(lane >> 1) < m ? (lane >> 1) : m - 1;
    const uint32_t sc_off = (uint32_t)(srow * kb * 4) + (lane & 1) * 16u;
    const uint32_t w4_col = (r >> 3) * 1024u + (r & 7) * 128u + (kq & 1) * 8u, w4_shift = 4 * (kq >> 1);
    uint32_t w_col[4], a_col[4];
    {
        const uint32_t row = r < 8u * RT ? r : 8u * RT - 1;
#pragma unroll
        for (uint32_t c = 0; c < 4; c++) {
            w_col[c] = (r >> 3) * 2048u + (r & 7) * 128u + (((2 * c + (kq >> 1)) ^ (r & 7)) << 4) + (kq & 1) * 8u;
            a_col[c] = (row >> 3) * 2048u + (row & 7) * 128u + (((2 * c + (kq >> 1)) ^ (row & 7)) << 4) + (kq & 1) * 8u;
        }
    }
    uint8_t *act = smem + g * R::kActGrp;
    uint8_t *ring = wgt_base + (size_t)g * M::kSlots * M::kSlot;

    // ---- the wave's activation group, once
    if (has) {
#pragma unroll
        for (int i = 0; i < 2 * RT; i++) {
            const int rg = i >> 1, kh = i & 1;
            dma16(a.qs + (int64_t)(rg * 8) * k + g * 256 + kh * 128, row_off, act + i * 1024);
        }
        if (lane < 16 * RT) dma16((const uint8_t *)(a.d + g * 8), sc_off, act + R::oD);
        if (Q4 && lane < 16 * RT) dma16((const uint8_t *)(a.bsum32 + g * 8), sc_off, act + R::oBs);
    }
    for (int64_t t0 = blockIdx.x; t0 < tiles; t0 += kTilesPerRound * G) {
        int cnt = (int)((tiles - t0 + G - 1) / G);
        cnt = cnt < kTilesPerRound ? cnt : kTilesPerRound;
        if (has) {
            v4f o0 = {0.0f, 0.0f, 0.0f, 0.0f}, o1 = o0, o2 = o0, o3 = o0;
            blk32_multi_issue<DT, RT>(ring, w, t0 * 16, g, row_off, q4_off, ws_off, lane);
            if (M::kSlots == 2 && cnt > 1) blk32_multi_issue<DT, RT>(ring + M::kSlot, w, (t0 + G) * 16, g, row_off, q4_off, ws_off, lane);
#pragma nounroll
            for (int i = 0; i < cnt; i++) {
                // everything but the copies of a tile in flight ahead has landed
                if (M::kSlots == 2 && i + 1 < cnt) __builtin_amdgcn_s_waitcnt(kAhead);
                else __builtin_amdgcn_s_waitcnt(0x0F70);
                const int64_t tile = t0 + i * G;
                v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
                blk32_multi_step<DT, RT, DUMP>(ring + (M::kSlots == 2 ? (i & 1) * M::kSlot : 0), act, lane, w, i + M::kSlots < cnt,
                                               tile + M::kSlots * G, g, row_off, q4_off, ws_off, w4_col, w4_shift, w_col, a_col, acc, dump,
                                               (tile * 16 + r) * kb + g * 8, w.n * kb, m);
                if (i == 0) { o0 = acc; asm volatile(""); }
                else if (i == 1) { o1 = acc; asm volatile(""); }
                else if (i == 2) { o2 = acc; asm volatile(""); }
                else { o3 = acc; asm volatile(""); }
            }
            *(v4f *)(ring + lane * 16) = o0;
            *(v4f *)(ring + 1024 + lane * 16) = o1;
            *(v4f *)(ring + 2048 + lane * 16) = o2;
            *(v4f *)(ring + 3072 + lane * 16) = o3;
        }
        __syncthreads();
        if (wave < cnt && !DUMP) {   // wave i sums tile i of the round, in wave order
            v4f s = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
            const int64_t nw = kg < kWaves ? kg : kWaves;   // waves that own a group
            for (int64_t o = 0; o < nw; o++) {
                const v4f p = *(const v4f *)(wgt_base + (size_t)o * M::kSlots * M::kSlot + wave * 1024 + lane * 16);
                s += p;
            }
            const int64_t col = (t0 + wave * G) * 16 + r;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int64_t row = kq * 4 + i;
                if (row < m) y[row * w.n + col] = s[i];
            }
        }
        if (t0 + kTilesPerRound * G < tiles) __syncthreads();   // the sums have been read: the slots take the next round's copies
    }
}

template <int DT, int RT, int NW, bool DUMP>
hipError_t launch_blk32_multi_inst(const cq_weight *w, cq_act_view a, int64_t m, float *y, size_t lds, unsigned grid, cq_mfma_dump d,
                                   hipStream_t s) {
    if (hipError_t e = cq_ensure_lds<skinny_blk32_multi_kernel<DT, RT, NW, DUMP>>(w->dev, lds); e != hipSuccess) return e;
    CQ_LAUNCH((skinny_blk32_multi_kernel<DT, RT, NW, DUMP>), grid, NW * 64, lds, s, *w, a, m, y, d);
    return hipGetLastError();
}

template <int DT, int RT, int NW, bool DUMP>
hipError_t launch_blk32_res_inst(const cq_weight *w, cq_act_view a, int64_t m, float *y, size_t lds, cq_mfma_dump d, hipStream_t s) {
    if (hipError_t e = cq_ensure_lds<skinny_blk32_resident_kernel<DT, RT, NW, DUMP>>(w->dev, lds); e != hipSuccess) return e;
    CQ_LAUNCH((skinny_blk32_resident_kernel<DT, RT, NW, DUMP>), (unsigned)(w->n / 16), NW * 64, lds, s, *w, a, m, y, d);
    return hipGetLastError();
}
// Takes the launch (true) where the resident kernel applies: one tile per workgroup, all operands in the LDS.
template <int DT, int RT, bool DUMP>
bool launch_blk32_res_rt(const cq_weight *w, cq_act_view a, int64_t m, float *y, cq_mfma_dump d, hipStream_t s, hipError_t *err) {
    const int64_t kg = w->k >> 8, tiles = w->n / 16;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (cus <= 0) cus = 256;
    const bool sixteen = kg > 8;
    if (tiles > cus) {
        // several tiles per workgroup: rounds of tiles with one meeting each, where a wave has one K group
        if constexpr (RT <= 2) {
            const size_t lm = ResQ8Multi<DT, RT>::bytes(kg);
            if (sixteen && kg <= 16 && lm <= (size_t)kMaxLds && (uint64_t)w->n * (uint64_t)w->k < (1ull << 32)) {
                *err = launch_blk32_multi_inst<DT, RT, 16, DUMP>(w, a, m, y, lm, (unsigned)cus, d, s);
                return true;
            }
        }
        return false;
    }
    if (kg > (sixteen ? 16 : 8) * kMaxBpw) return false;
    const size_t lds = ResQ8<DT, RT>::bytes(kg);
    if (lds > (size_t)kMaxLds) return false;
    *err = sixteen ? launch_blk32_res_inst<DT, RT, 16, DUMP>(w, a, m, y, lds, d, s) : launch_blk32_res_inst<DT, RT, 8, DUMP>(w, a, m, y, lds, d, s);
    return true;
}
template <int DT, bool DUMP>
bool launch_blk32_res(const cq_weight *w, cq_act_view a, int64_t m, float *y, cq_mfma_dump d, hipStream_t s, hipError_t *err) {
    if (m <= 8) return launch_blk32_res_rt<DT, 1, DUMP>(w, a, m, y, d, s, err);
    if (m <= 16) return launch_blk32_res_rt<DT, 2, DUMP>(w, a, m, y, d, s, err);
    if (m <= 24) return launch_blk32_res_rt<DT, 3, DUMP>(w, a, m, y, d, s, err);
    if (m <= 32) return launch_blk32_res_rt<DT, 4, DUMP>(w, a, m, y, d, s, err);
    return false;
}

// DUMP (all launchers below): the launch cq_launch_skinny would make, storing the block integers through `d`.
template <int DT, int RT, bool DUMP>
hipError_t launch_blk32_rt(const cq_weight *w, cq_act_view a, int64_t m0, int64_t m, float *y, cq_mfma_dump d, hipStream_t s) {
    const size_t lds = (size_t)BufQ8<RT>::kBytes * kWaves;
    if (hipError_t e = cq_ensure_lds<skinny_blk32_kernel<DT, RT, DUMP>>(w->dev, lds); e != hipSuccess) return e;
    CQ_LAUNCH((skinny_blk32_kernel<DT, RT, DUMP>), (unsigned)(w->n / 16), kThreads, lds, s, *w, a, m0, m, y, d);
    return hipGetLastError();
}

template <int DT, bool DUMP>
hipError_t launch_blk32(const cq_weight *w, cq_act_view a, int64_t m, float *y, cq_mfma_dump d, hipStream_t s) {
    for (int64_t m0 = 0; m0 < m; m0 += 32) {
        const int64_t left = m - m0;
        hipError_t e;
        if (left <= 8) e = launch_blk32_rt<DT, 1, DUMP>(w, a, m0, m, y, d, s);
        else if (left <= 16) e = launch_blk32_rt<DT, 2, DUMP>(w, a, m0, m, y, d, s);
        else if (left <= 24) e = launch_blk32_rt<DT, 3, DUMP>(w, a, m0, m, y, d, s);
        else e = launch_blk32_rt<DT, 4, DUMP>(w, a, m0, m, y, d, s);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <int DT, int RT, bool DUMP>
hipError_t launch_rt(const cq_weight *w, cq_act_view a, int64_t m0, int64_t m, float *y, cq_mfma_dump d, hipStream_t s) {
    const size_t lds = (size_t)Buf<DT, RT>::kBytes * kWaves;
    if (hipError_t e = cq_ensure_lds<skinny_kernel<DT, RT, DUMP>>(w->dev, lds); e != hipSuccess) return e;
    CQ_LAUNCH((skinny_kernel<DT, RT, DUMP>), (unsigned)(w->n / 16), kThreads, lds, s, *w, a, m0, m, y, d);
    return hipGetLastError();
}

template <int DT, bool DUMP>
hipError_t launch_dt(const cq_weight *w, cq_act_view a, int64_t m, float *y, cq_mfma_dump d, hipStream_t s) {
    for (int64_t m0 = 0; m0 < m; m0 += 32) {
        const int64_t left = m - m0;
        hipError_t e;
        if (left <= 8) e = launch_rt<DT, 1, DUMP>(w, a, m0, m, y, d, s);
        else if (left <= 16) e = launch_rt<DT, 2, DUMP>(w, a, m0, m, y, d, s);
        else if (left <= 24) e = launch_rt<DT, 3, DUMP>(w, a, m0, m, y, d, s);
        else e = launch_rt<DT, 4, DUMP>(w, a, m0, m, y, d, s);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}


// The resident-activation kernel where the call's activations and the weight buffers fit the LDS (see above).
template <int DT, int RT, int NW, int NBUF, bool DUMP>
hipError_t launch_res_inst(const cq_weight *w, cq_act_view a, int64_t m, float *y, size_t lds, unsigned grid, cq_mfma_dump d,
                           hipStream_t s) {
    if (hipError_t e = cq_ensure_lds<skinny_resident_kernel<DT, RT, NW, NBUF, DUMP>>(w->dev, lds); e != hipSuccess) return e;
    CQ_LAUNCH((skinny_resident_kernel<DT, RT, NW, NBUF, DUMP>), grid, NW * 64, lds, s, *w, a, m, y, d);
    return hipGetLastError();
}
template <int DT, int RT, int NW, bool DUMP>
hipError_t launch_multi_inst(const cq_weight *w, cq_act_view a, int64_t m, float *y, size_t lds, unsigned grid, cq_mfma_dump d,
                             hipStream_t s) {
    if (hipError_t e = cq_ensure_lds<skinny_resident_multi_kernel<DT, RT, NW, DUMP>>(w->dev, lds); e != hipSuccess) return e;
    CQ_LAUNCH((skinny_resident_multi_kernel<DT, RT, NW, DUMP>), grid, NW * 64, lds, s, *w, a, m, y, d);
    return hipGetLastError();
}
template <int DT, int RT, bool DUMP>
bool launch_res_rt(const cq_weight *w, cq_act_view a, int64_t m, float *y, cq_mfma_dump d, hipStream_t s, hipError_t *err) {
    const int64_t kb = w->k >> 8, tiles = w->n / 16;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (cus <= 0) cus = 256;
    const unsigned grid = (unsigned)(tiles < cus ? tiles : cus);
    const bool sixteen = kb > 8;
    if (kb > (sixteen ? 16 : 8) * kMaxBpw) return false;
    // the copies address every plane with 32-bit byte offsets
    if ((uint64_t)w->n * (uint64_t)kb * 128u >= (1ull << 32) || (uint64_t)a.m_stride * (uint64_t)w->k >= (1ull << 32)) return false;
    // Measured (Q4K, 16 rows, matmul kernel alone): 4096 x 4096, one tile per workgroup, 5.95 us against 6.5 us for the
    // kernel that copies activations per block; 11008 x 4096, two or three tiles per workgroup, 12.7 against 12.5 us
    // (also with the next tile's weights copied ahead into a second buffer): taken where every workgroup has one tile.
    if (tiles > grid) {
        // several tiles per workgroup: the kernel that meets once per round of tiles, where a wave has one K block
        if constexpr (RT <= 2 && (DT == CQ_DTYPE_Q4K || DT == CQ_DTYPE_Q5K)) {
            const size_t two = ResMulti<DT, RT>::bytes(kb);
            // Measured (Q4K, whole calls in us, the kernel that copies activations per block -> this one): 16 rows 11008 x 4096
            // 13.6 -> 12.6, 14336 x 4096 15.9 -> 14.3, 32000 x 4096 28.3 -> 24.1; 8 rows 11.7 -> 12.2, 14.1 -> 13.6, 24.1 -> 23.6:
            // with up to 8 rows five of the other kernel's workgroups share a CU and hide each other's waits.
            // K = 2048 (eight waves): 16 rows 8192 x 2048 10.0 -> 10.2; left with the other kernel.
            const bool pays = RT == 2 || tiles > 3 * (int64_t)cus;
            if (pays && sixteen && kb <= 16 && two <= (size_t)kMaxLds) {
                *err = launch_multi_inst<DT, RT, 16, DUMP>(w, a, m, y, two, grid, d, s);
                return true;
            }
        }
        return false;
    }
    const size_t one = Res<DT, RT>::bytes(kb, 1);
    if (one <= (size_t)kMaxLds) {
        *err = sixteen ? launch_res_inst<DT, RT, 16, 1, DUMP>(w, a, m, y, one, grid, d, s)
                       : launch_res_inst<DT, RT, 8, 1, DUMP>(w, a, m, y, one, grid, d, s);
        return true;
    }
    return false;
}
template <int DT, bool DUMP>
bool launch_res(const cq_weight *w, cq_act_view a, int64_t m, float *y, cq_mfma_dump d, hipStream_t s, hipError_t *err) {
    if (m <= 8) return launch_res_rt<DT, 1, DUMP>(w, a, m, y, d, s, err);
    if (m <= 16) return launch_res_rt<DT, 2, DUMP>(w, a, m, y, d, s, err);
    if (m <= 24) return launch_res_rt<DT, 3, DUMP>(w, a, m, y, d, s, err);
    if (m <= 32) return launch_res_rt<DT, 4, DUMP>(w, a, m, y, d, s, err);
    return false;
}

template <bool DUMP>
hipError_t launch_any(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, cq_mfma_dump d, hipStream_t s) {
    if (!cq_skinny_supported(w, act_dtype)) return hipErrorNotSupported;
    if (m == 0) return hipSuccess;
    if (a.m_stride < (m + 31) / 32 * 32) return hipErrorInvalidValue;   // whole 8-row groups are copied
    hipError_t e = hipSuccess;
    if (w->dtype == CQ_DTYPE_Q8_0 && launch_blk32_res<CQ_DTYPE_Q8_0, DUMP>(w, a, m, y, d, s, &e)) return e;
    if (w->dtype == CQ_DTYPE_Q4_0 && launch_blk32_res<CQ_DTYPE_Q4_0, DUMP>(w, a, m, y, d, s, &e)) return e;
    if (w->dtype == CQ_DTYPE_Q8_0) return launch_blk32<CQ_DTYPE_Q8_0, DUMP>(w, a, m, y, d, s);
    if (w->dtype == CQ_DTYPE_Q4_0) return launch_blk32<CQ_DTYPE_Q4_0, DUMP>(w, a, m, y, d, s);
    if (w->dtype == CQ_DTYPE_Q4K && launch_res<CQ_DTYPE_Q4K, DUMP>(w, a, m, y, d, s, &e)) return e;
    if (w->dtype == CQ_DTYPE_Q5K && launch_res<CQ_DTYPE_Q5K, DUMP>(w, a, m, y, d, s, &e)) return e;
    if (w->dtype == CQ_DTYPE_Q6K && launch_res<CQ_DTYPE_Q6K, DUMP>(w, a, m, y, d, s, &e)) return e;
    if (w->dtype == CQ_DTYPE_Q4K) return launch_dt<CQ_DTYPE_Q4K, DUMP>(w, a, m, y, d, s);
    if (w->dtype == CQ_DTYPE_Q5K) return launch_dt<CQ_DTYPE_Q5K, DUMP>(w, a, m, y, d, s);
    return launch_dt<CQ_DTYPE_Q6K, DUMP>(w, a, m, y, d, s);
}

}  // namespace

bool cq_skinny_supported(const cq_weight *w, int act_dtype) {
    // the copies address 8 rows of activations and 16 rows of a weight plane with 32-bit offsets
    const bool kquant = (w->dtype == CQ_DTYPE_Q4K || w->dtype == CQ_DTYPE_Q5K || w->dtype == CQ_DTYPE_Q6K) && act_dtype == CQ_DTYPE_Q8K;
    const bool q8 = (w->dtype == CQ_DTYPE_Q8_0 || w->dtype == CQ_DTYPE_Q4_0) && act_dtype == CQ_DTYPE_Q8_0 && w->k % 256 == 0;
    return (kquant || q8) && w->k >= 256 && w->k <= (1 << 24) && w->n % 16 == 0 && w->n > 0;
}

hipError_t cq_launch_skinny(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, hipStream_t s) {
    return launch_any<false>(w, a, act_dtype, m, y, cq_mfma_dump{nullptr, nullptr, 0}, s);
}

hipError_t cq_launch_skinny_dump(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, cq_mfma_dump d, hipStream_t s) {
    return launch_any<true>(w, a, act_dtype, m, nullptr, d, s);
}
