// GGML array-of-blocks <-> device planes (and back).  Pure byte permutations:
// cq_launch_unpack(cq_launch_repack(x)) == x for every input.
//
// Replaces the plain host->device copy of cuda::load_quantized
// (candle-core/src/quantized/cuda.rs:591-612); the inverse serves QStorage::data
// (mod.rs:118-130).
#include "qhip_internal.h"

namespace {

// ---- Q4_0: 18-byte blocks {f16 d; u8 qs[16]} --------------------------------
__global__ void repack_q4_0(const uint8_t *__restrict__ aos, uint8_t *__restrict__ qs, uint16_t *__restrict__ d,
                            int64_t nblocks, bool inverse) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    uint16_t *a16 = (uint16_t *)(aos + b * 18);   // 18*b is even
    uint16_t *q16 = (uint16_t *)(qs + b * 16);
    if (!inverse) {
        d[b] = a16[0];
        for (int i = 0; i < 8; i++) q16[i] = a16[1 + i];
    } else {
        a16[0] = d[b];
        for (int i = 0; i < 8; i++) a16[1 + i] = q16[i];
    }
}

// ---- Q8_0: 34-byte blocks {f16 d; i8 qs[32]} --------------------------------
__global__ void repack_q8_0(const uint8_t *__restrict__ aos, uint8_t *__restrict__ qs, uint16_t *__restrict__ d,
                            int64_t nblocks, bool inverse) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    uint16_t *a16 = (uint16_t *)(aos + b * 34);
    uint16_t *q16 = (uint16_t *)(qs + b * 32);
    if (!inverse) {
        d[b] = a16[0];
        for (int i = 0; i < 16; i++) q16[i] = a16[1 + i];
    } else {
        a16[0] = d[b];
        for (int i = 0; i < 16; i++) a16[1 + i] = q16[i];
    }
}

// The 16 header bytes {f16 d; f16 dmin; u8 scales[12]} of a Q4K / Q5K block <-> the 20-byte device
// record: the twelve bytes of 6-bit fields (utils.rs:49-59 get_scale_min_k4) unpacked to one byte
// per field and grouped per 32 qs bytes, record g = {sc[2g], sc[2g+1], mn[2g], mn[2g+1]}; the
// inverse packs them back (every one of the 96 bits is a field bit, so the round trip is exact).
__device__ void k4_header(uint4 *a, uint32_t *h, bool inverse) {
    if (!inverse) {
        const uint4 v = *a;
        h[0] = v.x;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            int s0, m0, s1, m1;
            cq_scale_min_k4(2 * g, v.y, v.z, v.w, s0, m0);
            cq_scale_min_k4(2 * g + 1, v.y, v.z, v.w, s1, m1);
            h[1 + g] = (uint32_t)s0 | ((uint32_t)s1 << 8) | ((uint32_t)m0 << 16) | ((uint32_t)m1 << 24);
        }
    } else {
        uint32_t sc[8], mn[8];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t r = h[1 + g];
            sc[2 * g] = r & 0xff; sc[2 * g + 1] = (r >> 8) & 0xff;
            mn[2 * g] = (r >> 16) & 0xff; mn[2 * g + 1] = r >> 24;
        }
        uint32_t w[3] = {0, 0, 0};   // scales[0..3], scales[4..7], scales[8..11]
#pragma unroll
        for (int j = 0; j < 4; j++) {
            w[0] |= ((sc[j] & 63) | ((sc[j + 4] >> 4) << 6)) << (8 * j);
            w[1] |= ((mn[j] & 63) | ((mn[j + 4] >> 4) << 6)) << (8 * j);
            w[2] |= ((sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)) << (8 * j);
        }
        *a = make_uint4(h[0], w[0], w[1], w[2]);
    }
}

// ---- Q4K: 144-byte blocks {f16 d; f16 dmin; u8 scales[12]; u8 qs[128]} ------
// One thread per 16-byte unit: unit 0 is the header, units 1..8 the nibbles.
__global__ void repack_q4k(const uint8_t *__restrict__ aos, uint8_t *__restrict__ qs, uint8_t *__restrict__ hd,
                           int64_t nblocks, bool inverse) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t b = t / 9;
    int u = (int)(t - b * 9);
    if (b >= nblocks) return;
    uint4 *a = (uint4 *)(aos + b * 144) + u;      // 144 = 9 * 16, base is 256-byte aligned
    if (u != 0) {
        uint4 *p = (uint4 *)(qs + b * 128) + (u - 1);
        if (!inverse) *p = *a; else *a = *p;
        return;
    }
    k4_header(a, (uint32_t *)(hd + b * CQ_Q4K_HDR), inverse);
}

// ---- Q5K: 176-byte blocks {f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]} ------
// (k_quants.rs:119-127).  Header and nibbles as Q4K.  Bit j of qh[l] is the fifth bit of element
// l of sub-block j, i.e. of the low (j even) or high (j odd) nibble of qs byte 32*(j/2) + l.  The
// device plane holds, per 32 qs bytes g, two words L (sub-block 2g) and H (sub-block 2g+1) with
//   bit 8c + i  =  fifth bit belonging to byte c of qs word i  (l = 4i + c),
// so that (W >> i) & 0x01010101 lines the four bits up with the four nibbles of word i.
// One thread per 16-byte unit of the block: 0 header, 1 the whole qh (32 bytes), 2 idle, 3..10 qs.
__global__ void repack_q5k(const uint8_t *__restrict__ aos, uint8_t *__restrict__ qs, uint8_t *__restrict__ hd,
                           uint8_t *__restrict__ qh, int64_t nblocks, bool inverse) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t b = t / 11;
    int u = (int)(t - b * 11);
    if (b >= nblocks) return;
    uint4 *a = (uint4 *)(aos + b * 176) + u;      // 176 = 11 * 16, base is 256-byte aligned
    if (u >= 3) {
        uint4 *p = (uint4 *)(qs + b * 128) + (u - 3);
        if (!inverse) *p = *a; else *a = *p;
        return;
    }
    if (u == 2) return;
    if (u == 1) {
        uint8_t *src = (uint8_t *)aos + b * 176 + 16;   // GGML qh[32]
        uint32_t *dst = (uint32_t *)(qh + b * 32);      // {L, H} x 4
        if (!inverse) {
            for (int g = 0; g < 4; g++) {
                uint32_t L = 0, H = 0;
                for (int i = 0; i < 8; i++)
                    for (int c = 0; c < 4; c++) {
                        const uint32_t v = src[4 * i + c];
                        L |= ((v >> (2 * g)) & 1u) << (8 * c + i);
                        H |= ((v >> (2 * g + 1)) & 1u) << (8 * c + i);
                    }
                dst[2 * g] = L;
                dst[2 * g + 1] = H;
            }
        } else {
            for (int i = 0; i < 8; i++)
                for (int c = 0; c < 4; c++) {
                    uint32_t v = 0;
                    for (int g = 0; g < 4; g++) {
                        v |= ((dst[2 * g] >> (8 * c + i)) & 1u) << (2 * g);
                        v |= ((dst[2 * g + 1] >> (8 * c + i)) & 1u) << (2 * g + 1);
                    }
                    src[4 * i + c] = (uint8_t)v;
                }
        }
        return;
    }
    k4_header(a, (uint32_t *)(hd + b * CQ_Q4K_HDR), inverse);
}

// ---- Q6K: 210-byte blocks {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d} -----
// qh is re-ordered so that the thread that owns ql bytes [16u, 16u+16) of a block
// finds the high bits of exactly those 32 elements in qh' bytes [8u, 8u+8):
//   u = 4h + 2t + i  ->  ql byte 64h + 32t + 16i + e  (e < 16)
//   low  nibble: element 128h + 32t + 16i + e        hi bits = qh[32h + 16i + e] >> 2t
//   high nibble: element 128h + 64 + 32t + 16i + e   hi bits = qh[32h + 16i + e] >> (2t + 4)
//   qh'[8u + 4x + c] (x < 2, c < 4) =   lo2(8x + c)       | hi2(8x + c) << 2
//                                      | lo2(8x + 4 + c) << 4 | hi2(8x + 4 + c) << 6
//   sc'[2u], sc'[2u + 1] = scales[js], scales[js + 4] with js = u + 4h: the scales of the lane's
//   low-nibble and high-nibble 16-element groups, one 2-byte load per lane.
// i.e. for the two ql words 2x and 2x+1 of the lane, (H >> {0,2,4,6}) & 0x03030303 lines the
// two high bits up with each byte of {word 2x low, word 2x high, word 2x+1 low, word 2x+1 high}.
__global__ void repack_q6k(const uint8_t *__restrict__ aos, uint8_t *__restrict__ ql, uint8_t *__restrict__ qh,
                           uint8_t *__restrict__ sc, uint16_t *__restrict__ d, int64_t nblocks, bool inverse) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t b = t / 8;
    int u = (int)(t & 7);
    if (b >= nblocks) return;
    uint8_t *a = (uint8_t *)aos + b * 210;
    uint8_t *a_ql = a, *a_qh = a + 128, *a_sc = a + 192, *a_d = a + 208;
    const int h = u >> 2, tt = (u >> 1) & 1, i0 = (u & 1) * 16;
    uint8_t *pql = ql + b * 128 + 16 * u;
    uint8_t *pqh = qh + b * 64 + 8 * u;
    if (!inverse) {
        for (int e = 0; e < 16; e++) pql[e] = a_ql[16 * u + e];
        for (int x = 0; x < 2; x++)
            for (int c = 0; c < 4; c++) {
                uint8_t s0 = a_qh[32 * h + i0 + 8 * x + c];
                uint8_t s1 = a_qh[32 * h + i0 + 8 * x + 4 + c];
                uint8_t v = (uint8_t)(((s0 >> (2 * tt)) & 3) | (((s0 >> (2 * tt + 4)) & 3) << 2) |
                                      (((s1 >> (2 * tt)) & 3) << 4) | (((s1 >> (2 * tt + 4)) & 3) << 6));
                pqh[4 * x + c] = v;
            }
        // the lane's two 16-element scale groups (low nibbles: js, high nibbles: js + 4) side by side
        const int js = u + 4 * h;
        sc[b * 16 + 2 * u] = a_sc[js];
        sc[b * 16 + 2 * u + 1] = a_sc[js + 4];
        if (u == 0) d[b] = (uint16_t)(a_d[0] | (a_d[1] << 8));
    } else {
        for (int e = 0; e < 16; e++) a_ql[16 * u + e] = pql[e];
        const int js = u + 4 * h;
        a_sc[js] = sc[b * 16 + 2 * u];
        a_sc[js + 4] = sc[b * 16 + 2 * u + 1];
        if (u == 0) {
            a_d[0] = (uint8_t)(d[b] & 0xff);
            a_d[1] = (uint8_t)(d[b] >> 8);
        }
        // Each GGML qh byte 32h + j collects 2-bit fields from the two lanes t = 0, 1 that share
        // (h, i); lane (h, t = 0, i) rebuilds the 16 bytes 32h + 16i + e from both lanes' qh'.
        if (tt == 0) {
            const uint8_t *p0 = qh + b * 64 + 8 * u;        // t = 0
            const uint8_t *p1 = qh + b * 64 + 8 * (u + 2);  // t = 1
            for (int x = 0; x < 2; x++)
                for (int c = 0; c < 4; c++) {
                    uint8_t v0 = p0[4 * x + c], v1 = p1[4 * x + c];
                    // element e = 8x + c : fields lo2 (bits 0-1) and hi2 (bits 2-3)
                    a_qh[32 * h + i0 + 8 * x + c] =
                        (uint8_t)((v0 & 3) | ((v1 & 3) << 2) | (((v0 >> 2) & 3) << 4) | (((v1 >> 2) & 3) << 6));
                    // element e = 8x + 4 + c : fields at bits 4-5 and 6-7
                    a_qh[32 * h + i0 + 8 * x + 4 + c] = (uint8_t)(((v0 >> 4) & 3) | (((v1 >> 4) & 3) << 2) |
                                                                  (((v0 >> 6) & 3) << 4) | (((v1 >> 6) & 3) << 6));
                }
        }
    }
}

// ---- types held in another type's planes --------------------------------------------------------
// Q5_0 {f16 d; u8 qh[4]; u8 qs[16]} (k_quants.rs:61-67) holds d and 32 five-bit quants q, value d * (q - 16): exactly a
// Q8_0 block {f16 d; i8 qs[32]} with qs = q - 16, whose dequantization (k_quants.rs:568-584) and dot product with Q8_0
// activations (:631-649) are the arithmetic of Q5_0's (:428-451, :371-391) operation for operation.
__global__ void transcode_q5_0_q8_0(uint8_t *__restrict__ q5, uint8_t *__restrict__ q8, int64_t nblocks, bool inverse) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    uint8_t *x = q5 + b * 22, *y = q8 + b * 34;
    if (!inverse) {
        y[0] = x[0];
        y[1] = x[1];
        const uint32_t qh = (uint32_t)x[2] | ((uint32_t)x[3] << 8) | ((uint32_t)x[4] << 16) | ((uint32_t)x[5] << 24);
        for (int j = 0; j < 16; j++) {
            const int x0 = (int)((x[6 + j] & 0x0F) | (((qh >> j) & 1u) << 4)) - 16;
            const int x1 = (int)((x[6 + j] >> 4) | (((qh >> (j + 16)) & 1u) << 4)) - 16;
            y[2 + j] = (uint8_t)(int8_t)x0;
            y[2 + j + 16] = (uint8_t)(int8_t)x1;
        }
    } else {
        x[0] = y[0];
        x[1] = y[1];
        uint32_t qh = 0;
        for (int j = 0; j < 16; j++) {
            const uint32_t v0 = (uint32_t)((int)(int8_t)y[2 + j] + 16) & 31u, v1 = (uint32_t)((int)(int8_t)y[2 + j + 16] + 16) & 31u;
            x[6 + j] = (uint8_t)((v0 & 0x0F) | ((v1 & 0x0F) << 4));
            qh |= (v0 >> 4) << j;
            qh |= (v1 >> 4) << (j + 16);
        }
        x[2] = (uint8_t)qh; x[3] = (uint8_t)(qh >> 8); x[4] = (uint8_t)(qh >> 16); x[5] = (uint8_t)(qh >> 24);
    }
}

// Q4_1 {f16 d; f16 m; u8 qs[16]} and Q5_1 {f16 d; f16 m; u8 qh[4]; u8 qs[16]} (k_quants.rs:51-57, :69-76): value d * q + m.
// The quants (0..15, 0..31) and d go into a Q8_0 block, m into its own plane.
template <bool FIVE>
__global__ void transcode_q4_1_q8_0(uint8_t *__restrict__ src, uint8_t *__restrict__ q8, uint16_t *__restrict__ mins,
                                    int64_t nblocks, bool inverse) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    constexpr int TS = FIVE ? 24 : 20, QS = FIVE ? 8 : 4;
    uint8_t *x = src + b * TS, *y = q8 + b * 34;
    if (!inverse) {
        y[0] = x[0];
        y[1] = x[1];
        mins[b] = (uint16_t)(x[2] | (x[3] << 8));
        const uint32_t qh = FIVE ? ((uint32_t)x[4] | ((uint32_t)x[5] << 8) | ((uint32_t)x[6] << 16) | ((uint32_t)x[7] << 24)) : 0u;
        for (int j = 0; j < 16; j++) {
            y[2 + j] = (uint8_t)((x[QS + j] & 0x0F) | (((qh >> j) & 1u) << 4));
            y[2 + j + 16] = (uint8_t)((x[QS + j] >> 4) | (((qh >> (j + 16)) & 1u) << 4));
        }
    } else {
        x[0] = y[0];
        x[1] = y[1];
        x[2] = (uint8_t)(mins[b] & 0xff);
        x[3] = (uint8_t)(mins[b] >> 8);
        uint32_t qh = 0;
        for (int j = 0; j < 16; j++) {
            const uint32_t v0 = y[2 + j], v1 = y[2 + j + 16];
            x[QS + j] = (uint8_t)((v0 & 0x0F) | ((v1 & 0x0F) << 4));
            qh |= ((v0 >> 4) & 1u) << j;
            qh |= ((v1 >> 4) & 1u) << (j + 16);
        }
        if (FIVE) { x[4] = (uint8_t)qh; x[5] = (uint8_t)(qh >> 8); x[6] = (uint8_t)(qh >> 16); x[7] = (uint8_t)(qh >> 24); }
    }
}

// Q3K {u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d} (k_quants.rs:107-114): sixteen groups of sixteen three-bit quants,
// value (d * (sc_j - 32)) * (q - 4) with six-bit sc_j: exactly a Q6K block {ql, qh, i8 scales[16], f16 d} with
// scales[j] = sc_j - 32 and six-bit quants q + 28 (so that q6 - 32 = q - 4), whose dequantization (k_quants.rs:1716-1746)
// and dot product with Q8K activations (:1585-1641) are those of Q3K (:1094-1146, :890-1009): the same integers, the
// same products in the same order.
__device__ __forceinline__ int q3k_scale6(const uint8_t *sc, int j) {
    const int low = j < 8 ? (sc[j] & 0xF) : (sc[j - 8] >> 4);
    return low | (((sc[8 + j % 4] >> (2 * (j / 4))) & 3) << 4);
}
__global__ void transcode_q3k_q6k(uint8_t *__restrict__ q3, uint8_t *__restrict__ q6, int64_t nblocks, bool inverse) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    uint8_t *x = q3 + b * 110, *y = q6 + b * 210;
    uint8_t *hmask = x, *qs = x + 32, *sc3 = x + 96;
    uint8_t *ql = y, *qh = y + 128, *sc6 = y + 192;
    if (!inverse) {
        for (int i = 0; i < 192; i++) y[i] = 0;
        for (int e = 0; e < 256; e++) {
            const int half = e / 128, r = e % 128, quad = r / 32, l = r % 32;
            const int low = (qs[32 * half + l] >> (2 * quad)) & 3;
            const int v = low + 4 * ((hmask[e % 32] >> (e / 32)) & 1) + 28;   // (q - 4) + 32
            ql[64 * half + 32 * (quad & 1) + l] |= (uint8_t)((v & 0xF) << (4 * (quad >> 1)));
            qh[32 * half + l] |= (uint8_t)((v >> 4) << (2 * quad));
        }
        for (int j = 0; j < 16; j++) sc6[j] = (uint8_t)(int8_t)(q3k_scale6(sc3, j) - 32);
        y[208] = x[108];
        y[209] = x[109];
    } else {
        for (int i = 0; i < 108; i++) x[i] = 0;
        for (int e = 0; e < 256; e++) {
            const int half = e / 128, r = e % 128, quad = r / 32, l = r % 32;
            const int v6 = ((ql[64 * half + 32 * (quad & 1) + l] >> (4 * (quad >> 1))) & 0xF) | (((qh[32 * half + l] >> (2 * quad)) & 3) << 4);
            const int v = v6 - 28;   // 0..7
            qs[32 * half + l] |= (uint8_t)((v & 3) << (2 * quad));
            hmask[e % 32] |= (uint8_t)((v >> 2) << (e / 32));
        }
        for (int j = 0; j < 16; j++) {
            const int lv = (int)(int8_t)sc6[j] + 32;
            if (j < 8) sc3[j] |= (uint8_t)(lv & 0xF);
            else sc3[j - 8] |= (uint8_t)((lv & 0xF) << 4);
            sc3[8 + j % 4] |= (uint8_t)((lv >> 4) << (2 * (j / 4)));
        }
        x[108] = y[208];
        x[109] = y[209];
    }
}

// Q2K {u8 scales[16]; u8 qs[64]; f16 d; f16 dmin} (k_quants.rs:96-103): value (d * sc_j) * q - dmin * m_j, sc_j and m_j
// the nibbles of scales[j].  The first term is a Q6K block with scales sc_j and quants q + 32; m_j and dmin go to
// planes of their own.
__global__ void transcode_q2k_q6k(uint8_t *__restrict__ q2, uint8_t *__restrict__ q6, uint8_t *__restrict__ mins,
                                  uint16_t *__restrict__ dmins, int64_t nblocks, bool inverse) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    uint8_t *x = q2 + b * 84, *y = q6 + b * 210;
    uint8_t *sc2 = x, *qs = x + 16;
    uint8_t *ql = y, *qh = y + 128, *sc6 = y + 192, *mb = mins + b * 16;
    if (!inverse) {
        for (int i = 0; i < 192; i++) y[i] = 0;
        for (int e = 0; e < 256; e++) {
            const int half = e / 128, r = e % 128, quad = r / 32, l = r % 32;
            const int v = ((qs[32 * half + l] >> (2 * quad)) & 3) + 32;
            ql[64 * half + 32 * (quad & 1) + l] |= (uint8_t)((v & 0xF) << (4 * (quad >> 1)));
            qh[32 * half + l] |= (uint8_t)((v >> 4) << (2 * quad));
        }
        for (int j = 0; j < 16; j++) {
            sc6[j] = (uint8_t)(sc2[j] & 0xF);
            mb[j] = (uint8_t)(sc2[j] >> 4);
        }
        y[208] = x[80];
        y[209] = x[81];
        dmins[b] = (uint16_t)(x[82] | (x[83] << 8));
    } else {
        for (int i = 16; i < 80; i++) x[i] = 0;
        for (int e = 0; e < 256; e++) {
            const int half = e / 128, r = e % 128, quad = r / 32, l = r % 32;
            const int v6 = ((ql[64 * half + 32 * (quad & 1) + l] >> (4 * (quad >> 1))) & 0xF) | (((qh[32 * half + l] >> (2 * quad)) & 3) << 4);
            qs[32 * half + l] |= (uint8_t)(((v6 - 32) & 3) << (2 * quad));
        }
        for (int j = 0; j < 16; j++) sc2[j] = (uint8_t)((sc6[j] & 0xF) | (mb[j] << 4));
        x[80] = y[208];
        x[81] = y[209];
        x[82] = (uint8_t)(dmins[b] & 0xff);
        x[83] = (uint8_t)(dmins[b] >> 8);
    }
}

hipError_t launch(const cq_weight *w, uint8_t *aos, bool inverse, hipStream_t s) {
    const int64_t bs = cq_block_size(w->dtype);
    const int64_t nblocks = w->n * (w->k / bs);
    if (nblocks == 0) return hipSuccess;
    const int threads = 256;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: {
        unsigned grid = (unsigned)((nblocks + threads - 1) / threads);
        repack_q4_0<<<grid, threads, 0, s>>>(aos, w->p0, (uint16_t *)w->p1, nblocks, inverse);
        break;
    }
    case CQ_DTYPE_Q8_0: {
        unsigned grid = (unsigned)((nblocks + threads - 1) / threads);
        repack_q8_0<<<grid, threads, 0, s>>>(aos, w->p0, (uint16_t *)w->p1, nblocks, inverse);
        break;
    }
    case CQ_DTYPE_Q4K: {
        unsigned grid = (unsigned)((nblocks * 9 + threads - 1) / threads);
        repack_q4k<<<grid, threads, 0, s>>>(aos, w->p0, w->p1, nblocks, inverse);
        break;
    }
    case CQ_DTYPE_Q5K: {
        unsigned grid = (unsigned)((nblocks * 11 + threads - 1) / threads);
        repack_q5k<<<grid, threads, 0, s>>>(aos, w->p0, w->p1, w->p2, nblocks, inverse);
        break;
    }
    case CQ_DTYPE_Q6K: {
        unsigned grid = (unsigned)((nblocks * 8 + threads - 1) / threads);
        repack_q6k<<<grid, threads, 0, s>>>(aos, w->p0, w->p1, w->p2, (uint16_t *)w->p3, nblocks, inverse);
        break;
    }
    case CQ_DTYPE_Q8K: return cq_launch_repack_q8k(w, aos, inverse, s);
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

hipError_t cq_launch_repack(const cq_weight *w, const uint8_t *aos_dev, hipStream_t s) {
    return launch(w, (uint8_t *)aos_dev, false, s);
}
hipError_t cq_launch_unpack(const cq_weight *w, uint8_t *aos_dev, hipStream_t s) {
    return launch(w, aos_dev, true, s);
}

// GGML blocks of type `ggml_dtype` <-> GGML blocks of the type whose planes hold them (cq_storage_dtype).
hipError_t cq_launch_transcode(const cq_weight *w, uint8_t *ggml_aos_dev, uint8_t *storage_aos_dev, int64_t nblocks, bool inverse,
                               hipStream_t s) {
    const int ggml_dtype = w->ggml_dtype;
    uint16_t *min_plane = (uint16_t *)w->p2;
    if (nblocks == 0) return hipSuccess;
    const int threads = 128;
    const unsigned grid = (unsigned)((nblocks + threads - 1) / threads);
    switch (ggml_dtype) {
    case CQ_DTYPE_Q5_0: transcode_q5_0_q8_0<<<grid, threads, 0, s>>>(ggml_aos_dev, storage_aos_dev, nblocks, inverse); break;
    case CQ_DTYPE_Q4_1: transcode_q4_1_q8_0<false><<<grid, threads, 0, s>>>(ggml_aos_dev, storage_aos_dev, min_plane, nblocks, inverse); break;
    case CQ_DTYPE_Q5_1: transcode_q4_1_q8_0<true><<<grid, threads, 0, s>>>(ggml_aos_dev, storage_aos_dev, min_plane, nblocks, inverse); break;
    case CQ_DTYPE_Q3K: transcode_q3k_q6k<<<grid, threads, 0, s>>>(ggml_aos_dev, storage_aos_dev, nblocks, inverse); break;
    case CQ_DTYPE_Q2K: transcode_q2k_q6k<<<grid, threads, 0, s>>>(ggml_aos_dev, storage_aos_dev, w->p4, (uint16_t *)w->p5, nblocks, inverse); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
