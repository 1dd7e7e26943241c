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
