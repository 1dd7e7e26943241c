// The offset terms of weight types that are held in another type's planes.
//
// The m * s term of the Q4_1 / Q5_1 dot product with Q8_1 activations (k_quants.rs:267-294, :463-494):
//   y[r, c] += sum_b  h2f(m[c, b]) * h2f(s8[r, b]),   s8 = f16(h2f(f16(sum of the block's 32 quants)) * d8)
// (BlockQ8_1::from_float, k_quants.rs:665-691).  Those weights are held as Q8_0 planes (quants 0..15 / 0..31) plus the
// plane of minima; the Q8_0 kernels have already written sum_b sum_i * d * d8 into y, from activations quantized by the
// Q8_0 rule, which is the Q8_1 rule without the `s` field: the field is recomputed here from the workspace's block sums
// and scales.  The reference adds both terms block by block into one f32; here the two sums are formed separately and
// added, a difference of rounding only.
#include "qhip_internal.h"

namespace {

__device__ __forceinline__ float block_s(const cq_act_view &a, int64_t at) {
    const float hs = cq_h2f(cq_f2h((float)a.bsum32[at]));
    return cq_h2f(cq_f2h(hs * a.d[at]));
}

// Order of the f32 additions, the same in both kernels and for any number of rows (a row's result does not depend on the
// rows beside it): the blocks of a weight row in chunks of eight, a chunk's products added one after the other from
// zero, the chunk sums added one after the other.
constexpr int kChunk = 8;

// Many rows: a workgroup forms a 32 x 32 tile of outputs, thread (i, j) the 2 x 2 outputs (i, i+16) x (j, j+16); the
// minima and the s values of 32 blocks at a time go through LDS.
constexpr int kT = 32, kB = 32;
__global__ void __launch_bounds__(256) min32_tile_kernel(const uint16_t *__restrict__ mins, cq_act_view a, int64_t n, int64_t nb,
                                                         int64_t m, float *__restrict__ y) {
    __shared__ float sm[kT][kB + 1], ss[kT][kB + 1];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int64_t c0 = (int64_t)blockIdx.x * kT, r0 = (int64_t)blockIdx.y * kT;
    float acc[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
    for (int64_t b0 = 0; b0 < nb; b0 += kB) {
        for (int e = threadIdx.x; e < kT * kB; e += 256) {
            const int row = e / kB, bb = e % kB;
            const int64_t b = b0 + bb;
            const bool ok = b < nb;
            sm[row][bb] = ok && c0 + row < n ? cq_h2f(mins[(c0 + row) * nb + b]) : 0.0f;
            ss[row][bb] = ok && r0 + row < m ? block_s(a, (r0 + row) * nb + b) : 0.0f;
        }
        __syncthreads();
        for (int g = 0; g < kB && b0 + g < nb; g += kChunk) {
            float t[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
#pragma unroll
            for (int i = 0; i < kChunk; i++) {
                if (b0 + g + i < nb) {   // blocks past the end of the row are left out, not added as zeros
                    const float s0 = ss[ty][g + i], s1 = ss[ty + 16][g + i], m0 = sm[tx][g + i], m1 = sm[tx + 16][g + i];
                    t[0][0] += m0 * s0;
                    t[0][1] += m1 * s0;
                    t[1][0] += m0 * s1;
                    t[1][1] += m1 * s1;
                }
            }
            acc[0][0] += t[0][0];
            acc[0][1] += t[0][1];
            acc[1][0] += t[1][0];
            acc[1][1] += t[1][1];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int64_t r = r0 + ty + 16 * i, c = c0 + tx + 16 * j;
            if (r < m && c < n) y[r * n + c] += acc[i][j];
        }
}

// Few rows (decode, small batches): sixteen lanes per weight row, each a chunk of eight blocks out of 128 at a time; lane
// 0 of the sixteen adds the chunk sums in order.  Sixteen weight rows and four activation rows per workgroup.
constexpr int kSmallRows = 4;
__global__ void __launch_bounds__(256) min32_small_kernel(const uint16_t *__restrict__ mins, cq_act_view a, int64_t n, int64_t nb,
                                                          int64_t m, float *__restrict__ y) {
    __shared__ float part[kSmallRows][16][17];
    const int j = threadIdx.x & 15, cl = threadIdx.x >> 4;
    const int64_t c = (int64_t)blockIdx.x * 16 + cl;
    const uint16_t *mrow = mins + (c < n ? c : n - 1) * nb;
    const int64_t r0 = (int64_t)blockIdx.y * kSmallRows;
    float acc[kSmallRows] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t sb = 0; sb < nb; sb += 16 * kChunk) {
        const int64_t b = sb + j * kChunk;
        const int cnt = (int)(nb - b < kChunk ? (nb - b < 0 ? 0 : nb - b) : kChunk);
        float mv[kChunk];
#pragma unroll
        for (int i = 0; i < kChunk; i++) mv[i] = i < cnt ? cq_h2f(mrow[b + i]) : 0.0f;
#pragma unroll
        for (int r = 0; r < kSmallRows; r++) {
            float t = 0.0f;
            if (r0 + r < m) {
#pragma unroll
                for (int i = 0; i < kChunk; i++)
                    if (i < cnt) t += mv[i] * block_s(a, (r0 + r) * nb + b + i);
            }
            part[r][cl][j] = t;
        }
        __syncthreads();
        if (j == 0) {
            for (int jj = 0; jj < 16 && sb + jj * kChunk < nb; jj++)
#pragma unroll
                for (int r = 0; r < kSmallRows; r++) acc[r] += part[r][cl][jj];
        }
        __syncthreads();
    }
    if (j == 0 && c < n)
        for (int r = 0; r < kSmallRows && r0 + r < m; r++) y[(r0 + r) * n + c] += acc[r];
}

// ---- Q2K: the dmin term of its dot product with Q8K activations (k_quants.rs:727-733, :762) ----
//   y[r, c] -= sum_b (d8[r, b] * h2f(dmin[c, b])) * float(sum_j bsums[r, b, j] * m[c, b, j])
// One thread per weight row c and up to eight activation rows; the rows' bsums and scales of sixteen blocks at a time in
// LDS.  Every output adds its blocks one after the other, whatever the number of rows.
constexpr int kQ2Rows = 8, kQ2Blocks = 16;
__global__ void __launch_bounds__(64) min16_kernel(const uint8_t *__restrict__ mins, const uint16_t *__restrict__ dmins, cq_act_view a,
                                                   int64_t n, int64_t kb, int64_t m, float *__restrict__ y) {
    __shared__ int16_t sb[kQ2Rows][kQ2Blocks][16];
    __shared__ float sd[kQ2Rows][kQ2Blocks];
    const int64_t c = (int64_t)blockIdx.x * 64 + threadIdx.x, r0 = (int64_t)blockIdx.y * kQ2Rows;
    const int64_t cc = c < n ? c : n - 1;
    float acc[kQ2Rows];
#pragma unroll
    for (int r = 0; r < kQ2Rows; r++) acc[r] = 0.0f;
    for (int64_t b0 = 0; b0 < kb; b0 += kQ2Blocks) {
        const int cnt = (int)(kb - b0 < kQ2Blocks ? kb - b0 : kQ2Blocks);
        for (int e = threadIdx.x; e < kQ2Rows * kQ2Blocks * 16; e += 64) {
            const int r = e / (kQ2Blocks * 16), bb = (e / 16) % kQ2Blocks, j = e % 16;
            const bool ok = r0 + r < m && bb < cnt;
            sb[r][bb][j] = ok ? a.bsums[((r0 + r) * kb + b0 + bb) * 16 + j] : (int16_t)0;
            if (j == 0) sd[r][bb] = ok ? a.d[(r0 + r) * kb + b0 + bb] : 0.0f;
        }
        __syncthreads();
        for (int bb = 0; bb < cnt; bb++) {
            const uint4 mw = *(const uint4 *)(mins + (cc * kb + b0 + bb) * 16);
            const float dmin = cq_h2f(dmins[cc * kb + b0 + bb]);
            const uint32_t w[4] = {mw.x, mw.y, mw.z, mw.w};
#pragma unroll
            for (int r = 0; r < kQ2Rows; r++) {
                int summs = 0;
#pragma unroll
                for (int j = 0; j < 16; j++) summs += (int)sb[r][bb][j] * (int)((w[j >> 2] >> (8 * (j & 3))) & 0xff);
                acc[r] += (sd[r][bb] * dmin) * (float)summs;
            }
        }
        __syncthreads();
    }
    if (c < n)
        for (int r = 0; r < kQ2Rows && r0 + r < m; r++) y[(r0 + r) * n + c] -= acc[r];
}

// Few rows (decode, small batches): sixteen lanes per weight row, each one block out of sixteen at a time; lane 0 of the
// sixteen adds the block terms in order (the same terms, the same order as above).  Sixteen weight rows and four
// activation rows per workgroup, so that a launch has many workgroups where the kernel above would have few.
__global__ void __launch_bounds__(256) min16_small_kernel(const uint8_t *__restrict__ mins, const uint16_t *__restrict__ dmins,
                                                          cq_act_view a, int64_t n, int64_t kb, int64_t m, float *__restrict__ y) {
    __shared__ float part[kSmallRows][16][17];
    const int j = threadIdx.x & 15, cl = threadIdx.x >> 4;
    const int64_t c = (int64_t)blockIdx.x * 16 + cl;
    const int64_t cc = c < n ? c : n - 1, r0 = (int64_t)blockIdx.y * kSmallRows;
    float acc[kSmallRows] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t sb = 0; sb < kb; sb += 16) {
        const int64_t b = sb + j;
        if (b < kb) {
            const uint4 mw = *(const uint4 *)(mins + (cc * kb + b) * 16);
            const float dmin = cq_h2f(dmins[cc * kb + b]);
            const uint32_t w[4] = {mw.x, mw.y, mw.z, mw.w};
#pragma unroll
            for (int r = 0; r < kSmallRows; r++) {
                float term = 0.0f;
                if (r0 + r < m) {
                    const int16_t *bs = a.bsums + ((r0 + r) * kb + b) * 16;
                    int summs = 0;
#pragma unroll
                    for (int g = 0; g < 16; g++) summs += (int)bs[g] * (int)((w[g >> 2] >> (8 * (g & 3))) & 0xff);
                    term = (a.d[(r0 + r) * kb + b] * dmin) * (float)summs;
                }
                part[r][cl][j] = term;
            }
        }
        __syncthreads();
        if (j == 0) {
            for (int jj = 0; jj < 16 && sb + jj < kb; jj++)
#pragma unroll
                for (int r = 0; r < kSmallRows; r++) acc[r] += part[r][cl][jj];
        }
        __syncthreads();
    }
    if (j == 0 && c < n)
        for (int r = 0; r < kSmallRows && r0 + r < m; r++) y[(r0 + r) * n + c] -= acc[r];
}

}  // namespace

hipError_t cq_launch_min32_term(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    if (!cq_has_min32(w->ggml_dtype)) return hipErrorInvalidValue;
    if (m == 0 || w->n == 0 || w->k == 0) return hipSuccess;
    const int64_t nb = w->k / 32;
    const uint16_t *mins = (const uint16_t *)w->p2;
    if (m <= kSmallRows)   // (measured slower than the tile kernel from five rows on)
        CQ_LAUNCH(min32_small_kernel, dim3((unsigned)((w->n + 15) / 16), (unsigned)((m + kSmallRows - 1) / kSmallRows)), 256, 0, s, mins, a,
                  w->n, nb, m, y);
    else CQ_LAUNCH(min32_tile_kernel, dim3((unsigned)((w->n + kT - 1) / kT), (unsigned)((m + kT - 1) / kT)), 256, 0, s, mins, a, w->n, nb, m, y);
    return hipGetLastError();
}

hipError_t cq_launch_min16_term(const cq_weight *w, cq_act_view a, int64_t m, float *y, hipStream_t s) {
    if (!cq_has_min16(w->ggml_dtype)) return hipErrorInvalidValue;
    if (m == 0 || w->n == 0 || w->k == 0) return hipSuccess;
    if (m <= 64)
        CQ_LAUNCH(min16_small_kernel, dim3((unsigned)((w->n + 15) / 16), (unsigned)((m + kSmallRows - 1) / kSmallRows)), 256, 0, s, w->p4,
                  (const uint16_t *)w->p5, a, w->n, w->k / 256, m, y);
    else
        CQ_LAUNCH(min16_kernel, dim3((unsigned)((w->n + 63) / 64), (unsigned)((m + kQ2Rows - 1) / kQ2Rows)), 64, 0, s, w->p4,
                  (const uint16_t *)w->p5, a, w->n, w->k / 256, m, y);
    return hipGetLastError();
}
