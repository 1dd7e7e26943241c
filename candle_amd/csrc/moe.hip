// Glue kernels of the MoE FFN (candle-transformers/src/models/quantized_llama.rs:56-63, :116-135).
#include "qhip_internal.h"

namespace {

// h = silu(a) * b, silu(v) = v / (1 + exp(-v))  (candle-core/src/op.rs:607-609)
__global__ void silu_mul_kernel(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ h,
                                int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const float v = a[i];
    const float s = v / (1.0f + expf(-v));
    h[i] = s * b[i];
}

// ys[row_ids[p], j] += weights[p] * y[p, j], positions p visited in increasing order for every
// destination element (the reference's sequential index_add, cpu_backend/mod.rs:619-653, applied
// expert by expert).  One thread per destination element; no atomics, so the sum order is fixed.
__global__ void scatter_add_kernel(const float *__restrict__ y, const int32_t *__restrict__ row_ids,
                                   const float *__restrict__ weights, int64_t total_rows, int64_t hidden,
                                   float *__restrict__ ys, int64_t tokens) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= tokens * hidden) return;
    const int64_t t = i / hidden, j = i - t * hidden;
    float acc = ys[i];
    for (int64_t p = 0; p < total_rows; p++) {
        if (row_ids[p] == (int32_t)t) acc += y[p * hidden + j] * weights[p];
    }
    ys[i] = acc;
}

// The same sum for hidden % 4 == 0: a workgroup owns 1024 consecutive elements of one token, so the
// search for the token's rows is wave-uniform (scalar loads and branches) and only the matching
// rows cost vector work.
__global__ void scatter_add4_kernel(const float *__restrict__ y, const int32_t *__restrict__ row_ids,
                                    const float *__restrict__ weights, int total_rows, int64_t hidden,
                                    float *__restrict__ ys) {
    const int32_t t = (int32_t)blockIdx.y;
    const int64_t j = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    const int lane = threadIdx.x & 63;
    const bool live = j < hidden;
    float4 acc = live ? *(const float4 *)(ys + (int64_t)t * hidden + j) : make_float4(0.f, 0.f, 0.f, 0.f);
    // 64 row ids per step, one per lane; the matches come out of the lane mask in increasing order
    for (int base = 0; base < total_rows; base += 64) {
        const int q = base + lane;
        const int32_t rid = q < total_rows ? row_ids[q] : -1;
        uint64_t hits = __builtin_amdgcn_ballot_w64(rid == t);
        while (hits) {
            const int p = base + __builtin_ctzll(hits);
            hits &= hits - 1;
            if (live) {
                const float4 v = *(const float4 *)(y + (int64_t)p * hidden + j);
                const float wgt = weights[p];
                acc.x += v.x * wgt;
                acc.y += v.y * wgt;
                acc.z += v.z * wgt;
                acc.w += v.w * wgt;
            }
        }
    }
    if (live) *(float4 *)(ys + (int64_t)t * hidden + j) = acc;
}

__global__ void fill_zero_kernel(float *p, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] = 0.0f;
}

}  // namespace

hipError_t cq_launch_silu_mul(const float *a, const float *b, float *h, int64_t count, hipStream_t s) {
    silu_mul_kernel<<<(unsigned)((count + 255) / 256), 256, 0, s>>>(a, b, h, count);
    return hipGetLastError();
}

hipError_t cq_launch_scatter_add(const float *y, const int32_t *row_ids, const float *weights, int64_t total_rows,
                                 int64_t hidden, float *ys, int64_t tokens, hipStream_t s) {
    if (hidden % 4 == 0 && tokens <= 65535 && total_rows <= INT32_MAX && (((uintptr_t)y | (uintptr_t)ys) & 15) == 0) {
        if (tokens == 0 || hidden == 0) return hipSuccess;
        dim3 grid((unsigned)((hidden / 4 + 255) / 256), (unsigned)tokens);
        scatter_add4_kernel<<<grid, 256, 0, s>>>(y, row_ids, weights, (int)total_rows, hidden, ys);
        return hipGetLastError();
    }
    const int64_t count = tokens * hidden;
    scatter_add_kernel<<<(unsigned)((count + 255) / 256), 256, 0, s>>>(y, row_ids, weights, total_rows, hidden, ys,
                                                                        tokens);
    return hipGetLastError();
}

hipError_t cq_launch_fill_zero(float *p, int64_t count, hipStream_t s) {
    if (count == 0) return hipSuccess;
    fill_zero_kernel<<<(unsigned)((count + 255) / 256), 256, 0, s>>>(p, count);
    return hipGetLastError();
}
