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
