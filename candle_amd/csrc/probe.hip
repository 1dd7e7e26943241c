// Measurement aid, not part of the product library: two reference kernels that bound what any
// decode launch can reach on a device, built into libcandle_qhip_probe.so and driven by
// `bench.py --envelope`.
//   cqp_empty:       a kernel that does nothing, with a chosen grid / block / dynamic LDS size
//                    (the cost of one launch in a stream or a graph chain);
//   cqp_stream_read: every lane reads 16 bytes per step, `unroll` steps in flight, over `bytes`
//                    bytes, and keeps an xor of what it read (a pure HBM read at full width).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

__global__ void empty_kernel(uint32_t *sink, uint32_t magic) {
    extern __shared__ uint8_t smem[];
    if (magic == 0x12345678u && threadIdx.x == 0) sink[0] = smem[0];   // never true: keeps the LDS allocation
}

template <int U>
__global__ void stream_read_kernel(const uint4 *__restrict__ p, size_t n16, uint32_t *sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t acc = 0;
    uint4 v[U];
    for (; i + (U - 1) * stride < n16; i += U * stride) {
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = p[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) {
        const uint4 t = p[i];
        acc += t.x ^ t.y ^ t.z ^ t.w;
    }
    if (acc == 0x12345678u) sink[0] = acc;   // practically never: the loads must not be optimized away
}

}  // namespace

extern "C" int cqp_empty(int grid, int block, int lds_bytes, uint32_t *sink_dev, void *stream) {
    hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), (uint32_t)lds_bytes, (hipStream_t)stream, sink_dev, 0u);
    return (int)hipGetLastError();
}

extern "C" int cqp_stream_read(const void *buf_dev, size_t bytes, int grid, int block, int unroll, uint32_t *sink_dev,
                               void *stream) {
    const uint4 *p = (const uint4 *)buf_dev;
    const size_t n16 = bytes / 16;
    hipStream_t s = (hipStream_t)stream;
    switch (unroll) {
    case 1: hipLaunchKernelGGL(stream_read_kernel<1>, dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 2: hipLaunchKernelGGL(stream_read_kernel<2>, dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 4: hipLaunchKernelGGL(stream_read_kernel<4>, dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 8: hipLaunchKernelGGL(stream_read_kernel<8>, dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}
