// Measurement aid, not part of the product library: reference kernels that bound what any
// decode launch can reach on a device, built into libcandle_qhip_probe.so and driven by
// `bench.py --envelope`.
//   cqp_empty:           a kernel that does nothing, with a chosen grid / block / dynamic LDS size
//                        (the cost of one launch in a stream or a graph chain);
//   cqp_stream_read:     every lane reads 16 bytes per step, `unroll` steps in flight, over `bytes`
//                        bytes, and keeps an xor of what it read (a pure HBM read at full width);
//   cqp_stream_read_pol: the same through buffer loads with a chosen cache policy (the `aux` bits of
//                        the load: 1 = sc0, 2 = nt, 16 = sc1);
//   cqp_lds_read:        the same bytes requested as buffer loads that land in LDS (no registers per
//                        request), each wave with a ring of `ring` one-KiB requests in flight;
//   cqp_lds_read_rows:   the same with a wave owning whole rows of consecutive KiB (the decode kernels' ownership);
//   cqp_mfma_clock:      the shader clock the part holds while every matrix pipe runs int8 MFMAs (the published
//                        peaks assume 2.4 GHz), and the time per 32x32x32 int8 MFMA and SIMD at that clock.
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

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void *lptr_t;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_rsrc(const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, -1, 0x00020000);
}

// Buffer loads of 16 bytes per lane with the cache-policy bits AUX, U steps in flight.  The buffer is at most 4 GiB - 1.
template <int U, int AUX>
__global__ void stream_read_pol_kernel(const uint8_t *__restrict__ p, uint32_t n16, uint32_t *sink) {
    const uint32_t stride = gridDim.x * blockDim.x;
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p);
    uint32_t acc = 0;
    u32x4 v[U];
    for (; i + (U - 1) * stride < n16; i += U * stride) {
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)((i + u * stride) * 16u), 0, AUX);
#pragma unroll
        for (int u = 0; u < U; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) {
        const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(i * 16u), 0, AUX);
        acc += t.x ^ t.y ^ t.z ^ t.w;
    }
    if (acc == 0x12345678u) sink[0] = acc;
}

// Every wave requests one-KiB pieces (16 bytes per lane) that land in its own LDS ring of RING slots; piece j of the
// launch belongs to wave j mod (waves of the launch), so the launch reads a contiguous band at any time.  A slot is
// requested again once its previous request has landed (requests return in order: at most RING - 1 younger ones may be
// outstanding).  Nothing is computed; one word of the ring is read at the end.
template <int RING, int AUX>
__global__ void lds_read_kernel(const uint8_t *__restrict__ p, uint32_t pieces, uint32_t *sink) {
    extern __shared__ __align__(16) uint8_t smem[];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wpb = blockDim.x >> 6;
    const uint32_t gw = blockIdx.x * wpb + wave, tw = gridDim.x * wpb;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p);
    uint8_t *ring = smem + wave * (RING * 1024);
    uint32_t j = gw;
    // first RING requests (those that exist)
#pragma unroll
    for (int s = 0; s < RING; s++) {
        if (j < pieces) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(ring + s * 1024), 16, (int)(j * 1024u + lane * 16u), 0, 0, AUX);
        j += tw;
    }
    while (j < pieces) {
#pragma unroll
        for (int s = 0; s < RING; s++) {
            if (j < pieces) {
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(RING - 1) : "memory");
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(ring + s * 1024), 16, (int)(j * 1024u + lane * 16u), 0, 0, AUX);
            }
            j += tw;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const uint32_t v = *(const uint32_t *)(smem + threadIdx.x * 4);
    if (v == 0x12345679u) sink[0] = v;
}

// The same bytes with the decode kernels' ownership: the buffer is `rows` rows of P one-KiB pieces, wave g of the
// launch owns rows g, g + waves, ... and requests a row's pieces one after the other.
template <int RING, int AUX>
__global__ void lds_read_rows_kernel(const uint8_t *__restrict__ p, uint32_t rows, uint32_t P, uint32_t *sink) {
    extern __shared__ __align__(16) uint8_t smem[];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wpb = blockDim.x >> 6;
    const uint32_t gw = blockIdx.x * wpb + wave, tw = gridDim.x * wpb;
    const __amdgpu_buffer_rsrc_t rs = wave_rsrc(p);
    uint8_t *ring = smem + wave * (RING * 1024);
    const uint32_t my_rows = gw < rows ? (rows - gw + tw - 1) / tw : 0;
    const uint32_t total = my_rows * P;
    auto piece_off = [&](uint32_t s) { return ((gw + (s / P) * tw) * P + s % P) * 1024u + lane * 16u; };
    uint32_t s = 0;
#pragma unroll
    for (int i = 0; i < RING; i++) {
        if (s < total) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(ring + i * 1024), 16, (int)piece_off(s), 0, 0, AUX);
        s++;
    }
    while (s < total) {
#pragma unroll
        for (int i = 0; i < RING; i++) {
            if (s < total) {
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(RING - 1) : "memory");
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lptr_t)(ring + i * 1024), 16, (int)piece_off(s), 0, 0, AUX);
            }
            s++;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const uint32_t v = *(const uint32_t *)(smem + threadIdx.x * 4);
    if (v == 0x12345679u) sink[0] = v;
}

// Two waves per SIMD run dependent chains of 32x32x32 int8 MFMAs on pseudo-random operands; wave 0 of workgroup 0
// reads the shader-clock counter and the constant 100 MHz counter before and after.
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(512) mfma_clock_kernel(int iters, uint64_t *out, int *sink) {
    v4i_t a, b;
    for (int i = 0; i < 4; i++) {
        a[i] = (int)(threadIdx.x * 2654435761u + 977u * (i + 1));
        b[i] = (int)(threadIdx.x * 40503u + 131u * (i + 7));
    }
    v16i_t lo = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, hi = lo;
    const uint64_t c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; it++) {
        asm volatile("" : "+v"(a), "+v"(b));   // not loop-invariant
#pragma unroll
        for (int s = 0; s < 8; s++) {
            lo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, lo, 0, 0, 0);
            hi = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, a, hi, 0, 0, 0);
        }
    }
    int acc = 0;
    for (int i = 0; i < 16; i++) acc += lo[i] ^ hi[i];
    const uint64_t c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    if (acc == 0x12345678) sink[0] = acc;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        out[0] = c1 - c0;
        out[1] = r1 - r0;
    }
}

}  // namespace

// out_dev[0] = shader-clock cycles, out_dev[1] = ticks of the constant 100 MHz counter over `iters` x 16 MFMAs per wave
// (256 workgroups of eight waves: two per SIMD on every CU).
extern "C" int cqp_mfma_clock(int iters, uint64_t *out_dev, int *sink_dev, void *stream) {
    hipLaunchKernelGGL(mfma_clock_kernel, dim3(256), dim3(512), 0, (hipStream_t)stream, iters, out_dev, sink_dev);
    return (int)hipGetLastError();
}

extern "C" int cqp_lds_read_rows(const void *buf_dev, size_t bytes, int grid, int pieces_per_row, uint32_t *sink_dev, void *stream) {
    const uint8_t *p = (const uint8_t *)buf_dev;
    if (bytes >= ((size_t)1 << 32) || pieces_per_row < 1) return (int)hipErrorInvalidValue;
    const uint32_t rows = (uint32_t)(bytes / 1024 / (size_t)pieces_per_row);
    const uint32_t lds = 8 * 1024 * 8;
    static bool once = false;
    if (!once) {
        hipError_t e = hipFuncSetAttribute((const void *)lds_read_rows_kernel<8, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        once = true;
    }
    hipLaunchKernelGGL((lds_read_rows_kernel<8, 2>), dim3(grid), dim3(512), lds, (hipStream_t)stream, p, rows, (uint32_t)pieces_per_row, sink_dev);
    return (int)hipGetLastError();
}

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

extern "C" int cqp_stream_read_pol(const void *buf_dev, size_t bytes, int grid, int block, int aux, uint32_t *sink_dev,
                                   void *stream) {
    const uint8_t *p = (const uint8_t *)buf_dev;
    if (bytes >= ((size_t)1 << 32)) return (int)hipErrorInvalidValue;
    const uint32_t n16 = (uint32_t)(bytes / 16);
    hipStream_t s = (hipStream_t)stream;
    switch (aux) {
    case 0: hipLaunchKernelGGL((stream_read_pol_kernel<4, 0>), dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 1: hipLaunchKernelGGL((stream_read_pol_kernel<4, 1>), dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 2: hipLaunchKernelGGL((stream_read_pol_kernel<4, 2>), dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 3: hipLaunchKernelGGL((stream_read_pol_kernel<4, 3>), dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 16: hipLaunchKernelGGL((stream_read_pol_kernel<4, 16>), dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 17: hipLaunchKernelGGL((stream_read_pol_kernel<4, 17>), dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 18: hipLaunchKernelGGL((stream_read_pol_kernel<4, 18>), dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    case 19: hipLaunchKernelGGL((stream_read_pol_kernel<4, 19>), dim3(grid), dim3(block), 0, s, p, n16, sink_dev); break;
    default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

// block = 512 threads (8 waves); ring slots of 1 KiB per wave: 4, 8 or 16 (32 / 64 / 128 KiB of LDS per workgroup)
extern "C" int cqp_lds_read(const void *buf_dev, size_t bytes, int grid, int ring, int aux, uint32_t *sink_dev, void *stream) {
    const uint8_t *p = (const uint8_t *)buf_dev;
    if (bytes >= ((size_t)1 << 32)) return (int)hipErrorInvalidValue;
    const uint32_t pieces = (uint32_t)(bytes / 1024);
    hipStream_t s = (hipStream_t)stream;
    const int block = 512;
    const uint32_t lds = (uint32_t)(ring * 1024 * (block / 64));
    hipError_t e = hipSuccess;
#define CQP_LDS_CASE(R, A)                                                                                   \
    if (ring == R && aux == A) {                                                                             \
        static bool once = false;                                                                            \
        if (!once) {                                                                                         \
            e = hipFuncSetAttribute((const void *)lds_read_kernel<R, A>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)lds);                                                               \
            if (e != hipSuccess) return (int)e;                                                              \
            once = true;                                                                                     \
        }                                                                                                    \
        hipLaunchKernelGGL((lds_read_kernel<R, A>), dim3(grid), dim3(block), lds, s, p, pieces, sink_dev);   \
        return (int)hipGetLastError();                                                                       \
    }
    CQP_LDS_CASE(4, 0)
    CQP_LDS_CASE(8, 0)
    CQP_LDS_CASE(16, 0)
    CQP_LDS_CASE(8, 2)
    CQP_LDS_CASE(16, 2)
    CQP_LDS_CASE(16, 16)
#undef CQP_LDS_CASE
    return (int)hipErrorInvalidValue;
}
