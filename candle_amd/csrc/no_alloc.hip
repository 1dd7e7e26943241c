// cq_qmatmul_static: cq_qmatmul for callers that cannot allocate device memory (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc).  The quantized activations, which
// cq_qmatmul keeps in a workspace the caller allocates, live in a device array of this code object.
#include <atomic>

#include "qhip_internal.h"

// One copy of this array exists on every GPU the code object is loaded on, each at an address of its
// own.  In host code the name is only a handle for hipGetSymbolAddress: it is never passed to a
// kernel or a runtime call; host code uses the address looked up below, once per device, with that
// device current.
static __device__ __align__(256) uint8_t cq_static_scratch[CQ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxScratchDev = 64;
std::atomic<uint8_t *> g_scratch_ptr[kMaxScratchDev];
}  // namespace

// Device address of the scratch array on `dev`, which must be the current device.  nullptr (and a
// message for cq_last_error) when the lookup fails.
uint8_t *cq_static_scratch_ptr(int dev) {
    if (dev < 0 || dev >= kMaxScratchDev) {
        cq_set_error(CQ_ERR_INVALID, "device %d is beyond the %d devices the static scratch table holds", dev, kMaxScratchDev);
        return nullptr;
    }
    if (uint8_t *p = g_scratch_ptr[dev].load(std::memory_order_acquire)) return p;
    void *sym = nullptr;
    const hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(cq_static_scratch));
    if (e != hipSuccess || !sym) {
        cq_set_error(CQ_ERR_HIP, "hipGetSymbolAddress(cq_static_scratch) failed on device %d: %s", dev, hipGetErrorString(e));
        return nullptr;
    }
    g_scratch_ptr[dev].store((uint8_t *)sym, std::memory_order_release);   // racing threads store the same address
    return (uint8_t *)sym;
}

extern "C" int cq_qmatmul_static(const cq_weight *w, const float *x_dev, int64_t m, float *y_dev, int flags, void *stream) {
    if (!w) return cq_set_error(CQ_ERR_INVALID, "null weight");
    if (m < 0) return cq_set_error(CQ_ERR_INVALID, "negative row count");
    const size_t need = cq_workspace_bytes(w, m, flags);
    if (need > (size_t)CQ_STATIC_SCRATCH_BYTES)
        return cq_set_error(CQ_ERR_WORKSPACE,
                            "%lld rows of %lld elements need %zu bytes of scratch, the static array holds %zu: "
                            "use cq_qmatmul with a workspace",
                            (long long)m, (long long)w->k, need, (size_t)CQ_STATIC_SCRATCH_BYTES);
    CQ_HIP_CHECK(hipSetDevice(w->dev));
    uint8_t *scratch = cq_static_scratch_ptr(w->dev);   // looked up when the first weight of the device was created
    if (!scratch) return CQ_ERR_HIP;
    // Nothing in the scratch has to start at zero: the quantizer launch writes every byte the matmul
    // kernels use of it before they read it, as with a caller's workspace that is reused between calls.
    return cq_qmatmul(w, x_dev, m, y_dev, flags, scratch, (size_t)CQ_STATIC_SCRATCH_BYTES, stream);
}
