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
constexpr int kMaxScratchDev = 32;   // as many devices as the table of granted LDS sizes holds (cq_ensure_lds)
std::atomic<uint8_t *> g_scratch_ptr[kMaxScratchDev];
}  // namespace

// Device address of the scratch array on `dev`, which must be the current device, into *out.  Returns CQ_OK, or the
// error code it has set (with a message for cq_last_error) when the lookup fails.
static int scratch_lookup(int dev, uint8_t **out) {
    *out = nullptr;
    if (dev < 0 || dev >= kMaxScratchDev)
        return cq_set_error(CQ_ERR_INVALID, "device %d is beyond the %d devices the static scratch table holds", dev, kMaxScratchDev);
    if (uint8_t *p = g_scratch_ptr[dev].load(std::memory_order_acquire)) {
        *out = p;
        return CQ_OK;
    }
    void *sym = nullptr;
    const hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(cq_static_scratch));
    if (e != hipSuccess || !sym)
        return cq_set_error(CQ_ERR_HIP, "hipGetSymbolAddress(cq_static_scratch) failed on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev].store((uint8_t *)sym, std::memory_order_release);   // racing threads store the same address
    *out = (uint8_t *)sym;
    return CQ_OK;
}
uint8_t *cq_static_scratch_ptr(int dev) {
    uint8_t *p = nullptr;
    (void)scratch_lookup(dev, &p);
    return p;
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
    uint8_t *scratch = nullptr;   // looked up when the first weight of the device was created
    if (int rc = scratch_lookup(w->dev, &scratch)) return rc;
    // Nothing in the scratch has to start at zero: the quantizer launch writes every byte the matmul
    // kernels use of it before they read it, as with a caller's workspace that is reused between calls.
    return cq_qmatmul(w, x_dev, m, y_dev, flags, scratch, (size_t)CQ_STATIC_SCRATCH_BYTES, stream);
}
