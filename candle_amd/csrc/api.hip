// C ABI of libcandle_qhip (declarations and reference citations: include/candle_qhip.h).
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <new>

#include "qhip_internal.h"

// ------------------------------------------------------------------ errors ----
static thread_local char g_err[512] = "";

// ---- kernel timing hook ------------------------------------------------------------------------
namespace {
struct KernelTimer {
    hipEvent_t start = nullptr, stop = nullptr;
    bool armed = false, pending = false;
};
thread_local KernelTimer g_timer;
}  // namespace

namespace {
thread_local bool g_no_split = false;
// Scope of one entry point: launches planned inside it never split K when the call carries CQ_FLAG_DETERMINISTIC.
struct NoSplitScope {
    bool prev;
    explicit NoSplitScope(int flags) : prev(g_no_split) { g_no_split = (flags & CQ_FLAG_DETERMINISTIC) != 0; }
    ~NoSplitScope() { g_no_split = prev; }
};
}  // namespace
bool cq_no_split_k() { return g_no_split; }

bool cq_timing_take(hipEvent_t *start, hipEvent_t *stop) {
    if (!g_timer.armed) return false;
    g_timer.armed = false;
    g_timer.pending = true;
    *start = g_timer.start;
    *stop = g_timer.stop;
    return true;
}

int cq_set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" const char *cq_last_error(void) { return g_err; }
extern "C" const char *cq_version(void) { return "candle_qhip 0.1 (gfx950)"; }

extern "C" int cq_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

// ------------------------------------------------------------ dtype tables ----
extern "C" int64_t cq_block_size(int dt) {
    switch (dt) {
    case CQ_DTYPE_Q4_0: case CQ_DTYPE_Q4_1: case CQ_DTYPE_Q5_0: case CQ_DTYPE_Q5_1: case CQ_DTYPE_Q8_0: case CQ_DTYPE_Q8_1: return 32;
    case CQ_DTYPE_Q2K: case CQ_DTYPE_Q3K: case CQ_DTYPE_Q4K: case CQ_DTYPE_Q5K: case CQ_DTYPE_Q6K: case CQ_DTYPE_Q8K: return 256;
    default: return 0;
    }
}
extern "C" int64_t cq_type_size(int dt) {
    switch (dt) {
    case CQ_DTYPE_Q4_0: return 18;
    case CQ_DTYPE_Q4_1: return 20;
    case CQ_DTYPE_Q5_0: return 22;
    case CQ_DTYPE_Q5_1: return 24;
    case CQ_DTYPE_Q2K: return 84;
    case CQ_DTYPE_Q3K: return 110;
    case CQ_DTYPE_Q8_0: return 34;
    case CQ_DTYPE_Q8_1: return 36;
    case CQ_DTYPE_Q4K: return 144;
    case CQ_DTYPE_Q5K: return 176;
    case CQ_DTYPE_Q6K: return 210;
    case CQ_DTYPE_Q8K: return 292;
    default: return 0;
    }
}
extern "C" int cq_vec_dot_type(int dt) {
    switch (dt) {
    case CQ_DTYPE_Q4_0: case CQ_DTYPE_Q5_0: case CQ_DTYPE_Q8_0: return CQ_DTYPE_Q8_0;
    case CQ_DTYPE_Q4_1: case CQ_DTYPE_Q5_1: return CQ_DTYPE_Q8_1;   /* k_quants.rs:260, :457 */
    case CQ_DTYPE_Q2K: case CQ_DTYPE_Q3K: case CQ_DTYPE_Q4K: case CQ_DTYPE_Q5K: case CQ_DTYPE_Q6K: case CQ_DTYPE_Q8K: return CQ_DTYPE_Q8K;
    default: return -1;
    }
}

static bool is_weight_dtype(int dt) {
    return dt == CQ_DTYPE_Q4_0 || dt == CQ_DTYPE_Q4_1 || dt == CQ_DTYPE_Q5_0 || dt == CQ_DTYPE_Q5_1 || dt == CQ_DTYPE_Q8_0 ||
           dt == CQ_DTYPE_Q2K || dt == CQ_DTYPE_Q3K || dt == CQ_DTYPE_Q4K ||
           dt == CQ_DTYPE_Q5K || dt == CQ_DTYPE_Q6K || dt == CQ_DTYPE_Q8K;
}

// --------------------------------------------------------------- weights ----
static int weight_alloc(int dev, int dt, int64_t n, int64_t k, cq_weight **out) {
    if (!out) return cq_set_error(CQ_ERR_INVALID, "out is null");
    *out = nullptr;
    if (!is_weight_dtype(dt)) return cq_set_error(CQ_ERR_UNSUPPORTED, "unsupported weight dtype %d", dt);
    if (n < 0 || k < 0) return cq_set_error(CQ_ERR_INVALID, "negative shape [%lld, %lld]", (long long)n, (long long)k);
    const int64_t bs = cq_block_size(dt);
    // check_shape, candle-core/src/quantized/mod.rs:304-316
    if (k % bs != 0)
        return cq_set_error(CQ_ERR_INVALID,
                            "quantized tensor must have their last dim divisible by block size [%lld, %lld] %lld",
                            (long long)n, (long long)k, (long long)bs);
    int ndev = cq_device_count();
    if (dev < 0 || dev >= ndev) return cq_set_error(CQ_ERR_INVALID, "device %d out of range (%d visible)", dev, ndev);
    CQ_HIP_CHECK(hipSetDevice(dev));
    cq_weight *w = new (std::nothrow) cq_weight();
    if (!w) return cq_set_error(CQ_ERR_INVALID, "out of host memory");
    w->dev = dev; w->dtype = cq_storage_dtype(dt); w->ggml_dtype = dt; w->n = n; w->k = k;
    const int64_t nb = n * (k / bs);
    w->ggml_bytes = (size_t)nb * (size_t)cq_type_size(dt);
    size_t s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    switch (w->dtype) {
    case CQ_DTYPE_Q4_0: s0 = (size_t)nb * 16; s1 = (size_t)nb * 2; break;
    case CQ_DTYPE_Q8_0: s0 = (size_t)nb * 32; s1 = (size_t)nb * 2; break;
    case CQ_DTYPE_Q4K: s0 = (size_t)nb * 128; s1 = (size_t)nb * CQ_Q4K_HDR; break;
    case CQ_DTYPE_Q5K: s0 = (size_t)nb * 128; s1 = (size_t)nb * CQ_Q4K_HDR; s2 = (size_t)nb * 32; break;
    case CQ_DTYPE_Q6K: s0 = (size_t)nb * 128; s1 = (size_t)nb * 64; s2 = (size_t)nb * 16; s3 = (size_t)nb * 2; break;
    case CQ_DTYPE_Q8K: s0 = (size_t)nb * 256; s1 = (size_t)nb * 4; s2 = (size_t)nb * 32; break;
    }
    if (cq_has_min32(dt)) s2 = (size_t)nb * 2;   // the blocks' minima beside the Q8_0 planes
    size_t s4 = 0, s5 = 0;
    if (cq_has_min16(dt)) { s4 = (size_t)nb * 16; s5 = (size_t)nb * 2; }   // the groups' minima and dmin beside the Q6K planes
    const size_t o1 = cq_align_up(s0 + CQ_TAIL_PAD, 256);
    const size_t o2 = cq_align_up(o1 + s1 + CQ_TAIL_PAD, 256);
    const size_t o3 = cq_align_up(o2 + s2 + CQ_TAIL_PAD, 256);
    const size_t o4 = cq_align_up(o3 + s3 + CQ_TAIL_PAD, 256);
    const size_t o5 = cq_align_up(o4 + s4 + CQ_TAIL_PAD, 256);
    w->alloc_bytes = cq_align_up(o5 + s5 + CQ_TAIL_PAD, 256);
    hipError_t e = hipMalloc(&w->base, w->alloc_bytes);
    if (e != hipSuccess) {
        const size_t bytes = w->alloc_bytes;
        delete w;
        return cq_set_error(CQ_ERR_HIP, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    }
    w->p0 = (uint8_t *)w->base;
    w->p1 = (uint8_t *)w->base + o1;
    w->p2 = (uint8_t *)w->base + o2;
    w->p3 = (uint8_t *)w->base + o3;
    w->p4 = (uint8_t *)w->base + o4;
    w->p5 = (uint8_t *)w->base + o5;
    // creating a weight is the set-up call every user of a device goes through: the scratch array of
    // cq_qmatmul_static is looked up here, so that the first matmul on the device has nothing left to set up
    // (a failure is reported by cq_qmatmul_static itself, which looks again)
    (void)cq_static_scratch_ptr(dev);
    *out = w;
    return CQ_OK;
}

// GGML blocks of the caller's type (device memory) into the planes, and back.  A type held in another type's planes
// goes through that type's blocks in a temporary (set-up paths: they synchronize before freeing it).
static int64_t weight_blocks(const cq_weight *w) { return w->n * (w->k / cq_block_size(w->dtype)); }
static hipError_t blocks_to_planes(const cq_weight *w, uint8_t *ggml_aos_dev, hipStream_t s) {
    if (w->ggml_dtype == w->dtype) return cq_launch_repack(w, ggml_aos_dev, s);
    void *tmp = nullptr;
    hipError_t e = hipMalloc(&tmp, (size_t)weight_blocks(w) * (size_t)cq_type_size(w->dtype) + 256);
    if (e != hipSuccess) return e;
    e = cq_launch_transcode(w, ggml_aos_dev, (uint8_t *)tmp, weight_blocks(w), false, s);
    if (e == hipSuccess) e = cq_launch_repack(w, (const uint8_t *)tmp, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    (void)hipFree(tmp);
    return e;
}
static hipError_t planes_to_blocks(const cq_weight *w, uint8_t *ggml_aos_dev, hipStream_t s) {
    if (w->ggml_dtype == w->dtype) return cq_launch_unpack(w, ggml_aos_dev, s);
    void *tmp = nullptr;
    hipError_t e = hipMalloc(&tmp, (size_t)weight_blocks(w) * (size_t)cq_type_size(w->dtype) + 256);
    if (e != hipSuccess) return e;
    e = cq_launch_unpack(w, (uint8_t *)tmp, s);
    if (e == hipSuccess) e = cq_launch_transcode(w, ggml_aos_dev, (uint8_t *)tmp, weight_blocks(w), true, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    (void)hipFree(tmp);
    return e;
}

extern "C" int cq_weight_zeros(int dev, int dt, int64_t n, int64_t k, cq_weight **out) {
    int rc = weight_alloc(dev, dt, n, k, out);
    if (rc) return rc;
    hipError_t e = hipMemset((*out)->base, 0, (*out)->alloc_bytes);
    if (e == hipSuccess && (*out)->ggml_dtype != (*out)->dtype && (*out)->ggml_bytes) {
        // all-zero blocks of the caller's type are not all-zero planes of the holding type (a zero quant is stored
        // with its offset): encode them
        void *tmp = nullptr;
        e = hipMalloc(&tmp, (*out)->ggml_bytes + 256);
        if (e == hipSuccess) e = hipMemset(tmp, 0, (*out)->ggml_bytes);
        if (e == hipSuccess) e = blocks_to_planes(*out, (uint8_t *)tmp, nullptr);
        if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
        if (tmp) (void)hipFree(tmp);
    }
    if (e != hipSuccess) {
        cq_weight_destroy(*out);
        *out = nullptr;
        return cq_set_error(CQ_ERR_HIP, "hipMemset failed: %s", hipGetErrorString(e));
    }
    return CQ_OK;
}

extern "C" int cq_weight_create(int dev, int dt, const void *host_blocks, size_t nbytes, int64_t n, int64_t k,
                                cq_weight **out) {
    if (!host_blocks && nbytes) return cq_set_error(CQ_ERR_INVALID, "host_ggml_blocks is null");
    int rc = cq_weight_zeros(dev, dt, n, k, out);
    if (rc) return rc;
    cq_weight *w = *out;
    if (nbytes != w->ggml_bytes) {
        cq_weight_destroy(w);
        *out = nullptr;
        return cq_set_error(CQ_ERR_INVALID, "expected %zu bytes of GGML blocks for [%lld, %lld] dtype %d, got %zu",
                            w->ggml_bytes, (long long)n, (long long)k, dt, nbytes);
    }
    if (nbytes == 0) return CQ_OK;
    void *tmp = nullptr;
    hipError_t e = hipMalloc(&tmp, nbytes + 256);
    if (e == hipSuccess) e = hipMemcpy(tmp, host_blocks, nbytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = blocks_to_planes(w, (uint8_t *)tmp, nullptr);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    if (tmp) (void)hipFree(tmp);
    if (e != hipSuccess) {
        cq_weight_destroy(w);
        *out = nullptr;
        return cq_set_error(CQ_ERR_HIP, "weight upload failed: %s", hipGetErrorString(e));
    }
    return CQ_OK;
}

// QCudaStorage::zeros / load_quantized know an element count only (cuda.rs:368-381, :591-612): the storage is
// a flat run of blocks, and any [n, k] with n * k elements and k a multiple of the block size is a way of
// reading it (the planes are ordered by flat block index).  Until a shape is given it reads as one block per row.
extern "C" int cq_weight_zeros_flat(int dev, int dt, int64_t elem_count, cq_weight **out) {
    const int64_t bs = cq_block_size(dt);
    if (!out) return cq_set_error(CQ_ERR_INVALID, "out is null");
    *out = nullptr;
    if (bs == 0 || !is_weight_dtype(dt)) return cq_set_error(CQ_ERR_UNSUPPORTED, "unsupported weight dtype %d", dt);
    if (elem_count < 0 || elem_count % bs != 0)
        return cq_set_error(CQ_ERR_INVALID, "element count %lld is not a multiple of the block size %lld",
                            (long long)elem_count, (long long)bs);
    return cq_weight_zeros(dev, dt, elem_count / bs, bs, out);
}

extern "C" int cq_weight_create_flat(int dev, int dt, const void *host_blocks, size_t nbytes, cq_weight **out) {
    const int64_t bs = cq_block_size(dt), ts = cq_type_size(dt);
    if (!out) return cq_set_error(CQ_ERR_INVALID, "out is null");
    *out = nullptr;
    if (bs == 0 || !is_weight_dtype(dt)) return cq_set_error(CQ_ERR_UNSUPPORTED, "unsupported weight dtype %d", dt);
    if (nbytes % (size_t)ts != 0)
        return cq_set_error(CQ_ERR_INVALID, "%zu bytes are not a whole number of %lld-byte blocks", nbytes, (long long)ts);
    return cq_weight_create(dev, dt, host_blocks, nbytes, (int64_t)(nbytes / (size_t)ts), bs, out);
}

// check_shape (mod.rs:304-316) plus the element count of the storage
static int check_view_shape(const cq_weight *w, int64_t n, int64_t k) {
    if (!w) return cq_set_error(CQ_ERR_INVALID, "null weight");
    const int64_t bs = cq_block_size(w->dtype);
    if (n < 0 || k < 0) return cq_set_error(CQ_ERR_INVALID, "negative shape [%lld, %lld]", (long long)n, (long long)k);
    if (k % bs != 0)
        return cq_set_error(CQ_ERR_INVALID,
                            "quantized tensor must have their last dim divisible by block size [%lld, %lld] %lld",
                            (long long)n, (long long)k, (long long)bs);
    if (n * k != w->n * w->k)
        return cq_set_error(CQ_ERR_INVALID, "shape [%lld, %lld] does not cover the %lld elements of the storage",
                            (long long)n, (long long)k, (long long)(w->n * w->k));
    return CQ_OK;
}

extern "C" int64_t cq_weight_elem_count(const cq_weight *w) { return w ? w->n * w->k : 0; }

extern "C" int cq_weight_set_shape(cq_weight *w, int64_t n, int64_t k) {
    if (int rc = check_view_shape(w, n, k)) return rc;
    w->n = n;
    w->k = k;
    return CQ_OK;
}

extern "C" int cq_weight_quantize(cq_weight *w, const float *src_dev, void *stream) {
    if (!w || !src_dev) return cq_set_error(CQ_ERR_INVALID, "null argument");
    if (w->ggml_bytes == 0) return CQ_OK;
    CQ_HIP_CHECK(hipSetDevice(w->dev));
    hipStream_t s = (hipStream_t)stream;
    void *tmp = nullptr;
    CQ_HIP_CHECK(hipMalloc(&tmp, w->ggml_bytes + 256));
    const int64_t nb = w->n * (w->k / cq_block_size(w->dtype));
    hipError_t e = cq_launch_quantize_weight(w->ggml_dtype, src_dev, nb, (uint8_t *)tmp, s);
    if (e == hipSuccess) e = blocks_to_planes(w, (uint8_t *)tmp, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);  // the temporary is freed below
    (void)hipFree(tmp);
    if (e != hipSuccess) return cq_set_error(CQ_ERR_HIP, "weight quantize failed: %s", hipGetErrorString(e));
    return CQ_OK;
}

extern "C" int cq_weight_dequantize(const cq_weight *w, float *dst_dev, void *stream) {
    if (!w || !dst_dev) return cq_set_error(CQ_ERR_INVALID, "null argument");
    if ((uintptr_t)dst_dev & 15) return cq_set_error(CQ_ERR_INVALID, "dst must be 16-byte aligned");
    CQ_HIP_CHECK(hipSetDevice(w->dev));
    CQ_HIP_CHECK(cq_launch_dequantize(w, dst_dev, nullptr, (hipStream_t)stream));
    return CQ_OK;
}

extern "C" int cq_weight_dequantize_f16(const cq_weight *w, uint16_t *dst_dev, void *stream) {
    if (!w || !dst_dev) return cq_set_error(CQ_ERR_INVALID, "null argument");
    if ((uintptr_t)dst_dev & 15) return cq_set_error(CQ_ERR_INVALID, "dst must be 16-byte aligned");
    CQ_HIP_CHECK(hipSetDevice(w->dev));
    CQ_HIP_CHECK(cq_launch_dequantize(w, nullptr, dst_dev, (hipStream_t)stream));
    return CQ_OK;
}

extern "C" int cq_weight_to_ggml(const cq_weight *w, void *host_dst, size_t nbytes) {
    if (!w || (!host_dst && nbytes)) return cq_set_error(CQ_ERR_INVALID, "null argument");
    if (nbytes != w->ggml_bytes)
        return cq_set_error(CQ_ERR_INVALID, "expected a %zu-byte destination, got %zu", w->ggml_bytes, nbytes);
    if (nbytes == 0) return CQ_OK;
    CQ_HIP_CHECK(hipSetDevice(w->dev));
    void *tmp = nullptr;
    CQ_HIP_CHECK(hipMalloc(&tmp, nbytes + 256));
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = planes_to_blocks(w, (uint8_t *)tmp, nullptr);
    if (e == hipSuccess) e = hipMemcpy(host_dst, tmp, nbytes, hipMemcpyDeviceToHost);
    (void)hipFree(tmp);
    if (e != hipSuccess) return cq_set_error(CQ_ERR_HIP, "weight download failed: %s", hipGetErrorString(e));
    return CQ_OK;
}

extern "C" size_t cq_weight_size_in_bytes(const cq_weight *w) { return w ? w->ggml_bytes : 0; }
extern "C" int cq_weight_dtype(const cq_weight *w) { return w ? w->ggml_dtype : -1; }
extern "C" int cq_weight_device(const cq_weight *w) { return w ? w->dev : -1; }
extern "C" int cq_weight_shape(const cq_weight *w, int64_t *n, int64_t *k) {
    if (!w) return cq_set_error(CQ_ERR_INVALID, "null weight");
    if (n) *n = w->n;
    if (k) *k = w->k;
    return CQ_OK;
}

extern "C" void cq_weight_destroy(cq_weight *w) {
    if (!w) return;
    if (w->base) {
        (void)hipSetDevice(w->dev);
        (void)hipFree(w->base);
    }
    delete w;
}

// ----------------------------------------------------------- activations ----
static bool is_act_dtype(int dt) { return dt == CQ_DTYPE_Q8_0 || dt == CQ_DTYPE_Q8_1 || dt == CQ_DTYPE_Q8K; }

extern "C" size_t cq_act_bytes(int act_dtype, int64_t m, int64_t k) {
    if (!is_act_dtype(act_dtype) || m < 0 || k < 0 || k % cq_block_size(act_dtype) != 0) return 0;
    return (size_t)(m * (k / cq_block_size(act_dtype))) * (size_t)cq_type_size(act_dtype);
}

// Checks the description of a fused step; a null aux or an unknown kind is the caller's error.
static int check_pre(const cq_pre &pre) {
    if (pre.kind == CQ_PRE_NONE) return CQ_OK;
    if (pre.kind != CQ_PRE_RMS_NORM && pre.kind != CQ_PRE_SILU_MUL)
        return cq_set_error(CQ_ERR_INVALID, "unknown fused step %d", pre.kind);
    if (!pre.aux) return cq_set_error(CQ_ERR_INVALID, "null argument");
    if ((uintptr_t)pre.aux & 15) return cq_set_error(CQ_ERR_INVALID, "aux must be 16-byte aligned");
    return CQ_OK;
}

static int quantize_act_impl(int dev, int act_dtype, const float *x_dev, int64_t m, int64_t k, cq_pre pre, void *dst,
                             void *stream) {
    if (!is_act_dtype(act_dtype)) return cq_set_error(CQ_ERR_UNSUPPORTED, "unsupported activation dtype %d", act_dtype);
    if (m < 0 || k < 0) return cq_set_error(CQ_ERR_INVALID, "negative shape");
    if (k % cq_block_size(act_dtype) != 0)
        return cq_set_error(CQ_ERR_INVALID, "%lld is not divisible by %lld", (long long)k,
                            (long long)cq_block_size(act_dtype));
    if (m == 0 || k == 0) return CQ_OK;
    if (!x_dev || !dst) return cq_set_error(CQ_ERR_INVALID, "null argument");
    if (((uintptr_t)x_dev & 15) || ((uintptr_t)dst & 3))
        return cq_set_error(CQ_ERR_INVALID, "x must be 16-byte aligned and dst 4-byte aligned");
    if (int rc = check_pre(pre)) return rc;
    CQ_HIP_CHECK(hipSetDevice(dev));
    CQ_HIP_CHECK(cq_launch_quantize_act_aos(act_dtype, x_dev, m, k, pre, dst, (hipStream_t)stream));
    return CQ_OK;
}

extern "C" int cq_quantize_act(int dev, int act_dtype, const float *x_dev, int64_t m, int64_t k, void *dst,
                               void *stream) {
    return quantize_act_impl(dev, act_dtype, x_dev, m, k, cq_no_pre(), dst, stream);
}

extern "C" int cq_quantize_act_fused(int dev, int act_dtype, int pre, const float *x_dev, const float *aux_dev,
                                     float eps, int64_t m, int64_t k, void *dst, void *stream) {
    return quantize_act_impl(dev, act_dtype, x_dev, m, k, cq_pre{pre, aux_dev, eps}, dst, stream);
}

// Workspace layout for m rows of K elements (see cq_act_view).
static size_t act_ws_layout(int act_dtype, int64_t m, int64_t k, uint8_t *base, cq_act_view *v) {
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t o = off; off = cq_align_up(off + bytes, 256); return o; };
    // Q8K rows are padded (see cq_act_view::m_stride); the others to whole 32-row groups, which the
    // split-K MFMA kernel copies without looking at the row count
    // (beyond 32 rows to whole 128-row tiles, which the 32-element-block tile kernel reads, scales included)
    const int64_t m_pad = act_dtype == CQ_DTYPE_Q8K ? (m + 63) / 64 * 64 + 256 : m <= 32 ? (m + 31) / 32 * 32 : (m + 127) / 128 * 128;
    const size_t o_qs = take((size_t)(m_pad * k));
    cq_act_view view{};
    view.m_stride = m_pad;
    if (act_dtype == CQ_DTYPE_Q8K) {
        const size_t o_d = take((size_t)(m * (k / 256)) * 4);
        const size_t o_bs = take((size_t)(m * (k / 256)) * 32);
        const size_t o_dt = take((size_t)(m_pad * (k / 256)) * 4);
        const size_t o_bh = take((size_t)(m_pad * (k / 256)) * 32);
        if (base) {
            view.qs = (int8_t *)(base + o_qs); view.d = (float *)(base + o_d);
            view.bsums = (int16_t *)(base + o_bs); view.dT = (float *)(base + o_dt);
            view.bsh = (uint16_t *)(base + o_bh);
        }
    } else {
        const size_t o_d = take((size_t)(m_pad * (k / 32)) * 4);
        const size_t o_s = take((size_t)(m * (k / 32)) * 4);
        const size_t o_h = take((size_t)(m_pad * (k / 32)) * 2);   // padded: the Q8_1 tile kernel copies whole tiles
        if (base) {
            view.qs = (int8_t *)(base + o_qs); view.d = (float *)(base + o_d);
            view.bsum32 = (int32_t *)(base + o_s); view.s16 = (uint16_t *)(base + o_h);
        }
    }
    if (v) *v = view;
    return off;
}

static int act_dtype_for(const cq_weight *w, int flags) {
    int a = cq_vec_dot_type(w->dtype);
    if ((flags & CQ_FLAG_ACT_Q8_1) && (w->ggml_dtype == CQ_DTYPE_Q4K || w->ggml_dtype == CQ_DTYPE_Q6K)) a = CQ_DTYPE_Q8_1;
    return a;
}

extern "C" size_t cq_workspace_bytes(const cq_weight *w, int64_t m, int flags) {
    if (!w || m <= 0) return 0;
    return act_ws_layout(act_dtype_for(w, flags), m, w->k, nullptr, nullptr);
}

// candle's vec_dot of these three types refuses rows with an odd number of blocks (k_quants.rs:273, 363, 469)
static int check_vec_dot_rows(const cq_weight *w) {
    if ((w->ggml_dtype == CQ_DTYPE_Q4_1 || w->ggml_dtype == CQ_DTYPE_Q5_0 || w->ggml_dtype == CQ_DTYPE_Q5_1) && (w->k / 32) % 2)
        return cq_set_error(CQ_ERR_INVALID, "vec_dot: %lld, nb is not divisible by 2", (long long)w->k);
    return CQ_OK;
}

static int check_matmul_args(const cq_weight *w, const float *x, int64_t m, const void *y, void *ws, size_t ws_bytes,
                             size_t need) {
    if (!w) return cq_set_error(CQ_ERR_INVALID, "null weight");
    if (m < 0) return cq_set_error(CQ_ERR_INVALID, "negative row count");
    if (m == 0 || w->n == 0) return CQ_OK;
    if (int rc = check_vec_dot_rows(w)) return rc;
    if (!x || !y) return cq_set_error(CQ_ERR_INVALID, "null argument");
    if ((uintptr_t)x & 15) return cq_set_error(CQ_ERR_INVALID, "x must be 16-byte aligned");
    if (!ws || ws_bytes < need)
        return cq_set_error(CQ_ERR_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, ws ? ws_bytes : (size_t)0);
    if ((uintptr_t)ws & 255) return cq_set_error(CQ_ERR_INVALID, "workspace must be 256-byte aligned");
    return CQ_OK;
}

// The quantizer may clear the matmul's output while it reads the activations only if the two do not
// overlap (a caller may well compute in place when the launches are separate) and y takes 16-byte stores.
static bool ranges_overlap(const float *a, int64_t na, const float *b, int64_t nb) {
    return a && b && (uintptr_t)a < (uintptr_t)(b + nb) && (uintptr_t)b < (uintptr_t)(a + na);
}
static bool clear_in_quantizer_ok(const float *y, int64_t ny, const float *x, int64_t nx, cq_pre pre) {
    if ((uintptr_t)y & 15) return false;
    if (ranges_overlap(y, ny, x, nx)) return false;
    // rms_norm: aux is one row of weights; silu_mul: aux has the shape of x
    if (pre.kind != CQ_PRE_NONE && ranges_overlap(y, ny, pre.aux, nx)) return false;
    return true;
}

static int qmatmul_impl(const cq_weight *w, const float *x_dev, cq_pre pre, int64_t m, float *y_dev, int flags,
                        void *ws, size_t ws_bytes, void *stream) {
    const NoSplitScope no_split(flags);
    flags &= ~CQ_FLAG_DETERMINISTIC;   // (only the tile kernels' launch plans look at it; every other kernel is deterministic as it is)
    const size_t need = cq_workspace_bytes(w, m, flags);
    int rc = check_matmul_args(w, x_dev, m, y_dev, ws, ws_bytes, need);
    if (rc || m == 0 || w->n == 0) return rc;
    if ((rc = check_pre(pre))) return rc;
    if (pre.kind != CQ_PRE_NONE && (flags & CQ_FLAG_REUSE_ACT))
        return cq_set_error(CQ_ERR_INVALID, "a fused step and a reused workspace exclude each other");
    if (w->k == 0) {
        CQ_HIP_CHECK(hipSetDevice(w->dev));
        CQ_HIP_CHECK(cq_launch_fill_zero(y_dev, m * w->n, (hipStream_t)stream));
        return CQ_OK;
    }
    const int act = act_dtype_for(w, flags);
    CQ_HIP_CHECK(hipSetDevice(w->dev));
    hipStream_t s = (hipStream_t)stream;
    if (w->dtype == CQ_DTYPE_Q8K) {
        // Q8K weights (a type of the reference's tests, not of checkpoints): the quantizer launch and one dot-product kernel
        if (flags & ~(CQ_FLAG_REUSE_ACT | CQ_FLAG_FORCE_MATVEC | CQ_FLAG_STAGED_ACT))
            return cq_set_error(CQ_ERR_UNSUPPORTED, "Q8K weights have a dot-product kernel only (flags %d)", flags);
        cq_act_view v;
        act_ws_layout(act, m, w->k, (uint8_t *)ws, &v);
        if (!(flags & CQ_FLAG_REUSE_ACT))
            CQ_HIP_CHECK(cq_launch_quantize_act_ws(act, x_dev, nullptr, m, w->k, pre, v, cq_no_clear(), s));
        CQ_HIP_CHECK(cq_launch_q8k_weight_matmul(w, v, m, y_dev, s));
        return CQ_OK;
    }
    if (flags & CQ_FLAG_ACT_Q8_1) {
        // the reference's CUDA formulation (cuda.rs:298-365): activations to Q8_1; a dot-product kernel up to 32 rows, the matrix cores beyond
        if (act != CQ_DTYPE_Q8_1 || !cq_matmul_q8_1_supported(w))
            return cq_set_error(CQ_ERR_UNSUPPORTED, "Q8_1 activations are for Q4K and Q6K weights with rows that fit the LDS (dtype %d, k = %lld)",
                                w->ggml_dtype, (long long)w->k);
        if (flags & ~(CQ_FLAG_ACT_Q8_1 | CQ_FLAG_REUSE_ACT))
            return cq_set_error(CQ_ERR_INVALID, "CQ_FLAG_ACT_Q8_1 combines with CQ_FLAG_REUSE_ACT only");
        cq_act_view v;
        act_ws_layout(act, m, w->k, (uint8_t *)ws, &v);
        if (!(flags & CQ_FLAG_REUSE_ACT))
            CQ_HIP_CHECK(cq_launch_quantize_act_ws(act, x_dev, nullptr, m, w->k, pre, v, cq_no_clear(), s));
        if (cq_gemm_q81_supported(w, m)) CQ_HIP_CHECK(cq_launch_gemm_q81(w, v, m, y_dev, s));   // matrix cores beyond 32 rows
        else CQ_HIP_CHECK(cq_launch_matmul_q8_1(w, v, m, y_dev, s));
        return CQ_OK;
    }
    // In the one-launch kernels every workgroup reads x (and aux) in its prologue while others already store y:
    // an output that overlaps an input goes through the quantizer launch instead, which has read all of x
    // before the matmul kernel writes anything.
    const bool in_place = ranges_overlap(y_dev, m * w->n, x_dev, m * w->k) ||
                          (pre.kind != CQ_PRE_NONE &&
                           ranges_overlap(y_dev, m * w->n, pre.aux, pre.kind == CQ_PRE_RMS_NORM ? w->k : m * w->k));
    // decode (one activation row): a single launch that quantizes x in its prologue
    // (Q4_1 / Q5_1 / Q2K: the one-launch kernels add the offset term themselves when no model step is fused in front;
    // otherwise a second launch adds it from the quantized rows in the workspace)
    const bool min32 = cq_has_min32(w->ggml_dtype) || cq_has_min16(w->ggml_dtype);   // (Q2K: likewise, its dmin term)
    if (m == 1 && !in_place && !(min32 && pre.kind != CQ_PRE_NONE) &&
        !(flags & (CQ_FLAG_REUSE_ACT | CQ_FLAG_FORCE_GEMM | CQ_FLAG_STAGED_ACT | CQ_FLAG_ACT_Q8_1)) &&
        cq_matvec_fused_supported(w)) {
        CQ_HIP_CHECK(cq_launch_matvec_fused(w, x_dev, pre, y_dev, s));
        return CQ_OK;
    }
    // Which kernel takes the rows.  Decided before the quantizer runs, because the quantizer clears the
    // output of a launch that splits K on its way.
    enum { kSkinny, kGemm32, kGemm, kMatvec } path;
    // Few rows: split K over the waves instead of tiling rows.  Measured (weights from HBM, 4096..32000 weight rows,
    // k 4096..14336) faster than the dot-product kernels from 2 rows on and than the tile kernels
    //   up to 16 rows everywhere; up to 24 rows below 14336 weight rows; up to 32 rows below 12288 weight rows;
    //   up to 64 rows where n is small and k short, so that the tile kernel cannot fill the machine.
    // (the 32-element-block types from 4 rows (Q8_0) or 5 rows (Q4_0) on: below that the one-launch dot-product
    // kernel is as fast or faster, it has no per-block scaling of MFMA results to do - where it takes the rows)
    const bool rows_fused = flags == 0 && pre.kind == CQ_PRE_NONE && !in_place && cq_matvec_fused_rows_supported(w, m);
    const int64_t skinny_from = w->dtype == CQ_DTYPE_Q8_0 ? 4 : w->dtype == CQ_DTYPE_Q4_0 ? 5 : 2;
    const bool has_tile_kernel = cq_gemm_supported(w, m, act);
    const bool has_tile32 = m > 16 && cq_gemm32_supported(w, act);
    const bool skinny_rows = m <= 16 || (m <= 24 && w->n < 14336) || (m <= 32 && w->n < 12288) ||
                             (m <= 64 && w->n < 8192 && w->k <= 6144);
    if (flags & CQ_FLAG_FORCE_SKINNY) {
        if (!cq_skinny_supported(w, act))
            return cq_set_error(CQ_ERR_UNSUPPORTED, "no split-K MFMA kernel for dtype %d with activation dtype %d and n = %lld",
                                w->dtype, act, (long long)w->n);
        path = kSkinny;
    } else if (!(flags & CQ_FLAG_FORCE_MATVEC) && has_tile32) {
        // Q8_0 / Q4_0 beyond 16 rows: their own tile kernel (whole 256-element K steps, n a multiple of 32), measured
        // ahead of the split-K kernel from 17 rows on at every shape
        path = kGemm32;
    } else if (!(flags & (CQ_FLAG_FORCE_GEMM | CQ_FLAG_FORCE_MATVEC)) && (m >= skinny_from || (m >= 2 && !rows_fused)) &&
               cq_skinny_supported(w, act) && (skinny_rows || !has_tile_kernel)) {
        // (shapes the tile kernels do not take: the split-K kernel, 32 rows per pass over the weights, stays
        // ahead of the dot-product kernel, 8 rows per pass, at every row count)
        path = kSkinny;
    } else {
        bool use_gemm = false;
        if (flags & CQ_FLAG_FORCE_GEMM) {
            if (!has_tile_kernel)
                return cq_set_error(CQ_ERR_UNSUPPORTED, "no MFMA GEMM for dtype %d with activation dtype %d", w->dtype, act);
            use_gemm = true;
        } else if (!(flags & CQ_FLAG_FORCE_MATVEC)) {
            use_gemm = m > 8 && has_tile_kernel;  // the reference switches kernels at 8 rows (cuda.rs:484-498)
        }
        if (act == CQ_DTYPE_Q8_1 && !use_gemm)
            return cq_set_error(CQ_ERR_UNSUPPORTED, "Q8_1 activations are only handled by the GEMM kernel");
        path = use_gemm ? kGemm : kMatvec;
    }
    // (rows whose quantized image does not fit the 160 KiB of LDS go through the dot-product kernel that walks them in
    // chunks: no limit on k, as in k_quants::matmul)
    // two to four rows of short enough weight rows: the one-launch kernel again, every unpacked weight unit
    // contracted with each activation row
    if (rows_fused) {
        CQ_HIP_CHECK(cq_launch_matvec_fused_rows(w, x_dev, m, y_dev, s));
        return CQ_OK;
    }
    cq_act_view v;
    act_ws_layout(act, m, w->k, (uint8_t *)ws, &v);
    bool y_cleared = false;
    if (!(flags & CQ_FLAG_REUSE_ACT)) {
        cq_clear clear = cq_no_clear();
        const bool splits = path == kGemm32 ? cq_gemm32_splits_k(w, m) : path == kGemm ? cq_gemm_splits_k(w, m) : false;
        if (splits && clear_in_quantizer_ok(y_dev, m * w->n, x_dev, m * w->k, pre)) {
            clear = cq_clear{y_dev, m * w->n};
            y_cleared = true;
        }
        CQ_HIP_CHECK(cq_launch_quantize_act_ws(act, x_dev, nullptr, m, w->k, pre, v, clear, s));
    }
    switch (path) {
        case kSkinny: CQ_HIP_CHECK(cq_launch_skinny(w, v, act, m, y_dev, s)); break;
        case kGemm32: CQ_HIP_CHECK(cq_launch_gemm32(w, v, act, m, y_dev, y_cleared, s)); break;
        case kGemm: CQ_HIP_CHECK(cq_launch_gemm(w, v, act, m, y_dev, y_cleared, s)); break;
        case kMatvec: CQ_HIP_CHECK(cq_launch_matvec(w, v, act, m, y_dev, s)); break;
    }
    if (cq_has_min32(w->ggml_dtype)) CQ_HIP_CHECK(cq_launch_min32_term(w, v, m, y_dev, s));
    if (cq_has_min16(w->ggml_dtype)) CQ_HIP_CHECK(cq_launch_min16_term(w, v, m, y_dev, s));
    return CQ_OK;
}

extern "C" int cq_qmatmul(const cq_weight *w, const float *x_dev, int64_t m, float *y_dev, int flags, void *ws,
                          size_t ws_bytes, void *stream) {
    return qmatmul_impl(w, x_dev, cq_no_pre(), m, y_dev, flags, ws, ws_bytes, stream);
}

extern "C" size_t cq_workspace_bytes_shaped(const cq_weight *w, int64_t n, int64_t k, int64_t m, int flags) {
    if (!w || m <= 0 || check_view_shape(w, n, k) != CQ_OK) return 0;
    return act_ws_layout(act_dtype_for(w, flags), m, k, nullptr, nullptr);
}

extern "C" int cq_qmatmul_shaped(const cq_weight *w, int64_t n, int64_t k, const float *x_dev, int64_t m, float *y_dev,
                                 int flags, void *ws, size_t ws_bytes, void *stream) {
    if (int rc = check_view_shape(w, n, k)) return rc;
    cq_weight view = *w;   // the kernels take the descriptor by value; nothing keeps a pointer to it
    view.n = n;
    view.k = k;
    return qmatmul_impl(&view, x_dev, cq_no_pre(), m, y_dev, flags, ws, ws_bytes, stream);
}

extern "C" int cq_qmatmul_fused(const cq_weight *w, int pre, const float *x_dev, const float *aux_dev, float eps,
                                int64_t m, float *y_dev, int flags, void *ws, size_t ws_bytes, void *stream) {
    return qmatmul_impl(w, x_dev, cq_pre{pre, aux_dev, eps}, m, y_dev, flags, ws, ws_bytes, stream);
}

extern "C" int cq_qmatmul_multi(const cq_weight *const *ws, int count, int pre, const float *x_dev, const float *aux_dev,
                                float eps, int64_t m, float *const *ys_dev, int flags, void *workspace, size_t ws_bytes,
                                void *stream) {
    if (!ws || !ys_dev || count < 1) return cq_set_error(CQ_ERR_INVALID, "null argument");
    for (int i = 0; i < count; i++) {
        if (!ws[i]) return cq_set_error(CQ_ERR_INVALID, "null weight %d", i);
        if (ws[i]->ggml_dtype != ws[0]->ggml_dtype || ws[i]->k != ws[0]->k || ws[i]->dev != ws[0]->dev)
            return cq_set_error(CQ_ERR_INVALID, "weight %d differs in dtype, row length or device from weight 0", i);
    }
    const cq_pre p{pre, aux_dev, eps};
    // every weight reads the same x (and aux): an output on top of them would be read back by the weights behind it
    for (int i = 0; i < count && m > 0; i++) {
        if (ranges_overlap(ys_dev[i], m * ws[i]->n, x_dev, m * ws[0]->k) ||
            (pre != CQ_PRE_NONE && ranges_overlap(ys_dev[i], m * ws[i]->n, aux_dev, pre == CQ_PRE_RMS_NORM ? ws[0]->k : m * ws[0]->k)))
            return cq_set_error(CQ_ERR_INVALID, "output %d overlaps the activations: cq_qmatmul_multi does not work in place", i);
    }
    const int det = flags & CQ_FLAG_DETERMINISTIC;
    flags &= ~CQ_FLAG_DETERMINISTIC;
    // one activation row (or up to four of short weight rows), two or three weights: one launch over all their rows
    if (m >= 1 && m <= 4 && flags == 0 && !cq_has_min32(ws[0]->ggml_dtype) && !cq_has_min16(ws[0]->ggml_dtype) &&
        cq_matvec_fused_multi_supported(ws, count, pre, m)) {
        for (int i = 0; i < count; i++)
            if (ws[i]->n > 0)
                if (int rc = check_vec_dot_rows(ws[i])) return rc;
        if (!x_dev) return cq_set_error(CQ_ERR_INVALID, "null argument");
        if ((uintptr_t)x_dev & 15) return cq_set_error(CQ_ERR_INVALID, "x must be 16-byte aligned");
        for (int i = 0; i < count; i++)
            if (!ys_dev[i]) return cq_set_error(CQ_ERR_INVALID, "null argument");
        if (int rc = check_pre(p)) return rc;
        CQ_HIP_CHECK(hipSetDevice(ws[0]->dev));
        CQ_HIP_CHECK(cq_launch_matvec_fused_multi(ws, count, x_dev, p, m, ys_dev, (hipStream_t)stream));
        return CQ_OK;
    }
    // otherwise one matmul per weight; with more than one row the rows are quantized once, by the first
    // (two to four rows that the one-launch kernel takes need no quantizer launch to share)
    const bool share = m > 1 && !(flags & CQ_FLAG_REUSE_ACT) &&
                       !(flags == 0 && pre == CQ_PRE_NONE && cq_matvec_fused_rows_supported(ws[0], m));
    for (int i = 0; i < count; i++) {
        const bool reuse = share && i > 0;
        if (int rc = qmatmul_impl(ws[i], x_dev, reuse ? cq_no_pre() : p, m, ys_dev[i], (reuse ? flags | CQ_FLAG_REUSE_ACT : flags) | det,
                                  workspace, ws_bytes, stream))
            return rc;
    }
    return CQ_OK;
}

extern "C" int cq_qmatmul_int_dots(const cq_weight *w, const float *x_dev, int64_t m, int32_t *out_i, int32_t *out_mn,
                                   void *ws, size_t ws_bytes, void *stream) {
    const size_t need = cq_workspace_bytes(w, m, 0);
    int rc = check_matmul_args(w, x_dev, m, out_i, ws, ws_bytes, need);
    if (rc || m == 0 || w->n == 0 || w->k == 0) return rc;
    const int act = cq_vec_dot_type(w->dtype);
    if (w->dtype == CQ_DTYPE_Q8K) return cq_set_error(CQ_ERR_UNSUPPORTED, "no integer dump for Q8K weights");
    if (!cq_matvec_row_fits(w)) return cq_set_error(CQ_ERR_UNSUPPORTED, "rows of %lld elements do not fit the LDS", (long long)w->k);
    CQ_HIP_CHECK(hipSetDevice(w->dev));
    hipStream_t s = (hipStream_t)stream;
    cq_act_view v;
    act_ws_layout(act, m, w->k, (uint8_t *)ws, &v);
    CQ_HIP_CHECK(cq_launch_quantize_act_ws(act, x_dev, nullptr, m, w->k, cq_no_pre(), v, cq_no_clear(), s));
    CQ_HIP_CHECK(cq_launch_int_dots(w, v, m, out_i, (w->dtype == CQ_DTYPE_Q4K || w->dtype == CQ_DTYPE_Q5K) ? out_mn : nullptr, s));
    return CQ_OK;
}

extern "C" int cq_qmatmul_int_dots_mfma(const cq_weight *w, const float *x_dev, int64_t m, int kernel, int32_t *out_i,
                                        float *out_mn, void *ws, size_t ws_bytes, void *stream) {
    const size_t need = cq_workspace_bytes(w, m, 0);
    int rc = check_matmul_args(w, x_dev, m, out_i, ws, ws_bytes, need);
    if (rc || m == 0 || w->n == 0 || w->k == 0) return rc;
    const int act = cq_vec_dot_type(w->dtype);
    const bool kquant = w->dtype == CQ_DTYPE_Q4K || w->dtype == CQ_DTYPE_Q5K || w->dtype == CQ_DTYPE_Q6K;
    const int int_min = kernel & CQ_MFMA_INT_MIN;
    kernel &= ~CQ_MFMA_INT_MIN;
    bool ok = false;
    if (kernel == CQ_MFMA_SKINNY) ok = cq_skinny_supported(w, act);
    else if (kernel == CQ_MFMA_TILE) ok = kquant ? cq_gemm_supported(w, m, act) : m > 16 && cq_gemm32_supported(w, act);   // as cq_qmatmul
    else return cq_set_error(CQ_ERR_INVALID, "kernel must be CQ_MFMA_SKINNY or CQ_MFMA_TILE (plus CQ_MFMA_INT_MIN)");
    if (!ok) return cq_set_error(CQ_ERR_UNSUPPORTED, "that kernel does not take this weight (dtype %d, %lld x %lld) with %lld rows", w->dtype,
                                 (long long)w->n, (long long)w->k, (long long)m);
    CQ_HIP_CHECK(hipSetDevice(w->dev));
    hipStream_t s = (hipStream_t)stream;
    cq_act_view v;
    act_ws_layout(act, m, w->k, (uint8_t *)ws, &v);
    CQ_HIP_CHECK(cq_launch_quantize_act_ws(act, x_dev, nullptr, m, w->k, cq_no_pre(), v, cq_no_clear(), s));
    const cq_mfma_dump d{out_i, (w->dtype == CQ_DTYPE_Q4K || w->dtype == CQ_DTYPE_Q5K) ? out_mn : nullptr, int_min};
    if (kernel == CQ_MFMA_SKINNY) CQ_HIP_CHECK(cq_launch_skinny_dump(w, v, act, m, d, s));
    else if (kquant) CQ_HIP_CHECK(cq_launch_gemm_dump(w, v, act, m, d, s));
    else CQ_HIP_CHECK(cq_launch_gemm32_dump(w, v, act, m, d, s));
    return CQ_OK;
}

// ------------------------------------------------------------------- MoE ----
extern "C" size_t cq_grouped_workspace_bytes(const cq_weight *const *experts, int n_experts, int64_t total_rows,
                                             int flags) {
    if (!experts || n_experts <= 0 || !experts[0] || total_rows <= 0) return 0;
    return act_ws_layout(act_dtype_for(experts[0], flags), total_rows, experts[0]->k, nullptr, nullptr);
}

static int grouped_impl(const cq_weight *const *experts, int n_experts, const float *x_dev, cq_pre pre,
                        const int32_t *row_ids_dev, const int32_t *offsets, float *y_dev, int flags, void *ws,
                        size_t ws_bytes, void *stream) {
    if (!experts || n_experts <= 0 || !offsets) return cq_set_error(CQ_ERR_INVALID, "null argument");
    const NoSplitScope no_split(flags);
    flags &= ~CQ_FLAG_DETERMINISTIC;
    const cq_weight *w0 = experts[0];
    if (!w0) return cq_set_error(CQ_ERR_INVALID, "null expert");
    for (int e = 0; e < n_experts; e++) {
        if (!experts[e]) return cq_set_error(CQ_ERR_INVALID, "null expert %d", e);
        if (experts[e]->ggml_dtype != w0->ggml_dtype || experts[e]->n != w0->n || experts[e]->k != w0->k || experts[e]->dev != w0->dev)
            return cq_set_error(CQ_ERR_INVALID, "expert %d differs in dtype, shape or device from expert 0", e);
        if (offsets[e + 1] < offsets[e]) return cq_set_error(CQ_ERR_INVALID, "offsets must be non-decreasing");
    }
    if (offsets[0] != 0) return cq_set_error(CQ_ERR_INVALID, "offsets[0] must be 0");
    const int64_t total = offsets[n_experts];
    const size_t need = cq_grouped_workspace_bytes(experts, n_experts, total, flags);
    int rc = check_matmul_args(w0, x_dev, total, y_dev, ws, ws_bytes, need);
    if (rc || total == 0 || w0->n == 0 || w0->k == 0) return rc;
    const int act = act_dtype_for(w0, flags);
    if (act == CQ_DTYPE_Q8_1) return cq_set_error(CQ_ERR_UNSUPPORTED, "grouped matmul takes the CPU formulation only");
    if (cq_has_min32(w0->ggml_dtype) || cq_has_min16(w0->ggml_dtype) || w0->dtype == CQ_DTYPE_Q8K)
        return cq_set_error(CQ_ERR_UNSUPPORTED, "grouped matmul does not take Q4_1 / Q5_1 / Q2K / Q8K experts (no grouped launch for them)");
    if ((rc = check_pre(pre))) return rc;
    // (the same routed rows against a second set of experts, w1 and w3 of quantized_llama.rs:60-61: the workspace of the
    // first grouped call holds them)
    const bool reuse = (flags & CQ_FLAG_REUSE_ACT) != 0;
    if (reuse && pre.kind != CQ_PRE_NONE)
        return cq_set_error(CQ_ERR_INVALID, "a fused step and a reused workspace exclude each other");
    CQ_HIP_CHECK(hipSetDevice(w0->dev));
    hipStream_t s = (hipStream_t)stream;
    cq_act_view v;
    act_ws_layout(act, total, w0->k, (uint8_t *)ws, &v);
    // experts with more than eight rows among them: one tile-kernel launch for all experts
    int64_t most = 0;
    for (int e = 0; e < n_experts; e++) most = offsets[e + 1] - offsets[e] > most ? offsets[e + 1] - offsets[e] : most;
    const bool want_gemm = (flags & CQ_FLAG_FORCE_GEMM) ? true : (flags & CQ_FLAG_FORCE_MATVEC) ? false : most > 8;
    const bool grouped = want_gemm && cq_gemm_grouped_supported(experts, n_experts, offsets, act);
    // gather + quantize every routed row once (clearing the output on the way if the grouped launch splits K;
    // with row ids the extent of x is not known here, so nothing is cleared then)
    cq_clear clear = cq_no_clear();
    if (!reuse && grouped && !row_ids_dev && cq_gemm_grouped_splits_k(experts, n_experts, offsets) &&
        clear_in_quantizer_ok(y_dev, total * w0->n, x_dev, total * w0->k, pre))
        clear = cq_clear{y_dev, total * w0->n};
    if (!reuse) CQ_HIP_CHECK(cq_launch_quantize_act_ws(act, x_dev, row_ids_dev, total, w0->k, pre, v, clear, s));
    if (grouped) {
        CQ_HIP_CHECK(cq_launch_gemm_grouped(experts, n_experts, offsets, v, y_dev, clear.p != nullptr, s));
        return CQ_OK;
    }
    // otherwise one matmul per non-empty expert over its slice
    for (int e = 0; e < n_experts; e++) {
        const int64_t r0 = offsets[e], te = offsets[e + 1] - offsets[e];
        if (te == 0) continue;
        cq_act_view ve = v;
        ve.qs += r0 * w0->k;
        if (act == CQ_DTYPE_Q8K) {
            ve.d += r0 * (w0->k / 256);
            ve.bsums += r0 * (w0->k / 256) * 16;
            ve.dT += r0;
            ve.bsh += r0 * 16;
        } else {
            ve.d += r0 * (w0->k / 32);
            ve.bsum32 += r0 * (w0->k / 32);
        }
        float *ye = y_dev + r0 * w0->n;
        const bool use_gemm = (flags & CQ_FLAG_FORCE_GEMM) ? true
                              : (flags & CQ_FLAG_FORCE_MATVEC) ? false
                                                               : (te > 8 && cq_gemm_supported(experts[e], te, act));
        if (use_gemm) CQ_HIP_CHECK(cq_launch_gemm(experts[e], ve, act, te, ye, false, s));
        else CQ_HIP_CHECK(cq_launch_matvec(experts[e], ve, act, te, ye, s));
    }
    return CQ_OK;
}

extern "C" int cq_qmatmul_grouped(const cq_weight *const *experts, int n_experts, const float *x_dev,
                                  const int32_t *row_ids_dev, const int32_t *offsets, float *y_dev, int flags,
                                  void *ws, size_t ws_bytes, void *stream) {
    return grouped_impl(experts, n_experts, x_dev, cq_no_pre(), row_ids_dev, offsets, y_dev, flags, ws, ws_bytes, stream);
}

extern "C" int cq_qmatmul_grouped_fused(const cq_weight *const *experts, int n_experts, int pre, const float *x_dev,
                                        const float *aux_dev, float eps, const int32_t *row_ids_dev,
                                        const int32_t *offsets, float *y_dev, int flags, void *ws, size_t ws_bytes,
                                        void *stream) {
    return grouped_impl(experts, n_experts, x_dev, cq_pre{pre, aux_dev, eps}, row_ids_dev, offsets, y_dev, flags, ws,
                        ws_bytes, stream);
}

extern "C" int cq_silu_mul(int dev, const float *a, const float *b, float *h, int64_t count, void *stream) {
    if (count < 0) return cq_set_error(CQ_ERR_INVALID, "negative count");
    if (count == 0) return CQ_OK;
    if (!a || !b || !h) return cq_set_error(CQ_ERR_INVALID, "null argument");
    CQ_HIP_CHECK(hipSetDevice(dev));
    CQ_HIP_CHECK(cq_launch_silu_mul(a, b, h, count, (hipStream_t)stream));
    return CQ_OK;
}

extern "C" int cq_moe_scatter_add(int dev, const float *y, const int32_t *row_ids, const float *weights,
                                  int64_t total_rows, int64_t hidden, float *ys, int64_t tokens, void *stream) {
    if (total_rows < 0 || hidden < 0 || tokens < 0) return cq_set_error(CQ_ERR_INVALID, "negative size");
    if (tokens == 0 || hidden == 0) return CQ_OK;
    if (!ys || (total_rows && (!y || !row_ids || !weights))) return cq_set_error(CQ_ERR_INVALID, "null argument");
    CQ_HIP_CHECK(hipSetDevice(dev));
    CQ_HIP_CHECK(cq_launch_scatter_add(y, row_ids, weights, total_rows, hidden, ys, tokens, (hipStream_t)stream));
    return CQ_OK;
}

extern "C" int cq_timing_arm(void) {
    if (!g_timer.start) {
        CQ_HIP_CHECK(hipEventCreate(&g_timer.start));
        CQ_HIP_CHECK(hipEventCreate(&g_timer.stop));
    }
    g_timer.armed = true;
    g_timer.pending = false;
    return CQ_OK;
}

extern "C" int cq_timing_elapsed_us(double *us) {
    if (!us) return cq_set_error(CQ_ERR_INVALID, "us is null");
    if (!g_timer.pending) return cq_set_error(CQ_ERR_INVALID, "no armed kernel launch to read");
    g_timer.pending = false;
    CQ_HIP_CHECK(hipEventSynchronize(g_timer.stop));
    float ms = 0.0f;
    CQ_HIP_CHECK(hipEventElapsedTime(&ms, g_timer.start, g_timer.stop));
    *us = (double)ms * 1e3;
    return CQ_OK;
}

// ---- hardware self-check of the quantizers' rounding instruction -------------------------------
namespace {
__global__ void selfcheck_round_kernel(uint32_t last_bits, unsigned long long *bad) {
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    unsigned long long mine = 0;
    for (unsigned long long b = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; b <= last_bits; b += stride) {
        const float t = __builtin_bit_cast(float, (uint32_t)b);
        // exact: t has 24 significant bits, so t + 0.5 is exact in double
        const int want = (int)floor((double)t + 0.5);
        if (cq_round_away_i32(t) != want) mine++;
        if (cq_round_away_i32(-t) != -want) mine++;
    }
    if (mine) atomicAdd(bad, mine);
}
}  // namespace

extern "C" int cq_selfcheck_round(int dev, uint64_t *mismatches) {
    if (!mismatches) return cq_set_error(CQ_ERR_INVALID, "mismatches is null");
    CQ_HIP_CHECK(hipSetDevice(dev));
    unsigned long long *bad = nullptr;
    CQ_HIP_CHECK(hipMalloc((void **)&bad, sizeof(*bad)));
    hipError_t e = hipMemset(bad, 0, sizeof(*bad));
    if (e == hipSuccess) {
        hipLaunchKernelGGL(selfcheck_round_kernel, dim3(4096), dim3(256), 0, 0, 0x43020000u /* 130.0f */, bad);
        e = hipGetLastError();
    }
    unsigned long long host = 0;
    if (e == hipSuccess) e = hipMemcpy(&host, bad, sizeof(host), hipMemcpyDeviceToHost);
    (void)hipFree(bad);
    CQ_HIP_CHECK(e);
    *mismatches = host;
    return CQ_OK;
}
