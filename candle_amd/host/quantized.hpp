// C++ host side of the quantized-matmul path: the reference's `candle_core::quantized` surface
// (GgmlDType, QStorage's device arm, QTensor, QMatMul) over the C ABI of libcandle_qhip.so.
//
// The reference is Rust; names, argument meaning and error behaviour follow it so that a
// `quantized/hip.rs` can be written from this file line by line:
//   GgmlDType          candle-core/src/quantized/mod.rs:133-247
//   QHipStorage        the device arm of QStorage, as QCudaStorage in quantized/cuda.rs:367-500
//   QTensor            mod.rs:35-38, 318-392
//   QMatMul            mod.rs:394-462, 527-550 (forward)
// Errors are C++ exceptions of type candle_hip::Error (the reference returns Result and never
// panics on user error); nothing here aborts.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <memory>
#include <numeric>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/candle_qhip.h"

namespace candle_hip {

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline void check(int rc, const char *what) {
    if (rc != CQ_OK) throw Error(std::string(what) + ": " + cq_last_error());
}
inline void check_hip(hipError_t e, const char *what) {
    if (e != hipSuccess) throw Error(std::string(what) + ": " + hipGetErrorString(e));
}

// ---- GgmlDType (mod.rs:133-247) --------------------------------------------------------------
enum class GgmlDType : uint32_t { Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q8_1 = 9, Q2K = 10, Q3K = 11, Q4K = 12, Q5K = 13, Q6K = 14, Q8K = 15 };

inline GgmlDType ggml_dtype_from_u32(uint32_t u) {   // mod.rs:152-171
    switch (u) {
        case 2: case 3: case 6: case 7: case 8: case 9: case 10: case 11: case 12: case 13: case 14: case 15: return static_cast<GgmlDType>(u);
        default: throw Error("unknown or unsupported dtype for ggml: " + std::to_string(u));
    }
}
inline uint32_t to_u32(GgmlDType d) { return static_cast<uint32_t>(d); }                   // mod.rs:173-190
inline size_t block_size(GgmlDType d) { return (size_t)cq_block_size((int)to_u32(d)); }    // mod.rs:234-246
inline size_t type_size(GgmlDType d) { return (size_t)cq_type_size((int)to_u32(d)); }      // mod.rs:212-232

using Shape = std::vector<int64_t>;
inline int64_t elem_count(const Shape &s) {
    return std::accumulate(s.begin(), s.end(), (int64_t)1, [](int64_t a, int64_t b) { return a * b; });
}
inline std::string to_string(const Shape &s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? ", " : "") + std::to_string(s[i]);
    return r + "]";
}

// ---- a contiguous f32 device tensor: the only dense tensor the path needs ----------------------
template <typename T> class DeviceBuffer {
  public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(size_t count) : count_(count) {
        if (count) check_hip(hipMalloc((void **)&ptr_, count * sizeof(T)), "hipMalloc");
    }
    ~DeviceBuffer() { if (ptr_) (void)hipFree(ptr_); }
    DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), count_(o.count_) { o.ptr_ = nullptr; o.count_ = 0; }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
        if (this != &o) { if (ptr_) (void)hipFree(ptr_); ptr_ = o.ptr_; count_ = o.count_; o.ptr_ = nullptr; o.count_ = 0; }
        return *this;
    }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    T *get() const { return ptr_; }
    size_t size() const { return count_; }

  private:
    T *ptr_ = nullptr;
    size_t count_ = 0;
};

struct Tensor {
    Shape shape;
    DeviceBuffer<float> data;

    static Tensor from_host(const std::vector<float> &v, Shape shape) {
        if ((int64_t)v.size() != elem_count(shape)) throw Error("shape mismatch in Tensor::from_host");
        Tensor t{std::move(shape), DeviceBuffer<float>(v.size())};
        if (!v.empty()) check_hip(hipMemcpy(t.data.get(), v.data(), v.size() * 4, hipMemcpyHostToDevice), "hipMemcpy");
        return t;
    }
    std::vector<float> to_host() const {
        std::vector<float> v((size_t)elem_count(shape));
        check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize");
        if (!v.empty()) check_hip(hipMemcpy(v.data(), data.get(), v.size() * 4, hipMemcpyDeviceToHost), "hipMemcpy");
        return v;
    }
    size_t rank() const { return shape.size(); }
};

// ---- QHipStorage: what QCudaStorage offers (cuda.rs:367-500) ----------------------------------
class QHipStorage {
  public:
    // cuda.rs:368-381 `zeros(device, elem_count, dtype)`: the storage knows an element count, no shape
    static QHipStorage zeros(int device, int64_t elem_count, GgmlDType dtype) {
        cq_weight *w = nullptr;
        check(cq_weight_zeros_flat(device, (int)to_u32(dtype), elem_count, &w), "QHipStorage::zeros");
        return QHipStorage(w);
    }
    // cuda.rs:591-612 `load_quantized(device, data: &[T])`: host GGML blocks -> device, re-packed on upload
    static QHipStorage load_quantized(int device, GgmlDType dtype, const void *blocks, size_t nbytes) {
        cq_weight *w = nullptr;
        check(cq_weight_create_flat(device, (int)to_u32(dtype), blocks, nbytes, &w), "load_quantized");
        return QHipStorage(w);
    }
    ~QHipStorage() { if (w_) cq_weight_destroy(w_); }
    QHipStorage(QHipStorage &&o) noexcept : w_(o.w_) { o.w_ = nullptr; }
    QHipStorage &operator=(QHipStorage &&o) noexcept {
        if (this != &o) { if (w_) cq_weight_destroy(w_); w_ = o.w_; o.w_ = nullptr; }
        return *this;
    }
    QHipStorage(const QHipStorage &) = delete;
    QHipStorage &operator=(const QHipStorage &) = delete;

    GgmlDType dtype() const { return ggml_dtype_from_u32((uint32_t)cq_weight_dtype(w_)); }   // cuda.rs:382-384
    int device() const { return cq_weight_device(w_); }                                       // cuda.rs:386-388
    size_t storage_size_in_bytes() const { return cq_weight_size_in_bytes(w_); }              // cuda.rs:474-476
    int64_t elem_count() const { return cq_weight_elem_count(w_); }
    // The [n, k] the entry points without a shape argument read the storage as (QTensor::new fixes it).
    std::pair<int64_t, int64_t> dims() const {
        int64_t n = 0, k = 0;
        check(cq_weight_shape(w_, &n, &k), "QHipStorage::dims");
        return {n, k};
    }
    // (state of the handle: a set-up call, not concurrent with any use of the storage; QTensor owns its storage, so no
    // two tensors can fix different shapes on one handle)
    void set_dims(int64_t n, int64_t k) { check(cq_weight_set_shape(w_, n, k), "QHipStorage::set_dims"); }
    // cuda.rs:390-446
    Tensor dequantize(const Shape &shape, hipStream_t stream = nullptr) const {
        Tensor t{shape, DeviceBuffer<float>((size_t)candle_hip::elem_count(shape))};
        check(cq_weight_dequantize(w_, t.data.get(), stream), "QHipStorage::dequantize");
        return t;
    }
    // cuda.rs:448-472: f32 source on the same device; quantized on the device
    void quantize(const Tensor &src, hipStream_t stream = nullptr) {
        if (candle_hip::elem_count(src.shape) != elem_count()) throw Error("QHipStorage::quantize: size mismatch");
        check(cq_weight_quantize(w_, src.data.get(), stream), "QHipStorage::quantize");
    }
    std::vector<uint8_t> data() const {   // host GGML blocks (inverse re-pack)
        std::vector<uint8_t> out(storage_size_in_bytes());
        check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize");
        check(cq_weight_to_ggml(w_, out.data(), out.size()), "QHipStorage::data");
        return out;
    }
    // cuda.rs:478-499 `fwd(self_shape, storage, layout)`: x contiguous f32, rank 2 or 3 (any rank >= 2
    // here, as on the CPU), last dim == k; the result owns a fresh allocation.
    // `pre` != CQ_PRE_NONE: the model step in front of the projection computed inside the same
    // launches: rms_norm with alpha = *aux (candle-nn/src/ops.rs:641-652), or silu(x) * *aux
    // (quantized_llama.rs:60-62).
    Tensor fwd(const Shape &self_shape, const Tensor &x, hipStream_t stream = nullptr, int pre = CQ_PRE_NONE,
               const Tensor *aux = nullptr, float eps = 0.0f) const {
        if (self_shape.size() != 2) throw Error("QHipStorage::fwd: weight must be rank 2, got " + to_string(self_shape));
        const int64_t n = self_shape[0], k = self_shape[1];
        if (x.rank() < 2) throw Error("input tensor has only one dimension " + to_string(x.shape));       // mod.rs:480-482
        if (x.shape.back() != k)
            throw Error("input tensor " + to_string(x.shape) + " incompatible with " + to_string(self_shape));  // mod.rs:485-487
        if (pre == CQ_PRE_RMS_NORM && (!aux || aux->shape != Shape{k}))
            throw Error("shape mismatch in rms-norm " + to_string(x.shape) + " " + (aux ? to_string(aux->shape) : "none"));  // ops.rs:644-650
        if (pre == CQ_PRE_SILU_MUL && (!aux || aux->shape != x.shape))
            throw Error("shape mismatch in silu-mul " + to_string(x.shape) + " " + (aux ? to_string(aux->shape) : "none"));
        const int64_t m = k ? candle_hip::elem_count(x.shape) / k : 0;
        Shape out_shape = x.shape;
        out_shape.back() = n;
        Tensor y{out_shape, DeviceBuffer<float>((size_t)(m * n))};
        // the shape arrives with the call, as in the reference: the storage is read as [n, k] for this launch
        const size_t ws_bytes = cq_workspace_bytes_shaped(w_, n, k, m, CQ_FLAG_AUTO);
        if (m > 0 && n * k != elem_count()) throw Error("QHipStorage::fwd: " + to_string(self_shape) + " does not cover the storage");
        DeviceBuffer<uint8_t> ws(ws_bytes);   // per call, like the reference's quantized-activation buffer (cuda.rs:249-252)
        if (pre == CQ_PRE_NONE) {
            check(cq_qmatmul_shaped(w_, n, k, x.data.get(), m, y.data.get(), CQ_FLAG_AUTO, ws.get(), ws_bytes, stream),
                  "QHipStorage::fwd");
        } else {
            // the fused entry points read the shape QTensor::new fixed
            if (dims() != std::pair<int64_t, int64_t>{n, k}) throw Error("QHipStorage::fwd: fused steps need the tensor's own shape");
            check(cq_qmatmul_fused(w_, pre, x.data.get(), aux->data.get(), eps, m, y.data.get(), CQ_FLAG_AUTO, ws.get(),
                                   ws_bytes, stream), "QHipStorage::fwd");
        }
        // the workspace is freed when this returns; hipFree waits for the device, as dropping a
        // CudaSlice synchronises with its stream
        return y;
    }
    const cq_weight *raw() const { return w_; }

  private:
    explicit QHipStorage(cq_weight *w) : w_(w) {}
    cq_weight *w_ = nullptr;
};

// ---- QTensor (mod.rs:35-38, 318-392) ---------------------------------------------------------
inline void check_shape(const Shape &shape, size_t block) {   // mod.rs:304-316
    if (shape.empty()) throw Error("scalar tensor cannot be quantized " + to_string(shape));
    if (shape.back() % (int64_t)block != 0)
        throw Error("quantized tensor must have their last dim divisible by block size " + to_string(shape) + " " +
                    std::to_string(block));
}

class QTensor {
  public:
    QTensor(QHipStorage storage, Shape shape) : storage_(std::move(storage)), shape_(std::move(shape)) {
        check_shape(shape_, block_size(storage_.dtype()));                                   // mod.rs:319-323 `new`
        const int64_t k = shape_.back();
        storage_.set_dims(k ? elem_count(shape_) / k : 0, k);   // leading dims flattened into rows
    }
    // mod.rs:325-343
    static QTensor quantize(const Tensor &src, GgmlDType dtype, int device = 0) {
        check_shape(src.shape, block_size(dtype));
        QHipStorage s = QHipStorage::zeros(device, elem_count(src.shape), dtype);   // Device::qzeros, mod.rs:40-57
        s.quantize(src);
        return QTensor(std::move(s), src.shape);
    }
    GgmlDType dtype() const { return storage_.dtype(); }                 // mod.rs:345-347
    size_t rank() const { return shape_.size(); }                        // mod.rs:353-355
    const Shape &shape() const { return shape_; }                        // mod.rs:357-359
    Tensor dequantize() const { return storage_.dequantize(shape_); }    // mod.rs:361-365
    size_t storage_size_in_bytes() const { return storage_.storage_size_in_bytes(); }   // mod.rs:384-386
    std::vector<uint8_t> data() const { return storage_.data(); }        // mod.rs:388-391
    const QHipStorage &storage() const { return storage_; }

  private:
    QHipStorage storage_;
    Shape shape_;
};

// ---- QMatMul (mod.rs:394-462; forward :527-550) -------------------------------------------------
class QMatMul {
  public:
    static QMatMul from_arc(std::shared_ptr<QTensor> qtensor) { return QMatMul(std::move(qtensor)); }   // mod.rs:423-438
    static QMatMul from_qtensor(QTensor qtensor) {                                                      // mod.rs:440-442
        return QMatMul(std::make_shared<QTensor>(std::move(qtensor)));
    }
    // y = xs . W^T; xs [.., k] -> [.., n]
    Tensor forward(const Tensor &xs, hipStream_t stream = nullptr) const {
        return qtensor_->storage().fwd(qtensor_->shape(), xs, stream);
    }
    // forward(rms_norm(xs, alpha, eps)): RmsNorm::forward (candle-transformers/src/quantized_nn.rs:121-125)
    // in front of a projection (quantized_llama.rs:453-466), without the normalised tensor in memory
    Tensor forward_rms_norm(const Tensor &xs, const Tensor &alpha, float eps, hipStream_t stream = nullptr) const {
        return qtensor_->storage().fwd(qtensor_->shape(), xs, stream, CQ_PRE_RMS_NORM, &alpha, eps);
    }
    // forward(silu(gate) * up): the feed-forward's w2 (Mlp::forward, quantized_llama.rs:56-63)
    Tensor forward_silu_mul(const Tensor &gate, const Tensor &up, hipStream_t stream = nullptr) const {
        return qtensor_->storage().fwd(qtensor_->shape(), gate, stream, CQ_PRE_SILU_MUL, &up);
    }
    // {m.forward(xs) for m in mats} (with alpha: of rms_norm(xs, alpha, eps)) for matrices of one dtype and row
    // length, as q, k, v (quantized_llama.rs:206-208) or w1, w3 (:60-61): one launch for one activation row,
    // the rows quantized once otherwise
    static std::vector<Tensor> forward_multi(const std::vector<const QMatMul *> &mats, const Tensor &xs,
                                             const Tensor *alpha = nullptr, float eps = 0.0f, hipStream_t stream = nullptr) {
        if (mats.empty()) throw Error("forward_multi: no matrices");
        const int64_t k = mats[0]->qtensor_->shape().back();
        if (xs.rank() < 2) throw Error("input tensor has only one dimension " + to_string(xs.shape));
        if (alpha && alpha->shape != Shape{k})
            throw Error("shape mismatch in rms-norm " + to_string(xs.shape) + " " + to_string(alpha->shape));
        const int64_t m = k ? elem_count(xs.shape) / k : 0;
        std::vector<const cq_weight *> ws;
        std::vector<Tensor> ys;
        std::vector<float *> yp;
        size_t ws_bytes = 0;
        for (const QMatMul *mm : mats) {
            const Shape &sh = mm->qtensor_->shape();
            if (sh.size() != 2 || xs.shape.back() != sh[1])
                throw Error("input tensor " + to_string(xs.shape) + " incompatible with " + to_string(sh));
            Shape out_shape = xs.shape;
            out_shape.back() = sh[0];
            ys.push_back(Tensor{out_shape, DeviceBuffer<float>((size_t)(m * sh[0]))});
            yp.push_back(ys.back().data.get());
            ws.push_back(mm->qtensor_->storage().raw());
            ws_bytes = std::max(ws_bytes, cq_workspace_bytes(ws.back(), m, CQ_FLAG_AUTO));
        }
        DeviceBuffer<uint8_t> wsp(ws_bytes);
        check(cq_qmatmul_multi(ws.data(), (int)ws.size(), alpha ? CQ_PRE_RMS_NORM : CQ_PRE_NONE, xs.data.get(),
                               alpha ? alpha->data.get() : nullptr, eps, m, yp.data(), CQ_FLAG_AUTO, wsp.get(), ws_bytes,
                               stream), "QMatMul::forward_multi");
        return ys;
    }
    const QTensor &qtensor() const { return *qtensor_; }

  private:
    explicit QMatMul(std::shared_ptr<QTensor> q) : qtensor_(std::move(q)) {}
    std::shared_ptr<QTensor> qtensor_;
};

}  // namespace candle_hip
