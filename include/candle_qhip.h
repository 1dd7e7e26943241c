/*
 * candle_qhip.h - C ABI of the MI355X (gfx950) quantized-matmul library.
 *
 * This is the boundary a `Hip` arm of candle's `QStorage` enum binds to: each
 * entry point names the reference interface it replaces (paths relative to the
 * candle repository).  Plain pointers and sizes only; every function returns 0
 * on success or a negative code and leaves a message for cq_last_error().
 *
 * Conventions
 *  - dtype ids are GgmlDType::to_u32 (candle-core/src/quantized/mod.rs:173-190).
 *  - weights are logical [n, k] row-major, row = k/block consecutive blocks
 *    (k_quants.rs:1875); activations [m, k] contiguous f32; outputs [m, n] f32.
 *  - pointers named *_dev are device pointers on the weight's device; work is
 *    enqueued on `stream` (a hipStream_t, NULL = default stream) with no host
 *    synchronisation, like the reference's CUDA arm (cuda.rs:478-499).
 *  - the device layout of a cq_weight is private (re-packed planes), as
 *    QStorage::data() is "not implemented" for device arms (mod.rs:126-128).
 *  - aliasing: cq_qmatmul / cq_qmatmul_fused / cq_qmatmul_shaped may be called in place (y on top of
 *    x or aux): such a call goes through the separate quantizer launch, which has read every input
 *    before the matmul kernel stores anything.  cq_qmatmul_multi and the grouped calls refuse /
 *    do not support outputs that overlap their inputs.  The workspace never overlaps anything.
 *  - every matmul call needs its workspace (size from cq_workspace_bytes*), also the calls that
 *    usually finish in one launch without touching it: which kernels run is the library's choice.
 *  - no C++ exception or abort crosses this boundary.
 */
#ifndef CANDLE_QHIP_H
#define CANDLE_QHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GgmlDType ids handled by this library (mod.rs:133-190). */
enum {
    CQ_DTYPE_Q4_0 = 2,
    CQ_DTYPE_Q4_1 = 3,  /* held as Q8_0 planes (qs = q) plus a plane of block minima; the m * s term of the dot
                           product with Q8_1 activations (k_quants.rs:267-294) is added by the one-launch decode kernels
                           themselves, by a second small launch otherwise                                           */
    CQ_DTYPE_Q5_0 = 6,  /* held on the device as Q8_0 planes (qs = q - 16): the same values, the same arithmetic     */
    CQ_DTYPE_Q5_1 = 7,  /* like Q4_1, with five-bit quants                                                            */
    CQ_DTYPE_Q8_0 = 8,
    CQ_DTYPE_Q8_1 = 9,  /* activation format only */
    CQ_DTYPE_Q2K = 10,  /* held as Q6K planes (scale, quant + 32) plus the groups' minima and dmin; the dmin term of the
                           dot product (k_quants.rs:717-767) is subtracted the same way                                */
    CQ_DTYPE_Q3K = 11,  /* held on the device as Q6K planes (scale - 32, quant + 28): the same values and arithmetic */
    CQ_DTYPE_Q4K = 12,
    CQ_DTYPE_Q5K = 13,
    CQ_DTYPE_Q6K = 14,
    CQ_DTYPE_Q8K = 15   /* the activation format of the K-quants; as a weight type (k_quants.rs:1749-1839, a type of the
                           reference's tests rather than of checkpoints) it has one plain dot-product kernel, which
                           reads the weights once per activation row: m rows cost m passes over n * k bytes     */
};

/* error codes */
enum {
    CQ_OK = 0,
    CQ_ERR_INVALID = -1,     /* bad argument (shape, dtype, null pointer)      */
    CQ_ERR_UNSUPPORTED = -2, /* dtype / combination not handled by this build  */
    CQ_ERR_HIP = -3,         /* a HIP runtime call failed                      */
    CQ_ERR_WORKSPACE = -4    /* workspace missing or too small                 */
};

/* flags of cq_qmatmul / cq_workspace_bytes */
enum {
    CQ_FLAG_AUTO = 0,
    CQ_FLAG_FORCE_MATVEC = 1, /* row-streaming kernel whatever m is (A/B runs; replaces cuda.rs:22-26 set_force_dmmv) */
    CQ_FLAG_FORCE_GEMM = 2,   /* int8-MFMA tile kernel whatever m is                                                  */
    CQ_FLAG_ACT_Q8_1 = 4,     /* Q4K / Q6K weights x Q8_1 activations: the formulation of the reference's CUDA arm
                                 (mul_mat_via_q8_1, cuda.rs:298-365; quantized.cu:2141-2166, :2258-2281) with the
                                 activations quantized by BlockQ8_1::from_float (k_quants.rs:665-691), instead of the
                                 CPU formulation's Q8K.  A dot-product kernel up to 32 rows, the matrix cores beyond; combines with
                                 CQ_FLAG_REUSE_ACT only; the grouped calls do not take it.  Its results differ from
                                 the CPU QMatMul's by the two activation quantizers' noise (about 1e-2 relative:
                                 rel-L2 8.7e-3 measured on M = 512, K = 4096 activations with 1 % outliers).         */
    CQ_FLAG_REUSE_ACT = 8,    /* the workspace already holds this x, quantized by an earlier cq_qmatmul call with the
                                 same m, k and activation format (q/k/v or gate/up share their input): skip the
                                 quantizer launch.  The earlier call must have gone through the workspace: more than
                                 four rows, or CQ_FLAG_STAGED_ACT (calls of up to four rows may quantize inside their
                                 single launch and leave the workspace alone); cq_qmatmul_multi takes care of this
                                 by itself.  cq_qmatmul_grouped takes it too: the routed rows of the previous grouped
                                 call (same x, row ids, offsets, k and activation format) against another set of
                                 experts, w1 and w3 of an expert FFN.  No counterpart in the reference, which
                                 re-quantizes per call.                                                              */
    CQ_FLAG_FORCE_SKINNY = 32, /* the split-K MFMA kernel for few rows whatever m is (A/B runs)                                */
    CQ_FLAG_STAGED_ACT = 16,  /* up to four rows: run the stand-alone quantizer into the workspace and a matmul kernel
                                 (two launches, as cuda.rs:249-293 does) instead of the single fused launch           */
    CQ_FLAG_DETERMINISTIC = 64 /* the same bits on every run, like the CPU QMatMul.  Without it one family of launches is
                                 not: the tile kernels (17 rows and more; grouped experts with more than 8 rows) split K
                                 over several workgroups when the weight has few row tiles - n = 4096 at 33 .. 1024
                                 rows, the w2 projection of an expert - and add the partial sums atomically in
                                 arrival order, so the last bits of a result can differ between two runs (far inside
                                 the 1e-4 bar; the reference's CUDA arm is allowed 1e-4 of drift between batch sizes,
                                 quantized_tests.rs:203-209).  With the flag those launches never split K: each
                                 result is one sum in a fixed order, at the price of fewer workgroups in flight.
                                 Every other kernel is deterministic as it is.  Accepted by all matmul entry points. */
};

/* the model step a fused call computes on the way into the activation quantizer */
enum {
    CQ_PRE_NONE = 0,
    CQ_PRE_RMS_NORM = 1, /* x / sqrt(mean(x^2) + eps) * alpha[k]   (candle-nn/src/ops.rs:482-495)                  */
    CQ_PRE_SILU_MUL = 2  /* silu(x) * x2, x2 shaped like x         (quantized_llama.rs:56-63, candle-core op.rs:607-609) */
};

typedef struct cq_weight cq_weight;

/* ---- library / device ---------------------------------------------------- */
/* Number of usable HIP devices; 0 when no GPU is visible (Device::new_cuda's role, device.rs). */
int cq_device_count(void);
/* Thread-local message of the last failing call on this thread (candle_core::Error's role). */
const char *cq_last_error(void);
const char *cq_version(void);

/* ---- GgmlDType helpers (mod.rs:211-246) ---------------------------------- */
int64_t cq_block_size(int ggml_dtype); /* GgmlDType::block_size, 0 if unknown */
int64_t cq_type_size(int ggml_dtype);  /* GgmlDType::type_size,  0 if unknown */
/* The activation block type a weight type is contracted with on the CPU path
 * (GgmlType::VecDotType, k_quants.rs:160,565,1155,1569); -1 if unknown. */
int cq_vec_dot_type(int ggml_dtype);

/* ---- weight storage ------------------------------------------------------ */
/* cuda::load_quantized (cuda.rs:591-612; funnel ggml_file.rs:120-135): host GGML blocks of a
 * [n, k] matrix -> device storage.  Uploads and re-packs; k % block_size must be 0. */
int cq_weight_create(int dev, int ggml_dtype, const void *host_ggml_blocks, size_t nbytes,
                     int64_t n, int64_t k, cq_weight **out);
/* QCudaStorage::zeros (cuda.rs:368-381): zero-filled storage for n*k elements. */
int cq_weight_zeros(int dev, int ggml_dtype, int64_t n, int64_t k, cq_weight **out);
/* The same two constructors with the reference's own signatures, which know an element count and no
 * shape: QCudaStorage::zeros(device, el_count, dtype) (cuda.rs:368-381; Device::qzeros, mod.rs:40-57) and
 * load_quantized(device, data: &[T]) (cuda.rs:591-612).  The storage is a flat run of blocks (the device
 * planes are ordered by flat block index), so it can be read as any [n, k] with n * k == elem_count and
 * k % block_size == 0; until told otherwise it reads as [elem_count / block_size, block_size].  The shape
 * arrives with the call (cq_qmatmul_shaped, as QCudaStorage::fwd takes self_shape, cuda.rs:478-499) or is
 * fixed once with cq_weight_set_shape (QTensor::new, mod.rs:318-323), which the entry points without a
 * shape argument then use.  That shape is state of the handle: cq_weight_set_shape is a set-up call, not to run
 * while another thread uses the handle (the matmul entry points read n and k without a lock), and two views of one
 * storage with different shapes take cq_qmatmul_shaped / cq_workspace_bytes_shaped, which leave the handle alone. */
int cq_weight_zeros_flat(int dev, int ggml_dtype, int64_t elem_count, cq_weight **out);
int cq_weight_create_flat(int dev, int ggml_dtype, const void *host_ggml_blocks, size_t nbytes, cq_weight **out);
int64_t cq_weight_elem_count(const cq_weight *w);                /* QTensor::shape().elem_count() */
int cq_weight_set_shape(cq_weight *w, int64_t n, int64_t k);     /* check_shape, mod.rs:304-316   */
/* QCudaStorage::quantize (cuda.rs:448-472): f32 [n*k] on the device -> this storage.  The
 * reference copies to the host and runs T::from_float there; here the same arithmetic runs in
 * a HIP kernel and yields the same bytes. */
int cq_weight_quantize(cq_weight *w, const float *src_dev, void *stream);
/* QCudaStorage::dequantize / dequantize_f16 (cuda.rs:391-446): dst has n*k elements and is
 * 16-byte aligned (the kernels store whole 16-byte groups). */
int cq_weight_dequantize(const cq_weight *w, float *dst_dev, void *stream);
int cq_weight_dequantize_f16(const cq_weight *w, uint16_t *dst_dev, void *stream);
/* Inverse re-pack: the exact GGML bytes back on the host (QStorage::data, mod.rs:118-130; what
 * gguf_file::write needs).  Synchronises the device. */
int cq_weight_to_ggml(const cq_weight *w, void *host_dst, size_t nbytes);
/* QCudaStorage::storage_size_in_bytes (cuda.rs:474-476): unpadded GGML byte size. */
size_t cq_weight_size_in_bytes(const cq_weight *w);
int cq_weight_dtype(const cq_weight *w);                        /* QCudaStorage::dtype  (cuda.rs:383) */
int cq_weight_device(const cq_weight *w);                       /* QCudaStorage::device (cuda.rs:387) */
int cq_weight_shape(const cq_weight *w, int64_t *n, int64_t *k); /* QTensor::shape (mod.rs:357)       */
void cq_weight_destroy(cq_weight *w);                           /* Drop of the storage                */

/* ---- activation quantizer ------------------------------------------------ */
/* T::VecDotType::from_float over m rows (k_quants.rs:1857-1862; launch precedent cuda.rs:46-67).
 * act_dtype in {Q8_0, Q8_1, Q8K}.  dst receives m * k/block GGML blocks in the reference's
 * struct layout (k_quants.rs:78-93, 148-155), byte-comparable with the CPU path. */
size_t cq_act_bytes(int act_dtype, int64_t m, int64_t k);
int cq_quantize_act(int dev, int act_dtype, const float *x_dev, int64_t m, int64_t k,
                    void *dst_blocks_dev, void *stream);

/* ---- matmul -------------------------------------------------------------- */
/* Scratch the caller must provide to cq_qmatmul for m activation rows (the reference allocates
 * its quantized-activation buffer per call, cuda.rs:249-252, 322-325). */
size_t cq_workspace_bytes(const cq_weight *w, int64_t m, int flags);
/* QCudaStorage::fwd (cuda.rs:478-499) = <QTensor as CustomOp1>::cuda_fwd (mod.rs:514-524):
 * y[m, n] = x[m, k] . W[n, k]^T with x quantized to W's VecDotType first (k_quants.rs:1842-1883).
 * x contiguous f32; m = product of the leading dims of the input tensor.
 * Q4_1, Q5_0 and Q5_1 weights with an odd number of 32-element blocks per row are refused with
 * CQ_ERR_INVALID, as their vec_dot refuses them (k_quants.rs:273, 363, 469); so do the other matmul
 * entry points. */
int cq_qmatmul(const cq_weight *w, const float *x_dev, int64_t m, float *y_dev, int flags,
               void *workspace_dev, size_t workspace_bytes, void *stream);
/* The same with the weight's shape given at the call, exactly as QCudaStorage::fwd(&self, self_shape, ..)
 * receives it (cuda.rs:478-499): [n, k] must cover the storage's elements, k % block_size == 0. */
size_t cq_workspace_bytes_shaped(const cq_weight *w, int64_t n, int64_t k, int64_t m, int flags);
int cq_qmatmul_shaped(const cq_weight *w, int64_t n, int64_t k, const float *x_dev, int64_t m, float *y_dev,
                      int flags, void *workspace_dev, size_t workspace_bytes, void *stream);
/* cq_qmatmul for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference (which allocates its quantized
 * activations per call, cuda.rs:249-252).  Same arguments and results as cq_qmatmul without the workspace:
 * the quantized activations go to an array of CQ_STATIC_SCRATCH_BYTES that is part of the library's device
 * code, so every GPU the library runs on holds that much until the process ends.  Calls that need more
 * (cq_workspace_bytes(w, m, flags) > CQ_STATIC_SCRATCH_BYTES) fail with CQ_ERR_WORKSPACE.  The call itself
 * allocates and frees nothing; the array's address is looked up when the first weight is created on a device.
 * The first launch of a kernel instance on a device that needs more than 48 KiB of LDS sets that function attribute
 * once (hipFuncSetAttribute, as in every other entry point): make one call of each shape outside stream capture
 * before capturing.
 * All calls on one GPU share the array: calls that overlap in time on one GPU (two streams, two host threads)
 * race on it; calls in stream order do not. */
#define CQ_STATIC_SCRATCH_BYTES (16u << 20)
int cq_qmatmul_static(const cq_weight *w, const float *x_dev, int64_t m, float *y_dev, int flags, void *stream);
/* Debug/verification: the per-block integer dot products the f32 result is combined from
 * (k_quants.rs:1221-1241 for Q4K, :1418-1438 for Q5K, :1615-1633 for Q6K, :245-250 / :640-645 for Q4_0/Q8_0).
 * out_i[(r*n + c)*kb + b] = I_b; out_mn likewise = sum_j bsums_j*min_j (Q4K and Q5K, else NULL). */
int cq_qmatmul_int_dots(const cq_weight *w, const float *x_dev, int64_t m, int32_t *out_i_dev,
                        int32_t *out_mn_dev, void *workspace_dev, size_t workspace_bytes,
                        void *stream);

/* The same integers out of the matrix-core kernels (the verification above runs the dot-product kernels): `kernel`
 * picks the small-batch kernel (CQ_MFMA_SKINNY: the launch cq_qmatmul makes for few rows, whatever m is here) or
 * the tile kernel of the prefill path (CQ_MFMA_TILE, with the tile height and K split cq_qmatmul picks for m;
 * Q8_0 and Q4_0 weights: more than 16 rows, as in cq_qmatmul).
 * out_i as above.  out_mn (Q4K, Q5K; else NULL) is a float: those kernels contract the min term on the f16 matrix
 * core and never hold the integer sum: -dmin * sum_j min_{j/2}*bsums_j over the sixteen sums of a block (exact in
 * f16) with -dmin*min in two f16 pieces, stored as that contraction delivers it for one block (small-batch kernels) or
 * times the activation block's scale (tile kernel).  With CQ_MFMA_INT_MIN added to `kernel` the weight operand of
 * that contraction is the group minima themselves instead of -dmin * min, and out_mn receives the integer
 * Mn_b = sum_j min_{j/2} * bsums_j of k_quants.rs:1221-1241 (at most 16 * 2048 * 63, exact in a float): the same
 * instructions on the same sums, checked bit for bit.  No counterpart in the reference. */
#define CQ_MFMA_SKINNY 1
#define CQ_MFMA_TILE 2
#define CQ_MFMA_INT_MIN 16
int cq_qmatmul_int_dots_mfma(const cq_weight *w, const float *x_dev, int64_t m, int kernel, int32_t *out_i_dev,
                             float *out_mn_dev, void *workspace_dev, size_t workspace_bytes, void *stream);

/* ---- grouped experts (MoE FFN) ------------------------------------------- */
/* One QMatMul per expert over gathered rows, as MlpOrMoe::forward does sequentially
 * (candle-transformers/src/models/quantized_llama.rs:117-135): for expert e and p in
 * [offsets[e], offsets[e+1]):  y[p, :] = x[row_ids[p], :] . W_e^T   (row_ids == NULL: x[p, :]).
 * All experts share dtype and shape.  y has offsets[n_experts] rows. */
size_t cq_grouped_workspace_bytes(const cq_weight *const *experts, int n_experts, int64_t total_rows,
                                  int flags);
int cq_qmatmul_grouped(const cq_weight *const *experts, int n_experts, const float *x_dev,
                       const int32_t *row_ids_dev, const int32_t *offsets_host, float *y_dev,
                       int flags, void *workspace_dev, size_t workspace_bytes, void *stream);
/* h[i] = silu(a[i]) * b[i], silu(v) = v / (1 + exp(-v))  (Mlp::forward, quantized_llama.rs:56-63;
 * candle-core/src/op.rs:607-609). */
int cq_silu_mul(int dev, const float *a_dev, const float *b_dev, float *h_dev, int64_t count, void *stream);
/* ys[row_ids[p], :] += weights[p] * y[p, :] for p in expert order (broadcast_mul + index_add,
 * quantized_llama.rs:132-134; cpu_backend/mod.rs:619-653).  Each destination element is summed in
 * increasing p, which is increasing expert index, like the reference's sequential loop. */
int cq_moe_scatter_add(int dev, const float *y_dev, const int32_t *row_ids_dev, const float *weights_dev,
                       int64_t total_rows, int64_t hidden, float *ys_dev, int64_t tokens, void *stream);

/* ---- the matmul with the preceding model step fused in --------------------------------------
 * What the quantized models run directly in front of a QMatMul, computed on the way into the
 * activation quantizer so that the intermediate tensor never goes to memory:
 *   CQ_PRE_RMS_NORM: RmsNorm::forward (candle-transformers/src/quantized_nn.rs:121-125 ->
 *     candle_nn::ops::rms_norm, candle-nn/src/ops.rs:482-495) in front of the attention and
 *     feed-forward projections (quantized_llama.rs:453-466): aux = alpha[k], eps as given.
 *   CQ_PRE_SILU_MUL: silu(w1 x) * (w3 x) in front of w2 (Mlp::forward, quantized_llama.rs:56-63;
 *     the expert loop :124-131): x = w1's output, aux = w3's output, both [m, k]; eps unused.
 * Equivalent to the unfused sequence up to rounding: rms_norm is computed as the reference's device
 * kernel does, (1 / sqrt(mean + eps)) * x * alpha (candle-kernels/src/reduce.cu:161-172), with the
 * squares added pairwise in an order that does not depend on m; the CPU code adds them one by one
 * and divides.  silu * mul is the reference's sequence of operations (the exp is the device's).
 * aux is 16-byte aligned like x.  For one row this is still one launch.
 * cq_quantize_act_fused is the quantizer half on its own, for byte comparison with the CPU path. */
int cq_quantize_act_fused(int dev, int act_dtype, int pre, const float *x_dev, const float *aux_dev, float eps,
                          int64_t m, int64_t k, void *dst_blocks_dev, void *stream);
int cq_qmatmul_fused(const cq_weight *w, int pre, const float *x_dev, const float *aux_dev, float eps, int64_t m,
                     float *y_dev, int flags, void *workspace_dev, size_t workspace_bytes, void *stream);
/* Several weights on the same activations: ys[i] = x . ws[i]^T, i < count (the q, k, v projections of an
 * attention block, quantized_llama.rs:206-208; w1 and w3 of the feed-forward block, :60-61), with the step
 * `pre` in front as in cq_qmatmul_fused (CQ_PRE_NONE for none).  The weights share dtype, row length k and
 * device; their row counts may differ.  One activation row and two or three weights with rows of at most
 * 256 lane units (k <= 16384 for Q4K/Q5K, 8192 for Q6K/Q4_0, 4096 for Q8_0), flags == 0: a single launch
 * for all of them, each output bit-identical to its own cq_qmatmul_fused call; the same for two to four
 * rows without a step in front when the weight rows are short enough for the one-launch kernel (k <= 4096
 * always).  More rows: the rows are quantized once and every weight takes its matmul from the shared
 * workspace (size: the largest cq_workspace_bytes among the weights).  Anything else: one call per weight.  The reference has no
 * counterpart, it calls QMatMul::forward once per weight; a `Hip` arm can offer it to the model code beside
 * forward(). */
int cq_qmatmul_multi(const cq_weight *const *ws, int count, int pre, const float *x_dev, const float *aux_dev, float eps,
                     int64_t m, float *const *ys_dev, int flags, void *workspace_dev, size_t workspace_bytes,
                     void *stream);
/* cq_qmatmul_grouped with the same step applied to the gathered rows (row p reads x and aux at
 * row_ids[p], or p when row_ids is NULL). */
int cq_qmatmul_grouped_fused(const cq_weight *const *experts, int n_experts, int pre, const float *x_dev,
                             const float *aux_dev, float eps, const int32_t *row_ids_dev,
                             const int32_t *offsets_host, float *y_dev, int flags, void *workspace_dev,
                             size_t workspace_bytes, void *stream);

/* ---- measurement aid (no counterpart in the reference) ---------------------------------------
 * cq_timing_arm(): the next matmul kernel this host thread launches through cq_qmatmul (the
 * matvec / GEMM kernel proper, not a separate activation-quantizer launch) is bracketed by a pair
 * of HIP events owned by the library, recorded on the stream of that launch.
 * cq_timing_elapsed_us(): waits for that kernel and returns its duration in microseconds;
 * CQ_ERR_INVALID when no armed launch has happened since the last call. */
int cq_timing_arm(void);
int cq_timing_elapsed_us(double *us);

/* ---- hardware self-check (no counterpart in the reference) -------------------------------------
 * The activation quantizers round with `f32::round` (half away from zero; k_quants.rs:605, :1812).
 * On the device that is one conversion instruction (floor(|t| + 0.5) without an intermediate
 * rounding) plus the sign.  This call compares it with round-half-away computed the long way for
 * every f32 t with |t| <= 130 (both signs, denormals included) and stores the number of
 * mismatches, which must be zero on any device the library is used on. */
int cq_selfcheck_round(int dev, uint64_t *mismatches);

#ifdef __cplusplus
}
#endif
#endif /* CANDLE_QHIP_H */
