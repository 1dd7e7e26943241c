// Self-test of the C++ host layer: the reference's own Q4_0 matmul tests
// (candle-core/tests/quantized_tests.rs:49-64 `quantized_matmul`, :109-129 `quantized_matmul_neg`)
// driven through QTensor::quantize -> QMatMul::from_qtensor -> forward, plus the error behaviour of
// the shape checks.  `--host-only` stops before anything needs a GPU.
#include <cmath>
#include <cstdio>
#include <cstring>

#include "quantized.hpp"

using namespace candle_hip;

static int g_failed = 0;
#define EXPECT(cond, ...)                                   \
    do {                                                    \
        if (!(cond)) {                                      \
            g_failed++;                                     \
            std::printf("FAIL %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                       \
            std::printf("\n");                              \
        }                                                   \
    } while (0)

template <typename F> static bool throws(F f) {
    try { f(); } catch (const Error &) { return true; }
    return false;
}

static void host_only() {
    // GgmlDType::block_size / type_size (mod.rs:212-246)
    EXPECT(block_size(GgmlDType::Q4_0) == 32 && type_size(GgmlDType::Q4_0) == 18, "Q4_0 sizes");
    EXPECT(block_size(GgmlDType::Q8_0) == 32 && type_size(GgmlDType::Q8_0) == 34, "Q8_0 sizes");
    EXPECT(block_size(GgmlDType::Q8_1) == 32 && type_size(GgmlDType::Q8_1) == 36, "Q8_1 sizes");
    EXPECT(block_size(GgmlDType::Q4K) == 256 && type_size(GgmlDType::Q4K) == 144, "Q4K sizes");
    EXPECT(block_size(GgmlDType::Q5K) == 256 && type_size(GgmlDType::Q5K) == 176, "Q5K sizes");
    EXPECT(block_size(GgmlDType::Q6K) == 256 && type_size(GgmlDType::Q6K) == 210, "Q6K sizes");
    EXPECT(block_size(GgmlDType::Q8K) == 256 && type_size(GgmlDType::Q8K) == 292, "Q8K sizes");
    EXPECT(to_u32(ggml_dtype_from_u32(12)) == 12, "dtype id round trip");
    EXPECT(throws([] { ggml_dtype_from_u32(5); }), "unknown dtype id must be an error");
    // check_shape (mod.rs:304-316)
    EXPECT(throws([] { check_shape({}, 32); }), "scalar shape must be an error");
    EXPECT(throws([] { check_shape({4, 33}, 32); }), "last dim not divisible by the block size must be an error");
    EXPECT(!throws([] { check_shape({4, 64}, 32); }), "valid shape rejected");
}

static std::vector<float> ramp(int count, float shift) {
    std::vector<float> v((size_t)count);
    for (int i = 0; i < count; i++) v[(size_t)i] = (float)i - shift;
    return v;
}

static void q4_0_matmul(const char *name, float lhs_shift, float rhs_shift, const double (&want)[12]) {
    const int m = 3, k = 64, n = 4;
    Tensor lhs = Tensor::from_host(ramp(m * k, lhs_shift), {m, k});
    Tensor rhs = Tensor::from_host(ramp(k * n, rhs_shift), {n, k});
    QTensor q = QTensor::quantize(rhs, GgmlDType::Q4_0);
    EXPECT(q.storage_size_in_bytes() == 8 * 18, "%s: storage size %zu", name, q.storage_size_in_bytes());
    EXPECT(q.dtype() == GgmlDType::Q4_0 && q.rank() == 2, "%s: dtype/rank", name);
    QMatMul mm = QMatMul::from_qtensor(std::move(q));
    Tensor y = mm.forward(lhs);
    EXPECT(y.shape == (Shape{m, n}), "%s: output shape %s", name, to_string(y.shape).c_str());
    std::vector<float> got = y.to_host();
    for (int i = 0; i < m * n; i++)
        EXPECT(std::round((double)got[(size_t)i]) == want[i], "%s: element %d = %f, want %f", name, i, got[(size_t)i], want[i]);
    // rank-3 input keeps its leading dims (mod.rs:488-490)
    Tensor lhs3 = Tensor::from_host(ramp(m * k, lhs_shift), {1, m, k});
    Tensor y3 = mm.forward(lhs3);
    EXPECT(y3.shape == (Shape{1, m, n}), "%s: rank-3 output shape %s", name, to_string(y3.shape).c_str());
    EXPECT(y3.to_host() == got, "%s: rank-3 result differs", name);
    // error behaviour (mod.rs:480-487)
    Tensor bad = Tensor::from_host(ramp(m * 32, 0.f), {m, 32});
    EXPECT(throws([&] { mm.forward(bad); }), "%s: wrong last dim must be an error", name);
    Tensor one = Tensor::from_host(ramp(k, 0.f), {k});
    EXPECT(throws([&] { mm.forward(one); }), "%s: rank-1 input must be an error", name);
}

static void roundtrip() {
    // QTensor::quantize + dequantize + data(): 2 x 256 Q4K, error bound of quantized_tests.rs:546
    const int n = 2, k = 256;
    std::vector<float> src((size_t)(n * k));
    for (int i = 0; i < n * k; i++) src[(size_t)i] = -0.5f + (float)i / (float)(n * k);
    QTensor q = QTensor::quantize(Tensor::from_host(src, {n, k}), GgmlDType::Q4K);
    EXPECT(q.data().size() == 2 * 144, "Q4K data size");
    std::vector<float> back = q.dequantize().to_host();
    float worst = 0.f;
    for (size_t i = 0; i < src.size(); i++) worst = std::fmax(worst, std::fabs(back[i] - src[i]));
    EXPECT(worst < 0.017f, "Q4K round-trip max error %f", worst);
    // load_quantized(device, blocks) knows no shape (cuda.rs:591-612): the tensor's shape arrives with QTensor::new
    // and reaches the kernel with the call (fwd(self_shape, ..), cuda.rs:478-499)
    std::vector<uint8_t> blocks = q.data();
    QHipStorage st = QHipStorage::load_quantized(0, GgmlDType::Q4K, blocks.data(), blocks.size());
    EXPECT(st.elem_count() == n * k && st.storage_size_in_bytes() == blocks.size(), "flat storage size");
    std::vector<float> x((size_t)k);
    for (int i = 0; i < k; i++) x[(size_t)i] = std::cos(0.3f * (float)i);
    Tensor xt = Tensor::from_host(x, {1, k});
    std::vector<float> direct = st.fwd({n, k}, xt).to_host();
    QMatMul mm = QMatMul::from_qtensor(QTensor(std::move(st), {n, k}));
    EXPECT(mm.forward(xt).to_host() == direct, "flat storage: forward through QTensor differs from fwd(self_shape)");
    EXPECT(QMatMul::from_qtensor(std::move(q)).forward(xt).to_host() == direct, "flat storage: differs from the quantized tensor");
    EXPECT(throws([&] { QHipStorage::zeros(0, 100, GgmlDType::Q4K); }), "element count that is no whole number of blocks");
    EXPECT(throws([&] { QTensor(QHipStorage::zeros(0, 512, GgmlDType::Q4K), {3, 256}); }), "shape that does not cover the storage");
}

static void fused_neighbours() {
    // forward_rms_norm / forward_silu_mul against forward() on inputs prepared on the host
    const int m = 3, k = 512, n = 16;
    std::vector<float> w((size_t)(n * k)), x((size_t)(m * k)), u((size_t)(m * k)), alpha((size_t)k);
    for (int i = 0; i < n * k; i++) w[(size_t)i] = 0.02f * std::sin(0.37f * (float)i);
    for (int i = 0; i < m * k; i++) { x[(size_t)i] = 2.0f * std::cos(0.11f * (float)i); u[(size_t)i] = std::sin(0.05f * (float)i); }
    for (int i = 0; i < k; i++) alpha[(size_t)i] = 1.0f + 0.1f * std::sin((float)i);
    QMatMul mm = QMatMul::from_qtensor(QTensor::quantize(Tensor::from_host(w, {n, k}), GgmlDType::Q4K));
    const float eps = 1e-5f;
    std::vector<float> xn(x.size()), su(x.size());
    for (int r = 0; r < m; r++) {
        float sum2 = 0.f;
        for (int i = 0; i < k; i++) sum2 += x[(size_t)(r * k + i)] * x[(size_t)(r * k + i)];
        const float root = std::sqrt(sum2 / (float)k + eps);
        for (int i = 0; i < k; i++) xn[(size_t)(r * k + i)] = x[(size_t)(r * k + i)] / root * alpha[(size_t)i];
    }
    for (size_t i = 0; i < x.size(); i++) su[i] = x[i] / (1.0f + std::exp(-x[i])) * u[i];
    auto close = [&](const std::vector<float> &a, const std::vector<float> &b, const char *what) {
        double num = 0, den = 0;
        for (size_t i = 0; i < a.size(); i++) { num += ((double)a[i] - b[i]) * ((double)a[i] - b[i]); den += (double)b[i] * b[i]; }
        EXPECT(a.size() == b.size() && std::sqrt(num) <= 1e-4 * std::sqrt(den), "%s: relative L2 %g", what, std::sqrt(num / den));
    };
    Tensor xt = Tensor::from_host(x, {m, k}), ut = Tensor::from_host(u, {m, k}), at = Tensor::from_host(alpha, {k});
    close(mm.forward_rms_norm(xt, at, eps).to_host(), mm.forward(Tensor::from_host(xn, {m, k})).to_host(), "forward_rms_norm");
    close(mm.forward_silu_mul(xt, ut).to_host(), mm.forward(Tensor::from_host(su, {m, k})).to_host(), "forward_silu_mul");
    Tensor one = Tensor::from_host(std::vector<float>(x.begin(), x.begin() + k), {1, k});
    Tensor one_n = Tensor::from_host(std::vector<float>(xn.begin(), xn.begin() + k), {1, k});
    close(mm.forward_rms_norm(one, at, eps).to_host(), mm.forward(one_n).to_host(), "forward_rms_norm, one row");
    Tensor short_alpha = Tensor::from_host(std::vector<float>((size_t)(k - 1), 1.f), {k - 1});
    EXPECT(throws([&] { mm.forward_rms_norm(xt, short_alpha, eps); }), "alpha of the wrong length must be an error");
    EXPECT(throws([&] { mm.forward_silu_mul(xt, one); }), "operands of different shapes must be an error");
    // forward_multi: every output equals the matrix's own forward(), one row (one launch) and several
    std::vector<float> w2((size_t)(2 * n * k));
    for (size_t i = 0; i < w2.size(); i++) w2[i] = 0.02f * std::cos(0.23f * (float)i);
    QMatMul mm2 = QMatMul::from_qtensor(QTensor::quantize(Tensor::from_host(w2, {2 * n, k}), GgmlDType::Q4K));
    for (const Tensor *in : {&one, &xt}) {
        std::vector<Tensor> ys = QMatMul::forward_multi({&mm, &mm2}, *in);
        EXPECT(ys.size() == 2 && ys[1].shape.back() == 2 * n, "forward_multi: output shapes");
        close(ys[0].to_host(), mm.forward(*in).to_host(), "forward_multi, first matrix");
        close(ys[1].to_host(), mm2.forward(*in).to_host(), "forward_multi, second matrix");
        std::vector<Tensor> yn = QMatMul::forward_multi({&mm, &mm2}, *in, &at, eps);
        close(yn[1].to_host(), mm2.forward_rms_norm(*in, at, eps).to_host(), "forward_multi with rms_norm");
    }
    QMatMul other = QMatMul::from_qtensor(QTensor::quantize(Tensor::from_host(w, {n, k}), GgmlDType::Q6K));
    EXPECT(throws([&] { QMatMul::forward_multi({&mm, &other}, xt); }), "matrices of different dtypes must be an error");
}

int main(int argc, char **argv) {
    const bool host = argc > 1 && std::strcmp(argv[1], "--host-only") == 0;
    try {
        host_only();
        if (!host) {
            if (cq_device_count() <= 0) {
                std::printf("selftest: no GPU visible\n");
                return 2;
            }
            const double g1[12] = {85120, 214562, 345455, 474748, 213475, 604465, 1000686, 1388317, 341876, 994283, 1655709, 2301518};
            const double g2[12] = {243524, -19596, -285051, -549815, 23777, 21651, 19398, 18367, -196472, 63012, 324585, 587902};
            q4_0_matmul("quantized_matmul", 0.f, 0.f, g1);
            q4_0_matmul("quantized_matmul_neg", 3 * 64 / 2.0f, 64 * 4 / 3.0f, g2);
            roundtrip();
            fused_neighbours();
        }
    } catch (const std::exception &e) {
        std::printf("FAIL: exception: %s\n", e.what());
        return 1;
    }
    std::printf(g_failed ? "selftest: %d check(s) failed\n" : "selftest: ok%.0d\n", g_failed);
    return g_failed ? 1 : 0;
}
