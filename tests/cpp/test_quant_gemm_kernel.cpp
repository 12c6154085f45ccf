// Tests of MI355QuantGemmKernel / QuantGemmRegistry in the style of the reference's
// operator tests (tests/v2/.../Test__CPUNativeVNNI_GEMV.cpp): build an operator from
// synthetic GGUF blocks, call the ITensorGemm-shaped methods, compare with the CPU
// oracle on the same inputs.
//
//   test_quant_gemm_kernel --cpu   host logic only (no device needed)
//   test_quant_gemm_kernel         everything (needs an MI355X)
#include "llaminar_amd/quant_gemm.hpp"
#include "ql_oracle.h"

#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

using namespace llaminar_amd;

static int g_failed = 0, g_checks = 0;
static const char *g_case = "";

#define CHECK(cond)                                                                      \
    do                                                                                   \
    {                                                                                    \
        ++g_checks;                                                                      \
        if (!(cond))                                                                     \
        {                                                                                \
            ++g_failed;                                                                  \
            printf("  FAIL %s:%d [%s] %s\n", __FILE__, __LINE__, g_case, #cond);         \
            fflush(stdout);                                                              \
        }                                                                                \
    } while (0)

#define HIP_OK(call)                                                                     \
    do                                                                                   \
    {                                                                                    \
        hipError_t e_ = (call);                                                          \
        if (e_ != hipSuccess)                                                            \
        {                                                                                \
            printf("  HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            fflush(stdout);                                                              \
            exit(3);                                                                     \
        }                                                                                \
    } while (0)

static void begin(const char *name)
{
    g_case = name;
    printf("[ RUN ] %s\n", name);
    fflush(stdout);
}

static bool contains(const char *hay, const char *needle) { return strstr(hay, needle) != nullptr; }

// ---- synthetic data ---------------------------------------------------------------

static const uint8_t FORMATS[3] = {LLAM_FMT_Q4_K, LLAM_FMT_Q6_K, LLAM_FMT_IQ3_S};
static const char *fmt_name(uint8_t f) { return f == LLAM_FMT_Q4_K ? "Q4_K" : f == LLAM_FMT_Q6_K ? "Q6_K" : "IQ3_S"; }

// Uniform-random block bytes with the fp16 super-block scales drawn from [0.001, 0.02].
static std::vector<uint8_t> make_weights(uint8_t fmt, int N, int K, unsigned seed)
{
    const size_t bb = llam_format_block_bytes(fmt);
    const size_t nb = (size_t)N * (K / 256);
    std::vector<uint8_t> w(nb * bb);
    std::mt19937 rng(seed);
    for (auto &b : w)
        b = (uint8_t)(rng() & 0xFF);
    std::uniform_real_distribution<float> d(0.001f, 0.02f);
    for (size_t i = 0; i < nb; ++i)
    {
        uint8_t *blk = w.data() + i * bb;
        auto put = [&](size_t off) {
            const uint16_t h = qlo_f32_to_f16_rne(d(rng));
            memcpy(blk + off, &h, 2);
        };
        if (fmt == LLAM_FMT_Q4_K)
        {
            put(0);
            put(2);
        }
        else if (fmt == LLAM_FMT_Q6_K)
            put(208);
        else
            put(0);
    }
    return w;
}

static std::vector<float> make_floats(size_t n, unsigned seed, float scale = 1.0f)
{
    std::mt19937 rng(seed);
    std::normal_distribution<float> d(0.0f, scale);
    std::vector<float> v(n);
    for (auto &x : v)
        x = d(rng);
    return v;
}

template <class T>
struct DevBuf
{
    T *p = nullptr;
    size_t n = 0;
    explicit DevBuf(size_t count) : n(count) { HIP_OK(hipMalloc((void **)&p, std::max<size_t>(count, 1) * sizeof(T))); }
    explicit DevBuf(const std::vector<T> &h) : DevBuf(h.size()) { upload(h); }
    ~DevBuf() { (void)hipFree(p); }
    void upload(const std::vector<T> &h) { HIP_OK(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); }
    std::vector<T> download() const
    {
        std::vector<T> h(n);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
        return h;
    }
};

// Oracle product: quantise A (M x K) and multiply with all N rows.
static std::vector<float> oracle_product(uint8_t fmt, const std::vector<uint8_t> &w, int N, int K,
                                         const float *A, int M)
{
    std::vector<llam_block_q8_1> q8((size_t)M * (K / 32));
    qlo_quantize_q8_1(A, M, K, q8.data());
    std::vector<float> c((size_t)M * N);
    qlo_gemm_rows(fmt, w.data(), K, 0, N, q8.data(), M, c.data(), N, nullptr, 0);
    return c;
}

static float max_abs(const std::vector<float> &v)
{
    float m = 0;
    for (float x : v)
        m = std::max(m, std::fabs(x));
    return m;
}

// max |a-b| / max |b|
static float rel_err(const std::vector<float> &a, const std::vector<float> &b)
{
    float e = 0;
    for (size_t i = 0; i < a.size(); ++i)
        e = std::max(e, std::fabs(a[i] - b[i]));
    return e / std::max(max_abs(b), 1e-30f);
}

// fp32 results differ from the oracle only by the association of per-block sums.
static const float TOL = 2e-6f;

// ---- host-logic cases -----------------------------------------------------------------

static void test_invalid_construction()
{
    begin("InvalidConstructionLeavesOperatorInvalid");
    std::vector<uint8_t> bytes(144 * 4);
    MI355QuantGemmKernel bad_fmt(3, bytes.data(), 1, 1024, 0);
    CHECK(!bad_fmt.isValid());
    CHECK(contains(quant_gemm_last_error(), "unsupported weight format"));
    MI355QuantGemmKernel bad_k(LLAM_FMT_Q4_K, bytes.data(), 4, 200, 0);
    CHECK(!bad_k.isValid());
    CHECK(contains(quant_gemm_last_error(), "multiple of 256"));
    MI355QuantGemmKernel null_w(LLAM_FMT_Q4_K, nullptr, 4, 256, 0);
    CHECK(!null_w.isValid());
    CHECK(!null_w.hasWeights());
    CHECK(null_w.packedWeightBytes() == 0);
    float x = 0;
    DeviceTensor A(&x, 1, 1024), C(&x, 1, 1);
    CHECK(!bad_fmt.multiply_tensor(&A, &C, 1, 1, 1024));
    CHECK(contains(quant_gemm_last_error(), "multiply_tensor"));
}

static void test_shape_checks()
{
    begin("DimensionMismatchIsRejectedBeforeAnyLaunch");
    std::vector<uint8_t> bytes(144 * 8);
    MI355QuantGemmKernel k(LLAM_FMT_Q4_K, bytes.data(), 4, 512, 0);
    CHECK(k.isValid());
    CHECK(k.get_n() == 4 && k.get_k() == 512);
    CHECK(k.codebookId() == LLAM_FMT_Q4_K);
    CHECK(k.supports_device(0) && !k.supports_device(-1) && !k.supports_device(1));
    CHECK(k.supports_fused_projection() && k.supports_activation_sharing());
    float x = 0;
    DeviceTensor A(&x, 1, 512), C(&x, 1, 4);
    CHECK(!k.multiply_tensor(&A, &C, 1, 4, 256));
    CHECK(contains(quant_gemm_last_error(), "Dimension mismatch"));
    CHECK(!k.multiply_tensor(&A, &C, 1, 8, 512));
    CHECK(!k.multiply_tensor(&A, &C, 1, 4, 512, true, 1.0f, 0.0f, nullptr, 3));
    CHECK(contains(quant_gemm_last_error(), "device"));
    CHECK(!k.multiply_tensor(nullptr, &C, 1, 4, 512));
    DeviceTensor small(&x, 1, 100);
    CHECK(!k.multiply_tensor(&small, &C, 1, 4, 512));
    CHECK(!k.multiply_tensor(&A, &C, 2, 4, 512)); // A has one row
    CHECK(!k.multiply_with_precomputed_q8_1(nullptr, &x, 1, 4, 512));
    MI355QuantGemmKernel::FusedExpertDownDesc d{&k, &x, &x, 4};
    CHECK(!k.multiply_fused_expert_down(&d, 1, 2, 512));
    CHECK(contains(quant_gemm_last_error(), "single-token"));
    std::vector<MI355QuantGemmKernel::TensorProjectionDesc> none;
    CHECK(k.multiply_fused_tensor(&A, none, 1, 512));
}

static void test_workspace_sizes()
{
    begin("WorkspaceRequirements");
    CHECK(MI355QuantGemmKernel::getWorkspaceRequirements(1, 5120, 5120) == 5888u + 20480u);
    CHECK(MI355QuantGemmKernel::getWorkspaceRequirements(0, 5120, 5120) == 0u);
    std::vector<uint8_t> bytes(144);
    MI355QuantGemmKernel k(LLAM_FMT_Q4_K, bytes.data(), 1, 256, 0);
    CHECK(k.get_quantized_activation_buffer_size(2, 5120) == 2u * 160u * 36u);
    CHECK(k.get_quantized_activation_buffer_size(2, 100) == 0u);
    CHECK(k.packedWeightBytes() == 144u);
}

static void test_registry()
{
    begin("RegistryHandlesAndLookups");
    QuantGemmRegistry reg;
    bool threw = false;
    try
    {
        reg.prepareGemmHandleLocal(nullptr, 0);
    }
    catch (const std::runtime_error &)
    {
        threw = true;
    }
    CHECK(threw);
    std::vector<uint8_t> bytes(210 * 2 * 3);
    QuantWeightTensor bad{"blk.0.bad", 7, bytes.data(), 3, 512};
    threw = false;
    try
    {
        reg.prepareGemmHandleLocal(&bad, 0);
    }
    catch (const std::runtime_error &e)
    {
        threw = contains(e.what(), "blk.0.bad");
    }
    CHECK(threw);
    QuantWeightTensor bad_shape{"blk.0.odd", LLAM_FMT_Q6_K, bytes.data(), 3, 500};
    threw = false;
    try
    {
        reg.prepareGemmHandleLocal(&bad_shape, 0);
    }
    catch (const std::runtime_error &)
    {
        threw = true;
    }
    CHECK(threw);

    QuantWeightTensor t{"blk.0.ffn_down.weight", LLAM_FMT_Q6_K, bytes.data(), 3, 512};
    auto h = reg.prepareGemmHandleLocal(&t, 0);
    CHECK(h && h->tensor == &t && h->device_id == 0 && h->variant == LLAM_FMT_Q6_K);
    CHECK(h->kind == GemmPreparationKind::MI355_NATIVE_BLOCKS);
    CHECK(reg.prepareGemmHandleLocal(&t, 0) == h); // cached
    CHECK(reg.prepareGemmHandleLocal(&t, 1) != h); // other device, other handle
    MI355QuantGemmKernel *e = reg.getOrCreateGemmEngine(h.get());
    CHECK(e && e->isValid() && e->get_n() == 3 && e->get_k() == 512);
    CHECK(reg.getOrCreateGemmEngine(nullptr) == nullptr);
    reg.registerPreparedGemmHandle("layer0.down", h);
    CHECK(reg.gemmKernel("layer0.down") == e);
    CHECK(reg.gemmKernel("layer0.up") == nullptr);
    threw = false;
    try
    {
        reg.registerPreparedGemmHandle("x", nullptr);
    }
    catch (const std::runtime_error &)
    {
        threw = true;
    }
    CHECK(threw);
    auto ex = std::make_shared<MI355QuantGemmKernel>(LLAM_FMT_Q6_K, bytes.data(), 3, 512, 0);
    reg.registerEngine(0, 5, 17, ExpertRole::DOWN, ex);
    CHECK(reg.getEngine(0, 5, 17, ExpertRole::DOWN) == ex.get());
    CHECK(reg.getEngine(0, 5, 17, ExpertRole::UP) == nullptr);
    CHECK(reg.size() == 3);
    reg.clear();
    CHECK(reg.size() == 0 && reg.gemmKernel("layer0.down") == nullptr);
}

// Without a device nothing is computed: the operator reports failure.
static void test_no_device_fails_loudly()
{
    begin("NoDeviceFailsLoudly");
    auto w = make_weights(LLAM_FMT_Q4_K, 4, 256, 1);
    MI355QuantGemmKernel k(LLAM_FMT_Q4_K, w.data(), 4, 256, 0);
    k.prepareWeights();
    CHECK(!k.weights_converted());
    std::vector<float> a(256), c(4);
    DeviceTensor A(a.data(), 1, 256), C(c.data(), 1, 4);
    CHECK(!k.multiply_tensor(&A, &C, 1, 4, 256));
    CHECK(contains(quant_gemm_last_error(), "device"));
    DeviceQuantMatrixDesc d;
    CHECK(!k.exportMatrixDesc(d) && !d.valid());
}

// ---- device cases ---------------------------------------------------------------------------

static void test_multiply_tensor(uint8_t fmt)
{
    const std::string name = std::string("MultiplyTensor_") + fmt_name(fmt);
    begin(name.c_str());
    const int N = 640, K = 1024;
    auto w = make_weights(fmt, N, K, 11 + fmt);
    MI355QuantGemmKernel k(fmt, w.data(), N, K, 0);
    CHECK(k.isValid() && !k.weights_converted());
    k.prepareWeights();
    CHECK(k.weights_converted());
    CHECK(k.packedWeightBytes() == llam_ql_prepared_bytes(fmt, N, K));

    // m = 1 (GEMV), rows 2.. of a larger activation buffer
    const int rows = 40;
    auto a = make_floats((size_t)rows * K, 5);
    DevBuf<float> dA(a);
    for (int m : {1, 3, 8, 33})
    {
        const int off = 2;
        DevBuf<float> dC((size_t)m * N);
        DeviceTensor A(dA.p, rows, K), C(dC.p, m, N);
        CHECK(k.multiply_tensor(&A, &C, m, N, K, true, 1.0f, 0.0f, nullptr, -1, nullptr, off));
        auto ref = oracle_product(fmt, w, N, K, a.data() + (size_t)off * K, m);
        const float e = rel_err(dC.download(), ref);
        printf("    m=%d max rel err %.3g\n", m, e);
        CHECK(e <= TOL);
    }

    // alpha / beta / bias into a wider C
    {
        const int m = 4, ldc = N + 24;
        auto c0 = make_floats((size_t)m * ldc, 6);
        auto bias = make_floats(N, 7);
        DevBuf<float> dC(c0), dB(bias);
        DeviceTensor A(dA.p, rows, K), C(dC.p, m, ldc), B(dB.p, 1, N);
        CHECK(k.multiply_tensor(&A, &C, m, N, K, true, 0.5f, -1.5f, &B));
        auto prod = oracle_product(fmt, w, N, K, a.data(), m);
        std::vector<float> ref = c0;
        qlo_epilogue(ref.data(), prod.data(), m, N, ldc, 0.5f, -1.5f, bias.data());
        const float e = rel_err(dC.download(), ref);
        printf("    alpha/beta/bias max rel err %.3g\n", e);
        CHECK(e <= TOL);
        // columns beyond n are untouched
        auto got = dC.download();
        bool untouched = true;
        for (int r = 0; r < m; ++r)
            for (int j = N; j < ldc; ++j)
                untouched = untouched && got[(size_t)r * ldc + j] == c0[(size_t)r * ldc + j];
        CHECK(untouched);
    }

    // bias only, dense C (in-place epilogue) and beta = 1 accumulate
    {
        const int m = 2;
        auto bias = make_floats(N, 8);
        DevBuf<float> dC((size_t)m * N), dB(bias);
        DeviceTensor A(dA.p, rows, K), C(dC.p, m, N), B(dB.p, 1, N);
        CHECK(k.multiply_tensor(&A, &C, m, N, K, true, 1.0f, 0.0f, &B));
        auto prod = oracle_product(fmt, w, N, K, a.data(), m);
        std::vector<float> ref((size_t)m * N, 0.0f);
        qlo_epilogue(ref.data(), prod.data(), m, N, N, 1.0f, 0.0f, bias.data());
        CHECK(rel_err(dC.download(), ref) <= TOL);
        CHECK(k.multiply_tensor(&A, &C, m, N, K, true, 1.0f, 1.0f));
        qlo_epilogue(ref.data(), prod.data(), m, N, N, 1.0f, 1.0f, nullptr);
        CHECK(rel_err(dC.download(), ref) <= TOL);
    }
    HIP_OK(hipDeviceSynchronize());
}

// detachWeights / cloneWeights / attachWeights (TensorKernels.h:1335-1394) and the snapshot
// description: a clone attached to another operator of the same shape computes the donor's
// result bit for bit; a detached operator has no weights and fails until they come back.
// enableBatchPlane: a Q6_K operator reads its int8 batch plane for batches of 5..8 rows; the
// result is within tolerance of the CPU restatement, batches of 1..4 do not change, the plane
// goes away with the weights, and the other formats have none.
static void test_batch_plane()
{
    begin("BatchPlane");
    const int N = 136, K = 4096;
    auto w = make_weights(LLAM_FMT_Q6_K, N, K, 91);
    MI355QuantGemmKernel k(LLAM_FMT_Q6_K, w.data(), N, K, 0);
    auto a = make_floats((size_t)8 * K, 92);
    DevBuf<float> dA(a), d4((size_t)4 * N), d8((size_t)8 * N);
    DeviceTensor A(dA.p, 8, K), C4(d4.p, 4, N), C8(d8.p, 8, N);
    CHECK(k.multiply_tensor(&A, &C4, 4, N, K));
    CHECK(k.multiply_tensor(&A, &C8, 8, N, K));
    const auto y4 = d4.download();
    const auto ref = oracle_product(LLAM_FMT_Q6_K, w, N, K, a.data(), 8);
    CHECK(rel_err(d8.download(), ref) <= TOL);

    CHECK(!k.hasBatchPlane() && k.batchPlaneBytes() == 0);
    CHECK(k.enableBatchPlane());
    CHECK(k.hasBatchPlane() && k.batchPlaneBytes() == llam_ql_batch_plane_bytes(LLAM_FMT_Q6_K, N, K));
    CHECK(k.enableBatchPlane()); // idempotent
    CHECK(k.multiply_tensor(&A, &C8, 8, N, K));
    const float e = rel_err(d8.download(), ref);
    printf("    m=8 from the plane: max rel err %.3g\n", e);
    CHECK(e <= TOL);
    CHECK(k.multiply_tensor(&A, &C4, 4, N, K));
    CHECK(d4.download() == y4); // batches of 1..4 never read the plane

    auto taken = k.detachWeights(); // the plane does not travel with the weights
    CHECK(taken && !k.hasBatchPlane());
    CHECK(k.attachWeights(std::move(taken)));
    CHECK(k.multiply_tensor(&A, &C8, 8, N, K));
    CHECK(rel_err(d8.download(), ref) <= TOL);
    CHECK(k.enableBatchPlane());
    k.dropBatchPlane();
    CHECK(!k.hasBatchPlane());

    auto w4 = make_weights(LLAM_FMT_Q4_K, N, K, 93);
    MI355QuantGemmKernel k4(LLAM_FMT_Q4_K, w4.data(), N, K, 0);
    CHECK(!k4.enableBatchPlane() && contains(quant_gemm_last_error(), "no batch plane"));
}

static void test_weight_handover(uint8_t fmt)
{
    const std::string name = std::string("WeightHandover_") + fmt_name(fmt);
    begin(name.c_str());
    const int N = 96, K = 1024, m = 2;
    auto wa = make_weights(fmt, N, K, 61), wb = make_weights(fmt, N, K, 62);
    MI355QuantGemmKernel a(fmt, wa.data(), N, K, 0), b(fmt, wb.data(), N, K, 0);
    auto x = make_floats((size_t)m * K, 63);
    DevBuf<float> dX(x), dA((size_t)m * N), dB((size_t)m * N);
    DeviceTensor X(dX.p, m, K), CA(dA.p, m, N), CB(dB.p, m, N);
    CHECK(a.multiply_tensor(&X, &CA, m, N, K));
    CHECK(b.multiply_tensor(&X, &CB, m, N, K));
    const auto ya = dA.download();
    CHECK(ya != dB.download());

    auto copy = a.cloneWeights();
    CHECK(copy && copy->format() == fmt && copy->N() == N && copy->K() == K && copy->device() == 0);
    CHECK(copy && copy->sizeBytes() == a.packedWeightBytes() && copy->data() != nullptr);
    CHECK(a.hasWeights()); // the donor keeps its own
    CHECK(b.attachWeights(std::move(copy)));
    CHECK(b.multiply_tensor(&X, &CB, m, N, K));
    CHECK(dB.download() == ya);

    auto taken = a.detachWeights();
    CHECK(taken && taken->sizeBytes() == llam_ql_prepared_bytes(fmt, N, K));
    CHECK(!a.hasWeights() && a.packedWeightBytes() == 0);
    CHECK(!a.multiply_tensor(&X, &CA, m, N, K)); // no weights: fails, does not crash
    CHECK(strstr(quant_gemm_last_error(), "weights") != nullptr);
    auto second = taken ? taken->clone() : nullptr; // a copy of a detached payload
    CHECK(second != nullptr);
    CHECK(a.attachWeights(std::move(taken)));
    CHECK(a.hasWeights());
    CHECK(a.multiply_tensor(&X, &CA, m, N, K));
    CHECK(dA.download() == ya);

    // a payload of another shape or format is refused
    auto wz = make_weights(fmt, 64, 256, 64);
    MI355QuantGemmKernel z(fmt, wz.data(), 64, 256, 0);
    CHECK(!z.attachWeights(std::move(second)));
    CHECK(!z.attachWeights(nullptr));

    const KernelSnapshotInfo info = a.getKernelSnapshotInfo();
    CHECK(std::string(info.kernel_name) == "GEMM" && !info.is_passthrough);
    CHECK(info.inputs.size() == 1 && std::string(info.inputs[0].name) == "A");
    CHECK(info.weights.size() == 1 && std::string(info.weights[0].name) == "B");
    CHECK(info.outputs.size() == 1 && std::string(info.outputs[0].name) == "C");
    CHECK(info.scalars.size() == 4 && std::string(info.scalars[3].name) == "weights_converted");
    HIP_OK(hipDeviceSynchronize());
}

static void test_fused_and_verifier_rows(uint8_t fmt)
{
    const std::string name = std::string("FusedProjections_") + fmt_name(fmt);
    begin(name.c_str());
    const int K = 1280, Nq = 512, Nk = 128, Nv = 128;
    auto wq = make_weights(fmt, Nq, K, 21), wk = make_weights(fmt, Nk, K, 22), wv = make_weights(fmt, Nv, K, 23);
    MI355QuantGemmKernel q(fmt, wq.data(), Nq, K, 0), kk(fmt, wk.data(), Nk, K, 0), v(fmt, wv.data(), Nv, K, 0);
    const int m = 4;
    auto a = make_floats((size_t)m * K, 24);
    auto bias = make_floats(Nk, 25);
    DevBuf<float> dA(a), dQ((size_t)m * Nq), dK((size_t)m * Nk), dV((size_t)m * Nv), dB(bias);
    DeviceTensor A(dA.p, m, K), Q(dQ.p, m, Nq), Kt(dK.p, m, Nk), V(dV.p, m, Nv), B(dB.p, 1, Nk);
    using P = MI355QuantGemmKernel::TensorProjectionDesc;

    std::vector<P> projs = {P(&q, &Q, Nq, nullptr, "q"), P(&kk, &Kt, Nk, nullptr, "k"), P(&v, &V, Nv, nullptr, "v")};
    CHECK(q.multiply_fused_verifier_rows_decode_equivalent(&A, projs, m, K));
    auto got_q = dQ.download(), got_k = dK.download(), got_v = dV.download();
    CHECK(rel_err(got_q, oracle_product(fmt, wq, Nq, K, a.data(), m)) <= TOL);
    CHECK(rel_err(got_k, oracle_product(fmt, wk, Nk, K, a.data(), m)) <= TOL);
    CHECK(rel_err(got_v, oracle_product(fmt, wv, Nv, K, a.data(), m)) <= TOL);

    // every verifier row equals the single-row decode result bit for bit
    bool same = true;
    for (int r = 0; r < m; ++r)
    {
        DevBuf<float> d1(Nq);
        DeviceTensor A1(dA.p + (size_t)r * K, 1, K), C1(d1.p, 1, Nq);
        CHECK(q.multiply_tensor(&A1, &C1, 1, Nq, K));
        auto one = d1.download();
        same = same && memcmp(one.data(), got_q.data() + (size_t)r * Nq, Nq * sizeof(float)) == 0;
    }
    CHECK(same);
    CHECK(!q.multiply_fused_verifier_rows_decode_equivalent(&A, projs, 5, K));

    // the down projection's row length (K = 25600) at three and four rows: accepted, and every
    // row carries the bits of the single-row call
    {
        const int KL = 25600, NL = 48;
        auto wl = make_weights(fmt, NL, KL, 27);
        MI355QuantGemmKernel dl(fmt, wl.data(), NL, KL, 0);
        auto al = make_floats((size_t)4 * KL, 28);
        DevBuf<float> dAl(al), dCl((size_t)4 * NL);
        DeviceTensor Al(dAl.p, 4, KL), Cl(dCl.p, 4, NL);
        std::vector<P> one_proj = {P(&dl, &Cl, NL, nullptr, "down")};
        for (int mm = 3; mm <= 4; ++mm)
        {
            CHECK(dl.multiply_fused_verifier_rows_decode_equivalent(&Al, one_proj, mm, KL));
            auto got = dCl.download();
            bool eq = true;
            for (int r = 0; r < mm; ++r)
            {
                DevBuf<float> d1(NL);
                DeviceTensor A1(dAl.p + (size_t)r * KL, 1, KL), C1(d1.p, 1, NL);
                CHECK(dl.multiply_tensor(&A1, &C1, 1, NL, KL));
                auto one = d1.download();
                eq = eq && memcmp(one.data(), got.data() + (size_t)r * NL, NL * sizeof(float)) == 0;
            }
            CHECK(eq);
        }
    }

    // a projection with a bias takes the per-projection route
    std::vector<P> with_bias = {P(&q, &Q, Nq), P(&kk, &Kt, Nk, &B, "k")};
    CHECK(q.multiply_fused_tensor(&A, with_bias, 2, K));
    auto prod = oracle_product(fmt, wk, Nk, K, a.data(), 2);
    std::vector<float> ref((size_t)2 * Nk);
    qlo_epilogue(ref.data(), prod.data(), 2, Nk, Nk, 1.0f, 0.0f, bias.data());
    auto kb = dK.download();
    kb.resize((size_t)2 * Nk);
    CHECK(rel_err(kb, ref) <= TOL);

    // mismatching K is refused
    auto wz = make_weights(fmt, 64, 256, 26);
    MI355QuantGemmKernel z(fmt, wz.data(), 64, 256, 0);
    DevBuf<float> dZ(64);
    DeviceTensor Z(dZ.p, 1, 64);
    std::vector<P> bad = {P(&q, &Q, Nq), P(&z, &Z, 64)};
    CHECK(!q.multiply_fused_tensor(&A, bad, 1, K));
    CHECK(contains(quant_gemm_last_error(), "Dimension mismatch"));
    HIP_OK(hipDeviceSynchronize());
}

static void test_precomputed_q8_1(uint8_t fmt)
{
    const std::string name = std::string("PrecomputedQ8_1_") + fmt_name(fmt);
    begin(name.c_str());
    const int N = 256, K = 768, m = 2;
    auto w = make_weights(fmt, N, K, 31);
    MI355QuantGemmKernel k(fmt, w.data(), N, K, 0);
    auto a = make_floats((size_t)m * K, 32, 3.0f);
    DevBuf<float> dA(a), dC((size_t)m * N);
    DevBuf<uint8_t> dQ(k.get_quantized_activation_buffer_size(m, K));
    CHECK(k.quantize_activations(dA.p, dQ.p, m, K));
    std::vector<llam_block_q8_1> q8((size_t)m * (K / 32));
    qlo_quantize_q8_1(a.data(), m, K, q8.data());
    auto got_q8 = dQ.download();
    CHECK(got_q8.size() == q8.size() * sizeof(llam_block_q8_1));
    CHECK(memcmp(got_q8.data(), q8.data(), got_q8.size()) == 0); // bit-exact
    CHECK(k.multiply_with_precomputed_q8_1(dQ.p, dC.p, m, N, K));
    auto ref = oracle_product(fmt, w, N, K, a.data(), m);
    CHECK(rel_err(dC.download(), ref) <= TOL);
    CHECK(k.multiply_with_precomputed_q8_1(dQ.p, dC.p, m, N, K, nullptr, true)); // accumulate
    for (auto &x : ref)
        x *= 2.0f;
    CHECK(rel_err(dC.download(), ref) <= TOL);
    HIP_OK(hipDeviceSynchronize());
}

static void test_swiglu_and_expert_down(uint8_t fmt)
{
    const std::string name = std::string("SwiGLUAndExpertDown_") + fmt_name(fmt);
    begin(name.c_str());
    const int N = 512, K = 768;
    auto w = make_weights(fmt, N, K, 41);
    MI355QuantGemmKernel k(fmt, w.data(), N, K, 0);
    const int m = 2;
    auto g = make_floats((size_t)m * K, 42), u = make_floats((size_t)m * K, 43);
    DevBuf<float> dG(g), dU(u), dO((size_t)m * N);
    DeviceTensor G(dG.p, m, K), U(dU.p, m, K), O(dO.p, m, N);
    CHECK(k.multiply_tensor_with_fused_swiglu(&G, &U, &O, m, N, K));
    std::vector<float> act((size_t)m * K);
    qlo_swiglu(g.data(), u.data(), m * K, act.data());
    auto ref = oracle_product(fmt, w, N, K, act.data(), m);
    // expf on the device may differ by an ulp from libm's, which can move a
    // quantised activation by one step: envelope of the path, not bit parity
    const float e = rel_err(dO.download(), ref);
    printf("    swiglu max rel err %.3g\n", e);
    CHECK(e <= 2e-3f);

    // three experts' down projections, each with its own input
    auto w2 = make_weights(fmt, N, K, 44), w3 = make_weights(fmt, N, K, 45);
    MI355QuantGemmKernel k2(fmt, w2.data(), N, K, 0), k3(fmt, w3.data(), N, K, 0);
    auto in = make_floats((size_t)3 * K, 46);
    DevBuf<float> dIn(in), dOut((size_t)3 * N);
    MI355QuantGemmKernel::FusedExpertDownDesc descs[3] = {
        {&k, dIn.p, dOut.p, N}, {&k2, dIn.p + K, dOut.p + N, N}, {&k3, dIn.p + 2 * K, dOut.p + 2 * N, N}};
    CHECK(k.multiply_fused_expert_down(descs, 3, 1, K));
    auto out = dOut.download();
    const std::vector<uint8_t> *ws[3] = {&w, &w2, &w3};
    for (int i = 0; i < 3; ++i)
    {
        auto r = oracle_product(fmt, *ws[i], N, K, in.data() + (size_t)i * K, 1);
        std::vector<float> got(out.begin() + (size_t)i * N, out.begin() + (size_t)(i + 1) * N);
        CHECK(rel_err(got, r) <= TOL);
    }
    HIP_OK(hipDeviceSynchronize());
}

static void test_workspace_and_preuploaded()
{
    begin("BoundWorkspaceAndPreUploadedWeights");
    const uint8_t fmt = LLAM_FMT_Q6_K;
    const int N = 384, K = 512, m = 3;
    auto w = make_weights(fmt, N, K, 51);
    auto owner = std::make_shared<MI355QuantGemmKernel>(fmt, w.data(), N, K, 0);
    DeviceQuantMatrixDesc desc;
    CHECK(owner->exportMatrixDesc(desc) && desc.valid());
    CHECK(desc.n == N && desc.k == K && desc.blocks_per_row == (uint32_t)K / 32 && desc.codebook_id == fmt);
    // a second operator over the same device bytes, keeping the first alive
    MI355QuantGemmKernel k(fmt, desc.weights, N, K, 0, owner);
    CHECK(k.isValid() && k.weights_converted());

    auto a = make_floats((size_t)m * K, 52);
    DevBuf<float> dA(a), dC((size_t)m * N);
    DeviceTensor A(dA.p, m, K), C(dC.p, m, N);
    const size_t need = MI355QuantGemmKernel::getWorkspaceRequirements(m, N, K);
    DevBuf<uint8_t> ws(need + 256);
    DeviceWorkspace tiny{ws.p, 64};
    CHECK(!k.multiply_tensor(&A, &C, m, N, K, true, 1.0f, 0.0f, nullptr, -1, &tiny));
    CHECK(contains(quant_gemm_last_error(), "workspace"));
    k.bindWorkspace(DeviceWorkspace{ws.p + 4, need + 252}); // unaligned base is tolerated
    hipStream_t st;
    HIP_OK(hipStreamCreate(&st));
    k.setGPUStream(st);
    CHECK(k.multiply_tensor(&A, &C, m, N, K, true, 2.0f, 0.0f));
    HIP_OK(hipStreamSynchronize(st));
    auto ref = oracle_product(fmt, w, N, K, a.data(), m);
    for (auto &x : ref)
        x *= 2.0f;
    CHECK(rel_err(dC.download(), ref) <= TOL);
    k.setGPUStream(nullptr);
    HIP_OK(hipStreamDestroy(st));
    k.releaseWeights();
    CHECK(!k.isValid() && !k.multiply_tensor(&A, &C, m, N, K));
}

static void test_registry_end_to_end()
{
    begin("RegistryEndToEnd");
    const int N = 256, K = 512;
    auto w = make_weights(LLAM_FMT_IQ3_S, N, K, 61);
    QuantWeightTensor t{"blk.3.ffn_gate.weight", LLAM_FMT_IQ3_S, w.data(), N, K};
    QuantGemmRegistry reg;
    auto h = reg.prepareGemmHandleLocal(&t, 0);
    reg.registerPreparedGemmHandle(t.name, h);
    MI355QuantGemmKernel *k = reg.gemmKernel(t.name);
    CHECK(k != nullptr);
    k->prepareWeights();
    CHECK(k->weights_converted());
    auto a = make_floats(K, 62);
    DevBuf<float> dA(a), dC(N);
    DeviceTensor A(dA.p, 1, K), C(dC.p, 1, N);
    CHECK(k->multiply_tensor(&A, &C, 1, N, K));
    CHECK(rel_err(dC.download(), oracle_product(LLAM_FMT_IQ3_S, w, N, K, a.data(), 1)) <= TOL);
}

int main(int argc, char **argv)
{
    const bool cpu_only = argc > 1 && strcmp(argv[1], "--cpu") == 0;
    test_invalid_construction();
    test_shape_checks();
    test_workspace_sizes();
    test_registry();
    int ndev = 0;
    const bool have_gpu = hipGetDeviceCount(&ndev) == hipSuccess && ndev > 0;
    if (!have_gpu)
        test_no_device_fails_loudly();
    if (!cpu_only)
    {
        if (!have_gpu)
        {
            printf("no HIP device: the device cases need an MI355X\n");
            return 2;
        }
        for (uint8_t fmt : FORMATS)
        {
            test_multiply_tensor(fmt);
            test_fused_and_verifier_rows(fmt);
            test_weight_handover(fmt);
            test_precomputed_q8_1(fmt);
            test_swiglu_and_expert_down(fmt);
        }
        test_batch_plane();
        test_workspace_and_preuploaded();
        test_registry_end_to_end();
    }
    printf("%s: %d checks, %d failed\n", g_failed ? "FAILED" : "PASSED", g_checks, g_failed);
    return g_failed ? 1 : 0;
}
