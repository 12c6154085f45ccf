// Tests of MI355MoEKernel (the decode methods of the reference's IMoEKernel over device
// memory): descriptor tables, routing from the router matrix, grouped gate/up and down
// projections, the fused decode sequence, the shared-expert gate -- against the CPU
// oracle on the same inputs.
//
//   test_moe_kernel --cpu   host logic only (no device needed)
//   test_moe_kernel         everything (needs an MI355X)
#include "llaminar_amd/moe_kernel.hpp"
#include "ql_oracle.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <random>
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

static float rel_err(const std::vector<float> &a, const std::vector<float> &b)
{
    float e = 0, m = 0;
    for (size_t i = 0; i < a.size(); ++i)
    {
        e = std::max(e, std::fabs(a[i] - b[i]));
        m = std::max(m, std::fabs(b[i]));
    }
    return e / std::max(m, 1e-30f);
}

// ---- host logic --------------------------------------------------------------------------------
static void test_host_logic()
{
    begin("host logic");
    MI355MoEKernel bad(-1);
    CHECK(!bad.isValid());
    CHECK(contains(moe_kernel_last_error(), "bad device id"));
    MI355MoEKernel k(0);
    CHECK(k.isValid() && k.supports_device(0) && !k.supports_device(1));
    CHECK(MI355MoEKernel::getWorkspaceRequirements(0, 9, 2048, 512, 256) == 0);
    const size_t ws = MI355MoEKernel::getWorkspaceRequirements(1, 9, 2048, 512, 256);
    // logits 1 KiB, Q8_1 hidden 2304 B, gate and up 18 KiB each, Q8_1 activations 5184 B, each rounded to 256
    // logits, Q8_1 hidden, gate and up rows, Q8_1 SwiGLU, pair table, per-pair down rows, ids and weights
    CHECK(ws == 1024 + 2304 + 2 * 18432 + 5376 + 256 + 73728 + 2 * 256);
    DeviceQuantMatrixDesc d[2];
    CHECK(k.uploadGroupedExpertDownDescriptorTable(nullptr, 2, 512, 256) == -1);
    CHECK(k.uploadGroupedExpertDownDescriptorTable(d, 2, 500, 256) == -1 && contains(moe_kernel_last_error(), "bad shape"));
    CHECK(k.uploadGroupedExpertDownDescriptorTable(d, 2, 512, 256) == -1 &&
          contains(moe_kernel_last_error(), "no valid expert"));
    d[0].weights = reinterpret_cast<const void *>(0x1000);
    d[0].n = 100;
    d[0].k = 256;
    d[0].blocks_per_row = 8;
    d[0].codebook_id = LLAM_FMT_Q4_K;
    CHECK(k.uploadGroupedExpertDownDescriptorTable(d, 2, 512, 256) == -1 && contains(moe_kernel_last_error(), "expected 512 x 256"));
    DeviceMoELayerRuntime rt;
    DeviceTensor h(reinterpret_cast<float *>(0x1000), 1, 512), o(reinterpret_cast<float *>(0x2000), 1, 512);
    CHECK(!k.groupedExpertDecodeFromRuntime(&rt, &h, 0, 0, 2, &o, 512, 256));
    CHECK(contains(moe_kernel_last_error(), "descriptor table id 0 outside"));
    CHECK(!k.decodeRouteSelect(&rt, &h, &h, 512, 1, 1, true) && contains(moe_kernel_last_error(), "no top-k buffers"));
    CHECK(k.tableCount() == 0);
}

// ---- device ------------------------------------------------------------------------------------------
static void test_decode(uint8_t fmt, int T)
{
    static char name[96];
    snprintf(name, sizeof name, "decode %s, %d token(s)", fmt == LLAM_FMT_Q4_K ? "Q4_K" : "IQ3_S", T);
    begin(name);
    const int D = 512, I = 256, E = 6, TOPK = 2, SLOTS = TOPK + 1; // slot 2: the shared expert (entry E)
    std::vector<std::vector<uint8_t>> wg, wu, wd;
    std::vector<std::unique_ptr<MI355QuantGemmKernel>> eg, eu, ed;
    std::vector<DeviceQuantMatrixDesc> dg(E + 1), du(E + 1), dd(E + 1);
    for (int e = 0; e <= E; ++e)
    {
        wg.push_back(make_weights(fmt, I, D, 100 + e));
        wu.push_back(make_weights(fmt, I, D, 200 + e));
        wd.push_back(make_weights(fmt, D, I, 300 + e));
        eg.emplace_back(new MI355QuantGemmKernel(fmt, wg[e].data(), I, D, 0));
        eu.emplace_back(new MI355QuantGemmKernel(fmt, wu[e].data(), I, D, 0));
        ed.emplace_back(new MI355QuantGemmKernel(fmt, wd[e].data(), D, I, 0));
        CHECK(eg[e]->exportMatrixDesc(dg[e]) && eu[e]->exportMatrixDesc(du[e]) && ed[e]->exportMatrixDesc(dd[e]));
    }
    dg[1] = du[1] = dd[1] = DeviceQuantMatrixDesc(); // expert 1 lives elsewhere: its slots are skipped
    MI355MoEKernel k(0);
    const int tg = k.uploadGroupedExpertGateUpDescriptorTables(dg.data(), du.data(), E + 1, D, I);
    const int td = k.uploadGroupedExpertDownDescriptorTable(dd.data(), E + 1, D, I);
    CHECK(tg == 0 && td == 1 && k.tableCount() == 2);

    const std::vector<float> hidden = make_floats((size_t)T * D, 7 + T);
    const std::vector<float> gate_w = make_floats((size_t)E * D, 8, 0.05f);
    DevBuf<float> d_hidden(hidden), d_gate_w(gate_w), d_out((size_t)T * D), d_out2((size_t)T * D);
    DevBuf<float> d_gate((size_t)T * SLOTS * I), d_up((size_t)T * SLOTS * I);
    DevBuf<int32_t> d_ids(std::vector<int32_t>((size_t)T * SLOTS, E)); // shared expert in every last slot
    DevBuf<float> d_w(std::vector<float>((size_t)T * SLOTS, 1.0f));
    DevBuf<uint8_t> d_ws(MI355MoEKernel::getWorkspaceRequirements(T, SLOTS, D, I, E));
    k.bindWorkspace(DeviceWorkspace{d_ws.p, d_ws.n});
    DeviceMoELayerRuntime rt;
    rt.topk_expert_ids = d_ids.p;
    rt.topk_weights = d_w.p;
    rt.slot_stride = SLOTS;
    DeviceTensor th(d_hidden.p, T, D), tw(d_gate_w.p, E, D), to(d_out.p, T, D), to2(d_out2.p, T, D);

    // routing: logits on the device against the oracle's router on double-accumulated logits
    CHECK(k.decodeRouteSelect(&rt, &th, &tw, D, E, TOPK, true));
    const std::vector<int32_t> ids = d_ids.download();
    const std::vector<float> w = d_w.download();
    std::vector<float> logits((size_t)T * E);
    for (int t = 0; t < T; ++t)
        for (int e = 0; e < E; ++e)
        {
            double a = 0;
            for (int c = 0; c < D; ++c)
                a += (double)hidden[(size_t)t * D + c] * (double)gate_w[(size_t)e * D + c];
            logits[(size_t)t * E + e] = (float)a;
        }
    std::vector<int32_t> oids((size_t)T * TOPK);
    std::vector<float> ow((size_t)T * TOPK), probs((size_t)T * E);
    qlo_moe_route(logits.data(), T, E, TOPK, 1, oids.data(), ow.data(), probs.data());
    for (int t = 0; t < T; ++t)
    {
        for (int s = 0; s < TOPK; ++s)
        {
            CHECK(ids[(size_t)t * SLOTS + s] == oids[(size_t)t * TOPK + s]);
            CHECK(std::fabs(w[(size_t)t * SLOTS + s] - ow[(size_t)t * TOPK + s]) <= 1e-5f);
        }
        CHECK(ids[(size_t)t * SLOTS + TOPK] == E && w[(size_t)t * SLOTS + TOPK] == 1.0f); // left alone
    }

    // fused sequence == staged calls, bit for bit
    CHECK(k.groupedExpertDecodeFromRuntime(&rt, &th, tg, td, SLOTS, &to, D, I));
    CHECK(k.groupedExpertGateUpDecodeFromRuntime(&rt, &th, tg, SLOTS, d_gate.p, d_up.p, D, I));
    CHECK(k.groupedExpertDownDecodeFromRuntime(d_gate.p, d_up.p, &rt, td, SLOTS, &to2, D, I));
    const std::vector<float> out = d_out.download(), out2 = d_out2.download();
    CHECK(memcmp(out.data(), out2.data(), out.size() * 4) == 0);

    // against the oracle chain (SwiGLU through the accurate expf on both sides)
    std::vector<float> ref((size_t)T * D, 0.0f);
    for (int t = 0; t < T; ++t)
    {
        std::vector<llam_block_q8_1> q8(D / 32);
        qlo_quantize_q8_1(hidden.data() + (size_t)t * D, 1, D, q8.data());
        for (int s = 0; s < SLOTS; ++s)
        {
            const int e = ids[(size_t)t * SLOTS + s];
            if (e == 1)
                continue; // not on this device
            std::vector<float> g(I), u(I), act(I), dn(D);
            qlo_gemm_rows(fmt, wg[e].data(), D, 0, I, q8.data(), 1, g.data(), I, nullptr, 0);
            qlo_gemm_rows(fmt, wu[e].data(), D, 0, I, q8.data(), 1, u.data(), I, nullptr, 0);
            qlo_swiglu(g.data(), u.data(), I, act.data());
            std::vector<llam_block_q8_1> qa(I / 32);
            qlo_quantize_q8_1(act.data(), 1, I, qa.data());
            qlo_gemm_rows(fmt, wd[e].data(), I, 0, D, qa.data(), 1, dn.data(), D, nullptr, 0);
            for (int c = 0; c < D; ++c)
                ref[(size_t)t * D + c] += w[(size_t)t * SLOTS + s] * dn[c];
        }
    }
    CHECK(rel_err(out, ref) <= (fmt == LLAM_FMT_IQ3_S ? 1e-2f : 1e-3f));
    int skipped = 0;
    for (int32_t id : ids)
        skipped += id == 1;
    printf("  (%d slot(s) routed to the absent expert)\n", skipped);

    // shared-expert gate: out += sigmoid(dot(gate_inp, hidden)) * shared
    const std::vector<float> gate_inp = make_floats(D, 99, 0.05f), shared = make_floats((size_t)T * D, 98);
    DevBuf<float> d_gi(gate_inp), d_sh(shared);
    DeviceTensor tsh(d_sh.p, T, D);
    CHECK(k.sharedExpertGateAdd(&to, &tsh, &th, d_gi.p, T, D));
    const std::vector<float> out3 = d_out.download();
    std::vector<float> ref3 = out;
    for (int t = 0; t < T; ++t)
    {
        double dot = 0;
        for (int c = 0; c < D; ++c)
            dot += (double)gate_inp[c] * (double)hidden[(size_t)t * D + c];
        const double g = 1.0 / (1.0 + std::exp(-dot));
        for (int c = 0; c < D; ++c)
            ref3[(size_t)t * D + c] += (float)(g * shared[(size_t)t * D + c]);
    }
    CHECK(rel_err(out3, ref3) <= 1e-5f);

    // IMoEKernel::route: the same routing with the result on the host, probabilities included
    {
        MoERoutingResult rr;
        CHECK(k.route(d_hidden.p, d_gate_w.p, T, D, E, TOPK, true, rr));
        CHECK(rr.expert_indices.size() == (size_t)T * TOPK && rr.router_logits.size() == (size_t)T * E);
        for (int t = 0; t < T; ++t)
        {
            for (int s = 0; s < TOPK; ++s)
            {
                CHECK(rr.expert_indices[(size_t)t * TOPK + s] == oids[(size_t)t * TOPK + s]);
                CHECK(std::fabs(rr.expert_weights[(size_t)t * TOPK + s] - ow[(size_t)t * TOPK + s]) <= 1e-5f);
            }
            for (int e = 0; e < E; ++e)
                CHECK(std::fabs(rr.router_logits[(size_t)t * E + e] - probs[(size_t)t * E + e]) <= 1e-5f);
        }
    }

    // single-token calls driven by host ids (FromTable) and by fp32 device routing tensors
    // (FromRouting): the bits of the FromRuntime calls on token 0
    {
        std::vector<int> hid(SLOTS);
        std::vector<float> hw(SLOTS), fidx(SLOTS);
        for (int s = 0; s < SLOTS; ++s)
        {
            hid[s] = ids[s];
            hw[s] = w[s];
            fidx[s] = (float)ids[s];
        }
        DevBuf<float> d_fidx(fidx), d_fw(hw), g1((size_t)SLOTS * I), u1((size_t)SLOTS * I), g2((size_t)SLOTS * I),
            u2((size_t)SLOTS * I), o1(D), o2(D), o0(D), g0((size_t)SLOTS * I), u0((size_t)SLOTS * I);
        DevBuf<int32_t> d_ids0(std::vector<int32_t>(ids.begin(), ids.begin() + SLOTS));
        DeviceMoELayerRuntime rt0;
        rt0.topk_expert_ids = d_ids0.p;
        rt0.topk_weights = d_fw.p;
        rt0.slot_stride = SLOTS;
        DeviceTensor th0(d_hidden.p, 1, D), to0(o0.p, 1, D), to1(o1.p, 1, D), to2b(o2.p, 1, D);
        CHECK(k.groupedExpertGateUpDecodeFromRuntime(&rt0, &th0, tg, SLOTS, g0.p, u0.p, D, I));
        CHECK(k.groupedExpertDownDecodeFromRuntime(g0.p, u0.p, &rt0, td, SLOTS, &to0, D, I));
        CHECK(k.groupedExpertGateUpDecodeFromTable(&th0, hid.data(), tg, SLOTS, g1.p, u1.p, D, I));
        CHECK(k.groupedExpertDownDecodeFromTable(g1.p, u1.p, hid.data(), hw.data(), td, SLOTS, &to1, D, I));
        CHECK(k.groupedExpertGateUpDecodeFromRouting(&th0, d_fidx.p, tg, SLOTS, g2.p, u2.p, D, I));
        CHECK(k.groupedExpertDownDecodeFromRouting(g2.p, u2.p, d_fidx.p, d_fw.p, td, SLOTS, &to2b, D, I));
        const std::vector<float> a0 = o0.download(), a1 = o1.download(), a2 = o2.download();
        CHECK(memcmp(a0.data(), a1.data(), a0.size() * 4) == 0);
        CHECK(memcmp(a0.data(), a2.data(), a0.size() * 4) == 0);
        CHECK(memcmp(a0.data(), out.data(), a0.size() * 4) == 0); // token 0 of the batch
        // weightedAdd: o1 += 0.25 * o2
        CHECK(k.weightedAdd(o1.p, o2.p, 0.25f, D));
        const std::vector<float> a3 = o1.download();
        float worst = 0.0f;
        for (int c = 0; c < D; ++c)
            worst = std::max(worst, std::fabs(a3[c] - (a1[c] + 0.25f * a2[c])));
        CHECK(worst <= 1e-6f * std::max(1.0f, std::fabs(a1[0])) + 1e-5f);

        // the token-batching helpers of the interface: gather two rows of o0's buffer (one token
        // here, so index 0 twice), scatter them back with weights, gate and SwiGLU in place
        const std::vector<int> idx = {0, 0};
        const std::vector<float> ws = {0.5f, 0.25f};
        DevBuf<int> d_idx(idx);
        DevBuf<float> d_ws(ws), d_batch((size_t)2 * D);
        CHECK(k.gatherTokenBatch(o0.p, d_batch.p, d_idx.p, 2, D, 1));
        const std::vector<float> gb = d_batch.download();
        CHECK(memcmp(gb.data(), a0.data(), D * 4) == 0 && memcmp(gb.data() + D, a0.data(), D * 4) == 0);
        CHECK(k.scatterAddWeighted(o2.p, d_batch.p, d_idx.p, d_ws.p, 2, D, 1));
        const std::vector<float> a4 = o2.download();
        worst = 0.0f;
        for (int c = 0; c < D; ++c)
            worst = std::max(worst, std::fabs(a4[c] - (a2[c] + 0.75f * a0[c])));
        CHECK(worst <= 1e-5f * std::max(1.0f, std::fabs(a2[0])) + 1e-5f);
        CHECK(!k.gatherTokenBatch(nullptr, d_batch.p, d_idx.p, 2, D, 1));
        CHECK(contains(moe_kernel_last_error(), "null pointer"));
    }

    // errors keep their reason
    CHECK(!k.groupedExpertDecodeFromRuntime(&rt, &th, td, td, SLOTS, &to, D, I));
    CHECK(contains(moe_kernel_last_error(), "holds no gate/up"));
    CHECK(!k.groupedExpertDecodeFromRuntime(&rt, &th, tg, td, TOPK, &to, D, I));
    CHECK(contains(moe_kernel_last_error(), "must cover"));
}

int main(int argc, char **argv)
{
    const bool cpu_only = argc > 1 && std::string(argv[1]) == "--cpu";
    test_host_logic();
    if (!cpu_only)
    {
        test_decode(LLAM_FMT_Q4_K, 1);
        test_decode(LLAM_FMT_Q4_K, 5);
        test_decode(LLAM_FMT_IQ3_S, 3);
        test_decode(LLAM_FMT_IQ3_S, 100); // 300 (token, slot) pairs: the fused sequence groups tokens by expert
    }
    printf("%d checks, %d failed\n%s\n", g_checks, g_failed, g_failed ? "FAILED" : "PASSED");
    return g_failed ? 1 : 0;
}
