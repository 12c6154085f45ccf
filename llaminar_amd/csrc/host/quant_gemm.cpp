// MI355QuantGemmKernel and QuantGemmRegistry: host logic above the C entry points.
// Device memory is touched only through the HIP runtime (allocation, upload) and
// the entry points of ql_api.h (all arithmetic).
#include "llaminar_amd/quant_gemm.hpp"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <stdexcept>

namespace llaminar_amd
{
    namespace
    {
        thread_local char g_error[512] = "";

        bool fail(const char *fn, const char *fmt, ...)
        {
            char msg[400];
            va_list ap;
            va_start(ap, fmt);
            vsnprintf(msg, sizeof msg, fmt, ap);
            va_end(ap);
            snprintf(g_error, sizeof g_error, "[MI355QuantGemmKernel::%s] %s", fn, msg);
            fprintf(stderr, "%s\n", g_error);
            return false;
        }

        // A failed entry point has already printed its reason; keep it as ours too.
        bool forward(const char *fn, bool ok)
        {
            if (!ok)
                snprintf(g_error, sizeof g_error, "[MI355QuantGemmKernel::%s] %s", fn, llam_ql_last_error());
            return ok;
        }

        constexpr size_t ALIGN = 256;
        size_t round_up(size_t b) { return (b + ALIGN - 1) / ALIGN * ALIGN; }
        size_t q8_bytes(int m, int k) { return (size_t)m * (size_t)(k / 32) * sizeof(llam_block_q8_1); }

        bool format_ok(uint8_t fmt) { return llam_format_block_bytes(fmt) != 0; }

        // Fallback scratch when the caller neither passes nor binds a workspace: one
        // grow-only buffer per thread and device, so operators shared between threads
        // never hand two calls the same memory.
        struct OwnScratch
        {
            void *p[16] = {};
            size_t cap[16] = {};
            ~OwnScratch()
            {
                for (int d = 0; d < 16; ++d)
                    if (p[d])
                        (void)hipFree(p[d]);
            }
        };
        thread_local OwnScratch g_own;
    } // namespace

    const char *quant_gemm_last_error() { return g_error; }

    // ---- construction ------------------------------------------------------------

    MI355QuantGemmKernel::MI355QuantGemmKernel(uint8_t fmt, const void *host_gguf, int N, int K, int device_id)
        : fmt_(fmt), N_(N), K_(K), device_id_(device_id), host_gguf_(host_gguf)
    {
        if (!format_ok(fmt))
            fail("ctor", "unsupported weight format id %d", (int)fmt);
        else if (!host_gguf)
            fail("ctor", "null weight pointer");
        else if (N <= 0 || K <= 0 || K % 256 != 0)
            fail("ctor", "bad shape N=%d K=%d (K must be a positive multiple of 256)", N, K);
        else if (device_id < 0 || device_id >= 16)
            fail("ctor", "bad device id %d", device_id);
        else
            valid_ = true;
    }

    MI355QuantGemmKernel::MI355QuantGemmKernel(uint8_t fmt, const void *d_prepared, int N, int K, int device_id,
                                               std::shared_ptr<void> lifetime_owner)
        : fmt_(fmt), N_(N), K_(K), device_id_(device_id), lifetime_owner_(std::move(lifetime_owner))
    {
        if (!format_ok(fmt))
            fail("ctor", "unsupported weight format id %d", (int)fmt);
        else if (!d_prepared)
            fail("ctor", "null device weight pointer");
        else if (N <= 0 || K <= 0 || K % 256 != 0)
            fail("ctor", "bad shape N=%d K=%d (K must be a positive multiple of 256)", N, K);
        else if (device_id < 0 || device_id >= 16)
            fail("ctor", "bad device id %d", device_id);
        else
        {
            d_weights_ = d_prepared;
            valid_ = true;
        }
    }

    MI355QuantGemmKernel::~MI355QuantGemmKernel() { releaseWeights(); }

    void MI355QuantGemmKernel::releaseWeights()
    {
        std::lock_guard<std::mutex> lock(prepare_mutex_);
        drop_plane_locked();
        if (d_owned_)
        {
            (void)hipSetDevice(device_id_);
            (void)hipFree(d_owned_);
        }
        d_owned_ = nullptr;
        d_weights_ = nullptr;
        host_gguf_ = nullptr;
        lifetime_owner_.reset();
        valid_ = false;
    }

    size_t MI355QuantGemmKernel::packedWeightBytes() const
    {
        return (valid_ && (d_weights_ || host_gguf_)) ? llam_ql_prepared_bytes(fmt_, N_, K_) : 0;
    }

    // ---- weight hand-over ----------------------------------------------------------

    MI355PackedWeights::~MI355PackedWeights()
    {
        if (owned_)
        {
            (void)hipSetDevice(device_id_);
            (void)hipFree(owned_);
        }
    }

    std::unique_ptr<MI355PackedWeights> MI355PackedWeights::clone(void *stream) const
    {
        static const char *fn = "MI355PackedWeights::clone";
        if (!d_ || bytes_ == 0)
        {
            fail(fn, "no weights to copy");
            return nullptr;
        }
        if (hipSetDevice(device_id_) != hipSuccess)
        {
            fail(fn, "no HIP device %d", device_id_);
            return nullptr;
        }
        void *copy = nullptr;
        if (hipMalloc(&copy, bytes_) != hipSuccess)
        {
            (void)hipGetLastError();
            fail(fn, "device allocation of %zu bytes failed", bytes_);
            return nullptr;
        }
        hipStream_t st = static_cast<hipStream_t>(stream);
        if (hipMemcpyAsync(copy, d_, bytes_, hipMemcpyDeviceToDevice, st) != hipSuccess ||
            hipStreamSynchronize(st) != hipSuccess)
        {
            (void)hipGetLastError();
            (void)hipFree(copy);
            fail(fn, "device copy of %zu bytes failed", bytes_);
            return nullptr;
        }
        std::unique_ptr<MI355PackedWeights> w(new MI355PackedWeights());
        w->fmt_ = fmt_;
        w->n_ = n_;
        w->k_ = k_;
        w->device_id_ = device_id_;
        w->bytes_ = bytes_;
        w->d_ = copy;
        w->owned_ = copy;
        return w;
    }

    std::unique_ptr<MI355PackedWeights> MI355QuantGemmKernel::detachWeights()
    {
        if (!ready("detachWeights"))
            return nullptr;
        std::lock_guard<std::mutex> lock(prepare_mutex_);
        drop_plane_locked(); // the plane belongs to this operator, not to the weights handed over
        std::unique_ptr<MI355PackedWeights> w(new MI355PackedWeights());
        w->fmt_ = fmt_;
        w->n_ = N_;
        w->k_ = K_;
        w->device_id_ = device_id_;
        w->bytes_ = llam_ql_prepared_bytes(fmt_, N_, K_);
        w->d_ = d_weights_;
        w->owned_ = d_owned_;
        w->keepalive_ = std::move(lifetime_owner_);
        d_owned_ = nullptr;
        d_weights_ = nullptr;
        lifetime_owner_.reset();
        return w; // valid_ stays: the shape is known, attachWeights() makes the operator usable again
    }

    std::unique_ptr<MI355PackedWeights> MI355QuantGemmKernel::cloneWeights()
    {
        if (!ready("cloneWeights"))
            return nullptr;
        MI355PackedWeights view;
        view.fmt_ = fmt_;
        view.n_ = N_;
        view.k_ = K_;
        view.device_id_ = device_id_;
        view.bytes_ = llam_ql_prepared_bytes(fmt_, N_, K_);
        view.d_ = d_weights_; // not owned: the view frees nothing
        return view.clone(stream_);
    }

    bool MI355QuantGemmKernel::attachWeights(std::unique_ptr<MI355PackedWeights> weights)
    {
        static const char *fn = "attachWeights";
        if (!valid_)
            return fail(fn, "operator is not valid");
        if (!weights || !weights->d_)
            return fail(fn, "null weights");
        if (weights->fmt_ != fmt_ || weights->n_ != N_ || weights->k_ != K_ || weights->device_id_ != device_id_)
            return fail(fn, "weights are format %d [%d x %d] on device %d, the operator is format %d [%d x %d] on device %d",
                        (int)weights->fmt_, weights->n_, weights->k_, weights->device_id_, (int)fmt_, N_, K_, device_id_);
        std::lock_guard<std::mutex> lock(prepare_mutex_);
        drop_plane_locked();
        if (d_owned_)
        {
            (void)hipSetDevice(device_id_);
            (void)hipFree(d_owned_);
        }
        d_owned_ = weights->owned_;
        d_weights_ = weights->d_;
        lifetime_owner_ = std::move(weights->keepalive_);
        host_gguf_ = nullptr;
        weights->owned_ = nullptr; // ownership moved
        weights->d_ = nullptr;
        return true;
    }

    KernelSnapshotInfo MI355QuantGemmKernel::getKernelSnapshotInfo() const
    {
        KernelSnapshotInfo info;
        info.kernel_name = "GEMM";
        info.kernel_description = "block-quantized linear projection: C = alpha * A @ W^T + beta * C (+ bias)";
        info.inputs = {{"A", "input activations [m, k]", "FP32"}};
        info.weights = {{"B", "quantized weight matrix [n, k] (GGUF blocks in the prepared device layout)", "INT8"}};
        info.outputs = {{"C", "output matrix [m, n]", "FP32"}};
        info.scalars = {{"N", "output features", "INT32"},
                        {"K", "input features", "INT32"},
                        {"rocm_device_id", "HIP device ID", "INT32"},
                        {"weights_converted", "whether the weights are on the device in the prepared layout", "INT32"}};
        return info;
    }

    // Upload the GGUF bytes and bring them into the prepared layout.  The staging copy
    // is freed again; only the prepared buffer stays.  Runs once.
    void MI355QuantGemmKernel::prepareWeights()
    {
        static const char *fn = "prepareWeights";
        std::lock_guard<std::mutex> lock(prepare_mutex_);
        if (!valid_ || d_weights_ || !host_gguf_) // nothing to upload (also after detachWeights)
            return;
        if (hipSetDevice(device_id_) != hipSuccess)
        {
            fail(fn, "no HIP device %d", device_id_);
            return;
        }
        const size_t raw = (size_t)N_ * (size_t)(K_ / 256) * llam_format_block_bytes(fmt_);
        const size_t prepared = llam_ql_prepared_bytes(fmt_, N_, K_);
        void *d_raw = nullptr, *d_prep = nullptr;
        if (hipMalloc(&d_raw, raw) != hipSuccess || hipMalloc(&d_prep, prepared) != hipSuccess)
        {
            if (d_raw)
                (void)hipFree(d_raw);
            fail(fn, "device allocation of %zu + %zu bytes failed", raw, prepared);
            return;
        }
        hipStream_t st = static_cast<hipStream_t>(stream_);
        bool ok = hipMemcpyAsync(d_raw, host_gguf_, raw, hipMemcpyHostToDevice, st) == hipSuccess;
        ok = ok && forward(fn, llam_ql_prepare_weights(fmt_, d_raw, d_prep, N_, K_, device_id_, stream_));
        ok = ok && hipStreamSynchronize(st) == hipSuccess;
        (void)hipFree(d_raw);
        if (!ok)
        {
            (void)hipFree(d_prep);
            fail(fn, "upload failed");
            return;
        }
        d_owned_ = d_prep;
        d_weights_ = d_prep;
        host_gguf_ = nullptr; // the borrowed bytes are not needed any more
    }

    bool MI355QuantGemmKernel::exportMatrixDesc(DeviceQuantMatrixDesc &out)
    {
        out = {};
        if (!ready("exportMatrixDesc"))
            return false;
        out.weights = d_weights_;
        out.n = N_;
        out.k = K_;
        out.blocks_per_row = (uint32_t)(K_ / 32);
        out.codebook_id = fmt_;
        return true;
    }

    // ---- batch plane ----------------------------------------------------------------

    void MI355QuantGemmKernel::drop_plane_locked()
    {
        if (!d_plane_)
            return;
        (void)hipSetDevice(device_id_);
        (void)hipFree(d_plane_); // waits for the launches that read it
        d_plane_ = nullptr;
    }

    void MI355QuantGemmKernel::dropBatchPlane()
    {
        std::lock_guard<std::mutex> lock(prepare_mutex_);
        drop_plane_locked();
    }

    bool MI355QuantGemmKernel::enableBatchPlane()
    {
        static const char *fn = "enableBatchPlane";
        if (!ready(fn))
            return false;
        std::lock_guard<std::mutex> lock(prepare_mutex_);
        if (d_plane_)
            return true;
        const size_t bytes = llam_ql_batch_plane_bytes(fmt_, N_, K_);
        if (bytes == 0)
            return fail(fn, "format %d [%d x %d] has no batch plane", (int)fmt_, N_, K_);
        void *p = nullptr;
        if (hipSetDevice(device_id_) != hipSuccess || hipMalloc(&p, bytes) != hipSuccess)
            return fail(fn, "hipMalloc of %zu bytes failed", bytes);
        // finished before any launch gets it: a launch on another stream must not read a half-written plane
        if (!llam_ql_build_batch_plane(fmt_, d_weights_, p, N_, K_, device_id_, stream_) ||
            hipStreamSynchronize(static_cast<hipStream_t>(stream_)) != hipSuccess)
        {
            (void)hipFree(p);
            return fail(fn, "%s", llam_ql_last_error());
        }
        d_plane_ = p;
        return true;
    }

    bool MI355QuantGemmKernel::ready(const char *fn)
    {
        if (!valid_)
            return fail(fn, "operator is not valid");
        if (!d_weights_)
            prepareWeights();
        if (!d_weights_)
            return fail(fn, "weights are not on the device");
        return true;
    }

    // ---- workspace -----------------------------------------------------------------

    size_t MI355QuantGemmKernel::getWorkspaceRequirements(int m, int n, int k)
    {
        if (m <= 0 || n <= 0 || k <= 0)
            return 0;
        return round_up(q8_bytes(m, k)) + round_up((size_t)m * n * sizeof(float));
    }

    void *MI355QuantGemmKernel::Scratch::take(size_t bytes)
    {
        bytes = round_up(bytes);
        if (bytes > left)
            return nullptr;
        void *r = p;
        p += bytes;
        left -= bytes;
        return r;
    }

    bool MI355QuantGemmKernel::open_scratch(const char *fn, size_t bytes, DeviceWorkspace *ws, Scratch &s)
    {
        const DeviceWorkspace *use = (ws && ws->base) ? ws : (bound_.base ? &bound_ : nullptr);
        if (use)
        {
            const size_t skew = (ALIGN - (uintptr_t)use->base % ALIGN) % ALIGN;
            if (use->bytes < bytes + skew)
                return fail(fn, "workspace of %zu bytes is smaller than the %zu needed", use->bytes, bytes + skew);
            s.p = static_cast<uint8_t *>(use->base) + skew;
            s.left = use->bytes - skew;
            return true;
        }
        if (g_own.cap[device_id_] < bytes)
        {
            if (hipSetDevice(device_id_) != hipSuccess)
                return fail(fn, "no HIP device %d", device_id_);
            // The old buffer may still be read by work queued earlier on this thread.
            if (g_own.p[device_id_] && (hipDeviceSynchronize() != hipSuccess || hipFree(g_own.p[device_id_]) != hipSuccess))
                return fail(fn, "could not release the previous scratch buffer");
            g_own.p[device_id_] = nullptr;
            g_own.cap[device_id_] = 0;
            if (hipMalloc(&g_own.p[device_id_], bytes) != hipSuccess)
                return fail(fn, "scratch allocation of %zu bytes failed (bind a workspace when allocation is not possible)",
                            bytes);
            g_own.cap[device_id_] = bytes;
        }
        s.p = static_cast<uint8_t *>(g_own.p[device_id_]);
        s.left = g_own.cap[device_id_];
        return true;
    }

    // ---- product ---------------------------------------------------------------------

    // d_C[m x n] (row stride ldc) from quantised activations.
    bool MI355QuantGemmKernel::run(const char *fn, const void *d_q8, float *d_C, int ldc, int m, int n,
                                   const DeviceTensor *bias, float alpha, float beta, Scratch &s,
                                   void *stream)
    {
        auto product = [&](float *dst, int ld) {
            return m <= LLAM_QL_MAX_GEMV_M
                       ? llam_ql_gemv_plane(fmt_, d_weights_, d_plane_, d_q8, dst, m, n, K_, ld, device_id_, stream)
                       : llam_ql_gemm(fmt_, d_weights_, d_q8, dst, m, n, K_, ld, device_id_, stream);
        };
        const float *d_bias = bias ? bias->data : nullptr;
        if (bias && bias->cols * (bias->rows ? bias->rows : 1) < n)
            return fail(fn, "bias has fewer than n=%d elements", n);
        const bool plain = alpha == 1.0f && beta == 0.0f;
        if (plain && (!d_bias || ldc == n))
        {
            if (!forward(fn, product(d_C, ldc)))
                return false;
            // dense C: the bias is added in place (element i is read and written by one lane)
            return !d_bias ||
                   forward(fn, llam_ql_epilogue(d_C, d_C, d_bias, m, n, ldc, 1.0f, 0.0f, device_id_, stream));
        }
        float *tmp = static_cast<float *>(s.take((size_t)m * n * sizeof(float)));
        if (!tmp)
            return fail(fn, "workspace too small for the [%d x %d] intermediate", m, n);
        return forward(fn, product(tmp, n)) &&
               forward(fn, llam_ql_epilogue(d_C, tmp, d_bias, m, n, ldc, alpha, beta, device_id_, stream));
    }

    bool MI355QuantGemmKernel::multiply_tensor(const DeviceTensor *A, DeviceTensor *C, int m, int n, int k,
                                               bool transpose_B, float alpha, float beta, const DeviceTensor *bias,
                                               int device_idx, DeviceWorkspace *workspace, int activation_row_offset)
    {
        static const char *fn = "multiply_tensor";
        (void)transpose_B; // weights are always [N x K], as in the reference operator
        if (device_idx != -1 && device_idx != device_id_)
            return fail(fn, "operator lives on device %d, not %d", device_id_, device_idx);
        if (!A || !C || !A->data || !C->data)
            return fail(fn, "null tensor");
        if (m < 0 || activation_row_offset < 0)
            return fail(fn, "negative size");
        if (n != N_ || k != K_)
            return fail(fn, "Dimension mismatch: requested n=%d k=%d packed N=%d K=%d", n, k, N_, K_);
        if (A->cols < k || C->cols < n || A->rows < activation_row_offset + m || C->rows < m)
            return fail(fn, "tensor smaller than the requested [%d x %d] @ [%d x %d]", m, k, n, k);
        if (A->stride() != k)
            return fail(fn, "activation rows must be dense (stride %d, k %d)", A->stride(), k);
        if (m == 0)
            return true;
        if (!ready(fn))
            return false;
        Scratch s;
        if (!open_scratch(fn, getWorkspaceRequirements(m, n, k), workspace, s))
            return false;
        void *q8 = s.take(q8_bytes(m, k));
        const float *a = A->data + (size_t)activation_row_offset * k;
        // plain decode product: the fp32-input GEMV quantises inside its kernel where that
        // saves the quantiser launch (same bits), else through q8
        if (m <= LLAM_QL_MAX_GEMV_M && alpha == 1.0f && beta == 0.0f && !bias)
        {
            const llam_ql_proj one{d_weights_, C->data, n, C->stride(), fmt_, d_plane_};
            return forward(fn, llam_ql_gemv_fused_f32(&one, 1, a, k, m, k, q8, device_id_, stream_));
        }
        return forward(fn, llam_ql_quantize_q8_1(a, q8, m, k, device_id_, stream_)) &&
               run(fn, q8, C->data, C->stride(), m, n, bias, alpha, beta, s, stream_);
    }

    size_t MI355QuantGemmKernel::get_quantized_activation_buffer_size(int m, int k) const
    {
        return (m > 0 && k > 0 && k % 32 == 0) ? q8_bytes(m, k) : 0;
    }

    bool MI355QuantGemmKernel::quantize_activations(const float *d_A, void *d_q8_1, int m, int k)
    {
        static const char *fn = "quantize_activations";
        if (!valid_)
            return fail(fn, "operator is not valid");
        return forward(fn, llam_ql_quantize_q8_1(d_A, d_q8_1, m, k, device_id_, stream_));
    }

    bool MI355QuantGemmKernel::multiply_with_precomputed_q8_1(const void *d_q8_1, float *d_C, int m, int n, int k,
                                                              const DeviceTensor *bias, bool accumulate, float alpha,
                                                              float beta, int device_idx, DeviceWorkspace *workspace)
    {
        static const char *fn = "multiply_with_precomputed_q8_1";
        if (device_idx != -1 && device_idx != device_id_)
            return fail(fn, "operator lives on device %d, not %d", device_id_, device_idx);
        if (!d_q8_1 || !d_C)
            return fail(fn, "null pointer");
        if (n != N_ || k != K_)
            return fail(fn, "Dimension mismatch: requested n=%d k=%d packed N=%d K=%d", n, k, N_, K_);
        if (m < 0)
            return fail(fn, "negative size");
        if (m == 0)
            return true;
        if (!ready(fn))
            return false;
        if (accumulate)
            beta = 1.0f;
        Scratch s;
        const bool direct = alpha == 1.0f && beta == 0.0f;
        if (!direct && !open_scratch(fn, round_up((size_t)m * n * sizeof(float)), workspace, s))
            return false;
        return run(fn, d_q8_1, d_C, n, m, n, bias, alpha, beta, s, stream_);
    }

    bool MI355QuantGemmKernel::multiply_fused_tensor(const DeviceTensor *input,
                                                     const std::vector<TensorProjectionDesc> &projections, int m,
                                                     int k, DeviceWorkspace *workspace)
    {
        static const char *fn = "multiply_fused_tensor";
        if (!input || !input->data)
            return fail(fn, "null input");
        if (projections.empty())
            return true;
        if ((int)projections.size() > LLAM_QL_MAX_FUSED)
            return fail(fn, "%zu projections, at most %d", projections.size(), LLAM_QL_MAX_FUSED);
        if (m < 0 || input->rows < m || input->cols < k || input->stride() != k)
            return fail(fn, "input is not a dense [%d x %d] matrix", m, k);
        size_t tmp_bytes = 0;
        for (const auto &p : projections)
        {
            if (!p.kernel || !p.output || !p.output->data)
                return fail(fn, "invalid projection%s%s", p.name ? " " : "", p.name ? p.name : "");
            if (p.kernel->device_id_ != device_id_)
                return fail(fn, "projection on device %d, input operator on %d", p.kernel->device_id_, device_id_);
            if (p.kernel->K_ != k || p.n != p.kernel->N_)
                return fail(fn, "Dimension mismatch: projection n=%d k=%d packed N=%d K=%d", p.n, k, p.kernel->N_,
                            p.kernel->K_);
            if (p.output->rows < m || p.output->cols < p.n)
                return fail(fn, "output smaller than [%d x %d]", m, p.n);
            if (!p.kernel->ready(fn))
                return false;
            if (p.bias && p.output->stride() != p.n)
                tmp_bytes = std::max(tmp_bytes, round_up((size_t)m * p.n * sizeof(float)));
        }
        if (m == 0)
            return true;
        Scratch s;
        if (!open_scratch(fn, round_up(q8_bytes(m, k)) + tmp_bytes, workspace, s))
            return false;
        void *q8 = s.take(q8_bytes(m, k));

        bool any_bias = false;
        for (const auto &p : projections)
            any_bias = any_bias || p.bias;
        if (m <= LLAM_QL_MAX_GEMV_M && !any_bias)
        {
            llam_ql_proj projs[LLAM_QL_MAX_FUSED];
            for (size_t i = 0; i < projections.size(); ++i)
            {
                const auto &p = projections[i];
                projs[i].d_w = p.kernel->d_weights_;
                projs[i].d_y = p.output->data;
                projs[i].N = p.n;
                projs[i].ldy = p.output->stride();
                projs[i].fmt = p.kernel->fmt_;
                projs[i].d_plane = p.kernel->d_plane_;
            }
            return forward(fn, llam_ql_gemv_fused_f32(projs, (int)projections.size(), input->data, k, m, k, q8,
                                                      device_id_, stream_));
        }
        if (!forward(fn, llam_ql_quantize_q8_1(input->data, q8, m, k, device_id_, stream_)))
            return false;
        for (const auto &p : projections)
        {
            Scratch each = s; // the intermediate, if any, is reused by every projection
            if (!p.kernel->run(fn, q8, p.output->data, p.output->stride(), m, p.n, p.bias, 1.0f, 0.0f, each, stream_))
                return false;
        }
        return true;
    }

    bool MI355QuantGemmKernel::multiply_fused_verifier_rows_decode_equivalent(
        const DeviceTensor *input, const std::vector<TensorProjectionDesc> &projections, int m, int k,
        DeviceWorkspace *workspace)
    {
        static const char *fn = "multiply_fused_verifier_rows_decode_equivalent";
        // A row is bit-identical to its m == 1 result when the launcher serves both batch sizes
        // with the same kernel on the same row partition and K slices: asked of the launcher
        // itself, per projection (llam_ql_gemv_describe reports the plan llam_ql_gemv executes).
        if (m < 1 || m > 4)
            return fail(fn, "m=%d is outside the decode-equivalent range 1..4", m);
        for (const auto &p : projections)
        {
            if (!p.kernel)
                return fail(fn, "null projection kernel");
            llam_ql_gemv_plan plan;
            if (!forward(fn, llam_ql_gemv_describe(p.kernel->fmt_, m, p.n, k, p.kernel->d_plane_ != nullptr, device_id_, &plan)))
                return false;
            if (!plan.decode_equivalent)
                return fail(fn, "m=%d n=%d k=%d (format %d) is not served like m=1: rows would differ in the last bits",
                            m, p.n, k, (int)p.kernel->fmt_);
        }
        return multiply_fused_tensor(input, projections, m, k, workspace);
    }

    bool MI355QuantGemmKernel::multiply_tensor_with_fused_swiglu(const DeviceTensor *gate, const DeviceTensor *up,
                                                                 DeviceTensor *output, int m, int n, int k,
                                                                 float alpha, float beta, DeviceWorkspace *workspace)
    {
        static const char *fn = "multiply_tensor_with_fused_swiglu";
        if (!gate || !up || !output || !gate->data || !up->data || !output->data)
            return fail(fn, "null tensor");
        if (n != N_ || k != K_)
            return fail(fn, "Dimension mismatch: requested n=%d k=%d packed N=%d K=%d", n, k, N_, K_);
        if (m < 0 || gate->rows < m || up->rows < m || output->rows < m || gate->cols < k || up->cols < k ||
            output->cols < n || gate->stride() != k || up->stride() != k)
            return fail(fn, "gate/up must be dense [%d x %d], output at least [%d x %d]", m, k, m, n);
        if (m == 0)
            return true;
        if (!ready(fn))
            return false;
        Scratch s;
        if (!open_scratch(fn, getWorkspaceRequirements(m, n, k), workspace, s))
            return false;
        void *q8 = s.take(q8_bytes(m, k));
        if (m <= LLAM_QL_MAX_GEMV_M && alpha == 1.0f && beta == 0.0f)
            return forward(fn, llam_ql_gemv_swiglu_f32(fmt_, d_weights_, d_plane_, gate->data, up->data, k, output->data, m, n,
                                                       k, output->stride(), q8, device_id_, stream_));
        return forward(fn, llam_ql_swiglu_quantize(gate->data, up->data, nullptr, q8, m, k, device_id_, stream_)) &&
               run(fn, q8, output->data, output->stride(), m, n, nullptr, alpha, beta, s, stream_);
    }

    bool MI355QuantGemmKernel::multiply_fused_expert_down(const FusedExpertDownDesc *descs, int num_descs, int m,
                                                          int k)
    {
        static const char *fn = "multiply_fused_expert_down";
        if (m != 1)
            return fail(fn, "m=%d: only single-token decode is fused", m);
        if (num_descs < 0 || (num_descs > 0 && !descs))
            return fail(fn, "bad descriptor array");
        for (int i = 0; i < num_descs; ++i)
        {
            const auto &d = descs[i];
            if (!d.kernel || !d.input || !d.output)
                return fail(fn, "descriptor %d is incomplete", i);
            if (d.kernel->K_ != k || d.n != d.kernel->N_ || d.kernel->device_id_ != device_id_)
                return fail(fn, "Dimension mismatch: descriptor %d n=%d k=%d packed N=%d K=%d", i, d.n, k,
                            d.kernel->N_, d.kernel->K_);
            if (!d.kernel->ready(fn))
                return false;
        }
        if (num_descs == 0)
            return true;
        Scratch s;
        if (!open_scratch(fn, (size_t)num_descs * round_up(q8_bytes(1, k)), nullptr, s))
            return false;
        for (int i = 0; i < num_descs; ++i)
        {
            const auto &d = descs[i];
            void *q8 = s.take(q8_bytes(1, k));
            if (!forward(fn, llam_ql_quantize_q8_1(d.input, q8, 1, k, device_id_, stream_)) ||
                !forward(fn, llam_ql_gemv(d.kernel->fmt_, d.kernel->d_weights_, q8, d.output, 1, d.n, k, d.n,
                                          device_id_, stream_)))
                return false;
        }
        return true;
    }

    // ---- registry ----------------------------------------------------------------------

    std::shared_ptr<PreparedGemmHandle> QuantGemmRegistry::prepareGemmHandleLocal(const QuantWeightTensor *tensor,
                                                                                 int device_id,
                                                                                 GemmPreparationKind kind)
    {
        if (!tensor)
            throw std::runtime_error("QuantGemmRegistry::prepareGemmHandleLocal: null tensor");
        if (!format_ok(tensor->fmt))
            throw std::runtime_error("QuantGemmRegistry::prepareGemmHandleLocal: tensor '" + tensor->name +
                                     "' has an unsupported weight format");
        std::lock_guard<std::mutex> lock(cache_mutex_);
        auto key = std::make_pair(tensor, device_id);
        auto it = handles_.find(key);
        if (it != handles_.end())
            return it->second;
        auto weights = std::make_shared<PreparedGemmWeights>();
        weights->kind = GemmPreparationKind::MI355_NATIVE_BLOCKS;
        weights->owned_kernel =
            std::make_shared<MI355QuantGemmKernel>(tensor->fmt, tensor->host_gguf, tensor->n, tensor->k, device_id);
        weights->kernel = weights->owned_kernel.get();
        if (!weights->kernel->isValid())
            throw std::runtime_error("QuantGemmRegistry::prepareGemmHandleLocal: tensor '" + tensor->name +
                                     "' cannot be prepared: " + quant_gemm_last_error());
        (void)kind; // AUTO and MI355_NATIVE_BLOCKS are the same thing here
        auto handle = std::make_shared<PreparedGemmHandle>();
        handle->tensor = tensor;
        handle->device_id = device_id;
        handle->kind = weights->kind;
        handle->variant = tensor->fmt;
        handle->prepared_weights = std::move(weights);
        handles_[key] = handle;
        return handle;
    }

    MI355QuantGemmKernel *QuantGemmRegistry::getOrCreateGemmEngine(const PreparedGemmHandle *prepared)
    {
        if (!prepared || !prepared->prepared_weights)
            return nullptr;
        return prepared->prepared_weights->kernel;
    }

    void QuantGemmRegistry::registerPreparedGemmHandle(const std::string &ref, std::shared_ptr<PreparedGemmHandle> handle)
    {
        if (!handle)
            throw std::runtime_error("QuantGemmRegistry::registerPreparedGemmHandle: null handle for '" + ref + "'");
        std::lock_guard<std::mutex> lock(cache_mutex_);
        by_ref_[ref] = std::move(handle);
    }

    MI355QuantGemmKernel *QuantGemmRegistry::gemmKernel(const std::string &ref)
    {
        std::lock_guard<std::mutex> lock(cache_mutex_);
        auto it = by_ref_.find(ref);
        return it == by_ref_.end() ? nullptr : getOrCreateGemmEngine(it->second.get());
    }

    void QuantGemmRegistry::registerEngine(int device, int layer, int expert, ExpertRole role,
                                           std::shared_ptr<MI355QuantGemmKernel> e)
    {
        std::unique_lock<std::shared_mutex> lock(expert_mutex_);
        experts_[std::make_tuple(device, layer, expert, (int)role)] = std::move(e);
    }

    MI355QuantGemmKernel *QuantGemmRegistry::getEngine(int device, int layer, int expert, ExpertRole role)
    {
        std::shared_lock<std::shared_mutex> lock(expert_mutex_);
        auto it = experts_.find(std::make_tuple(device, layer, expert, (int)role));
        return it == experts_.end() ? nullptr : it->second.get();
    }

    size_t QuantGemmRegistry::size()
    {
        std::lock_guard<std::mutex> lock(cache_mutex_);
        std::shared_lock<std::shared_mutex> elock(expert_mutex_);
        return handles_.size() + experts_.size();
    }

    void QuantGemmRegistry::clear()
    {
        std::lock_guard<std::mutex> lock(cache_mutex_);
        std::unique_lock<std::shared_mutex> elock(expert_mutex_);
        by_ref_.clear();
        handles_.clear();
        experts_.clear();
    }
} // namespace llaminar_amd
