// Host-side operator for the MI355X quantized-linear path.
//
// MI355QuantGemmKernel carries the method set the reference's stages call on an
// ITensorGemm (tensors/TensorKernels.h:348-1427) as implemented by its CPU
// operator CPUNativeVNNIGemmKernel (kernels/cpu/native_vnni/CPUNativeVNNIGemmKernel.h:42-1422):
// same method names, argument meaning and bool error convention, over tensors
// that live in device memory.  Every method only enqueues work on the stream set
// with setGPUStream(); nothing synchronises and, once a workspace is bound,
// nothing allocates.
//
// QuantGemmRegistry mirrors the prepared-GEMM registry the stages resolve their
// operator from (kernels/KernelFactory.h:1225-1330, loaders/PreparedWeightStore.h:68-79,
// loaders/ExpertGemmRegistry.h:43-120).
//
// The class sits on top of the C entry points in ql_api.h and adds no arithmetic.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <shared_mutex>
#include <string>
#include <tuple>
#include <vector>

#include "llaminar_amd/ql_api.h"

namespace llaminar_amd
{
    // fp32 row-major matrix in device memory: what the reference passes as TensorBase.
    struct DeviceTensor
    {
        float *data = nullptr;
        int rows = 0;
        int cols = 0;
        int ld = 0; // elements between rows; 0 means cols

        DeviceTensor() = default;
        DeviceTensor(float *d, int r, int c, int l = 0) : data(d), rows(r), cols(c), ld(l) {}
        int stride() const { return ld ? ld : cols; }
    };

    // Caller-owned device scratch (the role of the reference's DeviceWorkspaceManager,
    // interfaces/IWorkspaceConsumer.h:60-136).
    struct DeviceWorkspace
    {
        void *base = nullptr;
        size_t bytes = 0;
    };

    // What a grouped MoE launch needs to address one matrix (the role of
    // DeviceNativeVNNIMatrixDesc, tensors/TensorKernels.h:39-55).
    struct DeviceQuantMatrixDesc
    {
        const void *weights = nullptr; // prepared layout of ql_api.h
        int n = 0;
        int k = 0;
        uint32_t blocks_per_row = 0; // 32-column blocks
        uint8_t codebook_id = 0;     // llam_weight_format
        uint8_t reserved[3] = {0, 0, 0};
        bool valid() const { return weights && n > 0 && k > 0 && blocks_per_row > 0; }
    };

    // Reason of the calling thread's last failed operator or registry call.
    const char *quant_gemm_last_error();

    // Prepared weights outside an operator: what detachWeights() hands over, cloneWeights()
    // copies and attachWeights() takes (the reference's transferable packed weights,
    // kernels/IPackedWeights.h:62-130: format, shape, size, deep copy).  Device memory in the
    // prepared layout of llam_ql_prepare_weights, owned (freed with the object) or kept alive
    // by a shared owner.
    class MI355PackedWeights
    {
    public:
        ~MI355PackedWeights();
        MI355PackedWeights(const MI355PackedWeights &) = delete;
        MI355PackedWeights &operator=(const MI355PackedWeights &) = delete;

        uint8_t format() const { return fmt_; } // llam_weight_format
        int N() const { return n_; }
        int K() const { return k_; }
        int device() const { return device_id_; }
        size_t sizeBytes() const { return bytes_; }
        const void *data() const { return d_; }
        // Deep copy on the same device (stream-ordered copy, synchronised before it returns);
        // null when the allocation or the copy fails.
        std::unique_ptr<MI355PackedWeights> clone(void *stream = nullptr) const;

    private:
        friend class MI355QuantGemmKernel;
        MI355PackedWeights() = default;
        uint8_t fmt_ = 0;
        int n_ = 0, k_ = 0, device_id_ = 0;
        size_t bytes_ = 0;
        const void *d_ = nullptr;
        void *owned_ = nullptr;
        std::shared_ptr<void> keepalive_;
    };

    // What a snapshot tool may record around one call of the operator: the buffers and scalars
    // by name (tensors/KernelSnapshotInfo.h:249-300; kernels/rocm/gemm/ROCmQuantisedGemmKernel.cpp:5049-5059).
    struct KernelBufferDesc
    {
        const char *name;
        const char *description;
        const char *dtype; // "FP32", "INT8", "INT32"
    };
    struct KernelSnapshotInfo
    {
        const char *kernel_name = "";
        const char *kernel_description = "";
        std::vector<KernelBufferDesc> inputs, outputs, weights, scalars;
        bool is_passthrough = false; // nothing to snapshot
    };

    class MI355QuantGemmKernel
    {
    public:
        // Weights given as GGUF blocks in host memory, row-major [N][K/256].  The bytes
        // are borrowed until prepareWeights() has run (the first multiply runs it if the
        // caller did not); they may be released afterwards.  A bad format or shape leaves
        // the object invalid instead of throwing (CPUNativeVNNIGemmKernel.h:65-71).
        MI355QuantGemmKernel(uint8_t fmt, const void *host_gguf, int N, int K, int device_id);

        // Weights already in device memory in the prepared layout, kept alive by
        // lifetime_owner (a pooled VRAM slab, kernels/rocm/gemm/ROCmQuantisedGemmKernel.h:388-393).
        MI355QuantGemmKernel(uint8_t fmt, const void *d_prepared, int N, int K, int device_id,
                             std::shared_ptr<void> lifetime_owner);

        ~MI355QuantGemmKernel();
        MI355QuantGemmKernel(const MI355QuantGemmKernel &) = delete;
        MI355QuantGemmKernel &operator=(const MI355QuantGemmKernel &) = delete;

        // ---- ITensorKernel ---------------------------------------------------
        bool supports_device(int device_idx) const { return device_idx == device_id_; }
        void setGPUStream(void *stream) { stream_ = stream; }
        void resetDynamicState() {}

        // ---- weights ---------------------------------------------------------
        void prepareWeights();
        bool weights_converted() const { return d_weights_ != nullptr; }
        bool isValid() const { return valid_; }
        bool hasWeights() const { return valid_ && (d_weights_ || host_gguf_); }
        void releaseWeights();
        size_t packedWeightBytes() const;
        // Optional batch plane of the matrix (ql_api.h, llam_ql_build_batch_plane): built once,
        // owned by the operator and handed to every launch it makes, so that batches of 5..8
        // rows read weights laid out for the matrix unit (Q6_K: ready-made int8); dropped with
        // the weights (release, detach, attach).  The reference's packed matrix is int8 to begin with and has no such switch.
        // False (with the reason in last_error) where the format or shape has no plane.
        bool enableBatchPlane();
        bool hasBatchPlane() const { return d_plane_ != nullptr; }
        void dropBatchPlane();
        size_t batchPlaneBytes() const { return d_plane_ ? llam_ql_batch_plane_bytes(fmt_, N_, K_) : 0; }
        // Weight hand-over (TensorKernels.h:1335-1394).  detachWeights: the operator gives its
        // prepared weights away and has none until attachWeights (hasWeights() is false, every
        // multiply fails); cloneWeights: a deep copy, the operator keeps its own; attachWeights:
        // takes weights of the same format, shape and device in place of whatever it held,
        // false (and the argument destroyed) on a mismatch.  Host GGUF bytes that have not been
        // uploaded yet are prepared first.
        std::unique_ptr<MI355PackedWeights> detachWeights();
        std::unique_ptr<MI355PackedWeights> cloneWeights();
        bool attachWeights(std::unique_ptr<MI355PackedWeights> weights);
        KernelSnapshotInfo getKernelSnapshotInfo() const;
        uint8_t codebookId() const { return fmt_; }
        int get_n() const { return N_; }
        int get_k() const { return K_; }
        int device() const { return device_id_; }
        bool exportMatrixDesc(DeviceQuantMatrixDesc &out);

        // ---- workspace -------------------------------------------------------
        // Bytes multiply_* may need for an [m x k] input and [m x n] output.
        static size_t getWorkspaceRequirements(int m, int n, int k);
        void bindWorkspace(const DeviceWorkspace &ws) { bound_ = ws; }

        // ---- GEMM ------------------------------------------------------------
        // C[m x n] = alpha * A[m x k] @ W[n x k]^T + beta * C (+ bias).  m <= 8 runs the
        // decode GEMV, larger m the int8-MFMA GEMM.  n and k must equal get_n() and
        // get_k() (the reference operator computes all packed rows whatever n says);
        // C may be wider than n.  beta == 0 overwrites C.
        bool multiply_tensor(const DeviceTensor *A, DeviceTensor *C, int m, int n, int k,
                             bool transpose_B = true, float alpha = 1.0f, float beta = 0.0f,
                             const DeviceTensor *bias = nullptr, int device_idx = -1,
                             DeviceWorkspace *workspace = nullptr, int activation_row_offset = 0);

        struct TensorProjectionDesc
        {
            MI355QuantGemmKernel *kernel;
            DeviceTensor *output;
            int n;
            const DeviceTensor *bias;
            const char *name;
            TensorProjectionDesc(MI355QuantGemmKernel *k, DeviceTensor *out, int n_dim,
                                 const DeviceTensor *b = nullptr, const char *nm = nullptr)
                : kernel(k), output(out), n(n_dim), bias(b), name(nm) {}
        };

        // Several projections of one input: the input is quantised once.
        bool supports_fused_projection() const { return true; }
        bool multiply_fused_tensor(const DeviceTensor *input, const std::vector<TensorProjectionDesc> &projections,
                                   int m, int k, DeviceWorkspace *workspace = nullptr);

        // Rows 2..4 of a verifier batch with the arithmetic of the m == 1 path
        // (TensorKernels.h:676-709): here every m <= 4 GEMV row already is bit-identical
        // to its m == 1 result, so this is multiply_fused_tensor with that bound checked.
        bool multiply_fused_verifier_rows_decode_equivalent(const DeviceTensor *input,
                                                            const std::vector<TensorProjectionDesc> &projections,
                                                            int m, int k, DeviceWorkspace *workspace = nullptr);

        // output[m x n] = (silu(gate) * up)[m x k] @ W^T
        bool multiply_tensor_with_fused_swiglu(const DeviceTensor *gate, const DeviceTensor *up, DeviceTensor *output,
                                               int m, int n, int k, float alpha = 1.0f, float beta = 0.0f,
                                               DeviceWorkspace *workspace = nullptr);

        // ---- activation sharing ------------------------------------------------
        bool supports_activation_sharing() const { return true; }
        size_t get_quantized_activation_buffer_size(int m, int k) const;
        bool quantize_activations(const float *d_A, void *d_q8_1, int m, int k);
        bool multiply_with_precomputed_q8_1(const void *d_q8_1, float *d_C, int m, int n, int k,
                                            const DeviceTensor *bias = nullptr, bool accumulate = false,
                                            float alpha = 1.0f, float beta = 0.0f, int device_idx = -1,
                                            DeviceWorkspace *workspace = nullptr);

        // ---- MoE down projections ----------------------------------------------
        struct FusedExpertDownDesc
        {
            MI355QuantGemmKernel *kernel;
            const float *input; // device, [k]
            float *output;      // device, [n]
            int n;
        };
        bool multiply_fused_expert_down(const FusedExpertDownDesc *descs, int num_descs, int m, int k);

    private:
        struct Scratch
        {
            uint8_t *p = nullptr;
            size_t left = 0;
            void *take(size_t bytes);
        };
        bool open_scratch(const char *fn, size_t bytes, DeviceWorkspace *ws, Scratch &s);
        bool ready(const char *fn);
        bool run(const char *fn, const void *d_q8, float *d_C, int ldc, int m, int n, const DeviceTensor *bias,
                 float alpha, float beta, Scratch &s, void *stream);

        uint8_t fmt_ = 0;
        int N_ = 0, K_ = 0, device_id_ = 0;
        bool valid_ = false;
        const void *host_gguf_ = nullptr;
        const void *d_weights_ = nullptr;
        void *d_owned_ = nullptr;
        void *d_plane_ = nullptr; // the batch plane built from d_weights_
        void drop_plane_locked();
        std::shared_ptr<void> lifetime_owner_;
        void *stream_ = nullptr;
        DeviceWorkspace bound_;
        std::mutex prepare_mutex_;
    };

    // ---------------------------------------------------------------------------
    // Registry
    // ---------------------------------------------------------------------------

    enum class GemmPreparationKind
    {
        AUTO = 0,
        MI355_NATIVE_BLOCKS = 5, // device-resident GGUF blocks in the prepared layout
    };

    // The weight tensor as the loader sees it: GGUF blocks in host memory.
    struct QuantWeightTensor
    {
        std::string name;
        uint8_t fmt = 0;
        const void *host_gguf = nullptr;
        int n = 0;
        int k = 0;
    };

    struct PreparedGemmWeights
    {
        GemmPreparationKind kind{GemmPreparationKind::AUTO};
        MI355QuantGemmKernel *kernel{nullptr};
        std::shared_ptr<MI355QuantGemmKernel> owned_kernel;
    };

    struct PreparedGemmHandle
    {
        const QuantWeightTensor *tensor{nullptr};
        int device_id{0};
        GemmPreparationKind kind{GemmPreparationKind::AUTO};
        int variant{0}; // weight format id
        std::shared_ptr<PreparedGemmWeights> prepared_weights;
    };

    enum class ExpertRole
    {
        GATE = 0,
        UP = 1,
        DOWN = 2
    };

    class QuantGemmRegistry
    {
    public:
        // One handle per (tensor, device): a second call returns the first handle.
        // Throws std::runtime_error on a null tensor or unsupported format
        // (factory misuse throws in the reference too, kernels/KernelFactory.cpp:3235-3241).
        std::shared_ptr<PreparedGemmHandle> prepareGemmHandleLocal(const QuantWeightTensor *tensor, int device_id,
                                                                   GemmPreparationKind kind = GemmPreparationKind::AUTO);
        // The operator bound to a handle; nullptr for a null or unbound handle.
        MI355QuantGemmKernel *getOrCreateGemmEngine(const PreparedGemmHandle *prepared);

        // Name-keyed store the stages read (PreparedWeightStore).
        void registerPreparedGemmHandle(const std::string &ref, std::shared_ptr<PreparedGemmHandle> handle);
        MI355QuantGemmKernel *gemmKernel(const std::string &ref);

        // (device, layer, expert, role)-keyed store for MoE engines (ExpertGemmRegistry).
        void registerEngine(int device, int layer, int expert, ExpertRole role, std::shared_ptr<MI355QuantGemmKernel> e);
        MI355QuantGemmKernel *getEngine(int device, int layer, int expert, ExpertRole role);

        size_t size();
        void clear();

    private:
        std::mutex cache_mutex_;
        std::map<std::pair<const QuantWeightTensor *, int>, std::shared_ptr<PreparedGemmHandle>> handles_;
        std::map<std::string, std::shared_ptr<PreparedGemmHandle>> by_ref_;
        std::shared_mutex expert_mutex_;
        std::map<std::tuple<int, int, int, int>, std::shared_ptr<MI355QuantGemmKernel>> experts_;
    };
} // namespace llaminar_amd
