// Llaminar-side binding of the MI355X quantized-linear operator: an ITensorGemm
// (src/v2/tensors/TensorKernels.h:348-1427) and IWorkspaceConsumer
// (src/v2/interfaces/IWorkspaceConsumer.h:60-137) that forwards every call to
// llaminar_amd::MI355QuantGemmKernel.  This is the file a Llaminar maintainer drops beside
// kernels/rocm/gemm/ROCmQuantisedGemmKernel.h; it compiles only inside the Llaminar tree
// (include root src/v2) with this repository's include/ on the include path, and contains
// no arithmetic.
//
// Device pointers come from TensorBase::gpu_data_ptr() (tensors/TensorClasses.h:1001), as in
// ROCmQuantisedGemmKernel::multiply_tensor (kernels/rocm/gemm/ROCmQuantisedGemmKernel.cpp:2331);
// tensors that are not resident on the device make the call fail (return false), which the
// stages treat as "format combination not supported".
#pragma once

#include <cstring>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "execution/local_execution/device/DeviceWorkspaceManager.h"
#include "tensors/TensorKernels.h"
#include "tensors/Tensors.h"

#include <llaminar_amd/quant_gemm.hpp>

namespace llaminar2
{
    namespace mi355
    {
        // Name of the one workspace buffer the operator asks for.
        constexpr const char *kScratchBufferName = "mi355_ql_scratch";

        // GGUF codebook id (= llam_weight_format) of a weight tensor type; 0 = not served.
        inline uint8_t codebookIdOf(TensorType t)
        {
            switch (t)
            {
            case TensorType::Q4_K:
                return LLAM_FMT_Q4_K;
            case TensorType::Q6_K:
                return LLAM_FMT_Q6_K;
            case TensorType::IQ3_S:
                return LLAM_FMT_IQ3_S;
            default:
                return 0;
            }
        }

        inline size_t superblockBytes(uint8_t codebook_id)
        {
            return static_cast<size_t>(llam_format_block_bytes(codebook_id));
        }

        inline KernelBufferDtype dtypeOf(const char *name)
        {
            if (!name)
                return KernelBufferDtype::Unknown;
            if (!std::strcmp(name, "FP32"))
                return KernelBufferDtype::FP32;
            if (!std::strcmp(name, "INT8"))
                return KernelBufferDtype::INT8;
            if (!std::strcmp(name, "INT32"))
                return KernelBufferDtype::INT32;
            if (!std::strcmp(name, "Q8_1"))
                return KernelBufferDtype::Q8_1;
            if (!std::strcmp(name, "Q4_K"))
                return KernelBufferDtype::Q4_K;
            if (!std::strcmp(name, "Q6_K"))
                return KernelBufferDtype::Q6_K;
            if (!std::strcmp(name, "IQ3_S"))
                return KernelBufferDtype::IQ3_S;
            return KernelBufferDtype::Unknown;
        }

        // fp32 tensor on the device -> the operator's view of it; data == nullptr when the tensor
        // is not resident.
        inline llaminar_amd::DeviceTensor deviceView(const TensorBase *t)
        {
            if (!t)
                return {};
            auto *p = static_cast<float *>(const_cast<void *>(t->gpu_data_ptr()));
            return llaminar_amd::DeviceTensor(p, static_cast<int>(t->rows()), static_cast<int>(t->cols()));
        }

        inline llaminar_amd::DeviceWorkspace workspaceView(const DeviceWorkspaceManager *ws)
        {
            llaminar_amd::DeviceWorkspace out;
            if (ws && ws->hasBuffer(kScratchBufferName))
            {
                out.base = ws->getBuffer(kScratchBufferName);
                out.bytes = ws->getBufferSize(kScratchBufferName);
            }
            return out;
        }

        // Prepared weights outside an operator (kernels/IPackedWeights.h:62-130).
        class MI355PackedWeightsHandle final : public IPackedWeights
        {
        public:
            explicit MI355PackedWeightsHandle(std::unique_ptr<llaminar_amd::MI355PackedWeights> w) : w_(std::move(w)) {}
            PackedWeightsFormat format() const override { return PackedWeightsFormat::ROCM_INT8; }
            DeviceType deviceType() const override { return DeviceType::ROCm; }
            int N() const override { return w_ ? w_->N() : 0; }
            int K() const override { return w_ ? w_->K() : 0; }
            size_t sizeBytes() const override { return w_ ? w_->sizeBytes() : 0; }
            std::unique_ptr<IPackedWeights> clone() const override
            {
                if (!w_)
                    return nullptr;
                auto c = w_->clone();
                if (!c)
                    return nullptr;
                return std::make_unique<MI355PackedWeightsHandle>(std::move(c));
            }
            std::unique_ptr<llaminar_amd::MI355PackedWeights> take() { return std::move(w_); }

        private:
            std::unique_ptr<llaminar_amd::MI355PackedWeights> w_;
        };

        class MI355QuantGemmAdapter final : public ITensorGemm, public IWorkspaceConsumer
        {
        public:
            // GGUF super-blocks of rows [row_start, row_end) of a Q4_K / Q6_K / IQ3_S tensor in host
            // memory (TensorBase::raw_data, tensors/TensorClasses.h:724); row_end < 0 = all rows.
            MI355QuantGemmAdapter(const TensorBase *w, int rocm_ordinal, int row_start = 0, int row_end = -1,
                                  int serving_batch = 1)
                : impl_(codebookIdOf(w->native_type()),
                        static_cast<const uint8_t *>(w->raw_data()) +
                            size_t(row_start) * (w->cols() / 256) * superblockBytes(codebookIdOf(w->native_type())),
                        (row_end < 0 ? static_cast<int>(w->rows()) : row_end) - row_start, static_cast<int>(w->cols()),
                        rocm_ordinal),
                  serving_batch_(serving_batch)
            {
            }

            // Raw rows (an expert slice, a test).
            MI355QuantGemmAdapter(uint8_t codebook_id, const void *host_gguf_rows, int n, int k, int rocm_ordinal,
                                  int serving_batch = 1)
                : impl_(codebook_id, host_gguf_rows, n, k, rocm_ordinal), serving_batch_(serving_batch)
            {
            }

            llaminar_amd::MI355QuantGemmKernel &impl() { return impl_; }
            bool isValid() const { return impl_.isValid(); }

            // ---- ITensorKernel / IKernelSnapshotCapable ------------------------------------------
            bool supports_device(int device_idx) const override { return impl_.supports_device(device_idx); }
            void setGPUStream(void *stream) override { impl_.setGPUStream(stream); }
            KernelSnapshotInfo getKernelSnapshotInfo() const override
            {
                const llaminar_amd::KernelSnapshotInfo i = impl_.getKernelSnapshotInfo();
                KernelSnapshotInfo out = KernelSnapshotInfo::gemm();
                for (const auto &d : i.inputs)
                    out.withInput(d.name, d.description, dtypeOf(d.dtype));
                for (const auto &d : i.weights)
                    out.withWeight(d.name, d.description, dtypeOf(d.dtype));
                for (const auto &d : i.outputs)
                    out.withOutput(d.name, d.description, dtypeOf(d.dtype));
                for (const auto &d : i.scalars)
                    out.withScalar(d.name, d.description, dtypeOf(d.dtype));
                return out;
            }

            // ---- ITensorGemm: the primary interface (TensorKernels.h:470-479) ------------------------
            using ITensorGemm::multiply_tensor; // keep the shape-deducing overload visible (TensorKernels.h:415)
            bool multiply_tensor(const TensorBase *A, TensorBase *C, int m, int n, int k, bool transpose_B = true,
                                 float alpha = 1.0f, float beta = 0.0f, const TensorBase *bias = nullptr,
                                 const IMPIContext *mpi_ctx = nullptr, int device_idx = -1,
                                 DeviceWorkspaceManager *workspace = nullptr, int activation_row_offset = 0) override
            {
                (void)mpi_ctx;
                if (!A || !C)
                    return false;
                llaminar_amd::DeviceTensor a = deviceView(A), c = deviceView(C), b = deviceView(bias);
                if (!a.data || !c.data || (bias && !b.data))
                    return false;
                llaminar_amd::DeviceWorkspace w = workspaceView(workspace ? workspace : workspace_);
                return impl_.multiply_tensor(&a, &c, m, n, k, transpose_B, alpha, beta, bias ? &b : nullptr, device_idx,
                                             w.base ? &w : nullptr, activation_row_offset);
            }

            // TensorKernels.h:490-496
            bool multiply_tensor_with_fused_swiglu(const TensorBase *gate, const TensorBase *up, TensorBase *output, int m,
                                                   int n, int k, float alpha = 1.0f, float beta = 0.0f,
                                                   DeviceWorkspaceManager *workspace = nullptr) override
            {
                llaminar_amd::DeviceTensor g = deviceView(gate), u = deviceView(up), o = deviceView(output);
                if (!g.data || !u.data || !o.data)
                    return false;
                llaminar_amd::DeviceWorkspace w = workspaceView(workspace ? workspace : workspace_);
                return impl_.multiply_tensor_with_fused_swiglu(&g, &u, &o, m, n, k, alpha, beta, w.base ? &w : nullptr);
            }

            // TensorKernels.h:527-533: rows of m <= 4 carry the bits of their m == 1 call on this
            // engine, so the grouped verifier form is the ordinary one with that bound checked.
            bool multiply_tensor_with_fused_swiglu_verifier_rows_decode_equivalent(
                const TensorBase *gate, const TensorBase *up, TensorBase *output, int m, int n, int k, float alpha = 1.0f,
                float beta = 0.0f, DeviceWorkspaceManager *workspace = nullptr) override
            {
                llam_ql_gemv_plan plan{};
                if (m < 1 || m > LLAM_QL_MAX_GEMV_M ||
                    !llam_ql_gemv_describe(impl_.codebookId(), m, impl_.get_n(), impl_.get_k(), impl_.hasBatchPlane() ? 1 : 0, impl_.device(), &plan) ||
                    !plan.decode_equivalent)
                    return false;
                return multiply_tensor_with_fused_swiglu(gate, up, output, m, n, k, alpha, beta, workspace);
            }

            bool supports_fused_projection() const override { return true; }
            void prepareWeights() override
            {
                impl_.prepareWeights();
                if (serving_batch_ >= 5)
                    (void)impl_.enableBatchPlane(); // optional second copy for batches of 5..8
            }
            bool weights_converted() const override { return impl_.weights_converted(); }

            // TensorKernels.h:584.  The prepared matrix is ONE device buffer; `scales` repeats the
            // payload pointer so that DeviceNativeVNNIMatrixDesc::valid() holds.  Only
            // MI355MoEAdapter reads these descriptors, and it reads `payload` alone.
            bool exportNativeVNNIMatrixDesc(DeviceNativeVNNIMatrixDesc &out) override
            {
                out = {};
                llaminar_amd::DeviceQuantMatrixDesc d;
                if (!impl_.exportMatrixDesc(d))
                    return false;
                out.payload = static_cast<const uint8_t *>(d.weights);
                out.scales = d.weights;
                out.n = d.n;
                out.k = d.k;
                out.blocks_per_row = d.blocks_per_row;
                out.codebook_id = d.codebook_id;
                return out.valid();
            }

            // TensorKernels.h:639-645
            bool multiply_fused_tensor(const TensorBase *input, const std::vector<TensorProjectionDesc> &projections, int m,
                                       int k, const IMPIContext *mpi_ctx = nullptr,
                                       DeviceWorkspaceManager *workspace = nullptr) override
            {
                (void)mpi_ctx;
                return fused(input, projections, m, k, workspace, false);
            }

            // TensorKernels.h:695-701
            bool multiply_fused_verifier_rows_decode_equivalent(const TensorBase *input,
                                                                const std::vector<TensorProjectionDesc> &projections,
                                                                int m, int k, const IMPIContext *mpi_ctx = nullptr,
                                                                DeviceWorkspaceManager *workspace = nullptr) override
            {
                (void)mpi_ctx;
                return fused(input, projections, m, k, workspace, true);
            }

            // TensorKernels.h:738-741: descs[i].input / output are device pointers here
            bool multiply_fused_expert_down(const FusedExpertDownDesc *descs, int num_descs, int m, int k) override
            {
                if (!descs || num_descs <= 0)
                    return false;
                std::vector<llaminar_amd::MI355QuantGemmKernel::FusedExpertDownDesc> d;
                d.reserve(static_cast<size_t>(num_descs));
                for (int i = 0; i < num_descs; ++i)
                {
                    auto *peer = dynamic_cast<MI355QuantGemmAdapter *>(descs[i].kernel);
                    if (!peer)
                        return false;
                    d.push_back({&peer->impl_, descs[i].input, descs[i].output, descs[i].n});
                }
                return impl_.multiply_fused_expert_down(d.data(), num_descs, m, k);
            }

            // ---- activation sharing (TensorKernels.h:1169-1312) -----------------------------------------
            bool supports_activation_sharing() const override { return true; }
            bool quantize_activations(const float *A, void *q8_1_buffer, int m, int k) override
            {
                return impl_.quantize_activations(A, q8_1_buffer, m, k);
            }
            size_t get_quantized_activation_buffer_size(int m, int k) const override
            {
                return impl_.get_quantized_activation_buffer_size(m, k);
            }
            using ITensorGemm::multiply_with_precomputed_q8_1; // the overload without fused_ops delegates here
            bool multiply_with_precomputed_q8_1(const void *q8_1_activations, float *C, int m, int n, int k,
                                                const TensorBase *bias, bool accumulate, float alpha, float beta,
                                                const IMPIContext *mpi_ctx, int device_idx, const GemmFusedOps &fused_ops,
                                                DeviceWorkspaceManager *workspace = nullptr) override
            {
                (void)mpi_ctx;
                if (fused_ops.has_fusion())
                    return false; // SwiGLU / softmax epilogues are not part of this path
                llaminar_amd::DeviceTensor b = deviceView(bias);
                if (bias && !b.data)
                    return false;
                llaminar_amd::DeviceWorkspace w = workspaceView(workspace ? workspace : workspace_);
                return impl_.multiply_with_precomputed_q8_1(q8_1_activations, C, m, n, k, bias ? &b : nullptr, accumulate,
                                                            alpha, beta, device_idx, w.base ? &w : nullptr);
            }

            // ---- IWorkspaceConsumer (interfaces/IWorkspaceConsumer.h:87-136) -----------------------------
            WorkspaceRequirements getWorkspaceRequirements(int m, int n = 0, int k = 0) const override
            {
                WorkspaceRequirements req;
                const size_t bytes = llaminar_amd::MI355QuantGemmKernel::getWorkspaceRequirements(
                    m, n > 0 ? n : impl_.get_n(), k > 0 ? k : impl_.get_k());
                req.buffers.push_back({kScratchBufferName, bytes, 256, true});
                return req;
            }
            void bindWorkspace(DeviceWorkspaceManager *workspace) override
            {
                workspace_ = workspace;
                impl_.bindWorkspace(workspaceView(workspace));
            }
            bool hasWorkspace() const override { return workspace_ != nullptr; }
            DeviceWorkspaceManager *getWorkspace() const override { return workspace_; }

            // ---- weight life cycle (TensorKernels.h:1335-1394) -------------------------------------------
            std::unique_ptr<IPackedWeights> detachWeights() override { return wrap(impl_.detachWeights()); }
            std::unique_ptr<IPackedWeights> cloneWeights() const override
            {
                return wrap(const_cast<llaminar_amd::MI355QuantGemmKernel &>(impl_).cloneWeights());
            }
            bool attachWeights(std::unique_ptr<IPackedWeights> weights) override
            {
                auto *mine = dynamic_cast<MI355PackedWeightsHandle *>(weights.get());
                if (!mine)
                    return false;
                return impl_.attachWeights(mine->take());
            }
            void releaseWeights() override { impl_.releaseWeights(); }
            bool hasWeights() const override { return impl_.hasWeights(); }
            size_t packedWeightBytes() const override { return impl_.packedWeightBytes(); }
            int get_n() const override { return impl_.get_n(); }
            int get_k() const override { return impl_.get_k(); }

        private:
            static std::unique_ptr<IPackedWeights> wrap(std::unique_ptr<llaminar_amd::MI355PackedWeights> w)
            {
                if (!w)
                    return nullptr;
                return std::make_unique<MI355PackedWeightsHandle>(std::move(w));
            }

            bool fused(const TensorBase *input, const std::vector<TensorProjectionDesc> &projections, int m, int k,
                       DeviceWorkspaceManager *workspace, bool verifier_rows)
            {
                llaminar_amd::DeviceTensor in = deviceView(input);
                if (!in.data || projections.empty())
                    return false;
                const size_t n = projections.size();
                std::vector<llaminar_amd::DeviceTensor> outs(n), biases(n);
                std::vector<llaminar_amd::MI355QuantGemmKernel::TensorProjectionDesc> descs;
                descs.reserve(n);
                for (size_t i = 0; i < n; ++i)
                {
                    const TensorProjectionDesc &p = projections[i];
                    auto *peer = dynamic_cast<MI355QuantGemmAdapter *>(p.kernel);
                    if (!peer || !p.output)
                        return false;
                    outs[i] = deviceView(p.output);
                    biases[i] = deviceView(p.bias);
                    if (!outs[i].data || (p.bias && !biases[i].data))
                        return false;
                    descs.emplace_back(&peer->impl_, &outs[i], p.n, p.bias ? &biases[i] : nullptr, p.name);
                }
                llaminar_amd::DeviceWorkspace w = workspaceView(workspace ? workspace : workspace_);
                return verifier_rows
                           ? impl_.multiply_fused_verifier_rows_decode_equivalent(&in, descs, m, k, w.base ? &w : nullptr)
                           : impl_.multiply_fused_tensor(&in, descs, m, k, w.base ? &w : nullptr);
            }

            llaminar_amd::MI355QuantGemmKernel impl_;
            DeviceWorkspaceManager *workspace_ = nullptr;
            int serving_batch_ = 1;
        };
    } // namespace mi355
} // namespace llaminar2
