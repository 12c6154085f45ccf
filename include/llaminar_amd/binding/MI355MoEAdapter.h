// Llaminar-side binding of the MI355X MoE operator: an IMoEKernel
// (src/v2/kernels/IMoEKernel.h:56-660) that forwards the decode methods to
// llaminar_amd::MI355MoEKernel.  Like MI355QuantGemmAdapter.h this file compiles only inside
// the Llaminar tree (include root src/v2) and contains no arithmetic.
//
// All pointers are device pointers, as in ROCmMoEKernel (kernels/rocm/moe/ROCmMoEKernel.cpp:1785-1845).
// DeviceMoELayerRuntime (execution/moe/MoERuntimeTable.h:88-115) is a device-resident struct:
// the adapter only forms the addresses of its topk_expert_ids / topk_weights / decode_histogram
// members and never reads through the pointer on the host.
#pragma once

#include <cstddef>
#include <vector>

#include "execution/local_execution/device/DeviceWorkspaceManager.h"
#include "execution/moe/MoERuntimeTable.h"
#include "interfaces/IWorkspaceConsumer.h"
#include "kernels/IMoEKernel.h"
#include "tensors/Tensors.h"

#include <llaminar_amd/moe_kernel.hpp>

namespace llaminar2
{
    namespace mi355
    {
        constexpr const char *kMoEScratchBufferName = "mi355_moe_scratch";

        class MI355MoEAdapter final : public IMoEKernel, public IWorkspaceConsumer
        {
        public:
            explicit MI355MoEAdapter(int rocm_ordinal) : impl_(rocm_ordinal), device_(rocm_ordinal) {}
            llaminar_amd::MI355MoEKernel &impl() { return impl_; }
            bool isValid() const { return impl_.isValid(); }

            // ---- ITensorKernel -------------------------------------------------------------------
            bool supports_device(int device_idx) const override { return impl_.supports_device(device_idx); }
            void setGPUStream(void *stream) override
            {
                stream_ = stream;
                impl_.setGPUStream(stream);
            }
            // nothing of its own to snapshot, as ROCmMoEKernel (kernels/rocm/moe/ROCmMoEKernel.h:387-390)
            KernelSnapshotInfo getKernelSnapshotInfo() const override { return KernelSnapshotInfo::passthrough(); }

            // ---- IWorkspaceConsumer (interfaces/IWorkspaceConsumer.h:87-136) ------------------------
            // m = tokens per call; n = expert intermediate width, k = d_model.  The slot count and the
            // expert count are those of the largest configuration the runtime table allows.
            WorkspaceRequirements getWorkspaceRequirements(int m, int n = 0, int k = 0) const override
            {
                WorkspaceRequirements req;
                req.buffers.push_back({kMoEScratchBufferName,
                                       llaminar_amd::MI355MoEKernel::getWorkspaceRequirements(
                                           m, static_cast<int>(kDeviceMoEMaxTopK), k, n, static_cast<int>(kDeviceMoEMaxExperts)),
                                       256, true});
                return req;
            }
            void bindWorkspace(DeviceWorkspaceManager *workspace) override
            {
                workspace_ = workspace;
                llaminar_amd::DeviceWorkspace w;
                if (workspace && workspace->hasBuffer(kMoEScratchBufferName))
                {
                    w.base = workspace->getBuffer(kMoEScratchBufferName);
                    w.bytes = workspace->getBufferSize(kMoEScratchBufferName);
                }
                impl_.bindWorkspace(w);
            }
            bool hasWorkspace() const override { return workspace_ != nullptr; }
            DeviceWorkspaceManager *getWorkspace() const override { return workspace_; }

            // ---- IMoEKernel: the five pure virtuals (IMoEKernel.h:84-171) --------------------------------
            bool route(const float *hidden, const float *gate_weights, int seq_len, int d_model, int num_experts, int top_k,
                       bool normalize_weights, MoERoutingResult &result) override
            {
                llaminar_amd::MoERoutingResult r;
                if (!impl_.route(hidden, gate_weights, seq_len, d_model, num_experts, top_k, normalize_weights, r))
                    return false;
                result.expert_indices = std::move(r.expert_indices);
                result.expert_weights = std::move(r.expert_weights);
                result.router_logits = std::move(r.router_logits);
                return true;
            }
            // The interface gives no row count for `hidden` / `output`: the indices come from the
            // router of the same call and are in range by construction, so the bound passed on is
            // the largest index an int can hold.
            void gatherTokenBatch(const float *hidden, float *batch_buffer, const int *token_indices, int num_tokens,
                                  int d_model) override
            {
                (void)impl_.gatherTokenBatch(hidden, batch_buffer, token_indices, num_tokens, d_model, kNoRowBound);
            }
            void scatterAddWeighted(float *output, const float *expert_output, const int *token_indices,
                                    const float *weights, int num_tokens, int d_model) override
            {
                (void)impl_.scatterAddWeighted(output, expert_output, token_indices, weights, num_tokens, d_model,
                                               kNoRowBound);
            }
            void sharedExpertGate(const float *input, const float *gate_inp, float *shared_output, int seq_len,
                                  int d_model) override
            {
                (void)impl_.sharedExpertGate(input, gate_inp, shared_output, seq_len, d_model);
            }
            void swiGLU(float *gate, const float *up, int count) override { (void)impl_.swiGLU(gate, up, count); }
            void weightedAdd(float *output, const float *input, float weight, int count) override
            {
                (void)impl_.weightedAdd(output, input, weight, count);
            }

            // ---- device-resident decode routing (IMoEKernel.h:245-258) -----------------------------------
            bool decodeRouteSelect(DeviceMoELayerRuntime *runtime_layer, ITensor *hidden, ITensor *gate_weights, int d_model,
                                   int num_experts, int top_k, bool normalize_weights, ITensor *output_indices,
                                   ITensor *output_weights, bool write_legacy_outputs,
                                   bool update_runtime_histogram) override
            {
                if (!runtime_layer || !hidden || !gate_weights || top_k <= 0 || top_k > static_cast<int>(kDeviceMoEMaxTopK))
                    return false;
                if (gate_weights->native_type() != TensorType::FP32)
                    return false; // the router matrix is multiplied in fp32
                llaminar_amd::DeviceTensor h = view(hidden), g = view(gate_weights);
                if (!h.data || !g.data)
                    return false;
                h.rows = 1; // decode: the runtime state holds ONE token's slots
                h.cols = d_model;
                g.rows = num_experts;
                g.cols = d_model;
                llaminar_amd::DeviceMoELayerRuntime rt = runtimeView(runtime_layer, top_k);
                if (!impl_.decodeRouteSelect(&rt, &h, &g, d_model, num_experts, top_k, normalize_weights))
                    return false;
                float *legacy_ids = nullptr, *legacy_w = nullptr;
                if (write_legacy_outputs)
                {
                    if (!output_indices || !output_weights)
                        return false;
                    legacy_ids = static_cast<float *>(output_indices->gpu_data_ptr());
                    legacy_w = static_cast<float *>(output_weights->gpu_data_ptr());
                    if (!legacy_ids || !legacy_w)
                        return false;
                }
                uint64_t *hist = update_runtime_histogram ? member<uint64_t>(runtime_layer, offsetof(DeviceMoELayerRuntime, decode_histogram)) : nullptr;
                return llam_ql_moe_publish_routing(rt.topk_expert_ids, rt.topk_weights, 1, top_k, top_k, legacy_ids, legacy_w,
                                                   hist, num_experts < static_cast<int>(kDeviceMoEMaxExperts) ? num_experts : static_cast<int>(kDeviceMoEMaxExperts),
                                                   device_, stream_);
            }

            // ---- descriptor tables (IMoEKernel.h:409-450) -----------------------------------------------
            int uploadGroupedExpertDownDescriptorTable(const DeviceNativeVNNIMatrixDesc *down_descs, int num_experts,
                                                       int d_model, int intermediate) override
            {
                if (!down_descs || num_experts <= 0)
                    return -1;
                const auto d = convert(down_descs, num_experts);
                return impl_.uploadGroupedExpertDownDescriptorTable(d.data(), num_experts, d_model, intermediate);
            }
            int uploadGroupedExpertGateUpDescriptorTables(const DeviceNativeVNNIMatrixDesc *gate_descs,
                                                          const DeviceNativeVNNIMatrixDesc *up_descs, int num_experts,
                                                          int d_model, int intermediate) override
            {
                if (!gate_descs || !up_descs || num_experts <= 0)
                    return -1;
                const auto g = convert(gate_descs, num_experts), u = convert(up_descs, num_experts);
                return impl_.uploadGroupedExpertGateUpDescriptorTables(g.data(), u.data(), num_experts, d_model, intermediate);
            }

            // ---- grouped decode from host ids (IMoEKernel.h:452-478, 530-552) ----------------------------
            bool groupedExpertGateUpDecodeFromTable(const TensorBase *input, const int *expert_ids, int descriptor_table_id,
                                                    int num_active, ITensor *const *gate_outputs, ITensor *const *up_outputs,
                                                    int d_model, int intermediate) override
            {
                llaminar_amd::DeviceTensor in = view(input);
                float *g = contiguous(gate_outputs, num_active, intermediate), *u = contiguous(up_outputs, num_active, intermediate);
                if (!in.data || !g || !u)
                    return false;
                in.rows = 1;
                in.cols = d_model;
                return impl_.groupedExpertGateUpDecodeFromTable(&in, expert_ids, descriptor_table_id, num_active, g, u, d_model,
                                                                intermediate);
            }
            bool groupedExpertDownDecodeFromTable(ITensor *const *gate_tensors, ITensor *const *up_tensors, const int *expert_ids,
                                                  const float *expert_weights, int descriptor_table_id, int num_active,
                                                  ITensor *output, int d_model, int intermediate) override
            {
                float *g = contiguous(gate_tensors, num_active, intermediate), *u = contiguous(up_tensors, num_active, intermediate);
                llaminar_amd::DeviceTensor out = view(output);
                if (!g || !u || !out.data)
                    return false;
                out.rows = 1;
                out.cols = d_model;
                return impl_.groupedExpertDownDecodeFromTable(g, u, expert_ids, expert_weights, descriptor_table_id, num_active,
                                                              &out, d_model, intermediate);
            }

            // ---- grouped decode from fp32 routing tensors (IMoEKernel.h:480-506, 554-575) ---------------
            bool groupedExpertGateUpDecodeFromRouting(const TensorBase *input, ITensor *routing_indices, int descriptor_table_id,
                                                      int top_k, ITensor *const *gate_outputs, ITensor *const *up_outputs,
                                                      int d_model, int intermediate) override
            {
                llaminar_amd::DeviceTensor in = view(input);
                const float *idx = routing_indices ? static_cast<const float *>(routing_indices->gpu_data_ptr()) : nullptr;
                float *g = contiguous(gate_outputs, top_k, intermediate), *u = contiguous(up_outputs, top_k, intermediate);
                if (!in.data || !idx || !g || !u)
                    return false;
                in.rows = 1;
                in.cols = d_model;
                return impl_.groupedExpertGateUpDecodeFromRouting(&in, idx, descriptor_table_id, top_k, g, u, d_model,
                                                                  intermediate);
            }
            bool groupedExpertDownDecodeFromRouting(ITensor *const *gate_tensors, ITensor *const *up_tensors,
                                                    ITensor *routing_indices, ITensor *routing_weights, int descriptor_table_id,
                                                    int top_k, ITensor *output, int d_model, int intermediate) override
            {
                float *g = contiguous(gate_tensors, top_k, intermediate), *u = contiguous(up_tensors, top_k, intermediate);
                const float *idx = routing_indices ? static_cast<const float *>(routing_indices->gpu_data_ptr()) : nullptr;
                const float *wts = routing_weights ? static_cast<const float *>(routing_weights->gpu_data_ptr()) : nullptr;
                llaminar_amd::DeviceTensor out = view(output);
                if (!g || !u || !idx || !wts || !out.data)
                    return false;
                out.rows = 1;
                out.cols = d_model;
                return impl_.groupedExpertDownDecodeFromRouting(g, u, idx, wts, descriptor_table_id, top_k, &out, d_model,
                                                                intermediate);
            }

            // ---- grouped decode from the runtime state (IMoEKernel.h:508-528, 577-645) -------------------
            bool groupedExpertGateUpDecodeFromRuntime(DeviceMoELayerRuntime *runtime_layer, const TensorBase *input,
                                                      int descriptor_table_id, int top_k, ITensor *const *gate_outputs,
                                                      ITensor *const *up_outputs, int d_model, int intermediate) override
            {
                llaminar_amd::DeviceTensor in = view(input);
                float *g = contiguous(gate_outputs, top_k, intermediate), *u = contiguous(up_outputs, top_k, intermediate);
                if (!runtime_layer || !in.data || !g || !u)
                    return false;
                in.rows = 1;
                in.cols = d_model;
                llaminar_amd::DeviceMoELayerRuntime rt = runtimeView(runtime_layer, top_k);
                return impl_.groupedExpertGateUpDecodeFromRuntime(&rt, &in, descriptor_table_id, top_k, g, u, d_model,
                                                                  intermediate);
            }
            bool groupedExpertDownDecodeFromRuntime(ITensor *const *gate_tensors, ITensor *const *up_tensors,
                                                    DeviceMoELayerRuntime *runtime_layer, int descriptor_table_id, int top_k,
                                                    ITensor *output, int d_model, int intermediate) override
            {
                float *g = contiguous(gate_tensors, top_k, intermediate), *u = contiguous(up_tensors, top_k, intermediate);
                llaminar_amd::DeviceTensor out = view(output);
                if (!runtime_layer || !g || !u || !out.data)
                    return false;
                out.rows = 1;
                out.cols = d_model;
                llaminar_amd::DeviceMoELayerRuntime rt = runtimeView(runtime_layer, top_k);
                return impl_.groupedExpertDownDecodeFromRuntime(g, u, &rt, descriptor_table_id, top_k, &out, d_model,
                                                                intermediate);
            }
            // The path MoEExpertComputeStage prefers on GPUs (MoEExpertComputeStage.cpp:1141-1149).
            bool groupedExpertDecodeFromRuntime(DeviceMoELayerRuntime *runtime_layer, const TensorBase *input,
                                                int gateup_descriptor_table_id, int down_descriptor_table_id, int top_k,
                                                ITensor *output, int d_model, int intermediate) override
            {
                llaminar_amd::DeviceTensor in = view(input), out = view(output);
                if (!runtime_layer || !in.data || !out.data)
                    return false;
                in.rows = out.rows = 1;
                in.cols = out.cols = d_model;
                llaminar_amd::DeviceMoELayerRuntime rt = runtimeView(runtime_layer, top_k);
                return impl_.groupedExpertDecodeFromRuntime(&rt, &in, gateup_descriptor_table_id, down_descriptor_table_id, top_k,
                                                            &out, d_model, intermediate);
            }

            // ---- shared expert (IMoEKernel.h:344-356; default body kernels/IMoEKernel.cpp:131-158) --------
            // shared_output *= sigmoid(dot(gate_inp, input)); combined = routed_residual + shared_output.
            // Served in place (combined_output == routed_residual), which is how MoEExpertComputeStage
            // calls it (MoEExpertComputeStage.cpp:2716); anything else goes to the interface's default.
            void sharedExpertGateAddFromTensors(ITensor *input, ITensor *gate_inp, ITensor *shared_output,
                                                ITensor *routed_residual, ITensor *combined_output, int seq_len,
                                                int d_model) override
            {
                const float *in = input ? static_cast<const float *>(input->gpu_data_ptr()) : nullptr;
                const float *gi = gate_inp ? static_cast<const float *>(gate_inp->gpu_data_ptr()) : nullptr;
                float *sh = shared_output ? static_cast<float *>(shared_output->gpu_data_ptr()) : nullptr;
                float *out = combined_output ? static_cast<float *>(combined_output->gpu_data_ptr()) : nullptr;
                if (!in || !gi || !sh || !out || !routed_residual || routed_residual->gpu_data_ptr() != out)
                {
                    IMoEKernel::sharedExpertGateAddFromTensors(input, gate_inp, shared_output, routed_residual, combined_output,
                                                               seq_len, d_model);
                    return;
                }
                if (impl_.sharedExpertGate(in, gi, sh, seq_len, d_model))
                    (void)impl_.weightedAdd(out, sh, 1.0f, seq_len * d_model);
            }

        private:
            static constexpr int kNoRowBound = 0x7fffffff;

            static llaminar_amd::DeviceTensor view(const ITensor *t)
            {
                if (!t)
                    return {};
                auto *p = static_cast<float *>(const_cast<void *>(t->gpu_data_ptr()));
                return llaminar_amd::DeviceTensor(p, static_cast<int>(t->rows()), static_cast<int>(t->cols()));
            }
            template <typename T>
            static T *member(DeviceMoELayerRuntime *device_struct, size_t offset)
            {
                return reinterpret_cast<T *>(reinterpret_cast<unsigned char *>(device_struct) + offset);
            }
            // The operator's view of one token's slots inside the device-resident runtime struct.
            static llaminar_amd::DeviceMoELayerRuntime runtimeView(DeviceMoELayerRuntime *device_struct, int top_k)
            {
                llaminar_amd::DeviceMoELayerRuntime rt;
                rt.topk_expert_ids = member<int32_t>(device_struct, offsetof(DeviceMoELayerRuntime, topk_expert_ids));
                rt.topk_weights = member<float>(device_struct, offsetof(DeviceMoELayerRuntime, topk_weights));
                rt.top_k = top_k;
                rt.slot_stride = top_k;
                return rt;
            }
            // The reference passes one tensor per slot; the operator wants [slots x intermediate] in one
            // piece.  Returns the base when the slot tensors already lie that way (a stage that carves its
            // per-slot scratch from one buffer), else null and the caller reports "not served".
            static float *contiguous(ITensor *const *slots, int n, int intermediate)
            {
                if (!slots || n <= 0 || !slots[0])
                    return nullptr;
                auto *base = static_cast<float *>(slots[0]->gpu_data_ptr());
                if (!base)
                    return nullptr;
                for (int i = 1; i < n; ++i)
                    if (!slots[i] || static_cast<float *>(slots[i]->gpu_data_ptr()) != base + static_cast<size_t>(i) * intermediate)
                        return nullptr;
                return base;
            }
            static std::vector<llaminar_amd::DeviceQuantMatrixDesc> convert(const DeviceNativeVNNIMatrixDesc *descs, int n)
            {
                std::vector<llaminar_amd::DeviceQuantMatrixDesc> out(static_cast<size_t>(n));
                for (int i = 0; i < n; ++i)
                {
                    // entries of experts that live elsewhere stay invalid and are skipped by the launches
                    if (!descs[i].valid())
                        continue;
                    out[i].weights = descs[i].payload;
                    out[i].n = descs[i].n;
                    out[i].k = descs[i].k;
                    out[i].blocks_per_row = descs[i].blocks_per_row;
                    out[i].codebook_id = descs[i].codebook_id;
                }
                return out;
            }

            llaminar_amd::MI355MoEKernel impl_;
            DeviceWorkspaceManager *workspace_ = nullptr;
            void *stream_ = nullptr;
            int device_ = 0;
        };
    } // namespace mi355
} // namespace llaminar2
