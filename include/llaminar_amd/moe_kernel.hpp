// Host-side MoE operator for the MI355X path: the decode methods of the reference's
// IMoEKernel (src/v2/kernels/IMoEKernel.h:56-660) over device memory -- routing from the
// router matrix, persistent expert descriptor tables, grouped gate/up and down
// projections driven by device-resident top-k state, the fused decode sequence, the
// shared-expert gate.  Same method names, argument meaning and bool error convention;
// every method only enqueues work on the stream set with setGPUStream() and, once a
// workspace is bound, allocates nothing.  No arithmetic of its own: all of it is behind
// the llam_ql_moe_* entry points of ql_api.h.
//
// Differences from the reference interface, all because tensors here are plain device
// buffers: per-slot ITensor* arrays (gate_outputs[i], up_outputs[i]) are one contiguous
// [slots x intermediate] buffer; DeviceMoELayerRuntime carries raw device pointers.
#pragma once

#include <cstddef>
#include <cstdint>
#include <mutex>
#include <vector>

#include "llaminar_amd/quant_gemm.hpp"

namespace llaminar_amd
{
    // Device-resident top-k state of one MoE layer (the role of the reference's
    // DeviceMoELayerRuntime: topk_expert_ids / topk_weights written by decodeRouteSelect and
    // read by the grouped launches without a host round trip).  Slots of a token are
    // slot_stride apart; slots top_k..slot_stride-1 belong to the caller (always-on experts
    // such as the shared expert, with their weights).
    struct DeviceMoELayerRuntime
    {
        int32_t *topk_expert_ids = nullptr; // [n_tokens][slot_stride]
        float *topk_weights = nullptr;      // [n_tokens][slot_stride]
        int top_k = 0;
        int slot_stride = 0; // 0 means top_k
        int stride() const { return slot_stride ? slot_stride : top_k; }
    };

    // Host-side routing result (reference: MoERoutingResult, src/v2/kernels/IMoEKernel.h:37-42).
    struct MoERoutingResult
    {
        std::vector<int> expert_indices;   // [seq_len * top_k]
        std::vector<float> expert_weights; // [seq_len * top_k]
        std::vector<float> router_logits;  // [seq_len * num_experts] probabilities after the softmax
    };

    // Reason of the calling thread's last failed MI355MoEKernel call.
    const char *moe_kernel_last_error();

    class MI355MoEKernel
    {
    public:
        explicit MI355MoEKernel(int device_id);
        ~MI355MoEKernel();
        MI355MoEKernel(const MI355MoEKernel &) = delete;
        MI355MoEKernel &operator=(const MI355MoEKernel &) = delete;

        bool supports_device(int device_idx) const { return device_idx == device_id_; }
        void setGPUStream(void *stream) { stream_ = stream; }
        bool isValid() const { return valid_; }
        // nothing of its own to snapshot: the expert matrices belong to their GEMM operators
        // (kernels/rocm/moe/ROCmMoEKernel.h:387-390)
        KernelSnapshotInfo getKernelSnapshotInfo() const
        {
            KernelSnapshotInfo info;
            info.kernel_name = "MoE";
            info.kernel_description = "pass-through";
            info.is_passthrough = true;
            return info;
        }

        // ---- workspace -----------------------------------------------------------------
        // Bytes the decode methods need for n_tokens tokens of `slots` expert slots each:
        // router logits, the Q8_1 hidden state, the gate/up outputs and their Q8_1 SwiGLU.
        static size_t getWorkspaceRequirements(int n_tokens, int slots, int d_model, int intermediate, int num_experts);
        void bindWorkspace(const DeviceWorkspace &ws) { bound_ = ws; }

        // ---- descriptor tables (IMoEKernel.h:409-450) ----------------------------------------
        // Persistent all-expert tables in device memory; entries that are not valid() (experts
        // that live elsewhere) stay null and are skipped by the launches.  Returns a table id,
        // -1 on error.  All experts of a table share one weight format.
        int uploadGroupedExpertGateUpDescriptorTables(const DeviceQuantMatrixDesc *gate_descs,
                                                      const DeviceQuantMatrixDesc *up_descs, int num_experts,
                                                      int d_model, int intermediate);
        int uploadGroupedExpertDownDescriptorTable(const DeviceQuantMatrixDesc *down_descs, int num_experts,
                                                   int d_model, int intermediate);

        // ---- routing (IMoEKernel.h:245-258; CPUMoEKernel::route) -------------------------------
        // hidden [n_tokens x d_model] and gate_weights [num_experts x d_model] fp32 in device
        // memory -> runtime_layer's top-k ids and weights (device).  output_probs (optional)
        // is not written; the softmax lives in registers.
        bool decodeRouteSelect(DeviceMoELayerRuntime *runtime_layer, const DeviceTensor *hidden,
                               const DeviceTensor *gate_weights, int d_model, int num_experts, int top_k,
                               bool normalize_weights);

        // IMoEKernel::route (IMoEKernel.h:84-90): the same routing with the result on the host.
        // hidden and gate_weights are device pointers; the call waits for the stream (the result
        // is host memory by its interface).
        bool route(const float *hidden, const float *gate_weights, int seq_len, int d_model, int num_experts,
                   int top_k, bool normalize_weights, MoERoutingResult &result);
        // IMoEKernel::weightedAdd (IMoEKernel.h:189-195): output[i] += weight * input[i], device buffers.
        bool weightedAdd(float *output, const float *input, float weight, int count);
        // The other device helpers of the interface (IMoEKernel.h:92-171), all over device
        // pointers, enqueued on the operator's stream.  token_indices are device int32; num_rows
        // bounds them (rows of `hidden` / `output`).
        bool gatherTokenBatch(const float *hidden, float *batch_buffer, const int *token_indices, int num_tokens,
                              int d_model, int num_rows);
        bool scatterAddWeighted(float *output, const float *expert_output, const int *token_indices,
                                const float *weights, int num_tokens, int d_model, int num_rows);
        bool sharedExpertGate(const float *input, const float *gate_inp, float *shared_output, int seq_len,
                              int d_model);
        bool swiGLU(float *gate, const float *up, int count);

        // ---- single-token grouped projections from host or fp32 device routing ------------------
        // (IMoEKernel.h:452-575)  FromTable: expert_ids / expert_weights are HOST arrays of the
        // num_active slots, uploaded as per-call metadata.  FromRouting: routing_indices /
        // routing_weights are DEVICE tensors of top_k fp32 values.  gate_outputs / up_outputs:
        // one contiguous [slots x intermediate] device buffer; output [1 x d_model], overwritten.
        bool groupedExpertGateUpDecodeFromTable(const DeviceTensor *input, const int *expert_ids,
                                                int descriptor_table_id, int num_active, float *gate_outputs,
                                                float *up_outputs, int d_model, int intermediate);
        bool groupedExpertGateUpDecodeFromRouting(const DeviceTensor *input, const float *routing_indices,
                                                  int descriptor_table_id, int top_k, float *gate_outputs,
                                                  float *up_outputs, int d_model, int intermediate);
        bool groupedExpertDownDecodeFromTable(const float *gate_tensors, const float *up_tensors,
                                              const int *expert_ids, const float *expert_weights,
                                              int descriptor_table_id, int num_active, DeviceTensor *output,
                                              int d_model, int intermediate);
        bool groupedExpertDownDecodeFromRouting(const float *gate_tensors, const float *up_tensors,
                                                const float *routing_indices, const float *routing_weights,
                                                int descriptor_table_id, int top_k, DeviceTensor *output, int d_model,
                                                int intermediate);

        // ---- grouped projections (IMoEKernel.h:508-620) ------------------------------------------
        // input [n_tokens x d_model] fp32; gate_outputs / up_outputs [n_tokens*slots x intermediate].
        bool groupedExpertGateUpDecodeFromRuntime(DeviceMoELayerRuntime *runtime_layer, const DeviceTensor *input,
                                                  int descriptor_table_id, int top_k, float *gate_outputs,
                                                  float *up_outputs, int d_model, int intermediate);
        // output [n_tokens x d_model] = sum over slots of weight * W_down (silu(gate) * up); overwrites.
        bool groupedExpertDownDecodeFromRuntime(const float *gate_tensors, const float *up_tensors,
                                                DeviceMoELayerRuntime *runtime_layer, int descriptor_table_id,
                                                int top_k, DeviceTensor *output, int d_model, int intermediate);
        // gate/up, SwiGLU + quantise, down as one graph-capturable launch sequence (IMoEKernel.h:624-645).
        bool groupedExpertDecodeFromRuntime(DeviceMoELayerRuntime *runtime_layer, const DeviceTensor *input,
                                            int gateup_descriptor_table_id, int down_descriptor_table_id, int top_k,
                                            DeviceTensor *output, int d_model, int intermediate);

        // ---- shared expert (IMoEKernel.h:151-170, 344-356) ------------------------------------------
        // output[t,:] += sigmoid(dot(gate_inp, hidden[t,:])) * shared[t,:]  (gate 1 when gate_inp is null)
        bool sharedExpertGateAdd(DeviceTensor *output, const DeviceTensor *shared, const DeviceTensor *hidden,
                                 const float *gate_inp, int seq_len, int d_model);

        int tableCount() const { return (int)tables_.size(); }

    private:
        struct Table
        {
            llam_ql_expert *d_entries = nullptr;
            int num_experts = 0, d_model = 0, intermediate = 0;
            uint8_t fmt = 0;
            bool has_gate_up = false, has_down = false;
        };
        const Table *table(const char *fn, int id, bool want_down, int d_model, int intermediate) const;
        int add_table(const char *fn, const DeviceQuantMatrixDesc *a, const DeviceQuantMatrixDesc *b,
                      const DeviceQuantMatrixDesc *c, int num_experts, int d_model, int intermediate);
        bool gate_up_ids(const char *fn, const DeviceTensor *input, const int32_t *d_ids, uint8_t *scratch_after_ids,
                         size_t scratch_left, const Table *t, int slots, float *gate_outputs, float *up_outputs);
        bool down_ids(const char *fn, const float *gate_tensors, const float *up_tensors, const int32_t *d_ids,
                      const float *d_weights, uint8_t *scratch, size_t scratch_left, const Table *t, int slots,
                      DeviceTensor *output);
        struct Scratch
        {
            uint8_t *p = nullptr;
            size_t left = 0;
            void *take(size_t bytes);
        };
        bool open_scratch(const char *fn, size_t bytes, Scratch &s);

        int device_id_;
        bool valid_ = false;
        void *stream_ = nullptr;
        DeviceWorkspace bound_;
        void *own_ = nullptr; // grow-only fallback when no workspace is bound
        size_t own_bytes_ = 0;
        std::vector<Table> tables_;
        std::mutex mu_;
    };
} // namespace llaminar_amd
