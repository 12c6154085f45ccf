// MI355MoEKernel: host logic above the llam_ql_moe_* entry points.
#include "llaminar_amd/moe_kernel.hpp"

#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>

namespace llaminar_amd
{
    namespace
    {
        thread_local char g_moe_error[512] = "";

        bool fail(const char *fn, const char *fmt, ...)
        {
            char msg[400];
            va_list ap;
            va_start(ap, fmt);
            vsnprintf(msg, sizeof msg, fmt, ap);
            va_end(ap);
            snprintf(g_moe_error, sizeof g_moe_error, "[MI355MoEKernel::%s] %s", fn, msg);
            fprintf(stderr, "%s\n", g_moe_error);
            return false;
        }
        bool forward(const char *fn, bool ok)
        {
            if (!ok)
                snprintf(g_moe_error, sizeof g_moe_error, "[MI355MoEKernel::%s] %s", fn, llam_ql_last_error());
            return ok;
        }
        constexpr size_t ALIGN = 256;
        constexpr size_t GROUP_MIN_PAIRS = 432; // (token, slot) pairs from which batches are grouped by expert
        size_t round_up(size_t b) { return (b + ALIGN - 1) / ALIGN * ALIGN; }
        size_t q8_bytes(size_t rows, int k) { return rows * (size_t)(k / 32) * sizeof(llam_block_q8_1); }
    } // namespace

    const char *moe_kernel_last_error() { return g_moe_error; }

    MI355MoEKernel::MI355MoEKernel(int device_id) : device_id_(device_id)
    {
        if (device_id < 0 || device_id >= 16)
            fail("ctor", "bad device id %d", device_id);
        else
            valid_ = true;
    }

    MI355MoEKernel::~MI355MoEKernel()
    {
        for (Table &t : tables_)
            if (t.d_entries)
                (void)hipFree(t.d_entries);
        if (own_)
            (void)hipFree(own_);
    }

    size_t MI355MoEKernel::getWorkspaceRequirements(int n_tokens, int slots, int d_model, int intermediate,
                                                    int num_experts)
    {
        if (n_tokens < 1 || slots < 1 || d_model < 32 || intermediate < 32 || num_experts < 1)
            return 0;
        const size_t rows = (size_t)n_tokens * slots;
        // (+ the pair table and the per-pair down rows of the grouped path, + ids and weights of
        // the FromTable / FromRouting calls)
        return round_up((size_t)n_tokens * num_experts * 4) + round_up(q8_bytes(n_tokens, d_model)) +
               2 * round_up(rows * intermediate * 4) + round_up(q8_bytes(rows, intermediate)) +
               round_up(llam_ql_moe_group_bytes(n_tokens, slots)) + round_up(rows * d_model * 4) +
               2 * round_up(rows * 4);
    }

    void *MI355MoEKernel::Scratch::take(size_t bytes)
    {
        bytes = round_up(bytes);
        if (bytes > left)
            return nullptr;
        void *r = p;
        p += bytes;
        left -= bytes;
        return r;
    }

    bool MI355MoEKernel::open_scratch(const char *fn, size_t bytes, Scratch &s)
    {
        if (bound_.base)
        {
            if (bound_.bytes < bytes)
                return fail(fn, "bound workspace of %zu bytes is smaller than the %zu needed", bound_.bytes, bytes);
            s.p = static_cast<uint8_t *>(bound_.base);
            s.left = bound_.bytes;
            return true;
        }
        std::lock_guard<std::mutex> lock(mu_);
        if (own_bytes_ < bytes)
        {
            if (hipSetDevice(device_id_) != hipSuccess)
                return fail(fn, "hipSetDevice(%d) failed", device_id_);
            if (own_)
                (void)hipFree(own_);
            own_ = nullptr;
            own_bytes_ = 0;
            if (hipMalloc(&own_, bytes) != hipSuccess)
                return fail(fn, "cannot allocate %zu bytes of scratch", bytes);
            own_bytes_ = bytes;
        }
        s.p = static_cast<uint8_t *>(own_);
        s.left = own_bytes_;
        return true;
    }

    int MI355MoEKernel::add_table(const char *fn, const DeviceQuantMatrixDesc *a, const DeviceQuantMatrixDesc *b,
                                  const DeviceQuantMatrixDesc *c, int num_experts, int d_model, int intermediate)
    {
        if (!valid_)
            return fail(fn, "invalid kernel object"), -1;
        if (num_experts < 1 || d_model < 256 || d_model % 256 || intermediate < 256 || intermediate % 256)
            return fail(fn, "bad shape (num_experts=%d d_model=%d intermediate=%d)", num_experts, d_model, intermediate), -1;
        std::vector<llam_ql_expert> host((size_t)num_experts);
        uint8_t fmt = 0;
        for (int e = 0; e < num_experts; ++e)
        {
            host[e] = llam_ql_expert{nullptr, nullptr, nullptr};
            const DeviceQuantMatrixDesc *set[3] = {a ? a + e : nullptr, b ? b + e : nullptr, c ? c + e : nullptr};
            for (int i = 0; i < 3; ++i)
            {
                const DeviceQuantMatrixDesc *d = set[i];
                if (!d || !d->valid())
                    continue; // a non-local expert: skipped by the launches
                const int want_n = i == 2 ? d_model : intermediate, want_k = i == 2 ? intermediate : d_model;
                if (d->n != want_n || d->k != want_k)
                    return fail(fn, "expert %d: matrix is %d x %d, expected %d x %d", e, d->n, d->k, want_n, want_k), -1;
                if (fmt == 0)
                    fmt = d->codebook_id;
                else if (fmt != d->codebook_id)
                    return fail(fn, "expert %d: format %d differs from the table's %d", e, (int)d->codebook_id, (int)fmt), -1;
                (i == 0 ? host[e].d_gate : i == 1 ? host[e].d_up : host[e].d_down) = d->weights;
            }
        }
        if (fmt == 0 || llam_format_block_bytes(fmt) == 0)
            return fail(fn, "no valid expert in the table"), -1;
        Table t;
        t.num_experts = num_experts;
        t.d_model = d_model;
        t.intermediate = intermediate;
        t.fmt = fmt;
        t.has_gate_up = a != nullptr;
        t.has_down = c != nullptr;
        if (hipSetDevice(device_id_) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&t.d_entries), host.size() * sizeof(llam_ql_expert)) != hipSuccess)
            return fail(fn, "cannot allocate the descriptor table"), -1;
        if (hipMemcpy(t.d_entries, host.data(), host.size() * sizeof(llam_ql_expert), hipMemcpyHostToDevice) !=
            hipSuccess)
        {
            (void)hipFree(t.d_entries);
            return fail(fn, "descriptor table upload failed"), -1;
        }
        std::lock_guard<std::mutex> lock(mu_);
        tables_.push_back(t);
        return (int)tables_.size() - 1;
    }

    int MI355MoEKernel::uploadGroupedExpertGateUpDescriptorTables(const DeviceQuantMatrixDesc *gate_descs,
                                                                  const DeviceQuantMatrixDesc *up_descs,
                                                                  int num_experts, int d_model, int intermediate)
    {
        static const char *fn = "uploadGroupedExpertGateUpDescriptorTables";
        if (!gate_descs || !up_descs)
            return fail(fn, "null descriptor array"), -1;
        return add_table(fn, gate_descs, up_descs, nullptr, num_experts, d_model, intermediate);
    }

    int MI355MoEKernel::uploadGroupedExpertDownDescriptorTable(const DeviceQuantMatrixDesc *down_descs, int num_experts,
                                                               int d_model, int intermediate)
    {
        static const char *fn = "uploadGroupedExpertDownDescriptorTable";
        if (!down_descs)
            return fail(fn, "null descriptor array"), -1;
        return add_table(fn, nullptr, nullptr, down_descs, num_experts, d_model, intermediate);
    }

    const MI355MoEKernel::Table *MI355MoEKernel::table(const char *fn, int id, bool want_down, int d_model,
                                                       int intermediate) const
    {
        if (id < 0 || id >= (int)tables_.size())
        {
            fail(fn, "descriptor table id %d outside [0,%d)", id, (int)tables_.size());
            return nullptr;
        }
        const Table &t = tables_[id];
        if (want_down ? !t.has_down : !t.has_gate_up)
        {
            fail(fn, "descriptor table %d holds no %s matrices", id, want_down ? "down" : "gate/up");
            return nullptr;
        }
        if (t.d_model != d_model || t.intermediate != intermediate)
        {
            fail(fn, "descriptor table %d is for %d x %d, call says %d x %d", id, t.d_model, t.intermediate, d_model,
                 intermediate);
            return nullptr;
        }
        return &t;
    }

    bool MI355MoEKernel::decodeRouteSelect(DeviceMoELayerRuntime *rt, const DeviceTensor *hidden,
                                           const DeviceTensor *gate_weights, int d_model, int num_experts, int top_k,
                                           bool normalize_weights)
    {
        static const char *fn = "decodeRouteSelect";
        if (!valid_)
            return false;
        if (!rt || !hidden || !gate_weights || !hidden->data || !gate_weights->data)
            return fail(fn, "null tensor");
        if (!rt->topk_expert_ids || !rt->topk_weights)
            return fail(fn, "runtime layer has no top-k buffers");
        if (hidden->cols != d_model || gate_weights->cols != d_model || gate_weights->rows != num_experts)
            return fail(fn, "shapes: hidden %d x %d, gate %d x %d, call d_model=%d num_experts=%d", hidden->rows,
                        hidden->cols, gate_weights->rows, gate_weights->cols, d_model, num_experts);
        if (hidden->stride() != d_model || gate_weights->stride() != d_model)
            return fail(fn, "hidden and gate_weights must be dense rows");
        const int stride = rt->slot_stride ? rt->slot_stride : top_k;
        if (stride < top_k)
            return fail(fn, "slot_stride=%d smaller than top_k=%d", stride, top_k);
        const int T = hidden->rows;
        Scratch s;
        if (!open_scratch(fn, round_up((size_t)T * num_experts * 4), s))
            return false;
        float *logits = static_cast<float *>(s.take((size_t)T * num_experts * 4));
        if (!forward(fn, llam_ql_moe_router_logits(hidden->data, gate_weights->data, logits, T, d_model, num_experts,
                                                   device_id_, stream_)))
            return false;
        rt->top_k = top_k;
        return forward(fn, llam_ql_moe_route_ex(logits, T, num_experts, top_k, normalize_weights ? 1 : 0,
                                                rt->topk_expert_ids, rt->topk_weights, stride, device_id_, stream_));
    }

    bool MI355MoEKernel::groupedExpertGateUpDecodeFromRuntime(DeviceMoELayerRuntime *rt, const DeviceTensor *input,
                                                              int table_id, int top_k, float *gate_outputs,
                                                              float *up_outputs, int d_model, int intermediate)
    {
        static const char *fn = "groupedExpertGateUpDecodeFromRuntime";
        if (!valid_)
            return false;
        if (!rt || !rt->topk_expert_ids || !input || !input->data || !gate_outputs || !up_outputs)
            return fail(fn, "null argument");
        const Table *t = table(fn, table_id, false, d_model, intermediate);
        if (!t)
            return false;
        if (input->cols != d_model || input->stride() != d_model)
            return fail(fn, "input must be dense rows of d_model=%d", d_model);
        if (rt->stride() != top_k)
            return fail(fn, "top_k=%d must cover the runtime layer's %d slots per token", top_k, rt->stride());
        const int T = input->rows;
        Scratch s;
        if (!open_scratch(fn, round_up(q8_bytes(T, d_model)), s))
            return false;
        void *q8 = s.take(q8_bytes(T, d_model));
        if (!forward(fn, llam_ql_quantize_q8_1(input->data, q8, T, d_model, device_id_, stream_)))
            return false;
        return forward(fn, llam_ql_moe_gate_up(t->fmt, t->d_entries, t->num_experts, rt->topk_expert_ids, q8,
                                               gate_outputs, up_outputs, T, top_k, d_model, intermediate, device_id_,
                                               stream_));
    }

    bool MI355MoEKernel::groupedExpertDownDecodeFromRuntime(const float *gate_tensors, const float *up_tensors,
                                                            DeviceMoELayerRuntime *rt, int table_id, int top_k,
                                                            DeviceTensor *output, int d_model, int intermediate)
    {
        static const char *fn = "groupedExpertDownDecodeFromRuntime";
        if (!valid_)
            return false;
        if (!rt || !rt->topk_expert_ids || !rt->topk_weights || !gate_tensors || !up_tensors || !output ||
            !output->data)
            return fail(fn, "null argument");
        const Table *t = table(fn, table_id, true, d_model, intermediate);
        if (!t)
            return false;
        if (output->cols != d_model || output->stride() != d_model)
            return fail(fn, "output must be dense rows of d_model=%d", d_model);
        if (rt->stride() != top_k)
            return fail(fn, "top_k=%d must cover the runtime layer's %d slots per token", top_k, rt->stride());
        const int T = output->rows;
        const size_t rows = (size_t)T * top_k;
        Scratch s;
        if (!open_scratch(fn, round_up(q8_bytes(rows, intermediate)), s))
            return false;
        void *qa = s.take(q8_bytes(rows, intermediate));
        if (!forward(fn, llam_ql_swiglu_quantize(gate_tensors, up_tensors, nullptr, qa, (int)rows, intermediate,
                                                 device_id_, stream_)))
            return false;
        return forward(fn, llam_ql_moe_down(t->fmt, t->d_entries, t->num_experts, rt->topk_expert_ids,
                                            rt->topk_weights, qa, output->data, T, top_k, d_model, intermediate, 0,
                                            device_id_, stream_));
    }

    bool MI355MoEKernel::groupedExpertDecodeFromRuntime(DeviceMoELayerRuntime *rt, const DeviceTensor *input,
                                                        int gu_table, int down_table, int top_k, DeviceTensor *output,
                                                        int d_model, int intermediate)
    {
        static const char *fn = "groupedExpertDecodeFromRuntime";
        if (!valid_)
            return false;
        if (!rt || !input || !input->data || !output || !output->data)
            return fail(fn, "null argument");
        const Table *tg = table(fn, gu_table, false, d_model, intermediate);
        const Table *td = tg ? table(fn, down_table, true, d_model, intermediate) : nullptr;
        if (!tg || !td)
            return false;
        if (input->cols != d_model || input->stride() != d_model || output->cols != d_model ||
            output->stride() != d_model || input->rows != output->rows)
            return fail(fn, "input and output must be dense [tokens x d_model=%d]", d_model);
        if (rt->stride() != top_k || !rt->topk_expert_ids || !rt->topk_weights)
            return fail(fn, "top_k=%d must cover the runtime layer's %d slots per token", top_k, rt->stride());
        const int T = input->rows;
        const size_t rows = (size_t)T * top_k;
        // Batches of GROUP_MIN_PAIRS (token, slot) pairs and more are sorted by expert on the
        // device, so that every distinct expert's matrices are decoded once per chunk of its
        // tokens (measured on the 256-expert IQ3_S shape with 9 slots per token, grouped against per slot:
        // 40 tokens 126 / 127 us, 48 tokens 142 / 144, 64 tokens 155 / 188, 128 tokens 228 / 340 us).
        const bool grouped = rows >= GROUP_MIN_PAIRS && rows <= 4096 && tg->num_experts <= 2048 &&
                             tg->num_experts == td->num_experts;
        Scratch s;
        if (!open_scratch(fn, round_up(q8_bytes(T, d_model)) + 2 * round_up(rows * intermediate * 4) +
                                  round_up(q8_bytes(rows, intermediate)) +
                                  (grouped ? round_up(llam_ql_moe_group_bytes(T, top_k)) + round_up(rows * d_model * 4)
                                           : 0),
                          s))
            return false;
        void *q8 = s.take(q8_bytes(T, d_model));
        float *gate = static_cast<float *>(s.take(rows * intermediate * 4));
        float *up = static_cast<float *>(s.take(rows * intermediate * 4));
        void *qa = s.take(q8_bytes(rows, intermediate));
        if (grouped)
        {
            void *grp = s.take(llam_ql_moe_group_bytes(T, top_k));
            float *pair_out = static_cast<float *>(s.take(rows * d_model * 4));
            return forward(fn, llam_ql_quantize_q8_1(input->data, q8, T, d_model, device_id_, stream_)) &&
                   forward(fn, llam_ql_moe_group(rt->topk_expert_ids, T, top_k, tg->num_experts, grp, device_id_,
                                                 stream_)) &&
                   forward(fn, llam_ql_moe_gate_up_grouped(tg->fmt, tg->d_entries, tg->num_experts, grp, q8, gate, up,
                                                           T, top_k, d_model, intermediate, device_id_, stream_)) &&
                   forward(fn, llam_ql_swiglu_quantize(gate, up, nullptr, qa, (int)rows, intermediate, device_id_,
                                                       stream_)) &&
                   forward(fn, llam_ql_moe_down_grouped(td->fmt, td->d_entries, td->num_experts, grp,
                                                        rt->topk_expert_ids, rt->topk_weights, qa, pair_out,
                                                        output->data, T, top_k, d_model, intermediate, 0, device_id_,
                                                        stream_));
        }
        return forward(fn, llam_ql_quantize_q8_1(input->data, q8, T, d_model, device_id_, stream_)) &&
               // gate/up, SwiGLU and its Q8_1 quantiser: one launch where the format and row length allow,
               // else two through the fp32 rows
               forward(fn, llam_ql_moe_gate_up_swiglu(tg->fmt, tg->d_entries, tg->num_experts, rt->topk_expert_ids, q8,
                                                      gate, up, qa, T, top_k, d_model, intermediate, device_id_,
                                                      stream_)) &&
               forward(fn, llam_ql_moe_down(td->fmt, td->d_entries, td->num_experts, rt->topk_expert_ids,
                                            rt->topk_weights, qa, output->data, T, top_k, d_model, intermediate, 0,
                                            device_id_, stream_));
    }

    // ---- routing with a host-side result -------------------------------------------------------------
    bool MI355MoEKernel::route(const float *hidden, const float *gate_weights, int seq_len, int d_model,
                               int num_experts, int top_k, bool normalize_weights, MoERoutingResult &result)
    {
        static const char *fn = "route";
        if (!valid_)
            return false;
        if (!hidden || !gate_weights || seq_len < 1 || top_k < 1 || top_k > num_experts)
            return fail(fn, "bad argument (seq_len=%d top_k=%d num_experts=%d)", seq_len, top_k, num_experts);
        const size_t nl = (size_t)seq_len * num_experts, nk = (size_t)seq_len * top_k;
        Scratch s;
        if (!open_scratch(fn, round_up(nl * 4) + 2 * round_up(nk * 4), s))
            return false;
        float *logits = static_cast<float *>(s.take(nl * 4));
        int32_t *ids = static_cast<int32_t *>(s.take(nk * 4));
        float *w = static_cast<float *>(s.take(nk * 4));
        if (!forward(fn, llam_ql_moe_router_logits(hidden, gate_weights, logits, seq_len, d_model, num_experts,
                                                   device_id_, stream_)) ||
            !forward(fn, llam_ql_moe_route_ex(logits, seq_len, num_experts, top_k, normalize_weights ? 1 : 0, ids, w,
                                              top_k, device_id_, stream_)))
            return false;
        result.expert_indices.resize(nk);
        result.expert_weights.resize(nk);
        result.router_logits.resize(nl);
        hipStream_t st = static_cast<hipStream_t>(stream_);
        static_assert(sizeof(int) == sizeof(int32_t), "expert ids are 32-bit");
        if (hipMemcpyAsync(result.expert_indices.data(), ids, nk * 4, hipMemcpyDeviceToHost, st) != hipSuccess ||
            hipMemcpyAsync(result.expert_weights.data(), w, nk * 4, hipMemcpyDeviceToHost, st) != hipSuccess ||
            hipMemcpyAsync(result.router_logits.data(), logits, nl * 4, hipMemcpyDeviceToHost, st) != hipSuccess ||
            hipStreamSynchronize(st) != hipSuccess)
            return fail(fn, "copy of the routing result to the host failed");
        // the probabilities the reference reports (CPUMoEKernel.cpp:87-110): exp(l - max) * (1 / sum)
        for (int t = 0; t < seq_len; ++t)
        {
            float *row = result.router_logits.data() + (size_t)t * num_experts;
            float mx = row[0];
            for (int e = 1; e < num_experts; ++e)
                mx = row[e] > mx ? row[e] : mx;
            double sum = 0.0;
            for (int e = 0; e < num_experts; ++e)
            {
                row[e] = expf(row[e] - mx);
                sum += (double)row[e];
            }
            const float inv = (float)(1.0 / (sum > 0.0 ? sum : 1.0));
            for (int e = 0; e < num_experts; ++e)
                row[e] *= inv;
        }
        return true;
    }

    bool MI355MoEKernel::gatherTokenBatch(const float *hidden, float *batch_buffer, const int *token_indices,
                                          int num_tokens, int d_model, int num_rows)
    {
        static const char *fn = "gatherTokenBatch";
        if (!valid_)
            return fail(fn, "operator is not valid");
        return forward(fn, llam_ql_moe_gather_rows(hidden, batch_buffer, token_indices, num_tokens, num_rows, d_model,
                                                   device_id_, stream_));
    }

    bool MI355MoEKernel::scatterAddWeighted(float *output, const float *expert_output, const int *token_indices,
                                            const float *weights, int num_tokens, int d_model, int num_rows)
    {
        static const char *fn = "scatterAddWeighted";
        if (!valid_)
            return fail(fn, "operator is not valid");
        return forward(fn, llam_ql_moe_scatter_add_weighted(output, expert_output, token_indices, weights, num_tokens,
                                                            num_rows, d_model, device_id_, stream_));
    }

    bool MI355MoEKernel::sharedExpertGate(const float *input, const float *gate_inp, float *shared_output, int seq_len,
                                          int d_model)
    {
        static const char *fn = "sharedExpertGate";
        if (!valid_)
            return fail(fn, "operator is not valid");
        return forward(fn, llam_ql_shared_expert_gate(shared_output, input, gate_inp, seq_len, d_model, device_id_,
                                                      stream_));
    }

    bool MI355MoEKernel::swiGLU(float *gate, const float *up, int count)
    {
        static const char *fn = "swiGLU";
        if (!valid_)
            return fail(fn, "operator is not valid");
        return forward(fn, llam_ql_swiglu_inplace(gate, up, count, device_id_, stream_));
    }

    bool MI355MoEKernel::weightedAdd(float *output, const float *input, float weight, int count)
    {
        static const char *fn = "weightedAdd";
        if (!valid_)
            return false;
        if (count < 0 || (count > 0 && (!output || !input)))
            return fail(fn, "bad argument");
        // C = 1 * C + weight * T over one row of `count` values
        return forward(fn, llam_ql_epilogue(output, input, nullptr, 1, count, count, weight, 1.0f, device_id_, stream_));
    }

    // ---- single-token projections driven by host ids or fp32 device routing ----------------------------
    bool MI355MoEKernel::gate_up_ids(const char *fn, const DeviceTensor *input, const int32_t *d_ids, uint8_t *scratch,
                                     size_t scratch_left, const Table *t, int slots, float *gate_outputs,
                                     float *up_outputs)
    {
        const size_t need = round_up(q8_bytes(1, t->d_model));
        if (scratch_left < need)
            return fail(fn, "scratch too small");
        return forward(fn, llam_ql_quantize_q8_1(input->data, scratch, 1, t->d_model, device_id_, stream_)) &&
               forward(fn, llam_ql_moe_gate_up(t->fmt, t->d_entries, t->num_experts, d_ids, scratch, gate_outputs,
                                               up_outputs, 1, slots, t->d_model, t->intermediate, device_id_, stream_));
    }

    bool MI355MoEKernel::down_ids(const char *fn, const float *gate_tensors, const float *up_tensors,
                                  const int32_t *d_ids, const float *d_weights, uint8_t *scratch, size_t scratch_left,
                                  const Table *t, int slots, DeviceTensor *output)
    {
        const size_t need = round_up(q8_bytes(slots, t->intermediate));
        if (scratch_left < need)
            return fail(fn, "scratch too small");
        return forward(fn, llam_ql_swiglu_quantize(gate_tensors, up_tensors, nullptr, scratch, slots, t->intermediate,
                                                   device_id_, stream_)) &&
               forward(fn, llam_ql_moe_down(t->fmt, t->d_entries, t->num_experts, d_ids, d_weights, scratch,
                                            output->data, 1, slots, t->d_model, t->intermediate, 0, device_id_,
                                            stream_));
    }

    bool MI355MoEKernel::groupedExpertGateUpDecodeFromTable(const DeviceTensor *input, const int *expert_ids,
                                                            int table_id, int num_active, float *gate_outputs,
                                                            float *up_outputs, int d_model, int intermediate)
    {
        static const char *fn = "groupedExpertGateUpDecodeFromTable";
        if (!valid_)
            return false;
        if (!input || !input->data || !expert_ids || !gate_outputs || !up_outputs || num_active < 1)
            return fail(fn, "null argument or no active expert");
        const Table *t = table(fn, table_id, false, d_model, intermediate);
        if (!t)
            return false;
        if (input->rows != 1 || input->cols != d_model)
            return fail(fn, "input must be one row of d_model=%d", d_model);
        Scratch s;
        if (!open_scratch(fn, round_up((size_t)num_active * 4) + round_up(q8_bytes(1, d_model)), s))
            return false;
        int32_t *ids = static_cast<int32_t *>(s.take((size_t)num_active * 4));
        // per-call routing metadata (IMoEKernel.h:528-531): a few ids, copied in stream order
        if (hipMemcpyAsync(ids, expert_ids, (size_t)num_active * 4, hipMemcpyHostToDevice,
                           static_cast<hipStream_t>(stream_)) != hipSuccess)
            return fail(fn, "upload of the expert ids failed");
        return gate_up_ids(fn, input, ids, s.p, s.left, t, num_active, gate_outputs, up_outputs);
    }

    bool MI355MoEKernel::groupedExpertGateUpDecodeFromRouting(const DeviceTensor *input, const float *routing_indices,
                                                              int table_id, int top_k, float *gate_outputs,
                                                              float *up_outputs, int d_model, int intermediate)
    {
        static const char *fn = "groupedExpertGateUpDecodeFromRouting";
        if (!valid_)
            return false;
        if (!input || !input->data || !routing_indices || !gate_outputs || !up_outputs || top_k < 1)
            return fail(fn, "null argument");
        const Table *t = table(fn, table_id, false, d_model, intermediate);
        if (!t)
            return false;
        if (input->rows != 1 || input->cols != d_model)
            return fail(fn, "input must be one row of d_model=%d", d_model);
        Scratch s;
        if (!open_scratch(fn, round_up((size_t)top_k * 4) + round_up(q8_bytes(1, d_model)), s))
            return false;
        int32_t *ids = static_cast<int32_t *>(s.take((size_t)top_k * 4));
        return forward(fn, llam_ql_moe_ids_from_f32(routing_indices, ids, top_k, device_id_, stream_)) &&
               gate_up_ids(fn, input, ids, s.p, s.left, t, top_k, gate_outputs, up_outputs);
    }

    bool MI355MoEKernel::groupedExpertDownDecodeFromTable(const float *gate_tensors, const float *up_tensors,
                                                          const int *expert_ids, const float *expert_weights,
                                                          int table_id, int num_active, DeviceTensor *output,
                                                          int d_model, int intermediate)
    {
        static const char *fn = "groupedExpertDownDecodeFromTable";
        if (!valid_)
            return false;
        if (!gate_tensors || !up_tensors || !expert_ids || !expert_weights || !output || !output->data ||
            num_active < 1)
            return fail(fn, "null argument or no active expert");
        const Table *t = table(fn, table_id, true, d_model, intermediate);
        if (!t)
            return false;
        if (output->rows != 1 || output->cols != d_model)
            return fail(fn, "output must be one row of d_model=%d", d_model);
        Scratch s;
        if (!open_scratch(fn, 2 * round_up((size_t)num_active * 4) + round_up(q8_bytes(num_active, intermediate)), s))
            return false;
        int32_t *ids = static_cast<int32_t *>(s.take((size_t)num_active * 4));
        float *w = static_cast<float *>(s.take((size_t)num_active * 4));
        hipStream_t st = static_cast<hipStream_t>(stream_);
        if (hipMemcpyAsync(ids, expert_ids, (size_t)num_active * 4, hipMemcpyHostToDevice, st) != hipSuccess ||
            hipMemcpyAsync(w, expert_weights, (size_t)num_active * 4, hipMemcpyHostToDevice, st) != hipSuccess)
            return fail(fn, "upload of the expert ids and weights failed");
        return down_ids(fn, gate_tensors, up_tensors, ids, w, s.p, s.left, t, num_active, output);
    }

    bool MI355MoEKernel::groupedExpertDownDecodeFromRouting(const float *gate_tensors, const float *up_tensors,
                                                            const float *routing_indices, const float *routing_weights,
                                                            int table_id, int top_k, DeviceTensor *output, int d_model,
                                                            int intermediate)
    {
        static const char *fn = "groupedExpertDownDecodeFromRouting";
        if (!valid_)
            return false;
        if (!gate_tensors || !up_tensors || !routing_indices || !routing_weights || !output || !output->data ||
            top_k < 1)
            return fail(fn, "null argument");
        const Table *t = table(fn, table_id, true, d_model, intermediate);
        if (!t)
            return false;
        if (output->rows != 1 || output->cols != d_model)
            return fail(fn, "output must be one row of d_model=%d", d_model);
        Scratch s;
        if (!open_scratch(fn, round_up((size_t)top_k * 4) + round_up(q8_bytes(top_k, intermediate)), s))
            return false;
        int32_t *ids = static_cast<int32_t *>(s.take((size_t)top_k * 4));
        return forward(fn, llam_ql_moe_ids_from_f32(routing_indices, ids, top_k, device_id_, stream_)) &&
               down_ids(fn, gate_tensors, up_tensors, ids, routing_weights, s.p, s.left, t, top_k, output);
    }

    bool MI355MoEKernel::sharedExpertGateAdd(DeviceTensor *output, const DeviceTensor *shared,
                                             const DeviceTensor *hidden, const float *gate_inp, int seq_len,
                                             int d_model)
    {
        static const char *fn = "sharedExpertGateAdd";
        if (!valid_)
            return false;
        if (!output || !shared || !output->data || !shared->data || (gate_inp && (!hidden || !hidden->data)))
            return fail(fn, "null tensor");
        if (output->stride() != d_model || shared->stride() != d_model || (hidden && hidden->stride() != d_model))
            return fail(fn, "tensors must be dense rows of d_model=%d", d_model);
        return forward(fn, llam_ql_shared_expert_add(output->data, shared->data, hidden ? hidden->data : nullptr,
                                                     gate_inp, seq_len, d_model, device_id_, stream_));
    }
} // namespace llaminar_amd
