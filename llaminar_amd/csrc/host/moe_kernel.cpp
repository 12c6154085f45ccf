// MI355MoEKernel: host logic above the llam_ql_moe_* entry points.
#include "llaminar_amd/moe_kernel.hpp"

#include <hip/hip_runtime_api.h>

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
        return round_up((size_t)n_tokens * num_experts * 4) + round_up(q8_bytes(n_tokens, d_model)) +
               2 * round_up(rows * intermediate * 4) + round_up(q8_bytes(rows, intermediate));
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
        Scratch s;
        if (!open_scratch(fn, round_up(q8_bytes(T, d_model)) + 2 * round_up(rows * intermediate * 4) +
                                  round_up(q8_bytes(rows, intermediate)),
                          s))
            return false;
        void *q8 = s.take(q8_bytes(T, d_model));
        float *gate = static_cast<float *>(s.take(rows * intermediate * 4));
        float *up = static_cast<float *>(s.take(rows * intermediate * 4));
        void *qa = s.take(q8_bytes(rows, intermediate));
        return forward(fn, llam_ql_quantize_q8_1(input->data, q8, T, d_model, device_id_, stream_)) &&
               forward(fn, llam_ql_moe_gate_up(tg->fmt, tg->d_entries, tg->num_experts, rt->topk_expert_ids, q8, gate,
                                               up, T, top_k, d_model, intermediate, device_id_, stream_)) &&
               forward(fn, llam_ql_swiglu_quantize(gate, up, nullptr, qa, (int)rows, intermediate, device_id_,
                                                   stream_)) &&
               forward(fn, llam_ql_moe_down(td->fmt, td->d_entries, td->num_experts, rt->topk_expert_ids,
                                            rt->topk_weights, qa, output->data, T, top_k, d_model, intermediate, 0,
                                            device_id_, stream_));
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
