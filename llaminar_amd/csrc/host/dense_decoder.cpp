// Greedy decode step of a dense decoder-only model: buffers and the order of launches.
// All arithmetic is behind the entry points of ql_api.h and decode_api.h.
#include "llaminar_amd/dense_decoder.h"

#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <utility>
#include <vector>

#include "llaminar_amd/decode_api.h"
#include "llaminar_amd/ql_api.h"

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
        snprintf(g_error, sizeof g_error, "[llam_decoder_%s] %s", fn, msg);
        fprintf(stderr, "%s\n", g_error);
        return false;
    }

    // a failed entry point has already printed its reason
    bool forward(const char *fn, bool ok)
    {
        if (!ok)
            snprintf(g_error, sizeof g_error, "[llam_decoder_%s] %s", fn, llam_ql_last_error());
        return ok;
    }

    size_t q8_bytes(int m, int k) { return (size_t)m * (size_t)(k / 32) * sizeof(llam_block_q8_1); }

    struct Decoder
    {
        llam_decoder_config cfg{};
        std::vector<llam_decoder_layer> layers;
        std::vector<bool> layer_set;
        llam_decoder_globals globals{};
        bool globals_set = false;

        std::vector<void *> owned;
        size_t owned_bytes = 0;

        int32_t *ids = nullptr, *pos = nullptr;
        int host_max_pos = 0; // the furthest sequence's position as the host counts it
        float *last_res = nullptr; // where the last step left the residual stream (x or x_alt)
        float *x = nullptr, *x_alt = nullptr, *delta = nullptr, *delta2 = nullptr, *qkv = nullptr, *attn = nullptr, *gate = nullptr, *up = nullptr;
        float *logits = nullptr, *inv_freq = nullptr, *rope_table = nullptr, *att_scratch = nullptr;
        void *q8_h = nullptr, *q8_attn = nullptr, *q8_act = nullptr, *argmax_scratch = nullptr;
        std::vector<void *> kcache, vcache;

        int qdim() const { return cfg.n_heads * cfg.head_dim; }
        int kvdim() const { return cfg.n_kv * cfg.head_dim; }

        template <class T>
        bool alloc(T *&p, size_t bytes)
        {
            void *raw = nullptr;
            if (hipMalloc(&raw, bytes ? bytes : 16) != hipSuccess)
                return fail("create", "hipMalloc of %zu bytes failed", bytes);
            owned.push_back(raw);
            owned_bytes += bytes;
            p = static_cast<T *>(raw);
            return true;
        }

        ~Decoder()
        {
            for (void *p : owned)
                (void)hipFree(p);
        }
    };

    bool fmt_ok(uint8_t f) { return llam_format_block_bytes(f) != 0; }
} // namespace

extern "C" const char *llam_decoder_last_error(void) { return g_error; }

extern "C" void *llam_decoder_create(const llam_decoder_config *c)
{
    if (!c)
    {
        fail("create", "null config");
        return nullptr;
    }
    if (c->hidden < 256 || c->hidden % 256 || c->ffn < 256 || c->ffn % 256)
    {
        fail("create", "hidden=%d and ffn=%d must be positive multiples of 256", c->hidden, c->ffn);
        return nullptr;
    }
    if (c->head_dim != 128 || c->n_heads < 1 || c->n_kv < 1 || c->n_heads % c->n_kv)
    {
        fail("create", "heads %d/%d of %d: head_dim must be 128 and n_heads a multiple of n_kv", c->n_heads, c->n_kv,
             c->head_dim);
        return nullptr;
    }
    const int G = c->n_heads / c->n_kv;
    if (G != 1 && G != 2 && G != 4 && G != 8)
    {
        fail("create", "n_heads/n_kv=%d: 1, 2, 4 or 8", G);
        return nullptr;
    }
    if (c->batch < 1 || c->batch > LLAM_QL_MAX_GEMV_M || c->n_layers < 1 || c->vocab < 1 || c->ctx_cap < 1 ||
        (c->ctx_cap % 32) != 0)
    {
        fail("create", "batch=%d (1..%d), n_layers=%d, vocab=%d, ctx_cap=%d (a multiple of 32)", c->batch, LLAM_QL_MAX_GEMV_M, c->n_layers,
             c->vocab, c->ctx_cap);
        return nullptr;
    }
    if (!(c->rms_eps >= 0.0f) || !(c->rope_theta > 1.0f))
    {
        fail("create", "rms_eps=%g rope_theta=%g", (double)c->rms_eps, (double)c->rope_theta);
        return nullptr;
    }
    if (hipSetDevice(c->device_id) != hipSuccess)
    {
        fail("create", "hipSetDevice(%d) failed", c->device_id);
        return nullptr;
    }
    Decoder *d = new Decoder;
    d->cfg = *c;
    d->layers.resize(c->n_layers);
    d->layer_set.assign(c->n_layers, false);
    const int B = c->batch, H = c->hidden, F = c->ffn;
    const int wide = H > d->qdim() ? H : d->qdim();
    bool ok = d->alloc(d->ids, (size_t)B * 4) && d->alloc(d->pos, (size_t)B * 4) &&
              d->alloc(d->x, (size_t)B * H * 4) && d->alloc(d->x_alt, (size_t)B * H * 4) &&
              d->alloc(d->delta, (size_t)B * H * 4) && d->alloc(d->delta2, (size_t)B * H * 4) &&
              d->alloc(d->qkv, (size_t)B * (d->qdim() + 2 * d->kvdim()) * 4) &&
              d->alloc(d->attn, (size_t)B * d->qdim() * 4) && d->alloc(d->gate, (size_t)B * F * 4) &&
              d->alloc(d->up, (size_t)B * F * 4) && d->alloc(d->logits, (size_t)B * c->vocab * 4) &&
              d->alloc(d->inv_freq, (size_t)(c->head_dim / 2) * 4) &&
              d->alloc(d->rope_table, (size_t)B * c->head_dim * 4) &&
              d->alloc(d->att_scratch,
                       llam_dec_attention_scratch_floats(B, c->n_heads, c->head_dim, c->ctx_cap) * 4) &&
              d->alloc(d->q8_h, q8_bytes(B, wide)) && d->alloc(d->q8_attn, q8_bytes(B, d->qdim())) &&
              d->alloc(d->q8_act, q8_bytes(B, F)) &&
              d->alloc(d->argmax_scratch, llam_dec_argmax_scratch_bytes(B, c->vocab));
    const size_t cache_bytes = (size_t)B * c->n_kv * c->ctx_cap * c->head_dim * 2;
    d->kcache.resize(c->n_layers);
    d->vcache.resize(c->n_layers);
    for (int l = 0; ok && l < c->n_layers; ++l)
        ok = d->alloc(d->kcache[l], cache_bytes) && d->alloc(d->vcache[l], cache_bytes);
    if (ok)
    {
        std::vector<float> f(c->head_dim / 2);
        llam_dec_rope_inv_freq(c->head_dim, c->rope_theta, f.data());
        ok = hipMemcpy(d->inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice) == hipSuccess &&
             hipMemset(d->ids, 0, (size_t)B * 4) == hipSuccess && hipMemset(d->pos, 0, (size_t)B * 4) == hipSuccess;
        if (!ok)
            fail("create", "initial upload failed");
    }
    if (!ok)
    {
        delete d;
        return nullptr;
    }
    return d;
}

extern "C" void llam_decoder_destroy(void *dec) { delete static_cast<Decoder *>(dec); }

extern "C" size_t llam_decoder_device_bytes(void *dec) { return dec ? static_cast<Decoder *>(dec)->owned_bytes : 0; }

extern "C" bool llam_decoder_set_layer(void *dec, int layer, const llam_decoder_layer *w)
{
    Decoder *d = static_cast<Decoder *>(dec);
    if (!d || !w)
        return fail("set_layer", "null argument");
    if (layer < 0 || layer >= d->cfg.n_layers)
        return fail("set_layer", "layer %d outside [0,%d)", layer, d->cfg.n_layers);
    if (!w->wq || !w->wk || !w->wv || !w->wo || !w->wgate || !w->wup || !w->wdown || !w->attn_norm || !w->ffn_norm)
        return fail("set_layer", "layer %d: null weight pointer", layer);
    if (!fmt_ok(w->fmt_q) || !fmt_ok(w->fmt_k) || !fmt_ok(w->fmt_v) || !fmt_ok(w->fmt_o) || !fmt_ok(w->fmt_gate) ||
        !fmt_ok(w->fmt_up) || !fmt_ok(w->fmt_down))
        return fail("set_layer", "layer %d: unsupported weight format", layer);
    d->layers[layer] = *w;
    d->layer_set[layer] = true;
    return true;
}

extern "C" bool llam_decoder_set_globals(void *dec, const llam_decoder_globals *g)
{
    Decoder *d = static_cast<Decoder *>(dec);
    if (!d || !g)
        return fail("set_globals", "null argument");
    if (!g->embed_q4k || !g->final_norm || !g->lm_head || !fmt_ok(g->fmt_lm_head))
        return fail("set_globals", "null pointer or unsupported lm_head format");
    d->globals = *g;
    d->globals_set = true;
    return true;
}

extern "C" bool llam_decoder_set_state(void *dec, const int32_t *h_ids, const int32_t *h_pos)
{
    Decoder *d = static_cast<Decoder *>(dec);
    if (!d || !h_ids || !h_pos)
        return fail("set_state", "null argument");
    for (int b = 0; b < d->cfg.batch; ++b)
        if (h_pos[b] < 0 || h_pos[b] >= d->cfg.ctx_cap)
            return fail("set_state", "position %d of sequence %d outside [0,%d)", h_pos[b], b, d->cfg.ctx_cap);
    if (hipSetDevice(d->cfg.device_id) != hipSuccess ||
        hipMemcpy(d->ids, h_ids, (size_t)d->cfg.batch * 4, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(d->pos, h_pos, (size_t)d->cfg.batch * 4, hipMemcpyHostToDevice) != hipSuccess)
        return fail("set_state", "upload failed");
    d->host_max_pos = 0;
    for (int b = 0; b < d->cfg.batch; ++b)
        d->host_max_pos = h_pos[b] > d->host_max_pos ? h_pos[b] : d->host_max_pos;
    return true;
}

extern "C" int llam_decoder_steps_left(void *dec)
{
    Decoder *d = static_cast<Decoder *>(dec);
    if (!d)
        return 0;
    const int left = d->cfg.ctx_cap - d->host_max_pos;
    return left > 0 ? left : 0;
}

extern "C" bool llam_decoder_advance(void *dec, int n)
{
    Decoder *d = static_cast<Decoder *>(dec);
    if (!d || n < 0)
        return fail("advance", "bad argument");
    if (n > llam_decoder_steps_left(dec))
        return fail("advance", "context full: %d step(s) asked for, %d left of ctx_cap=%d", n,
                    llam_decoder_steps_left(dec), d->cfg.ctx_cap);
    d->host_max_pos += n;
    return true;
}

extern "C" void *llam_decoder_buffer(void *dec, const char *name, int layer)
{
    Decoder *d = static_cast<Decoder *>(dec);
    if (!d || !name)
        return nullptr;
    if (!strcmp(name, "ids"))
        return d->ids;
    if (!strcmp(name, "pos"))
        return d->pos;
    if (!strcmp(name, "logits"))
        return d->logits;
    if (!strcmp(name, "x"))
        return d->last_res ? d->last_res : d->x;
    if (layer >= 0 && layer < d->cfg.n_layers)
    {
        if (!strcmp(name, "kcache"))
            return d->kcache[layer];
        if (!strcmp(name, "vcache"))
            return d->vcache[layer];
    }
    fail("buffer", "no buffer '%s' (layer %d)", name, layer);
    return nullptr;
}

extern "C" bool llam_decoder_step(void *dec, void *stream)
{
    static const char *fn = "step";
    Decoder *d = static_cast<Decoder *>(dec);
    if (!d)
        return fail(fn, "null handle");
    if (!d->globals_set)
        return fail(fn, "globals not set");
    for (int l = 0; l < d->cfg.n_layers; ++l)
        if (!d->layer_set[l])
            return fail(fn, "layer %d not set", l);
    const llam_decoder_config &c = d->cfg;
    const int B = c.batch, H = c.hidden, F = c.ffn, dev = c.device_id;
    const int QD = d->qdim(), KV = d->kvdim(), ldqkv = QD + 2 * KV;
    // a position at ctx_cap would neither be appended to the cache nor attended to
    if (d->host_max_pos >= c.ctx_cap)
        return fail(fn, "context full: a sequence is at position %d of ctx_cap=%d", d->host_max_pos, c.ctx_cap);

    if (!forward(fn, llam_dec_embed_q4k(d->globals.embed_q4k, c.vocab, d->ids, d->x, B, H, H, dev, stream)))
        return false;
    // the rotation of this step's positions, shared by every layer
    if (!forward(fn, llam_dec_rope_table(d->pos, d->inv_freq, d->rope_table, B, c.head_dim, dev, stream)))
        return false;
    // The residual stream: the rows in `res`, and `pending`, a delta still to be added to them (or null).
    // A projection that can add its result to its output (llam_ql_gemv_accumulate) updates `res`
    // itself and leaves nothing pending; otherwise its result waits in d->delta for the next norm.
    // Where the projections' kernels can run the norm themselves (llam_ql_gemv_fused_rmsnorm: no
    // launch for the norm) a pending delta is added into the other of the two buffers, elsewhere the
    // norm updates `res` in place.
    // (a projection whose rows were summed in two halves leaves two deltas: pending and pending2)
    float *res = d->x, *spare = d->x_alt;
    const float *pending = nullptr, *pending2 = nullptr;
    auto norm_and_project = [&](const llam_ql_proj *projs, int num, const float *gamma) {
        if (!pending2 && llam_ql_gemv_fused_rmsnorm_supported(projs, num, B, H))
        {
            if (!forward(fn, llam_ql_gemv_fused_rmsnorm(projs, num, res, pending, gamma, c.rms_eps, spare, B, H, dev,
                                                        stream)))
                return false;
            if (pending)
                std::swap(res, spare);
        }
        else
        {
            if (!forward(fn, llam_dec_rmsnorm2_q8_1(res, pending, pending2, gamma, c.rms_eps, nullptr, d->q8_h, B, H, dev, stream)))
                return false;
            if (!forward(fn, llam_ql_gemv_fused(projs, num, d->q8_h, B, H, dev, stream)))
                return false;
        }
        pending = pending2 = nullptr;
        return true;
    };
    // res += W q8 where the launch can, else delta = W q8 and pending
    auto project_into_residual = [&](uint8_t fmt, const void *w, const void *plane, const void *q8, int K) {
        if (llam_ql_gemv_accumulate_supported(fmt, B, H, K, dev))
            return forward(fn, llam_ql_gemv_accumulate(fmt, w, q8, res, B, H, K, H, dev, stream));
        pending = d->delta;
        // long rows at batches the matrix unit serves: the row's halves as two launches' worth of workgroups, each
        // staging half of the activations; the next norm adds both partial sums
        if (plane && llam_ql_gemv_plane_split_supported(fmt, B, H, K))
        {
            pending2 = d->delta2;
            return forward(fn, llam_ql_gemv_plane_split(fmt, plane, q8, d->delta, d->delta2, B, H, K, H, dev, stream));
        }
        return forward(fn, llam_ql_gemv_plane(fmt, w, plane, q8, d->delta, B, H, K, H, dev, stream));
    };
    for (int l = 0; l < c.n_layers; ++l)
    {
        const llam_decoder_layer &w = d->layers[l];
        // attention half
        llam_ql_proj qkv[3];
        qkv[0] = llam_ql_proj{w.wq, d->qkv, QD, ldqkv, w.fmt_q, w.plane_q};
        qkv[1] = llam_ql_proj{w.wk, d->qkv + QD, KV, ldqkv, w.fmt_k, w.plane_k};
        qkv[2] = llam_ql_proj{w.wv, d->qkv + QD + KV, KV, ldqkv, w.fmt_v, w.plane_v};
        if (!norm_and_project(qkv, 3, w.attn_norm))
            return false;
        // rotary embedding, the cache append and the attention in one operator; its output leaves the
        // merge kernel as Q8_1 blocks: the output projection's quantiser costs no launch of its own
        if (!forward(fn, llam_dec_rope_attention(d->qkv, ldqkv, d->rope_table, d->pos, d->kcache[l], d->vcache[l], nullptr,
                                                 0, d->q8_attn, d->att_scratch, B, c.n_heads, c.n_kv, c.head_dim,
                                                 c.ctx_cap, dev, stream)))
            return false;
        if (!project_into_residual(w.fmt_o, w.wo, w.plane_o, d->q8_attn, QD))
            return false;
        // feed-forward half
        llam_ql_proj gu[2];
        gu[0] = llam_ql_proj{w.wgate, d->gate, F, F, w.fmt_gate, w.plane_gate};
        gu[1] = llam_ql_proj{w.wup, d->up, F, F, w.fmt_up, w.plane_up};
        // batches the matrix unit serves: gate, up, SwiGLU and the Q8_1 quantiser of the result in one launch
        if (w.fmt_gate == w.fmt_up && (w.plane_gate != nullptr) == (w.plane_up != nullptr) &&
            llam_ql_gemv_gate_up_swiglu_supported(w.fmt_gate, B, F, H))
        {
            if (!forward(fn, llam_dec_rmsnorm2_q8_1(res, pending, pending2, w.ffn_norm, c.rms_eps, nullptr, d->q8_h, B, H, dev,
                                                    stream)))
                return false;
            pending = pending2 = nullptr;
            if (!forward(fn, llam_ql_gemv_gate_up_swiglu(w.fmt_gate, w.wgate, w.plane_gate, w.wup, w.plane_up, d->q8_h,
                                                         nullptr, nullptr, 0, d->q8_act, B, F, H, dev, stream)))
                return false;
            if (!project_into_residual(w.fmt_down, w.wdown, w.plane_down, d->q8_act, F))
                return false;
            continue;
        }
        if (!norm_and_project(gu, 2, w.ffn_norm))
            return false;
        if (llam_ql_gemv_accumulate_supported(w.fmt_down, B, H, F, dev))
        {
            // SwiGLU and its quantiser as a launch of their own (rows this long are not quantised
            // again by every workgroup of the projection), then res += W_down act
            if (!forward(fn, llam_ql_swiglu_quantize(d->gate, d->up, nullptr, d->q8_act, B, F, dev, stream)))
                return false;
            if (!project_into_residual(w.fmt_down, w.wdown, w.plane_down, d->q8_act, F))
                return false;
        }
        else
        {
            if (!forward(fn, llam_ql_gemv_swiglu_f32(w.fmt_down, w.wdown, w.plane_down, d->gate, d->up, F, d->delta, B, H, F, H,
                                                     d->q8_act, dev, stream)))
                return false;
            pending = d->delta;
        }
    }
    if (!forward(fn, llam_dec_rmsnorm2_q8_1(res, pending, pending2, d->globals.final_norm, c.rms_eps, nullptr, d->q8_h, B,
                                            H, dev, stream)))
        return false;
    d->last_res = res; // the final norm has added what was pending
    if (!forward(fn, llam_ql_gemv_plane(d->globals.fmt_lm_head, d->globals.lm_head, d->globals.plane_lm_head, d->q8_h,
                                        d->logits, B, c.vocab, H, c.vocab, dev, stream)))
        return false;
    if (!forward(fn, llam_dec_argmax(d->logits, c.vocab, c.vocab, B, d->ids, d->pos, d->argmax_scratch, dev, stream)))
        return false;
    d->host_max_pos += 1; // (a call recorded under stream capture counts too: the count errs on the safe side)
    return true;
}
