/* Host-side driver of one greedy decode step of a dense decoder-only model: the order
 * in which a layer's operators are enqueued, and the buffers between them.  C ABI over
 * an opaque handle, exported by the host library next to the C++ operator classes.
 *
 * The step follows the node order the reference builds for a decoder layer
 * (src/v2/models/qwen/QwenGraphBase.cpp: addPreAttentionNorm :2586, fused QKV projection,
 * addRoPE :2691, addKVCacheAppend :2736, addKVCacheAndAttention :2785,
 * addWoProjectionAndAllreduce :2937, buildFFNGraph :1974, addFinalNormToGraph :2447,
 * buildLMHeadGraph :1789) followed by greedy sampling:
 *
 *   x = embed[ids]
 *   per layer:  h  = Q8_1(rmsnorm(x += down_prev) * attn_norm)       (no add in layer 0)
 *               q,k,v = W{q,k,v} h ; rope(q, k, pos) ; cache[pos] = fp16(k, v)
 *               a  = attention(q, cache[0..pos])
 *               o  = Wo Q8_1(a)
 *               h2 = Q8_1(rmsnorm(x += o) * ffn_norm)
 *               down = Wdown Q8_1(silu(Wgate h2) * (Wup h2))
 *   logits = Wlm Q8_1(rmsnorm(x += down) * final_norm) ; ids = argmax(logits) ; pos += 1
 *
 * llam_decoder_step() only enqueues kernels on the given stream (9 per layer up to batch 4):
 * no allocation, no synchronisation, no host read of device data.  Token ids and
 * positions live in device memory and are advanced by the step itself, so a step can
 * be captured in a HIP graph once and replayed for every following token.
 *
 * Weights are borrowed: device pointers in the layouts of ql_api.h, owned by the caller
 * for the life of the handle.  All functions return false (NULL) on error and keep the
 * reason for llam_decoder_last_error(). */
#ifndef LLAMINAR_AMD_DENSE_DECODER_H
#define LLAMINAR_AMD_DENSE_DECODER_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct
{
    int hidden;    /* model width, multiple of 256 */
    int n_heads;   /* query heads */
    int n_kv;      /* key/value heads (n_heads / n_kv in {1,2,4,8}) */
    int head_dim;  /* 128 */
    int ffn;       /* feed-forward width, multiple of 256 */
    int vocab;
    int n_layers;
    int ctx_cap;   /* KV-cache positions per sequence, a multiple of 32 */
    int batch;     /* sequences decoded together, 1..8 */
    float rope_theta;
    float rms_eps;
    int device_id;
} llam_decoder_config;

typedef struct
{
    const void *wq, *wk, *wv, *wo, *wgate, *wup, *wdown; /* prepared weights (llam_ql_prepare_weights) */
    uint8_t fmt_q, fmt_k, fmt_v, fmt_o, fmt_gate, fmt_up, fmt_down;
    const float *attn_norm; /* [hidden] */
    const float *ffn_norm;  /* [hidden] */
    /* optional batch planes of the seven matrices (llam_ql_build_batch_plane), read by batches of
     * 5..8 sequences; NULL = none */
    const void *plane_q, *plane_k, *plane_v, *plane_o, *plane_gate, *plane_up, *plane_down;
} llam_decoder_layer;

typedef struct
{
    const void *embed_q4k;   /* GGUF Q4_K [vocab][hidden/256] */
    const float *final_norm; /* [hidden] */
    const void *lm_head;     /* prepared weights [vocab x hidden] */
    uint8_t fmt_lm_head;
    const void *plane_lm_head; /* optional batch plane of lm_head, or NULL */
} llam_decoder_globals;

/* Allocates the activation buffers, the KV caches (2 * n_layers * batch * n_kv * ctx_cap *
 * head_dim fp16) and the scratch of the operators on cfg->device_id. */
void *llam_decoder_create(const llam_decoder_config *cfg);
void llam_decoder_destroy(void *dec);

bool llam_decoder_set_layer(void *dec, int layer, const llam_decoder_layer *w);
bool llam_decoder_set_globals(void *dec, const llam_decoder_globals *g);

/* Current token and its position per sequence (host arrays of `batch` entries); copies
 * synchronously.  The cache must hold positions 0..pos-1 already (llam_decoder_buffer). */
bool llam_decoder_set_state(void *dec, const int32_t *h_ids, const int32_t *h_pos);

/* One token for every sequence; see the file comment.  Fails, enqueuing nothing, when a
 * sequence has reached ctx_cap: the handle counts, on the host, the position llam_decoder_set_state
 * gave plus one per call (the device advances its own copy), so the check costs no
 * synchronisation. */
bool llam_decoder_step(void *dec, void *stream);

/* Steps that may still run before the furthest sequence reaches ctx_cap, by that host count. */
int llam_decoder_steps_left(void *dec);

/* Replays of a captured step do not pass through llam_decoder_step: a caller that replays a
 * graph of the step reports the replays here (before launching them), which advances the host
 * count by n and fails, changing nothing, when fewer than n steps are left. */
bool llam_decoder_advance(void *dec, int n);

/* Device buffers, for filling caches, reading results and parity checks:
 *   "ids" int32[batch], "pos" int32[batch], "logits" fp32[batch][vocab], "x" fp32[batch][hidden]
 *   (the residual stream as the last step left it: every layer's outputs added, the input of the
 *   final norm; before the first step, the buffer the embedding will fill),
 *   "kcache" and "vcache" fp16[batch][n_kv][ctx_cap * head_dim] of `layer`,
 *   each (sequence, head) slice in the tiles llam_dec_rope_kv_append documents. */
void *llam_decoder_buffer(void *dec, const char *name, int layer);

/* Bytes of device memory the handle owns. */
size_t llam_decoder_device_bytes(void *dec);

const char *llam_decoder_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
