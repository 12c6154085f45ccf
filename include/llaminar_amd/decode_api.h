/* C ABI of the decode-step operators that sit between the quantized-linear launches
 * of a dense decoder layer (ql_api.h): token embedding, RMSNorm (with the residual
 * add in front and the Q8_1 quantisation behind it), rotary embedding with the fp16
 * KV-cache append, single-token GQA attention over that cache, and greedy sampling.
 *
 * Conventions are those of ql_api.h: every pointer named d_* is device memory, every
 * call only enqueues work on `stream` for `device_id`, returns false and records a
 * message for llam_ql_last_error() on bad arguments or a failed launch, allocates
 * nothing, and synchronises nothing.  Positions and token ids live in device memory
 * so that a captured graph of a whole step can be replayed as generation proceeds.
 *
 * Floating point throughout (no bit-exact contract): results are compared with the
 * CPU restatement at 1e-5 (RMSNorm, RoPE, embedding) and 1e-4 (attention) relative
 * to the largest output; the sampler's index is exact. */
#ifndef LLAMINAR_AMD_DECODE_API_H
#define LLAMINAR_AMD_DECODE_API_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Rows of a Q4_K embedding table as fp32: d_x[b*ldx + c] = dequant(table[d_ids[b]][c]),
 * y = (d*sc)*q - dmin*m per 32-element sub-block.  The table is GGUF Q4_K, row-major
 * [vocab][H/256] super-blocks (what llam_ql_prepare_weights leaves unchanged).
 * Replaces Q4_KTensor::decodeBlockScalar / dequantize_row (src/v2/tensors/Q4_KTensor.cpp:345-389)
 * as used by the embedding lookup.  H % 256 == 0; ids outside [0, vocab) give a zero row. */
bool llam_dec_embed_q4k(const void *d_table, int vocab, const int32_t *d_ids, float *d_x,
                        int B, int H, int ldx, int device_id, void *stream);

/* RMSNorm of M rows of H floats, optionally with the residual add in front and the
 * Q8_1 quantiser behind:
 *     if d_delta: d_x[m] += d_delta[m]              (fp32 add, d_x updated in place)
 *     rms = sqrt(float(sum_sq / H) + eps), sum of squares accumulated in double
 *     y = (x * (1/rms)) * gamma
 *     if d_y:  d_y[m]  = y (fp32, row stride H)
 *     if d_q8: d_q8[m] = Q8_1 blocks of y, the arithmetic of llam_ql_quantize_q8_1
 * Replaces rmsnorm_fused_row_* and fused_residual_rmsnorm_row_*
 * (src/v2/kernels/cpu/primitives/RMSNormPrimitives.cpp:1295-1319, 1491-1562, 1564-1650)
 * behind CPURMSNormKernelT<FP32>::apply_typed / apply_with_residual_add
 * (src/v2/kernels/cpu/ops/CPURMSNormKernelT.h:134-176, 300-322), followed by the
 * activation quantiser of the next projection.  H % 32 == 0, rows 16-byte aligned. */
bool llam_dec_rmsnorm_q8_1(float *d_x, const float *d_delta, const float *d_gamma, float eps,
                           float *d_y, void *d_q8, int M, int H, int device_id, void *stream);
/* The same with the delta in two partial sums (a projection whose rows were summed in two halves,
 * llam_ql_gemv_plane_split): d_x[m] += (d_delta[m] + d_delta2[m]).  d_delta2 == NULL is the call above. */
bool llam_dec_rmsnorm2_q8_1(float *d_x, const float *d_delta, const float *d_delta2, const float *d_gamma,
                            float eps, float *d_y, void *d_q8, int M, int H, int device_id, void *stream);

/* inv_freq[i] = exp(-log(theta) * (2 i / head_dim)), i < head_dim/2, in fp32 with the
 * host's libm: get_inv_freq_cached (src/v2/kernels/cpu/primitives/RoPEPrimitives.cpp:50-77).
 * Host function; the caller uploads the table once. */
void llam_dec_rope_inv_freq(int head_dim, float theta, float *h_inv_freq);

/* Rotary embedding of one new token per sequence and the KV-cache append.
 * d_qkv: [B][ld_qkv] fp32 with the Q heads at column 0, the K heads at column
 * n_heads*head_dim and the V heads after them (the output of the fused QKV launch).
 * Pairs (i, i + head_dim/2) of every Q and K head are rotated by
 * angle = float(pos) * inv_freq[i] (apply_rope_to_head_scalar,
 * RoPEPrimitives.cpp:180-203).  Q is rotated in place; rotated K and V are rounded
 * to fp16 (nearest even) into the caches at position d_pos[b].  Cache layouts: per
 * (sequence, KV head) a slice of ctx_cap * head_dim fp16 values, [B][n_kv] slices, tiled
 * for the matrix operands of llam_dec_attention so that each of its load instructions
 * reads one contiguous kilobyte (head_dim a multiple of 16, ctx_cap of 32):
 *   K: element (p, d) at (p/16)*16*head_dim + (d/8)*128 + (p%16)*8 + d%8
 *      (tiles of 16 positions; a 16-byte piece = 8 dims of one position)
 *   V: element (p, d) at (p/32)*32*head_dim + (d/16)*512 + ((p/8)%4)*128 + (d%16)*8 + p%8
 *      (tiles of 32 positions; a 16-byte piece = 8 positions of one dim).
 * 0 <= d_pos[b] < ctx_cap is the caller's duty (a position outside is not written).
 * Replaces RoPEStage + KVCacheAppendStage for decode
 * (src/v2/models/qwen/QwenGraphBase.cpp:2691-2736, 2738-2790). */
bool llam_dec_rope_kv_append(float *d_qkv, int ld_qkv, const float *d_inv_freq,
                             const int32_t *d_pos, void *d_kcache, void *d_vcache, int B,
                             int n_heads, int n_kv, int head_dim, int ctx_cap, int device_id,
                             void *stream);

/* Scratch floats llam_dec_attention needs for its per-chunk partial results. */
size_t llam_dec_attention_scratch_floats(int B, int n_heads, int head_dim, int ctx_cap);

/* Single-token grouped-query attention over the fp16 caches:
 * d_out[b][h][:] = softmax_p(q[b][h] . K[b][h / (n_heads/n_kv)][p] / sqrt(head_dim)) . V[...][p]
 * over p = 0 .. d_pos[b] inclusive (the token appended last).  Q heads are read from
 * d_q (row stride ld_q); outputs go to d_out (fp32, row stride ld_out) and / or to d_q8_out
 * as the Q8_1 blocks [B][n_heads*head_dim/32] of the same rows (the quantiser of the output
 * projection, with the arithmetic of llam_ql_quantize_q8_1); either may be NULL.
 * Replaces CPUFlashAttentionKernelT::compute_decode with fp16 KV
 * (src/v2/kernels/cpu/attention/CPUFlashAttentionKernelT.h:507-545, 633-662).
 * Cache layouts as llam_dec_rope_kv_append writes them; what the caches hold past
 * position d_pos[b] is never used, whatever its bits.  Both products run on the matrix
 * unit in fp16 x fp16 -> fp32: K and V are exact operands, the fp32 factors (q / sqrt(d),
 * the softmax weights) enter as the sum of two fp16 numbers, i.e. to about 2^-22;
 * |q| / sqrt(head_dim) must stay below the fp16 range (65504).
 * head_dim == 128, n_heads / n_kv in {1, 2, 4, 8}, ctx_cap a multiple of 32. */
bool llam_dec_attention(const float *d_q, int ld_q, const void *d_kcache, const void *d_vcache,
                        const int32_t *d_pos, float *d_out, int ld_out, void *d_q8_out,
                        float *d_scratch, int B, int n_heads, int n_kv, int head_dim, int ctx_cap,
                        int device_id, void *stream);

/* d_table[b][i] = (cos, sin) of float(d_pos[b]) * d_inv_freq[i], i < head_dim/2, as two
 * floats each: the rotation of a decode step, which is the same in every layer.  One call
 * per step serves the llam_dec_rope_attention call of every layer.  d_table holds
 * B * head_dim floats. */
bool llam_dec_rope_table(const int32_t *d_pos, const float *d_inv_freq, float *d_table, int B,
                         int head_dim, int device_id, void *stream);

/* llam_dec_rope_kv_append and llam_dec_attention as one operator, two launches instead of
 * three: d_qkv is the unrotated row of the fused Q/K/V projection (layout as for
 * llam_dec_rope_kv_append), d_rope_table what llam_dec_rope_table wrote for the same
 * d_pos.  Every workgroup of the attention kernel rotates the query heads it serves; the
 * one whose chunk of the cache holds position d_pos[b] rotates the K head, rounds it and
 * the V head to fp16, appends both to the caches and attends over them.
 * Results and cache contents are those of the two calls in sequence, with one difference:
 * d_qkv is only read (the rotated Q is not written back).  Same limits as llam_dec_attention.
 * Replaces RoPEStage + KVCacheAppendStage + the decode attention stage
 * (src/v2/models/qwen/QwenGraphBase.cpp:2691-2790;
 * src/v2/kernels/cpu/attention/CPUFlashAttentionKernelT.h:507-545). */
bool llam_dec_rope_attention(const float *d_qkv, int ld_qkv, const float *d_rope_table,
                             const int32_t *d_pos, void *d_kcache, void *d_vcache, float *d_out,
                             int ld_out, void *d_q8_out, float *d_scratch, int B, int n_heads,
                             int n_kv, int head_dim, int ctx_cap, int device_id, void *stream);

/* Scratch bytes llam_dec_argmax needs for its per-workgroup partial results. */
size_t llam_dec_argmax_scratch_bytes(int B, int n);

/* Greedy sampling: d_ids[b] = index of the largest of d_logits[b*ld .. +n), the lower
 * index on ties, NaN never chosen (rocm_argmax_better,
 * src/v2/kernels/rocm/ops/ROCmArgmaxKernels.hip:28-35; two passes as there, :37-140).
 * If d_pos is not NULL, d_pos[b] += 1 afterwards (the next token's position). */
bool llam_dec_argmax(const float *d_logits, int ld, int n, int B, int32_t *d_ids, int32_t *d_pos,
                     void *d_scratch, int device_id, void *stream);

#ifdef __cplusplus
}
#endif
#endif
