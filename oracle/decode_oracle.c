/* TEST INFRASTRUCTURE ONLY -- CPU restatement of the decode-step operators around
 * the quantized-linear path (embedding rows, RMSNorm, rotary embedding + fp16 KV
 * append, single-token GQA attention, greedy sampling).  Scalar C, one function per
 * reference routine, each citing the reference lines it follows.  Nothing in the
 * shipped library calls into this file.
 *
 * How each function is pinned (tests/test_oracle_decode.py):
 *   qlo_dequant_row_q4k   against the int8/scale/min sub-block decoder of ql_oracle.c,
 *                         itself pinned on the reference's golden vectors (same nibble
 *                         order, same 6-bit scales), and against a numpy restatement of
 *                         the published ggml dequantize_row_q4_K
 *   qlo_rmsnorm           closed form in float64 numpy (x / sqrt(mean(x^2) + eps) * gamma),
 *                         unit-gamma rows of constant value, scale invariance
 *   qlo_rope_inv_freq/
 *   qlo_rope_head         norm preservation per pair, position 0 = identity, composition
 *                         R(p) R(q) = R(p+q), numpy float64 closed form
 *   qlo_attention_decode  one position = V row; uniform keys = mean of V; numpy float64
 *                         softmax closed form
 *   qlo_argmax            numpy argmax incl. ties (first index) and NaN rows
 * These are floating-point operators: the reference's own SIMD variants differ from its
 * scalar ones in the last bits (summation order, libm), so the contract is a tolerance,
 * stated with each GPU test, not bit equality. */
#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "ql_oracle.h"

/* Q4_KTensor::decodeBlockScalar (src/v2/tensors/Q4_KTensor.cpp:345-389): four groups of
 * 64 elements; sub-block 2g takes the low nibbles of qs[32g..32g+31], sub-block 2g+1 the
 * high nibbles; y = (d*sc)*q - (dmin*m). */
void qlo_dequant_row_q4k(const llam_block_q4_K *blocks, int nblocks, float *out)
{
    for (int b = 0; b < nblocks; ++b)
    {
        const llam_block_q4_K *blk = blocks + b;
        const float d = qlo_f16_to_f32(blk->d);
        const float dmin = qlo_f16_to_f32(blk->dmin);
        const uint8_t *q = blk->qs;
        float *y = out + (size_t)b * 256;
        int is = 0;
        for (int j = 0; j < 256; j += 64)
        {
            uint8_t sc1, m1, sc2, m2;
            qlo_get_scale_min_k4(is + 0, blk->scales, &sc1, &m1);
            qlo_get_scale_min_k4(is + 1, blk->scales, &sc2, &m2);
            const float d1 = d * (float)sc1, mv1 = dmin * (float)m1;
            const float d2 = d * (float)sc2, mv2 = dmin * (float)m2;
            for (int l = 0; l < 32; ++l)
                *y++ = d1 * (float)(q[l] & 0xF) - mv1;
            for (int l = 0; l < 32; ++l)
                *y++ = d2 * (float)(q[l] >> 4) - mv2;
            q += 32;
            is += 2;
        }
    }
}

/* rmsnorm_fused_row_scalar / fused_residual_rmsnorm_row
 * (src/v2/kernels/cpu/primitives/RMSNormPrimitives.cpp:1295-1319, 1564-1650):
 * optional residual += delta first (fp32 add, residual updated), sum of squares in
 * double, rms = sqrtf((float)(sum_sq / cols) + eps), y = x * (1/rms) * gamma. */
void qlo_rmsnorm(float *x, const float *delta, const float *gamma, float eps, float *y, int rows, int cols)
{
    for (int r = 0; r < rows; ++r)
    {
        float *xr = x + (size_t)r * cols;
        double sum_sq = 0.0;
        for (int c = 0; c < cols; ++c)
        {
            if (delta)
                xr[c] = xr[c] + delta[(size_t)r * cols + c];
            sum_sq += (double)xr[c] * (double)xr[c];
        }
        const float rms = sqrtf((float)(sum_sq / (double)cols) + eps);
        const float inv_rms = 1.0f / rms;
        for (int c = 0; c < cols; ++c)
            y[(size_t)r * cols + c] = xr[c] * inv_rms * gamma[c];
    }
}

/* get_inv_freq_cached (src/v2/kernels/cpu/primitives/RoPEPrimitives.cpp:50-77). */
void qlo_rope_inv_freq(int head_dim, float theta, float *inv_freq)
{
    const int half_dim = head_dim / 2;
    const float log_base = logf(theta);
    for (int i = 0; i < half_dim; ++i)
    {
        const float exponent = (2.0f * (float)i) / (float)head_dim;
        inv_freq[i] = expf(-log_base * exponent);
    }
}

/* apply_rope_to_head_scalar (RoPEPrimitives.cpp:180-203): pairs (i, i + head_dim/2). */
void qlo_rope_head(float *head, int position, const float *inv_freq, int head_dim)
{
    const int half_dim = head_dim / 2;
    for (int i = 0; i < half_dim; ++i)
    {
        const float angle = (float)position * inv_freq[i];
        const float c = cosf(angle), s = sinf(angle);
        const float x0 = head[i], x1 = head[i + half_dim];
        head[i] = x0 * c - x1 * s;
        head[i + half_dim] = x0 * s + x1 * c;
    }
}

/* RoPE of the Q and K heads of one token and the fp16 KV append
 * (RoPEStage + KVCacheAppendStage of a decode step, src/v2/models/qwen/QwenGraphBase.cpp:2691-2790).
 * qkv: [n_heads + 2 n_kv][head_dim]; caches [n_kv][ctx_cap][head_dim] as fp16 bits. */
void qlo_rope_kv_append(float *qkv, const float *inv_freq, int position, uint16_t *kcache, uint16_t *vcache,
                        int n_heads, int n_kv, int head_dim, int ctx_cap)
{
    for (int h = 0; h < n_heads + n_kv; ++h)
        qlo_rope_head(qkv + (size_t)h * head_dim, position, inv_freq, head_dim);
    for (int kh = 0; kh < n_kv; ++kh)
    {
        const float *k = qkv + (size_t)(n_heads + kh) * head_dim;
        const float *v = qkv + (size_t)(n_heads + n_kv + kh) * head_dim;
        uint16_t *kd = kcache + ((size_t)kh * ctx_cap + position) * head_dim;
        uint16_t *vd = vcache + ((size_t)kh * ctx_cap + position) * head_dim;
        for (int i = 0; i < head_dim; ++i)
        {
            kd[i] = qlo_f32_to_f16_rne(k[i]);
            vd[i] = qlo_f32_to_f16_rne(v[i]);
        }
    }
}

/* Single-token attention over fp16 K/V, positions 0..last inclusive:
 * out_h = softmax(q_h . K / sqrt(d)) . V  (CPUFlashAttentionKernelT::compute_decode with
 * fp16 KV, src/v2/kernels/cpu/attention/CPUFlashAttentionKernelT.h:507-545, 633-662).
 * The reference streams tiles with an online softmax in fp32; this restatement evaluates
 * the same expression in double, which every tile order rounds to. */
void qlo_attention_decode(const float *q, const uint16_t *kcache, const uint16_t *vcache, int last, float *out,
                          int n_heads, int n_kv, int head_dim, int ctx_cap)
{
    const int G = n_heads / n_kv;
    const double scale = 1.0 / sqrt((double)head_dim);
    double *s = (double *)malloc((size_t)(last + 1) * sizeof(double));
    double *acc = (double *)malloc((size_t)head_dim * sizeof(double));
    for (int h = 0; h < n_heads; ++h)
    {
        const int kh = h / G;
        const uint16_t *K = kcache + (size_t)kh * ctx_cap * head_dim;
        const uint16_t *V = vcache + (size_t)kh * ctx_cap * head_dim;
        double mx = -INFINITY;
        for (int p = 0; p <= last; ++p)
        {
            double d = 0.0;
            for (int i = 0; i < head_dim; ++i)
                d += (double)q[(size_t)h * head_dim + i] * (double)qlo_f16_to_f32(K[(size_t)p * head_dim + i]);
            s[p] = d * scale;
            if (s[p] > mx)
                mx = s[p];
        }
        double l = 0.0;
        memset(acc, 0, (size_t)head_dim * sizeof(double));
        for (int p = 0; p <= last; ++p)
        {
            const double e = exp(s[p] - mx);
            l += e;
            for (int i = 0; i < head_dim; ++i)
                acc[i] += e * (double)qlo_f16_to_f32(V[(size_t)p * head_dim + i]);
        }
        for (int i = 0; i < head_dim; ++i)
            out[(size_t)h * head_dim + i] = (float)(acc[i] / l);
    }
    free(s);
    free(acc);
}

/* rocm_argmax_better (src/v2/kernels/rocm/ops/ROCmArgmaxKernels.hip:28-35): larger value
 * wins, equal values -> lower index; start (-FLT_MAX, INT_MAX), so NaN never wins. */
int qlo_argmax(const float *x, int n)
{
    float best = -FLT_MAX;
    int idx = INT_MAX;
    for (int i = 0; i < n; ++i)
        if (x[i] > best || (x[i] == best && i < idx))
        {
            best = x[i];
            idx = i;
        }
    return idx;
}
