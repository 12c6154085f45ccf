/*
 * TEST INFRASTRUCTURE ONLY -- see ql_oracle.h.  Scalar restatement of the
 * reference's CPU quantized-linear arithmetic; never linked into the product.
 *
 * Build with -ffp-contract=off: every fused multiply-add below is an explicit
 * fmaf() because the reference's kernels fuse exactly those and nothing else.
 */
#include "ql_oracle.h"

#include <math.h>
#include <omp.h>
#include <stdlib.h>
#include <string.h>

#include "llaminar_amd/iq3s_grid.h"

static inline uint32_t f32_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float bits_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* tensors/FP16Utils.h:25-66 -- exact widening (subnormals normalised). */
float qlo_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    const uint32_t m = h & 0x3FFu;
    if (e == 0x1Fu)
        return bits_f32(sign | 0x7F800000u | (m << 13));
    if (e != 0)
        return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
    if (m == 0)
        return bits_f32(sign);
    /* subnormal: m * 2^-24, exactly representable in binary32 */
    float v = (float)m * 5.9604644775390625e-08f;
    return (sign ? -v : v);
}

/* tensors/FP16Utils.h:75-118.  Normal results round to nearest even; results
 * below the fp16 normal range are TRUNCATED toward zero (no rounding) and
 * anything below 2^-25 becomes a signed zero. */
uint16_t qlo_f32_to_f16_sw(float f)
{
    const uint32_t u = f32_bits(f);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const int32_t e = (int32_t)((u >> 23) & 0xFFu) - 112; /* rebias 127 -> 15 */
    uint32_t m = u & 0x007FFFFFu;

    if (e >= 31)
    {
        if (((u >> 23) & 0xFFu) == 0xFFu && m != 0)
            return (uint16_t)(sign | 0x7C00u | (m >> 13)); /* NaN */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (e <= 0)
    {
        if (e < -10)
            return sign;
        m = (m | 0x00800000u) >> (1 - e);
        return (uint16_t)(sign | (m >> 13)); /* truncation */
    }
    uint32_t he = (uint32_t)e;
    m += 0x0FFFu + ((m >> 13) & 1u);
    if (m >= 0x00800000u)
    {
        m = 0;
        he += 1;
    }
    return (uint16_t)(sign | (he << 10) | (m >> 13));
}

/* IEEE-754 binary32 -> binary16, round-to-nearest-even everywhere (what the
 * F16C conversion in tensors/SIMDHelpers.h:4743-4745 produces). */
uint16_t qlo_f32_to_f16_rne(float f)
{
    uint32_t x = f32_bits(f);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7FFFFFFFu;
    if (x > 0x7F800000u)
        return (uint16_t)(sign | 0x7E00u | ((x >> 13) & 0x3FFu)); /* quiet NaN */
    if (x >= 0x38800000u)
    { /* >= 2^-14: normal half (or overflow) */
        uint32_t r = x + 0x0FFFu + ((x >> 13) & 1u);
        uint32_t h = (r - 0x38000000u) >> 13;
        if (h >= 0x7C00u)
            h = 0x7C00u;
        return (uint16_t)(sign | h);
    }
    if (x < 0x33000000u)
        return sign; /* < 2^-25 rounds to zero */
    /* subnormal half: units of 2^-24 */
    const int e = (int)(x >> 23);
    const uint32_t m = (x & 0x007FFFFFu) | 0x00800000u;
    const int shift = 126 - e; /* 14..24 */
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u)))
        q += 1;
    return (uint16_t)(sign | q);
}

/* ------------------------------------------------------------------------- */
/* Q8_1 activation quantiser                                                  */
/* ------------------------------------------------------------------------- */

void qlo_quantize_block_q8_1(const float *x, int valid, llam_block_q8_1 *out)
{
    float amax = 0.0f;
    for (int i = 0; i < valid; ++i)
    {
        float a = fabsf(x[i]);
        if (a > amax)
            amax = a;
    }
    if (amax < 1e-10f)
    {
        memset(out, 0, sizeof(*out));
        return;
    }
    const float d = amax / 127.0f;
    const float id = 1.0f / d;
    int32_t sum = 0;
    if (valid == 32)
    {
        /* SIMD path: RNE convert, saturating narrow, hardware fp16 convert. */
        out->d = qlo_f32_to_f16_rne(d);
        for (int i = 0; i < 32; ++i)
        {
            long q = lrintf(x[i] * id); /* default rounding mode: nearest-even */
            if (q > 127)
                q = 127;
            if (q < -128)
                q = -128;
            out->qs[i] = (int8_t)q;
            sum += (int32_t)q;
        }
    }
    else
    {
        /* Scalar tail: round-half-away, C++ narrowing cast, software fp16. */
        out->d = qlo_f32_to_f16_sw(d);
        for (int i = 0; i < valid; ++i)
        {
            int8_t q = (int8_t)roundf(x[i] * id);
            out->qs[i] = q;
            sum += q;
        }
        for (int i = valid; i < 32; ++i)
            out->qs[i] = 0;
    }
    out->sum_qs = (int16_t)sum;
}

void qlo_quantize_q8_1(const float *x, int M, int K, llam_block_q8_1 *out)
{
    const int KB = (K + 31) / 32;
    for (int m = 0; m < M; ++m)
        for (int kb = 0; kb < KB; ++kb)
        {
            int len = K - kb * 32;
            if (len > 32)
                len = 32;
            qlo_quantize_block_q8_1(x + (size_t)m * K + kb * 32, len, out + (size_t)m * KB + kb);
        }
}

/* ------------------------------------------------------------------------- */
/* Weight-side effective sub-blocks                                           */
/* ------------------------------------------------------------------------- */

void qlo_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m)
{
    if (j < 4)
    {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    }
    else
    {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

void qlo_subblocks_q4k(const llam_block_q4_K *sb, int8_t *w, uint16_t *scale8, uint16_t *min8)
{
    const float d = qlo_f16_to_f32(sb->d);
    const float dmin = qlo_f16_to_f32(sb->dmin);
    for (int j = 0; j < 8; ++j)
    {
        const uint8_t *src = sb->qs + 32 * (j >> 1);
        for (int i = 0; i < 32; ++i)
            w[32 * j + i] = (int8_t)((j & 1) ? (src[i] >> 4) : (src[i] & 0x0F));
        uint8_t sc, m;
        qlo_get_scale_min_k4(j, sb->scales, &sc, &m);
        scale8[j] = qlo_f32_to_f16_sw(d * (float)sc);
        min8[j] = qlo_f32_to_f16_sw(-dmin * (float)m);
    }
}

void qlo_subblocks_q6k(const llam_block_q6_K *sb, int8_t *w, uint16_t *scale8, uint16_t *min8)
{
    const float d = qlo_f16_to_f32(sb->d);
    for (int j = 0; j < 8; ++j)
    {
        const int half = j >> 2, s = j & 3;
        const int8_t sc0 = sb->scales[8 * half + 2 * s];
        const int8_t sc1 = sb->scales[8 * half + 2 * s + 1];
        const float a0 = fabsf((float)sc0), a1 = fabsf((float)sc1);
        const float msc = a0 > a1 ? a0 : a1;
        int16_t f[2] = {0, 0};
        float out_scale = 0.0f;
        if (msc != 0.0f)
        {
            out_scale = d * msc * 32.0f / 127.0f; /* left to right */
            f[0] = (int16_t)nearbyintf((float)sc0 * 127.0f * 256.0f / (msc * 32.0f));
            f[1] = (int16_t)nearbyintf((float)sc1 * 127.0f * 256.0f / (msc * 32.0f));
        }
        const uint8_t *ql = sb->ql + 64 * half + 32 * (s & 1);
        const uint8_t *qh = sb->qh + 32 * half;
        for (int i = 0; i < 32; ++i)
        {
            const int nib = (s >= 2) ? (ql[i] >> 4) : (ql[i] & 0x0F);
            const int hi = (qh[i] >> (2 * s)) & 3;
            const int16_t q = (int16_t)((nib | (hi << 4)) - 32);
            /* int16 lanes: mullo, add 128, arithmetic shift right 8, truncate to byte */
            const int16_t prod = (int16_t)(q * f[i >> 4]);
            const int16_t r = (int16_t)((int16_t)(prod + 128) >> 8);
            w[32 * j + i] = (int8_t)r;
        }
        scale8[j] = qlo_f32_to_f16_sw(out_scale);
        min8[j] = qlo_f32_to_f16_sw(0.0f);
    }
}

void qlo_subblocks_iq3s(const llam_block_iq3_s *sb, int8_t *w, uint16_t *scale8, uint16_t *min8)
{
    const float d = qlo_f16_to_f32(sb->d);
    for (int j = 0; j < 8; ++j)
    {
        const uint8_t sbyte = sb->scales[j >> 1];
        const int nib = (j & 1) ? (sbyte >> 4) : (sbyte & 0x0F);
        const float db = d * (1.0f + 2.0f * (float)nib);
        uint32_t signs;
        memcpy(&signs, sb->signs + 4 * j, 4);
        float v[32];
        float amax = 0.0f;
        for (int l = 0; l < 8; ++l)
        {
            const uint32_t idx = (uint32_t)sb->qs[8 * j + l] | ((((uint32_t)sb->qh[j] >> l) & 1u) << 8);
            const uint32_t g = llam_iq3s_grid[idx];
            for (int t = 0; t < 4; ++t)
            {
                const int e = 4 * l + t;
                float x = (float)(int8_t)((g >> (8 * t)) & 0xFF) * db;
                if ((signs >> e) & 1u)
                    x = 0.0f - x;
                v[e] = x;
                const float a = fabsf(x);
                if (a > amax)
                    amax = a;
            }
        }
        float scale = amax / 127.0f;
        if (scale > 65504.0f)
            scale = 65504.0f;
        if (amax < 1e-6f)
            scale = 0.0f;
        if (scale == 0.0f)
        {
            memset(w + 32 * j, 0, 32);
        }
        else
        {
            const float inv = 1.0f / scale;
            for (int e = 0; e < 32; ++e)
                w[32 * j + e] = (int8_t)(int32_t)lrintf(v[e] * inv); /* RNE, byte truncation */
        }
        scale8[j] = qlo_f32_to_f16_sw(scale);
        min8[j] = 0;
    }
}

void qlo_subblocks(int fmt, const void *sb, int8_t *w, uint16_t *scale8, uint16_t *min8)
{
    switch (fmt)
    {
    case LLAM_FMT_Q4_K: qlo_subblocks_q4k((const llam_block_q4_K *)sb, w, scale8, min8); break;
    case LLAM_FMT_Q6_K: qlo_subblocks_q6k((const llam_block_q6_K *)sb, w, scale8, min8); break;
    case LLAM_FMT_IQ3_S: qlo_subblocks_iq3s((const llam_block_iq3_s *)sb, w, scale8, min8); break;
    default: abort();
    }
}

/* ------------------------------------------------------------------------- */
/* GEMV / GEMM                                                                */
/* ------------------------------------------------------------------------- */

void qlo_gemm_rows(int fmt, const void *W, int K, int n0, int n1,
                   const llam_block_q8_1 *A, int M, float *C, int ldc,
                   int32_t *block_sums, int k_tiles)
{
    const int SB = K / 256;
    const int KB = K / 32;
    const size_t bb = (size_t)llam_format_block_bytes(fmt);
    /* The reference treats Q4_K and Q6_K as "asymmetric" (a mins plane exists,
     * all-zero for Q6_K); IQ3_S is symmetric (TensorClasses.h:6223,5530,7608). */
    const int asym = (fmt != LLAM_FMT_IQ3_S);
    const int tiles = k_tiles > 1 ? k_tiles : 1;
    const int kb_per_tile = (KB + tiles - 1) / tiles;

#pragma omp parallel
    {
        int8_t *w = (int8_t *)malloc((size_t)K);
        uint16_t *sc = (uint16_t *)malloc((size_t)KB * 2);
        uint16_t *mn = (uint16_t *)malloc((size_t)KB * 2);
#pragma omp for schedule(static)
        for (int n = n0; n < n1; ++n)
        {
            const uint8_t *row = (const uint8_t *)W + (size_t)n * SB * bb;
            for (int s = 0; s < SB; ++s)
                qlo_subblocks(fmt, row + (size_t)s * bb, w + 256 * s, sc + 8 * s, mn + 8 * s);
            for (int m = 0; m < M; ++m)
            {
                const llam_block_q8_1 *a = A + (size_t)m * KB;
                float total = 0.0f;
                for (int t = 0; t < tiles; ++t)
                {
                    int kb0 = t * kb_per_tile, kb1 = kb0 + kb_per_tile;
                    if (kb1 > KB)
                        kb1 = KB;
                    float acc = 0.0f;
                    for (int kb = kb0; kb < kb1; ++kb)
                    {
                        int32_t idot = 0;
                        for (int i = 0; i < 32; ++i)
                            idot += (int32_t)a[kb].qs[i] * (int32_t)w[32 * kb + i];
                        if (block_sums)
                            block_sums[((size_t)m * (n1 - n0) + (n - n0)) * KB + kb] = idot;
                        const float a_d = qlo_f16_to_f32(a[kb].d);
                        const float cs = a_d * qlo_f16_to_f32(sc[kb]);
                        acc = fmaf((float)idot, cs, acc);
                        if (asym)
                            acc = fmaf((float)a[kb].sum_qs * a_d, qlo_f16_to_f32(mn[kb]), acc);
                    }
                    total = (tiles == 1) ? acc : (t == 0 ? acc : total + acc);
                }
                C[(size_t)m * ldc + n] = total;
            }
        }
        free(w);
        free(sc);
        free(mn);
    }
}

void qlo_epilogue(float *C, const float *tmp, int M, int N, int ldc,
                  float alpha, float beta, const float *bias)
{
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n)
        {
            float c = (beta == 0.0f) ? 0.0f : beta * C[(size_t)m * ldc + n];
            c += alpha * tmp[(size_t)m * N + n];
            if (bias)
                c += bias[n];
            C[(size_t)m * ldc + n] = c;
        }
}

/* ------------------------------------------------------------------------- */
/* MoE router and SwiGLU                                                      */
/* ------------------------------------------------------------------------- */

void qlo_moe_route(const float *logits, int n_tokens, int n_experts, int top_k,
                   int normalize, int32_t *ids, float *weights, float *probs)
{
    float *p = (float *)malloc((size_t)n_experts * sizeof(float));
    char *taken = (char *)malloc((size_t)n_experts);
    for (int t = 0; t < n_tokens; ++t)
    {
        const float *l = logits + (size_t)t * n_experts;
        float mx = -INFINITY;
        for (int e = 0; e < n_experts; ++e)
            if (l[e] > mx)
                mx = l[e];
        if (!isfinite(mx))
            mx = 0.0f;
        double sum = 0.0;
        for (int e = 0; e < n_experts; ++e)
            sum += (double)expf(l[e] - mx);
        if (sum <= 0.0)
            sum = 1.0;
        const float inv = (float)(1.0 / sum);
        for (int e = 0; e < n_experts; ++e)
            p[e] = expf(l[e] - mx) * inv;
        if (probs)
            memcpy(probs + (size_t)t * n_experts, p, (size_t)n_experts * sizeof(float));
        memset(taken, 0, (size_t)n_experts);
        float topk_sum = 0.0f;
        for (int k = 0; k < top_k; ++k)
        {
            int best = -1;
            for (int e = 0; e < n_experts; ++e)
                if (!taken[e] && (best < 0 || p[e] > p[best]))
                    best = e;
            taken[best] = 1;
            ids[(size_t)t * top_k + k] = best;
            topk_sum += p[best];
        }
        for (int k = 0; k < top_k; ++k)
        {
            const float pk = p[ids[(size_t)t * top_k + k]];
            weights[(size_t)t * top_k + k] = normalize ? pk / topk_sum : pk;
        }
    }
    free(p);
    free(taken);
}

void qlo_swiglu(const float *gate, const float *up, int n, float *out)
{
    for (int i = 0; i < n; ++i)
    {
        const float g = gate[i];
        out[i] = (g / (1.0f + expf(-g))) * up[i];
    }
}

/* ---- exhaustive checks of two division-free forms the GPU kernels use ---------------
 * Both return the number of inputs on which the cheap form differs from the division the
 * reference performs (SIMDHelpers.h:12023-12204); the tests expect 0.
 *
 * x / 127 for x = (f32(d) * msc) * 32, every fp16 d and msc = 1..128 (the Q6_K block scale
 * before its fp16 rounding): q0 = x * c, r = fma(-q0, 127, x), q1 = fma(r, c, q0) with
 * c = RN(1/127) -- Markstein's correction step; zero and non-finite x take q0 (sign of zero). */
long qlo_check_div127(void)
{
    const float c = 0x1.020408p-7f;
    long bad = 0;
    for (unsigned h = 0; h < 65536u; ++h)
    {
        const float d = qlo_f16_to_f32((uint16_t)h);
        for (int msc = 1; msc <= 128; ++msc)
        {
            const float x = d * (float)msc * 32.0f;
            const float want = x / 127.0f;
            const float q0 = x * c;
            const float r = fmaf(-q0, 127.0f, x);
            const float q1 = fmaf(r, c, q0);
            const float got = (isfinite(x) && x != 0.0f) ? q1 : q0;
            uint32_t a, b;
            memcpy(&a, &want, 4);
            memcpy(&b, &got, 4);
            if (a != b && !(want != want && got != got))
                ++bad;
        }
    }
    return bad;
}

/* The same correction step for EVERY finite x: the result of the sequence depends on the
 * significand of x only (each operation scales with x by an exact power of two as long as
 * nothing leaves the normal range), so all 2^23 significands at two exponents far from the
 * ends of the range cover every x between 2^-100 and 2^100.  Used by the IQ3_S block scale
 * (gmax * d * (1 + 2 nib)) / 127 of the GPU decoder. */
long qlo_check_div127_all_significands(void)
{
    const float c = 0x1.020408p-7f;
    long bad = 0;
    for (int pass = 0; pass < 2; ++pass)
    {
        const uint32_t expo = pass == 0 ? 127u : 127u - 20u;
        for (uint32_t m = 0; m < (1u << 23); ++m)
        {
            const uint32_t bits = (expo << 23) | m;
            float x;
            memcpy(&x, &bits, 4);
            const float want = x / 127.0f;
            const float q0 = x * c;
            const float r = fmaf(-q0, 127.0f, x);
            const float got = fmaf(r, c, q0);
            uint32_t a, b;
            memcpy(&a, &want, 4);
            memcpy(&b, &got, 4);
            bad += a != b;
        }
    }
    return bad;
}

/* nearbyint(s * 32512 / (msc * 32)) for |s| <= msc <= 128 (the 8.8 factor of the smaller
 * sub-scale) against rint of one Newton step on s * 1016 * r, for EVERY r within `ulps`
 * units in the last place of the correctly rounded 1/msc (the GPU's reciprocal instruction
 * is accurate to one).                                                                    */
long qlo_check_q6k_factor(int ulps)
{
    long bad = 0;
    for (int msc = 1; msc <= 128; ++msc)
    {
        const float fm = (float)msc;
        const float r0 = 1.0f / fm;
        for (int u = -ulps; u <= ulps; ++u)
        {
            float r = r0;
            for (int i = 0; i < (u < 0 ? -u : u); ++i)
                r = nextafterf(r, u < 0 ? 0.0f : 2.0f);
            for (int sv = -msc; sv <= msc; ++sv)
            {
                if (sv < -128 || sv > 127)
                    continue;
                const float want = nearbyintf((float)sv * 127 * 256 / (fm * 32));
                const float num = (float)(sv * 1016);
                const float q0 = num * r;
                const float q1 = fmaf(fmaf(-fm, q0, num), r, q0);
                if (nearbyintf(q1) != want)
                    ++bad;
            }
        }
    }
    return bad;
}


/* Host memory bandwidth for the CPU baseline's context: the triad a[i] = b[i] + s * c[i] over
 * three arrays of n doubles with every OpenMP thread, `reps` passes, best pass.  Returns bytes per
 * second counting 24 bytes per element (the STREAM convention: no write-allocate traffic), as
 * the reference's performance harness reports beside its GEMV figures
 * (tests/v2/performance/kernels/cpu/native_vnni/Perf__CPUNativeVNNI_GEMV.cpp:120-177). */
double qlo_stream_triad(double *a, const double *b, const double *c, long n, int reps)
{
    double best = 0.0;
    for (int r = 0; r < reps; ++r) {
        const double t0 = omp_get_wtime();
#pragma omp parallel for schedule(static)
        for (long i = 0; i < n; ++i)
            a[i] = b[i] + 3.0 * c[i];
        const double dt = omp_get_wtime() - t0;
        if (dt > 0.0) {
            const double bw = 24.0 * (double)n / dt;
            if (bw > best)
                best = bw;
        }
    }
    return best;
}
