// Operators between the quantized-linear launches of a decode step, for gfx950:
// embedding rows, RMSNorm (+ residual add, + Q8_1), rotary embedding with the fp16
// KV-cache append, single-token GQA attention, greedy sampling.
//
// All of them move a few KB to a few MB per launch and are bound by launch latency or,
// for attention, by streaming the KV cache once; none is GEMM-shaped.
#include "ql_device.h"
#include "ql_host.h"

#include <cfloat>
#include <climits>
#include <cmath>

#include "llaminar_amd/decode_api.h"
#include "llaminar_amd/ql_api.h"

namespace llamql
{
    // ---- embedding ---------------------------------------------------------------------
    // One workgroup of 256 threads per (token, super-block); thread e owns element e.
    // Element e of a super-block: group g = e/64 of 32 bytes, low nibbles for e%64 < 32
    // (sub-block 2g), high nibbles otherwise (sub-block 2g+1).
    __global__ void __launch_bounds__(256)
        embed_q4k_kernel(const llam_block_q4_K *__restrict__ table, int vocab, const int32_t *__restrict__ ids,
                         float *__restrict__ x, int nsb, int ldx)
    {
        const int b = blockIdx.y, sb = blockIdx.x, e = threadIdx.x;
        const int id = ids[b];
        float y = 0.0f;
        if (id >= 0 && id < vocab)
        {
            const llam_block_q4_K *blk = table + (size_t)id * nsb + sb;
            const int g = e >> 6, l = e & 31, hi = (e >> 5) & 1;
            const uint32_t *sc32 = reinterpret_cast<const uint32_t *>(blk->scales);
            uint32_t sc, mn;
            q4k_scale_min(2 * g + hi, sc32[0], sc32[1], sc32[2], sc, mn);
            const float d = h2f(blk->d), dmin = h2f(blk->dmin);
            const uint32_t byte = blk->qs[g * 32 + l];
            const float q = (float)(hi ? (byte >> 4) : (byte & 0xFu));
            const float d1 = d * (float)sc;
            const float m1 = dmin * (float)mn;
            y = d1 * q - m1;
        }
        x[(size_t)b * ldx + sb * 256 + e] = y;
    }

    // ---- RMSNorm -------------------------------------------------------------------------
    // One workgroup per row.  Pass 1 adds the delta (when given), stores the new residual
    // and accumulates the sum of squares in double; pass 2 scales the row and, eight
    // threads per 32-element block, quantises it.  A thread keeps its first NORM_KEEP
    // float4 of the row and of gamma in registers (rows of up to 8192 values: all of
    // them), so every global load of the kernel is issued before the reduction and pass 2
    // waits for no memory; longer rows re-read the rest (the same thread reads what it wrote).
    constexpr int NORM_THREADS = 512;
    constexpr int NORM_KEEP = 4;

    __global__ void __launch_bounds__(NORM_THREADS)
        rmsnorm_q8_1_kernel(float *__restrict__ x, const float *__restrict__ delta, const float *__restrict__ delta2,
                            const float *__restrict__ gamma, float eps, float *__restrict__ y,
                            uint32_t *__restrict__ q8, int H)
    {
        // delta2 (only with delta): the delta arrives as two partial sums, x += (delta + delta2)
        __shared__ double s_part[NORM_THREADS / WAVE];
        const int m = blockIdx.x;
        const int nvec = H >> 2;
        float4 *row = reinterpret_cast<float4 *>(x + (size_t)m * H);
        const float4 *drow = delta ? reinterpret_cast<const float4 *>(delta + (size_t)m * H) : nullptr;
        const float4 *d2row = delta && delta2 ? reinterpret_cast<const float4 *>(delta2 + (size_t)m * H) : nullptr;
        const float4 *g4 = reinterpret_cast<const float4 *>(gamma);

        float4 keep[NORM_KEEP], dk[NORM_KEEP], gk[NORM_KEEP];
#pragma unroll
        for (int t = 0; t < NORM_KEEP; ++t)
        {
            const int i = threadIdx.x + t * NORM_THREADS;
            keep[t] = dk[t] = gk[t] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (i < nvec)
            {
                keep[t] = row[i];
                if (drow)
                    dk[t] = drow[i];
                gk[t] = g4[i];
            }
        }
        if (d2row) // (uniform; its loads go out with the others, before anything is waited for)
        {
            float4 d2[NORM_KEEP];
#pragma unroll
            for (int t = 0; t < NORM_KEEP; ++t)
            {
                const int i = threadIdx.x + t * NORM_THREADS;
                d2[t] = i < nvec ? d2row[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
#pragma unroll
            for (int t = 0; t < NORM_KEEP; ++t)
            {
                dk[t].x += d2[t].x;
                dk[t].y += d2[t].y;
                dk[t].z += d2[t].z;
                dk[t].w += d2[t].w;
            }
        }

        double acc = 0.0;
        auto square = [&acc](const float4 &v) {
            acc += (double)v.x * (double)v.x;
            acc += (double)v.y * (double)v.y;
            acc += (double)v.z * (double)v.z;
            acc += (double)v.w * (double)v.w;
        };
#pragma unroll
        for (int t = 0; t < NORM_KEEP; ++t)
        {
            const int i = threadIdx.x + t * NORM_THREADS;
            if (i < nvec)
            {
                if (drow)
                {
                    keep[t].x += dk[t].x;
                    keep[t].y += dk[t].y;
                    keep[t].z += dk[t].z;
                    keep[t].w += dk[t].w;
                    row[i] = keep[t];
                }
                square(keep[t]);
            }
        }
        for (int i = threadIdx.x + NORM_KEEP * NORM_THREADS; i < nvec; i += NORM_THREADS)
        {
            float4 v = row[i];
            if (drow)
            {
                float4 d = drow[i];
                if (d2row)
                {
                    const float4 e = d2row[i];
                    d.x += e.x;
                    d.y += e.y;
                    d.z += e.z;
                    d.w += e.w;
                }
                v.x += d.x;
                v.y += d.y;
                v.z += d.z;
                v.w += d.w;
                row[i] = v;
            }
            square(v);
        }
        acc = wave_sum(acc);
        if ((threadIdx.x & (WAVE - 1)) == 0)
            s_part[threadIdx.x >> 6] = acc;
        __syncthreads();
        double sum_sq = 0.0;
#pragma unroll
        for (int w = 0; w < NORM_THREADS / WAVE; ++w)
            sum_sq += s_part[w];

        const float rms = __fsqrt_rn(__fadd_rn((float)(sum_sq / (double)H), eps));
        const float inv = __fdiv_rn(1.0f, rms);

        float4 *yrow = y ? reinterpret_cast<float4 *>(y + (size_t)m * H) : nullptr;
        uint32_t *qrow = q8 ? q8 + (size_t)m * (H >> 5) * 9 : nullptr;
        auto emit = [&](int i, const float4 &v, const float4 &g) { // whole 8-thread groups stay together
            float4 o;
            o.x = __fmul_rn(__fmul_rn(v.x, inv), g.x);
            o.y = __fmul_rn(__fmul_rn(v.y, inv), g.y);
            o.z = __fmul_rn(__fmul_rn(v.z, inv), g.z);
            o.w = __fmul_rn(__fmul_rn(v.w, inv), g.w);
            if (yrow)
                yrow[i] = o;
            if (qrow)
            {
                const Q8Lane q = q8_1_quantize_lane(o);
                uint32_t *dst = qrow + (size_t)(i >> 3) * 9;
                dst[1 + (i & 7)] = q.packed;
                if ((i & 7) == 0)
                    dst[0] = q.head;
            }
        };
#pragma unroll
        for (int t = 0; t < NORM_KEEP; ++t)
        {
            const int i = threadIdx.x + t * NORM_THREADS;
            if (i < nvec)
                emit(i, keep[t], gk[t]);
        }
        for (int i = threadIdx.x + NORM_KEEP * NORM_THREADS; i < nvec; i += NORM_THREADS)
            emit(i, row[i], g4[i]);
    }

    // ---- the caches' tiles ---------------------------------------------------------------
    // Both caches hold, per (sequence, KV head), ctx_cap x head_dim fp16 values in tiles laid out for
    // the attention kernel's matrix operands, so that every load instruction of a wavefront (64
    // lanes x 16 bytes) reads ONE contiguous kilobyte instead of 64 pieces of 16 bytes:
    //   K: tiles of 16 positions, [position / 16][dim / 8][position % 16][dim % 8]
    //      (a lane's operand: 8 dims of one position; 16 neighbouring lanes: 16 positions)
    //   V: tiles of 32 positions, [position / 32][dim / 16][(position / 8) % 4][dim % 16][position % 8]
    //      (a lane's operand: 8 positions of one dim; 16 neighbouring lanes: 16 dims)
    // Element offsets inside the (sequence, head) slice; head_dim a multiple of 16, ctx_cap of 32.
    __host__ __device__ inline size_t kv_k_offset(int p, int d, int head_dim)
    {
        return (size_t)(p >> 4) * (size_t)(16 * head_dim) + (size_t)(d >> 3) * 128 + (size_t)(p & 15) * 8 + (size_t)(d & 7);
    }
    __host__ __device__ inline size_t kv_v_offset(int p, int d, int head_dim)
    {
        return (size_t)(p >> 5) * (size_t)(32 * head_dim) + (size_t)(d >> 4) * 512 + (size_t)((p >> 3) & 3) * 128 +
               (size_t)(d & 15) * 8 + (size_t)(p & 7);
    }

    // ---- rotary embedding + KV append -----------------------------------------------------
    // One workgroup of head_dim/2 threads per (sequence, head); heads n_heads.. are the K
    // heads, whose workgroups also copy the matching V head.
    // (x0, x1) rotated by the angle whose cosine and sine are c and s; every product and sum is
    // rounded on its own, as in the scalar host code (apply_rope_to_head_scalar)
    __device__ __forceinline__ void rope_pair(float x0, float x1, float c, float s, float &r0, float &r1)
    {
        r0 = __fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, s));
        r1 = __fadd_rn(__fmul_rn(x0, s), __fmul_rn(x1, c));
    }

    __global__ void rope_kv_append_kernel(float *__restrict__ qkv, int ld_qkv, const float *__restrict__ inv_freq,
                                          const int32_t *__restrict__ pos, __half *__restrict__ kcache,
                                          __half *__restrict__ vcache, int n_heads, int n_kv, int head_dim,
                                          int ctx_cap)
    {
        const int b = blockIdx.y, h = blockIdx.x, i = threadIdx.x;
        const int half_dim = head_dim >> 1;
        const int p = pos[b];
        float *row = qkv + (size_t)b * ld_qkv;
        const float angle = (float)p * inv_freq[i];
        const float c = cosf(angle), s = sinf(angle);
        float *head = row + (size_t)h * head_dim;
        const float x0 = head[i], x1 = head[i + half_dim];
        float r0, r1;
        rope_pair(x0, x1, c, s, r0, r1);
        if (h < n_heads)
        {
            head[i] = r0;
            head[i + half_dim] = r1;
            return;
        }
        if (p < 0 || p >= ctx_cap)
            return;
        const int kh = h - n_heads;
        const size_t slice = ((size_t)b * n_kv + kh) * (size_t)ctx_cap * head_dim;
        kcache[slice + kv_k_offset(p, i, head_dim)] = __float2half_rn(r0);
        kcache[slice + kv_k_offset(p, i + half_dim, head_dim)] = __float2half_rn(r1);
        const float *vhead = row + (size_t)(n_heads + n_kv + kh) * head_dim;
        vcache[slice + kv_v_offset(p, i, head_dim)] = __float2half_rn(vhead[i]);
        vcache[slice + kv_v_offset(p, i + half_dim, head_dim)] = __float2half_rn(vhead[i + half_dim]);
    }

    // cos and sin of float(pos[b]) * inv_freq[i]: the same for every layer of a decode step
    __global__ void rope_table_kernel(const int32_t *__restrict__ pos, const float *__restrict__ inv_freq,
                                      float2 *__restrict__ table, int half_dim)
    {
        const int b = blockIdx.x, i = threadIdx.x;
        const float angle = (float)pos[b] * inv_freq[i];
        table[(size_t)b * half_dim + i] = make_float2(cosf(angle), sinf(angle));
    }

    // ---- attention --------------------------------------------------------------------------
    // Workgroup = (chunk of ATT_CHUNK = 128 cache positions, KV head, sequence); its G = n_heads/n_kv
    // query heads share every K and V element it reads.  Each of the four wavefronts takes 32
    // positions and runs both products on the matrix unit (v_mfma_f32_16x16x32_f16, fp32 sums):
    //   scores  S[head][pos] = sum_d Q[head][d] K[pos][d]     A = Q rows (heads, padded to 16),
    //                                                          B = K rows as columns: lane (pos, g)
    //                                                          holds 8 dims of its position
    //   softmax statistics of the chunk per head: m = max, e = exp(s - m), l = sum e
    //   output  O[head][d] = sum_pos e[head][pos] V[pos][d]   A = e rows, B = V columns: lane (d, g)
    //                                                          holds 8 positions of its dim, which
    //                                                          are contiguous in the V cache's
    //                                                          tiles (kv_v_offset)
    // K and V are exact fp16 operands.  The fp32 factors (Q, e) enter as the sum of two fp16 numbers,
    // high part and remainder, after a scaling by a power of two that keeps the remainders out of
    // the subnormal range, so every product is that of the fp32 value to about 2^-22.
    // A second kernel merges the chunks: o = sum_c o_c exp(m_c - M) / sum_c l_c exp(m_c - M).
    constexpr int ATT_CHUNK = 128;
    constexpr int ATT_THREADS = 256;
    constexpr int ATT_HD = 128;
    constexpr int ATT_WAVES = ATT_THREADS / WAVE;
    constexpr int ATT_PER_WAVE = ATT_CHUNK / ATT_WAVES; // 32 positions: two score tiles, one output step
    constexpr float ATT_P_SCALE = 32768.0f;             // e <= 1 is split after scaling: remainders stay normal fp16

    typedef _Float16 att_v8h __attribute__((ext_vector_type(8)));
    typedef float att_v4f __attribute__((ext_vector_type(4)));

    // x = hi + lo up to 2^-22 |x|, both fp16 (the remainder is exact in fp32)
    __device__ __forceinline__ void att_split(const float (&x)[8], att_v8h &hi, att_v8h &lo)
    {
#pragma unroll
        for (int j = 0; j < 8; ++j)
        {
            const _Float16 h = (_Float16)x[j];
            hi[j] = h;
            lo[j] = (_Float16)(x[j] - (float)h);
        }
    }

    // ROPE: q is the unrotated output row of the fused Q/K/V projection (Q heads, then K heads,
    // then V heads).  The workgroup rotates its G query heads itself, and the workgroup whose chunk
    // holds the new position also rotates that K head, rounds it and the V head to fp16, appends
    // both to the caches and uses them in place of what the caches held: the work of
    // rope_kv_append_kernel without its launch.  The cosines and sines come from the table that
    // rope_table_kernel writes once per decode step (computing them here, in every workgroup of
    // every layer, cost more than the launch saved).
    template <int G, bool ROPE>
    __global__ void __launch_bounds__(ATT_THREADS)
        attention_partial_kernel(const float *__restrict__ q, int ld_q, const float2 *__restrict__ rope_table,
                                 __half *__restrict__ kcache, __half *__restrict__ vcache,
                                 const int32_t *__restrict__ pos, float *__restrict__ part_o,
                                 float *__restrict__ part_ml, int n_heads, int n_kv, int ctx_cap, int n_chunks)
    {
        __shared__ __attribute__((aligned(16))) float s_sc[G][ATT_CHUNK];       // scores, then e
        __shared__ __attribute__((aligned(16))) float s_o[ATT_WAVES][G][ATT_HD]; // per-wavefront outputs; first the rotated Q
        __shared__ __attribute__((aligned(16))) __half s_new[2][ATT_HD];         // the appended K and V rows
        const int chunk = blockIdx.x, kh = blockIdx.y, b = blockIdx.z;
        const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
        const int n = lane & 15, gq = lane >> 4; // matrix-unit lane: row/column n, k-group gq
        const int last = pos[b] < ctx_cap - 1 ? pos[b] : ctx_cap - 1; // newest position, inclusive
        const int p0 = chunk * ATT_CHUNK;
        const size_t out_base = ((size_t)b * n_heads + (size_t)kh * G) * n_chunks + chunk;
        if (p0 > last)
            return; // no position in this chunk yet: the merge does not read it
        const __half *kbase = kcache + ((size_t)b * n_kv + kh) * ctx_cap * ATT_HD;
        const __half *vbase = vcache + ((size_t)b * n_kv + kh) * ctx_cap * ATT_HD;
        const int pw = p0 + wave * ATT_PER_WAVE; // first position of this wavefront

        // ROPE: the few values of the rotation are requested first: loads return in order, and the
        // rotation then runs while the K and V loads behind them are in flight
        constexpr int HALF = ATT_HD / 2;
        constexpr int Q_PAIRS = (G * HALF + ATT_THREADS - 1) / ATT_THREADS; // head pairs per thread
        const int ri = threadIdx.x & (HALF - 1);
        float2 rope_cs = make_float2(1.0f, 0.0f);
        float rope_x0[Q_PAIRS], rope_x1[Q_PAIRS], new_x0 = 0.0f, new_x1 = 0.0f;
        int rope_p = -1;
        bool owner = false;
        if (ROPE)
        {
            rope_p = pos[b];
            owner = rope_p >= 0 && rope_p < ctx_cap && rope_p / ATT_CHUNK == chunk; // the append is this workgroup's
            rope_cs = rope_table[(size_t)b * HALF + ri];
            const float *row = q + (size_t)b * ld_q;
#pragma unroll
            for (int k = 0; k < Q_PAIRS; ++k)
            {
                const int g = threadIdx.x / HALF + k * (ATT_THREADS / HALF);
                const float *head = row + (size_t)(kh * G + (g < G ? g : 0)) * ATT_HD;
                rope_x0[k] = head[ri];
                rope_x1[k] = head[ri + HALF];
            }
            if (owner && threadIdx.x < ATT_HD) // first 64 threads: the K head, next 64: the V head
            {
                const float *head = row + (size_t)(n_heads + (threadIdx.x >= HALF ? n_kv : 0) + kh) * ATT_HD;
                new_x0 = head[ri];
                new_x1 = head[ri + HALF];
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        // Every K and V element this wavefront will need is requested before the first use.
        // K: tile t holds positions pw + 16 t + n, step s the dims 32 s + 8 gq .. + 7.
        uint4 kraw[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
        {
            const int p = pw + 16 * t + n;
            const __half *row = kbase + kv_k_offset(p <= last ? p : last, 8 * gq, ATT_HD); // rows past the end: weight 0
#pragma unroll
            for (int s = 0; s < 4; ++s)
                kraw[t][s] = *reinterpret_cast<const uint4 *>(row + 512 * s); // dims 32 s further: four 8-dim groups of 128 values
        }
        // V: column tile ct holds dims 16 ct + n, positions pw + 8 gq .. + 7 (a group that starts
        // past the newest position is read at the newest one's group; the mask below clears it)
        uint4 vraw[8];
        const int pg = pw + 8 * gq;
        {
            const __half *colp = vbase + kv_v_offset(pg <= last ? pg : (last & ~7), n, ATT_HD);
#pragma unroll
            for (int ct = 0; ct < 8; ++ct)
                vraw[ct] = *reinterpret_cast<const uint4 *>(colp + 512 * ct); // dims 16 ct further
        }

        if (ROPE)
        {
            __builtin_amdgcn_sched_barrier(0);
            const int p = rope_p, i = ri;
            const float c = rope_cs.x, sn = rope_cs.y;
            float(*s_q)[ATT_HD] = s_o[0];
#pragma unroll
            for (int k = 0; k < Q_PAIRS; ++k)
            {
                const int g = threadIdx.x / HALF + k * (ATT_THREADS / HALF);
                if (g < G)
                    rope_pair(rope_x0[k], rope_x1[k], c, sn, s_q[g][i], s_q[g][i + HALF]);
            }
            if (owner && threadIdx.x < ATT_HD)
            {
                const bool is_v = threadIdx.x >= HALF;
                float r0 = new_x0, r1 = new_x1;
                if (!is_v)
                    rope_pair(new_x0, new_x1, c, sn, r0, r1);
                const __half h0 = __float2half_rn(r0), h1 = __float2half_rn(r1);
                s_new[is_v][i] = h0;
                s_new[is_v][i + HALF] = h1;
                if (is_v)
                {
                    __half *vhead = vcache + ((size_t)b * n_kv + kh) * ctx_cap * ATT_HD;
                    vhead[kv_v_offset(p, i, ATT_HD)] = h0;
                    vhead[kv_v_offset(p, i + HALF, ATT_HD)] = h1;
                }
                else
                {
                    __half *khead = kcache + ((size_t)b * n_kv + kh) * ctx_cap * ATT_HD;
                    khead[kv_k_offset(p, i, ATT_HD)] = h0;
                    khead[kv_k_offset(p, i + HALF, ATT_HD)] = h1;
                }
            }
            __syncthreads();
            if (owner)
            {
                // the new row replaces what was loaded for its position
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    if (pw + 16 * t + n == p)
                    {
#pragma unroll
                        for (int s = 0; s < 4; ++s)
                            kraw[t][s] = *reinterpret_cast<const uint4 *>(&s_new[0][32 * s + 8 * gq]);
                    }
                const int j = p - pg;
                if (j >= 0 && j < 8)
                {
                    const uint32_t sh = (j & 1) * 16, clear = ~(0xffffu << sh);
#pragma unroll
                    for (int ct = 0; ct < 8; ++ct)
                    {
                        const uint32_t nv = (uint32_t)__half_as_ushort(s_new[1][16 * ct + n]) << sh;
                        uint32_t *w = reinterpret_cast<uint32_t *>(&vraw[ct]);
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            if (k == (j >> 1))
                                w[k] = (w[k] & clear) | nv;
                    }
                }
            }
        }

        // Q rows: lane (head n, gq) holds dims 32 s + 8 gq .. + 7, scaled by 1/sqrt(128) and by the
        // power of two that brings the head's largest magnitude to [2^14, 2^15): the matrix unit
        // treats subnormal fp16 operands as zero, and the remainders of values near 0.1 would be
        // subnormal.  q_down undoes the power of two on the scores, exactly.
        att_v8h qhi[4], qlo[4];
        float q_down;
        {
            const float scale = 0.08838834764831845f;
            const float *qh = ROPE ? &s_o[0][n < G ? n : 0][8 * gq]
                                   : q + (size_t)b * ld_q + (size_t)(kh * G + (n < G ? n : 0)) * ATT_HD + 8 * gq;
            const float live = n < G ? scale : 0.0f; // rows past the group's heads are zero
            float x[4][8];
            float mx = 0.0f;
#pragma unroll
            for (int s = 0; s < 4; ++s)
            {
                const float4 a = *reinterpret_cast<const float4 *>(qh + 32 * s);
                const float4 c = *reinterpret_cast<const float4 *>(qh + 32 * s + 4);
                x[s][0] = a.x * live, x[s][1] = a.y * live, x[s][2] = a.z * live, x[s][3] = a.w * live;
                x[s][4] = c.x * live, x[s][5] = c.y * live, x[s][6] = c.z * live, x[s][7] = c.w * live;
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    mx = fmaxf(mx, fabsf(x[s][j]));
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE)); // the head's four lanes agree
            int sh = 15 - __builtin_amdgcn_frexp_expf(mx); // mx = f 2^e with 0.5 <= f < 1
            sh = sh > 100 ? 100 : (sh < -100 ? -100 : sh);
            const float up = ldexpf(1.0f, sh);
            q_down = ldexpf(1.0f, -sh);
#pragma unroll
            for (int s = 0; s < 4; ++s)
            {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    x[s][j] *= up;
                att_split(x[s], qhi[s], qlo[s]);
            }
        }

        // scores: lane (position n of tile t, gq) receives heads 4 gq .. 4 gq + 3
#pragma unroll
        for (int t = 0; t < 2; ++t)
        {
            att_v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < 4; ++s)
            {
                const att_v8h kv = __builtin_bit_cast(att_v8h, kraw[t][s]);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(qhi[s], kv, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(qlo[s], kv, acc, 0, 0, 0);
            }
            const int pl = wave * ATT_PER_WAVE + 16 * t + n;
            const bool valid = p0 + pl <= last;
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                const float down = __shfl(q_down, 4 * gq + r, WAVE); // lane h < 16 holds head h
                if (4 * gq + r < G)
                    s_sc[4 * gq + r][pl] = valid ? acc[r] * down : -INFINITY;
            }
        }
        __syncthreads();

        // statistics: wavefront w takes heads w, w + 4, ..., all of them side by side (their reductions are
        // chains of dependent cross-lane steps: one after the other they were a tenth of the kernel)
        {
            constexpr int PER_LANE = ATT_CHUNK / WAVE;
            constexpr int HEADS = (G + ATT_WAVES - 1) / ATT_WAVES; // heads per wavefront
            float sc[HEADS][PER_LANE], mx[HEADS], l[HEADS];
#pragma unroll
            for (int h = 0; h < HEADS; ++h)
            {
                const int g = wave + ATT_WAVES * h;
                mx[h] = -INFINITY;
#pragma unroll
                for (int k = 0; k < PER_LANE; ++k)
                {
                    sc[h][k] = s_sc[g < G ? g : 0][lane + WAVE * k];
                    mx[h] = fmaxf(mx[h], sc[h][k]);
                }
            }
#pragma unroll
            for (int h = 0; h < HEADS; ++h)
                mx[h] = wave_max(mx[h]);
#pragma unroll
            for (int h = 0; h < HEADS; ++h)
            {
                const int g = wave + ATT_WAVES * h;
                l[h] = 0.0f;
#pragma unroll
                for (int k = 0; k < PER_LANE; ++k)
                {
                    const float e = expf(sc[h][k] - mx[h]); // position p0 is valid: mx is finite
                    if (g < G)
                        s_sc[g][lane + WAVE * k] = e;
                    l[h] += e;
                }
            }
#pragma unroll
            for (int h = 0; h < HEADS; ++h)
                l[h] = wave_sum(l[h]);
#pragma unroll
            for (int h = 0; h < HEADS; ++h)
            {
                const int g = wave + ATT_WAVES * h;
                if (lane == 0 && g < G)
                {
                    part_ml[(out_base + (size_t)g * n_chunks) * 2 + 0] = mx[h];
                    part_ml[(out_base + (size_t)g * n_chunks) * 2 + 1] = l[h];
                }
            }
        }
        __syncthreads();

        // output: A = e rows, lane (head n, gq) holds positions pw + 8 gq .. + 7
        att_v8h phi, plo;
        {
            float x[8];
            const float4 *src = reinterpret_cast<const float4 *>(&s_sc[n < G ? n : 0][wave * ATT_PER_WAVE + 8 * gq]);
            const float4 a = src[0], c = src[1];
            const float live = n < G ? ATT_P_SCALE : 0.0f;
            x[0] = a.x * live, x[1] = a.y * live, x[2] = a.z * live, x[3] = a.w * live;
            x[4] = c.x * live, x[5] = c.y * live, x[6] = c.z * live, x[7] = c.w * live;
            att_split(x, phi, plo);
        }
        // V elements of positions past the newest one may be anything, NaN included: clear them
        uint4 keep;
        {
            const int left = last - pg; // halves 0 .. left of the group are live
            uint32_t m[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                m[j] = (2 * j <= left ? 0x0000ffffu : 0u) | (2 * j + 1 <= left ? 0xffff0000u : 0u);
            keep = make_uint4(m[0], m[1], m[2], m[3]);
        }
#pragma unroll
        for (int ct = 0; ct < 8; ++ct)
        {
            uint4 v = vraw[ct];
            v.x &= keep.x, v.y &= keep.y, v.z &= keep.z, v.w &= keep.w;
            const att_v8h vv = __builtin_bit_cast(att_v8h, v);
            att_v4f o = {0.0f, 0.0f, 0.0f, 0.0f};
            o = __builtin_amdgcn_mfma_f32_16x16x32_f16(phi, vv, o, 0, 0, 0);
            o = __builtin_amdgcn_mfma_f32_16x16x32_f16(plo, vv, o, 0, 0, 0);
            // lane (dim 16 ct + n, gq) holds heads 4 gq .. 4 gq + 3
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (4 * gq + r < G)
                    s_o[wave][4 * gq + r][16 * ct + n] = o[r] * (1.0f / ATT_P_SCALE);
        }
        __syncthreads();
        for (int i = threadIdx.x; i < G * (ATT_HD / 4); i += ATT_THREADS)
        {
            const int g = i / (ATT_HD / 4), c4 = (i % (ATT_HD / 4)) * 4;
            float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
            for (int w = 0; w < ATT_WAVES; ++w)
            {
                const float4 v = *reinterpret_cast<const float4 *>(&s_o[w][g][c4]);
                a.x += v.x, a.y += v.y, a.z += v.z, a.w += v.w;
            }
            *reinterpret_cast<float4 *>(part_o + (out_base + (size_t)g * n_chunks) * ATT_HD + c4) = a;
        }
    }

    template <int G>
    void attention_partial_launch(dim3 grid, hipStream_t st, const float *q, int ld_q, const float2 *inv_freq,
                                  __half *kc, __half *vc, const int32_t *pos, float *part_o, float *part_ml,
                                  int n_heads, int n_kv, int ctx_cap, int n_chunks)
    {
        if (inv_freq)
            hipLaunchKernelGGL((attention_partial_kernel<G, true>), grid, dim3(ATT_THREADS), 0, st, q, ld_q, inv_freq, kc,
                               vc, pos, part_o, part_ml, n_heads, n_kv, ctx_cap, n_chunks);
        else
            hipLaunchKernelGGL((attention_partial_kernel<G, false>), grid, dim3(ATT_THREADS), 0, st, q, ld_q, inv_freq, kc,
                               vc, pos, part_o, part_ml, n_heads, n_kv, ctx_cap, n_chunks);
    }

    // One workgroup of 128 threads per (sequence, head): thread k weighs chunk k, then thread c
    // sums column c over the chunks that hold positions.
    constexpr int ATT_MAX_CHUNKS = 1024; // 131072 cache positions
    constexpr int ATT_MERGE_KEEP = 40;   // chunks whose partial outputs a thread holds in registers (5120 positions)

    __global__ void __launch_bounds__(ATT_HD)
        attention_merge_kernel(const float *__restrict__ part_o, const float *__restrict__ part_ml,
                               const int32_t *__restrict__ pos, float *__restrict__ out, int ld_out,
                               uint32_t *__restrict__ q8, int n_heads, int n_chunks, int ctx_cap)
    {
        __shared__ __attribute__((aligned(16))) float s_val[ATT_HD];
        __shared__ float s_w[ATT_MAX_CHUNKS];
        __shared__ float s_red[ATT_HD / WAVE];
        const int h = blockIdx.x, b = blockIdx.y, c = threadIdx.x;
        const int last = pos[b] < ctx_cap - 1 ? pos[b] : ctx_cap - 1;
        const int used = last < 0 ? 0 : last / ATT_CHUNK + 1; // chunks that were written
        const size_t base = ((size_t)b * n_heads + h) * n_chunks;

        // The first ATT_MERGE_KEEP chunks' column values are requested before anything is
        // waited for: they do not depend on the weights, and the kernel is then one memory
        // latency deep instead of one per few chunks.
        float po[ATT_MERGE_KEEP];
#pragma unroll
        for (int k = 0; k < ATT_MERGE_KEEP; ++k)
            po[k] = k < used ? part_o[(base + k) * ATT_HD + c] : 0.0f;

        float mx = -INFINITY;
        for (int k = c; k < used; k += ATT_HD)
            mx = fmaxf(mx, part_ml[(base + k) * 2]);
        mx = wave_max(mx);
        if ((c & (WAVE - 1)) == 0)
            s_red[c >> 6] = mx;
        __syncthreads();
        const float M = fmaxf(s_red[0], s_red[1]);
        __syncthreads();
        float l = 0.0f;
        for (int k = c; k < used; k += ATT_HD)
        {
            const float w = expf(part_ml[(base + k) * 2] - M);
            s_w[k] = w;
            l = fmaf(part_ml[(base + k) * 2 + 1], w, l);
        }
        l = wave_sum(l);
        if ((c & (WAVE - 1)) == 0)
            s_red[c >> 6] = l;
        __syncthreads();
        const float L = s_red[0] + s_red[1];

        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < ATT_MERGE_KEEP; ++k)
            if (k < used)
                acc = fmaf(po[k], s_w[k], acc);
#pragma unroll 4
        for (int k = ATT_MERGE_KEEP; k < used; ++k)
            acc = fmaf(part_o[(base + k) * ATT_HD + c], s_w[k], acc);
        const float val = L > 0.0f ? __fdiv_rn(acc, L) : 0.0f; // pos < 0: nothing attended
        if (out)
            out[(size_t)b * ld_out + (size_t)h * ATT_HD + c] = val;
        if (q8)
        {
            // the head's 128 outputs are four Q8_1 blocks of the row the next projection reads
            s_val[c] = val;
            __syncthreads();
            if (c < ATT_HD / 4) // 32 threads, eight per block
            {
                const Q8Lane q = q8_1_quantize_lane(*reinterpret_cast<const float4 *>(&s_val[4 * c]));
                uint32_t *dst = q8 + (((size_t)b * n_heads + h) * (ATT_HD / 32) + (c >> 3)) * 9;
                dst[1 + (c & 7)] = q.packed;
                if ((c & 7) == 0)
                    dst[0] = q.head;
            }
        }
    }

    // ---- greedy sampling -----------------------------------------------------------------------
    constexpr int ARGMAX_THREADS = 256;
    constexpr int ARGMAX_PER_THREAD = 8;

    __device__ __forceinline__ bool argmax_better(float cv, int ci, float v, int i)
    {
        return cv > v || (cv == v && ci < i);
    }

    __device__ __forceinline__ void argmax_block_reduce(float &v, int &idx, float *s_v, int *s_i)
    {
#pragma unroll
        for (int off = WAVE / 2; off > 0; off >>= 1)
        {
            const float ov = __shfl_xor(v, off, WAVE);
            const int oi = __shfl_xor(idx, off, WAVE);
            if (argmax_better(ov, oi, v, idx))
            {
                v = ov;
                idx = oi;
            }
        }
        if ((threadIdx.x & (WAVE - 1)) == 0)
        {
            s_v[threadIdx.x >> 6] = v;
            s_i[threadIdx.x >> 6] = idx;
        }
        __syncthreads();
        if (threadIdx.x == 0)
        {
            for (int w = 1; w < ARGMAX_THREADS / WAVE; ++w)
                if (argmax_better(s_v[w], s_i[w], v, idx))
                {
                    v = s_v[w];
                    idx = s_i[w];
                }
        }
    }

    __global__ void __launch_bounds__(ARGMAX_THREADS)
        argmax_partial_kernel(const float *__restrict__ logits, int ld, int n, float *__restrict__ pv,
                              int *__restrict__ pi)
    {
        __shared__ float s_v[ARGMAX_THREADS / WAVE];
        __shared__ int s_i[ARGMAX_THREADS / WAVE];
        const int b = blockIdx.y;
        const float *row = logits + (size_t)b * ld;
        float v = -FLT_MAX;
        int idx = INT_MAX;
        const int stride = ARGMAX_THREADS * gridDim.x;
        for (int i = blockIdx.x * ARGMAX_THREADS + threadIdx.x; i < n; i += stride)
        {
            const float x = row[i];
            if (argmax_better(x, i, v, idx))
            {
                v = x;
                idx = i;
            }
        }
        argmax_block_reduce(v, idx, s_v, s_i);
        if (threadIdx.x == 0)
        {
            pv[(size_t)b * gridDim.x + blockIdx.x] = v;
            pi[(size_t)b * gridDim.x + blockIdx.x] = idx;
        }
    }

    __global__ void __launch_bounds__(ARGMAX_THREADS)
        argmax_final_kernel(const float *__restrict__ pv, const int *__restrict__ pi, int n_part,
                            int32_t *__restrict__ ids, int32_t *__restrict__ pos)
    {
        __shared__ float s_v[ARGMAX_THREADS / WAVE];
        __shared__ int s_i[ARGMAX_THREADS / WAVE];
        const int b = blockIdx.x;
        float v = -FLT_MAX;
        int idx = INT_MAX;
        for (int i = threadIdx.x; i < n_part; i += ARGMAX_THREADS)
        {
            const float x = pv[(size_t)b * n_part + i];
            const int xi = pi[(size_t)b * n_part + i];
            if (argmax_better(x, xi, v, idx))
            {
                v = x;
                idx = xi;
            }
        }
        argmax_block_reduce(v, idx, s_v, s_i);
        if (threadIdx.x == 0)
        {
            ids[b] = idx;
            if (pos)
                pos[b] += 1;
        }
    }

    inline int argmax_blocks(int n)
    {
        const int per_block = ARGMAX_THREADS * ARGMAX_PER_THREAD;
        return (n + per_block - 1) / per_block;
    }
} // namespace llamql

using namespace llamql;

extern "C" bool llam_dec_embed_q4k(const void *d_table, int vocab, const int32_t *d_ids, float *d_x,
                                   int B, int H, int ldx, int device_id, void *stream)
{
    static const char *fn = "llam_dec_embed_q4k";
    if (B < 0 || vocab < 1 || H < 1)
        return fail(fn, "bad size (B=%d vocab=%d H=%d)", B, vocab, H);
    if (B == 0)
        return true;
    if ((H % 256) != 0 || ldx < H)
        return fail(fn, "H=%d must be a multiple of 256 and ldx=%d at least H", H, ldx);
    if (!d_table || !d_ids || !d_x)
        return fail(fn, "null pointer");
    if (!aligned16(d_table) || !aligned4(d_ids) || !aligned4(d_x))
        return fail(fn, "misaligned pointer");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(embed_q4k_kernel, dim3(H / 256, B), dim3(256), 0, as_stream(stream),
                       static_cast<const llam_block_q4_K *>(d_table), vocab, d_ids, d_x, H / 256, ldx);
    return launched(fn);
}

extern "C" bool llam_dec_rmsnorm_q8_1(float *d_x, const float *d_delta, const float *d_gamma, float eps,
                                      float *d_y, void *d_q8, int M, int H, int device_id, void *stream)
{
    return llam_dec_rmsnorm2_q8_1(d_x, d_delta, nullptr, d_gamma, eps, d_y, d_q8, M, H, device_id, stream);
}

extern "C" bool llam_dec_rmsnorm2_q8_1(float *d_x, const float *d_delta, const float *d_delta2, const float *d_gamma,
                                       float eps, float *d_y, void *d_q8, int M, int H, int device_id, void *stream)
{
    static const char *fn = "llam_dec_rmsnorm_q8_1";
    if (d_delta2 && (!d_delta || !aligned16(d_delta2)))
        return fail(fn, "a second delta needs the first, and 16-byte alignment");
    if (M < 0 || H < 1)
        return fail(fn, "bad size (M=%d H=%d)", M, H);
    if (M == 0)
        return true;
    if ((H % 32) != 0)
        return fail(fn, "H=%d must be a multiple of 32", H);
    if (!d_x || !d_gamma)
        return fail(fn, "null pointer");
    if (!aligned16(d_x) || !aligned16(d_gamma) || (d_delta && !aligned16(d_delta)) || (d_y && !aligned16(d_y)) ||
        (d_q8 && !aligned4(d_q8)))
        return fail(fn, "fp32 rows must be 16-byte aligned, d_q8 4-byte aligned");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(rmsnorm_q8_1_kernel, dim3(M), dim3(NORM_THREADS), 0, as_stream(stream), d_x, d_delta, d_delta2,
                       d_gamma, eps, d_y, static_cast<uint32_t *>(d_q8), H);
    return launched(fn);
}

extern "C" void llam_dec_rope_inv_freq(int head_dim, float theta, float *h_inv_freq)
{
    const int half_dim = head_dim / 2;
    const float log_base = std::log(theta);
    for (int i = 0; i < half_dim; ++i)
    {
        const float exponent = (2.0f * (float)i) / (float)head_dim;
        h_inv_freq[i] = std::exp(-log_base * exponent);
    }
}

extern "C" bool llam_dec_rope_kv_append(float *d_qkv, int ld_qkv, const float *d_inv_freq,
                                        const int32_t *d_pos, void *d_kcache, void *d_vcache, int B,
                                        int n_heads, int n_kv, int head_dim, int ctx_cap, int device_id,
                                        void *stream)
{
    static const char *fn = "llam_dec_rope_kv_append";
    if (B < 0 || n_heads < 1 || n_kv < 1 || head_dim < 2 || ctx_cap < 1)
        return fail(fn, "bad size");
    if (B == 0)
        return true;
    if ((head_dim % 16) != 0 || head_dim / 2 > 1024)
        return fail(fn, "head_dim=%d must be a multiple of 16 and at most 2048", head_dim);
    if ((ctx_cap % 32) != 0)
        return fail(fn, "ctx_cap=%d must be a multiple of 32 (the caches are kept in tiles of 16 and 32 positions)", ctx_cap);
    if (ld_qkv < (n_heads + 2 * n_kv) * head_dim)
        return fail(fn, "ld_qkv=%d smaller than (n_heads + 2 n_kv) * head_dim", ld_qkv);
    if (!d_qkv || !d_inv_freq || !d_pos || !d_kcache || !d_vcache)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(rope_kv_append_kernel, dim3(n_heads + n_kv, B), dim3(head_dim / 2), 0, as_stream(stream),
                       d_qkv, ld_qkv, d_inv_freq, d_pos, static_cast<__half *>(d_kcache),
                       static_cast<__half *>(d_vcache), n_heads, n_kv, head_dim, ctx_cap);
    return launched(fn);
}

extern "C" size_t llam_dec_attention_scratch_floats(int B, int n_heads, int head_dim, int ctx_cap)
{
    if (B < 1 || n_heads < 1 || head_dim < 1 || ctx_cap < 1)
        return 0;
    const size_t chunks = ((size_t)ctx_cap + ATT_CHUNK - 1) / ATT_CHUNK;
    return (size_t)B * n_heads * chunks * ((size_t)head_dim + 2);
}

namespace
{
    // llam_dec_attention (no table of cosines and sines: d_inv_freq == nullptr, d_q holds rotated query heads) and
    // llam_dec_rope_attention (d_q is the unrotated Q/K/V row) share everything but the kernel variant.
    bool attention_run(const char *fn, const float *d_q, int ld_q, const float2 *d_inv_freq, void *d_kcache,
                       void *d_vcache, const int32_t *d_pos, float *d_out, int ld_out, void *d_q8_out,
                       float *d_scratch, int B, int n_heads, int n_kv, int head_dim, int ctx_cap, int device_id,
                       void *stream)
    {
        using namespace llamql;
        if (B < 0 || n_heads < 1 || n_kv < 1 || ctx_cap < 1)
            return fail(fn, "bad size");
        if (B == 0)
            return true;
        if (head_dim != ATT_HD)
            return fail(fn, "head_dim=%d: only 128 is built", head_dim);
        if ((n_heads % n_kv) != 0)
            return fail(fn, "n_heads=%d not a multiple of n_kv=%d", n_heads, n_kv);
        const int G = n_heads / n_kv;
        if (G != 1 && G != 2 && G != 4 && G != 8)
            return fail(fn, "n_heads/n_kv=%d: only 1, 2, 4 and 8 are built", G);
        const int width = (d_inv_freq ? n_heads + 2 * n_kv : n_heads) * head_dim;
        if (ld_q < width || (d_out && ld_out < n_heads * head_dim))
            return fail(fn, "row strides smaller than the rows");
        if (!d_q || !d_kcache || !d_vcache || !d_pos || (!d_out && !d_q8_out) || !d_scratch)
            return fail(fn, "null pointer");
        if (!aligned16(d_q) || (ld_q % 4) != 0 || !aligned16(d_kcache) || !aligned16(d_vcache) ||
            (d_out && !aligned4(d_out)) || (d_q8_out && !aligned4(d_q8_out)) || !aligned16(d_scratch))
            return fail(fn, "misaligned pointer (q, caches and scratch 16-byte, out 4-byte)");
        if ((ctx_cap % 32) != 0)
            return fail(fn, "ctx_cap=%d must be a multiple of 32 (the caches are kept in tiles of 16 and 32 positions)",
                        ctx_cap);
        const int n_chunks = (ctx_cap + ATT_CHUNK - 1) / ATT_CHUNK;
        if (n_chunks > ATT_MAX_CHUNKS || B > 65535)
            return fail(fn, "ctx_cap=%d beyond %d positions, or too many sequences", ctx_cap,
                        ATT_MAX_CHUNKS * ATT_CHUNK);
        if (!set_device(fn, device_id))
            return false;
        float *part_o = d_scratch;
        float *part_ml = d_scratch + (size_t)B * n_heads * n_chunks * ATT_HD;
        __half *kc = static_cast<__half *>(d_kcache);
        __half *vc = static_cast<__half *>(d_vcache);
        const dim3 grid(n_chunks, n_kv, B);
        hipStream_t st = as_stream(stream);
        switch (G)
        {
        case 1: attention_partial_launch<1>(grid, st, d_q, ld_q, d_inv_freq, kc, vc, d_pos, part_o, part_ml, n_heads, n_kv, ctx_cap, n_chunks); break;
        case 2: attention_partial_launch<2>(grid, st, d_q, ld_q, d_inv_freq, kc, vc, d_pos, part_o, part_ml, n_heads, n_kv, ctx_cap, n_chunks); break;
        case 4: attention_partial_launch<4>(grid, st, d_q, ld_q, d_inv_freq, kc, vc, d_pos, part_o, part_ml, n_heads, n_kv, ctx_cap, n_chunks); break;
        default: attention_partial_launch<8>(grid, st, d_q, ld_q, d_inv_freq, kc, vc, d_pos, part_o, part_ml, n_heads, n_kv, ctx_cap, n_chunks); break;
        }
        if (!launched(fn))
            return false;
        hipLaunchKernelGGL(attention_merge_kernel, dim3(n_heads, B), dim3(ATT_HD), 0, st, part_o, part_ml, d_pos, d_out,
                           ld_out, static_cast<uint32_t *>(d_q8_out), n_heads, n_chunks, ctx_cap);
        return launched(fn);
    }
} // namespace

extern "C" bool llam_dec_attention(const float *d_q, int ld_q, const void *d_kcache, const void *d_vcache,
                                   const int32_t *d_pos, float *d_out, int ld_out, void *d_q8_out,
                                   float *d_scratch, int B, int n_heads, int n_kv, int head_dim, int ctx_cap,
                                   int device_id, void *stream)
{
    // without the table of frequencies the kernel only reads the caches
    return attention_run("llam_dec_attention", d_q, ld_q, nullptr, const_cast<void *>(d_kcache),
                         const_cast<void *>(d_vcache), d_pos, d_out, ld_out, d_q8_out, d_scratch, B, n_heads, n_kv,
                         head_dim, ctx_cap, device_id, stream);
}

extern "C" bool llam_dec_rope_table(const int32_t *d_pos, const float *d_inv_freq, float *d_table, int B, int head_dim,
                                    int device_id, void *stream)
{
    static const char *fn = "llam_dec_rope_table";
    if (B < 0 || head_dim < 2 || (head_dim % 2) != 0 || head_dim / 2 > 1024)
        return fail(fn, "bad size");
    if (B == 0)
        return true;
    if (!d_pos || !d_inv_freq || !d_table)
        return fail(fn, "null pointer");
    if (((uintptr_t)d_table & 7) != 0)
        return fail(fn, "table not 8-byte aligned");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(rope_table_kernel, dim3(B), dim3(head_dim / 2), 0, as_stream(stream), d_pos, d_inv_freq,
                       reinterpret_cast<float2 *>(d_table), head_dim / 2);
    return launched(fn);
}

extern "C" bool llam_dec_rope_attention(const float *d_qkv, int ld_qkv, const float *d_rope_table, const int32_t *d_pos,
                                        void *d_kcache, void *d_vcache, float *d_out, int ld_out, void *d_q8_out,
                                        float *d_scratch, int B, int n_heads, int n_kv, int head_dim, int ctx_cap,
                                        int device_id, void *stream)
{
    static const char *fn = "llam_dec_rope_attention";
    if (!d_rope_table)
        return fail(fn, "null pointer");
    if (((uintptr_t)d_rope_table & 7) != 0)
        return fail(fn, "table not 8-byte aligned");
    return attention_run(fn, d_qkv, ld_qkv, reinterpret_cast<const float2 *>(d_rope_table), d_kcache, d_vcache, d_pos,
                         d_out, ld_out, d_q8_out, d_scratch, B, n_heads, n_kv, head_dim, ctx_cap, device_id, stream);
}

extern "C" size_t llam_dec_argmax_scratch_bytes(int B, int n)
{
    if (B < 1 || n < 1)
        return 0;
    return (size_t)B * argmax_blocks(n) * (sizeof(float) + sizeof(int));
}

extern "C" bool llam_dec_argmax(const float *d_logits, int ld, int n, int B, int32_t *d_ids, int32_t *d_pos,
                                void *d_scratch, int device_id, void *stream)
{
    static const char *fn = "llam_dec_argmax";
    if (B < 0 || n < 1 || ld < n)
        return fail(fn, "bad size (B=%d n=%d ld=%d)", B, n, ld);
    if (B == 0)
        return true;
    if (!d_logits || !d_ids || !d_scratch)
        return fail(fn, "null pointer");
    if (!aligned4(d_logits) || !aligned4(d_ids) || !aligned4(d_scratch) || (d_pos && !aligned4(d_pos)))
        return fail(fn, "misaligned pointer");
    if (B > 65535)
        return fail(fn, "too many rows");
    if (!set_device(fn, device_id))
        return false;
    const int blocks = argmax_blocks(n);
    float *pv = static_cast<float *>(d_scratch);
    int *pi = reinterpret_cast<int *>(pv + (size_t)B * blocks);
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(blocks, B), dim3(ARGMAX_THREADS), 0, as_stream(stream), d_logits,
                       ld, n, pv, pi);
    if (!launched(fn))
        return false;
    hipLaunchKernelGGL(argmax_final_kernel, dim3(B), dim3(ARGMAX_THREADS), 0, as_stream(stream), pv, pi, blocks,
                       d_ids, d_pos);
    return launched(fn);
}
