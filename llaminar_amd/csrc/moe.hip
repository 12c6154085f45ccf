// MoE expert-bucketed GEMV for gfx950: router, routed gate/up and down GEMVs
// driven by device-resident top-k ids, fused SwiGLU + Q8_1 quantise, shared
// expert gate.  The GEMVs reuse the decode-GEMV skeleton; the per-workgroup
// launch description is assembled on the device from the expert table and the
// routing ids, so no host round trip separates routing from expert compute.
#include "gemv_traits_all.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    // ---- router ------------------------------------------------------------------
    // One wavefront per token; lane l owns experts l, l+64, ...  Softmax as the
    // reference computes it (kernels/cpu/primitives/SoftmaxPrimitivesImpl.h:584-693):
    // max, sum of exp(l-max) in double, p = exp(l-max) * float(1/sum); then top_k
    // rounds of arg-max (ties -> lower expert id) and optional renormalisation over
    // the top_k.  All reductions are wavefront shuffles: no LDS, no barriers.
    constexpr int ROUTE_MAX_PER_LANE = 32; // up to 2048 experts

    // One wavefront routes one token: l its n_experts logits; lane k < top_k returns the k-th expert and
    // its weight (other lanes: unspecified).
    template <int PER>
    __device__ __forceinline__ void moe_route_wave(const float *__restrict__ l, int n_experts, int top_k, int normalize,
                                                   int lane, int &out_id, float &out_weight)
    {
        float p[PER];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < PER; ++i)
        {
            const int e = lane + i * WAVE;
            p[i] = (e < n_experts) ? l[e] : -INFINITY;
            mx = fmaxf(mx, p[i]);
        }
        mx = wave_max(mx);
        if (!isfinite(mx))
            mx = 0.0f;

        double sum = 0.0;
#pragma unroll
        for (int i = 0; i < PER; ++i)
        {
            const int e = lane + i * WAVE;
            if (e < n_experts)
            {
                p[i] = expf(p[i] - mx);
                sum += (double)p[i];
            }
            else
            {
                p[i] = -1.0f; // never selected: probabilities are >= 0
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
            sum += __shfl_xor(sum, off);
        if (sum <= 0.0)
            sum = 1.0;
        const float inv = (float)(1.0 / sum);
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (p[i] >= 0.0f)
                p[i] = p[i] * inv;

        // top_k rounds of arg-max: the largest live probability over the wavefront, then the lowest
        // expert id that holds it (expert e sits in p[e / 64] of lane e % 64: the first i with a
        // match, then the lowest matching lane); retired and padding entries are -1, below every
        // probability.  Lane k keeps the k-th winner.
        float my_top = 0.0f;
        int my_id = -1;
        float topk_sum = 0.0f;
        for (int k = 0; k < top_k; ++k)
        {
            float best = p[0];
#pragma unroll
            for (int i = 1; i < PER; ++i)
                best = fmaxf(best, p[i]);
            best = wave_max(best); // every lane now holds the winner's probability
            int best_e = -1;
            float bp = 0.0f;
            if (best >= 0.0f) // uniform; false only when nothing selectable is left (NaN logits)
            {
                bp = best;
#pragma unroll
                for (int i = PER - 1; i >= 0; --i)
                {
                    const unsigned long long hit = __ballot(p[i] == best);
                    if (hit) // uniform
                        best_e = i * WAVE + (int)__builtin_ctzll(hit);
                }
            }
            if (lane == k)
            {
                my_top = bp;
                my_id = best_e;
            }
            topk_sum += bp; // same order on every lane: k = 0, 1, ...
#pragma unroll
            for (int i = 0; i < PER; ++i)
                if (lane + i * WAVE == best_e)
                    p[i] = -1.0f; // retire the winner
        }
        out_id = my_id;
        out_weight = normalize ? __fdiv_rn(my_top, topk_sum) : my_top;
    }

    // Workgroups past the tokens (optional) quantise `q_blocks` 32-element blocks of q_x to Q8_1
    // with the stand-alone quantiser's arithmetic: the hidden state the expert GEMVs read does
    // not depend on the routing, so its quantiser rides in the same launch.
    template <int PER>
    __global__ void __launch_bounds__(WAVE)
        moe_route_kernel(const float *__restrict__ logits, int n_tokens, int n_experts, int top_k, int normalize,
                         int32_t *__restrict__ ids, float *__restrict__ weights, int slot_stride,
                         const float4 *__restrict__ q_x, uint32_t *__restrict__ q_out, long q_blocks)
    {
        if ((int)blockIdx.x >= n_tokens) // uniform
        {
            const long lane_global = (long)((int)blockIdx.x - n_tokens) * WAVE + threadIdx.x;
            const long blk = lane_global >> 3;
            if (blk >= q_blocks)
                return; // whole 8-lane groups leave together
            const Q8Lane q = q8_1_quantize_lane(q_x[lane_global]);
            uint32_t *dst = q_out + blk * 9;
            dst[1 + (lane_global & 7)] = q.packed;
            if ((lane_global & 7) == 0)
                dst[0] = q.head;
            return;
        }
        const int t = blockIdx.x;
        const int lane = threadIdx.x;
        int my_id;
        float my_weight;
        moe_route_wave<PER>(logits + (size_t)t * n_experts, n_experts, top_k, normalize, lane, my_id, my_weight);
        if (lane < top_k)
        {
            ids[(size_t)t * slot_stride + lane] = my_id;
            weights[(size_t)t * slot_stride + lane] = my_weight;
        }
    }

    // ---- router logits -------------------------------------------------------------------
    // logits[t][e] = dot(hidden[t], gate_w[e]) in fp32: one wavefront per (token, expert),
    // float4 loads, fused multiply-adds per lane, then the fixed-order wavefront sum.
    __global__ void __launch_bounds__(256)
        moe_router_logits_kernel(const float *__restrict__ hidden, const float *__restrict__ gate_w,
                                 float *__restrict__ logits, int d_model, int n_experts)
    {
        const int t = blockIdx.y;
        const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
        const int lane = threadIdx.x & (WAVE - 1);
        if (e >= n_experts)
            return; // whole wavefronts leave together
        const float4 *h = reinterpret_cast<const float4 *>(hidden + (size_t)t * d_model);
        const float4 *w = reinterpret_cast<const float4 *>(gate_w + (size_t)e * d_model);
        float acc = 0.0f;
        for (int i = lane; i < (d_model >> 2); i += WAVE)
        {
            const float4 a = h[i], b = w[i];
            acc = fmaf(a.x, b.x, acc);
            acc = fmaf(a.y, b.y, acc);
            acc = fmaf(a.z, b.z, acc);
            acc = fmaf(a.w, b.w, acc);
        }
        acc = wave_sum(acc);
        if (lane == 0)
            logits[(size_t)t * n_experts + e] = acc;
    }

    // ---- routed gate/up ---------------------------------------------------------
    struct MoEArgs
    {
        const llam_ql_expert *experts;
        const int32_t *ids;
        const float *weights;
        const uint32_t *q8;
        float *out0;
        float *out1;
        int n_experts, top_k, hidden, inter;
        int rows_per_wave, gshift, accumulate;
    };

    // A pointer every lane holds, moved to scalar registers (the weight loads take their base there).
    __device__ __forceinline__ const void *uniform_ptr(const void *p)
    {
        const uint64_t v = (uint64_t)p;
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return reinterpret_cast<const void *>(((uint64_t)hi << 32) | lo);
    }

    // grid: (workgroups per matrix, n_tokens*top_k, 2 = gate|up)
    template <class F>
    __global__ void __launch_bounds__(GEMV_WAVES *WAVE) moe_gate_up_kernel(const MoEArgs m)
    {
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        const int slot = blockIdx.y;
        const int t = slot / m.top_k;
        const int e = m.ids[slot];
        if (e < 0 || e >= m.n_experts)
            return; // uniform for the workgroup; outputs of a bad id stay untouched
        GemvArgs a;
        a.w = blockIdx.z == 0 ? m.experts[e].d_gate : m.experts[e].d_up;
        if (!a.w)
            return; // an expert whose matrices live elsewhere: skipped like a bad id (uniform)
        a.q8 = m.q8 + (size_t)t * (m.hidden / 32) * 9;
        a.y = (blockIdx.z == 0 ? m.out0 : m.out1) + (size_t)slot * m.inter;
        a.sums = nullptr;
        a.ldy = m.inter;
        a.N = m.inter;
        a.SB = m.hidden / 256;
        a.sb0 = 0;
        a.nsb = a.SB;
        a.rows_per_wave = m.rows_per_wave;
        a.gshift = m.gshift;
        a.accumulate = 0;
        a.out_scale = 1.0f;
        a.row0 = 0;
        a.nrows = 0;
        a.pairs = nullptr;
        a.pair_div = 1;
        gemv_body<F, 1, 1, false>(a, (long)blockIdx.x, lds);
    }

    // ---- the same with the quad-lane decoders (gemv_quad.h) ---------------------------------
    // Expert rows are short (2..16 super-blocks): a wavefront step of 16 super-blocks covers 16 / nsb
    // WHOLE rows, so a lane's product is final after one step and a segmented sum over the
    // 4 nsb lanes of a row ends it -- no run across rows, no ring.  A lane decodes two 32-element
    // blocks of a super-block with the format's quad-lane decoder (per super-block work shared by
    // four lanes instead of repeated by eight), loads are issued as in the quad-lane GEMV (two
    // steps in flight).  nsb: a power of two, 2..16.
    constexpr int MOE_QUAD_WAVES = 8;

    // sum over the 4 << nsb_log2 lanes of a row (nsb_log2 = 1..4); every lane gets the total
    __device__ __forceinline__ float moe_quad_row_sum(float v, int nsb_log2) { return segment_sum(v, nsb_log2 - 1); }

    // One wavefront step: decode, dot with the activation row at `aq` (quad-lane layout), this lane's share.
    template <class Q>
    __device__ __forceinline__ float moe_quad_step(const typename Q::Raw &r, const typename Q::Lane &lc,
                                                   const uint8_t *aq_lane)
    {
        v4i w[4];
        typename Q::Scale S;
        Q::decode(r, lc, w, S);
        const v4i a0 = *reinterpret_cast<const v4i *>(aq_lane);
        const v4i a1 = *reinterpret_cast<const v4i *>(aq_lane + 64);
        const v4i a2 = *reinterpret_cast<const v4i *>(aq_lane + 128);
        const v4i a3 = *reinterpret_cast<const v4i *>(aq_lane + 192);
        const float4 sd = *reinterpret_cast<const float4 *>(aq_lane + 256);
        const int i0 = dot16(a1, w[1], dot16z(a0, w[0]));
        const int i1 = dot16(a3, w[3], dot16z(a2, w[2]));
        return Q::apply(S, i0, i1, sd, 0.0f);
    }

    // grid: (workgroups per matrix, n_tokens*top_k, 2 = gate|up), MOE_QUAD_WAVES wavefronts;
    // m.rows_per_wave: STEPS per wavefront, m.gshift: log2(nsb)
    template <class Q>
    __global__ void __launch_bounds__(MOE_QUAD_WAVES *WAVE) moe_gate_up_quad_kernel(const MoEArgs m)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t moe_quad_lds[];
        const int slot = blockIdx.y;
        const int t = slot / m.top_k;
        const int nsb_log2 = m.gshift, nsb = 1 << nsb_log2;
        // what does not depend on the routing goes first: the decode tables and the token's Q8_1 row
        typename Q::TablesRaw tab;
        Q::tables_issue(tab);
        QuadActRaw act[1]; // nsb * 8 <= 128 blocks: one per thread at most
        quad_act_issue(act, m.q8 + (size_t)t * (m.hidden / 32) * 9, nsb * 8);
        const int e = m.ids[slot];
        if (e < 0 || e >= m.n_experts)
            return; // uniform for the workgroup; outputs of a bad id stay untouched
        GemvArgs a;
        a.w = blockIdx.z == 0 ? m.experts[e].d_gate : m.experts[e].d_up;
        if (!a.w)
            return; // an expert whose matrices live elsewhere: skipped like a bad id (uniform)
        a.w = uniform_ptr(a.w);
        a.N = m.inter;
        a.SB = nsb;
        float *y = (blockIdx.z == 0 ? m.out0 : m.out1) + (size_t)slot * m.inter;

        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int l = lane & 3, grp = lane >> 2;
        const typename Q::Lane lc = Q::lane_consts(l);
        const int total = m.inter * nsb;                       // super-blocks of the matrix
        const int step0 = ((int)blockIdx.x * MOE_QUAD_WAVES + wave) * m.rows_per_wave;
        const int nsteps = min(m.rows_per_wave, max(0, (total + QUAD_STEP_SB - 1) / QUAD_STEP_SB - step0));
        // loads are never predicated: past the end a lane re-reads its first super-block
        const size_t t0 = (size_t)min(step0 * QUAD_STEP_SB + grp, total - 1);
        typename Q::Cursor wc = Q::cursor(a, t0, t0, lc);
        const typename Q::Stride stride = Q::stride(0);
        int ld_step = 0;
        auto issue = [&](typename Q::Raw &buf) {
            Q::load(buf, wc, lc, ld_step < nsteps && (step0 + ld_step) * QUAD_STEP_SB + grp < total);
            Q::next(wc, false, stride);
            ++ld_step;
        };
        typename Q::Raw bufA, bufB;
        issue(bufA);
        issue(bufB);
        quad_act_wait<2 * Q::LOADS>(act);
        Q::template tables_wait<2 * Q::LOADS>(tab); // asked for before the activations
        quad_act_store<Q>(act, nsb, nsb * 8, moe_quad_lds, 0);
        Q::tables_store(tab);
        __syncthreads();
        Q::keep(bufA);
        Q::keep(bufB);

        const uint8_t *aq_lane = moe_quad_lds + (grp & (nsb - 1)) * QUAD_SB_LDS + (l << 4);
        const int seg_mask = (4 << nsb_log2) - 1;
        int step = 0;
        auto compute = [&](const typename Q::Raw &buf) {
            const int sb = (step0 + step) * QUAD_STEP_SB + grp;
            float v = moe_quad_step<Q>(buf, lc, aq_lane);
            v = sb < total ? v : 0.0f;
            const float tot = moe_quad_row_sum(v, nsb_log2);
            if (sb < total && (lane & seg_mask) == 0)
                y[sb >> nsb_log2] = tot;
            ++step;
        };
        for (int c0 = 0; c0 < nsteps; c0 += 2)
        {
            Q::template wait<Q::LOADS>(bufA);
            if (step < nsteps) // uniform
                compute(bufA);
            __builtin_amdgcn_sched_barrier(0);
            issue(bufA);
            Q::template wait<Q::LOADS>(bufB);
            if (step < nsteps)
                compute(bufB);
            __builtin_amdgcn_sched_barrier(0);
            issue(bufB);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // loads issued past the end
        Q::keep(bufA);
        Q::keep(bufB);
    }

    // Down projection of one token's slots with the quad-lane decoder: a wavefront walks its steps
    // (16 / nsb whole rows each) slot after slot, so a row's slots are added in ascending order by
    // the one lane that writes it (moe_down_kernel's arithmetic).  The live slots (good id, matrix
    // present) are listed in LDS; two (step, slot) items are in flight per wavefront.
    // grid: (workgroups per matrix, n_tokens); m.rows_per_wave: steps per wavefront, m.gshift: log2(nsb).
    struct MoEQuadSlot
    {
        const void *w;
        float weight;
        int slot; // within the token
    };
    constexpr int MOE_QUAD_MAX_SLOTS = 16;

    template <class Q>
    __global__ void __launch_bounds__(MOE_QUAD_WAVES *WAVE) moe_down_quad_kernel(const MoEArgs m)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t moe_quad_lds[];
        __shared__ MoEQuadSlot live[MOE_QUAD_MAX_SLOTS];
        __shared__ int n_live_s;
        const int t = blockIdx.y;
        const int nsb_log2 = m.gshift, nsb = 1 << nsb_log2;
        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int l = lane & 3, grp = lane >> 2;
        const typename Q::Lane lc = Q::lane_consts(l);
        const int total = m.hidden * nsb; // super-blocks of one down matrix
        const int step0 = ((int)blockIdx.x * MOE_QUAD_WAVES + wave) * m.rows_per_wave;
        const int nsteps = min(m.rows_per_wave, max(0, (total + QUAD_STEP_SB - 1) / QUAD_STEP_SB - step0));

        // what does not depend on the routing goes first: the decode tables and the token's Q8_1
        // rows (its slots form one long activation row: slot s at super-blocks s * nsb ..)
        typename Q::TablesRaw tab;
        Q::tables_issue(tab);
        QuadActRaw act[QUAD_ACT_PASSES];
        const int total_blk = nsb * 8 * m.top_k;
        const uint32_t *q8_token = m.q8 + (size_t)t * m.top_k * (m.inter / 32) * 9;
        quad_act_issue(act, q8_token, total_blk);
        if (wave == 0)
        {
            // the live slots (good id, matrix present), in ascending order: a lane per slot
            const bool in = lane < m.top_k;
            const int e = in ? m.ids[t * m.top_k + lane] : -1;
            const void *w = (e >= 0 && e < m.n_experts) ? m.experts[e].d_down : nullptr;
            const unsigned long long mask = __ballot(w != nullptr);
            if (w) // a bad id, or an expert whose matrices live elsewhere, is skipped
            {
                const int pos = __popcll(mask & ((1ull << lane) - 1ull));
                live[pos].w = w;
                live[pos].weight = m.weights[t * m.top_k + lane];
                live[pos].slot = lane;
            }
            if (lane == 0)
                n_live_s = __popcll(mask);
        }
        quad_act_wait<0>(act);
        Q::template tables_wait<0>(tab);
        if (total_blk <= QUAD_ACT_PASSES * (int)blockDim.x) // uniform
            quad_act_store<Q>(act, nsb * m.top_k, total_blk, moe_quad_lds, 0);
        else
            quad_stage_q8<Q, 1>(q8_token, nsb * m.top_k, moe_quad_lds, moe_quad_lds, 0, 0);
        Q::tables_store(tab);
        __syncthreads();
        const int n_live = n_live_s;
        if (n_live == 0) // uniform
        {
            if (m.accumulate == 0) // no live slot: the token's output is zero, not what the buffer held
            {
                const long r0 = (long)blockIdx.x * MOE_QUAD_WAVES * m.rows_per_wave * (QUAD_STEP_SB >> nsb_log2);
                const long r1 = r0 + (long)MOE_QUAD_WAVES * m.rows_per_wave * (QUAD_STEP_SB >> nsb_log2);
                for (long r = r0 + threadIdx.x; r < r1 && r < m.hidden; r += blockDim.x)
                    m.out0[(size_t)t * m.hidden + r] = 0.0f;
            }
            return;
        }

        GemvArgs a; // weight addressing only
        a.N = m.hidden;
        a.SB = nsb;
        int ld_step = 0, ld_k = 0;
        // loads are never predicated: past the end a lane re-reads its first super-block of the slot
        auto issue = [&](typename Q::Raw &buf) {
            const uint64_t wp = (uint64_t)live[ld_k].w;
            const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)wp);
            const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(wp >> 32));
            a.w = reinterpret_cast<const void *>(((uint64_t)hi << 32) | lo);
            const int st = ld_step < nsteps ? ld_step : 0;
            const size_t ti = (size_t)min((step0 + st) * QUAD_STEP_SB + grp, total - 1);
            const typename Q::Cursor wc = Q::cursor(a, ti, ti, lc);
            Q::load(buf, wc, lc, true);
            if (++ld_k == n_live)
            {
                ld_k = 0;
                ++ld_step;
            }
        };
        typename Q::Raw bufA, bufB;
        issue(bufA);
        issue(bufB);

        const uint8_t *aq_lane = moe_quad_lds + (grp & (nsb - 1)) * QUAD_SB_LDS + (l << 4);
        const int seg_mask = (4 << nsb_log2) - 1;
        const int n_items = nsteps * n_live;
        int item = 0, step = 0, k = 0;
        float y = 0.0f;
        auto compute = [&](const typename Q::Raw &buf) {
            const int sb = (step0 + step) * QUAD_STEP_SB + grp;
            const int slot = live[k].slot;
            float v = moe_quad_step<Q>(buf, lc, aq_lane + (size_t)slot * nsb * QUAD_SB_LDS);
            v = sb < total ? v : 0.0f;
            const float val = weighted(live[k].weight, moe_quad_row_sum(v, nsb_log2));
            const bool writer = sb < total && (lane & seg_mask) == 0;
            float *const dst = m.out0 + (size_t)t * m.hidden + (writer ? (sb >> nsb_log2) : 0);
            // the first live slot starts the sum: from what the output holds when accumulating
            // (((out + v0) + v1) + .., the per-slot kernel's order), else from nothing
            if (k == 0)
                y = (m.accumulate && writer) ? add_rounded(*dst, val) : val;
            else
                y = add_rounded(y, val);
            if (++k == n_live)
            {
                if (writer)
                    *dst = y;
                k = 0;
                ++step;
            }
            ++item;
        };
        for (int c0 = 0; c0 < n_items; c0 += 2)
        {
            Q::template wait<Q::LOADS>(bufA);
            if (item < n_items) // uniform
                compute(bufA);
            __builtin_amdgcn_sched_barrier(0);
            issue(bufA);
            Q::template wait<Q::LOADS>(bufB);
            if (item < n_items)
                compute(bufB);
            __builtin_amdgcn_sched_barrier(0);
            issue(bufB);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // loads issued past the end
        Q::keep(bufA);
        Q::keep(bufB);
    }

    // Down projection of ONE token's slots when there is little work per compute unit (a few tokens):
    // wavefront s of the workgroup takes slot s, so the loads of every slot of a row range are in
    // flight at once and the launch is one memory round trip deep instead of one per slot.  The
    // launch is a chain of dependent loads (id -> expert table -> weights); what does not depend on
    // the routing -- the decode tables and the wavefront's own Q8_1 row -- is asked for first and
    // staged while the weights travel.  The wavefronts leave their rows' dot products in LDS; after
    // one barrier a lane per row adds the live slots in ascending order with their routing weights
    // -- the arithmetic and order of moe_down_quad_kernel, the same bits.
    // grid: (workgroups per matrix, n_tokens), top_k wavefronts (more where the decode tables need a thread a piece);
    // m.rows_per_wave: steps per wavefront (1..MOE_SLOTWAVE_MAX_STEPS), m.gshift: log2(nsb).
    constexpr int MOE_SLOTWAVE_MAX_STEPS = 4;
    template <class Q>
    __global__ void __launch_bounds__(MOE_QUAD_MAX_SLOTS *WAVE) moe_down_slotwave_kernel(const MoEArgs m)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t moe_quad_lds[];
        __shared__ float slot_weight[MOE_QUAD_MAX_SLOTS];
        __shared__ int slot_live[MOE_QUAD_MAX_SLOTS];
        constexpr int NS = MOE_SLOTWAVE_MAX_STEPS;
        const int t = blockIdx.y;
        const int nsb_log2 = m.gshift, nsb = 1 << nsb_log2;
        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int l = lane & 3, grp = lane >> 2;
        const typename Q::Lane lc = Q::lane_consts(l);
        const int total = m.hidden * nsb; // super-blocks of one down matrix
        const int spw = m.rows_per_wave;
        const int step0 = (int)blockIdx.x * spw;
        const int all_steps = (total + QUAD_STEP_SB - 1) / QUAD_STEP_SB;
        const int nsteps = min(spw, max(0, all_steps - step0));
        const int rows_per_step = QUAD_STEP_SB >> nsb_log2;
        const int rows_wg = spw * rows_per_step;
        float *part = reinterpret_cast<float *>(moe_quad_lds + (size_t)m.top_k * nsb * QUAD_SB_LDS); // [slot][rows_wg]

        typename Q::TablesRaw tab;
        Q::tables_issue(tab);
        const bool has_slot = wave < m.top_k; // uniform per wavefront
        const int slot = has_slot ? wave : 0;
        // this wavefront's slot: its Q8_1 row (nsb * 8 <= 128 blocks: two per lane at most)
        QuadActRaw act[QUAD_ACT_PASSES];
        const int nkb = nsb * 8;
        quad_act_issue(act, m.q8 + ((size_t)t * m.top_k + slot) * (size_t)nkb * 9, nkb, lane, WAVE);
        const int e = has_slot ? m.ids[t * m.top_k + slot] : -1;
        const void *w = (e >= 0 && e < m.n_experts) ? m.experts[e].d_down : nullptr;
        const bool mine = w != nullptr; // a bad id, or an expert whose matrices live elsewhere, is skipped
        if (has_slot && lane == 0)
        {
            slot_live[slot] = mine ? 1 : 0;
            slot_weight[slot] = mine ? m.weights[t * m.top_k + slot] : 0.0f;
        }
        typename Q::Raw buf[NS];
        uint8_t *aq = moe_quad_lds + (size_t)slot * nsb * QUAD_SB_LDS;
        if (mine) // uniform
        {
            GemvArgs a; // weight addressing only
            a.N = m.hidden;
            a.SB = nsb;
            a.w = uniform_ptr(w);
            // every step's loads go out at once; never predicated: past the end a lane re-reads an earlier super-block
#pragma unroll
            for (int i = 0; i < NS; ++i)
            {
                const int st = i < nsteps ? i : 0;
                const size_t ti = (size_t)min((step0 + st) * QUAD_STEP_SB + grp, total - 1);
                const typename Q::Cursor wc = Q::cursor(a, ti, ti, lc);
                Q::load(buf[i], wc, lc, true);
            }
            quad_act_wait<NS * Q::LOADS>(act);
            Q::template tables_wait<NS * Q::LOADS>(tab); // asked for before the activations
            quad_act_store<Q>(act, nsb, nkb, aq, 0, lane, WAVE);
        }
        else
        {
            quad_act_wait<0>(act);
            Q::template tables_wait<0>(tab);
        }
        Q::tables_store(tab);
        __syncthreads(); // decode tables, every wavefront's activations, the slots' weights and flags
        if (mine)
        {
#pragma unroll
            for (int i = 0; i < NS; ++i)
                Q::keep(buf[i]);
            const uint8_t *aq_lane = aq + (grp & (nsb - 1)) * QUAD_SB_LDS + (l << 4);
            const int seg_mask = (4 << nsb_log2) - 1;
#pragma unroll
            for (int i = 0; i < NS; ++i)
            {
                // loads issued after step i's: those of the steps behind it
                switch (i)
                {
                case 0: Q::template wait<Q::LOADS *(NS - 1)>(buf[i]); break;
                case 1: Q::template wait<Q::LOADS *(NS - 2)>(buf[i]); break;
                case 2: Q::template wait<Q::LOADS *(NS - 3)>(buf[i]); break;
                default: Q::template wait<0>(buf[i]); break;
                }
                if (i < nsteps) // uniform
                {
                    const int sb = (step0 + i) * QUAD_STEP_SB + grp;
                    float v = moe_quad_step<Q>(buf[i], lc, aq_lane);
                    v = sb < total ? v : 0.0f;
                    const float tot = moe_quad_row_sum(v, nsb_log2);
                    if ((lane & seg_mask) == 0)
                        part[slot * rows_wg + i * rows_per_step + (grp >> nsb_log2)] = tot;
                }
            }
        }
        __syncthreads();
        // one lane per row: the live slots in ascending order
        for (int r = threadIdx.x; r < rows_wg; r += blockDim.x)
        {
            const long row = (long)step0 * rows_per_step + r;
            if (row >= m.hidden)
                break;
            float *dst = m.out0 + (size_t)t * m.hidden + row;
            float y = 0.0f;
            bool first = true;
            for (int s = 0; s < m.top_k; ++s)
            {
                if (!slot_live[s])
                    continue;
                const float val = weighted(slot_weight[s], part[s * rows_wg + r]);
                if (first)
                    y = m.accumulate ? add_rounded(*dst, val) : val;
                else
                    y = add_rounded(y, val);
                first = false;
            }
            if (!first || m.accumulate == 0) // no live slot: zeros unless accumulating
                *dst = y;
        }
    }

    // Gate and up projections of one token slot with SwiGLU and the Q8_1 quantiser of the result in the
    // same launch: a workgroup owns 32 consecutive intermediate rows of BOTH matrices of its slot's
    // expert, so it holds the 32 gate and 32 up values of one Q8_1 block of silu(gate) * up and
    // quantises it itself -- the bits of llam_ql_moe_gate_up (quad-lane kernel) followed by
    // llam_ql_swiglu_quantize, without the fp32 round trip and the second launch.  The decode
    // tables and the token's Q8_1 row do not depend on the routing: they are asked for before the
    // id -> expert table -> weights chain and staged while the weights travel.
    // grid: (inter / 32, n_tokens * top_k), MOE_QUAD_WAVES wavefronts; m.gshift: log2(nsb); the
    // 4 nsb steps of a workgroup (2 nsb per matrix) are dealt to its wavefronts in order.
    // q8_out: Q8_1 blocks [n_tokens * top_k][inter / 32]; blocks of skipped slots are left untouched.
    // NB: steps in flight per wavefront -- 4 when the launch is a latency chain (few slots), 2 (fewer
    // registers, twice the resident workgroups) when there is work to overlap it with.
    // PER > 0: the router and the Q8_1 quantiser of the hidden state run here as well.  Every workgroup
    // quantises its token's fp32 row straight into its LDS (the arithmetic of the stand-alone quantiser) and
    // one of its wavefronts routes the token (moe_route_wave with PER experts per lane) -- work repeated by
    // every workgroup of the token, all of it before the first weight can be asked for anyway -- so the step
    // needs no routing launch; the first workgroup of a token writes the ids and weights out for the down
    // projection.  Slots past the routed ones (always-on experts) take their id from m.ids.
    struct MoERouteArgs
    {
        const float *logits; // [n_tokens][n_route]
        const float *x;      // [n_tokens][hidden] fp32
        int32_t *ids;        // [n_tokens][m.top_k]: columns < top_k are written
        float *weights;
        int n_route, top_k, normalize;
    };

    template <class Q, int NB, int PER = 0>
    __device__ __forceinline__ void moe_gate_up_swiglu_body(const MoEArgs &m, uint32_t *q8_out, const MoERouteArgs *rt = nullptr)
    {
        static_assert(MOE_QUAD_WAVES * WAVE >= Q::TABLE_THREADS, "one table piece per thread");
        static_assert(NB == 2 || NB == 4, "the wait counts below are written for 2 or 4 steps");
        extern __shared__ __attribute__((aligned(16))) uint8_t moe_quad_lds[];
        __shared__ int routed_id[WAVE];
        const int slot = blockIdx.y;
        const int t = slot / m.top_k;
        const int nsb_log2 = m.gshift, nsb = 1 << nsb_log2;
        typename Q::TablesRaw tab;
        Q::tables_issue(tab);
        QuadActRaw act[1]; // nsb * 8 <= 128 blocks: one per thread at most
        int e;
        if constexpr (PER > 0)
        {
            // float4 number i of the row is one lane's share of block i / 8 (whole 8-lane groups: hidden is
            // a multiple of 256)
            const float4 *x4 = reinterpret_cast<const float4 *>(rt->x + (size_t)t * m.hidden);
            for (int i = threadIdx.x; i < m.hidden / 4; i += blockDim.x)
                quad_store_q8_lane<Q>(q8_1_quantize_lane(x4[i]), i, moe_quad_lds);
            if (threadIdx.x < WAVE) // uniform per wavefront
            {
                int id;
                float w;
                moe_route_wave<PER>(rt->logits + (size_t)t * rt->n_route, rt->n_route, rt->top_k, rt->normalize,
                                    (int)threadIdx.x, id, w);
                if ((int)threadIdx.x < rt->top_k)
                {
                    routed_id[threadIdx.x] = id;
                    if (blockIdx.x == 0 && slot == t * m.top_k) // one workgroup per token publishes the routing
                    {
                        rt->ids[(size_t)t * m.top_k + threadIdx.x] = id;
                        rt->weights[(size_t)t * m.top_k + threadIdx.x] = w;
                    }
                }
            }
            Q::template tables_wait<0>(tab);
            Q::tables_store(tab);
            __syncthreads();
            const int s_in_t = slot - t * m.top_k;
            e = s_in_t < rt->top_k ? routed_id[s_in_t] : m.ids[slot];
        }
        else
        {
            quad_act_issue(act, m.q8 + (size_t)t * (m.hidden / 32) * 9, nsb * 8);
            e = m.ids[slot];
        }
        if (e < 0 || e >= m.n_experts)
            return; // uniform for the workgroup
        const void *wg = m.experts[e].d_gate, *wu = m.experts[e].d_up;
        if (!wg || !wu)
            return; // an expert whose matrices live elsewhere: skipped like a bad id (uniform)
        wg = uniform_ptr(wg);
        wu = uniform_ptr(wu);
        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int l = lane & 3, grp = lane >> 2;
        const typename Q::Lane lc = Q::lane_consts(l);
        const int per_mat = 2 * nsb;                                         // steps of 32 rows of one matrix
        const int spw = (2 * per_mat + MOE_QUAD_WAVES - 1) / MOE_QUAD_WAVES; // steps per wavefront (1, 2, 4, 8)
        const int s0 = wave * spw;                                           // this wavefront's first of the 2 * per_mat steps
        float *res = reinterpret_cast<float *>(moe_quad_lds + (size_t)nsb * QUAD_SB_LDS); // [2][32]: gate rows, up rows

        GemvArgs a; // weight addressing only
        a.N = m.inter;
        a.SB = nsb;
        auto issue = [&](typename Q::Raw &buf, int i) {
            const int s = min(s0 + i, 2 * per_mat - 1); // past the end: the last step again, never predicated
            const int mat = s >= per_mat ? 1 : 0;
            a.w = uniform_ptr(mat ? wu : wg);
            const size_t ti = (size_t)blockIdx.x * 32 * nsb + (size_t)(s - mat * per_mat) * QUAD_STEP_SB + grp;
            const typename Q::Cursor wc = Q::cursor(a, ti, ti, lc);
            Q::load(buf, wc, lc, true);
        };
        typename Q::Raw buf[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i)
            issue(buf[i], i);
        if constexpr (PER == 0)
        {
            quad_act_wait<NB * Q::LOADS>(act);
            Q::template tables_wait<NB * Q::LOADS>(tab); // asked for before the activations
            quad_act_store<Q>(act, nsb, nsb * 8, moe_quad_lds, 0);
            Q::tables_store(tab);
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < NB; ++i)
            Q::keep(buf[i]);

        const uint8_t *aq_lane = moe_quad_lds + (grp & (nsb - 1)) * QUAD_SB_LDS + (l << 4);
        const int seg_mask = (4 << nsb_log2) - 1;
        auto compute = [&](const typename Q::Raw &r, int s) {
            if (s < s0 + spw) // uniform (a wavefront with fewer steps than buffers)
            {
                const int mat = s >= per_mat ? 1 : 0;
                const int sb = (s - mat * per_mat) * QUAD_STEP_SB + grp; // within the 32 rows
                const float v = moe_quad_step<Q>(r, lc, aq_lane);
                const float tot = moe_quad_row_sum(v, nsb_log2);
                if ((lane & seg_mask) == 0)
                    res[mat * 32 + (sb >> nsb_log2)] = tot;
            }
        };
        // Rounds of NB steps.  spw and NB are powers of two, so a round is followed by a whole round
        // or by none: while one follows, a buffer is asked for again as soon as it is used up and
        // every wait leaves the other NB - 1 buffers' loads in flight; the last round drains.
        int i0 = 0;
        for (; i0 + NB < spw; i0 += NB)
        {
#pragma unroll
            for (int i = 0; i < NB; ++i)
            {
                Q::template wait<Q::LOADS *(NB - 1)>(buf[i]);
                compute(buf[i], s0 + i0 + i);
                __builtin_amdgcn_sched_barrier(0);
                issue(buf[i], i0 + NB + i);
            }
        }
#pragma unroll
        for (int i = 0; i < NB; ++i)
        {
            // loads issued after step i's: those of the steps behind it
            switch (NB - 1 - i)
            {
            case 3: Q::template wait<Q::LOADS * 3>(buf[i]); break;
            case 2: Q::template wait<Q::LOADS * 2>(buf[i]); break;
            case 1: Q::template wait<Q::LOADS * 1>(buf[i]); break;
            default: Q::template wait<0>(buf[i]); break;
            }
            compute(buf[i], s0 + i0 + i);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < NB; ++i)
            Q::keep(buf[i]);
        __syncthreads();
        if (wave == 0)
        {
            // eight lanes quantise the block (the lane mapping of the stand-alone quantiser); the
            // other lanes of the wavefront run along on the same values and store nothing
            const int sub = lane & 7;
            const float4 g = reinterpret_cast<const float4 *>(res)[sub];
            const float4 u = reinterpret_cast<const float4 *>(res + 32)[sub];
            const Q8Lane q = q8_1_quantize_lane(swiglu4(g, u));
            if (lane < 8)
            {
                uint32_t *dst = q8_out + ((size_t)slot * (m.inter / 32) + blockIdx.x) * 9;
                dst[1 + sub] = q.packed;
                if (sub == 0)
                    dst[0] = q.head;
            }
        }
    }

    template <class Q>
    __global__ void __launch_bounds__(MOE_QUAD_WAVES *WAVE) moe_gate_up_swiglu_kernel(const MoEArgs m, uint32_t *q8_out)
    {
        moe_gate_up_swiglu_body<Q, 4>(m, q8_out);
    }
    // many slots: two steps in flight, fewer registers, three resident workgroups per compute unit
    template <class Q>
    __global__ void __launch_bounds__(MOE_QUAD_WAVES *WAVE)
    moe_gate_up_swiglu_dense_kernel(const MoEArgs m, uint32_t *q8_out)
    {
        moe_gate_up_swiglu_body<Q, 2>(m, q8_out);
    }
    // the same with the router and the hidden state's quantiser inside (PER experts per lane of the routing wavefront)
    template <class Q, int NB, int PER>
    __global__ void __launch_bounds__(MOE_QUAD_WAVES *WAVE)
    moe_route_gate_up_swiglu_kernel(const MoEArgs m, uint32_t *q8_out, const MoERouteArgs r)
    {
        moe_gate_up_swiglu_body<Q, NB, PER>(m, q8_out, &r);
    }

    // grid: (workgroups per matrix, n_tokens).  Slots are walked in ascending
    // order inside the workgroup, so each output element is accumulated by one
    // lane in a fixed order.
    template <class F>
    __global__ void __launch_bounds__(GEMV_WAVES *WAVE) moe_down_kernel(const MoEArgs m)
    {
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        const int t = blockIdx.y;
        bool first = (m.accumulate == 0);
        for (int s = 0; s < m.top_k; ++s)
        {
            const int slot = t * m.top_k + s;
            const int e = m.ids[slot];
            if (e < 0 || e >= m.n_experts || !m.experts[e].d_down)
                continue; // bad id, or an expert whose matrices live elsewhere
            GemvArgs a;
            a.w = m.experts[e].d_down;
            a.q8 = m.q8 + (size_t)slot * (m.inter / 32) * 9;
            a.y = m.out0 + (size_t)t * m.hidden;
            a.sums = nullptr;
            a.ldy = m.hidden;
            a.N = m.hidden;
            a.SB = m.inter / 256;
            a.sb0 = 0;
            a.nsb = a.SB;
            a.rows_per_wave = m.rows_per_wave;
            a.gshift = m.gshift;
            a.accumulate = first ? 0 : 1;
            a.out_scale = m.weights[slot];
            a.row0 = 0;
            a.nrows = 0;
            a.pairs = nullptr;
            a.pair_div = 1;
            gemv_body<F, 1, 1, false>(a, (long)blockIdx.x, lds);
            first = false;
            __syncthreads(); // LDS is restaged by the next slot
        }
        if (first)
        {
            // accumulate == 0 and no live slot: the token's output is zero, not what the buffer held
            const int gsh = m.gshift;
            const int rows_per_wg = GEMV_WAVES * (8 >> gsh) * m.rows_per_wave;
            const long r0 = (long)blockIdx.x * rows_per_wg;
            for (long r = r0 + threadIdx.x; r < r0 + rows_per_wg && r < m.hidden; r += blockDim.x)
                m.out0[(size_t)t * m.hidden + r] = 0.0f;
        }
    }

    // Down projection for short expert rows (at most 8 super-blocks, i.e. one load per
    // lane and row) and up to S slots per token.  The activations of all slots of the
    // token (contiguous Q8_1 rows) are staged in ONE pass, and for each row batch the
    // weight loads of ALL slots are issued before the first is decoded, so a workgroup
    // waits for memory once per row batch instead of once per slot.  Same arithmetic and
    // slot order as moe_down_kernel.  grid: (workgroups per matrix, n_tokens).
    template <class F, int S>
    __global__ void __launch_bounds__(GEMV_WAVES *WAVE) moe_down_multi_kernel(const MoEArgs m)
    {
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        const int t = blockIdx.y;
        const int nsb = m.inter / 256;
        const int nkb = nsb * 8;
        const int nkb_all = nkb * m.top_k; // the token's slots form one long activation row
        uint32_t *aq = lds;
        float *ad = reinterpret_cast<float *>(aq + nkb_all * 8);
        float *asd = ad + nkb_all;
        void *tab = format_tables_lds<F>();

        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = threadIdx.x >> 6;
        const int c = lane & 7;
        const int grp = lane >> 3;
        const bool odd = (c & 1) != 0;
        const int G = 1 << m.gshift;
        const int R = 8 >> m.gshift;
        const int rsub = grp >> m.gshift;
        const int sb = grp & (G - 1); // the one super-block of this lane

        GemvArgs a; // weight addressing only
        a.N = m.hidden;
        a.SB = nsb;
        int e[S];
        float wt[S];
#pragma unroll
        for (int s = 0; s < S; ++s)
        {
            e[s] = (s < m.top_k) ? m.ids[t * m.top_k + s] : -1;
            if (e[s] >= m.n_experts)
                e[s] = -1;
            wt[s] = (s < m.top_k) ? m.weights[t * m.top_k + s] : 0.0f;
        }
        const void *wdown[S];
#pragma unroll
        for (int s = 0; s < S; ++s)
        {
            wdown[s] = e[s] >= 0 ? m.experts[e[s]].d_down : nullptr;
            if (!wdown[s])
                e[s] = -1; // an expert whose matrices live elsewhere: skipped like a bad id
        }

        const long wg_row0 = (long)blockIdx.x * (GEMV_WAVES * R * m.rows_per_wave);
        auto load_rows = [&](typename F::Raw(&raw)[S], long row) {
#pragma unroll
            for (int s = 0; s < S; ++s)
            {
                raw[s] = typename F::Raw{};
                if (e[s] >= 0 && row < m.hidden && sb < nsb)
                {
                    a.w = wdown[s];
                    raw[s] = F::load(a, row, sb, c);
                }
            }
        };
        typename F::Raw raw[S];
        load_rows(raw, wg_row0 + (long)wave * R + rsub); // in flight during the staging

        if (F::TABLE_BYTES > 0)
            F::stage_tables(tab);
        stage_q8<F, 1>(m.q8 + (size_t)t * nkb_all * 9, nkb_all, 0, nkb_all, aq, ad, asd);
        __syncthreads();

        for (int r = 0; r < m.rows_per_wave; ++r)
        {
            const long row = wg_row0 + ((long)r * GEMV_WAVES + wave) * R + rsub;
            if (wg_row0 + ((long)r * GEMV_WAVES + wave) * R >= m.hidden) // uniform
                break;
            const bool row_ok = row < m.hidden && sb < nsb;
            typename F::Raw cur[S];
#pragma unroll
            for (int s = 0; s < S; ++s)
                cur[s] = raw[s];
            if (r + 1 < m.rows_per_wave)
                load_rows(raw, row + (long)GEMV_WAVES * R);

            // accumulate: the slots are added one by one onto what the output holds,
            // ((out + v0) + v1) + .., as the per-slot kernel does (the reference's vec_axpy per slot)
            const bool writer = row < m.hidden && (lane & (8 * G - 1)) == 0;
            float *const dst = m.out0 + (size_t)t * m.hidden + (row < m.hidden ? row : 0);
            float y = (m.accumulate && writer) ? *dst : 0.0f;
            bool first = (m.accumulate == 0);
#pragma unroll
            for (int s = 0; s < S; ++s)
            {
                if (e[s] < 0) // uniform
                    continue;
                float acc = 0.0f;
                if (row_ok)
                {
                    v4i w0, w1;
                    int j;
                    float bscale, bmin;
                    F::decode(cur[s], c, w0, w1, j, bscale, bmin, tab);
                    const v4i *ap = reinterpret_cast<const v4i *>(aq + (size_t)((s * nsb + sb) * 8 + c) * 8);
                    const v4i a0 = ap[0];
                    const v4i a1 = ap[1];
                    int idot;
                    if (F::PAIR)
                    {
                        const int p0 = dot16(a0, w0, 0);
                        const int p1 = dot16(a1, w1, 0);
                        const int got = dpp_i32<DPP_QUAD_XOR1>(odd ? p0 : p1);
                        idot = (odd ? p1 : p0) + got;
                    }
                    else
                    {
                        idot = dot16(a1, w1, dot16(a0, w0, 0));
                    }
                    const int kb = (s * nsb + sb) * 8 + j;
                    acc = fmaf((float)idot, ad[kb] * bscale, 0.0f);
                    if (F::HAS_MIN)
                        acc = fmaf(asd[kb], bmin, acc);
                }
                const float total = segment_sum(acc, m.gshift);
                const float v = weighted(wt[s], total);
                if (first)
                {
                    y = v; // accumulate == 0: the first live slot overwrites
                    first = false;
                }
                else
                    y = add_rounded(y, v);
            }
            // (a token without a live slot: y is 0, which overwrites when accumulate == 0)
            if (writer)
                *dst = y;
        }
    }


    // ---- token grouping by expert ---------------------------------------------------------
    // Batches: the (token, slot) pairs sorted by expert id, so that the grouped launches read
    // every distinct expert's matrices once per chunk of four of its tokens
    // (MoEExpertComputeStage::execute buckets the same way on the host,
    // src/v2/execution/compute_stages/stages/MoEExpertComputeStage.cpp:884-979; device
    // counterpart IMoEKernel::groupTokensByExpertDevice, src/v2/kernels/IMoEKernel.h:737).
    // Workspace, int32, P = n_tokens * slot_stride:
    //   [0] segments  [1] valid pairs  [2] chunks  [3] pairs per chunk
    //   seg_expert[P]  seg_begin[P+1]  pair_sorted[P]  chunk_expert[P]  chunk_begin[P]  chunk_count[P]
    // A segment is the run of one expert's pairs in pair_sorted (stable: ascending pair index);
    // a chunk is up to moe_chunk_size(P) consecutive pairs of a segment, the unit of work of the grouped
    // launches.  Pairs with an id outside [0, n_experts) are left out.
    constexpr int MOE_GROUP_THREADS = 1024;
    constexpr int MOE_GROUP_MAX_PAIRS = 4096;
    constexpr int MOE_GROUP_MAX_EXPERTS = 2 * MOE_GROUP_THREADS; // two experts per thread
    // Tokens of one expert that share a workgroup's pass over its matrix.  Measured on the
    // 256-expert IQ3_S shape: four pay from about 500 pairs on (64 tokens: 217 against 247 us
    // per step); below that the larger register footprint of the four-row body costs more than
    // the second read of the few experts with more than two tokens saves (16 tokens: 107
    // against 104 us).
    constexpr int MOE_CHUNK_MAX = 4;
    __host__ __device__ inline int moe_chunk_size(int P) { return P >= 512 ? 4 : 2; }
    struct MoEGroupView
    {
        int32_t *head, *seg_expert, *seg_begin, *pair_sorted, *chunk_expert, *chunk_begin, *chunk_count;
    };
    __host__ __device__ inline MoEGroupView moe_group_view(void *ws, int P)
    {
        int32_t *w = static_cast<int32_t *>(ws);
        MoEGroupView g;
        g.head = w;
        g.seg_expert = w + 4;
        g.seg_begin = g.seg_expert + P;
        g.pair_sorted = g.seg_begin + (P + 1);
        g.chunk_expert = g.pair_sorted + P;
        g.chunk_begin = g.chunk_expert + P;
        g.chunk_count = g.chunk_begin + P;
        return g;
    }
    __host__ __device__ inline size_t moe_group_bytes(int P) { return ((size_t)(4 + 6 * (size_t)P + 1) * 4 + 15) & ~(size_t)15; }

    // exclusive sums of three counters over the workgroup's threads, and the totals
    struct Int3
    {
        int a, b, c;
    };
    __device__ __forceinline__ Int3 block_exclusive_scan3(Int3 v, Int3 &total, int (*wave_sums)[3])
    {
        const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
        Int3 inc = v;
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1)
        {
            const int a = __shfl_up(inc.a, off), b = __shfl_up(inc.b, off), c = __shfl_up(inc.c, off);
            if (lane >= off)
            {
                inc.a += a;
                inc.b += b;
                inc.c += c;
            }
        }
        if (lane == WAVE - 1)
        {
            wave_sums[wave][0] = inc.a;
            wave_sums[wave][1] = inc.b;
            wave_sums[wave][2] = inc.c;
        }
        __syncthreads();
        Int3 base{0, 0, 0};
        total = Int3{0, 0, 0};
        for (int w = 0; w < nwaves; ++w)
        {
            if (w < wave)
            {
                base.a += wave_sums[w][0];
                base.b += wave_sums[w][1];
                base.c += wave_sums[w][2];
            }
            total.a += wave_sums[w][0];
            total.b += wave_sums[w][1];
            total.c += wave_sums[w][2];
        }
        return Int3{base.a + inc.a - v.a, base.b + inc.b - v.b, base.c + inc.c - v.c};
    }

    __global__ void __launch_bounds__(MOE_GROUP_THREADS)
        moe_group_kernel(const int32_t *__restrict__ ids, int P, int n_experts, void *ws)
    {
        extern __shared__ int32_t grp_se[]; // expert of every pair (INT_MAX: left out), padded to a multiple of 4
        __shared__ int hist[MOE_GROUP_MAX_EXPERTS];
        __shared__ int wave_sums[MOE_GROUP_THREADS / WAVE][3];
        const MoEGroupView g = moe_group_view(ws, P);
        const int tid = threadIdx.x;
        for (int e = tid; e < MOE_GROUP_MAX_EXPERTS; e += blockDim.x)
            hist[e] = 0;
        __syncthreads();
        const int P4 = (P + 3) & ~3;
        for (int p = tid; p < P4; p += blockDim.x)
        {
            const int e = p < P ? ids[p] : -1;
            const bool ok = e >= 0 && e < n_experts;
            grp_se[p] = ok ? e : 0x7FFFFFFF;
            if (ok)
                atomicAdd(&hist[e], 1); // integer: the counts do not depend on the order
        }
        __syncthreads();
        // thread i owns experts 2i and 2i+1: pairs, non-empty experts and chunks before them
        const int c0 = hist[2 * tid], c1 = hist[2 * tid + 1];
        const int MOE_CHUNK = moe_chunk_size(P);
        const int k0 = (c0 + MOE_CHUNK - 1) / MOE_CHUNK, k1 = (c1 + MOE_CHUNK - 1) / MOE_CHUNK;
        Int3 total;
        const Int3 ex = block_exclusive_scan3(Int3{c0 + c1, (c0 > 0) + (c1 > 0), k0 + k1}, total, wave_sums);
        __syncthreads(); // everybody has read its counts: hist becomes the experts' offsets
        hist[2 * tid] = ex.a;
        hist[2 * tid + 1] = ex.a + c0;
        auto emit = [&](int e, int cnt, int seg, int begin, int chunk) {
            g.seg_expert[seg] = e;
            g.seg_begin[seg] = begin;
            for (int j = 0; j * MOE_CHUNK < cnt; ++j)
            {
                g.chunk_expert[chunk + j] = e;
                g.chunk_begin[chunk + j] = begin + j * MOE_CHUNK;
                g.chunk_count[chunk + j] = cnt - j * MOE_CHUNK < MOE_CHUNK ? cnt - j * MOE_CHUNK : MOE_CHUNK;
            }
        };
        if (c0 > 0)
            emit(2 * tid, c0, ex.b, ex.a, ex.c);
        if (c1 > 0)
            emit(2 * tid + 1, c1, ex.b + (c0 > 0), ex.a + c0, ex.c + k0);
        if (tid == 0)
        {
            g.head[0] = total.b;
            g.head[1] = total.a;
            g.head[2] = total.c;
            g.head[3] = MOE_CHUNK;
            g.seg_begin[total.b] = total.a;
        }
        __syncthreads();
        // stable place of every pair: its expert's offset plus the earlier pairs of that expert
        for (int p = tid; p < P; p += blockDim.x)
        {
            const int e = grp_se[p];
            if (e == 0x7FFFFFFF)
                continue;
            int same = 0;
            const int4 *v = reinterpret_cast<const int4 *>(grp_se);
            const int full = p >> 2;
            for (int q = 0; q < full; ++q)
            {
                const int4 x = v[q];
                same += (x.x == e) + (x.y == e) + (x.z == e) + (x.w == e);
            }
            for (int q = full * 4; q < p; ++q)
                same += grp_se[q] == e;
            g.pair_sorted[hist[e] + same] = p;
        }
    }

    // One chunk of the grouped launches: the expert's matrix (gate, up or down) against the
    // chunk's 1..MOE_CHUNK tokens, through the generic GEMV body with its batch rows gathered
    // through the sorted pair list.  Every output row carries the bits of the ungrouped launch:
    // a batch row's arithmetic does not depend on the batch it rides in.
    template <class F, int MAXM>
    __device__ __forceinline__ void moe_chunk_body(GemvArgs &a, const MoEGroupView &g, int chunk, uint32_t *lds)
    {
        a.pairs = g.pair_sorted + g.chunk_begin[chunk];
        const int n = g.chunk_count[chunk]; // uniform
        if constexpr (MAXM >= 4)
        {
            if (n == 4)
            {
                gemv_body<F, 4, 1, false>(a, (long)blockIdx.x, lds);
                return;
            }
            if (n == 3)
            {
                gemv_body<F, 3, 1, false>(a, (long)blockIdx.x, lds);
                return;
            }
        }
        if (n == 2)
            gemv_body<F, 2, 1, false>(a, (long)blockIdx.x, lds);
        else
            gemv_body<F, 1, 1, false>(a, (long)blockIdx.x, lds);
    }

    // grid: (workgroups per matrix, chunks (upper bound), 2 = gate|up)
    template <class F, int MAXM>
    __global__ void __launch_bounds__(GEMV_WAVES *WAVE) moe_gate_up_grouped_kernel(const MoEArgs m, void *ws, int P)
    {
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        const MoEGroupView g = moe_group_view(ws, P);
        const int chunk = blockIdx.y;
        if (chunk >= g.head[2])
            return; // uniform
        const int e = g.chunk_expert[chunk];
        GemvArgs a;
        a.w = blockIdx.z == 0 ? m.experts[e].d_gate : m.experts[e].d_up;
        if (!a.w)
            return; // an expert whose matrices live elsewhere (uniform)
        a.q8 = m.q8;
        a.y = blockIdx.z == 0 ? m.out0 : m.out1;
        a.sums = nullptr;
        a.ldy = m.inter;
        a.N = m.inter;
        a.SB = m.hidden / 256;
        a.sb0 = 0;
        a.nsb = a.SB;
        a.rows_per_wave = m.rows_per_wave;
        a.gshift = m.gshift;
        a.accumulate = 0;
        a.out_scale = 1.0f;
        a.row0 = 0;
        a.nrows = 0;
        a.pair_div = m.top_k; // pair = token * slot_stride + slot
        moe_chunk_body<F, MAXM>(a, g, chunk, lds);
    }

    // Down projection of one chunk into per-pair rows: pair_out[pair][:] = W_down[e] . act[pair]
    // (unweighted; moe_pair_reduce_kernel adds a token's slots).  grid: (workgroups per matrix, chunks)
    template <class F, int MAXM>
    __global__ void __launch_bounds__(GEMV_WAVES *WAVE) moe_down_grouped_kernel(const MoEArgs m, void *ws, int P)
    {
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        const MoEGroupView g = moe_group_view(ws, P);
        const int chunk = blockIdx.y;
        if (chunk >= g.head[2])
            return;
        const int e = g.chunk_expert[chunk];
        GemvArgs a;
        a.w = m.experts[e].d_down;
        if (!a.w)
            return;
        a.q8 = m.q8;  // Q8_1 activations, one row per pair
        a.y = m.out1; // [P x hidden]
        a.sums = nullptr;
        a.ldy = m.hidden;
        a.N = m.hidden;
        a.SB = m.inter / 256;
        a.sb0 = 0;
        a.nsb = a.SB;
        a.rows_per_wave = m.rows_per_wave;
        a.gshift = m.gshift;
        a.accumulate = 0;
        a.out_scale = 1.0f;
        a.row0 = 0;
        a.nrows = 0;
        a.pair_div = 1;
        moe_chunk_body<F, MAXM>(a, g, chunk, lds);
    }

    // The grouped launches on the quad-lane decoder (expert rows of 2, 4, 8 or 16 super-blocks): a workgroup
    // row takes one chunk -- an expert and 1..MAXM of its (token, slot) pairs -- decodes every step of the
    // expert's matrix ONCE and multiplies it with each pair's activation row: per pair the decode, the dots
    // and the row sum of moe_gate_up_quad_kernel / moe_down_quad_kernel, the same bits.
    // DOWN = false: grid (workgroups per matrix, chunks (upper bound), 2 = gate|up), activations = the
    // pair's token's hidden row, outputs out0/out1[pair][inter].  DOWN = true: grid (workgroups, chunks),
    // activations = the pair's own row of inter values, outputs out1[pair][hidden] (unweighted).
    // m.rows_per_wave: steps per wavefront, m.gshift: log2(nsb).
    template <class Q, int MAXM, bool DOWN>
    __global__ void __launch_bounds__(MOE_QUAD_WAVES *WAVE) moe_grouped_quad_kernel(const MoEArgs m, void *ws, int P)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t moe_quad_lds[];
        const MoEGroupView g = moe_group_view(ws, P);
        const int chunk = blockIdx.y;
        if (chunk >= g.head[2])
            return; // uniform
        const int e = g.chunk_expert[chunk];
        const void *w = DOWN ? m.experts[e].d_down : (blockIdx.z == 0 ? m.experts[e].d_gate : m.experts[e].d_up);
        if (!w)
            return; // an expert whose matrices live elsewhere (uniform)
        const int n = g.chunk_count[chunk]; // uniform, 1..MAXM
        const int32_t *pairs = g.pair_sorted + g.chunk_begin[chunk];
        const int K = DOWN ? m.inter : m.hidden, N = DOWN ? m.hidden : m.inter;
        const int nsb_log2 = m.gshift, nsb = 1 << nsb_log2;
        GemvArgs a; // weight addressing only
        a.w = uniform_ptr(w);
        a.N = N;
        a.SB = nsb;

        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int l = lane & 3, grp = lane >> 2;
        const typename Q::Lane lc = Q::lane_consts(l);
        const int total = N * nsb; // super-blocks of the matrix
        const int step0 = ((int)blockIdx.x * MOE_QUAD_WAVES + wave) * m.rows_per_wave;
        const int nsteps = min(m.rows_per_wave, max(0, (total + QUAD_STEP_SB - 1) / QUAD_STEP_SB - step0));
        // loads are never predicated: past the end a lane re-reads its first super-block
        const size_t t0 = (size_t)min(step0 * QUAD_STEP_SB + grp, total - 1);
        typename Q::Cursor wc = Q::cursor(a, t0, t0, lc);
        const typename Q::Stride stride = Q::stride(0);
        int ld_step = 0;
        auto issue = [&](typename Q::Raw &buf) {
            Q::load(buf, wc, lc, ld_step < nsteps && (step0 + ld_step) * QUAD_STEP_SB + grp < total);
            Q::next(wc, false, stride);
            ++ld_step;
        };
        typename Q::Raw bufA, bufB;
        issue(bufA);
        issue(bufB);
        // the chunk's activation rows, one thread per Q8_1 block (row mm of the chunk at mm * nsb super-blocks)
        const int nkb = nsb * 8;
        for (int idx = threadIdx.x; idx < n * nkb; idx += blockDim.x)
        {
            const int mm = idx / nkb, kb = idx - mm * nkb;
            const int pair = pairs[mm];
            const uint32_t *src = m.q8 + ((size_t)(DOWN ? pair : pair / m.top_k) * nkb + kb) * 9;
            uint32_t v[9];
#pragma unroll
            for (int i = 0; i < 9; ++i)
                v[i] = src[i];
            const float d = h2f((uint16_t)(v[0] & 0xFFFFu));
            const int sb = kb >> 3, j = kb & 7;
            int ll, odd;
            Q::owner(j, ll, odd);
            uint8_t *base = moe_quad_lds + ((size_t)mm * nsb + sb) * QUAD_SB_LDS + ll * 16;
            *reinterpret_cast<float2 *>(base + 256 + odd * 8) = make_float2(d, (float)(int16_t)(v[0] >> 16) * d);
            *reinterpret_cast<uint4 *>(base + (odd * 2) * 64) = make_uint4(v[1], v[2], v[3], v[4]);
            *reinterpret_cast<uint4 *>(base + (odd * 2 + 1) * 64) = make_uint4(v[5], v[6], v[7], v[8]);
        }
        Q::stage();
        __syncthreads();
        Q::keep(bufA);
        Q::keep(bufB);

        const uint8_t *aq_lane = moe_quad_lds + (grp & (nsb - 1)) * QUAD_SB_LDS + (l << 4);
        const int seg_mask = (4 << nsb_log2) - 1;
        float *out = DOWN ? m.out1 : (blockIdx.z == 0 ? m.out0 : m.out1);
        int step = 0;
        auto compute = [&](const typename Q::Raw &buf) {
            const int sb = (step0 + step) * QUAD_STEP_SB + grp;
            v4i wq[4];
            typename Q::Scale S;
            Q::decode(buf, lc, wq, S);
#pragma unroll
            for (int mm = 0; mm < MAXM; ++mm)
            {
                if (mm < n) // uniform
                {
                    const uint8_t *ar = aq_lane + (size_t)mm * nsb * QUAD_SB_LDS;
                    const v4i a0 = *reinterpret_cast<const v4i *>(ar);
                    const v4i a1 = *reinterpret_cast<const v4i *>(ar + 64);
                    const v4i a2 = *reinterpret_cast<const v4i *>(ar + 128);
                    const v4i a3 = *reinterpret_cast<const v4i *>(ar + 192);
                    const float4 sd = *reinterpret_cast<const float4 *>(ar + 256);
                    const int i0 = dot16(a1, wq[1], dot16z(a0, wq[0]));
                    const int i1 = dot16(a3, wq[3], dot16z(a2, wq[2]));
                    float v = Q::apply(S, i0, i1, sd, 0.0f);
                    v = sb < total ? v : 0.0f;
                    const float tot = moe_quad_row_sum(v, nsb_log2);
                    if (sb < total && (lane & seg_mask) == 0)
                        out[(size_t)pairs[mm] * N + (sb >> nsb_log2)] = tot;
                }
            }
            ++step;
        };
        for (int c0 = 0; c0 < nsteps; c0 += 2)
        {
            Q::template wait<Q::LOADS>(bufA);
            if (step < nsteps) // uniform
                compute(bufA);
            __builtin_amdgcn_sched_barrier(0);
            issue(bufA);
            Q::template wait<Q::LOADS>(bufB);
            if (step < nsteps)
                compute(bufB);
            __builtin_amdgcn_sched_barrier(0);
            issue(bufB);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // loads issued past the end
        Q::keep(bufA);
        Q::keep(bufB);
    }

    // out[t][h] (+)= sum over the token's live slots, ascending, of weight * pair_out[pair][h]:
    // the arithmetic and order of moe_down_kernel, so the same bits.  A token without a live
    // slot gets zeros when accumulate == 0.
    __global__ void __launch_bounds__(256)
        moe_pair_reduce_kernel(const float *__restrict__ pair_out, const int32_t *__restrict__ ids,
                               const float *__restrict__ weights, const llam_ql_expert *__restrict__ experts,
                               int n_experts, float *__restrict__ out, int slots, int hidden, int accumulate)
    {
        const int t = blockIdx.y;
        const int h = blockIdx.x * blockDim.x + threadIdx.x;
        if (h >= hidden)
            return;
        // accumulate: the sum starts from what the output holds and takes the slots one by one,
        // ((out + v0) + v1) + .., as the per-slot launches do
        float *dst = out + (size_t)t * hidden + h;
        float y = accumulate ? *dst : 0.0f;
        bool first = accumulate == 0;
        for (int s = 0; s < slots; ++s)
        {
            const int pair = t * slots + s;
            const int e = ids[pair];
            if (e < 0 || e >= n_experts || !experts[e].d_down)
                continue;
            const float v = weighted(weights[pair], pair_out[(size_t)pair * hidden + h]);
            if (first)
            {
                y = v;
                first = false;
            }
            else
                y = add_rounded(y, v);
        }
        *dst = y;
    }

    // ---- SwiGLU + Q8_1 ---------------------------------------------------------------
    // Same lane mapping as the plain quantiser: 8 lanes per 32-element block.
    __global__ void __launch_bounds__(256)
        swiglu_quantize_kernel(const float4 *__restrict__ gate, const float4 *__restrict__ up,
                               float4 *__restrict__ act_out, uint32_t *__restrict__ out, long n_blocks)
    {
        const long lane_global = (long)blockIdx.x * blockDim.x + threadIdx.x;
        const long blk = lane_global >> 3;
        const int sub = (int)(lane_global & 7);
        if (blk >= n_blocks)
            return;
        const float4 g = gate[lane_global];
        const float4 u = up[lane_global];
        const float4 v = swiglu4(g, u);
        if (act_out)
            act_out[lane_global] = v;

        const Q8Lane q = q8_1_quantize_lane(v);
        uint32_t *dst = out + blk * 9;
        dst[1 + sub] = q.packed;
        if (sub == 0)
            dst[0] = q.head;
    }

    // ---- fp32 routing indices -> int32 ids ----------------------------------------------------
    // The reference's device routing tensors hold expert indices as fp32 values
    // (IMoEKernel::groupedExpert*DecodeFromRouting, src/v2/kernels/IMoEKernel.h:480-575).
    __global__ void __launch_bounds__(256)
        moe_ids_from_f32_kernel(const float *__restrict__ src, int32_t *__restrict__ dst, int n)
    {
        const int i = blockIdx.x * blockDim.x + threadIdx.x;
        if (i < n)
        {
            const float v = src[i];
            dst[i] = (v >= 0.0f && v < 2147483520.0f) ? (int32_t)v : -1; // NaN, negative, huge: no expert
        }
    }

    // What decodeRouteSelect publishes beside the runtime top-k state (IMoEKernel.h:245-258;
    // kernels/rocm/moe/ROCmMoEKernel.cpp:2956-3019): the routing as fp32 tensors for stages that
    // still read those, and one count per selected expert in the layer's decode histogram.
    // Integer atomics: the counts do not depend on the order of the adds.
    __global__ void __launch_bounds__(256)
        moe_publish_routing_kernel(const int32_t *__restrict__ ids, const float *__restrict__ weights, int n_tokens,
                                   int top_k, int slot_stride, float *__restrict__ indices_f32,
                                   float *__restrict__ weights_f32, unsigned long long *__restrict__ histogram,
                                   int n_experts)
    {
        const int i = blockIdx.x * blockDim.x + threadIdx.x;
        if (i >= n_tokens * top_k)
            return;
        const int t = i / top_k, s = i - t * top_k;
        const int32_t e = ids[(size_t)t * slot_stride + s];
        if (indices_f32)
            indices_f32[i] = (float)e;
        if (weights_f32)
            weights_f32[i] = weights[(size_t)t * slot_stride + s];
        if (histogram && e >= 0 && e < n_experts)
            atomicAdd(histogram + e, 1ull);
    }

    // ---- shared expert gate -----------------------------------------------------------
    // out[t,:] += sigmoid(dot(gate_inp, hidden[t,:])) * shared[t,:]
    // (CPUMoEKernel::sharedExpertGate, kernels/cpu/moe/CPUMoEKernel.cpp:162-197, followed by
    // the add into the token output).  One workgroup per token.
    __global__ void __launch_bounds__(256)
        shared_expert_add_kernel(float *__restrict__ out, const float *__restrict__ shared,
                                 const float *__restrict__ hidden, const float *__restrict__ gate_inp, int d_model)
    {
        __shared__ float s_part[256];
        const int t = blockIdx.x;
        const float *x = hidden + (size_t)t * d_model;
        float gate = 1.0f;
        if (gate_inp)
        {
            float part = 0.0f;
            for (int i = threadIdx.x; i < d_model; i += blockDim.x)
                part = fmaf(gate_inp[i], x[i], part);
            s_part[threadIdx.x] = part;
            __syncthreads();
            for (int off = 128; off > 0; off >>= 1)
            {
                if ((int)threadIdx.x < off)
                    s_part[threadIdx.x] += s_part[threadIdx.x + off];
                __syncthreads();
            }
            gate = __fdiv_rn(1.0f, 1.0f + expf(-s_part[0]));
        }
        for (int i = threadIdx.x; i < d_model; i += blockDim.x)
            out[(size_t)t * d_model + i] += gate * shared[(size_t)t * d_model + i];
    }

    // shared[t,:] *= sigmoid(dot(gate_inp, hidden[t,:])) in place (IMoEKernel::sharedExpertGate,
    // kernels/cpu/moe/CPUMoEKernel.cpp:162-197).  One workgroup per token.
    __global__ void __launch_bounds__(256)
        shared_expert_gate_kernel(float *__restrict__ shared, const float *__restrict__ hidden,
                                  const float *__restrict__ gate_inp, int d_model)
    {
        __shared__ float s_part[256];
        const int t = blockIdx.x;
        const float *x = hidden + (size_t)t * d_model;
        float part = 0.0f;
        for (int i = threadIdx.x; i < d_model; i += blockDim.x)
            part = fmaf(gate_inp[i], x[i], part);
        s_part[threadIdx.x] = part;
        __syncthreads();
        for (int off = 128; off > 0; off >>= 1)
        {
            if ((int)threadIdx.x < off)
                s_part[threadIdx.x] += s_part[threadIdx.x + off];
            __syncthreads();
        }
        const float gate = __fdiv_rn(1.0f, 1.0f + expf(-s_part[0]));
        for (int i = threadIdx.x; i < d_model; i += blockDim.x)
            shared[(size_t)t * d_model + i] *= gate;
    }

    // batch[i,:] = hidden[idx[i],:] (IMoEKernel::gatherTokenBatch, CPUMoEKernel.cpp:133-144);
    // rows whose index is outside [0, n_rows) are filled with zeros.
    __global__ void __launch_bounds__(256)
        moe_gather_rows_kernel(const float *__restrict__ hidden, float *__restrict__ batch,
                               const int32_t *__restrict__ idx, int n_rows, int d_model)
    {
        const int i = blockIdx.x;
        const int src = idx[i];
        const bool ok = src >= 0 && src < n_rows;
        for (int c = threadIdx.x; c < d_model; c += blockDim.x)
            batch[(size_t)i * d_model + c] = ok ? hidden[(size_t)src * d_model + c] : 0.0f;
    }

    // out[idx[i],:] += w[i] * expert_out[i,:] (IMoEKernel::scatterAddWeighted, CPUMoEKernel.cpp:146-160).
    // One workgroup per COLUMN block walks the batch rows in ascending order, so rows that name
    // the same token are added one after the other, as the reference's loop adds them.
    __global__ void __launch_bounds__(256)
        moe_scatter_add_weighted_kernel(float *__restrict__ out, const float *__restrict__ expert_out,
                                        const int32_t *__restrict__ idx, const float *__restrict__ w, int num_tokens,
                                        int n_rows, int d_model)
    {
        const int c = blockIdx.x * blockDim.x + threadIdx.x;
        if (c >= d_model)
            return;
        for (int i = 0; i < num_tokens; ++i)
        {
            const int dst = idx[i];
            if (dst < 0 || dst >= n_rows)
                continue;
            float *o = out + (size_t)dst * d_model + c;
            *o = fmaf(w[i], expert_out[(size_t)i * d_model + c], *o);
        }
    }

    // gate[i] = silu(gate[i]) * up[i] in place (IMoEKernel::swiGLU, CPUMoEKernel.cpp:199-202), four
    // values per thread with the arithmetic of swiglu4.
    __global__ void __launch_bounds__(256)
        swiglu_inplace_kernel(float *__restrict__ gate, const float *__restrict__ up, long n4, long n)
    {
        const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
        if (i < n4)
        {
            float4 *g = reinterpret_cast<float4 *>(gate) + i;
            *g = swiglu4(*g, reinterpret_cast<const float4 *>(up)[i]);
        }
        else if (i < n4 + (n - 4 * n4)) // the last n % 4 values, one thread each
        {
            const long e = 4 * n4 + (i - n4);
            const float4 v = swiglu4(make_float4(gate[e], 0.f, 0.f, 0.f), make_float4(up[e], 0.f, 0.f, 0.f));
            gate[e] = v.x;
        }
    }

    namespace
    {
        // matrices: how many [N x SB] matrices the launch walks (slots x tokens x gate|up).
        // Every workgroup stages its activations (and the format's tables) once, so it
        // should own as many rows as still leaves a few workgroups per compute unit.
        void moe_shape(int N, int SB, long matrices, int device_id, int &gshift, int &rpw, long &grid_x)
        {
            gshift = 3;
            while (gshift > 0 && (1 << (gshift - 1)) >= SB)
                --gshift;
            const int R = 8 >> gshift;
            const long rows_total = (long)N * matrices;
            const long per_cu = rows_total / cu_count(device_id);
            rpw = 1;
            while (rpw < 8 && (long)GEMV_WAVES * R * rpw * 2 * 4 <= per_cu && (long)GEMV_WAVES * R * rpw * 2 <= N)
                rpw *= 2;
            const int rows_per_wg = GEMV_WAVES * R * rpw;
            grid_x = ((long)N + rows_per_wg - 1) / rows_per_wg;
        }

        // rows the short-row quad-lane kernels take: 2, 4, 8 or 16 super-blocks
        bool moe_quad_rows(int nsb) { return nsb >= 2 && nsb <= QUAD_STEP_SB && (nsb & (nsb - 1)) == 0; }
        int moe_log2(int v)
        {
            int l = 0;
            while ((1 << l) < v)
                ++l;
            return l;
        }

        bool check_moe(const char *fn, uint8_t fmt, int n_tokens, int n_experts, int top_k, int hidden, int inter)
        {
            if (fmt != LLAM_FMT_Q4_K && fmt != LLAM_FMT_Q6_K && fmt != LLAM_FMT_IQ3_S)
                return fail(fn, "unsupported weight format id %d", (int)fmt);
            if (n_tokens < 1 || n_experts < 1 || top_k < 1)
                return fail(fn, "need n_tokens, n_experts, top_k >= 1 (%d, %d, %d)", n_tokens, n_experts, top_k);
            if (hidden < 256 || inter < 256 || (hidden % 256) != 0 || (inter % 256) != 0)
                return fail(fn, "hidden=%d and inter=%d must be positive multiples of 256", hidden, inter);
            if ((long)n_tokens * top_k > 65535 || n_tokens > 65535)
                return fail(fn, "too many token slots for one launch (%d x %d)", n_tokens, top_k);
            return true;
        }

        // Short expert rows with few slots: one launch whose loads for all slots are in
        // flight together; otherwise the slot-by-slot kernel.
        template <class F>
        bool moe_down_launch(const char *fn, const MoEArgs &m, dim3 grid, dim3 block, hipStream_t st)
        {
            const int nsb = m.inter / 256;
            if (nsb <= 8 && m.top_k <= 12)
            {
                const int S = m.top_k <= 4 ? 4 : (m.top_k <= 8 ? 8 : 12);
                const size_t lds = (size_t)m.top_k * nsb * GEMV_LDS_PER_SB;
                if (lds + F::TABLE_BYTES <= 64 * 1024)
                {
                    if (S == 4)
                        hipLaunchKernelGGL((moe_down_multi_kernel<F, 4>), grid, block, lds, st, m);
                    else if (S == 8)
                        hipLaunchKernelGGL((moe_down_multi_kernel<F, 8>), grid, block, lds, st, m);
                    else
                        hipLaunchKernelGGL((moe_down_multi_kernel<F, 12>), grid, block, lds, st, m);
                    return launched(fn);
                }
            }
            const size_t lds = gemv_lds_bytes<F>(1, nsb);
            if (lds + F::TABLE_BYTES > 64 * 1024)
                return fail(fn, "inter=%d too large for one LDS stage", m.inter);
            hipLaunchKernelGGL((moe_down_kernel<F>), grid, block, lds, st, m);
            return launched(fn);
        }
    } // namespace
} // namespace llamql

extern "C" bool llam_ql_moe_router_logits(const float *d_hidden, const float *d_gate_w, float *d_logits,
                                          int n_tokens, int d_model, int n_experts, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_router_logits";
    if (n_tokens < 0 || d_model < 1 || n_experts < 1)
        return fail(fn, "bad size (n_tokens=%d d_model=%d n_experts=%d)", n_tokens, d_model, n_experts);
    if (n_tokens == 0)
        return true;
    if ((d_model % 4) != 0)
        return fail(fn, "d_model=%d must be a multiple of 4", d_model);
    if (!d_hidden || !d_gate_w || !d_logits)
        return fail(fn, "null pointer");
    if (!aligned16(d_hidden) || !aligned16(d_gate_w) || !aligned4(d_logits))
        return fail(fn, "d_hidden and d_gate_w must be 16-byte aligned");
    if (n_tokens > 65535)
        return fail(fn, "too many tokens for one launch");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(moe_router_logits_kernel, dim3((unsigned)((n_experts + 3) / 4), (unsigned)n_tokens), dim3(256),
                       0, as_stream(stream), d_hidden, d_gate_w, d_logits, d_model, n_experts);
    return launched(fn);
}

namespace llamql
{
    namespace
    {
        bool moe_route_run(const char *fn, const float *d_logits, int n_tokens, int n_experts, int top_k,
                           int normalize, int32_t *d_ids, float *d_weights, int slot_stride, const float *d_x,
                           void *d_q8, long q_blocks, int device_id, void *stream)
        {
            if (n_tokens < 0)
                return fail(fn, "negative n_tokens");
            if (n_tokens == 0)
                return true;
            if (n_experts < 1 || n_experts > WAVE * ROUTE_MAX_PER_LANE)
                return fail(fn, "n_experts=%d outside 1..%d", n_experts, WAVE * ROUTE_MAX_PER_LANE);
            if (top_k < 1 || top_k > n_experts || top_k > 64)
                return fail(fn, "top_k=%d outside 1..min(n_experts,64)", top_k);
            if (slot_stride < top_k)
                return fail(fn, "slot_stride=%d smaller than top_k=%d", slot_stride, top_k);
            if (!d_logits || !d_ids || !d_weights)
                return fail(fn, "null pointer");
            if (!set_device(fn, device_id))
                return false;
            const long q_wgs = (q_blocks * 8 + WAVE - 1) / WAVE;
            if ((long)n_tokens + q_wgs > 0x7FFFFFFFl)
                return fail(fn, "too much work for one launch");
            const dim3 grid((unsigned)(n_tokens + q_wgs)), block(WAVE);
            hipStream_t st = as_stream(stream);
            const float4 *qx = reinterpret_cast<const float4 *>(d_x);
            uint32_t *qo = static_cast<uint32_t *>(d_q8);
            const int per = (n_experts + WAVE - 1) / WAVE;
            if (per <= 4)
                hipLaunchKernelGGL((moe_route_kernel<4>), grid, block, 0, st, d_logits, n_tokens, n_experts, top_k,
                                   normalize, d_ids, d_weights, slot_stride, qx, qo, q_blocks);
            else if (per <= 8)
                hipLaunchKernelGGL((moe_route_kernel<8>), grid, block, 0, st, d_logits, n_tokens, n_experts, top_k,
                                   normalize, d_ids, d_weights, slot_stride, qx, qo, q_blocks);
            else if (per <= 16)
                hipLaunchKernelGGL((moe_route_kernel<16>), grid, block, 0, st, d_logits, n_tokens, n_experts, top_k,
                                   normalize, d_ids, d_weights, slot_stride, qx, qo, q_blocks);
            else
                hipLaunchKernelGGL((moe_route_kernel<32>), grid, block, 0, st, d_logits, n_tokens, n_experts, top_k,
                                   normalize, d_ids, d_weights, slot_stride, qx, qo, q_blocks);
            return launched(fn);
        }
        // ---- the quad-lane kernels on expert rows of 2, 4, 8 or 16 super-blocks, any format with such a decoder ----
        template <class F>
        bool moe_quad_ok(int rows, int nsb)
        {
            return moe_quad_rows(nsb) && F::Quad::addressable(rows, nsb);
        }

        // gate/up as fp32 rows: steps per wavefront so that a compute unit sees a few workgroups, each long
        // enough to be worth its staging
        template <class F>
        bool moe_gate_up_quad_launch(const char *fn, MoEArgs m, int n_tokens, int device_id, hipStream_t st)
        {
            typedef typename F::Quad Q;
            const int nsb = m.hidden / 256;
            const long steps = ((long)m.inter * nsb + QUAD_STEP_SB - 1) / QUAD_STEP_SB;
            const long all_steps = steps * n_tokens * m.top_k * 2;
            int spw = 2;
            while (spw < 8 && all_steps / ((long)cu_count(device_id) * MOE_QUAD_WAVES * 2) >= 2 * spw)
                spw *= 2;
            m.rows_per_wave = spw;
            m.gshift = moe_log2(nsb);
            const long gx = (steps + (long)MOE_QUAD_WAVES * spw - 1) / ((long)MOE_QUAD_WAVES * spw);
            const dim3 grid((unsigned)gx, (unsigned)(n_tokens * m.top_k), 2);
            hipLaunchKernelGGL((moe_gate_up_quad_kernel<Q>), grid, dim3(MOE_QUAD_WAVES * WAVE),
                               (size_t)nsb * QUAD_SB_LDS, st, m);
            return launched(fn);
        }

        // gate/up + SwiGLU + Q8_1 in one launch; rt: with the router and the hidden state's quantiser inside
        template <class F>
        bool moe_gate_up_swiglu_launch(const char *fn, MoEArgs m, uint32_t *q8_out, int n_tokens, int device_id,
                                       hipStream_t st, const MoERouteArgs *rt = nullptr)
        {
            typedef typename F::Quad Q;
            const int nsb = m.hidden / 256;
            m.gshift = moe_log2(nsb);
            m.rows_per_wave = 0;
            const dim3 grid((unsigned)(m.inter / 32), (unsigned)(n_tokens * m.top_k)), block(MOE_QUAD_WAVES * WAVE);
            const size_t lds = (size_t)nsb * QUAD_SB_LDS + 2 * 32 * sizeof(float);
            if (rt)
            {
                if ((rt->n_route + WAVE - 1) / WAVE <= 4)
                    hipLaunchKernelGGL((moe_route_gate_up_swiglu_kernel<Q, 4, 4>), grid, block, lds, st, m, q8_out, *rt);
                else
                    hipLaunchKernelGGL((moe_route_gate_up_swiglu_kernel<Q, 4, 8>), grid, block, lds, st, m, q8_out, *rt);
            }
            else if ((long)grid.x * grid.y >= 4L * cu_count(device_id))
                hipLaunchKernelGGL((moe_gate_up_swiglu_dense_kernel<Q>), grid, block, lds, st, m, q8_out);
            else
                hipLaunchKernelGGL((moe_gate_up_swiglu_kernel<Q>), grid, block, lds, st, m, q8_out);
            return launched(fn);
        }

        // down projection: 1 launched, 0 failed, -1 this format and shape have no quad-lane launch
        template <class F>
        int moe_down_quad_launch(const char *fn, MoEArgs m, int n_tokens, int device_id, hipStream_t st)
        {
            typedef typename F::Quad Q;
            const int nsb = m.inter / 256, top_k = m.top_k;
            if (!(moe_quad_ok<F>(m.hidden, nsb) && top_k <= MOE_QUAD_MAX_SLOTS &&
                  (size_t)top_k * nsb * QUAD_SB_LDS + Q::STATIC_LDS + 4096 <= 64 * 1024))
                return -1;
            const long steps = ((long)m.hidden * nsb + QUAD_STEP_SB - 1) / QUAD_STEP_SB;
            m.gshift = moe_log2(nsb);
            // (with little work per compute unit the launch is a chain of memory round trips: there a wavefront
            // per slot has every slot's loads of a row range in flight at once; it loses from 8 tokens of the
            // 9-slot, 2-super-block shape on: 41.5 against 39.9 us per step)
            if ((long)m.hidden * nsb / QUAD_STEP_SB * n_tokens * top_k < 48L * cu_count(device_id))
            {
                int spw = 1;
                while (spw < MOE_SLOTWAVE_MAX_STEPS && steps * n_tokens / (2L * cu_count(device_id)) >= 2 * spw)
                    spw *= 2;
                m.rows_per_wave = spw;
                const long gx = (steps + spw - 1) / spw;
                const size_t lds = (size_t)top_k * nsb * QUAD_SB_LDS + (size_t)top_k * spw * (QUAD_STEP_SB / nsb) * sizeof(float);
                // a wavefront per slot, and enough threads to fetch the decode tables a piece each
                const int waves = top_k * WAVE >= Q::TABLE_THREADS ? top_k : (Q::TABLE_THREADS + WAVE - 1) / WAVE;
                hipLaunchKernelGGL((moe_down_slotwave_kernel<Q>), dim3((unsigned)gx, (unsigned)n_tokens), dim3(waves * WAVE),
                                   lds, st, m);
                return launched(fn) ? 1 : 0;
            }
            // workgroups of a step or more per wavefront, at least two of them per compute unit
            int spw = 1;
            while (spw < 8 && steps * n_tokens / ((long)cu_count(device_id) * MOE_QUAD_WAVES * 2) >= 2 * spw)
                spw *= 2;
            m.rows_per_wave = spw;
            const long gx = (steps + (long)MOE_QUAD_WAVES * spw - 1) / ((long)MOE_QUAD_WAVES * spw);
            hipLaunchKernelGGL((moe_down_quad_kernel<Q>), dim3((unsigned)gx, (unsigned)n_tokens), dim3(MOE_QUAD_WAVES * WAVE),
                               (size_t)top_k * nsb * QUAD_SB_LDS, st, m);
            return launched(fn) ? 1 : 0;
        }
    } // namespace
} // namespace llamql

extern "C" bool llam_ql_moe_route_ex(const float *d_logits, int n_tokens, int n_experts,
                                     int top_k, int normalize, int32_t *d_ids,
                                     float *d_weights, int slot_stride, int device_id, void *stream)
{
    return llamql::moe_route_run("llam_ql_moe_route", d_logits, n_tokens, n_experts, top_k, normalize, d_ids, d_weights,
                                 slot_stride, nullptr, nullptr, 0, device_id, stream);
}

extern "C" bool llam_ql_moe_route_quantize(const float *d_logits, int n_tokens, int n_experts, int top_k,
                                           int normalize, int32_t *d_ids, float *d_weights, int slot_stride,
                                           const float *d_hidden, int d_model, void *d_q8, int device_id,
                                           void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_route_quantize";
    if (d_model < 32 || (d_model % 32) != 0)
        return fail(fn, "d_model=%d must be a positive multiple of 32", d_model);
    if (n_tokens > 0 && (!d_hidden || !d_q8))
        return fail(fn, "null pointer");
    if (n_tokens > 0 && (!aligned16(d_hidden) || !aligned4(d_q8)))
        return fail(fn, "d_hidden must be 16-byte aligned, d_q8 4-byte aligned");
    return moe_route_run(fn, d_logits, n_tokens, n_experts, top_k, normalize, d_ids, d_weights, slot_stride, d_hidden,
                         d_q8, (long)(n_tokens > 0 ? n_tokens : 0) * (d_model / 32), device_id, stream);
}

extern "C" bool llam_ql_moe_route(const float *d_logits, int n_tokens, int n_experts,
                                  int top_k, int normalize, int32_t *d_ids,
                                  float *d_weights, int device_id, void *stream)
{
    return llam_ql_moe_route_ex(d_logits, n_tokens, n_experts, top_k, normalize, d_ids, d_weights, top_k, device_id,
                                stream);
}

extern "C" bool llam_ql_moe_gate_up(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                    const int32_t *d_ids, const void *d_q8,
                                    float *d_gate_out, float *d_up_out, int n_tokens,
                                    int top_k, int hidden, int inter, int device_id,
                                    void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_gate_up";
    if (!check_moe(fn, fmt, n_tokens, n_experts, top_k, hidden, inter))
        return false;
    if (!d_experts || !d_ids || !d_q8 || !d_gate_out || !d_up_out)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    MoEArgs m;
    m.experts = d_experts;
    m.ids = d_ids;
    m.weights = nullptr;
    m.q8 = static_cast<const uint32_t *>(d_q8);
    m.out0 = d_gate_out;
    m.out1 = d_up_out;
    m.n_experts = n_experts;
    m.top_k = top_k;
    m.hidden = hidden;
    m.inter = inter;
    m.accumulate = 0;
    hipStream_t st = as_stream(stream);
    switch (fmt) // the quad-lane decoder on short rows
    {
    case LLAM_FMT_Q4_K:
        if (moe_quad_ok<Q4KTraits>(inter, hidden / 256))
            return moe_gate_up_quad_launch<Q4KTraits>(fn, m, n_tokens, device_id, st);
        break;
    case LLAM_FMT_Q6_K:
        if (moe_quad_ok<Q6KTraits>(inter, hidden / 256))
            return moe_gate_up_quad_launch<Q6KTraits>(fn, m, n_tokens, device_id, st);
        break;
    default:
        if (moe_quad_ok<IQ3STraits>(inter, hidden / 256))
            return moe_gate_up_quad_launch<IQ3STraits>(fn, m, n_tokens, device_id, st);
        break;
    }
    long gx;
    moe_shape(inter, hidden / 256, (long)n_tokens * top_k * 2, device_id, m.gshift, m.rows_per_wave, gx);
    const dim3 grid((unsigned)gx, (unsigned)(n_tokens * top_k), 2);
    const dim3 block(GEMV_WAVES * WAVE);
    switch (fmt)
    {
    case LLAM_FMT_Q4_K:
    {
        const size_t lds = gemv_lds_bytes<Q4KTraits>(1, hidden / 256);
        if (lds + Q4KTraits::TABLE_BYTES > 64 * 1024)
            return fail(fn, "hidden=%d too large for one LDS stage", hidden);
        hipLaunchKernelGGL((moe_gate_up_kernel<Q4KTraits>), grid, block, lds, st, m);
        break;
    }
    case LLAM_FMT_Q6_K:
    {
        const size_t lds = gemv_lds_bytes<Q6KTraits>(1, hidden / 256);
        if (lds + Q6KTraits::TABLE_BYTES > 64 * 1024)
            return fail(fn, "hidden=%d too large for one LDS stage", hidden);
        hipLaunchKernelGGL((moe_gate_up_kernel<Q6KTraits>), grid, block, lds, st, m);
        break;
    }
    default:
    {
        const size_t lds = gemv_lds_bytes<IQ3STraits>(1, hidden / 256);
        if (lds + IQ3STraits::TABLE_BYTES > 64 * 1024)
            return fail(fn, "hidden=%d too large for one LDS stage", hidden);
        hipLaunchKernelGGL((moe_gate_up_kernel<IQ3STraits>), grid, block, lds, st, m);
        break;
    }
    }
    return launched(fn);
}

extern "C" bool llam_ql_moe_gate_up_swiglu(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                           const int32_t *d_ids, const void *d_q8, float *d_gate_scratch,
                                           float *d_up_scratch, void *d_q8_out, int n_tokens, int top_k, int hidden,
                                           int inter, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_gate_up_swiglu";
    if (!check_moe(fn, fmt, n_tokens, n_experts, top_k, hidden, inter))
        return false;
    if (!d_experts || !d_ids || !d_q8 || !d_q8_out)
        return fail(fn, "null pointer");
    if (!aligned4(d_q8_out))
        return fail(fn, "d_q8_out must be 4-byte aligned");
    const bool one_launch = fmt == LLAM_FMT_Q4_K   ? moe_quad_ok<Q4KTraits>(inter, hidden / 256)
                            : fmt == LLAM_FMT_Q6_K ? moe_quad_ok<Q6KTraits>(inter, hidden / 256)
                                                   : moe_quad_ok<IQ3STraits>(inter, hidden / 256);
    if (one_launch) // (inter is a multiple of 256: whole Q8_1 blocks per workgroup)
    {
        if (!set_device(fn, device_id))
            return false;
        MoEArgs m;
        m.experts = d_experts;
        m.ids = d_ids;
        m.weights = nullptr;
        m.q8 = static_cast<const uint32_t *>(d_q8);
        m.out0 = nullptr;
        m.out1 = nullptr;
        m.n_experts = n_experts;
        m.top_k = top_k;
        m.hidden = hidden;
        m.inter = inter;
        m.accumulate = 0;
        uint32_t *out = static_cast<uint32_t *>(d_q8_out);
        hipStream_t st = as_stream(stream);
        switch (fmt)
        {
        case LLAM_FMT_Q4_K: return moe_gate_up_swiglu_launch<Q4KTraits>(fn, m, out, n_tokens, device_id, st);
        case LLAM_FMT_Q6_K: return moe_gate_up_swiglu_launch<Q6KTraits>(fn, m, out, n_tokens, device_id, st);
        default: return moe_gate_up_swiglu_launch<IQ3STraits>(fn, m, out, n_tokens, device_id, st);
        }
    }
    // other row lengths: the two launches, through the caller's fp32 scratch
    if (!d_gate_scratch || !d_up_scratch)
        return fail(fn, "this shape needs the fp32 scratch rows (d_gate_scratch, d_up_scratch)");
    if (!llam_ql_moe_gate_up(fmt, d_experts, n_experts, d_ids, d_q8, d_gate_scratch, d_up_scratch, n_tokens, top_k,
                             hidden, inter, device_id, stream))
        return false;
    return llam_ql_swiglu_quantize(d_gate_scratch, d_up_scratch, nullptr, d_q8_out, n_tokens * top_k, inter, device_id,
                                   stream);
}

extern "C" bool llam_ql_moe_route_gate_up_swiglu(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                                 const float *d_logits, int n_route_experts, int top_k, int normalize,
                                                 int32_t *d_ids, float *d_weights, int slot_stride,
                                                 const float *d_hidden, void *d_q8_hidden_scratch,
                                                 float *d_gate_scratch, float *d_up_scratch, void *d_q8_out,
                                                 int n_tokens, int hidden, int inter, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_route_gate_up_swiglu";
    if (!check_moe(fn, fmt, n_tokens, n_experts, slot_stride, hidden, inter))
        return false;
    if (!d_experts || !d_logits || !d_ids || !d_weights || !d_hidden || !d_q8_out)
        return fail(fn, "null pointer");
    if (n_route_experts < 1 || n_route_experts > n_experts)
        return fail(fn, "n_route_experts=%d outside 1..n_experts=%d", n_route_experts, n_experts);
    if (top_k < 1 || top_k > n_route_experts || top_k > 64 || top_k > slot_stride)
        return fail(fn, "top_k=%d outside 1..min(n_route_experts, 64, slot_stride=%d)", top_k, slot_stride);
    if (!aligned16(d_hidden) || !aligned4(d_q8_out))
        return fail(fn, "d_hidden must be 16-byte aligned, d_q8_out 4-byte aligned");
    const int per = (n_route_experts + WAVE - 1) / WAVE;
    // One launch while the step is a chain of latencies (fewer workgroups than two per compute unit: one or
    // two tokens of the 256-expert shape: 16.2 against 17.5 us per step at 1 token); with more work the
    // routing repeated by every workgroup costs more than the launch it saves (4 tokens 30.4 against 29.7 us,
    // 16 tokens 64.3 against 59.4-61.8 us).
    const bool few = (long)(inter / 32) * n_tokens * slot_stride < 2L * cu_count(device_id);
    const bool quad = fmt == LLAM_FMT_Q4_K   ? moe_quad_ok<Q4KTraits>(inter, hidden / 256)
                      : fmt == LLAM_FMT_Q6_K ? moe_quad_ok<Q6KTraits>(inter, hidden / 256)
                                             : moe_quad_ok<IQ3STraits>(inter, hidden / 256);
    if (quad && per <= 8 && few)
    {
        if (!set_device(fn, device_id))
            return false;
        MoEArgs m;
        m.experts = d_experts;
        m.ids = d_ids;
        m.weights = nullptr;
        m.q8 = nullptr;
        m.out0 = nullptr;
        m.out1 = nullptr;
        m.n_experts = n_experts;
        m.top_k = slot_stride;
        m.hidden = hidden;
        m.inter = inter;
        m.accumulate = 0;
        MoERouteArgs r;
        r.logits = d_logits;
        r.x = d_hidden;
        r.ids = d_ids;
        r.weights = d_weights;
        r.n_route = n_route_experts;
        r.top_k = top_k;
        r.normalize = normalize;
        hipStream_t st = as_stream(stream);
        uint32_t *out = static_cast<uint32_t *>(d_q8_out);
        switch (fmt)
        {
        case LLAM_FMT_Q4_K: return moe_gate_up_swiglu_launch<Q4KTraits>(fn, m, out, n_tokens, device_id, st, &r);
        case LLAM_FMT_Q6_K: return moe_gate_up_swiglu_launch<Q6KTraits>(fn, m, out, n_tokens, device_id, st, &r);
        default: return moe_gate_up_swiglu_launch<IQ3STraits>(fn, m, out, n_tokens, device_id, st, &r);
        }
    }
    // more tokens, other row lengths, more than 512 routed experts: the launches one by one
    if (!d_q8_hidden_scratch)
        return fail(fn, "this shape or token count needs the Q8_1 scratch of the hidden state (d_q8_hidden_scratch)");
    if (!llam_ql_moe_route_quantize(d_logits, n_tokens, n_route_experts, top_k, normalize, d_ids, d_weights, slot_stride,
                                    d_hidden, hidden, d_q8_hidden_scratch, device_id, stream))
        return false;
    return llam_ql_moe_gate_up_swiglu(fmt, d_experts, n_experts, d_ids, d_q8_hidden_scratch, d_gate_scratch, d_up_scratch,
                                      d_q8_out, n_tokens, slot_stride, hidden, inter, device_id, stream);
}

extern "C" size_t llam_ql_moe_group_bytes(int n_tokens, int slot_stride)
{
    if (n_tokens < 1 || slot_stride < 1)
        return 0;
    return llamql::moe_group_bytes(n_tokens * slot_stride);
}

extern "C" bool llam_ql_moe_group(const int32_t *d_ids, int n_tokens, int slot_stride, int n_experts, void *d_group,
                                  int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_group";
    if (n_tokens < 1 || slot_stride < 1 || n_experts < 1)
        return fail(fn, "need n_tokens, slot_stride, n_experts >= 1 (%d, %d, %d)", n_tokens, slot_stride, n_experts);
    const long P = (long)n_tokens * slot_stride;
    if (P > MOE_GROUP_MAX_PAIRS)
        return fail(fn, "%ld (token, slot) pairs: at most %d are grouped in one call", P, MOE_GROUP_MAX_PAIRS);
    if (!d_ids || !d_group)
        return fail(fn, "null pointer");
    if (!aligned16(d_group))
        return fail(fn, "d_group must be 16-byte aligned");
    if (!set_device(fn, device_id))
        return false;
    if (n_experts > MOE_GROUP_MAX_EXPERTS)
        return fail(fn, "n_experts=%d: at most %d experts are grouped", n_experts, MOE_GROUP_MAX_EXPERTS);
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(MOE_GROUP_THREADS), (size_t)((P + 3) & ~3L) * 4,
                       as_stream(stream), d_ids, (int)P, n_experts, d_group);
    return launched(fn);
}

namespace llamql
{
    namespace
    {
        template <class Q, bool DOWN>
        void moe_grouped_quad_launch_m(bool four, dim3 grid, size_t lds, hipStream_t st, const MoEArgs &m, void *ws, int P)
        {
            if (four)
                hipLaunchKernelGGL((moe_grouped_quad_kernel<Q, 4, DOWN>), grid, dim3(MOE_QUAD_WAVES * WAVE), lds, st, m, ws, P);
            else
                hipLaunchKernelGGL((moe_grouped_quad_kernel<Q, 2, DOWN>), grid, dim3(MOE_QUAD_WAVES * WAVE), lds, st, m, ws, P);
        }

        template <class F>
        bool moe_grouped_launch(const char *fn, bool down, const MoEArgs &m_in, void *ws, int P, dim3 grid, int device_id,
                                hipStream_t st)
        {
            const MoEArgs &m = m_in;
            {
                // expert rows of 2, 4, 8 or 16 super-blocks: the quad-lane decoder, every step decoded once per chunk
                const int rows = down ? m.hidden : m.inter, nsbq = (down ? m.inter : m.hidden) / 256;
                if (moe_quad_ok<F>(rows, nsbq))
                {
                    typedef typename F::Quad Q;
                    MoEArgs q = m;
                    const long steps = ((long)rows * nsbq + QUAD_STEP_SB - 1) / QUAD_STEP_SB;
                    // about the chunks there are: two pairs a chunk below 512 pairs, four from there on
                    const long chunks = (P + moe_chunk_size(P) - 1) / moe_chunk_size(P) + (P >= 64 ? P / 8 : P / 2);
                    const long all_steps = steps * chunks * (down ? 1 : 2);
                    int spw = 1;
                    while (spw < 8 && all_steps / ((long)cu_count(device_id) * MOE_QUAD_WAVES * 2) >= 2 * spw)
                        spw *= 2;
                    q.rows_per_wave = spw;
                    q.gshift = moe_log2(nsbq);
                    const long gx = (steps + (long)MOE_QUAD_WAVES * spw - 1) / ((long)MOE_QUAD_WAVES * spw);
                    const bool four = moe_chunk_size(P) > 2;
                    const size_t lds = (size_t)(four ? 4 : 2) * nsbq * QUAD_SB_LDS;
                    const dim3 qgrid((unsigned)gx, grid.y, down ? 1 : 2);
                    if (down)
                        moe_grouped_quad_launch_m<Q, true>(four, qgrid, lds, st, q, ws, P);
                    else
                        moe_grouped_quad_launch_m<Q, false>(four, qgrid, lds, st, q, ws, P);
                    return launched(fn);
                }
            }
            const int nsb = (down ? m.inter : m.hidden) / 256;
            const size_t lds = gemv_lds_bytes<F>(4, nsb);
            if (lds + F::TABLE_BYTES > 64 * 1024)
                return fail(fn, "%s=%d too large for one LDS stage of four tokens", down ? "inter" : "hidden",
                            down ? m.inter : m.hidden);
            const dim3 block(GEMV_WAVES * WAVE);
            const bool four = moe_chunk_size(P) > 2; // the chunk size llam_ql_moe_group used for P pairs
            if (down && four)
                hipLaunchKernelGGL((moe_down_grouped_kernel<F, 4>), grid, block, lds, st, m, ws, P);
            else if (down)
                hipLaunchKernelGGL((moe_down_grouped_kernel<F, 2>), grid, block, lds, st, m, ws, P);
            else if (four)
                hipLaunchKernelGGL((moe_gate_up_grouped_kernel<F, 4>), grid, block, lds, st, m, ws, P);
            else
                hipLaunchKernelGGL((moe_gate_up_grouped_kernel<F, 2>), grid, block, lds, st, m, ws, P);
            return launched(fn);
        }
    } // namespace
} // namespace llamql

extern "C" bool llam_ql_moe_gate_up_grouped(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                            const void *d_group, const void *d_q8, float *d_gate_out,
                                            float *d_up_out, int n_tokens, int slot_stride, int hidden, int inter,
                                            int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_gate_up_grouped";
    if (!check_moe(fn, fmt, n_tokens, n_experts, slot_stride, hidden, inter))
        return false;
    const long P = (long)n_tokens * slot_stride;
    if (P > MOE_GROUP_MAX_PAIRS)
        return fail(fn, "%ld (token, slot) pairs: at most %d are grouped", P, MOE_GROUP_MAX_PAIRS);
    if (!d_experts || !d_group || !d_q8 || !d_gate_out || !d_up_out)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    MoEArgs m;
    m.experts = d_experts;
    m.ids = nullptr;
    m.weights = nullptr;
    m.q8 = static_cast<const uint32_t *>(d_q8);
    m.out0 = d_gate_out;
    m.out1 = d_up_out;
    m.n_experts = n_experts;
    m.top_k = slot_stride;
    m.hidden = hidden;
    m.inter = inter;
    m.accumulate = 0;
    long gx;
    moe_shape(inter, hidden / 256, P * 2, device_id, m.gshift, m.rows_per_wave, gx);
    const dim3 grid((unsigned)gx, (unsigned)P, 2); // one chunk per workgroup row; P bounds their number
    void *ws = const_cast<void *>(d_group);
    hipStream_t st = as_stream(stream);
    switch (fmt)
    {
    case LLAM_FMT_Q4_K: return moe_grouped_launch<Q4KTraits>(fn, false, m, ws, (int)P, grid, device_id, st);
    case LLAM_FMT_Q6_K: return moe_grouped_launch<Q6KTraits>(fn, false, m, ws, (int)P, grid, device_id, st);
    default: return moe_grouped_launch<IQ3STraits>(fn, false, m, ws, (int)P, grid, device_id, st);
    }
}

extern "C" bool llam_ql_moe_down_grouped(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                         const void *d_group, const int32_t *d_ids, const float *d_weights,
                                         const void *d_q8_act, float *d_pair_out, float *d_out, int n_tokens,
                                         int slot_stride, int hidden, int inter, int accumulate, int device_id,
                                         void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_down_grouped";
    if (!check_moe(fn, fmt, n_tokens, n_experts, slot_stride, hidden, inter))
        return false;
    const long P = (long)n_tokens * slot_stride;
    if (P > MOE_GROUP_MAX_PAIRS)
        return fail(fn, "%ld (token, slot) pairs: at most %d are grouped", P, MOE_GROUP_MAX_PAIRS);
    if (!d_experts || !d_group || !d_ids || !d_weights || !d_q8_act || !d_pair_out || !d_out)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    MoEArgs m;
    m.experts = d_experts;
    m.ids = d_ids;
    m.weights = d_weights;
    m.q8 = static_cast<const uint32_t *>(d_q8_act);
    m.out0 = d_out;
    m.out1 = d_pair_out;
    m.n_experts = n_experts;
    m.top_k = slot_stride;
    m.hidden = hidden;
    m.inter = inter;
    m.accumulate = accumulate;
    long gx;
    moe_shape(hidden, inter / 256, P, device_id, m.gshift, m.rows_per_wave, gx);
    const dim3 grid((unsigned)gx, (unsigned)P);
    void *ws = const_cast<void *>(d_group);
    hipStream_t st = as_stream(stream);
    bool ok;
    switch (fmt)
    {
    case LLAM_FMT_Q4_K: ok = moe_grouped_launch<Q4KTraits>(fn, true, m, ws, (int)P, grid, device_id, st); break;
    case LLAM_FMT_Q6_K: ok = moe_grouped_launch<Q6KTraits>(fn, true, m, ws, (int)P, grid, device_id, st); break;
    default: ok = moe_grouped_launch<IQ3STraits>(fn, true, m, ws, (int)P, grid, device_id, st); break;
    }
    if (!ok)
        return false;
    hipLaunchKernelGGL(moe_pair_reduce_kernel, dim3((unsigned)((hidden + 255) / 256), (unsigned)n_tokens), dim3(256), 0,
                       st, d_pair_out, d_ids, d_weights, d_experts, n_experts, d_out, slot_stride, hidden, accumulate);
    return launched(fn);
}

extern "C" bool llam_ql_swiglu_quantize(const float *d_gate, const float *d_up,
                                        float *d_act_out, void *d_q8_out, int rows,
                                        int inter, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_swiglu_quantize";
    if (rows < 0 || inter < 0)
        return fail(fn, "negative size");
    if (rows == 0 || inter == 0)
        return true;
    if ((inter % 32) != 0)
        return fail(fn, "inter=%d must be a multiple of 32", inter);
    if (!d_gate || !d_up || !d_q8_out)
        return fail(fn, "null pointer");
    if (!aligned16(d_gate) || !aligned16(d_up) || (d_act_out && !aligned16(d_act_out)) || !aligned4(d_q8_out))
        return fail(fn, "fp32 buffers must be 16-byte aligned, d_q8_out 4-byte aligned");
    if (!set_device(fn, device_id))
        return false;
    const long n_blocks = (long)rows * (inter / 32);
    const long grid = (n_blocks * 8 + 255) / 256;
    hipLaunchKernelGGL(swiglu_quantize_kernel, dim3((unsigned)grid), dim3(256), 0, as_stream(stream),
                       reinterpret_cast<const float4 *>(d_gate), reinterpret_cast<const float4 *>(d_up),
                       reinterpret_cast<float4 *>(d_act_out), static_cast<uint32_t *>(d_q8_out), n_blocks);
    return launched(fn);
}

extern "C" bool llam_ql_moe_down(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                 const int32_t *d_ids, const float *d_weights,
                                 const void *d_q8_act, float *d_out, int n_tokens,
                                 int top_k, int hidden, int inter, int accumulate,
                                 int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_down";
    if (!check_moe(fn, fmt, n_tokens, n_experts, top_k, hidden, inter))
        return false;
    if (!d_experts || !d_ids || !d_weights || !d_q8_act || !d_out)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    MoEArgs m;
    m.experts = d_experts;
    m.ids = d_ids;
    m.weights = d_weights;
    m.q8 = static_cast<const uint32_t *>(d_q8_act);
    m.out0 = d_out;
    m.out1 = nullptr;
    m.n_experts = n_experts;
    m.top_k = top_k;
    m.hidden = hidden;
    m.inter = inter;
    m.accumulate = accumulate;
    hipStream_t st = as_stream(stream);
    {
        const int r = fmt == LLAM_FMT_Q4_K   ? moe_down_quad_launch<Q4KTraits>(fn, m, n_tokens, device_id, st)
                      : fmt == LLAM_FMT_Q6_K ? moe_down_quad_launch<Q6KTraits>(fn, m, n_tokens, device_id, st)
                                             : moe_down_quad_launch<IQ3STraits>(fn, m, n_tokens, device_id, st);
        if (r >= 0)
            return r == 1;
    }
    long gx;
    moe_shape(hidden, inter / 256, (long)n_tokens, device_id, m.gshift, m.rows_per_wave, gx);
    const dim3 grid((unsigned)gx, (unsigned)n_tokens);
    const dim3 block(GEMV_WAVES * WAVE);
    switch (fmt)
    {
    case LLAM_FMT_Q4_K: return moe_down_launch<Q4KTraits>(fn, m, grid, block, st);
    case LLAM_FMT_Q6_K: return moe_down_launch<Q6KTraits>(fn, m, grid, block, st);
    default: return moe_down_launch<IQ3STraits>(fn, m, grid, block, st);
    }
}

extern "C" bool llam_ql_moe_ids_from_f32(const float *d_indices, int32_t *d_ids, int n, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_ids_from_f32";
    if (n < 0)
        return fail(fn, "negative count");
    if (n == 0)
        return true;
    if (!d_indices || !d_ids)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(moe_ids_from_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream),
                       d_indices, d_ids, n);
    return launched(fn);
}

extern "C" bool llam_ql_moe_publish_routing(const int32_t *d_ids, const float *d_weights, int n_tokens, int top_k,
                                            int slot_stride, float *d_indices_f32, float *d_weights_f32,
                                            uint64_t *d_histogram, int n_experts, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_publish_routing";
    if (n_tokens < 0 || top_k < 0 || slot_stride < top_k)
        return fail(fn, "bad sizes: n_tokens=%d top_k=%d slot_stride=%d", n_tokens, top_k, slot_stride);
    if (n_tokens == 0 || top_k == 0 || (!d_indices_f32 && !d_weights_f32 && !d_histogram))
        return true;
    if (!d_ids || (d_weights_f32 && !d_weights))
        return fail(fn, "null pointer");
    if (d_histogram && n_experts <= 0)
        return fail(fn, "a histogram needs n_experts > 0");
    if ((long)n_tokens * top_k > (1L << 30))
        return fail(fn, "too many (token, slot) pairs");
    if (!set_device(fn, device_id))
        return false;
    const int n = n_tokens * top_k;
    hipLaunchKernelGGL(moe_publish_routing_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream),
                       d_ids, d_weights, n_tokens, top_k, slot_stride, d_indices_f32, d_weights_f32,
                       reinterpret_cast<unsigned long long *>(d_histogram), n_experts);
    return launched(fn);
}

extern "C" bool llam_ql_shared_expert_add(float *d_out, const float *d_shared,
                                          const float *d_hidden, const float *d_gate_inp,
                                          int n_tokens, int d_model, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_shared_expert_add";
    if (n_tokens < 0 || d_model < 0)
        return fail(fn, "negative size");
    if (n_tokens == 0 || d_model == 0)
        return true;
    if (!d_out || !d_shared || (d_gate_inp && !d_hidden))
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(shared_expert_add_kernel, dim3((unsigned)n_tokens), dim3(256), 0, as_stream(stream),
                       d_out, d_shared, d_hidden, d_gate_inp, d_model);
    return launched(fn);
}

extern "C" bool llam_ql_shared_expert_gate(float *d_shared, const float *d_hidden, const float *d_gate_inp,
                                           int n_tokens, int d_model, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_shared_expert_gate";
    if (n_tokens < 0 || d_model < 0)
        return fail(fn, "negative size");
    if (n_tokens == 0 || d_model == 0)
        return true;
    if (!d_shared || !d_hidden || !d_gate_inp)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(shared_expert_gate_kernel, dim3((unsigned)n_tokens), dim3(256), 0, as_stream(stream), d_shared,
                       d_hidden, d_gate_inp, d_model);
    return launched(fn);
}

extern "C" bool llam_ql_moe_gather_rows(const float *d_hidden, float *d_batch, const int32_t *d_token_indices,
                                        int num_tokens, int n_rows, int d_model, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_gather_rows";
    if (num_tokens < 0 || n_rows < 0 || d_model < 0)
        return fail(fn, "negative size");
    if (num_tokens == 0 || d_model == 0)
        return true;
    if (!d_hidden || !d_batch || !d_token_indices)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(moe_gather_rows_kernel, dim3((unsigned)num_tokens), dim3(256), 0, as_stream(stream), d_hidden,
                       d_batch, d_token_indices, n_rows, d_model);
    return launched(fn);
}

extern "C" bool llam_ql_moe_scatter_add_weighted(float *d_output, const float *d_expert_output,
                                                 const int32_t *d_token_indices, const float *d_weights,
                                                 int num_tokens, int n_rows, int d_model, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_scatter_add_weighted";
    if (num_tokens < 0 || n_rows < 0 || d_model < 0)
        return fail(fn, "negative size");
    if (num_tokens == 0 || d_model == 0)
        return true;
    if (!d_output || !d_expert_output || !d_token_indices || !d_weights)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(moe_scatter_add_weighted_kernel, dim3((unsigned)((d_model + 255) / 256)), dim3(256), 0,
                       as_stream(stream), d_output, d_expert_output, d_token_indices, d_weights, num_tokens, n_rows,
                       d_model);
    return launched(fn);
}

extern "C" bool llam_ql_swiglu_inplace(float *d_gate, const float *d_up, long count, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_swiglu_inplace";
    if (count < 0)
        return fail(fn, "negative size");
    if (count == 0)
        return true;
    if (!d_gate || !d_up)
        return fail(fn, "null pointer");
    if (!aligned16(d_gate) || !aligned16(d_up))
        return fail(fn, "d_gate and d_up must be 16-byte aligned");
    if (!set_device(fn, device_id))
        return false;
    const long n4 = count / 4, work = n4 + (count - 4 * n4);
    const long grid = (work + 255) / 256;
    if (grid > 0x7FFFFFFFL)
        return fail(fn, "count too large for one launch");
    hipLaunchKernelGGL(swiglu_inplace_kernel, dim3((unsigned)grid), dim3(256), 0, as_stream(stream), d_gate, d_up, n4,
                       count);
    return launched(fn);
}
