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
    // One workgroup (256 threads) per token.  Softmax as the reference computes it
    // (kernels/cpu/primitives/SoftmaxPrimitivesImpl.h:584-693): max, sum of
    // exp(l-max) in double, p = exp(l-max) * float(1/sum); then top_k rounds of
    // arg-max (ties -> lower expert id) and optional renormalisation over the top_k.
    constexpr int ROUTE_THREADS = 256;
    constexpr int ROUTE_MAX_PER_THREAD = 8; // up to 2048 experts

    __global__ void __launch_bounds__(ROUTE_THREADS)
        moe_route_kernel(const float *__restrict__ logits, int n_experts, int top_k, int normalize,
                         int32_t *__restrict__ ids, float *__restrict__ weights)
    {
        __shared__ float s_f[ROUTE_THREADS];
        __shared__ double s_d[ROUTE_THREADS];
        __shared__ int s_i[ROUTE_THREADS];
        __shared__ float s_top[64];

        const int t = blockIdx.x;
        const int tid = threadIdx.x;
        const float *l = logits + (size_t)t * n_experts;

        float p[ROUTE_MAX_PER_THREAD];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_THREAD; ++i)
        {
            const int e = tid + i * ROUTE_THREADS;
            p[i] = (e < n_experts) ? l[e] : -INFINITY;
            mx = fmaxf(mx, p[i]);
        }
        s_f[tid] = mx;
        __syncthreads();
        for (int off = ROUTE_THREADS / 2; off > 0; off >>= 1)
        {
            if (tid < off)
                s_f[tid] = fmaxf(s_f[tid], s_f[tid + off]);
            __syncthreads();
        }
        mx = s_f[0];
        if (!isfinite(mx))
            mx = 0.0f;
        __syncthreads();

        double sum = 0.0;
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_THREAD; ++i)
        {
            const int e = tid + i * ROUTE_THREADS;
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
        s_d[tid] = sum;
        __syncthreads();
        for (int off = ROUTE_THREADS / 2; off > 0; off >>= 1)
        {
            if (tid < off)
                s_d[tid] += s_d[tid + off];
            __syncthreads();
        }
        sum = s_d[0];
        if (sum <= 0.0)
            sum = 1.0;
        const float inv = (float)(1.0 / sum);
#pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_THREAD; ++i)
            if (p[i] >= 0.0f)
                p[i] = p[i] * inv;
        __syncthreads();

        for (int k = 0; k < top_k; ++k)
        {
            float best = -1.0f;
            int best_e = 0x7FFFFFFF;
#pragma unroll
            for (int i = 0; i < ROUTE_MAX_PER_THREAD; ++i)
            {
                const int e = tid + i * ROUTE_THREADS;
                if (p[i] > best) // ascending e within a thread: first maximum wins
                {
                    best = p[i];
                    best_e = e;
                }
            }
            s_f[tid] = best;
            s_i[tid] = best_e;
            __syncthreads();
            for (int off = ROUTE_THREADS / 2; off > 0; off >>= 1)
            {
                if (tid < off)
                {
                    const float ov = s_f[tid + off];
                    const int oe = s_i[tid + off];
                    if (ov > s_f[tid] || (ov == s_f[tid] && oe < s_i[tid]))
                    {
                        s_f[tid] = ov;
                        s_i[tid] = oe;
                    }
                }
                __syncthreads();
            }
            const int win = s_i[0];
            const float winp = s_f[0];
            __syncthreads();
            if (tid == 0)
            {
                ids[(size_t)t * top_k + k] = win;
                s_top[k] = winp;
            }
            // retire the winner
#pragma unroll
            for (int i = 0; i < ROUTE_MAX_PER_THREAD; ++i)
                if (tid + i * ROUTE_THREADS == win)
                    p[i] = -1.0f;
        }
        __syncthreads();
        if (tid == 0)
        {
            float topk_sum = 0.0f;
            for (int k = 0; k < top_k; ++k)
                topk_sum += s_top[k];
            for (int k = 0; k < top_k; ++k)
                weights[(size_t)t * top_k + k] = normalize ? __fdiv_rn(s_top[k], topk_sum) : s_top[k];
        }
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
        gemv_body<F, 1, 1, false>(a, (long)blockIdx.x, lds);
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
            if (e < 0 || e >= m.n_experts)
                continue;
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
            gemv_body<F, 1, 1, false>(a, (long)blockIdx.x, lds);
            first = false;
            __syncthreads(); // LDS is restaged by the next slot
        }
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
        float4 v;
        v.x = __fdiv_rn(g.x, 1.0f + expf(-g.x)) * u.x;
        v.y = __fdiv_rn(g.y, 1.0f + expf(-g.y)) * u.y;
        v.z = __fdiv_rn(g.z, 1.0f + expf(-g.z)) * u.z;
        v.w = __fdiv_rn(g.w, 1.0f + expf(-g.w)) * u.w;
        if (act_out)
            act_out[lane_global] = v;

        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = fmaxf(amax, dpp_f32<DPP_QUAD_XOR1>(amax));
        amax = fmaxf(amax, dpp_f32<DPP_QUAD_XOR2>(amax));
        amax = fmaxf(amax, dpp_f32<DPP_ROW_HALF_MIRROR>(amax));
        uint32_t packed = 0, head = 0;
        if (amax >= 1e-10f)
        {
            const float d = __fdiv_rn(amax, 127.0f);
            const float id = __fdiv_rn(1.0f, d);
            int q0 = max(-128, min(127, (int)rintf(v.x * id)));
            int q1 = max(-128, min(127, (int)rintf(v.y * id)));
            int q2 = max(-128, min(127, (int)rintf(v.z * id)));
            int q3 = max(-128, min(127, (int)rintf(v.w * id)));
            int sum = q0 + q1 + q2 + q3;
            sum += dpp_i32<DPP_QUAD_XOR1>(sum);
            sum += dpp_i32<DPP_QUAD_XOR2>(sum);
            sum += dpp_i32<DPP_ROW_HALF_MIRROR>(sum);
            packed = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) |
                     ((uint32_t)(q2 & 0xFF) << 16) | ((uint32_t)(q3 & 0xFF) << 24);
            head = (uint32_t)__half_as_ushort(__float2half_rn(d)) | ((uint32_t)(sum & 0xFFFF) << 16);
        }
        uint32_t *dst = out + blk * 9;
        dst[1 + sub] = packed;
        if (sub == 0)
            dst[0] = head;
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

    namespace
    {
        void moe_shape(int N, int SB, int device_id, int &gshift, int &rpw, long &grid_x)
        {
            gshift = 3;
            while (gshift > 0 && (1 << (gshift - 1)) >= SB)
                --gshift;
            const int R = 8 >> gshift;
            rpw = 1;
            const int rows_per_wg = GEMV_WAVES * R * rpw;
            grid_x = ((long)N + rows_per_wg - 1) / rows_per_wg;
            (void)device_id;
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
    } // namespace
} // namespace llamql

extern "C" bool llam_ql_moe_route(const float *d_logits, int n_tokens, int n_experts,
                                  int top_k, int normalize, int32_t *d_ids,
                                  float *d_weights, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_moe_route";
    if (n_tokens < 0)
        return fail(fn, "negative n_tokens");
    if (n_tokens == 0)
        return true;
    if (n_experts < 1 || n_experts > ROUTE_THREADS * ROUTE_MAX_PER_THREAD)
        return fail(fn, "n_experts=%d outside 1..%d", n_experts, ROUTE_THREADS * ROUTE_MAX_PER_THREAD);
    if (top_k < 1 || top_k > n_experts || top_k > 64)
        return fail(fn, "top_k=%d outside 1..min(n_experts,64)", top_k);
    if (!d_logits || !d_ids || !d_weights)
        return fail(fn, "null pointer");
    if (!set_device(fn, device_id))
        return false;
    hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)n_tokens), dim3(ROUTE_THREADS), 0, as_stream(stream),
                       d_logits, n_experts, top_k, normalize, d_ids, d_weights);
    return launched(fn);
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
    long gx;
    moe_shape(inter, hidden / 256, device_id, m.gshift, m.rows_per_wave, gx);
    const dim3 grid((unsigned)gx, (unsigned)(n_tokens * top_k), 2);
    const dim3 block(GEMV_WAVES * WAVE);
    hipStream_t st = as_stream(stream);
    switch (fmt)
    {
    case LLAM_FMT_Q4_K:
    {
        const size_t lds = gemv_lds_bytes<Q4KTraits>(1, hidden / 256);
        if (lds > 64 * 1024)
            return fail(fn, "hidden=%d too large for one LDS stage", hidden);
        hipLaunchKernelGGL((moe_gate_up_kernel<Q4KTraits>), grid, block, lds, st, m);
        break;
    }
    case LLAM_FMT_Q6_K:
    {
        const size_t lds = gemv_lds_bytes<Q6KTraits>(1, hidden / 256);
        if (lds > 64 * 1024)
            return fail(fn, "hidden=%d too large for one LDS stage", hidden);
        hipLaunchKernelGGL((moe_gate_up_kernel<Q6KTraits>), grid, block, lds, st, m);
        break;
    }
    default:
    {
        const size_t lds = gemv_lds_bytes<IQ3STraits>(1, hidden / 256);
        if (lds > 64 * 1024)
            return fail(fn, "hidden=%d too large for one LDS stage", hidden);
        hipLaunchKernelGGL((moe_gate_up_kernel<IQ3STraits>), grid, block, lds, st, m);
        break;
    }
    }
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
    long gx;
    moe_shape(hidden, inter / 256, device_id, m.gshift, m.rows_per_wave, gx);
    const dim3 grid((unsigned)gx, (unsigned)n_tokens);
    const dim3 block(GEMV_WAVES * WAVE);
    hipStream_t st = as_stream(stream);
    switch (fmt)
    {
    case LLAM_FMT_Q4_K:
    {
        const size_t lds = gemv_lds_bytes<Q4KTraits>(1, inter / 256);
        if (lds > 64 * 1024)
            return fail(fn, "inter=%d too large for one LDS stage", inter);
        hipLaunchKernelGGL((moe_down_kernel<Q4KTraits>), grid, block, lds, st, m);
        break;
    }
    case LLAM_FMT_Q6_K:
    {
        const size_t lds = gemv_lds_bytes<Q6KTraits>(1, inter / 256);
        if (lds > 64 * 1024)
            return fail(fn, "inter=%d too large for one LDS stage", inter);
        hipLaunchKernelGGL((moe_down_kernel<Q6KTraits>), grid, block, lds, st, m);
        break;
    }
    default:
    {
        const size_t lds = gemv_lds_bytes<IQ3STraits>(1, inter / 256);
        if (lds > 64 * 1024)
            return fail(fn, "inter=%d too large for one LDS stage", inter);
        hipLaunchKernelGGL((moe_down_kernel<IQ3STraits>), grid, block, lds, st, m);
        break;
    }
    }
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
