// Row-streaming decode GEMV (gfx950): the kernel for the dense-layer shapes.
//
// Weight rows are contiguous runs of super-blocks, so RP consecutive rows form
// one run of RP*nsb super-blocks that a wavefront walks 8 at a time with every
// lane busy in every step:
//     RP = 1 when nsb % 8 == 0 (e.g. K = 8192: 32 super-blocks, 4 steps per row)
//     RP = 2 when nsb % 8 == 4 (e.g. K = 5120: 2 x 20 = 40 super-blocks, 5 steps;
//            K = 25600: 200 super-blocks, 25 steps) -- in the middle step lane
//            groups 0-3 finish row A while groups 4-7 start row B.
// A "pass" is those P = RP*nsb/8 steps.  Steps are issued in chunks of U loads per
// lane with two register buffers used alternately, so the next chunk (of this pass
// or of the wavefront's next pass) is always in flight while one is decoded, and
// no per-lane predicates or register copies remain in the loop.
//
// Arithmetic, lane roles, LDS layout and reduction order are those of
// gemv_core.h / gemv_fast.h; per lane the blocks of a row are still accumulated
// in ascending order, so results are bit-identical to the other GEMV kernels.
#pragma once

#include "gemv_fast.h"

namespace llamql
{
    template <class F, int M, int U, int RP>
    struct StreamCtx
    {
        typename F::Lane3 l3;
        const uint8_t *aq_lane;  // LDS: this lane's 32-byte unit of super-block 0
        const uint8_t *ads_lane; // LDS: {f32 d, sum*d} of this lane's block of super-block 0
        int m_stride_aq, m_stride_ads;
        int grp, nsb, P, mid;
        bool odd, low_half;
        const void *tab;
    };

    // Decode and accumulate one chunk (steps i0 .. i0+U-1 of a pass).
    template <class F, int M, int U, int RP>
    __device__ __forceinline__ void stream_chunk(const typename F::Raw (&buf)[U], const StreamCtx<F, M, U, RP> &cx,
                                                 int i0, float (&accA)[M], float (&accB)[M])
    {
#pragma unroll
        for (int u = 0; u < U; ++u)
        {
            const int i = i0 + u;
            if (i >= cx.P) // uniform: only the last chunk of a pass can be short
                break;
            v4i w0, w1;
            typename F::Scale S;
            F::decode3(buf[u], cx.l3, w0, w1, S, cx.tab);

            // super-block of this lane inside its row
            int s = i * 8 + cx.grp;
            if (RP == 2)
                s = (int)min((uint32_t)s, (uint32_t)(s - cx.nsb));
            const uint8_t *aql = cx.aq_lane + s * 256;
            const uint8_t *adl = cx.ads_lane + s * 64;
#pragma unroll
            for (int m = 0; m < M; ++m)
            {
                const v4i *ap = reinterpret_cast<const v4i *>(aql + m * cx.m_stride_aq);
                const v4i a0 = ap[0];
                const v4i a1 = ap[1];
                const float2 sd = *reinterpret_cast<const float2 *>(adl + m * cx.m_stride_ads);
                int idot;
                if (F::PAIR)
                {
                    const int p0 = dot16(a0, w0, 0);
                    const int p1 = dot16(a1, w1, 0);
                    const int got = dpp_i32<DPP_QUAD_XOR1>(cx.odd ? p0 : p1);
                    idot = (cx.odd ? p1 : p0) + got;
                }
                else
                {
                    idot = dot16(a1, w1, dot16(a0, w0, 0));
                }
                const float cs = F::cs(S, sd.x);
                if (RP == 1 || i < cx.mid)
                {
                    accA[m] = F::add_min(S, sd.y, fmaf((float)idot, cs, accA[m]));
                }
                else if (i > cx.mid)
                {
                    accB[m] = F::add_min(S, sd.y, fmaf((float)idot, cs, accB[m]));
                }
                else
                {
                    // middle step: lane groups 0-3 end row A, groups 4-7 begin row B
                    const float t = F::add_min(S, sd.y, fmaf((float)idot, cs, cx.low_half ? accA[m] : accB[m]));
                    accA[m] = cx.low_half ? t : accA[m];
                    accB[m] = cx.low_half ? accB[m] : t;
                }
            }
        }
    }

    template <class F, int M, int U, int RP>
    __global__ void __launch_bounds__(F::STREAM_MAX_THREADS) gemv_stream_kernel(const GemvArgs a)
    {
        const int NW = (int)(blockDim.x >> 6); // wavefronts in this workgroup (launch parameter)
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        const int nsb = a.nsb; // == a.SB: this kernel is only launched on whole rows
        const int nkb = nsb * 8;
        uint32_t *aq = lds;
        float2 *ads = reinterpret_cast<float2 *>(aq + M * nkb * 8);
        void *tab = ads + M * nkb;

        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = threadIdx.x >> 6;
        const int c = lane & 7;
        const int grp = lane >> 3;

        StreamCtx<F, M, U, RP> cx;
        cx.l3 = F::lane3_consts(c);
        cx.grp = grp;
        cx.nsb = nsb;
        cx.P = RP * nsb / 8;
        cx.mid = nsb / 8;
        cx.odd = (c & 1) != 0;
        cx.low_half = grp < 4;
        cx.tab = tab;
        cx.m_stride_aq = nkb * 32;
        cx.m_stride_ads = nkb * 8;
        cx.aq_lane = reinterpret_cast<const uint8_t *>(aq) + c * 32;
        cx.ads_lane = reinterpret_cast<const uint8_t *>(ads) + F::lane_consts(c).j * 8;

        const int NC = (cx.P + U - 1) / U;                 // chunks per pass
        const long npass = a.N / RP;
        const long pass0 = (long)blockIdx.x * (NW * a.rows_per_wave) + wave;
        // passes this wavefront owns: pass0, pass0+NW, ... (rows_per_wave of them at most)
        int my_passes = 0;
        if (pass0 < npass)
        {
            const long left = (npass - pass0 + NW - 1) / NW;
            my_passes = left < a.rows_per_wave ? (int)left : a.rows_per_wave;
        }
        const int total = my_passes * NC; // chunks this wavefront will process

        // Chunk g of the wavefront = chunk (g % NC) of its pass (g / NC).  The weight
        // pointer walks the run; between passes it skips the passes of the other wavefronts.
        typename F::Ptr p = F::ptr(a, (pass0 < npass ? pass0 : 0) * RP, grp, c);
        int ld_ch = 0; // chunk index (within its pass) of the next chunk to load
        auto load_chunk = [&](typename F::Raw(&buf)[U]) {
            const int i0 = ld_ch * U;
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (i0 + u < cx.P)
                    buf[u] = F::load_at(p, 8 * u);
            if (ld_ch + 1 < NC)
            {
                F::advance(p, 8 * U);
                ++ld_ch;
            }
            else
            {
                // to step 0 of this wavefront's next pass
                F::advance(p, NW * RP * nsb - 8 * U * ld_ch);
                ld_ch = 0;
            }
        };

        typename F::Raw bufA[U], bufB[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
        {
            bufA[u] = typename F::Raw{};
            bufB[u] = typename F::Raw{};
        }
        if (total > 0)
            load_chunk(bufA); // in flight while the activations are staged

        if (F::TABLE_BYTES > 0)
            F::stage_tables(tab);
        stage_q8_blocks<F, M>(a.q8, a.SB * 8, 0, nkb, aq, ads);
        __syncthreads();

        float accA[M], accB[M];
#pragma unroll
        for (int m = 0; m < M; ++m)
            accA[m] = accB[m] = 0.0f;
        int ch = 0;        // chunk (within its pass) being computed
        long pass = pass0; // pass being computed

        auto finish_chunk = [&]() {
            if (++ch < NC)
                return;
            ch = 0;
            // end of pass: reduce and store RP rows
#pragma unroll
            for (int m = 0; m < M; ++m)
            {
                const float ta = wave_sum(accA[m]);
                float tb = 0.0f;
                if (RP == 2)
                    tb = wave_sum(accB[m]);
                if (lane == 0)
                {
                    float *dst = a.y + (size_t)m * a.ldy + pass * RP;
                    dst[0] = a.accumulate ? (dst[0] + a.out_scale * ta) : a.out_scale * ta;
                    if (RP == 2)
                        dst[1] = a.accumulate ? (dst[1] + a.out_scale * tb) : a.out_scale * tb;
                }
                accA[m] = accB[m] = 0.0f;
            }
            pass += NW;
        };

        for (int g = 0; g < total; g += 2)
        {
            if (g + 1 < total)
                load_chunk(bufB);
            stream_chunk<F, M, U, RP>(bufA, cx, ch * U, accA, accB);
            finish_chunk();
            if (g + 1 >= total)
                break;
            if (g + 2 < total)
                load_chunk(bufA);
            stream_chunk<F, M, U, RP>(bufB, cx, ch * U, accA, accB);
            finish_chunk();
        }
    }

    template <class F, int M>
    inline void gemv_stream_launch_rp(int RP, int waves, dim3 grid, size_t lds, hipStream_t st, const GemvArgs &a)
    {
        dim3 block(waves * WAVE);
        if (RP == 2)
            hipLaunchKernelGGL((gemv_stream_kernel<F, M, F::STREAM_U_PAIR, 2>), grid, block, lds, st, a);
        else
            hipLaunchKernelGGL((gemv_stream_kernel<F, M, F::STREAM_U_SINGLE, 1>), grid, block, lds, st, a);
    }

    // M is 1 or 2 (larger batches use the chunked kernel).
    template <class F>
    inline void gemv_stream_launch(int M, int RP, int waves, dim3 grid, size_t lds, hipStream_t st, const GemvArgs &a)
    {
        if (M == 1)
            gemv_stream_launch_rp<F, 1>(RP, waves, grid, lds, st, a);
        else
            gemv_stream_launch_rp<F, 2>(RP, waves, grid, lds, st, a);
    }
} // namespace llamql
