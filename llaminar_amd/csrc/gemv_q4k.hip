// Q4_K x Q8_1 decode GEMV for gfx950 (M = 1..8 activation rows).
//
// Weights stay in GGUF layout: a row is K/256 super-blocks of 144 B = nine
// 16-byte pieces (piece 0: d, dmin, 12 packed scale bytes; pieces 1..8: 128
// nibble bytes).  One wavefront owns one output row at a time; 8 lanes own one
// super-block, lane c of the group loading nibble piece c (one
// global_load_dwordx4) plus the shared header piece.  Piece c = 2g+h holds
// elements 16h..16h+15 of sub-block 2g (low nibbles) and of sub-block 2g+1
// (high nibbles); the two lanes h=0/1 of a pair swap one partial through DPP so
// that lane c ends up with the complete int32 dot of sub-block c -- the exact
// per-block sum the reference forms (CPUNativeVNNIGemv.h:417-487) -- and applies
// that sub-block's fp16-rounded scale and min (Q4_KTensor.cpp:794-799).
//
// Activations are staged once per workgroup in LDS, re-laid so each lane's 32
// int8 are contiguous (two ds_read_b128), with f32(d) and float(sum_qs)*f32(d)
// beside them.  HBM-bound: 144 B per 256 weights.
#include "ql_device.h"
#include "ql_host.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    constexpr int Q4K_WAVES = 4;              // wavefronts per workgroup
    constexpr int Q4K_LDS_PER_SB = 256 + 64;  // int8 quants + 8 x (f32 d, f32 sum*d)

    struct GemvArgs
    {
        const void *w;      // prepared weights, row-major super-blocks
        const uint32_t *q8; // Q8_1 activations as dwords (9 per block)
        float *y;
        int32_t *sums;      // DUMP only
        int ldy;
        int N;
        int SB;             // super-blocks per weight row
        int sb0, nsb;       // K slice handled by this launch
        int rows_per_wave;
        int accumulate;     // add onto y instead of overwriting
        int row0, nrows;    // DUMP only: rows [row0,row0+nrows) of the matrix
    };

    // Stage `nsb` super-blocks worth of Q8_1 activations (M rows) into LDS.
    //   aq  [M][nsb*256] int8, permuted: 32-byte unit (s,c) = elements 16h..+15 of
    //       sub-block 2g followed by the same elements of sub-block 2g+1 (c = 2g+h)
    //   ad  [M][nsb*8] f32(d) ; asd [M][nsb*8] float(sum_qs)*f32(d)
    template <int M>
    __device__ __forceinline__ void stage_q8_q4k(const uint32_t *__restrict__ q8, int KB_total, int kb0, int nkb,
                                                 uint32_t *aq, float *ad, float *asd)
    {
        const int ndw = nkb * 9;
        constexpr int U = 8; // loads in flight per thread
        for (int m = 0; m < M; ++m)
        {
            const uint32_t *src = q8 + ((size_t)m * KB_total + kb0) * 9;
            for (int base = 0; base < ndw; base += U * (int)blockDim.x)
            {
                uint32_t v[U];
#pragma unroll
                for (int u = 0; u < U; ++u)
                {
                    const int i = base + u * (int)blockDim.x + (int)threadIdx.x;
                    v[u] = (i < ndw) ? src[i] : 0u;
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
                {
                    const int i = base + u * (int)blockDim.x + (int)threadIdx.x;
                    if (i >= ndw)
                        continue;
                    const int kb = i / 9;
                    const int r = i - kb * 9;
                    if (r == 0)
                    {
                        const float d = h2f((uint16_t)(v[u] & 0xFFFFu));
                        ad[m * nkb + kb] = d;
                        asd[m * nkb + kb] = (float)(int16_t)(v[u] >> 16) * d;
                    }
                    else
                    {
                        const int q = r - 1;          // dword q = elements 4q..4q+3
                        const int s = kb >> 3, j = kb & 7;
                        const int g = j >> 1, p = j & 1, h = q >> 2;
                        const int c = 2 * g + h;
                        aq[m * nkb * 8 + ((s * 8 + c) * 8 + p * 4 + (q & 3))] = v[u];
                    }
                }
            }
        }
    }

    template <int M, bool DUMP>
    __global__ void __launch_bounds__(Q4K_WAVES * WAVE)
        gemv_q4k_kernel(const GemvArgs a)
    {
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        const int nkb = a.nsb * 8;
        uint32_t *aq = lds;                                   // M * nkb * 8 dwords
        float *ad = reinterpret_cast<float *>(aq + M * nkb * 8); // M * nkb
        float *asd = ad + M * nkb;                            // M * nkb

        stage_q8_q4k<M>(a.q8, a.SB * 8, a.sb0 * 8, nkb, aq, ad, asd);
        __syncthreads();

        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = threadIdx.x >> 6;
        const int c = lane & 7;        // nibble piece / sub-block owned by this lane
        const int grp = lane >> 3;     // super-block slot inside an iteration
        const bool odd = (c & 1) != 0;
        const int rows_per_wg = Q4K_WAVES * a.rows_per_wave;
        const long wg_row0 = (long)blockIdx.x * rows_per_wg;

        for (int r = 0; r < a.rows_per_wave; ++r)
        {
            const long row = wg_row0 + (long)r * Q4K_WAVES + wave;
            if (row >= a.N)
                break;
            const uint4 *wrow = static_cast<const uint4 *>(a.w) + ((size_t)row * a.SB + a.sb0) * 9;

            float acc[M];
#pragma unroll
            for (int m = 0; m < M; ++m)
                acc[m] = 0.0f;

            int s = grp;
            uint4 qn = make_uint4(0, 0, 0, 0), hn = make_uint4(0, 0, 0, 0);
            if (s < a.nsb)
            {
                hn = wrow[(size_t)s * 9];
                qn = wrow[(size_t)s * 9 + 1 + c];
            }
            for (; s < a.nsb; s += 8)
            {
                const uint4 q = qn, hd = hn;
                const int sn = s + 8;
                if (sn < a.nsb)
                {
                    hn = wrow[(size_t)sn * 9];
                    qn = wrow[(size_t)sn * 9 + 1 + c];
                }

                v4i wlo, whi;
                wlo.x = (int)(q.x & 0x0F0F0F0Fu); whi.x = (int)((q.x >> 4) & 0x0F0F0F0Fu);
                wlo.y = (int)(q.y & 0x0F0F0F0Fu); whi.y = (int)((q.y >> 4) & 0x0F0F0F0Fu);
                wlo.z = (int)(q.z & 0x0F0F0F0Fu); whi.z = (int)((q.z >> 4) & 0x0F0F0F0Fu);
                wlo.w = (int)(q.w & 0x0F0F0F0Fu); whi.w = (int)((q.w >> 4) & 0x0F0F0F0Fu);

                uint32_t sc, mn;
                q4k_scale_min(c, hd.y, hd.z, hd.w, sc, mn);
                const float d = h2f((uint16_t)(hd.x & 0xFFFFu));
                const float dmin = h2f((uint16_t)(hd.x >> 16));
                const float bscale = f16_round_packer(d * (float)sc);
                const float bmin = f16_round_packer(-dmin * (float)mn);

                const int kb = s * 8 + c;
#pragma unroll
                for (int m = 0; m < M; ++m)
                {
                    const v4i *ap = reinterpret_cast<const v4i *>(aq + (size_t)m * nkb * 8 + (size_t)kb * 8);
                    const v4i alo = ap[0];
                    const v4i ahi = ap[1];
                    const int lo = dot16(alo, wlo, 0);
                    const int hi = dot16(ahi, whi, 0);
                    // even lane completes sub-block c (low nibbles), odd lane sub-block c (high nibbles)
                    const int give = odd ? lo : hi;
                    const int got = dpp_i32<DPP_QUAD_XOR1>(give);
                    const int idot = (odd ? hi : lo) + got;
                    if (DUMP)
                    {
                        const long rr = row - a.row0;
                        if (rr >= 0 && rr < a.nrows)
                            a.sums[((size_t)m * a.nrows + rr) * ((size_t)a.SB * 8) + (size_t)(a.sb0 + s) * 8 + c] = idot;
                    }
                    const float cs = ad[m * nkb + kb] * bscale;
                    acc[m] = fmaf((float)idot, cs, acc[m]);
                    acc[m] = fmaf(asd[m * nkb + kb], bmin, acc[m]);
                }
            }

            if (!DUMP)
            {
#pragma unroll
                for (int m = 0; m < M; ++m)
                {
                    const float total = wave_sum(acc[m]);
                    if (lane == 0)
                    {
                        float *dst = a.y + (size_t)m * a.ldy + row;
                        *dst = a.accumulate ? (*dst + total) : total;
                    }
                }
            }
        }
    }

    namespace
    {
        int g_rows_per_wave_override = 0;

        template <bool DUMP>
        void launch_m(int M, dim3 grid, size_t lds, hipStream_t st, const GemvArgs &a)
        {
            dim3 block(Q4K_WAVES * WAVE);
            switch (M)
            {
            case 1: hipLaunchKernelGGL((gemv_q4k_kernel<1, DUMP>), grid, block, lds, st, a); break;
            case 2: hipLaunchKernelGGL((gemv_q4k_kernel<2, DUMP>), grid, block, lds, st, a); break;
            case 3: hipLaunchKernelGGL((gemv_q4k_kernel<3, DUMP>), grid, block, lds, st, a); break;
            case 4: hipLaunchKernelGGL((gemv_q4k_kernel<4, DUMP>), grid, block, lds, st, a); break;
            case 5: hipLaunchKernelGGL((gemv_q4k_kernel<5, DUMP>), grid, block, lds, st, a); break;
            case 6: hipLaunchKernelGGL((gemv_q4k_kernel<6, DUMP>), grid, block, lds, st, a); break;
            case 7: hipLaunchKernelGGL((gemv_q4k_kernel<7, DUMP>), grid, block, lds, st, a); break;
            default: hipLaunchKernelGGL((gemv_q4k_kernel<8, DUMP>), grid, block, lds, st, a); break;
            }
        }
    } // namespace

    void q4k_set_rows_per_wave(int v) { g_rows_per_wave_override = v; }

    // Shared by llam_ql_gemv / llam_ql_gemv_block_sums.  Arguments are validated
    // by the callers; the device is current.
    bool q4k_gemv_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int32_t *d_sums,
                         int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st)
    {
        const int SB = K / 256;
        const bool dump = d_sums != nullptr;
        // K slices keep the staged activations within 64 KiB of LDS.
        int slice = (64 * 1024) / (M * Q4K_LDS_PER_SB);
        if (slice > SB)
            slice = SB;
        if (slice < 1)
            return fail(fn, "activation rows do not fit LDS (M=%d)", M);

        int rpw = g_rows_per_wave_override;
        if (rpw <= 0)
        {
            // enough workgroups for every CU several times over, but amortise the LDS staging
            const long target_wgs = (long)cu_count(device_id) * 8;
            rpw = (int)((long)N / (target_wgs * Q4K_WAVES));
            if (rpw < 1)
                rpw = 1;
            if (rpw > 8)
                rpw = 8;
        }
        const int rows_per_wg = Q4K_WAVES * rpw;
        const long grid = ((long)N + rows_per_wg - 1) / rows_per_wg;

        for (int sb0 = 0; sb0 < SB; sb0 += slice)
        {
            GemvArgs a;
            a.w = d_w;
            a.q8 = static_cast<const uint32_t *>(d_q8);
            a.y = d_y;
            a.sums = d_sums;
            a.ldy = ldy;
            a.N = N;
            a.SB = SB;
            a.sb0 = sb0;
            a.nsb = (SB - sb0 < slice) ? (SB - sb0) : slice;
            a.rows_per_wave = rpw;
            a.accumulate = sb0 > 0;
            a.row0 = row0;
            a.nrows = nrows;
            const size_t lds = (size_t)M * a.nsb * Q4K_LDS_PER_SB;
            if (dump)
                launch_m<true>(M, dim3((unsigned)grid), lds, st, a);
            else
                launch_m<false>(M, dim3((unsigned)grid), lds, st, a);
            if (!launched(fn))
                return false;
        }
        return true;
    }
} // namespace llamql
