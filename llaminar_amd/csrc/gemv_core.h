// Decode-GEMV skeleton shared by the weight formats (gfx950, M = 1..8).
//
// One wavefront owns one output row at a time; 8 lanes own one 256-element
// super-block and a wavefront therefore walks 8 super-blocks per iteration with
// the next iteration's loads already in flight.  Lane c of a group decodes 32
// weight values into two 16-byte int8 vectors (w0, w1):
//
//   PAIR formats (Q4_K, Q6_K): w0 / w1 are the lane's 16 elements of two
//     different 32-element sub-blocks; lanes c and c^1 hold the two halves of
//     the same two sub-blocks and swap one partial through DPP, so each lane
//     finishes ONE sub-block's exact int32 dot.
//   whole-block formats (IQ3_S): w0, w1 are the two halves of sub-block c.
//
// Either way a lane ends with `idot`, the exact per-32-block integer sum the
// reference forms (CPUNativeVNNIGemv.h:417-487, :560-640), and applies
//   acc = fma(float(idot), f32(a.d)*b_scale, acc) ; acc = fma(float(a.sum)*f32(a.d), b_min, acc)
// with the block's fp16-rounded effective scale/min.  The 64 per-lane partial
// sums of a row are added in a fixed order (deterministic).
//
// Activations (Q8_1) are staged once per workgroup in LDS in 32-byte units laid
// out so unit (s, c) is exactly what lane c needs for super-block s (two
// ds_read_b128), plus f32(d) and float(sum_qs)*f32(d) per block.
//
// A format supplies a traits struct F:
//   static constexpr bool PAIR, HAS_MIN;
//   struct Raw;                                   registers loaded per lane
//   static void unit_of(int j, int q, int &c, int &p)   LDS slot of dword q of block j
//   static Raw  load(const GemvArgs&, long row, int sb, int c)
//   static void decode(const Raw&, int c, v4i &w0, v4i &w1, int &j, float &bscale, float &bmin, const void *tab)
//   static constexpr int TABLE_BYTES; static void *tables_lds(); static void stage_tables(void *lds_tab)
#pragma once

#include "ql_device.h"
#include "ql_host.h"

namespace llamql
{
    constexpr int GEMV_WAVES = 4;             // wavefronts per workgroup
    constexpr int GEMV_LDS_PER_SB = 256 + 64; // int8 quants + 8 x (f32 d, f32 sum*d)

    struct GemvArgs
    {
        const void *w;      // prepared weights
        const uint32_t *q8; // Q8_1 activations as dwords (9 per block)
        float *y;
        int32_t *sums;      // DUMP only
        int ldy;
        int N;
        int SB;             // super-blocks per weight row
        int sb0, nsb;       // K slice handled by this launch
        int rows_per_wave;  // row batches one wavefront walks
        int gshift;         // log2(G): G = 8-lane groups that share one row (1,2,4,8)
        int accumulate;     // add onto y instead of overwriting
        float out_scale;    // y (+)= out_scale * (row dot); 1 for plain GEMV
        int row0, nrows;    // DUMP only: rows [row0,row0+nrows) of the matrix
        // Optional gather of the batch rows (MoE token groups): batch row m takes the activation
        // row pairs[m] / pair_div of q8 and writes output row pairs[m] of y.  Null: row m both.
        const int32_t *pairs;
        int pair_div;
    };

    // The format's decode tables (IQ3_S: codebook, maps, sign masks) live in STATIC LDS: their
    // address is a link-time constant, so every table look-up is a ds_read with an immediate
    // offset instead of an address addition.  Null for formats without tables.
    template <class F>
    __device__ __forceinline__ void *format_tables_lds()
    {
        return F::tables_lds();
    }

    // Stage `nkb` Q8_1 blocks of each of M activation rows into LDS.
    template <class F, int M>
    __device__ __forceinline__ void stage_q8(const uint32_t *__restrict__ q8, int KB_total, int kb0, int nkb,
                                             uint32_t *aq, float *ad, float *asd, const int32_t *pairs = nullptr,
                                             int pair_div = 1)
    {
        const int ndw = nkb * 9;
        constexpr int U = 8; // loads in flight per thread
        for (int m = 0; m < M; ++m)
        {
            const size_t arow = pairs ? (size_t)(pairs[m] / pair_div) : (size_t)m;
            const uint32_t *src = q8 + (arow * KB_total + kb0) * 9;
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
                        int c, p;
                        F::unit_of(kb & 7, r - 1, c, p);
                        aq[m * nkb * 8 + (((kb >> 3) * 8 + c) * 8 + p * 4 + ((r - 1) & 3))] = v[u];
                    }
                }
            }
        }
    }

    // Sum over the 8*G lanes that share a row (G = 1,2,4,8 groups of 8 lanes);
    // every lane of the segment returns the segment total.  Fixed order.
    __device__ __forceinline__ float segment_sum(float v, int gshift)
    {
        v += dpp_f32<DPP_QUAD_XOR1>(v);
        v += dpp_f32<DPP_QUAD_XOR2>(v);
        v += dpp_f32<DPP_ROW_HALF_MIRROR>(v);
        if (gshift >= 1)
            v += dpp_f32<DPP_ROW_MIRROR>(v);
        if (gshift >= 2)
        {
            const int lane = threadIdx.x & (WAVE - 1);
            const int b = __float_as_int(v);
            const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
            const float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
            const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
            const float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
            if (gshift == 2)
                v = (lane < 32) ? (r0 + r1) : (r2 + r3);
            else
                v = (r0 + r1) + (r2 + r3);
        }
        return v;
    }

    // The workgroup-level GEMV: workgroup `wg` of the launch described by `a`.
    // Requires blockDim.x == GEMV_WAVES*WAVE and the dynamic LDS of gemv_lds_bytes().
    //
    // U = iterations (8 super-blocks each, or G when rows are short) whose loads are
    // issued together; the next chunk -- of this row or of the wavefront's next row --
    // is already in flight while the current one is decoded, so a wavefront keeps
    // 2*U global loads per lane outstanding.
    template <class F, int M, int U, bool DUMP>
    __device__ __forceinline__ void gemv_body(const GemvArgs &a, long wg, uint32_t *lds)
    {
        const int nkb = a.nsb * 8;
        uint32_t *aq = lds;                                      // M * nkb * 8 dwords
        float *ad = reinterpret_cast<float *>(aq + M * nkb * 8); // M * nkb
        float *asd = ad + M * nkb;                               // M * nkb
        void *tab = format_tables_lds<F>();

        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = threadIdx.x >> 6;
        const int c = lane & 7;    // piece / sub-block slot owned by this lane
        const int grp = lane >> 3; // 8-lane group
        const bool odd = (c & 1) != 0;
        const int G = 1 << a.gshift;          // groups per row
        const int R = 8 >> a.gshift;          // rows a wavefront handles at once
        const int rsub = grp >> a.gshift;     // which of those rows this lane is on
        const int s_first = grp & (G - 1);    // first super-block of this lane
        const int rows_per_wg = GEMV_WAVES * R * a.rows_per_wave;
        const long wg_row0 = wg * rows_per_wg;
        const int chunk_sb = G * U;                                // super-blocks per chunk and row
        const int nchunks = (a.nsb + chunk_sb - 1) / chunk_sb;

        // Issue the first chunk's weight loads before touching the activations, so HBM
        // latency overlaps the LDS staging.
        typename F::Raw buf[U];
        {
            const long row = wg_row0 + (long)wave * R + rsub;
#pragma unroll
            for (int u = 0; u < U; ++u)
            {
                const int s = s_first + u * G;
                buf[u] = typename F::Raw{};
                if (row < a.N && s < a.nsb)
                    buf[u] = F::load(a, row, a.sb0 + s, c);
            }
        }

        if (F::TABLE_BYTES > 0)
            F::stage_tables(tab);
        stage_q8<F, M>(a.q8, a.SB * 8, a.sb0 * 8, nkb, aq, ad, asd, a.pairs, a.pair_div);
        __syncthreads();

        for (int r = 0; r < a.rows_per_wave; ++r)
        {
            const long row_base = wg_row0 + ((long)r * GEMV_WAVES + wave) * R;
            if (row_base >= a.N)
                break;
            const long row = row_base + rsub;
            const bool row_ok = row < a.N;

            float acc[M];
#pragma unroll
            for (int m = 0; m < M; ++m)
                acc[m] = 0.0f;

            for (int ch = 0; ch < nchunks; ++ch)
            {
                typename F::Raw cur[U];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    cur[u] = buf[u];

                // prefetch the next chunk: same row, or the first chunk of the next row
                {
                    const bool same_row = (ch + 1 < nchunks);
                    const long nrow = same_row ? row : row + (long)GEMV_WAVES * R;
                    const int nch = same_row ? ch + 1 : 0;
                    const bool more = same_row || (r + 1 < a.rows_per_wave);
#pragma unroll
                    for (int u = 0; u < U; ++u)
                    {
                        const int s = s_first + (nch * U + u) * G;
                        if (more && nrow < a.N && s < a.nsb)
                            buf[u] = F::load(a, nrow, a.sb0 + s, c);
                    }
                }

#pragma unroll
                for (int u = 0; u < U; ++u)
                {
                    const int s = s_first + (ch * U + u) * G;
                    if (!row_ok || s >= a.nsb)
                        continue;
                    v4i w0, w1;
                    int j;
                    float bscale, bmin;
                    F::decode(cur[u], c, w0, w1, j, bscale, bmin, tab);

                    const int unit = s * 8 + c; // LDS unit of this lane
                    const int kb = s * 8 + j;   // block this lane finishes (slice-relative)
#pragma unroll
                    for (int m = 0; m < M; ++m)
                    {
                        const v4i *ap = reinterpret_cast<const v4i *>(aq + (size_t)m * nkb * 8 + (size_t)unit * 8);
                        const v4i a0 = ap[0];
                        const v4i a1 = ap[1];
                        int idot;
                        if (F::PAIR)
                        {
                            const int p0 = dot16(a0, w0, 0);
                            const int p1 = dot16(a1, w1, 0);
                            // even lane finishes the w0 sub-block, odd lane the w1 sub-block
                            const int got = dpp_i32<DPP_QUAD_XOR1>(odd ? p0 : p1);
                            idot = (odd ? p1 : p0) + got;
                        }
                        else
                        {
                            idot = dot16(a1, w1, dot16(a0, w0, 0));
                        }
                        if (DUMP)
                        {
                            const long rr = row - a.row0;
                            if (rr >= 0 && rr < a.nrows)
                                a.sums[((size_t)m * a.nrows + rr) * ((size_t)a.SB * 8) + (size_t)(a.sb0 + s) * 8 + j] = idot;
                        }
                        const float cs = ad[m * nkb + kb] * bscale;
                        acc[m] = fmaf((float)idot, cs, acc[m]);
                        if (F::HAS_MIN)
                            acc[m] = fmaf(asd[m * nkb + kb], bmin, acc[m]);
                    }
                }
            }

            if (!DUMP)
            {
#pragma unroll
                for (int m = 0; m < M; ++m)
                {
                    const float total = segment_sum(acc[m], a.gshift);
                    if (row_ok && (lane & (8 * G - 1)) == 0)
                    {
                        const size_t orow = a.pairs ? (size_t)a.pairs[m] : (size_t)m;
                        float *dst = a.y + orow * a.ldy + row;
                        const float v = weighted(a.out_scale, total);
                        *dst = a.accumulate ? add_rounded(*dst, v) : v;
                    }
                }
            }
        }
    }

    template <class F, int M, int U, bool DUMP>
    __global__ void __launch_bounds__(GEMV_WAVES *WAVE) gemv_kernel(const GemvArgs a)
    {
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        gemv_body<F, M, U, DUMP>(a, (long)blockIdx.x, lds);
    }

    // The generic kernel is only instantiated with U = 1: it serves short rows, the
    // block-sum dump and the MoE kernels; long rows go through gemv_fast.h.
    template <class F, int M>
    inline void gemv_launch_u(bool dump, dim3 grid, size_t lds, hipStream_t st, const GemvArgs &a)
    {
        dim3 block(GEMV_WAVES * WAVE);
        if (dump)
            hipLaunchKernelGGL((gemv_kernel<F, M, 1, true>), grid, block, lds, st, a);
        else
            hipLaunchKernelGGL((gemv_kernel<F, M, 1, false>), grid, block, lds, st, a);
    }

    // M is one of 1,2,3,4,8 (other batch sizes are split by the caller).
    template <class F>
    inline void gemv_launch_m(int M, bool dump, dim3 grid, size_t lds, hipStream_t st, const GemvArgs &a)
    {
        switch (M)
        {
        case 1: gemv_launch_u<F, 1>(dump, grid, lds, st, a); break;
        case 2: gemv_launch_u<F, 2>(dump, grid, lds, st, a); break;
        case 3: gemv_launch_u<F, 3>(dump, grid, lds, st, a); break;
        case 4: gemv_launch_u<F, 4>(dump, grid, lds, st, a); break;
        default: gemv_launch_u<F, 8>(dump, grid, lds, st, a); break;
        }
    }

    int gemv_rows_per_wave_override();

    template <class F>
    inline size_t gemv_lds_bytes(int M, int nsb)
    {
        return (size_t)M * nsb * GEMV_LDS_PER_SB; // dynamic part; F::TABLE_BYTES more are static
    }

} // namespace llamql
