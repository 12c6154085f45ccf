// Prefill GEMM for gfx950: GGUF block-quantized weights x Q8_1 activations on
// int8 MFMA with int32 accumulation per 32-column block and fp32 rescale.
//
//   C[m,n] = sum_kb float(idot[m,n,kb]) * (f32(a.d[m,kb]) * b_scale[n,kb])
//          + sum_kb (float(a.sum[m,kb]) * f32(a.d[m,kb])) * b_min[n,kb]
//
// idot is formed by ONE v_mfma_i32_32x32x32_i8 per 32x32 output tile and K-block
// (K depth 32 = exactly one Q8_1 block, zero accumulator input), so it is the
// same exact integer the reference forms with vpdpbusd
// (CPUNativeVNNIGemv.h:1046-1231); the per-block rescale is fp32 VALU work and
// the rank-1 min term goes through v_mfma_f32_32x32x2f32 into its own
// accumulator.
//
// Workgroup: 512 threads = 8 wavefronts, tile 128 tokens x 128 weight rows,
// K advanced one 256-column super-block at a time.  Per step the weights of the
// tile are decoded (nibble unpack / requantise, shared with the GEMV traits)
// into LDS as int8 [row][k], the activations copied beside them, both with a
// 272-byte row stride (conflict-free ds_read_b128 for MFMA operands).  Wavefront
// w owns weight rows 32*(w%4).. and tokens 64*(w/4)..: two 32x32 MFMA tiles that
// share the weight operand.  The MFMA's A operand is the activation tile, B the
// weight tile, so a lane holds one weight row n and 16 tokens: stores of C are
// 128-byte coalesced and b_scale is one register per block.
#include "gemv_traits_all.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    typedef float v16f __attribute__((ext_vector_type(16)));

    constexpr int GEMM_BM = 128;        // tokens per workgroup
    constexpr int GEMM_BN = 128;        // weight rows per workgroup
    constexpr int GEMM_THREADS = 512;
    constexpr int GEMM_STRIDE = 256 + 16; // bytes per LDS row (one super-block + pad)

    struct GemmArgs
    {
        GemvArgs w;         // only w.w, w.N, w.SB are used (weight addressing)
        const uint32_t *q8; // [M][K/32] blocks as dwords
        float *y;
        int M, ldy;
    };

    template <class F>
    constexpr size_t gemm_lds_bytes()
    {
        return (size_t)(GEMM_BM + GEMM_BN) * GEMM_STRIDE + (size_t)4 * 8 * 128 * sizeof(float) + F::TABLE_BYTES;
    }

    template <class F>
    __global__ void __launch_bounds__(GEMM_THREADS) gemm_kernel(const GemmArgs g)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        uint8_t *Al = smem;                             // [BM][STRIDE] activations int8
        uint8_t *Wl = Al + GEMM_BM * GEMM_STRIDE;       // [BN][STRIDE] weights int8
        float *ad = reinterpret_cast<float *>(Wl + GEMM_BN * GEMM_STRIDE); // [8][BM]
        float *asd = ad + 8 * GEMM_BM;                  // [8][BM]
        float *bs = asd + 8 * GEMM_BM;                  // [8][BN]
        float *bm = bs + 8 * GEMM_BN;                   // [8][BN]
        void *tab = bm + 8 * GEMM_BN;

        if (F::TABLE_BYTES > 0)
            F::stage_tables(tab);

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int ntile = wave & 3;
        const int mhalf = wave >> 2;
        const int l32 = lane & 31;
        const int lh = lane >> 5;

        const long n0 = (long)blockIdx.x * GEMM_BN;
        const long m0 = (long)blockIdx.y * GEMM_BM;
        const int KB = g.w.SB * 8;

        v16f acc[2], accmin[2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                acc[t][r] = 0.0f;
                accmin[t][r] = 0.0f;
            }

        for (int sb = 0; sb < g.w.SB; ++sb)
        {
            __syncthreads(); // previous step's LDS reads (and the table staging) are done

            // ---- weights: 128 rows x 8 lanes each -> int8 + scales -------------------
#pragma unroll
            for (int it = 0; it < (GEMM_BN * 8) / GEMM_THREADS; ++it)
            {
                const int task = tid + it * GEMM_THREADS;
                const int row = task >> 3;
                const int c = task & 7;
                long n = n0 + row;
                if (n >= g.w.N)
                    n = g.w.N - 1; // tail rows: decode a valid row, never stored
                const typename F::Raw raw = F::load(g.w, n, sb, c);
                v4i w0, w1;
                int j;
                float bscale, bmin;
                F::decode(raw, c, w0, w1, j, bscale, bmin, tab);
                int j0, e0, j1, e1;
                F::where(c, j0, e0, j1, e1);
                *reinterpret_cast<v4i *>(Wl + row * GEMM_STRIDE + 32 * j0 + e0) = w0;
                *reinterpret_cast<v4i *>(Wl + row * GEMM_STRIDE + 32 * j1 + e1) = w1;
                bs[j * GEMM_BN + row] = bscale;
                bm[j * GEMM_BN + row] = bmin;
            }

            // ---- activations: 128 tokens x 8 blocks x 9 dwords ------------------------
#pragma unroll
            for (int it = 0; it < (GEMM_BM * 72) / GEMM_THREADS; ++it)
            {
                const int i = tid + it * GEMM_THREADS;
                const int m = i / 72;
                const int rem = i - m * 72;
                const int kb = rem / 9;
                const int r = rem - kb * 9;
                uint32_t v = 0;
                if (m0 + m < g.M)
                    v = g.q8[((size_t)(m0 + m) * KB + (size_t)sb * 8 + kb) * 9 + r];
                if (r == 0)
                {
                    const float d = h2f((uint16_t)(v & 0xFFFFu));
                    ad[kb * GEMM_BM + m] = d;
                    asd[kb * GEMM_BM + m] = (float)(int16_t)(v >> 16) * d;
                }
                else
                {
                    *reinterpret_cast<uint32_t *>(Al + m * GEMM_STRIDE + kb * 32 + (r - 1) * 4) = v;
                }
            }
            __syncthreads();

            // ---- multiply ------------------------------------------------------------------
            const uint8_t *wrow = Wl + (ntile * 32 + l32) * GEMM_STRIDE + lh * 16;
            const uint8_t *arow = Al + (mhalf * 64 + l32) * GEMM_STRIDE + lh * 16;
#pragma unroll
            for (int kb = 0; kb < 8; ++kb)
            {
                const v4i bw = *reinterpret_cast<const v4i *>(wrow + kb * 32);
                const float bscale = bs[kb * GEMM_BN + ntile * 32 + l32];
#pragma unroll
                for (int t = 0; t < 2; ++t)
                {
                    const v4i aa = *reinterpret_cast<const v4i *>(arow + t * 32 * GEMM_STRIDE + kb * 32);
                    v16i zero;
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        zero[r] = 0;
                    const v16i idot = __builtin_amdgcn_mfma_i32_32x32x32_i8(aa, bw, zero, 0, 0, 0);
                    const float *adp = ad + kb * GEMM_BM + mhalf * 64 + t * 32 + 4 * lh;
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                    {
                        const float4 a4 = *reinterpret_cast<const float4 *>(adp + 8 * q);
                        acc[t][4 * q + 0] = fmaf((float)idot[4 * q + 0], a4.x * bscale, acc[t][4 * q + 0]);
                        acc[t][4 * q + 1] = fmaf((float)idot[4 * q + 1], a4.y * bscale, acc[t][4 * q + 1]);
                        acc[t][4 * q + 2] = fmaf((float)idot[4 * q + 2], a4.z * bscale, acc[t][4 * q + 2]);
                        acc[t][4 * q + 3] = fmaf((float)idot[4 * q + 3], a4.w * bscale, acc[t][4 * q + 3]);
                    }
                }
                if (F::HAS_MIN && (kb & 1))
                {
                    // rank-2 update over blocks kb-1, kb: lane half lh supplies block kb-1+lh
                    const int kk = kb - 1 + lh;
                    const float bmin = bm[kk * GEMM_BN + ntile * 32 + l32];
#pragma unroll
                    for (int t = 0; t < 2; ++t)
                    {
                        const float av = asd[kk * GEMM_BM + mhalf * 64 + t * 32 + l32];
                        accmin[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bmin, accmin[t], 0, 0, 0);
                    }
                }
            }
        }

        // ---- store: lane holds weight row n, 16 tokens per tile --------------------------
        const long n = n0 + ntile * 32 + l32;
        if (n < g.w.N)
        {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    const long m = m0 + mhalf * 64 + t * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                    if (m < g.M)
                        g.y[(size_t)m * g.ldy + n] = F::HAS_MIN ? (acc[t][r] + accmin[t][r]) : acc[t][r];
                }
        }
    }

    __global__ void __launch_bounds__(256)
        epilogue_kernel(float *__restrict__ c, const float *__restrict__ t, const float *__restrict__ bias,
                        long M, int N, int ldc, float alpha, float beta)
    {
        const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
        if (i >= M * N)
            return;
        const long m = i / N;
        const int n = (int)(i - m * N);
        float *dst = c + m * ldc + n;
        float v = (beta == 0.0f) ? 0.0f : beta * *dst;
        v += alpha * t[i];
        if (bias)
            v += bias[n];
        *dst = v;
    }

    template <class F>
    bool gemm_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int M, int N, int K, int ldy,
                     hipStream_t st)
    {
        GemmArgs g;
        g.w = GemvArgs{};
        g.w.w = d_w;
        g.w.N = N;
        g.w.SB = K / 256;
        g.q8 = static_cast<const uint32_t *>(d_q8);
        g.y = d_y;
        g.M = M;
        g.ldy = ldy;
        constexpr size_t lds = gemm_lds_bytes<F>();
        static bool attr_set = false;
        if (!attr_set)
        {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kernel<F>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess)
                return fail(fn, "cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
            attr_set = true;
        }
        const dim3 grid((unsigned)((N + GEMM_BN - 1) / GEMM_BN), (unsigned)((M + GEMM_BM - 1) / GEMM_BM));
        hipLaunchKernelGGL((gemm_kernel<F>), grid, dim3(GEMM_THREADS), lds, st, g);
        return launched(fn);
    }
} // namespace llamql

extern "C" bool llam_ql_gemm(uint8_t fmt, const void *d_w, const void *d_q8, float *d_y,
                             int M, int N, int K, int ldy, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemm";
    if (fmt != LLAM_FMT_Q4_K && fmt != LLAM_FMT_Q6_K && fmt != LLAM_FMT_IQ3_S)
        return fail(fn, "unsupported weight format id %d", (int)fmt);
    if (M < 0)
        return fail(fn, "negative M");
    if (M == 0)
        return true;
    if (N < 1 || K < 1 || (K % 256) != 0)
        return fail(fn, "need N >= 1 and K a positive multiple of 256 (N=%d K=%d)", N, K);
    if (!d_w || !d_q8 || !d_y)
        return fail(fn, "null pointer");
    if (!aligned16(d_w) || !aligned4(d_q8))
        return fail(fn, "d_w must be 16-byte and d_q8 4-byte aligned");
    if (ldy < N)
        return fail(fn, "ldy=%d smaller than N=%d", ldy, N);
    if ((M + GEMM_BM - 1) / GEMM_BM > 65535)
        return fail(fn, "M=%d too large for one launch", M);
    if (!set_device(fn, device_id))
        return false;
    hipStream_t st = as_stream(stream);
    switch (fmt)
    {
    case LLAM_FMT_Q4_K: return gemm_launch<Q4KTraits>(fn, d_w, d_q8, d_y, M, N, K, ldy, st);
    case LLAM_FMT_Q6_K: return gemm_launch<Q6KTraits>(fn, d_w, d_q8, d_y, M, N, K, ldy, st);
    default: return gemm_launch<IQ3STraits>(fn, d_w, d_q8, d_y, M, N, K, ldy, st);
    }
}

extern "C" bool llam_ql_epilogue(float *d_c, const float *d_t, const float *d_bias, int M,
                                 int N, int ldc, float alpha, float beta, int device_id,
                                 void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_epilogue";
    if (M < 0 || N < 0)
        return fail(fn, "negative size");
    if (M == 0 || N == 0)
        return true;
    if (!d_c || !d_t)
        return fail(fn, "null pointer");
    if (ldc < N)
        return fail(fn, "ldc=%d smaller than N=%d", ldc, N);
    if (!set_device(fn, device_id))
        return false;
    const long total = (long)M * N;
    const long grid = (total + 255) / 256;
    if (grid > 0x7FFFFFFFL)
        return fail(fn, "problem too large");
    hipLaunchKernelGGL(epilogue_kernel, dim3((unsigned)grid), dim3(256), 0, as_stream(stream), d_c, d_t, d_bias,
                       (long)M, N, ldc, alpha, beta);
    return launched(fn);
}
