// Prefill GEMM for gfx950: GGUF block-quantized weights x Q8_1 activations on
// int8 MFMA with int32 accumulation per 32-column block and fp32 rescale.
//
//   C[m,n] = sum_kb float(idot[m,n,kb]) * (f32(a.d[m,kb]) * b_scale[n,kb])
//          + sum_kb (float(a.sum[m,kb]) * f32(a.d[m,kb])) * b_min[n,kb]
//
// idot is formed by ONE v_mfma_i32_32x32x32_i8 per 32x32 output tile and K-block
// (K depth 32 = exactly one Q8_1 block, zero accumulator input), so it is the
// same exact integer the reference forms with vpdpbusd
// (CPUNativeVNNIGemv.h:1046-1231); the per-block rescale is fp32 work: the scale
// products a_d[m] * b_scale[n] of a block, a rank-1 matrix, come from the matrix unit too
// (v_mfma_f32_32x32x1_2b_f32: two blocks per instruction, exact), convert and multiply-add per
// output element stay on
// the vector unit (two operations against 64 int8 MFMA operations: this, not the int8
// rate of the matrix unit, bounds the kernel), and the rank-1 min term goes through
// another v_mfma_f32_32x32x2f32 straight into the accumulator.
//
// Workgroup: 512 threads = 8 wavefronts, tile 128 tokens x 64 weight rows, 64 KiB
// of LDS, so two workgroups share a compute unit and one's staging overlaps the
// other's multiply.  K advances one 256-column super-block at a time.  The global
// data of a step (raw weight blocks, 72 bytes of Q8_1 per thread) is fetched into
// registers while the previous step is multiplied; then the weights are decoded
// (nibble unpack / requantise, shared with the GEMV decoders) into LDS as int8
// [row][k], the activations copied beside them, both with a 272-byte row stride
// (conflict-free ds_read_b128 for MFMA operands).  Wavefront w owns weight rows
// 32*(w%2).. and tokens 32*(w/2)..: one 32x32 MFMA tile.  The MFMA's A operand is
// the activation tile, B the weight tile, so a lane holds one weight row n and 16
// tokens: stores of C are 128-byte coalesced and b_scale is one register per block.
#include "gemv_traits_all.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    typedef float v16f __attribute__((ext_vector_type(16)));
    typedef float v32f __attribute__((ext_vector_type(32)));

    constexpr int GEMM_BM = 128;        // tokens per workgroup
    // (launches of up to 32 and up to 64 tokens run tiles of 32 and 64 tokens: gemm_kernel's BM)
    constexpr int GEMM_BN = 64;         // weight rows per workgroup
    constexpr int GEMM_THREADS = 512;
    constexpr int GEMM_STRIDE = 256 + 16; // bytes per LDS row (one super-block + pad)
    // per-block scale tables [8][rows + 8]: the pad spreads the four threads that write one
    // row's scales of different blocks over different banks
    constexpr int GEMM_SN = GEMM_BN + 8;

    struct GemmArgs
    {
        GemvArgs w;         // only w.w, w.N, w.SB are used (weight addressing)
        const uint32_t *q8; // [M][K/32] blocks as dwords
        float *y;
        int M, ldy;
        // DUMP kernels only: the exact per-block int32 sums of weight rows [row0, row0+nrows) go to
        // sums[(m * nrows + n - row0) * (K/32) + block]
        int32_t *sums;
        int row0, nrows;
        int tile0; // first 64-row tile of the launch (0 unless DUMP)
    };

    template <class F, int BM>
    constexpr size_t gemm_lds_bytes()
    {
        return (size_t)(BM + GEMM_BN) * GEMM_STRIDE + (size_t)2 * 8 * (BM + 8 + GEMM_SN) * sizeof(float);
    }

    // Two adjacent Q8_1 blocks (72 bytes, 4-byte aligned) of one token, fetched with loads
    // the kernel waits for itself: written as ordinary loads the compiler moves them down
    // to their first use, behind the multiply they are meant to overlap.
    typedef int v2i __attribute__((ext_vector_type(2)));
    struct GemmActRaw
    {
        v4i q0, q1, q2, q3;
        v2i q4;
        __device__ __forceinline__ void load(const uint32_t *p)
        {
            asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(q0) : "v"(p));
            asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=&v"(q1) : "v"(p));
            asm volatile("global_load_dwordx4 %0, %1, off offset:32" : "=&v"(q2) : "v"(p));
            asm volatile("global_load_dwordx4 %0, %1, off offset:48" : "=&v"(q3) : "v"(p));
            asm volatile("global_load_dwordx2 %0, %1, off offset:64" : "=&v"(q4) : "v"(p));
        }
        // every load issued so far has arrived
        __device__ __forceinline__ void wait()
        {
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(q0), "+v"(q1), "+v"(q2), "+v"(q3), "+v"(q4));
        }
        __device__ __forceinline__ uint32_t dword(int i) const
        {
            // i is a compile-time constant after unrolling
            return (uint32_t)(i < 4 ? q0[i] : i < 8 ? q1[i - 4] : i < 12 ? q2[i - 8] : i < 16 ? q3[i - 12] : q4[i - 16]);
        }
    };

    // Weight data of one K step held in registers while the previous step is multiplied.
    template <class F, bool QUAD = F::USE_QUAD>
    struct GemmPrefetch;

    // Formats with a quad-lane decoder: thread = (weight row, quad lane), 64 weights.
    template <class F>
    struct GemmPrefetch<F, true>
    {
        typedef typename F::Quad Q;
        typename Q::Raw raw;
        typename Q::Lane lc;
        typename Q::Cursor wc;
        int row, l;
        bool active; // wavefront-uniform: BN rows x 4 quad lanes = the first 4*BN threads

        // first: the first of the 4 BN decoding threads (a multiple of 4 BN)
        __device__ __forceinline__ void init(const GemmArgs &g, long n0, int tid, int first)
        {
            const int t0 = __builtin_amdgcn_readfirstlane(tid);
            active = t0 >= first && t0 < first + GEMM_BN * 4;
            row = (tid >> 2) & (GEMM_BN - 1);
            l = tid & 3;
            lc = Q::lane_consts(l);
            long n = n0 + row;
            if (n >= g.w.N)
                n = g.w.N - 1; // tail rows: decode a valid row, never stored
            wc = Q::cursor(g.w, (size_t)n * g.w.SB, (size_t)n * g.w.SB, lc);
        }
        __device__ __forceinline__ void issue(const GemmArgs &, int sb)
        {
            // the other wavefronts load the same bytes again (cache hits) and drop them: a
            // load under a condition would need a register copy that waits for it at once
            // (asking for the rows of a later step instead, to warm the L2 cache, changed nothing)
            Q::load_at(raw, wc, lc, sb);
        }
        __device__ __forceinline__ void store(uint8_t *Wl, float *bs, float *bm, const void *)
        {
            Q::template wait<0>(raw);
            if (!active)
                return;
            v4i w[4];
            typename Q::Scale S;
            Q::decode(raw, lc, w, S);
#pragma unroll
            for (int i = 0; i < 2; ++i)
            {
                const int j = Q::block_of(l, i);
                v4i *dst = reinterpret_cast<v4i *>(Wl + row * GEMM_STRIDE + 32 * j);
                dst[0] = w[2 * i];
                dst[1] = w[2 * i + 1];
                bs[j * GEMM_SN + row] = Q::scale_f32(S, i);
                bm[j * GEMM_SN + row] = Q::min_f32(S, i);
            }
        }
        __device__ __forceinline__ void finish() { Q::template wait<0>(raw); }
    };

    // Other formats: the 8-lane decode of the GEMV skeleton, one task per thread.
    template <class F>
    struct GemmPrefetch<F, false>
    {
        static_assert(GEMM_BN * 8 == GEMM_THREADS, "one (row, lane) task per thread");
        typename F::Raw raw;
        long n;
        int row, c;

        __device__ __forceinline__ void init(const GemmArgs &g, long n0, int tid, int)
        {
            row = tid >> 3;
            c = tid & 7;
            n = n0 + row;
            if (n >= g.w.N)
                n = g.w.N - 1;
        }
        __device__ __forceinline__ void issue(const GemmArgs &g, int sb) { raw = F::load(g.w, n, sb, c); }
        __device__ __forceinline__ void store(uint8_t *Wl, float *bs, float *bm, const void *tab)
        {
            v4i w0, w1;
            int j;
            float bscale, bmin;
            F::decode(raw, c, w0, w1, j, bscale, bmin, tab);
            int j0, e0, j1, e1;
            F::where(c, j0, e0, j1, e1);
            *reinterpret_cast<v4i *>(Wl + row * GEMM_STRIDE + 32 * j0 + e0) = w0;
            *reinterpret_cast<v4i *>(Wl + row * GEMM_STRIDE + 32 * j1 + e1) = w1;
            bs[j * GEMM_SN + row] = bscale;
            bm[j * GEMM_SN + row] = bmin;
        }
        __device__ __forceinline__ void finish() {}
    };

    // DUMP: also store the matrix unit's results, the exact int32 block sums (the parity hook of
    // the C-ABI), for a window of weight rows; otherwise the same code.
    // BM = 128: wavefront w owns one 32x32 tile (tokens 32 (w / 2).., weight rows 32 (w % 2)..) and all eight
    // blocks of a K step.  BM = 64 and 32 (few tokens): the workgroup has four or two tiles only, so two or
    // four wavefronts share a tile and take four or two of a step's eight blocks each -- the rescale work per
    // wavefront falls with the tokens -- and their partial accumulators are added in wavefront order at the
    // end.
    template <class F, bool DUMP = false, int BM = GEMM_BM>
    // (the block-sum variant of the small tile also carries the addresses of the sums: it may take the
    // registers of three wavefronts per SIMD unit; it is the parity hook, not a timed path)
    __global__ void __launch_bounds__(GEMM_THREADS)
        __attribute__((amdgpu_waves_per_eu(DUMP && BM != GEMM_BM ? 3 : 4, 4)))
        gemm_kernel(const GemmArgs g)
    {
        static_assert(BM == 128 || BM == 64 || BM == 32, "tiles of 128, 64 or 32 tokens");
        constexpr int GEMM_SM = BM + 8; // per-block scale table [8][tokens + 8]
        constexpr int MTILES = BM / 32;             // 32-token tiles of the workgroup
        constexpr int KPARTS = 4 / MTILES;          // wavefronts that share a tile's K step
        constexpr int KB_PER = 8 / KPARTS;          // blocks of a K step per wavefront
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        uint8_t *Al = smem;                             // [BM][STRIDE] activations int8
        uint8_t *Wl = Al + BM * GEMM_STRIDE;            // [BN][STRIDE] weights int8
        float *ad = reinterpret_cast<float *>(Wl + GEMM_BN * GEMM_STRIDE); // [8][SM] a_d
        float *asd = ad + 8 * GEMM_SM;                  // [8][SM]
        float *bs = asd + 8 * GEMM_SM;                  // [8][SN]
        float *bm = bs + 8 * GEMM_SN;                   // [8][SN]
        void *tab = format_tables_lds<F>(); // static LDS beside the dynamic tiles

        if (F::TABLE_BYTES > 0)
            F::stage_tables(tab);

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        // (small tiles: in a scalar register, like all it leads to -- they have no vector register to spare)
        const int wave = BM == GEMM_BM ? tid >> 6 : __builtin_amdgcn_readfirstlane(tid >> 6);
        const int ntile = wave & 1;
        const int mtile = KPARTS == 1 ? wave >> 1 : (wave >> 1) % MTILES;
        const int kpart = KPARTS == 1 ? 0 : (wave >> 1) / MTILES; // this wavefront's blocks of a step: kpart * KB_PER ..
        const int l32 = lane & 31;
        const int lh = lane >> 5;

        const long n0 = ((long)blockIdx.x + g.tile0) * GEMM_BN;
        const long m0 = (long)blockIdx.y * BM;
        const int KB = g.w.SB * 8;

        // activations: thread = (token, pair of adjacent Q8_1 blocks) -> 72 contiguous bytes; the first
        // 4 BM threads (whole wavefronts) have a token, the others load and store nothing
        const bool a_thread = BM * 4 >= GEMM_THREADS || __builtin_amdgcn_readfirstlane(tid) < BM * 4; // per wavefront
        const int am = (tid >> 2) & (BM - 1);
        const int ap = tid & 3;
        long am_src = m0 + am;
        if (am_src >= g.M)
            am_src = g.M - 1; // tail tokens: a valid row, never stored
        const uint32_t *asrc = g.q8 + ((size_t)am_src * KB + 2 * ap) * 9;
        GemmActRaw areg;

        GemmPrefetch<F> pf;
        // small tiles: the wavefronts that stage no activations decode the weights (the second half of
        // the workgroup), so that the two kinds of staging run side by side
        pf.init(g, n0, tid, BM == GEMM_BM ? 0 : GEMM_THREADS - GEMM_BN * 4);

        auto issue = [&](int sb) {
            pf.issue(g, sb);
            if (a_thread)
                areg.load(asrc + (size_t)sb * 72);
        };

        // One K step's staging: registers -> LDS (weights as int8 [row][k] + scales, activations
        // beside them), then the next step's global data is asked for, to travel while this one
        // is multiplied (the last step re-reads itself: every issued load is consumed, none is
        // conditional).
        auto stage = [&](int sb) {
            __syncthreads(); // previous step's LDS reads (and the table staging) are done
            pf.store(Wl, bs, bm, tab);
            areg.wait();
            if (a_thread)
            {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                {
                    const uint32_t h = areg.dword(9 * i);
                    const float d = h2f((uint16_t)(h & 0xFFFFu));
                    const int kb = 2 * ap + i;
                    ad[kb * GEMM_SM + am] = d;
                    asd[kb * GEMM_SM + am] = (float)(int16_t)(h >> 16) * d;
                    v4i *dst = reinterpret_cast<v4i *>(Al + am * GEMM_STRIDE + kb * 32);
                    dst[0] = (v4i){(int)areg.dword(9 * i + 1), (int)areg.dword(9 * i + 2), (int)areg.dword(9 * i + 3),
                                   (int)areg.dword(9 * i + 4)};
                    dst[1] = (v4i){(int)areg.dword(9 * i + 5), (int)areg.dword(9 * i + 6), (int)areg.dword(9 * i + 7),
                                   (int)areg.dword(9 * i + 8)};
                }
            }
            __syncthreads();
            issue(sb + 1 < g.w.SB ? sb + 1 : sb);
        };

        v16f acc;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[r] = 0.0f;

        issue(0);
        for (int sb = 0; sb < g.w.SB; ++sb)
        {
            stage(sb);

            // ---- multiply ------------------------------------------------------------------
            // 8 block products per step; the other wavefronts of the SIMD unit keep the vector
            // unit busy while this one waits for the matrix unit.
            const uint8_t *wrow = Wl + (ntile * 32 + l32) * GEMM_STRIDE + lh * 16;
            const uint8_t *arow = Al + (mtile * 32 + l32) * GEMM_STRIDE + lh * 16;
            v16i zero;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                zero[r] = 0;
            v32f zero2f;
#pragma unroll
            for (int r = 0; r < 32; ++r)
                zero2f[r] = 0.0f;
            v16f zero1f;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                zero1f[r] = 0.0f;
            auto product = [&](int kb) {
                const v4i bw = *reinterpret_cast<const v4i *>(wrow + kb * 32);
                const v4i aa = *reinterpret_cast<const v4i *>(arow + kb * 32);
                return __builtin_amdgcn_mfma_i32_32x32x32_i8(aa, bw, zero, 0, 0, 0);
            };
            // The scale products a_d[m] * b_scale[n] of a block are a rank-1 matrix: the matrix
            // unit forms them in the layout of the block sums instead of 16 multiplies per lane,
            // two blocks per instruction (v_mfma_f32_32x32x1_2b_f32: lane half lh supplies block
            // kb + lh, results 0-15 belong to block kb, 16-31 to block kb + 1).  Exact: both
            // factors are fp16 values.
            auto scales = [&](int kb) {
                const float av = ad[(kb + lh) * GEMM_SM + mtile * 32 + l32];
                const float bv = bs[(kb + lh) * GEMM_SN + ntile * 32 + l32];
                return __builtin_amdgcn_mfma_f32_32x32x1f32(av, bv, zero2f, 0, 0, 0);
            };
            // Formats whose prefetch registers leave no room for two blocks' scale products form
            // them one block at a time (v_mfma_f32_32x32x2_f32 adds (a_d/2) * b_scale twice: exact).
            auto scales1 = [&](int kb) {
                const float av = 0.5f * ad[kb * GEMM_SM + mtile * 32 + l32];
                const float bv = bs[kb * GEMM_SN + ntile * 32 + l32];
                return __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, zero1f, 0, 0, 0);
            };
            v32f cs;
            v16f cs1;
            const int kb0 = kpart * KB_PER; // (KB_PER is even: the pairs of the scale and min-term products stay whole)
            if constexpr (F::GEMM_PAIR_SCALES)
                cs = scales(kb0);
            else
                cs1 = scales1(kb0);
#pragma unroll
            for (int kk8 = 0; kk8 < KB_PER; ++kk8)
            {
                const int kb = kb0 + kk8;
                // (one set of result registers: with the scale products held as well, a second
                // set would not fit the 128 registers that four wavefronts per SIMD unit leave;
                // the other wavefronts cover the product's latency)
                const v16i d = product(kb);
                if constexpr (DUMP)
                {
                    const long n = n0 + ntile * 32 + l32;
                    const long nn = n - g.row0;
                    if (n < g.w.N && nn >= 0 && nn < g.nrows)
                    {
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                        {
                            const long m = m0 + mtile * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                            if (m < g.M)
                                g.sums[((size_t)m * g.nrows + (size_t)nn) * (size_t)KB + (size_t)sb * 8 + kb] = d[r];
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[r] = fmaf((float)d[r], F::GEMM_PAIR_SCALES ? cs[16 * (kk8 & 1) + r] : cs1[r], acc[r]);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (F::GEMM_PAIR_SCALES)
                {
                    if ((kk8 & 1) && kk8 + 1 < KB_PER)
                        cs = scales(kb + 1); // the other wavefronts of the unit cover its latency
                }
                else
                {
                    if (kk8 + 1 < KB_PER)
                        cs1 = scales1(kb + 1);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (F::HAS_MIN && (kk8 & 1))
                {
                    // rank-2 update over blocks kb-1, kb, straight into the accumulator: lane
                    // half lh supplies block kb-1+lh
                    const int kk = kb - 1 + lh;
                    const float bmin = bm[kk * GEMM_SN + ntile * 32 + l32];
                    const float av = asd[kk * GEMM_SM + mtile * 32 + l32];
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bmin, acc, 0, 0, 0);
                }
            }
        }
        pf.finish();
        areg.wait();

        if constexpr (KPARTS > 1 && !DUMP)
        {
            // the tile's wavefronts add their partial accumulators in wavefront order (kpart 0 + 1 + ..)
            __syncthreads(); // every wavefront is done with the step's LDS
            float *red = reinterpret_cast<float *>(smem); // [wavefront][16][64]
#pragma unroll
            for (int r = 0; r < 16; ++r)
                red[(wave * 16 + r) * 64 + lane] = acc[r];
            __syncthreads();
            if (kpart != 0)
                return;
#pragma unroll
            for (int p = 1; p < KPARTS; ++p)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[r] += red[((wave + 2 * MTILES * p) * 16 + r) * 64 + lane];
        }

        // ---- store: lane holds weight row n, 16 tokens -------------------------------------
        const long n = n0 + ntile * 32 + l32;
        if (!DUMP && n < g.w.N)
        {
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                const long m = m0 + mtile * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                if (m < g.M)
                    g.y[(size_t)m * g.ldy + n] = acc[r];
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

    template <class F, bool DUMP, int BM>
    bool gemm_launch_bm(const char *fn, const GemmArgs &g, int tiles_n, int M, hipStream_t st)
    {
        constexpr size_t lds = gemm_lds_bytes<F, BM>();
        static_assert(lds >= (size_t)8 * 16 * 64 * sizeof(float), "room for the partial accumulators");
        static LdsGrant grant;
        const hipError_t e = allow_lds(grant, reinterpret_cast<const void *>(&gemm_kernel<F, DUMP, BM>), lds);
        if (e != hipSuccess)
            return fail(fn, "cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        const dim3 grid((unsigned)tiles_n, (unsigned)((M + BM - 1) / BM));
        hipLaunchKernelGGL((gemm_kernel<F, DUMP, BM>), grid, dim3(GEMM_THREADS), lds, st, g);
        return launched(fn);
    }

    // d_sums: the block-sum variant over weight rows [row0, row0+nrows); only the workgroups
    // whose 64-row tile meets the window are launched.
    template <class F, bool DUMP = false>
    bool gemm_launch(const char *fn, const void *d_w, const void *d_q8, float *d_y, int M, int N, int K, int ldy,
                     hipStream_t st, int32_t *d_sums = nullptr, int row0 = 0, int nrows = 0)
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
        g.sums = d_sums;
        g.row0 = row0;
        g.nrows = nrows;
        g.tile0 = DUMP ? row0 / GEMM_BN : 0;
        // (the quad-lane decoders address a matrix through 32-bit offsets)
        if constexpr (F::USE_QUAD)
        {
            if (!F::Quad::addressable(N, K / 256))
                return fail(fn, "matrix too large for the kernel's 32-bit offsets (N=%d K=%d)", N, K);
        }
        const int tile_end = DUMP ? (row0 + nrows + GEMM_BN - 1) / GEMM_BN : (N + GEMM_BN - 1) / GEMM_BN;
        // few tokens: one smaller tile of tokens (a 128-token tile would rescale 128 rows for them)
        if (M <= 32)
            return gemm_launch_bm<F, DUMP, 32>(fn, g, tile_end - g.tile0, M, st);
        if (M <= 64)
            return gemm_launch_bm<F, DUMP, 64>(fn, g, tile_end - g.tile0, M, st);
        return gemm_launch_bm<F, DUMP, GEMM_BM>(fn, g, tile_end - g.tile0, M, st);
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

extern "C" bool llam_ql_gemm_block_sums(uint8_t fmt, const void *d_w, const void *d_q8, int32_t *d_sums,
                                        int M, int N, int K, int row0, int nrows, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_gemm_block_sums";
    if (fmt != LLAM_FMT_Q4_K && fmt != LLAM_FMT_Q6_K && fmt != LLAM_FMT_IQ3_S)
        return fail(fn, "unsupported weight format id %d", (int)fmt);
    if (M < 1 || N < 1 || K < 1 || (K % 256) != 0)
        return fail(fn, "need M, N >= 1 and K a positive multiple of 256 (M=%d N=%d K=%d)", M, N, K);
    if (!d_w || !d_q8 || !d_sums)
        return fail(fn, "null pointer");
    if (!aligned16(d_w) || !aligned4(d_q8) || !aligned4(d_sums))
        return fail(fn, "d_w must be 16-byte, d_q8 and d_sums 4-byte aligned");
    if (row0 < 0 || nrows < 1 || (long)row0 + nrows > N)
        return fail(fn, "row window [%d,%d) outside [0,%d)", row0, row0 + nrows, N);
    if ((M + GEMM_BM - 1) / GEMM_BM > 65535)
        return fail(fn, "M=%d too large for one launch", M);
    if ((size_t)M * (size_t)nrows * (size_t)(K / 32) * sizeof(int32_t) >= ((size_t)1 << 31))
        return fail(fn, "M=%d x %d rows x %d blocks of sums exceed 2 GiB", M, nrows, K / 32);
    if (!set_device(fn, device_id))
        return false;
    hipStream_t st = as_stream(stream);
    switch (fmt)
    {
    case LLAM_FMT_Q4_K: return gemm_launch<Q4KTraits, true>(fn, d_w, d_q8, nullptr, M, N, K, 0, st, d_sums, row0, nrows);
    case LLAM_FMT_Q6_K: return gemm_launch<Q6KTraits, true>(fn, d_w, d_q8, nullptr, M, N, K, 0, st, d_sums, row0, nrows);
    default: return gemm_launch<IQ3STraits, true>(fn, d_w, d_q8, nullptr, M, N, K, 0, st, d_sums, row0, nrows);
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
