// Chunked full-row decode GEMV (gfx950): rows of at least five super-blocks in
// formats without a quad-lane decoder (Q6_K, IQ3_S), Q4_K rows shorter than 16
// super-blocks, and the host-side launcher that picks a kernel for every shape.
//
// Same arithmetic and lane roles as the generic skeleton in gemv_core.h; what
// differs is how the work is fed:
//   - one wavefront per row at a time (8 lanes per super-block, 8 super-blocks per
//     load batch), U load batches issued together, and the next U -- of this row
//     or of the wavefront's next row -- already in flight while the current ones
//     are decoded, so a wavefront keeps 2*U x (16..52) bytes per lane outstanding;
//   - per-lane weight pointers advanced by constants (immediate offsets inside a
//     chunk), per-lane bit-field constants for the header decode, no per-element
//     predicates on full chunks;
//   - the first chunk's loads are issued BEFORE the activations are staged in LDS,
//     so HBM latency overlaps the staging.
//
// LDS: aq [M][K/32 units of 32 B]  int8 quants laid out per lane (see gemv_core.h)
//      ads[M][K/32] float2 = { f32(d), float(sum_qs)*f32(d) }
#pragma once

#include "gemv_core.h"
#include "gemv_quad.h"
#include "gemv_mfma.h"
#include "gemv_mfma_q6k.h"
#include "gemv_mfma_q4k_long.h"
#include <atomic>
#include <type_traits>

namespace llamql
{
    // Stage nkb Q8_1 blocks of each of M activation rows: one thread per block.
    template <class F, int M>
    __device__ __forceinline__ void stage_q8_blocks(const uint32_t *__restrict__ q8, int KB_total, int kb0, int nkb,
                                                    uint32_t *aq, float2 *ads)
    {
#pragma unroll
        for (int m = 0; m < M; ++m)
        {
            for (int kb = threadIdx.x; kb < nkb; kb += blockDim.x)
            {
                const uint32_t *src = q8 + ((size_t)m * KB_total + kb0 + kb) * 9;
                uint32_t v[9];
#pragma unroll
                for (int i = 0; i < 9; ++i)
                    v[i] = src[i];
                const float d = h2f((uint16_t)(v[0] & 0xFFFFu));
                ads[m * nkb + kb] = make_float2(d, (float)(int16_t)(v[0] >> 16) * d);
                int c0, p0, c1, p1;
                F::unit_of(kb & 7, 0, c0, p0);
                F::unit_of(kb & 7, 4, c1, p1);
                uint32_t *base = aq + (size_t)m * nkb * 8 + (size_t)(kb >> 3) * 64;
                *reinterpret_cast<uint4 *>(base + c0 * 8 + p0 * 4) = make_uint4(v[1], v[2], v[3], v[4]);
                *reinterpret_cast<uint4 *>(base + c1 * 8 + p1 * 4) = make_uint4(v[5], v[6], v[7], v[8]);
            }
        }
    }

    // dump_row: with DUMP, where the block sums of this lane's row go (sums + (row - row0) * blocks
    // per row, null outside the window); the sums of activation row m lie dump_m_stride further
    template <class F, int M, int U, bool PARTIAL, bool DUMP>
    __device__ __forceinline__ void gemv_fast_chunk(const typename F::Raw (&cur)[U], const typename F::Lane &lc,
                                                    bool odd, int s_base, int nsb, const uint8_t *aq_lane,
                                                    const uint8_t *ads_lane, int m_stride_aq, int m_stride_ads,
                                                    const void *tab, float (&acc)[M], int32_t *dump_row,
                                                    size_t dump_m_stride, int dump_sb0)
    {
#pragma unroll
        for (int u = 0; u < U; ++u)
        {
            if (PARTIAL && s_base + 8 * u >= nsb)
                continue;
            v4i w0, w1;
            float bscale, bmin;
            F::decode2(cur[u], lc, w0, w1, bscale, bmin, tab);
#pragma unroll
            for (int m = 0; m < M; ++m)
            {
                const v4i *ap = reinterpret_cast<const v4i *>(aq_lane + m * m_stride_aq + u * 2048);
                const v4i a0 = ap[0];
                const v4i a1 = ap[1];
                const float2 sd = *reinterpret_cast<const float2 *>(ads_lane + m * m_stride_ads + u * 512);
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
                if constexpr (DUMP)
                {
                    if (dump_row)
                        dump_row[(size_t)m * dump_m_stride + (size_t)(dump_sb0 + s_base + 8 * u) * 8 + lc.j] = idot;
                }
                const float cs = sd.x * bscale;
                acc[m] = fmaf((float)idot, cs, acc[m]);
                if (F::HAS_MIN)
                    acc[m] = fmaf(sd.y, bmin, acc[m]);
            }
        }
    }

    // DUMP: also store the exact int32 block sums (the parity hook); otherwise the same code.
    template <class F, int M, int U, bool DUMP = false>
    __global__ void __launch_bounds__(GEMV_WAVES *WAVE) gemv_fast_kernel(const GemvArgs a)
    {
        extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
        const int nkb = a.nsb * 8;
        uint32_t *aq = lds;                                          // M * nkb * 8 dwords
        float2 *ads = reinterpret_cast<float2 *>(aq + M * nkb * 8);  // M * nkb
        void *tab = format_tables_lds<F>();

        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = threadIdx.x >> 6;
        const int c = lane & 7;
        const int grp = lane >> 3;
        const bool odd = (c & 1) != 0;
        const typename F::Lane lc = F::lane_consts(c);

        const long wg_row0 = (long)blockIdx.x * (GEMV_WAVES * a.rows_per_wave);
        const int chunk_sb = 8 * U;
        const int nfull = a.nsb / chunk_sb;
        const int nchunks = (a.nsb + chunk_sb - 1) / chunk_sb;

        // weight loads of the first chunk go out before anything else
        long row = wg_row0 + wave;
        const bool any_row = row < a.N;
        typename F::Ptr p = F::ptr(a, any_row ? row : (long)a.N - 1, a.sb0 + grp, c);
        typename F::Raw buf[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
        {
            buf[u] = typename F::Raw{};
            if (any_row && grp + 8 * u < a.nsb)
                buf[u] = F::load_at(p, 8 * u);
        }

        if (F::TABLE_BYTES > 0)
            F::stage_tables(tab);
        stage_q8_blocks<F, M>(a.q8, a.SB * 8, a.sb0 * 8, nkb, aq, ads);
        __syncthreads();

        const uint8_t *aq_lane0 = reinterpret_cast<const uint8_t *>(aq) + (grp * 8 + c) * 32;
        const uint8_t *ads_lane0 = reinterpret_cast<const uint8_t *>(ads) + (grp * 8 + lc.j) * 8;
        const int m_stride_aq = nkb * 32;
        const int m_stride_ads = nkb * 8;

        for (int r = 0; r < a.rows_per_wave; ++r, row += GEMV_WAVES)
        {
            if (row >= a.N)
                break;
            float acc[M];
#pragma unroll
            for (int m = 0; m < M; ++m)
                acc[m] = 0.0f;
            int32_t *dump_row = nullptr;
            const size_t dump_m_stride = (size_t)a.nrows * ((size_t)a.SB * 8);
            if constexpr (DUMP)
            {
                if (row >= a.row0 && row < (long)a.row0 + a.nrows)
                    dump_row = a.sums + (size_t)(row - a.row0) * ((size_t)a.SB * 8);
            }

            for (int ch = 0; ch < nchunks; ++ch)
            {
                typename F::Raw cur[U];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    cur[u] = buf[u];

                // ---- prefetch: next chunk of this row, else first chunk of the next row
                const bool last = (ch + 1 == nchunks);
                int next_base; // first super-block (of this lane) in the chunk being fetched
                bool more;
                if (!last)
                {
                    F::advance(p, chunk_sb);
                    next_base = grp + (ch + 1) * chunk_sb;
                    more = true;
                }
                else
                {
                    F::advance(p, GEMV_WAVES * a.SB - ch * chunk_sb);
                    next_base = grp;
                    more = (r + 1 < a.rows_per_wave) && (row + GEMV_WAVES < a.N);
                }
                if (more)
                {
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (next_base + 8 * u < a.nsb)
                            buf[u] = F::load_at(p, 8 * u);
                }

                // ---- decode + dot
                const uint8_t *aql = aq_lane0 + ch * (U * 2048);
                const uint8_t *adl = ads_lane0 + ch * (U * 512);
                if (ch < nfull)
                    gemv_fast_chunk<F, M, U, false, DUMP>(cur, lc, odd, grp + ch * chunk_sb, a.nsb, aql, adl,
                                                          m_stride_aq, m_stride_ads, tab, acc, dump_row, dump_m_stride,
                                                          a.sb0);
                else
                    gemv_fast_chunk<F, M, U, true, DUMP>(cur, lc, odd, grp + ch * chunk_sb, a.nsb, aql, adl,
                                                         m_stride_aq, m_stride_ads, tab, acc, dump_row, dump_m_stride,
                                                         a.sb0);
            }

            if constexpr (!DUMP) // the block-sum variant has no fp32 output
            {
#pragma unroll
                for (int m = 0; m < M; ++m)
                {
                    const float total = wave_sum(acc[m]);
                    if (lane == 0)
                    {
                        float *dst = a.y + (size_t)m * a.ldy + row;
                        const float v = weighted(a.out_scale, total);
                        *dst = a.accumulate ? add_rounded(*dst, v) : v;
                    }
                }
            }
        }
    }

    template <class F, int M, bool DUMP>
    inline void gemv_fast_launch_u(int U, dim3 grid, size_t lds, hipStream_t st, const GemvArgs &a)
    {
        dim3 block(GEMV_WAVES * WAVE);
        // formats whose decode is register-hungry only build (and run) the shallow variant
        if constexpr (F::FAST_MAX_U >= 4)
        {
            switch (U)
            {
            case 1: hipLaunchKernelGGL((gemv_fast_kernel<F, M, 1, DUMP>), grid, block, lds, st, a); break;
            case 2: hipLaunchKernelGGL((gemv_fast_kernel<F, M, 2, DUMP>), grid, block, lds, st, a); break;
            case 3: hipLaunchKernelGGL((gemv_fast_kernel<F, M, 3, DUMP>), grid, block, lds, st, a); break;
            default: hipLaunchKernelGGL((gemv_fast_kernel<F, M, 4, DUMP>), grid, block, lds, st, a); break;
            }
        }
        else
        {
            (void)U;
            hipLaunchKernelGGL((gemv_fast_kernel<F, M, 1, DUMP>), grid, block, lds, st, a);
        }
    }

    // M is one of 1,2,3,4,8.  a.sums set: the block-sum variant of the same kernel.
    template <class F>
    inline void gemv_fast_launch(int M, int U, dim3 grid, size_t lds, hipStream_t st, const GemvArgs &a)
    {
        if (a.sums)
        {
            switch (M)
            {
            case 1: gemv_fast_launch_u<F, 1, true>(U, grid, lds, st, a); break;
            case 2: gemv_fast_launch_u<F, 2, true>(U, grid, lds, st, a); break;
            case 3: gemv_fast_launch_u<F, 3, true>(U, grid, lds, st, a); break;
            case 4: gemv_fast_launch_u<F, 4, true>(U, grid, lds, st, a); break;
            default: gemv_fast_launch_u<F, 8, true>(U, grid, lds, st, a); break;
            }
            return;
        }
        switch (M)
        {
        case 1: gemv_fast_launch_u<F, 1, false>(U, grid, lds, st, a); break;
        case 2: gemv_fast_launch_u<F, 2, false>(U, grid, lds, st, a); break;
        case 3: gemv_fast_launch_u<F, 3, false>(U, grid, lds, st, a); break;
        case 4: gemv_fast_launch_u<F, 4, false>(U, grid, lds, st, a); break;
        default: gemv_fast_launch_u<F, 8, false>(U, grid, lds, st, a); break;
        }
    }

    // Wavefronts of gemv_fast_kernel<F, M, U> a compute unit holds at once, as far as registers
    // allow (asked of the runtime once per instantiation; the LDS limit is the caller's).
    template <class F, int M, int U>
    inline int gemv_fast_resident_waves_mu()
    {
        static std::atomic<int> cached{0};
        int w = cached.load(std::memory_order_relaxed);
        if (w == 0)
        {
            int blocks = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, gemv_fast_kernel<F, M, U, false>,
                                                             GEMV_WAVES * WAVE, 0) != hipSuccess ||
                blocks < 1)
            {
                (void)hipGetLastError();
                blocks = 32 / GEMV_WAVES;
            }
            w = blocks * GEMV_WAVES;
            cached.store(w, std::memory_order_relaxed);
        }
        return w;
    }

    template <class F, int M>
    inline int gemv_fast_resident_waves_m(int U)
    {
        if constexpr (F::FAST_MAX_U >= 4)
        {
            switch (U)
            {
            case 1: return gemv_fast_resident_waves_mu<F, M, 1>();
            case 2: return gemv_fast_resident_waves_mu<F, M, 2>();
            case 3: return gemv_fast_resident_waves_mu<F, M, 3>();
            default: return gemv_fast_resident_waves_mu<F, M, 4>();
            }
        }
        else
            return gemv_fast_resident_waves_mu<F, M, 1>();
    }

    // M is one of 1,2,3,4,8; lds: dynamic LDS of a workgroup.
    template <class F>
    inline int gemv_fast_resident_waves(int M, int U, size_t lds)
    {
        int w;
        switch (M)
        {
        case 1: w = gemv_fast_resident_waves_m<F, 1>(U); break;
        case 2: w = gemv_fast_resident_waves_m<F, 2>(U); break;
        case 3: w = gemv_fast_resident_waves_m<F, 3>(U); break;
        case 4: w = gemv_fast_resident_waves_m<F, 4>(U); break;
        default: w = gemv_fast_resident_waves_m<F, 8>(U); break;
        }
        const size_t per_wg = lds + F::TABLE_BYTES + 256;
        const long by_lds = (long)(160 * 1024 / per_wg) * GEMV_WAVES;
        if (by_lds < w)
            w = (int)by_lds;
        return w < GEMV_WAVES ? GEMV_WAVES : w;
    }

    int gemv_unroll_override();
    // Launch shape for N rows of nsb super-blocks (one LDS slice) on a device with
    // `cus` compute units.  Rows are dealt to workgroups so that every compute unit
    // receives (nearly) the same number of rows in a single round of workgroups.
    struct GemvShape
    {
        int gshift, rpw, U;
        long grid;
    };

    // max_u: deepest unroll the format builds; resident(U): wavefronts of the kernel with that
    // unroll a compute unit holds at once.
    template <class Resident>
    inline GemvShape gemv_shape(long N, int nsb, int cus, int max_u, Resident resident)
    {
        GemvShape sh;
        sh.gshift = 3;
        while (sh.gshift > 0 && (1 << (sh.gshift - 1)) >= nsb)
            --sh.gshift;
        const int G = 1 << sh.gshift;
        const int R = 8 >> sh.gshift;
        const int iters = (nsb + G - 1) / G; // wavefront iterations per row
        // unroll: whole row when short, else the depth that wastes the fewest slots
        sh.U = iters;
        if (iters > 4)
        {
            int best = 4, waste = (4 - iters % 4) % 4;
            for (int u = 3; u >= 2; --u)
            {
                const int w = (u - iters % u) % u;
                if (w < waste)
                {
                    best = u;
                    waste = w;
                }
            }
            sh.U = best;
        }
        if (gemv_unroll_override() > 0)
            sh.U = gemv_unroll_override() > 4 ? 4 : gemv_unroll_override();
        else if (sh.U > max_u)
            sh.U = max_u;
        int cap = sh.gshift == 3 ? resident(sh.U) : 32; // wavefronts a compute unit holds
        if (cap > 32)
            cap = 32;
        const int floor_waves = cap < 16 ? cap : 16;

        // rows (in units of R) each compute unit must cover
        const long units = (N + R - 1) / R;
        const long per_cu = (units + cus - 1) / cus;
        int rpw = gemv_rows_per_wave_override();
        if (rpw <= 0)
        {
            // candidates: row batches per wavefront; cost = padded work per CU, with at least
            // 16 wavefronts per CU when there is enough work (and they fit), at most what a
            // compute unit holds at once: a second round runs at a fraction of the occupancy
            double best_cost = 1e30;
            rpw = 1;
            for (int cand = 1; cand <= 64; ++cand)
            {
                const long wg_units = (long)GEMV_WAVES * cand;
                const long wgs_per_cu = (per_cu + wg_units - 1) / wg_units;
                double cost = (double)(wgs_per_cu * wg_units) / (double)per_cu;
                const long waves = wgs_per_cu * GEMV_WAVES;
                if (waves > cap)
                    cost *= 1.0 + 0.25 * (double)((waves + cap - 1) / cap - 1); // extra rounds: restaging + tail
                if (waves < floor_waves && per_cu >= floor_waves)
                    cost *= 1.25; // too little memory-level parallelism
                if (cost < best_cost - 1e-9)
                {
                    best_cost = cost;
                    rpw = cand;
                }
            }
        }
        sh.rpw = rpw;
        const long rows_per_wg = (long)GEMV_WAVES * R * rpw;
        sh.grid = (N + rows_per_wg - 1) / rows_per_wg;
        return sh;
    }

    // Quad-lane kernel over up to QUAD_MAX_PROJ matrices of one format and row length that
    // share their activations.  Every matrix keeps the rows-per-wavefront it has when it is
    // launched alone, so results do not depend on what it is launched together with.
    struct QuadProj
    {
        const void *w;
        float *y;
        int N, ldy;
    };
    template <class F>
    bool quad_eligible(int M, int N, int K)
    {
        if constexpr (F::USE_QUAD)
            return K / 256 >= QUAD_STEP_SB && gemv_unroll_override() == 0 && F::Quad::addressable(N, K / 256) &&
                   quad_lds_bytes(M, K / 256) + F::Quad::STATIC_LDS <= QUAD_MAX_LDS;
        else
            return false;
    }
    // Batches of 5..8 rows on rows of 8 super-blocks or more (the activations of the whole batch
    // and the wavefronts' bounce buffers must fit the 160 KiB of LDS) go to the matrix-unit
    // kernel, in formats that have one.
    // below this many rows a Q4_K matrix at batch 5..8 stays on the quad-lane kernel (measured on
    // 5120-column matrices: 1024 rows 10.6 us on the matrix unit, 8192 rows and more faster there)
    constexpr int MFMA_MIN_ROWS = 4096;

    template <class F>
    bool mfma_eligible(int M, int N, int K)
    {
        if constexpr (!F::USE_MFMA_BATCH)
            return false;
        else if (M < 5 || N < 1 || K / 256 < 8 || gemv_unroll_override() != 0 || gemv_rows_per_wave_override() != 0)
            return false;
        else if constexpr (std::is_same<typename F::Quad, Q6KQuad>::value)
            // where the quad-lane kernel cannot keep the batch in LDS and would run it as two
            // (any row length works here: long rows are walked in chunks)
            return quad_lds_bytes(M, K / 256) > QUAD_MAX_LDS && Q6KQuad::addressable(N, K / 256);
        else
            // a matrix of few 32-row tiles leaves most compute units idle here: the quad-lane kernel
            // spreads it over all of them (and shares its launch with a following Q6_K matrix)
            // (long rows are walked in chunks, gemv_mfma_q4k_long.h; where not even one buffer of the whole
            // batch fits the LDS but the quad-lane kernel still holds the batch in one launch, that one is
            // faster: 5 rows of K = 25600 28 against 32 us)
            return N >= MFMA_MIN_ROWS && (mfma_max_slices(K / 256) >= 1 || quad_lds_bytes(M, K / 256) > QUAD_MAX_LDS);
    }

    template <int SRC, bool DUMP = false, bool PLANE = false>
    void gemv_mfma_q4k_launch_src(dim3 grid, dim3 block, size_t lds, hipStream_t st, const MfmaArgs &a)
    {
        static LdsGrant grant;
        (void)allow_lds(grant, reinterpret_cast<const void *>(&gemv_mfma_q4k_kernel<SRC, DUMP, PLANE>), QUAD_MAX_LDS);
        hipLaunchKernelGGL((gemv_mfma_q4k_kernel<SRC, DUMP, PLANE>), grid, block, lds, st, a);
    }

    // Rows that take the chunked kernel: those whose activations leave gemv_mfma_q4k_kernel fewer than its
    // eight wavefronts per tile (measured at batch 8 on 5120 rows: 50 super-blocks 19.0 against 23.5 us
    // chunked; 32 super-blocks 13.4 against 12.6 us, and 25600 rows of 20 super-blocks 32.7 against 25.1 us).
    inline bool mfma4_long_rows(int SB) { return mfma_max_slices(SB) < MFMA_MAX_SLICES; }

    template <int SRC, bool DUMP = false, bool PLANE = false>
    void gemv_mfma_q4k_long_launch_src(dim3 grid, dim3 block, size_t lds, hipStream_t st, const MfmaLongArgs &a)
    {
        static LdsGrant grant;
        (void)allow_lds(grant, reinterpret_cast<const void *>(&gemv_mfma_q4k_long_kernel<SRC, DUMP, PLANE>), QUAD_MAX_LDS);
        hipLaunchKernelGGL((gemv_mfma_q4k_long_kernel<SRC, DUMP, PLANE>), grid, block, lds, st, a);
    }

    // Rows too long for gemv_mfma_q4k_kernel (the batch's activations do not fit the LDS).
    inline bool gemv_mfma_q4k_long_launch(const char *fn, const void *d_w, const void *d_plane, const ActSource &src,
                                          float *d_y, int M, int N, int K, int ldy, int device_id, hipStream_t st,
                                          int32_t *d_sums, int row0, int nrows)
    {
        const int SB = K / 256;
        const Mfma6Shape sh = gemv_mfma6_shape(N, SB, cu_count(device_id), d_sums ? MFMA4_LONG_DUMP_COMPUTE : MFMA4_LONG_COMPUTE,
                                               d_plane != nullptr, MFMA_BOUNCE);
        MfmaLongArgs a{};
        a.ksplit = 1;
        a.w = static_cast<const uint8_t *>(d_w);
        a.plane = static_cast<const uint8_t *>(d_plane);
        a.q8 = static_cast<const uint32_t *>(src.q8);
        a.x = src.x;
        a.x2 = src.x2;
        a.ldx = src.ldx;
        a.y = d_y;
        a.ldy = ldy;
        a.N = N;
        a.SB = SB;
        a.M = M;
        a.slices = sh.slices;
        a.tile_rows = sh.tile_rows;
        a.tiles = sh.tiles;
        a.chunk = sh.chunk;
        a.sums = d_sums;
        a.row0 = row0;
        a.nrows = nrows;
        const dim3 grid((unsigned)sh.grid), block((unsigned)(sh.slices * sh.tiles + MFMA4_LONG_PRODUCERS) * WAVE);
        const size_t lds = mfma6_act_bytes(SB, sh.chunk) + (a.plane ? 0 : (size_t)sh.slices * sh.tiles * MFMA_BOUNCE);
        if (d_sums)
        {
            if (src.kind != ACT_SRC_Q8)
                return fail(fn, "block sums are dumped on Q8_1 input");
            if (a.plane)
                gemv_mfma_q4k_long_launch_src<QUAD_SRC_Q8, true, true>(grid, block, lds, st, a);
            else
                gemv_mfma_q4k_long_launch_src<QUAD_SRC_Q8, true>(grid, block, lds, st, a);
            return launched(fn);
        }
        if (a.plane)
        {
            switch (src.kind)
            {
            case ACT_SRC_F32: gemv_mfma_q4k_long_launch_src<QUAD_SRC_F32, false, true>(grid, block, lds, st, a); break;
            case ACT_SRC_SWIGLU: gemv_mfma_q4k_long_launch_src<QUAD_SRC_SWIGLU, false, true>(grid, block, lds, st, a); break;
            default: gemv_mfma_q4k_long_launch_src<QUAD_SRC_Q8, false, true>(grid, block, lds, st, a); break;
            }
            return launched(fn);
        }
        switch (src.kind)
        {
        case ACT_SRC_F32: gemv_mfma_q4k_long_launch_src<QUAD_SRC_F32>(grid, block, lds, st, a); break;
        case ACT_SRC_SWIGLU: gemv_mfma_q4k_long_launch_src<QUAD_SRC_SWIGLU>(grid, block, lds, st, a); break;
        default: gemv_mfma_q4k_long_launch_src<QUAD_SRC_Q8>(grid, block, lds, st, a); break;
        }
        return launched(fn);
    }

    // d_plane: the matrix's batch plane (q4k_plane_bytes) or null; with one, the kernel reads it
    // instead of the prepared matrix, the block-sum variant included.
    inline bool gemv_mfma_q4k_launch(const char *fn, const void *d_w, const void *d_plane, const ActSource &src,
                                     float *d_y, int M, int N, int K, int ldy, int device_id, hipStream_t st,
                                     int32_t *d_sums = nullptr, int row0 = 0, int nrows = 0)
    {
        const int SB = K / 256;
        if (mfma4_long_rows(SB))
            return gemv_mfma_q4k_long_launch(fn, d_w, d_plane, src, d_y, M, N, K, ldy, device_id, st, d_sums, row0, nrows);
        const MfmaShape sh = gemv_mfma_shape(N, SB, cu_count(device_id), d_sums ? MFMA_DUMP_WAVES : MFMA_MAX_WAVES);
        MfmaArgs a{};
        a.w = static_cast<const uint8_t *>(d_w);
        a.plane = static_cast<const uint8_t *>(d_plane);
        a.q8 = static_cast<const uint32_t *>(src.q8);
        a.x = src.x;
        a.x2 = src.x2;
        a.ldx = src.ldx;
        a.y = d_y;
        a.ldy = ldy;
        a.N = N;
        a.SB = SB;
        a.M = M;
        a.slices = sh.slices;
        a.tiles_per_wg = sh.tiles_per_wg;
        a.tile_rows = sh.tile_rows;
        a.sums = d_sums;
        a.row0 = row0;
        a.nrows = nrows;
        const dim3 grid((unsigned)sh.grid), block((unsigned)(sh.slices * sh.tiles_per_wg) * WAVE);
        const size_t lds = a.plane ? mfma_act_bytes(SB) : mfma_lds_bytes(SB, sh.slices * sh.tiles_per_wg);
        if (d_sums)
        {
            if (src.kind != ACT_SRC_Q8)
                return fail(fn, "block sums are dumped on Q8_1 input");
            if (a.plane)
                gemv_mfma_q4k_launch_src<QUAD_SRC_Q8, true, true>(grid, block, lds, st, a);
            else
                gemv_mfma_q4k_launch_src<QUAD_SRC_Q8, true>(grid, block, lds, st, a);
            return launched(fn);
        }
        if (a.plane)
        {
            switch (src.kind)
            {
            case ACT_SRC_F32: gemv_mfma_q4k_launch_src<QUAD_SRC_F32, false, true>(grid, block, lds, st, a); break;
            case ACT_SRC_SWIGLU: gemv_mfma_q4k_launch_src<QUAD_SRC_SWIGLU, false, true>(grid, block, lds, st, a); break;
            default: gemv_mfma_q4k_launch_src<QUAD_SRC_Q8, false, true>(grid, block, lds, st, a); break;
            }
            return launched(fn);
        }
        switch (src.kind)
        {
        case ACT_SRC_F32: gemv_mfma_q4k_launch_src<QUAD_SRC_F32>(grid, block, lds, st, a); break;
        case ACT_SRC_SWIGLU: gemv_mfma_q4k_launch_src<QUAD_SRC_SWIGLU>(grid, block, lds, st, a); break;
        default: gemv_mfma_q4k_launch_src<QUAD_SRC_Q8>(grid, block, lds, st, a); break;
        }
        return launched(fn);
    }

    // Smallest batch the entry points that NAME the matrix-unit kernels serve (the fused feed-forward launch, the
    // projection summed in two halves).  llam_ql_gemv keeps batches of up to 4 on the quad-lane kernel, whose rows
    // carry the bits of their single-row calls; a caller that does not need that (independent sequences of a
    // decode batch) is faster on the matrix unit from two rows on: the 64-layer decode step at batches of 2, 3 and 4
    // 279 -> 292, 359 -> 395 and 430 -> 500 tokens/s.
    constexpr int MFMA_NAMED_MIN_M = 2;
    // Gate and up projection with SwiGLU and the Q8_1 quantiser of the result in one launch
    // (gemv_mfma_q4k_kernel<.., SWIGLU>): Q4_K, batches of 5..8, rows the unchunked matrix-unit kernel
    // walks, N a multiple of 32; both matrices with a batch plane or neither.
    inline bool gemv_mfma_q4k_swiglu_ok(int M, int N, int K)
    {
        // (the shape rules of a batch of 5..8; the entry point itself serves smaller batches too: its caller asks
        // for the matrix unit by name and does not need a row to carry the bits of its single-row call)
        return M >= MFMA_NAMED_MIN_M && M <= 8 && K % 256 == 0 && mfma_eligible<Q4KTraits>(M < 5 ? 5 : M, N, K) &&
               !mfma4_long_rows(K / 256) && N % MFMA_TILE_ROWS == 0;
    }
    inline bool gemv_mfma_q4k_swiglu_launch(const char *fn, const void *d_w_gate, const void *d_plane_gate,
                                            const void *d_w_up, const void *d_plane_up, const void *d_q8,
                                            float *d_y_gate, float *d_y_up, int ldy, void *d_q8_out, int M, int N,
                                            int K, int device_id, hipStream_t st)
    {
        const int SB = K / 256;
        const MfmaShape sh = gemv_mfma_swiglu_shape(N, SB, cu_count(device_id));
        MfmaArgs a{};
        a.w = static_cast<const uint8_t *>(d_w_gate);
        a.plane = static_cast<const uint8_t *>(d_plane_gate);
        a.w2 = static_cast<const uint8_t *>(d_w_up);
        a.plane2 = static_cast<const uint8_t *>(d_plane_up);
        a.q8 = static_cast<const uint32_t *>(d_q8);
        a.y = d_y_gate;
        a.y2 = d_y_up;
        a.ldy = ldy;
        a.q8_out = static_cast<uint32_t *>(d_q8_out);
        a.N = N;
        a.SB = SB;
        a.M = M;
        a.slices = sh.slices;
        a.tiles_per_wg = sh.tiles_per_wg;
        a.tile_rows = MFMA_TILE_ROWS;
        const int waves = sh.slices * sh.tiles_per_wg;
        if (waves > MFMA_MAX_WAVES)
            return fail(fn, "launch shape of %d wavefronts (N=%d K=%d)", waves, N, K);
        const dim3 grid((unsigned)sh.grid), block((unsigned)waves * WAVE);
        const size_t lds = mfma_swiglu_lds_bytes(SB, waves, sh.tiles_per_wg, a.plane != nullptr);
        if (lds > QUAD_MAX_LDS)
            return fail(fn, "%zu bytes of LDS (N=%d K=%d)", lds, N, K);
        static LdsGrant grant_plane, grant_plain;
        if (a.plane)
        {
            (void)allow_lds(grant_plane, reinterpret_cast<const void *>(&gemv_mfma_q4k_kernel<QUAD_SRC_Q8, false, true, true>), QUAD_MAX_LDS);
            hipLaunchKernelGGL((gemv_mfma_q4k_kernel<QUAD_SRC_Q8, false, true, true>), grid, block, lds, st, a);
        }
        else
        {
            (void)allow_lds(grant_plain, reinterpret_cast<const void *>(&gemv_mfma_q4k_kernel<QUAD_SRC_Q8, false, false, true>), QUAD_MAX_LDS);
            hipLaunchKernelGGL((gemv_mfma_q4k_kernel<QUAD_SRC_Q8, false, false, true>), grid, block, lds, st, a);
        }
        return launched(fn);
    }

    template <int SRC, bool DUMP = false>
    void gemv_mfma_q6k_launch_src(dim3 grid, dim3 block, size_t lds, hipStream_t st, const Mfma6Args &a)
    {
        static LdsGrant grant;
        (void)allow_lds(grant, reinterpret_cast<const void *>(&gemv_mfma_q6k_kernel<SRC, DUMP>), QUAD_MAX_LDS);
        hipLaunchKernelGGL((gemv_mfma_q6k_kernel<SRC, DUMP>), grid, block, lds, st, a);
    }

    inline bool batch_plane_usable_q6k(int M, int N, int K)
    {
        return M >= 5 && M <= 8 && gemv_unroll_override() == 0 && gemv_rows_per_wave_override() == 0 && K / 256 >= 8 &&
               q6k_plane_bytes(N, K / 256) < ((size_t)1 << 32);
    }

    template <int SRC, bool DUMP = false>
    void gemv_mfma_q6k_plane_launch_src(dim3 grid, dim3 block, size_t lds, hipStream_t st, const Mfma6Args &a)
    {
        static LdsGrant grant;
        (void)allow_lds(grant, reinterpret_cast<const void *>(&gemv_mfma_q6k_plane_kernel<SRC, DUMP>), QUAD_MAX_LDS);
        hipLaunchKernelGGL((gemv_mfma_q6k_plane_kernel<SRC, DUMP>), grid, block, lds, st, a);
    }

    // d_plane: the matrix's batch plane (q6k_plane_bytes) or null; with one, the plane kernel runs,
    // also as the block-sum variant.
    inline bool gemv_mfma_q6k_launch(const char *fn, const void *d_w, const void *d_plane, const ActSource &src,
                                     float *d_y, int M, int N, int K, int ldy, int device_id, hipStream_t st,
                                     int32_t *d_sums = nullptr, int row0 = 0, int nrows = 0)
    {
        const int SB = K / 256;
        const uint8_t *plane = static_cast<const uint8_t *>(d_plane);
        const Mfma6Shape sh =
            gemv_mfma6_shape(N, SB, cu_count(device_id), plane ? MFMA6_PLANE_COMPUTE : d_sums ? MFMA6_DUMP_COMPUTE : MFMA6_MAX_COMPUTE,
                             plane != nullptr);
        Mfma6Args a{};
        a.ksplit = 1;
        a.w = static_cast<const uint8_t *>(d_w);
        a.plane = plane;
        a.q8 = static_cast<const uint32_t *>(src.q8);
        a.x = src.x;
        a.x2 = src.x2;
        a.ldx = src.ldx;
        a.y = d_y;
        a.ldy = ldy;
        a.N = N;
        a.SB = SB;
        a.M = M;
        a.slices = sh.slices;
        a.tiles = sh.tiles;
        a.tile_rows = sh.tile_rows;
        a.chunk = sh.chunk;
        a.sums = d_sums;
        a.row0 = row0;
        a.nrows = nrows;
        const dim3 grid((unsigned)sh.grid), block((unsigned)(sh.slices * sh.tiles + (plane ? MFMA6_PLANE_PRODUCERS : MFMA6_PRODUCERS)) * WAVE);
        const size_t lds = plane ? mfma6_act_bytes(SB, sh.chunk) : mfma6_lds_bytes(SB, sh.chunk, sh.slices * sh.tiles);
        if (d_sums)
        {
            if (src.kind != ACT_SRC_Q8)
                return fail(fn, "block sums are dumped on Q8_1 input");
            if (plane)
                gemv_mfma_q6k_plane_launch_src<QUAD_SRC_Q8, true>(grid, block, lds, st, a);
            else
                gemv_mfma_q6k_launch_src<QUAD_SRC_Q8, true>(grid, block, lds, st, a);
            return launched(fn);
        }
        if (plane)
        {
            switch (src.kind)
            {
            case ACT_SRC_F32: gemv_mfma_q6k_plane_launch_src<QUAD_SRC_F32>(grid, block, lds, st, a); break;
            case ACT_SRC_SWIGLU: gemv_mfma_q6k_plane_launch_src<QUAD_SRC_SWIGLU>(grid, block, lds, st, a); break;
            default: gemv_mfma_q6k_plane_launch_src<QUAD_SRC_Q8>(grid, block, lds, st, a); break;
            }
            return launched(fn);
        }
        switch (src.kind)
        {
        case ACT_SRC_F32: gemv_mfma_q6k_launch_src<QUAD_SRC_F32>(grid, block, lds, st, a); break;
        case ACT_SRC_SWIGLU: gemv_mfma_q6k_launch_src<QUAD_SRC_SWIGLU>(grid, block, lds, st, a); break;
        default: gemv_mfma_q6k_launch_src<QUAD_SRC_Q8>(grid, block, lds, st, a); break;
        }
        return launched(fn);
    }

    // The plane kernel with the rows' super-blocks in two halves, one workgroup per (two tiles, half): a
    // workgroup stages half of the batch's activations (what every workgroup stages of a long row costs as much
    // as its weights: 8 rows of K = 25600 are 230 KB), the halves' sums go to two outputs and the caller adds them.
    // Served for long rows only: each half must keep the wavefronts of a tile busy for several steps.
    inline bool gemv_mfma_q6k_split_ok(int M, int N, int K)
    {
        return M >= MFMA_NAMED_MIN_M && M <= 8 && K % 512 == 0 && K / 256 >= 64 && N >= 1 &&
               batch_plane_usable_q6k(M < 5 ? 5 : M, N, K);
    }
    inline bool gemv_mfma_q6k_split_launch(const char *fn, const void *d_plane, const void *d_q8, float *d_y_lo,
                                           float *d_y_hi, int M, int N, int K, int ldy, int device_id, hipStream_t st)
    {
        const int SB = K / 256;
        // the shape of a matrix with rows of half the length, two tiles per workgroup (half the wavefronts per tile)
        Mfma6Shape sh = gemv_mfma6_shape(N, SB / 2, cu_count(device_id), MFMA6_PLANE_COMPUTE, true);
        if (sh.tiles == 1 && sh.slices >= 2)
        {
            sh.tiles = 2;
            sh.slices /= 2;
            sh.grid = (sh.grid + 1) / 2;
            if (sh.chunk < SB / 2)
                sh.chunk = sh.chunk / sh.slices * sh.slices;
        }
        Mfma6Args a{};
        a.ksplit = 2;
        a.plane = static_cast<const uint8_t *>(d_plane);
        a.q8 = static_cast<const uint32_t *>(d_q8);
        a.y = d_y_lo;
        a.y2 = d_y_hi;
        a.ldy = ldy;
        a.N = N;
        a.SB = SB;
        a.M = M;
        a.slices = sh.slices;
        a.tiles = sh.tiles;
        a.tile_rows = sh.tile_rows;
        a.chunk = sh.chunk;
        const dim3 grid((unsigned)(sh.grid * 2)), block((unsigned)(sh.slices * sh.tiles + MFMA6_PLANE_PRODUCERS) * WAVE);
        const size_t lds = mfma6_act_bytes(SB / 2, sh.chunk);
        if (lds > QUAD_MAX_LDS || sh.chunk < sh.slices)
            return fail(fn, "launch shape (N=%d K=%d)", N, K);
        gemv_mfma_q6k_plane_launch_src<QUAD_SRC_Q8>(grid, block, lds, st, a);
        return launched(fn);
    }

    // The same for Q4_K rows the chunked kernel walks (gemv_mfma_q4k_long_kernel), from the matrix's batch plane.
    inline bool gemv_mfma_q4k_split_ok(int M, int N, int K)
    {
        return M >= 5 && M <= 8 && K % 512 == 0 && K / 256 >= 64 && N >= 1 && mfma_eligible<Q4KTraits>(M, N, K) &&
               mfma4_long_rows(K / 256) && q4k_plane_bytes(N, K / 256) < ((size_t)1 << 32);
    }
    inline bool gemv_mfma_q4k_split_launch(const char *fn, const void *d_plane, const void *d_q8, float *d_y_lo,
                                           float *d_y_hi, int M, int N, int K, int ldy, int device_id, hipStream_t st)
    {
        const int SB = K / 256;
        Mfma6Shape sh = gemv_mfma6_shape(N, SB / 2, cu_count(device_id), MFMA4_LONG_COMPUTE, true, MFMA_BOUNCE);
        if (sh.tiles == 1 && sh.slices >= 2)
        {
            sh.tiles = 2;
            sh.slices /= 2;
            sh.grid = (sh.grid + 1) / 2;
            if (sh.chunk < SB / 2)
                sh.chunk = sh.chunk / sh.slices * sh.slices;
        }
        MfmaLongArgs a{};
        a.ksplit = 2;
        a.plane = static_cast<const uint8_t *>(d_plane);
        a.q8 = static_cast<const uint32_t *>(d_q8);
        a.y = d_y_lo;
        a.y2 = d_y_hi;
        a.ldy = ldy;
        a.N = N;
        a.SB = SB;
        a.M = M;
        a.slices = sh.slices;
        a.tile_rows = sh.tile_rows;
        a.tiles = sh.tiles;
        a.chunk = sh.chunk;
        const dim3 grid((unsigned)(sh.grid * 2)), block((unsigned)(sh.slices * sh.tiles + MFMA4_LONG_PRODUCERS) * WAVE);
        const size_t lds = mfma6_act_bytes(SB / 2, sh.chunk);
        if (lds > QUAD_MAX_LDS || sh.chunk < sh.slices)
            return fail(fn, "launch shape (N=%d K=%d)", N, K);
        gemv_mfma_q4k_long_launch_src<QUAD_SRC_Q8, false, true>(grid, block, lds, st, a);
        return launched(fn);
    }

    // Whether a batch of M rows of this matrix is served from its batch plane when the caller
    // brings one: 5..8 rows, no tuning override in force; Q6_K: rows of eight super-blocks and
    // more, Q4_K: where the batch goes to the matrix-unit kernel anyway.
    template <class F>
    bool batch_plane_usable(int M, int N, int K)
    {
        if constexpr (F::USE_MFMA_BATCH)
            if (M >= 5 && M <= 8 && gemv_unroll_override() == 0 && gemv_rows_per_wave_override() == 0)
            {
                if constexpr (std::is_same<typename F::Quad, Q6KQuad>::value)
                    return K / 256 >= 8 && q6k_plane_bytes(N, K / 256) < ((size_t)1 << 32);
                else
                    return mfma_eligible<F>(M, N, K) && q4k_plane_bytes(N, K / 256) < ((size_t)1 << 32);
            }
        return false;
    }
    // The plane a launch reads: d_plane where it is usable, else null.
    template <class F>
    const void *batch_plane_for(const void *d_plane, int M, int N, int K)
    {
        return d_plane && batch_plane_usable<F>(M, N, K) ? d_plane : nullptr;
    }

    // The matrix-unit kernel of format F (mfma_eligible<F> or batch_plane_for<F> has said yes).
    template <class F>
    bool gemv_mfma_launch(const char *fn, const void *d_w, const void *d_plane, const ActSource &src, float *d_y,
                          int M, int N, int K, int ldy, int device_id, hipStream_t st, int32_t *d_sums = nullptr,
                          int row0 = 0, int nrows = 0)
    {
        if constexpr (std::is_same<typename F::Quad, Q6KQuad>::value)
            return gemv_mfma_q6k_launch(fn, d_w, d_plane, src, d_y, M, N, K, ldy, device_id, st, d_sums, row0, nrows);
        else
            return gemv_mfma_q4k_launch(fn, d_w, d_plane, src, d_y, M, N, K, ldy, device_id, st, d_sums, row0, nrows);
    }

    static_assert(ACT_SRC_Q8 == QUAD_SRC_Q8 && ACT_SRC_F32 == QUAD_SRC_F32 && ACT_SRC_SWIGLU == QUAD_SRC_SWIGLU &&
                      ACT_SRC_RMSNORM == QUAD_SRC_RMSNORM,
                  "activation source kinds");

    // Wavefronts that share the N rows of a matrix when none walks more than R.  (Rows are dealt
    // round robin, so any count would do; a count rounded up to a whole number per compute unit
    // measured no faster.)
    inline int quad_wavefronts(long N, int R, int) { return (int)((N + R - 1) / R); }

    // d_sums (one matrix, Q8_1 input): run the block-sum variant over rows [row0, row0+nrows).
    // accumulate (one matrix): QUAD_ACC_LAUNCH adds the row sums to what the output holds, which the
    // kernel can do where it reduces rows through the ring and a wavefront's rows fit one flush;
    // QUAD_ACC_QUERY only answers whether this launch could (no launch, no error text).
    constexpr int QUAD_ACC_NONE = 0, QUAD_ACC_LAUNCH = 1, QUAD_ACC_QUERY = 2;
    template <class F>
    bool gemv_quad_multi(const char *fn, const QuadProj *pr, int n, const ActSource &src, int M, int K,
                         int device_id, hipStream_t st, int32_t *d_sums = nullptr, int row0 = 0, int nrows = 0,
                         int accumulate = QUAD_ACC_NONE)
    {
        if constexpr (F::USE_QUAD)
        {
            const int SB = K / 256;
            const int cus = cu_count(device_id);
            const int max_waves = F::Quad::max_threads(M) / WAVE;
            QuadArgs a;
            a.q8 = static_cast<const uint32_t *>(src.q8);
            a.x = src.x;
            a.x2 = src.x2;
            a.ldx = src.ldx;
            a.gamma = src.gamma;
            a.x_out = src.x_out;
            a.eps = src.eps;
            a.norm_lds = 0;
            a.SB = SB;
            a.nproj = n;
            a.first_b = n;
            a.sums = d_sums;
            a.row0 = row0;
            a.nrows = nrows;
            if (d_sums && (n != 1 || src.kind != ACT_SRC_Q8))
                return fail(fn, "block sums are dumped for one matrix on Q8_1 input");
            long waves = 0;
            for (int i = 0; i < QUAD_MAX_PROJ; ++i)
            {
                const int j = i < n ? i : n - 1; // unused entries repeat the last matrix
                a.w[i] = pr[j].w;
                a.y[i] = pr[j].y;
                a.N[i] = pr[j].N;
                a.ldy[i] = pr[j].ldy;
                a.R[i] = gemv_quad_shape(pr[j].N, SB, cus, max_waves, F::Quad::RESIDENT_WAVES).rows_per_wave;
                a.TW[i] = quad_wavefronts(pr[j].N, a.R[i], cus);
                a.rows_min[i] = pr[j].N / a.TW[i];
                a.wave_begin[i] = (int)waves;
                if (i < n)
                    waves += a.TW[i];
            }
            if (waves > 0x7FFFFFFFL / WAVE)
                return fail(fn, "too many rows for one launch");
            // wavefronts per workgroup: an even share of what one compute unit gets
            const long wpc = (waves + cus - 1) / cus;
            const long wgs_per_cu = (wpc + max_waves - 1) / max_waves;
            long nw = (wpc + wgs_per_cu - 1) / wgs_per_cu;
            if (nw > waves)
                nw = waves;
            if (nw < 1)
                nw = 1;
            const long grid = (waves + nw - 1) / nw;
            size_t lds = quad_lds_bytes(M, SB);
            const size_t norm = src.kind == ACT_SRC_RMSNORM ? QUAD_NORM_LDS : 0;
            if (norm && M > QUAD_NORM_MAX_M)
                return fail(fn, "the fused norm serves batches of 1..%d", QUAD_NORM_MAX_M);
            // (the ring must not cost a compute unit one of the workgroups it would hold at once)
            a.ring = M <= QUAD_RING_MAX_M && !d_sums &&
                     (size_t)wgs_per_cu * (lds + norm + (size_t)nw * M * QUAD_RING_BYTES + F::Quad::STATIC_LDS) <=
                         QUAD_MAX_LDS;
            if (a.ring)
                lds += (size_t)nw * M * QUAD_RING_BYTES;
            a.norm_lds = (int)lds;
            lds += norm;
            if (lds + F::Quad::STATIC_LDS > QUAD_MAX_LDS)
                return fail(fn, "K=%d: %d activation row(s) and the norm's scratch do not fit the LDS", K, M);
            a.accumulate = 0;
            if (accumulate != QUAD_ACC_NONE)
            {
                const bool can = n == 1 && a.ring && a.R[0] <= QUAD_RING_ROWS;
                if (accumulate == QUAD_ACC_QUERY)
                    return can;
                if (!can)
                    return fail(fn, "M=%d N=%d K=%d: this launch cannot add to its output", M, pr[0].N, K);
                a.accumulate = 1;
            }
            gemv_quad_launch<typename F::Quad>(M, src.kind, dim3((unsigned)grid), dim3((unsigned)nw * WAVE), lds, st, a);
            return launched(fn);
        }
        else
        {
            (void)pr; (void)n; (void)src; (void)M; (void)K; (void)device_id; (void)st;
            return fail(fn, "format has no quad-lane kernel");
        }
    }

    // The same over two runs of matrices in two formats (na of FA, then nb of FB; na + nb <=
    // QUAD_MAX_PROJ), Q8_1 or plain fp32 activations.  The second format starts at a
    // workgroup boundary.
    // What a two-format launch is made of.  force_nw: wavefronts per workgroup the caller needs (0: chosen here).
    struct QuadDualLaunch
    {
        QuadArgs a;
        long grid, nw;
        size_t lds;
    };
    template <class FA, class FB>
    bool gemv_quad_dual_setup(const char *fn, const QuadProj *pr, int na, int nb, const ActSource &src, int M, int K,
                              int device_id, int force_nw, QuadDualLaunch &out)
    {
        if constexpr (FA::USE_QUAD && FB::USE_QUAD)
        {
            typedef typename FA::Quad QA;
            typedef typename FB::Quad QB;
            QuadArgs &a = out.a;
            const int SB = K / 256;
            const int cus = cu_count(device_id);
            const int mta = QA::max_threads(M), mtb = QB::max_threads(M);
            const int max_waves = (mta < mtb ? mta : mtb) / WAVE;
            const int n = na + nb;
            a.q8 = static_cast<const uint32_t *>(src.q8);
            a.x = src.x;
            a.x2 = src.x2;
            a.ldx = src.ldx;
            a.gamma = src.gamma;
            a.x_out = src.x_out;
            a.eps = src.eps;
            a.norm_lds = 0;
            a.SB = SB;
            a.nproj = n;
            a.first_b = na;
            a.sums = nullptr;
            a.row0 = a.nrows = 0;
            a.accumulate = 0;
            long cnt[QUAD_MAX_PROJ], waves = 0;
            for (int i = 0; i < QUAD_MAX_PROJ; ++i)
            {
                const int j = i < n ? i : n - 1;
                a.w[i] = pr[j].w;
                a.y[i] = pr[j].y;
                a.N[i] = pr[j].N;
                a.ldy[i] = pr[j].ldy;
                // every matrix keeps the rows per wavefront of its own single launch
                const int resident = j < na ? QA::RESIDENT_WAVES : QB::RESIDENT_WAVES;
                const int own_max = (j < na ? mta : mtb) / WAVE;
                a.R[i] = gemv_quad_shape(pr[j].N, SB, cus, own_max, resident).rows_per_wave;
                a.TW[i] = quad_wavefronts(pr[j].N, a.R[i], cus);
                a.rows_min[i] = pr[j].N / a.TW[i];
                cnt[i] = i < n ? a.TW[i] : 0;
                waves += cnt[i];
            }
            const long wpc = (waves + cus - 1) / cus;
            const long wgs_per_cu = (wpc + max_waves - 1) / max_waves;
            long nw = (wpc + wgs_per_cu - 1) / wgs_per_cu;
            if (nw > waves)
                nw = waves;
            if (nw < 1)
                nw = 1;
            if (force_nw > 0)
            {
                if (force_nw > max_waves)
                    return fail(fn, "workgroups of %d wavefronts at M=%d", force_nw, M);
                nw = force_nw;
            }
            long at = 0;
            for (int i = 0; i < QUAD_MAX_PROJ; ++i)
            {
                if (i == na)
                    at = (at + nw - 1) / nw * nw; // the second format starts a workgroup
                a.wave_begin[i] = (int)at;
                at += cnt[i];
            }
            if (at > 0x7FFFFFFFL / WAVE)
                return fail(fn, "too many rows for one launch");
            const long grid = (at + nw - 1) / nw;
            size_t lds = quad_lds_bytes(M, SB);
            const size_t norm = src.kind == ACT_SRC_RMSNORM ? QUAD_NORM_LDS : 0;
            if (norm && M > QUAD_NORM_MAX_M)
                return fail(fn, "the fused norm serves batches of 1..%d", QUAD_NORM_MAX_M);
            a.ring = M <= QUAD_RING_MAX_M &&
                     (size_t)wgs_per_cu * (lds + norm + (size_t)nw * M * QUAD_RING_BYTES) <= QUAD_MAX_LDS;
            if (a.ring)
                lds += (size_t)nw * M * QUAD_RING_BYTES;
            a.norm_lds = (int)lds;
            lds += norm;
            if (lds > QUAD_MAX_LDS)
                return fail(fn, "K=%d: %d activation row(s) and the norm's scratch do not fit the LDS", K, M);
            out.grid = grid;
            out.nw = nw;
            out.lds = lds;
            return true;
        }
        else
        {
            (void)pr; (void)na; (void)nb; (void)src; (void)M; (void)K; (void)device_id; (void)force_nw; (void)out;
            return fail(fn, "formats have no quad-lane kernel");
        }
    }

    template <class FA, class FB>
    bool gemv_quad_dual(const char *fn, const QuadProj *pr, int na, int nb, const ActSource &src, int M, int K,
                        int device_id, hipStream_t st)
    {
        if constexpr (FA::USE_QUAD && FB::USE_QUAD)
        {
            QuadDualLaunch L;
            if (!gemv_quad_dual_setup<FA, FB>(fn, pr, na, nb, src, M, K, device_id, 0, L))
                return false;
            gemv_quad_dual_launch<typename FA::Quad, typename FB::Quad>(M, src.kind, dim3((unsigned)L.grid),
                                                                         dim3((unsigned)L.nw * WAVE), L.lds, st, L.a);
            return launched(fn);
        }
        else
        {
            (void)pr; (void)na; (void)nb; (void)src; (void)M; (void)K; (void)device_id; (void)st;
            return fail(fn, "formats have no quad-lane kernel");
        }
    }

    // ---- a matrix-unit matrix and a quad-lane group in ONE launch (batches of 5..8) -------------------------------
    // Q (thousands of rows: the matrix unit) and K, V (a thousand rows each: the quad-lane kernel) read the
    // same activations and used to be two launches of about 10 us each, most of it the latency chain of a
    // launch.  Here the first workgroups of the launch run the matrix-unit body on Q, the others the
    // quad-lane bodies on the group: every matrix keeps the tiling, slices and rows per wavefront of its
    // own launch, so the results are those of the separate launches bit for bit.
    constexpr int MIXED_WAVES = 8; // wavefronts per workgroup: what the quad-lane kernels run at these batches
    template <bool PLANE, int M>
    __global__ void __launch_bounds__(MIXED_WAVES *WAVE)
        gemv_mfma_quad_kernel(const MfmaArgs a, const QuadArgs qa, const int mfma_blocks)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t mixed_lds[];
        if ((int)blockIdx.x < mfma_blocks) // uniform per workgroup
        {
            gemv_mfma_q4k_body<QUAD_SRC_Q8, false, PLANE, false>(a, mixed_lds, (int)blockIdx.x);
            return;
        }
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int wid_all = ((int)blockIdx.x - mfma_blocks) * MIXED_WAVES + wave;
        int p, w_first;
        quad_which(qa, wid_all, p, w_first);
        if (p < qa.first_b)
            quad_body<Q4KQuad, M, quad_unroll<Q4KQuad>(M), QUAD_SRC_Q8>(qa, mixed_lds, p, w_first, wid_all);
        else
            quad_body<Q6KQuad, M, quad_unroll<Q6KQuad>(M), QUAD_SRC_Q8>(qa, mixed_lds, p, w_first, wid_all);
    }

    template <bool PLANE, int M>
    void gemv_mfma_quad_launch_pm(dim3 grid, size_t lds, hipStream_t st, const MfmaArgs &a, const QuadArgs &qa,
                                  int mfma_blocks)
    {
        static LdsGrant grant;
        (void)allow_lds(grant, reinterpret_cast<const void *>(&gemv_mfma_quad_kernel<PLANE, M>), QUAD_MAX_LDS);
        hipLaunchKernelGGL((gemv_mfma_quad_kernel<PLANE, M>), grid, dim3(MIXED_WAVES * WAVE), lds, st, a, qa, mfma_blocks);
    }

    // Whether the Q4_K matrix's own matrix-unit launch fits workgroups of MIXED_WAVES wavefronts (then the
    // mixed launch can run it unchanged).
    inline bool gemv_mfma_quad_ok(int M, int N, int K, int device_id)
    {
        if (M < 5 || M > 8 || !mfma_eligible<Q4KTraits>(M, N, K) || mfma4_long_rows(K / 256))
            return false;
        const MfmaShape sh = gemv_mfma_shape(N, K / 256, cu_count(device_id), MFMA_MAX_WAVES);
        return sh.slices * sh.tiles_per_wg <= MIXED_WAVES;
    }

    // d_w / d_plane / d_y / N / ldy: the matrix-unit matrix (Q4_K); pr: na Q4_K then nb Q6_K matrices for the
    // quad-lane kernel (na + nb >= 1); Q8_1 activations.
    inline bool gemv_mfma_quad_launch(const char *fn, const void *d_w, const void *d_plane, float *d_y, int N, int ldy,
                                      const QuadProj *pr, int na, int nb, const void *d_q8, int M, int K,
                                      int device_id, hipStream_t st)
    {
        const int SB = K / 256;
        const MfmaShape sh = gemv_mfma_shape(N, SB, cu_count(device_id), MFMA_MAX_WAVES);
        MfmaArgs a{};
        a.w = static_cast<const uint8_t *>(d_w);
        a.plane = static_cast<const uint8_t *>(d_plane);
        a.q8 = static_cast<const uint32_t *>(d_q8);
        a.y = d_y;
        a.ldy = ldy;
        a.N = N;
        a.SB = SB;
        a.M = M;
        a.slices = sh.slices;
        a.tiles_per_wg = sh.tiles_per_wg;
        a.tile_rows = sh.tile_rows;
        QuadDualLaunch L;
        if (!gemv_quad_dual_setup<Q4KTraits, Q6KTraits>(fn, pr, na, nb, act_source_q8(d_q8), M, K, device_id, MIXED_WAVES, L))
            return false;
        const size_t lds_mfma = a.plane ? mfma_act_bytes(SB) : mfma_lds_bytes(SB, sh.slices * sh.tiles_per_wg);
        // (the partial sums of all eight wavefronts lie over the activations at the end)
        const size_t lds = lds_mfma > L.lds ? lds_mfma : L.lds;
        if (lds > QUAD_MAX_LDS || lds < (size_t)MIXED_WAVES * 4 * WAVE * sizeof(float))
            return fail(fn, "%zu bytes of LDS (N=%d K=%d)", lds, N, K);
        const dim3 grid((unsigned)(sh.grid + L.grid));
        const int mb = (int)sh.grid;
#define LLAM_MIXED_CASE(m)                                                                                             \
    case m:                                                                                                            \
        if (a.plane)                                                                                                   \
            gemv_mfma_quad_launch_pm<true, m>(grid, lds, st, a, L.a, mb);                                              \
        else                                                                                                           \
            gemv_mfma_quad_launch_pm<false, m>(grid, lds, st, a, L.a, mb);                                             \
        break;
        switch (M)
        {
            LLAM_MIXED_CASE(5)
            LLAM_MIXED_CASE(6)
            LLAM_MIXED_CASE(7)
        default:
            LLAM_MIXED_CASE(8)
        }
#undef LLAM_MIXED_CASE
        return launched(fn);
    }

    // What the launcher does with a shape: the one place where the kernel, the batch split and
    // the K slices are decided.  gemv_launch() executes a plan; llam_ql_gemv_describe() reports it.
    constexpr int GEMV_KERNEL_GENERIC = 0; // gemv_kernel: rows shorter than 5 super-blocks
    constexpr int GEMV_KERNEL_CHUNKED = 1; // gemv_fast_kernel
    constexpr int GEMV_KERNEL_QUAD = 2;    // gemv_quad_kernel
    constexpr int GEMV_KERNEL_MFMA = 3;    // gemv_mfma_q4k_kernel / gemv_mfma_q6k_kernel
    struct GemvPlan
    {
        int kernel;        // GEMV_KERNEL_*; -1: the shape cannot be served
        int m_first;       // batch rows of the first launch group; the rest (M - m_first > 0) is
                           // planned and launched the same way after it
        int slice_sb;      // super-blocks per K slice (generic and chunked kernels; others: the row)
        int rows_per_wave; // row (batches) a wavefront walks
        int unroll;        // load batches in flight (chunked kernel)
        int gshift;        // 8-lane groups per row, log2 (generic and chunked kernels)
        long grid;
    };

    template <class F>
    GemvPlan gemv_plan(int M, int N, int K, int device_id)
    {
        const int SB = K / 256;
        GemvPlan p{};
        p.m_first = M;
        p.slice_sb = SB;
        if constexpr (F::USE_MFMA_BATCH)
            if (mfma_eligible<F>(M, N, K))
            {
                p.kernel = GEMV_KERNEL_MFMA;
                return p;
            }
        // Rows of at least 16 super-blocks in a format with a quad-lane decoder: the
        // quad kernel, which stages whole activation rows (up to 160 KiB of LDS).
        if constexpr (F::USE_QUAD)
            if (SB >= QUAD_STEP_SB && gemv_unroll_override() == 0 && F::Quad::addressable(N, SB))
            {
                p.kernel = GEMV_KERNEL_QUAD;
                if (quad_lds_bytes(M, SB) + F::Quad::STATIC_LDS > QUAD_MAX_LDS)
                {
                    if (M == 1)
                    {
                        p.kernel = -1; // one activation row does not fit the LDS
                        return p;
                    }
                    p.m_first = M / 2;
                }
                const QuadShape sh = gemv_quad_shape(N, SB, cu_count(device_id), F::Quad::max_threads(p.m_first) / WAVE,
                                                     F::Quad::RESIDENT_WAVES);
                p.rows_per_wave = sh.rows_per_wave;
                p.grid = sh.grid;
                return p;
            }
        // batch sizes without a dedicated kernel are run as 4 + (M-4)
        if (M > 4 && M < 8)
            p.m_first = 4;
        // K slices keep the staged activations (+ tables) within 64 KiB of LDS.
        int slice = (64 * 1024 - F::TABLE_BYTES) / (p.m_first * GEMV_LDS_PER_SB);
        if (slice > SB)
            slice = SB;
        if (slice < 1)
        {
            p.kernel = -1;
            return p;
        }
        const int m_first = p.m_first;
        const GemvShape sh = gemv_shape(N, slice, cu_count(device_id), F::FAST_MAX_U, [=](int U) {
            return gemv_fast_resident_waves<F>(m_first, U, gemv_lds_bytes<F>(m_first, slice));
        });
        p.kernel = sh.gshift == 3 ? GEMV_KERNEL_CHUNKED : GEMV_KERNEL_GENERIC;
        p.slice_sb = slice;
        p.rows_per_wave = sh.rpw;
        p.unroll = sh.U;
        p.gshift = sh.gshift;
        p.grid = sh.grid;
        return p;
    }

    // Whether every activation row of an M-row call gets the bits of its own M = 1 call: the
    // same kernel walks the same rows and K slices in the same order for both batch sizes.
    // (The quad-lane kernel picks its rows per wavefront from N and K alone and a batch split
    // runs the same kernel on each part; the chunked and generic kernels add a lane's
    // super-blocks in ascending order whatever the unroll, so only the K slicing, which
    // shrinks with M, can differ; the matrix-unit kernels add blocks in another order.)
    template <class F>
    bool gemv_decode_equivalent(int M, int N, int K, int device_id)
    {
        const GemvPlan one = gemv_plan<F>(1, N, K, device_id);
        for (int m0 = 0; m0 < M;)
        {
            const GemvPlan p = gemv_plan<F>(M - m0, N, K, device_id);
            if (p.kernel < 0 || one.kernel < 0 || p.kernel != one.kernel || p.kernel == GEMV_KERNEL_MFMA)
                return false;
            if (p.kernel != GEMV_KERNEL_QUAD && (p.slice_sb != one.slice_sb || p.gshift != one.gshift))
                return false;
            m0 += p.m_first;
        }
        return true;
    }

    // Shared host launcher.  Arguments are validated by the callers; the device
    // is current.  M is 1..8.  With d_sums the same plan is executed with the chosen kernel's
    // block-sum variant: the parity hook reads the integer pipeline that serves this
    // (format, M, N, K).
    // d_plane: the matrix's batch plane or null; a batch it serves goes to the plane kernel
    // whatever the plan says for the matrix alone.
    template <class F>
    bool gemv_launch(const char *fn, const void *d_w, const void *d_plane, const void *d_q8, float *d_y,
                     int32_t *d_sums, int M, int N, int K, int ldy, int row0, int nrows, int device_id, hipStream_t st)
    {
        const int SB = K / 256;
        const bool dump = d_sums != nullptr;
        if constexpr (F::USE_MFMA_BATCH)
            if (const void *plane = batch_plane_for<F>(d_plane, M, N, K))
                return gemv_mfma_launch<F>(fn, d_w, plane, act_source_q8(d_q8), d_y, M, N, K, ldy, device_id, st,
                                           d_sums, row0, nrows);
        const GemvPlan p = gemv_plan<F>(M, N, K, device_id);
        if (p.kernel < 0)
            return fail(fn, "K=%d is too long for %d activation row(s) in LDS", K, p.m_first);
        if (p.m_first < M)
        {
            // the first p.m_first rows now, the others after them
            if (!gemv_launch<F>(fn, d_w, nullptr, d_q8, d_y, d_sums, p.m_first, N, K, ldy, row0, nrows, device_id, st))
                return false;
            const uint8_t *q8b = static_cast<const uint8_t *>(d_q8) + (size_t)p.m_first * (K / 32) * 36;
            return gemv_launch<F>(fn, d_w, nullptr, q8b, d_y ? d_y + (size_t)p.m_first * ldy : nullptr,
                                  d_sums ? d_sums + (size_t)p.m_first * nrows * (K / 32) : nullptr, M - p.m_first, N,
                                  K, ldy, row0, nrows, device_id, st);
        }
        if constexpr (F::USE_MFMA_BATCH)
            if (p.kernel == GEMV_KERNEL_MFMA)
                return gemv_mfma_launch<F>(fn, d_w, nullptr, act_source_q8(d_q8), d_y, M, N, K, ldy, device_id, st,
                                           d_sums, row0, nrows);
        if constexpr (F::USE_QUAD)
            if (p.kernel == GEMV_KERNEL_QUAD)
            {
                QuadProj one{d_w, d_y, N, ldy};
                return gemv_quad_multi<F>(fn, &one, 1, act_source_q8(d_q8), M, K, device_id, st, d_sums, row0, nrows);
            }
        for (int sb0 = 0; sb0 < SB; sb0 += p.slice_sb)
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
            a.nsb = (SB - sb0 < p.slice_sb) ? (SB - sb0) : p.slice_sb;
            a.rows_per_wave = p.rows_per_wave;
            a.gshift = p.gshift;
            a.accumulate = sb0 > 0;
            a.out_scale = 1.0f;
            a.row0 = row0;
            a.nrows = nrows;
            a.pairs = nullptr;
            a.pair_div = 1;
            const size_t lds = gemv_lds_bytes<F>(M, a.nsb);
            if (p.kernel == GEMV_KERNEL_CHUNKED)
                gemv_fast_launch<F>(M, p.unroll, dim3((unsigned)p.grid), lds, st, a);
            else
                gemv_launch_m<F>(M, dump, dim3((unsigned)p.grid), lds, st, a);
            if (!launched(fn))
                return false;
        }
        return true;
    }
} // namespace llamql
