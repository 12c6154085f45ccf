// Q6_K x Q8_1 decode GEMV for batches of 5..8 activation rows on the matrix unit.
//
// The exact 8.8 fixed-point requantisation of the 6-bit weights is what a Q6_K product costs
// (several vector instructions per weight; its per-block factors and scales come ready-made
// from the factor plane of the prepared layout).  The quad-lane kernel keeps four activation rows
// in LDS at most when the row is long, so a batch of eight pays that requantisation twice.
// Here every weight is requantised once: lane (r = l%32, h = l/32) turns elements
// 16h..16h+15 of each 32-column block of weight row r into int8 (one Q6_K sub-scale covers
// exactly those 16 elements) and hands them to v_mfma_i32_32x32x32_i8 as the B operand; the A
// operand is the batch's activations from LDS, the result the reference's per-block int32
// sums of rows 4h..4h+3, rescaled in fp32 in ascending block order (gemv_mfma.h has the
// operand layout).
//
// Long rows do not fit the LDS (K = 25600, eight rows: 269 KB): the row is walked in chunks
// of at most 30 super-blocks, staged alternately into two LDS buffers by two producer
// wavefronts of the workgroup while the compute wavefronts work on the other buffer -- one
// barrier per chunk.  The compute wavefronts of a 32-row tile share the super-blocks round
// robin (wavefront j takes j, j + slices, ..); with the chunk a multiple of `slices` that
// sequence does not depend on the chunking.  Their partial sums are added in wavefront order.
//
// Weight loads are coalesced: of the 32 x 128 bytes of ql and 32 x 64 bytes of qh of a step,
// lane l loads the 16-byte pieces l, l+64, .. (eight neighbouring lanes cover a row's cache
// line of ql) and the wavefront passes them through a private LDS buffer to the two lanes of
// the row (rows 144 and 80 bytes apart there, so that the 128-bit reads of neighbouring rows
// fall into different banks).  The 32 bytes of factor records of a row's super-block go
// straight to its two lanes.  No barrier for the buffer: LDS instructions of one wavefront run
// in order.
#pragma once
#include "gemv_mfma.h"
#include <type_traits>

namespace llamql
{
    constexpr int MFMA6_PRODUCERS = 2;     // wavefronts that only stage activations
    constexpr int MFMA6_MAX_COMPUTE = 8;   // compute wavefronts per workgroup
    constexpr int MFMA6_DUMP_COMPUTE = 6;  // the same for the block-sum variant
    constexpr int MFMA6_LOADS = 8;         // vector memory loads per super-block and lane
    constexpr int MFMA6_QL_STRIDE = 144;   // bounce buffer: bytes between the ql lines of two rows
    constexpr int MFMA6_QH_STRIDE = 80;    // and between their 64 bytes of qh
    constexpr int MFMA6_BOUNCE = 32 * (MFMA6_QL_STRIDE + MFMA6_QH_STRIDE); // per compute wavefront

    struct Mfma6Args
    {
        const uint8_t *w;   // prepared Q6_K planes: ql | qh | scales | d over all N*SB super-blocks
        const uint8_t *plane; // PLANE kernels: the matrix's batch plane (q6k_plane_bytes), w is not read
        const uint32_t *q8; // Q8_1 activations as dwords (QUAD_SRC_Q8)
        const float *x;     // fp32 rows (QUAD_SRC_F32); the gate rows for QUAD_SRC_SWIGLU
        const float *x2;    // the up rows for QUAD_SRC_SWIGLU
        int ldx;
        float *y;
        int ldy;
        int N;
        int SB;     // super-blocks per weight row
        int M;      // activation rows, 1..8
        int slices; // compute wavefronts per tile
        int tile_rows; // weight rows of a tile, 1..32 (gemv_mfma.h)
        int tiles;  // tiles per workgroup
        int chunk;  // super-blocks per activation buffer; a multiple of slices when SB > chunk
        // DUMP kernels only: the exact per-block int32 sums of rows [row0, row0+nrows) go to
        // sums[(m * nrows + row - row0) * (SB * 8) + block]
        int32_t *sums;
        int row0, nrows;
        // gemv_mfma_q6k_plane_kernel only: the row's super-blocks in ksplit (1 or 2) equal parts, one workgroup
        // per (tiles, part); part 1's sums go to y2 (the caller adds the two)
        int ksplit;
        float *y2;
    };

    struct Mfma6Raw
    {
        v4i ql0, ql1, ql2, ql3, qh0, qh1, fc0, fc1;
    };
    // Plane bases advanced to the step's super-block (wavefront-uniform, scalar registers) and
    // this lane's byte offsets from them: four pieces of ql, two of qh, its row's factor records.
    struct Mfma6Ptr
    {
        const uint8_t *ql, *qh, *fc;
    };
    struct Mfma6Off
    {
        uint32_t ql[4], qh[2], fc;
    };
    __device__ __forceinline__ void mfma6_load(Mfma6Raw &r, const Mfma6Ptr &p, const Mfma6Off &o)
    {
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.ql0) : "v"(o.ql[0]), "s"(p.ql));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.ql1) : "v"(o.ql[1]), "s"(p.ql));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.ql2) : "v"(o.ql[2]), "s"(p.ql));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.ql3) : "v"(o.ql[3]), "s"(p.ql));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.qh0) : "v"(o.qh[0]), "s"(p.qh));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.qh1) : "v"(o.qh[1]), "s"(p.qh));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.fc0) : "v"(o.fc), "s"(p.fc));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:16" : "=&v"(r.fc1) : "v"(o.fc), "s"(p.fc));
    }
    // The same for the batch plane: the eight blocks of this lane's row, ready as operands, and
    // the row's eight block scales.
    constexpr int MFMA6_PLANE_LOADS = 9;
    constexpr int MFMA6_PLANE_PRODUCERS = 2; // wavefronts that only stage activations there (4: 33.8 against 34.5 us at batch 8, 31.4 against 30.4 us at batch 5)
    constexpr int MFMA6_PLANE_COMPUTE = 8; // compute wavefronts per workgroup of the plane kernel (12: 39.9 us, 14: 38.9 us against 34.7 us at 5120 x 25600)
    struct Mfma6PlaneRaw
    {
        v4i w0, w1, w2, w3, w4, w5, w6, w7, sc;
    };
    __device__ __forceinline__ void mfma6_plane_load(Mfma6PlaneRaw &r, const uint8_t *pw, const uint8_t *ps, uint32_t ow,
                                                     uint32_t os)
    {
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.w0) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:128" : "=&v"(r.w1) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:256" : "=&v"(r.w2) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:384" : "=&v"(r.w3) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:512" : "=&v"(r.w4) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:640" : "=&v"(r.w5) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:768" : "=&v"(r.w6) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:896" : "=&v"(r.w7) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.sc) : "v"(os), "s"(ps));
    }
    __device__ __forceinline__ void mfma6_keep(Mfma6PlaneRaw &r)
    {
        asm volatile(""
                     : "+v"(r.w0), "+v"(r.w1), "+v"(r.w2), "+v"(r.w3), "+v"(r.w4), "+v"(r.w5), "+v"(r.w6), "+v"(r.w7),
                       "+v"(r.sc));
    }
    template <int NEWER>
    __device__ __forceinline__ void mfma6_wait(Mfma6PlaneRaw &r)
    {
        asm volatile("s_waitcnt vmcnt(%9)"
                     : "+v"(r.w0), "+v"(r.w1), "+v"(r.w2), "+v"(r.w3), "+v"(r.w4), "+v"(r.w5), "+v"(r.w6), "+v"(r.w7),
                       "+v"(r.sc)
                     : "n"(NEWER));
    }
    __device__ __forceinline__ void mfma6_keep(Mfma6Raw &r)
    {
        asm volatile(""
                     : "+v"(r.ql0), "+v"(r.ql1), "+v"(r.ql2), "+v"(r.ql3), "+v"(r.qh0), "+v"(r.qh1), "+v"(r.fc0),
                       "+v"(r.fc1));
    }
    template <int NEWER>
    __device__ __forceinline__ void mfma6_wait(Mfma6Raw &r)
    {
        asm volatile("s_waitcnt vmcnt(%8)"
                     : "+v"(r.ql0), "+v"(r.ql1), "+v"(r.ql2), "+v"(r.ql3), "+v"(r.qh0), "+v"(r.qh1), "+v"(r.fc0),
                       "+v"(r.fc1)
                     : "n"(NEWER));
    }

    // Workgroup barrier of a compute wavefront: its own LDS reads are done (their results have
    // been consumed), and it must NOT wait for its weight loads in flight, which a
    // __syncthreads() would.  The producers publish their LDS writes with __syncthreads().
    __device__ __forceinline__ void mfma6_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

    __host__ __device__ inline size_t mfma6_act_bytes(int nsb, int chunk)
    {
        return mfma_act_bytes(chunk) * (nsb > chunk ? 2 : 1);
    }
    inline size_t mfma6_lds_bytes(int nsb, int chunk, int ncomp)
    {
        return mfma6_act_bytes(nsb, chunk) + (size_t)ncomp * MFMA6_BOUNCE;
    }

    // DUMP: also store the matrix unit's results, the exact int32 block sums (the parity hook).
    // Its stores need a few registers more than ten wavefronts leave each lane (and the build
    // refuses to spill): the variant runs with at most MFMA6_DUMP_COMPUTE compute wavefronts.
    template <int SRC, bool DUMP = false>
    __global__ void __launch_bounds__(((DUMP ? MFMA6_DUMP_COMPUTE : MFMA6_MAX_COMPUTE) + MFMA6_PRODUCERS) * WAVE)
        gemv_mfma_q6k_kernel(const Mfma6Args a)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t mfma6_lds[];
        const int nsb = a.SB;
        const int nph = (nsb + a.chunk - 1) / a.chunk; // activation chunks
        const size_t buf_bytes = mfma_act_bytes(a.chunk);
        const int ncomp = a.slices * a.tiles; // compute wavefronts
        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};

        auto buf_aq = [&](int ph) { return mfma6_lds + (size_t)(ph & 1) * buf_bytes; };
        auto buf_asc = [&](int ph) {
            return reinterpret_cast<float *>(mfma6_lds + (size_t)(ph & 1) * buf_bytes + (size_t)a.chunk * 8 * MFMA_AQ_STRIDE);
        };

        // chunk ph into its buffer, by `nthreads` threads that keep UN loads in flight each
        auto stage = [&](int ph, int tid, int nthreads, auto un) {
            const int c0 = ph * a.chunk;
            const int c1 = c0 + a.chunk < nsb ? c0 + a.chunk : nsb;
            mfma_stage_acts<SRC, decltype(un)::value>(a.q8, a.x, a.x2, a.ldx, a.M, nsb * 8, c0 * 8, (c1 - c0) * 8,
                                                      buf_aq(ph), buf_asc(ph), tid, nthreads);
        };
        typedef std::integral_constant<int, 3> Together; // everybody stages the first chunk
        typedef std::integral_constant<int, 8> Alone;    // two wavefronts stage the others: a chunk of 16
                                                         // super-blocks is 8 blocks a thread, all in flight

        if (wave >= ncomp)
        {
            // ---- producers: the first chunk together with everybody, then chunk ph+1 into the
            // buffer nobody reads during chunk ph ------------------------------------------------
            stage(0, (int)threadIdx.x, (int)blockDim.x, Together());
            __syncthreads();
            for (int ph = 0; ph + 1 < nph; ++ph)
            {
                stage(ph + 1, (int)threadIdx.x - ncomp * WAVE, MFMA6_PRODUCERS * WAVE, Alone());
                __syncthreads();
            }
        }
        else
        {
            // ---- compute wavefronts --------------------------------------------------------------
            const int l32 = lane & 31, lh = lane >> 5;
            const uint32_t lh_second = lh ? Q6K_CODE_BIG1 : 0u; // the record bit that says this lane's sub-scale is the larger one
            const int tile_local = wave / a.slices, slice = wave - tile_local * a.slices;
            const int nsteps = slice < nsb ? (nsb - slice + a.slices - 1) / a.slices : 0;
            const int last_step = nsteps > 0 ? nsteps - 1 : 0;
            const long tile_row0 = ((long)blockIdx.x * a.tiles + tile_local) * a.tile_rows;
            const size_t T = (size_t)a.N * nsb;
            // rows past the end of the tile or of the matrix re-read the last one
            auto sb_index = [&](int local_row) {
                const long r = tile_row0 + (local_row < a.tile_rows ? local_row : a.tile_rows - 1);
                return (uint32_t)((r < a.N ? r : a.N - 1) * nsb);
            };
            Mfma6Off off;
#pragma unroll
            for (int i = 0; i < 4; ++i) // ql piece lane + 64 i: row (lane >> 3) + 8 i, 16 bytes at 16 (lane & 7)
                off.ql[i] = sb_index((lane >> 3) + 8 * i) * 128u + 16u * (uint32_t)(lane & 7);
#pragma unroll
            for (int i = 0; i < 2; ++i) // qh piece lane + 64 i: row (lane >> 2) + 16 i, 16 bytes at 16 (lane & 3)
                off.qh[i] = sb_index((lane >> 2) + 16 * i) * 64u + 16u * (uint32_t)(lane & 3);
            off.fc = sb_index(l32) * 32u;
            uint8_t *bounce = mfma6_lds + mfma6_act_bytes(nsb, a.chunk) + (size_t)wave * MFMA6_BOUNCE;
            uint8_t *wr_ql = bounce + (lane >> 3) * MFMA6_QL_STRIDE + (lane & 7) * 16;  // piece i at + 8 i rows
            uint8_t *wr_qh = bounce + 32 * MFMA6_QL_STRIDE + (lane >> 2) * MFMA6_QH_STRIDE + (lane & 3) * 16;
            const uint8_t *rd_ql = bounce + l32 * MFMA6_QL_STRIDE + 16 * lh;            // piece c at + 32 c
            const uint8_t *rd_qh = bounce + 32 * MFMA6_QL_STRIDE + l32 * MFMA6_QH_STRIDE + 16 * lh;

            // loads are never predicated: past its last step a lane re-reads that step
            auto issue = [&](Mfma6Raw &r, int step) {
                const uint32_t sb = nsteps > 0 ? (uint32_t)(slice + (step < last_step ? step : last_step) * a.slices) : 0u;
                auto uniform = [](const uint8_t *p) {
                    const uint64_t b = (uint64_t)p;
                    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
                    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
                    return reinterpret_cast<const uint8_t *>(((uint64_t)hi << 32) | lo);
                };
                Mfma6Ptr pl;
                pl.ql = uniform(a.w + (size_t)sb * 128);
                pl.qh = uniform(a.w + T * 128 + (size_t)sb * 64);
                pl.fc = uniform(a.w + q6k_factors_offset(T) + (size_t)sb * 32);
                mfma6_load(r, pl, off);
            };
            Mfma6Raw bufA, bufB;
            issue(bufA, 0);
            issue(bufB, 1);
            stage(0, (int)threadIdx.x, (int)blockDim.x, Together()); // while the first weights are in flight
            __syncthreads();
            mfma6_keep(bufA); // the staging code must not reuse the registers of the loads in flight
            mfma6_keep(bufB);

            // DUMP: byte offset from a.sums of this lane's sums of its first activation row (4 lh); the
            // following rows lie dump_stride sums further each.  All ones outside the row window.  (The
            // host keeps the whole dump below 4 GiB.)
            uint32_t dump_off = 0xFFFFFFFFu;
            const size_t dump_stride = (size_t)a.nrows * ((size_t)nsb * 8);
            if constexpr (DUMP)
            {
                const long row = tile_row0 + l32;
                const long rr = row - a.row0;
                if (l32 < a.tile_rows && row < a.N && rr >= 0 && rr < a.nrows)
                    dump_off = (uint32_t)((((size_t)(4 * lh) * a.nrows + (size_t)rr) * ((size_t)nsb * 8)) * sizeof(int32_t));
            }
            v16i zero;
#pragma unroll
            for (int i = 0; i < 16; ++i)
                zero[i] = 0;
            const int a_lane = (l32 & 7) * 32 + lh * 16; // rows beyond the batch: any row, result unused
            int step = 0, cur_ph = 0;

            // the coalesced pieces of a step into the bounce buffer; its factor records stay behind
            v4i fc_cur0, fc_cur1;
            auto stage_w = [&](const Mfma6Raw &r) {
                mfma_wave_sync(); // the previous step's reads are done
                *reinterpret_cast<v4i *>(wr_ql) = r.ql0;
                *reinterpret_cast<v4i *>(wr_ql + 8 * MFMA6_QL_STRIDE) = r.ql1;
                *reinterpret_cast<v4i *>(wr_ql + 16 * MFMA6_QL_STRIDE) = r.ql2;
                *reinterpret_cast<v4i *>(wr_ql + 24 * MFMA6_QL_STRIDE) = r.ql3;
                *reinterpret_cast<v4i *>(wr_qh) = r.qh0;
                *reinterpret_cast<v4i *>(wr_qh + 16 * MFMA6_QH_STRIDE) = r.qh1;
                fc_cur0 = r.fc0;
                fc_cur1 = r.fc1;
                mfma_wave_sync();
            };

            auto compute = [&]() {
                const int sb = slice + step * a.slices;
                const int ph = sb / a.chunk;
                while (cur_ph < ph) // uniform: wait until the chunk this step needs has been staged
                {
                    mfma6_barrier();
                    ++cur_ph;
                }
                const int kb0 = (sb - ph * a.chunk) * 8;
                const uint8_t *ab = buf_aq(ph) + (size_t)kb0 * MFMA_AQ_STRIDE + a_lane;
                const float *sb_sc = buf_asc(ph) + (size_t)kb0 * 16 + lh * 8;
                const v4i ql[4] = {*reinterpret_cast<const v4i *>(rd_ql), *reinterpret_cast<const v4i *>(rd_ql + 32),
                                   *reinterpret_cast<const v4i *>(rd_ql + 64), *reinterpret_cast<const v4i *>(rd_ql + 96)};
                const v4i qh[2] = {*reinterpret_cast<const v4i *>(rd_qh), *reinterpret_cast<const v4i *>(rd_qh + 32)};
                const uint32_t k4 = 0x0F0F0F0Fu, k2 = 0x03030303u;
                // the records of the super-block's eight blocks, in the order the plane keeps them
                const uint32_t rec[8] = {(uint32_t)fc_cur0.x, (uint32_t)fc_cur0.y, (uint32_t)fc_cur0.z, (uint32_t)fc_cur0.w,
                                         (uint32_t)fc_cur1.x, (uint32_t)fc_cur1.y, (uint32_t)fc_cur1.z, (uint32_t)fc_cur1.w};
                // block j = 4n + s: nibbles of ql piece (n, s & 1), low for s < 2, high otherwise;
                // bits 2s, 2s+1 of qh piece n; sub-scales 8n + 2s and 8n + 2s + 1
                auto product = [&](int j, float &bscale) {
                    const int n = j >> 2, s = j & 3;
                    int f; // this lane's 16 elements share one sub-scale
                    q6k_block_factor(rec[q6k_code_pos(j)], lh_second, f, bscale);
                    const unsigned short fu = (unsigned short)f, ku = (unsigned short)(128 - 32 * f);
                    const Q6KQuad::v2s ff = {fu, fu}, cc = {ku, ku};
                    const v4i lo = ql[2 * n + (s & 1)], hi = qh[n];
                    auto q4 = [&](int l, int h) {
                        const uint32_t nib = (s >= 2 ? (uint32_t)l >> 4 : (uint32_t)l) & k4;
                        const uint32_t q = nib | ((((uint32_t)h >> (2 * s)) & k2) << 4);
                        return Q6KQuad::requant4(q, ff, cc); // f == 0 (both sub-scales 0) yields 0 bytes
                    };
                    const v4i w = {q4(lo.x, hi.x), q4(lo.y, hi.y), q4(lo.z, hi.z), q4(lo.w, hi.w)};
                    const v4i av = *reinterpret_cast<const v4i *>(ab + j * MFMA_AQ_STRIDE);
                    return __builtin_amdgcn_mfma_i32_32x32x32_i8(av, w, zero, 0, 0, 0);
                };
                // the product of block j+1 is issued before block j is rescaled
                v16i idot[2];
                float bs[2];
                idot[0] = product(0, bs[0]);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                {
                    if (j + 1 < 8)
                        idot[(j + 1) & 1] = product(j + 1, bs[(j + 1) & 1]);
                    const float4 ad = *reinterpret_cast<const float4 *>(sb_sc + j * 16);
                    const v16i dd = idot[j & 1];
                    const float b = bs[j & 1];
                    if constexpr (DUMP)
                    {
                        if (dump_off != 0xFFFFFFFFu)
                        {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                if (4 * lh + i < a.M)
                                {
                                    // uniform base in scalar registers, one 32-bit lane offset
                                    char *base = reinterpret_cast<char *>(a.sums) + ((size_t)(sb * 8 + j) + (size_t)i * dump_stride) * sizeof(int32_t);
                                    *reinterpret_cast<int32_t *>(base + dump_off) = dd[i];
                                }
                        }
                    }
                    acc[0] = fmaf((float)dd[0], ad.x * b, acc[0]);
                    acc[1] = fmaf((float)dd[1], ad.y * b, acc[1]);
                    acc[2] = fmaf((float)dd[2], ad.z * b, acc[2]);
                    acc[3] = fmaf((float)dd[3], ad.w * b, acc[3]);
                }
                ++step;
            };

            // Two register buffers alternate; each is reloaded (two steps ahead) as soon as its
            // pieces are in LDS, before the step is computed.  Every buffer is waited for, also
            // past the end: a register whose load is still in flight must not look free to the
            // compiler.
            for (int c0 = 0; c0 < nsteps; c0 += 2)
            {
                mfma6_wait<MFMA6_LOADS>(bufA);
                if (step < nsteps) // uniform
                    stage_w(bufA);
                __builtin_amdgcn_sched_barrier(0);
                issue(bufA, c0 + 2);
                if (step < nsteps)
                    compute();
                __builtin_amdgcn_sched_barrier(0);
                mfma6_wait<MFMA6_LOADS>(bufB);
                if (step < nsteps)
                    stage_w(bufB);
                __builtin_amdgcn_sched_barrier(0);
                issue(bufB, c0 + 3);
                if (step < nsteps)
                    compute();
                __builtin_amdgcn_sched_barrier(0);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // loads issued past the end
            mfma6_keep(bufA);
            mfma6_keep(bufB);
            while (cur_ph < nph - 1) // the barriers of chunks this wavefront had no part in
            {
                mfma6_barrier();
                ++cur_ph;
            }
        }

        // ---- partial sums of the slices, added in slice order -------------------------------------
        __syncthreads(); // every wavefront is done with the activations
        float *red = reinterpret_cast<float *>(mfma6_lds); // [compute wavefront][4][64]
        if (wave < ncomp)
        {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                red[(wave * 4 + i) * WAVE + lane] = acc[i];
        }
        __syncthreads();
        if (wave < ncomp)
        {
            const int tile_local = wave / a.slices, slice = wave - tile_local * a.slices;
            const long row = ((long)blockIdx.x * a.tiles + tile_local) * a.tile_rows + (lane & 31);
            if (slice == 0 && (lane & 31) < a.tile_rows)
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    float v = acc[i];
                    for (int s = 1; s < a.slices; ++s)
                        v += red[((wave + s) * 4 + i) * WAVE + lane];
                    const int m = 4 * (lane >> 5) + i;
                    if constexpr (!DUMP) // the block-sum variant has no fp32 output (y is null)
                    {
                        if (m < a.M && row < a.N)
                            a.y[(size_t)m * a.ldy + row] = v;
                    }
                }
            }
        }
    }

    // The same product from the matrix's batch plane (q6k_plane_bytes): the int8 weights and
    // block scales that the kernel above works out per launch are read ready-made, 272 bytes per
    // super-block and row against 224, and nothing is left to decode.  Lane (n, h) loads the
    // 16 bytes of elements 16h..16h+15 of every block of its row straight into the B operand
    // (eight lanes read one 128-byte line of the plane; a group's super-block is 1 KB in one
    // place), so there is no bounce buffer either.  Same block sums, same scales, same order of
    // the fp32 operations: the results are those of gemv_mfma_q6k_kernel bit for bit.
    // DUMP: also store the matrix unit's exact int32 block sums (the parity hook), no fp32 output.
    template <int SRC, bool DUMP = false>
    __global__ void __launch_bounds__((MFMA6_PLANE_COMPUTE + MFMA6_PLANE_PRODUCERS) * WAVE) gemv_mfma_q6k_plane_kernel(const Mfma6Args a)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t mfma6_lds[];
        const int nsb = a.SB;
        // this workgroup's part of the rows: super-blocks sb0 .. sb0 + nsbp (the whole row unless ksplit = 2)
        const int part = a.ksplit > 1 ? (int)(blockIdx.x % (unsigned)a.ksplit) : 0;
        const int wg = a.ksplit > 1 ? (int)(blockIdx.x / (unsigned)a.ksplit) : (int)blockIdx.x;
        const int sb_per = (nsb + a.ksplit - 1) / a.ksplit;
        const int sb0 = part * sb_per;
        const int nsbp = sb0 + sb_per <= nsb ? sb_per : (nsb > sb0 ? nsb - sb0 : 0);
        const int nph = (nsbp + a.chunk - 1) / a.chunk; // activation chunks
        const size_t buf_bytes = mfma_act_bytes(a.chunk);
        const int ncomp = a.slices * a.tiles; // compute wavefronts
        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};

        auto buf_aq = [&](int ph) { return mfma6_lds + (size_t)(ph & 1) * buf_bytes; };
        auto buf_asc = [&](int ph) {
            return reinterpret_cast<float *>(mfma6_lds + (size_t)(ph & 1) * buf_bytes + (size_t)a.chunk * 8 * MFMA_AQ_STRIDE);
        };
        auto stage = [&](int ph, int tid, int nthreads, auto un) {
            const int c0 = sb0 + ph * a.chunk;
            const int c1 = ph * a.chunk + a.chunk < nsbp ? c0 + a.chunk : sb0 + nsbp;
            mfma_stage_acts<SRC, decltype(un)::value>(a.q8, a.x, a.x2, a.ldx, a.M, nsb * 8, c0 * 8, (c1 - c0) * 8,
                                                      buf_aq(ph), buf_asc(ph), tid, nthreads);
        };
        typedef std::integral_constant<int, 3> Together;
        typedef std::integral_constant<int, 8> Alone;

        if (wave >= ncomp)
        {
            stage(0, (int)threadIdx.x, (int)blockDim.x, Together());
            __syncthreads();
            for (int ph = 0; ph + 1 < nph; ++ph)
            {
                stage(ph + 1, (int)threadIdx.x - ncomp * WAVE, MFMA6_PLANE_PRODUCERS * WAVE, Alone());
                __syncthreads();
            }
        }
        else
        {
            const int l32 = lane & 31, lh = lane >> 5;
            const int tile_local = wave / a.slices, slice = wave - tile_local * a.slices;
            const int nsteps = slice < nsbp ? (nsbp - slice + a.slices - 1) / a.slices : 0;
            const int last_step = nsteps > 0 ? nsteps - 1 : 0;
            const long tile_row0 = ((long)wg * a.tiles + tile_local) * a.tile_rows;
            // rows past the end of the tile or of the matrix re-read the last one
            const long r_tile = tile_row0 + (l32 < a.tile_rows ? l32 : a.tile_rows - 1);
            const long row = r_tile < a.N ? r_tile : a.N - 1;
            const uint32_t grp = (uint32_t)(row >> 2) * (uint32_t)nsb; // the group's first super-block
            const uint32_t off_w = grp * 1024u + (uint32_t)(row & 3) * 32u + 16u * (uint32_t)lh;
            const uint32_t off_s = grp * 64u + (uint32_t)(row & 3) * 16u;
            const uint8_t *scales = a.plane + q6k_plane_scales_offset(a.N, nsb);

            // loads are never predicated: past its last step a lane re-reads that step
            auto issue = [&](Mfma6PlaneRaw &r, int step) {
                const uint32_t sb = (uint32_t)sb0 + (nsteps > 0 ? (uint32_t)(slice + (step < last_step ? step : last_step) * a.slices) : 0u);
                auto uniform = [](const uint8_t *p) {
                    const uint64_t b = (uint64_t)p;
                    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
                    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
                    return reinterpret_cast<const uint8_t *>(((uint64_t)hi << 32) | lo);
                };
                mfma6_plane_load(r, uniform(a.plane + (size_t)sb * 1024), uniform(scales + (size_t)sb * 64), off_w, off_s);
            };
            Mfma6PlaneRaw bufA, bufB;
            issue(bufA, 0);
            issue(bufB, 1);
            stage(0, (int)threadIdx.x, (int)blockDim.x, Together()); // while the first weights are in flight
            __syncthreads();
            mfma6_keep(bufA); // the staging code must not reuse the registers of the loads in flight
            mfma6_keep(bufB);

            // DUMP: byte offset from a.sums of this lane's sums of its first activation row (4 lh); the
            // following rows lie dump_stride sums further each.  All ones outside the row window.
            uint32_t dump_off = 0xFFFFFFFFu;
            const size_t dump_stride = (size_t)a.nrows * ((size_t)nsb * 8);
            if constexpr (DUMP)
            {
                const long own = tile_row0 + l32;
                const long rr = own - a.row0;
                if (l32 < a.tile_rows && own < a.N && rr >= 0 && rr < a.nrows)
                    dump_off = (uint32_t)((((size_t)(4 * lh) * a.nrows + (size_t)rr) * ((size_t)nsb * 8)) * sizeof(int32_t));
            }
            v16i zero;
#pragma unroll
            for (int i = 0; i < 16; ++i)
                zero[i] = 0;
            const int a_lane = (l32 & 7) * 32 + lh * 16; // rows beyond the batch: any row, result unused
            int step = 0, cur_ph = 0;

            auto compute = [&](const Mfma6PlaneRaw &r) {
                const int sbl = slice + step * a.slices; // within the part
                const int sb = sb0 + sbl;
                const int ph = sbl / a.chunk;
                while (cur_ph < ph) // uniform: wait until the chunk this step needs has been staged
                {
                    mfma6_barrier();
                    ++cur_ph;
                }
                const int kb0 = (sbl - ph * a.chunk) * 8;
                const uint8_t *ab = buf_aq(ph) + (size_t)kb0 * MFMA_AQ_STRIDE + a_lane;
                const float *sb_sc = buf_asc(ph) + (size_t)kb0 * 16 + lh * 8;
                const v4i wv[8] = {r.w0, r.w1, r.w2, r.w3, r.w4, r.w5, r.w6, r.w7};
                const uint32_t sc[4] = {(uint32_t)r.sc.x, (uint32_t)r.sc.y, (uint32_t)r.sc.z, (uint32_t)r.sc.w};
                auto product = [&](int j) {
                    const v4i av = *reinterpret_cast<const v4i *>(ab + j * MFMA_AQ_STRIDE);
                    return __builtin_amdgcn_mfma_i32_32x32x32_i8(av, wv[j], zero, 0, 0, 0);
                };
                // the product of block j+1 is issued before block j is rescaled
                v16i idot[2];
                idot[0] = product(0);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                {
                    if (j + 1 < 8)
                        idot[(j + 1) & 1] = product(j + 1);
                    const float4 ad = *reinterpret_cast<const float4 *>(sb_sc + j * 16);
                    const v16i dd = idot[j & 1];
                    const float b = h2f((uint16_t)(sc[j >> 1] >> (16 * (j & 1))));
                    if constexpr (DUMP)
                    {
                        if (dump_off != 0xFFFFFFFFu)
                        {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                if (4 * lh + i < a.M)
                                {
                                    char *base = reinterpret_cast<char *>(a.sums) + ((size_t)(sb * 8 + j) + (size_t)i * dump_stride) * sizeof(int32_t);
                                    *reinterpret_cast<int32_t *>(base + dump_off) = dd[i];
                                }
                        }
                    }
                    acc[0] = fmaf((float)dd[0], ad.x * b, acc[0]);
                    acc[1] = fmaf((float)dd[1], ad.y * b, acc[1]);
                    acc[2] = fmaf((float)dd[2], ad.z * b, acc[2]);
                    acc[3] = fmaf((float)dd[3], ad.w * b, acc[3]);
                }
                ++step;
            };

            // Two register buffers alternate; each is reloaded, two steps ahead, once its step has
            // been computed from it (three buffers, 155 registers: 35.4 against 34.4 us).  Every buffer is waited for, also past the end: a register
            // whose load is still in flight must not look free to the compiler.
            for (int c0 = 0; c0 < nsteps; c0 += 2)
            {
                mfma6_wait<MFMA6_PLANE_LOADS>(bufA);
                if (step < nsteps) // uniform
                    compute(bufA);
                __builtin_amdgcn_sched_barrier(0);
                issue(bufA, c0 + 2);
                mfma6_wait<MFMA6_PLANE_LOADS>(bufB);
                if (step < nsteps)
                    compute(bufB);
                __builtin_amdgcn_sched_barrier(0);
                issue(bufB, c0 + 3);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // loads issued past the end
            mfma6_keep(bufA);
            mfma6_keep(bufB);
            while (cur_ph < nph - 1) // the barriers of chunks this wavefront had no part in
            {
                mfma6_barrier();
                ++cur_ph;
            }
        }

        // ---- partial sums of the slices, added in slice order -------------------------------------
        __syncthreads(); // every wavefront is done with the activations
        float *red = reinterpret_cast<float *>(mfma6_lds); // [compute wavefront][4][64]
        if (wave < ncomp)
        {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                red[(wave * 4 + i) * WAVE + lane] = acc[i];
        }
        __syncthreads();
        if (wave < ncomp)
        {
            const int tile_local = wave / a.slices, slice = wave - tile_local * a.slices;
            const long row = ((long)wg * a.tiles + tile_local) * a.tile_rows + (lane & 31);
            float *const y_part = part ? a.y2 : a.y;
            if (slice == 0 && (lane & 31) < a.tile_rows)
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    float v = acc[i];
                    for (int s = 1; s < a.slices; ++s)
                        v += red[((wave + s) * 4 + i) * WAVE + lane];
                    const int m = 4 * (lane >> 5) + i;
                    if constexpr (!DUMP) // the block-sum variant has no fp32 output (y is null)
                    {
                        if (m < a.M && row < a.N)
                            y_part[(size_t)m * a.ldy + row] = v;
                    }
                }
            }
        }
    }

    struct Mfma6Shape
    {
        int slices, tiles, chunk, tile_rows;
        long grid;
    };
    // The launch for tiles of `tile_rows` rows.  Slices so that a compute unit sees about eight
    // compute wavefronts, five at least (the scales of eight neighbouring super-blocks share a
    // cache line) and each two steps long; tiles per workgroup to fill its compute wavefronts
    // when there are tiles to spare.
    // bounce_per_wave: LDS bytes of a compute wavefront's bounce buffer (none when the weights come from a batch plane)
    inline Mfma6Shape gemv_mfma6_shape_of(long N, int nsb, int cus, int max_compute, int tile_rows, bool plane = false,
                                          size_t bounce_per_wave = MFMA6_BOUNCE)
    {
        const long tiles = (N + tile_rows - 1) / tile_rows;
        long want = ((long)cus * max_compute + tiles - 1) / tiles;
        if (want < 5)
            want = 5;
        if (want > max_compute)
            want = max_compute;
        if (want > nsb / 2)
            want = nsb / 2;
        if (want < 1)
            want = 1;
        Mfma6Shape sh;
        sh.tile_rows = tile_rows;
        sh.slices = (int)want;
        int t = 1;
        while ((t * 2) * sh.slices <= max_compute && tiles / (t * 2) >= 2L * cus)
            t *= 2;
        sh.tiles = t;
        sh.grid = (tiles + t - 1) / t;
        // one buffer if the whole row fits beside the bounce buffers and leaves half the LDS
        // free, else two buffers of a whole number of rounds of the slices
        const size_t bounce = plane ? 0 : (size_t)sh.slices * t * bounce_per_wave; // the plane kernels have no bounce buffers
        if (mfma_act_bytes(nsb) * 2 + bounce <= QUAD_MAX_LDS)
            sh.chunk = nsb;
        else
        {
            const int fit = (int)((QUAD_MAX_LDS - bounce) / (2 * mfma_act_bytes(1)));
            sh.chunk = (fit / sh.slices) * sh.slices;
        }
        return sh;
    }
    // The tile height that leaves the busiest compute unit the fewest rows (gemv_mfma_shape):
    // 5120 rows are 160 full tiles, and 256 tiles of 20 rows.
    inline Mfma6Shape gemv_mfma6_shape(long N, int nsb, int cus, int max_compute = MFMA6_MAX_COMPUTE, bool plane = false,
                                       size_t bounce_per_wave = MFMA6_BOUNCE)
    {
        const int forced = gemv_mfma_tile_rows_override();
        Mfma6Shape best;
        long best_cost = -1;
        for (int tr = MFMA_TILE_ROWS; tr >= MFMA_MIN_TILE_ROWS; --tr)
        {
            if (forced > 0 && tr != forced)
                continue;
            const Mfma6Shape sh = gemv_mfma6_shape_of(N, nsb, cus, max_compute, tr, plane, bounce_per_wave);
            const long cost = ((sh.grid + cus - 1) / cus) * sh.tiles * tr;
            if (best_cost < 0 || cost * 20 < best_cost * 19) // a shorter tile has to win 5 %
            {
                best = sh;
                best_cost = cost;
            }
        }
        return best;
    }
} // namespace llamql
