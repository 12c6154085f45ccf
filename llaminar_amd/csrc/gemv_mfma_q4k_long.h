// Q4_K x Q8_1 decode GEMV for batches of 5..8 activation rows on the matrix unit, rows too long
// for the batch's activations in LDS (K = 25600 at eight rows: 269 KB).
//
// The product of gemv_mfma_q4k_kernel (gemv_mfma.h: operand layout, decode, block order, the
// coalesced weight loads through a per-wavefront bounce buffer, or the batch plane read in
// place) inside the workgroup of gemv_mfma_q6k_kernel (gemv_mfma_q6k.h): the row is walked in
// chunks of super-blocks that two producer wavefronts stage alternately into two LDS buffers
// while the compute wavefronts work on the other buffer, one barrier per chunk; the compute
// wavefronts of a 32-row tile share the super-blocks round robin, and with the chunk a multiple
// of their number that sequence does not depend on the chunking.  Their partial sums are added
// in wavefront order.
#pragma once
#include "gemv_mfma_q6k.h"

namespace llamql
{
    struct MfmaLongArgs : MfmaArgs // slices: compute wavefronts per tile
    {
        int tiles; // tiles per workgroup
        int chunk; // super-blocks per activation buffer; a multiple of slices when SB > chunk
        // the row's super-blocks in ksplit (1 or 2) equal parts, one workgroup per (tiles, part); part 1's sums go
        // to y2 (the caller adds the two: gemv_mfma_q6k_plane_kernel has the same)
        int ksplit;
        float *y2;
    };

    constexpr int MFMA4_LONG_COMPUTE = MFMA6_MAX_COMPUTE; // compute wavefronts per workgroup
    constexpr int MFMA4_LONG_DUMP_COMPUTE = MFMA6_DUMP_COMPUTE; // the same for the block-sum variant (its stores need registers)
    constexpr int MFMA4_LONG_PRODUCERS = MFMA6_PRODUCERS; // wavefronts that only stage activations

    // DUMP: also store the matrix unit's results, the exact int32 block sums (the parity hook), no fp32 output.
    // PLANE: the weights come from the matrix's batch plane (no bounce buffer).
    template <int SRC, bool DUMP = false, bool PLANE = false>
    __global__ void __launch_bounds__(((DUMP ? MFMA4_LONG_DUMP_COMPUTE : MFMA4_LONG_COMPUTE) + MFMA4_LONG_PRODUCERS) * WAVE)
        gemv_mfma_q4k_long_kernel(const MfmaLongArgs a)
    {
        typedef typename std::conditional<PLANE, MfmaPlaneRaw, MfmaRaw>::type Raw;
        constexpr int LOADS = PLANE ? MFMA_PLANE_LOADS : MFMA_LOADS;
        extern __shared__ __attribute__((aligned(16))) uint8_t mfma4_lds[];
        const int nsb = a.SB;
        const int nkb = nsb * 8;
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

        auto buf_aq = [&](int ph) { return mfma4_lds + (size_t)(ph & 1) * buf_bytes; };
        auto buf_asc = [&](int ph) {
            return reinterpret_cast<float *>(mfma4_lds + (size_t)(ph & 1) * buf_bytes + (size_t)a.chunk * 8 * MFMA_AQ_STRIDE);
        };
        // chunk ph into its buffer, by `nthreads` threads that keep UN loads in flight each
        auto stage_acts = [&](int ph, int tid, int nthreads, auto un) {
            const int c0 = sb0 + ph * a.chunk;
            const int c1 = ph * a.chunk + a.chunk < nsbp ? c0 + a.chunk : sb0 + nsbp;
            mfma_stage_acts<SRC, decltype(un)::value>(a.q8, a.x, a.x2, a.ldx, a.M, nkb, c0 * 8, (c1 - c0) * 8, buf_aq(ph),
                                                      buf_asc(ph), tid, nthreads);
        };
        typedef std::integral_constant<int, 3> Together; // everybody stages the first chunk
        typedef std::integral_constant<int, 8> Alone;    // the producers stage the others

        if (wave >= ncomp)
        {
            // ---- producers: the first chunk together with everybody, then chunk ph+1 into the
            // buffer nobody reads during chunk ph ------------------------------------------------
            stage_acts(0, (int)threadIdx.x, (int)blockDim.x, Together());
            __syncthreads();
            for (int ph = 0; ph + 1 < nph; ++ph)
            {
                stage_acts(ph + 1, (int)threadIdx.x - ncomp * WAVE, MFMA4_LONG_PRODUCERS * WAVE, Alone());
                __syncthreads();
            }
        }
        else
        {
            // ---- compute wavefronts --------------------------------------------------------------
            const int l32 = lane & 31, lh = lane >> 5;
            const int tile_local = wave / a.slices, slice = wave - tile_local * a.slices;
            const int nsteps = slice < nsbp ? (nsbp - slice + a.slices - 1) / a.slices : 0;
            const int last_step = nsteps > 0 ? nsteps - 1 : 0;
            const long tile_row0 = ((long)wg * a.tiles + tile_local) * a.tile_rows;
            const long row = tile_row0 + l32;
            const bool row_ok = l32 < a.tile_rows && row < a.N;

            // piece p = lane + 64 i of the step: 16 bytes at offset 16 (p % 9) of row p / 9.  Rows
            // past the end of the tile or of the matrix (and the 32 pieces past row 31) re-read the
            // last row.
            const long base_row = tile_row0 < a.N ? tile_row0 : a.N - 1;
            const int max_local = (int)(a.N - 1 - base_row) < a.tile_rows - 1 ? (int)(a.N - 1 - base_row)
                                                                              : a.tile_rows - 1;
            uint32_t off[5];
#pragma unroll
            for (int i = 0; i < 5; ++i)
            {
                const int p = lane + WAVE * i;
                int r = p / 9;
                const int piece = p - r * 9;
                if (r > max_local)
                    r = max_local;
                off[i] = (uint32_t)r * (uint32_t)(nsb * 144) + (uint32_t)(piece * 16);
            }
            const uint8_t *tile_base = a.w + (size_t)base_row * nsb * 144;
            uint8_t *bounce = mfma4_lds + mfma6_act_bytes(nsb, a.chunk) + (size_t)wave * MFMA_BOUNCE;
            uint8_t *bounce_wr = bounce + lane * 16;              // piece lane + 64 i at + 1024 i
            const uint8_t *bounce_rd = bounce + l32 * 144;        // this lane's weight row
            const uint8_t *bounce_rdq = bounce_rd + 16 + 16 * lh; // its half of every group
            // PLANE: this lane's row (past the tile or the matrix: the last one), its group's first
            // super-block and its byte offsets in the two planes
            const long prow = base_row + (l32 < max_local ? l32 : max_local);
            const uint32_t pgrp = (uint32_t)(prow >> 2) * (uint32_t)nsb;
            const uint32_t poff_w = pgrp * 512u + (uint32_t)(prow & 3) * 32u + 16u * (uint32_t)lh;
            const uint32_t poff_h = pgrp * 64u + (uint32_t)(prow & 3) * 16u;
            auto uniform = [](const uint8_t *p) {
                const uint64_t b = (uint64_t)p;
                const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
                const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
                return reinterpret_cast<const uint8_t *>(((uint64_t)hi << 32) | lo);
            };
            // loads are never predicated: past its last step a lane re-reads that step
            auto issue = [&](Raw &r, int step) {
                const int sb = sb0 + (nsteps > 0 ? slice + (step < last_step ? step : last_step) * a.slices : 0);
                if constexpr (PLANE)
                    mfma_plane_load(r, uniform(a.plane + (size_t)sb * 512),
                                    uniform(a.plane + q4k_plane_heads_offset(a.N, nsb) + (size_t)sb * 64), poff_w, poff_h);
                else
                    mfma_load(r, uniform(tile_base + (size_t)sb * 144), off);
            };
            Raw bufA, bufB;
            issue(bufA, 0);
            issue(bufB, 1);
            stage_acts(0, (int)threadIdx.x, (int)blockDim.x, Together()); // while the first weights are in flight
            __syncthreads();
            mfma_keep(bufA); // the staging code must not reuse the registers of the loads in flight
            mfma_keep(bufB);

            // DUMP: byte offset from a.sums of this lane's sums of its first activation row (4 lh); the
            // following rows lie dump_stride sums further each.  All ones outside the row window.  (The
            // host keeps the whole dump below 4 GiB.)
            uint32_t dump_off = 0xFFFFFFFFu;
            const size_t dump_stride = (size_t)a.nrows * (size_t)nkb;
            if constexpr (DUMP)
            {
                const long rr = row - a.row0;
                if (row_ok && rr >= 0 && rr < a.nrows)
                    dump_off = (uint32_t)((((size_t)(4 * lh) * a.nrows + (size_t)rr) * (size_t)nkb) * sizeof(int32_t));
            }
            v16i zero;
#pragma unroll
            for (int i = 0; i < 16; ++i)
                zero[i] = 0;
            const int a_lane = (l32 & 7) * 32 + lh * 16; // rows beyond the batch: any row, result unused
            int step = 0, cur_ph = 0;

            // the loaded pieces go to the wavefront's bounce buffer in piece order
            auto stage_w = [&](const MfmaRaw &r) {
                mfma_wave_sync(); // the previous step's reads are done
                *reinterpret_cast<v4i *>(bounce_wr) = r.c0;
                *reinterpret_cast<v4i *>(bounce_wr + 1024) = r.c1;
                *reinterpret_cast<v4i *>(bounce_wr + 2048) = r.c2;
                *reinterpret_cast<v4i *>(bounce_wr + 3072) = r.c3;
                *reinterpret_cast<v4i *>(bounce_wr + 4096) = r.c4;
                mfma_wave_sync();
            };

            // this lane's operands: the head of its row's super-block and its half of the four groups
            auto compute = [&](const v4i head, const v4i q0, const v4i q1, const v4i q2, const v4i q3) {
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
                const v4i q[4] = {q0, q1, q2, q3};
                Q4KQuad::Scale S[4];
                Q4KQuad::decode_scales(head, Q4KQuad::lane_consts(0), S[0]);
                Q4KQuad::decode_scales(head, Q4KQuad::lane_consts(1), S[1]);
                Q4KQuad::decode_scales(head, Q4KQuad::lane_consts(2), S[2]);
                Q4KQuad::decode_scales(head, Q4KQuad::lane_consts(3), S[3]);
                const uint32_t k = 0x0F0F0F0Fu;
                // block 2g+h of the super-block: h = 0 low nibbles, 1 high nibbles
                auto product = [&](int j) {
                    const v4i x = q[j >> 1];
                    v4i w;
                    if (j & 1)
                        w = (v4i){(int)(((uint32_t)x.x >> 4) & k), (int)(((uint32_t)x.y >> 4) & k),
                                  (int)(((uint32_t)x.z >> 4) & k), (int)(((uint32_t)x.w >> 4) & k)};
                    else
                        w = (v4i){(int)((uint32_t)x.x & k), (int)((uint32_t)x.y & k), (int)((uint32_t)x.z & k),
                                  (int)((uint32_t)x.w & k)};
                    const v4i av = *reinterpret_cast<const v4i *>(ab + j * MFMA_AQ_STRIDE);
                    return __builtin_amdgcn_mfma_i32_32x32x32_i8(av, w, zero, 0, 0, 0);
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
                    const float4 asd = *reinterpret_cast<const float4 *>(sb_sc + j * 16 + 4);
                    const float bs = Q4KQuad::scale_f32(S[j >> 1], j & 1);
                    const float bm = Q4KQuad::min_f32(S[j >> 1], j & 1);
                    const v16i d = idot[j & 1];
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
                                    *reinterpret_cast<int32_t *>(base + dump_off) = d[i];
                                }
                        }
                    }
                    acc[0] = fmaf((float)d[0], ad.x * bs, acc[0]);
                    acc[0] = fmaf(asd.x, bm, acc[0]);
                    acc[1] = fmaf((float)d[1], ad.y * bs, acc[1]);
                    acc[1] = fmaf(asd.y, bm, acc[1]);
                    acc[2] = fmaf((float)d[2], ad.z * bs, acc[2]);
                    acc[2] = fmaf(asd.z, bm, acc[2]);
                    acc[3] = fmaf((float)d[3], ad.w * bs, acc[3]);
                    acc[3] = fmaf(asd.w, bm, acc[3]);
                }
                ++step;
            };
            auto compute_lds = [&]() {
                compute(*reinterpret_cast<const v4i *>(bounce_rd), *reinterpret_cast<const v4i *>(bounce_rdq),
                        *reinterpret_cast<const v4i *>(bounce_rdq + 32), *reinterpret_cast<const v4i *>(bounce_rdq + 64),
                        *reinterpret_cast<const v4i *>(bounce_rdq + 96));
            };

            // Two register buffers alternate; every buffer is waited for, also past the end of the
            // slice: a register whose load is still in flight must not look free to the compiler.
            for (int c0 = 0; c0 < nsteps; c0 += 2)
            {
                if constexpr (PLANE)
                {
                    mfma_wait<LOADS>(bufA);
                    if (step < nsteps) // uniform
                        compute(bufA.head, bufA.q0, bufA.q1, bufA.q2, bufA.q3);
                    __builtin_amdgcn_sched_barrier(0);
                    issue(bufA, c0 + 2);
                    mfma_wait<LOADS>(bufB);
                    if (step < nsteps)
                        compute(bufB.head, bufB.q0, bufB.q1, bufB.q2, bufB.q3);
                    __builtin_amdgcn_sched_barrier(0);
                    issue(bufB, c0 + 3);
                }
                else
                {
                    mfma_wait<LOADS>(bufA);
                    if (step < nsteps) // uniform
                        stage_w(bufA);
                    __builtin_amdgcn_sched_barrier(0);
                    issue(bufA, c0 + 2);
                    if (step < nsteps)
                        compute_lds();
                    __builtin_amdgcn_sched_barrier(0);
                    mfma_wait<LOADS>(bufB);
                    if (step < nsteps)
                        stage_w(bufB);
                    __builtin_amdgcn_sched_barrier(0);
                    issue(bufB, c0 + 3);
                    if (step < nsteps)
                        compute_lds();
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // loads issued past the end of the slice
            mfma_keep(bufA);
            mfma_keep(bufB);
            while (cur_ph < nph - 1) // the barriers of chunks this wavefront had no part in
            {
                mfma6_barrier();
                ++cur_ph;
            }
        }

        // ---- partial sums of the slices, added in slice order -------------------------------------
        __syncthreads(); // every wavefront is done with the activations
        float *red = reinterpret_cast<float *>(mfma4_lds); // [compute wavefront][4][64]
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
} // namespace llamql
