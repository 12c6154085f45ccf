// Q4_K x Q8_1 decode GEMV for batches of 5..8 activation rows on the matrix unit.
//
// With several activation rows the quad-lane kernel pays 16 dot instructions and five
// 128-bit LDS reads per 64 weights for EVERY row.  Here one v_mfma_i32_32x32x32_i8 per
// 32-column block multiplies 32 weight rows with all activation rows at once:
//   A operand = activations (rows m of the batch, padded to 32), lane (m = l%32, h = l/32)
//               supplies bytes 16h..16h+15 of the block, read from LDS;
//   B operand = weights, lane (r = l%32, h) supplies elements 16h..16h+15 of row r's block,
//               straight from the registers the lane decoded them into: a 16-byte piece of
//               a Q4_K group holds exactly those elements of block 2g (low nibbles) and of
//               block 2g+1 (high nibbles);
//   result    = the exact int32 block sums: lane (r, h) holds rows m = 4h..4h+3 of column r,
//               i.e. the lane that decoded row r's scales also rescales row r's sums.
// The accumulator is zero for every block, so the MFMA result is the reference's per-block
// int32 sum, rescaled in fp32 block after block in ascending order.
//
// The wavefronts of a 32-row tile share its super-blocks round robin (K = 5120: 4 wavefronts,
// wavefront j takes super-blocks j, j+4, ..: at any moment they read neighbouring super-blocks
// of every row); their partial sums are added in wavefront order at the end.
//
// Weight loads are coalesced: the 32 x 144 bytes of a step are 288 16-byte pieces; lane l loads
// pieces l, l+64, .. (nine neighbouring lanes cover one super-block, so an instruction touches
// 8 rows instead of 64) and the wavefront passes them through a private LDS buffer to the lane
// that needs them as an operand.  No barrier: LDS instructions of one wavefront run in order.
#pragma once
#include "gemv_core.h"
#include "gemv_quad.h"
#include <type_traits>

namespace llamql
{
    constexpr int MFMA_TILE_ROWS = 32;     // rows of a full tile (columns of the matrix instruction)
    constexpr int MFMA_MIN_TILE_ROWS = 16; // shortest tile the launch shapes consider
    constexpr int MFMA_MAX_SLICES = 8;
    constexpr int MFMA_MAX_WAVES = 16;     // wavefronts per workgroup
    constexpr int MFMA_DUMP_WAVES = 8;     // the same for the block-sum variant
    constexpr int MFMA_LOADS = 5;          // vector memory loads per step and lane
    constexpr int MFMA_BOUNCE = 5 * 1024;  // LDS bytes of a wavefront's bounce buffer (320 pieces, 288 used)

    struct MfmaArgs
    {
        const uint8_t *w;   // Q4_K super-blocks, row-major
        const uint8_t *plane; // PLANE kernels: the matrix's batch plane (q4k_plane_bytes), w is not read
        const uint32_t *q8; // Q8_1 activations as dwords (9 per block), M rows (QUAD_SRC_Q8)
        const float *x;     // fp32 rows of ldx floats (QUAD_SRC_F32); the gate rows for QUAD_SRC_SWIGLU
        const float *x2;    // the up rows for QUAD_SRC_SWIGLU
        int ldx;
        float *y;
        int ldy;
        int N;
        int SB;           // super-blocks per weight row
        int M;            // activation rows, 1..8
        int slices;       // wavefronts per tile (wavefront j walks super-blocks j, j + slices, ..)
        int tiles_per_wg; // tiles of a workgroup; wavefronts beyond slices * tiles_per_wg help to stage the
                          // activations and idle otherwise
        int tile_rows;    // weight rows of a tile, 1..32: fewer than 32 leave columns of the matrix
                          // instruction unused, and let the tiles of a launch fill every compute unit
        // DUMP kernels only: the exact per-block int32 sums of rows [row0, row0+nrows) go to
        // sums[(m * nrows + row - row0) * (SB * 8) + block]
        int32_t *sums;
        int row0, nrows;
        // SWIGLU kernels only (gate and up projection in one launch): the second matrix (w, plane are the
        // gate matrix) and its optional fp32 output (y: the gate's, may be null too), and the Q8_1 blocks of
        // silu(gate) * up, [M][N/32] blocks of 9 dwords
        const uint8_t *w2;
        const uint8_t *plane2;
        float *y2;
        uint32_t *q8_out;
    };

    // LDS: per 32-column block 8 activation rows x 32 int8 (16 bytes of padding: neighbouring
    // blocks start four banks apart, so the staging writes do not collide) and
    // 2 x {d[4], sum*d[4]}
    constexpr int MFMA_AQ_STRIDE = 256 + 16;
    __host__ __device__ inline size_t mfma_act_bytes(int nsb) { return (size_t)nsb * 8 * (MFMA_AQ_STRIDE + 64); }
    inline size_t mfma_lds_bytes(int nsb, int waves) { return mfma_act_bytes(nsb) + (size_t)waves * MFMA_BOUNCE; }

    // pieces l, l+64, .., l+256 of a step, as loaded
    struct MfmaRaw
    {
        v4i c0, c1, c2, c3, c4;
    };

    // base: the step's super-block of the tile's first row (wavefront-uniform, scalar registers);
    // off: this lane's five byte offsets from it
    __device__ __forceinline__ void mfma_load(MfmaRaw &r, const uint8_t *base, const uint32_t (&off)[5])
    {
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.c0) : "v"(off[0]), "s"(base));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.c1) : "v"(off[1]), "s"(base));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.c2) : "v"(off[2]), "s"(base));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.c3) : "v"(off[3]), "s"(base));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.c4) : "v"(off[4]), "s"(base));
    }
    __device__ __forceinline__ void mfma_keep(MfmaRaw &r)
    {
        asm volatile("" : "+v"(r.c0), "+v"(r.c1), "+v"(r.c2), "+v"(r.c3), "+v"(r.c4));
    }
    template <int NEWER>
    __device__ __forceinline__ void mfma_wait(MfmaRaw &r)
    {
        asm volatile("s_waitcnt vmcnt(%5)"
                     : "+v"(r.c0), "+v"(r.c1), "+v"(r.c2), "+v"(r.c3), "+v"(r.c4)
                     : "n"(NEWER));
    }
    // The same bytes from the matrix's batch plane, where they lie in the order the lanes take
    // them: the head of this lane's row's super-block (d, dmin, scales) and its half of the four
    // 32-byte groups.
    constexpr int MFMA_PLANE_LOADS = 5;
    struct MfmaPlaneRaw
    {
        v4i head, q0, q1, q2, q3;
    };
    __device__ __forceinline__ void mfma_plane_load(MfmaPlaneRaw &r, const uint8_t *pw, const uint8_t *ph, uint32_t ow,
                                                    uint32_t oh)
    {
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.head) : "v"(oh), "s"(ph));
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.q0) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:128" : "=&v"(r.q1) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:256" : "=&v"(r.q2) : "v"(ow), "s"(pw));
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:384" : "=&v"(r.q3) : "v"(ow), "s"(pw));
    }
    __device__ __forceinline__ void mfma_keep(MfmaPlaneRaw &r)
    {
        asm volatile("" : "+v"(r.head), "+v"(r.q0), "+v"(r.q1), "+v"(r.q2), "+v"(r.q3));
    }
    template <int NEWER>
    __device__ __forceinline__ void mfma_wait(MfmaPlaneRaw &r)
    {
        asm volatile("s_waitcnt vmcnt(%5)"
                     : "+v"(r.head), "+v"(r.q0), "+v"(r.q1), "+v"(r.q2), "+v"(r.q3)
                     : "n"(NEWER));
    }
    // orders the LDS traffic of one wavefront as seen by the compiler; the hardware runs a
    // wavefront's LDS instructions in order, so no instruction is needed
    __device__ __forceinline__ void mfma_wave_sync()
    {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }

    // Activation blocks kb0 .. kb0+nkb of all M rows into LDS, by `nthreads` threads (tid among
    // them): aq[kb][8 rows][32 int8] (stride MFMA_AQ_STRIDE) and asc[kb][2 halves][d x4, sum*d x4].
    // nkb_row: blocks in a whole activation row.  UN: loads a thread keeps in flight (Q8_1
    // blocks, or 16-byte pieces of fp32 rows): the latency of a round trip is paid per batch of
    // loads, so few threads staging much want a large UN.
    template <int SRC, int UN = 3>
    __device__ __forceinline__ void mfma_stage_acts(const uint32_t *q8, const float *x, const float *x2, int ldx, int M,
                                                    int nkb_row, int kb0, int nkb, uint8_t *aq, float *asc, int tid,
                                                    int nthreads)
    {
        if constexpr (SRC == QUAD_SRC_Q8)
        {
            // one thread per Q8_1 block
            const int total = M * nkb;
            for (int i0 = tid; i0 < total; i0 += UN * nthreads)
            {
                uint32_t v[UN][9];
#pragma unroll
                for (int u = 0; u < UN; ++u)
                {
                    const int idx = min(i0 + u * nthreads, total - 1);
                    const int m = idx / nkb, kb = idx - m * nkb;
                    const uint32_t *src = q8 + ((size_t)m * nkb_row + kb0 + kb) * 9;
#pragma unroll
                    for (int i = 0; i < 9; ++i)
                        v[u][i] = src[i];
                }
#pragma unroll
                for (int u = 0; u < UN; ++u)
                {
                    const int idx = i0 + u * nthreads;
                    if (idx < total)
                    {
                        const int m = idx / nkb, kb = idx - m * nkb;
                        const float d = h2f((uint16_t)(v[u][0] & 0xFFFFu));
                        uint4 *dst = reinterpret_cast<uint4 *>(aq + (size_t)kb * MFMA_AQ_STRIDE + m * 32);
                        dst[0] = make_uint4(v[u][1], v[u][2], v[u][3], v[u][4]);
                        dst[1] = make_uint4(v[u][5], v[u][6], v[u][7], v[u][8]);
                        float *sc = asc + (size_t)kb * 16 + (m >> 2) * 8 + (m & 3);
                        sc[0] = d;
                        sc[4] = (float)(int16_t)(v[u][0] >> 16) * d;
                    }
                }
            }
        }
        else
        {
            // eight neighbouring threads quantise one 32-element block (the stand-alone
            // quantiser's arithmetic); pieces of all rows are dealt round robin, whole 8-thread
            // groups stay together (nthreads and the pieces of a row are multiples of 8)
            constexpr int UF = UN < 4 ? UN : 4;
            const int nvec = nkb * 8, total = M * nvec;
            for (int i0 = tid; i0 < total; i0 += UF * nthreads)
            {
                float4 v[UF], v2[UF];
#pragma unroll
                for (int u = 0; u < UF; ++u)
                {
                    const int idx = min(i0 + u * nthreads, total - 8 + (tid & 7)); // past the end: the last block again
                    const int m = idx / nvec, i = idx - m * nvec;
                    v[u] = (reinterpret_cast<const float4 *>(x + (size_t)m * ldx) + (size_t)kb0 * 8)[i];
                    if constexpr (SRC == QUAD_SRC_SWIGLU)
                        v2[u] = (reinterpret_cast<const float4 *>(x2 + (size_t)m * ldx) + (size_t)kb0 * 8)[i];
                }
#pragma unroll
                for (int u = 0; u < UF; ++u)
                {
                    const int idx = i0 + u * nthreads;
                    float4 w = v[u];
                    if constexpr (SRC == QUAD_SRC_SWIGLU)
                        w = swiglu4(w, v2[u]);
                    const Q8Lane q = q8_1_quantize_lane(w); // exchanges with the 7 neighbours: no divergence before it
                    if (idx < total)
                    {
                        const int m = idx / nvec, i = idx - m * nvec;
                        const int kb = i >> 3, sub = i & 7;
                        *reinterpret_cast<uint32_t *>(aq + (size_t)kb * MFMA_AQ_STRIDE + m * 32 + sub * 4) = q.packed;
                        if (sub == 0)
                        {
                            const float d = h2f((uint16_t)(q.head & 0xFFFFu));
                            float *sc = asc + (size_t)kb * 16 + (m >> 2) * 8 + (m & 3);
                            sc[0] = d;
                            sc[4] = (float)(int16_t)(q.head >> 16) * d;
                        }
                    }
                }
            }
        }
    }

    // The same layout from blocks fetched ahead (quad_act_issue: block idx = m * nkb + kb of whole rows).
    constexpr int MFMA_ACT_PASSES = 4; // eight rows of 8192 over eight wavefronts
    __device__ __forceinline__ void mfma_act_store(const QuadActRaw (&r)[MFMA_ACT_PASSES], int nkb, int total, uint8_t *aq,
                                                   float *asc)
    {
#pragma unroll
        for (int p = 0; p < MFMA_ACT_PASSES; ++p)
        {
            const int idx = (int)threadIdx.x + p * (int)blockDim.x;
            if (idx < total)
            {
                const int m = idx / nkb, kb = idx - m * nkb;
                const uint32_t head = (uint32_t)r[p].lo.x;
                const float d = h2f((uint16_t)(head & 0xFFFFu));
                uint4 *dst = reinterpret_cast<uint4 *>(aq + (size_t)kb * MFMA_AQ_STRIDE + m * 32);
                dst[0] = make_uint4((uint32_t)r[p].lo.y, (uint32_t)r[p].lo.z, (uint32_t)r[p].lo.w, (uint32_t)r[p].hi.x);
                dst[1] = make_uint4((uint32_t)r[p].hi.y, (uint32_t)r[p].hi.z, (uint32_t)r[p].hi.w, (uint32_t)r[p].tail);
                float *sc = asc + (size_t)kb * 16 + (m >> 2) * 8 + (m & 3);
                sc[0] = d;
                sc[4] = (float)(int16_t)(head >> 16) * d;
            }
        }
    }

    // SRC: where the activations come from (QUAD_SRC_*): Q8_1 blocks, or fp32 rows quantised here.
    // DUMP: also store the matrix unit's results, the exact int32 block sums (the parity hook).
    // Its stores need registers the 16-wavefront workgroup does not have (and the build refuses to
    // spill): the variant runs in workgroups of at most MFMA_DUMP_WAVES wavefronts, fewer tiles per
    // workgroup, the same code per tile.
    // PLANE: the weights come from the matrix's batch plane (ql_host.h: the super-blocks' bytes
    // regrouped so that lane (row, h) finds its operands at one address, 128-byte lines shared by
    // four rows): no bounce buffer, a step is computed straight from the registers its loads
    // filled.  Same decode, same products, same order: bit-identical results.
    // SWIGLU: the gate and the up projection of a feed-forward block in one launch.  The tiles of a
    // workgroup come in pairs (rows 32 t .. 32 t + 31 of the gate matrix, the same rows of the up matrix),
    // so the workgroup holds both operands of silu(gate) * up for 32 consecutive columns of every
    // activation row: one Q8_1 block of the down projection's input each, quantised here with the
    // stand-alone quantiser's arithmetic (the bits of the two projections followed by
    // llam_ql_swiglu_quantize for the same partition of the rows into slices); the fp32 results go to
    // memory only if asked for.  Tiles are 32 rows, N a multiple of 32.
    // block: the workgroup's index among those of this kernel body (a launch may hold other workgroups).
    template <int SRC, bool DUMP = false, bool PLANE = false, bool SWIGLU = false>
    __device__ __forceinline__ void gemv_mfma_q4k_body(const MfmaArgs &a, uint8_t *mfma_lds, const int block)
    {
        static_assert(!(SWIGLU && DUMP), "the block-sum variant walks one matrix");
        typedef typename std::conditional<PLANE, MfmaPlaneRaw, MfmaRaw>::type Raw;
        constexpr int LOADS = PLANE ? MFMA_PLANE_LOADS : MFMA_LOADS;
        const int nsb = a.SB;
        const int nkb = nsb * 8;
        uint8_t *aq = mfma_lds;                                                 // [kb][8 rows][32 B] (+16)
        float *asc = reinterpret_cast<float *>(mfma_lds + nkb * MFMA_AQ_STRIDE); // [kb][2 halves][d x4, sum*d x4]

        const int lane = threadIdx.x & (WAVE - 1);
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        const int l32 = lane & 31, lh = lane >> 5;

        // this wavefront's tile and slice of the row, and this lane's weight row
        const int tile_local = wave / a.slices, slice = wave - tile_local * a.slices;
        const int tiles_per_wg = a.tiles_per_wg;
        const bool idle = tile_local >= tiles_per_wg; // (uniform) a wavefront without a tile
        // slice j walks super-blocks j, j + slices, ..: at any moment the wavefronts of a tile
        // read NEIGHBOURING super-blocks of every row, so a 128-byte line that straddles two
        // super-blocks (144 bytes each) is asked for by two wavefronts of the workgroup at the
        // same time and crosses the fabric once
        const int nsteps = !idle && slice < nsb ? (nsb - slice + a.slices - 1) / a.slices : 0;
        // SWIGLU: tile 2 p of the workgroup is the gate half, tile 2 p + 1 the up half of pair p
        const int mat = SWIGLU ? tile_local & 1 : 0;
        const long tile_idx = SWIGLU ? (long)block * (tiles_per_wg >> 1) + (tile_local >> 1)
                                     : (long)block * tiles_per_wg + tile_local;
        const long tile_row0 = tile_idx * a.tile_rows;
        const uint8_t *const w_mat = SWIGLU && mat ? a.w2 : a.w;
        const uint8_t *const plane_mat = SWIGLU && mat ? a.plane2 : a.plane;
        const long row = tile_row0 + l32;
        const bool row_ok = !idle && l32 < a.tile_rows && row < a.N;
        const int last_step = nsteps > 0 ? nsteps - 1 : 0;

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
        const uint8_t *tile_base = w_mat + (size_t)base_row * nsb * 144;
        uint8_t *bounce = mfma_lds + nkb * (MFMA_AQ_STRIDE + 64) + wave * MFMA_BOUNCE;
        uint8_t *bounce_wr = bounce + lane * 16;                     // piece lane + 64 i at + 1024 i
        const uint8_t *bounce_rd = bounce + l32 * 144;               // this lane's weight row
        const uint8_t *bounce_rdq = bounce_rd + 16 + 16 * lh;        // its half of every group

        // loads are never predicated: past the end of the slice a lane re-reads its last block
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
        auto issue = [&](Raw &r, int step) {
            const int sb = nsteps > 0 ? slice + (step < last_step ? step : last_step) * a.slices : 0;
            if constexpr (PLANE)
                mfma_plane_load(r, uniform(plane_mat + (size_t)sb * 512),
                                uniform(plane_mat + q4k_plane_heads_offset(a.N, nsb) + (size_t)sb * 64), poff_w, poff_h);
            else
                mfma_load(r, uniform(tile_base + (size_t)sb * 144), off);
        };
        Raw bufA, bufB;
        // ---- activations into LDS ------------------------------------------------------------
        if constexpr (SRC == QUAD_SRC_Q8)
        {
            // Q8_1 blocks are asked for BEFORE the weights and waited for by themselves (a wavefront's
            // loads return in issue order: behind two steps of weights per wavefront, 100 KB and more
            // per compute unit, the staging and its barrier would wait for all of those first)
            const int total = a.M * nkb;
            QuadActRaw ar[MFMA_ACT_PASSES];
            quad_act_issue(ar, a.q8, total);
            issue(bufA, 0);
            issue(bufB, 1);
            quad_act_wait<2 * LOADS>(ar);
            if (total <= MFMA_ACT_PASSES * (int)blockDim.x) // uniform
                mfma_act_store(ar, nkb, total, aq, asc);
            else
                mfma_stage_acts<SRC>(a.q8, a.x, a.x2, a.ldx, a.M, nkb, 0, nkb, aq, asc, (int)threadIdx.x, (int)blockDim.x);
        }
        else
        {
            issue(bufA, 0);
            issue(bufB, 1);
            mfma_stage_acts<SRC>(a.q8, a.x, a.x2, a.ldx, a.M, nkb, 0, nkb, aq, asc, (int)threadIdx.x, (int)blockDim.x);
        }
        __syncthreads();
        mfma_keep(bufA); // the staging code must not reuse the registers of the loads in flight
        mfma_keep(bufB);

        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
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
        const uint8_t *aq_lane = aq + (l32 & 7) * 32 + lh * 16; // rows beyond the batch: any row, result unused
        const float *asc_lane = asc + lh * 8;
        int step = 0;

        // the loaded pieces go to the wavefront's bounce buffer in piece order
        auto stage = [&](const MfmaRaw &r) {
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
            const int sb = slice + step * a.slices;
            const v4i q[4] = {q0, q1, q2, q3};
            Q4KQuad::Scale S[4];
            Q4KQuad::decode_scales(head, Q4KQuad::lane_consts(0), S[0]);
            Q4KQuad::decode_scales(head, Q4KQuad::lane_consts(1), S[1]);
            Q4KQuad::decode_scales(head, Q4KQuad::lane_consts(2), S[2]);
            Q4KQuad::decode_scales(head, Q4KQuad::lane_consts(3), S[3]);
            const uint8_t *ab = aq_lane + (size_t)sb * (8 * MFMA_AQ_STRIDE);
            const float *sb_sc = asc_lane + (size_t)sb * (8 * 16);
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
            // the product of block j+1 is issued before block j is rescaled: matrix unit and
            // vector unit work side by side
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

        // Two register buffers alternate; each is reloaded (two steps ahead) as soon as its
        // pieces are in LDS, before the step is computed.  Every buffer is waited for, also past
        // the end of the slice: a register whose load is still in flight must not look free to
        // the compiler.
        auto compute_lds = [&]() {
            compute(*reinterpret_cast<const v4i *>(bounce_rd), *reinterpret_cast<const v4i *>(bounce_rdq),
                    *reinterpret_cast<const v4i *>(bounce_rdq + 32), *reinterpret_cast<const v4i *>(bounce_rdq + 64),
                    *reinterpret_cast<const v4i *>(bounce_rdq + 96));
        };
        for (int c0 = 0; c0 < nsteps; c0 += 2)
        {
            if constexpr (PLANE)
            {
                // a buffer is reloaded once its step has been computed from it (a third buffer in the
                // rotation: 21.7 against 20.3 us at 25600 x 5120, batch 8)
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
                    stage(bufA);
                __builtin_amdgcn_sched_barrier(0);
                issue(bufA, c0 + 2);
                if (step < nsteps)
                    compute_lds();
                __builtin_amdgcn_sched_barrier(0);
                mfma_wait<LOADS>(bufB);
                if (step < nsteps)
                    stage(bufB);
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

        // ---- partial sums of the slices, added in slice order ---------------------------------
        __syncthreads(); // every wavefront is done with the activations
        float *red = reinterpret_cast<float *>(mfma_lds); // [wavefront][4][64]
#pragma unroll
        for (int i = 0; i < 4; ++i)
            red[(wave * 4 + i) * WAVE + lane] = acc[i];
        __syncthreads();
        // SWIGLU: the tiles' sums meet in LDS behind the partial sums, [tile][8 activation rows][32 weight rows]
        float *res = red + (size_t)(blockDim.x >> 6) * 4 * WAVE;
        if (slice == 0 && !idle)
        {
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                float v = acc[i];
                for (int s = 1; s < a.slices; ++s)
                    v += red[((wave + s) * 4 + i) * WAVE + lane];
                const int m = 4 * lh + i;
                if constexpr (SWIGLU)
                {
                    res[(tile_local * 8 + m) * 32 + l32] = v; // (rows past the batch: never read as results)
                    float *const y_mat = mat ? a.y2 : a.y;
                    if (y_mat && m < a.M && row_ok)
                        y_mat[(size_t)m * a.ldy + row] = v;
                }
                else if constexpr (!DUMP) // the block-sum variant has no fp32 output (y is null)
                {
                    if (m < a.M && row_ok)
                        a.y[(size_t)m * a.ldy + row] = v;
                }
            }
        }
        if constexpr (SWIGLU)
        {
            __syncthreads();
            // the first wavefront of a pair: eight lanes per activation row quantise its block (the lane
            // mapping of the stand-alone quantiser)
            if (slice == 0 && mat == 0 && !idle)
            {
                const int m = lane >> 3, sub = lane & 7;
                const float4 g = reinterpret_cast<const float4 *>(res + (tile_local * 8 + m) * 32)[sub];
                const float4 u = reinterpret_cast<const float4 *>(res + ((tile_local + 1) * 8 + m) * 32)[sub];
                const Q8Lane q = q8_1_quantize_lane(swiglu4(g, u));
                if (m < a.M && tile_row0 < a.N)
                {
                    uint32_t *dst = a.q8_out + ((size_t)m * (size_t)(a.N / 32) + (size_t)tile_idx) * 9;
                    dst[1 + sub] = q.packed;
                    if (sub == 0)
                        dst[0] = q.head;
                }
            }
        }
    }

    template <int SRC, bool DUMP = false, bool PLANE = false, bool SWIGLU = false>
    __global__ void __launch_bounds__((DUMP ? MFMA_DUMP_WAVES : MFMA_MAX_WAVES) * WAVE)
        gemv_mfma_q4k_kernel(const MfmaArgs a)
    {
        extern __shared__ __attribute__((aligned(16))) uint8_t mfma_lds[];
        gemv_mfma_q4k_body<SRC, DUMP, PLANE, SWIGLU>(a, mfma_lds, (int)blockIdx.x);
    }

    struct MfmaShape
    {
        int slices, tiles_per_wg, tile_rows;
        long grid;
    };
    // Most slices the LDS of a compute unit leaves room for (0: the row is too long for this kernel).
    inline int mfma_max_slices(int nsb)
    {
        const size_t act = mfma_act_bytes(nsb);
        if (act + MFMA_BOUNCE > QUAD_MAX_LDS)
            return 0;
        const size_t fit = (QUAD_MAX_LDS - act) / MFMA_BOUNCE;
        return fit < (size_t)MFMA_MAX_SLICES ? (int)fit : MFMA_MAX_SLICES;
    }
    int gemv_mfma_tile_rows_override();
    // The launch for tiles of `tile_rows` rows.  Slices so that a compute unit sees about a dozen
    // wavefronts, each at least two super-blocks long; tiles per workgroup so that every workgroup
    // of the launch is resident at once (a second round of workgroups would run nearly alone on
    // the chip and cost a workgroup's whole latency again) and the activations are staged less
    // often.
    inline MfmaShape gemv_mfma_shape_of(long N, int nsb, int cus, int max_waves, int tile_rows)
    {
        const long tiles = (N + tile_rows - 1) / tile_rows;
        long want = ((long)cus * 12 + tiles - 1) / tiles;
        if (want > mfma_max_slices(nsb))
            want = mfma_max_slices(nsb);
        if (want > nsb / 2)
            want = nsb / 2;
        if (want < 1)
            want = 1;
        MfmaShape sh;
        sh.tile_rows = tile_rows;
        const int per_slice = (int)((nsb + want - 1) / want);
        sh.slices = (nsb + per_slice - 1) / per_slice;
        // workgroups a compute unit holds at once: by LDS, and 16 wavefronts at this kernel's registers
        auto resident = [&](int t) {
            const long by_lds = (long)(QUAD_MAX_LDS / mfma_lds_bytes(nsb, t * sh.slices));
            const long by_waves = max_waves / (t * sh.slices);
            const long r = by_lds < by_waves ? by_lds : by_waves;
            return r < 1 ? 1 : r;
        };
        int t = 1;
        while (t * 2 * sh.slices <= max_waves && mfma_lds_bytes(nsb, t * 2 * sh.slices) <= QUAD_MAX_LDS &&
               (tiles + t - 1) / t > (long)cus * resident(t))
            t *= 2;
        sh.tiles_per_wg = t;
        sh.grid = (tiles + t - 1) / t;
        return sh;
    }
    // Tiles of 32 rows use every column of the matrix instruction, but their count rarely fits
    // the chip: 25600 rows are 800 tiles, 200 workgroups of four, and 56 compute units idle while
    // the others walk 128 rows each.  A compute unit's time goes with the rows it streams, so the
    // tile height that leaves the busiest compute unit the fewest rows wins; ties go to the
    // taller tile.
    // Gate and up in one launch: 2 N / 32 full tiles, an even number per workgroup.
    inline MfmaShape gemv_mfma_swiglu_shape(long N, int nsb, int cus)
    {
        MfmaShape sh = gemv_mfma_shape_of(2 * N, nsb, cus, MFMA_MAX_WAVES, MFMA_TILE_ROWS);
        if (sh.tiles_per_wg < 2)
        {
            // a pair needs both tiles in the workgroup: fewer wavefronts per tile where two tiles of the
            // chosen slices do not fit the LDS (slices <= 8, so 16 wavefronts always suffice)
            sh.tiles_per_wg = 2;
            while (sh.slices > 1 && mfma_lds_bytes(nsb, 2 * sh.slices) > QUAD_MAX_LDS)
                --sh.slices;
        }
        const long pairs = N / MFMA_TILE_ROWS, per_wg = sh.tiles_per_wg / 2;
        sh.grid = (pairs + per_wg - 1) / per_wg;
        return sh;
    }
    // LDS bytes of the launch: the activations (and bounce buffers), and at the end the partial sums of
    // every wavefront with the tiles' sums behind them
    inline size_t mfma_swiglu_lds_bytes(int nsb, int waves, int tiles, bool plane)
    {
        const size_t run = plane ? mfma_act_bytes(nsb) : mfma_lds_bytes(nsb, waves);
        const size_t end = (size_t)waves * 4 * WAVE * sizeof(float) + (size_t)tiles * 8 * 32 * sizeof(float);
        return run > end ? run : end;
    }

    inline MfmaShape gemv_mfma_shape(long N, int nsb, int cus, int max_waves = MFMA_MAX_WAVES)
    {
        const int forced = gemv_mfma_tile_rows_override();
        MfmaShape best;
        long best_cost = -1;
        for (int tr = MFMA_TILE_ROWS; tr >= MFMA_MIN_TILE_ROWS; --tr)
        {
            if (forced > 0 && tr != forced)
                continue;
            const MfmaShape sh = gemv_mfma_shape_of(N, nsb, cus, max_waves, tr);
            const long cost = ((sh.grid + cus - 1) / cus) * sh.tiles_per_wg * tr; // rows of the busiest compute unit
            if (best_cost < 0 || cost * 20 < best_cost * 19) // a shorter tile has to win 5 %
            {
                best = sh;
                best_cost = cost;
            }
        }
        return best;
    }
} // namespace llamql
