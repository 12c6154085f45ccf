// Q4_K x Q8_1 decode GEMV for gfx950: format traits for the shared skeleton.
//
// Weights stay in GGUF layout: a row is K/256 super-blocks of 144 B = nine
// 16-byte pieces (piece 0: d, dmin, 12 packed scale bytes; pieces 1..8: 128
// nibble bytes).  Lane c of an 8-lane group loads nibble piece c (one
// global_load_dwordx4) plus the shared header piece.  Piece c = 2g+h holds
// elements 16h..16h+15 of sub-block 2g (low nibbles) and of sub-block 2g+1
// (high nibbles) -- the nibble order of Q4_KTensor::packVnniBlock
// (src/v2/tensors/Q4_KTensor.cpp:768-792).  After the pair exchange lane c owns
// sub-block c and applies its effective scale f16(d*sc) and min f16(-dmin*m)
// (Q4_KTensor.cpp:794-799).  HBM-bound: 144 B per 256 weights.
#pragma once
#include "gemv_core.h"
#include "gemv_quad.h"


namespace llamql
{
    struct Q4KTraits
    {
        static constexpr bool PAIR = true;
        static constexpr bool HAS_MIN = true;
        static constexpr bool USE_QUAD = true;        // quad-lane kernel for rows of >= 16 super-blocks
        static constexpr bool GEMM_PAIR_SCALES = true;   // prefill GEMM: scale products of two blocks per matrix instruction
        static constexpr bool USE_MFMA_BATCH = true;  // matrix-unit kernel for 5..8 activation rows
        typedef Q4KQuad Quad;
        static constexpr int FAST_MAX_U = 4;          // load batches in flight in the chunked kernel
        static constexpr int TABLE_BYTES = 0;
        __device__ static void *tables_lds() { return nullptr; }
        __device__ static void stage_tables(void *) {}

        struct Raw
        {
            uint4 head;
            uint4 q;
        };

        // Block j (0..7) of a super-block, dword q (elements 4q..4q+3): piece
        // c = 2*(j/2) + (q/4); low-nibble blocks (even j) fill the first 16 bytes.
        __device__ __forceinline__ static void unit_of(int j, int q, int &c, int &p)
        {
            c = (j & ~1) + (q >> 2);
            p = j & 1;
        }

        // Where decode()'s w0 / w1 sit inside the super-block: block index and
        // first element (for kernels that lay the int8 values out again).
        __device__ __forceinline__ static void where(int c, int &j0, int &e0, int &j1, int &e1)
        {
            j0 = c & ~1;
            j1 = j0 + 1;
            e0 = e1 = 16 * (c & 1);
        }

        __device__ __forceinline__ static Raw load(const GemvArgs &a, long row, int sb, int c)
        {
            const uint4 *blk = static_cast<const uint4 *>(a.w) + ((size_t)row * a.SB + sb) * 9;
            Raw r;
            r.head = blk[0];
            r.q = blk[1 + c];
            return r;
        }

        __device__ __forceinline__ static void decode(const Raw &r, int c, v4i &w0, v4i &w1, int &j,
                                                      float &bscale, float &bmin, const void *)
        {
            w0.x = (int)(r.q.x & 0x0F0F0F0Fu); w1.x = (int)((r.q.x >> 4) & 0x0F0F0F0Fu);
            w0.y = (int)(r.q.y & 0x0F0F0F0Fu); w1.y = (int)((r.q.y >> 4) & 0x0F0F0F0Fu);
            w0.z = (int)(r.q.z & 0x0F0F0F0Fu); w1.z = (int)((r.q.z >> 4) & 0x0F0F0F0Fu);
            w0.w = (int)(r.q.w & 0x0F0F0F0Fu); w1.w = (int)((r.q.w >> 4) & 0x0F0F0F0Fu);
            j = c; // even lane: low-nibble sub-block 2g = c ; odd lane: high-nibble sub-block 2g+1 = c
            uint32_t sc, mn;
            q4k_scale_min(c, r.head.y, r.head.z, r.head.w, sc, mn);
            const float d = h2f((uint16_t)(r.head.x & 0xFFFFu));
            const float dmin = h2f((uint16_t)(r.head.x >> 16));
            bscale = f16_round_packer(d * (float)sc);
            bmin = f16_round_packer(-dmin * (float)mn);
        }

        // ---- streaming interface of the full-row kernel ------------------------------
        // Per-lane constants: where this lane's 6-bit scale and min sit in the 12 packed
        // bytes, as bit-field (offset, width) triples so the extraction is branch-free.
        struct Lane
        {
            int c, j;
            uint32_t sh, w_lo, w_hi2, w_p;
        };
        __device__ __forceinline__ static Lane lane_consts(int c)
        {
            Lane l;
            l.c = c;
            l.j = c;
            l.sh = 8u * (uint32_t)(c & 3);
            l.w_lo = (c < 4) ? 6u : 0u;  // j<4: six bits of byte j
            l.w_hi2 = (c < 4) ? 0u : 2u; // j>=4: top two bits of byte j-4 (scale) / j (min)
            l.w_p = (c < 4) ? 0u : 4u;   // j>=4: a nibble of byte j+4
            return l;
        }

        struct Ptr
        {
            const uint4 *head; // super-block header piece
            const uint4 *q;    // this lane's nibble piece
        };
        __device__ __forceinline__ static Ptr ptr(const GemvArgs &a, long row, int sb, int c)
        {
            Ptr p;
            p.head = static_cast<const uint4 *>(a.w) + ((size_t)row * a.SB + sb) * 9;
            p.q = p.head + 1 + c;
            return p;
        }
        __device__ __forceinline__ static void advance(Ptr &p, int nsb)
        {
            p.head += (size_t)nsb * 9;
            p.q += (size_t)nsb * 9;
        }
        __device__ __forceinline__ static Raw load_at(const Ptr &p, int off_sb)
        {
            Raw r;
            r.head = p.head[off_sb * 9];
            r.q = p.q[off_sb * 9];
            return r;
        }

        __device__ __forceinline__ static void decode2(const Raw &r, const Lane &l, v4i &w0, v4i &w1,
                                                       float &bscale, float &bmin, const void *)
        {
            w0.x = (int)(r.q.x & 0x0F0F0F0Fu); w1.x = (int)((r.q.x >> 4) & 0x0F0F0F0Fu);
            w0.y = (int)(r.q.y & 0x0F0F0F0Fu); w1.y = (int)((r.q.y >> 4) & 0x0F0F0F0Fu);
            w0.z = (int)(r.q.z & 0x0F0F0F0Fu); w1.z = (int)((r.q.z >> 4) & 0x0F0F0F0Fu);
            w0.w = (int)(r.q.w & 0x0F0F0F0Fu); w1.w = (int)((r.q.w >> 4) & 0x0F0F0F0Fu);
            const uint32_t u0 = r.head.y, u1 = r.head.z, u2 = r.head.w;
            const uint32_t sc = __builtin_amdgcn_ubfe(u0, l.sh, l.w_lo) |
                                (__builtin_amdgcn_ubfe(u0, l.sh + 6u, l.w_hi2) << 4) |
                                __builtin_amdgcn_ubfe(u2, l.sh, l.w_p);
            const uint32_t mn = __builtin_amdgcn_ubfe(u1, l.sh, l.w_lo) |
                                (__builtin_amdgcn_ubfe(u1, l.sh + 6u, l.w_hi2) << 4) |
                                __builtin_amdgcn_ubfe(u2, l.sh + 4u, l.w_p);
            const float d = h2f((uint16_t)(r.head.x & 0xFFFFu));
            const float dmin = h2f((uint16_t)(r.head.x >> 16));
            f16_round_packer2(d * (float)sc, -dmin * (float)mn, bscale, bmin);
        }
    };
} // namespace llamql
