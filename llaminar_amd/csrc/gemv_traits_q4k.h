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
        typedef Q4KQuad Quad;
        static constexpr bool USE_STREAM = true;      // row-streaming kernel pays off for this format
        static constexpr int FAST_MAX_U = 4;          // load batches in flight in the chunked kernel
        static constexpr int STREAM_MAX_THREADS = 1024; // workgroup size bound of the row-streaming kernel
        static constexpr int STREAM_U_PAIR = 5;   // loads per lane and chunk, row-pair passes
        static constexpr int STREAM_U_SINGLE = 4; // ... single-row passes
        static constexpr int TABLE_BYTES = 0;
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

        // ---- leanest form, used by the row-streaming kernel ------------------------------
        // The two fp16 products are formed directly in packed half precision: d (11-bit
        // significand) times a 6-bit integer is exact before rounding, so one
        // round-to-nearest-even f16 multiply equals f16(fp32 product); the packer's
        // truncating rule for fp16-subnormal results is applied on a rarely taken branch
        // (only possible when d or dmin is below 2^-13).  Scale holds {b_scale, |b_min|}.
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        struct Scale
        {
            h2 p;
        };
        struct Lane3
        {
            uint32_t sel, psh, m1, m2, m3;
        };
        __device__ __forceinline__ static Lane3 lane3_consts(int c)
        {
            Lane3 l;
            const uint32_t b = (uint32_t)(c & 3);
            l.sel = b | (0x0Cu << 8) | ((4u + b) << 16) | (0x0Cu << 24);
            l.psh = 8u * b;
            l.m1 = (c < 4) ? 0x003F003Fu : 0u;
            l.m2 = (c < 4) ? 0u : 0x00300030u;
            l.m3 = (c < 4) ? 0u : 0x000F000Fu;
            return l;
        }
        __device__ __forceinline__ static uint16_t f16_trunc_bits(float x)
        {
            // fp16 bit pattern of x truncated toward zero in the subnormal range (|x| < 2^-14)
            const uint32_t mag = (uint32_t)truncf(fabsf(x) * 16777216.0f);
            return (uint16_t)(mag | ((__float_as_uint(x) >> 16) & 0x8000u));
        }
        __device__ __forceinline__ static void decode3(const Raw &r, const Lane3 &l, v4i &w0, v4i &w1, Scale &S,
                                                       const void *)
        {
            w0.x = (int)(r.q.x & 0x0F0F0F0Fu); w1.x = (int)((r.q.x >> 4) & 0x0F0F0F0Fu);
            w0.y = (int)(r.q.y & 0x0F0F0F0Fu); w1.y = (int)((r.q.y >> 4) & 0x0F0F0F0Fu);
            w0.z = (int)(r.q.z & 0x0F0F0F0Fu); w1.z = (int)((r.q.z >> 4) & 0x0F0F0F0Fu);
            w0.w = (int)(r.q.w & 0x0F0F0F0Fu); w1.w = (int)((r.q.w >> 4) & 0x0F0F0F0Fu);
            // {sc, mn} as two 16-bit integers
            const uint32_t X = __builtin_amdgcn_perm(r.head.z, r.head.y, l.sel); // {scales[b], scales[b+4]}
            const uint32_t P = __builtin_amdgcn_ubfe(r.head.w, l.psh, 8u);      // scales[b+8]
            const uint32_t Pp = P | (P << 12);
            const uint32_t sm = (X & l.m1) | ((X >> 2) & l.m2) | (Pp & l.m3);
            // integer n in 0..63 -> f16: 0x6400|n is 1024+n
            const h2 f = __builtin_bit_cast(h2, sm | 0x64006400u) - (h2){(_Float16)1024.0f, (_Float16)1024.0f};
            const uint32_t dd = r.head.x; // {d, dmin}
            S.p = __builtin_bit_cast(h2, dd) * f;
            const uint32_t e = dd & 0x7C007C00u;
            if (__builtin_expect(((e - 0x08000800u) & 0x80008000u) != 0u, 0))
            {
                const float xs = h2f((uint16_t)(dd & 0xFFFFu)) * (float)(sm & 0xFFFFu);
                const float xm = h2f((uint16_t)(dd >> 16)) * (float)(sm >> 16);
                uint32_t bits = __builtin_bit_cast(uint32_t, S.p);
                if (fabsf(xs) < 6.103515625e-05f)
                    bits = (bits & 0xFFFF0000u) | f16_trunc_bits(xs);
                if (fabsf(xm) < 6.103515625e-05f)
                    bits = (bits & 0x0000FFFFu) | ((uint32_t)f16_trunc_bits(xm) << 16);
                S.p = __builtin_bit_cast(h2, bits);
            }
        }
        __device__ __forceinline__ static float cs(const Scale &S, float ad) { return fmaf(ad, (float)S.p.x, 0.0f); }
        __device__ __forceinline__ static float add_min(const Scale &S, float asd, float acc)
        {
            return fmaf(asd, -(float)S.p.y, acc);
        }
    };
} // namespace llamql
