// Q6_K x Q8_1 decode GEMV for gfx950: format traits for the shared skeleton.
//
// The reference's CPU path does not multiply Q6_K natively: at pack time it
// REQUANTISES every 32-element sub-block to int8 with one fp16 scale
// (src/v2/tensors/SIMDHelpers.h:12023-12204, 8.8 fixed point):
//     msc = max(|sc0|,|sc1|)              (the two 16-element Q6_K scales)
//     f_h = rne(sc_h*127*256 / (msc*32))  (int16), 0 when msc == 0
//     w   = ((q-32)*f_h + 128) >> 8       (int16 arithmetic, low byte kept)
//     b_scale = f16(d*msc*32/127)
// and the contract's per-block int32 sums are sums over those w.  This kernel
// performs the same requantisation in registers, straight from the 6-bit data,
// so HBM traffic stays at 210 B per 256 weights.
//
// Device layout (llam_ql_prepare_weights): four planes over T = N*K/256
// super-blocks -- ql [T][128], qh [T][64], scales [T][16], d [T] (fp16) -- so
// every load is 16-byte aligned (a raw 210-byte block is only 2-byte aligned).
//
// Lane c of an 8-lane group loads ql piece c (16 bytes).  With half = c/4,
// u = (c/2)&1, v = c&1 that piece holds elements 16v..16v+15 of sub-block
// 4*half+u (low nibbles) and of sub-block 4*half+2+u (high nibbles); their two
// upper bits sit in qh piece 2*half+v at bit offsets 2u and 2u+4.  The lane's 16
// elements of either sub-block share one 16-element Q6_K scale, hence one
// factor f.
#pragma once
#include "gemv_core.h"
#include "gemv_quad.h"


namespace llamql
{
    typedef unsigned short v2s __attribute__((ext_vector_type(2))); // wraps mod 2^16 by definition

    // ((q-32)*f + 128) >> 8 on four unsigned 6-bit values packed in `q`, bytewise.
    // (q-32)*f + 128 = q*f + (128 - 32 f) (mod 2^16); the true value is below 2^15 in
    // magnitude for |f| <= 1016, so wrapping 16-bit arithmetic is exact and
    // ">> 8, keep the low byte" is "take the high byte".
    __device__ __forceinline__ int q6k_requant4(uint32_t q, v2s ff, v2s cc)
    {
        const uint32_t e = q & 0x00FF00FFu;        // elements 0 and 2
        const uint32_t o = (q >> 8) & 0x00FF00FFu; // elements 1 and 3
        const v2s re = __builtin_bit_cast(v2s, e) * ff + cc;
        const v2s ro = __builtin_bit_cast(v2s, o) * ff + cc;
        // result bytes: [re.hi0, ro.hi0, re.hi1, ro.hi1]
        return (int)__builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, ro), __builtin_bit_cast(uint32_t, re),
                                          0x07030501u);
    }

    struct Q6KTraits
    {
        static constexpr bool PAIR = true;
        static constexpr bool HAS_MIN = false; // the reference's mins plane is all zero for Q6_K
        static constexpr bool USE_QUAD = true;        // quad-lane kernel for rows of >= 16 super-blocks
        static constexpr bool GEMM_PAIR_SCALES = false;   // prefill GEMM: scale products of two blocks per matrix instruction
        static constexpr bool USE_MFMA_BATCH = true;   // matrix-unit kernel for 5..8 activation rows
        typedef Q6KQuad Quad;
        static constexpr int FAST_MAX_U = 1;          // load batches in flight in the chunked kernel
        static constexpr int TABLE_BYTES = 0;
        __device__ static void *tables_lds() { return nullptr; }
        __device__ static void stage_tables(void *) {}

        struct Raw
        {
            uint4 ql;
            uint4 qh;
            uint4 sc;
            uint32_t d;
        };

        // Block j = 4*half + jj: jj&1 = u selects the 32-byte run of ql, jj>>1 says
        // low (0) or high (1) nibbles.  Dword q of the block -> v = q/4.
        __device__ __forceinline__ static void unit_of(int j, int q, int &c, int &p)
        {
            c = (j & 4) + 2 * (j & 1) + (q >> 2);
            p = (j >> 1) & 1;
        }

        __device__ __forceinline__ static void where(int c, int &j0, int &e0, int &j1, int &e1)
        {
            j0 = (c & 4) + ((c >> 1) & 1);
            j1 = j0 + 2;
            e0 = e1 = 16 * (c & 1);
        }

        __device__ __forceinline__ static Raw load(const GemvArgs &a, long row, int sb, int c)
        {
            const size_t T = (size_t)a.N * a.SB;
            const size_t t = (size_t)row * a.SB + sb;
            const uint8_t *base = static_cast<const uint8_t *>(a.w);
            const uint4 *ql = reinterpret_cast<const uint4 *>(base);
            const uint4 *qh = reinterpret_cast<const uint4 *>(base + T * 128);
            const uint4 *sc = reinterpret_cast<const uint4 *>(base + T * 192);
            const uint16_t *d = reinterpret_cast<const uint16_t *>(base + T * 208);
            Raw r;
            r.ql = ql[t * 8 + c];
            r.qh = qh[t * 4 + 2 * (c >> 2) + (c & 1)];
            r.sc = sc[t];
            r.d = d[t];
            return r;
        }

        // Byte i (0..15) of the 16 int8 sub-scales, sign-extended.  Dwords are picked with
        // bit masks rather than a conditional on the vector's members, which would turn
        // into an indexed access through memory.
        __device__ __forceinline__ static int sc_byte(const uint4 &s, int i)
        {
            const uint32_t m8 = (uint32_t)0 - (uint32_t)((i >> 3) & 1);
            const uint32_t m4 = (uint32_t)0 - (uint32_t)((i >> 2) & 1);
            const uint32_t lo = (s.y & m4) | (s.x & ~m4);
            const uint32_t hi = (s.w & m4) | (s.z & ~m4);
            const uint32_t w = (hi & m8) | (lo & ~m8);
            return __builtin_amdgcn_sbfe((int)w, 8u * (uint32_t)(i & 3), 8u);
        }

        __device__ __forceinline__ static void factor(int sc, float msc, v2s &ff, v2s &cc)
        {
            int f = 0;
            if (msc != 0.0f)
                f = (int)rintf(__fdiv_rn((float)sc * 127.0f * 256.0f, msc * 32.0f));
            const unsigned short fs = (unsigned short)f;
            const unsigned short cs = (unsigned short)(128 - 32 * f);
            ff = (v2s){fs, fs};
            cc = (v2s){cs, cs};
        }

        __device__ __forceinline__ static void decode(const Raw &r, int c, v4i &w0, v4i &w1, int &j,
                                                      float &bscale, float &bmin, const void *)
        {
            const int half = c >> 2, u = (c >> 1) & 1, v = c & 1;
            const int i_lo = 8 * half + 2 * u + v; // scale of the lane's low-nibble 16 elements
            const int i_hi = i_lo + 4;             // ... and of its high-nibble 16 elements
            const int sc_lo = sc_byte(r.sc, i_lo), sc_lo_other = sc_byte(r.sc, i_lo ^ 1);
            const int sc_hi = sc_byte(r.sc, i_hi), sc_hi_other = sc_byte(r.sc, i_hi ^ 1);
            const float msc_lo = fmaxf(fabsf((float)sc_lo), fabsf((float)sc_lo_other));
            const float msc_hi = fmaxf(fabsf((float)sc_hi), fabsf((float)sc_hi_other));
            v2s f_lo, c_lo, f_hi, c_hi;
            factor(sc_lo, msc_lo, f_lo, c_lo);
            factor(sc_hi, msc_hi, f_hi, c_hi);

            const int sh = 2 * u;
            const uint32_t ql[4] = {r.ql.x, r.ql.y, r.ql.z, r.ql.w};
            const uint32_t qh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
            int o0[4], o1[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                const uint32_t lo4 = ql[k] & 0x0F0F0F0Fu;
                const uint32_t hi4 = (ql[k] >> 4) & 0x0F0F0F0Fu;
                const uint32_t h = qh[k] >> sh;
                const uint32_t q_lo = lo4 | ((h & 0x03030303u) << 4);
                const uint32_t q_hi = hi4 | (((h >> 4) & 0x03030303u) << 4);
                o0[k] = q6k_requant4(q_lo, f_lo, c_lo); // f == 0 (msc == 0) yields 0 bytes
                o1[k] = q6k_requant4(q_hi, f_hi, c_hi);
            }
            w0 = (v4i){o0[0], o0[1], o0[2], o0[3]};
            w1 = (v4i){o1[0], o1[1], o1[2], o1[3]};

            // even lane (v=0) finishes the low-nibble sub-block, odd lane the high-nibble one
            j = 4 * half + u + 2 * v;
            const float msc = v ? msc_hi : msc_lo;
            const float d = h2f((uint16_t)r.d);
            bscale = (msc != 0.0f) ? f16_round_packer(__fdiv_rn(d * msc * 32.0f, 127.0f)) : 0.0f;
            bmin = 0.0f;
        }

        // ---- streaming interface of the full-row kernel ------------------------------
        struct Lane
        {
            int c, j;
        };
        __device__ __forceinline__ static Lane lane_consts(int c)
        {
            Lane l;
            l.c = c;
            l.j = (c & 4) + ((c >> 1) & 1) + 2 * (c & 1);
            return l;
        }

        struct Ptr
        {
            const uint4 *ql;
            const uint4 *qh;
            const uint4 *sc;
            const uint16_t *d;
        };
        __device__ __forceinline__ static Ptr ptr(const GemvArgs &a, long row, int sb, int c)
        {
            const size_t T = (size_t)a.N * a.SB;
            const size_t t = (size_t)row * a.SB + sb;
            const uint8_t *base = static_cast<const uint8_t *>(a.w);
            Ptr p;
            p.ql = reinterpret_cast<const uint4 *>(base) + t * 8 + c;
            p.qh = reinterpret_cast<const uint4 *>(base + T * 128) + t * 4 + 2 * (c >> 2) + (c & 1);
            p.sc = reinterpret_cast<const uint4 *>(base + T * 192) + t;
            p.d = reinterpret_cast<const uint16_t *>(base + T * 208) + t;
            return p;
        }
        __device__ __forceinline__ static void advance(Ptr &p, int nsb)
        {
            p.ql += (size_t)nsb * 8;
            p.qh += (size_t)nsb * 4;
            p.sc += nsb;
            p.d += nsb;
        }
        __device__ __forceinline__ static Raw load_at(const Ptr &p, int off_sb)
        {
            Raw r;
            r.ql = p.ql[off_sb * 8];
            r.qh = p.qh[off_sb * 4];
            r.sc = p.sc[off_sb];
            r.d = p.d[off_sb];
            return r;
        }
        __device__ __forceinline__ static void decode2(const Raw &r, const Lane &l, v4i &w0, v4i &w1,
                                                       float &bscale, float &bmin, const void *tab)
        {
            int j;
            decode(r, l.c, w0, w1, j, bscale, bmin, tab);
        }
    };
} // namespace llamql
