// IQ3_S x Q8_1 decode GEMV for gfx950: format traits for the shared skeleton.
//
// The reference's CPU path REQUANTISES every 32-element IQ3_S sub-block to int8
// at pack time (src/v2/tensors/SIMDHelpers.h:8612-8768): codebook magnitudes
// g in {1,3,..,15} times db = d*(1+2*nib), signed, then scale = max|v|/127 and
// w = rne(v/scale).  Because v = +-g*db with one db per sub-block this is the pure
// integer map  w = +-round(g*127/gmax)  (gmax = largest magnitude in the
// sub-block; never a tie) with  b_scale = f16((gmax*db)/127).  Every magnitude is odd,
// g = 2k+1 with k in 0..7, so for a given gmax the map is an 8-entry byte table.  The kernel
// keeps in LDS (4.6 KB): the codebook as k-bytes (2 KB), the eight maps, and a 256-entry table
// that turns eight sign bits into two byte masks; a sub-block costs eight codebook gathers,
// one map fetch and four sign-mask gathers, and per four weights one v_perm_b32 (map), one
// subtraction (bytewise negation: every magnitude is 1..127) and one v_bfi_b32 (signs).
// Which map a sub-block needs -- its gmax -- is worked out when the weights are prepared and
// kept as a two-bit hint per sub-block in the two spare bytes of the super-block's meta
// record: 0, 1, 2 mean gmax 15, 13, 11 (93 %, 6 % and 1 % of sub-blocks with uniform codebook
// indices); 3 means "smaller": those few look their entries' maxima up in a byte table.  HBM
// traffic stays at the format's 110 B per 256 weights (+2 B alignment padding, which now
// carries the hints).
//
// Device layout (llam_ql_prepare_weights): three planes over T = N*K/256
// super-blocks -- qs [T][64], signs [T][32], meta [T][16] = qh[8] scales[4] d[2]
// hints[2].  Lane c of an 8-lane group owns sub-block c.
#pragma once
#include "gemv_core.h"
#include <cstddef>

#define LLAM_IQ3S_GRID_QUALIFIER static constexpr
#include "llaminar_amd/iq3s_grid.h"

namespace llamql
{
    struct IQ3STables
    {
        uint32_t cb[512];    // codebook entry idx as bytes k = g >> 1
        uint8_t cbmax[512];  // the entry's largest k
        uint32_t map[8][2];  // map[gi]: bytes round((2k+1)*127/(2*gi+1)) for k = 0..7 (k > gi is never looked up)
        uint32_t sgn[256][2]; // eight sign bits -> 0xFF bytes where the bit is set: elements 0-3, 4-7
        bool odd;            // every codebook magnitude is odd and at most 15
    };

    constexpr IQ3STables make_iq3s_tables()
    {
        IQ3STables t{};
        t.odd = true;
        for (int idx = 0; idx < 512; ++idx)
        {
            const uint32_t g4 = llam_iq3s_grid[idx];
            uint32_t mx = 0, e = 0;
            for (int b = 0; b < 4; ++b)
            {
                const uint32_t g = (g4 >> (8 * b)) & 0xFFu;
                if ((g & 1u) == 0u || g > 15u)
                    t.odd = false;
                const uint32_t k = g >> 1;
                if (k > mx)
                    mx = k;
                e |= k << (8 * b);
            }
            t.cb[idx] = e;
            t.cbmax[idx] = (uint8_t)mx;
        }
        for (int gi = 0; gi < 8; ++gi)
        {
            const uint32_t gm = 2u * (uint32_t)gi + 1u;
            for (int k = 0; k < 8; ++k)
            {
                const uint32_t g = 2u * (uint32_t)k + 1u;
                uint32_t q = (2u * g * 127u + gm) / (2u * gm); // round half up; never exactly half
                if (q > 127u)
                    q = 127u; // g > gm: never looked up
                t.map[gi][k >> 2] |= q << (8 * (k & 3));
            }
        }
        for (int s8 = 0; s8 < 256; ++s8)
            for (int b = 0; b < 8; ++b)
                if (s8 & (1 << b))
                    t.sgn[s8][b >> 2] |= 0xFFu << (8 * (b & 3));
        return t;
    }
    static_assert(make_iq3s_tables().odd, "IQ3_S codebook magnitudes must be odd and at most 15");

    static __device__ const IQ3STables g_iq3s_tables = make_iq3s_tables();

    // The gmax hint of a sub-block (two bits): the largest k of its eight codebook entries as
    // 7 - k for k = 7, 6, 5, and 3 for anything smaller.
    constexpr uint32_t IQ3S_HINT_OTHER = 3;
    __device__ __forceinline__ uint32_t iq3s_gmax_hint(const uint8_t *qs8, uint32_t qh)
    {
        uint32_t mx = 0;
#pragma unroll
        for (int l = 0; l < 8; ++l)
        {
            const uint32_t k = g_iq3s_tables.cbmax[qs8[l] | (((qh >> l) & 1u) << 8)];
            mx = k > mx ? k : mx;
        }
        return mx >= 5u ? 7u - mx : IQ3S_HINT_OTHER;
    }

    // (byte N of x) << sh in one instruction (sub-dword addressing of the operand).  sh is a
    // register operand; it holds a small constant.
    template <int N>
    __device__ __forceinline__ uint32_t byte_shl(uint32_t x, uint32_t sh)
    {
        uint32_t r;
        if constexpr (N == 0)
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(sh), "v"(x));
        else if constexpr (N == 1)
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(sh), "v"(x));
        else if constexpr (N == 2)
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(sh), "v"(x));
        else
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(sh), "v"(x));
        return r;
    }

    struct IQ3STraits
    {
        static constexpr bool PAIR = false;
        static constexpr bool HAS_MIN = false;
        static constexpr bool USE_QUAD = false;
        static constexpr bool USE_MFMA_BATCH = false;  // matrix-unit kernel for 5..8 activation rows
        static constexpr int FAST_MAX_U = 3;          // load batches in flight in the chunked kernel
        static constexpr int TABLE_BYTES = 2048 + 512 + 64 + 2048; // cb, cbmax, map, sgn

        __device__ static void stage_tables(void *lds_tab)
        {
            static_assert(offsetof(IQ3STables, cbmax) == 2048 && offsetof(IQ3STables, map) == 2560 &&
                              offsetof(IQ3STables, sgn) == 2624 && offsetof(IQ3STables, odd) == TABLE_BYTES,
                          "table offsets the decoder assumes");
            const uint4 *src = reinterpret_cast<const uint4 *>(&g_iq3s_tables);
            uint4 *dst = static_cast<uint4 *>(lds_tab);
            constexpr int n = TABLE_BYTES / 16;
            for (int i = threadIdx.x; i < n; i += blockDim.x)
                dst[i] = src[i];
        }

        struct Raw // no padding between members: arrays of it stay in registers
        {
            uint4 meta;
            uint2 qs;
            uint32_t signs;
            uint32_t spare;
        };

        // natural layout: block j is unit j, dword q at position q
        __device__ __forceinline__ static void unit_of(int j, int q, int &c, int &p)
        {
            c = j;
            p = q >> 2;
        }

        __device__ __forceinline__ static void where(int c, int &j0, int &e0, int &j1, int &e1)
        {
            j0 = j1 = c;
            e0 = 0;
            e1 = 16;
        }

        __device__ __forceinline__ static Raw load(const GemvArgs &a, long row, int sb, int c)
        {
            const size_t T = (size_t)a.N * a.SB;
            const size_t t = (size_t)row * a.SB + sb;
            const uint8_t *base = static_cast<const uint8_t *>(a.w);
            Raw r;
            r.spare = 0;
            r.qs = reinterpret_cast<const uint2 *>(base)[t * 8 + c];
            r.signs = reinterpret_cast<const uint32_t *>(base + T * 64)[t * 8 + c];
            r.meta = reinterpret_cast<const uint4 *>(base + T * 96)[t];
            return r;
        }

        __device__ __forceinline__ static void decode(const Raw &r, int c, v4i &w0, v4i &w1, int &j,
                                                      float &bscale, float &bmin, const void *tab)
        {
            const uint32_t *cb = static_cast<const uint32_t *>(tab);
            const uint8_t *cbmax = static_cast<const uint8_t *>(tab) + 2048;
            const uint2 *maps = reinterpret_cast<const uint2 *>(static_cast<const uint8_t *>(tab) + 2560);
            const uint2 *sgn = reinterpret_cast<const uint2 *>(static_cast<const uint8_t *>(tab) + 2624);

            // picked with a bit mask: a conditional on two members of r would become a load
            // through a computed address and force arrays of Raw into memory
            const uint32_t m4 = (uint32_t)0 - (uint32_t)((c >> 2) & 1);
            const uint32_t qh = ((((r.meta.y & m4) | (r.meta.x & ~m4))) >> (8 * (c & 3))) & 0xFFu;
            const uint32_t nib = (r.meta.z >> (4 * c)) & 0xFu; // scales[c/2], low nibble for even c
            const float d = h2f((uint16_t)(r.meta.w & 0xFFFFu));
            const uint32_t hint = (r.meta.w >> (16 + 2 * c)) & 3u;

            // byte offsets of the eight codebook entries: (qs byte l) * 4 + (bit l of qh) * 1024
            const uint8_t *cbb = static_cast<const uint8_t *>(tab);
            uint32_t off[8];
            {
                const uint32_t two = 2u;
                const uint32_t a0 = byte_shl<0>(r.qs.x, two), a1 = byte_shl<1>(r.qs.x, two), a2 = byte_shl<2>(r.qs.x, two),
                               a3 = byte_shl<3>(r.qs.x, two), a4 = byte_shl<0>(r.qs.y, two), a5 = byte_shl<1>(r.qs.y, two),
                               a6 = byte_shl<2>(r.qs.y, two), a7 = byte_shl<3>(r.qs.y, two);
                const uint32_t a[8] = {a0, a1, a2, a3, a4, a5, a6, a7};
#pragma unroll
                for (int l = 0; l < 8; ++l)
                    off[l] = (((qh >> l) & 1u) << 10) | a[l]; // v_bfe_u32 + v_lshl_or_b32
            }
            uint32_t e[8];
#pragma unroll
            for (int l = 0; l < 8; ++l)
                e[l] = *reinterpret_cast<const uint32_t *>(cbb + off[l]);
            uint32_t km = 7u - hint;
            if (__builtin_expect(hint == IQ3S_HINT_OTHER, 0))
            {
                // a sub-block whose largest magnitude is 9 or less (3 in 10000 with uniform indices)
                km = 0;
#pragma unroll
                for (int l = 0; l < 8; ++l)
                    km = max(km, (uint32_t)cbmax[off[l] >> 2]);
            }

            // amax = gmax * (d * (1 + 2 nib)) is exact in fp32 (11 x 5 x 4 bits), so is d * (gmax * (1 + 2 nib))
            const float amax = d * (float)((2u * km + 1u) * (2u * nib + 1u));
            float scale = div_by_127(amax);
            if (scale > 65504.0f)
                scale = 65504.0f;
            if (amax < 1e-6f)
                scale = 0.0f;

            uint2 mp = maps[km];
            uint32_t sg_all = r.signs;
            if (scale == 0.0f) // all-zero sub-block: zero magnitudes, and no sign to apply to them
            {
                mp = make_uint2(0u, 0u);
                sg_all = 0u;
            }
            int ws[8];
            {
                const uint8_t *sgb = reinterpret_cast<const uint8_t *>(sgn);
                const uint32_t three = 3u;
                // byte masks of elements 8p..8p+3 (x) and 8p+4..8p+7 (y)
                const uint2 sm[4] = {*reinterpret_cast<const uint2 *>(sgb + byte_shl<0>(sg_all, three)),
                                     *reinterpret_cast<const uint2 *>(sgb + byte_shl<1>(sg_all, three)),
                                     *reinterpret_cast<const uint2 *>(sgb + byte_shl<2>(sg_all, three)),
                                     *reinterpret_cast<const uint2 *>(sgb + byte_shl<3>(sg_all, three))};
#pragma unroll
                for (int l = 0; l < 8; ++l)
                {
                    const uint32_t w = __builtin_amdgcn_perm(mp.y, mp.x, e[l]);
                    const uint32_t neg = 0x01010100u - w; // bytewise -w: every byte of w is in 1..127 (or all are 0)
                    const uint32_t mask = (l & 1) ? sm[l >> 1].y : sm[l >> 1].x;
                    ws[l] = (int)((neg & mask) | (w & ~mask)); // v_bfi_b32
                }
            }
            w0 = (v4i){ws[0], ws[1], ws[2], ws[3]};
            w1 = (v4i){ws[4], ws[5], ws[6], ws[7]};
            j = c;
            bscale = f16_round_packer(scale);
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
            l.j = c;
            return l;
        }

        struct Ptr
        {
            const uint2 *qs;
            const uint32_t *signs;
            const uint4 *meta;
        };
        __device__ __forceinline__ static Ptr ptr(const GemvArgs &a, long row, int sb, int c)
        {
            const size_t T = (size_t)a.N * a.SB;
            const size_t t = (size_t)row * a.SB + sb;
            const uint8_t *base = static_cast<const uint8_t *>(a.w);
            Ptr p;
            p.qs = reinterpret_cast<const uint2 *>(base) + t * 8 + c;
            p.signs = reinterpret_cast<const uint32_t *>(base + T * 64) + t * 8 + c;
            p.meta = reinterpret_cast<const uint4 *>(base + T * 96) + t;
            return p;
        }
        __device__ __forceinline__ static void advance(Ptr &p, int nsb)
        {
            p.qs += (size_t)nsb * 8;
            p.signs += (size_t)nsb * 8;
            p.meta += nsb;
        }
        __device__ __forceinline__ static Raw load_at(const Ptr &p, int off_sb)
        {
            Raw r;
            r.qs = p.qs[off_sb * 8];
            r.signs = p.signs[off_sb * 8];
            r.meta = p.meta[off_sb];
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
