// IQ3_S x Q8_1 decode GEMV for gfx950: format traits for the shared skeleton.
//
// The reference's CPU path REQUANTISES every 32-element IQ3_S sub-block to int8
// at pack time (src/v2/tensors/SIMDHelpers.h:8612-8768): codebook magnitudes
// g in {1,3,..,15} times db = d*(1+2*nib), signed, then scale = max|v|/127 and
// w = rne(v/scale).  Because v = +-g*db with one db per sub-block this is the pure
// integer map  w = +-round(g*127/gmax)  (gmax = largest magnitude in the
// sub-block; never a tie) with  b_scale = f16((gmax*db)/127).  Every magnitude is odd,
// g = 2k+1 with k in 0..7, so for a given gmax the map is an 8-entry byte table: the
// kernel keeps the codebook in LDS as k-bytes (2 KB; bits 28..30 of an entry hold its
// largest k, so the largest of a sub-block's eight raw entries carries gmax), fetches
// that gmax's table (two dwords) and applies it with one byte permute per four weights;
// signs are applied with a second permute whose selector is spread out of the sign nibble.
// One LDS gather per four weights, none of them dependent on another.  HBM traffic stays
// at the format's 110 B per 256 weights (+2 B alignment padding).
//
// Device layout (llam_ql_prepare_weights): three planes over T = N*K/256
// super-blocks -- qs [T][64], signs [T][32], meta [T][16] = qh[8] scales[4] d[2]
// pad[2].  Lane c of an 8-lane group owns sub-block c.
#pragma once
#include "gemv_core.h"

#define LLAM_IQ3S_GRID_QUALIFIER static constexpr
#include "llaminar_amd/iq3s_grid.h"

namespace llamql
{
    struct IQ3STables
    {
        uint32_t cb[512];   // codebook entry idx as bytes k = g >> 1; bits 28..30: the entry's largest k
        uint32_t map[8][2]; // map[gi]: bytes round((2k+1)*127/(2*gi+1)) for k = 0..7 (k > gi is never looked up)
        bool odd;           // every codebook magnitude is odd and at most 15
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
            t.cb[idx] = e | (mx << 28);
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
        return t;
    }
    static_assert(make_iq3s_tables().odd, "IQ3_S codebook magnitudes must be odd and at most 15");

    static __device__ const IQ3STables g_iq3s_tables = make_iq3s_tables();

    struct IQ3STraits
    {
        static constexpr bool PAIR = false;
        static constexpr bool HAS_MIN = false;
        static constexpr bool USE_QUAD = false;
        static constexpr bool USE_MFMA_BATCH = false;  // matrix-unit kernel for 5..8 activation rows
        static constexpr int FAST_MAX_U = 3;          // load batches in flight in the chunked kernel
        static constexpr int TABLE_BYTES = (512 + 16) * 4; // cb, map

        __device__ static void stage_tables(void *lds_tab)
        {
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
            const uint2 *maps = reinterpret_cast<const uint2 *>(cb + 512);

            // picked with a bit mask: a conditional on two members of r would become a load
            // through a computed address and force arrays of Raw into memory
            const uint32_t m4 = (uint32_t)0 - (uint32_t)((c >> 2) & 1);
            const uint32_t qh = ((((r.meta.y & m4) | (r.meta.x & ~m4))) >> (8 * (c & 3))) & 0xFFu;
            const uint32_t nib = (r.meta.z >> (4 * c)) & 0xFu; // scales[c/2], low nibble for even c
            const float d = h2f((uint16_t)(r.meta.w & 0xFFFFu));

            uint32_t idx[8];
#pragma unroll
            for (int l = 0; l < 8; ++l)
            {
                const uint32_t qsb = ((l < 4 ? r.qs.x : r.qs.y) >> (8 * (l & 3))) & 0xFFu;
                idx[l] = qsb | (((qh >> l) & 1u) << 8);
            }
            uint32_t e[8];
#pragma unroll
            for (int l = 0; l < 8; ++l)
                e[l] = cb[idx[l]];
            uint32_t km = 0;
#pragma unroll
            for (int l = 0; l < 8; ++l)
                km = max(km, e[l]); // the field above every k byte decides
            km >>= 28;
            const uint32_t gm = 2u * km + 1u;

            const float db = d * (1.0f + 2.0f * (float)nib);
            const float amax = (float)gm * db;
            float scale = __fdiv_rn(amax, 127.0f);
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
#pragma unroll
            for (int l = 0; l < 8; ++l)
            {
                const uint32_t w = __builtin_amdgcn_perm(mp.y, mp.x, e[l] & 0x07070707u);
                const uint32_t sg = (sg_all >> (4 * l)) & 0xFu;
                // bit k of sg -> bit 0 of byte k, then selector byte k = k (keep) or k+4 (negated)
                const uint32_t sel = 0x03020100u | (((sg * 0x00204081u) & 0x01010101u) << 2);
                const uint32_t neg = 0x01010100u - w; // bytewise -w: every byte of w is in 1..127 (or all are 0)
                ws[l] = (int)__builtin_amdgcn_perm(neg, w, sel);
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
