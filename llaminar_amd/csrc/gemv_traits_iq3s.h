// IQ3_S x Q8_1 decode GEMV for gfx950: format traits for the shared skeleton and the
// quad-lane decoder.
//
// The reference's CPU path REQUANTISES every 32-element IQ3_S sub-block to int8
// at pack time (src/v2/tensors/SIMDHelpers.h:8612-8768): codebook magnitudes
// g in {1,3,..,15} times db = d*(1+2*nib), signed, then scale = max|v|/127 and
// w = rne(v/scale).  Because v = +-g*db with one db per sub-block this is the pure
// integer map  w = +-round(g*127/gmax)  (gmax = largest magnitude in the
// sub-block; never a tie) with  b_scale = f16((gmax*db)/127).  Every magnitude is odd,
// g = 2k+1 with k in 0..7, so for a given gmax the map is an 8-entry byte table.  The kernels
// keep in (static) LDS, 4.9 KB: the codebook as k-bytes (2 KB), the maps, a 256-entry
// table that turns eight sign bits into two byte masks, and the 48 products (15 - 2 hint) *
// (1 + 2 nib) as floats; a sub-block costs eight codebook gathers, one map fetch, four sign-mask
// gathers and one scale fetch, and per four weights one v_perm_b32 (map), one subtraction
// (bytewise negation: every magnitude is 1..127) and one v_bfi_b32 (signs).  (Signs through one
// v_xad_u32, (w ^ mask) + ones, need the masks' 0x01 bytes from the table as well: eight vector
// instructions fewer per sub-block and 16-byte gathers for 8-byte ones, 5 % slower -- the LDS
// is as busy as the vector unit here.)
//
// What a sub-block needs beyond its bytes is worked out when the weights are prepared and kept
// as a two-bit hint per sub-block in the two spare bytes of the super-block's meta record:
// 0, 1, 2 mean "regular, gmax 15, 13, 11" (93 %, 6 % and 1 % of sub-blocks with uniform
// codebook indices), where regular says that the scale is an ordinary fp16 number, so that the
// decoder needs no test for zero, overflow, subnormal or non-finite scales; 3 means "anything
// else": those few take the general path (maxima from a byte table, every special case).  HBM
// traffic stays at the format's 110 B per 256 weights (+2 B alignment padding, which now
// carries the hints).
//
// Device layout (llam_ql_prepare_weights): three planes over T = N*K/256
// super-blocks -- qs [T][64], signs [T][32], meta [T][16] = qh[8] scales[4] d[2]
// hints[2].  In the shared skeleton lane c of an 8-lane group owns sub-block c; in the
// quad-lane kernel lane l of a quad owns sub-blocks 2l and 2l+1.
#pragma once
#include "gemv_core.h"
#include "gemv_quad.h"
#include <cstddef>

#define LLAM_IQ3S_GRID_QUALIFIER static constexpr
#include "llaminar_amd/iq3s_grid.h"

namespace llamql
{
    struct IQ3STables
    {
        uint32_t cb[512];     // codebook entry idx as bytes k = g >> 1
        uint8_t cbmax[512];   // the entry's largest k
        uint32_t map[10][2];  // map[7 - gi]: bytes round((2k+1)*127/(2*gi+1)) for k = 0..7 (k > gi is never
                              // looked up); map[8], map[9]: zeros (an all-zero sub-block)
        uint32_t sgn[256][2]; // eight sign bits -> 0xFF bytes where the bit is set: elements 0-3, 4-7
        float gmul[4][16];    // [hint][nib]: (15 - 2 hint) * (1 + 2 nib), what d is multiplied by in a regular sub-block
        bool odd;             // every codebook magnitude is odd and at most 15
    };
    constexpr int IQ3S_TABLE_BYTES = 2048 + 512 + 80 + 2048 + 256;
    constexpr int IQ3S_OFF_CBMAX = 2048, IQ3S_OFF_MAP = 2560, IQ3S_OFF_SGN = 2640, IQ3S_OFF_GMUL = 4688;
    constexpr uint32_t IQ3S_MAP_ZERO = 8; // index of the all-zero map

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
                t.map[7 - gi][k >> 2] |= q << (8 * (k & 3));
            }
        }
        for (int s8 = 0; s8 < 256; ++s8)
            for (int b = 0; b < 8; ++b)
                if (s8 & (1 << b))
                    t.sgn[s8][b >> 2] |= 0xFFu << (8 * (b & 3));
        for (int h = 0; h < 3; ++h)
            for (int nib = 0; nib < 16; ++nib)
                t.gmul[h][nib] = (float)((15 - 2 * h) * (1 + 2 * nib));
        return t;
    }
    static_assert(make_iq3s_tables().odd, "IQ3_S codebook magnitudes must be odd and at most 15");
    static_assert(offsetof(IQ3STables, cbmax) == IQ3S_OFF_CBMAX && offsetof(IQ3STables, map) == IQ3S_OFF_MAP &&
                      offsetof(IQ3STables, sgn) == IQ3S_OFF_SGN && offsetof(IQ3STables, gmul) == IQ3S_OFF_GMUL &&
                      offsetof(IQ3STables, odd) == IQ3S_TABLE_BYTES &&
                      IQ3S_TABLE_BYTES % 16 == 0,
                  "table offsets the decoder assumes");

    static __device__ const IQ3STables g_iq3s_tables = make_iq3s_tables();

    // The tables' place in LDS: a static array, so that its address is a link-time constant and
    // every look-up is a ds_read with an immediate offset.  Every kernel that decodes IQ3_S
    // fills it (iq3s_stage_tables) before its first barrier.
    __device__ __forceinline__ uint8_t *iq3s_tables_lds()
    {
        __shared__ __attribute__((aligned(16))) uint8_t iq3s_tables[IQ3S_TABLE_BYTES];
        return iq3s_tables;
    }
    __device__ __forceinline__ void iq3s_stage_tables()
    {
        const uint4 *src = reinterpret_cast<const uint4 *>(&g_iq3s_tables);
        uint4 *dst = reinterpret_cast<uint4 *>(iq3s_tables_lds());
        constexpr int n = IQ3S_TABLE_BYTES / 16;
        for (int i = threadIdx.x; i < n; i += blockDim.x)
            dst[i] = src[i];
    }

    // The same in two halves, for a kernel that has dependent loads to wait for while the tables
    // travel: one 16-byte piece per thread (workgroups of at least IQ3S_TABLE_BYTES / 16 threads),
    // asked for with an assembly load so that the kernel decides where it is waited for; never
    // predicated (threads past the end re-read the last piece).
    struct IQ3STablesRaw
    {
        int v __attribute__((ext_vector_type(4)));
    };
    constexpr int IQ3S_TABLE_THREADS = IQ3S_TABLE_BYTES / 16;
    __device__ __forceinline__ void iq3s_tables_issue(IQ3STablesRaw &r)
    {
        const int i = min((int)threadIdx.x, IQ3S_TABLE_THREADS - 1);
        const uint4 *src = reinterpret_cast<const uint4 *>(&g_iq3s_tables) + i;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(r.v) : "v"(src));
    }
    // until at most NEWER vector memory operations issued after the tables' load are pending
    template <int NEWER>
    __device__ __forceinline__ void iq3s_tables_wait(IQ3STablesRaw &r)
    {
        static_assert(NEWER <= 63, "vmcnt is a 6-bit counter");
        asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r.v) : "n"(NEWER));
    }
    __device__ __forceinline__ void iq3s_tables_store(const IQ3STablesRaw &r)
    {
        typedef int v4 __attribute__((ext_vector_type(4)));
        if (threadIdx.x < IQ3S_TABLE_THREADS)
            reinterpret_cast<v4 *>(iq3s_tables_lds())[threadIdx.x] = r.v;
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

    // The general scale of a sub-block whose largest codebook byte is km: amax = gmax * (d * (1 + 2 nib))
    // is exact in fp32 (11 x 5 x 4 bits), so is d * (gmax * (1 + 2 nib)).  Returns the scale before
    // its fp16 rounding; 0 for a sub-block the packer treats as all zero.
    __device__ __forceinline__ float iq3s_scale_general(float d, uint32_t km, uint32_t nib)
    {
        const float amax = d * (float)((2u * km + 1u) * (2u * nib + 1u));
        float scale = div_by_127(amax);
        if (scale > 65504.0f)
            scale = 65504.0f;
        if (amax < 1e-6f)
            scale = 0.0f;
        return scale;
    }

    // The hint of a sub-block (two bits), worked out when the weights are prepared.
    constexpr uint32_t IQ3S_HINT_OTHER = 3;
    __device__ __forceinline__ uint32_t iq3s_block_hint(const uint8_t *qs8, uint32_t qh, uint32_t nib, float d)
    {
        uint32_t mx = 0;
#pragma unroll
        for (int l = 0; l < 8; ++l)
        {
            const uint32_t k = g_iq3s_tables.cbmax[qs8[l] | (((qh >> l) & 1u) << 8)];
            mx = k > mx ? k : mx;
        }
        if (mx < 5u)
            return IQ3S_HINT_OTHER;
        // regular: a positive scale inside the normal fp16 range (which excludes zeros, clamped,
        // subnormal-after-rounding and non-finite scales; a NaN fails both comparisons)
        const float scale = iq3s_scale_general(d, mx, nib);
        const bool regular = scale >= 6.103515625e-05f && scale < 65504.0f;
        return regular ? 7u - mx : IQ3S_HINT_OTHER;
    }

    // One 32-element sub-block to int8 weights and its scale.
    //   qs: the eight low index bytes; qh: bit l is the ninth bit of index l (bits above 7 are ignored);
    //   nib: the 4-bit sub-block scale; hint: see above; signs: the 32 sign bits; d: the super-block scale
    __device__ __forceinline__ void iq3s_decode_block(const uint2 qs, const uint32_t qh, const uint32_t nib,
                                                      const uint32_t hint, const float d, const uint32_t signs,
                                                      v4i &w0, v4i &w1, float &bscale)
    {
        const uint8_t *tab = iq3s_tables_lds();

        // Byte offsets of the eight codebook entries: (qs byte l) * 4 + (bit l of qh) * 1024, that is
        // low byte (b << 2) & 0xFC and high byte (b >> 6) | bit << 2.  Four at a time: the dword of
        // index bytes rotated right by six holds, in byte l, the two top bits of index byte l at the
        // bottom and the six low bits of index byte l + 1 above them; four bits of qh times a constant
        // with one bit per byte land on bit 2 of bytes 0..3 (the shifted copies of the four bits do
        // not overlap: nothing carries).  One v_perm_b32 per offset then picks its two bytes: 6 + 4
        // instructions per dword where shifting and merging each offset by itself took 12.
        uint32_t off[8];
#pragma unroll
        for (int h = 0; h < 2; ++h)
        {
            const uint32_t q = h ? qs.y : qs.x;
            const uint32_t rot = __builtin_amdgcn_alignbit(q, q, 6);
            const uint32_t lo = rot & 0xFCFCFCFCu;  // byte l: (index byte (l + 1) & 3) << 2, truncated
            const uint32_t top = rot & 0x03030303u; // byte l: (index byte l) >> 6
            const uint32_t nib4 = h ? (qh >> 4) & 0xFu : qh & 0xFu;
            const uint32_t spread = __umul24(nib4, (1u << 2) | (1u << 9) | (1u << 16) | (1u << 23)); // bit l -> bit 8 l + 2
            const uint32_t hi = (spread & 0x04040404u) | top;
            off[4 * h + 0] = __builtin_amdgcn_perm(hi, lo, 0x0C0C0403u);
            off[4 * h + 1] = __builtin_amdgcn_perm(hi, lo, 0x0C0C0500u);
            off[4 * h + 2] = __builtin_amdgcn_perm(hi, lo, 0x0C0C0601u);
            off[4 * h + 3] = __builtin_amdgcn_perm(hi, lo, 0x0C0C0702u);
        }
        uint32_t e[8];
#pragma unroll
        for (int l = 0; l < 8; ++l)
            e[l] = *reinterpret_cast<const uint32_t *>(tab + off[l]);

        // regular sub-block: gmax = 15 - 2 hint; scale = f16(d * gmax * (1 + 2 nib) / 127), finite,
        // not zero and a normal fp16 number, so nearest-even is the packer's rounding
        uint32_t mi = hint; // which map
        uint32_t sg_all = signs;
        {
            // (15 - 2 hint) * (1 + 2 nib) as a float from a 64-entry table: three instructions for seven
            const float amax = d * *reinterpret_cast<const float *>(tab + IQ3S_OFF_GMUL + ((hint << 6) | (nib << 2)));
            const float c = 0x1.020408p-7f;
            const float q0 = amax * c;
            const float q1 = fmaf(fmaf(-q0, 127.0f, amax), c, q0); // div_by_127 of a finite non-zero value
            bscale = __half2float(__float2half_rn(q1));
        }
        if (__builtin_expect(hint == IQ3S_HINT_OTHER, 0))
        {
            // 3 in 10000 with uniform indices: largest magnitude 9 or less, or a special scale
            uint32_t km = 0;
#pragma unroll
            for (int l = 0; l < 8; ++l)
                km = max(km, (uint32_t)tab[IQ3S_OFF_CBMAX + (off[l] >> 2)]);
            const float scale = iq3s_scale_general(d, km, nib);
            bscale = f16_round_packer(scale);
            mi = 7u - km;
            if (scale == 0.0f) // all-zero sub-block: zero magnitudes, and no sign to apply to them
            {
                mi = IQ3S_MAP_ZERO;
                sg_all = 0u;
            }
        }
        const uint2 mp = *reinterpret_cast<const uint2 *>(tab + IQ3S_OFF_MAP + mi * 8u);

        int ws[8];
        {
            const uint8_t *sgb = tab + IQ3S_OFF_SGN;
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
    }

    // ---- quad-lane decoder -------------------------------------------------------------
    // Lane l of a quad decodes sub-blocks 2l and 2l+1: 16 bytes of qs, 8 of signs, and the
    // super-block's meta record (the four lanes ask for the same 16 bytes).  Weight addresses
    // are 32-bit offsets from the plane bases.
    struct IQ3SQuad
    {
        typedef int v2i_ __attribute__((ext_vector_type(2)));
        static constexpr int LOADS = 3;
        static constexpr int STATIC_LDS = IQ3S_TABLE_BYTES;
        // 16 wavefronts of 128 registers for a single activation row
        static constexpr int max_threads(int M) { return M == 1 ? 1024 : 512; }
        // the decoder is arithmetic-bound: a compute unit should hold 16 wavefronts
        static constexpr int RESIDENT_WAVES = 16;
        static bool addressable(long N, int SB) { return (double)N * SB * 64.0 < 4.0e9; }
        __device__ __forceinline__ static void stage() { iq3s_stage_tables(); }
        // the tables fetched ahead (workgroups of at least TABLE_THREADS threads)
        typedef IQ3STablesRaw TablesRaw;
        static constexpr int TABLE_THREADS = IQ3S_TABLE_THREADS;
        __device__ __forceinline__ static void tables_issue(TablesRaw &r) { iq3s_tables_issue(r); }
        template <int NEWER>
        __device__ __forceinline__ static void tables_wait(TablesRaw &r) { iq3s_tables_wait<NEWER>(r); }
        __device__ __forceinline__ static void tables_store(const TablesRaw &r) { iq3s_tables_store(r); }

        struct Raw
        {
            v4i qs, meta;
            v2i_ sg;
        };
        struct Lane
        {
            uint32_t l;
            uint32_t qh_sel; // v_perm selector: qh bytes 2l and 2l+1 of {meta.x, meta.y} into bits 0-7 and 16-23
        };
        struct Scale
        {
            float bs0, bs1;
        };
        struct Cursor
        {
            const uint8_t *qs, *sg, *meta; // plane bases (uniform)
            uint32_t t, first;             // this lane's super-block index: current, and the one read
                                           // instead past the end of the run
        };

        __device__ __forceinline__ static Lane lane_consts(int l)
        {
            Lane c;
            c.l = (uint32_t)l;
            const uint32_t b = 2u * (uint32_t)l;
            c.qh_sel = b | (0x0Cu << 8) | ((b + 1u) << 16) | (0x0Cu << 24);
            return c;
        }
        __device__ __forceinline__ static void owner(int j, int &l, int &which)
        {
            l = j >> 1;
            which = j & 1;
        }
        __device__ __forceinline__ static int block_of(int l, int which) { return 2 * l + which; }

        __device__ __forceinline__ static Cursor cursor(const GemvArgs &a, size_t t, size_t t_safe, const Lane &)
        {
            const size_t T = (size_t)a.N * a.SB;
            Cursor c;
            c.qs = static_cast<const uint8_t *>(a.w);
            c.sg = c.qs + T * 64;
            c.meta = c.qs + T * 96;
            c.t = (uint32_t)t;
            c.first = (uint32_t)t_safe;
            return c;
        }
        // super-blocks a lane moves by per step, without and with a row crossing (Q4KQuad::Stride)
        struct Stride
        {
            uint32_t plain, cross;
        };
        __device__ __forceinline__ static Stride stride(uint32_t jump)
        {
            Stride st;
            st.plain = (uint32_t)QUAD_STEP_SB;
            st.cross = (uint32_t)QUAD_STEP_SB + jump;
            return st;
        }
        __device__ __forceinline__ static void next(Cursor &c, bool cross, const Stride &st)
        {
            c.t += cross ? st.cross : st.plain;
        }
        __device__ __forceinline__ static void load(Raw &r, const Cursor &c, const Lane &lc, bool valid)
        {
            load_index(r, c, lc, valid ? c.t : c.first);
        }
        __device__ __forceinline__ static void load_at(Raw &r, const Cursor &c, const Lane &lc, int sb_off)
        {
            load_index(r, c, lc, c.t + (uint32_t)sb_off);
        }
        // Loads issued as assembly so that the kernel decides where they are waited for.
        __device__ __forceinline__ static void load_index(Raw &r, const Cursor &c, const Lane &lc, uint32_t t)
        {
            const uint32_t oqs = t * 64u + lc.l * 16u, osg = t * 32u + lc.l * 8u, om = t * 16u;
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.qs) : "v"(oqs), "s"(c.qs));
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(r.meta) : "v"(om), "s"(c.meta));
            asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(r.sg) : "v"(osg), "s"(c.sg));
        }
        __device__ __forceinline__ static void keep(Raw &r)
        {
            asm volatile("" : "+v"(r.qs), "+v"(r.meta), "+v"(r.sg));
        }
        template <int NEWER>
        __device__ __forceinline__ static void wait(Raw &r)
        {
            asm volatile("s_waitcnt vmcnt(%3)" : "+v"(r.qs), "+v"(r.meta), "+v"(r.sg) : "n"(NEWER));
        }

        // w[0], w[1]: elements 0-15, 16-31 of sub-block 2l; w[2], w[3]: of sub-block 2l+1.
        __device__ __forceinline__ static void decode(const Raw &r, const Lane &lc, v4i (&w)[4], Scale &S)
        {
            const uint32_t qh2 = __builtin_amdgcn_perm((uint32_t)r.meta.y, (uint32_t)r.meta.x, lc.qh_sel);
            const uint32_t nibs = ((uint32_t)r.meta.z >> (8u * lc.l)); // scales[l]: low nibble 2l, high nibble 2l+1
            const uint32_t hints = ((uint32_t)r.meta.w >> (16u + 4u * lc.l));
            const float d = h2f((uint16_t)((uint32_t)r.meta.w & 0xFFFFu));
            iq3s_decode_block(make_uint2((uint32_t)r.qs.x, (uint32_t)r.qs.y), qh2, nibs & 0xFu, hints & 3u, d,
                              (uint32_t)r.sg.x, w[0], w[1], S.bs0);
            iq3s_decode_block(make_uint2((uint32_t)r.qs.z, (uint32_t)r.qs.w), qh2 >> 16, (nibs >> 4) & 0xFu,
                              (hints >> 2) & 3u, d, (uint32_t)r.sg.y, w[2], w[3], S.bs1);
        }

        __device__ __forceinline__ static float scale_f32(const Scale &S, int i) { return i ? S.bs1 : S.bs0; }
        __device__ __forceinline__ static float min_f32(const Scale &, int) { return 0.0f; }

        // the format has no block minimum
        __device__ __forceinline__ static float apply(const Scale &S, int idot0, int idot1, const float4 sd, float acc)
        {
            acc = fmaf((float)idot0, sd.x * S.bs0, acc);
            acc = fmaf((float)idot1, sd.z * S.bs1, acc);
            return acc;
        }
    };

    struct IQ3STraits
    {
        static constexpr bool PAIR = false;
        static constexpr bool HAS_MIN = false;
        static constexpr bool USE_QUAD = true;         // quad-lane kernel for rows of >= 16 super-blocks
        static constexpr bool GEMM_PAIR_SCALES = true;   // prefill GEMM: scale products of two blocks per matrix instruction
        static constexpr bool USE_MFMA_BATCH = false;  // matrix-unit kernel for 5..8 activation rows
        typedef IQ3SQuad Quad;
        static constexpr int FAST_MAX_U = 3;          // load batches in flight in the chunked kernel
        static constexpr int TABLE_BYTES = IQ3S_TABLE_BYTES;

        __device__ static void *tables_lds() { return iq3s_tables_lds(); }
        __device__ static void stage_tables(void *) { iq3s_stage_tables(); }

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
                                                      float &bscale, float &bmin, const void *)
        {
            // picked with a bit mask: a conditional on two members of r would become a load
            // through a computed address and force arrays of Raw into memory
            const uint32_t m4 = (uint32_t)0 - (uint32_t)((c >> 2) & 1);
            const uint32_t qh = (((r.meta.y & m4) | (r.meta.x & ~m4))) >> (8 * (c & 3));
            const uint32_t nib = (r.meta.z >> (4 * c)) & 0xFu; // scales[c/2], low nibble for even c
            const float d = h2f((uint16_t)(r.meta.w & 0xFFFFu));
            const uint32_t hint = (r.meta.w >> (16 + 2 * c)) & 3u;
            iq3s_decode_block(r.qs, qh, nib, hint, d, r.signs, w0, w1, bscale);
            j = c;
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
