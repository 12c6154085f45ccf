// Device-side helpers shared by the gfx950 quantized-linear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "llaminar_amd/ql_blocks.h"

namespace llamql
{
    typedef int v4i __attribute__((ext_vector_type(4)));
    typedef int v16i __attribute__((ext_vector_type(16)));

    constexpr int WAVE = 64;

    // ---- binary16 helpers ---------------------------------------------------

    __device__ __forceinline__ float h2f(uint16_t bits)
    {
        return __half2float(__ushort_as_half(bits));
    }

    // fp32 -> fp16 -> fp32 with the rounding the reference's weight packer
    // applies to effective block scales and mins (tensors/FP16Utils.h:75-118):
    // nearest-even when the fp16 result is normal, truncation toward zero when
    // it is subnormal (|x| < 2^-14), signed zero below 2^-25.
    __device__ __forceinline__ float f16_round_packer(float x)
    {
        float r = __half2float(__float2half_rn(x));
        if (fabsf(x) < 6.103515625e-05f)
            r = truncf(x * 16777216.0f) * 5.9604644775390625e-08f;
        return r;
    }

    // x / 127 as an IEEE division gives it, for the values a Q6_K block scale takes before its
    // fp16 rounding (x = f32(d) * msc * 32, d any fp16, msc = 1..128: checked exhaustively on the
    // host): q0 = x * RN(1/127), one correction step through the exact remainder.  Zeros,
    // infinities and NaN take q0, which has their sign and kind.
    __device__ __forceinline__ float div_by_127(float x)
    {
        const float c = 0x1.020408p-7f;
        const float q0 = x * c;
        const float q1 = fmaf(fmaf(-q0, 127.0f, x), c, q0);
        return __builtin_amdgcn_classf(x, 0x198) ? q1 : q0; // finite and not zero
    }

    // ---- Q6_K block factors, worked out once when the weights are prepared ---------------
    // A 32-element block has two int8 sub-scales s0, s1.  With msc = max(|s0|, |s1|) the
    // reference requantises w = ((q - 32) * f_h + 128) >> 8, f_h = rne(s_h * 32512 / (msc * 32)),
    // and scales the block by f16(d * msc * 32 / 127) (SIMDHelpers.h:12023-12204).  The larger
    // sub-scale's factor is +-1016; the record keeps the other one:
    //   bits  0..11  f of the smaller sub-scale (two's complement)
    //   bit   12     the larger sub-scale is the second one (ties: the first)
    //   bits 13..14  the sign of the larger sub-scale as a two-bit two's complement number: +1, -1, or
    //                0 when both sub-scales are zero (weights and scale are zero) -- times 1016 it is
    //                the larger one's factor
    //   bits 16..31  the block scale as fp16 bits
    constexpr uint32_t Q6K_CODE_BIG1 = 1u << 12, Q6K_CODE_SIGN_SHIFT = 13;
    constexpr uint32_t Q6K_CODE_POS = 1u << Q6K_CODE_SIGN_SHIFT, Q6K_CODE_NEG = 3u << Q6K_CODE_SIGN_SHIFT;

    __device__ __forceinline__ uint32_t q6k_block_code(int s0, int s1, float d)
    {
        const int a0 = s0 < 0 ? -s0 : s0, a1 = s1 < 0 ? -s1 : s1;
        const bool big0 = a0 >= a1;
        const int msc = big0 ? a0 : a1;
        if (msc == 0)
            return 0u;
        const int s_small = big0 ? s1 : s0, s_big = big0 ? s0 : s1;
        const float fm = (float)msc;
        // rne(s_small * 1016 / msc) without a division: the quotient has a denominator of at most
        // 128, so unless it is a half-integer it lies 1/256 or more from one and any value within
        // 1e-3 rounds alike; a half-integer is a float, and one Newton step on the reciprocal
        // reproduces representable quotients.
        const float num = (float)(s_small * 1016);
        const float r = __builtin_amdgcn_rcpf(fm);
        const float q0 = num * r;
        const int f_small = (int)rintf(fmaf(fmaf(-fm, q0, num), r, q0));
        const float bscale = f16_round_packer(div_by_127(d * fm * 32.0f));
        return ((uint32_t)f_small & 0xFFFu) | (big0 ? 0u : Q6K_CODE_BIG1) | (s_big < 0 ? Q6K_CODE_NEG : Q6K_CODE_POS) |
               ((uint32_t)__half_as_ushort(__float2half_rn(bscale)) << 16); // bscale is an fp16 value: exact
    }
    // the two 8.8 factors and the block scale of a record
    __device__ __forceinline__ void q6k_block_decode(uint32_t c, int &f0, int &f1, float &bscale)
    {
        const int fs = __builtin_amdgcn_sbfe((int)c, 0u, 12u);
        const int fb = __builtin_amdgcn_sbfe((int)c, Q6K_CODE_SIGN_SHIFT, 2u) * 1016;
        const bool big1 = (c & Q6K_CODE_BIG1) != 0;
        f0 = big1 ? fs : fb;
        f1 = big1 ? fb : fs;
        bscale = h2f((uint16_t)(c >> 16));
    }
    // the factor of one of the two sub-scales (second: 0 or Q6K_CODE_BIG1, the lane's constant) and the
    // block scale: what a lane needs that requantises 16 elements of a block
    __device__ __forceinline__ void q6k_block_factor(uint32_t c, uint32_t second, int &f, float &bscale)
    {
        const int fs = __builtin_amdgcn_sbfe((int)c, 0u, 12u);
        const int fb = __builtin_amdgcn_sbfe((int)c, Q6K_CODE_SIGN_SHIFT, 2u) * 1016;
        f = (c & Q6K_CODE_BIG1) == second ? fb : fs;
        bscale = h2f((uint16_t)(c >> 16));
    }
    // where the record of block j sits among the eight of its super-block: the two blocks a
    // quad lane decodes (4n + h and 4n + 2 + h for lane 2n + h) are neighbours
    __host__ __device__ constexpr int q6k_code_pos(int j) { return (j & 4) | ((j & 1) << 1) | ((j >> 1) & 1); }

    // Same rounding for two values at once.  The truncating branch is only needed when a
    // value lies below the fp16 normal range, which real weights almost never produce:
    // one rarely-taken branch (fp16 exponent field 0 or 1 in either result) guards the
    // exact test for both.
    __device__ __forceinline__ void f16_round_packer2(float x0, float x1, float &r0, float &r1)
    {
        const __half h0 = __float2half_rn(x0);
        const __half h1 = __float2half_rn(x1);
        r0 = __half2float(h0);
        r1 = __half2float(h1);
        const uint32_t e = ((uint32_t)__half_as_ushort(h0) | ((uint32_t)__half_as_ushort(h1) << 16)) & 0x7C007C00u;
        // a 16-bit half below 0x0800 makes the subtraction borrow into bit 15 / bit 31
        if (__builtin_expect(((e - 0x08000800u) & 0x80008000u) != 0u, 0))
        {
            if (fabsf(x0) < 6.103515625e-05f)
                r0 = truncf(x0 * 16777216.0f) * 5.9604644775390625e-08f;
            if (fabsf(x1) < 6.103515625e-05f)
                r1 = truncf(x1 * 16777216.0f) * 5.9604644775390625e-08f;
        }
    }

    // ---- cross-lane -----------------------------------------------------------

    template <int CTRL>
    __device__ __forceinline__ int dpp_i32(int v)
    {
        return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
    }
    template <int CTRL>
    __device__ __forceinline__ float dpp_f32(float v)
    {
        return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
    }

    constexpr int DPP_QUAD_XOR1 = 0xB1;     // quad_perm [1,0,3,2]
    constexpr int DPP_QUAD_XOR2 = 0x4E;     // quad_perm [2,3,0,1]
    constexpr int DPP_ROW_HALF_MIRROR = 0x141;
    constexpr int DPP_ROW_MIRROR = 0x140;

    // Sum over the 64 lanes of a wavefront; every lane returns the total.
    // Fixed association order, so results are run-to-run identical.
    __device__ __forceinline__ float wave_sum(float v)
    {
        v += dpp_f32<DPP_QUAD_XOR1>(v);
        v += dpp_f32<DPP_QUAD_XOR2>(v);
        v += dpp_f32<DPP_ROW_HALF_MIRROR>(v);
        v += dpp_f32<DPP_ROW_MIRROR>(v);
        const int b = __float_as_int(v);
        const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
        const float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
        const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
        const float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
        return (r0 + r1) + (r2 + r3);
    }

    // The same for a double (two 32-bit halves travel per step); every lane returns the total.
    template <int CTRL>
    __device__ __forceinline__ double dpp_f64(double v)
    {
        const long long b = __double_as_longlong(v);
        const int lo = dpp_i32<CTRL>((int)(b & 0xFFFFFFFFLL)), hi = dpp_i32<CTRL>((int)(b >> 32));
        return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
    }
    __device__ __forceinline__ double wave_sum(double v)
    {
        v += dpp_f64<DPP_QUAD_XOR1>(v);
        v += dpp_f64<DPP_QUAD_XOR2>(v);
        v += dpp_f64<DPP_ROW_HALF_MIRROR>(v);
        v += dpp_f64<DPP_ROW_MIRROR>(v);
        const long long b = __double_as_longlong(v);
        const int lo = (int)(b & 0xFFFFFFFFLL), hi = (int)(b >> 32);
        auto row = [&](int lane) {
            const unsigned int l = (unsigned int)__builtin_amdgcn_readlane(lo, lane);
            const int h = __builtin_amdgcn_readlane(hi, lane);
            return __longlong_as_double(((long long)h << 32) | l);
        };
        return (row(0) + row(16)) + (row(32) + row(48));
    }

    // Maximum over the 64 lanes of a wavefront; every lane returns it.
    __device__ __forceinline__ float wave_max(float v)
    {
        v = fmaxf(v, dpp_f32<DPP_QUAD_XOR1>(v));
        v = fmaxf(v, dpp_f32<DPP_QUAD_XOR2>(v));
        v = fmaxf(v, dpp_f32<DPP_ROW_HALF_MIRROR>(v));
        v = fmaxf(v, dpp_f32<DPP_ROW_MIRROR>(v));
        const int b = __float_as_int(v);
        const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
        const float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
        const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
        const float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
        return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
    }

    // ---- Q8_1 quantiser, one lane's share ---------------------------------------------
    // Eight neighbouring lanes (lane & 7 = 0..7) own one 32-element block, four values
    // each; all eight must be active.  Arithmetic of the reference's quantiser
    // (src/v2/tensors/SIMDHelpers.h:4716-4785): amax = max|x|, below 1e-10 an all-zero
    // block; d = amax/127 and id = 1/d as IEEE divides; q = saturate(rne(x*id));
    // d stored as nearest-even fp16 next to the int16 sum of the 32 quants.
    struct Q8Lane
    {
        uint32_t packed; // this lane's four quants
        uint32_t head;   // fp16 d | int16 sum << 16 (the same in all eight lanes)
    };
    __device__ __forceinline__ Q8Lane q8_1_quantize_lane(const float4 v)
    {
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = fmaxf(amax, dpp_f32<DPP_QUAD_XOR1>(amax));
        amax = fmaxf(amax, dpp_f32<DPP_QUAD_XOR2>(amax));
        amax = fmaxf(amax, dpp_f32<DPP_ROW_HALF_MIRROR>(amax));
        Q8Lane r;
        r.packed = 0;
        r.head = 0;
        if (amax >= 1e-10f)
        {
            const float d = __fdiv_rn(amax, 127.0f);
            const float id = __fdiv_rn(1.0f, d);
            const int q0 = max(-128, min(127, (int)rintf(v.x * id)));
            const int q1 = max(-128, min(127, (int)rintf(v.y * id)));
            const int q2 = max(-128, min(127, (int)rintf(v.z * id)));
            const int q3 = max(-128, min(127, (int)rintf(v.w * id)));
            int sum = q0 + q1 + q2 + q3;
            sum += dpp_i32<DPP_QUAD_XOR1>(sum);
            sum += dpp_i32<DPP_QUAD_XOR2>(sum);
            sum += dpp_i32<DPP_ROW_HALF_MIRROR>(sum);
            r.packed = (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
                       ((uint32_t)(q3 & 0xFF) << 24);
            r.head = (uint32_t)__half_as_ushort(__float2half_rn(d)) | ((uint32_t)(sum & 0xFFFF) << 16);
        }
        return r;
    }

    // silu(gate) * up, element by element (gate / (1 + exp(-gate)) with an IEEE divide).
    __device__ __forceinline__ float4 swiglu4(const float4 g, const float4 u)
    {
        float4 v;
        v.x = __fdiv_rn(g.x, 1.0f + expf(-g.x)) * u.x;
        v.y = __fdiv_rn(g.y, 1.0f + expf(-g.y)) * u.y;
        v.z = __fdiv_rn(g.z, 1.0f + expf(-g.z)) * u.z;
        v.w = __fdiv_rn(g.w, 1.0f + expf(-g.w)) * u.w;
        return v;
    }

    // weight * v, and that added to y, each rounded on its own: never contracted into a fused multiply-add, so
    // that every kernel that weighs and adds partial results (expert slots, accumulating launches) forms
    // the same bits whatever the compiler makes of the code around it.
    // (contraction is switched off for these two operations themselves: __fmul_rn / __fadd_rn are plain
    // operators to this compiler and fuse like any others)
    __device__ __forceinline__ float weighted(float weight, float v)
    {
#pragma clang fp contract(off)
        return weight * v;
    }
    __device__ __forceinline__ float add_rounded(float y, float v)
    {
#pragma clang fp contract(off)
        return y + v;
    }

    // ---- integer dot ------------------------------------------------------------

    // acc + sum of four signed-byte products (v_dot4_i32_i8).
    __device__ __forceinline__ int dot4(int a, int b, int acc)
    {
        return __builtin_amdgcn_sdot4(a, b, acc, false);
    }

    __device__ __forceinline__ int dot16(const v4i a, const v4i b, int acc)
    {
        acc = dot4(a.x, b.x, acc);
        acc = dot4(a.y, b.y, acc);
        acc = dot4(a.z, b.z, acc);
        acc = dot4(a.w, b.w, acc);
        return acc;
    }

    // Same with a zero start value.  Spelled as the three-operand VOP3P form so no
    // register has to be cleared first.
    __device__ __forceinline__ int dot4z(int a, int b)
    {
        int r;
        asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
        return r;
    }

    __device__ __forceinline__ int dot16z(const v4i a, const v4i b)
    {
        int acc = dot4z(a.x, b.x);
        acc = dot4(a.y, b.y, acc);
        acc = dot4(a.z, b.z, acc);
        acc = dot4(a.w, b.w, acc);
        return acc;
    }

    // ---- Q4_K -------------------------------------------------------------------

    // 6-bit (scale, min) pair j of a Q4_K super-block whose 12 packed bytes are
    // given as three little-endian words (bytes 0-3, 4-7, 8-11).
    __device__ __forceinline__ void q4k_scale_min(int j, uint32_t s0, uint32_t s1, uint32_t s2,
                                                  uint32_t &sc, uint32_t &mn)
    {
        const int sh = 8 * (j & 3);
        const uint32_t a = (s0 >> sh) & 0xFFu;
        const uint32_t b = (s1 >> sh) & 0xFFu;
        const uint32_t p = (s2 >> sh) & 0xFFu;
        if (j < 4)
        {
            sc = a & 63u;
            mn = b & 63u;
        }
        else
        {
            sc = (p & 15u) | ((a >> 6) << 4);
            mn = (p >> 4) | ((b >> 6) << 4);
        }
    }
} // namespace llamql
