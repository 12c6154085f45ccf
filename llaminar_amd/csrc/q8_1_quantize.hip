// FP32 -> Q8_1 activation quantiser for gfx950.
//
// Arithmetic follows the reference's SIMD quantiser operation for operation
// (src/v2/tensors/SIMDHelpers.h:4716-4785) so the 36-byte blocks are identical:
//   amax = max|x| ; amax < 1e-10 -> all-zero block
//   d = amax / 127 (IEEE divide) ; id = 1 / d (IEEE divide)
//   q = saturate_int8(round_nearest_even(x * id)) ; sum = sum q ; d stored as RNE fp16
//
// Mapping: 8 lanes own one 32-element block (a float4 each), a wavefront owns 8
// consecutive blocks = 1 KiB of contiguous input; max and sum are reduced inside
// the 8-lane group with DPP.  HBM-bound: 4 B read + 1.125 B written per element.
#include "ql_device.h"
#include "ql_host.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    __global__ void __launch_bounds__(256)
        q8_1_quantize_kernel(const float4 *__restrict__ x, uint32_t *__restrict__ out, long n_blocks)
    {
        const long lane_global = (long)blockIdx.x * blockDim.x + threadIdx.x;
        const long blk = lane_global >> 3;
        const int sub = (int)(lane_global & 7);
        if (blk >= n_blocks)
            return; // whole 8-lane groups leave together, DPP below stays inside a group

        const float4 v = x[lane_global];

        const Q8Lane q = q8_1_quantize_lane(v);
        // 36-byte block = 9 dwords: [d|sum][8 x 4 quants]
        uint32_t *dst = out + blk * 9;
        dst[1 + sub] = q.packed;
        if (sub == 0)
            dst[0] = q.head;
    }

    // The reference's software binary32 -> binary16 (tensors/FP16Utils.h:75-118), which its
    // scalar quantiser uses for partial blocks: nearest-even for normal results, truncation for
    // subnormal ones, zero below 2^-25.
    __device__ __forceinline__ uint16_t f32_to_f16_software(float f)
    {
        const uint32_t bits = __float_as_uint(f);
        const uint32_t sign = (bits & 0x80000000u) >> 16;
        int e = (int)((bits & 0x7F800000u) >> 23) - 127 + 15;
        uint32_t m = bits & 0x007FFFFFu;
        if (e <= 0)
        {
            if (e < -10)
                return (uint16_t)sign;
            m = (m | 0x00800000u) >> (1 - e);
            return (uint16_t)(sign | (m >> 13));
        }
        if (e >= 0x1F)
        {
            if (e == 0xFF - 127 + 15 && m != 0)
                return (uint16_t)(sign | 0x7C00u | (m >> 13));
            return (uint16_t)(sign | 0x7C00u);
        }
        m += 0x0FFFu + ((m >> 13) & 1u);
        if (m >= 0x00800000u)
        {
            m = 0;
            e += 1;
        }
        return (uint16_t)(sign | ((uint32_t)e << 10) | (m >> 13));
    }

    // Rows whose length is not a multiple of 32 (or not 16-byte aligned): ceil(K/32) blocks per
    // row.  Full blocks take the arithmetic above; the partial last block of a row follows the
    // reference's scalar quantiser (tensors/SIMDHelpers.h:4554-4596): round half away from
    // zero, the software fp16 conversion, zero padding.
    __global__ void __launch_bounds__(256)
        q8_1_quantize_ragged_kernel(const float *__restrict__ x, uint32_t *__restrict__ out, long n_blocks, int K, int KB)
    {
        const long lane_global = (long)blockIdx.x * blockDim.x + threadIdx.x;
        const long blk = lane_global >> 3;
        const int sub = (int)(lane_global & 7);
        if (blk >= n_blocks)
            return; // whole 8-lane groups leave together
        const long m = blk / KB;
        const int kb = (int)(blk - m * KB);
        const int valid = min(32, K - kb * 32);
        const float *src = x + (size_t)m * K + (size_t)kb * 32 + 4 * sub;
        float e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            e[i] = (4 * sub + i < valid) ? src[i] : 0.0f;
        const float4 v = make_float4(e[0], e[1], e[2], e[3]);
        uint32_t *dst = out + blk * 9;
        if (valid == 32) // uniform inside the 8-lane group
        {
            const Q8Lane q = q8_1_quantize_lane(v);
            dst[1 + sub] = q.packed;
            if (sub == 0)
                dst[0] = q.head;
            return;
        }
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = fmaxf(amax, dpp_f32<DPP_QUAD_XOR1>(amax));
        amax = fmaxf(amax, dpp_f32<DPP_QUAD_XOR2>(amax));
        amax = fmaxf(amax, dpp_f32<DPP_ROW_HALF_MIRROR>(amax));
        uint32_t packed = 0, head = 0;
        if (amax >= 1e-10f)
        {
            const float d = __fdiv_rn(amax, 127.0f);
            const float id = __fdiv_rn(1.0f, d);
            int q[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                q[i] = (4 * sub + i < valid) ? (int)(int8_t)(int)roundf(e[i] * id) : 0;
            int sum = q[0] + q[1] + q[2] + q[3];
            sum += dpp_i32<DPP_QUAD_XOR1>(sum);
            sum += dpp_i32<DPP_QUAD_XOR2>(sum);
            sum += dpp_i32<DPP_ROW_HALF_MIRROR>(sum);
            packed = (uint32_t)(q[0] & 0xFF) | ((uint32_t)(q[1] & 0xFF) << 8) | ((uint32_t)(q[2] & 0xFF) << 16) |
                     ((uint32_t)(q[3] & 0xFF) << 24);
            head = (uint32_t)f32_to_f16_software(d) | ((uint32_t)(sum & 0xFFFF) << 16);
        }
        dst[1 + sub] = packed;
        if (sub == 0)
            dst[0] = head;
    }
} // namespace llamql

extern "C" bool llam_ql_quantize_q8_1(const float *d_x, void *d_q8, int M, int K,
                                      int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_quantize_q8_1";
    if (M < 0 || K < 0)
        return fail(fn, "negative size (M=%d K=%d)", M, K);
    if (M == 0 || K == 0)
        return true;
    if (!d_x || !d_q8)
        return fail(fn, "null pointer");
    if (!aligned4(d_x) || !aligned4(d_q8))
        return fail(fn, "d_x and d_q8 must be 4-byte aligned");
    if ((K % 32) != 0)
    {
        // rows end in a partial block: ceil(K/32) blocks per row
        if (!set_device(fn, device_id))
            return false;
        const int KB = (K + 31) / 32;
        const long nb = (long)M * KB;
        const long g = (nb * 8 + 255) / 256;
        if (g > 0x7FFFFFFFL)
            return fail(fn, "problem too large (M=%d K=%d)", M, K);
        hipLaunchKernelGGL(q8_1_quantize_ragged_kernel, dim3((unsigned)g), dim3(256), 0, as_stream(stream), d_x,
                           static_cast<uint32_t *>(d_q8), nb, K, KB);
        return launched(fn);
    }
    if (!aligned16(d_x))
        return fail(fn, "d_x must be 16-byte aligned");
    if (!set_device(fn, device_id))
        return false;
    const long n_blocks = (long)M * (K / 32);
    const long lanes = n_blocks * 8;
    const int threads = 256;
    const long grid = (lanes + threads - 1) / threads;
    if (grid > 0x7FFFFFFFL)
        return fail(fn, "problem too large (M=%d K=%d)", M, K);
    hipLaunchKernelGGL(q8_1_quantize_kernel, dim3((unsigned)grid), dim3(threads), 0, as_stream(stream),
                       reinterpret_cast<const float4 *>(d_x), static_cast<uint32_t *>(d_q8), n_blocks);
    return launched(fn);
}
