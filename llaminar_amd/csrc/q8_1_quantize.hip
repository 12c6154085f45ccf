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
    if ((K % 32) != 0)
        return fail(fn, "K must be a multiple of 32 (M=%d K=%d)", M, K);
    if (!aligned16(d_x) || !aligned4(d_q8))
        return fail(fn, "d_x must be 16-byte and d_q8 4-byte aligned");
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
