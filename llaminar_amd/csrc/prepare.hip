// Weight preparation: raw GGUF super-blocks -> the device layout the kernels
// read.  Moves bytes; for Q6_K it also works out, once, the per-block requantisation
// factors and scales that every product would otherwise recompute.
//
//   Q4_K  : unchanged (144-byte blocks are 16-byte aligned)
//   Q6_K  : planes ql [T][128] | qh [T][64] | scales [T][16] | d [T] fp16      (T*210 B)
//           | pad to 16 | factors [T][8] x 4 B (q6k_block_code, ql_device.h)    (T*32 B)
//   IQ3_S : planes qs [T][64] | signs [T][32] | meta [T][16]                   (T*112 B)
//           meta = qh[8] scales[4] d[2] hints[2]: two bits per 32-element block, which of the
//           requantisation maps the block needs (its largest codebook magnitude) when its scale is
//           an ordinary fp16 number, else "take the general path" (iq3s_block_hint)
// with T = N*K/256 super-blocks in row-major order.  Raw Q6_K / IQ3_S blocks are
// 210 / 110 bytes, i.e. only 2-byte aligned, so the copy works in halfwords.
#include "gemv_traits_iq3s.h"
#include "ql_device.h"
#include "ql_host.h"

#include "llaminar_amd/ql_api.h"

namespace llamql
{
    __global__ void __launch_bounds__(256)
        prepare_q6k_kernel(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst, size_t T)
    {
        const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (i >= T * 105)
            return;
        const size_t t = i / 105;
        const int u = (int)(i - t * 105);
        const uint16_t v = src[i];
        size_t o;
        if (u < 64)
            o = t * 64 + u; // ql
        else if (u < 96)
            o = T * 64 + t * 32 + (u - 64); // qh
        else if (u < 104)
            o = T * 96 + t * 8 + (u - 96); // scales
        else
            o = T * 104 + t; // d
        dst[o] = v;
    }

    // one thread per 32-element block: its two sub-scales and the super-block's d -> record
    __global__ void __launch_bounds__(256)
        prepare_q6k_factors_kernel(const uint16_t *__restrict__ src, uint32_t *__restrict__ fac, size_t T)
    {
        const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (i >= T * 8)
            return;
        const size_t t = i >> 3;
        const int j = (int)(i & 7);
        const uint16_t pair = src[t * 105 + 96 + j]; // scales[2j], scales[2j+1] (block j = 4n+s: 8n+2s = 2j)
        const int s0 = (int)(int8_t)(pair & 0xFF), s1 = (int)(int8_t)(pair >> 8);
        const float d = h2f(src[t * 105 + 104]);
        fac[t * 8 + q6k_code_pos(j)] = q6k_block_code(s0, s1, d);
    }

    __global__ void __launch_bounds__(256)
        prepare_iq3s_kernel(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst, size_t T)
    {
        // 56 halfwords are written per block (55 copied + the gmax hints in place of padding)
        const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (i >= T * 56)
            return;
        const size_t t = i / 56;
        const int u = (int)(i - t * 56);
        uint16_t v = 0;
        size_t o;
        if (u == 55)
        {
            o = T * 48 + t * 8 + 7; // hints: block j in bits 2j, 2j+1
            const uint8_t *blk = reinterpret_cast<const uint8_t *>(src + t * 55); // d[2] qs[64] qh[8] signs[32] scales[4]
            const float d = h2f((uint16_t)(blk[0] | (blk[1] << 8)));
#pragma unroll
            for (int j = 0; j < 8; ++j)
            {
                const uint32_t nib = ((uint32_t)blk[106 + (j >> 1)] >> (4 * (j & 1))) & 0xFu;
                v |= (uint16_t)(iq3s_block_hint(blk + 2 + 8 * j, blk[66 + j], nib, d) << (2 * j));
            }
        }
        else
        {
            v = src[t * 55 + u];
            if (u == 0)
                o = T * 48 + t * 8 + 6; // d
            else if (u < 33)
                o = t * 32 + (u - 1); // qs
            else if (u < 37)
                o = T * 48 + t * 8 + (u - 33); // qh
            else if (u < 53)
                o = T * 32 + t * 16 + (u - 37); // signs
            else
                o = T * 48 + t * 8 + 4 + (u - 53); // scales
        }
        dst[o] = v;
    }
} // namespace llamql

extern "C" size_t llam_ql_prepared_bytes(uint8_t fmt, int N, int K)
{
    if (N <= 0 || K <= 0 || (K % 256) != 0)
        return 0;
    const size_t T = (size_t)N * (size_t)(K / 256);
    switch (fmt)
    {
    case LLAM_FMT_Q4_K: return T * 144;
    case LLAM_FMT_Q6_K: return llamql::q6k_factors_offset(T) + T * 32;
    case LLAM_FMT_IQ3_S: return T * 112;
    default: return 0;
    }
}

extern "C" bool llam_ql_prepare_weights(uint8_t fmt, const void *d_gguf, void *d_prepared,
                                        int N, int K, int device_id, void *stream)
{
    using namespace llamql;
    static const char *fn = "llam_ql_prepare_weights";
    if (fmt != LLAM_FMT_Q4_K && fmt != LLAM_FMT_Q6_K && fmt != LLAM_FMT_IQ3_S)
        return fail(fn, "unsupported weight format id %d", (int)fmt);
    if (N < 1 || K < 1 || (K % 256) != 0)
        return fail(fn, "need N >= 1 and K a positive multiple of 256 (N=%d K=%d)", N, K);
    if (!d_gguf || !d_prepared)
        return fail(fn, "null pointer");
    if (!aligned16(d_prepared))
        return fail(fn, "d_prepared must be 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(d_gguf) & 1u) != 0)
        return fail(fn, "d_gguf must be 2-byte aligned");
    if (!set_device(fn, device_id))
        return false;
    const size_t T = (size_t)N * (size_t)(K / 256);
    hipStream_t st = as_stream(stream);
    if (fmt == LLAM_FMT_Q4_K)
    {
        if (d_gguf == d_prepared)
            return true;
        if (!aligned16(d_gguf))
            return fail(fn, "Q4_K source must be 16-byte aligned");
        hipError_t e = hipMemcpyAsync(d_prepared, d_gguf, T * 144, hipMemcpyDeviceToDevice, st);
        if (e != hipSuccess)
            return fail(fn, "hipMemcpyAsync: %s", hipGetErrorString(e));
        return true;
    }
    if (d_gguf == d_prepared)
        return fail(fn, "in-place preparation is only possible for Q4_K");
    const size_t items = T * (fmt == LLAM_FMT_Q6_K ? 105 : 56);
    const size_t grid = (items + 255) / 256;
    if (grid > 0x7FFFFFFFull)
        return fail(fn, "matrix too large (N=%d K=%d)", N, K);
    if (fmt == LLAM_FMT_Q6_K)
    {
        hipLaunchKernelGGL(prepare_q6k_kernel, dim3((unsigned)grid), dim3(256), 0, st,
                           static_cast<const uint16_t *>(d_gguf), static_cast<uint16_t *>(d_prepared), T);
        uint32_t *fac = reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(d_prepared) + q6k_factors_offset(T));
        hipLaunchKernelGGL(prepare_q6k_factors_kernel, dim3((unsigned)((T * 8 + 255) / 256)), dim3(256), 0, st,
                           static_cast<const uint16_t *>(d_gguf), fac, T);
    }
    else
        hipLaunchKernelGGL(prepare_iq3s_kernel, dim3((unsigned)grid), dim3(256), 0, st,
                           static_cast<const uint16_t *>(d_gguf), static_cast<uint16_t *>(d_prepared), T);
    return launched(fn);
}
