// TEST INFRASTRUCTURE ONLY.  Thin extern "C" doorway onto the REFERENCE's own
// CPU code, compiled straight from the reference's headers where they lie
// (see oracle/Makefile: -I$(REFERENCE)/src/v2).  No reference source is copied
// here: every arithmetic routine called below is the reference's.  The result,
// oracle/_ref/libllaminar_ref.so, is used to (1) pin oracle/ql_oracle.c,
// (2) write the golden vectors under tests/golden/, (3) optionally serve as
// the timed CPU baseline.
//
// The one thing this file does itself is fill a CPUNativeVNNIPackedWeights the
// way packWeightsCPUNativeVNNI (CPUNativeVNNIWeightPacker.h:598-1136) does,
// because that function wants a TensorBase whose implementation drags in the
// whole engine.  The fill only moves bytes the reference's simd::unpack_*
// routines produced into the slots the reference's accessors name
// (interleavedB / chunkComp / chunkScales / chunkMins).
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <numeric>
#include <vector>

#include "kernels/cpu/native_vnni/CPUNativeVNNIGemv.h"
#include "kernels/cpu/primitives/RMSNormPrimitives.h"
#include "kernels/cpu/primitives/RoPEPrimitives.h"
#include "kernels/cpu/primitives/SoftmaxPrimitivesImpl.h"
#include "kernels/cpu/primitives/SwiGLUPrimitives.h"
#include "tensors/BlockStructures.h"
#include "tensors/FP16Utils.h"
#include "tensors/IQQuantTables.h"
#include "tensors/SIMDHelpers.h"

using namespace llaminar2;
using namespace llaminar2::cpu::native_vnni;

namespace
{
    enum Fmt
    {
        FMT_Q4_K = 5,
        FMT_Q6_K = 8,
        FMT_IQ3_S = 11
    };

    size_t block_bytes(int fmt)
    {
        return fmt == FMT_Q4_K ? sizeof(Q4_KBlock) : fmt == FMT_Q6_K ? sizeof(Q6_KBlock) : sizeof(IQ3_SBlock);
    }

    // variant: 0 = the dispatcher the packer reaches, 1 scalar, 2 AVX2, 3 AVX512
    void unpack_sb(int fmt, const void *sb, int8_t *w, float *scales, float *mins, int variant)
    {
        if (fmt == FMT_Q4_K)
        {
            const Q4_KBlock &b = *static_cast<const Q4_KBlock *>(sb);
            if (variant == 1)
                simd::unpack_q4_k_superblock_to_int8_scalar(b, w, scales, mins);
            else if (variant == 2)
                simd::unpack_q4_k_superblock_to_int8_avx2(b, w, scales, mins);
            else
                simd::unpack_q4_k_superblock_to_int8(b, w, scales, mins);
        }
        else if (fmt == FMT_Q6_K)
        {
            const Q6_KBlock &b = *static_cast<const Q6_KBlock *>(sb);
            if (variant == 1)
                simd::unpack_q6_k_superblock_to_int8_scalar(b, w, scales, mins);
            else if (variant == 2)
                simd::unpack_q6_k_superblock_to_int8_avx2(b, w, scales, mins);
            else if (variant == 3)
                simd::unpack_q6_k_superblock_to_int8_avx512(b, w, scales, mins);
            else
                simd::unpack_q6_k_superblock_to_int8(b, w, scales, mins);
        }
        else
        {
            const IQ3_SBlock &b = *static_cast<const IQ3_SBlock *>(sb);
            if (variant == 3)
                simd::unpack_iq3_s_superblock_to_int8_avx512(b, w, scales);
            else
                simd::unpack_iq3_s_superblock_to_int8(b, w, scales);
            if (mins)
                std::fill(mins, mins + 8, 0.0f);
        }
    }

    // Mirror of the packer's bookkeeping for one weight matrix.
    bool fill_packed(int fmt, const uint8_t *W, int N, int K, CPUNativeVNNIPackedWeights &out)
    {
        if (K % 256 != 0)
            return false;
        const bool nibble = (fmt == FMT_Q4_K);
        out.N = N;
        out.K = K;
        out.N_padded = (N + 63) / 64 * 64;
        out.blocks_per_row = K / 32;
        out.codebook_id = static_cast<uint8_t>(fmt);
        out.payload_bytes = fmt == FMT_Q4_K ? 16 : fmt == FMT_Q6_K ? 24 : 13;
        out.is_asymmetric = (fmt != FMT_IQ3_S);
        out.is_superblock = true;
        out.is_nibble_lut = nibble;
        out.data_stride = nibble ? 1024 : 2048;
        out.interleaved_block_stride = out.data_stride + 256 + (out.is_asymmetric ? 128 : 0);

        const int bpr = out.blocks_per_row;
        const int n_chunks = out.N_padded / 64;
        const size_t bb = block_bytes(fmt);
        const int sbpr = K / 256;

        out.native_interleaved.resize((size_t)n_chunks * bpr * out.interleaved_block_stride);
        std::memset(out.native_interleaved.data(), 0, out.native_interleaved.size());
        if (nibble)
            out.payload.assign((size_t)n_chunks * bpr * 64 * 16, 0);
        else
            out.int8_flat.assign((size_t)n_chunks * bpr * 64 * 32, 0);

#pragma omp parallel for schedule(static)
        for (int n = 0; n < N; ++n)
        {
            const int chunk = n / 64, col = n % 64;
            for (int sb = 0; sb < sbpr; ++sb)
            {
                const uint8_t *blk = W + ((size_t)n * sbpr + sb) * bb;
                int8_t vals[256];
                float sc[8], mn[8];
                unpack_sb(fmt, blk, vals, sc, mn, 0);
                for (int i = 0; i < 8; ++i)
                {
                    const int kb = sb * 8 + i;
                    uint8_t *dst = out.native_interleaved.data() +
                                   ((size_t)chunk * bpr + kb) * out.interleaved_block_stride;
                    auto *comp = reinterpret_cast<int16_t *>(dst + out.data_stride);
                    auto *scales = reinterpret_cast<uint16_t *>(dst + out.data_stride + 128);
                    auto *mins = reinterpret_cast<uint16_t *>(dst + out.data_stride + 256);
                    scales[col] = fp32_to_fp16(sc[i]);
                    if (out.is_asymmetric)
                        mins[col] = fp32_to_fp16(mn[i]);
                    const int z = col / 16, lane = col % 16;
                    if (nibble)
                    {
                        // payload rule of Q4_KTensor::packVnniBlock (Q4_KTensor.cpp:776-792)
                        const Q4_KBlock &q = *reinterpret_cast<const Q4_KBlock *>(blk);
                        const uint8_t *src32 = q.qs + (i / 2) * 32;
                        uint8_t p16[16];
                        for (int t = 0; t < 16; ++t)
                            p16[t] = (i & 1) ? static_cast<uint8_t>((src32[t] >> 4) | (src32[t + 16] & 0xF0))
                                             : static_cast<uint8_t>((src32[t] & 0xF) | ((src32[t + 16] & 0xF) << 4));
                        std::memcpy(out.payload.data() + (((size_t)chunk * bpr + kb) * 64 + col) * 16, p16, 16);
                        for (int g = 0; g < 4; ++g)
                            std::memcpy(dst + g * 256 + z * 64 + lane * 4, p16 + g * 4, 4);
                        int8_t decoded[32];
                        decode_native_block(out.codebook_id, p16, decoded);
                        int32_t s = 0;
                        for (int t = 0; t < 32; ++t)
                            s += decoded[t];
                        comp[col] = static_cast<int16_t>(s);
                    }
                    else
                    {
                        const int8_t *v = vals + i * 32;
                        std::memcpy(out.int8_flat.data() + (((size_t)chunk * bpr + kb) * 64 + col) * 32, v, 32);
                        for (int g = 0; g < 8; ++g)
                            std::memcpy(dst + g * 256 + z * 64 + lane * 4, v + g * 4, 4);
                        int32_t s = 0;
                        for (int t = 0; t < 32; ++t)
                            s += v[t];
                        comp[col] = static_cast<int16_t>(s);
                    }
                }
            }
        }
        return true;
    }

    ISAPath isa_of(int isa)
    {
        return isa == 1 ? ISAPath::AVX512 : isa == 2 ? ISAPath::AVX2 : isa == 3 ? ISAPath::SCALAR : ISAPath::AUTO;
    }
} // namespace

extern "C"
{
    float ref_f16_to_f32(uint16_t h) { return fp16_to_fp32(h); }
    uint16_t ref_f32_to_f16(float f) { return fp32_to_fp16(f); }
    uint16_t ref_f32_to_f16_f16c(float f)
    {
        return (uint16_t)_mm_cvtsi128_si32(_mm_cvtps_ph(_mm_set_ss(f), _MM_FROUND_TO_NEAREST_INT));
    }
    const uint32_t *ref_iq3s_grid() { return iq3s_grid; }
    void ref_get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) { simd::get_scale_min_k4(j, q, d, m); }

    // variant: 0 dispatch (what the GEMV path calls), 1 scalar, 2 AVX2, 3 AVX512
    void ref_quantize_block_q8_1(const float *x, int valid, void *out, int variant)
    {
        Q8_1Block &b = *static_cast<Q8_1Block *>(out);
        if (variant == 1)
            simd::quantize_single_block_scalar(x, b, valid);
        else if (variant == 2)
            simd::quantize_single_block_avx2(x, b);
        else if (variant == 3)
            simd::quantize_single_block_avx512(x, b);
        else
            simd::quantize_single_block(x, b, valid);
    }

    void ref_quantize_q8_1(const float *x, int M, int K, void *out)
    {
        quantize_activations_to_q8_1(x, static_cast<Q8_1Block *>(out), M, K, (K + 31) / 32);
    }

    void ref_unpack_superblock(int fmt, const void *sb, int8_t *w256, float *scales8, float *mins8, int variant)
    {
        unpack_sb(fmt, sb, w256, scales8, mins8, variant);
    }

    // Opaque packed-weight handle so timing loops do not re-pack.
    void *ref_pack(int fmt, const void *W, int N, int K)
    {
        auto *p = new CPUNativeVNNIPackedWeights();
        if (!fill_packed(fmt, static_cast<const uint8_t *>(W), N, K, *p))
        {
            delete p;
            return nullptr;
        }
        return p;
    }
    void ref_pack_free(void *p) { delete static_cast<CPUNativeVNNIPackedWeights *>(p); }
    long ref_pack_bytes(void *p) { return (long)static_cast<CPUNativeVNNIPackedWeights *>(p)->native_interleaved.size(); }

    // M == 1 -> gemv_native_vnni_preq, else gemm_native_vnni_preq.
    void ref_gemm_packed(void *p, const void *A_q8, int M, float *C, int ldc, int isa)
    {
        const auto &pk = *static_cast<CPUNativeVNNIPackedWeights *>(p);
        if (M == 1)
            gemv_native_vnni_preq(pk, static_cast<const Q8_1Block *>(A_q8), C, isa_of(isa));
        else
            gemm_native_vnni_preq(pk, static_cast<const Q8_1Block *>(A_q8), C, M, ldc, isa_of(isa));
    }

    // fp32 activations in: quantise + multiply, the way multiply_tensor reaches them
    // (gemv_native_vnni CPUNativeVNNIGemv.h:974-1020, gemm_native_vnni :3554-3570).
    void ref_gemm_fp32_packed(void *p, const float *A, int M, float *C, int ldc)
    {
        const auto &pk = *static_cast<CPUNativeVNNIPackedWeights *>(p);
        if (M == 1)
            gemv_native_vnni(pk, A, C);
        else
            gemm_native_vnni(pk, A, C, M, ldc);
    }

    int ref_gemm(int fmt, const void *W, int N, int K, const void *A_q8, int M, float *C, int ldc, int isa)
    {
        void *p = ref_pack(fmt, W, N, K);
        if (!p)
            return 0;
        ref_gemm_packed(p, A_q8, M, C, ldc, isa);
        ref_pack_free(p);
        return 1;
    }

    int ref_omp_threads() { return omp_get_max_threads(); }

    // ---- decode-step operators: the reference's primitives, compiled by the Makefile from
    // kernels/cpu/primitives/{RMSNormPrimitives,RoPEPrimitives}.cpp where they lie ----------
    // variant: 1 scalar, 2 AVX2, 3 AVX512
    void ref_rmsnorm_row(int variant, const float *src, const float *gamma, float *dst, long cols, float eps)
    {
        if (variant == 1)
            primitives::rmsnorm_fused_row_scalar(src, gamma, dst, (std::size_t)cols, eps);
        else if (variant == 2)
            primitives::rmsnorm_fused_row_avx2(src, gamma, dst, (std::size_t)cols, eps);
        else
            primitives::rmsnorm_fused_row_avx512(src, gamma, dst, (std::size_t)cols, eps);
    }
    // residual += input, then RMSNorm of the new residual
    void ref_residual_rmsnorm_row(const float *input, float *residual, const float *gamma, float *output, long cols,
                                  float eps)
    {
        primitives::fused_residual_rmsnorm_row_avx512(input, residual, gamma, output, (std::size_t)cols, eps);
    }
    void ref_rope_inv_freq(int head_dim, float theta, float *out)
    {
        const std::vector<float> &f = primitives::get_inv_freq_cached(head_dim, theta);
        std::memcpy(out, f.data(), f.size() * sizeof(float));
    }
    // one token at position n_past: q [q_heads*head_dim], k [k_heads*head_dim], in place
    void ref_rope_token(float *q, float *k, int head_dim, int q_heads, int k_heads, int n_past, float theta)
    {
        primitives::apply_rope_vectorized(q, k, 1, head_dim, q_heads, k_heads, n_past, theta, nullptr);
    }
    void ref_rope_head_scalar(float *head, int position, int head_dim, float theta)
    {
        primitives::apply_rope_to_head_scalar(head, position, primitives::get_inv_freq_cached(head_dim, theta),
                                              head_dim, 0);
    }
    // silu(gate) * up as the CPU FFN computes it (ISA dispatch, no OpenMP region):
    // compute_swiglu_serial, SwiGLUPrimitives.cpp:254
    void ref_swiglu(const float *gate, const float *up, float *out, int n)
    {
        primitives::compute_swiglu_serial(gate, up, out, n);
    }
    // The router's softmax (primitives::softmax_row_fp32, SoftmaxPrimitivesImpl.h:412-709), in place.
    // variant: 0 = the dispatcher CPUMoEKernel::route reaches, 1 scalar, 2 AVX2, 3 AVX512
    void ref_softmax_row(float *row, int cols, int variant)
    {
        if (variant == 1)
            primitives::softmax_row_fp32_scalar(row, cols, false, 1.0f, 0);
        else if (variant == 2)
            primitives::softmax_row_fp32_avx2(row, cols, false, 1.0f, 0);
        else if (variant == 3)
            primitives::softmax_row_fp32_avx512(row, cols, false, 1.0f, 0);
        else
            primitives::softmax_row_fp32(row, cols, false, 1.0f, 0);
    }
    // CPUMoEKernel::route from the logits on (CPUMoEKernel.cpp:51-78): the reference's softmax,
    // then the statements of its selection -- iota, std::partial_sort by probability, the sum of
    // the top_k and the division -- which live in a translation unit that needs the whole engine.
    // probs [n_tokens x n_experts] receives the probabilities.
    void ref_moe_route(const float *logits, int n_tokens, int n_experts, int top_k, int normalize, int variant,
                       int32_t *ids, float *weights, float *probs)
    {
        std::vector<int> indices(n_experts);
        for (int t = 0; t < n_tokens; ++t)
        {
            float *p = probs + (size_t)t * n_experts;
            std::memcpy(p, logits + (size_t)t * n_experts, (size_t)n_experts * sizeof(float));
            ref_softmax_row(p, n_experts, variant);
            std::iota(indices.begin(), indices.end(), 0);
            std::partial_sort(indices.begin(), indices.begin() + top_k, indices.end(),
                              [p](int a, int b) { return p[a] > p[b]; });
            float topk_sum = 0.0f;
            for (int k = 0; k < top_k; ++k)
                topk_sum += p[indices[k]];
            for (int k = 0; k < top_k; ++k)
            {
                ids[(size_t)t * top_k + k] = indices[k];
                weights[(size_t)t * top_k + k] = normalize ? p[indices[k]] / topk_sum : p[indices[k]];
            }
        }
    }
}
