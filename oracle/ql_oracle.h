/*
 * TEST INFRASTRUCTURE ONLY -- not part of the shipped library.
 *
 * Scalar CPU restatement of the reference's quantized-linear arithmetic
 * (GGUF block-quantized weight x Q8_1-quantized activation).  It exists so the
 * HIP kernels can be checked against something that follows the reference's
 * CPU AVX512-VNNI / AVX2 path operation for operation.  Only tests, the smoke
 * check and the benchmark's cpu_baseline leg may link or load it; the product
 * library never does.
 *
 * Every function names the reference code it follows.  All of them are pinned
 * against the reference itself (oracle/_ref, built from the reference's own
 * headers where those are present) and against the golden vectors under
 * tests/golden/ that were produced by that build; see tests/test_oracle_*.py.
 */
#ifndef QL_ORACLE_H
#define QL_ORACLE_H

#include <stdint.h>
#include "llaminar_amd/ql_blocks.h"

#ifdef __cplusplus
extern "C" {
#endif

/* binary16 <-> binary32.
 *  qlo_f16_to_f32      exact widening           (tensors/FP16Utils.h:25-66)
 *  qlo_f32_to_f16_sw   the software narrowing the weight packer uses: RNE for
 *                      fp16-normal results, TRUNCATION for fp16-subnormal
 *                      results, flush to zero below 2^-25 (tensors/FP16Utils.h:75-118)
 *  qlo_f32_to_f16_rne  IEEE round-to-nearest-even including subnormals, i.e.
 *                      what _mm_cvtps_ph(.., _MM_FROUND_TO_NEAREST_INT) returns
 *                      (used for Q8_1 d, tensors/SIMDHelpers.h:4743-4745)      */
float qlo_f16_to_f32(uint16_t h);
uint16_t qlo_f32_to_f16_sw(float f);
uint16_t qlo_f32_to_f16_rne(float f);

/* One Q8_1 block from `valid` (1..32) fp32 values.
 * valid == 32: the SIMD quantizer   (tensors/SIMDHelpers.h:4716-4785)
 * valid <  32: the scalar tail path (tensors/SIMDHelpers.h:4554-4596)          */
void qlo_quantize_block_q8_1(const float *x, int valid, llam_block_q8_1 *out);

/* M rows of K fp32 -> M * ceil(K/32) blocks, row-major
 * (kernels/cpu/native_vnni/CPUNativeVNNIGemv.h:2000-2036).                      */
void qlo_quantize_q8_1(const float *x, int M, int K, llam_block_q8_1 *out);

/* (scale, min) 6-bit pair j of a Q4_K super-block (tensors/SIMDHelpers.h:10791-10803). */
void qlo_get_scale_min_k4(int j, const uint8_t *scales12, uint8_t *sc, uint8_t *m);

/* Effective 32-element weight sub-blocks of one super-block, as the reference's
 * weight packer defines them: 256 int8 values, 8 fp16 scales, 8 fp16 mins.
 *  Q4_K : nibble values 0..15, scale=f16(d*sc), min=f16(-dmin*m)
 *         (tensors/Q4_KTensor.cpp:768-800, SIMDHelpers.h:10974-11014,
 *          CPUNativeVNNIWeightPacker.h:836-843)
 *  Q6_K : 8.8 fixed-point requantisation to int8, one scale per 32
 *         (tensors/SIMDHelpers.h:12023-12204, WeightPacker.h:1009-1019)
 *  IQ3_S: codebook decode then float requantisation to int8
 *         (tensors/SIMDHelpers.h:8612-8768, WeightPacker.h:1009-1019)           */
void qlo_subblocks_q4k(const llam_block_q4_K *sb, int8_t *w256, uint16_t *scale8, uint16_t *min8);
void qlo_subblocks_q6k(const llam_block_q6_K *sb, int8_t *w256, uint16_t *scale8, uint16_t *min8);
void qlo_subblocks_iq3s(const llam_block_iq3_s *sb, int8_t *w256, uint16_t *scale8, uint16_t *min8);
void qlo_subblocks(int fmt, const void *sb, int8_t *w256, uint16_t *scale8, uint16_t *min8);

/* C[m*ldc + n] for rows n in [n0,n1) of an [N x K] weight matrix stored as
 * row-major GGUF super-blocks, against M rows of Q8_1 activations
 * (A[m*(K/32) + kb]).  Per output element, kb ascending
 * (CPUNativeVNNIGemv.h:412-518 / :549-646):
 *     idot = sum_i a.qs[i]*w[i]                       (int32, exact)
 *     acc  = fmaf((float)idot, f32(a.d)*f32(b_scale), acc)
 *     acc  = fmaf((float)a.sum_qs*f32(a.d), f32(b_min), acc)   (Q4_K, Q6_K)
 * k_tiles <= 1: one chain over all blocks (default GEMV, all GEMM rows);
 * k_tiles  > 1: per-tile chains of ceil(KB/k_tiles) blocks summed in tile
 *               order (CPUNativeVNNIGemv.h:756-892).
 * block_sums, if not NULL, receives idot as [M][n1-n0][K/32] int32.            */
void qlo_gemm_rows(int fmt, const void *W, int K, int n0, int n1,
                   const llam_block_q8_1 *A, int M, float *C, int ldc,
                   int32_t *block_sums, int k_tiles);

/* alpha/beta/bias epilogue of the operator (CPUNativeVNNIGemmKernel.h:154-214):
 * C = beta*C (0 when beta==0) then C += alpha*tmp, then C += bias.             */
void qlo_epilogue(float *C, const float *tmp, int M, int N, int ldc,
                  float alpha, float beta, const float *bias);

/* Router (kernels/cpu/moe/CPUMoEKernel.cpp:24-131): softmax over all experts
 * with exp(l-max)*(1/sum), top_k by probability (ties: lower index first),
 * weights p_k / sum_topk p when normalize != 0.  probs may be NULL.             */
void qlo_moe_route(const float *logits, int n_tokens, int n_experts, int top_k,
                   int normalize, int32_t *ids, float *weights, float *probs);

/* silu(g)*u = (g / (1 + expf(-g))) * u, the reference's scalar routine
 * (kernels/cpu/primitives/SwiGLUPrimitives.cpp:40-51, bit-identical on the same libm).
 * Its vector paths (:137-208: a degree-5 exp polynomial, rcp14 and one Newton step)
 * approximate the same function; measured against the reference's compiled code they
 * stay within 8e-6 relative per element, which the tests check where oracle/_ref is
 * built and on the committed vectors. */
void qlo_swiglu(const float *gate, const float *up, int n, float *out);

/* Exhaustive checks of division-free forms used by the GPU kernels: number of inputs on
 * which they differ from the reference's divisions (0 expected).                          */
long qlo_check_div127(void);
long qlo_check_div127_all_significands(void);
long qlo_check_q6k_factor(int ulps);

/* ---- decode-step operators (decode_oracle.c) ------------------------------------- */
void qlo_dequant_row_q4k(const llam_block_q4_K *blocks, int nblocks, float *out);
void qlo_rmsnorm(float *x, const float *delta, const float *gamma, float eps, float *y, int rows, int cols);
void qlo_rope_inv_freq(int head_dim, float theta, float *inv_freq);
void qlo_rope_head(float *head, int position, const float *inv_freq, int head_dim);
void qlo_rope_kv_append(float *qkv, const float *inv_freq, int position, uint16_t *kcache, uint16_t *vcache,
                        int n_heads, int n_kv, int head_dim, int ctx_cap);
void qlo_attention_decode(const float *q, const uint16_t *kcache, const uint16_t *vcache, int last, float *out,
                          int n_heads, int n_kv, int head_dim, int ctx_cap);
int qlo_argmax(const float *x, int n);

/* STREAM triad over three arrays of n doubles, all OpenMP threads; bytes per second of the best of `reps` passes */
double qlo_stream_triad(double *a, const double *b, const double *c, long n, int reps);

#ifdef __cplusplus
}
#endif
#endif
