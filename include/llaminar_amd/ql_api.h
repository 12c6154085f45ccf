/*
 * C-ABI of the MI355X (gfx950) quantized-linear library: GGUF block-quantized
 * weight x Q8_1-quantized activation products.  This is the whole boundary a
 * host engine binds: plain device pointers and sizes, no C++ or framework
 * types.
 *
 * Conventions (the ones the reference's own extern "C" HIP launchers follow,
 * e.g. rocmGemv_native_vnni_fp32, src/v2/kernels/rocm/gemm/ROCmGemvKernel_native_VNNI.hip:5228-5260):
 *   - every entry point returns bool; false = invalid argument or launch
 *     failure, with a "[fn] reason" line on stderr and llam_ql_last_error()
 *     holding the same text for the calling thread;
 *   - all pointers named d_* are device pointers on `device_id`; the call makes
 *     that device current, enqueues on `stream` (a hipStream_t, NULL = default
 *     stream) and returns without synchronising;
 *   - nothing is allocated, freed or synchronised inside a call;
 *   - results are deterministic: no floating-point atomics, fixed reduction
 *     order (the reference's LLAMINAR_DETERMINISTIC contract,
 *     ROCmGemvKernel_native_VNNI.hip:5260-5261).
 *
 * Weight matrices are [N rows x K columns], row-major in super-blocks of 256
 * columns (K % 256 == 0).  `fmt` is a llam_weight_format value.
 *
 * Arithmetic contract (reference CPU path, CPUNativeVNNIGemv.h:412-518):
 *   per 32-column block  idot = sum_i a.qs[i]*w[i]           (int32, exact)
 *                        acc += float(idot) * (f32(a.d)*f32(b_scale))
 *                        acc += (float(a.sum_qs)*f32(a.d)) * f32(b_min)
 * with (w, b_scale, b_min) the effective int8 sub-block the reference's weight
 * packer derives from the GGUF block (CPUNativeVNNIWeightPacker.h:598-1136).
 */
#ifndef LLAMINAR_AMD_QL_API_H
#define LLAMINAR_AMD_QL_API_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include "llaminar_amd/ql_blocks.h"

#ifdef __cplusplus
extern "C" {
#endif

#define LLAM_QL_MAX_GEMV_M 8      /* rows of activations one GEMV launch accepts */
#define LLAM_QL_MAX_FUSED 16      /* projections per fused launch (reference: <=16 FusedGemvDesc) */

/* Text of the calling thread's most recent failure ("" if none). */
const char *llam_ql_last_error(void);

/* Library ABI version (bumped on any signature change). */
int llam_ql_abi_version(void);

/* Tuning overrides for sweeps (reference: rocmGemv_native_vnni_set_tuning_overrides /
 * ..._reset_tuning_overrides, ROCmGemvKernel_native_VNNI.hip:182-196).
 * rows_per_wave: rows (row batches) one wavefront walks; unroll: 1..4 forces the
 * chunked kernel with that many load batches in flight, also where the quad-lane
 * kernel would be used.  Values <= 0 restore the built-in choice.  Not thread-safe. */
void llam_ql_set_gemv_tuning(int rows_per_wave, int unroll);
void llam_ql_reset_gemv_tuning(void);
/* Batch plane of a prepared matrix: an optional second copy for callers that decode batches of
 * 5..8 rows, laid out as the matrix unit takes its operands (rows in groups of four, a 128-byte
 * line per group and block), separate from the prepared matrix.
 *   Q6_K: the weights requantised to int8 once (the 8.8 requantisation of
 *     packWeightsCPUNativeVNNI's Q6_K branch, SIMDHelpers.h:12023-12204, which the decode
 *     kernels otherwise repeat on every launch) beside their fp16 block scales, 272 bytes per
 *     super-block and row; rows of eight super-blocks and more.  A batch of 5..8 rows of that
 *     matrix launched with its plane runs on the matrix-unit plane kernel.
 *   Q4_K: the 144 bytes of every super-block regrouped, not changed; shapes whose batches of
 *     5..8 go to the matrix-unit kernel (4096 rows and more).  The kernel then finds a lane's
 *     operands at one address and needs no LDS bounce.
 * Results are bit-identical to the matrix-unit kernels without a plane.  The reference's packed
 * matrix is int8 in operand order to begin with; here that is the optional copy.
 *   llam_ql_batch_plane_bytes: size of the plane, 0 if the format or shape has none (Q4_K: also
 *     while llam_ql_set_gemv_tuning overrides are in force, which keep batches off the matrix unit).
 *   llam_ql_build_batch_plane: fills d_plane (16-byte aligned) from the prepared matrix.
 * The caller owns the plane and hands it to every launch that may use it: the d_plane argument
 * of llam_ql_gemv_plane, llam_ql_gemv_swiglu_f32 and llam_ql_gemv_block_sums, the d_plane field
 * of llam_ql_proj.  NULL means "no plane" everywhere; a plane is only read by batches of 5..8
 * rows.  The library keeps no record of planes: a plane handed to a launch must be the one built
 * from the d_w of the same launch, and both must stay alive until the launch has finished. */
size_t llam_ql_batch_plane_bytes(uint8_t fmt, int N, int K);
bool llam_ql_build_batch_plane(uint8_t fmt, const void* d_prepared, void* d_plane, int N, int K,
                               int device_id, void* stream);

/* ---- P1: activation quantiser --------------------------------------------------
 * fp32 [M x K] (row stride K) -> llam_block_q8_1 [M x ceil(K/32)].  d_x 16-byte aligned when
 * K % 32 == 0 (every shape the GEMV and GEMM entry points take), 4-byte aligned otherwise: a row's
 * partial last block then follows the reference's scalar quantiser (round half away from zero,
 * software fp16 conversion, zero padding; src/v2/tensors/SIMDHelpers.h:4554-4596).
 * Replaces simd::quantize_single_block / quantize_two_blocks_avx512 and
 * quantize_activations_to_q8_1 (src/v2/tensors/SIMDHelpers.h:4716-4959,
 * src/v2/kernels/cpu/native_vnni/CPUNativeVNNIGemv.h:2000-2036); device-side
 * counterpart of rocmQuantGemm_quantizeActivationsBlockwise
 * (src/v2/kernels/rocm/gemm/ROCmQuantisedGemmKernel.hip:1187-1193).
 * Output bytes equal the reference CPU quantiser's bit for bit. */
bool llam_ql_quantize_q8_1(const float *d_x, void *d_q8, int M, int K,
                           int device_id, void *stream);

/* ---- weight preparation -----------------------------------------------------------
 * Device layout the GEMV/GEMM kernels read.  Q4_K: the GGUF super-blocks
 * unchanged (144 B is 16-byte aligned).  Q6_K (210 B) and IQ3_S (110 B) are
 * split into 16-byte-aligned planes (IQ3_S +2 B/block padding); no weight byte is
 * changed.  Q6_K additionally gets a plane of one 4-byte record per 32-element block
 * (+32 B per super-block): the two 8.8 requantisation factors of the block and its
 * fp16 scale, i.e. what unpack_q6_k_superblock_to_int8 (SIMDHelpers.h:12023-12204)
 * derives from the sub-scales, worked out once instead of in every product.
 * Replaces packWeightsCPUNativeVNNI (CPUNativeVNNIWeightPacker.h:598) /
 * repack_*_to_vnni (src/v2/kernels/rocm/repack/VnniRepackKernels.hip:65-887).
 * d_prepared must be 16-byte aligned and llam_ql_prepared_bytes() large; it may
 * equal d_gguf for Q4_K only. */
size_t llam_ql_prepared_bytes(uint8_t fmt, int N, int K);
bool llam_ql_prepare_weights(uint8_t fmt, const void *d_gguf, void *d_prepared,
                             int N, int K, int device_id, void *stream);

/* ---- P2: decode GEMV (M = 1..LLAM_QL_MAX_GEMV_M) -----------------------------------
 * d_y[m*ldy + n] = sum_k W[n,k] * A[m,k] for prepared weights and Q8_1
 * activations A[m][K/32].  Replaces gemv_native_vnni_preq
 * (CPUNativeVNNIGemv.h:712-954) and, for M>1, the small-M decode rows;
 * device-side counterpart of rocmGemv_native_vnni_fp32
 * (ROCmGemvKernel_native_VNNI.hip:5228). */
bool llam_ql_gemv(uint8_t fmt, const void *d_w, const void *d_q8, float *d_y,
                  int M, int N, int K, int ldy, int device_id, void *stream);
/* The same with the matrix's batch plane (llam_ql_build_batch_plane; NULL: llam_ql_gemv): batches
 * of 5..8 rows read the plane instead of d_w, smaller batches ignore it. */
bool llam_ql_gemv_plane(uint8_t fmt, const void *d_w, const void *d_plane, const void *d_q8,
                        float *d_y, int M, int N, int K, int ldy, int device_id, void *stream);

/* One projection of a fused launch (reference: FusedGemvDesc,
 * CPUNativeVNNIGemv.h:3782-3881 / TensorProjectionDesc, TensorKernels.h:601). */
typedef struct
{
    const void *d_w;   /* prepared weights [N x K] */
    float *d_y;        /* output, row stride ldy   */
    int N;
    int ldy;
    uint8_t fmt;
    const void *d_plane; /* the matrix's batch plane (llam_ql_build_batch_plane), or NULL */
} llam_ql_proj;

/* Several projections of ONE quantised input in one launch (QKV, gate+up,
 * 2*top_k MoE gate/up).  Replaces gemv_native_vnni_fused_preq
 * (CPUNativeVNNIGemv.h:3807-3881).  num <= LLAM_QL_MAX_FUSED; `projs` is a host
 * array read during the call.  Neighbours in the array share a launch where their kernels
 * allow it (up to four quad-lane matrices of one format, a second run in the other quad-lane
 * format behind them, and at batches of 5..8 a Q4_K matrix on the matrix unit with the small
 * quad-lane matrices that follow it: Q, then K and V); every output carries the bits of its own
 * llam_ql_gemv / llam_ql_gemv_plane call. */
bool llam_ql_gemv_fused(const llam_ql_proj *projs, int num, const void *d_q8,
                        int M, int K, int device_id, void *stream);

/* The same from fp32 activations (rows of ldx floats, 16-byte aligned, ldx % 4 == 0):
 * the Q8_1 quantisation of llam_ql_quantize_q8_1 happens inside the GEMV kernels, so
 * the results are the bits of "quantise, then llam_ql_gemv / llam_ql_gemv_fused" without
 * the quantiser's launch and its round trip through memory.  These are the operator's
 * fp32-input decode calls: multiply_tensor with small m and multiply_fused_tensor
 * (CPUNativeVNNIGemmKernel.h:154-214, 572-700: quantize_activations_to_q8_1 followed by
 * gemv_native_vnni_preq / gemv_native_vnni_fused_preq).
 * d_q8_scratch: M * K/32 * 36 bytes, or NULL.  It is written only when a projection's
 * kernel cannot quantise for itself (IQ3_S, K < 4096, M*K too large for LDS); with NULL
 * such a call fails. */
bool llam_ql_gemv_f32(uint8_t fmt, const void *d_w, const float *d_x, int ldx, float *d_y,
                      int M, int N, int K, int ldy, void *d_q8_scratch, int device_id,
                      void *stream);
bool llam_ql_gemv_fused_f32(const llam_ql_proj *projs, int num, const float *d_x, int ldx,
                            int M, int K, void *d_q8_scratch, int device_id, void *stream);

/* llam_ql_gemv_f32 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the Q8_1 scratch is a
 * buffer of LLAM_QL_STATIC_SCRATCH_BYTES built into the library's device image, so the
 * caller passes inputs and outputs only and the results are the bits of llam_ql_gemv_f32
 * with a scratch buffer.  It has no counterpart in the reference, whose operators draw
 * scratch from a caller-bound DeviceWorkspaceManager.
 * Limits: M * (K/32) * 36 <= LLAM_QL_STATIC_SCRATCH_BYTES (8 rows of K = 32768), otherwise
 * the call fails with a message.  All calls on one GPU share that GPU's buffer: two calls that
 * overlap on one GPU (different streams or host threads) race; calls on one stream are
 * ordered and safe.  Nothing in the buffer needs clearing between calls. */
#define LLAM_QL_STATIC_SCRATCH_BYTES (8 * (32768 / 32) * 36)
bool llam_ql_gemv_f32_static(uint8_t fmt, const void *d_w, const float *d_x, int ldx, float *d_y,
                             int M, int N, int K, int ldy, int device_id, void *stream);

/* d_y = (silu(gate) * up) @ W^T for fp32 gate/up rows of ld_gu floats: the bits of
 * llam_ql_swiglu_quantize followed by llam_ql_gemv, in one launch.  Replaces
 * multiply_tensor_with_fused_swiglu (CPUNativeVNNIGemmKernel.h:325-431: compute_swiglu,
 * then the quantising GEMV).  d_q8_scratch as above; d_plane: the matrix's batch plane or NULL. */
bool llam_ql_gemv_swiglu_f32(uint8_t fmt, const void *d_w, const void *d_plane, const float *d_gate,
                             const float *d_up, int ld_gu, float *d_y, int M, int N, int K,
                             int ldy, void *d_q8_scratch, int device_id, void *stream);

/* The feed-forward block's first half in one launch, batches of 2..8 rows:
 *   d_q8_out = Q8_1( silu(W_gate a) * (W_up a) )   [M x N/32 blocks], the down projection's input.
 * Both projections run on the matrix unit with their 32-row tiles paired inside a workgroup, which then
 * holds both operands of 32 consecutive columns and quantises the block itself: no launch for the
 * second projection, none for llam_ql_swiglu_quantize, no fp32 round trip.  d_y_gate / d_y_up (row
 * stride ldy) receive the fp32 projections when not NULL; d_q8_out is bit for bit
 * llam_ql_swiglu_quantize of those.  The projections are those of the matrix-unit kernel (the
 * reference's ascending block order within a wavefront's share of the row, llam_ql_gemv's contract for
 * batches of 5..8); their last bits may differ from two llam_ql_gemv calls, which split a row into
 * other shares -- and at M = 2..4 a row does not carry the bits of its single-row call, which llam_ql_gemv
 * guarantees there: the entry point is for callers whose rows are independent sequences.
 * Served (llam_ql_gemv_gate_up_swiglu_supported) for Q4_K, M = 2..8, N a multiple of 32
 * and at least 4096, rows of 8..45 super-blocks (K = 2048..11520); d_plane_gate / d_plane_up: both matrices' batch planes
 * or both NULL.  Replaces multiply_fused_tensor over {gate, up} + compute_swiglu + the quantiser of
 * the down projection (CPUNativeVNNIGemmKernel.h:572, :325-431; the decode flow of
 * MoEExpertComputeStage.cpp:1450-1708 for a dense block). */
bool llam_ql_gemv_gate_up_swiglu_supported(uint8_t fmt, int M, int N, int K);

/* A projection with long rows at batches of 2..8 (Q4_K: 5..8), its rows summed in two halves:
 *     d_y_lo[m][n] = sum over the first K/2 columns,  d_y_hi[m][n] = sum over the last K/2
 * from the matrix's batch plane (d_plane, llam_ql_build_batch_plane), per 32-column block the arithmetic of
 * llam_ql_gemv_plane.  The caller adds the two (llam_dec_rmsnorm2_q8_1 does, in front of the next norm).
 * Why: every workgroup of a matrix-unit launch stages the batch's activations for the columns it
 * walks; for K = 25600 that is 230 KB per workgroup, as much traffic as its weights.  Here a workgroup
 * walks half of the columns of twice the rows: 5120 x 25600 at batch 8 31 against 36 us.  The split is
 * the reference's row-parallel tensor split of this projection run on one device (each K slice yields a
 * partial sum, TPAllreduceStage adds them), without the exchange.  Served
 * (llam_ql_gemv_plane_split_supported) for K a multiple of 512 with K >= 16384: Q6_K at M = 2..8 (like the
 * entry point above it names the matrix-unit kernel: rows of batches of 2..4 do not carry the bits of their
 * single-row calls), and Q4_K matrices whose batch goes to the chunked matrix-unit kernel (4096 rows and more,
 * a batch too large for the LDS whole: M = 5..8 at most); both outputs have row stride ldy and must be
 * different buffers. */
bool llam_ql_gemv_plane_split_supported(uint8_t fmt, int M, int N, int K);
bool llam_ql_gemv_plane_split(uint8_t fmt, const void *d_plane, const void *d_q8, float *d_y_lo, float *d_y_hi, int M,
                              int N, int K, int ldy, int device_id, void *stream);
bool llam_ql_gemv_gate_up_swiglu(uint8_t fmt, const void *d_w_gate, const void *d_plane_gate,
                                 const void *d_w_up, const void *d_plane_up, const void *d_q8,
                                 float *d_y_gate, float *d_y_up, int ldy, void *d_q8_out, int M, int N,
                                 int K, int device_id, void *stream);

/* Parity hook: the exact per-block int32 sums the GEMV forms, for rows
 * [row0, row0+nrows): d_sums[(m*nrows + r)*(K/32) + kb].  The call makes the choices
 * llam_ql_gemv makes for (fmt, M, N, K) -- quad-lane, matrix-unit, chunked or generic
 * kernel, K slices, batch splits -- and runs the chosen kernel's block-sum variant: the
 * same code compiled with the stores of the sums switched on and the fp32 output off.
 * (The reference exposes the same quantity only inside its kernels: int_acc in
 * CPUNativeVNNIGemv.h:417-487.)  d_plane: the batch plane the launch to be checked would get, or
 * NULL -- with a plane and a batch it serves, the plane kernel's block-sum variant runs.
 * M * nrows * (K/32) * 4 bytes must stay below 2 GiB. */
bool llam_ql_gemv_block_sums(uint8_t fmt, const void *d_w, const void *d_plane, const void *d_q8,
                             int32_t *d_sums, int M, int N, int K, int row0,
                             int nrows, int device_id, void *stream);

/* d_y[m, n] += dot(W[n, :], x[m, :]): llam_ql_gemv whose row sums are added (one fp32 add each) to
 * what d_y holds -- the residual add in front of the next norm (fused_residual_rmsnorm_row_*,
 * RMSNormPrimitives.cpp:1491-1562) done by the projection that produces the delta, with the bits of
 * llam_ql_gemv followed by that add.  Served where llam_ql_gemv_accumulate_supported says so
 * (a single quad-lane launch that reduces its rows in LDS); elsewhere the call fails and the
 * caller keeps the delta in a buffer of its own. */
bool llam_ql_gemv_accumulate_supported(uint8_t fmt, int M, int N, int K, int device_id);
bool llam_ql_gemv_accumulate(uint8_t fmt, const void *d_w, const void *d_q8, float *d_y, int M,
                             int N, int K, int ldy, int device_id, void *stream);

/* RMSNorm, Q8_1 quantiser and the projections of the normalised row in the projections' own
 * launches: every workgroup normalises and quantises the M rows for itself (rows of a few
 * thousand floats), which saves the norm's launch.
 *     v = d_x[m] (+ d_delta[m] when d_delta is given; then d_x_out[m] = v, d_x is not written)
 *     y = (v * (1/rms)) * gamma,  rms = sqrt(float(sum_sq / K) + eps), sum_sq in double
 *     projections of the Q8_1 blocks of y, as llam_ql_gemv_fused
 * with the bits of llam_dec_rmsnorm_q8_1 followed by llam_ql_gemv_fused (the fused form of
 * CPURMSNormKernelT<FP32>::apply_with_residual_add, CPURMSNormKernelT.h:300-322, in front of the
 * activation quantiser).  Rows of d_x, d_delta and d_x_out are K floats apart.  Served where
 * llam_ql_gemv_fused_rmsnorm_supported says so (single rows, M == 1, of shapes the quad-lane
 * kernel takes); elsewhere the call fails and the norm and the projections run as two calls.
 * d_x_out must not overlap d_x or d_delta. */
bool llam_ql_gemv_fused_rmsnorm_supported(const llam_ql_proj *projs, int num, int M, int K);
bool llam_ql_gemv_fused_rmsnorm(const llam_ql_proj *projs, int num, const float *d_x,
                                const float *d_delta, const float *d_gamma, float eps,
                                float *d_x_out, int M, int K, int device_id, void *stream);

/* What llam_ql_gemv (has_plane == 0) or a launch that brings the matrix's batch plane
 * (has_plane != 0) does with a shape: which kernel runs, how the batch and the row are split.  For tests, tuning and the operator's decode-equivalence guard; the launcher
 * executes exactly this plan.  (Reference: the dispatch tables behind
 * rocmGemv_native_vnni_fp32, ROCmNativeVNNIDecodeDispatchGenerated.inc.) */
#define LLAM_QL_KERNEL_GENERIC 0 /* rows shorter than 5 super-blocks */
#define LLAM_QL_KERNEL_CHUNKED 1 /* 8 lanes per super-block, whole rows per wavefront */
#define LLAM_QL_KERNEL_QUAD 2    /* 4 lanes per super-block, runs of rows per wavefront */
#define LLAM_QL_KERNEL_MFMA 3    /* batches of 5..8 on the matrix unit */
typedef struct
{
    int kernel;            /* LLAM_QL_KERNEL_*, or -1 when the shape cannot be served */
    int m_first;           /* activation rows of the first launch group (the rest follows alike) */
    int slice_sb;          /* super-blocks per K slice (one slice = the whole row) */
    int rows_per_wave;
    int decode_equivalent; /* 1: every row of the M-row call has the bits of its own M = 1 call */
} llam_ql_gemv_plan;
bool llam_ql_gemv_describe(uint8_t fmt, int M, int N, int K, int has_plane, int device_id,
                           llam_ql_gemv_plan *out);

/* ---- P3: prefill GEMM (any M) -------------------------------------------------------
 * Same contract as llam_ql_gemv for many activation rows, on int8 MFMA with
 * int32 accumulation per 32-column block and fp32 rescale.  Replaces
 * gemm_native_vnni_preq (CPUNativeVNNIGemv.h:2046-2287); device-side
 * counterpart of launch_native_vnni_gemm
 * (src/v2/kernels/rocm/gemm/ROCmQuantisedGemmKernel_native_VNNI.hip:2580-2632).
 * Token tiles of 32 (M <= 32), 64 (M <= 64) or 128 tokens: the fp32 sum of a row's blocks
 * is formed in an order that depends on the tile, so a row's last bits may differ between
 * calls of different M (the per-block int32 sums never do). */
bool llam_ql_gemm(uint8_t fmt, const void *d_w, const void *d_q8, float *d_y,
                  int M, int N, int K, int ldy, int device_id, void *stream);

/* Parity hook of the GEMM: the matrix unit's exact per-block int32 sums of weight rows
 * [row0, row0+nrows) for all M activation rows, d_sums[(m*nrows + r)*(K/32) + kb], from
 * the block-sum variant of llam_ql_gemm's kernel (same tiles, same decode, same MFMA).
 * Counterpart of the reference's int32 accumulators in gemm_2row_native_chunk /
 * gemm_2row_int8_chunk (CPUNativeVNNIGemv.h:1046-1376). */
bool llam_ql_gemm_block_sums(uint8_t fmt, const void *d_w, const void *d_q8, int32_t *d_sums,
                             int M, int N, int K, int row0, int nrows, int device_id,
                             void *stream);

/* C = beta*C + alpha*T (+ bias per column), the operator's epilogue
 * (CPUNativeVNNIGemmKernel.h:154-214).  beta == 0 overwrites.  T row stride N. */
bool llam_ql_epilogue(float *d_c, const float *d_t, const float *d_bias, int M,
                      int N, int ldc, float alpha, float beta, int device_id,
                      void *stream);

/* ---- P4: MoE ---------------------------------------------------------------------------
 * Router logits: d_logits[t*n_experts + e] = dot(d_hidden[t,:], d_gate_w[e,:]) in fp32
 * (the router matrix is not quantised).  Replaces the vec_dot loop at the top of
 * CPUMoEKernel::route (src/v2/kernels/cpu/moe/CPUMoEKernel.cpp:45-49); floating point,
 * summation order differs from the reference's SIMD dot (tests: 1e-5 of the largest
 * logit).  d_model % 4 == 0. */
bool llam_ql_moe_router_logits(const float *d_hidden, const float *d_gate_w, float *d_logits,
                               int n_tokens, int d_model, int n_experts, int device_id,
                               void *stream);

/* Router: softmax over all experts, top_k by probability (ties: lower expert
 * id first), weights renormalised over the top_k when normalize != 0.
 * Replaces CPUMoEKernel::route's selection stage
 * (src/v2/kernels/cpu/moe/CPUMoEKernel.cpp:87-124; IMoEKernel::route,
 * src/v2/kernels/IMoEKernel.h:56).  d_logits [n_tokens x n_experts]. */
bool llam_ql_moe_route(const float *d_logits, int n_tokens, int n_experts,
                       int top_k, int normalize, int32_t *d_ids,
                       float *d_weights, int device_id, void *stream);

/* llam_ql_moe_route_ex and llam_ql_quantize_q8_1(d_hidden, d_q8, n_tokens, d_model) in one
 * launch: the hidden state the expert GEMVs read does not depend on the routing, so its
 * quantiser rides along (same bits as the two calls).  No counterpart in the reference, whose
 * stage quantises inside the first expert GEMV (MoEExpertComputeStage.cpp:1450-1500). */
bool llam_ql_moe_route_quantize(const float *d_logits, int n_tokens, int n_experts, int top_k,
                                int normalize, int32_t *d_ids, float *d_weights, int slot_stride,
                                const float *d_hidden, int d_model, void *d_q8, int device_id,
                                void *stream);

/* Same with the slots of a token slot_stride (>= top_k) entries apart in d_ids and
 * d_weights: columns top_k.. are left alone, so a caller can keep always-on experts
 * (the shared expert of MoEExpertComputeStage.cpp:1450-1708, weight 1 or its sigmoid
 * gate) in them and run routed and shared experts through one gate/up and one down
 * launch with top_k = slot_stride. */
bool llam_ql_moe_route_ex(const float *d_logits, int n_tokens, int n_experts,
                          int top_k, int normalize, int32_t *d_ids,
                          float *d_weights, int slot_stride, int device_id,
                          void *stream);

/* Expert weight table on the device: one entry per expert id (reference:
 * DeviceNativeVNNIMatrixDesc tables, src/v2/tensors/TensorKernels.h:39-55,
 * uploaded via IMoEKernel::upload...DescriptorTable, IMoEKernel.h:378-643). */
typedef struct
{
    const void *d_gate; /* prepared [inter x hidden] */
    const void *d_up;   /* prepared [inter x hidden] */
    const void *d_down; /* prepared [hidden x inter] */
} llam_ql_expert;

/* Gate/up GEMVs of the routed experts, driven by device-resident routing ids:
 * for token t, slot s, expert e = d_ids[t*top_k+s]:
 *   d_gate_out[(t*top_k+s)*inter + i] = W_gate[e][i,:] . q8(hidden[t])
 *   d_up_out  [(t*top_k+s)*inter + i] = W_up  [e][i,:] . q8(hidden[t])
 * d_q8 holds the Q8_1 hidden state [n_tokens x hidden/32].  Replaces the
 * 2*top_k-projection multiply_fused_tensor of MoEExpertComputeStage
 * (src/v2/execution/compute_stages/stages/MoEExpertComputeStage.cpp:1450-1482);
 * counterpart of groupedExpertGateUpDecodeFromRouting (IMoEKernel.h:378-643).
 * The table has n_experts entries; a slot whose id is outside [0,n_experts), or whose
 * expert has a NULL matrix in the table (an expert that lives on another device), is
 * skipped (its outputs are left untouched). */
bool llam_ql_moe_gate_up(uint8_t fmt, const llam_ql_expert *d_experts,
                         int n_experts, const int32_t *d_ids, const void *d_q8,
                         float *d_gate_out, float *d_up_out, int n_tokens,
                         int top_k, int hidden, int inter, int device_id,
                         void *stream);

/* act[i] = silu(gate[i]) * up[i] over n values, then Q8_1-quantise rows of
 * `inter` values: d_q8_out [rows x inter/32].  d_act_out (optional) receives the
 * fp32 activations.  Replaces compute_swiglu_serial + the per-expert quantise
 * of multiply_fused_expert_down (MoEExpertComputeStage.cpp:1646,
 * CPUNativeVNNIGemmKernel.h:1094-1107). */
bool llam_ql_swiglu_quantize(const float *d_gate, const float *d_up,
                             float *d_act_out, void *d_q8_out, int rows,
                             int inter, int device_id, void *stream);

/* Down GEMVs and weighted accumulation:
 *   d_out[t*hidden + h] (+)= sum_s d_weights[t*top_k+s] * (W_down[e_s][h,:] . q8_act[t,s])
 * Slots are added in ascending s; accumulate != 0 adds onto d_out, else
 * overwrites (a token all of whose slots are skipped gets zeros).  Replaces multiply_fused_expert_down + vec_axpy
 * (MoEExpertComputeStage.cpp:1664-1673); counterpart of
 * groupedExpertDownDecode* (IMoEKernel.h:378-643). */
bool llam_ql_moe_down(uint8_t fmt, const llam_ql_expert *d_experts,
                      int n_experts, const int32_t *d_ids, const float *d_weights,
                      const void *d_q8_act, float *d_out, int n_tokens,
                      int top_k, int hidden, int inter, int accumulate,
                      int device_id, void *stream);

/* llam_ql_moe_gate_up followed by llam_ql_swiglu_quantize, the same Q8_1 bytes:
 *   d_q8_out [(t*top_k+s)][inter/32] = Q8_1(silu(W_gate[e] . q8(hidden[t])) * (W_up[e] . q8(hidden[t])))
 * For expert rows of 2, 4, 8 or 16 super-blocks (hidden/256) this is ONE launch: a workgroup owns the 32
 * gate and 32 up rows of one Q8_1 block, so the fp32 intermediate never leaves the chip and
 * d_gate_scratch / d_up_scratch may be NULL.  Every other row length runs the two
 * launches through the scratch rows (fp32 [n_tokens*top_k x inter] each; NULL is refused there).
 * Blocks of skipped slots (id outside [0,n_experts), NULL matrix) are left untouched in the
 * one-launch form and are quantised from whatever the scratch holds in the other; no later
 * stage reads them.  Counterpart of the fused decode epilogue of
 * groupedExpertGateUpDecodeFromRouting + swiGLU (IMoEKernel.h:378-643, :168-180). */
bool llam_ql_moe_gate_up_swiglu(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                const int32_t *d_ids, const void *d_q8, float *d_gate_scratch,
                                float *d_up_scratch, void *d_q8_out, int n_tokens, int top_k,
                                int hidden, int inter, int device_id, void *stream);

/* llam_ql_moe_route_quantize followed by llam_ql_moe_gate_up_swiglu: the same ids, weights and Q8_1
 * bytes.  For expert rows of 2, 4, 8 or 16 super-blocks (hidden/256), at most 512 routed experts and few tokens
 * (fewer workgroups than two per compute unit: one or two tokens of a 9-slot, 512-row expert shape)
 * this is ONE launch: every workgroup quantises its token's hidden row into its LDS and routes the
 * token for itself (work that precedes the first weight load in any case), so a decode step is two
 * launches: this one and llam_ql_moe_down.  With more tokens the repeated routing costs more than the
 * launch it saves and the call runs the two launches.  d_logits [n_tokens x n_route_experts]; d_ids / d_weights
 * [n_tokens x slot_stride]: columns < top_k are written, columns top_k.. are READ as always-on slots
 * (the shared expert: its table index and weight, set by the caller once); the expert table has
 * n_experts >= n_route_experts entries.  d_hidden fp32 [n_tokens x hidden].  The two-launch form
 * needs d_q8_hidden_scratch (Q8_1 [n_tokens x hidden/32]) and, for row lengths outside
 * llam_ql_moe_gate_up_swiglu's one-launch kernel, its fp32 scratch rows; a caller that cannot tell
 * passes all three (they are left untouched when not needed).
 * Counterpart of decodeRouteSelect + groupedExpertGateUpDecodeFromRuntime + swiGLU
 * (IMoEKernel.h:245-258, :378-643, :171). */
bool llam_ql_moe_route_gate_up_swiglu(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                      const float *d_logits, int n_route_experts, int top_k, int normalize,
                                      int32_t *d_ids, float *d_weights, int slot_stride,
                                      const float *d_hidden, void *d_q8_hidden_scratch,
                                      float *d_gate_scratch, float *d_up_scratch, void *d_q8_out,
                                      int n_tokens, int hidden, int inter, int device_id, void *stream);

/* ---- batches: tokens grouped by expert ---------------------------------------------------
 * With several tokens the same expert is usually picked more than once (16 tokens x 8 slots
 * of 256 experts hit about 100 distinct ones, and an always-on shared expert serves all 16).
 * llam_ql_moe_group sorts the (token, slot) pairs by expert id on the device (stable; ids
 * outside [0, n_experts) are left out) into a caller-provided workspace of
 * llam_ql_moe_group_bytes(); the _grouped launches then read every distinct expert's matrices
 * once per chunk of two of its tokens (four from 512 pairs on).  Outputs are the bits of the
 * ungrouped launches.  At most 4096 pairs per call.  Replaces the per-expert bucketing of
 * MoEExpertComputeStage::execute (MoEExpertComputeStage.cpp:884-979: gatherTokenBatch,
 * multiply_fused_tensor with m = tokens of the expert, scatterAddWeighted); device counterpart
 * IMoEKernel::groupTokensByExpertDevice (src/v2/kernels/IMoEKernel.h:737) and
 * moe_grouped_prefill (src/v2/kernels/rocm/gemm/ROCmMoEGroupedPrefillKernels.hip:1465).
 * d_ids [n_tokens x slot_stride] as written by llam_ql_moe_route_ex (every column is a slot). */
size_t llam_ql_moe_group_bytes(int n_tokens, int slot_stride);
bool llam_ql_moe_group(const int32_t *d_ids, int n_tokens, int slot_stride, int n_experts,
                       void *d_group, int device_id, void *stream);
/* llam_ql_moe_gate_up over the grouped pairs: same outputs, same layout
 * (d_gate_out[(t*slot_stride+s)*inter + i]). */
bool llam_ql_moe_gate_up_grouped(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                                 const void *d_group, const void *d_q8, float *d_gate_out,
                                 float *d_up_out, int n_tokens, int slot_stride, int hidden,
                                 int inter, int device_id, void *stream);
/* llam_ql_moe_down over the grouped pairs: the down products of every pair go to
 * d_pair_out [n_tokens*slot_stride x hidden] (scratch), then a token's live slots are added
 * in ascending order with their routing weights -- the order and arithmetic of
 * llam_ql_moe_down, the same bits.  A token without a live slot gets zeros when
 * accumulate == 0. */
bool llam_ql_moe_down_grouped(uint8_t fmt, const llam_ql_expert *d_experts, int n_experts,
                              const void *d_group, const int32_t *d_ids, const float *d_weights,
                              const void *d_q8_act, float *d_pair_out, float *d_out, int n_tokens,
                              int slot_stride, int hidden, int inter, int accumulate,
                              int device_id, void *stream);

/* Expert ids from a device tensor that holds them as fp32 values (the reference's routing_indices
 * tensors of groupedExpert*DecodeFromRouting, src/v2/kernels/IMoEKernel.h:480-575): truncation
 * toward zero; NaN, negative and out-of-range values become -1, which every launch skips. */
bool llam_ql_moe_ids_from_f32(const float *d_indices, int32_t *d_ids, int n, int device_id,
                              void *stream);

/* The other direction, and what else IMoEKernel::decodeRouteSelect publishes beside the runtime
 * top-k state (src/v2/kernels/IMoEKernel.h:245-258, write_legacy_outputs / update_runtime_histogram;
 * src/v2/kernels/rocm/moe/ROCmMoEKernel.cpp:2956-3019): for every token t and slot s < top_k,
 *   d_indices_f32[t*top_k+s] = float(d_ids[t*slot_stride+s]),  d_weights_f32[t*top_k+s] = d_weights[t*slot_stride+s],
 *   d_histogram[id] += 1 for ids inside [0, n_experts)   (uint64 counts, integer atomics).
 * Each of the three outputs may be NULL. */
bool llam_ql_moe_publish_routing(const int32_t *d_ids, const float *d_weights, int n_tokens, int top_k,
                                 int slot_stride, float *d_indices_f32, float *d_weights_f32,
                                 uint64_t *d_histogram, int n_experts, int device_id, void *stream);

/* Shared expert: d_out[t,:] += g_t * d_shared[t,:] with
 * g_t = sigmoid(dot(d_gate_inp, d_hidden[t,:])), or g_t = 1 when d_gate_inp is
 * NULL.  Replaces CPUMoEKernel::sharedExpertGate + the add into the token output
 * (src/v2/kernels/cpu/moe/CPUMoEKernel.cpp:162-197; IMoEKernel::weightedAdd,
 * src/v2/kernels/IMoEKernel.h:189). */
bool llam_ql_shared_expert_add(float *d_out, const float *d_shared,
                               const float *d_hidden, const float *d_gate_inp,
                               int n_tokens, int d_model, int device_id,
                               void *stream);

/* The remaining device helpers of the MoE operator interface (src/v2/kernels/IMoEKernel.h:92-171;
 * CPU forms in src/v2/kernels/cpu/moe/CPUMoEKernel.cpp:133-202), for callers that batch tokens
 * per expert themselves:
 *   shared_expert_gate    d_shared[t,:] *= sigmoid(dot(d_gate_inp, d_hidden[t,:]))     (sharedExpertGate)
 *   gather_rows           d_batch[i,:] = d_hidden[d_token_indices[i],:]                (gatherTokenBatch)
 *   scatter_add_weighted  d_output[d_token_indices[i],:] += d_weights[i] * d_expert_output[i,:], rows
 *                         taken in ascending i, so repeated indices add up in order   (scatterAddWeighted)
 *   swiglu_inplace        d_gate[i] = silu(d_gate[i]) * d_up[i]                        (swiGLU)
 * n_rows bounds the token indices: an index outside [0, n_rows) reads as a row of zeros
 * (gather) or is skipped (scatter). */
bool llam_ql_shared_expert_gate(float *d_shared, const float *d_hidden, const float *d_gate_inp,
                                int n_tokens, int d_model, int device_id, void *stream);
bool llam_ql_moe_gather_rows(const float *d_hidden, float *d_batch, const int32_t *d_token_indices,
                             int num_tokens, int n_rows, int d_model, int device_id, void *stream);
bool llam_ql_moe_scatter_add_weighted(float *d_output, const float *d_expert_output,
                                      const int32_t *d_token_indices, const float *d_weights,
                                      int num_tokens, int n_rows, int d_model, int device_id,
                                      void *stream);
bool llam_ql_swiglu_inplace(float *d_gate, const float *d_up, long count, int device_id, void *stream);

#ifdef __cplusplus
}
#endif
#endif
