/*
 * GGUF block layouts on the quantized-linear path.  Plain C PODs, usable from
 * C, C++ and HIP device code.  Byte-for-byte identical to the reference's
 * structs so raw GGUF tensor bytes (and Q8_1 activation buffers) can be handed
 * across the boundary unchanged:
 *
 *   llam_block_q8_1  <-> Q8_1Block   src/v2/tensors/BlockStructures.h:69-76
 *   llam_block_q4_K  <-> Q4_KBlock   src/v2/tensors/BlockStructures.h:461-469
 *   llam_block_q6_K  <-> Q6_KBlock   src/v2/tensors/BlockStructures.h:484-492
 *   llam_block_iq3_s <-> IQ3_SBlock  src/v2/tensors/BlockStructures.h:547-556
 */
#ifndef LLAMINAR_AMD_QL_BLOCKS_H
#define LLAMINAR_AMD_QL_BLOCKS_H

#include <stdint.h>

#define LLAM_QK8_1 32   /* elements per Q8_1 activation block            */
#define LLAM_QK_K 256   /* elements per K-quant / IQ weight super-block  */

/* Activation block: d is IEEE binary16 bits; sum_qs is the RAW integer sum of
 * qs[] (not d*sum). */
typedef struct
{
    uint16_t d;
    int16_t sum_qs;
    int8_t qs[LLAM_QK8_1];
} llam_block_q8_1;

/* 4-bit K-quant: 8 sub-blocks of 32; 6-bit (scale,min) pairs packed in scales[12]. */
typedef struct
{
    uint16_t d;
    uint16_t dmin;
    uint8_t scales[12];
    uint8_t qs[128];
} llam_block_q4_K;

/* 6-bit K-quant: 16 sub-blocks of 16 with int8 scales. */
typedef struct
{
    uint8_t ql[128];
    uint8_t qh[64];
    int8_t scales[16];
    uint16_t d;
} llam_block_q6_K;

/* 3-bit codebook quant: 9-bit indices (qs + one bit of qh) into llam_iq3s_grid. */
typedef struct __attribute__((packed))
{
    uint16_t d;
    uint8_t qs[64];
    uint8_t qh[8];
    uint8_t signs[32];
    uint8_t scales[4];
} llam_block_iq3_s;

#ifdef __cplusplus
static_assert(sizeof(llam_block_q8_1) == 36, "Q8_1 block is 36 bytes");
static_assert(sizeof(llam_block_q4_K) == 144, "Q4_K block is 144 bytes");
static_assert(sizeof(llam_block_q6_K) == 210, "Q6_K block is 210 bytes");
static_assert(sizeof(llam_block_iq3_s) == 110, "IQ3_S block is 110 bytes");
#else
_Static_assert(sizeof(llam_block_q8_1) == 36, "Q8_1 block is 36 bytes");
_Static_assert(sizeof(llam_block_q4_K) == 144, "Q4_K block is 144 bytes");
_Static_assert(sizeof(llam_block_q6_K) == 210, "Q6_K block is 210 bytes");
_Static_assert(sizeof(llam_block_iq3_s) == 110, "IQ3_S block is 110 bytes");
#endif

/* Weight formats this library multiplies.  The numeric values are the
 * "codebook_id" kernel-dispatch ids the reference's launchers take for the same
 * formats (NativeVnniFormatInfo::codebook_id: Q4_K src/v2/tensors/TensorClasses.h:6223,
 * Q6_K :5530, IQ3_S :7608). */
typedef enum
{
    LLAM_FMT_Q4_K = 5,
    LLAM_FMT_Q6_K = 8,
    LLAM_FMT_IQ3_S = 11
} llam_weight_format;

static inline int llam_format_block_bytes(int fmt)
{
    switch (fmt)
    {
    case LLAM_FMT_Q4_K: return 144;
    case LLAM_FMT_Q6_K: return 210;
    case LLAM_FMT_IQ3_S: return 110;
    default: return 0;
    }
}

#endif
