/* Where prepared weights come from and where they can be kept: a reader of GGUF files that
 * hands out the raw super-block rows of their tensors, and a small container for a matrix
 * in the prepared layout, so that a model is prepared once and re-loaded without its GGUF
 * file.  Host functions of the host library; C ABI, no device types in the signatures.
 *
 * The reader covers what the reference's loader does before a tensor reaches a kernel:
 * ModelLoader::parseHeader / parseTensorInfo and the alignment of the data section
 * (src/v2/loaders/ModelLoader.cpp:2245-2300, 2459-2530, 409; type ids ModelLoader.h:86-111).
 * The container stands where the reference serialises device-packed weights
 * (GpuPackedWeightsHeader, buildGpuPackedHeader, validateGpuPackedHeader,
 * parseGpuPackedBuffer: src/v2/loaders/gpu_pipeline/GpuPackedWeightsFormat.h:52-180): a fixed
 * 64-byte little-endian header followed by the payload, here the bytes
 * llam_ql_prepare_weights wrote, with a checksum the reference's header does not have.
 *
 * Files are untrusted input: every count, length and offset is checked against the size of
 * the file before it is used.  Functions return false / NULL on error and keep the reason
 * for llam_weights_last_error(). */
#ifndef LLAMINAR_AMD_WEIGHTS_IO_H
#define LLAMINAR_AMD_WEIGHTS_IO_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *llam_weights_last_error(void);

/* ---- GGUF ------------------------------------------------------------------------- */

typedef struct
{
    const char *name;   /* owned by the handle */
    uint32_t ggml_type; /* the file's type id: 0 F32, 1 F16, 12 Q4_K, 14 Q6_K, 21 IQ3_S, ... */
    uint8_t fmt;        /* LLAM_FMT_* when a kernel of this library reads the type, else 0 */
    uint32_t n_dims;    /* 1..4 */
    uint64_t dims[4];   /* dims[0] is the row length (K), dims[1] the number of rows (N) */
    uint64_t nbytes;    /* 0 for a type whose block size this reader does not know */
    const void *data;   /* inside the read-only mapping of the file, 32-byte aligned or as
                         * general.alignment says; valid until llam_gguf_close */
} llam_gguf_tensor;

/* Maps the file read-only and parses header, metadata and tensor directory (GGUF versions 2
 * and 3, little-endian). */
void *llam_gguf_open(const char *path);
void llam_gguf_close(void *gguf);
uint64_t llam_gguf_tensor_count(const void *gguf);
bool llam_gguf_tensor_at(const void *gguf, uint64_t index, llam_gguf_tensor *out);
bool llam_gguf_find(const void *gguf, const char *name, llam_gguf_tensor *out);
/* Scalar metadata by key: any integer or bool type as u64 (negative values are refused), any
 * float type as double, strings as a NUL-terminated copy owned by the handle (NULL if absent). */
bool llam_gguf_meta_u64(const void *gguf, const char *key, uint64_t *out);
bool llam_gguf_meta_f64(const void *gguf, const char *key, double *out);
const char *llam_gguf_meta_str(const void *gguf, const char *key);

/* ---- prepared-weights container --------------------------------------------------- */

#define LLAM_PREPARED_MAGIC 0x5750514Cu /* "LQPW" */
#define LLAM_PREPARED_VERSION 2u

typedef struct
{
    uint32_t magic;
    uint32_t version;
    uint8_t fmt;             /* LLAM_FMT_* */
    uint8_t reserved0[3];    /* zero */
    int32_t N;               /* rows */
    int32_t K;               /* columns, a multiple of 256 */
    uint32_t block_bytes;    /* bytes of one GGUF super-block of the format */
    uint64_t prepared_bytes; /* payload size = llam_ql_prepared_bytes(fmt, N, K) */
    uint64_t gguf_bytes;     /* N * K / 256 * block_bytes: the size of the source tensor */
    uint64_t checksum;       /* llam_weights_checksum of the payload */
    uint8_t reserved1[16];   /* zero */
} llam_prepared_header;      /* 64 bytes */

/* FNV-1a, 64 bit, over 8-byte little-endian words (a tail of fewer bytes is zero-padded). */
uint64_t llam_weights_checksum(const void *bytes, uint64_t n);

/* Header of a prepared fmt matrix of N x K whose payload is `payload` (host memory). */
bool llam_prepared_header_build(uint8_t fmt, int N, int K, const void *payload, llam_prepared_header *out);
/* Magic, version, format, shape and sizes are consistent and `buffer_bytes` (header +
 * payload) holds the whole payload; with verify_checksum the payload behind the header is
 * hashed as well. */
bool llam_prepared_buffer_check(const void *buffer, uint64_t buffer_bytes, bool verify_checksum);

/* Copies a prepared matrix from device memory and writes header + payload to `path`. */
bool llam_prepared_save(const char *path, uint8_t fmt, int N, int K, const void *d_prepared, int device_id);
/* Reads `path`, checks it (checksum included) and copies the payload to d_prepared, which
 * holds `capacity` bytes; *out receives the header.  With d_prepared == NULL only the
 * header is read and checked against the file size (to size the allocation). */
bool llam_prepared_load(const char *path, llam_prepared_header *out, void *d_prepared, uint64_t capacity,
                        int device_id);

#ifdef __cplusplus
}
#endif
#endif
