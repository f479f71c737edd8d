/*
 * C ABI of the host-side pieces on either side of the ternary operators: the ternarise+pack
 * producer and the .tllm model file reader / synthetic writer.
 *
 * Everything here runs on the HOST except tllm_model_file_upload, which copies the ternary weight
 * arrays of a file into ONE caller-provided device buffer (the reference loader makes one
 * cudaMalloc + cudaMemcpy per array, reference src/model.cpp:19-43, 46-60).
 * Return values as in tllm_ternary.h: 0, a negative TLLM_ERR_* code, or a positive hipError_t.
 */
#ifndef TLLM_MODEL_FILE_H
#define TLLM_MODEL_FILE_H

#include <stddef.h>
#include <stdint.h>

#include "tllm_ternary.h"

#ifdef __cplusplus
extern "C" {
#endif

enum {
    TLLM_ERR_IO = -8,        /* file cannot be opened, is truncated, or a write failed */
    TLLM_ERR_BAD_FILE = -9   /* bad magic / version, or a header field out of range */
};

/*
 * Ternarise a row-major fp32 matrix [rows, cols] and pack it into the dual-bitmask layout.
 * Per group of `group_size` consecutive columns of a row: threshold = threshold_factor *
 * mean|w|; w > threshold -> +1, w < -threshold -> -1, else 0; scale = mean|w| over the non-zero
 * entries (0 for an all-zero group), stored as fp16 (round to nearest even).
 * Replaces ternarize_tensor + pack_ternary_to_bitmasks, reference ternarize/pack.py:41-101,
 * 120-169 (the reference's default threshold_factor is 0.7). Sums are taken in fp32 in column
 * order (the reference sums in torch's order; on the seeded tensors of its own packing test,
 * tests/test_packing.py:92-111 and 141-173, masks and fp16 scales agree bit for bit). cols % group_size must be 0 and group_size % 32 must be 0 (the reference pads the input
 * dimension to a multiple of 32 with zero weights, pack.py:24-34; here the caller passes padded
 * matrices). Outputs are HOST arrays: nonzero_masks / sign_masks uint32 [rows, cols/32] (the sign
 * bit of a zero weight is written as 0), scales fp16 bits [rows, cols/group_size].
 */
int tllm_ternarize_pack_f32(const float *weight, int rows, int cols, int group_size,
                            float threshold_factor, uint32_t *nonzero_masks, uint32_t *sign_masks,
                            uint16_t *scales);

/* The 256-byte on-disk header (reference include/format.h:20-37), little endian. */
typedef struct tllm_file_header {
    uint32_t magic;   /* 0x544C4C4D */
    uint32_t version; /* 1 */
    uint32_t arch;    /* 0 = llama, 1 = mistral */
    uint32_t vocab_size;
    uint32_t hidden_dim;
    uint32_t intermediate_dim;
    uint32_t n_layers;
    uint32_t n_heads;
    uint32_t n_kv_heads;
    uint32_t max_seq_len;
    uint32_t head_dim;
    uint32_t rope_theta_bits; /* float bits */
    uint32_t group_size;
    uint32_t rms_norm_eps_bits; /* float bits */
    uint32_t flags;             /* bit 0: lm_head is ternary */
    uint8_t reserved[256 - 15 * 4];
} tllm_file_header;

/* One ternary linear of a model file. Offsets are in bytes; *_file from the start of the file,
 * *_pool from the start of the device pool (each array starts on a 256-byte boundary). */
typedef struct tllm_file_linear {
    uint64_t nonzero_file, sign_file, scales_file;
    uint64_t nonzero_pool, sign_pool, scales_pool;
    int32_t rows;  /* out_features */
    int32_t cols;  /* in_features, padded to a multiple of 32 as stored */
    int32_t layer; /* decoder layer, or -1 for the lm_head */
    int32_t kind;  /* 0 q, 1 k, 2 v, 3 o, 4 gate, 5 up, 6 down, 7 lm_head */
} tllm_file_linear;

typedef struct tllm_model_file tllm_model_file;

/*
 * Opens a .tllm file, validates the header and lays out its arrays in file order (reference
 * src/model.cpp:72-212: header, fp16 embedding table, per layer q k v o gate up down as
 * (nonzero, sign, scales) triples followed by the two fp16 norm vectors, final norm, lm_head,
 * tokenizer blob). Touches no GPU.
 */
int tllm_model_file_open(const char *path, tllm_model_file **file);
void tllm_model_file_close(tllm_model_file *file);
int tllm_model_file_header(const tllm_model_file *file, tllm_file_header *header);
/* Number of ternary linears: 7 per layer, plus the lm_head when it is ternary. */
int tllm_model_file_linear_count(const tllm_model_file *file);
int tllm_model_file_linear(const tllm_model_file *file, int index, tllm_file_linear *out);
/* Bytes of the device pool that holds every ternary array of the file. */
uint64_t tllm_model_file_pool_bytes(const tllm_model_file *file);
/*
 * Reads the ternary arrays and copies them into `device_pool` (DEVICE pointer, at least
 * tllm_model_file_pool_bytes, 256-byte aligned) through a pinned staging buffer; returns after
 * the copies have completed. Allocates only the pinned staging buffer (freed before returning).
 */
int tllm_model_file_upload(const tllm_model_file *file, void *device_pool, uint64_t pool_bytes,
                           tllm_stream_t stream);
/* Fills the weight pointers, rows and cols of `problem` for linear `index` inside `device_pool`;
 * input, output and batch are left to the caller. */
int tllm_model_file_problem(const tllm_model_file *file, int index, void *device_pool,
                            tllm_linear_problem *problem);

/*
 * Writes a synthetic model in the .tllm format: fp32 weights drawn N(0, 0.02^2) from a seeded
 * generator are ternarised with tllm_ternarize_pack_f32 (threshold factor 0.7), the fp16 tables are
 * small random values, the tokenizer blob is empty. `header` supplies the dimensions (magic and
 * version are filled in; hidden_dim, n_heads*head_dim and intermediate_dim must be multiples of
 * group_size). Counterpart of the reference's writer, ternarize/ternarize.py:73-111, 254-349,
 * for tests and benchmarks without a checkpoint.
 */
int tllm_model_file_write_synthetic(const char *path, const tllm_file_header *header, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif /* TLLM_MODEL_FILE_H */
