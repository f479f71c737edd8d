// Drop-in C++ operator interface over the C ABI (include/tllm_ternary.h).
//
// Re-declares the four ternary operators of the reference's `namespace ternary`
// (include/kernels.cuh:11-40) and the two element-wise operators next to them
// (include/kernels.cuh:45-48, 60-62) with the same names, argument order and default stream,
// so the call expressions in src/transformer.cpp:107-116, 132-142, 193-196, 201-217, 258-261,
// 266-278, 285-286 compile unchanged against this header. `half` is HIP's __half (hip/hip_fp16.h) and the
// stream is a hipStream_t. Like the reference these return void. The C ABI underneath checks what the
// reference never checked (null pointers, cols % group_size, 16-byte alignment of masks and activations,
// output overlapping the input) and REJECTS such a call without writing the output: the rejection goes
// to the handler below (default: a line on stderr) and stays readable in ternary::last_error() until the
// caller clears it, so a caller ported from the reference cannot consume a stale buffer unnoticed.
// Compile with -DTERNARY_ABORT_ON_ERROR to abort on the first rejected call instead.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <atomic>
#include <cstdio>
#include <cstdlib>

#include "tllm_ternary.h"

namespace ternary {

using error_handler_t = void (*)(const char *op, int code);

inline void default_error_handler(const char *op, int code) {
    std::fprintf(stderr, "[ternary] %s rejected: %s (%d)\n", op, tllm_error_string(code), code);
}

inline error_handler_t &error_handler() {
    static error_handler_t h = default_error_handler;
    return h;
}

// First non-zero code since the caller last set it to 0 (negative: TLLM_ERR_*, positive: hipError_t). One atomic for
// the whole process, shared by every thread and stream: the first rejected call wins (compare-and-swap from 0), later
// ones leave it alone, `ternary::last_error() = 0` clears it. A caller that needs to know WHICH call failed installs
// an error_handler, which receives the operator's name with every code.
inline std::atomic<int> &last_error() {
    static std::atomic<int> e{0};
    return e;
}

inline void report(const char *op, int code) {
    if (code == 0) return;
    int none = 0;
    last_error().compare_exchange_strong(none, code, std::memory_order_relaxed);
    if (error_handler()) error_handler()(op, code);
#ifdef TERNARY_ABORT_ON_ERROR
    std::abort();
#endif
}

// Reference include/kernels.cuh:11-14.
inline void ternary_gemv(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                         const half *scales, const half *input, half *output, int rows, int cols,
                         int group_size, hipStream_t stream = 0) {
    report("ternary_gemv",
           tllm_ternary_gemv_f16(nonzero_masks, sign_masks,
                                 reinterpret_cast<const uint16_t *>(scales),
                                 reinterpret_cast<const uint16_t *>(input),
                                 reinterpret_cast<uint16_t *>(output), rows, cols, group_size, stream));
}

// Reference include/kernels.cuh:19-24.
inline void ternary_gemv_int8(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                              const half *weight_scales, const int8_t *input_int8,
                              float input_scale, half *output, int rows, int cols, int group_size,
                              hipStream_t stream = 0) {
    report("ternary_gemv_int8",
           tllm_ternary_gemv_i8(nonzero_masks, sign_masks,
                                reinterpret_cast<const uint16_t *>(weight_scales), input_int8,
                                input_scale, reinterpret_cast<uint16_t *>(output), rows, cols,
                                group_size, stream));
}

// Reference include/kernels.cuh:30-32.
inline void quantize_absmax_int8(const half *input, int8_t *output, float *scale, int n,
                                 hipStream_t stream = 0) {
    report("quantize_absmax_int8",
           tllm_quantize_absmax_i8(reinterpret_cast<const uint16_t *>(input), output, scale, n, stream));
}

// The reference's INT8 linear as one call (no counterpart in include/kernels.cuh: there it is the member function
// Transformer::ternary_linear_int8, src/transformer.cpp:126-143, which quantises, copies the scale to the host and
// calls ternary_gemv_int8). Same result bit for bit; no int8 buffer, no scale, no copy.
inline void ternary_linear_int8(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                                const half *weight_scales, const half *input, half *output, int rows,
                                int cols, int group_size, hipStream_t stream = 0) {
    report("ternary_linear_int8",
           tllm_ternary_linear_int8_f16(nonzero_masks, sign_masks,
                                        reinterpret_cast<const uint16_t *>(weight_scales),
                                        reinterpret_cast<const uint16_t *>(input),
                                        reinterpret_cast<uint16_t *>(output), rows, cols, group_size, stream));
}

// The FFN front half of a prefill step as one call (no counterpart in include/kernels.cuh: there it is ternary_gemm on
// the gate matrix, ternary_gemm on the up matrix and silu_mul_forward, src/transformer.cpp:264-286). C = silu(A gate^T) * (A up^T).
inline void ternary_gemm_swiglu(const half *A, const uint32_t *nz_gate, const uint32_t *sign_gate, const half *scales_gate,
                                const uint32_t *nz_up, const uint32_t *sign_up, const half *scales_up, half *C, int M,
                                int N, int K, int group_size, hipStream_t stream = 0) {
    report("ternary_gemm_swiglu",
           tllm_ternary_gemm_swiglu_f16(reinterpret_cast<const uint16_t *>(A), nz_gate, sign_gate,
                                        reinterpret_cast<const uint16_t *>(scales_gate), nz_up, sign_up,
                                        reinterpret_cast<const uint16_t *>(scales_up), reinterpret_cast<uint16_t *>(C), M, N,
                                        K, group_size, stream));
}

// The q, k and v projections of a prefill step (or any `count` <= TLLM_MAX_GEMM_GROUP matrices on the same activations)
// as one launch; no counterpart in include/kernels.cuh: there it is one ternary_gemm per matrix
// (src/transformer.cpp:199-217). C[i] = A B[i]^T, the pointer arrays live in host memory.
inline void ternary_gemm_group(const half *A, const uint32_t *const *nz_B, const uint32_t *const *sign_B,
                               const half *const *scales_B, half *const *C, const int *N, int count, int M, int K,
                               int group_size, hipStream_t stream = 0) {
    report("ternary_gemm_group",
           tllm_ternary_gemm_group_f16(reinterpret_cast<const uint16_t *>(A), nz_B, sign_B,
                                       reinterpret_cast<const uint16_t *const *>(scales_B),
                                       reinterpret_cast<uint16_t *const *>(C), N, count, M, K, group_size, stream));
}

// Reference include/kernels.cuh:37-40.
inline void ternary_gemm(const half *A, const uint32_t *nz_B, const uint32_t *sign_B,
                         const half *scales_B, half *C, int M, int N, int K, int group_size,
                         hipStream_t stream = 0) {
    report("ternary_gemm",
           tllm_ternary_gemm_f16(reinterpret_cast<const uint16_t *>(A), nz_B, sign_B,
                                 reinterpret_cast<const uint16_t *>(scales_B),
                                 reinterpret_cast<uint16_t *>(C), M, N, K, group_size, stream));
}

// Reference include/kernels.cuh:45-48.
inline void rmsnorm_forward(const half *input, const half *weight, half *output, const half *residual,
                            half *residual_out, int batch, int dim, float eps, hipStream_t stream = 0) {
    report("rmsnorm_forward",
           tllm_rmsnorm_f16(reinterpret_cast<const uint16_t *>(input), reinterpret_cast<const uint16_t *>(weight),
                            reinterpret_cast<uint16_t *>(output), reinterpret_cast<const uint16_t *>(residual),
                            reinterpret_cast<uint16_t *>(residual_out), batch, dim, eps, stream));
}

// Reference include/kernels.cuh:60-62.
inline void silu_mul_forward(const half *gate, const half *up, half *output, int size, hipStream_t stream = 0) {
    report("silu_mul_forward",
           tllm_silu_mul_f16(reinterpret_cast<const uint16_t *>(gate), reinterpret_cast<const uint16_t *>(up),
                             reinterpret_cast<uint16_t *>(output), size, stream));
}

// Reference include/kernels.cuh:50-53.
inline void rope_forward(half *q, half *k, int batch, int seq_len, int n_heads, int n_kv_heads, int head_dim,
                         int start_pos, float theta, hipStream_t stream = 0) {
    report("rope_forward", tllm_rope_f16(reinterpret_cast<uint16_t *>(q), reinterpret_cast<uint16_t *>(k), batch, seq_len,
                                         n_heads, n_kv_heads, head_dim, start_pos, theta, stream));
}

// Reference include/kernels.cuh:64-66.
inline void add_forward(const half *a, const half *b, half *output, int size, hipStream_t stream = 0) {
    report("add_forward", tllm_add_f16(reinterpret_cast<const uint16_t *>(a), reinterpret_cast<const uint16_t *>(b),
                                       reinterpret_cast<uint16_t *>(output), size, stream));
}

// Reference include/kernels.cuh:68-70.
inline void embedding_lookup(const half *table, const int *indices, half *output, int n_tokens, int dim,
                             hipStream_t stream = 0) {
    report("embedding_lookup", tllm_embedding_lookup_f16(reinterpret_cast<const uint16_t *>(table), indices,
                                                         reinterpret_cast<uint16_t *>(output), n_tokens, dim, stream));
}

// Reference include/kernels.cuh:72-76.
inline void copy_to_kv_cache(const half *k, const half *v, half *k_cache, half *v_cache, int batch, int n_kv_heads,
                             int head_dim, int seq_len, int start_pos, int max_seq_len, hipStream_t stream = 0) {
    report("copy_to_kv_cache",
           tllm_copy_to_kv_cache_f16(reinterpret_cast<const uint16_t *>(k), reinterpret_cast<const uint16_t *>(v),
                                     reinterpret_cast<uint16_t *>(k_cache), reinterpret_cast<uint16_t *>(v_cache), batch,
                                     n_kv_heads, head_dim, seq_len, start_pos, max_seq_len, stream));
}

}  // namespace ternary
