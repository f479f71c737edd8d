/*
 * C ABI of the MI355X ternary linear-layer operators.
 *
 * Weight layout (the .tllm dual-bitmask layout, reference include/model.h:17-36):
 *   nonzero_masks  uint32 [rows, cols/32]   bit b of word j of row r <-> w[r, 32*j+b] != 0
 *   sign_masks     uint32 [rows, cols/32]   same position, 1 <-> w > 0; ignored where nz bit is 0
 *   scales         fp16   [rows, cols/group_size], one per `group_size` consecutive columns
 * fp16 values cross this boundary as IEEE binary16 bit patterns (uint16_t).
 * Every pointer is a borrowed DEVICE pointer unless said otherwise; the three weight
 * arrays may live in separate allocations. Calls are asynchronous on `stream`.
 *
 * Return value: 0 on success; a negative TLLM_ERR_* code when the arguments are
 * rejected before anything is launched; a positive value is a hipError_t from the
 * launch. (The reference operators return void and check nothing; this is a strict
 * superset. Unlike the reference, cols % group_size != 0 is rejected, not truncated.)
 */
#ifndef TLLM_TERNARY_H
#define TLLM_TERNARY_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *tllm_stream_t; /* a hipStream_t; NULL is the default stream */

enum {
    TLLM_OK = 0,
    TLLM_ERR_NULL_POINTER = -1, /* a required pointer is NULL */
    TLLM_ERR_BAD_SHAPE = -2,    /* rows/cols/M/N/K/n < 1, or cols % 32 != 0 */
    TLLM_ERR_BAD_GROUP = -3,    /* group_size < 32, group_size % 32 != 0 or cols % group_size != 0 */
    TLLM_ERR_TOO_LARGE = -4,    /* an element count does not fit the index type, or exceeds a stated limit */
    TLLM_ERR_ALIAS = -5,        /* output overlaps the activation input */
    TLLM_ERR_BAD_PLAN = -6,     /* plan handle is NULL, count < 1, batch out of range, or a pair / prologue rule is broken */
    TLLM_ERR_MISALIGNED = -7,   /* masks/activations not 16-byte aligned, scales/outputs not 2-byte aligned */
    /* -8 and -9 belong to tllm_model_file.h */
    TLLM_ERR_SCRATCH_TOO_SMALL = -10, /* tllm_ternary_gemm_f16_static: the shape needs more exchange memory than the fixed scratch */
    TLLM_ERR_STAGE_TIMEOUT = -11      /* tllm_linear_plan_status: a launch of a staged plan gave up waiting between two stages */
};

/* Human-readable text for a negative TLLM_ERR_* code (host pointer, static storage). */
const char *tllm_error_string(int code);

/* ABI revision of this header. */
int tllm_abi_version(void);

/*
 * y[r] = fp16( sum_g float(scales[r,g]) * sum_{k in g} w[r,k] * float(input[k]) ),  fp32 accumulation.
 * Replaces ternary::ternary_gemv, reference include/kernels.cuh:11-14
 * (kernels/ternary_gemv.cu:27-100). input fp16 [cols], output fp16 [rows].
 * Inf, NaN and outliers in `input` (group_size 128, the matrix-core kernels; the same holds for the int8 variant,
 * tllm_ternary_gemm_f16 with M <= 16 and the plans): as in the reference, which adds term by term
 * (kernels/ternary_gemv.cu:60-82), a non-finite activation makes exactly the rows non-finite that hold a non-zero
 * weight on its column, and an activation of any magnitude leaves the accuracy of the rows that hold none
 * untouched. (The kernels meet weights and activations in a matrix multiply, where every activation enters the
 * fp32 sums of every row; an activation that is non-finite, or more than 2^8 times the typical magnitude of its
 * 128-column group, is therefore kept out of the operand and added afterwards, scale * w * x in fp32, to the rows
 * that hold a weight there.) Limit: a workgroup holds 64 such activations per vector (128 for all activation rows
 * of a 2..16-row call together); further ones stay inside the matrix operand, where a finite one costs the rows
 * that do not use it about 2^-21 of its magnitude and a non-finite one makes every output of that activation row
 * non-finite.
 */
int tllm_ternary_gemv_f16(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                          const uint16_t *scales, const uint16_t *input, uint16_t *output,
                          int rows, int cols, int group_size, tllm_stream_t stream);

/*
 * y[r] = fp16( input_scale * sum_g float(weight_scales[r,g]) * float(sum_{k in g} w[r,k] * input_int8[k]) ).
 * Replaces ternary::ternary_gemv_int8, reference include/kernels.cuh:19-24
 * (kernels/ternary_gemv.cu:116-216). `input_scale` is passed by value from the host,
 * as the reference does.
 */
int tllm_ternary_gemv_i8(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                         const uint16_t *weight_scales, const int8_t *input_int8,
                         float input_scale, uint16_t *output, int rows, int cols, int group_size,
                         tllm_stream_t stream);

/*
 * The reference's whole INT8 linear in one launch: absmax-quantises the fp16 `input` (as tllm_quantize_absmax_i8
 * does) inside the GEMV and multiplies (as tllm_ternary_gemv_i8 does); `output` holds, bit for bit, what the two
 * calls store. No int8 buffer, no scale, no device-to-host copy. Replaces Transformer::ternary_linear_int8,
 * reference src/transformer.cpp:126-143 (kernels/activations.cu:88-151 + kernels/ternary_gemv.cu:116-216).
 */
int tllm_ternary_linear_int8_f16(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                                 const uint16_t *weight_scales, const uint16_t *input, uint16_t *output,
                                 int rows, int cols, int group_size, tllm_stream_t stream);

/*
 * Same as tllm_ternary_gemv_i8 but reads the activation scale from DEVICE memory
 * (the float written by tllm_quantize_absmax_i8), so a decode step needs no
 * device-to-host copy between the two calls. No counterpart in the reference, which
 * copies the scale to the host first (src/transformer.cpp:134-142).
 */
int tllm_ternary_gemv_i8_dscale(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                                const uint16_t *weight_scales, const int8_t *input_int8,
                                const float *input_scale_device, uint16_t *output, int rows,
                                int cols, int group_size, tllm_stream_t stream);

/*
 * absmax = max|input|; *scale = absmax > 0 ? absmax/127 : 1;
 * output[i] = clamp(rint(input[i] * (127/absmax)), -127, 127)  (0 when absmax is 0).
 * Replaces ternary::quantize_absmax_int8, reference include/kernels.cuh:30-32
 * (kernels/activations.cu:88-151). `scale` is a device pointer to one float.
 */
int tllm_quantize_absmax_i8(const uint16_t *input, int8_t *output, float *scale, int n,
                            tllm_stream_t stream);

/*
 * C[m,n] = fp16( sum_k float(scales_B[n, k/group]) * w[n,k] * float(A[m,k]) ),  fp32 accumulation.
 * A fp16 [M,K] row-major, packed weight [N,K], C fp16 [M,N] row-major.
 * Replaces ternary::ternary_gemm, reference include/kernels.cuh:37-40
 * (kernels/ternary_gemm.cu:33-195). Any M >= 1 is accepted.
 * Allocation: none per call, with one exception: a workspace that belongs to (device, stream). Two kinds
 * of shapes use it. Shapes whose output tiles do not fill the chip, or not its last round (M > 16), split K
 * over several workgroups per tile, which exchange fp32 partial sums through it (at most 32 MiB); so do shapes
 * of 2 to 16 activation rows (and wider ones that run as passes of 16) with so few weight rows that their
 * 64-row blocks would leave half the chip idle (N <= 64 * CUs / 2, K >= 4096: at most 1 MiB). The first such call on a stream creates
 * the workspace: ONE allocation of TLLM_GEMM_STATIC_SCRATCH_BYTES (the most any shape is allowed to need: the kernel
 * choice works under that limit), with its arrival counters cleared before the call returns (one device
 * synchronisation, that once). It is never grown, moved or freed afterwards, except by tllm_gemm_workspace_release:
 * a graph captured on the stream keeps pointing at valid memory whatever shapes run on the stream later.
 * tllm_gemm_workspace_reserve creates it ahead of time. While `stream` is being captured into a graph
 * nothing is allocated: a call whose stream has no workspace yet then runs the kernel that needs
 * none (same result up to the order of the fp32 additions, slower). Calls that use one stream's workspace
 * must not overlap in time: replays of a captured graph on another stream count as calls on the stream
 * the graph was captured on.
 */
int tllm_ternary_gemm_f16(const uint16_t *A, const uint32_t *nz_B, const uint32_t *sign_B,
                          const uint16_t *scales_B, uint16_t *C, int M, int N, int K,
                          int group_size, tllm_stream_t stream);

/*
 * Up to TLLM_MAX_GEMM_GROUP weight matrices on the SAME activations in one launch: C[i][m, n] = fp16(A[m, :] . row n of
 * matrix i), what `count` calls of tllm_ternary_gemm_f16 store (reference src/transformer.cpp:199-217 at n_tokens > 1:
 * ternary_linear on q_proj, k_proj and v_proj with the same hidden_buf_). The tiles of all matrices are dealt to the
 * workgroups together, so three small matrices fill the chip where each alone leaves most of it idle. nz, sign,
 * scales, C and N are HOST arrays of `count` entries (device pointers / row counts); every matrix is [N[i], K] in the
 * packed layout, every output [M, N[i]], no two outputs overlapping. Same arithmetic as tllm_ternary_gemm_f16 in its
 * row-split kernel (fp32 accumulation; tiles that do not fill the last round over the CUs are split along K through
 * the stream's workspace, like there: tllm_gemm_workspace_reserve(M, 256 * sum over i of ceil(N[i] / 256), K, ...)
 * reserves it; under graph capture without it the tiles run whole). group_size 128; K a multiple of 256, or of 128 from
 * 384 on (another K: TLLM_ERR_BAD_SHAPE, another group size: TLLM_ERR_BAD_GROUP; issue the calls one by one then); count
 * outside 1 .. TLLM_MAX_GEMM_GROUP: TLLM_ERR_BAD_SHAPE; outputs that overlap each other or A: TLLM_ERR_ALIAS.
 */
enum { TLLM_MAX_GEMM_GROUP = 4 };
int tllm_ternary_gemm_group_f16(const uint16_t *A, const uint32_t *const *nz, const uint32_t *const *sign,
                                const uint16_t *const *scales, uint16_t *const *C, const int *N, int count, int M, int K,
                                int group_size, tllm_stream_t stream);

/*
 * The FFN front half of a prefill step in ONE launch: C[m, n] = fp16( silu(g) * u ) with g = fp16(A[m, :] . gate row n),
 * u = fp16(A[m, :] . up row n), i.e. what tllm_ternary_gemm_f16 on the gate matrix, tllm_ternary_gemm_f16 on the up
 * matrix and tllm_silu_mul_f16 store (reference src/transformer.cpp:264-286 at n_tokens > 1: ternary_linear(gate),
 * ternary_linear(up), silu_mul_forward). A workgroup multiplies one tile of the activations with the same 128 rows of
 * both matrices, so the activations are fetched once and the two M x N intermediates are never written. Same arithmetic
 * as tllm_ternary_gemm_f16 (fp32 accumulation; the order of the additions is that of its row-split kernel in the
 * four-wave form). Both matrices are [N, K] in the packed layout; group_size 128; K a multiple of 256, or of 128 from
 * 384 on (else TLLM_ERR_BAD_SHAPE / TLLM_ERR_BAD_GROUP: issue the three launches); A and the mask planes 16-byte aligned.
 * Any M >= 1 (for M = 1 the decode plans with TLLM_PROBLEM_SWIGLU_GATE are the faster form). Allocation-free.
 */
int tllm_ternary_gemm_swiglu_f16(const uint16_t *A, const uint32_t *nz_gate, const uint32_t *sign_gate,
                                 const uint16_t *scales_gate, const uint32_t *nz_up, const uint32_t *sign_up,
                                 const uint16_t *scales_up, uint16_t *C, int M, int N, int K, int group_size,
                                 tllm_stream_t stream);

/*
 * tllm_ternary_gemm_f16 for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc): same arguments, same kernels, same results bit for
 * bit, but the workspace (the split-K exchange) is a fixed array of
 * TLLM_GEMM_STATIC_SCRATCH_BYTES in device memory that the library holds on every GPU it runs on until
 * the process ends. The call never allocates, frees or synchronises. Both entry points choose their kernel among those whose workspace
 * fits the array (a split needs at most CUs * 128 KiB),
 * so on a 256-CU MI355X every shape runs; a configuration that would not fit is rejected with
 * TLLM_ERR_SCRATCH_TOO_SMALL before anything is launched. All calls on one GPU share the one
 * array: calls that overlap in time on one GPU (two streams, two threads, two graph branches) race on it;
 * issue them on one stream, or use tllm_ternary_gemm_f16 with its per-stream workspaces.
 * No counterpart in the reference, whose GEMM needs no exchange memory.
 */
#define TLLM_GEMM_STATIC_SCRATCH_BYTES (32 * 1024 * 1024 + 4096)
int tllm_ternary_gemm_f16_static(const uint16_t *A, const uint32_t *nz_B, const uint32_t *sign_B,
                                 const uint16_t *scales_B, uint16_t *C, int M, int N, int K,
                                 int group_size, tllm_stream_t stream);

/*
 * Name of the kernel tllm_ternary_gemm_f16 runs for a shape on the current device (static string, "" for a
 * shape the entry point would reject; for reports and profiles: the choice depends on M, N, K and the
 * number of CUs). No counterpart in the reference.
 */
const char *tllm_ternary_gemm_kernel(int M, int N, int K, int group_size);

/*
 * Creates the workspace of `stream` if the GEMM shape (M, N, K) uses one and the stream has none yet, so that
 * later tllm_ternary_gemm_f16 calls on that stream allocate nothing, e.g. before capturing them into a graph
 * (the workspace has one size, so reserving for any shape that needs it serves every shape). May synchronise
 * the device, once per stream. No counterpart in the reference (its GEMM needs no workspace).
 * tllm_gemm_workspace_release frees every workspace of the process: no GEMM call may be in flight, and a
 * graph that was captured with a call that used a workspace must not be replayed afterwards (it holds the
 * freed address): destroy such graphs first, or never release.
 */
int tllm_gemm_workspace_reserve(int M, int N, int K, int group_size, tllm_stream_t stream);
void tllm_gemm_workspace_release(void);

/*
 * output[b, i] = fp16( t[b, i] / sqrt(mean_i t[b, i]^2 + eps) * weight[i] ),  t = input (+ residual), fp32.
 * residual may be NULL; residual_out, when given (with a residual), receives fp16(t) and the
 * normalised output is then computed from that rounded value, as the reference does.
 * Replaces ternary::rmsnorm_forward, reference include/kernels.cuh:45-48 (kernels/rmsnorm.cu:20-127):
 * the operator in front of every projection group (src/transformer.cpp:193-196, 258-261).
 */
int tllm_rmsnorm_f16(const uint16_t *input, const uint16_t *weight, uint16_t *output,
                     const uint16_t *residual, uint16_t *residual_out, int batch, int dim, float eps,
                     tllm_stream_t stream);

/*
 * output[i] = fp16( gate[i] / (1 + exp(-gate[i])) * up[i] ), fp32 arithmetic.
 * Replaces ternary::silu_mul_forward, reference include/kernels.cuh:60-62
 * (kernels/activations.cu:18-74): the operator between the gate/up and the down projection.
 */
int tllm_silu_mul_f16(const uint16_t *gate, const uint16_t *up, uint16_t *output, int size,
                      tllm_stream_t stream);

/*
 * output[i] = a[i] + b[i], one correctly rounded fp16 addition per element; output may be a or b.
 * Replaces ternary::add_forward, reference include/kernels.cuh:64-66 (kernels/elementwise.cu:18-48),
 * the residual add of src/transformer.cpp.
 */
int tllm_add_f16(const uint16_t *a, const uint16_t *b, uint16_t *output, int size, tllm_stream_t stream);

/*
 * Rotary position embedding, in place: q is fp16 [batch, seq_len, n_heads, head_dim], k is
 * [batch, seq_len, n_kv_heads, head_dim]; the pair (2i, 2i+1) of every head of token (b, s) is
 * rotated by the angle (start_pos + s) * theta^(-2i / head_dim):
 *   (x0, x1) -> (x0 cos - x1 sin, x0 sin + x1 cos), fp32 arithmetic, fp16 store.
 * head_dim must be even. The angle, its sine and cosine are evaluated in fp64 and rounded to fp32
 * (the reference evaluates them in fp32, which leaves the angle off by up to pos * 2^-23 rad).
 * Replaces ternary::rope_forward, reference include/kernels.cuh:50-53 (kernels/rope.cu:22-104).
 */
int tllm_rope_f16(uint16_t *q, uint16_t *k, int batch, int seq_len, int n_heads, int n_kv_heads,
                  int head_dim, int start_pos, float theta, tllm_stream_t stream);

/*
 * output[t, :] = table[indices[t], :] for t < n_tokens; rows of dim fp16 values, indices are int32
 * on the device and are not range-checked (the operator does not know the table's height).
 * Replaces ternary::embedding_lookup, reference include/kernels.cuh:68-70
 * (kernels/elementwise.cu:54-89).
 */
int tllm_embedding_lookup_f16(const uint16_t *table, const int32_t *indices, uint16_t *output,
                              int n_tokens, int dim, tllm_stream_t stream);

/*
 * Copies the new rows k, v [batch, seq_len, n_kv_heads, head_dim] into the caches
 * [batch, n_kv_heads, max_seq_len, head_dim] at positions start_pos .. start_pos + seq_len - 1;
 * positions at or beyond max_seq_len are dropped, as in the reference.
 * Replaces ternary::copy_to_kv_cache, reference include/kernels.cuh:72-76
 * (kernels/elementwise.cu:97-147).
 */
int tllm_copy_to_kv_cache_f16(const uint16_t *k, const uint16_t *v, uint16_t *k_cache,
                              uint16_t *v_cache, int batch, int n_kv_heads, int head_dim,
                              int seq_len, int start_pos, int max_seq_len, tllm_stream_t stream);

/*
 * Several independent ternary linears in ONE launch (e.g. q/k/v, gate/up, or a whole
 * back-to-back projection sweep). Each problem is what one tllm_ternary_gemv_f16 /
 * small-M tllm_ternary_gemm_f16 call would take: input fp16 [batch, cols],
 * output fp16 [batch, rows]. The reference issues these as separate launches
 * (src/transformer.cpp:206-217, 266-278).
 */
typedef struct tllm_linear_problem {
    const uint32_t *nonzero_masks;
    const uint32_t *sign_masks;
    const uint16_t *scales;
    const uint16_t *input;
    uint16_t *output;
    int32_t rows;
    int32_t cols;
    int32_t batch; /* 1..TLLM_MAX_PLAN_BATCH */
    int32_t flags; /* 0 or any of TLLM_PROBLEM_SWIGLU_GATE, TLLM_PROBLEM_QUANTIZE_INPUT */
} tllm_linear_problem;

enum { TLLM_MAX_PLAN_BATCH = 16 };

/*
 * Flag of a problem that is the GATE projection of a SwiGLU pair. The next problem of the array must
 * then be the UP projection: same rows, cols, batch (1 only) and input. The pair is computed together
 * and ONE result is stored, in the gate problem's output:
 *   output[b, r] = fp16( silu(g) * u ),  g = fp16(gate row r . x_b),  u = fp16(up row r . x_b),
 * i.e. exactly what the two projections followed by tllm_silu_mul_f16 store (the up problem's output
 * pointer is not written and may be NULL). Replaces the three launches of the reference's FFN front
 * half, src/transformer.cpp:266-286 (gate GEMV, up GEMV, silu_mul_forward).
 */
enum { TLLM_PROBLEM_SWIGLU_GATE = 1 };

/*
 * Flag of a problem whose fp16 input the launch quantises to int8 itself before it multiplies (batch 1): the output
 * is what tllm_quantize_absmax_i8 followed by tllm_ternary_gemv_i8_dscale stores for that matrix, bit for bit, without
 * the int8 vector and its scale ever being written. Replaces the reference's ternary_linear_int8
 * (src/transformer.cpp:126-143: quantise, copy the scale to the host, int8 GEMV) for every linear of a group in one
 * launch. It combines with the other two fusions in the order of the reference's INT8 decode step
 * (src/transformer.cpp:193-217, 258-286): behind an RMSNorm prologue the normalised, fp16-rounded row is what gets
 * quantised (rmsnorm_forward, then quantize_absmax_int8, then the projections that share the int8 vector); on the gate
 * problem of a SwiGLU pair both halves multiply the same quantised row and the epilogue stores silu(gate) * up of the
 * two fp16-rounded INT8 results (the up problem carries no flag of its own).
 */
enum { TLLM_PROBLEM_QUANTIZE_INPUT = 2 };

typedef struct tllm_linear_plan tllm_linear_plan;

/* Validates and copies `problems` (HOST array) into a device-resident schedule.
 * Allocates device memory; not for the per-token path. group_size must be 128. */
int tllm_linear_plan_create(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                            int count, int group_size);
/*
 * The same with an RMSNorm prologue: where norm_weights[i] is not NULL, problem i reads its input
 * through   x' = fp16( x / sqrt(mean(x^2) + eps) * norm_weights[i] )   (fp32 arithmetic, the sums taken
 * in the order of tllm_rmsnorm_f16, whose output it reproduces bit for bit when cols is a multiple of
 * 2048), so the normalised vector is never written to memory. Such problems need batch 1 and
 * cols <= 16384; both halves of a SwiGLU pair carry the same weights. norm_weights is a HOST array of
 * `count` DEVICE pointers (fp16 [cols], 16-byte aligned). Replaces the rmsnorm_forward launch in
 * front of each projection group, reference src/transformer.cpp:193-196, 258-261.
 */
int tllm_linear_plan_create_normed(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                                   const uint16_t *const *norm_weights, float eps, int count,
                                   int group_size);
/*
 * The same on INT8 activations: problem i's `input` points at int8 [cols] (cast to the field's type; 16-byte
 * aligned) and input_scales[i] (HOST array of `count` DEVICE pointers) at the float tllm_quantize_absmax_i8
 * wrote for that vector; batch 1, flags 0. Every output is what tllm_ternary_gemv_i8_dscale gives for that
 * matrix, bit for bit:
 *   output[r] = fp16( *input_scales[i] * sum_g float(scales[r,g]) * float(sum_{k in g} w[r,k] * input_int8[k]) ).
 * One launch then replaces the ternary_gemv_int8 calls of a decode step that do not depend on each other
 * (reference src/transformer.cpp:132-142 per linear, 199-217 and 264-278 for the groups). Shapes that the
 * matrix-core kernel does not serve (cols below 512 or not a multiple of 128) are rejected with
 * TLLM_ERR_BAD_PLAN: issue those with tllm_ternary_gemv_i8.
 */
int tllm_linear_plan_create_i8(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                               const float *const *input_scales, int count, int group_size);
/*
 * A plan whose problems DEPEND on each other, run in stages inside ONE launch: stages[i] (HOST array, ascending from 0,
 * at most 8 stages) says after which problems problem i runs; the problems of one stage are independent, and every
 * problem of stage s + 1 may read what stage s stored. The kernel does not end between two stages. How a stage gets
 * the results of the stage before, chosen when the plan is created:
 *   - as tagged words (the usual case): a problem whose output a later stage reads also stores every output row as a
 *     32-bit word (fp16 bits and a tag of the launch) in memory the plan owns; the workgroups that need it poll those
 *     words and take the values from them, so each waits for exactly the data it needs. This needs buffers that
 *     relate plainly: an input or residual is either exactly one earlier stage's output (same pointer, same length)
 *     or touches no output of the plan (a residual may be its own problem's output: in place); two outputs are
 *     either the same buffer in different stages (the reference's residual stream, updated in place twice) or do
 *     not overlap; a buffer that a later stage overwrites is only overwritten by a problem that depends, through
 *     such hand-overs, on every problem that reads or writes it earlier; rows of at most 16384 columns, at most
 *     64 problems.
 *   - otherwise at a barrier in device memory between every two stages (counters, bounded polling), after which
 *     the outputs of the stage before are read from memory, not from a stale cache line.
 * tllm_linear_plan_kernel names the way a plan runs. Either way the launches of a decode step that depend on each
 * other become one, reference src/transformer.cpp:239-296, e.g.
 *   stage 0  o_proj, residuals[0] = the residual stream (output = stream + projection, in place allowed)
 *   stage 1  gate / up as a SwiGLU pair with norm_weights = the FFN norm: reads the stream through RMSNorm
 *   stage 2  down_proj on the pair's output, residuals = the stream again
 *   stage 3  q / k / v of the next layer with that layer's attention norm
 * Every output equals, bit for bit, what the separate launches store (tllm_ternary_gemv_f16, tllm_add_f16, the
 * normed / paired plans). residuals[i] (HOST array of DEVICE pointers, entries or the array itself may be NULL) is
 * fp16 [rows]: the problem then stores fp16(residual[r] + fp16(projection)), the reference's add_forward behind the
 * projection; it may be the problem's own output, not its input. norm_weights as in
 * tllm_linear_plan_create_normed (may be NULL). Every problem: batch 1, group_size 128, cols a multiple of 128 between
 * 2048 and 28672, rows >= 16 (else TLLM_ERR_BAD_PLAN). TLLM_PROBLEM_QUANTIZE_INPUT is allowed where the other plans allow it.
 * The launch is sized so that all its workgroups are resident together; should they not be (the GPU is shared
 * with kernels that hold its CUs for long), a workgroup gives up after about a second of waiting, every workgroup
 * ends normally, outputs are then incomplete, and tllm_linear_plan_status reports it.
 */
int tllm_linear_plan_create_staged(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                                   const uint16_t *const *norm_weights, const uint16_t *const *residuals,
                                   const int32_t *stages, float eps, int count, int group_size);
/* TLLM_OK, or TLLM_ERR_STAGE_TIMEOUT if a launch of this staged plan gave up waiting since the last call (the flag
 * is read from the device and cleared; synchronise the launches you ask about first). Until it is cleared, further
 * launches of the plan do not wait either. Plans without stages: always TLLM_OK. */
int tllm_linear_plan_status(const tllm_linear_plan *plan);

/* One launch over every problem of the plan. Allocation-free. Besides the outputs a launch uses two device
 * counters that deal the tail of a large plan out to the workgroups (the kernel resets them when it ends, so
 * replays of a captured graph need no clearing). The plan holds 16 such pairs and launches take them in turn:
 * launches of one plan may overlap in time (several streams, graph branches) as long as no two of them that
 * are in flight together are 16 launches apart or were captured as the same launch (a captured launch keeps the
 * pair it was captured with: do not replay one graph concurrently with itself). They still write the same
 * outputs, like two calls of any operator on the same buffers. */
int tllm_linear_plan_launch(const tllm_linear_plan *plan, tllm_stream_t stream);
/* Algorithmic weight-stream bytes (masks + scales) one launch reads. */
int64_t tllm_linear_plan_weight_bytes(const tllm_linear_plan *plan);
/* Name of the kernel a launch of this plan runs (static string; for reports and profiles). The
 * choice depends on the activation-row counts, the shapes and the size of the plan. No counterpart in
 * the reference. */
const char *tllm_linear_plan_kernel(const tllm_linear_plan *plan);
void tllm_linear_plan_destroy(tllm_linear_plan *plan);

/*
 * Measurement aid: one pass of 16-byte loads over `bytes` of device memory (16-byte aligned), nothing
 * written (`sink` may be NULL). Timed, it gives the read-only streaming ceiling of the GPU at hand, the
 * figure a weight stream can be compared with besides the published HBM peak. No counterpart in the
 * reference operators; its benchmark prints a copy bandwidth for the same purpose (tests/benchmark.cu:87-95).
 */
int tllm_read_stream(const void *src, size_t bytes, uint32_t *sink, tllm_stream_t stream);

/*
 * Testing and tuning aid: the kernel-choice switches of the library. Each is read from its environment variable
 * once per process (TLLM_GEMM_PATH, TLLM_GEMM_ROWSPLIT, TLLM_BATCH_K_PARTS, TLLM_TALL_MAX_BATCH,
 * TLLM_TALL_MIN_SHARE, TLLM_READ_SHAPE) when the library first needs one; no operator call reads the environment.
 * These two calls change and read them afterwards, by name: "gemm_path" (0 cost model, 1 prefill GEMM, 2 passes of
 * the decode kernel), "gemm_rowsplit" (-1 cost model, 0 never, 1 or 2 forced), "batch_k_parts", "tall_max_batch",
 * "tall_min_share_milli", "stage_spin_limit" (polls a staged plan waits; 0: about a second), "stage_exchange" (read when
 * a staged plan is created: 0 makes it wait at barriers even where tagged words would do), "stage_epoch_start" (the
 * launch count a staged plan created afterwards starts its 16-bit tags from: tests put it just below the wrap), "read_wgs_per_cu",
 * "read_in_flight". An unknown name returns
 * TLLM_ERR_BAD_SHAPE. Results never depend on them beyond the order of fp32 additions. Not for concurrent use
 * with operator calls whose choice should be stable. No counterpart in the reference.
 */
int tllm_debug_set_tuning(const char *name, int value);
int tllm_debug_get_tuning(const char *name, int *value);

#ifdef __cplusplus
}
#endif
#endif /* TLLM_TERNARY_H */
