// The C ABI: argument validation and dispatch. No kernel code lives here.
#include <new>
#include <vector>

#include "common.h"

namespace tllm {
namespace {

inline bool misaligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

inline bool overlaps(const void *a, size_t na, const void *b, size_t nb) {
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + nb && b0 < a0 + na;
}

// Checks shared by every operator over a packed rows x cols weight.
int check_weight(const void *nz, const void *sg, const void *scales, int rows, int cols, int group) {
    if (!nz || !sg || !scales) return TLLM_ERR_NULL_POINTER;
    if (rows < 1 || cols < 1 || cols % 32 != 0) return TLLM_ERR_BAD_SHAPE;
    if (group < 32 || group % 32 != 0 || cols % group != 0) return TLLM_ERR_BAD_GROUP;
    if (misaligned(nz, 16) || misaligned(sg, 16) || misaligned(scales, 2)) return TLLM_ERR_MISALIGNED;
    return TLLM_OK;
}

int check_linear(const Problem &p, int group) {
    if (int e = check_weight(p.nz, p.sg, p.scales, p.rows, p.cols, group)) return e;
    if (!p.x || !p.y) return TLLM_ERR_NULL_POINTER;
    if (p.batch < 1) return TLLM_ERR_BAD_SHAPE;
    if (misaligned(p.x, 16) || misaligned(p.y, 2)) return TLLM_ERR_MISALIGNED;
    if ((int64_t)p.batch * p.cols > INT32_MAX || (int64_t)p.batch * p.rows > INT32_MAX)
        return TLLM_ERR_TOO_LARGE;
    if (overlaps(p.x, (size_t)p.batch * p.cols * 2, p.y, (size_t)p.batch * p.rows * 2))
        return TLLM_ERR_ALIAS;
    return TLLM_OK;
}

int run_linear(const Problem &p, int group, hipStream_t s) {
    if (int e = check_linear(p, group)) return e;
    return (int)dispatch_linear(p, group, s);
}

}  // namespace
}  // namespace tllm

using tllm::Problem;

struct tllm_linear_plan {
    std::vector<Problem> host;
    tllm::PlanDevice dev;
    int group;
    int64_t weight_bytes;
};

extern "C" {

const char *tllm_error_string(int code) {
    switch (code) {
        case TLLM_OK: return "ok";
        case TLLM_ERR_NULL_POINTER: return "a required pointer is NULL";
        case TLLM_ERR_BAD_SHAPE: return "bad shape: sizes must be >= 1 and cols a multiple of 32";
        case TLLM_ERR_BAD_GROUP: return "bad group_size: must be a multiple of 32 that divides cols";
        case TLLM_ERR_TOO_LARGE: return "size exceeds the supported maximum";
        case TLLM_ERR_ALIAS: return "output overlaps the activation input";
        case TLLM_ERR_BAD_PLAN: return "invalid plan: handle, problem count, batch, SwiGLU pair or RMSNorm prologue";
        case TLLM_ERR_MISALIGNED: return "pointer alignment: masks/activations need 16 bytes, fp16 arrays 2";
        case -8: return "file cannot be opened, is truncated, or a write failed";   // TLLM_ERR_IO
        case -9: return "not a .tllm file of a supported version, or a header field is out of range";  // TLLM_ERR_BAD_FILE
        case TLLM_ERR_STAGE_TIMEOUT:
            return "a launch of a staged plan gave up waiting for a stage (its workgroups were not all running at the same time)";
        case TLLM_ERR_SCRATCH_TOO_SMALL:
            return "the split-K exchange of this GEMM shape needs more than the fixed device scratch of "
                   "tllm_ternary_gemm_f16_static (TLLM_GEMM_STATIC_SCRATCH_BYTES): use tllm_ternary_gemm_f16";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error code";
    }
}

int tllm_abi_version(void) { return 1; }

int tllm_ternary_gemv_f16(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                          const uint16_t *scales, const uint16_t *input, uint16_t *output,
                          int rows, int cols, int group_size, tllm_stream_t stream) {
    Problem p{nonzero_masks, sign_masks, scales, input, output, rows, cols, 1, 0};
    return tllm::run_linear(p, group_size, (hipStream_t)stream);
}

int tllm_ternary_gemm_f16(const uint16_t *A, const uint32_t *nz_B, const uint32_t *sign_B,
                          const uint16_t *scales_B, uint16_t *C, int M, int N, int K,
                          int group_size, tllm_stream_t stream) {
    if (M < 1) return TLLM_ERR_BAD_SHAPE;
    Problem p{nz_B, sign_B, scales_B, A, C, N, K, M, 0};
    return tllm::run_linear(p, group_size, (hipStream_t)stream);
}

int tllm_ternary_gemm_f16_static(const uint16_t *A, const uint32_t *nz_B, const uint32_t *sign_B,
                                 const uint16_t *scales_B, uint16_t *C, int M, int N, int K,
                                 int group_size, tllm_stream_t stream) {
    if (M < 1) return TLLM_ERR_BAD_SHAPE;
    Problem p{nz_B, sign_B, scales_B, A, C, N, K, M, 0};
    if (int e = tllm::check_linear(p, group_size)) return e;
    if (tllm::dispatch_takes_gemm(p, group_size) && !tllm::gemm_mfma_static_fits(p)) return TLLM_ERR_SCRATCH_TOO_SMALL;
    return (int)tllm::dispatch_linear(p, group_size, (hipStream_t)stream, true);
}

int tllm_ternary_gemm_swiglu_f16(const uint16_t *A, const uint32_t *nz_gate, const uint32_t *sign_gate,
                                 const uint16_t *scales_gate, const uint32_t *nz_up, const uint32_t *sign_up,
                                 const uint16_t *scales_up, uint16_t *C, int M, int N, int K, int group_size,
                                 tllm_stream_t stream) {
    if (M < 1) return TLLM_ERR_BAD_SHAPE;
    Problem gate{nz_gate, sign_gate, scales_gate, A, C, N, K, M, 0};
    Problem up{nz_up, sign_up, scales_up, A, C, N, K, M, 0};
    if (int e = tllm::check_linear(gate, group_size)) return e;
    if (int e = tllm::check_weight(nz_up, sign_up, scales_up, N, K, group_size)) return e;
    // (one kernel serves the pair: group 128, K a multiple of 256 or of 128 from 384 on; other shapes: the three launches)
    if (group_size != 128) return TLLM_ERR_BAD_GROUP;
    if (!tllm::gemm_swiglu_supports(gate, up)) return TLLM_ERR_BAD_SHAPE;
    return (int)tllm::launch_gemm_swiglu(gate, up, (hipStream_t)stream);
}

int tllm_ternary_gemm_group_f16(const uint16_t *A, const uint32_t *const *nz, const uint32_t *const *sign,
                                const uint16_t *const *scales, uint16_t *const *C, const int *N, int count, int M, int K,
                                int group_size, tllm_stream_t stream) {
    if (!nz || !sign || !scales || !C || !N) return TLLM_ERR_NULL_POINTER;
    if (count < 1 || count > TLLM_MAX_GEMM_GROUP || M < 1) return TLLM_ERR_BAD_SHAPE;
    Problem ps[TLLM_MAX_GEMM_GROUP];
    for (int i = 0; i < count; i++) {
        ps[i] = Problem{nz[i], sign[i], scales[i], A, C[i], N[i], K, M, 0};
        if (int e = tllm::check_linear(ps[i], group_size)) return e;
        for (int j = 0; j < i; j++)
            if (tllm::overlaps(C[i], (size_t)M * N[i] * 2, C[j], (size_t)M * N[j] * 2)) return TLLM_ERR_ALIAS;
    }
    if (group_size != 128) return TLLM_ERR_BAD_GROUP;
    if (!tllm::gemm_group_supports(ps, count)) return TLLM_ERR_BAD_SHAPE;
    return (int)tllm::launch_gemm_group(ps, count, (hipStream_t)stream);
}

int tllm_gemm_workspace_reserve(int M, int N, int K, int group_size, tllm_stream_t stream) {
    if (M < 1 || N < 1 || K < 1 || K % 32 != 0) return TLLM_ERR_BAD_SHAPE;
    if (group_size < 32 || group_size % 32 != 0 || K % group_size != 0) return TLLM_ERR_BAD_GROUP;
    if ((int64_t)M * K > INT32_MAX || (int64_t)M * N > INT32_MAX) return TLLM_ERR_TOO_LARGE;
    // only the shape matters here: the pointers are never dereferenced
    Problem p{nullptr, nullptr, nullptr, nullptr, nullptr, N, K, M, 0};
    return (int)tllm::dispatch_reserve(p, group_size, (hipStream_t)stream);
}

void tllm_gemm_workspace_release(void) { tllm::gemm_mfma_release_all(); }

const char *tllm_ternary_gemm_kernel(int M, int N, int K, int group_size) {
    if (M < 1 || N < 1 || K < 1 || K % 32 != 0 || group_size < 32 || group_size % 32 != 0 || K % group_size != 0) return "";
    Problem p{nullptr, nullptr, nullptr, nullptr, nullptr, N, K, M, 0};
    return tllm::dispatch_kernel_name(p, group_size);
}

static int gemv_i8_common(const uint32_t *nz, const uint32_t *sg, const uint16_t *scales,
                          const int8_t *xq, float scale_value, const float *scale_dev,
                          uint16_t *y, int rows, int cols, int group, tllm_stream_t stream) {
    if (int e = tllm::check_weight(nz, sg, scales, rows, cols, group)) return e;
    if (!xq || !y) return TLLM_ERR_NULL_POINTER;
    if (tllm::misaligned(xq, 16) || tllm::misaligned(y, 2)) return TLLM_ERR_MISALIGNED;
    if (tllm::overlaps(xq, (size_t)cols, y, (size_t)rows * 2)) return TLLM_ERR_ALIAS;
    // int8 values are exact in fp16 and the group sums stay exact in the fp32 accumulators, so the
    // fp16 matrix-core kernel computes the reference's integer arithmetic on them
    Problem p{nz, sg, scales, reinterpret_cast<const uint16_t *>(xq), y, rows, cols, 1, 0};
    if (group == 128 && tllm::gemv_mfma_supports(p, group))
        return (int)tllm::launch_gemv_mfma_i8(p, scale_value, scale_dev, (hipStream_t)stream);
    return (int)tllm::launch_gemv_rowwave_i8(nz, sg, scales, xq, scale_value, scale_dev, y, rows,
                                             cols, group, (hipStream_t)stream);
}

int tllm_ternary_gemv_i8(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                         const uint16_t *weight_scales, const int8_t *input_int8,
                         float input_scale, uint16_t *output, int rows, int cols, int group_size,
                         tllm_stream_t stream) {
    return gemv_i8_common(nonzero_masks, sign_masks, weight_scales, input_int8, input_scale,
                          nullptr, output, rows, cols, group_size, stream);
}

int tllm_ternary_linear_int8_f16(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                                 const uint16_t *weight_scales, const uint16_t *input, uint16_t *output,
                                 int rows, int cols, int group_size, tllm_stream_t stream) {
    Problem p{nonzero_masks, sign_masks, weight_scales, input, output, rows, cols, 1, tllm::kProblemQuantInput};
    if (int e = tllm::check_linear(p, group_size)) return e;
    if (group_size == 128 && tllm::gemv_mfma_supports(p, group_size)) return (int)tllm::launch_gemv_mfma(p, (hipStream_t)stream);
    return (int)tllm::launch_gemv_rowwave_q8(p, group_size, (hipStream_t)stream);
}

int tllm_ternary_gemv_i8_dscale(const uint32_t *nonzero_masks, const uint32_t *sign_masks,
                                const uint16_t *weight_scales, const int8_t *input_int8,
                                const float *input_scale_device, uint16_t *output, int rows,
                                int cols, int group_size, tllm_stream_t stream) {
    if (!input_scale_device) return TLLM_ERR_NULL_POINTER;
    return gemv_i8_common(nonzero_masks, sign_masks, weight_scales, input_int8, 0.0f,
                          input_scale_device, output, rows, cols, group_size, stream);
}

int tllm_quantize_absmax_i8(const uint16_t *input, int8_t *output, float *scale, int n,
                            tllm_stream_t stream) {
    if (!input || !output || !scale) return TLLM_ERR_NULL_POINTER;
    if (n < 1) return TLLM_ERR_BAD_SHAPE;
    if (tllm::misaligned(input, 2) || tllm::misaligned(scale, 4)) return TLLM_ERR_MISALIGNED;
    return (int)tllm::launch_quantize_absmax_i8(input, output, scale, n, (hipStream_t)stream);
}

int tllm_rmsnorm_f16(const uint16_t *input, const uint16_t *weight, uint16_t *output, const uint16_t *residual,
                     uint16_t *residual_out, int batch, int dim, float eps, tllm_stream_t stream) {
    if (!input || !weight || !output) return TLLM_ERR_NULL_POINTER;
    if (batch < 1 || dim < 1) return TLLM_ERR_BAD_SHAPE;
    if ((int64_t)batch * dim > INT32_MAX) return TLLM_ERR_TOO_LARGE;
    if (residual_out && !residual) return TLLM_ERR_NULL_POINTER;
    return (int)tllm::launch_rmsnorm(input, weight, output, residual, residual_out, batch, dim, eps, (hipStream_t)stream);
}

int tllm_silu_mul_f16(const uint16_t *gate, const uint16_t *up, uint16_t *output, int size, tllm_stream_t stream) {
    if (!gate || !up || !output) return TLLM_ERR_NULL_POINTER;
    if (size < 1) return TLLM_ERR_BAD_SHAPE;
    return (int)tllm::launch_silu_mul(gate, up, output, size, (hipStream_t)stream);
}

int tllm_add_f16(const uint16_t *a, const uint16_t *b, uint16_t *output, int size, tllm_stream_t stream) {
    if (!a || !b || !output) return TLLM_ERR_NULL_POINTER;
    if (size < 1) return TLLM_ERR_BAD_SHAPE;
    return (int)tllm::launch_add(a, b, output, size, (hipStream_t)stream);
}

int tllm_rope_f16(uint16_t *q, uint16_t *k, int batch, int seq_len, int n_heads, int n_kv_heads, int head_dim,
                  int start_pos, float theta, tllm_stream_t stream) {
    if (!q || !k) return TLLM_ERR_NULL_POINTER;
    if (batch < 1 || seq_len < 1 || n_heads < 1 || n_kv_heads < 1 || head_dim < 2 || head_dim % 2 || start_pos < 0 ||
        !(theta > 0.0f))
        return TLLM_ERR_BAD_SHAPE;
    const long long heads = n_heads > n_kv_heads ? n_heads : n_kv_heads;
    if ((long long)batch * seq_len * heads * head_dim >= (1ll << 40) || (long long)start_pos + seq_len > INT32_MAX)
        return TLLM_ERR_BAD_SHAPE;
    if (((uintptr_t)q | (uintptr_t)k) & 3) return TLLM_ERR_MISALIGNED;
    return (int)tllm::launch_rope(q, k, batch, seq_len, n_heads, n_kv_heads, head_dim, start_pos, theta, (hipStream_t)stream);
}

int tllm_embedding_lookup_f16(const uint16_t *table, const int32_t *indices, uint16_t *output, int n_tokens, int dim,
                              tllm_stream_t stream) {
    if (!table || !indices || !output) return TLLM_ERR_NULL_POINTER;
    if (n_tokens < 1 || dim < 1) return TLLM_ERR_BAD_SHAPE;
    return (int)tllm::launch_embedding_lookup(table, indices, output, n_tokens, dim, (hipStream_t)stream);
}

int tllm_copy_to_kv_cache_f16(const uint16_t *k, const uint16_t *v, uint16_t *k_cache, uint16_t *v_cache, int batch,
                              int n_kv_heads, int head_dim, int seq_len, int start_pos, int max_seq_len,
                              tllm_stream_t stream) {
    if (!k || !v || !k_cache || !v_cache) return TLLM_ERR_NULL_POINTER;
    if (batch < 1 || batch > 65535 || n_kv_heads < 1 || n_kv_heads > 65535 || head_dim < 1 || seq_len < 1 ||
        start_pos < 0 || max_seq_len < 1 || (long long)start_pos + seq_len > INT32_MAX)
        return TLLM_ERR_BAD_SHAPE;
    return (int)tllm::launch_copy_to_kv_cache(k, v, k_cache, v_cache, batch, n_kv_heads, head_dim, seq_len, start_pos,
                                              max_seq_len, (hipStream_t)stream);
}

int tllm_debug_set_tuning(const char *name, int value) {
    std::atomic<int> *v = tllm::tuning_by_name(name);
    if (!v) return TLLM_ERR_BAD_SHAPE;
    v->store(value, std::memory_order_relaxed);
    return TLLM_OK;
}

int tllm_debug_get_tuning(const char *name, int *value) {
    std::atomic<int> *v = tllm::tuning_by_name(name);
    if (!v || !value) return v ? TLLM_ERR_NULL_POINTER : TLLM_ERR_BAD_SHAPE;
    *value = v->load(std::memory_order_relaxed);
    return TLLM_OK;
}

int tllm_read_stream(const void *src, size_t bytes, uint32_t *sink, tllm_stream_t stream) {
    if (!src) return TLLM_ERR_NULL_POINTER;
    if (bytes < 16) return TLLM_ERR_BAD_SHAPE;
    if (tllm::misaligned(src, 16)) return TLLM_ERR_MISALIGNED;
    return (int)tllm::launch_read_stream(src, bytes, sink, (hipStream_t)stream);
}

static int create_plan(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                       const uint16_t *const *norm_weights, float eps, int count, int group_size,
                       const float *const *input_scales = nullptr, const uint16_t *const *residuals = nullptr,
                       const int32_t *stages = nullptr) {
    if (!plan || !problems) return TLLM_ERR_NULL_POINTER;
    *plan = nullptr;
    if (count < 1) return TLLM_ERR_BAD_PLAN;
    if (group_size != 128) return TLLM_ERR_BAD_GROUP;
    std::vector<Problem> host(count);
    int64_t bytes = 0;
    for (int i = 0; i < count; i++) {
        const tllm_linear_problem &q = problems[i];
        host[i] = Problem{q.nonzero_masks, q.sign_masks, q.scales, q.input, q.output,
                          q.rows, q.cols, q.batch, q.flags};
        if (q.batch < 1 || q.batch > TLLM_MAX_PLAN_BATCH) return TLLM_ERR_BAD_PLAN;
        if (q.flags & ~(TLLM_PROBLEM_SWIGLU_GATE | TLLM_PROBLEM_QUANTIZE_INPUT)) return TLLM_ERR_BAD_PLAN;
        if (q.flags & TLLM_PROBLEM_QUANTIZE_INPUT) {
            // quantised inside the launch: one activation row, fp16 input. A norm prologue comes first (the normalised,
            // fp16-rounded row is what gets quantised, as when rmsnorm_forward runs in front of the quantiser); the two
            // halves of a SwiGLU pair share the quantised row (the flag sits on the gate problem).
            if (q.batch != 1 || input_scales) return TLLM_ERR_BAD_PLAN;
        }
        const bool is_up = i > 0 && (problems[i - 1].flags & TLLM_PROBLEM_SWIGLU_GATE);
        if (is_up) {
            // the up half of a SwiGLU pair: same shape and activations as its gate, no output of its own
            const tllm_linear_problem &g = problems[i - 1];
            if (q.flags || q.rows != g.rows || q.cols != g.cols || q.batch != g.batch || q.input != g.input)
                return TLLM_ERR_BAD_PLAN;
            host[i].y = host[i - 1].y;
        }
        if (q.flags & TLLM_PROBLEM_SWIGLU_GATE) {
            if (i + 1 >= count || q.batch != 1) return TLLM_ERR_BAD_PLAN;
        }
        if (input_scales) {
            // int8 activations: `input` points at int8 [cols]; one row, no pairs; the scale lives on the device
            if (q.batch != 1 || q.flags) return TLLM_ERR_BAD_PLAN;
            if (!input_scales[i] || !q.input || !q.output) return TLLM_ERR_NULL_POINTER;
            if (int e = tllm::check_weight(host[i].nz, host[i].sg, host[i].scales, q.rows, q.cols, group_size)) return e;
            if (tllm::misaligned(q.input, 16) || tllm::misaligned(q.output, 2) || tllm::misaligned(input_scales[i], 4))
                return TLLM_ERR_MISALIGNED;
            if (tllm::overlaps(q.input, (size_t)q.cols, q.output, (size_t)q.rows * 2)) return TLLM_ERR_ALIAS;
            host[i].flags |= tllm::kProblemInt8Input;
            host[i].x_scale = input_scales[i];
        } else if (int e = tllm::check_linear(host[i], group_size)) {
            return e;
        }
        if (norm_weights && norm_weights[i]) {
            // RMSNorm prologue: batch 1, a row that the one-pass staging holds, 16-byte aligned weights
            if (q.batch != 1 || q.cols > 16384 || !(eps >= 0.0f)) return TLLM_ERR_BAD_PLAN;
            if (tllm::misaligned(norm_weights[i], 16)) return TLLM_ERR_MISALIGNED;
            if (is_up && norm_weights[i] != norm_weights[i - 1]) return TLLM_ERR_BAD_PLAN;
            host[i].norm_w = norm_weights[i];
            host[i].eps = eps;
        } else if (is_up && norm_weights && norm_weights[i - 1]) {
            return TLLM_ERR_BAD_PLAN;  // the halves of a pair see the same activations
        }
        if (stages) {
            // staged plans: one activation row; an up problem shares its gate's stage; the residual of the epilogue is
            // fp16 [rows] and may be the output itself, but not the input
            if (q.batch != 1 || stages[i] < 0 || stages[i] >= tllm::kMaxStages) return TLLM_ERR_BAD_PLAN;
            if (is_up && stages[i] != stages[i - 1]) return TLLM_ERR_BAD_PLAN;
            host[i].stage = stages[i];
            if (residuals && residuals[i]) {
                if (is_up || (q.flags & TLLM_PROBLEM_SWIGLU_GATE)) return TLLM_ERR_BAD_PLAN;
                if (tllm::misaligned(residuals[i], 2)) return TLLM_ERR_MISALIGNED;
                if (tllm::overlaps(residuals[i], (size_t)q.rows * 2, q.input, (size_t)q.cols * 2)) return TLLM_ERR_ALIAS;
                host[i].residual = residuals[i];
            }
        }
        bytes += (int64_t)q.rows * (q.cols / 32) * 8 + (int64_t)q.rows * (q.cols / group_size) * 2;
    }
    tllm_linear_plan *pl = new (std::nothrow) tllm_linear_plan{std::move(host), {}, group_size, bytes};
    if (!pl) return TLLM_ERR_TOO_LARGE;
    if (hipError_t e = stages ? tllm::plan_device_create_staged(pl->host, &pl->dev) : tllm::plan_device_create(pl->host, &pl->dev)) {
        delete pl;
        // (invalid value: a shape that only the general kernel serves, which knows neither int8 activations nor pairs nor prologues)
        return e == hipErrorInvalidValue ? TLLM_ERR_BAD_PLAN : (int)e;
    }
    if (pl->dev.extras && !pl->dev.use_mfma) {  // a shape that only the general kernel serves: no pairs, no prologue
        tllm::plan_device_destroy(&pl->dev);
        delete pl;
        return TLLM_ERR_BAD_PLAN;
    }
    *plan = pl;
    return TLLM_OK;
}

int tllm_linear_plan_create(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                            int count, int group_size) {
    return create_plan(plan, problems, nullptr, 0.0f, count, group_size);
}

int tllm_linear_plan_create_normed(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                                   const uint16_t *const *norm_weights, float eps, int count,
                                   int group_size) {
    if (!norm_weights) return TLLM_ERR_NULL_POINTER;
    return create_plan(plan, problems, norm_weights, eps, count, group_size);
}

int tllm_linear_plan_create_i8(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                               const float *const *input_scales, int count, int group_size) {
    if (!input_scales) return TLLM_ERR_NULL_POINTER;
    return create_plan(plan, problems, nullptr, 0.0f, count, group_size, input_scales);
}

int tllm_linear_plan_create_staged(tllm_linear_plan **plan, const tllm_linear_problem *problems,
                                   const uint16_t *const *norm_weights, const uint16_t *const *residuals,
                                   const int32_t *stages, float eps, int count, int group_size) {
    if (!stages) return TLLM_ERR_NULL_POINTER;
    return create_plan(plan, problems, norm_weights, eps, count, group_size, nullptr, residuals, stages);
}

int tllm_linear_plan_status(const tllm_linear_plan *plan) {
    if (!plan) return TLLM_ERR_BAD_PLAN;
    if (!plan->dev.status) return TLLM_OK;
    int v = 0;
    if (hipError_t e = hipMemcpy(&v, plan->dev.status, sizeof v, hipMemcpyDeviceToHost)) return (int)e;
    if (v != 0) {
        // (the launch that gave up left its barrier half counted: all barriers and the status word start again)
        if (hipError_t e = hipMemset(plan->dev.stage_counters, 0, plan->dev.barrier_bytes)) return (int)e;
        return TLLM_ERR_STAGE_TIMEOUT;
    }
    return TLLM_OK;
}

int tllm_linear_plan_launch(const tllm_linear_plan *plan, tllm_stream_t stream) {
    if (!plan || plan->host.empty()) return TLLM_ERR_BAD_PLAN;
    return (int)tllm::plan_device_launch(plan->dev, (hipStream_t)stream);
}

int64_t tllm_linear_plan_weight_bytes(const tllm_linear_plan *plan) {
    return plan ? plan->weight_bytes : 0;
}

const char *tllm_linear_plan_kernel(const tllm_linear_plan *plan) {
    if (!plan) return "";
    const tllm::PlanDevice &d = plan->dev;
    if (d.batch_kernel) return "tllm::gemv_batch_kernel";
    if (!d.use_mfma) return "tllm::gemv_rowwave_f16_table_kernel";
    if (d.n_stages > 0 && d.exchange) return "tllm::gemv_mfma_kernel<Wide, extras, fine>, staged, results handed over as tagged words";
    if (d.n_stages > 0) return "tllm::gemv_mfma_kernel<Wide, extras, fine>, staged, barriers between the stages";
    if (!d.wide) return d.fine ? "tllm::gemv_mfma_kernel<Tall, fine>" : "tllm::gemv_mfma_kernel<Tall>";
    if (d.extras) return d.fine ? "tllm::gemv_mfma_kernel<Wide, extras, fine>" : "tllm::gemv_mfma_kernel<Wide, extras>";
    return d.fine ? "tllm::gemv_mfma_kernel<Wide, fine>" : "tllm::gemv_mfma_kernel<Wide>";
}

void tllm_linear_plan_destroy(tllm_linear_plan *plan) {
    if (!plan) return;
    tllm::plan_device_destroy(&plan->dev);
    delete plan;
}

}  // extern "C"
