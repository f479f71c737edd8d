// Shared declarations of the ternary linear-layer library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <vector>

#include "../../include/tllm_ternary.h"

namespace tllm {

constexpr int kWave = 64;

// Load of weight-stream data that is read once per launch: marked non-temporal, so that it does not
// displace what is reused (activations, scales) from the caches. -DTLLM_STREAM_PLAIN keeps ordinary loads.
#ifdef TLLM_STREAM_PLAIN
#define TLLM_STREAM_LOAD(ptr) (*(ptr))
#else
#define TLLM_STREAM_LOAD(ptr) __builtin_nontemporal_load(ptr)
#endif

// One ternary linear: y[batch, rows] = x[batch, cols] * W^T with W packed as two bit planes.
struct Problem {
    const uint32_t *nz;
    const uint32_t *sg;
    const uint16_t *scales;
    const uint16_t *x;
    uint16_t *y;
    int32_t rows;
    int32_t cols;
    int32_t batch;
    int32_t flags;  // kProblemSwigluGate, kProblemQuantInput, kProblemInt8Input
    union {
        // optional prologue (plans only): x is RMS-normalised with these weights before it is used
        const uint16_t *norm_w;
        // plans on int8 activations (kProblemInt8Input: x points at int8 values, batch 1): the activation scale in
        // device memory, as tllm_quantize_absmax_i8 writes it
        const float *x_scale;
    };
    float eps;
    int32_t stage;  // staged plans: the problem runs after every problem of the stages before it has stored its output
    // optional epilogue (staged plans): the output is fp16(residual[r] + fp16(projection)), the reference's add_forward
    // behind the projection; may point at the output itself (in place)
    const uint16_t *residual;
    // Staged plans that hand results from stage to stage as tagged words (PlanDevice::exchange): where the launch
    // finds the problem's activations / its residual / where it leaves its output, as an index into the launch
    // slot's array of 32-bit words (fp16 bits | tag << 16), or -1: activations and residual are read from x and
    // residual as they are (nothing in the plan writes them), no later stage reads the output.
    int32_t x_words, res_words, y_words;
    int32_t pad_;
};
static_assert(sizeof(Problem) == sizeof(tllm_linear_problem) + 40, "tllm_linear_problem, then the prologue, the epilogue and the hand-over");
// What a workgroup of a staged plan needs to start a stage, in one 128-byte record (one round trip to memory instead
// of three dependent ones: its span, the span's place in the unit prefix, the problem): the span, the problem its
// first unit lies in, that problem's first unit and number of units, and the problem itself.
struct WgStart {
    int32_t u, u_end, pi, first_unit, p_units, pad[3];
    Problem p;
};
static_assert(sizeof(WgStart) == 128, "one record per 128-byte line");
constexpr int kProblemSwigluGate = TLLM_PROBLEM_SWIGLU_GATE;
constexpr int kProblemInt8Input = 0x100;  // set by tllm_linear_plan_create_i8, not a public flag
// staged plans, set by the library: a later stage overwrites y, so the store to y is complete before the tagged word goes out
constexpr int kProblemOrderedStore = 0x200;
// fp16 activations that the kernel quantises to int8 itself (absmax, reference kernels/activations.cu:88-142) before it
// multiplies: quantize_absmax_int8 + ternary_gemv_int8 in one launch, bit for bit (batch 1)
constexpr int kProblemQuantInput = TLLM_PROBLEM_QUANTIZE_INPUT;

// Tuning switches. Each is read from its environment variable ONCE, when the library first asks for any of them;
// afterwards only tllm_debug_set_tuning changes them (tests force kernel choices through it). No call path reads the
// environment again.
struct Tuning {
    std::atomic<int> gemm_path{0};              // TLLM_GEMM_PATH=mfma|stream: 1 | 2 forces prefill GEMM | passes of the batched decode kernel for M > 16
    std::atomic<int> gemm_rowsplit{-1};         // TLLM_GEMM_ROWSPLIT: 0 never, 1 / 2 whenever the shape allows (eight-wave / four-wave form)
    std::atomic<int> batch_k_parts{0};          // TLLM_BATCH_K_PARTS: n parts where they fit, 1 never share out K
    std::atomic<int> tall_max_batch{4};         // TLLM_TALL_MAX_BATCH: most activation rows of a plan on the tall-tile kernel
    std::atomic<int> tall_min_share_milli{1000};  // TLLM_TALL_MIN_SHARE (x 1000): share of the plan per workgroup, in units, from which tall tiles run
    std::atomic<int> stage_exchange{1};         // staged plans hand results over as tagged words where the plan allows (0: always the barrier)
    std::atomic<int> stage_epoch_start{0};      // launch count a new staged plan starts its tags from (tests put it just below the 16-bit wrap)
    std::atomic<int> stage_spin_limit{0};       // polls a workgroup of a staged plan waits for a stage (0: the plan's own limit); tests force a wait to expire with 1
    std::atomic<int> read_wgs_per_cu{8};        // TLLM_READ_SHAPE="wgs_per_cu,loads_in_flight" of tllm_read_stream
    std::atomic<int> read_in_flight{8};
};
Tuning &tuning();
std::atomic<int> *tuning_by_name(const char *name);  // nullptr: no such switch

// CU count of the current device, asked once per device (256 if the runtime cannot tell). Safe to
// call from several host threads.
inline int current_device_cus() {
    static std::atomic<int> cache[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cache[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        cache[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

__device__ __forceinline__ float h2f(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);
}
__device__ __forceinline__ uint16_t f2h(float v) {  // round to nearest even
    return __builtin_bit_cast(uint16_t, (_Float16)v);
}

// fp16(v) of an fp32 value the compiler must take as it is: without this it may fold the multiplication that
// produced v into a mixed-precision instruction that rounds the exact product once, straight to fp16, and whether it
// does depends on the code around. Two kernels that promise the same bits (RMSNorm on its own and as a prologue)
// round twice, fp32 then fp16, like the reference's __float2half of an fp32 product (kernels/rmsnorm.cu:20-106).
__device__ __forceinline__ uint16_t f2h_of_rounded(float v) {
    asm("" : "+v"(v));
    return f2h(v);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// ---- launchers implemented in the kernel files; all return a hipError_t ----
// General fallback (any group size that is a multiple of 32): one wave per output row.
hipError_t launch_gemv_rowwave_f16(const Problem &p, int group, hipStream_t s);
hipError_t launch_gemv_rowwave_f16_table(const Problem *table, int count, int max_rows,
                                         int max_batch, int group, hipStream_t s);
hipError_t launch_gemv_rowwave_i8(const uint32_t *nz, const uint32_t *sg, const uint16_t *scales,
                                  const int8_t *xq, float scale_value, const float *scale_dev,
                                  uint16_t *y, int rows, int cols, int group, hipStream_t s);
hipError_t launch_quantize_absmax_i8(const uint16_t *x, int8_t *q, float *scale, int n,
                                     hipStream_t s);
// quantize_absmax_int8 + ternary_gemv_int8 in one launch for the shapes the matrix-core kernel does not serve
hipError_t launch_gemv_rowwave_q8(const Problem &p, int group, hipStream_t s);

// Element-wise neighbours of the linears (elementwise.hip).
hipError_t launch_rmsnorm(const uint16_t *input, const uint16_t *weight, uint16_t *output, const uint16_t *residual,
                          uint16_t *residual_out, int batch, int dim, float eps, hipStream_t s);
hipError_t launch_silu_mul(const uint16_t *gate, const uint16_t *up, uint16_t *output, int size, hipStream_t s);
hipError_t launch_add(const uint16_t *a, const uint16_t *b, uint16_t *output, int size, hipStream_t s);
hipError_t launch_rope(uint16_t *q, uint16_t *k, int batch, int seq_len, int n_heads, int n_kv_heads, int head_dim,
                       int start_pos, float theta, hipStream_t s);
hipError_t launch_embedding_lookup(const uint16_t *table, const int *indices, uint16_t *output, int n_tokens, int dim,
                                   hipStream_t s);
hipError_t launch_copy_to_kv_cache(const uint16_t *k, const uint16_t *v, uint16_t *k_cache, uint16_t *v_cache, int batch,
                                   int n_kv_heads, int head_dim, int seq_len, int start_pos, int max_seq_len,
                                   hipStream_t s);

// Measurement aid (elementwise.hip): reads `bytes` of device memory once.
hipError_t launch_read_stream(const void *src, size_t bytes, uint32_t *sink, hipStream_t s);

// 128-group MFMA GEMV, batch 1..4 (gemv_mfma.hip).
bool gemv_mfma_supports(const Problem &p, int group);
hipError_t launch_gemv_mfma(const Problem &p, hipStream_t s);
// The same kernel on INT8 activations (p.x is an int8 pointer, batch 1): y = scale * sum_g s_g * (integer sum).
hipError_t launch_gemv_mfma_i8(const Problem &p, float scale_value, const float *scale_dev, hipStream_t s);

// 128-group MFMA kernel for 2..16 activation rows, K a multiple of 512 (gemv_batch.hip).
bool gemv_batch_supports(const Problem &p, int group);
// fixed_scratch: a launch that shares out K among workgroups exchanges its sums through the library's fixed device
// array instead of the stream's workspace (no allocation, ever).
hipError_t launch_gemv_batch(const Problem &p, hipStream_t s, bool fixed_scratch = false);
// Creates (or grows) the exchange workspace of stream s for this shape, if its launch would share out K at all.
hipError_t gemv_batch_reserve(const Problem &p, hipStream_t s);
const char *gemv_batch_kernel_name(const Problem &p);  // what launch_gemv_batch would run, given exchange memory (static string)
int gemv_batch_block_rows();
float gemv_batch_cost_us(const Problem &p);  // rough time of one launch_gemv_batch
hipError_t launch_gemv_batch_table(const Problem *table, const int *unit_prefix, const int *wg_first, int grid,
                                   int pool_begin, int pool_end, const int *pool_problem, int *counters,
                                   hipStream_t s);

// 128-group MFMA GEMM for M >= 16 (gemm_mfma.hip); Problem.batch is M, rows is N, cols is K.
bool gemm_mfma_supports(const Problem &p, int group);
hipError_t launch_gemm_mfma(const Problem &p, hipStream_t s);
float gemm_mfma_cost_us(const Problem &p);
const char *gemm_mfma_kernel_name(const Problem &p);  // the kernel launch_gemm_mfma would run (static string)  // rough time of launch_gemm_mfma, to choose between kernels
// Exchange memory for launches that share out K among workgroups (gemm_mfma.hip): `floats` fp32 slots and
// kSplitArrivalSlots arrival counters that are zero between launches. fixed: the library's fixed device array
// (*partial stays null if it is too small); else the workspace of (device, stream s), created or grown unless the
// stream is being captured (then *partial stays null when what exists is too small). Launches on one stream run in
// order and so may share it.
constexpr int kSplitArrivalSlots = 1024;
hipError_t split_exchange_memory(hipStream_t s, size_t floats, bool fixed, float **partial, unsigned **arrivals);
// Creates (or grows) the split-K workspace of stream s for this shape, if the shape splits K at all.
hipError_t gemm_mfma_reserve(const Problem &p, hipStream_t s);
void gemm_mfma_release_all();  // frees every split-K workspace (nothing may still be running on them)
// The same launch with the split-K exchange in the library's fixed device array (no allocation, ever).
// Up to four weight matrices on the same activations in one launch of the prefill GEMM (same x, batch and cols; K a
// multiple of 256 or of 128 from 384 on; 16-byte aligned masks and activations).
bool gemm_group_supports(const Problem *ps, int count);
hipError_t launch_gemm_group(const Problem *ps, int count, hipStream_t s);
// The prefill form of a SwiGLU pair in one launch (gate.y = silu(gate product) * up product); shapes: K a multiple of 128
// from 384 on, 16-byte aligned masks and activations.
bool gemm_swiglu_supports(const Problem &gate, const Problem &up);
hipError_t launch_gemm_swiglu(const Problem &gate, const Problem &up, hipStream_t s);
bool gemm_mfma_static_fits(const Problem &p);
hipError_t launch_gemm_mfma_static(const Problem &p, hipStream_t s);

// Picks the kernel for one linear (fast 128-group paths when they apply, else the row-wave kernel).
// static_scratch: a launch that splits K exchanges its partial sums through the fixed device array.
hipError_t dispatch_linear(const Problem &p, int group, hipStream_t s, bool static_scratch = false);
// Creates (or grows) the exchange workspace of stream s that dispatch_linear would use for this shape, if any.
hipError_t dispatch_reserve(const Problem &p, int group, hipStream_t s);
// True if dispatch_linear would run the prefill GEMM kernel (the only path that may need exchange memory).
bool dispatch_takes_gemm(const Problem &p, int group);
// Name of the kernel dispatch_linear would launch for this shape (static string; pointers may be null).
const char *dispatch_kernel_name(const Problem &p, int group);

// Launches of one plan that are in flight at the same time need hand-out counters of their own: a launch
// takes pair (launch number % kPlanSlots), so any kPlanSlots consecutive launches never share one.
constexpr int kPlanSlots = 16;

// Device-resident schedule of a multi-problem launch.
struct PlanDevice {
    Problem *problems = nullptr;  // device copy of the table
    int count = 0;
    int device = -1;
    int max_rows = 0;
    int max_batch = 0;
    // schedule of the MFMA kernel (use_mfma == false: the row-wave table kernel runs instead)
    bool use_mfma = false;
    bool wide = false;  // 4 x 2048 tiles (every problem at batch 1) instead of 16 x 512
    bool batch_kernel = false;  // the 2..16-row kernel runs (its blocks are the units below)
    int *unit_prefix = nullptr;
    int *wg_first = nullptr;
    int *pool_first = nullptr;  // shared pool of small tasks (MFMA kernel, large plans)
    int pool_count = 0;
    int pool_begin = 0, pool_end = 0;  // batched kernel: blocks handed out at run time, their problems in pool_first
    int *counters = nullptr;  // kPlanSlots pairs of hand-out counters; a launch takes the next pair in turn
    std::atomic<unsigned> *next_slot = nullptr;
    int grid = 0;
    int max_units = 0;
    int pair_stride = 0;  // floats between the two partial-sum areas of a SwiGLU pair (0: no pairs)
    bool fine = false;    // units of 16 rows (decode-size plans that would leave most workgroup slots empty)
    bool extras = false;  // SwiGLU pairs or RMSNorm prologues present: the kernel instance that knows them
    bool x_is_i8 = false; // every problem reads int8 activations and its own device-resident scale
    int image_bytes = 0;
    int lds_bytes = 0;
    // staged plans: the spans of stage s start at wg_first + s * (2 * grid + 1); between two stages every workgroup
    // waits for all workgroups at a barrier in device memory (stage_counters: one barrier per launch slot), for at
    // most spin_limit polls; a wait that expires sets *status
    int n_stages = 0;
    int *stage_counters = nullptr;
    int *status = nullptr;
    int spin_limit = 0;
    size_t barrier_bytes = 0;  // all barriers and the status word: cleared when a timeout is read
    bool stage_fence = false;  // the workgroups invalidate their cache behind each barrier (else: loads of device scope)
    // Hand-over by tagged words instead of barriers: per launch slot an array of words_per_slot 32-bit words (one per
    // output row that a later stage reads) and one launch count per workgroup (epochs), from which the tag comes.
    bool exchange = false;
    WgStart *starts = nullptr;  // [n_stages * grid]
    uint32_t *words = nullptr;  // per launch slot: the words, then one launch count per workgroup
    size_t words_per_slot = 0, ints_per_slot = 0;
};
hipError_t plan_device_create(const std::vector<Problem> &host, PlanDevice *out);
// A plan whose problems run in stages inside one launch (Problem::stage, ascending); batch 1, shapes the wide-tile
// kernel serves with whole rows in LDS. hipErrorInvalidValue for a plan that does not qualify.
hipError_t plan_device_create_staged(const std::vector<Problem> &host, PlanDevice *out);
constexpr int kMaxStages = 8;
hipError_t plan_device_launch(const PlanDevice &plan, hipStream_t s);
void plan_device_destroy(PlanDevice *plan);

}  // namespace tllm
