// Kernel selection for one linear.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "common.h"

namespace tllm {

Tuning &tuning() {
    static Tuning t;
    static const bool from_env = [] {
        if (const char *e = getenv("TLLM_GEMM_PATH")) t.gemm_path = e[0] == 'm' ? 1 : e[0] == 's' ? 2 : 0;
        if (const char *e = getenv("TLLM_GEMM_ROWSPLIT")) t.gemm_rowsplit = atoi(e);
        if (const char *e = getenv("TLLM_BATCH_K_PARTS")) t.batch_k_parts = atoi(e);
        if (const char *e = getenv("TLLM_TALL_MAX_BATCH")) t.tall_max_batch = atoi(e);
        if (const char *e = getenv("TLLM_TALL_MIN_SHARE")) t.tall_min_share_milli = (int)(atof(e) * 1000.0 + 0.5);
        if (const char *e = getenv("TLLM_READ_SHAPE")) {
            int a = 8, b = 8;
            if (sscanf(e, "%d,%d", &a, &b) == 2) {
                t.read_wgs_per_cu = a;
                t.read_in_flight = b;
            }
        }
        return true;
    }();
    (void)from_env;
    return t;
}

std::atomic<int> *tuning_by_name(const char *name) {
    Tuning &t = tuning();
    const struct {
        const char *name;
        std::atomic<int> *value;
    } all[] = {{"gemm_path", &t.gemm_path},           {"gemm_rowsplit", &t.gemm_rowsplit},
               {"batch_k_parts", &t.batch_k_parts},
               {"tall_max_batch", &t.tall_max_batch}, {"tall_min_share_milli", &t.tall_min_share_milli},
               {"read_wgs_per_cu", &t.read_wgs_per_cu}, {"read_in_flight", &t.read_in_flight},
               {"stage_spin_limit", &t.stage_spin_limit}, {"stage_exchange", &t.stage_exchange}, {"stage_epoch_start", &t.stage_epoch_start}};
    for (const auto &e : all)
        if (name && !strcmp(name, e.name)) return e.value;
    return nullptr;
}

namespace {
constexpr int kTallBatch = 4;    // activation rows per pass of the batch-1 family's tall tiles
constexpr int kBatchRows = 16;   // activation rows per pass of the batched decode kernel

// gemm_path 1 | 2 forces the choice between the prefill GEMM and passes of the batched decode kernel for M > 16
// (a tuning aid; 0: the cost model decides)
int forced_path() { return tuning().gemm_path.load(std::memory_order_relaxed); }
}  // namespace

namespace {
// The activation rows go through the batched decode kernel in passes of 16 (true), or not (false).
bool streams_in_passes(const Problem &p, int group) {
    Problem probe = p;
    probe.batch = p.batch < kBatchRows ? p.batch : kBatchRows;
    if (p.batch <= 1 || !gemv_batch_supports(probe, group)) return false;
    const int passes = (p.batch + kBatchRows - 1) / kBatchRows;
    const bool gemm_ok = gemm_mfma_supports(p, group);
    bool stream = passes == 1 || !gemm_ok || (float)passes * gemv_batch_cost_us(probe) < gemm_mfma_cost_us(p);
    if (passes > 1 && gemm_ok && forced_path()) stream = forced_path() == 2;
    return stream;
}
}  // namespace

bool dispatch_takes_gemm(const Problem &p, int group) {
    if (group != 128) return false;
    if (p.batch == 1 && gemv_mfma_supports(p, group)) return false;
    if (streams_in_passes(p, group)) return false;
    return !gemv_mfma_supports(p, group) && gemm_mfma_supports(p, group);
}

hipError_t dispatch_linear(const Problem &p, int group, hipStream_t s, bool static_scratch) {
    if (group != 128) return launch_gemv_rowwave_f16(p, group, s);
    if (p.batch == 1 && gemv_mfma_supports(p, group)) return launch_gemv_mfma(p, s);
    if (streams_in_passes(p, group)) {
        for (int b0 = 0; b0 < p.batch; b0 += kBatchRows) {
            Problem q = p;
            q.batch = p.batch - b0 < kBatchRows ? p.batch - b0 : kBatchRows;
            q.x = p.x + (size_t)b0 * p.cols;
            q.y = p.y + (size_t)b0 * p.rows;
            if (hipError_t e = launch_gemv_batch(q, s, static_scratch)) return e;
        }
        return hipSuccess;
    }
    if (gemv_mfma_supports(p, group)) return launch_gemv_mfma(p, s);
    if (gemm_mfma_supports(p, group)) return static_scratch ? launch_gemm_mfma_static(p, s) : launch_gemm_mfma(p, s);
    // wider batches: four activation rows at a time through the tall-tile kernel
    for (int b0 = 0; b0 < p.batch; b0 += kTallBatch) {
        Problem q = p;
        q.batch = p.batch - b0 < kTallBatch ? p.batch - b0 : kTallBatch;
        q.x = p.x + (size_t)b0 * p.cols;
        q.y = p.y + (size_t)b0 * p.rows;
        while (q.batch > 1 && !gemv_mfma_supports(q, group)) q.batch /= 2;  // very long K: fewer rows per pass
        if (!gemv_mfma_supports(q, group)) return launch_gemv_rowwave_f16(p, group, s);
        if (hipError_t e = launch_gemv_mfma(q, s)) return e;
        b0 -= kTallBatch - q.batch;
    }
    return hipSuccess;
}


hipError_t dispatch_reserve(const Problem &p, int group, hipStream_t s) {
    if (group != 128 || (p.batch == 1 && gemv_mfma_supports(p, group))) return hipSuccess;
    if (streams_in_passes(p, group)) {
        Problem q = p;
        q.batch = p.batch < kBatchRows ? p.batch : kBatchRows;
        return gemv_batch_reserve(q, s);
    }
    if (gemv_mfma_supports(p, group) || !gemm_mfma_supports(p, group)) return hipSuccess;
    return gemm_mfma_reserve(p, s);
}

const char *dispatch_kernel_name(const Problem &p, int group) {
    if (group != 128) return "tllm::gemv_rowwave_f16_kernel";
    if (p.batch == 1 && gemv_mfma_supports(p, group)) return "tllm::gemv_mfma_kernel";
    if (streams_in_passes(p, group)) {
        Problem q = p;
        q.batch = p.batch < kBatchRows ? p.batch : kBatchRows;
        return gemv_batch_kernel_name(q);
    }
    if (gemv_mfma_supports(p, group)) return "tllm::gemv_mfma_kernel<Tall>";
    if (gemm_mfma_supports(p, group)) return gemm_mfma_kernel_name(p);
    return "tllm::gemv_mfma_kernel<Tall>, passes";
}

}  // namespace tllm
