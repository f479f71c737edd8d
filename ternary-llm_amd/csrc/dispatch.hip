// Kernel selection for one linear.
#include "common.h"

namespace tllm {

namespace {
constexpr int kTallBatch = 4;    // activation rows per pass of the batch-1 family's tall tiles
constexpr int kBatchRows = 16;   // activation rows per pass of the batched decode kernel

// rough time of `passes` sweeps over the packed weights at the rate the streaming kernels sustain
float stream_cost_us(const Problem &p, int passes) {
    const float bytes = 0.265625f * (float)p.rows * (float)p.cols;
    return (float)passes * (bytes / 4.0e6f + 3.0f);
}
}  // namespace

hipError_t dispatch_linear(const Problem &p, int group, hipStream_t s) {
    if (group != 128) return launch_gemv_rowwave_f16(p, group, s);
    if (p.batch == 1 && gemv_mfma_supports(p, group)) return launch_gemv_mfma(p, s);
    Problem probe = p;
    probe.batch = p.batch < kBatchRows ? p.batch : kBatchRows;
    if (p.batch > 1 && gemv_batch_supports(probe, group)) {
        const int passes = (p.batch + kBatchRows - 1) / kBatchRows;
        const bool gemm_ok = gemm_mfma_supports(p, group);
        if (passes == 1 || !gemm_ok || stream_cost_us(p, passes) < gemm_mfma_cost_us(p)) {
            for (int b0 = 0; b0 < p.batch; b0 += kBatchRows) {
                Problem q = p;
                q.batch = p.batch - b0 < kBatchRows ? p.batch - b0 : kBatchRows;
                q.x = p.x + (size_t)b0 * p.cols;
                q.y = p.y + (size_t)b0 * p.rows;
                if (hipError_t e = launch_gemv_batch(q, s)) return e;
            }
            return hipSuccess;
        }
    }
    if (gemv_mfma_supports(p, group)) return launch_gemv_mfma(p, s);
    if (gemm_mfma_supports(p, group)) return launch_gemm_mfma(p, s);
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

}  // namespace tllm
