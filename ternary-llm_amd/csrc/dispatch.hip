// Kernel selection for one linear.
#include "common.h"

namespace tllm {

hipError_t dispatch_linear(const Problem &p, int group, hipStream_t s) {
    if (group != 128) return launch_gemv_rowwave_f16(p, group, s);
    if (gemv_mfma_supports(p, group)) return launch_gemv_mfma(p, s);
    if (gemm_mfma_supports(p, group)) return launch_gemm_mfma(p, s);
    // wider batches: four activation rows at a time through the same kernel
    for (int b0 = 0; b0 < p.batch; b0 += TLLM_MAX_PLAN_BATCH) {
        Problem q = p;
        q.batch = p.batch - b0 < TLLM_MAX_PLAN_BATCH ? p.batch - b0 : TLLM_MAX_PLAN_BATCH;
        q.x = p.x + (size_t)b0 * p.cols;
        q.y = p.y + (size_t)b0 * p.rows;
        while (q.batch > 1 && !gemv_mfma_supports(q, group)) q.batch /= 2;  // very long K: fewer rows per pass
        if (!gemv_mfma_supports(q, group)) return launch_gemv_rowwave_f16(p, group, s);
        if (hipError_t e = launch_gemv_mfma(q, s)) return e;
        b0 -= TLLM_MAX_PLAN_BATCH - q.batch;
    }
    return hipSuccess;
}

}  // namespace tllm
