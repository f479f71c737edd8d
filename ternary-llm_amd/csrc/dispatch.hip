// Kernel selection for one linear and the multi-problem plan.
#include "common.h"

namespace tllm {

hipError_t dispatch_linear(const Problem &p, int group, hipStream_t s) {
    return launch_gemv_rowwave_f16(p, group, s);
}

hipError_t plan_device_create(const std::vector<Problem> &host, PlanDevice *out) {
    PlanDevice d;
    d.count = (int)host.size();
    for (const Problem &p : host) {
        d.max_rows = p.rows > d.max_rows ? p.rows : d.max_rows;
        d.max_batch = p.batch > d.max_batch ? p.batch : d.max_batch;
    }
    if (hipError_t e = hipGetDevice(&d.device)) return e;
    if (hipError_t e = hipMalloc(&d.problems, sizeof(Problem) * host.size())) return e;
    if (hipError_t e = hipMemcpy(d.problems, host.data(), sizeof(Problem) * host.size(),
                                 hipMemcpyHostToDevice)) {
        (void)hipFree(d.problems);
        return e;
    }
    *out = d;
    return hipSuccess;
}

hipError_t plan_device_launch(const PlanDevice &plan, hipStream_t s) {
    return launch_gemv_rowwave_f16_table(plan.problems, plan.count, plan.max_rows, plan.max_batch,
                                         128, s);
}

void plan_device_destroy(PlanDevice *plan) {
    if (plan->problems) (void)hipFree(plan->problems);
    plan->problems = nullptr;
}

}  // namespace tllm
