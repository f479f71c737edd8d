// Decode GEMV on the matrix cores (gfx950), group size 128, batch 1..4.
//
// Arithmetic (reference kernels/ternary_gemv.cu:47-86): y[r] = sum_g s[r,g] * sum_{k in g} w[r,k] x[k],
// fp32 accumulation, fp16 store with round-to-nearest-even.
//
// Dataflow. A workgroup of 4 waves owns a range of rows of one matrix. Each wave owns 512-column
// slices of K: it keeps the slice's activations in 64 VGPRs as ready-made MFMA B operands and
// walks down the rows 16 at a time. Per iteration a lane loads 16 B of each mask plane (the 128
// weights of one scale group of one row, so a 16-lane group reads 64 contiguous bytes per row),
// turns them into 16 MFMA A operands with ~0.75 VALU ops per weight (see gemv_layout.h) and issues
// 16 v_mfma_f32_16x16x32_f16. The B operand of lane (k-quarter q, column j) is non-zero only when
// j % 4 == q, so output column j collects exactly one scale group (j % 4) of one batch column
// (j / 4): the per-group fp32 scale is applied to a 16x16 tile once per 4 groups. Partial sums of
// the K slices meet in LDS, one slot per wave, and are added in a fixed order (deterministic).
#include "common.h"
#include "gemv_layout.h"

namespace tllm {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int kNW = 4;  // waves per workgroup
constexpr int kThreads = kNW * kWave;
constexpr int kMaxBatch = TLLM_MAX_PLAN_BATCH;

struct Sched {
    const Problem *table;    // device table, or nullptr: use the by-value problem
    const int *task_prefix;  // [count + 1] first task of each problem
    const int *wg_first;     // [grid + 1] first task of each workgroup
    int count;
    int range_rows;   // rows per task, a multiple of 16
    int image_bytes;  // LDS bytes reserved for the activation image (the partial sums follow)
};

struct Tile {
    u4 nz, sg;
    uint16_t sc[4];
};

// Weight streams are read through global-address-space pointers (pointers fetched from the
// problem table would otherwise be treated as generic and use slower flat loads).
typedef __attribute__((address_space(1))) const uint32_t GU32;
typedef __attribute__((address_space(1))) const uint16_t GU16;
typedef __attribute__((address_space(1))) const u4 GU4;
template <class T>
__device__ __forceinline__ __attribute__((address_space(1))) const T *as_global(const T *p) {
    return (__attribute__((address_space(1))) const T *)p;
}

__device__ __forceinline__ float dpp_quad(float v, int ctrl_b1_or_4e) {
    // quad_perm swaps inside groups of 4 lanes; 0xB1 = [1,0,3,2], 0x4E = [2,3,0,1]
    int r = ctrl_b1_or_4e == 0xB1
                ? __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)
                : __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true);
    return __builtin_bit_cast(float, r);
}

__device__ __forceinline__ f4 mfma16(const uint32_t *o, u4 b, f4 c) {
    const u4 a = {o[0], o[1], o[2], o[3]};
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a),
                                                  __builtin_bit_cast(h8, b), c, 0, 0, 0);
}

// 16 rows x 512 columns: D[i][j] = 2^-24 * sum over the 128 columns of group (j % 4) of
// (w + 1) * x'' for row i and batch column j / 4.
__device__ __forceinline__ f4 slice_product(const u4 nz, const u4 sg, const u4 (&B)[kMfmaPerSlice]) {
    f4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t o[16];
        decode_word(nz[w], sg[w], o);
        d0 = mfma16(o + 0, B[4 * w + 0], d0);
        d1 = mfma16(o + 4, B[4 * w + 1], d1);
        d0 = mfma16(o + 8, B[4 * w + 2], d0);
        d1 = mfma16(o + 12, B[4 * w + 3], d1);
    }
    return d0 + d1;
}

__global__ __launch_bounds__(kThreads, 2) void gemv_mfma_kernel(Problem single, Sched sc) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    uint16_t *image = reinterpret_cast<uint16_t *>(lds);
    float *partial = reinterpret_cast<float *>(lds + sc.image_bytes);
    __shared__ uint32_t red_amax[kNW][kMaxBatch];
    __shared__ float fscale[kMaxBatch];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int li = lane & 15;  // A row / D column
    const int lq = lane >> 4;  // k quarter / D row quad

    int task_begin, task_end;
    if (sc.table) {
        task_begin = sc.wg_first[blockIdx.x];
        task_end = sc.wg_first[blockIdx.x + 1];
    } else {
        const int total = (single.rows + sc.range_rows - 1) / sc.range_rows;
        task_begin = (int)((int64_t)total * blockIdx.x / gridDim.x);
        task_end = (int)((int64_t)total * (blockIdx.x + 1) / gridDim.x);
    }

    int cur = -1;  // problem whose activations are staged
    int pi = 0;
    Problem p = single;
    int slices = 0, groups = 0, words = 0, img_stride = 0;

    for (int task = task_begin; task < task_end; task++) {
        int first_task = 0;
        if (sc.table) {
            while (sc.task_prefix[pi + 1] <= task) pi++;
            first_task = sc.task_prefix[pi];
        }
        if (pi != cur) {
            // ------------------------------------------------ stage the activations of problem pi
            if (sc.table) p = sc.table[pi];
            cur = pi;
            words = p.cols / 32;
            groups = p.cols / 128;
            slices = (p.cols + kSliceCols - 1) / kSliceCols;
            img_stride = slices * kSliceCols;
            // (a) per batch column: largest magnitude -> power-of-two normalisation
            for (int b = 0; b < p.batch; b++) {
                const uint4 *xv = reinterpret_cast<const uint4 *>(p.x + (size_t)b * p.cols);
                uint32_t m = 0;
                for (int c8 = tid; c8 < p.cols / 8; c8 += kThreads) {
                    const uint4 v = xv[c8];
                    const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        m = max(m, w4[e] & 0x7FFFu);
                        m = max(m, (w4[e] >> 16) & 0x7FFFu);
                    }
                }
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, kWave));
                if (lane == 0) red_amax[wave][b] = m;
            }
            __syncthreads();
            for (int b = 0; b < p.batch; b++) {
                uint32_t m = 0;
#pragma unroll
                for (int w = 0; w < kNW; w++) m = max(m, red_amax[w][b]);
                // amax in [2^ex, 2^(ex+1)); x'' = x * 2^(14-ex) stays below 2^15
                int ex = 0;  // all-zero activations: the image is zero whatever the exponent
                if (m >= 0x7C00u) ex = 15;  // inf/nan present: they propagate to the outputs
                else if (m) ex = (int)((__builtin_bit_cast(uint32_t, h2f((uint16_t)m)) >> 23) & 0xFF) - 127;
                if (tid == 0) fscale[b] = m ? __builtin_bit_cast(float, (uint32_t)(127 + ex + 10) << 23) : 0.0f;
                // (b) image: operand element (slice, t, q, e) = fp16(x[col] * 2^(14-ex-p))
                const uint4 *xv = reinterpret_cast<const uint4 *>(p.x + (size_t)b * p.cols);
                uint16_t *img = image + (size_t)b * img_stride;
                for (int c8 = tid; c8 < img_stride / 8; c8 += kThreads) {
                    uint4 v = {0u, 0u, 0u, 0u};
                    if (c8 * 8 < p.cols && m) v = xv[c8];
                    const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const int col = c8 * 8 + e;
                        const OperandSlot s = column_slot(col & (kSliceCols - 1));
                        const float mult = __builtin_bit_cast(float, (uint32_t)(127 + 14 - ex - s.p) << 23);
                        const uint16_t hx = (uint16_t)(w4[e >> 1] >> (16 * (e & 1)));
                        img[(col / kSliceCols) * kSliceCols + image_index(s.t, s.q, s.e)] = f2h(h2f(hx) * mult);
                    }
                }
            }
            __syncthreads();
        }

        const int r_begin = (task - first_task) * sc.range_rows;
        const int r_end = min(p.rows, r_begin + sc.range_rows);
        const int nrows = r_end - r_begin;
        const int bcol = li >> 2;               // batch column of this lane's D column
        const bool b_active = (li & 3) == lq && bcol < p.batch;
        float *my_part = partial + (size_t)wave * sc.range_rows * p.batch;
        const bool part_lane = (li & 3) == 0 && bcol < p.batch;

        // This wave's tiles: its slices (wave, wave + kNW, ...) times the 16-row blocks of the range,
        // slice-major. Tile loads are issued three tiles ahead and never branch, so the hardware
        // counters let two tiles stay in flight while one is being consumed.
        const int n_rb = (nrows + kIterRows - 1) / kIterRows;
        const int n_sl = slices > wave ? (slices - wave + kNW - 1) / kNW : 0;
        const int n_tiles = n_sl * n_rb;
        const GU32 *nz_g = as_global(p.nz);
        const GU32 *sg_g = as_global(p.sg);
        const GU16 *sc_g = as_global(p.scales);

        // Groups past the end of a row (last slice when cols % 512 != 0) are read from the row's last
        // group instead: their activations in the image are zero, so they add nothing.
        auto load_tile = [&](int slice, int rb) -> Tile {
            Tile t;
            const int ga = min(4 * slice + lq, groups - 1);
            const int gs = min(4 * slice + (li & 3), groups - 1);
            const int ra = min(rb + li, p.rows - 1);
            const size_t off = (size_t)ra * words + 4 * ga;
            t.nz = *reinterpret_cast<const GU4 *>(nz_g + off);
            t.sg = *reinterpret_cast<const GU4 *>(sg_g + off);
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int rs = min(rb + 4 * lq + v, p.rows - 1);
                t.sc[v] = sc_g[(size_t)rs * groups + gs];
            }
            return t;
        };

        u4 B[kMfmaPerSlice];
        f4 bias = {0.f, 0.f, 0.f, 0.f};
        const u4 zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int t = 0; t < kMfmaPerSlice; t++) B[t] = zero4;

        auto process = [&](const Tile &t, int slice, int rb) {
            if (rb == r_begin) {
                // new slice: its activations become the B operands (zero outside the lane's own
                // group / batch column), and an all-zero weight row gives the "+1" term of the code
                const u4 *src = reinterpret_cast<const u4 *>(image + (size_t)bcol * img_stride +
                                                             slice * kSliceCols) + lq;
                if (b_active) {
#pragma unroll
                    for (int k = 0; k < kMfmaPerSlice; k++) B[k] = src[k * 4];
                }
                bias = slice_product(zero4, zero4, B);
            }
            const f4 d = slice_product(t.nz, t.sg, B);
            float r[4];
#pragma unroll
            for (int v = 0; v < 4; v++) {
                float x = h2f(t.sc[v]) * (d[v] - bias[v]);
                x += dpp_quad(x, 0xB1);
                x += dpp_quad(x, 0x4E);
                r[v] = x;
            }
            if (part_lane) {
                const bool first_slice = slice == wave;
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    float *dst = my_part + (size_t)(rb - r_begin + 4 * lq + v) * p.batch + bcol;
                    *dst = first_slice ? r[v] : *dst + r[v];
                }
            }
        };

        if (n_tiles > 0) {
            // load cursor (ls, lrb) runs three tiles ahead of the compute cursor (cs, crb)
            int ls = wave, lrb = r_begin, cs = wave, crb = r_begin;
            auto advance = [&](int &s_, int &rb_) {
                rb_ += kIterRows;
                if (rb_ >= r_end) { rb_ = r_begin; s_ += kNW; }
            };
            auto next_load = [&]() -> Tile {
                // past the last tile the cursor is parked on it (a cached re-read, never out of range)
                const Tile t = load_tile(ls < slices ? ls : cs, ls < slices ? lrb : crb);
                if (ls < slices) advance(ls, lrb);
                return t;
            };
            Tile t0 = next_load(), t1 = next_load(), t2 = next_load();
            for (int i = 0; i < n_tiles; i += 3) {
                process(t0, cs, crb);
                advance(cs, crb);
                t0 = next_load();
                if (i + 1 >= n_tiles) break;
                process(t1, cs, crb);
                advance(cs, crb);
                t1 = next_load();
                if (i + 2 >= n_tiles) break;
                process(t2, cs, crb);
                advance(cs, crb);
                t2 = next_load();
            }
        }
        __syncthreads();
        // ------------------------------------------------ add the K slices in wave order, store fp16
        const int live = min(kNW, slices);
        for (int idx = tid; idx < nrows * p.batch; idx += kThreads) {
            const int b = idx / nrows, rl = idx - b * nrows;
            float sum = 0.0f;
            for (int w = 0; w < live; w++)
                sum += partial[((size_t)w * sc.range_rows + rl) * p.batch + b];
            p.y[(size_t)b * p.rows + r_begin + rl] = f2h(sum * fscale[b]);
        }
        __syncthreads();
    }
}

struct DeviceInfo {
    int cus = 0;
    bool attr_set = false;
};

DeviceInfo &device_info(int dev) {
    static DeviceInfo info[64];
    return info[dev < 0 || dev >= 64 ? 0 : dev];
}

constexpr int kLdsLimit = 80 * 1024;  // two workgroups per CU inside the 160 KB LDS

int round16(int v) { return (v + 15) / 16 * 16; }

hipError_t prepare_device(int *cus) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    DeviceInfo &di = device_info(dev);
    if (di.cus == 0) {
        int n = 0;
        if (hipError_t e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev)) return e;
        di.cus = n > 0 ? n : 256;
    }
    if (!di.attr_set) {
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_mfma_kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit))
            return e;
        di.attr_set = true;
    }
    *cus = di.cus;
    return hipSuccess;
}

int image_bytes_of(int cols, int batch) {
    return (cols + kSliceCols - 1) / kSliceCols * kSliceCols * 2 * batch;
}

}  // namespace

bool gemv_mfma_supports(const Problem &p, int group) {
    return group == 128 && p.batch >= 1 && p.batch <= kMaxBatch &&
           image_bytes_of(p.cols, p.batch) + kNW * 16 * p.batch * 4 <= kLdsLimit;
}

hipError_t launch_gemv_mfma(const Problem &p, hipStream_t s) {
    int cus = 0;
    if (hipError_t e = prepare_device(&cus)) return e;
    Sched sc{};
    sc.table = nullptr;
    sc.count = 1;
    sc.image_bytes = image_bytes_of(p.cols, p.batch);
    const int room = (kLdsLimit - sc.image_bytes) / (kNW * p.batch * 4) / 16 * 16;  // rows the partials can hold
    int range = round16((p.rows + 2 * cus - 1) / (2 * cus));
    range = range < 16 ? 16 : range;
    range = range > 512 ? 512 : range;
    range = range > room ? room : range;
    sc.range_rows = range;
    const int tasks = (p.rows + range - 1) / range;
    const int grid = tasks < 2 * cus ? tasks : 2 * cus;
    const size_t lds = (size_t)sc.image_bytes + (size_t)kNW * range * p.batch * 4;
    gemv_mfma_kernel<<<grid, kThreads, lds, s>>>(p, sc);
    return hipGetLastError();
}

// ------------------------------------------------------------------ multi-problem plan
hipError_t plan_device_create(const std::vector<Problem> &host, PlanDevice *out) {
    PlanDevice d;
    d.count = (int)host.size();
    if (hipError_t e = hipGetDevice(&d.device)) return e;
    int cus = 0;
    if (hipError_t e = prepare_device(&cus)) return e;

    int64_t total_rows = 0;
    int max_image = 0, max_batch = 1;
    for (const Problem &p : host) {
        total_rows += p.rows;
        const int ib = image_bytes_of(p.cols, p.batch);
        max_image = ib > max_image ? ib : max_image;
        max_batch = p.batch > max_batch ? p.batch : max_batch;
        d.max_rows = p.rows > d.max_rows ? p.rows : d.max_rows;
        d.max_batch = max_batch;
    }
    d.use_mfma = true;
    for (const Problem &p : host) d.use_mfma = d.use_mfma && gemv_mfma_supports(p, 128);
    const int room = (kLdsLimit - max_image) / (kNW * max_batch * 4) / 16 * 16;
    if (room < 16) d.use_mfma = false;

    std::vector<int> prefix(host.size() + 1, 0), wg_first;
    if (d.use_mfma) {
        // about 8 tasks per workgroup, each a multiple of 16 rows that fits the partial-sum area
        int range = round16((int)((total_rows + 16LL * cus - 1) / (16LL * cus)));
        range = range < 16 ? 16 : range;
        range = range > 512 ? 512 : range;
        range = range > room ? room : range;
        std::vector<int64_t> weight;
        for (size_t i = 0; i < host.size(); i++) {
            const int n = (host[i].rows + range - 1) / range;
            prefix[i + 1] = prefix[i] + n;
            for (int t = 0; t < n; t++) {
                const int r0 = t * range;
                const int nr = host[i].rows - r0 < range ? host[i].rows - r0 : range;
                weight.push_back((int64_t)nr * host[i].cols + 4096);  // + a fixed per-task cost
            }
        }
        const int tasks = prefix.back();
        const int grid = tasks < 2 * cus ? tasks : 2 * cus;
        int64_t total_w = 0;
        for (int64_t w : weight) total_w += w;
        // contiguous shares of about equal weight; every workgroup gets at least one task
        wg_first.assign(grid + 1, tasks);
        wg_first[0] = 0;
        int64_t acc = 0;  // weight of tasks [0, t)
        int t = 0;
        for (int g = 1; g < grid; g++) {
            const int lo = wg_first[g - 1] + 1, hi = tasks - (grid - g);
            while (t < hi && (t < lo || acc * grid < total_w * g)) acc += weight[t++];
            wg_first[g] = t;
        }
        d.grid = grid;
        d.range_rows = range;
        d.image_bytes = max_image;
        d.lds_bytes = max_image + kNW * range * max_batch * 4;
    }

    const size_t bytes_table = sizeof(Problem) * host.size();
    const size_t bytes_prefix = sizeof(int) * prefix.size();
    const size_t bytes_wg = sizeof(int) * wg_first.size();
    char *base = nullptr;
    if (hipError_t e = hipMalloc(&base, bytes_table + bytes_prefix + bytes_wg + 64)) return e;
    d.problems = reinterpret_cast<Problem *>(base);
    d.task_prefix = reinterpret_cast<int *>(base + bytes_table);
    d.wg_first = reinterpret_cast<int *>(base + bytes_table + bytes_prefix);
    hipError_t e = hipMemcpy(d.problems, host.data(), bytes_table, hipMemcpyHostToDevice);
    if (!e) e = hipMemcpy(d.task_prefix, prefix.data(), bytes_prefix, hipMemcpyHostToDevice);
    if (!e && bytes_wg) e = hipMemcpy(d.wg_first, wg_first.data(), bytes_wg, hipMemcpyHostToDevice);
    if (e) {
        (void)hipFree(base);
        return e;
    }
    *out = d;
    return hipSuccess;
}

hipError_t plan_device_launch(const PlanDevice &plan, hipStream_t s) {
    if (!plan.use_mfma)
        return launch_gemv_rowwave_f16_table(plan.problems, plan.count, plan.max_rows, plan.max_batch, 128, s);
    Sched sc{};
    sc.table = plan.problems;
    sc.task_prefix = plan.task_prefix;
    sc.wg_first = plan.wg_first;
    sc.count = plan.count;
    sc.range_rows = plan.range_rows;
    sc.image_bytes = plan.image_bytes;
    Problem none{};
    gemv_mfma_kernel<<<plan.grid, kThreads, plan.lds_bytes, s>>>(none, sc);
    return hipGetLastError();
}

void plan_device_destroy(PlanDevice *plan) {
    if (plan->problems) (void)hipFree(plan->problems);
    plan->problems = nullptr;
}

}  // namespace tllm
