// Decode GEMV on the matrix cores (gfx950), group size 128.
//
// Arithmetic (reference kernels/ternary_gemv.cu:47-86): y[r] = sum_g s[r,g] * sum_{k in g} w[r,k] x[k],
// fp32 accumulation, fp16 store with round-to-nearest-even.
//
// Dataflow. A workgroup of 4 waves owns a range of rows of one matrix; the activations of the matrix
// are staged once in LDS as ready-made MFMA B operands (power-of-two normalised, see below). The
// work of a range is cut into tiles of 64 (row, 128-column chunk) pairs: every lane loads 16 B of
// each mask plane (one chunk = one scale group of one row), turns them into 16 MFMA A operands
// with ~0.8 VALU operations per weight (gemv_layout.h) and the wave issues 16
// v_mfma_f32_16x16x32_f16. Tiles are ordered slice-major (a slice = the columns whose activations
// sit in the wave's 64 B-operand registers), split evenly over the waves, and loaded three tiles
// ahead. The B operands are sparse by construction - lane (k-quarter q, column j) is non-zero for
// one q only - so each output column of the 16x16 result collects exactly one scale group, and the
// fp32 group scale is applied to whole result tiles, not to weights. Partial sums meet in LDS,
// one slot per wave, and are added in a fixed order (deterministic).
//
// Two tile geometries:
//   Wide (batch 1):   4 rows x 2048 columns. Lanes 4a..4a+3 read 64 contiguous bytes of row a, so
//                     the loads coalesce; result column j is scale group j of the slice.
//   Tall (batch 1-4): 16 rows x 512 columns. Result column j is group j % 4 of batch column j / 4. The four
//                     scales of (row, slice) come as one 8-byte load and are transposed inside the lane quad.
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <new>

#include "common.h"
#include "gemv_layout.h"

namespace tllm {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

// Weight streams are read through global-address-space pointers (pointers fetched from the
// problem table would otherwise be treated as generic and use slower flat loads).
typedef __attribute__((address_space(1))) const uint32_t GU32;
typedef __attribute__((address_space(1))) const uint16_t GU16;
typedef __attribute__((address_space(1))) const u4 GU4;
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
// (a row of scales starts on any even byte when the number of groups is odd)
typedef __attribute__((address_space(1))) const u2 __attribute__((aligned(2))) GU2;
#define GB __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ __attribute__((address_space(1))) const T *as_global(const T *p) {
    return (__attribute__((address_space(1))) const T *)p;
}

constexpr int kNW = 4;  // waves per workgroup
// Most slices of a row (wide tiles: 2048 columns each) whose operand image is in LDS at one time;
// longer rows are staged and walked in segments. 8 slices = 32 KB keep three workgroups on a CU.
constexpr int kSegSlices = 8;
// The limit for tall tiles, in slices of 512 columns: 8192 elements of all batch columns together
// (16 KB; the partial sums need the room more).
__host__ __device__ constexpr int tall_seg_slices(int batch) { return 8192 / 512 / batch; }
constexpr int kThreads = kNW * kWave;
constexpr int kMaxBatch = 4;  // activation rows the tall tiles carry
// Outlier activations a workgroup can hold per staged row (all batch columns together); more stay in the image.
constexpr int kMaxOutliers = 64;
// kAhead of a tile geometry: tile loads in flight per wave (register ring, unrolled) = tiles per wave in a unit of work.
// Wide tiles: two, three and four give the same rate on long plans (8B sweep within 0.5 %); two make units of 32 rows
// instead of 48 and leave more registers to the rest, which takes 6 % off a single call and 5 % off the 16-layer 1B
// plan. Tall tiles: two are 9 - 11 % faster than three on the 8B sweep at two and four activation rows (one 13 % and
// four 8 % slower): units of 128 rows, and the kernel fits its 168 registers without spilling. (Since the scales of a
// tall tile come as one 8-byte load the kernel needs 157 registers and three tiles fit without spills too: still 7 - 10 %
// slower than two at two to four rows.)
struct Wide {
    static constexpr int kCols = 2048, kRows = 4, kChunks = 16, kWgPerCu = 3, kAhead = 2;
};
struct Tall {
    static constexpr int kCols = 512, kRows = 16, kChunks = 4, kWgPerCu = 3, kAhead = 2;
};

// Work is counted in units of kNW * kRows * kAhead rows of one matrix. A workgroup owns a
// contiguous span of units (of about equal weight, cut by the host) and processes it in tasks of
// up to max_units units that stay inside one matrix.
struct Sched {
    const Problem *table;    // device table, or nullptr: use the by-value problem
    const int *unit_prefix;  // [count + 1] first unit of each problem
    const int *wg_first;     // [grid + 1] first unit of each workgroup, then [grid] the problem that unit is in
    // Shared pool (large plans): tasks that belong to no span. A workgroup that has finished its
    // span takes them one at a time through counters[0]; counters[1] counts the workgroups that
    // have left, and the last one to leave sets both back to zero for the next launch. Launches of
    // one plan must therefore not overlap (they would also race on the outputs).
    const int *pool_first;  // [pool_count + 1] first unit of each pool task, then [pool_count] its problem
    int pool_count;
    int *counters;
    int count;
    int pair_stride;  // floats between the partial sums of a gate matrix and of its up matrix; 0: no pairs
    int max_units;    // units per task (bounds the partial-sum area)
    int max_batch;    // largest batch of any problem (sizes the per-wave partial-sum areas)
    int image_bytes;  // LDS bytes reserved for the activation image (the partial sums follow)
    // INT8 activations (single problem, batch 1): x points at int8 values; every output is multiplied
    // by the activation scale, given by value or read from device memory (reference
    // kernels/ternary_gemv.cu:116-216: exact integer group sums, fp32 scales).
    int x_is_i8;
    float i8_scale;
    const float *i8_scale_dev;
    // Staged plans (kExtras instances): n_stages > 0; the spans of stage s start at wg_first + s * (2 * grid + 1).
    // Between two stages the workgroups meet at a barrier in device memory (`barrier`, kBarrierInts ints, one per
    // launch slot): a workgroup whose outputs of the stage have reached memory adds one to the counter of its group of
    // kBarrierGroup workgroups; the last of a group adds one to the top counter; the last group sets the counters back
    // to zero and flips the flag word every other workgroup polls (plain loads, no read-modify-write: hundreds of
    // atomics on ONE address cost tens of microseconds here, since each is served in turn at the memory side). The flag
    // alternates from barrier to barrier and across launches; every counter is zero again when a launch ends, so a
    // replayed graph needs no clearing. Every workgroup is resident (the host sizes the grid for that); a wait gives up
    // after spin_limit polls, sets *status to the stage's number + 1, and the workgroup leaves; so do the others when
    // they see it (the host clears the barrier when it reads the status).
    int n_stages;
    int spin_limit;
    int *barrier;
    int *status;
    // How a stage sees what the stage before wrote. 0: its loads of activations and residuals ask for memory's copy
    // themselves (loads of device scope, no cache is invalidated: every problem's row is staged in one pass from
    // registers). 1: every workgroup invalidates its cache behind the barrier (any shape; costs about 2 us per stage).
    int stage_fence;
    // Hand-over without barriers (exchange != 0). A problem whose output a later stage reads also stores every
    // output row as a 32-bit word, fp16 bits | tag << 16, written through to memory (words + Problem::y_words); the
    // problems that read it poll those words with loads of device scope until every one carries the tag of this
    // launch, and take the values from them: a workgroup waits for exactly the data it needs, and the wait and the
    // transfer are one round trip. The tag is the low 16 bits of (launches of this slot so far + 1): every workgroup
    // keeps that count in a word of its own (epochs[blockIdx.x]), reads it when it starts and adds one when it
    // leaves, so all workgroups agree on it without talking, also when a captured launch is replayed. Every word is
    // rewritten by every launch, so a stale word carries the tag before. Waits are bounded as at the barrier.
    int exchange;
    uint32_t *words;
    int *epochs;
    const WgStart *starts;  // plans: [grid] (staged plans: [n_stages * grid]) what each workgroup starts (each stage) with
};
// Layout of a stage barrier, in ints: [0] the flag, [32] the top counter, [64 + 32 g] the counter of group g: every
// word that takes atomics from many workgroups sits on a 128-byte line of its own.
constexpr int kBarrierGroup = 16;
constexpr int kBarrierMaxGroups = 64;  // grids of up to 1024 workgroups
constexpr int kBarrierInts = 64 + 32 * kBarrierMaxGroups;

// The scales that travel with a tile. Wide: the one scale of the lane's (row, group). Tall: the four scales (one
// slice) of row 4 * lq + (li & 3) as one 8-byte load; the lane needs the scale of its own group li & 3 for each of the
// rows 4 * lq + v instead, which is the 4 x 4 transpose of these halfwords inside the quad (quad_scales).
template <class G>
struct Tile;
template <>
struct Tile<Wide> {
    u4 nz, sg;
    uint16_t sc[1];
};
template <>
struct Tile<Tall> {
    u4 nz, sg;
    uint32_t sc[2];
};

template <int kCtrl>
__device__ __forceinline__ float dpp_add(float v) {
    // v + (v moved across lanes by the DPP control); all lanes and banks enabled
    const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xF, 0xF, true);
    return v + __builtin_bit_cast(float, r);
}
// The largest value any lane of the wave holds, as a wave-uniform number: four DPP rotations inside the rows of 16
// lanes, then one lane of each row read into a scalar (much shorter than a butterfly of cross-lane permutes).
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t m) {
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x128, 0xF, 0xF, true));  // row_ror:8
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x124, 0xF, 0xF, true));  // row_ror:4
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x122, 0xF, 0xF, true));  // row_ror:2
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x121, 0xF, 0xF, true));  // row_ror:1
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)m, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)m, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)m, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)m, 48);
    return max(max(a, b), max(c, d));
}
// fp16 bits -> magnitude bits for a maximum that skips NaN the way fmaxf does (Inf counts)
__device__ __forceinline__ uint32_t finite_magnitude(uint32_t half_bits) {
    const uint32_t mag = half_bits & 0x7FFFu;
    return mag > 0x7C00u ? 0u : mag;
}
constexpr int kQuadSwap1 = 0xB1;       // quad_perm [1,0,3,2]
constexpr int kQuadSwap2 = 0x4E;       // quad_perm [2,3,0,1]
constexpr int kRowHalfMirror = 0x141;  // lane k <-> 7-k inside each 8 lanes
constexpr int kRowMirror = 0x140;      // lane k <-> 15-k inside each 16 lanes

// dst = mask[lane] ? b : a, with the 64-bit lane mask held in scalar registers. Written out because
// the compiler otherwise recomputes the lane compare in front of every select.
__device__ __forceinline__ float lane_select(float a, float b, uint64_t mask) {
    float r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "s"(mask));
    return r;
}

// 4 x 4 transpose of 16-bit values inside every quad of lanes. In: lane q of a quad holds a0 = (e0 | e1 << 16),
// a1 = (e2 | e3 << 16), the four elements of its row q. Out: t0 = (element q of row 0 | element q of row 1 << 16),
// t1 = the same of rows 2 and 3. Step 1 trades halfwords with lane q ^ 1 (sel: 0x05040100 in even lanes = own low half,
// partner's low half; 0x03020706 in odd lanes = partner's high half, own high half; v_perm bytes 0-3 come from the
// second operand, 4-7 from the first), step 2 trades one word with lane q ^ 2 (hi: the lanes with q >= 2).
__device__ __forceinline__ void quad_scales(uint32_t a0, uint32_t a1, uint32_t sel, uint64_t hi, uint32_t &t0, uint32_t &t1) {
    const uint32_t p0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)a0, kQuadSwap1, 0xF, 0xF, true);
    const uint32_t p1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)a1, kQuadSwap1, 0xF, 0xF, true);
    const uint32_t d0 = __builtin_amdgcn_perm(p0, a0, sel);  // rows {q & ~1, q | 1}, element (q & 1)
    const uint32_t d1 = __builtin_amdgcn_perm(p1, a1, sel);  // the same rows, element 2 + (q & 1)
    const uint32_t send = __builtin_bit_cast(uint32_t, lane_select(__builtin_bit_cast(float, d1), __builtin_bit_cast(float, d0), hi));
    const uint32_t got = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, kQuadSwap2, 0xF, 0xF, true);
    t0 = __builtin_bit_cast(uint32_t, lane_select(__builtin_bit_cast(float, d0), __builtin_bit_cast(float, got), hi));
    t1 = __builtin_bit_cast(uint32_t, lane_select(__builtin_bit_cast(float, got), __builtin_bit_cast(float, d1), hi));
}

__device__ __forceinline__ f4 mfma16(const uint32_t *o, u4 b, f4 c) {
    const u4 a = {o[0], o[1], o[2], o[3]};
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a),
                                                  __builtin_bit_cast(h8, b), c, 0, 0, 0);
}

// One tile: D[i][j] = 2^-24 * sum over the lanes' chunks that B lets through of (w + 1) * x''.
// Two accumulator chains keep dependent MFMAs apart; the caller adds them.
__device__ __forceinline__ void tile_product2(const u4 nz, const u4 sg, const u4 (&B)[kMfmaPerTile],
                                              f4 &d0, f4 &d1) {
    d0 = f4{0.f, 0.f, 0.f, 0.f};
    d1 = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t o[16];
        decode_word(nz[w], sg[w], o);
        d0 = mfma16(o + 0, B[4 * w + 0], d0);
        d1 = mfma16(o + 4, B[4 * w + 1], d1);
        d0 = mfma16(o + 8, B[4 * w + 2], d0);
        d1 = mfma16(o + 12, B[4 * w + 3], d1);
    }
}

__device__ __forceinline__ f4 tile_product(const u4 nz, const u4 sg, const u4 (&B)[kMfmaPerTile]) {
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

// Loads of device scope (they fetch memory's copy, not a line of this XCD's cache that another XCD has made stale),
// issued together and waited for inside ONE asm statement: the compiler never sees a register whose load is still in
// flight, so it cannot copy or spill one (it takes the outputs of an asm statement for complete when it ends).
__device__ __forceinline__ void load8_device_scope(const uint4 *const (&src)[8], u4 (&got)[8]) {
    asm volatile(
        "global_load_dwordx4 %0, %8, off sc1\n\t"
        "global_load_dwordx4 %1, %9, off sc1\n\t"
        "global_load_dwordx4 %2, %10, off sc1\n\t"
        "global_load_dwordx4 %3, %11, off sc1\n\t"
        "global_load_dwordx4 %4, %12, off sc1\n\t"
        "global_load_dwordx4 %5, %13, off sc1\n\t"
        "global_load_dwordx4 %6, %14, off sc1\n\t"
        "global_load_dwordx4 %7, %15, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(got[0]), "=&v"(got[1]), "=&v"(got[2]), "=&v"(got[3]), "=&v"(got[4]), "=&v"(got[5]), "=&v"(got[6]), "=&v"(got[7])
        : "v"(src[0]), "v"(src[1]), "v"(src[2]), "v"(src[3]), "v"(src[4]), "v"(src[5]), "v"(src[6]), "v"(src[7])
        : "memory");
}
// the same for four runs of eight 32-bit words (32 bytes each)
__device__ __forceinline__ void load4x8_words_device_scope(const uint32_t *const (&src)[4], u4 (&lo)[4], u4 (&hi)[4]) {
    asm volatile(
        "global_load_dwordx4 %0, %8, off sc1\n\t"
        "global_load_dwordx4 %1, %8, off offset:16 sc1\n\t"
        "global_load_dwordx4 %2, %9, off sc1\n\t"
        "global_load_dwordx4 %3, %9, off offset:16 sc1\n\t"
        "global_load_dwordx4 %4, %10, off sc1\n\t"
        "global_load_dwordx4 %5, %10, off offset:16 sc1\n\t"
        "global_load_dwordx4 %6, %11, off sc1\n\t"
        "global_load_dwordx4 %7, %11, off offset:16 sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(lo[0]), "=&v"(hi[0]), "=&v"(lo[1]), "=&v"(hi[1]), "=&v"(lo[2]), "=&v"(hi[2]), "=&v"(lo[3]), "=&v"(hi[3])
        : "v"(src[0]), "v"(src[1]), "v"(src[2]), "v"(src[3])
        : "memory");
}

// kExtras: the table may hold SwiGLU pairs and RMSNorm prologues (a separate instance, so that plans
// without them keep the register allocation of the plain kernel).
// kFine: units of one tile per wave (16 rows for wide tiles) instead of kAhead, for launches
// that would otherwise leave most of the chip's workgroup slots empty; the tile ring then runs
// across the walks of a wave and the B operands are reloaded for every tile.
template <class G, bool kExtras = false, bool kFine = false>
__global__ __launch_bounds__(kThreads, kExtras ? 2 : G::kWgPerCu) void gemv_mfma_kernel(Problem single, Sched sc) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    // [group factors | operand image | partial sums]: image_bytes counts the first two, 1 : 64 (one float per 128
    // two-byte image elements)
    float *gfac = reinterpret_cast<float *>(lds);
    uint16_t *image = reinterpret_cast<uint16_t *>(lds + sc.image_bytes / 65);
    float *partial = reinterpret_cast<float *>(lds + sc.image_bytes);
    __shared__ float red_ss[kNW];
    __shared__ float q_inv, q_scale;  // absmax quantisation of the staged problem's activations (kProblemQuantInput)
    __shared__ float fscale[kMaxBatch];
    __shared__ u4 zero_operand;  // what the idle lanes of a B operand read
    // Activations that stay out of the operand image (see stage_piece): column, fp16 bits | batch column << 16
    __shared__ int n_outliers;
    __shared__ int out_col[kMaxOutliers];
    __shared__ uint32_t out_val[kMaxOutliers];
    if (threadIdx.x == 0) zero_operand = u4{0u, 0u, 0u, 0u};

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    // the wave index is uniform inside a wave: say so, or every loop counter and tile address that
    // depends on it is computed per lane in vector registers
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15;  // MFMA A row / D column
    const int lq = lane >> 4;  // MFMA k quarter / D row quad

    // (Fine-grained wide tiles in units of 8 rows, where the waves share out the slices of two row blocks, were
    // measured: a 4096 x 14336 matrix then spreads over twice the workgroups and every wave fetches half the tiles,
    // but twice as many workgroups stage the 28 KB of activations, and a call takes the same time.)
    constexpr int kUnitRows = kNW * G::kRows * (kFine ? 1 : G::kAhead);
    constexpr int kChunkStep = G::kRows * (kFine ? 1 : G::kAhead);  // a wave's share of a task's rows is a multiple of this
    int u = 0, u_end = 0, pi = 0;
    if (sc.table) {
        // (plans: the span, its place among the units and the problem come in one record, below)
    } else {
        const int total = (single.rows + kUnitRows - 1) / kUnitRows;
        u = (int)((int64_t)total * blockIdx.x / gridDim.x);
        u_end = (int)((int64_t)total * (blockIdx.x + 1) / gridDim.x);
    }

    int cur = -1;      // problem whose activations are staged
    int cur_seg = -1;  // and which segment of its columns
    constexpr int kSegBatch = G::kRows == 4 ? 1 : kMaxBatch;
    Problem p = single;
    int slices = 0, groups = 0, words = 0, img_stride = 0;
    int seg_lo = 0, seg_n = 0;  // slices of the staged segment

    __shared__ int pool_task;
    __shared__ int stage_reached;
    // the flag of the stage barrier as this launch finds it (only thread 0 uses it): no workgroup can flip it before
    // every workgroup has read it here, because flipping takes the arrival of all of them
    int barrier_sense = 0;
    if (kExtras && sc.n_stages > 1 && !sc.exchange && tid == 0) barrier_sense = __hip_atomic_load(sc.barrier, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int n_stages = kExtras && sc.n_stages > 0 ? sc.n_stages : 1;
    const bool staged = kExtras && sc.n_stages > 0;
    const bool exchange = staged && sc.exchange != 0;
    uint32_t epoch = 0;  // (launches of this slot so far; counted modulo 2^32, used modulo 2^16)
    if (exchange) epoch = (uint32_t)sc.epochs[blockIdx.x];
    const uint32_t tag_hi = ((epoch + 1u) & 0xFFFFu) << 16;
    bool gave_up = false;  // a bounded wait of this workgroup expired (the same value in every thread)
    for (int stage = 0; stage < n_stages; stage++) {
    bool from_record = false;  // the first task of the stage takes its problem and unit numbers from the record
    int rec_first = 0, rec_units = 0;
    Problem rec_p = single;
    if (sc.table) {
        // one round trip to memory instead of three dependent ones (the span, the unit prefix around it, the problem)
        const WgStart &ws = sc.starts[(size_t)stage * gridDim.x + blockIdx.x];
        u = ws.u;
        u_end = ws.u_end;
        pi = ws.pi;
        rec_first = ws.first_unit;
        rec_units = ws.p_units;
        rec_p = ws.p;
        from_record = true;
    }
    for (;;) {
        if (u >= u_end) {
            // The span (or pool task) is done: go on with the pool task that was asked for when the
            // walks of the task before ended. The two barriers that end a task lie between the write
            // of pool_task and this read, and between this read and the next write.
            if (sc.pool_count == 0) break;
            const int t = __builtin_amdgcn_readfirstlane(pool_task);
            if (t >= sc.pool_count) break;
            u = sc.pool_first[t];
            u_end = sc.pool_first[t + 1];
            pi = sc.pool_first[sc.pool_count + 1 + t];
        }
        int first_unit = 0;
        int p_units = (single.rows + kUnitRows - 1) / kUnitRows;
        if (from_record) {
            first_unit = rec_first;
            p_units = rec_units;
        } else if (sc.table) {
            while (sc.unit_prefix[pi + 1] <= u) pi++;
            first_unit = sc.unit_prefix[pi];
            p_units = sc.unit_prefix[pi + 1] - first_unit;
        }
        const bool with_record = from_record;
        from_record = false;
        const int n_units = min(min(u_end - u, first_unit + p_units - u), sc.max_units);
        const int task_first_row = (u - first_unit) * kUnitRows;
        u += n_units;
        const bool fresh = pi != cur;
        if (fresh) {
            if (with_record) p = rec_p;
            else if (sc.table) p = sc.table[pi];
            cur = pi;
            cur_seg = -1;
            words = p.cols / 32;
            groups = p.cols / kChunkCols;
            slices = (p.cols + G::kCols - 1) / G::kCols;
        }
        // Rows longer than kSegSlices slices are staged and walked in segments of equal length, so
        // that the operand image never takes more than kSegSlices slices of LDS (wide tiles only).
        // (fine-grained wide-tile instances: whole rows, the host sees to it that they fit)
        const int seg_max = G::kRows == 4 ? kSegSlices : tall_seg_slices(p.batch);
        const int n_seg = kFine && G::kRows == 4 ? 1 : (slices + seg_max - 1) / seg_max;
        const int seg_len = (slices + n_seg - 1) / n_seg;

        const int r_begin = task_first_row;
        const int r_end = min(p.rows, r_begin + n_units * kUnitRows);
        const bool pair = kExtras && (p.flags & kProblemSwigluGate) != 0;
        const size_t wave_stride = (size_t)(sc.max_units * kUnitRows) * sc.max_batch;
        for (int mat = 0; mat < (pair ? 2 : 1); mat++) {
            float *part = partial + (size_t)mat * sc.pair_stride + (size_t)wave * wave_stride;
            for (int k = lane; k < n_units * kUnitRows * p.batch; k += kWave) part[k] = 0.0f;
        }
        for (int seg = 0; seg < n_seg; seg++) {
        if (seg != cur_seg) {
            // ------------------------------------------------ stage the activations of problem pi
            // (the list of outliers belongs to the whole row: it starts again with the row's first segment; the
            // barrier that ended the task before lies between its last reader and this write)
            if (seg == 0 && tid == 0) n_outliers = 0;
            if (kExtras && tid == 0) stage_reached = 1;  // (a wave whose wait for tagged words expires clears it)
            __syncthreads();  // every wave is done with the image that was staged before
            cur_seg = seg;
            seg_lo = seg * seg_len;
            seg_n = min(seg_len, slices - seg_lo);
            img_stride = seg_n * G::kCols;
            // Activations that the launch quantises itself (reference kernels/activations.cu:100-141): the largest
            // magnitude of the whole row first (one pass, also for rows staged in segments: when the row's first
            // segment is staged), then every element becomes the integer the quantisation gives it, as an fp16
            // number, and the kernel goes on as for int8 input.
            const bool quant = (p.flags & kProblemQuantInput) != 0;
            // (rows that the one-pass staging below keeps in registers find their maximum there, without a second read)
            const bool quant_from_registers = quant && n_seg == 1 && p.batch == 1 && img_stride / 8 <= 8 * kThreads;
            if (quant && seg == 0 && !quant_from_registers) {
                // (the magnitudes compare as their fp16 bit patterns; NaN is skipped, as fmaxf skips it)
                uint32_t m = 0;
                for (int c8 = tid; c8 < p.cols / 8; c8 += kThreads) {
                    const uint4 v = reinterpret_cast<const uint4 *>(p.x)[c8];
                    const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) m = max(m, max(finite_magnitude(w4[e]), finite_magnitude(w4[e] >> 16)));
                }
                m = wave_max_u32(m);
                if (lane == 0) red_ss[wave] = h2f((uint16_t)m);
                __syncthreads();
                if (tid == 0) {
                    float amax = 0.0f;
#pragma unroll
                    for (int w = 0; w < kNW; w++) amax = fmaxf(amax, red_ss[w]);
                    q_inv = amax > 0.0f ? 127.0f / amax : 0.0f;
                    q_scale = amax > 0.0f ? amax / 127.0f : 1.0f;
                }
                __syncthreads();
            }
            const float quant_inv = quant && !quant_from_registers ? q_inv : 0.0f;
            // eight fp16 activations -> the integers the quantisation gives them, as fp16 numbers (exact)
            auto quantised = [](const uint4 &v, float inv) -> uint4 {
                const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
                uint32_t h[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    // (no clamp needed: |x| <= amax and inv = fl(127 / amax) keep the product within 127 (1 + 2^-23), which
                    // rounds to 127; a non-finite x gives NaN here and the conversion to int makes it 0, as in the quantiser)
                    const int r = (int)rintf(h2f((uint16_t)(w4[e >> 1] >> (16 * (e & 1)))) * inv);
                    h[e] = f2h((float)r);
                }
                return uint4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
            };
            // eight consecutive activations as fp16 bits; int8 values convert exactly
            auto load8 = [&](int b, int c8) -> uint4 {
                if (!sc.x_is_i8) {
                    const uint4 v = reinterpret_cast<const uint4 *>(p.x + (size_t)b * p.cols)[c8];
                    return quant && !quant_from_registers ? quantised(v, quant_inv) : v;
                }
                const uint2 q = reinterpret_cast<const uint2 *>(p.x)[c8];
                const uint32_t w2[2] = {q.x, q.y};
                uint32_t h[8];
#pragma unroll
                for (int e = 0; e < 8; e++) h[e] = f2h((float)(int8_t)(w2[e >> 2] >> (8 * (e & 3))));
                return uint4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
            };
            // Image element (slice, t, chunk, e) = fp16(x[col] * 2^(14-ex-p)), where 2^ex is the power
            // of two at or below the largest magnitude of the element's SCALE GROUP (its 128-column chunk): every
            // group is normalised by itself, so an outlier activation costs precision only inside its own group (a
            // result column of the matrix product collects exactly one group, and 2^(ex+10) of the group joins its
            // fp32 scale when the column is taken out of the accumulators). The last slice of a row
            // that is not a whole number of slices is moved left so that it ends with the row; the
            // chunks it then shares with the slice before it are zero in the image. Eight-element
            // pieces are numbered in image order; piece_of() loads the activations of one.
            const int pieces = img_stride / 8;
            auto piece_of = [&](int b, int c8) -> uint4 {
                const int slice = seg_lo + (c8 * 8) / G::kCols;
                const int chunk = ((c8 * 8) % G::kCols) / kChunkCols;
                const int g = min(slice * G::kChunks, groups - G::kChunks) + chunk;
                if (g < slice * G::kChunks) return uint4{0u, 0u, 0u, 0u};
                return load8(b, (g * kChunkCols + (c8 * 8) % kChunkCols) / 8);
            };
            // the RMSNorm weights of the columns of piece c8 (zero where the piece is a duplicate)
            auto norm_piece = [&](int c8) -> uint4 {
                const int slice = (c8 * 8) / G::kCols;
                const int chunk = ((c8 * 8) % G::kCols) / kChunkCols;
                const int g = min(slice * G::kChunks, groups - G::kChunks) + chunk;
                if (g < slice * G::kChunks) return uint4{0u, 0u, 0u, 0u};
                return reinterpret_cast<const uint4 *>(p.norm_w)[(g * kChunkCols + (c8 * 8) % kChunkCols) / 8];
            };
            auto magnitude = [](uint32_t m, const uint4 &v) -> uint32_t {
                const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    m = max(m, w4[e] & 0x7FFFu);
                    m = max(m, (w4[e] >> 16) & 0x7FFFu);
                }
                return m;
            };
            auto write_piece = [&](uint16_t *img, int c8, const uint4 &v, int ex) {
                const int slice = (c8 * 8) / G::kCols;
                const int chunk = ((c8 * 8) % G::kCols) / kChunkCols;
                const int cc0 = (c8 * 8) % kChunkCols;
                const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
                uint16_t *dst = img + slice * G::kCols;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const OperandSlot s = chunk_slot(cc0 + e);
                    const float mult = __builtin_bit_cast(float, (uint32_t)(127 + 14 - ex - s.p) << 23);
                    const uint16_t hx = (uint16_t)(w4[e >> 1] >> (16 * (e & 1)));
                    dst[image_index(s.t, chunk, s.e, G::kChunks)] = f2h(h2f(hx) * mult);
                }
            };
            // One piece into the image. The 16 pieces of a 128-column group are held by 16 neighbouring threads
            // (one DPP row), whatever the staging path.
            // Outliers first. The matrix product sees the codes w + 1, so an activation also enters the fp32 sums of
            // the rows whose weight on its column is ZERO, to be cancelled against the all-zero-row product later:
            // that costs every such row about 2^-21 of the activation's magnitude, too much once it is some hundred
            // times the magnitude of its neighbours, and it would carry an Inf or NaN into every row. An element more
            // than 2^8 times the smallest non-zero piece maximum of its group (a robust "typical magnitude"; Inf and
            // NaN always) therefore stays OUT of the image: it goes to a short list, and the epilogue adds
            // scale * w * x for it to the rows that hold a weight there, term by term in fp32 like the reference
            // (kernels/ternary_gemv.cu:60-82). When the list is full the element stays in the image.
            // Then the exponent of the group's largest remaining magnitude; 2^(ex+10) goes to the table of group
            // factors (the image of an all-zero group is zero whatever the exponent).
            auto stage_piece = [&](int b, int c8, uint4 v) {
                uint32_t m = magnitude(0u, v);
                uint32_t t = m ? m : 0xFFFFu;
                t = min(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x128, 0xF, 0xF, true));  // row_ror:8
                t = min(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x124, 0xF, 0xF, true));  // row_ror:4
                t = min(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x122, 0xF, 0xF, true));  // row_ror:2
                t = min(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x121, 0xF, 0xF, true));  // row_ror:1
                const uint32_t limit = min(t + (8u << 10), 0x7BFFu);  // fp16 bits: 2^8 times t, at most the largest finite number
                if (m > limit) {
                    const int slice = seg_lo + (c8 * 8) / G::kCols;
                    const int chunk = ((c8 * 8) % G::kCols) / kChunkCols;
                    const int col0 = (min(slice * G::kChunks, groups - G::kChunks) + chunk) * kChunkCols + (c8 * 8) % kChunkCols;
                    uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const uint32_t bits = (w4[e >> 1] >> (16 * (e & 1))) & 0xFFFFu;
                        if ((bits & 0x7FFFu) > limit) {
                            const int slot = __hip_atomic_fetch_add(&n_outliers, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                            if (slot < kMaxOutliers) {
                                out_col[slot] = col0 + e;
                                out_val[slot] = bits | (uint32_t)b << 16;
                                w4[e >> 1] &= ~(0xFFFFu << (16 * (e & 1)));
                            }
                        }
                    }
                    v = uint4{w4[0], w4[1], w4[2], w4[3]};
                    m = magnitude(0u, v);
                }
                m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x128, 0xF, 0xF, true));
                m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x124, 0xF, 0xF, true));
                m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x122, 0xF, 0xF, true));
                m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x121, 0xF, 0xF, true));
                // amax in [2^ex, 2^(ex+1)); x'' = x * 2^(14-ex) stays below 2^15
                int ex = 0;
                if (m >= 0x7C00u) ex = 15;  // inf/nan left in the image (full list): they propagate to every output
                else if (m) ex = (int)((__builtin_bit_cast(uint32_t, h2f((uint16_t)m)) >> 23) & 0xFF) - 127;
                if ((c8 & 15) == 0) gfac[b * (pieces / 16) + c8 / 16] = __builtin_bit_cast(float, (uint32_t)(127 + ex + 10) << 23);
                write_piece(image + (size_t)b * img_stride, c8, v, ex);
            };
            // what every output of a batch column is multiplied with at the end: the activation scale of int8 input
            if (tid < kMaxBatch) {
                float f = 1.0f;
                if (sc.x_is_i8) f = sc.table ? *p.x_scale : (sc.i8_scale_dev ? *sc.i8_scale_dev : sc.i8_scale);
                if (quant && !quant_from_registers) f = q_scale;
                fscale[tid] = f;  // (rows quantised from registers: set there)
            }
            // The piece addresses depend on the thread index only; hidden behind an empty asm they are
            // worked out here, each time, instead of living in registers across the whole kernel.
            int stid = tid;
            asm volatile("" : "+v"(stid));
            constexpr int kKeep = 8;  // pieces per thread that stay in registers between the two steps
            if (n_seg == 1 && p.batch == 1 && pieces <= kKeep * kThreads) {
                // one pass over x: all loads are issued together and kept for the image
                uint4 keep[kKeep];
                // RMSNorm prologue on a row of up to 8192 columns: the norm weights are asked for now, with (or before)
                // the activations, not after the sum of squares: one round trip to memory less
                uint4 early_w[kKeep / 2];
                const bool early_norm = kExtras && p.norm_w != nullptr && pieces <= (kKeep / 2) * kThreads;
                if (early_norm) {
#pragma unroll
                    for (int k = 0; k < kKeep / 2; k++) {
                        const int c8 = stid + k * kThreads;
                        early_w[k] = c8 < pieces ? norm_piece(c8) : uint4{0u, 0u, 0u, 0u};
                    }
                }
                if (kExtras && exchange && p.x_words >= 0) {
                    // The activations are the tagged words of an earlier stage: eight words per piece, asked for
                    // again until all of this wave's carry the tag of this launch (four pieces at a time: 32
                    // registers in flight). The fp16 bits are then packed into the piece as if loaded from x.
                    const uint32_t *xw = sc.words + p.x_words;
                    bool wave_ok = true;
#pragma unroll
                    for (int half = 0; half < 2; half++) {
                        u4 lo[kKeep / 2], hi[kKeep / 2];
                        for (int spins = wave_ok ? 0 : sc.spin_limit;; spins++) {  // (a wave that has given up asks once more, no longer)
                            uint32_t bad = 0;
                            const uint32_t *src[kKeep / 2];
                            bool live[kKeep / 2];
#pragma unroll
                            for (int k = 0; k < kKeep / 2; k++) {
                                const int c8 = stid + (half * (kKeep / 2) + k) * kThreads;
                                const int slice = seg_lo + (c8 * 8) / G::kCols;
                                const int chunk = ((c8 * 8) % G::kCols) / kChunkCols;
                                const int g = min(slice * G::kChunks, groups - G::kChunks) + chunk;
                                live[k] = c8 < pieces && g >= slice * G::kChunks;
                                // (pieces that are not needed load the row's first words and count as zeros)
                                src[k] = live[k] ? xw + g * kChunkCols + (c8 * 8) % kChunkCols : xw;
                            }
                            load4x8_words_device_scope(src, lo, hi);
#pragma unroll
                            for (int k = 0; k < kKeep / 2; k++) {
                                if (!live[k]) lo[k] = hi[k] = u4{tag_hi, tag_hi, tag_hi, tag_hi};
#pragma unroll
                                for (int e = 0; e < 4; e++) bad |= (lo[k][e] ^ tag_hi) | (hi[k][e] ^ tag_hi);
                            }
                            if (__builtin_amdgcn_ballot_w64((bad >> 16) != 0) == 0) break;  // (uniform in the wave)
                            if (spins >= sc.spin_limit ||
                                ((spins & 15) == 15 && __hip_atomic_load(sc.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
                                wave_ok = false;
                                break;
                            }
                            __builtin_amdgcn_s_sleep(2);
                        }
#pragma unroll
                        for (int k = 0; k < kKeep / 2; k++)
                            keep[half * (kKeep / 2) + k] = uint4{__builtin_amdgcn_perm(lo[k][1], lo[k][0], 0x05040100u),
                                                                 __builtin_amdgcn_perm(lo[k][3], lo[k][2], 0x05040100u),
                                                                 __builtin_amdgcn_perm(hi[k][1], hi[k][0], 0x05040100u),
                                                                 __builtin_amdgcn_perm(hi[k][3], hi[k][2], 0x05040100u)};
                        if (pieces <= (kKeep / 2) * kThreads) {  // (rows of up to 8192 columns: the second half holds nothing)
#pragma unroll
                            for (int k = kKeep / 2; k < kKeep; k++) keep[k] = uint4{0u, 0u, 0u, 0u};
                            break;
                        }
                    }
                    if (!wave_ok && lane == 0) stage_reached = 0;
                } else if (kExtras && staged && !exchange && !sc.stage_fence) {
                    // The stage before wrote these activations, maybe on another XCD: loads of device scope fetch
                    // memory's copy instead of a stale line of this XCD's cache.
                    u4 got[kKeep];
                    const uint4 *src[kKeep];
                    bool live[kKeep];
#pragma unroll
                    for (int k = 0; k < kKeep; k++) {
                        const int c8 = stid + k * kThreads;
                        const int slice = seg_lo + (c8 * 8) / G::kCols;
                        const int chunk = ((c8 * 8) % G::kCols) / kChunkCols;
                        const int g = min(slice * G::kChunks, groups - G::kChunks) + chunk;
                        live[k] = c8 < pieces && g >= slice * G::kChunks;
                        // (pieces that are not needed load the row's first one and become zeros)
                        src[k] = reinterpret_cast<const uint4 *>(p.x) + (live[k] ? (g * kChunkCols + (c8 * 8) % kChunkCols) / 8 : 0);
                    }
                    load8_device_scope(src, got);
#pragma unroll
                    for (int k = 0; k < kKeep; k++) keep[k] = live[k] ? uint4{got[k][0], got[k][1], got[k][2], got[k][3]} : uint4{0u, 0u, 0u, 0u};
                } else {
#pragma unroll
                for (int k = 0; k < kKeep; k++) {
                    const int c8 = stid + k * kThreads;
                    keep[k] = c8 < pieces ? piece_of(0, c8) : uint4{0u, 0u, 0u, 0u};
                }
                }
                if (kExtras && p.norm_w) {
                    // RMSNorm prologue, reference kernels/rmsnorm.cu:20-106 without residual: the kept
                    // pieces become fp16(x * rsqrt(mean x^2 + eps) * w). Same sums in the same order as
                    // the stand-alone operator (elementwise.hip), so both give the same bits.
                    float ss = 0.0f;
#pragma unroll
                    for (int k = 0; k < kKeep; k++) {
                        const uint32_t w4[4] = {keep[k].x, keep[k].y, keep[k].z, keep[k].w};
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float lo = h2f((uint16_t)w4[e]), hi = h2f((uint16_t)(w4[e] >> 16));
                            ss = __builtin_fmaf(lo, lo, ss);
                            ss = __builtin_fmaf(hi, hi, ss);
                        }
                        __builtin_amdgcn_sched_barrier(0);  // piece by piece: few registers
                    }
                    ss = wave_sum(ss);
                    if (lane == 0) red_ss[wave] = ss;
                    __syncthreads();
                    float total = 0.0f;
#pragma unroll
                    for (int w = 0; w < kNW; w++) total += red_ss[w];
                    const float inv = 1.0f / sqrtf(total / (float)p.cols + p.eps);
                    // the weights come in two batches of loads, to keep the register need of this
                    // rarely run code below that of the tile loop
#pragma unroll
                    for (int half = 0; half < 2; half++) {
                        if (early_norm && half == 1) break;  // (nothing in the second half of the pieces)
                        uint4 wk[kKeep / 2];
#pragma unroll
                        for (int k = 0; k < kKeep / 2; k++) {
                            const int c8 = stid + (half * (kKeep / 2) + k) * kThreads;
                            if (early_norm) wk[k] = early_w[k];
                            else wk[k] = c8 < pieces ? norm_piece(c8) : uint4{0u, 0u, 0u, 0u};
                        }
#pragma unroll
                        for (int k = 0; k < kKeep / 2; k++) {
                            uint4 &x = keep[half * (kKeep / 2) + k];
                            const uint32_t x4[4] = {x.x, x.y, x.z, x.w};
                            const uint32_t n4[4] = {wk[k].x, wk[k].y, wk[k].z, wk[k].w};
                            uint32_t o[4];
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                o[e] = (uint32_t)f2h_of_rounded(h2f((uint16_t)x4[e]) * inv * h2f((uint16_t)n4[e])) |
                                       (uint32_t)f2h_of_rounded(h2f((uint16_t)(x4[e] >> 16)) * inv * h2f((uint16_t)(n4[e] >> 16))) << 16;
                            x = uint4{o[0], o[1], o[2], o[3]};
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
                if (quant_from_registers) {
                    // absmax quantisation of the kept pieces (pieces a moved-back last slice repeats are zeros here
                    // and their originals are among the others: the maximum is the row's)
                    uint32_t m = 0;
#pragma unroll
                    for (int k = 0; k < kKeep; k++) {
                        const uint32_t w4[4] = {keep[k].x, keep[k].y, keep[k].z, keep[k].w};
#pragma unroll
                        for (int e = 0; e < 4; e++) m = max(m, max(finite_magnitude(w4[e]), finite_magnitude(w4[e] >> 16)));
                    }
                    m = wave_max_u32(m);
                    if (lane == 0) red_ss[wave] = h2f((uint16_t)m);
                    __syncthreads();
                    float amax = 0.0f;
#pragma unroll
                    for (int w = 0; w < kNW; w++) amax = fmaxf(amax, red_ss[w]);
                    const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
                    if (tid == 0) fscale[0] = amax > 0.0f ? amax / 127.0f : 1.0f;
#pragma unroll
                    for (int k = 0; k < kKeep; k++) {
                        if (stid + k * kThreads < pieces) keep[k] = quantised(keep[k], inv);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
#pragma unroll
                for (int k = 0; k < kKeep; k++) {
                    const int c8 = stid + k * kThreads;
                    if (c8 < pieces) stage_piece(0, c8, keep[k]);
                    __builtin_amdgcn_sched_barrier(0);  // one piece at a time: keeps the register need low
                }
            } else if constexpr (kFine && G::kRows == 4) {
                // a whole row too long for the registers (the fine-grained instances do not stage in
                // segments): piece by piece (the trip count is the same for the 16 threads of a group)
                for (int c8 = stid; c8 < pieces; c8 += kThreads) stage_piece(0, c8, piece_of(0, c8));
            } else {
                // Long rows or several batch columns. The (column, piece) pairs are numbered column-major and
                // taken kFlat * kThreads at a time, so that a thread has kFlat loads in flight whatever the shape
                // (the pieces of a column are a multiple of 16, so the 16 threads of a DPP row always hold one group).
                constexpr int kFlat = G::kRows == 4 ? kKeep / 2 : kKeep;  // loads in flight per thread (wide tiles: fewer registers to spare)
                auto column_of = [&](int item, int per_col) -> int {  // item / per_col for at most kSegBatch columns
                    int b = 0;
#pragma unroll
                    for (int c = 1; c < kSegBatch; c++) b += item >= c * per_col;
                    return b;
                };
                const int items = pieces * p.batch;
                for (int base = 0; base < items; base += kFlat * kThreads) {
                    uint4 kp[kFlat];
#pragma unroll
                    for (int k = 0; k < kFlat; k++) {
                        const int item = base + stid + k * kThreads;
                        const int b = column_of(item, pieces);
                        kp[k] = item < items ? piece_of(b, item - b * pieces) : uint4{0u, 0u, 0u, 0u};
                    }
#pragma unroll
                    for (int k = 0; k < kFlat; k++) {
                        const int item = base + stid + k * kThreads;
                        const int b = column_of(item, pieces);
                        if (item < items) stage_piece(b, item - b * pieces, kp[k]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            __syncthreads();
            if (kExtras && exchange && !stage_reached) {  // (the same in every thread: read behind the barrier)
                gave_up = true;
                break;
            }
        }

        // The task's rows are cut into kNW chunks; a "walk" is one chunk under one slice (the B
        // operands stay put during a walk). Walks are numbered chunk-major, slice-minor and dealt to
        // the waves round-robin, so at any time the waves of a workgroup work on neighbouring
        // slices of the same rows: the cache lines of a row (masks and, above all, the 2-byte
        // scales) are fetched from HBM once and shared, not once per slice.
        // chunk size: a quarter of the rows that exist, rounded up to whole groups of G::kAhead tiles
        const int chunk_rows = ((r_end - r_begin + kNW - 1) / kNW + kChunkStep - 1) / kChunkStep * kChunkStep;
        const int n_walks = kNW * seg_n;
        const int my_walks = seg_n;  // walks wave, wave + kNW, ...
        // fine-grained instances: only the walks of chunks that have rows (the first ones of every wave)
        const int live_walks = (r_end - r_begin + chunk_rows - 1) / chunk_rows * seg_n;
        const int my_live = max(0, (live_walks - wave + kNW - 1) / kNW);
        const int park_walk = kFine ? wave + (max(my_live, 1) - 1) * kNW : n_walks - kNW + wave;
        // A SwiGLU pair (flag on the gate problem; the up problem follows it in the table, same shape
        // and activations, no units of its own) runs the walks twice over the same rows, with the same
        // operand image, into two partial-sum areas; the epilogue below joins them.
        // (The fine-grained instance that knows pairs takes both matrices in ONE pass, below: the tiles of gate and
        // up travel through the same ring, so a unit's four tiles at K = 4096 are one round trip to memory, not two.)
        constexpr bool kBothInOnePass = kFine && kExtras && G::kRows == 4;
        for (int mat = 0; mat < (pair && !kBothInOnePass ? 2 : 1); mat++) {
        const uint32_t *w_nz = p.nz, *w_sg = p.sg;
        const uint16_t *w_sc = p.scales;
        if (mat == 1) {
            w_nz = sc.table[pi + 1].nz;
            w_sg = sc.table[pi + 1].sg;
            w_sc = sc.table[pi + 1].scales;
        }
        float *my_part = partial + (size_t)mat * sc.pair_stride + (size_t)wave * wave_stride;

        // ---- which operand lanes are live, and what each lane loads
        int bcol;       // batch column of this lane's D column
        bool b_active;  // this lane's B operand is non-zero
        int b_chunk;    // chunk (of the slice) the lane's B operand holds
        int a_chunk;    // chunk (of the slice) whose weights the lane loads
        int a_row;      // row (of the tile) whose weights the lane loads
        if constexpr (G::kRows == 4) {
            bcol = 0;
            b_active = lq == (li >> 2);
            b_chunk = li;
            a_chunk = 4 * lq + (lane & 3);
            a_row = (lane >> 2) & 3;
        } else {
            bcol = li >> 2;
            b_active = (li & 3) == lq && bcol < p.batch;
            b_chunk = lq;
            a_chunk = lq;
            a_row = li;
        }

        // Tile addresses: a wave-uniform base (row block, slice) plus a per-lane offset that never
        // changes, so the hot loop spends no vector operations on addressing. The last row block and
        // the last slice are moved back to end exactly at the matrix edge (rows >= kRows and
        // groups >= kChunks are guaranteed by the dispatcher); the rows such a block repeats are
        // dropped again in the epilogue, the repeated columns are zero in the image.
        const char GB *nz_g = reinterpret_cast<const char GB *>(as_global(w_nz));
        const char GB *sg_g = reinterpret_cast<const char GB *>(as_global(w_sg));
        const char GB *sc_g = reinterpret_cast<const char GB *>(as_global(w_sc));
        const uint32_t lane_a = ((uint32_t)a_row * words + 4u * a_chunk) * 4u;
        const uint32_t lane_s = G::kRows == 4 ? ((uint32_t)lq * groups + li) * 2u
                                              : (uint32_t)(4 * lq + (li & 3)) * groups * 2u;

        auto load_tile = [&](int slice, int rb) -> Tile<G> {
            Tile<G> t;
            const int rbe = min(rb, p.rows - G::kRows);
            const int c0 = min((seg_lo + slice) * G::kChunks, groups - G::kChunks);
            const size_t base_a = ((size_t)rbe * words + (size_t)c0 * 4) * 4;
            const size_t base_s = ((size_t)rbe * groups + c0) * 2;
            if constexpr (G::kRows == 4) {
                // wide tiles read every mask line once, whole (a quad of lanes = 64 bytes, the next quad the
                // rest of the line): streamed past the caches. Tall tiles come back to a line for the next
                // slice and keep ordinary loads (non-temporal ones cost them 12 %).
                t.nz = TLLM_STREAM_LOAD(reinterpret_cast<const GU4 *>(nz_g + base_a + lane_a));
                t.sg = TLLM_STREAM_LOAD(reinterpret_cast<const GU4 *>(sg_g + base_a + lane_a));
            } else {
                t.nz = *reinterpret_cast<const GU4 *>(nz_g + base_a + lane_a);
                t.sg = *reinterpret_cast<const GU4 *>(sg_g + base_a + lane_a);
            }
            if constexpr (G::kRows == 4) {
                t.sc[0] = *reinterpret_cast<const GU16 *>(sc_g + base_s + lane_s);
            } else {
                // (a slice starts on a multiple of four groups: 8-byte aligned when the scale array is)
                const u2 w = *reinterpret_cast<const GU2 *>(sc_g + base_s + lane_s);
                t.sc[0] = w[0];
                t.sc[1] = w[1];
            }
            return t;
        };

        // rows of chunk c that exist, as a number of tiles; slots round that up to whole groups of
        // G::kAhead (slots past the live tiles re-read the last one, their results are dropped)
        auto chunk_tiles = [&](int c) -> int {
            const int rows_c = max(0, min(r_end - (r_begin + c * chunk_rows), chunk_rows));
            return (rows_c + G::kRows - 1) / G::kRows;
        };
        const int n_slots = chunk_rows / G::kRows;  // a multiple of G::kAhead

        {
            // Load cursor over this wave's walks; it runs G::kAhead slots ahead of the compute
            // loop, across walks. Walks of chunks without rows are skipped by both cursors alike.
            int l_walk = wave, l_slot = 0;
            auto next_load = [&]() -> Tile<G> {
                // past the last walk the cursor parks on the wave's last tile
                const int w_ = min(l_walk, park_walk);
                const int c = w_ / seg_n, sl = w_ - c * seg_n;
                const int live_tiles = max(chunk_tiles(c), 1);
                const Tile<G> t = load_tile(sl, r_begin + c * chunk_rows + min(l_slot, live_tiles - 1) * G::kRows);
                if (++l_slot == n_slots) { l_slot = 0; l_walk += kNW; }
                return t;
            };
            Tile<G> ring[G::kAhead];
            if constexpr (!kBothInOnePass) {
#pragma unroll
                for (int k = 0; k < G::kAhead; k++) {
                    ring[k] = next_load();
                    __builtin_amdgcn_sched_barrier(0);  // same issue order as in the loop below
                }
            }

            const u4 zero4 = {0u, 0u, 0u, 0u};
            // lanes whose result row (li & 3) is odd / is 2 or 3 (wide tiles pick one of four D rows)
            const uint64_t odd_lanes = __builtin_amdgcn_ballot_w64((li & 1) != 0);
            const uint64_t hi_lanes = __builtin_amdgcn_ballot_w64((li & 2) != 0);
            // tall tiles, transpose of the scales: byte selector of the first step, lanes of the second
            const uint32_t quad_sel = (li & 1) ? 0x03020706u : 0x05040100u;
            const uint64_t quad_hi = hi_lanes;
            // tall tiles: the lane adds the results of rows 4 lq + v, batch column bcol, if it is the first of its quad
            const bool adds = (li & 3) == 0 && bcol < p.batch;
            float *part_lane = my_part + 4 * lq * p.batch + bcol;
            // bias, bias_sel: the all-zero-row product of the slice, already multiplied by the group factor gf
            auto process_tile = [&](const Tile<G> &t, int rb, bool live, const u4 (&B)[kMfmaPerTile], const f4 &bias,
                                    float bias_sel, float gf) {
                f4 d0, d1;
                tile_product2(t.nz, t.sg, B, d0, d1);
                const f4 d = d0 + d1;
                const int sh = rb - min(rb, p.rows - G::kRows);  // rows a moved-back block repeats
                if constexpr (G::kRows == 4) {
                    // lane (row quad lq, column li): only D row 4*lq + (li & 3) pairs this column's
                    // chunk with the row that loaded it; it is group li of row rb - sh + lq.
                    // (bias_sel was formed the same way and its product with the power of two gf is exact, so an
                    // all-zero row still gives exactly 0)
                    const float dv = lane_select(lane_select(d[0], d[1], odd_lanes),
                                                 lane_select(d[2], d[3], odd_lanes), hi_lanes);
                    float x = h2f(t.sc[0]) * __builtin_fmaf(dv, gf, -bias_sel);
                    x = dpp_add<kQuadSwap1>(x);
                    x = dpp_add<kQuadSwap2>(x);
                    x = dpp_add<kRowHalfMirror>(x);
                    x = dpp_add<kRowMirror>(x);
                    if (li == 0 && lq >= sh && live) my_part[rb - sh - r_begin + lq] += x;
                } else {
                    float r[4];
                    uint32_t rows01, rows23;  // this lane's group of rows 4 lq, 4 lq + 1 and of rows 4 lq + 2, 4 lq + 3
                    quad_scales(t.sc[0], t.sc[1], quad_sel, quad_hi, rows01, rows23);
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const uint32_t pair = v < 2 ? rows01 : rows23;
                        float x = h2f((uint16_t)((v & 1) ? pair >> 16 : pair)) * __builtin_fmaf(d[v], gf, -bias[v]);
                        x = dpp_add<kQuadSwap1>(x);
                        x = dpp_add<kQuadSwap2>(x);
                        r[v] = x;
                    }
                    if (adds && live) {
                        // rows 4 lq + v of the tile, column bcol: the lane's part of the address never
                        // changes, the tile's part is wave-uniform
                        float *row0 = part_lane + (rb - sh - r_begin) * p.batch;
                        if (sh == 0) {
#pragma unroll
                            for (int v = 0; v < 4; v++) row0[v * p.batch] += r[v];
                        } else {
#pragma unroll
                            for (int v = 0; v < 4; v++)
                                if (4 * lq + v >= sh) row0[v * p.batch] += r[v];
                        }
                    }
                }
            };

            // the B operands of a slice, and what an all-zero weight row gives with them
            // this lane's result column collects one scale group of one batch column: the factor 2^(ex+10) of that
            // group, from the table the staging left
            const float *gfac_lane = gfac + (G::kRows == 4 ? li : min(bcol, p.batch - 1) * (seg_n * G::kChunks) + (li & 3));
            auto load_operands = [&](int slice, u4 (&B)[kMfmaPerTile], f4 &bias, float &bias_sel, float &gf) {
                // Every lane reads (no branch): the idle lanes read the zero operand with stride 0.
                const u4 *src = b_active ? reinterpret_cast<const u4 *>(image + (size_t)bcol * img_stride +
                                                                        slice * G::kCols) + b_chunk
                                         : &zero_operand;
                const int stride = b_active ? G::kChunks : 0;
#pragma unroll
                for (int k = 0; k < kMfmaPerTile; k++) B[k] = src[k * stride];
                gf = gfac_lane[slice * G::kChunks];
                // an all-zero weight row gives the "+1" term of the code, to be subtracted
                bias = tile_product(zero4, zero4, B);
                // wide tiles: the one bias entry this lane uses
                bias_sel = gf * lane_select(lane_select(bias[0], bias[1], odd_lanes),
                                            lane_select(bias[2], bias[3], odd_lanes), hi_lanes);
                bias = bias * gf;
            };
            if constexpr (kBothInOnePass) {
                // One flat sequence of (walk, matrix, slot) triples through a ring of four tiles. Per matrix the
                // tiles come in the order of the two-pass form, so every partial sum adds up in the same order;
                // the B operands of a walk serve both matrices.
                constexpr int kRing = 4;
                const int n_mats = pair ? 2 : 1;
                const char GB *bases[2][3] = {{nz_g, sg_g, sc_g}, {nz_g, sg_g, sc_g}};
                if (pair) {
                    bases[1][0] = reinterpret_cast<const char GB *>(as_global(sc.table[pi + 1].nz));
                    bases[1][1] = reinterpret_cast<const char GB *>(as_global(sc.table[pi + 1].sg));
                    bases[1][2] = reinterpret_cast<const char GB *>(as_global(sc.table[pi + 1].scales));
                }
                float *const part0 = my_part;
                int lw = wave, lm = 0, ls = 0;  // load cursor; past the last walk it parks on the wave's last walk
                auto next_of_both = [&]() -> Tile<G> {
                    const int w_ = min(lw, park_walk);
                    const int c = w_ / seg_n, sl = w_ - c * seg_n;
                    const int live_tiles = max(chunk_tiles(c), 1);
                    nz_g = bases[lm][0];
                    sg_g = bases[lm][1];
                    sc_g = bases[lm][2];
                    const Tile<G> t = load_tile(sl, r_begin + c * chunk_rows + min(ls, live_tiles - 1) * G::kRows);
                    if (++ls == n_slots) {
                        ls = 0;
                        if (++lm == n_mats) {
                            lm = 0;
                            lw += kNW;
                        }
                    }
                    return t;
                };
                Tile<G> ring4[kRing];
#pragma unroll
                for (int k = 0; k < kRing; k++) {
                    ring4[k] = next_of_both();
                    __builtin_amdgcn_sched_barrier(0);
                }
                u4 B[kMfmaPerTile];
                f4 bias;
                float bias_sel = 0.0f, gf = 0.0f;
                int wi = 0, m = 0, j = 0, c_begin = 0, n_rb = 0;
                const int total = my_live * n_mats * n_slots;
                for (int t0 = 0; t0 < total; t0 += kRing) {
#pragma unroll
                    for (int k = 0; k < kRing; k++) {
                        if (t0 + k < total) {
                            if (j == 0 && m == 0) {
                                const int walk = wave + wi * kNW;
                                const int chunk = walk / seg_n, slice = walk - chunk * seg_n;
                                c_begin = r_begin + chunk * chunk_rows;
                                n_rb = chunk_tiles(chunk);
                                load_operands(slice, B, bias, bias_sel, gf);
                            }
                            my_part = part0 + (size_t)m * sc.pair_stride;
                            process_tile(ring4[k], c_begin + min(j, max(n_rb, 1) - 1) * G::kRows, j < n_rb, B, bias, bias_sel, gf);
                            if (++j == n_slots) {
                                j = 0;
                                if (++m == n_mats) {
                                    m = 0;
                                    wi++;
                                }
                            }
                        }
                        ring4[k] = next_of_both();
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            } else if constexpr (kFine) {
                // one flat sequence of (walk, slot) pairs, G::kAhead at a time through the ring
                u4 B[kMfmaPerTile];
                f4 bias;
                float bias_sel = 0.0f, gf = 0.0f;
                int wi = 0, j = 0, c_begin = 0, n_rb = 0;
                const int total = my_live * n_slots;
                for (int t0 = 0; t0 < total; t0 += G::kAhead) {
#pragma unroll
                    for (int k = 0; k < G::kAhead; k++) {
                        if (t0 + k < total) {
                            if (j == 0) {
                                const int walk = wave + wi * kNW;
                                const int chunk = walk / seg_n, slice = walk - chunk * seg_n;
                                c_begin = r_begin + chunk * chunk_rows;
                                n_rb = chunk_tiles(chunk);
                                load_operands(slice, B, bias, bias_sel, gf);
                            }
                            process_tile(ring[k], c_begin + min(j, max(n_rb, 1) - 1) * G::kRows, j < n_rb, B, bias, bias_sel, gf);
                            if (++j == n_slots) {
                                j = 0;
                                wi++;
                            }
                        }
                        ring[k] = next_load();
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            } else
            for (int wi = 0; wi < my_walks; wi++) {
                const int walk = wave + wi * kNW;
                const int chunk = walk / seg_n, slice = walk - chunk * seg_n;
                const int c_begin = r_begin + chunk * chunk_rows;
                const int n_rb = chunk_tiles(chunk);  // live tiles of this walk (0: nothing to add)
                // this slice's activations become the B operands
                u4 B[kMfmaPerTile];
                f4 bias;
                float bias_sel, gf;
                load_operands(slice, B, bias, bias_sel, gf);

                auto process = [&](const Tile<G> &t, int rb, bool live) { process_tile(t, rb, live, B, bias, bias_sel, gf); };

                // No branch surrounds a load or an MFMA, so the wait counters stay exact and
                // G::kAhead - 1 tiles remain in flight while one is consumed.
                for (int j = 0; j < n_slots; j += G::kAhead) {
#pragma unroll
                    for (int k = 0; k < G::kAhead; k++) {
                        process(ring[k], c_begin + min(j + k, max(n_rb, 1) - 1) * G::kRows, j + k < n_rb);
                        ring[k] = next_load();
                        // keep the scheduler from interleaving whole tiles: that would need the
                        // registers of several decodes at once and cost a resident wave per SIMD
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
        }  // matrices of the task
        }  // segments of the row
        if (kExtras && gave_up) break;
        // last task of the span, or a pool task: ask for the next pool task now (not earlier: a
        // request is a claim, and a workgroup must not claim work long before it can start it); the
        // answer arrives while the partial sums are added up
        const bool request = sc.pool_count != 0 && u >= u_end && tid == 0;
        int requested = 0;
        if (request) requested = __hip_atomic_fetch_add(sc.counters, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        // ------------------------------------------------ add the waves' partial sums in wave order, store fp16
        {
            const int nrows = r_end - r_begin;
            // what the activations that stayed out of the image add to a row: scale * (+-x) where the row holds a
            // weight on the column, nothing where it holds none
            const int n_out = min(n_outliers, kMaxOutliers);
            auto outlier_sum = [&](const uint32_t *w_nz, const uint32_t *w_sg, const uint16_t *w_sc, int row, int b) -> float {
                float corr = 0.0f;
                for (int o = 0; o < n_out; o++) {
                    const uint32_t vb = out_val[o];
                    if ((int)(vb >> 16) != b) continue;
                    const int col = out_col[o];
                    const size_t at = (size_t)row * words + (col >> 5);
                    const uint32_t bit = 1u << (col & 31);
                    if (w_nz[at] & bit) {
                        const float xv = h2f((uint16_t)vb);
                        corr += h2f(w_sc[(size_t)row * groups + (col >> 7)]) * ((w_sg[at] & bit) ? xv : -xv);
                    }
                }
                return corr;
            };
            for (int idx = tid; idx < nrows * p.batch; idx += kThreads) {
                const int b = idx / nrows, rl = idx - b * nrows;
                float sum = 0.0f;
#pragma unroll
                for (int w = 0; w < kNW; w++) sum += partial[w * wave_stride + (size_t)rl * p.batch + b];
                if (n_out) sum += outlier_sum(p.nz, p.sg, p.scales, r_begin + rl, b);
                uint16_t out = f2h(sum * fscale[b]);
                if (pair) {
                    // out = silu(gate) * up on the fp16-rounded projections, in fp32: what the two
                    // launches and the element-wise kernel after them would store
                    float sum_up = 0.0f;
#pragma unroll
                    for (int w = 0; w < kNW; w++)
                        sum_up += partial[sc.pair_stride + w * wave_stride + (size_t)rl * p.batch + b];
                    if (n_out) sum_up += outlier_sum(sc.table[pi + 1].nz, sc.table[pi + 1].sg, sc.table[pi + 1].scales, r_begin + rl, b);
                    const float g = h2f(out), up = h2f(f2h(sum_up * fscale[b]));
                    out = f2h(g / (1.0f + expf(-g)) * up);
                }
                if (kExtras && p.residual) {
                    // the reference's add_forward behind the projection (src/transformer.cpp:247-250, 293-296): one
                    // correctly rounded fp16 add of the residual stream and the fp16-rounded projection
                    // (a load of device scope: an earlier stage may have written the residual stream)
                    uint16_t res_bits;
                    if (exchange && p.res_words >= 0) {
                        // the tagged word of the stage that wrote the residual stream (it has arrived long ago when the
                        // stages in between have run; the wait is bounded all the same)
                        uint32_t w = 0;
                        for (int spins = 0;; spins++) {
                            w = __hip_atomic_load(sc.words + p.res_words + r_begin + rl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            if (((w ^ tag_hi) >> 16) == 0) break;
                            if (spins >= sc.spin_limit) {
                                __hip_atomic_store(sc.status, stage + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                break;
                            }
                            __builtin_amdgcn_s_sleep(2);
                        }
                        res_bits = (uint16_t)w;
                    } else if (exchange) {
                        res_bits = p.residual[r_begin + rl];  // (nothing in the plan writes it, or only this row's own store below)
                    } else {
                        res_bits = __hip_atomic_load(p.residual + r_begin + rl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    const _Float16 res = __builtin_bit_cast(_Float16, res_bits);
                    out = __builtin_bit_cast(uint16_t, (_Float16)(res + __builtin_bit_cast(_Float16, out)));
                }
                uint16_t *dst = p.y + (size_t)b * p.rows + r_begin + rl;
                // (staged plans: written through to memory, where the workgroups of the next stage find it whatever
                // XCD they run on)
                if (staged) __hip_atomic_store(dst, out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else *dst = out;
                if (exchange && p.y_words >= 0) {
                    // (a later stage stores to y as well: this store has reached memory before any workgroup can know
                    // that the stage is complete, so the two stores cannot arrive in the wrong order)
                    if (p.flags & kProblemOrderedStore) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __hip_atomic_store(sc.words + p.y_words + r_begin + rl, (uint32_t)out | tag_hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        if (request) pool_task = requested;
        __syncthreads();
    }
    if (kExtras && gave_up) {
        if (tid == 0) __hip_atomic_store(sc.status, stage + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
    }
    if (exchange) {
        cur = -1;  // (the next stage waits for its own activations where it stages them)
    } else if (staged && stage + 1 < n_stages) {
        // ---- between two stages: every output of this workgroup's span has reached memory, then count and wait
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const int want = barrier_sense ^ 1;  // what the flag reads when every workgroup has arrived
            int *group = sc.barrier + 64 + 32 * ((int)blockIdx.x / kBarrierGroup);
            const int n_groups = ((int)gridDim.x + kBarrierGroup - 1) / kBarrierGroup;
            const int in_group = min(kBarrierGroup, (int)gridDim.x - (int)blockIdx.x / kBarrierGroup * kBarrierGroup);
            int reached = 0;
            bool last = false;
            if (__hip_atomic_fetch_add(group, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == in_group - 1) {
                __hip_atomic_store(group, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (__hip_atomic_fetch_add(sc.barrier + 32, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == n_groups - 1) {
                    __hip_atomic_store(sc.barrier + 32, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    // (the two stores above complete before the flag: nobody passes the barrier, let alone arrives
                    // at the next one, before the counters are zero)
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __hip_atomic_store(sc.barrier, want, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    last = true;
                    reached = 1;
                }
            }
            for (int spins = 0; !last && spins < sc.spin_limit; spins++) {
                if (__hip_atomic_load(sc.barrier, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == want) {
                    reached = 1;
                    break;
                }
                // (another workgroup has given up: the flag will never flip)
                if ((spins & 15) == 15 && __hip_atomic_load(sc.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
                __builtin_amdgcn_s_sleep(4);
            }
            if (!reached) __hip_atomic_store(sc.status, stage + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            stage_reached = reached;
            barrier_sense = want;
        }
        __syncthreads();
        if (!stage_reached) break;  // (the same for the whole workgroup: every wave leaves through the code below)
        // what the stage before wrote is read from memory, not from a stale line of this XCD's cache
        if (sc.stage_fence) {
            if (wave == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            __syncthreads();
        }
        cur = -1;
    }
    }  // stages
    if (exchange && tid == 0) sc.epochs[blockIdx.x] = (int)(epoch + 1u);
    if (sc.pool_count != 0 && tid == 0) {
        const int left = __hip_atomic_fetch_add(sc.counters + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left == (int)gridDim.x - 1) {  // every other workgroup has made its last request
            __hip_atomic_store(sc.counters, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(sc.counters + 1, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

struct DeviceInfo {
    int cus = 0;
};

constexpr int kLdsLimit = 64 * 1024;  // per workgroup; 160 KB per CU leaves room for two or three
// The tall-tile instance keeps one partial sum per wave, row and batch column: it gets all the LDS
// that three workgroups per CU can have (three resident workgroups beat two with 78 KB each: +4.5 %
// at four batch columns, equal at two and three).
constexpr int kTallLdsLimit = 53 * 1024;

template <class G, bool kExtras = false, bool kFine = false>
const void *kernel_ptr() {
    return reinterpret_cast<const void *>(&gemv_mfma_kernel<G, kExtras, kFine>);
}

// Per device, once: the kernels may use up to kLdsLimit of dynamic LDS. Safe from several host threads.
hipError_t prepare_device(DeviceInfo **out) {
    static DeviceInfo info[64];
    static std::atomic<bool> ready[64];
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    if (!ready[dev].load(std::memory_order_acquire)) {
        static std::mutex init_mutex;
        std::lock_guard<std::mutex> lock(init_mutex);
        for (const void *k : {kernel_ptr<Wide>(), kernel_ptr<Tall>(), kernel_ptr<Wide, true>(),
                              kernel_ptr<Wide, false, true>(), kernel_ptr<Wide, true, true>(),
                              kernel_ptr<Tall, false, true>()})
            if (hipError_t e = hipFuncSetAttribute(
                    k, hipFuncAttributeMaxDynamicSharedMemorySize,
                    k == kernel_ptr<Tall>() || k == kernel_ptr<Tall, false, true>() ? kTallLdsLimit : kLdsLimit))
                return e;
        info[dev].cus = current_device_cus();
        ready[dev].store(true, std::memory_order_release);
    }
    *out = &info[dev];
    return hipSuccess;
}

// Resident workgroups per CU for a given dynamic LDS size (asked from the runtime, capped at 4).
template <class G, bool kExtras = false, bool kFine = false>
int resident_wgs(size_t lds_bytes) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gemv_mfma_kernel<G, kExtras, kFine>, kThreads, lds_bytes) != hipSuccess || n < 1)
        n = 1;
    return n > 4 ? 4 : n;
}

template <class G>
constexpr int range_unit() {  // rows: every wave walks whole groups of G::kAhead tiles
    return kNW * G::kRows * G::kAhead;
}
constexpr int kFineUnit = kNW * Wide::kRows;  // rows of a unit of the fine-grained instances: one tile per wave
constexpr int kTallFineUnit = kNW * Tall::kRows;
// A launch with no more 32-row units than the chip has workgroup slots runs in units of 16 rows instead (one tile per
// wave): a single matrix of the 8B shapes takes 9.2 us per call so against 9.6 us. Beyond one unit per slot the coarse
// units win (8B shapes, one plan launch for 2 / 3 / 4 / 6 / 8 layers, i.e. 3.5 to 14 units per slot: 32.2 / 46.0 / 51.0 /
// 67.7 / 90.0 us against 35.9 / 49.9 / 57.8 / 78.9 / 99.1 us in units of 16 rows; the gate/up plan of a decode step,
// 1.2 units per slot, 4 us faster; only one whole layer, 1.75 per slot, loses 0.5 us of 22).
bool wants_fine(int64_t coarse_units, int slots) { return coarse_units <= (int64_t)slots; }

template <class G>
int image_bytes_of(int cols, int batch, bool segmented = true) {
    int slices = (cols + G::kCols - 1) / G::kCols;
    if (segmented) {  // long rows are staged in equal segments (the kernel works out the same numbers)
        const int seg_max = G::kRows == 4 ? kSegSlices : tall_seg_slices(batch);
        const int n_seg = (slices + seg_max - 1) / seg_max;
        slices = (slices + n_seg - 1) / n_seg;
    }
    const int image = slices * G::kCols * 2 * batch;
    return image + image / 64;  // and one fp32 factor per 128-column group
}

// Geometry limits: a tile must fit inside the matrix (edge tiles are moved back, not clipped).
bool wide_ok(const Problem &p) {
    return p.batch == 1 && p.rows >= 16 && p.cols >= Wide::kCols &&
           image_bytes_of<Wide>(p.cols, 1) + kNW * range_unit<Wide>() * 4 <= kLdsLimit;
}
bool tall_ok(const Problem &p) {
    return p.batch >= 1 && p.batch <= kMaxBatch && p.rows >= 16 && p.cols >= Tall::kCols &&
           image_bytes_of<Tall>(p.cols, p.batch) + kNW * range_unit<Tall>() * p.batch * 4 <= kTallLdsLimit;
}

#ifndef TLLM_MAX_TASK_UNITS
#define TLLM_MAX_TASK_UNITS 20
#endif
constexpr int kMaxTaskUnits = TLLM_MAX_TASK_UNITS;  // longer tasks amortise the per-slice operand reload

// The workgroups of one launch all start together, three per CU, and the CU serves its oldest
// waves first: measured on the 8B sweep with equal spans, the first 256 workgroups (one per CU)
// finished after 233 us, the second 256 after 280 us and the last after 333 us; the odd XCDs
// (workgroups go to the eight XCDs in turn, so XCD = index % 8 and its parity = index & 1) ran 8 % slower
// than the even ones, and what is left after these two effects
// is +-2 %. Spans are therefore cut in proportion to the speed of the place a workgroup will run in,
// so that they end together. TLLM_SPAN_SHARES="s0,s1,s2,odd" overrides the four factors.
struct SpanShares {
    double slot[3] = {1.4, 1.0, 0.65};
    double odd_xcd = 0.92;
};
const SpanShares &span_shares() {
    static const SpanShares shares = [] {
        SpanShares v;
        if (const char *e = getenv("TLLM_SPAN_SHARES")) {
            SpanShares w;
            if (sscanf(e, "%lf,%lf,%lf,%lf", &w.slot[0], &w.slot[1], &w.slot[2], &w.odd_xcd) == 4 && w.slot[0] > 0 &&
                w.slot[1] > 0 && w.slot[2] > 0 && w.odd_xcd > 0)
                v = w;
        }
        return v;
    }();
    return shares;
}
double span_share(int wg, int cus, int grid) {
    if (grid != 3 * cus) return 1.0;  // measured for three full rounds of workgroups only
    const SpanShares &v = span_shares();
    return v.slot[wg / cus] * ((wg & 1) ? v.odd_xcd : 1.0);
}

// Part of a large plan's weights that is kept out of the spans and dealt out at run time in pieces
// of about kPoolTaskWeights weights: spans of the right average size still do not end together
// (+-4 % from workgroup to workgroup and launch to launch), and the last workgroup sets the time.
// Measured on the 8B sweep in steady state with units of 48 rows: 0 -> 5375 GB/s, 0.10 -> 5495, 0.15 -> 5517, 0.30
// slower again (a pool task of 768 K weights spends a quarter of its 25 us on staging and hand-over); with the
// units of 32 rows the spans end closer together and a smaller pool is enough: 0 -> 5766, 0.03 -> 5816, 0.05 -> 5865,
// 0.07 -> 5830, 0.10 -> 5817, 0.15 -> 5770, 0.30 -> 5648 (70B, 80 layers: 0.15 -> 5865, 0.05 -> 5895).
// Plans of two to four activation rows (units of 128 rows, four times the work per unit) keep the larger pool:
// 8B sweep at four rows 0 -> 3938 GB/s, 0.05 -> 3885, 0.10 -> 4003, 0.15 -> 4040, 0.25 -> 3989; at two rows
// 0 -> 3982, 0.05 -> 3916, 0.10 -> 4220, 0.15 -> 4240, 0.25 -> 4284; on a faster box 0.15 / 0.20 / 0.25 at four
// rows 4136 / 4114 / 4084, at three 4021 / 4167 / 4120, at two 4254 / 4440 / 4336.
// TLLM_POOL_FRACTION and TLLM_TALL_POOL_FRACTION override them (0 switches the pool off).
double pool_fraction(bool wide) {
    static const double f[2] = {
        [] {
            const char *e = getenv("TLLM_TALL_POOL_FRACTION");
            const double v = e ? atof(e) : 0.2;
            return v < 0.0 ? 0.0 : v > 0.5 ? 0.5 : v;
        }(),
        [] {
            const char *e = getenv("TLLM_POOL_FRACTION");
            const double v = e ? atof(e) : 0.05;
            return v < 0.0 ? 0.0 : v > 0.5 ? 0.5 : v;
        }()};
    return f[wide ? 1 : 0];
}
#ifndef TLLM_POOL_TASK_WEIGHTS
#define TLLM_POOL_TASK_WEIGHTS (768 * 1024)
#endif
constexpr int64_t kPoolTaskWeights = TLLM_POOL_TASK_WEIGHTS;
// The same for the batched kernel, whose blocks are all independent (TLLM_BLOCK_POOL_FRACTION).
double block_pool_fraction() {
    static const double f = [] {
        const char *e = getenv("TLLM_BLOCK_POOL_FRACTION");
        const double v = e ? atof(e) : 0.4;
        return v < 0.0 ? 0.0 : v > 0.9 ? 0.9 : v;
    }();
    return f;
}

// units per task that the partial-sum area can hold
int max_units_for(int image_bytes, int batch, int unit, int mats = 1, int lds_limit = kLdsLimit) {
    // one partial sum per wave, row and matrix of the task (two for a SwiGLU pair)
    const int room_rows = (lds_limit - image_bytes) / (kNW * batch * 4 * mats);
    const int n = room_rows / unit;
    return n > kMaxTaskUnits ? kMaxTaskUnits : n;
}

}  // namespace

bool gemv_mfma_supports(const Problem &p, int group) {
    return group == 128 && (size_t)p.rows * (p.cols / 8) < (size_t)1 << 32 && (wide_ok(p) || tall_ok(p));
}

static hipError_t launch_single(const Problem &p, bool x_is_i8, float i8_scale, const float *i8_scale_dev,
                                hipStream_t s) {
    DeviceInfo *di = nullptr;
    if (hipError_t e = prepare_device(&di)) return e;
    Sched sc{};
    sc.x_is_i8 = x_is_i8 ? 1 : 0;
    sc.i8_scale = i8_scale;
    sc.i8_scale_dev = i8_scale_dev;
    sc.table = nullptr;
    sc.count = 1;
    const bool wide = wide_ok(p);
    const int wgs = (wide ? Wide::kWgPerCu : Tall::kWgPerCu) * di->cus;
    // the fine-grained instances keep the whole row in LDS: possible while it fits
    const bool fine = wide && image_bytes_of<Wide>(p.cols, 1, false) + kNW * kFineUnit * 4 <= kLdsLimit &&
                      wants_fine((p.rows + range_unit<Wide>() - 1) / range_unit<Wide>(), wgs);
    const int unit = fine ? kFineUnit : wide ? range_unit<Wide>() : range_unit<Tall>();
    sc.image_bytes = wide ? image_bytes_of<Wide>(p.cols, 1, !fine) : image_bytes_of<Tall>(p.cols, p.batch);
    sc.max_units = max_units_for(sc.image_bytes, p.batch, unit, 1, wide ? kLdsLimit : kTallLdsLimit);
    sc.max_batch = p.batch;
    const int units = (p.rows + unit - 1) / unit;
    const int grid = units < wgs ? units : wgs;
    const size_t lds = (size_t)sc.image_bytes + (size_t)kNW * sc.max_units * unit * p.batch * 4;
    if (fine)
        gemv_mfma_kernel<Wide, false, true><<<grid, kThreads, lds, s>>>(p, sc);
    else if (wide)
        gemv_mfma_kernel<Wide><<<grid, kThreads, lds, s>>>(p, sc);
    else
        gemv_mfma_kernel<Tall><<<grid, kThreads, lds, s>>>(p, sc);
    return hipGetLastError();
}

hipError_t launch_gemv_mfma(const Problem &p, hipStream_t s) { return launch_single(p, false, 0.0f, nullptr, s); }

// p.x points at int8 activations (batch 1, 8-byte aligned)
hipError_t launch_gemv_mfma_i8(const Problem &p, float scale_value, const float *scale_dev, hipStream_t s) {
    return launch_single(p, true, scale_value, scale_dev, s);
}

// ------------------------------------------------------------------ multi-problem plan
hipError_t plan_device_create(const std::vector<Problem> &host, PlanDevice *out) {
    PlanDevice d;
    d.count = (int)host.size();
    if (hipError_t e = hipGetDevice(&d.device)) return e;
    DeviceInfo *di = nullptr;
    if (hipError_t e = prepare_device(&di)) return e;

    int max_image = 0, max_batch = 1;
    for (const Problem &p : host) {
        max_batch = p.batch > max_batch ? p.batch : max_batch;
        d.max_rows = p.rows > d.max_rows ? p.rows : d.max_rows;
    }
    d.max_batch = max_batch;
    // Device table order: the problems whose units are dealt out as spans, then those of the shared
    // pool; `prefix` counts units in that order.
    std::vector<Problem> ordered = host;
    std::vector<int> prefix(host.size() + 1, 0), wg_first, pool_first;
    // Contiguous spans of units, one per workgroup, cut by weight (a unit's weights plus a fixed
    // cost) in proportion to the workgroup's share; at least one unit per workgroup. With
    // max_task_units > 0 and enough work, the last problems with short rows (staging x is cheap
    // there) go to the shared pool instead, cut into small tasks inside one problem each.
    auto partition = [&](int unit, int wgs, int max_task_units, bool wide) {
        const int n = (int)host.size();
        // the up half of a SwiGLU pair has no units: its rows are done with the gate's
        auto is_up = [&](const std::vector<Problem> &v, int i) { return i > 0 && (v[i - 1].flags & kProblemSwigluGate); };
        auto mats = [&](const Problem &p) { return (p.flags & kProblemSwigluGate) ? 2 : 1; };
        auto units_in = [&](const std::vector<Problem> &v, int i) { return is_up(v, i) ? 0 : (v[i].rows + unit - 1) / unit; };
        std::vector<char> pooled(n, 0);
        int64_t all_w = 0;
        int all_units = 0, min_cols = host[0].cols;
        for (int i = 0; i < n; i++) {
            all_w += (int64_t)host[i].rows * host[i].cols;
            all_units += units_in(host, i);
            min_cols = host[i].cols < min_cols ? host[i].cols : min_cols;
        }
        // no pool for plans that give a workgroup less than about two pool tasks of work: a quarter of
        // the workgroups would then end with one more task than the rest (1B shapes, 16 layers: 54 us
        // without the pool, 60.5 us with it; 8B shapes, 8 layers: 100 / 99 us)
        if (max_task_units > 0 && all_units >= 8 * wgs && (double)all_w / wgs >= 2.3 * (double)kPoolTaskWeights) {
            const int64_t want = (int64_t)((double)all_w * pool_fraction(wide));
            int64_t got = 0;
            int left_units = all_units;
            for (int pass = 0; pass < 2 && got < want; pass++)
                for (int i = n - 1; i >= 0 && got < want; i--) {
                    if (pooled[i] || is_up(host, i) || (pass == 0 && host[i].cols > 2 * min_cols)) continue;
                    if (left_units - units_in(host, i) < 4 * wgs) continue;
                    pooled[i] = 1;
                    got += (int64_t)host[i].rows * host[i].cols * mats(host[i]);
                    left_units -= units_in(host, i);
                    if (mats(host[i]) == 2) pooled[i + 1] = 1;  // a pair stays together
                }
        }
        int k = 0, n_static = 0;
        for (int pass = 0; pass < 2; pass++) {
            for (int i = 0; i < n; i++)
                if (pooled[i] == pass) ordered[k++] = host[i];
            if (pass == 0) n_static = k;
        }
        std::vector<int64_t> weight;
        for (int i = 0; i < n; i++) {
            const int nu = units_in(ordered, i);
            prefix[i + 1] = prefix[i] + nu;
            for (int t = 0; t < nu && i < n_static; t++) {
                const int nr = ordered[i].rows - t * unit < unit ? ordered[i].rows - t * unit : unit;
                weight.push_back((int64_t)nr * ordered[i].cols * mats(ordered[i]) + 16384);
            }
        }
        const int units = prefix[n_static];
        const int grid = units < wgs ? units : wgs;
        int64_t total_w = 0;
        for (int64_t w : weight) total_w += w;
        std::vector<double> upto(grid + 1, 0.0);  // shares of the workgroups before g
        for (int g = 0; g < grid; g++)
            upto[g + 1] = upto[g] + (max_task_units > 0 ? span_share(g, di->cus, grid) : 1.0);
        wg_first.assign(grid + 1, units);
        wg_first[0] = 0;
        int64_t acc = 0;  // weight of units [0, t)
        int t = 0;
        for (int g = 1; g < grid; g++) {
            const int lo = wg_first[g - 1] + 1, hi = units - (grid - g);
            const double want = (double)total_w * upto[g] / upto[grid];
            while (t < hi && (t < lo || (double)acc < want)) acc += weight[t++];
            wg_first[g] = t;
        }
        // the problem each span starts in, so that a workgroup does not scan the prefix from 0
        for (int g = 0, pr = 0; g < grid; g++) {
            while (prefix[pr + 1] <= wg_first[g]) pr++;
            wg_first.push_back(pr);
        }
        std::vector<int> pool_problem;
        for (int i = n_static; i < n; i++) {
            const int64_t unit_w = (int64_t)unit * ordered[i].cols * mats(ordered[i]);
            int64_t per = (kPoolTaskWeights + unit_w / 2) / unit_w;
            per = per < 1 ? 1 : per > max_task_units ? max_task_units : per;
            for (int u0 = prefix[i]; u0 < prefix[i + 1]; u0 += (int)per) {
                pool_first.push_back(u0);
                pool_problem.push_back(i);
            }
        }
        d.pool_count = (int)pool_problem.size();
        if (d.pool_count) {
            pool_first.push_back(prefix[n]);
            pool_first.insert(pool_first.end(), pool_problem.begin(), pool_problem.end());
        }
        d.grid = grid;
    };

    // The batched kernel works in blocks of rows that need nothing from the block before: equal
    // spans of blocks over the first part of the list, the blocks of the last part handed out one by
    // one at run time (the XCDs of one box differed by 15 % in speed under this kernel).
    auto partition_blocks = [&](int unit, int wgs) {
        std::vector<int64_t> weight;
        std::vector<int> block_problem;
        for (size_t i = 0; i < host.size(); i++) {
            const int n = (host[i].rows + unit - 1) / unit;
            prefix[i + 1] = prefix[i] + n;
            for (int t = 0; t < n; t++) {
                const int nr = host[i].rows - t * unit < unit ? host[i].rows - t * unit : unit;
                weight.push_back((int64_t)nr * host[i].cols + 16384);
                block_problem.push_back((int)i);
            }
        }
        const int all_units = prefix.back();
        int64_t all_w = 0;
        for (int64_t w : weight) all_w += w;
        int units = all_units;  // blocks that belong to spans
        if (all_units >= 8 * wgs) {
            int64_t acc = 0;
            units = 0;
            while (units < all_units && (double)acc < (double)all_w * (1.0 - block_pool_fraction())) acc += weight[units++];
            units = units < 4 * wgs ? 4 * wgs : units;
        }
        const int grid = units < wgs ? units : wgs;
        // List scheduling on the host, in the order the blocks lie in memory: chunks of consecutive blocks
        // go to the XCD with the least work so far (workgroup ids w, w + 8, ... share an XCD), and
        // inside the XCD each block to the workgroup with the least work so far. At run time the workgroups of an XCD
        // are then on the same chunk at about the same time, which is mostly one matrix: its activation rows come from
        // HBM once per XCD and from that XCD's L2 afterwards, not once per block. A workgroup's blocks ascend.
        const int n_xcd = grid % 8 == 0 ? 8 : 1, per_xcd = grid / n_xcd;
        std::vector<std::vector<int>> mine(grid);
        std::vector<int64_t> wg_load(grid, 0), xcd_load(n_xcd, 0);
        // (chunks of 8: whole XCD-loads of 32 neighbouring blocks put all of an XCD's workgroups into the same phase of
        // their blocks and cost 3 % on the 8B sweep at sixteen rows; with 8 an XCD is in four places at a time, the
        // activation rows of four matrices still fit its L2, and the 70B sweep keeps its + 4 %)
        const int chunk = per_xcd < 8 ? per_xcd : 8;
        for (int b0 = 0; b0 < units; b0 += chunk) {
            int x = 0;
            for (int i = 1; i < n_xcd; i++)
                if (xcd_load[i] < xcd_load[x]) x = i;
            for (int b = b0; b < units && b < b0 + chunk; b++) {
                int w = x;
                for (int i = 1; i < per_xcd; i++)
                    if (wg_load[x + n_xcd * i] < wg_load[w]) w = x + n_xcd * i;
                mine[w].push_back(b);
                wg_load[w] += weight[b];
                xcd_load[x] += weight[b];
            }
        }
        // The kernel asks for its first run-time block while it works on its last own one: every workgroup needs a
        // block of its own. The first chunks go to the XCDs that have none yet and fill all their workgroups, so none is
        // left empty as long as there are at least `grid` blocks; should weights ever defeat that, deal the blocks out
        // in turn instead.
        bool some_empty = false;
        for (int w = 0; w < grid; w++) some_empty = some_empty || mine[w].empty();
        if (some_empty) {
            for (int w = 0; w < grid; w++) mine[w].clear();
            for (int b = 0; b < units; b++) mine[b % grid].push_back(b);
        }
        std::vector<int> order, first_problem;
        wg_first.assign(grid + 1, 0);
        for (int w = 0; w < grid; w++) {
            wg_first[w] = (int)order.size();
            first_problem.push_back(block_problem[mine[w][0]]);
            order.insert(order.end(), mine[w].begin(), mine[w].end());
        }
        wg_first[grid] = (int)order.size();
        wg_first.insert(wg_first.end(), first_problem.begin(), first_problem.end());
        wg_first.insert(wg_first.end(), order.begin(), order.end());
        pool_first.assign(block_problem.begin() + units, block_problem.end());
        d.pool_begin = units;
        d.pool_end = all_units;
        d.grid = grid;
    };

    // several activation rows: the batched kernel if every problem fits it
    bool has_pairs = false, has_norm = false, has_quant = false;
    for (const Problem &p : host) {
        has_pairs = has_pairs || (p.flags & kProblemSwigluGate);
        has_norm = has_norm || (p.norm_w != nullptr && !(p.flags & kProblemInt8Input));
        has_quant = has_quant || (p.flags & kProblemQuantInput);  // (batch 1: the caller has checked)
    }
    // int8 activations: all problems or none, batch 1 (the caller has checked), MFMA kernel only
    bool any_i8 = false, all_i8 = true;
    for (const Problem &p : host) {
        any_i8 = any_i8 || (p.flags & kProblemInt8Input);
        all_i8 = all_i8 && (p.flags & kProblemInt8Input);
    }
    if (any_i8 && (!all_i8 || max_batch != 1 || has_pairs)) return hipErrorInvalidValue;
    d.x_is_i8 = any_i8;
    // SwiGLU pairs and RMSNorm prologues exist in the wide-tile MFMA GEMV kernel only (batch 1)
    d.extras = has_pairs || has_norm;
    bool all_batch = max_batch >= 2 && !d.extras && !has_quant;  // (only the batch-1 family quantises its input itself)
    for (const Problem &p : host) all_batch = all_batch && gemv_batch_supports(p, 128);
    // one geometry per launch otherwise: wide tiles if every problem allows them, else tall ones
    bool all_wide = true, all_tall = true;
    for (const Problem &p : host) {
        const bool addressable = (size_t)p.rows * (p.cols / 8) < (size_t)1 << 32;
        all_wide = all_wide && addressable && wide_ok(p);
        all_tall = all_tall && addressable && tall_ok(p);
    }
    // Up to this many activation rows the tall-tile MFMA kernel is the faster of the two (8B and 70B
    // sweeps: +17 % at two rows, +13 % at three, +5 % at four). The tuning switch tall_max_batch overrides.
    const int tall_max_batch = tuning().tall_max_batch.load(std::memory_order_relaxed);
    // ... for plans large enough: its units (128 rows of one matrix) are what spans are cut in, and a unit of a
    // long-row matrix must not outweigh a workgroup's share of the plan: the tall tiles are taken from a share of one
    // unit on (the tuning switch tall_min_share_milli overrides the ratio), and in units of 64 rows (one tile per wave) from a share of
    // 1.75 of those. One plan launch, us, batched kernel / tall tiles, at four activation rows: 8B shapes 2, 4, 6, 8, 12
    // layers (shares 0.3 to 1.8): 77 / 93, 97 / 119, 155 / 154, 178 / 165, 246 / 212; 70B 1, 2, 4, 8 layers (0.3 to
    // 2.4): 142 / 177, 211 / 234, 345 / 332, 587 / 563. At two rows the tall tiles win from 6 layers of 8B (154 / 133)
    // and 2 of 70B (211 / 198) on.
    bool tall_pays = all_tall && max_batch <= tall_max_batch, tall_fine = false;
    if (tall_pays) {
        int64_t total = 0;
        int max_cols = 0;
        for (const Problem &p : host) {
            total += (int64_t)p.rows * p.cols;
            max_cols = std::max(max_cols, (int)p.cols);
        }
        const double min_share = tuning().tall_min_share_milli.load(std::memory_order_relaxed) / 1000.0;
        const double share = (double)total / (Tall::kWgPerCu * di->cus);
        tall_pays = share >= min_share * (double)range_unit<Tall>() * max_cols;
        if (!tall_pays) tall_pays = tall_fine = share >= 1.75 * min_share * (double)kTallFineUnit * max_cols;
    }
    if (all_batch && !tall_pays) {
        d.batch_kernel = true;
        partition_blocks(gemv_batch_block_rows(), di->cus);
    } else {
        d.wide = all_wide;
        d.use_mfma = d.extras ? all_wide : all_wide || all_tall;
        if (d.x_is_i8 && !d.use_mfma) return hipErrorInvalidValue;  // the table kernel for general shapes is fp16 only
        if (d.wide) {  // decode-size plans: fine-grained units
            int64_t coarse = 0;
            int whole = 0;  // largest image of a whole row: the fine-grained instances do not stage in segments
            for (size_t i = 0; i < host.size(); i++) {
                whole = std::max(whole, image_bytes_of<Wide>(host[i].cols, 1, false));
                if (!(i > 0 && (host[i - 1].flags & kProblemSwigluGate)))
                    coarse += (host[i].rows + range_unit<Wide>() - 1) / range_unit<Wide>();
            }
            d.fine = whole + kNW * kFineUnit * 4 * (has_pairs ? 2 : 1) <= kLdsLimit &&
                     wants_fine(coarse, Wide::kWgPerCu * di->cus);
        }
        if (!d.wide) d.fine = tall_fine;
        for (const Problem &p : host) {
            const int ib = d.wide ? image_bytes_of<Wide>(p.cols, 1, !d.fine) : image_bytes_of<Tall>(p.cols, p.batch);
            max_image = ib > max_image ? ib : max_image;
        }
        const int unit = d.wide ? (d.fine ? kFineUnit : range_unit<Wide>()) : (d.fine ? kTallFineUnit : range_unit<Tall>());
        const int mats = has_pairs ? 2 : 1;
        const int max_units = max_units_for(max_image, max_batch, unit, mats, d.wide ? kLdsLimit : kTallLdsLimit);
        if (max_units < 1) d.use_mfma = false;
        // (again, after the demotion: the table kernel for general shapes reads fp16 activations and knows neither
        // SwiGLU pairs nor RMSNorm prologues)
        if ((d.x_is_i8 || d.extras || has_quant) && !d.use_mfma) return hipErrorInvalidValue;
        if (d.use_mfma) {
            d.pair_stride = has_pairs ? kNW * max_units * unit * max_batch : 0;
            d.lds_bytes = max_image + kNW * max_units * unit * max_batch * 4 * mats;
            const int per_cu = d.extras && d.fine ? resident_wgs<Wide, true, true>(d.lds_bytes)
                               : d.extras         ? resident_wgs<Wide, true>(d.lds_bytes)
                               : d.wide && d.fine ? resident_wgs<Wide, false, true>(d.lds_bytes)
                               : d.wide           ? resident_wgs<Wide>(d.lds_bytes)
                               : d.fine           ? resident_wgs<Tall, false, true>(d.lds_bytes)
                                                  : resident_wgs<Tall>(d.lds_bytes);
            partition(unit, per_cu * di->cus, max_units, d.wide);
            d.max_units = max_units;
            d.image_bytes = max_image;
        }
    }

    // one allocation: table | unit prefix | spans | pool tasks | the two counters
    auto round16 = [](size_t v) { return (v + 15) / 16 * 16; };
    const size_t bytes_table = round16(sizeof(Problem) * ordered.size());
    const size_t bytes_prefix = round16(sizeof(int) * prefix.size());
    const size_t bytes_wg = round16(sizeof(int) * wg_first.size());
    const size_t bytes_pool = round16(sizeof(int) * pool_first.size());
    // what every workgroup of the MFMA kernel starts with (wg_first: [grid + 1] first units, then [grid] problems)
    std::vector<WgStart> starts;
    if (d.use_mfma && !d.batch_kernel) {
        starts.resize(d.grid);
        for (int g = 0; g < d.grid; g++) {
            WgStart &ws = starts[g];
            ws = WgStart{};
            ws.u = wg_first[g];
            ws.u_end = wg_first[g + 1];
            ws.pi = wg_first[d.grid + 1 + g];
            ws.first_unit = prefix[ws.pi];
            ws.p_units = prefix[ws.pi + 1] - prefix[ws.pi];
            ws.p = ordered[ws.pi];
        }
    }
    const size_t bytes_starts = starts.empty() ? 0 : sizeof(WgStart) * starts.size() + 128;
    char *base = nullptr;
    if (hipError_t e = hipMalloc(&base, bytes_table + bytes_prefix + bytes_wg + bytes_pool + round16(8 * kPlanSlots) + bytes_starts)) return e;
    d.problems = reinterpret_cast<Problem *>(base);
    d.unit_prefix = reinterpret_cast<int *>(base + bytes_table);
    d.wg_first = reinterpret_cast<int *>(base + bytes_table + bytes_prefix);
    d.pool_first = reinterpret_cast<int *>(base + bytes_table + bytes_prefix + bytes_wg);
    d.counters = reinterpret_cast<int *>(base + bytes_table + bytes_prefix + bytes_wg + bytes_pool);
    hipError_t e = hipMemcpy(d.problems, ordered.data(), sizeof(Problem) * ordered.size(), hipMemcpyHostToDevice);
    if (!e) e = hipMemcpy(d.unit_prefix, prefix.data(), sizeof(int) * prefix.size(), hipMemcpyHostToDevice);
    if (!e && !wg_first.empty())
        e = hipMemcpy(d.wg_first, wg_first.data(), sizeof(int) * wg_first.size(), hipMemcpyHostToDevice);
    if (!e && !pool_first.empty())
        e = hipMemcpy(d.pool_first, pool_first.data(), sizeof(int) * pool_first.size(), hipMemcpyHostToDevice);
    if (!e) e = hipMemset(d.counters, 0, 8 * kPlanSlots);
    if (!e && !starts.empty()) {
        d.starts = reinterpret_cast<WgStart *>((reinterpret_cast<uintptr_t>(d.counters) + round16(8 * kPlanSlots) + 127) / 128 * 128);
        e = hipMemcpy(d.starts, starts.data(), sizeof(WgStart) * starts.size(), hipMemcpyHostToDevice);
    }
    d.next_slot = new (std::nothrow) std::atomic<unsigned>(0);
    if (!e && !d.next_slot) e = hipErrorOutOfMemory;
    if (e) {
        (void)hipFree(base);
        delete d.next_slot;
        return e;
    }
    *out = d;
    return hipSuccess;
}

// ------------------------------------------------------------------ staged plan
// The dependent linears of a decode step in ONE launch (reference src/transformer.cpp:239-296: o_proj, residual add,
// RMSNorm, gate/up, SiLU * up, down_proj, residual add, and the RMSNorm + q/k/v of the next layer): the problems of a
// stage are spread over all workgroups of the launch in units of 16 rows, and between two stages the workgroups wait
// for each other at a device counter instead of ending the kernel. Everything a problem computes is what the
// single-stage plan computes for it (same kernel instance, same units), so the outputs equal those of separate
// launches bit for bit.
hipError_t plan_device_create_staged(const std::vector<Problem> &host, PlanDevice *out) {
    PlanDevice d;
    d.count = (int)host.size();
    if (hipError_t e = hipGetDevice(&d.device)) return e;
    DeviceInfo *di = nullptr;
    if (hipError_t e = prepare_device(&di)) return e;
    const int n = d.count;
    bool has_pairs = false;
    int whole = 0, stage = 0;
    for (int i = 0; i < n; i++) {
        const Problem &p = host[i];
        const bool addressable = (size_t)p.rows * (p.cols / 8) < (size_t)1 << 32;
        if (p.batch != 1 || !addressable || !wide_ok(p) || (p.flags & kProblemInt8Input)) return hipErrorInvalidValue;
        if (p.stage < stage || p.stage > stage + 1 || p.stage >= kMaxStages || (i == 0 && p.stage != 0)) return hipErrorInvalidValue;
        stage = p.stage;
        has_pairs = has_pairs || (p.flags & kProblemSwigluGate);
        d.max_rows = std::max(d.max_rows, (int)p.rows);
        whole = std::max(whole, image_bytes_of<Wide>(p.cols, 1, false));
    }
    d.n_stages = stage + 1;
    d.max_batch = 1;
    // rows that the one-pass staging holds in registers (K <= 16384; also when the launch quantises them: it does so
    // from those registers) are read with loads of device scope, or as tagged words; longer rows make the workgroups
    // wait at barriers and invalidate their cache behind each
    for (const Problem &p : host)
        if (p.cols > 16384) d.stage_fence = true;
    const int mats = has_pairs ? 2 : 1;
    if (whole + kNW * kFineUnit * 4 * mats > kLdsLimit) return hipErrorInvalidValue;  // whole rows in LDS (K <= 28672)
    const int max_units = max_units_for(whole, 1, kFineUnit, mats);
    d.use_mfma = d.wide = d.fine = d.extras = true;
    d.max_units = max_units;
    d.image_bytes = whole;
    d.pair_stride = has_pairs ? kNW * max_units * kFineUnit : 0;
    d.lds_bytes = whole + kNW * max_units * kFineUnit * 4 * mats;
    // every workgroup of the launch must be resident at the same time: no more than the chip holds
    const int slots = resident_wgs<Wide, true, true>(d.lds_bytes) * di->cus;

    auto is_up = [&](int i) { return i > 0 && (host[i - 1].flags & kProblemSwigluGate); };
    auto units_in = [&](int i) { return is_up(i) ? 0 : (host[i].rows + kFineUnit - 1) / kFineUnit; };
    std::vector<int> prefix(n + 1, 0), stage_begin(d.n_stages + 1, n);
    for (int i = 0; i < n; i++) {
        prefix[i + 1] = prefix[i] + units_in(i);
        if (i == 0 || host[i].stage != host[i - 1].stage) stage_begin[host[i].stage] = i;
    }
    stage_begin[d.n_stages] = n;
    int grid = 1;
    for (int st = 0; st < d.n_stages; st++) grid = std::max(grid, prefix[stage_begin[st + 1]] - prefix[stage_begin[st]]);
    grid = std::min(std::min(grid, slots), kBarrierGroup * kBarrierMaxGroups);
    d.grid = grid;
    // spans of each stage: contiguous, of about equal weight (a unit's weights plus a fixed cost); a stage with
    // fewer units than workgroups gives one unit each to the first workgroups (the dispatcher hands the first
    // workgroups of a launch to different CUs)
    std::vector<int> spans;
    for (int st = 0; st < d.n_stages; st++) {
        const int u0 = prefix[stage_begin[st]], u1 = prefix[stage_begin[st + 1]];
        std::vector<int64_t> weight;
        for (int i = stage_begin[st]; i < stage_begin[st + 1]; i++)
            for (int t = 0; t < units_in(i); t++) {
                const int nr = std::min(kFineUnit, host[i].rows - t * kFineUnit);
                weight.push_back((int64_t)nr * host[i].cols * ((host[i].flags & kProblemSwigluGate) ? 2 : 1) + 16384);
            }
        int64_t total_w = 0;
        for (int64_t w : weight) total_w += w;
        std::vector<int> first(grid + 1, u1);
        first[0] = u0;
        const int units = u1 - u0;
        int64_t acc = 0;
        int t = 0;
        for (int g = 1; g < grid; g++) {
            if (units <= grid) {
                t = std::min(g, units);
            } else {
                const int lo = (first[g - 1] - u0) + 1, hi = units - (grid - g);
                const double want = (double)total_w * g / grid;
                while (t < hi && (t < lo || (double)acc < want)) acc += weight[t++];
            }
            first[g] = u0 + t;
        }
        spans.insert(spans.end(), first.begin(), first.end());
        for (int g = 0, pr = stage_begin[st]; g < grid; g++) {
            while (pr + 1 < stage_begin[st + 1] && prefix[pr + 1] <= first[g]) pr++;
            spans.push_back(pr);
        }
    }

    // Hand-over by tagged words (see Sched::exchange) where the plan allows: rows that the one-pass staging holds in
    // registers, nothing quantised inside the launch, and buffers that relate in the plain ways: an input or residual
    // is either exactly the output of an earlier stage (then it is read from that problem's words; the latest such
    // stage counts) or touches no output of the plan (a residual may be its own problem's output: in place); two
    // outputs are either the same buffer in different stages (the earlier store is then completed first) or apart.
    std::vector<Problem> table(host);
    size_t n_words = 0;
    bool exchange = tuning().stage_exchange.load(std::memory_order_relaxed) != 0 && !d.stage_fence && d.n_stages > 1;
    {
        auto lo = [](const void *q) { return reinterpret_cast<uintptr_t>(q); };
        auto cross = [&](const void *a, size_t na, const void *b, size_t nb) { return lo(a) < lo(b) + nb && lo(b) < lo(a) + na; };
        for (Problem &p : table) p.x_words = p.res_words = p.y_words = -1, p.pad_ = 0;
        // the producer of a buffer of `count` halfwords for a reader in stage `st`: -1 none, -2 the buffer relates
        // to some output in a way the words cannot serve
        auto producer_of = [&](const uint16_t *buf, int count, int st, int self) -> int {
            int best = -1;
            for (int j = 0; j < n && best != -2; j++) {
                if (is_up(j) || j == self) continue;
                const Problem &w = host[j];
                if (!cross(buf, (size_t)count * 2, w.y, (size_t)w.rows * 2)) continue;
                if (buf == w.y && count == w.rows) {
                    if (w.stage < st && (best < 0 || host[best].stage <= w.stage)) best = j;
                    else if (w.stage == st) best = -2;  // written and read in one stage
                } else {
                    best = -2;
                }
            }
            return best;
        };
        for (int i = 0; i < n && exchange; i++) {
            Problem &p = table[i];
            const int src = producer_of(p.x, p.cols, p.stage, -1);
            if (src == -2) exchange = false;
            else if (src >= 0) p.x_words = src;  // (the producer's index for now; its words are numbered below)
            if (p.residual) {
                const bool in_place = p.residual == p.y;
                const int r = producer_of(p.residual, p.rows, p.stage, in_place ? i : -1);
                if (r == -2) exchange = false;
                else if (r >= 0) p.res_words = r;
            }
            for (int j = 0; j < i && exchange; j++) {
                if (is_up(i) || is_up(j) || !cross(p.y, (size_t)p.rows * 2, host[j].y, (size_t)host[j].rows * 2)) continue;
                if (p.y == host[j].y && p.rows == host[j].rows && host[j].stage < p.stage) table[j].flags |= kProblemOrderedStore;
                else exchange = false;
            }
        }
        // Without barriers only data orders the stages: a problem may overwrite a buffer that an earlier stage's
        // problem reads as it is (or has written) only if it comes after that problem by a chain of hand-overs.
        if (exchange && n > 64) exchange = false;
        if (exchange) {
            std::vector<uint64_t> after(n, 0);  // bit j: problem i starts after problem j has stored all its outputs
            for (int i = 0; i < n; i++)
                for (int which = 0; which < 2; which++) {
                    int j = which ? table[i].res_words : table[i].x_words;
                    if (j < 0) continue;
                    after[i] |= (uint64_t)1 << j | after[j];
                    if (host[j].flags & kProblemSwigluGate) after[i] |= (uint64_t)1 << (j + 1);  // (the pair's up half)
                }
            for (int i = 0; i < n && exchange; i++) {
                if (is_up(i)) continue;
                const Problem &w = host[i];
                for (int j = 0; j < n && exchange; j++) {
                    if (j == i || host[j].stage >= w.stage) continue;
                    const Problem &r = host[j];
                    const bool reads_x = table[j].x_words < 0 && cross(w.y, (size_t)w.rows * 2, r.x, (size_t)r.cols * 2);
                    const bool reads_res = r.residual && table[j].res_words < 0 && cross(w.y, (size_t)w.rows * 2, r.residual, (size_t)r.rows * 2);
                    const bool wrote = !is_up(j) && cross(w.y, (size_t)w.rows * 2, r.y, (size_t)r.rows * 2);
                    if ((reads_x || reads_res || wrote) && !(after[i] >> j & 1)) exchange = false;
                }
            }
        }
        if (exchange) {
            std::vector<int> first_word(n, -1);
            for (int i = 0; i < n; i++)
                for (int which = 0; which < 2; which++) {
                    const int j = which ? table[i].res_words : table[i].x_words;
                    if (j >= 0 && first_word[j] < 0) {
                        first_word[j] = (int)n_words;
                        n_words += ((size_t)host[j].rows + 31) / 32 * 32;
                    }
                }
            for (int i = 0; i < n; i++) {
                if (table[i].x_words >= 0) table[i].x_words = first_word[table[i].x_words];
                if (table[i].res_words >= 0) table[i].res_words = first_word[table[i].res_words];
                table[i].y_words = first_word[i];
            }
        } else {
            for (Problem &p : table) p.x_words = p.res_words = p.y_words = -1, p.pad_ = 0, p.flags &= ~kProblemOrderedStore;
        }
    }
    d.exchange = exchange;
    d.words_per_slot = n_words;
    d.ints_per_slot = n_words + (size_t)grid;
    // what every workgroup starts every stage with (spans: per stage [grid + 1] first units, then [grid] problems)
    std::vector<WgStart> starts((size_t)d.n_stages * grid);
    for (int st = 0; st < d.n_stages; st++) {
        const int *first = spans.data() + (size_t)st * (2 * grid + 1);
        for (int g = 0; g < grid; g++) {
            WgStart &ws = starts[(size_t)st * grid + g];
            ws = WgStart{};
            ws.u = first[g];
            ws.u_end = first[g + 1];
            ws.pi = first[grid + 1 + g];
            ws.first_unit = prefix[ws.pi];
            ws.p_units = prefix[ws.pi + 1] - prefix[ws.pi];
            ws.p = table[ws.pi];
        }
    }

    auto round16 = [](size_t v) { return (v + 15) / 16 * 16; };
    const size_t bytes_table = round16(sizeof(Problem) * n), bytes_prefix = round16(sizeof(int) * prefix.size());
    const size_t bytes_spans = round16(sizeof(int) * spans.size());
    const size_t bytes_counters = round16(sizeof(int) * (32 + kPlanSlots * kBarrierInts + 32)) + 128;
    const size_t bytes_words = exchange ? (size_t)kPlanSlots * d.ints_per_slot * 4 + 128 : 0;
    const size_t bytes_starts = sizeof(WgStart) * starts.size() + 128;
    char *base = nullptr;
    if (hipError_t e = hipMalloc(&base, bytes_table + bytes_prefix + bytes_spans + bytes_counters + bytes_words + bytes_starts)) return e;
    d.problems = reinterpret_cast<Problem *>(base);
    d.unit_prefix = reinterpret_cast<int *>(base + bytes_table);
    d.wg_first = reinterpret_cast<int *>(base + bytes_table + bytes_prefix);
    // the hand-out counters (unused by staged plans), then, on 128-byte lines, the barriers of the launch slots and the status word
    d.counters = reinterpret_cast<int *>(base + bytes_table + bytes_prefix + bytes_spans);
    d.stage_counters = reinterpret_cast<int *>((reinterpret_cast<uintptr_t>(d.counters + 32) + 127) / 128 * 128);
    d.status = d.stage_counters + kPlanSlots * kBarrierInts;
    d.barrier_bytes = sizeof(int) * ((size_t)kPlanSlots * kBarrierInts + 1);
    // a poll is an uncached load and a short sleep, a microsecond or two: the wait gives up after about a second
    d.spin_limit = 500000;
    if (exchange) {
        // the words of all launch slots (each on a 128-byte line), then every slot's launch counts
        char *w0 = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(base + bytes_table + bytes_prefix + bytes_spans + bytes_counters) + 127) / 128 * 128);
        d.words = reinterpret_cast<uint32_t *>(w0);
    }
    d.starts = reinterpret_cast<WgStart *>((reinterpret_cast<uintptr_t>(base + bytes_table + bytes_prefix + bytes_spans + bytes_counters + bytes_words) + 127) / 128 * 128);
    hipError_t e = hipMemcpy(d.problems, table.data(), sizeof(Problem) * n, hipMemcpyHostToDevice);
    if (!e) e = hipMemcpy(d.starts, starts.data(), sizeof(WgStart) * starts.size(), hipMemcpyHostToDevice);
    if (!e) e = hipMemcpy(d.unit_prefix, prefix.data(), sizeof(int) * prefix.size(), hipMemcpyHostToDevice);
    if (!e) e = hipMemcpy(d.wg_first, spans.data(), sizeof(int) * spans.size(), hipMemcpyHostToDevice);
    if (!e) e = hipMemset(d.counters, 0, bytes_counters);
    if (!e && exchange) e = hipMemset(d.words, 0, (size_t)kPlanSlots * d.ints_per_slot * 4);
    if (const int start = tuning().stage_epoch_start.load(std::memory_order_relaxed); !e && exchange && start != 0) {
        // (every workgroup of every slot starts counting its launches from `start`)
        const std::vector<int> counts((size_t)grid, start);
        for (int slot = 0; slot < kPlanSlots && !e; slot++)
            e = hipMemcpy(d.words + (size_t)slot * d.ints_per_slot + n_words, counts.data(), sizeof(int) * counts.size(), hipMemcpyHostToDevice);
    }
    d.next_slot = new (std::nothrow) std::atomic<unsigned>(0);
    if (!e && !d.next_slot) e = hipErrorOutOfMemory;
    if (e) {
        (void)hipFree(base);
        delete d.next_slot;
        return e;
    }
    *out = d;
    return hipSuccess;
}

hipError_t plan_device_launch(const PlanDevice &plan, hipStream_t s) {
    // the schedule, the table and the counters live on the device the plan was created on
    int dev = -1;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    if (dev != plan.device) return hipErrorInvalidDevice;
    const unsigned slot = plan.next_slot->fetch_add(1, std::memory_order_relaxed) % kPlanSlots;
    int *counters = plan.counters + 2 * slot;
    if (plan.batch_kernel)
        return launch_gemv_batch_table(plan.problems, plan.unit_prefix, plan.wg_first, plan.grid, plan.pool_begin,
                                       plan.pool_end, plan.pool_first, counters, s);
    if (!plan.use_mfma)
        return launch_gemv_rowwave_f16_table(plan.problems, plan.count, plan.max_rows, plan.max_batch, 128, s);
    Sched sc{};
    sc.table = plan.problems;
    sc.unit_prefix = plan.unit_prefix;
    sc.wg_first = plan.wg_first;
    sc.pool_first = plan.pool_first;
    sc.pool_count = plan.pool_count;
    sc.counters = counters;
    sc.x_is_i8 = plan.x_is_i8 ? 1 : 0;
    sc.count = plan.count;
    sc.pair_stride = plan.pair_stride;
    sc.max_units = plan.max_units;
    sc.max_batch = plan.max_batch;
    sc.image_bytes = plan.image_bytes;
    sc.starts = plan.starts;
    if (plan.n_stages > 0) {
        sc.n_stages = plan.n_stages;
        sc.barrier = plan.stage_counters + slot * kBarrierInts;
        sc.stage_fence = plan.stage_fence ? 1 : 0;
        sc.status = plan.status;
        const int limit = tuning().stage_spin_limit.load(std::memory_order_relaxed);
        sc.spin_limit = limit > 0 ? limit : plan.spin_limit;
        if (plan.exchange) {
            sc.exchange = 1;
            sc.words = plan.words + (size_t)slot * plan.ints_per_slot;
            sc.epochs = reinterpret_cast<int *>(sc.words + plan.words_per_slot);
        }
    }
    Problem none{};
    if (plan.extras && plan.fine)
        gemv_mfma_kernel<Wide, true, true><<<plan.grid, kThreads, plan.lds_bytes, s>>>(none, sc);
    else if (plan.extras)
        gemv_mfma_kernel<Wide, true><<<plan.grid, kThreads, plan.lds_bytes, s>>>(none, sc);
    else if (plan.fine && plan.wide)
        gemv_mfma_kernel<Wide, false, true><<<plan.grid, kThreads, plan.lds_bytes, s>>>(none, sc);
    else if (plan.fine)
        gemv_mfma_kernel<Tall, false, true><<<plan.grid, kThreads, plan.lds_bytes, s>>>(none, sc);
    else if (plan.wide)
        gemv_mfma_kernel<Wide><<<plan.grid, kThreads, plan.lds_bytes, s>>>(none, sc);
    else
        gemv_mfma_kernel<Tall><<<plan.grid, kThreads, plan.lds_bytes, s>>>(none, sc);
    return hipGetLastError();
}

void plan_device_destroy(PlanDevice *plan) {
    if (plan->problems) (void)hipFree(plan->problems);
    plan->problems = nullptr;
    delete plan->next_slot;
    plan->next_slot = nullptr;
}

}  // namespace tllm
