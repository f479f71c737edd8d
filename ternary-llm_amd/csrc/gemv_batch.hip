// Batched decode (2..16 activation rows) on the matrix cores (gfx950), group size 128, K % 512 == 0.
//
// Arithmetic (reference kernels/ternary_gemm.cu:106-175 at small M, kernels/ternary_gemv.cu:47-86 per
// row): y[b, r] = sum_g s[r,g] * sum_{k in g} w[r,k] x[b,k], fp32 accumulation, fp16 store (RNE).
// The weights are streamed once for all activation rows: HBM-bound like the batch-1 kernel.
//
// Dataflow. A workgroup of 4 waves owns a block of up to 256 weight rows and walks K in slices of
// 512 columns. Per slice the workgroup turns x[0..16, slice] into ready-made MFMA B operands in LDS
// (power-of-two normalised per activation row and scale group, laid out in the element order of the
// decode below), every wave copies them into 64 registers, and then each wave streams its own tiles
// of 16 rows x 512 columns: lane (row i, chunk q) loads 16 bytes of each mask plane (one scale group
// of one row), four lane-row swaps transpose the 4 x 4 (chunk, word) block held by lanes i, i+16,
// i+32, i+48 so that in each of the four registers all four k-quarters of an MFMA belong to ONE scale
// group, the 2-bit codes are cut out with one AND per two weights (gemv_layout.h) and 4 x 4
// v_mfma_f32_16x16x32_f16 give one 16 x 16 result per scale group: rows x activation rows. The fp32
// group scales multiply whole result tiles; results stay in registers over all slices (every wave
// owns its rows for the whole of K, the two waves that share a tile add up once at the end), so
// there are no atomics.
// The "+1" of the code c = w + 1 is removed by subtracting the product of an all-zero weight row,
// computed once per slice with the same instructions (exact zeros stay exact).
#include <stdlib.h>

#include "common.h"
#include "gemv_layout.h"

namespace tllm {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
typedef uint16_t us2 __attribute__((ext_vector_type(2)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(1))) const u4 GU4;
typedef __attribute__((address_space(1))) const u2 GU2;
#define GB __attribute__((address_space(1)))

constexpr int kNW = 8;                          // waves: 4 tile quarters x 2 slice parities
constexpr int kThreads = kNW * kWave;
constexpr int kSliceCols = 512;                 // 4 scale groups
constexpr int kTileRows = 16;
constexpr int kMaxTilesPerWave = 4;             // tiles of one wave per slice = loads in flight
constexpr int kImageBytes = 16 * kSliceCols * 2;             // operands of one slice, 16 activation rows
constexpr int kMaxOutliers = 128;  // outlier activations a workgroup can hold per block of rows (all activation rows together); more stay in the image

struct BatchSched {
    const Problem *table;    // device table, or nullptr: use the by-value problem
    const int *unit_prefix;  // [count + 1] first block of each problem
    // [grid + 1] first position of each workgroup in `order`, then [grid] the problem its first block is in, then
    // `order`: [pool_begin] the block at each position. A workgroup walks consecutive positions; the blocks there ascend
    // and are chosen by the host so that the workgroups of an XCD work on neighbouring blocks at about the same time.
    const int *wg_first;
    // Blocks [pool_begin, pool_end) belong to no workgroup: whoever has finished its own blocks takes
    // them one at a time through counters[0]. counters[1] counts the workgroups that have left; the
    // last one sets both back to zero for the next launch (launches of one plan must not overlap).
    int pool_begin, pool_end;
    const int *pool_problem;  // [pool_end - pool_begin] the problem each pool block is in
    int *counters;            // nullptr: no pool
    // One problem with few rows and a long K: k_parts workgroups per block, each under its share of the steps
    // (workgroup b works on block b / k_parts, part b % k_parts). Each part leaves its fp32 sums in its slot of
    // `partial`; the part that arrives last at the block's counter in `arrivals` (zero before the launch, zero again
    // after it) adds all slots in part order, its own included, so the bits do not depend on the order of arrival.
    int k_parts;
    float *partial;
    unsigned *arrivals;
};

struct Tile {
    u4 nz, sg;
    u2 sc;  // scales of row 4*lq + (li & 3), groups 4*slice .. +3 (fp16 x 4)
};

__device__ __forceinline__ f4 mfma16(const uint32_t *o, u4 b, f4 c) {
    const u4 a = {o[0], o[1], o[2], o[3]};
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
}

// Lanes i, i+16, i+32, i+48 hold row q of a 4 x 4 matrix in a[0..3] (and of another in b[0..3]); afterwards they hold
// column q. The swaps work in place on the registers they are given; written through the builtins, which return new
// values, the same sequence cost 13 register copies per tile. The compiler does not see inside the block: a vector
// instruction that writes one of these registers must be two wait states away from the swap that reads it, hence
// the leading s_nop (the swaps themselves are interleaved so that each is two instructions behind its producer).
__device__ __forceinline__ void transpose4x2(u4 &a, u4 &b) {
    uint32_t a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3], b0 = b[0], b1 = b[1], b2 = b[2], b3 = b[3];
    asm volatile(
        "s_nop 1\n\t"
        "v_permlane32_swap_b32 %0, %2\n\t"
        "v_permlane32_swap_b32 %1, %3\n\t"
        "v_permlane32_swap_b32 %4, %6\n\t"
        "v_permlane32_swap_b32 %5, %7\n\t"
        "v_permlane16_swap_b32 %0, %1\n\t"
        "v_permlane16_swap_b32 %2, %3\n\t"
        "v_permlane16_swap_b32 %4, %5\n\t"
        "v_permlane16_swap_b32 %6, %7\n\t"
        "s_nop 1"
        : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(b0), "+v"(b1), "+v"(b2), "+v"(b3));
    a = u4{a0, a1, a2, a3};
    b = u4{b0, b1, b2, b3};
}

// The value lane `kFrom` of each quad holds, in all four lanes of the quad.
template <int kFrom>
__device__ __forceinline__ uint32_t quad_broadcast(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, kFrom * 0x55, 0xF, 0xF, true);
}

// kTilesPerWave: 4 for long streams (256-row blocks amortise the per-slice operand build best);
// 2 or 1 when one matrix alone must fill the chip (128- and 64-row blocks).
template <int kTilesPerWave>
__global__ __launch_bounds__(kThreads, 1) void gemv_batch_kernel(Problem single, BatchSched sc) {
    constexpr int kBlockRows = 4 * kTilesPerWave * kTileRows;
    // [buffer][slice parity]: the operands of two neighbouring slices are built per step
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    unsigned char (*image)[2][kImageBytes] = reinterpret_cast<unsigned char (*)[2][kImageBytes]>(lds_raw);
    // per scale group of the slice and activation row: 2^(ex + 10) of the group, 0 for an all-zero group
    float (*pow2)[2][4][16] = reinterpret_cast<float (*)[2][4][16]>(lds_raw + 4 * kImageBytes);

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    // Wave w works on tile quarter w % 4 under the slices of parity w / 4. The two waves that share
    // their tiles read the two 64-byte halves of every 128-byte line of the mask planes at about the
    // same time, so each line comes from HBM once (one wave walking all slices fetched it twice).
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = wave8 & 3;
    const int parity = wave8 >> 2;
    const int li = lane & 15;  // MFMA A row / D column (activation row)
    const int lq = lane >> 4;  // MFMA k quarter / D row quad

    // pos walks positions (plan: of `order`; single problem: the blocks themselves), u is the block there
    int pos = 0, pos_end = 0, pi = 0;
    const int *order = nullptr;
    if (sc.table) {
        pos = sc.wg_first[blockIdx.x];
        pos_end = sc.wg_first[blockIdx.x + 1];
        pi = sc.wg_first[gridDim.x + 1 + blockIdx.x];  // no scan over the problems before the first block
        order = sc.wg_first + 2 * gridDim.x + 1;
    } else if (sc.k_parts > 1) {
        pos = blockIdx.x / sc.k_parts;
        pos_end = pos + 1;
    } else {
        const int total = (single.rows + kBlockRows - 1) / kBlockRows;
        pos = (int)((int64_t)total * blockIdx.x / gridDim.x);
        pos_end = (int)((int64_t)total * (blockIdx.x + 1) / gridDim.x);
    }
    const int k_parts = sc.k_parts > 1 ? sc.k_parts : 1;
    const int k_part = sc.k_parts > 1 ? (int)(blockIdx.x % sc.k_parts) : 0;

    // operands of an all-zero weight row (every code = 1)
    uint32_t zero_o[16];
    decode_word(0u, 0u, zero_o);

    // Activations that stay out of the operand images (see build_image): column, fp16 bits | activation row << 16.
    // The list is rebuilt for every block of weight rows, since every block walks the whole of its K range.
    __shared__ int n_outliers;
    __shared__ int out_col[kMaxOutliers];
    __shared__ uint32_t out_val[kMaxOutliers];
    if (tid == 0) n_outliers = 0;
    __syncthreads();

    Problem p = single;
    __shared__ int pool_block;
    bool in_pool = false;
    for (;; pos++) {
        if (pos >= pos_end) {
            // own blocks done: go on with the pool block asked for while the last block was running
            // (the barriers that end a block separate the write of pool_block, this read, and the
            // next write)
            if (!sc.counters) break;
            const int t = __builtin_amdgcn_readfirstlane(pool_block);
            if (t >= sc.pool_end - sc.pool_begin) break;
            pos = sc.pool_begin + t;
            pos_end = pos + 1;
            pi = sc.pool_problem[t];
            in_pool = true;
        }
        // the pool's blocks come after all others and are their own positions; the blocks of a workgroup's own
        // positions ascend, so the scan for the problem below only moves forward
        const int u = order && !in_pool ? order[pos] : pos;
        // the last block of the span, or a pool block: ask for the next pool block
        const bool request = sc.counters != nullptr && pos + 1 >= pos_end && tid == 0;
        int requested = 0;
        if (request) requested = __hip_atomic_fetch_add(sc.counters, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int first_unit = 0;
        if (sc.table) {
            while (sc.unit_prefix[pi + 1] <= u) pi++;
            first_unit = sc.unit_prefix[pi];
            p = sc.table[pi];
        }
        const int r0 = (u - first_unit) * kBlockRows;
        const int n_tiles = (min(kBlockRows, p.rows - r0) + kTileRows - 1) / kTileRows;
        const int words = p.cols / 32, groups = p.cols / kChunkCols, slices = p.cols / kSliceCols;

        // ---- this wave's tiles: k-th tile is tile number 4k + wave of the block. Tiles past the end
        // of the block re-read its last tile (not stored); a tile that would pass the end of the
        // matrix is moved back to end with it, the rows it repeats are not stored.
        const char GB *nz_g = (const char GB *)p.nz;
        const char GB *sg_g = (const char GB *)p.sg;
        const char GB *sc_g = (const char GB *)p.scales;
        // Addresses: a wave-uniform part per tile (first row) plus one per-lane offset for all tiles.
        auto tile_first_row = [&](int k, int *skip) -> int {
            const int rb = r0 + min(4 * k + wave, n_tiles - 1) * kTileRows;
            const int rbe = min(rb, p.rows - kTileRows);
            if (skip) *skip = rb - rbe;
            return rbe;
        };
        const uint32_t lane_mask_off = ((uint32_t)li * words + 4u * lq) * 4u;
        // Scales: a lane holds the results of rows 4*lq + v, v = 0..3 (MFMA D layout). It loads the scales of row
        // 4*lq + (li & 3) only, so that the four lanes of every quad of lane quarter lq hold rows 4*lq .. 4*lq + 3, and
        // takes the other three from its quad neighbours (one DPP move per register): one load per tile whose 64 lanes
        // ask for 16 different addresses, four neighbouring lanes for four neighbouring rows. (With the MFMA operands
        // exchanged a lane would need the scales of one row only and no DPP moves, but its load, 16 different rows in
        // 16 neighbouring lanes, cost more than the moves save: 3 % slower at 5 and 8 activation rows.) They travel
        // with the masks of the same tile and slice, a whole step ahead: the loads of a wave return in order, and a
        // scale load asked for later than the masks it belongs to would make its tile wait for every mask load issued
        // before it.
        const uint32_t lane_scale_off = (uint32_t)(4 * lq + (li & 3)) * groups * 2u;
        auto load_tile = [&](int k, int slice) -> Tile {
            Tile t;
            const int first = tile_first_row(k, nullptr);
            const size_t base = (size_t)first * words * 4 + (size_t)slice * 64;
            t.nz = *reinterpret_cast<const GU4 *>(nz_g + base + lane_mask_off);
            t.sg = *reinterpret_cast<const GU4 *>(sg_g + base + lane_mask_off);
            t.sc = *reinterpret_cast<const GU2 *>(sc_g + (size_t)first * groups * 2 + (size_t)slice * 8 + lane_scale_off);
            return t;
        };

        // ---- activations: thread (row j = tid / 16, segment = tid % 16) owns 32 columns of a slice
        const int xpar = tid >> 8, xj = (tid >> 4) & 15, xseg = tid & 15;
        const bool x_live = xj < p.batch;
        const GU4 *x_src = (const GU4 *)(p.x + (size_t)(x_live ? xj : 0) * p.cols) + xseg * 4;
        // Every thread loads, also where the image is to be zeros (an activation row past the batch, the slice past
        // the end of an odd number of slices): loads under a branch would leave the number of loads in flight unknown
        // to the compiler, which then waits for all of them before a tile's masks are used.
        auto load_x = [&](u4 (&xr)[4], int slice) {
            const int sl = min(slice, slices - 1);
#pragma unroll
            for (int i = 0; i < 4; i++) xr[i] = x_src[sl * (kSliceCols / 8) + i];
        };
        // builds the operands of one slice: element (chunk c, word q, step t, row j, e) at
        // ((c*4 + t)*64 + q*16 + j)*16 + 2e bytes: lane (j, q) of MFMA (c, t) reads 16 contiguous bytes
        // (`dead`: write zeros whatever was loaded)
        auto build_image = [&](const u4 (&xr)[4], int buf, bool dead, int slice) {
            // largest magnitude of the activation row inside the thread's SCALE GROUP (128 columns: the four threads
            // of a quad): packed unsigned maximum of the sign-stripped halves, then across the quad (two DPP swaps).
            // Every group is normalised by itself, so an outlier activation costs precision only inside its own
            // group; 2^(ex+10) of the group meets the group's result tile beside its fp32 scale.
            us2 m2 = {0, 0};
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(us2, xr[i][e] & 0x7FFF7FFFu));
            uint32_t m = max((uint32_t)m2[0], (uint32_t)m2[1]);
            if (dead) m = 0;
            uint32_t src[16];
#pragma unroll
            for (int d = 0; d < 16; d++) src[d] = xr[d >> 2][d & 3];
            // Outliers first. The matrix product sees the codes w + 1, so an activation also enters the fp32 sums of the
            // rows whose weight on its column is ZERO, to be cancelled against the all-zero-row product: that costs every
            // such row about 2^-21 of the activation's magnitude, and would carry an Inf or NaN into every row. An element
            // more than 2^8 times the smallest non-zero thread maximum of its group (a robust "typical magnitude"; Inf and
            // NaN always) stays OUT of the image: it goes to a short list, and the end of the block adds scale * w * x
            // for it to the rows that hold a weight there, term by term in fp32 like the reference
            // (kernels/ternary_gemm.cu:131-155). When the list is full the element stays in the image.
            uint32_t t = m ? m : 0xFFFFu;
            t = min(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
            t = min(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
            const uint32_t limit = min(t + (8u << 10), 0x7BFFu);  // fp16 bits: 2^8 times t, at most the largest finite number
            if (m > limit) {
                m = 0;
#pragma unroll
                for (int d = 0; d < 16; d++)
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const uint32_t bits = (src[d] >> (16 * h)) & 0xFFFFu;
                        if ((bits & 0x7FFFu) > limit) {
                            const int slot = __hip_atomic_fetch_add(&n_outliers, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                            if (slot < kMaxOutliers) {
                                out_col[slot] = slice * kSliceCols + xseg * 32 + 2 * d + h;
                                out_val[slot] = bits | (uint32_t)xj << 16;
                                src[d] &= ~(0xFFFFu << (16 * h));
                            }
                        }
                        m = max(m, (src[d] >> (16 * h)) & 0x7FFFu);
                    }
            }
            m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
            m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
            // byte selectors of the permutes below; selector 0x0C yields a zero byte
            const uint32_t sel_lo = dead ? 0x0C0C0C0Cu : 0x05040100u, sel_hi = dead ? 0x0C0C0C0Cu : 0x07060302u;
            // amax in [2^ex, 2^(ex+1)); x'' = x * 2^(14-ex) stays below 2^15
            int ex = 0;
            if (m >= 0x7C00u) ex = 15;  // inf/nan present: they propagate to the outputs
            else if (m) ex = (int)((__builtin_bit_cast(uint32_t, h2f((uint16_t)m)) >> 23) & 0xFF) - 127;
            // The multipliers 2^(14-ex-p), p = 2..10, must be normal fp16 numbers: ex >= -3. Rows with
            // a smaller maximum are normalised as if it were 2^-3: their multipliers are then >= 2^7,
            // and multiplying an fp16 number by a power of two >= 1 is exact (no overflow: |x| < 2^-2).
            const int exl = max(ex, -3);
            if ((xseg & 3) == 0) pow2[buf][xpar][xseg >> 2][xj] = m ? __builtin_bit_cast(float, (uint32_t)(127 + exl + 10) << 23) : 0.0f;
            const int c = xseg >> 2, q = xseg & 3;
            // Operand t = 2z + h, dword d' holds the elements of decode dword m = 4h + d' (gemv_layout.h):
            // column 2m + z in its low half, column 2(m + 8) + z in its high half (m = 0: the other
            // way round); both sit in half z of source dwords m and m + 8. One byte permute and one
            // packed multiply by 2^(14-ex-p(m)) per dword; the product of an fp16 number and a power of
            // two is exact or rounded once to nearest even, as in the fp32 route.
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int z = t >> 1, h = t & 1;
                u4 v;
#pragma unroll
                for (int dq = 0; dq < 4; dq++) {
                    const int mm = 4 * h + dq;
                    const uint32_t lo = mm == 0 ? src[8] : src[mm], hi = mm == 0 ? src[0] : src[mm + 8];
                    const uint32_t pair = __builtin_amdgcn_perm(hi, lo, z ? sel_hi : sel_lo);
                    const uint16_t cbits = (uint16_t)((29 - exl - code_shift(mm)) << 10);
                    const h2 mult = __builtin_bit_cast(h2, (uint32_t)cbits | ((uint32_t)cbits << 16));
                    v[dq] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, pair) * mult);
                }
                *reinterpret_cast<u4 *>(&image[buf][xpar][(((c * 4 + t) * 64) + q * 16 + xj) * 16]) = v;
            }
        };

        f4 acc[kTilesPerWave];
#pragma unroll
        for (int k = 0; k < kTilesPerWave; k++) acc[k] = f4{0.f, 0.f, 0.f, 0.f};

        const int steps = (slices + 1) / 2;
        const int st_begin = steps * k_part / k_parts, st_end = steps * (k_part + 1) / k_parts;
        auto my_slice = [&](int step) -> int { return min(2 * step + parity, slices - 1); };  // weights: clamped
        u4 xr[4];
        load_x(xr, 2 * st_begin + xpar);
        // The first loads are issued in the order the loop issues them (activations, then tile by tile): the
        // compiler's count of loads in flight at the top of the loop is the worse of the two ways into it.
        __builtin_amdgcn_sched_barrier(0);
        Tile ring[kTilesPerWave];
#pragma unroll
        for (int k = 0; k < kTilesPerWave; k++) {
            ring[k] = load_tile(k, my_slice(st_begin));
            __builtin_amdgcn_sched_barrier(0);
        }

        for (int st = st_begin; st < st_end; st++) {
            const int buf = st & 1;
            build_image(xr, buf, !x_live || 2 * st + xpar >= slices, 2 * st + xpar);
            load_x(xr, 2 * (st + 1) + xpar);
            // one barrier per step: it publishes buffer `buf`; the other buffer is rewritten only in
            // the next iteration, after every wave has passed this barrier and so has finished
            // reading it into registers.
            __syncthreads();
            u4 B[16];
#pragma unroll
            for (int k = 0; k < 16; k++) B[k] = *reinterpret_cast<const u4 *>(&image[buf][parity][(k * 64 + lane) * 16]);
            // the product of an all-zero weight row (the "+1" of every code), formed exactly like a
            // tile's own product, so that subtracting it leaves exact zeros where the weights are zero; both meet
            // the group's factor 2^(ex+10) of this lane's activation row in one fused multiply-add (the product of
            // the bias and a power of two is exact)
            float pg[4];
            f4 bias[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                pg[c] = pow2[buf][parity][c][li];
                f4 d0 = {0.f, 0.f, 0.f, 0.f};
                d0 = mfma16(zero_o + 0, B[4 * c + 0], d0);
                d0 = mfma16(zero_o + 4, B[4 * c + 1], d0);
                d0 = mfma16(zero_o + 8, B[4 * c + 2], d0);
                d0 = mfma16(zero_o + 12, B[4 * c + 3], d0);
                bias[c] = d0 * pg[c];
            }
            const int s_next = my_slice(min(st + 1, st_end - 1));
#pragma unroll
            for (int k = 0; k < kTilesPerWave; k++) {
                Tile t = ring[k];
                transpose4x2(t.nz, t.sg);
                // sq[v][h]: scales of row 4*lq + v, groups 2h and 2h + 1 of the slice
                uint32_t sq[4][2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    sq[0][h] = quad_broadcast<0>(t.sc[h]);
                    sq[1][h] = quad_broadcast<1>(t.sc[h]);
                    sq[2][h] = quad_broadcast<2>(t.sc[h]);
                    sq[3][h] = quad_broadcast<3>(t.sc[h]);
                }
                f4 r = {0.f, 0.f, 0.f, 0.f};
                // One chain of four MFMAs per scale group. The chains of two groups are issued alternately, so that an
                // MFMA never follows the one it depends on directly, and the results of the first pair are touched only
                // after the second pair has been issued (+ 1 % against one chain after the other).
                f4 da[2], db[2];
                auto issue_pair = [&](int c, f4 (&d)[2]) {
                    uint32_t o0[16], o1[16];
                    decode_word(t.nz[c], t.sg[c], o0);
                    decode_word(t.nz[c + 1], t.sg[c + 1], o1);
                    d[0] = mfma16(o0 + 0, B[4 * c + 0], f4{0.f, 0.f, 0.f, 0.f});
                    d[1] = mfma16(o1 + 0, B[4 * c + 4], f4{0.f, 0.f, 0.f, 0.f});
                    d[0] = mfma16(o0 + 4, B[4 * c + 1], d[0]);
                    d[1] = mfma16(o1 + 4, B[4 * c + 5], d[1]);
                    d[0] = mfma16(o0 + 8, B[4 * c + 2], d[0]);
                    d[1] = mfma16(o1 + 8, B[4 * c + 6], d[1]);
                    d[0] = mfma16(o0 + 12, B[4 * c + 3], d[0]);
                    d[1] = mfma16(o1 + 12, B[4 * c + 7], d[1]);
                };
                auto retire = [&](int c, const f4 &dc) {
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const uint16_t sbits = (uint16_t)(sq[v][c >> 1] >> (16 * (c & 1)));
                        r[v] += h2f(sbits) * __builtin_fmaf(dc[v], pg[c], -bias[c][v]);
                    }
                };
                issue_pair(0, da);
                __builtin_amdgcn_sched_barrier(0);
                issue_pair(2, db);
                retire(0, da[0]);
                retire(1, da[1]);
                __builtin_amdgcn_sched_barrier(0);
                // The next slice of this tile is asked for only now that the registers of this one are dead (the masks,
                // in which the swaps above worked in place; the scales went to their quads at the top), so that the
                // loads write the registers the loop carries: a request placed earlier loads into other registers, and
                // the copies into the carried ones at the end of the step wait for every load in flight.
                __builtin_amdgcn_sched_barrier(0);
                ring[k] = load_tile(k, s_next);
                __builtin_amdgcn_sched_barrier(0);
                retire(2, db[0]);
                retire(3, db[1]);
                acc[k] += r;
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // ---- the odd-slice waves hand their sums to their even-slice partners through LDS (the image
        // buffers are free once every wave is past its last step), which add and store
        __syncthreads();
        float *hand = reinterpret_cast<float *>(&image[0][0][0]) + (size_t)wave * (kTilesPerWave * 4 * kWave);
        if (parity == 1) {
#pragma unroll
            for (int k = 0; k < kTilesPerWave; k++)
#pragma unroll
                for (int v = 0; v < 4; v++) hand[(k * 4 + v) * kWave + lane] = acc[k][v];
        }
        // (the list is complete: every append lies before the barrier above; it is cleared for the next block behind
        // the barrier below, so every thread takes its length here)
        const int n_out = min(n_outliers, kMaxOutliers);
        __syncthreads();
        if (parity == 0) {
#pragma unroll
            for (int k = 0; k < kTilesPerWave; k++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc[k][v] += hand[(k * 4 + v) * kWave + lane];
        }
        // what the activations that stayed out of the images add: scale * (+-x) to the rows that hold a weight on the
        // column (lane (lq, li) holds rows first + 4 lq + v of activation row li)
        if (n_out && parity == 0) {
            for (int o = 0; o < n_out; o++) {
                const uint32_t vb = out_val[o];
                if ((int)(vb >> 16) != li) continue;
                const int col = out_col[o];
                const uint32_t bit = 1u << (col & 31);
                const float xv = h2f((uint16_t)vb);
#pragma unroll
                for (int k = 0; k < kTilesPerWave; k++) {
                    const int first = tile_first_row(k, nullptr);
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const size_t row = (size_t)(first + 4 * lq + v);
                        const size_t at = row * words + (col >> 5);
                        if (p.nz[at] & bit) acc[k][v] += h2f(p.scales[row * groups + (col >> 7)]) * ((p.sg[at] & bit) ? xv : -xv);
                    }
                }
            }
        }
        bool stores = true;
        if (k_parts > 1) {  // (the same for the whole workgroup)
            // this part's sums into its slot, written through to memory: quad k of lane `lane` of wave `wave` at
            // ((wave * kTilesPerWave + k) * 64 + lane) * 4 floats
            constexpr int kSlot = 4 * kTilesPerWave * kWave * 4;
            float *slots = sc.partial + (size_t)u * k_parts * kSlot + ((size_t)wave * kTilesPerWave * kWave + lane) * 4;
            if (parity == 0) {
#pragma unroll
                for (int k = 0; k < kTilesPerWave; k++) {
                    float *dst = slots + (size_t)k_part * kSlot + k * kWave * 4;
                    const f4 v = acc[k];
                    // (two idle issue slots: a store of more than 8 bytes still reads its data registers after it
                    // has issued, and the compiler does not see inside the block)
                    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __shared__ unsigned last_part;
            __syncthreads();
            if (tid == 0) {
                const unsigned before = __hip_atomic_fetch_add(&sc.arrivals[u], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                last_part = before == (unsigned)k_parts - 1;
                if (last_part) __hip_atomic_store(&sc.arrivals[u], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();
            stores = last_part != 0;
            if (stores && parity == 0) {
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#pragma unroll
                for (int k = 0; k < kTilesPerWave; k++) acc[k] = f4{0.f, 0.f, 0.f, 0.f};
                for (int q = 0; q < k_parts; q++)
#pragma unroll
                    for (int k = 0; k < kTilesPerWave; k++)
                        acc[k] += *reinterpret_cast<const f4 *>(slots + (size_t)q * kSlot + k * kWave * 4);
            }
        }
        // lane (lq, li) holds rows first + 4*lq + v of activation row li
        if (stores && parity == 0 && li < p.batch) {
#pragma unroll
            for (int k = 0; k < kTilesPerWave; k++) {
                if (4 * k + wave >= n_tiles) continue;
                int skip = 0;
                const int first = tile_first_row(k, &skip);
#pragma unroll
                for (int v = 0; v < 4; v++)
                    if (4 * lq + v >= skip) p.y[(size_t)li * p.rows + first + 4 * lq + v] = f2h(acc[k][v]);
            }
        }
        if (request) pool_block = requested;
        if (tid == 0) n_outliers = 0;  // (every thread took the length before the second barrier of the hand-over)
        __syncthreads();  // the next block rewrites the image buffers
    }
    if (sc.counters && tid == 0) {
        const int left = __hip_atomic_fetch_add(sc.counters + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left == (int)gridDim.x - 1) {  // every other workgroup has made its last request
            __hip_atomic_store(sc.counters, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(sc.counters + 1, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

int device_cus() { return current_device_cus(); }

}  // namespace

bool gemv_batch_supports(const Problem &p, int group) {
    return group == 128 && p.batch >= 1 && p.batch <= 16 && p.rows >= kTileRows && p.cols >= kSliceCols &&
           p.cols % kSliceCols == 0 && (reinterpret_cast<uintptr_t>(p.scales) & 7) == 0 &&
           (size_t)p.rows * (p.cols / 8) < ((size_t)1 << 32) && (size_t)p.rows * (p.cols / 128) * 2 < ((size_t)1 << 32);
}

constexpr size_t kLdsBytes = 4 * kImageBytes + 2 * 2 * 4 * 16 * sizeof(float);

template <int T>
static hipError_t prepare_kernel() {
    static std::atomic<bool> done[64];  // per device; setting the attribute twice is harmless
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    if (dev < 0 || dev >= 64 || done[dev].load(std::memory_order_acquire)) return hipSuccess;
    if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_batch_kernel<T>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes))
        return e;
    done[dev].store(true, std::memory_order_release);
    return hipSuccess;
}

template <int T>
static hipError_t launch_single(const Problem &p, int wgs, int k_parts, float *partial, unsigned *arrivals, hipStream_t s) {
    if (hipError_t e = prepare_kernel<T>()) return e;
    const int blocks = (p.rows + 64 * T - 1) / (64 * T);
    BatchSched sc{};
    sc.k_parts = k_parts;
    sc.partial = partial;
    sc.arrivals = arrivals;
    const int grid = k_parts > 1 ? blocks * k_parts : blocks < wgs ? blocks : wgs;
    gemv_batch_kernel<T><<<grid, kThreads, kLdsBytes, s>>>(p, sc);
    return hipGetLastError();
}

// tiles per wave for one matrix alone: the largest block size that still gives every CU a block
static int single_tiles(const Problem &p, int cus) {
    for (int t = kMaxTilesPerWave; t > 1; t /= 2)
        if ((p.rows + 64 * t - 1) / (64 * t) >= cus) return t;
    return 1;
}

// Time of one matrix alone in 64-row blocks whose steps are shared out among `parts` workgroups each, in us, fitted to
// eleven shapes of 512 to 8192 rows and 4096 to 28672 columns (within 1.5 us on all of them): 3 us of launch and
// ramp, 1.78 us per step of 1024 columns, and for the exchange 1.5 us + 0.2 us per part + 0.027 us per workgroup of the
// launch (256 workgroups start and arrive noticeably later than 64).
static float single_split_us(int blocks, int steps, int parts) {
    const float chain = 3.0f + 1.78f * (float)((steps + parts - 1) / parts);
    return parts > 1 ? chain + 1.5f + 0.2f * (float)parts + 0.027f * (float)(blocks * parts) : chain;
}

// Workgroups per 64-row block along K for one matrix alone: with so few rows that CUs would stay without a block,
// the steps of a block may be shared out among up to 8 workgroups, as many as the estimate above likes best.
static int single_k_parts(const Problem &p, int cus) {
    if (single_tiles(p, cus) != 1) return 1;
    const int blocks = (p.rows + 63) / 64;
    const int steps = (p.cols / kSliceCols + 1) / 2;
    int most = cus / blocks;
    if (most > steps) most = steps;
    if (most > 8) most = 8;
    if (most < 2 || blocks > kSplitArrivalSlots) return 1;
    // tuning switch batch_k_parts = n: n parts where they fit, 1 = never share out K
    const int forced = tuning().batch_k_parts.load(std::memory_order_relaxed);
    if (forced > 0) return forced < most ? forced : most;
    int best = 1;
    for (int parts = 2; parts <= most; parts++)
        if (single_split_us(blocks, steps, parts) < single_split_us(blocks, steps, best)) best = parts;
    return best;
}
static size_t single_exchange_floats(const Problem &p, int parts) {
    return (size_t)((p.rows + 63) / 64) * parts * (4 * kWave * 4);
}

hipError_t launch_gemv_batch(const Problem &p, hipStream_t s, bool fixed_scratch) {
    const int cus = device_cus();  // one workgroup of 8 waves per CU
    int parts = single_k_parts(p, cus);
    float *partial = nullptr;
    unsigned *arrivals = nullptr;
    if (parts > 1) {
        // (no exchange memory to be had, e.g. under stream capture without a reserved workspace: one workgroup per block)
        if (hipError_t e = split_exchange_memory(s, single_exchange_floats(p, parts), fixed_scratch, &partial, &arrivals)) return e;
        if (!partial) parts = 1;
    }
    switch (single_tiles(p, cus)) {
        case 4: return launch_single<4>(p, cus, 1, nullptr, nullptr, s);
        case 2: return launch_single<2>(p, cus, 1, nullptr, nullptr, s);
        default: return launch_single<1>(p, cus, parts, partial, arrivals, s);
    }
}

const char *gemv_batch_kernel_name(const Problem &p) {
    return single_k_parts(p, device_cus()) > 1 ? "tllm::gemv_batch_kernel, K shared out" : "tllm::gemv_batch_kernel";
}

hipError_t gemv_batch_reserve(const Problem &p, hipStream_t s) {
    const int parts = single_k_parts(p, device_cus());
    float *partial = nullptr;
    unsigned *arrivals = nullptr;
    return parts > 1 ? split_exchange_memory(s, single_exchange_floats(p, parts), false, &partial, &arrivals) : hipSuccess;
}

float gemv_batch_cost_us(const Problem &p) {
    // measured on single matrices: 3 us of launch and ramp, then the larger of the streaming time
    // (a workgroup moves about 17 bytes of packed weights per ns with 256-row blocks, 13 with 64-row
    // blocks) and the latency chain of the K loop (1.8 us per step of 1024 columns; single_split_us when
    // the steps of a block are shared out)
    const int cus = device_cus();
    const int t = single_tiles(p, cus);
    const int parts = single_k_parts(p, cus);
    const int blocks = (p.rows + 64 * t - 1) / (64 * t);
    const int wgs = blocks * parts;
    const float rate = (t == 4 ? 17.0e3f : t == 2 ? 15.0e3f : 13.0e3f) * (float)(wgs < cus ? wgs : cus);
    const float stream = 3.0f + 0.265625f * (float)p.rows * (float)p.cols / rate;
    const float chain = single_split_us(blocks, (p.cols / kSliceCols + 1) / 2, parts);
    return stream > chain ? stream : chain;
}

int gemv_batch_block_rows() { return 64 * kMaxTilesPerWave; }

hipError_t launch_gemv_batch_table(const Problem *table, const int *unit_prefix, const int *wg_first, int grid,
                                   int pool_begin, int pool_end, const int *pool_problem, int *counters,
                                   hipStream_t s) {
    if (hipError_t e = prepare_kernel<kMaxTilesPerWave>()) return e;
    BatchSched sc{table, unit_prefix, wg_first, pool_begin, pool_end, pool_problem,
                  pool_end > pool_begin ? counters : nullptr, 1, nullptr, nullptr};
    Problem none{};
    gemv_batch_kernel<kMaxTilesPerWave><<<grid, kThreads, kLdsBytes, s>>>(none, sc);
    return hipGetLastError();
}

}  // namespace tllm
