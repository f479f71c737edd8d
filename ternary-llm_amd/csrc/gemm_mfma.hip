// Prefill GEMM on the matrix cores (gfx950), group size 128, M >= 16.
//
// Arithmetic (reference kernels/ternary_gemm.cu:106-175): C[m,n] = sum_k scale[n, k/128] * w[n,k] * A[m,k],
// the scale multiplied into every element, fp32 accumulation, fp16 store (round to nearest even).
// Here the product scale * w is formed exactly in fp16 (w in {-1,0,+1}), so the only difference to
// the reference is the order of the fp32 additions.
//
// Tiling. A workgroup (4 waves) computes 128 weight rows x BM activation rows; every wave owns all
// 128 weight rows and BM/4 activation rows of its own. Per stage of 64 columns of K:
//   * weights: each thread decodes one 32-bit mask word pair of one weight row into LDS. One
//     v_bitop3 puts the 2-bit field (negative, non-zero) of every even/odd weight in place, two
//     v_perm gather the fields of weights (2f, 2f+1) into the two halves of one dword; shifted to
//     the top of an fp16 half that field IS the number 0, +2.0 or -2.0 (bit 15 = sign, bit 14 =
//     exponent MSB), so a packed shift, an AND and a packed fp16 multiply by the group scale give
//     two elements +-2*scale: 1.7 vector operations per weight, once per workgroup. The factor 2
//     is undone on the fp32 accumulators at the end (exact);
//   * everything that comes from global memory (activations, mask words, scales) is written into
//     LDS by the load instruction itself (global_load_lds), two to three stages ahead, without
//     passing through registers. Activations are private to a wave: lane p of a load asks for the
//     16-byte chunk that belongs at byte 16 p of the destination block under the row swizzle, so
//     every load reads eight full 128-byte lines. (Loading the MFMA operand straight into
//     registers instead needs 16 different rows per 16 lanes and was 2.5 times slower.)
//   * each wave multiplies with v_mfma_f32_16x16x32_f16; inside a stage the MFMA with index ks
//     sums columns 16q + 8ks .. + 7 for lane quad q (both operands use the same assignment, so the
//     sum over the stage is complete); operands come from LDS as 16-byte chunks, XOR-swizzled by
//     row against bank conflicts.
// Three LDS buffers per operand, one barrier per stage; the loop body spells out the pipeline.
#include <stdlib.h>

#include <mutex>
#include <type_traits>

#include "common.h"

namespace tllm {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef uint16_t us2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int kBN = 128;     // weight rows per workgroup
constexpr int kBK = 64;      // K columns per stage (two MFMA steps of 32)
constexpr int kThreads = 256;
constexpr int kRowBytes = kBK * 2;  // one LDS row: 64 fp16 = 8 chunks of 16 bytes
constexpr int kNF = kBN / 32;       // MFMA row fragments (32 weight rows each) per wave
constexpr int kWBytes = kBN * kRowBytes;

// byte offset of 16-byte chunk c (0..7) of row r inside the [128][64] fp16 LDS tile
// The swizzle keeps a 16-byte fragment read free of bank conflicts both for 8 consecutive rows on 32 banks
// and for 16 consecutive rows on 64 banks (rows r and r + 8 lie 1 KB apart: same bank either way).
__device__ __forceinline__ int row_swizzle(int r) { return (r & 7) ^ ((r >> 3) & 1); }
__device__ __forceinline__ int chunk_off(int r, int c) { return r * kRowBytes + ((c ^ row_swizzle(r)) << 4); }

// Decoder of 32 weights (one mask word pair) into 16 dwords; dword d holds weights (2d, 2d + 1) as
// +-2*scale / 0. Split in steps so that the caller can spread the work between MFMAs.
struct Decoder {
    uint32_t q[2];
    h2 sp;
    __device__ __forceinline__ void begin(uint32_t nz, uint32_t sg, uint32_t scale) {
        const uint32_t neg = nz & ~sg;
        // field (negative, non-zero) of weight 2f+z at bits (2f+1, 2f) of t[z]:  (a & c) | (b & ~c), c = 0xAAAAAAAA
        const uint32_t t0 = __builtin_amdgcn_bitop3_b32(neg << 1, nz, 0xAAAAAAAAu, 0xE4);
        const uint32_t t1 = __builtin_amdgcn_bitop3_b32(neg, nz >> 1, 0xAAAAAAAAu, 0xE4);
        q[0] = __builtin_amdgcn_perm(t1, t0, 0x05040100u);  // low half: weights 0,2,..,14; high half: 1,3,..,15
        q[1] = __builtin_amdgcn_perm(t1, t0, 0x07060302u);  // the same for weights 16..31
        sp = __builtin_bit_cast(h2, scale | (scale << 16));
    }
    // dword d (0..15)
    __device__ __forceinline__ uint32_t dword(int d) const {
        us2 v = __builtin_bit_cast(us2, q[d >> 3]);
        v = v << (uint16_t)(14 - 2 * (d & 7));  // field of both halves to bits 15:14
        const uint32_t top = __builtin_bit_cast(uint32_t, v) & 0xC000C000u;  // 0, +2.0 or -2.0
        return __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, top) * sp);
    }
};

constexpr int kBufs = 3;  // LDS buffers per operand (stages in flight)

template <int MF>  // MFMA column fragments (32 activation rows each) per wave
__global__ __launch_bounds__(kThreads, 1) void gemm_mfma_kernel(
    const uint16_t *__restrict__ A, const uint32_t *__restrict__ nzB, const uint32_t *__restrict__ sgB,
    const uint16_t *__restrict__ scB, uint16_t *__restrict__ C, int M, int N, int K, int splits,
    float *__restrict__ partial, unsigned *__restrict__ arrivals) {
    constexpr int kWM = MF * 32;             // activation rows per wave
    constexpr int BM = 4 * kWM;
    constexpr int kActWave = kWM * kRowBytes;  // bytes of one wave's activation tile per stage
    constexpr int kActBytes = 4 * kActWave;
    constexpr int kActBase = kBufs * kWBytes;  // weights buffers first, activation buffers behind them
    constexpr int kMaskBase = kActBase + kBufs * kActBytes;  // raw mask words and scales: 3 planes of 1 KB per buffer
    constexpr int kMaskBytes = 3 * 1024;
    constexpr int kDma = kWM / 8;              // direct-to-LDS loads per wave and stage (8 rows of 128 bytes each)
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    typedef __attribute__((address_space(3))) unsigned char LB;
    LB *lds_dma = (LB *)lds;  // the same memory as a local-address-space pointer, for the direct loads

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lq = lane >> 5;  // MFMA 32x32x16: operand row / column, k half

    // tile coordinates: consecutive workgroups share the weight tile (same n0), so it stays in L2
    // With splits > 1, `splits` consecutive workgroups share a tile and take consecutive ranges of
    // whole scale groups of K; the last of them to finish adds the partial sums (below).
    const int m_tiles = (M + BM - 1) / BM;
    const int tile = blockIdx.x / splits, split = blockIdx.x - tile * splits;
    const int n0 = (tile / m_tiles) * kBN;
    const int m0 = (tile % m_tiles) * BM + wave * kWM;
    const int words = K / 32, groups = K / 128;
    const int g_begin = (int)((long)groups * split / splits), g_end = (int)((long)groups * (split + 1) / splits);
    const int k_begin = g_begin * 128;
    const int last = (g_end - g_begin) * 128 / kBK - 1;  // index of this workgroup's last stage

    // activations: load t of a stage brings rows 8t .. 8t+7 of the wave's tile, 128 bytes each, straight
    // into LDS. The hardware puts lane p's 16 bytes at byte 16 p of the 1 KB block, so lane p asks for
    // the chunk that belongs there under the row swizzle: row p / 8, chunk (p % 8) ^ (p / 8).
    // Rows past M re-read row M-1; their results are not stored.
    typedef __attribute__((address_space(1))) const unsigned char GB;
    GB *a_src[kDma];
#pragma unroll
    for (int t = 0; t < kDma; t++) {
        const int gm = min(m0 + 8 * t + (lane >> 3), M - 1);
        a_src[t] = (GB *)A + ((size_t)gm * K + k_begin + 8 * ((lane & 7) ^ row_swizzle(8 * t + (lane >> 3)))) * 2;
    }
    // weights: row w_row, 32-column word w_word of the stage
    const int w_row = tid >> 1, w_word = tid & 1;
    const int gn = min(n0 + w_row, N - 1);
    GB *nz_src = (GB *)nzB + ((size_t)gn * words + k_begin / 32 + w_word) * 4;
    GB *sg_src = (GB *)sgB + ((size_t)gn * words + k_begin / 32 + w_word) * 4;
    // the scale of group g travels as the aligned dword that contains it; sc_half picks the half
    GB *sc_src = (GB *)scB + ((size_t)gn * groups + g_begin) * 2;
    const int w_off = chunk_off(w_row, w_word * 4);      // chunk c of the word: w_off ^ (c << 4)
    const int fr_off = chunk_off(li, lq);                // fragment i, step ks: (fr_off ^ (ks << 5)) + i * 32 rows

    struct Masks {
        uint32_t nz, sg, sc;
        bool hi;  // the scale is the high half of sc
    };
    // Mask words and scales also come through LDS: thread t asks for its own three dwords, which the
    // hardware puts at byte 4 t of each 1 KB plane, and reads them back itself (no barrier involved).
    auto dma_masks = [&](int buf, int stage) {
        const int k0 = min(stage, last) * kBK;
        LB *dst = lds_dma + kMaskBase + buf * kMaskBytes + wave * 256;
        __builtin_amdgcn_global_load_lds((__attribute__((address_space(1))) const void *)(nz_src + k0 / 8),
                                         (__attribute__((address_space(3))) void *)dst, 4, 0, 0);
        __builtin_amdgcn_global_load_lds((__attribute__((address_space(1))) const void *)(sg_src + k0 / 8),
                                         (__attribute__((address_space(3))) void *)(dst + 1024), 4, 0, 0);
        const uintptr_t sc_addr = reinterpret_cast<uintptr_t>(sc_src) + (k0 / 128) * 2;
        __builtin_amdgcn_global_load_lds((__attribute__((address_space(1))) const void *)(sc_addr & ~(uintptr_t)3),
                                         (__attribute__((address_space(3))) void *)(dst + 2048), 4, 0, 0);
    };
    auto read_masks = [&](Masks &w, int buf, int stage) {
        const unsigned char *src = lds + kMaskBase + buf * kMaskBytes + tid * 4;
        w.nz = *reinterpret_cast<const uint32_t *>(src);
        w.sg = *reinterpret_cast<const uint32_t *>(src + 1024);
        w.sc = *reinterpret_cast<const uint32_t *>(src + 2048);  // the dword that holds the scale
        const uintptr_t sc_addr = reinterpret_cast<uintptr_t>(sc_src) + (min(stage, last) * kBK / 128) * 2;
        w.hi = (sc_addr & 2) != 0;
    };
    auto scale_of = [](const Masks &w) -> uint32_t { return w.hi ? w.sc >> 16 : w.sc & 0xFFFFu; };
    auto dma_acts = [&](int buf, int stage, int t_begin, int t_end) {
        const int k0 = min(stage, last) * kBK;
#pragma unroll
        for (int t = t_begin; t < t_end; t++)
            __builtin_amdgcn_global_load_lds(
                (__attribute__((address_space(1))) const void *)(a_src[t] + k0 * 2),
                (__attribute__((address_space(3))) void *)(lds_dma + kActBase + buf * kActBytes + wave * kActWave + t * 1024),
                16, 0, 0);
    };
    auto read_w = [&](u4 (&af)[kNF], int buf, int ks) {
        const unsigned char *Ws = lds + buf * kWBytes + (fr_off ^ (ks << 5));
#pragma unroll
        for (int i = 0; i < kNF; i++) af[i] = *reinterpret_cast<const u4 *>(Ws + i * 32 * kRowBytes);
    };
    auto read_a = [&](u4 (&bf)[MF], int buf, int ks) {
        const unsigned char *As = lds + kActBase + buf * kActBytes + wave * kActWave + (fr_off ^ (ks << 5));
#pragma unroll
        for (int j = 0; j < MF; j++) bf[j] = *reinterpret_cast<const u4 *>(As + j * 32 * kRowBytes);
    };

    f16v acc[kNF][MF];
#pragma unroll
    for (int i = 0; i < kNF; i++)
#pragma unroll
        for (int j = 0; j < MF; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    auto mfma_row = [&](const u4 &a, const u4 (&bf)[MF], int i) {
#pragma unroll
        for (int j = 0; j < MF; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, bf[j]),
                                                               acc[i][j], 0, 0, 0);
    };
    auto decode_all = [&](const Masks &w, int buf) {
        Decoder d;
        d.begin(w.nz, w.sg, scale_of(w));
        unsigned char *Ws = lds + buf * kWBytes;
#pragma unroll
        for (int c = 0; c < 4; c++)
            *reinterpret_cast<u4 *>(Ws + (w_off ^ (c << 4))) =
                u4{d.dword(4 * c), d.dword(4 * c + 1), d.dword(4 * c + 2), d.dword(4 * c + 3)};
    };

    // Software pipeline, per stage s (buffer indices modulo 3). Everything that comes from global
    // memory is written into LDS by the load itself; such loads complete in order, so "at most n
    // still in flight" is the test for the older ones. A stage is four MFMA steps of 16 columns;
    // the fragments of a step are read from LDS during the step before, after its first MFMAs.
    //   top:    activations of stage s+2 are requested;
    //   step 0: the masks of stage s+2 (requested in stage s-3) are read from LDS;
    //   steps 1-3: between the MFMAs the masks are decoded into weight buffer s+2;
    //   step 3: fragments of step 0 of stage s+1 are read; at the end the masks of stage s+5 are
    //           requested into the mask buffer just read; barrier.
    // The barrier at the end of stage s publishes weight buffer s+2 before its first read (step 3 of
    // stage s+1); that buffer was last read in step 2 of stage s-1. Activation and mask buffers are
    // private to a wave, ordered by the wave's own waits.
    Masks w;
    u4 af0[kNF], af1[kNF], bf0[MF], bf1[MF];
    dma_acts(0, 0, 0, kDma);
    dma_acts(1, 1, 0, kDma);
#pragma unroll
    for (int u = 0; u < kBufs; u++) dma_masks(u, u);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    read_masks(w, 0, 0);
    decode_all(w, 0);
    read_masks(w, 1, 1);
    decode_all(w, 1);
    dma_masks(0, 3);
    dma_masks(1, 4);
    // everything requested so far has landed: the in-loop waits count only requests made in the loop
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    read_w(af0, 0, 0);
    read_a(bf0, 0, 0);
    for (int s0 = 0; s0 <= last; s0 += kBufs) {
#pragma unroll
        for (int u = 0; u < kBufs; u++) {
            const int s = s0 + u;
            if (s > last) break;
            // Every LDS read is issued right AFTER the first MFMAs of a step, one step before its
            // data is used: the wait in front of a step's first MFMA then finds nothing younger in
            // the LDS queue and costs nothing.
            Decoder d;
            unsigned char *Ws = lds + ((u + 2) % kBufs) * kWBytes;
            uint32_t o[16];
            // the activation requests of stage s+2 are spread over the four steps (a quarter each, behind
            // the step's first MFMAs): issued back to back they hold the wave up
            constexpr int kQ = kDma / 4;
            // ---- step 0 (af0/bf0)
            mfma_row(af0[0], bf0, 0);
            __builtin_amdgcn_sched_barrier(0);
            // masks of stage s+2: requested in stage s-3; newer requests: 2 stages of (kDma + 3)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kDma + 6) : "memory");
            read_masks(w, (u + 2) % kBufs, s + 2);
            read_w(af1, u, 1);
            __builtin_amdgcn_sched_barrier(0);
            mfma_row(af0[1], bf0, 1);
            __builtin_amdgcn_sched_barrier(0);
            read_a(bf1, u, 1);
            dma_acts((u + 2) % kBufs, s + 2, 0, kQ);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 2; i < kNF; i++) mfma_row(af0[i], bf0, i);
            __builtin_amdgcn_sched_barrier(0);
            // ---- step 1 (af1/bf1): decode starts
            mfma_row(af1[0], bf1, 0);
            __builtin_amdgcn_sched_barrier(0);
            read_w(af0, u, 2);
            read_a(bf0, u, 2);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 1; i < kNF; i++) {
                mfma_row(af1[i], bf1, i);
                if (i == 1) {
                    dma_acts((u + 2) % kBufs, s + 2, kQ, 2 * kQ);
                    d.begin(w.nz, w.sg, scale_of(w));
                }
#pragma unroll
                for (int dw = 2 * (i - 1); dw < 2 * i; dw++) o[dw] = d.dword(dw);
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- step 2 (af0/bf0)
            mfma_row(af0[0], bf0, 0);
            o[6] = d.dword(6);
            o[7] = d.dword(7);
            __builtin_amdgcn_sched_barrier(0);
            read_w(af1, u, 3);
            read_a(bf1, u, 3);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 1; i < kNF; i++) {
                mfma_row(af0[i], bf0, i);
                if (i == 1) {
                    dma_acts((u + 2) % kBufs, s + 2, 2 * kQ, 3 * kQ);
                    *reinterpret_cast<u4 *>(Ws + (w_off ^ (0 << 4))) = u4{o[0], o[1], o[2], o[3]};
                    *reinterpret_cast<u4 *>(Ws + (w_off ^ (1 << 4))) = u4{o[4], o[5], o[6], o[7]};
                }
#pragma unroll
                for (int dw = 6 + 2 * i; dw < 8 + 2 * i; dw++) o[dw] = d.dword(dw);
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- step 3 (af1/bf1): fragments of step 0 of the next stage
            mfma_row(af1[0], bf1, 0);
            o[14] = d.dword(14);
            o[15] = d.dword(15);
            __builtin_amdgcn_sched_barrier(0);
            *reinterpret_cast<u4 *>(Ws + (w_off ^ (2 << 4))) = u4{o[8], o[9], o[10], o[11]};
            *reinterpret_cast<u4 *>(Ws + (w_off ^ (3 << 4))) = u4{o[12], o[13], o[14], o[15]};
            read_w(af0, (u + 1) % kBufs, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_row(af1[1], bf1, 1);
            __builtin_amdgcn_sched_barrier(0);
            dma_acts((u + 2) % kBufs, s + 2, 3 * kQ, kDma);
            // the activations of stage s+1 were requested during stage s-1; newer requests: the masks
            // of that stage (3) and this stage's activations (kDma)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kDma + 3) : "memory");
            read_a(bf0, (u + 1) % kBufs, 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 2; i < kNF; i++) mfma_row(af1[i], bf1, i);
            __builtin_amdgcn_sched_barrier(0);
            dma_masks((u + 2) % kBufs, s + 5);
            // plain barrier: a fence here would also wait for the requests in flight
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        }
    }

    // ---- split K: every workgroup of a tile leaves its fp32 sums in its own slot; the one that
    // arrives last adds all slots in split order (its own from its registers, in its place of the
    // order: the result does not depend on who is last) and stores. The slots are written with stores that go through to memory
    // (sc1) and are acknowledged (s_waitcnt vmcnt(0)) before the workgroup counts as arrived; the
    // reader drops what its L2 may still hold of the slots (acquire fence = invalidate, cheap) and
    // then reads them with ordinary 16-byte loads. A release fence instead of the write-through
    // stores would write back the whole L2 of the XCD and cost more than the GEMM.
    if (splits > 1) {
        constexpr int kSlot = BM * kBN;  // floats; element (c, tid, e) of a slot at (c * kThreads + tid) * 4 + e
        float *mine = partial + ((size_t)tile * splits + split) * kSlot + tid * 4;
#pragma unroll
        for (int i = 0; i < kNF; i++)
#pragma unroll
            for (int j = 0; j < MF; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const f4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    float *dst = mine + (size_t)((i * MF + j) * 4 + g) * kThreads * 4;
                    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
                }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __shared__ unsigned last_arrival;
        __syncthreads();
        if (tid == 0) {
            const unsigned before = __hip_atomic_fetch_add(&arrivals[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_arrival = before == (unsigned)splits - 1;
            if (last_arrival) __hip_atomic_store(&arrivals[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
        }
        __syncthreads();
        if (!last_arrival) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const float *slots = partial + (size_t)tile * splits * kSlot + tid * 4;
        // the sums of this workgroup stay in registers: its own slot is not read back (same values)
        f16v own[kNF][MF];
#pragma unroll
        for (int i = 0; i < kNF; i++)
#pragma unroll
            for (int j = 0; j < MF; j++) {
                own[i][j] = acc[i][j];
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
            }
        for (int q = 0; q < splits; q++) {
            if (q == split) {
#pragma unroll
                for (int i = 0; i < kNF; i++)
#pragma unroll
                    for (int j = 0; j < MF; j++) acc[i][j] += own[i][j];
                continue;
            }
            const float *slot = slots + (size_t)q * kSlot;
#pragma unroll
            for (int i = 0; i < kNF; i++)
#pragma unroll
                for (int j = 0; j < MF; j++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const f4 v = *reinterpret_cast<const f4 *>(slot + (size_t)((i * MF + j) * 4 + g) * kThreads * 4);
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[i][j][4 * g + e] += v[e];
                    }
        }
    }

    // ---- store: lane (k half lq, column li) of fragment (i, j) holds, for activation row m, the weight
    // rows n0 + 32 i + 8 g + 4 lq + v in register 4 g + v (g, v = 0..3)
    uint16_t *Cg = C;
    const bool vec_store = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 7) == 0;
#pragma unroll
    for (int j = 0; j < MF; j++) {
        const int m = m0 + j * 32 + li;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < kNF; i++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int n = n0 + i * 32 + 8 * g + 4 * lq;
                uint16_t h[4];
#pragma unroll
                for (int v = 0; v < 4; v++) h[v] = f2h(acc[i][j][4 * g + v] * 0.5f);
                uint16_t *dst = Cg + (size_t)m * N + n;
                if (n + 3 < N && vec_store) {
                    *reinterpret_cast<uint2 *>(dst) = uint2{(uint32_t)h[0] | ((uint32_t)h[1] << 16),
                                                            (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
                } else {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (n + v < N) dst[v] = h[v];
                }
            }
        }
    }
}


// ------------------------------------------------------------------------------------------------
// Eight-wave instance: two waves per SIMD, so that the loads, the decode and the LDS stores of one
// wave run under the MFMAs of the other. Same workgroup tile (128 weight rows x 128*MF activation
// rows) and the same LDS image of a stage; wave (wm, nh) owns activation rows 32*MF*wm .. and the
// weight rows 64*nh .. 64*nh+63 (a 64 x 32*MF tile: 2 x MF accumulator fragments). The activation
// tile of a wm is shared by its two waves (each requests half of its rows), the mask words and
// scales are requested by one wave and decoded by another, so everything that lands in LDS is
// published by the one barrier per phase.
//
// Phases. All LDS reads of the data of stage s happen between barrier s and barrier s+1 ("phase
// s"): the fragments of step 0 right after barrier s (under the last MFMAs of stage s-1), those of
// steps 1..3 one step ahead of their MFMAs. With three buffers per operand a buffer is therefore
// free for two whole phases before it is read again:
//   phase s: requests the activations of stage s+2 and the masks of stage s+3 (both waited for at
//            the end of phase s+1: in-order completion, vmcnt = this phase's own requests),
//            decodes the masks of stage s+1 (published by barrier s) into weight buffer s+1.
constexpr int kThreads8 = 512;

template <int MF>
__global__ __launch_bounds__(kThreads8, 1) void gemm_mfma8_kernel(
    const uint16_t *__restrict__ A, const uint32_t *__restrict__ nzB, const uint32_t *__restrict__ sgB,
    const uint16_t *__restrict__ scB, uint16_t *__restrict__ C, int M, int N, int K, int splits,
    float *__restrict__ partial, unsigned *__restrict__ arrivals) {
    constexpr int kWM = MF * 32;               // activation rows per wave pair
    constexpr int BM = 4 * kWM;
    constexpr int kActWave = kWM * kRowBytes;  // bytes of one pair's activation tile per stage
    constexpr int kActBytes = 4 * kActWave;
    constexpr int kActBase = kBufs * kWBytes;
    constexpr int kMaskBase = kActBase + kBufs * kActBytes;
    constexpr int kMaskBytes = 4 * 1024;       // nz words 1 KB | sign words 1 KB | scale dwords 8 x 256 B
    constexpr int kDmaPair = kWM / 8;          // 1 KB activation loads per pair and stage
    constexpr int kDma = kDmaPair / 2;         // ... per wave
    constexpr int kReq = kDma + 2;             // requests a wave makes per phase
    constexpr int kNF8 = 2;                    // weight-row fragments per wave
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    typedef __attribute__((address_space(3))) unsigned char LB;
    LB *lds_dma = (LB *)lds;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 3, nh = wave >> 2;
    const int li = lane & 31, lq = lane >> 5;

    const int m_tiles = (M + BM - 1) / BM;
    const int tile = blockIdx.x / splits, split = blockIdx.x - tile * splits;
    const int n0 = (tile / m_tiles) * kBN;
    const int m0 = (tile % m_tiles) * BM + wm * kWM;
    const int words = K / 32, groups = K / 128;
    const int g_begin = (int)((long)groups * split / splits), g_end = (int)((long)groups * (split + 1) / splits);
    const int k_begin = g_begin * 128;
    const int last = (g_end - g_begin) * 128 / kBK - 1;

    typedef __attribute__((address_space(1))) const unsigned char GB;
    // activations: this wave requests loads nh*kDma .. of its pair's tile (rows 8t .. 8t+7 each)
    GB *a_src[kDma];
#pragma unroll
    for (int t = 0; t < kDma; t++) {
        const int gm = min(m0 + 8 * (nh * kDma + t) + (lane >> 3), M - 1);
        a_src[t] = (GB *)A + ((size_t)gm * K + k_begin + 8 * ((lane & 7) ^ row_swizzle(8 * (nh * kDma + t) + (lane >> 3)))) * 2;
    }
    // masks: waves 0-3 request the non-zero words, waves 4-7 the sign words; lane l of wave w asks for
    // word (64 (w & 3) + l) of the stage = word (idx & 1) of weight row idx >> 1
    const int midx = 64 * (wave & 3) + lane;
    const int mrow = min(n0 + (midx >> 1), N - 1);
    GB *m_src = (GB *)(nh ? sgB : nzB) + ((size_t)mrow * words + k_begin / 32 + (midx & 1)) * 4;
    // scales: lane l of wave w asks for the aligned dword that holds the scale of weight row 16 w + (l & 15)
    const int srow = min(n0 + 16 * wave + (lane & 15), N - 1);
    const uintptr_t s_src = reinterpret_cast<uintptr_t>(scB) + ((size_t)srow * groups + g_begin) * 2;
    // decode: thread t turns 16 weights of row t >> 2 (columns 16 (t & 3) .. of the stage) into two chunks
    const int w_row = tid >> 2, w_qk = tid & 3;
    const int w_gn = min(n0 + w_row, N - 1);
    const int w_par = (int)(((size_t)w_gn * groups + g_begin) & 1);  // scale is the high half of its dword when (w_par + group) is odd
    const uint32_t w_sel = (w_qk & 1) ? 0x07060302u : 0x05040100u;   // which 16 weights of the word
    const int w_off = chunk_off(w_row, 2 * w_qk);
    const int w_mask_off = (w_row * 2 + (w_qk >> 1)) * 4;
    const int w_scale_off = 2048 + (w_row >> 4) * 256 + (w_row & 15) * 4;
    const int fr_off = chunk_off(li, lq);

    auto dma_masks = [&](int buf, int stage) {
        const int k0 = min(stage, last) * kBK;
        LB *dst = lds_dma + kMaskBase + buf * kMaskBytes;
        __builtin_amdgcn_global_load_lds((__attribute__((address_space(1))) const void *)(m_src + k0 / 8),
                                         (__attribute__((address_space(3))) void *)(dst + nh * 1024 + (wave & 3) * 256), 4, 0, 0);
        const uintptr_t sc_addr = s_src + (k0 / 128) * 2;
        __builtin_amdgcn_global_load_lds((__attribute__((address_space(1))) const void *)(sc_addr & ~(uintptr_t)3),
                                         (__attribute__((address_space(3))) void *)(dst + 2048 + wave * 256), 4, 0, 0);
    };
    auto dma_acts = [&](int buf, int stage, int t_begin, int t_end) {
        const int k0 = min(stage, last) * kBK;
#pragma unroll
        for (int t = t_begin; t < t_end; t++)
            __builtin_amdgcn_global_load_lds(
                (__attribute__((address_space(1))) const void *)(a_src[t] + k0 * 2),
                (__attribute__((address_space(3))) void *)(lds_dma + kActBase + buf * kActBytes + wm * kActWave + (nh * kDma + t) * 1024),
                16, 0, 0);
    };
    // 16 weights -> 8 dwords (two chunks) of +-2*scale / 0, see Decoder above
    struct Decoder16 {
        uint32_t q;
        h2 sp;
        __device__ __forceinline__ void begin(uint32_t nz, uint32_t sg, uint32_t scale, uint32_t sel) {
            const uint32_t neg = nz & ~sg;
            const uint32_t t0 = __builtin_amdgcn_bitop3_b32(neg << 1, nz, 0xAAAAAAAAu, 0xE4);
            const uint32_t t1 = __builtin_amdgcn_bitop3_b32(neg, nz >> 1, 0xAAAAAAAAu, 0xE4);
            q = __builtin_amdgcn_perm(t1, t0, sel);
            sp = __builtin_bit_cast(h2, scale | (scale << 16));
        }
        __device__ __forceinline__ uint32_t dword(int d) const {
            us2 v = __builtin_bit_cast(us2, q);
            v = v << (uint16_t)(14 - 2 * d);
            const uint32_t top = __builtin_bit_cast(uint32_t, v) & 0xC000C000u;
            return __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, top) * sp);
        }
    };

    f16v acc[kNF8][MF];
#pragma unroll
    for (int i = 0; i < kNF8; i++)
#pragma unroll
        for (int j = 0; j < MF; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // ---- prologue: masks of stages 0..2, activations of stages 0 and 1; weights of stage 0 decoded
    Decoder16 d;
    // Three sets of fragment registers: the fragments of a step are requested two steps before its
    // MFMAs, also across the barrier (the MFMAs of steps 2 and 3 of a stage run after the barrier that
    // ends its phase, from registers).
    struct Frags {
        u4 a[kNF8], b[MF];
    };
    Frags R[3];
#pragma unroll
    for (int q = 0; q < 3; q++) {
#pragma unroll
        for (int i = 0; i < kNF8; i++) R[q].a[i] = u4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < MF; j++) R[q].b[j] = u4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < kBufs; u++) dma_masks(u, u);
    dma_acts(0, 0, 0, kDma);
    dma_acts(1, 1, 0, kDma);
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    {
        const unsigned char *src = lds + kMaskBase;
        const uint32_t nz = *reinterpret_cast<const uint32_t *>(src + w_mask_off);
        const uint32_t sg = *reinterpret_cast<const uint32_t *>(src + 1024 + w_mask_off);
        const uint32_t sd = *reinterpret_cast<const uint32_t *>(src + w_scale_off);
        d.begin(nz, sg, (w_par & 1) ? sd >> 16 : sd & 0xFFFFu, w_sel);
        *reinterpret_cast<u4 *>(lds + w_off) = u4{d.dword(0), d.dword(1), d.dword(2), d.dword(3)};
        *reinterpret_cast<u4 *>(lds + (w_off ^ 16)) = u4{d.dword(4), d.dword(5), d.dword(6), d.dword(7)};
    }

    // In the loop every LDS instruction is written out and every wait for one names how many younger
    // ones may still be in flight (they complete in order), so that a wait never includes requests made
    // just before it. (Left to itself the compiler waits for the whole queue, lgkmcnt(0), in front of
    // each consumer.) Fragment reads are issued one at a time between MFMAs: bursts of them from all
    // eight waves at once fill the LDS queue and hold the MFMAs behind them.
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds_dma;
    uint32_t fo[4];  // this lane's fragment offset in steps 0..3
#pragma unroll
    for (int ks = 0; ks < 4; ks++) fo[ks] = lds0 + (uint32_t)(fr_off ^ (ks << 5));
    const uint32_t w_rd = (uint32_t)(nh * 64 * kRowBytes);                // + buf * kWBytes
    const uint32_t a_rd = (uint32_t)(kActBase + wm * kActWave);          // + buf * kActBytes
    const uint32_t m_rd = lds0 + (uint32_t)(kMaskBase + w_mask_off);     // imm: buf * kMaskBytes (+ 1024)
    const uint32_t s_rd = lds0 + (uint32_t)(kMaskBase + w_scale_off);
    const uint32_t w_wr0 = lds0 + (uint32_t)w_off, w_wr1 = lds0 + (uint32_t)(w_off ^ 16);  // imm: buf * kWBytes
#define TLLM_LDS_READ128(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))
#define TLLM_LDS_READ32(dst, addr, off) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))
#define TLLM_LDS_WRITE128(addr, val, off) asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(val), "i"(off) : "memory")
#define TLLM_LGKM(n) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(n) : "memory")
#define TLLM_FENCE() __builtin_amdgcn_sched_barrier(0)
    constexpr int kFr = kNF8 + MF;  // LDS reads of one step
    // read number r (0 .. kFr-1) of the fragments of step ks: weight rows first, then activation rows
    auto frag_read = [&](Frags &f, int buf, int ks, int r) {
        const uint32_t aw = fo[ks] + (w_rd + (uint32_t)(buf * kWBytes));
        const uint32_t aa = fo[ks] + (a_rd + (uint32_t)(buf * kActBytes));
        if (r == 0) TLLM_LDS_READ128(f.a[0], aw, 0);
        if (r == 1) TLLM_LDS_READ128(f.a[1], aw, 32 * kRowBytes);
        if (r == 2) TLLM_LDS_READ128(f.b[0], aa, 0);
        if constexpr (MF == 2)
            if (r == 3) TLLM_LDS_READ128(f.b[1], aa, 32 * kRowBytes);
    };
    // MFMA number m (0 .. 2 MF - 1) of a step
    auto mfma_one = [&](const Frags &f, int m) {
        const int i = m / MF, j = m % MF;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, f.a[i]), __builtin_bit_cast(h8, f.b[j]),
                                                           acc[i][j], 0, 0, 0);
    };
    constexpr int kMf = kNF8 * MF;  // MFMAs of one step
    // a slot: the MFMAs of one step (from set `use`) with the fragment reads of the step two ahead
    // (into set `get`) between them, one read behind each of the first MFMAs
    auto slot_spread = [&](const Frags &use, Frags &get, int buf, int ks) {
#pragma unroll
        for (int m = 0; m < (kMf > kFr ? kMf : kFr); m++) {
            if (m < kMf) mfma_one(use, m);
            TLLM_FENCE();
            if (m < kFr) frag_read(get, buf, ks, m);
            TLLM_FENCE();
        }
    };

    // one phase; the buffer index u = s % kBufs is a compile-time constant (it sits in instruction offsets)
    auto phase = [&](auto U, const int s) {
        constexpr int u = decltype(U)::value;
        constexpr int kH = kDma / 2 > 0 ? kDma / 2 : 1;
        constexpr int kNext = (u + 1) % kBufs;
        // slot j of this phase reads into set (4 u + j) % 3 and multiplies from set (4 u + j + 1) % 3
        constexpr int g0 = (4 * u + 0) % 3, g1 = (4 * u + 1) % 3, g2 = (4 * u + 2) % 3, g3 = (4 * u + 3) % 3;
        uint32_t o[8];
        uint32_t m_nz, m_sg, m_sc;
        // barrier s: publishes the weights decoded and the loads waited for in the phase before
        TLLM_LGKM(0);
        asm volatile("s_barrier" ::: "memory");
        TLLM_FENCE();
        // ---- slot 0: step 2 of the stage before (zero operands in the first phase); fragments of step 0
        slot_spread(R[g1], R[g0], u, 0);
        TLLM_LDS_READ32(m_nz, m_rd, kNext * kMaskBytes);
        TLLM_LDS_READ32(m_sg, m_rd, kNext * kMaskBytes + 1024);
        TLLM_LDS_READ32(m_sc, s_rd, kNext * kMaskBytes);
        dma_acts((u + 2) % kBufs, s + 2, 0, kH);
        TLLM_FENCE();
        // ---- slot 1: step 3 of the stage before; fragments of step 1
        slot_spread(R[g2], R[g1], u, 1);
        if (kDma > 1) dma_acts((u + 2) % kBufs, s + 2, kH, kDma);
        TLLM_FENCE();
        // ---- slot 2: step 0; fragments of step 2. In flight behind what it needs: the reads of slot 1.
        TLLM_LGKM(kFr);
        TLLM_FENCE();
        {
            const int odd = (w_par + min(s + 1, last) * kBK / 128) & 1;
            d.begin(m_nz, m_sg, odd ? m_sc >> 16 : m_sc & 0xFFFFu, w_sel);
        }
#pragma unroll
        for (int m = 0; m < (kMf > kFr ? kMf : kFr); m++) {
            if (m < kMf) mfma_one(R[g0], m);
            TLLM_FENCE();
            if (m < kFr) frag_read(R[g2], u, 2, m);
            if (m < 4) o[m] = d.dword(m);
            TLLM_FENCE();
        }
#pragma unroll
        for (int m = (kMf > kFr ? kMf : kFr); m < 4; m++) o[m] = d.dword(m);
        // ---- slot 3: step 1; fragments of step 3, requested early in the slot so that the wait in
        // front of the barrier finds them done. In flight behind what it needs: the reads of slot 2.
        TLLM_LGKM(kFr);
        TLLM_FENCE();
#pragma unroll
        for (int r = 0; r < kFr; r++) frag_read(R[g3], u, 3, r);
        TLLM_FENCE();
        mfma_one(R[g1], 0);
        TLLM_FENCE();
        o[4] = d.dword(4);
        o[5] = d.dword(5);
        {
            const u4 v = {o[0], o[1], o[2], o[3]};
            TLLM_LDS_WRITE128(w_wr0, v, kNext * kWBytes);
        }
        TLLM_FENCE();
        mfma_one(R[g1], 1);
        TLLM_FENCE();
        o[6] = d.dword(6);
        o[7] = d.dword(7);
        dma_masks(u, s + 3);
        {
            const u4 v = {o[4], o[5], o[6], o[7]};
            TLLM_LDS_WRITE128(w_wr1, v, kNext * kWBytes);
        }
        TLLM_FENCE();
#pragma unroll
        for (int m = 2; m < kMf; m++) mfma_one(R[g1], m);
        TLLM_FENCE();
        // everything requested before this phase has landed
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kReq) : "memory");
        if (s == last) {  // steps 2 and 3 of the last stage
            TLLM_LGKM(0);
            TLLM_FENCE();
#pragma unroll
            for (int m = 0; m < kMf; m++) mfma_one(R[g2], m);
#pragma unroll
            for (int m = 0; m < kMf; m++) mfma_one(R[g3], m);
        }
    };
    for (int s0 = 0; s0 <= last; s0 += kBufs) {
        phase(std::integral_constant<int, 0>{}, s0);
        if (s0 + 1 > last) break;
        phase(std::integral_constant<int, 1>{}, s0 + 1);
        if (s0 + 2 > last) break;
        phase(std::integral_constant<int, 2>{}, s0 + 2);
    }
#undef TLLM_LDS_READ128
#undef TLLM_LDS_READ32
#undef TLLM_LDS_WRITE128
#undef TLLM_LGKM
#undef TLLM_FENCE
    // requests past the last stage are still in flight into LDS: let them land before the workgroup ends
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if (splits > 1) {
        constexpr int kSlot = BM * kBN;  // floats; element (c, tid, e) of a slot at (c * kThreads8 + tid) * 4 + e
        float *mine = partial + ((size_t)tile * splits + split) * kSlot + tid * 4;
#pragma unroll
        for (int i = 0; i < kNF8; i++)
#pragma unroll
            for (int j = 0; j < MF; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const f4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    float *dst = mine + (size_t)((i * MF + j) * 4 + g) * kThreads8 * 4;
                    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
                }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __shared__ unsigned last_arrival8;
        __syncthreads();
        if (tid == 0) {
            const unsigned before = __hip_atomic_fetch_add(&arrivals[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_arrival8 = before == (unsigned)splits - 1;
            if (last_arrival8) __hip_atomic_store(&arrivals[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!last_arrival8) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const float *slots = partial + (size_t)tile * splits * kSlot + tid * 4;
        // The slots are added in split order whoever arrives last; this workgroup's own sums take
        // their place in that order from registers. All loads of a slot are in flight together.
        f16v own[kNF8][MF];
#pragma unroll
        for (int i = 0; i < kNF8; i++)
#pragma unroll
            for (int j = 0; j < MF; j++) {
                own[i][j] = acc[i][j];
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
            }
        for (int q = 0; q < splits; q++) {
            if (q == split) {
#pragma unroll
                for (int i = 0; i < kNF8; i++)
#pragma unroll
                    for (int j = 0; j < MF; j++) acc[i][j] += own[i][j];
                continue;
            }
            const float *slot = slots + (size_t)q * kSlot;
            f4 v[kNF8 * MF * 4];
#pragma unroll
            for (int c = 0; c < kNF8 * MF * 4; c++) v[c] = *reinterpret_cast<const f4 *>(slot + (size_t)c * kThreads8 * 4);
#pragma unroll
            for (int i = 0; i < kNF8; i++)
#pragma unroll
                for (int j = 0; j < MF; j++)
#pragma unroll
                    for (int g = 0; g < 4; g++)
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[i][j][4 * g + e] += v[(i * MF + j) * 4 + g][e];
        }
    }

    // ---- store: lane (k half lq, column li) of fragment (i, j) holds, for activation row m, the weight
    // rows n0 + 64 nh + 32 i + 8 g + 4 lq + v in register 4 g + v
    const bool vec_store = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 7) == 0;
#pragma unroll
    for (int j = 0; j < MF; j++) {
        const int m = m0 + j * 32 + li;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < kNF8; i++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int n = n0 + nh * 64 + i * 32 + 8 * g + 4 * lq;
                uint16_t h[4];
#pragma unroll
                for (int v = 0; v < 4; v++) h[v] = f2h(acc[i][j][4 * g + v] * 0.5f);
                uint16_t *dst = C + (size_t)m * N + n;
                if (n + 3 < N && vec_store) {
                    *reinterpret_cast<uint2 *>(dst) = uint2{(uint32_t)h[0] | ((uint32_t)h[1] << 16),
                                                            (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
                } else {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (n + v < N) dst[v] = h[v];
                }
            }
        }
    }
}


// ------------------------------------------------------------------------------------------------
// Four-wave instance with hand-placed instructions: one wave per SIMD, wave tile 128 weight rows x
// 32*MF activation rows (4 x MF accumulator fragments), the same LDS image of a stage as above.
// What a wave issues besides its MFMAs (fragment reads, the decode, direct-to-LDS loads) is dealt out
// one or two instructions at a time into the gaps between the MFMAs, every LDS instruction is written
// out, and every wait names how many younger requests may stay in flight. Activation tiles and mask
// words are private to a wave / thread (requested and read by the same one); only the decoded
// weights are shared, published by the one barrier per phase.
//   phase s: fragment reads of stage s (two steps ahead of their MFMAs, also across the barrier);
//            requests the activations of stage s+2 and the masks of stage s+3 (waited for at the end
//            of phase s+1: in-order completion, vmcnt = this phase's own requests);
//            decodes the masks of stage s+1 into weight buffer s+1.
template <int MF>
__global__ __launch_bounds__(kThreads, 1) void gemm_mfma4_kernel(
    const uint16_t *__restrict__ A, const uint32_t *__restrict__ nzB, const uint32_t *__restrict__ sgB,
    const uint16_t *__restrict__ scB, uint16_t *__restrict__ C, int M, int N, int K, int splits,
    float *__restrict__ partial, unsigned *__restrict__ arrivals) {
    constexpr int kWM = MF * 32;
    constexpr int BM = 4 * kWM;
    constexpr int kActWave = kWM * kRowBytes;
    constexpr int kActBytes = 4 * kActWave;
    constexpr int kActBase = kBufs * kWBytes;
    constexpr int kMaskBase = kActBase + kBufs * kActBytes;
    constexpr int kMaskBytes = 3 * 1024;  // per wave 768 bytes: nz words | sign words | scale dwords, 256 bytes each
    constexpr int kDma = kWM / 8;         // 1 KB activation loads per wave and stage
    constexpr int kReq = kDma + 3;        // requests a wave makes per phase
    constexpr int kFr = kNF + MF;         // LDS reads of one step
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    typedef __attribute__((address_space(3))) unsigned char LB;
    LB *lds_dma = (LB *)lds;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lq = lane >> 5;

    const int m_tiles = (M + BM - 1) / BM;
    const int tile = blockIdx.x / splits, split = blockIdx.x - tile * splits;
    const int n0 = (tile / m_tiles) * kBN;
    const int m0 = (tile % m_tiles) * BM + wave * kWM;
    const int words = K / 32, groups = K / 128;
    const int g_begin = (int)((long)groups * split / splits), g_end = (int)((long)groups * (split + 1) / splits);
    const int k_begin = g_begin * 128;
    const int last = (g_end - g_begin) * 128 / kBK - 1;

    typedef __attribute__((address_space(1))) const unsigned char GB;
    // Global addresses: a uniform base (which moves with the stage) plus a 32-bit lane offset that never changes.
    GB *a_base = (GB *)A + (size_t)k_begin * 2;
    uint32_t a_off[kDma];  // load t: rows 8t .. 8t+7 of the wave's tile, 128 bytes each, chunk order = LDS order
#pragma unroll
    for (int t = 0; t < kDma; t++) {
        const int gm = min(m0 + 8 * t + (lane >> 3), M - 1);
        a_off[t] = (uint32_t)(((size_t)gm * K + 8 * ((lane & 7) ^ row_swizzle(8 * t + (lane >> 3)))) * 2);
    }
    const int w_row = tid >> 1, w_word = tid & 1;  // this thread decodes 32 weights: one mask word pair per stage
    const int gn = min(n0 + w_row, N - 1);
    GB *nz_base = (GB *)nzB + (size_t)(k_begin / 32) * 4;
    GB *sg_base = (GB *)sgB + (size_t)(k_begin / 32) * 4;
    const uint32_t m_off = (uint32_t)(((size_t)gn * words + w_word) * 4);
    // the scale of a group travels as the aligned dword that holds it
    const size_t sc_elem = (size_t)gn * groups + g_begin;
    GB *sc_base = (GB *)scB;
    const uint32_t sc_off = (uint32_t)((sc_elem * 2) & ~(size_t)3);   // + 4 * ((sc_elem & 1) + group) / 2 ...
    const int w_par = (int)(sc_elem & 1);

    f16v acc[kNF][MF];
#pragma unroll
    for (int i = 0; i < kNF; i++)
#pragma unroll
        for (int j = 0; j < MF; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    struct Frags {
        u4 a[kNF], b[MF];
    };
    Frags R[3];
#pragma unroll
    for (int q = 0; q < 3; q++) {
#pragma unroll
        for (int i = 0; i < kNF; i++) R[q].a[i] = u4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < MF; j++) R[q].b[j] = u4{0u, 0u, 0u, 0u};
    }

    // LDS addresses (bytes from the start of LDS); buffer and fragment offsets sit in the instructions
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds_dma;
    const int fr_off = chunk_off(li, lq);
    uint32_t fw[4], fa[4];  // fragment reads of steps 0..3: weights, activations (buffers 0 and 1)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        fw[ks] = lds0 + (uint32_t)(fr_off ^ (ks << 5));
        fa[ks] = fw[ks] + (uint32_t)(kActBase + wave * kActWave);
    }
    const int w_off = chunk_off(w_row, w_word * 4);
    uint32_t w_wr[4];
#pragma unroll
    for (int c = 0; c < 4; c++) w_wr[c] = lds0 + (uint32_t)(w_off ^ (c << 4));
    const uint32_t m_rd = lds0 + (uint32_t)(kMaskBase + wave * 768 + lane * 4);
    const uint32_t m_rdb[3] = {m_rd, m_rd + (uint32_t)kMaskBytes, m_rd + 2u * (uint32_t)kMaskBytes};  // ds_read2 offsets are 8 bits
    // the scale is the low or the high half of its dword: the half flips from group to group
    const uint32_t s_rd_a = m_rd + 512u + 2u * (uint32_t)w_par, s_rd_b = m_rd + 512u + 2u * (uint32_t)(w_par ^ 1);

#define TLLM_GPTR(p) ((__attribute__((address_space(1))) const void *)(p))
#define TLLM_LPTR(p) ((__attribute__((address_space(3))) void *)(p))
    // stage index -> first column of the stage relative to k_begin (requests past the end repeat the last stage)
    auto stage_k0 = [&](int stage) -> int { return min(stage, last) * kBK; };
    auto dma_masks = [&](int buf, int stage) {
        const int k0 = stage_k0(stage);
        LB *dst = lds_dma + kMaskBase + buf * kMaskBytes + wave * 768;
        __builtin_amdgcn_global_load_lds(TLLM_GPTR(nz_base + (k0 / 8) + m_off), TLLM_LPTR(dst), 4, 0, 0);
        __builtin_amdgcn_global_load_lds(TLLM_GPTR(sg_base + (k0 / 8) + m_off), TLLM_LPTR(dst + 256), 4, 0, 0);
        // group k0 / 128 of this row: element sc_elem + k0 / 128, in dword (sc_elem + k0 / 128) / 2
        const uint32_t g2 = (uint32_t)(((w_par + k0 / 128) >> 1) * 4);
        __builtin_amdgcn_global_load_lds(TLLM_GPTR(sc_base + (sc_off + g2)), TLLM_LPTR(dst + 512), 4, 0, 0);
    };
    auto dma_act = [&](int buf, int stage, int t) {
        const int k0 = stage_k0(stage);
        __builtin_amdgcn_global_load_lds(TLLM_GPTR(a_base + (size_t)(k0 * 2) + a_off[t]),
                                         TLLM_LPTR(lds_dma + kActBase + buf * kActBytes + wave * kActWave + t * 1024), 16, 0, 0);
    };

    // ---- prologue: masks of stages 0..2, activations of stages 0 and 1; weights of stage 0 decoded
#pragma unroll
    for (int u = 0; u < kBufs; u++) dma_masks(u, u);
#pragma unroll
    for (int t = 0; t < kDma; t++) dma_act(0, 0, t);
#pragma unroll
    for (int t = 0; t < kDma; t++) dma_act(1, 1, t);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    Decoder d;
    {
        const unsigned char *src = lds + kMaskBase + wave * 768 + lane * 4;
        const uint32_t nz = *reinterpret_cast<const uint32_t *>(src);
        const uint32_t sg = *reinterpret_cast<const uint32_t *>(src + 256);
        const uint32_t sd = *reinterpret_cast<const uint32_t *>(src + 512);
        d.begin(nz, sg, (w_par & 1) ? sd >> 16 : sd & 0xFFFFu);
#pragma unroll
        for (int c = 0; c < 4; c++)
            *reinterpret_cast<u4 *>(lds + (w_off ^ (c << 4))) = u4{d.dword(4 * c), d.dword(4 * c + 1), d.dword(4 * c + 2), d.dword(4 * c + 3)};
    }

#define TLLM_LDS_READ128(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))
#define TLLM_LDS_READ2(dst, addr, o0, o1) asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(dst) : "v"(addr), "i"(o0), "i"(o1))
#define TLLM_LDS_READ16(dst, addr, off) asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "i"(off))
#define TLLM_LDS_WRITE128(addr, val, off) asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(val), "i"(off) : "memory")
#define TLLM_LGKM(n) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(n) : "memory")
#define TLLM_FENCE() __builtin_amdgcn_sched_barrier(0)
    // fragment reads of step ks of the stage in buffer u into set g
#define TLLM_RW(g, i, ks) TLLM_LDS_READ128(R[g].a[i], fw[ks], u * kWBytes + (i) * 32 * kRowBytes)
#define TLLM_RA(g, j, ks)                                                                              \
    do {                                                                                               \
        if constexpr ((j) < MF) {                                                                      \
            if constexpr (u * kActBytes + (j) * 32 * kRowBytes < 65536)                                \
                TLLM_LDS_READ128(R[g].b[(j) < MF ? (j) : 0], fa[ks], u * kActBytes + (j) * 32 * kRowBytes);            \
            else                                                                                       \
                TLLM_LDS_READ128(R[g].b[(j) < MF ? (j) : 0], fa_hi, u * kActBytes + (j) * 32 * kRowBytes - 65536);     \
        }                                                                                              \
    } while (0)
    // MFMA (i, j) of a step from set g
#define TLLM_MM(g, i, j)                                                                               \
    do {                                                                                               \
        if constexpr ((j) < MF)                                                                        \
            acc[i][(j) < MF ? (j) : 0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(                       \
                __builtin_bit_cast(h8, R[g].a[i]), __builtin_bit_cast(h8, R[g].b[(j) < MF ? (j) : 0]), \
                acc[i][(j) < MF ? (j) : 0], 0, 0, 0);                                                  \
        TLLM_FENCE();                                                                                  \
    } while (0)
#define TLLM_DMA(t)                                                    \
    do {                                                               \
        if constexpr ((t) < kDma) dma_act((u + 2) % kBufs, s + 2, (t) < kDma ? (t) : 0); \
        TLLM_FENCE();                                                  \
    } while (0)

    auto phase = [&](auto U, const int s) {
        constexpr int u = decltype(U)::value;
        constexpr int kNext = (u + 1) % kBufs;
        // slot j of this phase reads into set (4 u + j) % 3 and multiplies from set (4 u + j + 1) % 3
        constexpr int g0 = (4 * u + 0) % 3, g1 = (4 * u + 1) % 3, g2 = (4 * u + 2) % 3, g3 = (4 * u + 3) % 3;
        uint32_t o[16];
        uint32_t m_w[2], m_sc;
        const uint32_t fa_hi_base = 65536u;
        // barrier s: publishes the weights decoded in the phase before
        TLLM_LGKM(0);
        asm volatile("s_barrier" ::: "memory");
        TLLM_FENCE();
        // address of the scale half for stage s + 1 (group (s + 1) / 2 of this split)
        const uint32_t s_rd = ((stage_k0(s + 1) / 128) & 1) ? s_rd_b : s_rd_a;
        uint32_t fa_hi[4];  // only formed where a buffer offset does not fit the instruction (third buffer at MF = 2)
#pragma unroll
        for (int ks = 0; ks < 4; ks++) fa_hi[ks] = fa[ks] + fa_hi_base;
#define fa_hi fa_hi[ks_]
        // ---- slot 0: MFMAs of step 2 of the stage before (zero operands in the first phase); fragments of step 0
        {
            constexpr int ks_ = 0;
            TLLM_MM(g1, 0, 0); TLLM_RW(g0, 0, 0); TLLM_FENCE();
            TLLM_MM(g1, 0, 1); TLLM_RW(g0, 1, 0); TLLM_FENCE();
            TLLM_MM(g1, 1, 0); TLLM_RW(g0, 2, 0); TLLM_FENCE();
            TLLM_MM(g1, 1, 1); TLLM_RW(g0, 3, 0); TLLM_FENCE();
            TLLM_MM(g1, 2, 0); TLLM_RA(g0, 0, 0); TLLM_FENCE();
            TLLM_MM(g1, 2, 1); TLLM_RA(g0, 1, 0); TLLM_FENCE();
            TLLM_MM(g1, 3, 0);
            TLLM_LDS_READ2(m_w, m_rdb[kNext], 0, 64);
            TLLM_LDS_READ16(m_sc, s_rd, kNext * kMaskBytes);
            TLLM_FENCE();
            TLLM_MM(g1, 3, 1); TLLM_DMA(0); TLLM_DMA(1);
        }
        // ---- slot 1: MFMAs of step 3 of the stage before; fragments of step 1
        {
            constexpr int ks_ = 1;
            TLLM_MM(g2, 0, 0); TLLM_RW(g1, 0, 1); TLLM_FENCE();
            TLLM_MM(g2, 0, 1); TLLM_RW(g1, 1, 1); TLLM_FENCE();
            TLLM_MM(g2, 1, 0); TLLM_RW(g1, 2, 1); TLLM_FENCE();
            TLLM_MM(g2, 1, 1); TLLM_RW(g1, 3, 1); TLLM_FENCE();
            TLLM_MM(g2, 2, 0); TLLM_RA(g1, 0, 1); TLLM_FENCE();
            TLLM_MM(g2, 2, 1); TLLM_RA(g1, 1, 1); TLLM_FENCE();
            TLLM_MM(g2, 3, 0); TLLM_DMA(2); TLLM_DMA(3);
            TLLM_MM(g2, 3, 1); TLLM_DMA(4); TLLM_DMA(5);
        }
        // ---- slot 2: MFMAs of step 0; fragments of step 2; first half of the decode.
        // In flight behind what is needed (fragments of step 0, mask words, scale): the reads of slot 1.
        TLLM_LGKM(kFr);
        TLLM_FENCE();
        {
            constexpr int ks_ = 2;
            d.begin(m_w[0], m_w[1], m_sc);
            TLLM_FENCE();
            TLLM_MM(g0, 0, 0); TLLM_RW(g2, 0, 2); o[0] = d.dword(0); o[1] = d.dword(1); TLLM_FENCE();
            TLLM_MM(g0, 0, 1); TLLM_RW(g2, 1, 2); o[2] = d.dword(2); o[3] = d.dword(3); TLLM_FENCE();
            TLLM_MM(g0, 1, 0); TLLM_RW(g2, 2, 2); o[4] = d.dword(4); o[5] = d.dword(5); TLLM_FENCE();
            TLLM_MM(g0, 1, 1); TLLM_RW(g2, 3, 2); o[6] = d.dword(6); o[7] = d.dword(7); TLLM_FENCE();
            TLLM_MM(g0, 2, 0); TLLM_RA(g2, 0, 2); o[8] = d.dword(8); o[9] = d.dword(9); TLLM_FENCE();
            TLLM_MM(g0, 2, 1); TLLM_RA(g2, 1, 2); o[10] = d.dword(10); TLLM_FENCE();
            TLLM_MM(g0, 3, 0); TLLM_DMA(6); TLLM_DMA(7);
            o[11] = d.dword(11);
            TLLM_FENCE();
            TLLM_MM(g0, 3, 1);
            {
                const u4 v0 = {o[0], o[1], o[2], o[3]}, v1 = {o[4], o[5], o[6], o[7]};
                TLLM_LDS_WRITE128(w_wr[0], v0, kNext * kWBytes);
                TLLM_LDS_WRITE128(w_wr[1], v1, kNext * kWBytes);
            }
            TLLM_FENCE();
        }
        // ---- slot 3: MFMAs of step 1; fragments of step 3, requested early in the slot so that the wait
        // in front of the barrier finds them done. In flight behind what is needed: the reads and the two
        // stores of slot 2.
        TLLM_LGKM(kFr + 2);
        TLLM_FENCE();
        {
            constexpr int ks_ = 3;
            TLLM_MM(g1, 0, 0); TLLM_RW(g3, 0, 3); TLLM_RW(g3, 1, 3); TLLM_FENCE();
            TLLM_MM(g1, 0, 1); TLLM_RW(g3, 2, 3); TLLM_RW(g3, 3, 3); TLLM_FENCE();
            TLLM_MM(g1, 1, 0); TLLM_RA(g3, 0, 3); TLLM_RA(g3, 1, 3); TLLM_FENCE();
            TLLM_MM(g1, 1, 1); o[12] = d.dword(12); o[13] = d.dword(13); TLLM_FENCE();
            TLLM_MM(g1, 2, 0); o[14] = d.dword(14); o[15] = d.dword(15); TLLM_FENCE();
            TLLM_MM(g1, 2, 1);
            {
                const u4 v2 = {o[8], o[9], o[10], o[11]};
                TLLM_LDS_WRITE128(w_wr[2], v2, kNext * kWBytes);
            }
            TLLM_FENCE();
            TLLM_MM(g1, 3, 0);
            {
                const u4 v3 = {o[12], o[13], o[14], o[15]};
                TLLM_LDS_WRITE128(w_wr[3], v3, kNext * kWBytes);
            }
            TLLM_FENCE();
            TLLM_MM(g1, 3, 1);
            dma_masks(u, s + 3);
            TLLM_FENCE();
        }
#undef fa_hi
        // everything requested before this phase has landed
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kReq) : "memory");
        if (s == last) {  // steps 2 and 3 of the last stage
            TLLM_LGKM(0);
            TLLM_FENCE();
            TLLM_MM(g2, 0, 0); TLLM_MM(g2, 0, 1); TLLM_MM(g2, 1, 0); TLLM_MM(g2, 1, 1);
            TLLM_MM(g2, 2, 0); TLLM_MM(g2, 2, 1); TLLM_MM(g2, 3, 0); TLLM_MM(g2, 3, 1);
            TLLM_MM(g3, 0, 0); TLLM_MM(g3, 0, 1); TLLM_MM(g3, 1, 0); TLLM_MM(g3, 1, 1);
            TLLM_MM(g3, 2, 0); TLLM_MM(g3, 2, 1); TLLM_MM(g3, 3, 0); TLLM_MM(g3, 3, 1);
        }
    };
    for (int s0 = 0; s0 <= last; s0 += kBufs) {
        phase(std::integral_constant<int, 0>{}, s0);
        if (s0 + 1 > last) break;
        phase(std::integral_constant<int, 1>{}, s0 + 1);
        if (s0 + 2 > last) break;
        phase(std::integral_constant<int, 2>{}, s0 + 2);
    }
#undef TLLM_LDS_READ128
#undef TLLM_LDS_READ2
#undef TLLM_LDS_READ16
#undef TLLM_LDS_WRITE128
#undef TLLM_LGKM
#undef TLLM_FENCE
#undef TLLM_RW
#undef TLLM_RA
#undef TLLM_MM
#undef TLLM_DMA
#undef TLLM_GPTR
#undef TLLM_LPTR
    // requests past the last stage are still in flight into LDS: let them land before the workgroup ends
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if (splits > 1) {
        constexpr int kSlot = BM * kBN;  // floats; element (c, tid, e) of a slot at (c * kThreads + tid) * 4 + e
        float *mine = partial + ((size_t)tile * splits + split) * kSlot + tid * 4;
#pragma unroll
        for (int i = 0; i < kNF; i++)
#pragma unroll
            for (int j = 0; j < MF; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const f4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    float *dst = mine + (size_t)((i * MF + j) * 4 + g) * kThreads * 4;
                    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
                }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __shared__ unsigned last_arrival4;
        __syncthreads();
        if (tid == 0) {
            const unsigned before = __hip_atomic_fetch_add(&arrivals[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_arrival4 = before == (unsigned)splits - 1;
            if (last_arrival4) __hip_atomic_store(&arrivals[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!last_arrival4) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const float *slots = partial + (size_t)tile * splits * kSlot + tid * 4;
        // The slots are added in split order whoever arrives last; this workgroup's own sums take their
        // place in that order from registers. The loads of one fragment row are in flight together.
        f16v own[kNF][MF];
#pragma unroll
        for (int i = 0; i < kNF; i++)
#pragma unroll
            for (int j = 0; j < MF; j++) {
                own[i][j] = acc[i][j];
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
            }
        for (int q = 0; q < splits; q++) {
            if (q == split) {
#pragma unroll
                for (int i = 0; i < kNF; i++)
#pragma unroll
                    for (int j = 0; j < MF; j++) acc[i][j] += own[i][j];
                continue;
            }
            const float *slot = slots + (size_t)q * kSlot;
#pragma unroll
            for (int i = 0; i < kNF; i++) {
                f4 v[MF * 4];
#pragma unroll
                for (int c = 0; c < MF * 4; c++) v[c] = *reinterpret_cast<const f4 *>(slot + (size_t)(i * MF * 4 + c) * kThreads * 4);
#pragma unroll
                for (int j = 0; j < MF; j++)
#pragma unroll
                    for (int g = 0; g < 4; g++)
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[i][j][4 * g + e] += v[j * 4 + g][e];
            }
        }
    }

    // ---- store: lane (k half lq, column li) of fragment (i, j) holds, for activation row m, the weight
    // rows n0 + 32 i + 8 g + 4 lq + v in register 4 g + v
    const bool vec_store = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 7) == 0;
#pragma unroll
    for (int j = 0; j < MF; j++) {
        const int m = m0 + j * 32 + li;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < kNF; i++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int n = n0 + i * 32 + 8 * g + 4 * lq;
                uint16_t h[4];
#pragma unroll
                for (int v = 0; v < 4; v++) h[v] = f2h(acc[i][j][4 * g + v] * 0.5f);
                uint16_t *dst = C + (size_t)m * N + n;
                if (n + 3 < N && vec_store) {
                    *reinterpret_cast<uint2 *>(dst) = uint2{(uint32_t)h[0] | ((uint32_t)h[1] << 16),
                                                            (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
                } else {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (n + v < N) dst[v] = h[v];
                }
            }
        }
    }
}

// Split-K workspace: fp32 slots and arrival counters, one set per (device, stream), created on the
// first call that needs it and grown on demand (the only allocation this file makes; never during
// a call that does not split). Calls on one stream run in order and so may share a set.
struct SplitWorkspace {
    int device = -1;
    hipStream_t stream = nullptr;
    float *partial = nullptr;
    size_t floats = 0;
    unsigned *arrivals = nullptr;
    size_t tiles = 0;
};
std::mutex g_ws_mutex;
std::vector<SplitWorkspace> g_ws;

hipError_t split_workspace(hipStream_t s, size_t floats, size_t tiles, float **partial, unsigned **arrivals) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    SplitWorkspace *w = nullptr;
    for (SplitWorkspace &c : g_ws)
        if (c.device == dev && c.stream == s) w = &c;
    if (!w) {
        g_ws.push_back(SplitWorkspace{});
        w = &g_ws.back();
        w->device = dev;
        w->stream = s;
    }
    if (w->floats < floats || w->tiles < tiles) {
        if (hipError_t e = hipStreamSynchronize(s)) return e;  // earlier launches may still use the old buffers
        if (w->partial) (void)hipFree(w->partial);
        if (w->arrivals) (void)hipFree(w->arrivals);
        w->partial = nullptr;
        w->arrivals = nullptr;
        w->floats = w->tiles = 0;
        const size_t nf = floats > w->floats ? floats : w->floats, nt = tiles > 1024 ? tiles : 1024;
        if (hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->partial), nf * sizeof(float))) return e;
        if (hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->arrivals), nt * sizeof(unsigned))) return e;
        if (hipError_t e = hipMemset(w->arrivals, 0, nt * sizeof(unsigned))) return e;
        w->floats = nf;
        w->tiles = nt;
    }
    *partial = w->partial;
    *arrivals = w->arrivals;
    return hipSuccess;
}

// TLLM_GEMM_WAVES picks the instance, for comparisons: 4 = four waves with hand-placed instructions (default),
// 8 = eight waves, 1 = the first four-wave kernel (instruction order left to the compiler).
int gemm_instance() {
    static const int v = [] {
        const char *e = getenv("TLLM_GEMM_WAVES");
        return e && e[0] == '8' ? 8 : e && e[0] == '1' ? 1 : 4;
    }();
    return v;
}

template <int MF>
hipError_t launch(const Problem &p, int splits, hipStream_t s) {
    constexpr int BM = 128 * MF;
    static std::mutex attr_mutex;
    static bool attr_set[64][3] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    const int inst = gemm_instance(), slot = inst == 8 ? 2 : inst == 4 ? 1 : 0;
    const size_t lds = kBufs * (size_t)(kWBytes + BM * kRowBytes + (inst == 8 ? 4 : 3) * 1024);
    if (dev >= 0 && dev < 64) {
        std::lock_guard<std::mutex> lock(attr_mutex);
        if (!attr_set[dev][slot]) {
            const void *k = inst == 8   ? reinterpret_cast<const void *>(&gemm_mfma8_kernel<MF>)
                            : inst == 4 ? reinterpret_cast<const void *>(&gemm_mfma4_kernel<MF>)
                                        : reinterpret_cast<const void *>(&gemm_mfma_kernel<MF>);
            if (hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)) return e;
            attr_set[dev][slot] = true;
        }
    }
    const int m_tiles = (p.batch + BM - 1) / BM, n_tiles = (p.rows + kBN - 1) / kBN;
    const int tiles = m_tiles * n_tiles;
    float *partial = nullptr;
    unsigned *arrivals = nullptr;
    if (splits > 1)
        if (hipError_t e = split_workspace(s, (size_t)tiles * splits * BM * kBN, (size_t)tiles, &partial, &arrivals)) return e;
    if (inst == 8)
        gemm_mfma8_kernel<MF><<<tiles * splits, kThreads8, lds, s>>>(p.x, p.nz, p.sg, p.scales, p.y, p.batch, p.rows, p.cols,
                                                                     splits, partial, arrivals);
    else if (inst == 4)
        gemm_mfma4_kernel<MF><<<tiles * splits, kThreads, lds, s>>>(p.x, p.nz, p.sg, p.scales, p.y, p.batch, p.rows, p.cols,
                                                                   splits, partial, arrivals);
    else
        gemm_mfma_kernel<MF><<<tiles * splits, kThreads, lds, s>>>(p.x, p.nz, p.sg, p.scales, p.y, p.batch, p.rows, p.cols,
                                                                  splits, partial, arrivals);
    return hipGetLastError();
}

}  // namespace

bool gemm_mfma_supports(const Problem &p, int group) {
    // scales are fetched as aligned dwords: the array must start on one and hold an even count
    if ((reinterpret_cast<uintptr_t>(p.scales) & 3) || (((size_t)p.rows * (p.cols / 128)) & 1)) return false;
    return group == 128 && p.batch >= 16 && p.cols % 128 == 0 && (size_t)p.rows * (p.cols / 32) < ((size_t)1 << 31) &&
           (size_t)p.batch * p.cols < ((size_t)1 << 31);
}

namespace {
struct GemmConfig {
    int height;  // 0: 128 activation rows per workgroup, 1: 256
    int splits;  // workgroups per tile along K
    float us;    // estimated time
};

// One workgroup occupies a CU (LDS). Taller tiles do more per stage, shorter tiles fill the chip
// when there are few of them, and when even those leave CUs idle K is split across workgroups.
// Estimate: (rounds of workgroups over the CUs) x (stages per workgroup) x (time of one stage,
// measured: 1.19 / 0.70 us for 256 / 128 activation rows) + 5 us + the traffic of a split's exchange.
GemmConfig choose_config(const Problem &p) {
    const int n_cu = current_device_cus();
    const int n_tiles = (p.rows + kBN - 1) / kBN, groups = p.cols / 128;
    const float stage_us[2] = {0.70f, 1.19f};
    GemmConfig best{0, 1, 0.f};
    for (int c = 0; c < 2; c++) {
        const int bm = 128 << c;
        const long tiles = (long)n_tiles * ((p.batch + bm - 1) / bm);
        for (int splits = 1; splits <= 8; splits *= 2) {
            if (splits > 1 && (tiles * splits > n_cu || groups / splits < 4)) break;  // only to fill idle CUs
            const long wgs = tiles * splits;
            const float stages = (float)((groups + splits - 1) / splits * 2);
            // the exchange: all workgroups write their fp32 tile at once (about 5.5 us with the
            // hand-over), then the last one of a tile reads the `splits` slots on its own, at about
            // 29 GB/s (fitted to 14336x4096 and 4096x14336 at M = 128: 10 us with 2, 23.5 us with 8)
            const float exchange = splits > 1 ? 5.5f + (float)splits * (float)(bm * kBN * 4) / 29.0e3f : 0.0f;
            const float us = (float)((wgs + n_cu - 1) / n_cu) * stages * stage_us[c] + 5.0f + exchange;
            if (best.us == 0.f || us < best.us) best = GemmConfig{c, splits, us};
        }
    }
    return best;
}
}  // namespace

float gemm_mfma_cost_us(const Problem &p) { return choose_config(p).us; }

hipError_t launch_gemm_mfma(const Problem &p, hipStream_t s) {
    const GemmConfig c = choose_config(p);
    if (c.height == 1) return launch<2>(p, c.splits, s);
    return launch<1>(p, c.splits, s);
}

}  // namespace tllm
