// Prefill GEMM on the matrix cores (gfx950), group size 128, M >= 16.
//
// Arithmetic (reference kernels/ternary_gemm.cu:106-175): C[m,n] = sum_k scale[n, k/128] * w[n,k] * A[m,k],
// the scale multiplied into every element, fp32 accumulation, fp16 store (round to nearest even).
// Here the product scale * w is formed exactly in fp16 (w in {-1,0,+1}), so the only difference to
// the reference is the order of the fp32 additions.
//
// Two kernels, chosen per shape by a cost model (choose_config): the four-wave kernel described next and the row-split
// kernel (gemm_ns_kernel), described where it is defined.
//
// Tiling of the four-wave kernel. A workgroup (4 waves, one per SIMD) computes 128 weight rows x BM activation rows; every wave
// owns all 128 weight rows and BM/4 activation rows of its own. Per stage of 64 columns of K:
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
//   * each wave multiplies with v_mfma_f32_32x32x16_f16 in four steps of 16 columns; lane half q of
//     step ks sums columns 16 ks + 8 q .. + 7 (both operands use the same assignment); operands come
//     from LDS as 16-byte chunks, XOR-swizzled by row against bank conflicts.
// Three LDS buffers per operand, one barrier per stage; the kernel spells out the pipeline.
#include <stdlib.h>

#include <algorithm>
#include <mutex>
#include <type_traits>
#include <utility>

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
constexpr int kBK = 64;      // K columns per stage (four MFMA steps of 16)
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

// The kernel: one wave per SIMD, wave tile 128 weight rows x 32*MF activation rows (4 x MF accumulator
// fragments of 32 x 32).
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
__global__ __launch_bounds__(kThreads, 1) void gemm_mfma_kernel(
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
                    // A store of more than 8 bytes still reads its data registers for two issue slots after it
                    // has issued; the compiler keeps other writers away from its own stores but cannot see into
                    // this one, so the slots are filled here (without them the next address computation landed
                    // in the data registers of the store before it and a quarter of the lanes stored garbage).
                    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
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

// ---- The row-split kernel: the waves of a workgroup split the weight rows, weights decoded straight into MFMA operand
// registers.
//
// A workgroup computes 256 weight rows x 32 MF activation rows; a wave owns NF A-operand fragments of 32 weight rows and
// all the activation rows (NF x MF accumulator fragments). What this changes against the kernels above:
//   * decoded weights never pass through LDS (its write port was the slowest unit of those kernels): lane (li, lq) of wave
//     w loads the mask words of its own row, and the byte of a word IS the eight weights of one MFMA operand: one
//     v_perm puts byte t of the even-weight and odd-weight codes into the two halves of a dword, then a packed shift,
//     an AND and a packed multiply per weight pair: 13 vector instructions per MFMA step, used by MF MFMAs.
//     K is walked in an order that makes this possible: a block of 256 columns is four chunks of 64; in step t of chunk u
//     lane half lq multiplies the 8 columns 256 b + 64 u + 32 lq + 8 t .. + 7, i.e. byte t of mask word 2 u + lq. Both
//     operands use the same assignment, and a sum does not care in which order the columns are taken.
//     A lane loads mask words 4 lq .. 4 lq + 3 of a block (16 bytes per plane) and the two half-waves then trade words
//     with v_permlane32_swap; the two scales of a block come as one dword.
//   * the activations of the tile come straight from A[M][K] (no reordered copy): the load instruction writes them into
//     LDS (global_load_lds, 16 bytes per lane) in 1 KB pieces of 16 rows x 64 bytes, lane 16 t + r fetching step t of
//     row r, so that the B operand of (step t, fragment j) is one conflict-free ds_read_b128 per lane. A chunk is
//     MF x 4 KB; four chunks are in flight (ring of four slots, one barrier per chunk, taken one step before the
//     chunk's end so that the first fragment reads of the next chunk are already on their way).
//   * the vector work of step s + 1 is dealt out between the MFMAs of step s.
// Tiles that do not fill the last round of workgroups over the CUs are split along K between several workgroups
// (`splits`), which exchange fp32 sums through memory like the kernels above; the tiles before them (`full_tiles`)
// run whole. The workgroups of one XCD take consecutive work items of both kinds.
//
// Two shapes of workgroup compute the same 256 x 128 tile. NF = 1: eight waves (two per SIMD) with one weight fragment
// each: one workgroup per CU, the fastest when there are not enough tiles for two workgroups per CU. NF = 2: four waves
// (one per SIMD) with two weight fragments each, so that every activation fragment read from LDS feeds two MFMAs, and
// two workgroups per CU: the waves that share a SIMD then belong to different workgroups and do not wait for each
// other at barriers, and one workgroup's first loads and last stores hide behind the other's MFMAs.
constexpr int kNsBN = 256;
constexpr int kNsPitch = 2 * kNsBN + 16;  // bytes per activation row of the output tile in LDS

// kPair (NF = 2 only): the prefill form of a SwiGLU pair (reference src/transformer.cpp:264-286 at n_tokens > 1: gate GEMM,
// up GEMM, silu_mul_forward). A wave's two weight fragments are the SAME 32 rows of the gate matrix (B arrays) and of the
// up matrix (U arrays), so every activation fragment read from LDS feeds one MFMA of each, the activation tile is
// fetched once for both matrices, and the two accumulators that meet in the epilogue sit in the same lane: the tile
// (128 rows of each matrix x 128 activation rows) is stored once, as fp16(silu(fp16 gate) * fp16 up). No K split.
// kGroup: up to four weight matrices that share the activations in one launch (the q, k and v projections of a prefill
// step, reference src/transformer.cpp:199-217 at n_tokens > 1: three ternary_gemm calls on the same input). The tiles of
// the matrices are numbered one after the other (matrix g owns tiles prefix[g] .. prefix[g + 1] - 1) and dealt to the
// workgroups, whole or split along K, exactly as the tiles of one matrix are: three small matrices fill the chip
// together where each alone leaves most of it idle. Every output is what the single call computes when its tiles are
// split the same way.
struct GemmGroup {
    int count;
    int prefix[5];
    int N[4];
    const uint32_t *nz[4];
    const uint32_t *sg[4];
    const uint16_t *sc[4];
    uint16_t *C[4];
};
template <int MF, int NF, bool kPair = false, bool kGroup = false>
__global__ __launch_bounds__(512 / NF) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_ns_kernel(
    const uint16_t *__restrict__ A, const uint32_t *__restrict__ nzB_, const uint32_t *__restrict__ sgB_,
    const uint16_t *__restrict__ scB_, uint16_t *__restrict__ C_, int M, int N_, int K, int full_tiles, int splits,
    int n_fastest, float *__restrict__ partial, unsigned *__restrict__ arrivals, const uint32_t *__restrict__ nzU = nullptr,
    const uint32_t *__restrict__ sgU = nullptr, const uint16_t *__restrict__ scU = nullptr, GemmGroup grp = GemmGroup{}) {
    static_assert(!kPair || NF == 2, "a pair is the two fragments of a wave");
    static_assert(!(kPair && kGroup), "one or the other");
    const uint32_t *__restrict__ nzB = nzB_;
    const uint32_t *__restrict__ sgB = sgB_;
    const uint16_t *__restrict__ scB = scB_;
    uint16_t *__restrict__ C = C_;
    int N = N_;
    constexpr int BM = 32 * MF;
    constexpr int kTileN = kPair ? kNsBN / 2 : kNsBN;  // weight rows (of each matrix) per workgroup
    constexpr int kWaves = 8 / NF, kNsThreads = 64 * kWaves;
    constexpr int kChunk = 4 * MF * 1024;    // bytes of one chunk: four steps of MF fragments
    constexpr int kDma = MF * 4 / kWaves;    // 1 KB pieces per wave and chunk
    static_assert(MF == 4, "the ring of four chunks is addressed with 16-bit offsets: 4 x 16 KB");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    typedef __attribute__((address_space(3))) unsigned char LB;
    typedef __attribute__((address_space(1))) const unsigned char GB;
    LB *lds_l = (LB *)lds;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lq = lane >> 5;

    // ---- which tile, which part of K. Workgroup ids go round the XCDs: XCD x takes the x-th eighth of the whole tiles
    // first and the x-th eighth of the parts of split tiles afterwards.
    const int m_tiles = (M + BM - 1) / BM;
    int n_tiles = (N + kTileN - 1) / kTileN;
    const int tiles = kGroup ? grp.prefix[grp.count] : m_tiles * n_tiles, parts = (tiles - full_tiles) * splits;
    const int full_per = (full_tiles + 7) / 8, part_per = (parts + 7) / 8;
    const int xcd = (int)blockIdx.x & 7, slot_in_xcd = (int)blockIdx.x >> 3;
    int tile, split = 0;
    if (slot_in_xcd < full_per) {
        tile = xcd * full_per + slot_in_xcd;
        if (tile >= full_tiles) return;
    } else {
        const int part = xcd * part_per + (slot_in_xcd - full_per);
        if (part >= parts) return;
        tile = full_tiles + part / splits;
        split = part - (part / splits) * splits;
    }
    const bool is_split = tile >= full_tiles && splits > 1;
    // consecutive tiles (one XCD's share) walk the activation tiles of one weight tile first, or the weight tiles of one
    // activation tile first: whichever lets an XCD's L2 fetch fewer bytes for its share (the launcher decides)
    int local = tile;  // the tile's number inside its matrix
    if constexpr (kGroup) {
        int g = 0;
#pragma unroll
        for (int k = 1; k < 4; k++) g += k < grp.count && tile >= grp.prefix[k];
        local = tile - grp.prefix[g];
        nzB = grp.nz[g];
        sgB = grp.sg[g];
        scB = grp.sc[g];
        C = grp.C[g];
        N = grp.N[g];
        n_tiles = (N + kTileN - 1) / kTileN;
    }
    const int n0 = (n_fastest ? local % n_tiles : local / m_tiles) * kTileN;
    const int m0 = (n_fastest ? local / n_tiles : local % m_tiles) * BM;
    // K is a multiple of 128: a last block of 128 columns runs as a whole block whose upper mask words are zero
    // (its activation chunks past the row re-read the last chunk: they meet zero weights)
    const int words = K / 32, groups = K / 128, blocks = (K + 255) / 256;
    const int chunks = K / 64;
    const bool tail_half = (K & 255) != 0;
    const int b_begin = is_split ? (int)((long)blocks * split / splits) : 0;
    const int b_end = is_split ? (int)((long)blocks * (split + 1) / splits) : blocks;

    // fragment f of wave w: weight rows n0 + 32 (NF w + f) .. + 31
    GB *nz_g[NF], *sg_g[NF], *sc_g[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) {
        const int row = min(n0 + (kPair ? 32 * wave : 32 * (NF * wave + f)) + li, N - 1);
        const bool up = kPair && f == 1;
        nz_g[f] = (GB *)(up ? nzU : nzB) + ((size_t)row * words + 4 * lq) * 4;
        sg_g[f] = (GB *)(up ? sgU : sgB) + ((size_t)row * words + 4 * lq) * 4;
        sc_g[f] = (GB *)(up ? scU : scB) + (size_t)row * groups * 2;  // two scales per block: one aligned dword (groups is even)
    }

    // activation pieces this wave copies per chunk: piece p = wave * kDma + i covers fragment j = p / 4, rows
    // 16 h .. 16 h + 15 of it (h = (p / 2) % 2), column half q = p % 2; lane L of the copy fetches step L / 16 of row
    // L % 16. Rows past M repeat the last row (their outputs are not stored).
    GB *a_src[kDma];
    int a_dst[kDma];
#pragma unroll
    for (int i = 0; i < kDma; i++) {
        const int p = wave * kDma + i, j = p >> 2, h = (p >> 1) & 1, q = p & 1;
        const int m = min(m0 + 32 * j + 16 * h + (lane & 15), M - 1);
        a_src[i] = (GB *)A + ((size_t)m * K + 32 * q + 8 * (lane >> 4)) * 2;
        a_dst[i] = p * 1024;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds_l;
    const uint32_t b_rd = lds0 + (uint32_t)((((li >> 4) * 2 + lq) * 1024) + (li & 15) * 16);
#define TLLM_GPTR(p) ((__attribute__((address_space(1))) const void *)(p))
#define TLLM_LPTR(p) ((__attribute__((address_space(3))) void *)(p))
    // The destination of an asm load is "+v": the register that is being filled is then the one the variable had
    // before, and no copy of a register still in flight can appear on a loop edge.
#define TLLM_LDS_READ128(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "+v"(dst) : "v"(addr), "i"(off))
#define TLLM_FENCE() __builtin_amdgcn_sched_barrier(0)
    auto dma_chunk = [&](int c, int slot) {
        const int off = min(c, chunks - 1) * 128;
#pragma unroll
        for (int i = 0; i < kDma; i++)
            __builtin_amdgcn_global_load_lds(TLLM_GPTR(a_src[i] + off), TLLM_LPTR(lds_l + slot * kChunk + a_dst[i]), 16, 0, 0);
    };
    u4 nx_nz[NF], nx_sg[NF];
    uint32_t nx_sc[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) {
        nx_nz[f] = u4{0u, 0u, 0u, 0u};
        nx_sg[f] = u4{0u, 0u, 0u, 0u};
        nx_sc[f] = 0;
    }
    auto half_block = [&](int b) { return tail_half && b >= blocks - 1; };
    auto load_masks = [&](int b) {
        const int bb = min(b, blocks - 1);
        // a half block holds mask words 0..3 and one scale: the upper lane half, which would load words 4..7 from
        // the next row (or from beyond the array), loads the lower words again (dropped in take_masks); the scale
        // dword starts one scale earlier, so that it ends with the row
        const int back = half_block(b) ? 16 * lq : 0, sc_back = half_block(b) ? 2 : 0;
#pragma unroll
        for (int f = 0; f < NF; f++) {
            GB *p0 = nz_g[f] + (size_t)bb * 32 - back;
            GB *p1 = sg_g[f] + (size_t)bb * 32 - back;
            GB *p2 = sc_g[f] + (size_t)bb * 4 - sc_back;
            asm volatile("global_load_dwordx4 %0, %1, off" : "+v"(nx_nz[f]) : "v"(p0) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, off" : "+v"(nx_sg[f]) : "v"(p1) : "memory");
            asm volatile("global_load_dword %0, %1, off" : "+v"(nx_sc[f]) : "v"(p2) : "memory");
        }
    };

    f16v acc[NF][MF];
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int j = 0; j < MF; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[f][j][r] = 0.f;

    uint32_t cu_nz[NF][4], cu_sg[NF][4];  // mask word 2 u + lq of the current block
    h2 sp2[NF][2];                        // its two scales, each in both halves
    u4 Bv[2][MF];
#pragma unroll
    for (int q = 0; q < 2; q++)
#pragma unroll
        for (int j = 0; j < MF; j++) Bv[q][j] = u4{0u, 0u, 0u, 0u};
    u4 av[2][NF];
    uint32_t t0[NF] = {}, t1[NF] = {}, qn[NF] = {};
    h2 sp[NF] = {};
    auto codes = [&](int f, int u) {  // the two-bit codes (negative, non-zero) of mask word u: even weights in t0, odd weights in t1
        const uint32_t m_nz = cu_nz[f][u], m_sg = cu_sg[f][u];
        sp[f] = sp2[f][u >> 1];
        const uint32_t neg = m_nz & ~m_sg;
        t0[f] = __builtin_amdgcn_bitop3_b32(neg << 1, m_nz, 0xAAAAAAAAu, 0xE4);
        t1[f] = __builtin_amdgcn_bitop3_b32(neg, m_nz >> 1, 0xAAAAAAAAu, 0xE4);
    };
    auto pick = [&](int f, int t) {  // byte t of the even codes into the low half, of the odd codes into the high half
        qn[f] = __builtin_amdgcn_perm(t1[f], t0[f], 0x0C000C00u | (uint32_t)t | ((uint32_t)(4 + t) << 16));
    };
    auto pair = [&](int f, int e) -> uint32_t {  // weights 2 e, 2 e + 1 of the byte as +-2 scale / 0
        us2 v = __builtin_bit_cast(us2, qn[f]);
        v = v << (uint16_t)(14 - 2 * e);
        uint32_t top = __builtin_bit_cast(uint32_t, v);
        if (e > 0) top &= 0xC000C000u;  // (for e = 0 the shift leaves nothing below the field)
        return __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, top) * sp[f]);
    };
    auto take_masks = [&](bool half) {  // the loads into nx_* are complete where this is called; half: a last block of 128 columns
#pragma unroll
        for (int f = 0; f < NF; f++) {
            asm volatile("" : "+v"(nx_nz[f]), "+v"(nx_sg[f]), "+v"(nx_sc[f]));
            const auto s01 = __builtin_amdgcn_permlane32_swap(nx_nz[f][0], nx_nz[f][1], false, false);
            const auto s23 = __builtin_amdgcn_permlane32_swap(nx_nz[f][2], nx_nz[f][3], false, false);
            const auto g01 = __builtin_amdgcn_permlane32_swap(nx_sg[f][0], nx_sg[f][1], false, false);
            const auto g23 = __builtin_amdgcn_permlane32_swap(nx_sg[f][2], nx_sg[f][3], false, false);
            cu_nz[f][0] = s01[0]; cu_nz[f][2] = s01[1]; cu_nz[f][1] = s23[0]; cu_nz[f][3] = s23[1];
            cu_sg[f][0] = g01[0]; cu_sg[f][2] = g01[1]; cu_sg[f][1] = g23[0]; cu_sg[f][3] = g23[1];
            sp2[f][0] = __builtin_bit_cast(h2, __builtin_amdgcn_perm(nx_sc[f], nx_sc[f], half ? 0x03020302u : 0x01000100u));
            sp2[f][1] = __builtin_bit_cast(h2, __builtin_amdgcn_perm(nx_sc[f], nx_sc[f], 0x03020302u));
            if (half) {  // words 4..7 do not exist: no weights there
                cu_nz[f][2] = 0;
                cu_nz[f][3] = 0;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) asm volatile("" : "+v"(cu_nz[f][u]), "+v"(cu_sg[f][u]));
            asm volatile("" : "+v"(sp2[f][0]), "+v"(sp2[f][1]));
        }
    };

    // ---- prologue: masks of the first two blocks, the first four chunks; operands of the first step.
    // Requests complete in order; every wait below names how many younger ones may still be in flight.
    const int c_begin = 4 * b_begin;
    load_masks(b_begin);
    dma_chunk(c_begin, 0);
    dma_chunk(c_begin + 1, 1);
    dma_chunk(c_begin + 2, 2);
    TLLM_FENCE();
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kDma) : "memory");
    __builtin_amdgcn_s_barrier();
    TLLM_FENCE();
    take_masks(half_block(b_begin));
    load_masks(b_begin + 1);
    dma_chunk(c_begin + 3, 3);
    TLLM_FENCE();
#pragma unroll
    for (int j = 0; j < MF; j++) TLLM_LDS_READ128(Bv[0][j], b_rd, j * 4096);
#pragma unroll
    for (int f = 0; f < NF; f++) {
        codes(f, 0);
        pick(f, 0);
        av[0][f] = u4{pair(f, 0), pair(f, 1), pair(f, 2), pair(f, 3)};
    }
    TLLM_FENCE();

    // One step: the MFMAs of step s = (chunk c in ring slot u, t) with the decode of step s + 1 between them; the
    // activation fragments of step s + 1 are requested first. The last step of a chunk begins by taking the workgroup
    // across the barrier that frees the chunk's slot (every wave has its last fragments of it) and proves that the next
    // chunk has landed (every wave has waited for its own pieces); the slot is refilled with chunk c + 4. Request order
    // is: masks of block b + 2 (asked for in the last step of block b), then the chunks; a chunk's wait therefore
    // leaves the two younger chunks in flight and, in the two steps that follow a mask request, those three loads too.
    auto kstep = [&](auto U, auto T, int c) {
        constexpr int u = decltype(U)::value, t = decltype(T)::value;
        constexpr int cur = t & 1, nxt = cur ^ 1;
        constexpr int ru = t == 3 ? ((u + 1) & 3) : u, rt = (t + 1) & 3;
        if (t == 3) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (u < 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kDma + 3 * NF) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kDma) : "memory");
            __builtin_amdgcn_s_barrier();
            TLLM_FENCE();
            if (u == 3) {
                take_masks(half_block((c + 1) / 4));
                load_masks((c + 1) / 4 + 1);
            }
            dma_chunk(c + 4, u);
            TLLM_FENCE();
        }
#pragma unroll
        for (int j = 0; j < MF; j++) TLLM_LDS_READ128(Bv[nxt][j], b_rd, ru * kChunk + j * 4096 + rt * 256);
        if (t != 3) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(MF) : "memory");
        TLLM_FENCE();
        u4(&R)[MF] = Bv[cur];
        u4(&a_cur)[NF] = av[cur];
        uint32_t an[NF][4];
#pragma unroll
        for (int f = 0; f < NF; f++)
#pragma unroll
            for (int j = 0; j < MF; j++) {
                if (f == 0) asm volatile("" : "+v"(R[j]));
                acc[f][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a_cur[f]), __builtin_bit_cast(h8, R[j]), acc[f][j], 0, 0, 0);
                TLLM_FENCE();
                // the decode of fragment f of step s + 1 behind the MFMAs of fragment f
                if (j == 0) {
                    if (t == 3) codes(f, ru);
                    pick(f, rt);
                }
                an[f][j] = pair(f, j);
                asm volatile("" : "+v"(an[f][j]));  // computed here, between the MFMAs, not where it is used
                TLLM_FENCE();
            }
#pragma unroll
        for (int f = 0; f < NF; f++) av[nxt][f] = u4{an[f][0], an[f][1], an[f][2], an[f][3]};
    };
    std::integral_constant<int, 0> i0;
    std::integral_constant<int, 1> i1;
    std::integral_constant<int, 2> i2;
    std::integral_constant<int, 3> i3;
    for (int b = b_begin; b < b_end; b++) {
        kstep(i0, i0, 4 * b); kstep(i0, i1, 4 * b); kstep(i0, i2, 4 * b); kstep(i0, i3, 4 * b);
        kstep(i1, i0, 4 * b + 1); kstep(i1, i1, 4 * b + 1); kstep(i1, i2, 4 * b + 1); kstep(i1, i3, 4 * b + 1);
        kstep(i2, i0, 4 * b + 2); kstep(i2, i1, 4 * b + 2); kstep(i2, i2, 4 * b + 2); kstep(i2, i3, 4 * b + 2);
        kstep(i3, i0, 4 * b + 3); kstep(i3, i1, 4 * b + 3); kstep(i3, i2, 4 * b + 3); kstep(i3, i3, 4 * b + 3);
    }
    TLLM_FENCE();
    // copies and fragment reads past the last step are still in flight into LDS and registers
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    // the compiler cannot see that the asm stores below read matrix results: the slots a 16-pass product needs before
    // its result may be read by a memory instruction
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3" ::: "memory");
#undef TLLM_LDS_READ128
#undef TLLM_FENCE
#undef TLLM_GPTR
#undef TLLM_LPTR

    if (is_split) {
        // fp32 sums of this part into its slot (quad g of fragment (f, j) of thread tid at
        // (((f * MF + j) * 4 + g) * threads + tid) * 4), written through to memory; the last part of a tile to arrive adds
        // all slots in part order, its own included (read back: a second register set for its own sums would not fit),
        // so the bits do not depend on which part arrives last
        constexpr int kSlot = BM * kNsBN;
        const int st = tile - full_tiles;
        float *mine = partial + ((size_t)st * splits + split) * kSlot + tid * 4;
#pragma unroll
        for (int fj = 0; fj < NF * MF; fj++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const f16v &a = acc[fj / MF][fj % MF];
                const f4 v = {a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
                float *dst = mine + (size_t)(fj * 4 + g) * kNsThreads * 4;
                // (two idle issue slots: a store of more than 8 bytes still reads its data registers after it has issued)
                asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
            }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __shared__ unsigned last_arrival_ns;
        __syncthreads();
        if (tid == 0) {
            const unsigned before = __hip_atomic_fetch_add(&arrivals[st], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_arrival_ns = before == (unsigned)splits - 1;
            if (last_arrival_ns) __hip_atomic_store(&arrivals[st], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!last_arrival_ns) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const float *slots = partial + (size_t)st * splits * kSlot + tid * 4;
#pragma unroll
        for (int fj = 0; fj < NF * MF; fj++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[fj / MF][fj % MF][r] = 0.f;
        for (int q = 0; q < splits; q++) {
            const float *slot = slots + (size_t)q * kSlot;
#pragma unroll
            for (int fj = 0; fj < NF * MF; fj++) {
                f4 v[4];
#pragma unroll
                for (int g = 0; g < 4; g++) v[g] = *reinterpret_cast<const f4 *>(slot + (size_t)(fj * 4 + g) * kNsThreads * 4);
                f16v &a = acc[fj / MF][fj % MF];
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int e = 0; e < 4; e++) a[4 * g + e] += v[g][e];
            }
        }
    }

    // ---- store. Register 4 g + v of fragment (f, j) is weight row n0 + 32 (NF wave + f) + 8 g + 4 lq + v for activation row
    // m0 + 32 j + li: stored as they are these are 8-byte pieces in 32 different lines per instruction. The tile goes
    // through LDS instead (the ring is free now) and leaves as whole 512-byte rows, two rows per instruction.
    const bool wide_store = (N & 7) == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0;
    if constexpr (kPair) {
        // silu(gate) * up on the fp16-rounded products, in fp32: what the two GEMMs and the element-wise kernel store
        auto joined = [&](int j, int r) -> uint16_t {
            const float g = h2f(f2h(acc[0][j][r] * 0.5f)), u = h2f(f2h(acc[1][j][r] * 0.5f));
            return f2h(g / (1.0f + expf(-g)) * u);
        };
        if (wide_store) {
            __syncthreads();  // every wave is done with the ring
#pragma unroll
            for (int j = 0; j < MF; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    uint16_t hv[4];
#pragma unroll
                    for (int v = 0; v < 4; v++) hv[v] = joined(j, 4 * g + v);
                    *reinterpret_cast<uint2 *>(lds + (32 * j + li) * kNsPitch + (32 * wave + 8 * g + 4 * lq) * 2) =
                        uint2{(uint32_t)hv[0] | ((uint32_t)hv[1] << 16), (uint32_t)hv[2] | ((uint32_t)hv[3] << 16)};
                }
            __syncthreads();
            // rows of 128 outputs = 256 bytes: sixteen lanes per activation row, four rows per instruction
            const int piece = lane & 15;
            const int n = n0 + piece * 8;
#pragma unroll
            for (int r = 0; r < BM / (4 * kWaves); r++) {
                const int ml = wave * (BM / kWaves) + 4 * r + (lane >> 4);
                const int m = m0 + ml;
                if (m < M && n < N) *reinterpret_cast<u4 *>(C + (size_t)m * N + n) = *reinterpret_cast<const u4 *>(lds + ml * kNsPitch + piece * 16);
            }
        } else {
#pragma unroll
            for (int j = 0; j < MF; j++) {
                const int m = m0 + j * 32 + li;
                if (m >= M) continue;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int n = n0 + 32 * wave + 8 * g + 4 * lq;
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (n + v < N) C[(size_t)m * N + n + v] = joined(j, 4 * g + v);
                }
            }
        }
    } else if (wide_store) {
        __syncthreads();  // every wave is done with the ring
#pragma unroll
        for (int fj = 0; fj < NF * MF; fj++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int f = fj / MF, j = fj % MF;
                uint16_t hv[4];
#pragma unroll
                for (int v = 0; v < 4; v++) hv[v] = f2h(acc[f][j][4 * g + v] * 0.5f);
                *reinterpret_cast<uint2 *>(lds + (32 * j + li) * kNsPitch + (32 * (NF * wave + f) + 8 * g + 4 * lq) * 2) =
                    uint2{(uint32_t)hv[0] | ((uint32_t)hv[1] << 16), (uint32_t)hv[2] | ((uint32_t)hv[3] << 16)};
            }
        __syncthreads();
        const int piece = lane & 31;
        const int n = n0 + piece * 8;
#pragma unroll
        for (int r = 0; r < BM / (2 * kWaves); r++) {
            const int ml = wave * (BM / kWaves) + 2 * r + lq;
            const int m = m0 + ml;
            if (m < M && n < N) *reinterpret_cast<u4 *>(C + (size_t)m * N + n) = *reinterpret_cast<const u4 *>(lds + ml * kNsPitch + piece * 16);
        }
    } else {
#pragma unroll
        for (int fj = 0; fj < NF * MF; fj++) {
            const int f = fj / MF, j = fj % MF;
            const int m = m0 + j * 32 + li;
            if (m >= M) continue;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int n = n0 + 32 * (NF * wave + f) + 8 * g + 4 * lq;
#pragma unroll
                for (int v = 0; v < 4; v++)
                    if (n + v < N) C[(size_t)m * N + n + v] = f2h(acc[f][j][4 * g + v] * 0.5f);
            }
        }
    }
}

// ---- split-K exchange memory: fp32 slots and one arrival counter per tile.
//
// Ordinary calls use a workspace per (device, stream), created by tllm_gemm_workspace_reserve or by the first call
// that needs one. It is allocated ONCE, at the largest size any configuration is allowed to need (the limit the
// kernel choice works under, kStaticSlotFloats), and lives at that address until tllm_gemm_workspace_release: a graph
// captured on the stream keeps pointing at valid memory whatever shapes run on the stream afterwards. Calls on one
// stream run in order and so may share it. Nothing is allocated or synchronised while the stream is being captured
// into a graph: a call that would have to falls back to one workgroup per tile (no exchange).
struct SplitWorkspace {
    int device = -1;
    hipStream_t stream = nullptr;
    float *partial = nullptr;
    unsigned *arrivals = nullptr;
};
constexpr size_t kArrivalSlots = kSplitArrivalSlots;  // tiles of a split launch (at most one per CU pair)
constexpr size_t kWorkspaceFloats = (size_t)TLLM_GEMM_STATIC_SCRATCH_BYTES / 4 - kArrivalSlots;
std::mutex g_ws_mutex;
std::vector<SplitWorkspace> g_ws;

// may_allocate = false: only hands out what exists. *partial stays null when there is none (or the need exceeds
// what a workspace ever holds).
hipError_t split_workspace(hipStream_t s, size_t floats, bool may_allocate, float **partial, unsigned **arrivals) {
    if (floats > kWorkspaceFloats) return hipSuccess;
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    SplitWorkspace *w = nullptr;
    for (SplitWorkspace &c : g_ws)
        if (c.device == dev && c.stream == s) w = &c;
    if (!w) {
        if (!may_allocate) return hipSuccess;
        // counters first, then the slots: one allocation. The counters are cleared here, synchronously, so that they
        // are zero for whichever stream a launch (or the replay of a graph) that uses them runs on; every launch
        // leaves them at zero again.
        unsigned char *base = nullptr;
        if (hipError_t e = hipMalloc(reinterpret_cast<void **>(&base), (kArrivalSlots + kWorkspaceFloats) * 4)) return e;
        hipError_t e = hipMemset(base, 0, kArrivalSlots * sizeof(unsigned));
        if (!e) e = hipDeviceSynchronize();
        if (e) {
            (void)hipFree(base);
            return e;
        }
        g_ws.push_back(SplitWorkspace{dev, s, reinterpret_cast<float *>(base) + kArrivalSlots, reinterpret_cast<unsigned *>(base)});
        w = &g_ws.back();
    }
    *partial = w->partial;
    *arrivals = w->arrivals;
    return hipSuccess;
}

// The exchange memory of tllm_ternary_gemm_f16_static: a fixed array in device memory, one copy per GPU,
// held until the process ends. Arrival counters first (zero when the module is loaded, left at zero by
// every launch), then the fp32 slots.
constexpr size_t kStaticSlotFloats = kWorkspaceFloats;
static __device__ __align__(256) unsigned char scratch[TLLM_GEMM_STATIC_SCRATCH_BYTES];

// Device address of `scratch` on the current device, asked once per device.
hipError_t static_scratch(unsigned char **out) {
    static std::mutex m;
    static unsigned char *ptr[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(m);
    if (!ptr[dev]) {
        unsigned char *p = nullptr;
        if (hipError_t e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch))) return e;
        ptr[dev] = p;
    }
    *out = ptr[dev];
    return hipSuccess;
}

struct GemmConfig {
    int height;   // four-wave kernel: 0 = 128 activation rows per workgroup, 1 = 256
    int splits;   // workgroups per tile along K (four-wave kernel: every tile; row-split kernel: the tiles after full_tiles)
    float us;     // estimated time
    bool rowsplit = false;  // the row-split kernel (256 weight rows x 128 activation rows per workgroup)
    int full_tiles = 0;     // row-split kernel: tiles computed by one workgroup each
    int frags = 1;          // row-split kernel: weight fragments per wave (1: eight waves, one workgroup per CU; 2: four waves, two per CU)
};
GemmConfig choose_config(const Problem &p, size_t workspace_floats);

// Workspace a configuration needs, in floats: the fp32 slots of a split.
size_t workspace_floats(const Problem &p, const GemmConfig &c) {
    if (c.rowsplit) {
        const size_t tiles = (size_t)((p.batch + 127) / 128) * ((p.rows + kNsBN - 1) / kNsBN);
        return c.splits > 1 ? (tiles - c.full_tiles) * c.splits * 128 * kNsBN : 0;
    }
    const int bm = 128 << c.height;
    const size_t tiles = (size_t)((p.batch + bm - 1) / bm) * ((p.rows + kBN - 1) / kBN);
    return c.splits > 1 ? tiles * c.splits * bm * kBN : 0;
}

template <int MF>
hipError_t launch(const Problem &p, int splits, float *partial, unsigned *arrivals, hipStream_t s) {
    constexpr int BM = 128 * MF;
    static std::mutex attr_mutex;
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    const size_t lds = kBufs * (size_t)(kWBytes + BM * kRowBytes + 3 * 1024);
    if (dev >= 0 && dev < 64) {
        std::lock_guard<std::mutex> lock(attr_mutex);
        if (!attr_set[dev]) {
            if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_kernel<MF>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
                return e;
            attr_set[dev] = true;
        }
    }
    const int m_tiles = (p.batch + BM - 1) / BM, n_tiles = (p.rows + kBN - 1) / kBN;
    gemm_mfma_kernel<MF><<<m_tiles * n_tiles * splits, kThreads, lds, s>>>(p.x, p.nz, p.sg, p.scales, p.y, p.batch, p.rows,
                                                                          p.cols, splits, partial, arrivals);
    return hipGetLastError();
}


template <int NF>
hipError_t launch_rowsplit(const Problem &p, const GemmConfig &c, float *partial, unsigned *arrivals, hipStream_t s) {
    constexpr int MF = 4, BM = 32 * MF, kNsThreads = 512 / NF;
    static std::mutex attr_mutex;
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    // loop: a ring of four activation chunks; afterwards the output tile, one padded row per activation row
    const size_t ring = 4 * (size_t)(4 * MF * 1024), out_tile = (size_t)BM * kNsPitch;
    const size_t lds = ring > out_tile ? ring : out_tile;
    if (dev >= 0 && dev < 64) {
        std::lock_guard<std::mutex> lock(attr_mutex);
        if (!attr_set[dev]) {
            if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_ns_kernel<MF, NF>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
                return e;
            attr_set[dev] = true;
        }
    }
    const int m_tiles = (p.batch + BM - 1) / BM, n_tiles = (p.rows + kNsBN - 1) / kNsBN;
    const int tiles = m_tiles * n_tiles;
    const int parts = (tiles - c.full_tiles) * c.splits;
    const int wgs = 8 * ((c.full_tiles + 7) / 8 + (parts + 7) / 8);
    // bytes an XCD fetches for its eighth of the tiles in either order: (activation tiles touched) x 128 rows of A +
    // (weight tiles touched) x 256 rows of masks and scales
    const long per = (tiles + 7) / 8;
    const double a_bytes = 128.0 * p.cols * 2, w_bytes = 256.0 * p.cols * 0.265625;
    auto touched = [](long per_, long inner, long outer) { return std::pair<long, long>(std::min(inner, per_), std::min(outer, (per_ + inner - 1) / inner + 1)); };
    const auto mf = touched(per, m_tiles, n_tiles);  // activation tiles fastest: (m touched, n touched)
    const auto nf = touched(per, n_tiles, m_tiles);  // weight tiles fastest: (n touched, m touched)
    // Only on a clear gain (1.5 x), and only while an XCD then works on at most 16 weight tiles at a time: a mask line
    // holds four blocks of a row and has to survive in the L2 until the workgroup comes back to it (with 56 weight tiles
    // side by side the gate/up shape at M = 2048 lost 6 %).
    const int n_fastest = nf.first <= 16 && 1.5 * (nf.second * a_bytes + nf.first * w_bytes) < mf.first * a_bytes + mf.second * w_bytes;
    gemm_ns_kernel<MF, NF><<<wgs, kNsThreads, lds, s>>>(p.x, p.nz, p.sg, p.scales, p.y, p.batch, p.rows, p.cols, c.full_tiles,
                                                    c.splits, n_fastest, partial, arrivals);
    return hipGetLastError();
}

}  // namespace

namespace {
// The four-wave kernel fetches scales as aligned dwords: the array must start on one and hold an even count.
bool scales_dword_aligned(const Problem &p) {
    return !(reinterpret_cast<uintptr_t>(p.scales) & 3) && !(((size_t)p.rows * (p.cols / 128)) & 1);
}
// The row-split kernel: K a multiple of 256, or of 128 from 384 on (the last block then holds 128 columns); mask rows and
// activations in 16-byte pieces. (Its scale loads may start on any halfword.)
bool rowsplit_ok(const Problem &p) {
    return (p.cols % 256 == 0 || (p.cols % 128 == 0 && p.cols >= 384)) &&
           !((reinterpret_cast<uintptr_t>(p.x) | reinterpret_cast<uintptr_t>(p.nz) | reinterpret_cast<uintptr_t>(p.sg)) & 15);
}
}  // namespace

bool gemm_mfma_supports(const Problem &p, int group) {
    if (!(group == 128 && p.batch >= 16 && p.cols % 128 == 0 && (size_t)p.rows * (p.cols / 32) < ((size_t)1 << 31) &&
          (size_t)p.batch * p.cols < ((size_t)1 << 31)))
        return false;
    // (a shape-only query, pointers null: the answer for aligned arrays)
    return scales_dword_aligned(p) || rowsplit_ok(p);
}

namespace {
// The row-split kernel's configuration for `tiles` tiles of 256 weight rows x 128 activation rows (of one matrix, or of
// several that share the activations) over `blocks` blocks of 256 columns.
GemmConfig rowsplit_config(int tiles, int blocks, int n_cu, size_t limit_floats, int forced_rs) {
    const float block_us = 3.3f, fixed_us = 9.0f;
    GemmConfig rs{0, 1, 0.f};
    rs.rowsplit = true;
    rs.full_tiles = tiles;
    rs.us = (float)((tiles + n_cu - 1) / n_cu) * (float)blocks * block_us + fixed_us;
    const int rem = tiles % n_cu;
    if (rem) {
        int splits = n_cu / rem;
        if (splits > 8) splits = 8;
        if (splits > blocks / 2) splits = blocks / 2;
        while (splits > 1 && (size_t)rem * splits * 128 * kNsBN > limit_floats) splits--;
        if (splits > 1) {
            const float exchange = 6.0f + 1.5f * (float)splits;
            // (a launch that leaves CUs idle runs its blocks and its exchange faster: down to 3/4 of the time)
            const float parts = (float)rem * (float)splits;
            const float thin = tiles < n_cu ? 0.75f + 0.25f * std::min(1.0f, parts / (float)n_cu) : 1.0f;
            const float us = (float)(tiles / n_cu) * (float)blocks * block_us +
                             thin * ((float)((blocks + splits - 1) / splits) * block_us + exchange + fixed_us);
            if (us < rs.us) {
                rs.splits = splits;
                rs.full_tiles = tiles - rem;
                rs.us = us;
            }
        }
    }
    // Two workgroups of four waves per CU: a workgroup alone on its CU takes 3.7 us per block, two together 5.3 us
    // each; pays when there are more tiles than CUs. (No K split in this form.) TLLM_GEMM_ROWSPLIT=2 forces it.
    if (tiles > n_cu || forced_rs == 2) {
        const int slots = 2 * n_cu, last = tiles % slots;
        GemmConfig two = rs;
        two.frags = 2;
        two.splits = 1;
        two.full_tiles = tiles;
        two.us = (float)(tiles / slots) * (float)blocks * 5.3f + (last > n_cu ? 5.3f : last > 0 ? 3.7f : 0.f) * (float)blocks + fixed_us;
        if (forced_rs == 2 || (forced_rs != 1 && two.us < rs.us)) rs = two;
    }
    return rs;
}

// One workgroup occupies a CU (LDS). Taller tiles do more per stage, shorter tiles fill the chip
// when there are few of them, and when even those leave CUs idle K is split across workgroups.
// Estimate: (rounds of workgroups over the CUs) x (stages per workgroup) x (time of one stage,
// measured: 1.19 / 0.70 us for 256 / 128 activation rows) + 5 us + the traffic of a split's exchange.
GemmConfig choose_config(const Problem &p, size_t limit_floats) {
    const int n_cu = current_device_cus();
    const int n_tiles = (p.rows + kBN - 1) / kBN, groups = p.cols / 128;
    const float stage_us[2] = {0.70f, 1.19f};
    GemmConfig best{0, 1, 0.f};
    for (int c = 0; c < 2; c++) {
        const int bm = 128 << c;
        const long tiles = (long)n_tiles * ((p.batch + bm - 1) / bm);
        for (int splits = 1; splits <= 8; splits *= 2) {
            if (splits > 1 && (tiles * splits > n_cu || groups / splits < 4)) break;  // only to fill idle CUs
            const GemmConfig cand{c, splits, 0.f};
            if (workspace_floats(p, cand) > limit_floats) break;
            const long wgs = tiles * splits;
            const float stages = (float)((groups + splits - 1) / splits * 2);
            // the exchange: all workgroups write their fp32 tile at once, then the last one of a tile reads the
            // `splits` slots on its own: 2 us + 0.7 us per slot + 25 ns per workgroup of the launch for 64 KB slots
            // (fitted to fifteen shapes between 100 x 2048 x 2048 and 512 x 8192 x 28672)
            const float exchange = splits > 1 ? (2.0f + 0.7f * (float)splits + 0.025f * (float)(tiles * splits)) * (float)(bm / 128) : 0.0f;
            const float us = (float)((wgs + n_cu - 1) / n_cu) * stages * stage_us[c] + 5.0f + exchange;
            if (best.us == 0.f || us < best.us) best = GemmConfig{c, splits, us};
        }
    }
    // The row-split kernel: 3.3 us per block of 256 columns (1490 - 1530 cycles per chunk of 64 at the 1.8 GHz the chip
    // holds under this load), 9 us of launch, first loads and stores. The tiles that do not fill the last round over the
    // CUs are split along K (at most as far as the CUs reach, two blocks per part at least, and while the slots fit the
    // workspace) when that is cheaper than a last round of whole tiles; an exchange costs about 6 us + 1.5 us per part
    // (fitted to 4096 x 14336 at M = 128 ... 512). Tiles are 128 activation rows high: not for fewer than 96.
    const int forced_rs = tuning().gemm_rowsplit.load(std::memory_order_relaxed);  // 0: never, 1 / 2: whenever the shape allows, in its eight-wave / four-wave form
    const bool rs_ok = rowsplit_ok(p), four_ok = scales_dword_aligned(p);
    // (a shape whose scales the four-wave kernel cannot fetch runs the row-split kernel whatever its size)
    if ((forced_rs != 0 || !four_ok) && rs_ok && (forced_rs >= 1 || p.batch >= 96 || !four_ok)) {
        const GemmConfig rs = rowsplit_config(((p.batch + 127) / 128) * ((p.rows + kNsBN - 1) / kNsBN), (p.cols + 255) / 256, n_cu, limit_floats, forced_rs);
        if (forced_rs >= 1 || !four_ok || rs.us < best.us) best = rs;
    }
    return best;
}
}  // namespace

// Configurations are chosen among those whose workspace fits the fixed array of the entry point that
// allocates nothing, so that both entry points run the same kernels on every shape.
float gemm_mfma_cost_us(const Problem &p) { return choose_config(p, kStaticSlotFloats).us; }

const char *gemm_mfma_kernel_name(const Problem &p) {
    const GemmConfig c = choose_config(p, kStaticSlotFloats);
    if (c.rowsplit && c.frags == 2) return "tllm::gemm_ns_kernel<4, 2>";
    if (c.rowsplit) return c.splits > 1 ? "tllm::gemm_ns_kernel<4, 1>, last tiles K split" : "tllm::gemm_ns_kernel<4, 1>";
    if (c.height == 1) return c.splits > 1 ? "tllm::gemm_mfma_kernel<2>, K split" : "tllm::gemm_mfma_kernel<2>";
    return c.splits > 1 ? "tllm::gemm_mfma_kernel<1>, K split" : "tllm::gemm_mfma_kernel<1>";
}

namespace {
hipError_t launch_config(const Problem &p, const GemmConfig &c, float *workspace, unsigned *arrivals, hipStream_t s) {
    if (c.rowsplit) return c.frags == 2 ? launch_rowsplit<2>(p, c, workspace, arrivals, s) : launch_rowsplit<1>(p, c, workspace, arrivals, s);
    return c.height == 1 ? launch<2>(p, c.splits, workspace, arrivals, s) : launch<1>(p, c.splits, workspace, arrivals, s);
}
}  // namespace

hipError_t split_exchange_memory(hipStream_t s, size_t floats, bool fixed, float **partial, unsigned **arrivals) {
    *partial = nullptr;
    *arrivals = nullptr;
    if (fixed) {
        if (floats > kStaticSlotFloats) return hipSuccess;
        unsigned char *base = nullptr;
        if (hipError_t e = static_scratch(&base)) return e;
        *arrivals = reinterpret_cast<unsigned *>(base);
        *partial = reinterpret_cast<float *>(base) + kArrivalSlots;
        return hipSuccess;
    }
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipError_t e = hipStreamIsCapturing(s, &cap)) return e;
    return split_workspace(s, floats, cap == hipStreamCaptureStatusNone, partial, arrivals);
}

hipError_t launch_gemm_mfma(const Problem &p, hipStream_t s) {
    GemmConfig c = choose_config(p, kStaticSlotFloats);
    float *workspace = nullptr;
    unsigned *arrivals = nullptr;
    if (const size_t need = workspace_floats(p, c)) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipError_t e = hipStreamIsCapturing(s, &cap)) return e;
        if (hipError_t e = split_workspace(s, need, cap == hipStreamCaptureStatusNone, &workspace, &arrivals)) return e;
        if (!workspace) c = choose_config(p, 0);  // under capture without a reserved workspace: what needs none
    }
    return launch_config(p, c, workspace, arrivals, s);
}

hipError_t gemm_mfma_reserve(const Problem &p, hipStream_t s) {
    const GemmConfig c = choose_config(p, kStaticSlotFloats);
    float *workspace = nullptr;
    unsigned *arrivals = nullptr;
    const size_t need = workspace_floats(p, c);
    return need ? split_workspace(s, need, true, &workspace, &arrivals) : hipSuccess;
}

void gemm_mfma_release_all() {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    int dev = 0;
    (void)hipGetDevice(&dev);
    for (SplitWorkspace &w : g_ws) {
        (void)hipSetDevice(w.device);
        if (w.arrivals) (void)hipFree(w.arrivals);  // the one allocation: counters, then slots
    }
    g_ws.clear();
    (void)hipSetDevice(dev);
}

// Several weight matrices on the same activations in one launch of the row-split kernel (its group form): the
// problems share x, batch and cols; each stores its own [batch, rows] output. `fixed`: the exchange of split tiles uses
// the library's fixed device array (the entry point that never allocates is not offered for groups: false everywhere).
bool gemm_group_supports(const Problem *ps, int count) {
    if (count < 1 || count > 4) return false;
    for (int i = 0; i < count; i++) {
        const Problem shape{nullptr, nullptr, nullptr, nullptr, nullptr, ps[i].rows, ps[i].cols, std::max(ps[i].batch, 16), 0};
        if (!gemm_mfma_supports(shape, 128) || !rowsplit_ok(ps[i])) return false;
        if (ps[i].x != ps[0].x || ps[i].batch != ps[0].batch || ps[i].cols != ps[0].cols) return false;
    }
    return true;
}
namespace {
template <int NF>
hipError_t launch_group_form(const GemmGroup &grp, const Problem &first, const GemmConfig &c, float *partial, unsigned *arrivals,
                             hipStream_t s) {
    constexpr int MF = 4, BM = 32 * MF, kNsThreads = 512 / NF;
    static std::mutex attr_mutex;
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    const size_t ring = 4 * (size_t)(4 * MF * 1024), out_tile = (size_t)BM * kNsPitch;
    const size_t lds = ring > out_tile ? ring : out_tile;
    if (dev >= 0 && dev < 64) {
        std::lock_guard<std::mutex> lock(attr_mutex);
        if (!attr_set[dev]) {
            if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_ns_kernel<MF, NF, false, true>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
                return e;
            attr_set[dev] = true;
        }
    }
    const int tiles = grp.prefix[grp.count];
    const int parts = (tiles - c.full_tiles) * c.splits;
    const int wgs = 8 * ((c.full_tiles + 7) / 8 + (parts + 7) / 8);
    // (consecutive tiles of a matrix walk its activation tiles first: the weight tile stays, the few activation tiles
    // of a prefill step are shared by everybody anyway)
    gemm_ns_kernel<MF, NF, false, true><<<wgs, kNsThreads, lds, s>>>(first.x, nullptr, nullptr, nullptr, nullptr, first.batch, 0,
                                                                      first.cols, c.full_tiles, c.splits, 0, partial, arrivals,
                                                                      nullptr, nullptr, nullptr, grp);
    return hipGetLastError();
}
}  // namespace
hipError_t launch_gemm_group(const Problem *ps, int count, hipStream_t s) {
    constexpr int BM = 128;
    GemmGroup grp{};
    grp.count = count;
    const int m_tiles = (ps[0].batch + BM - 1) / BM;
    for (int i = 0; i < count; i++) {
        grp.prefix[i + 1] = grp.prefix[i] + m_tiles * ((ps[i].rows + kNsBN - 1) / kNsBN);
        grp.N[i] = ps[i].rows;
        grp.nz[i] = ps[i].nz;
        grp.sg[i] = ps[i].sg;
        grp.sc[i] = ps[i].scales;
        grp.C[i] = ps[i].y;
    }
    for (int i = count; i < 4; i++) grp.prefix[i + 1] = grp.prefix[count];
    const int tiles = grp.prefix[count], blocks = (ps[0].cols + 255) / 256;
    const int forced = tuning().gemm_rowsplit.load(std::memory_order_relaxed);
    GemmConfig c = rowsplit_config(tiles, blocks, current_device_cus(), kStaticSlotFloats, forced > 0 ? forced : -1);
    float *workspace = nullptr;
    unsigned *arrivals = nullptr;
    if (c.splits > 1) {
        const size_t need = (size_t)(tiles - c.full_tiles) * c.splits * 128 * kNsBN;
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipError_t e = hipStreamIsCapturing(s, &cap)) return e;
        if (hipError_t e = split_workspace(s, need, cap == hipStreamCaptureStatusNone, &workspace, &arrivals)) return e;
        if (!workspace) {  // under capture without a reserved workspace: whole tiles only
            c.splits = 1;
            c.full_tiles = tiles;
        }
    }
    return c.frags == 2 ? launch_group_form<2>(grp, ps[0], c, workspace, arrivals, s) : launch_group_form<1>(grp, ps[0], c, workspace, arrivals, s);
}

// The prefill form of a SwiGLU pair: one launch of the row-split kernel in its pair form. `gate.y` receives
// fp16(silu(fp16 gate product) * fp16 up product) [batch, rows]; `up` has the gate's shape and activations.
bool gemm_swiglu_supports(const Problem &gate, const Problem &up) {
    return gemm_mfma_supports(Problem{nullptr, nullptr, nullptr, nullptr, nullptr, gate.rows, gate.cols, std::max(gate.batch, 16), 0}, 128) &&
           rowsplit_ok(gate) && rowsplit_ok(up);
}
hipError_t launch_gemm_swiglu(const Problem &gate, const Problem &up, hipStream_t s) {
    constexpr int MF = 4, BM = 32 * MF, kTileN = kNsBN / 2;
    static std::mutex attr_mutex;
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    const size_t ring = 4 * (size_t)(4 * MF * 1024), out_tile = (size_t)BM * kNsPitch;
    const size_t lds = ring > out_tile ? ring : out_tile;
    if (dev >= 0 && dev < 64) {
        std::lock_guard<std::mutex> lock(attr_mutex);
        if (!attr_set[dev]) {
            if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_ns_kernel<MF, 2, true>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
                return e;
            attr_set[dev] = true;
        }
    }
    const int m_tiles = (gate.batch + BM - 1) / BM, n_tiles = (gate.rows + kTileN - 1) / kTileN;
    const int tiles = m_tiles * n_tiles;
    const int wgs = 8 * ((tiles + 7) / 8);
    // (the order of the tiles inside an XCD's share: as for the single matrix, with 128 rows of two matrices per tile)
    const long per = (tiles + 7) / 8;
    const double a_bytes = 128.0 * gate.cols * 2, w_bytes = 256.0 * gate.cols * 0.265625;
    auto touched = [](long per_, long inner, long outer) { return std::pair<long, long>(std::min(inner, per_), std::min(outer, (per_ + inner - 1) / inner + 1)); };
    const auto mf = touched(per, m_tiles, n_tiles);
    const auto nf = touched(per, n_tiles, m_tiles);
    const int n_fastest = nf.first <= 16 && 1.5 * (nf.second * a_bytes + nf.first * w_bytes) < mf.first * a_bytes + mf.second * w_bytes;
    gemm_ns_kernel<MF, 2, true><<<wgs, 256, lds, s>>>(gate.x, gate.nz, gate.sg, gate.scales, gate.y, gate.batch, gate.rows, gate.cols,
                                                      tiles, 1, n_fastest, nullptr, nullptr, up.nz, up.sg, up.scales);
    return hipGetLastError();
}

bool gemm_mfma_static_fits(const Problem &p) { return workspace_floats(p, choose_config(p, kStaticSlotFloats)) <= kStaticSlotFloats; }

hipError_t launch_gemm_mfma_static(const Problem &p, hipStream_t s) {
    const GemmConfig c = choose_config(p, kStaticSlotFloats);
    float *workspace = nullptr;
    unsigned *arrivals = nullptr;
    if (workspace_floats(p, c)) {
        unsigned char *base = nullptr;
        if (hipError_t e = static_scratch(&base)) return e;
        arrivals = reinterpret_cast<unsigned *>(base);
        workspace = reinterpret_cast<float *>(base) + kArrivalSlots;
    }
    return launch_config(p, c, workspace, arrivals, s);
}

}  // namespace tllm
