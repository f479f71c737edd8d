// Prefill GEMM on the matrix cores (gfx950), group size 128, M >= 16.
//
// Arithmetic (reference kernels/ternary_gemm.cu:106-175): C[m,n] = sum_k scale[n, k/128] * w[n,k] * A[m,k],
// the scale multiplied into every element, fp32 accumulation, fp16 store (round to nearest even).
// Here the product scale * w is formed exactly in fp16 (w in {-1,0,+1}), so the only difference to
// the reference is the order of the fp32 additions.
//
// Tiling. A workgroup (4 waves, one per SIMD) computes 128 weight rows x BM activation rows; every wave
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

// ---- split-K exchange memory: fp32 slots and one arrival counter per tile.
//
// Ordinary calls use a workspace per (device, stream), created by tllm_gemm_workspace_reserve or by the
// first call that needs it and grown on demand; calls on one stream run in order and so may share it.
// Nothing is allocated, freed or synchronised while the stream is being captured into a graph: a call
// that would have to falls back to one workgroup per tile (no exchange).
struct SplitWorkspace {
    int device = -1;
    hipStream_t stream = nullptr;
    float *partial = nullptr;
    size_t floats = 0;
    unsigned *arrivals = nullptr;
};
constexpr size_t kArrivalSlots = 1024;  // tiles of a split launch (at most one per CU pair)
std::mutex g_ws_mutex;
std::vector<SplitWorkspace> g_ws;

__global__ void clear_arrivals_kernel(unsigned *arrivals, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) arrivals[i] = 0u;
}

// may_allocate = false: only hands out what exists. *partial stays null when the workspace is too small.
hipError_t split_workspace(hipStream_t s, size_t floats, bool may_allocate, float **partial, unsigned **arrivals) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    SplitWorkspace *w = nullptr;
    for (SplitWorkspace &c : g_ws)
        if (c.device == dev && c.stream == s) w = &c;
    if ((!w || w->floats < floats) && !may_allocate) return hipSuccess;
    if (!w) {
        g_ws.push_back(SplitWorkspace{});
        w = &g_ws.back();
        w->device = dev;
        w->stream = s;
    }
    if (w->floats < floats) {
        if (hipError_t e = hipStreamSynchronize(s)) return e;  // earlier launches may still use the old buffers
        if (w->partial) (void)hipFree(w->partial);
        w->partial = nullptr;
        w->floats = 0;
        if (hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->partial), floats * sizeof(float))) return e;
        w->floats = floats;
        if (!w->arrivals) {
            if (hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->arrivals), kArrivalSlots * sizeof(unsigned))) return e;
            // cleared once, in stream order; every launch leaves the counters at zero again
            clear_arrivals_kernel<<<(int)(kArrivalSlots / 256), 256, 0, s>>>(w->arrivals, (int)kArrivalSlots);
            if (hipError_t e = hipGetLastError()) return e;
        }
    }
    *partial = w->partial;
    *arrivals = w->arrivals;
    return hipSuccess;
}

// The exchange memory of tllm_ternary_gemm_f16_static: a fixed array in device memory, one copy per GPU,
// held until the process ends. Arrival counters first (zero when the module is loaded, left at zero by
// every launch), then the fp32 slots.
constexpr size_t kStaticSlotFloats = (size_t)TLLM_GEMM_STATIC_SCRATCH_BYTES / 4 - kArrivalSlots;
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
    int height;  // 0: 128 activation rows per workgroup, 1: 256
    int splits;  // workgroups per tile along K
    float us;    // estimated time
};
GemmConfig choose_config(const Problem &p);

size_t split_floats(const Problem &p, const GemmConfig &c) {
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

}  // namespace

bool gemm_mfma_supports(const Problem &p, int group) {
    // scales are fetched as aligned dwords: the array must start on one and hold an even count
    if ((reinterpret_cast<uintptr_t>(p.scales) & 3) || (((size_t)p.rows * (p.cols / 128)) & 1)) return false;
    return group == 128 && p.batch >= 16 && p.cols % 128 == 0 && (size_t)p.rows * (p.cols / 32) < ((size_t)1 << 31) &&
           (size_t)p.batch * p.cols < ((size_t)1 << 31);
}

namespace {
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
    GemmConfig c = choose_config(p);
    float *partial = nullptr;
    unsigned *arrivals = nullptr;
    if (c.splits > 1) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipError_t e = hipStreamIsCapturing(s, &cap)) return e;
        if (hipError_t e = split_workspace(s, split_floats(p, c), cap == hipStreamCaptureStatusNone, &partial, &arrivals)) return e;
        if (!partial) c.splits = 1;  // under capture without a reserved workspace: one workgroup per tile
    }
    return c.height == 1 ? launch<2>(p, c.splits, partial, arrivals, s) : launch<1>(p, c.splits, partial, arrivals, s);
}

hipError_t gemm_mfma_reserve(const Problem &p, hipStream_t s) {
    const GemmConfig c = choose_config(p);
    float *partial = nullptr;
    unsigned *arrivals = nullptr;
    return c.splits > 1 ? split_workspace(s, split_floats(p, c), true, &partial, &arrivals) : hipSuccess;
}

void gemm_mfma_release_all() {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    int dev = 0;
    (void)hipGetDevice(&dev);
    for (SplitWorkspace &w : g_ws) {
        (void)hipSetDevice(w.device);
        if (w.partial) (void)hipFree(w.partial);
        if (w.arrivals) (void)hipFree(w.arrivals);
    }
    g_ws.clear();
    (void)hipSetDevice(dev);
}

bool gemm_mfma_static_fits(const Problem &p) { return split_floats(p, choose_config(p)) <= kStaticSlotFloats; }

hipError_t launch_gemm_mfma_static(const Problem &p, hipStream_t s) {
    const GemmConfig c = choose_config(p);
    float *partial = nullptr;
    unsigned *arrivals = nullptr;
    if (c.splits > 1) {
        unsigned char *base = nullptr;
        if (hipError_t e = static_scratch(&base)) return e;
        arrivals = reinterpret_cast<unsigned *>(base);
        partial = reinterpret_cast<float *>(base) + kArrivalSlots;
    }
    return c.height == 1 ? launch<2>(p, c.splits, partial, arrivals, s) : launch<1>(p, c.splits, partial, arrivals, s);
}

}  // namespace tllm
