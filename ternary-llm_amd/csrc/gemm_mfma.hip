// Prefill GEMM on the matrix cores (gfx950), group size 128, M >= 16.
//
// Arithmetic (reference kernels/ternary_gemm.cu:106-175): C[m,n] = sum_k scale[n, k/128] * w[n,k] * A[m,k],
// the scale multiplied into every element, fp32 accumulation, fp16 store (round to nearest even).
// Here the product scale * w is formed exactly in fp16 (w in {-1,0,+1}), so the only difference to
// the reference is the order of the fp32 additions.
//
// Tiling. A workgroup (4 waves, 2 x 2) computes BM activation rows x 128 weight rows. Per stage of
// 64 columns of K:
//   * activations: BM x 64 fp16 come from global memory into registers, are re-paired so that dword
//     u of every 32-column block holds columns (u, u+16), and go to LDS;
//   * weights: each thread decodes one 32-bit mask word pair of one weight row. One v_bitop3 puts the
//     2-bit field (negative, non-zero) of every even/odd weight in place; shifted to the top of an
//     fp16 half that field IS the number 0, +2.0 or -2.0 (bit 15 = sign, bit 14 = exponent MSB), so
//     a packed shift, an AND and a packed fp16 multiply by the group scale give two elements
//     +-2*scale: 1.6 vector operations per weight, once per workgroup. The factor 2 is undone on
//     the fp32 accumulators at the end (exact);
//   * each wave multiplies its 64 weight rows x BM/2 activation rows with v_mfma_f32_16x16x32_f16,
//     operands read from LDS as 16-byte chunks (XOR-swizzled by row against bank conflicts).
// Global loads for the next stage are issued before the MFMAs of the current one; LDS is double
// buffered, one barrier per stage.
#include "common.h"

namespace tllm {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef uint16_t us2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const u4 GU4;
typedef __attribute__((address_space(1))) const uint32_t GU32;
typedef __attribute__((address_space(1))) const uint16_t GU16;

constexpr int kBN = 128;     // weight rows per workgroup
constexpr int kBK = 64;      // K columns per stage (two MFMA steps of 32)
constexpr int kThreads = 256;
constexpr int kRowBytes = kBK * 2;  // one LDS row: 64 fp16 = 8 chunks of 16 bytes

// byte offset of 16-byte chunk c (0..7) of row r inside a [rows][64] fp16 LDS tile
__device__ __forceinline__ int chunk_off(int r, int c) { return r * kRowBytes + ((c ^ (r & 7)) << 4); }

// 32 weights (one mask word pair) -> 16 dwords; dword u holds weights (u, u + 16) as +-2*scale / 0.
__device__ __forceinline__ void decode_scaled(uint32_t nz, uint32_t sg, uint32_t scale_pair, uint32_t out[16]) {
    const uint32_t neg = nz & ~sg;
    uint32_t q[2];
    // field (negative, non-zero) of weight 2f+z at bits (2f+1, 2f) of q[z]:  (a & c) | (b & ~c), c = 0xAAAAAAAA
    q[0] = __builtin_amdgcn_bitop3_b32(neg << 1, nz, 0xAAAAAAAAu, 0xE4);
    q[1] = __builtin_amdgcn_bitop3_b32(neg, nz >> 1, 0xAAAAAAAAu, 0xE4);
    const h2 sp = __builtin_bit_cast(h2, scale_pair);
#pragma unroll
    for (int z = 0; z < 2; z++) {
#pragma unroll
        for (int f = 0; f < 8; f++) {
            us2 v = __builtin_bit_cast(us2, q[z]);
            v = v << (uint16_t)(14 - 2 * f);  // both halves: field f (and f + 8) to bits 15:14
            const uint32_t top = __builtin_bit_cast(uint32_t, v) & 0xC000C000u;  // 0, +2.0 or -2.0
            out[2 * f + z] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, top) * sp);
        }
    }
}

template <int BM>
__global__ __launch_bounds__(kThreads, 1) void gemm_mfma_kernel(
    const uint16_t *__restrict__ A, const uint32_t *__restrict__ nzB, const uint32_t *__restrict__ sgB,
    const uint16_t *__restrict__ scB, uint16_t *__restrict__ C, int M, int N, int K) {
    constexpr int kWM = BM / 2;          // activation rows per wave
    constexpr int kMF = kWM / 16;        // MFMA column fragments per wave
    constexpr int kNF = 4;               // MFMA row fragments per wave (64 weight rows)
    constexpr int kAUnits = BM * 4 / kThreads;  // (row, k-unit) pairs of the activation tile per thread
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    constexpr int kABytes = BM * kRowBytes, kWBytes = kBN * kRowBytes;
    // buffer b: activations at b * (kABytes + kWBytes), weights right behind them

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;
    const int wn = wave & 1, wm = wave >> 1;  // wave position: weight-row half, activation-row half

    // tile coordinates: consecutive workgroups share the weight tile (same n0), so it stays in L2
    const int m_tiles = (M + BM - 1) / BM;
    const int n0 = (blockIdx.x / m_tiles) * kBN;
    const int m0 = (blockIdx.x % m_tiles) * BM;
    const int words = K / 32, groups = K / 128;

    // ---- what this thread stages per 64-column stage
    // activations: unit (row r, u4 pair p): global chunks (p&1) + 4*(p>>1) and that + 2 of row r
    //   p = 0: columns 0-7 & 16-23 -> LDS chunks 0,1;  p = 1: 8-15 & 24-31 -> chunks 2,3;  p = 2,3: same in the second 32
    int a_row[kAUnits], a_p[kAUnits];
    const GU4 *a_src[kAUnits];
    bool a_ok[kAUnits];
#pragma unroll
    for (int i = 0; i < kAUnits; i++) {
        const int unit = tid + i * kThreads;
        a_row[i] = unit >> 2;
        a_p[i] = unit & 3;
        const int gm = m0 + a_row[i];
        a_ok[i] = gm < M;
        const int col = (a_p[i] >> 1) * 32 + (a_p[i] & 1) * 8;
        a_src[i] = reinterpret_cast<const GU4 *>((__attribute__((address_space(1))) const uint16_t *)A +
                                                 (size_t)(a_ok[i] ? gm : 0) * K + col);
    }
    // weights: row w_row, 32-column word w_word of the stage
    const int w_row = tid >> 1, w_word = tid & 1;
    const int gn = min(n0 + w_row, N - 1);
    const GU32 *nz_src = (GU32 *)nzB + (size_t)gn * words + w_word;
    const GU32 *sg_src = (GU32 *)sgB + (size_t)gn * words + w_word;
    const GU16 *sc_src = (GU16 *)scB + (size_t)gn * groups;

    u4 a_lo[kAUnits], a_hi[kAUnits];
    uint32_t w_nz, w_sg, w_sc;
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < kAUnits; i++) {
            const u4 z = {0u, 0u, 0u, 0u};
            a_lo[i] = a_ok[i] ? a_src[i][k0 / 8] : z;
            a_hi[i] = a_ok[i] ? a_src[i][k0 / 8 + 2] : z;
        }
        w_nz = nz_src[k0 / 32];
        w_sg = sg_src[k0 / 32];
        w_sc = sc_src[(k0 + 32 * w_word) / 128];
    };
    auto stage = [&](int buf) {
        unsigned char *As = lds + buf * (kABytes + kWBytes);
        unsigned char *Ws = As + kABytes;
#pragma unroll
        for (int i = 0; i < kAUnits; i++) {
            // dwords (a[u], a[u+16]): low halves of (lo, hi) -> even u, high halves -> odd u
            uint32_t o[8];
#pragma unroll
            for (int d = 0; d < 4; d++) {
                o[2 * d] = __builtin_amdgcn_perm(a_hi[i][d], a_lo[i][d], 0x05040100u);
                o[2 * d + 1] = __builtin_amdgcn_perm(a_hi[i][d], a_lo[i][d], 0x07060302u);
            }
            const int c = (a_p[i] >> 1) * 4 + (a_p[i] & 1) * 2;
            *reinterpret_cast<u4 *>(As + chunk_off(a_row[i], c)) = u4{o[0], o[1], o[2], o[3]};
            *reinterpret_cast<u4 *>(As + chunk_off(a_row[i], c + 1)) = u4{o[4], o[5], o[6], o[7]};
        }
        uint32_t o[16];
        decode_scaled(w_nz, w_sg, w_sc | (w_sc << 16), o);
#pragma unroll
        for (int c = 0; c < 4; c++)
            *reinterpret_cast<u4 *>(Ws + chunk_off(w_row, w_word * 4 + c)) =
                u4{o[4 * c], o[4 * c + 1], o[4 * c + 2], o[4 * c + 3]};
    };

    f4 acc[kNF][kMF];
#pragma unroll
    for (int i = 0; i < kNF; i++)
#pragma unroll
        for (int j = 0; j < kMF; j++) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};

    fetch(0);
    stage(0);
    __syncthreads();
    const int stages = K / kBK;
    for (int s = 0; s < stages; s++) {
        const int buf = s & 1;
        if (s + 1 < stages) fetch((s + 1) * kBK);
        const unsigned char *As = lds + buf * (kABytes + kWBytes);
        const unsigned char *Ws = As + kABytes;
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            u4 af[kNF], bf[kMF];
#pragma unroll
            for (int i = 0; i < kNF; i++)
                af[i] = *reinterpret_cast<const u4 *>(Ws + chunk_off(wn * 64 + i * 16 + li, ks * 4 + lq));
#pragma unroll
            for (int j = 0; j < kMF; j++)
                bf[j] = *reinterpret_cast<const u4 *>(As + chunk_off(wm * kWM + j * 16 + li, ks * 4 + lq));
#pragma unroll
            for (int i = 0; i < kNF; i++)
#pragma unroll
                for (int j = 0; j < kMF; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, af[i]),
                                                                       __builtin_bit_cast(h8, bf[j]),
                                                                       acc[i][j], 0, 0, 0);
        }
        if (s + 1 < stages) stage(buf ^ 1);
        __syncthreads();
    }

    // ---- store: lane (lq, li) of fragment (i, j) holds weight rows n .. n+3 for activation row m
    uint16_t *Cg = C;
    const bool vec_store = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 7) == 0;
#pragma unroll
    for (int j = 0; j < kMF; j++) {
        const int m = m0 + wm * kWM + j * 16 + li;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < kNF; i++) {
            const int n = n0 + wn * 64 + i * 16 + 4 * lq;
            uint16_t h[4];
#pragma unroll
            for (int v = 0; v < 4; v++) h[v] = f2h(acc[i][j][v] * 0.5f);
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

template <int BM>
hipError_t launch(const Problem &p, hipStream_t s) {
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    const size_t lds = 2 * (size_t)(BM + kBN) * kRowBytes;
    if (dev >= 0 && dev < 64 && !attr_set[dev]) {
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_kernel<BM>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
            return e;
        attr_set[dev] = true;
    }
    const int m_tiles = (p.batch + BM - 1) / BM, n_tiles = (p.rows + kBN - 1) / kBN;
    gemm_mfma_kernel<BM><<<m_tiles * n_tiles, kThreads, lds, s>>>(p.x, p.nz, p.sg, p.scales, p.y, p.batch,
                                                                  p.rows, p.cols);
    return hipGetLastError();
}

}  // namespace

bool gemm_mfma_supports(const Problem &p, int group) {
    return group == 128 && p.batch >= 16 && p.cols % 128 == 0 && (size_t)p.rows * (p.cols / 32) < ((size_t)1 << 31) &&
           (size_t)p.batch * p.cols < ((size_t)1 << 31);
}

hipError_t launch_gemm_mfma(const Problem &p, hipStream_t s) {
    return p.batch > 128 ? launch<256>(p, s) : launch<128>(p, s);
}

}  // namespace tllm
