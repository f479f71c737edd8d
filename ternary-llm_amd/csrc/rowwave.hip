// General-shape kernels: one 64-lane wave per output row, branch-free per-bit select.
// These accept every group size that is a multiple of 32; the 128-group fast paths live
// in their own files. Arithmetic follows the reference operators:
//   fp16 GEMV ......... kernels/ternary_gemv.cu:47-86   (fp32 group sum, then fp32 scale)
//   int8 GEMV ......... kernels/ternary_gemv.cu:148-198 (exact int group sum, fp32 scale)
//   absmax quantise ... kernels/activations.cu:100-141
#include "common.h"

namespace tllm {

namespace {

constexpr int kRowsPerBlock = 4;

__device__ __forceinline__ void gemv_rowwave_f16_body(const Problem &p, int group, int row, int b) {
    const int lane = threadIdx.x & (kWave - 1);
    if (row >= p.rows || b >= p.batch) return;
    const int words = p.cols / 32;
    const int groups = p.cols / group;
    const int words_per_group = group / 32;
    const uint32_t *nz = p.nz + (size_t)row * words;
    const uint32_t *sg = p.sg + (size_t)row * words;
    const uint16_t *sc = p.scales + (size_t)row * groups;
    const uint16_t *x = p.x + (size_t)b * p.cols;

    float acc = 0.0f;
    for (int j = lane; j < groups * words_per_group; j += kWave) {
        const uint32_t n = nz[j];
        const uint32_t pos = n & sg[j];
        const uint4 *xv = reinterpret_cast<const uint4 *>(x + 32 * j);  // 64 B aligned
        float part = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint4 v = xv[q];
            const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int bit = q * 8 + e;
                const float xf = h2f((uint16_t)(w4[e >> 1] >> (16 * (e & 1))));
                const float mag = ((n >> bit) & 1u) ? xf : 0.0f;
                part += ((pos >> bit) & 1u) ? mag : -mag;
            }
        }
        acc += h2f(sc[j / words_per_group]) * part;
    }
    acc = wave_sum(acc);
    if (lane == 0) p.y[(size_t)b * p.rows + row] = f2h(acc);
}

__global__ __launch_bounds__(kRowsPerBlock *kWave) void gemv_rowwave_f16_kernel(Problem p, int group) {
    gemv_rowwave_f16_body(p, group, blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6), blockIdx.y);
}

// blockIdx.y walks the problem table, blockIdx.z the batch; surplus blocks exit at once.
__global__ __launch_bounds__(kRowsPerBlock *kWave) void gemv_rowwave_f16_table_kernel(
    const Problem *__restrict__ table, int group) {
    const Problem p = table[blockIdx.y];
    gemv_rowwave_f16_body(p, group, blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6), blockIdx.z);
}

__global__ __launch_bounds__(kRowsPerBlock *kWave) void gemv_rowwave_i8_kernel(
    const uint32_t *__restrict__ nzp, const uint32_t *__restrict__ sgp,
    const uint16_t *__restrict__ scales, const int8_t *__restrict__ xq, float scale_value,
    const float *__restrict__ scale_dev, uint16_t *__restrict__ y, int rows, int cols, int group) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int words = cols / 32;
    const int groups = cols / group;
    const int words_per_group = group / 32;
    const uint32_t *nz = nzp + (size_t)row * words;
    const uint32_t *sg = sgp + (size_t)row * words;
    const uint16_t *sc = scales + (size_t)row * groups;

    float acc = 0.0f;
    for (int j = lane; j < groups * words_per_group; j += kWave) {
        const uint32_t n = nz[j];
        const uint32_t pos = n & sg[j];
        const uint4 *xv = reinterpret_cast<const uint4 *>(xq + 32 * j);  // 32 B aligned
        int part = 0;
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const uint4 v = xv[q];
            const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int bit = q * 16 + e;
                const int xi = (int)(int8_t)(w4[e >> 2] >> (8 * (e & 3)));
                const int mag = ((n >> bit) & 1u) ? xi : 0;
                part += ((pos >> bit) & 1u) ? mag : -mag;
            }
        }
        acc += h2f(sc[j / words_per_group]) * (float)part;
    }
    acc = wave_sum(acc);
    const float in_scale = scale_dev ? *scale_dev : scale_value;
    if (lane == 0) y[row] = f2h(acc * in_scale);
}

// quantize_absmax_int8 + ternary_gemv_int8 in one launch, any group size: every block first finds the largest
// magnitude of x (as the quantiser does, reference kernels/activations.cu:100-141), then each wave walks its row
// with the integers the quantisation gives (exact int32 group sums, fp32 scales, kernels/ternary_gemv.cu:148-198).
__global__ __launch_bounds__(kRowsPerBlock *kWave) void gemv_rowwave_q8_kernel(Problem p, int group) {
    __shared__ float wave_max[kRowsPerBlock];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    float m = 0.0f;
    for (int i = threadIdx.x; i < p.cols; i += kRowsPerBlock * kWave) m = fmaxf(m, fabsf(h2f(p.x[i])));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, kWave));
    if (lane == 0) wave_max[wave] = m;
    __syncthreads();
    float amax = 0.0f;
#pragma unroll
    for (int w = 0; w < kRowsPerBlock; w++) amax = fmaxf(amax, wave_max[w]);
    const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    const float in_scale = amax > 0.0f ? amax / 127.0f : 1.0f;
    const int row = blockIdx.x * kRowsPerBlock + wave;
    if (row >= p.rows) return;
    const int words = p.cols / 32;
    const int groups = p.cols / group;
    const int words_per_group = group / 32;
    const uint32_t *nz = p.nz + (size_t)row * words;
    const uint32_t *sg = p.sg + (size_t)row * words;
    const uint16_t *sc = p.scales + (size_t)row * groups;
    float acc = 0.0f;
    // (word by word, like gemv_rowwave_i8_kernel: the two give the same bits)
    for (int j = lane; j < groups * words_per_group; j += kWave) {
        const uint32_t n = nz[j];
        const uint32_t pos = n & sg[j];
        int part = 0;
        for (int bit = 0; bit < 32; bit++) {
            int xi = (int)rintf(h2f(p.x[32 * j + bit]) * inv);
            xi = max(-127, min(127, xi));
            const int mag = ((n >> bit) & 1u) ? xi : 0;
            part += ((pos >> bit) & 1u) ? mag : -mag;
        }
        acc += h2f(sc[j / words_per_group]) * (float)part;
    }
    acc = wave_sum(acc);
    if (lane == 0) p.y[row] = f2h(acc * in_scale);
}

constexpr int kQuantThreads = 1024;

__global__ __launch_bounds__(kQuantThreads) void quantize_absmax_i8_kernel(
    const uint16_t *__restrict__ x, int8_t *__restrict__ q, float *__restrict__ scale, int n) {
    __shared__ float wave_max[kQuantThreads / kWave];
    __shared__ float block_max;
    const int tid = threadIdx.x;
    float m = 0.0f;
    for (int i = tid; i < n; i += kQuantThreads) m = fmaxf(m, fabsf(h2f(x[i])));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, kWave));
    if ((tid & (kWave - 1)) == 0) wave_max[tid >> 6] = m;
    __syncthreads();
    if (tid == 0) {
        float t = 0.0f;
        for (int i = 0; i < kQuantThreads / kWave; i++) t = fmaxf(t, wave_max[i]);
        block_max = t;
        *scale = t > 0.0f ? t / 127.0f : 1.0f;
    }
    __syncthreads();
    const float amax = block_max;
    const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    for (int i = tid; i < n; i += kQuantThreads) {
        int r = (int)rintf(h2f(x[i]) * inv);
        r = max(-127, min(127, r));
        q[i] = (int8_t)r;
    }
}

// The same for vectors that fit the registers of one block (n <= 8192 * kPieces, a multiple of 8, aligned pointers):
// one pass over x, 16-byte loads, 8-byte stores. Same arithmetic, same bits.
template <int kPieces>
__global__ __launch_bounds__(kQuantThreads) void quantize_absmax_i8_regs_kernel(
    const uint4 *__restrict__ x, uint2 *__restrict__ q, float *__restrict__ scale, int n8) {
    __shared__ float wave_max[kQuantThreads / kWave];
    const int tid = threadIdx.x;
    uint4 v[kPieces];
    float m = 0.0f;
#pragma unroll
    for (int k = 0; k < kPieces; k++) {
        const int c = tid + k * kQuantThreads;
        v[k] = c < n8 ? x[c] : uint4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int k = 0; k < kPieces; k++) {
        const uint32_t w4[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            m = fmaxf(m, fabsf(h2f((uint16_t)w4[e])));
            m = fmaxf(m, fabsf(h2f((uint16_t)(w4[e] >> 16))));
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, kWave));
    if ((tid & (kWave - 1)) == 0) wave_max[tid >> 6] = m;
    __syncthreads();
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < kQuantThreads / kWave; i++) amax = fmaxf(amax, wave_max[i]);
    if (tid == 0) *scale = amax > 0.0f ? amax / 127.0f : 1.0f;
    const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
#pragma unroll
    for (int k = 0; k < kPieces; k++) {
        const int c = tid + k * kQuantThreads;
        if (c >= n8) continue;
        const uint32_t w4[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
        uint32_t out[2] = {0u, 0u};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            int r = (int)rintf(h2f((uint16_t)(w4[e >> 1] >> (16 * (e & 1)))) * inv);
            r = max(-127, min(127, r));
            out[e >> 2] |= (uint32_t)(r & 0xFF) << (8 * (e & 3));
        }
        q[c] = uint2{out[0], out[1]};
    }
}

}  // namespace

hipError_t launch_gemv_rowwave_f16(const Problem &p, int group, hipStream_t s) {
    dim3 grid((p.rows + kRowsPerBlock - 1) / kRowsPerBlock, p.batch);
    gemv_rowwave_f16_kernel<<<grid, kRowsPerBlock * kWave, 0, s>>>(p, group);
    return hipGetLastError();
}

hipError_t launch_gemv_rowwave_f16_table(const Problem *table, int count, int max_rows,
                                         int max_batch, int group, hipStream_t s) {
    dim3 grid((max_rows + kRowsPerBlock - 1) / kRowsPerBlock, count, max_batch);
    gemv_rowwave_f16_table_kernel<<<grid, kRowsPerBlock * kWave, 0, s>>>(table, group);
    return hipGetLastError();
}

hipError_t launch_gemv_rowwave_i8(const uint32_t *nz, const uint32_t *sg, const uint16_t *scales,
                                  const int8_t *xq, float scale_value, const float *scale_dev,
                                  uint16_t *y, int rows, int cols, int group, hipStream_t s) {
    dim3 grid((rows + kRowsPerBlock - 1) / kRowsPerBlock);
    gemv_rowwave_i8_kernel<<<grid, kRowsPerBlock * kWave, 0, s>>>(nz, sg, scales, xq, scale_value,
                                                                 scale_dev, y, rows, cols, group);
    return hipGetLastError();
}

hipError_t launch_gemv_rowwave_q8(const Problem &p, int group, hipStream_t s) {
    dim3 grid((p.rows + kRowsPerBlock - 1) / kRowsPerBlock);
    gemv_rowwave_q8_kernel<<<grid, kRowsPerBlock * kWave, 0, s>>>(p, group);
    return hipGetLastError();
}

hipError_t launch_quantize_absmax_i8(const uint16_t *x, int8_t *q, float *scale, int n,
                                     hipStream_t s) {
    const bool regs = n % 8 == 0 && n <= 8192 * 4 && !(reinterpret_cast<uintptr_t>(x) & 15) && !(reinterpret_cast<uintptr_t>(q) & 7);
    const uint4 *x4 = reinterpret_cast<const uint4 *>(x);
    uint2 *q2 = reinterpret_cast<uint2 *>(q);
    if (regs && n <= 8192) quantize_absmax_i8_regs_kernel<1><<<1, kQuantThreads, 0, s>>>(x4, q2, scale, n / 8);
    else if (regs && n <= 16384) quantize_absmax_i8_regs_kernel<2><<<1, kQuantThreads, 0, s>>>(x4, q2, scale, n / 8);
    else if (regs) quantize_absmax_i8_regs_kernel<4><<<1, kQuantThreads, 0, s>>>(x4, q2, scale, n / 8);
    else quantize_absmax_i8_kernel<<<1, kQuantThreads, 0, s>>>(x, q, scale, n);
    return hipGetLastError();
}

}  // namespace tllm
