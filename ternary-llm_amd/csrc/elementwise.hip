// The decode-step element-wise operators around the ternary linears: RMSNorm (with the optional
// fused residual add) in front of every projection group, SiLU(gate) * up between the FFN
// projections, the residual add, rotary position embedding of q and k, the embedding row lookup and
// the copy of new k/v rows into the cache. All are bandwidth-trivial (a few KB per token); fp16 in
// and out, arithmetic as the reference's kernels unless a comment says otherwise.
#include <cstdio>
#include <cstdlib>

#include "common.h"

namespace tllm {
namespace {

constexpr int kNormThreads = 256;

// Reference kernels/rmsnorm.cu:20-106. One workgroup per token row. With a residual the sum
// t = x + r is formed in fp32; the mean square uses that fp32 value, while the normalised output is
// computed from the fp16-rounded t when it is also stored to residual_out (the reference re-reads
// what it stored), else from the fp32 t. Every element is read and written by the same lane in both
// passes, so output may be input and residual_out may be residual.
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(const uint16_t *input, const uint16_t *__restrict__ weight,
                                                               uint16_t *output, const uint16_t *residual,
                                                               uint16_t *residual_out, int dim, float eps) {
    __shared__ float partial[kNormThreads / kWave];
    const size_t row = (size_t)blockIdx.x * dim;
    const uint16_t *x = input + row, *r = residual ? residual + row : nullptr;
    uint16_t *ro = residual_out ? residual_out + row : nullptr;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < dim; i += kNormThreads) {
        float v = h2f(x[i]);
        if (r) {
            v += h2f(r[i]);
            if (ro) ro[i] = f2h(v);
        }
        ss += v * v;
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & (kWave - 1)) == 0) partial[threadIdx.x / kWave] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kNormThreads / kWave; w++) total += partial[w];
    const float inv = 1.0f / sqrtf(total / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += kNormThreads) {
        float v;
        if (r) v = ro ? h2f(ro[i]) : h2f(x[i]) + h2f(r[i]);
        else v = h2f(x[i]);
        output[row + i] = f2h_of_rounded(v * inv * h2f(weight[i]));
    }
}

// The same operator for rows of up to 2048 * kChunks elements (kChunks 1, 2, 4, 8) whose pointers are 16-byte aligned and
// whose length is a multiple of 8: every lane keeps its 8-element chunks in registers between the
// two passes, so the row is read once, through 16-byte loads.
template <int kChunks>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_rows_kernel(const uint16_t *input,
                                                                    const uint16_t *__restrict__ weight,
                                                                    uint16_t *output, const uint16_t *residual,
                                                                    uint16_t *residual_out, int dim, float eps) {
    __shared__ float partial[kNormThreads / kWave];
    const size_t row = (size_t)blockIdx.x * dim;
    const int chunks = dim >> 3;
    float v[kChunks][8];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < kChunks; c++) {
        const int chunk = c * kNormThreads + threadIdx.x;
        if (chunk >= chunks) break;
        const size_t at = row + (size_t)chunk * 8;
        const uint4 xq = *(const uint4 *)(input + at);
        const uint32_t xw[4] = {xq.x, xq.y, xq.z, xq.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[c][2 * j] = h2f((uint16_t)xw[j]);
            v[c][2 * j + 1] = h2f((uint16_t)(xw[j] >> 16));
        }
        if (residual) {
            const uint4 rq = *(const uint4 *)(residual + at);
            const uint32_t rw[4] = {rq.x, rq.y, rq.z, rq.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[c][2 * j] += h2f((uint16_t)rw[j]);
                v[c][2 * j + 1] += h2f((uint16_t)(rw[j] >> 16));
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++) ss = __builtin_fmaf(v[c][j], v[c][j], ss);  // (written out: the prologue of the plan kernel takes the same sums in the same order)
        if (residual && residual_out) {
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint16_t lo = f2h(v[c][2 * j]), hi = f2h(v[c][2 * j + 1]);
                o[j] = (uint32_t)lo | (uint32_t)hi << 16;
                v[c][2 * j] = h2f(lo);  // the normalised value is taken from the rounded copy
                v[c][2 * j + 1] = h2f(hi);
            }
            *(uint4 *)(residual_out + at) = make_uint4(o[0], o[1], o[2], o[3]);
        }
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & (kWave - 1)) == 0) partial[threadIdx.x / kWave] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kNormThreads / kWave; w++) total += partial[w];
    const float inv = 1.0f / sqrtf(total / (float)dim + eps);
#pragma unroll
    for (int c = 0; c < kChunks; c++) {
        const int chunk = c * kNormThreads + threadIdx.x;
        if (chunk >= chunks) break;
        const uint4 wq = *(const uint4 *)(weight + (size_t)chunk * 8);
        const uint32_t ww[4] = {wq.x, wq.y, wq.z, wq.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            o[j] = (uint32_t)f2h_of_rounded(v[c][2 * j] * inv * h2f((uint16_t)ww[j])) |
                   (uint32_t)f2h_of_rounded(v[c][2 * j + 1] * inv * h2f((uint16_t)(ww[j] >> 16))) << 16;
        *(uint4 *)(output + row + (size_t)chunk * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// Reference kernels/activations.cu:18-59: out = gate / (1 + exp(-gate)) * up. The reference calls it
// in place (output == gate, src/transformer.cpp:285), so neither pointer is declared restrict.
__device__ __forceinline__ uint16_t silu_mul_one(uint16_t gate, uint16_t up) {
    const float g = h2f(gate);
    return f2h(g / (1.0f + expf(-g)) * h2f(up));
}

// Eight elements per lane through 16-byte loads; `vec8` counts the full groups, the remaining
// size - 8*vec8 elements are handled one per lane by the workgroups past the vector part.
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t *gate, const uint16_t *up, uint16_t *output,
                                                       int size, int vec8) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t < vec8) {
        const uint4 g = ((const uint4 *)gate)[t], u = ((const uint4 *)up)[t];
        const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            o[j] = (uint32_t)silu_mul_one((uint16_t)gw[j], (uint16_t)uw[j]) |
                   (uint32_t)silu_mul_one((uint16_t)(gw[j] >> 16), (uint16_t)(uw[j] >> 16)) << 16;
        ((uint4 *)output)[t] = make_uint4(o[0], o[1], o[2], o[3]);
        return;
    }
    const int i = vec8 * 8 + (t - vec8);
    if (i < size) output[i] = silu_mul_one(gate[i], up[i]);
}

// Reference kernels/elementwise.cu:18-48: out = a + b in fp16 (one correctly rounded fp16 addition per
// element, what __hadd / __hadd2 give). Eight elements per lane through 16-byte loads, the tail one
// per lane; output may be a or b.
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(256) void add_kernel(const uint16_t *a, const uint16_t *b, uint16_t *output, int size, int vec8) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t < vec8) {
        const half8 x = ((const half8 *)a)[t], y = ((const half8 *)b)[t];
        ((half8 *)output)[t] = x + y;
        return;
    }
    const int i = vec8 * 8 + (t - vec8);
    if (i < size)
        output[i] = __builtin_bit_cast(uint16_t, (_Float16)(__builtin_bit_cast(_Float16, a[i]) + __builtin_bit_cast(_Float16, b[i])));
}

// Reference kernels/rope.cu:22-80: q [batch, seq_len, n_heads, head_dim] and k [.., n_kv_heads, ..]
// are rotated in place, pair (2i, 2i+1) of every head by the angle (start_pos + seq_idx) *
// theta^(-2i / head_dim). One thread per (token, head slot, pair) as there; a head slot below
// n_heads rotates q, below n_kv_heads rotates k. The reference forms the angle and its sine and
// cosine in fp32 (the angle is then off by up to pos * 2^-23 rad); here they are computed in fp64
// and rounded to fp32 once, the rotation itself is the reference's fp32 arithmetic.
__global__ __launch_bounds__(256) void rope_kernel(uint16_t *q, uint16_t *k, int seq_len, int n_heads, int n_kv_heads,
                                                   int head_dim, int start_pos, double log2_theta, long long total) {
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int half_dim = head_dim / 2;
    const int max_heads = n_heads > n_kv_heads ? n_heads : n_kv_heads;
    const int pair = (int)(idx % half_dim);
    long long rest = idx / half_dim;
    const int head = (int)(rest % max_heads);
    const long long token = rest / max_heads;  // batch_idx * seq_len + seq_idx
    const int pos = start_pos + (int)(token % seq_len);
    const double angle = (double)pos * exp2(-log2_theta * (2.0 * pair) / (double)head_dim);
    double sd, cd;
    sincos(angle, &sd, &cd);
    const float sn = (float)sd, cs = (float)cd;
    auto rotate = [&](uint16_t *base, int heads) {
        uint32_t *at = (uint32_t *)(base + ((size_t)token * heads + head) * head_dim) + pair;
        const uint32_t v = *at;
        const float x0 = h2f((uint16_t)v), x1 = h2f((uint16_t)(v >> 16));
        *at = (uint32_t)f2h(x0 * cs - x1 * sn) | (uint32_t)f2h(x0 * sn + x1 * cs) << 16;
    };
    if (head < n_heads) rotate(q, n_heads);
    if (head < n_kv_heads) rotate(k, n_kv_heads);
}

// Reference kernels/elementwise.cu:54-89: output[t, :] = table[indices[t], :]. One workgroup per
// token; 16-byte copies when the rows allow it.
__global__ __launch_bounds__(256) void embedding_lookup_kernel(const uint16_t *__restrict__ table,
                                                               const int *__restrict__ indices,
                                                               uint16_t *__restrict__ output, int dim, int vec) {
    const size_t src = (size_t)indices[blockIdx.x] * dim, dst = (size_t)blockIdx.x * dim;
    if (vec) {
        const uint4 *s4 = (const uint4 *)(table + src);
        uint4 *d4 = (uint4 *)(output + dst);
        for (int i = threadIdx.x; i < dim / 8; i += 256) d4[i] = s4[i];
    } else {
        for (int i = threadIdx.x; i < dim; i += 256) output[dst + i] = table[src + i];
    }
}

// Reference kernels/elementwise.cu:97-147: row (batch b, position s, head h) of k and v
// [batch, seq_len, n_kv_heads, head_dim] goes to cache row (b, h, start_pos + s) of
// [batch, n_kv_heads, max_seq_len, head_dim]; positions at or past max_seq_len are dropped.
__global__ __launch_bounds__(128) void copy_to_kv_cache_kernel(const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,
                                                               uint16_t *__restrict__ k_cache, uint16_t *__restrict__ v_cache,
                                                               int n_kv_heads, int head_dim, int seq_len, int start_pos,
                                                               int max_seq_len, int vec) {
    const int b = blockIdx.z, h = blockIdx.y, sq = blockIdx.x;
    const int pos = start_pos + sq;
    if (pos >= max_seq_len) return;
    const size_t src = (((size_t)b * seq_len + sq) * n_kv_heads + h) * head_dim;
    const size_t dst = (((size_t)b * n_kv_heads + h) * max_seq_len + pos) * head_dim;
    if (vec) {
        for (int i = threadIdx.x; i < head_dim / 8; i += 128) {
            ((uint4 *)(k_cache + dst))[i] = ((const uint4 *)(k + src))[i];
            ((uint4 *)(v_cache + dst))[i] = ((const uint4 *)(v + src))[i];
        }
    } else {
        for (int i = threadIdx.x; i < head_dim; i += 128) {
            k_cache[dst + i] = k[src + i];
            v_cache[dst + i] = v[src + i];
        }
    }
}

}  // namespace

hipError_t launch_add(const uint16_t *a, const uint16_t *b, uint16_t *output, int size, hipStream_t s) {
    const bool aligned = (((uintptr_t)a | (uintptr_t)b | (uintptr_t)output) & 15) == 0;
    const int vec8 = aligned ? size / 8 : 0;
    const int lanes = vec8 + (size - vec8 * 8);
    add_kernel<<<(lanes + 255) / 256, 256, 0, s>>>(a, b, output, size, vec8);
    return hipGetLastError();
}

hipError_t launch_rope(uint16_t *q, uint16_t *k, int batch, int seq_len, int n_heads, int n_kv_heads, int head_dim,
                       int start_pos, float theta, hipStream_t s) {
    const int max_heads = n_heads > n_kv_heads ? n_heads : n_kv_heads;
    const long long total = (long long)batch * seq_len * max_heads * (head_dim / 2);
    rope_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(q, k, seq_len, n_heads, n_kv_heads, head_dim, start_pos,
                                                                log2((double)theta), total);
    return hipGetLastError();
}

hipError_t launch_embedding_lookup(const uint16_t *table, const int *indices, uint16_t *output, int n_tokens, int dim,
                                   hipStream_t s) {
    const int vec = dim % 8 == 0 && (((uintptr_t)table | (uintptr_t)output) & 15) == 0;
    embedding_lookup_kernel<<<n_tokens, 256, 0, s>>>(table, indices, output, dim, vec);
    return hipGetLastError();
}

hipError_t launch_copy_to_kv_cache(const uint16_t *k, const uint16_t *v, uint16_t *k_cache, uint16_t *v_cache, int batch,
                                   int n_kv_heads, int head_dim, int seq_len, int start_pos, int max_seq_len,
                                   hipStream_t s) {
    const int vec = head_dim % 8 == 0 &&
                    (((uintptr_t)k | (uintptr_t)v | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0;
    copy_to_kv_cache_kernel<<<dim3(seq_len, n_kv_heads, batch), 128, 0, s>>>(k, v, k_cache, v_cache, n_kv_heads, head_dim,
                                                                             seq_len, start_pos, max_seq_len, vec);
    return hipGetLastError();
}

hipError_t launch_rmsnorm(const uint16_t *input, const uint16_t *weight, uint16_t *output, const uint16_t *residual,
                          uint16_t *residual_out, int batch, int dim, float eps, hipStream_t s) {
    const uintptr_t all = (uintptr_t)input | (uintptr_t)weight | (uintptr_t)output | (uintptr_t)residual |
                          (uintptr_t)residual_out;
    const int per_pass = kNormThreads * 8;
    if ((all & 15) == 0 && dim % 8 == 0 && dim <= 8 * per_pass) {
        if (dim <= per_pass)
            rmsnorm_rows_kernel<1><<<batch, kNormThreads, 0, s>>>(input, weight, output, residual, residual_out, dim, eps);
        else if (dim <= 2 * per_pass)
            rmsnorm_rows_kernel<2><<<batch, kNormThreads, 0, s>>>(input, weight, output, residual, residual_out, dim, eps);
        else if (dim <= 4 * per_pass)
            rmsnorm_rows_kernel<4><<<batch, kNormThreads, 0, s>>>(input, weight, output, residual, residual_out, dim, eps);
        else
            rmsnorm_rows_kernel<8><<<batch, kNormThreads, 0, s>>>(input, weight, output, residual, residual_out, dim, eps);
    } else {
        rmsnorm_kernel<<<batch, kNormThreads, 0, s>>>(input, weight, output, residual, residual_out, dim, eps);
    }
    return hipGetLastError();
}

hipError_t launch_silu_mul(const uint16_t *gate, const uint16_t *up, uint16_t *output, int size, hipStream_t s) {
    const bool aligned = (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)output) & 15) == 0;
    const int vec8 = aligned ? size / 8 : 0;
    const int lanes = vec8 + (size - vec8 * 8);
    silu_mul_kernel<<<(lanes + 255) / 256, 256, 0, s>>>(gate, up, output, size, vec8);
    return hipGetLastError();
}

// ---- measurement aid: how fast can this GPU stream memory into registers at all?
// Every thread reads 16 bytes at a time, grid-stride, keeps eight loads in flight and folds the values
// into one word; the word is stored only if it equals a value it cannot have (keeps the loads alive).
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
template <int kFlight>
__global__ __launch_bounds__(256) void read_stream_kernel(const u4v *__restrict__ src, size_t n16, uint32_t *sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t acc = 0;
    for (; i + (kFlight - 1) * stride < n16; i += kFlight * stride) {
        u4v v[kFlight];
#pragma unroll
        for (int k = 0; k < kFlight; k++) v[k] = __builtin_nontemporal_load(src + i + k * stride);
#pragma unroll
        for (int k = 0; k < kFlight; k++) acc ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
    }
    for (; i < n16; i += stride) {
        const u4v v = src[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9E3779B9u && sink) *sink = acc;
}

hipError_t launch_read_stream(const void *src, size_t bytes, uint32_t *sink, hipStream_t s) {
    // launch shape from the tuning switches (TLLM_READ_SHAPE="wgs_per_cu,loads_in_flight"); default 8 workgroups per CU, 8 loads per thread
    const int per_cu = tuning().read_wgs_per_cu.load(std::memory_order_relaxed);
    const int flight = tuning().read_in_flight.load(std::memory_order_relaxed);
    const int grid = current_device_cus() * (per_cu < 1 ? 1 : per_cu > 64 ? 64 : per_cu);
    const u4v *p = reinterpret_cast<const u4v *>(src);
    if (flight >= 16) read_stream_kernel<16><<<grid, 256, 0, s>>>(p, bytes / 16, sink);
    else if (flight >= 8) read_stream_kernel<8><<<grid, 256, 0, s>>>(p, bytes / 16, sink);
    else read_stream_kernel<4><<<grid, 256, 0, s>>>(p, bytes / 16, sink);
    return hipGetLastError();
}

}  // namespace tllm
