/*
 * CPU oracle for the ternary linear-layer path. TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's ternary
 * operators so that the HIP kernels can be checked against it. Nothing in the
 * shipped library links, loads or calls it: only tests/, the smoke check and
 * the cpu_baseline leg of the benchmark may.
 *
 * Reference lines each function follows (paths relative to the reference tree):
 *   layout / bit order .......... ternarize/pack.py:120-169, include/model.h:17-36,
 *                                 tests/test_packing.py:25-41 (independent unpack loop)
 *   tllm_oracle_gemv_hostloop ... tests/test_ternary_gemv.cu:40-75 (cpu_reference)
 *   tllm_oracle_gemv_f64 ........ kernels/ternary_gemv.cu:47-86 (group sum, then scale)
 *   tllm_oracle_gemm_f64 ........ kernels/ternary_gemm.cu:106-156,163-175
 *   tllm_oracle_gemm_f32_elem ... kernels/ternary_gemm.cu:131-155 (scale per element, fp32)
 *   tllm_oracle_quantize_i8 ..... kernels/activations.cu:100-141
 *   tllm_oracle_gemv_i8_f64 ..... kernels/ternary_gemv.cu:148-198
 *   tllm_oracle_ternarize ....... ternarize/pack.py:41-101
 *   tllm_oracle_rmsnorm_f64 ..... kernels/rmsnorm.cu:20-106
 *   tllm_oracle_silu_mul_f64 .... kernels/activations.cu:18-59
 *   tllm_oracle_add_f64 ......... kernels/elementwise.cu:18-48
 *   tllm_oracle_rope_f64 ........ kernels/rope.cu:22-80
 *   tllm_oracle_rope_f32angle ... kernels/rope.cu:49-64 (the reference's fp32 angle arithmetic)
 *   (embedding_lookup and copy_to_kv_cache, kernels/elementwise.cu:54-147, are pure row copies;
 *    their restatement is numpy indexing in oracle.py)
 *
 * Pinning status (what each function is checked against in tests/test_oracle.py):
 *   pack/unpack ........ the known-answer words of tests/test_packing.py:55-81
 *                        (0x80000003 / 0x80000001 / 0xFFFFFFFF / 0x55555555) and a
 *                        numpy unpackbits round trip.
 *   gemv_f64, gemm_f64 . dense numpy float64 matmul of the unpacked matrix with
 *                        repeated scales; closed forms (all +1 -> sum(x), one
 *                        non-zero -> s*x[k], nz=0 -> 0, sign antisymmetry,
 *                        don't-care sign bits, linearity) and brute force.
 *   gemv_hostloop ...... agreement with gemv_f64 to fp32 accumulation error and
 *                        exact agreement on integer-valued inputs.
 *   quantize_i8 ........ closed forms (absmax=0 -> scale 1 / all zero, +-absmax ->
 *                        +-127, ties to even) and a numpy restatement via np.rint.
 *   gemv_i8_f64 ........ exact integer matmul in numpy int64.
 *   ternarize .......... the two degenerate cases of tests/test_packing.py:177-205,
 *                        a numpy restatement, and tests/golden/pack_seed42.json /
 *                        pack_seed123.json: inputs and outputs of the reference's own
 *                        ternarize_tensor + pack_ternary_to_bitmasks on the two seeded
 *                        tensors of tests/test_packing.py:92-111, 141-173 (written by
 *                        tests/golden/make_pack_fixtures.py); masks, ternary values and
 *                        fp16 scales are reproduced bit for bit.
 *   rmsnorm_f64 ........ the reference holds no test or fixture for it; pinned by closed
 *                        forms (constant row -> c/sqrt(c^2+eps); unit RMS of the output at
 *                        eps=0, w=1; invariance under x -> a*x at eps=0; linearity in w;
 *                        residual path == plain path on the pre-added fp16 sum) and a numpy
 *                        restatement through np.linalg.norm.
 *   silu_mul_f64 ....... closed forms (silu(0)=0, silu(g)-silu(-g)=g, g>>0 -> g*u) and
 *                        scipy.special.expit.
 *   add_f64 ............ exact by construction (the sum of two binary16 values is exact in
 *                        binary64); checked against numpy float16 addition.
 *   rope_f64 ........... the reference holds no test or fixture for it; pinned by closed forms
 *                        (position 0 -> identity; theta = 1 -> every pair turns by `pos` radians,
 *                        against math.cos/sin; the pair (1, 0) becomes (cos, sin): sign and
 *                        interleaved pair layout; pair norms are preserved; start_pos + seq index
 *                        composes; the angle of pair i is pos * theta^(-2i/head_dim) against a
 *                        complex-exponential numpy restatement; q heads past n_kv_heads leave k
 *                        untouched). The reference evaluates the angle in fp32; the oracle is the
 *                        exact-angle rotation, from which the reference itself is off by up to
 *                        pos * 2^-23 rad.
 *   embedding / kv copy  index arithmetic checked by brute-force Python loops on small cases.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ fp16 */

/* IEEE binary16 -> binary32, exact. */
float tllm_oracle_half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: value = man * 2^-24 */
            int e = -1;
            do { man <<= 1; e++; } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary64 -> binary16 with round-to-nearest-even (single rounding). */
uint16_t tllm_oracle_double_to_half(double d) {
    uint16_t sign = signbit(d) ? 0x8000u : 0;
    double a = fabs(d);
    if (isnan(d)) return (uint16_t)(sign | 0x7E00u);
    if (a >= 65520.0) return (uint16_t)(sign | 0x7C00u); /* rounds to inf */
    if (a < 5.9604644775390625e-8 * 0.5) return sign;    /* below half the min subnormal */
    int e;
    double m = frexp(a, &e); /* a = m * 2^e, m in [0.5,1) */
    int exp16 = e - 1;       /* a = (2m) * 2^(e-1) */
    double scaled;
    if (exp16 < -14) {
        scaled = ldexp(a, 24); /* subnormal: units of 2^-24 */
        double r = nearbyint(scaled);
        return (uint16_t)(sign | (uint16_t)r); /* r==1024 lands on the min normal */
    }
    scaled = ldexp(m, 11); /* [1024,2048) */
    double r = nearbyint(scaled);
    if (r >= 2048.0) { r = 1024.0; exp16++; }
    if (exp16 > 15) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | ((uint16_t)(exp16 + 15) << 10) | ((uint16_t)r - 1024u));
}

uint16_t tllm_oracle_float_to_half(float f) { return tllm_oracle_double_to_half((double)f); }

/* ---------------------------------------------------------------- layout */

/* w[r, 32*j + b] <-> bit b (LSB first) of word j of row r; nz bit = (w != 0),
 * sign bit = (w > 0). cols must be a multiple of 32. */
void tllm_oracle_pack(const int8_t *w, int rows, int cols, uint32_t *nz, uint32_t *sg) {
    int words = cols / 32;
    for (int r = 0; r < rows; r++)
        for (int j = 0; j < words; j++) {
            uint32_t n = 0, s = 0;
            for (int b = 0; b < 32; b++) {
                int8_t v = w[(size_t)r * cols + 32 * j + b];
                if (v != 0) n |= 1u << b;
                if (v > 0) s |= 1u << b;
            }
            nz[(size_t)r * words + j] = n;
            sg[(size_t)r * words + j] = s;
        }
}

/* Inverse; a sign bit under a clear nz bit is ignored (decodes to 0). */
void tllm_oracle_unpack(const uint32_t *nz, const uint32_t *sg, int rows, int cols, int8_t *w) {
    int words = cols / 32;
    for (int r = 0; r < rows; r++)
        for (int j = 0; j < words; j++) {
            uint32_t n = nz[(size_t)r * words + j], s = sg[(size_t)r * words + j];
            for (int b = 0; b < 32; b++) {
                int8_t v = 0;
                if ((n >> b) & 1u) v = ((s >> b) & 1u) ? 1 : -1;
                w[(size_t)r * cols + 32 * j + b] = v;
            }
        }
}

static inline int weight_at(const uint32_t *nz, const uint32_t *sg, size_t word, int bit) {
    if (!((nz[word] >> bit) & 1u)) return 0;
    return ((sg[word] >> bit) & 1u) ? 1 : -1;
}

/* ------------------------------------------------------------------ GEMV */

/* fp64 evaluation of y[r] = sum_g s[r,g] * sum_{k in g} w[r,k] * x[k] on the
 * fp16-rounded scales and activations. Columns past (cols/group)*group are
 * dropped, as the reference kernel does. */
void tllm_oracle_gemv_f64(const uint32_t *nz, const uint32_t *sg, const uint16_t *scales,
                          const uint16_t *x, double *y, int rows, int cols, int group) {
    int words = cols / 32, groups = cols / group;
    double *xd = (double *)malloc(sizeof(double) * (size_t)cols);
    for (int k = 0; k < cols; k++) xd[k] = (double)tllm_oracle_half_to_float(x[k]);
    for (int r = 0; r < rows; r++) {
        double acc = 0.0;
        for (int g = 0; g < groups; g++) {
            double gs = 0.0;
            for (int j = 0; j < group; j++) {
                int k = g * group + j;
                int w = weight_at(nz, sg, (size_t)r * words + k / 32, k % 32);
                if (w > 0) gs += xd[k];
                else if (w < 0) gs -= xd[k];
            }
            acc += (double)tllm_oracle_half_to_float(scales[(size_t)r * groups + g]) * gs;
        }
        y[r] = acc;
    }
    free(xd);
}

/* The reference's own host loop, in fp32, element at a time, on float copies of
 * the scales and activations. This is the loop timed as the CPU baseline. */
void tllm_oracle_gemv_hostloop_rows(const uint32_t *nz, const uint32_t *sg, const float *scales,
                                    const float *x, float *y, int row_begin, int row_end,
                                    int cols, int group) {
    int words = cols / 32, groups = cols / group;
    for (int r = row_begin; r < row_end; r++) {
        float total = 0.0f;
        for (int g = 0; g < groups; g++) {
            float part = 0.0f;
            int first = g * group;
            for (int j = 0; j < group; j++) {
                int k = first + j;
                uint32_t n = nz[(size_t)r * words + k / 32];
                uint32_t s = sg[(size_t)r * words + k / 32];
                int b = k % 32;
                float w = ((n >> b) & 1u) ? (((s >> b) & 1u) ? 1.0f : -1.0f) : 0.0f;
                part += w * x[k];
            }
            total += scales[(size_t)r * groups + g] * part;
        }
        y[r] = total;
    }
}

void tllm_oracle_gemv_hostloop(const uint32_t *nz, const uint32_t *sg, const float *scales,
                               const float *x, float *y, int rows, int cols, int group) {
    tllm_oracle_gemv_hostloop_rows(nz, sg, scales, x, y, 0, rows, cols, group);
}

typedef struct {
    const uint32_t *nz, *sg;
    const float *scales, *x;
    float *y;
    int r0, r1, cols, group;
} hostloop_job;

static void *hostloop_worker(void *p) {
    hostloop_job *j = (hostloop_job *)p;
    tllm_oracle_gemv_hostloop_rows(j->nz, j->sg, j->scales, j->x, j->y, j->r0, j->r1, j->cols,
                                   j->group);
    return NULL;
}

/* Same loop with the rows split over `threads` host threads. */
void tllm_oracle_gemv_hostloop_mt(const uint32_t *nz, const uint32_t *sg, const float *scales,
                                  const float *x, float *y, int rows, int cols, int group,
                                  int threads) {
    if (threads < 1) threads = 1;
    if (threads > rows) threads = rows > 0 ? rows : 1;
    pthread_t *tid = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)threads);
    hostloop_job *job = (hostloop_job *)malloc(sizeof(hostloop_job) * (size_t)threads);
    for (int t = 0; t < threads; t++) {
        job[t] = (hostloop_job){nz, sg, scales, x, y, (int)((int64_t)rows * t / threads),
                                (int)((int64_t)rows * (t + 1) / threads), cols, group};
        pthread_create(&tid[t], NULL, hostloop_worker, &job[t]);
    }
    for (int t = 0; t < threads; t++) pthread_join(tid[t], NULL);
    free(tid);
    free(job);
}

/* ------------------------------------------------------------------ GEMM */

/* C[m,n] = sum_g s[n,g] * sum_{k in g} w[n,k] * A[m,k] in fp64 on fp16 inputs. */
void tllm_oracle_gemm_f64(const uint16_t *A, const uint32_t *nz, const uint32_t *sg,
                          const uint16_t *scales, double *C, int M, int N, int K, int group) {
    int words = K / 32, groups = K / group;
    double *ad = (double *)malloc(sizeof(double) * (size_t)K);
    for (int m = 0; m < M; m++) {
        for (int k = 0; k < K; k++) ad[k] = (double)tllm_oracle_half_to_float(A[(size_t)m * K + k]);
        for (int n = 0; n < N; n++) {
            double acc = 0.0;
            for (int g = 0; g < groups; g++) {
                double gs = 0.0;
                for (int wd = 0; wd < group / 32; wd++) {
                    size_t word = (size_t)n * words + (size_t)g * (group / 32) + wd;
                    uint32_t nzw = nz[word], pos = nzw & sg[word], neg = nzw & ~sg[word];
                    int base = g * group + wd * 32;
                    for (int b = 0; b < 32; b++) {
                        if ((pos >> b) & 1u) gs += ad[base + b];
                        if ((neg >> b) & 1u) gs -= ad[base + b];
                    }
                }
                acc += (double)tllm_oracle_half_to_float(scales[(size_t)n * groups + g]) * gs;
            }
            C[(size_t)m * N + n] = acc;
        }
    }
    free(ad);
}

/* The reference GEMM kernel's own order: fp32 accumulator, scale multiplied into
 * every element, positive bits of a word first and then its negative bits. */
void tllm_oracle_gemm_f32_elem(const uint16_t *A, const uint32_t *nz, const uint32_t *sg,
                               const uint16_t *scales, float *C, int M, int N, int K, int group) {
    int words = K / 32, groups = K / group;
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int j = 0; j < words; j++) {
                float s = tllm_oracle_half_to_float(scales[(size_t)n * groups + (32 * j) / group]);
                uint32_t nzw = nz[(size_t)n * words + j], sgw = sg[(size_t)n * words + j];
                uint32_t pos = nzw & sgw, neg = nzw & ~sgw;
                for (int b = 0; b < 32; b++)
                    if ((pos >> b) & 1u)
                        acc += s * tllm_oracle_half_to_float(A[(size_t)m * K + 32 * j + b]);
                for (int b = 0; b < 32; b++)
                    if ((neg >> b) & 1u)
                        acc -= s * tllm_oracle_half_to_float(A[(size_t)m * K + 32 * j + b]);
            }
            C[(size_t)m * N + n] = acc;
        }
}

/* ------------------------------------------------------------- INT8 pair */

/* absmax quantisation: scale = absmax/127 (1 when absmax is 0);
 * q = clamp(rint(x * (127/absmax)), -127, 127), fp32 arithmetic, ties to even. */
void tllm_oracle_quantize_i8(const uint16_t *x, int8_t *q, float *scale, int n) {
    float amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float v = fabsf(tllm_oracle_half_to_float(x[i]));
        if (v > amax) amax = v;
    }
    *scale = amax > 0.0f ? amax / 127.0f : 1.0f;
    float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    for (int i = 0; i < n; i++) {
        float v = tllm_oracle_half_to_float(x[i]) * inv;
        int r = (int)nearbyintf(v);
        if (r > 127) r = 127;
        if (r < -127) r = -127;
        q[i] = (int8_t)r;
    }
}

/* y[r] = input_scale * sum_g s[r,g] * (exact integer group sum), fp64 scaling. */
void tllm_oracle_gemv_i8_f64(const uint32_t *nz, const uint32_t *sg, const uint16_t *scales,
                             const int8_t *xq, float input_scale, double *y, int rows, int cols,
                             int group) {
    int words = cols / 32, groups = cols / group;
    for (int r = 0; r < rows; r++) {
        double acc = 0.0;
        for (int g = 0; g < groups; g++) {
            int64_t gs = 0;
            for (int j = 0; j < group; j++) {
                int k = g * group + j;
                gs += (int64_t)weight_at(nz, sg, (size_t)r * words + k / 32, k % 32) * xq[k];
            }
            acc += (double)tllm_oracle_half_to_float(scales[(size_t)r * groups + g]) * (double)gs;
        }
        y[r] = (double)input_scale * acc;
    }
}

/* ----------------------------------------------------------- element-wise */

/* RMSNorm with the optional residual add. t = x (+ r), the sum formed in fp32 as the kernel does;
 * res_out (may be NULL) receives fp16(t) and, when given, the normalised value is taken from that
 * rounded copy. The mean square always uses the unrounded t. Everything else in fp64; out is left
 * unrounded. */
void tllm_oracle_rmsnorm_f64(const uint16_t *x, const uint16_t *w, const uint16_t *res,
                             uint16_t *res_out, double *out, int batch, int dim, float eps) {
    for (int b = 0; b < batch; b++) {
        size_t o = (size_t)b * dim;
        double ss = 0.0;
        for (int i = 0; i < dim; i++) {
            float t = tllm_oracle_half_to_float(x[o + i]);
            if (res) {
                t += tllm_oracle_half_to_float(res[o + i]);
                if (res_out) res_out[o + i] = tllm_oracle_float_to_half(t);
            }
            ss += (double)t * (double)t;
        }
        double inv = 1.0 / sqrt(ss / (double)dim + (double)eps);
        for (int i = 0; i < dim; i++) {
            double t;
            if (res && res_out)
                t = (double)tllm_oracle_half_to_float(res_out[o + i]);
            else if (res)
                t = (double)(tllm_oracle_half_to_float(x[o + i]) + tllm_oracle_half_to_float(res[o + i]));
            else
                t = (double)tllm_oracle_half_to_float(x[o + i]);
            out[o + i] = t * inv * (double)tllm_oracle_half_to_float(w[i]);
        }
    }
}

/* out = gate / (1 + exp(-gate)) * up, fp64, unrounded. */
void tllm_oracle_silu_mul_f64(const uint16_t *gate, const uint16_t *up, double *out, int n) {
    for (int i = 0; i < n; i++) {
        double g = (double)tllm_oracle_half_to_float(gate[i]);
        double u = (double)tllm_oracle_half_to_float(up[i]);
        out[i] = g / (1.0 + exp(-g)) * u;
    }
}

/* out = a + b, exact. */
void tllm_oracle_add_f64(const uint16_t *a, const uint16_t *b, double *out, int n) {
    for (int i = 0; i < n; i++)
        out[i] = (double)tllm_oracle_half_to_float(a[i]) + (double)tllm_oracle_half_to_float(b[i]);
}

/* Rotary embedding of x [tokens = batch * seq_len, heads, head_dim] (fp16 bits) into out (fp64,
 * unrounded): pair (2i, 2i+1) of every head of token t turns by (start_pos + t % seq_len) *
 * theta^(-2i / head_dim). */
void tllm_oracle_rope_f64(const uint16_t *x, double *out, int batch, int seq_len, int heads, int head_dim,
                          int start_pos, double theta) {
    for (int64_t t = 0; t < (int64_t)batch * seq_len; t++) {
        const double pos = (double)(start_pos + (int)(t % seq_len));
        for (int h = 0; h < heads; h++) {
            const int64_t base = (t * heads + h) * head_dim;
            for (int i = 0; i < head_dim / 2; i++) {
                const double angle = pos / pow(theta, (2.0 * i) / (double)head_dim);
                const double c = cos(angle), s = sin(angle);
                const double x0 = (double)tllm_oracle_half_to_float(x[base + 2 * i]);
                const double x1 = (double)tllm_oracle_half_to_float(x[base + 2 * i + 1]);
                out[base + 2 * i] = x0 * c - x1 * s;
                out[base + 2 * i + 1] = x0 * s + x1 * c;
            }
        }
    }
}

/* The same rotation in the reference's own arithmetic (kernels/rope.cu:49-64): frequency, angle, sine and
 * cosine formed in fp32 (`1.0f / powf(theta, 2i / head_dim)`, `(float)pos * freq`, `cosf`, `sinf`), the
 * rotation in fp32, the result rounded to fp16 (returned as fp16 bits). The host's powf/sinf/cosf stand in
 * for the device's: all are within an ulp or two of the exact functions of the fp32 angle, which itself
 * is off from the exact angle by up to about pos * 2^-23 rad. Used to bound the distance between the
 * exact-angle rotation the library computes and what the reference stores. */
void tllm_oracle_rope_f32angle(const uint16_t *x, uint16_t *out, int batch, int seq_len, int heads, int head_dim,
                               int start_pos, float theta) {
    for (int64_t t = 0; t < (int64_t)batch * seq_len; t++) {
        const int pos = start_pos + (int)(t % seq_len);
        for (int h = 0; h < heads; h++) {
            const int64_t base = (t * heads + h) * head_dim;
            for (int i = 0; i < head_dim / 2; i++) {
                const float freq = 1.0f / powf(theta, (2.0f * (float)i) / (float)head_dim);
                const float angle = (float)pos * freq;
                const float c = cosf(angle), sn = sinf(angle);
                const float x0 = tllm_oracle_half_to_float(x[base + 2 * i]);
                const float x1 = tllm_oracle_half_to_float(x[base + 2 * i + 1]);
                out[base + 2 * i] = tllm_oracle_float_to_half(x0 * c - x1 * sn);
                out[base + 2 * i + 1] = tllm_oracle_float_to_half(x0 * sn + x1 * c);
            }
        }
    }
}

/* -------------------------------------------------------------- producer */

/* Ternarise `numel` floats in consecutive groups of `group` (numel % group == 0):
 * threshold = factor * mean|w| of the group; t = +1 above, -1 below -threshold;
 * scale = mean|w| over the non-zero entries (0 for an all-zero group) -> fp16. */
void tllm_oracle_ternarize(const float *w, int64_t numel, int group, float factor, int8_t *t,
                           uint16_t *scales) {
    for (int64_t g = 0; g < numel / group; g++) {
        const float *p = w + g * group;
        float sum_abs = 0.0f;
        for (int j = 0; j < group; j++) sum_abs += fabsf(p[j]);
        float thr = factor * (sum_abs / (float)group);
        float nz_sum = 0.0f;
        int nz_cnt = 0;
        for (int j = 0; j < group; j++) {
            int8_t v = 0;
            if (p[j] > thr) v = 1;
            else if (p[j] < -thr) v = -1;
            t[g * group + j] = v;
            if (v) { nz_sum += fabsf(p[j]); nz_cnt++; }
        }
        scales[g] = tllm_oracle_float_to_half(nz_sum / (float)(nz_cnt > 0 ? nz_cnt : 1));
    }
}
