// Compile-and-run check of the C++ drop-in interface: the call expressions below have
// the shapes of the reference's callers (src/transformer.cpp:107-116 ternary_linear,
// :132-142 ternary_linear_int8, :193-196 rmsnorm_forward, :285-286 silu_mul_forward). With null pointers every call must be rejected by the
// argument validation before any GPU work, so this runs on a host without a GPU.
#include <cstdio>
#include <cstdlib>

#include "ternary_kernels.hpp"

struct TernaryWeight {  // same fields as the reference's include/model.h:17-23
    uint32_t *nonzero_masks = nullptr;
    uint32_t *sign_masks = nullptr;
    half *scales = nullptr;
    int out_features = 0;
    int in_features = 0;
};

static int rejected = 0;
static void count_handler(const char *, int code) { rejected += code < 0; }

int main() {
    ternary::error_handler() = count_handler;
    TernaryWeight w;
    w.out_features = 2048;
    w.in_features = 2048;
    const half *input = nullptr;
    half *output = nullptr;
    int8_t *int8_buf_ = nullptr;
    float *int8_scale_ = nullptr;
    int gs = 128, n_tokens = 7, dim = 2048;
    float h_scale = 0.5f;

    ternary::ternary_gemv(w.nonzero_masks, w.sign_masks, w.scales, input, output, w.out_features,
                          w.in_features, gs);
    ternary::ternary_gemm(input, w.nonzero_masks, w.sign_masks, w.scales, output, n_tokens,
                          w.out_features, w.in_features, gs);
    ternary::quantize_absmax_int8(input, int8_buf_, int8_scale_, dim);
    ternary::ternary_gemv_int8(w.nonzero_masks, w.sign_masks, w.scales, int8_buf_, h_scale, output,
                               w.out_features, w.in_features, gs);
    half *residual_buf_ = nullptr, *hidden_buf_ = nullptr, *gate_buf_ = nullptr, *up_buf_ = nullptr;
    const half *attn_norm_weight = nullptr;
    int hidden = 2048, inter = 5632;
    float rms_norm_eps = 1e-5f;
    ternary::rmsnorm_forward(residual_buf_, attn_norm_weight, hidden_buf_, nullptr, nullptr, n_tokens, hidden,
                             rms_norm_eps);
    ternary::silu_mul_forward(gate_buf_, up_buf_, gate_buf_, n_tokens * inter);
    // src/transformer.cpp:179-181 embedding, :225-236 RoPE and cache update, :253, 296 residual add
    half *q_buf_ = nullptr, *k_buf_ = nullptr, *v_buf_ = nullptr, *k_cache = nullptr, *v_cache = nullptr;
    const half *embed_tokens = nullptr;
    const int *d_tokens = nullptr;
    int n_heads = 32, n_kv_heads = 8, head_dim = 64, start_pos = 3, max_seq_len = 4096;
    float rope_theta = 500000.0f;
    ternary::embedding_lookup(embed_tokens, d_tokens, hidden_buf_, n_tokens, hidden);
    ternary::rope_forward(q_buf_, k_buf_, 1, n_tokens, n_heads, n_kv_heads, head_dim, start_pos, rope_theta);
    ternary::copy_to_kv_cache(k_buf_, v_buf_, k_cache, v_cache, 1, n_kv_heads, head_dim, n_tokens, start_pos, max_seq_len);
    ternary::add_forward(residual_buf_, hidden_buf_, residual_buf_, n_tokens * hidden);
    // the calls that replace member functions or groups of launches of the reference: ternary_linear_int8
    // (src/transformer.cpp:126-143) and the FFN front half of a prefill step (:264-286)
    ternary::ternary_linear_int8(w.nonzero_masks, w.sign_masks, w.scales, input, output, w.out_features, w.in_features, gs);
    ternary::ternary_gemm_swiglu(hidden_buf_, w.nonzero_masks, w.sign_masks, w.scales, w.nonzero_masks, w.sign_masks, w.scales,
                                 gate_buf_, n_tokens, inter, hidden, gs);
    // the q, k and v projections of a prefill step as one launch (:199-217)
    const uint32_t *nzs[3] = {w.nonzero_masks, w.nonzero_masks, w.nonzero_masks}, *sgs[3] = {w.sign_masks, w.sign_masks, w.sign_masks};
    const half *scs[3] = {w.scales, w.scales, w.scales};
    half *outs[3] = {q_buf_, k_buf_, v_buf_};
    const int ns[3] = {n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * head_dim};
    ternary::ternary_gemm_group(hidden_buf_, nzs, sgs, scs, outs, ns, 3, n_tokens, hidden, gs);
    std::printf("rejected=%d\n", rejected);
    return rejected == 13 ? 0 : 1;
}
