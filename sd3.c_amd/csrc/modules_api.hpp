// C++ overloads with the ORIGINAL names and argument lists of the raw-pointer layer of MichelHUANGGit/SD3.c
// modules.cpp, forwarding to the C ABI of include/sd3_hip.h. A translation unit of the reference that calls
// `layernorm(...)`, `linear(...)`, `dit_block(...)` ... compiles against this header unchanged; the only difference
// is that every pointer is a DEVICE pointer and the work is enqueued on `sd3::modules_stream()` (default: the null
// stream) of the context `sd3::modules_ctx()`.
// Failures throw std::runtime_error carrying sd3_last_error(), where the reference would assert or exit.
#pragma once
#include <functional>
#include <stdexcept>
#include <string>
#include <utility>

#include "../../include/sd3_hip.h"

namespace sd3 {
inline void*& modules_stream() {
    static void* s = nullptr;
    return s;
}
inline sd3_ctx*& modules_ctx() {  // created on first use on the current device; replace it to control device / lifetime
    static sd3_ctx* c = nullptr;
    return c;
}
inline int& modules_precision() {  // SD3_PREC_F32 (default) or SD3_PREC_BF16 for dit_block
    static int p = SD3_PREC_F32;
    return p;
}
inline void check(int status) {
    if (status != SD3_OK) throw std::runtime_error(std::string("sd3: ") + sd3_last_error());
}
}  // namespace sd3

// modules.cpp:10
inline void layernorm(float* x, float* y, float* mean, float* rstd, float* w, float* bias, float eps, int B, int T, int C) {
    sd3::check(sd3_layernorm(x, y, mean, rstd, w, bias, eps, B, T, C, sd3::modules_stream()));
}
// modules.cpp:154
inline void rmsnorm(float* x, float* y, float* w, float* rms, float eps, int B, int T, int C) {
    sd3::check(sd3_rmsnorm(x, y, w, rms, eps, B, T, C, sd3::modules_stream()));
}
// modules.cpp:192
inline void rmsnorm_group(float* x, float* y, float* w, float* rms, float eps, int groups, int B, int T, int C) {
    sd3::check(sd3_rmsnorm_group(x, y, w, rms, eps, groups, B, T, C, sd3::modules_stream()));
}
// modules.cpp:280 (erf form)
inline void gelu(float* x, float* y, long long n_elem) { sd3::check(sd3_gelu(x, y, n_elem, sd3::modules_stream())); }
// modules.cpp:293
inline void gelu_tanh(float* input, float* output, long long n_elem) { sd3::check(sd3_gelu_tanh(input, output, n_elem, sd3::modules_stream())); }
// modules.cpp:352
inline void silu(float* x, float* y, long long n_elem) { sd3::check(sd3_silu(x, y, n_elem, sd3::modules_stream())); }
// modules.cpp:475
inline void linear(float* x, float* W, float* b, float* y, int B, int C_in, int C_out) {
    sd3::check(sd3_linear(x, W, b, y, B, C_in, C_out, sd3::modules_stream()));
}
// modules.cpp:492
inline void partial_linear(float* x, float* W, float* b, float* y, int M, int K, int N, int Nmax, int n0) {
    sd3::check(sd3_partial_linear(x, W, b, y, M, K, N, Nmax, n0, sd3::modules_stream()));
}
// modules.cpp:513
inline void add(float* input, float* other, float* output, long long size) { sd3::check(sd3_add(input, other, output, size, sd3::modules_stream())); }
// modules.cpp:766
inline void multihead_attention(float* Q, float* K, float* V, float* output, int B, int num_heads, int T, int L, int head_dim) {
    sd3::check(sd3_multihead_attention(Q, K, V, output, B, num_heads, T, L, head_dim, sd3::modules_stream()));
}
// modules.cpp:946
inline void positional_embedding2D(float* output, int emb_dim, int height, int width, int base_size) {
    sd3::check(sd3_positional_embedding2D(output, emb_dim, height, width, base_size, sd3::modules_stream()));
}
// modules.cpp:977
inline void crop_positional_embedding2D(float* pos_embed, float* new_pos_embed, int pos_embed_max_size, int new_height, int new_width, int emb_dim) {
    sd3::check(sd3_crop_positional_embedding2D(pos_embed, new_pos_embed, pos_embed_max_size, new_height, new_width, emb_dim, sd3::modules_stream()));
}
// modules.cpp:1005
inline std::pair<int, int> get_conv2d_output_size(int in_height, int in_width, int kernel_height, int kernel_width, int stride, int padding) {
    return {(in_height + 2 * padding - kernel_height) / stride + 1, (in_width + 2 * padding - kernel_width) / stride + 1};
}
// modules.cpp:1037
inline void conv2d(float* input, float* output, float* kernel, float* bias, int B, int kernel_height, int kernel_width, int in_channels, int out_channels,
                   int in_height, int in_width, int out_height, int out_width, int stride, int padding) {
    sd3::check(sd3_conv2d(input, output, kernel, bias, B, kernel_height, kernel_width, in_channels, out_channels, in_height, in_width, out_height,
                          out_width, stride, padding, sd3::modules_stream()));
}
// modules.cpp:1093 -- the three scratch buffers (patches, pos_embed_max, pos_embed) are accepted and left untouched
inline void PatchEmbedding(float* latent_vector, float* /*patches*/, float* /*pos_embed_max*/, float* /*pos_embed*/, float* output, float* kernel,
                           float* bias, int B, int H, int W, int C, int emb_dim, int patch_size, int pos_embed_max_size, int base_height) {
    sd3::check(sd3_patch_embedding(latent_vector, output, kernel, bias, B, H, W, C, emb_dim, patch_size, pos_embed_max_size, base_height,
                                   sd3::modules_stream()));
}
// modules.cpp:1120 -- the reference passes its own `silu` or `gelu_tanh` as the std::function; they are recognised by address
inline void mlp(float* x, float* output, float* h1, float* W1, float* b1, float* W2, float* b2, int B, int C_in, int C_hid, int C_out,
                std::function<void(float*, float*, long long)> activation) {
    auto* fn = activation.target<void (*)(float*, float*, long long)>();
    int act;
    if (fn && *fn == &silu) act = SD3_ACT_SILU;
    else if (fn && *fn == &gelu_tanh) act = SD3_ACT_GELU_TANH;
    else throw std::invalid_argument("sd3: mlp supports the activations silu and gelu_tanh");
    sd3::check(sd3_mlp(x, output, h1, W1, b1, W2, b2, B, C_in, C_hid, C_out, act, sd3::modules_stream()));
}
// modules.cpp:1207
inline void scale_and_shift(float* input, float* output, float* shift, float* scale, int B, int T, int C) {
    sd3::check(sd3_scale_and_shift(input, output, shift, scale, B, T, C, sd3::modules_stream()));
}
// modules.cpp:1223
inline void gating_mechanism(float* input, float* output, float* gate, int B, int T, int C) {
    sd3::check(sd3_gating_mechanism(input, output, gate, B, T, C, sd3::modules_stream()));
}
// modules.cpp:1239
inline void concatenate_along_tokens(float* x, float* y, float* output, int B, int Tx, int Ty, int C) {
    sd3::check(sd3_concatenate_along_tokens(x, y, output, B, Tx, Ty, C, sd3::modules_stream()));
}
// modules.cpp:1268
inline void split_along_tokens(float* input, float* split1, float* split2, int B, int T1, int T2, int C) {
    sd3::check(sd3_split_along_tokens(input, split1, split2, B, T1, T2, C, sd3::modules_stream()));
}

// modules.cpp:1340-1365, same 49 pointers and 9 scalars in the same order. The 16 scratch pointers are accepted for
// source compatibility and not used: the library keeps its own (differently shaped) workspace in the context.
//
// WARNING for SD3_PREC_BF16: the bf16 copies of the weight matrices are made on first use and kept in the context, KEYED BY THE
// WEIGHT'S DEVICE ADDRESS. Raw pointers carry no notion of "changed": a caller that overwrites a weight buffer in place, or frees
// it and gets the same address back for other weights, must call sd3_weights_prepare(sd3::modules_ctx(), SD3_PREC_BF16) (drops
// and rebuilds every copy of the bound names) or sd3_weights_forget(sd3::modules_ctx(), ptr) for that buffer before the next
// dit_block, or the block runs on the old copies. SD3_PREC_F32 reads the weights in place and has no such state.
inline void dit_block(float* y, float* c, float* x,
                      float* c_ada_lnorm_weights, float* c_ada_lnorm_biases, float* c_Wqkv, float* c_bias_qkv, float* c_rms_Wq, float* c_rms_Wk,
                      float* c_Wout, float* c_bias_out, float* c_mlp_W1, float* c_mlp_b1, float* c_mlp_W2, float* c_mlp_b2,
                      float* x_ada_lnorm_weights, float* x_ada_lnorm_biases, float* x_Wqkv, float* x_bias_qkv, float* x_rms_Wq, float* x_rms_Wk,
                      float* x_Wout, float* x_bias_out,
                      float* x_Wqkv_dual, float* x_bias_qkv_dual, float* x_rms_Wq_dual, float* x_rms_Wk_dual, float* x_Wout_dual, float* x_bias_out_dual,
                      float* x_mlp_W1, float* x_mlp_b1, float* x_mlp_W2, float* x_mlp_b2,
                      float* /*c_hid*/, float* /*x_hid*/, float* /*x_hid_dual*/, float* /*c_query*/, float* /*c_key*/, float* /*c_value*/,
                      float* /*x_query*/, float* /*x_key*/, float* /*x_value*/, float* /*query*/, float* /*key*/, float* /*value*/,
                      float* /*c_mlp_hidden*/, float* /*x_mlp_hidden*/, float* /*y_hid1*/, float* /*y_hid2*/,
                      int B, int Tc, int Tx, int emb_dim, int attn_heads, int mlp_expand, bool use_dual_attention, bool use_qk_norm, bool discard_context) {
    if (!sd3::modules_ctx()) sd3::check(sd3_ctx_create(&sd3::modules_ctx(), 0));
    sd3::check(sd3_ctx_set_stream(sd3::modules_ctx(), sd3::modules_stream()));
    const sd3_block_weights w = {c_ada_lnorm_weights, c_ada_lnorm_biases, c_Wqkv, c_bias_qkv, c_rms_Wq, c_rms_Wk, c_Wout, c_bias_out,
                                 c_mlp_W1, c_mlp_b1, c_mlp_W2, c_mlp_b2,
                                 x_ada_lnorm_weights, x_ada_lnorm_biases, x_Wqkv, x_bias_qkv, x_rms_Wq, x_rms_Wk, x_Wout, x_bias_out,
                                 x_Wqkv_dual, x_bias_qkv_dual, x_rms_Wq_dual, x_rms_Wk_dual, x_Wout_dual, x_bias_out_dual,
                                 x_mlp_W1, x_mlp_b1, x_mlp_W2, x_mlp_b2};
    sd3::check(sd3_dit_block_w(sd3::modules_ctx(), y, c, x, &w, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm,
                               discard_context, sd3::modules_precision()));
}
