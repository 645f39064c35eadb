// TEST INFRASTRUCTURE ONLY. Never linked into, or loaded by, the shipped library.
//
// C-ABI shims around the *compiled reference* (MichelHUANGGit/SD3.c modules.cpp,
// built in place from /root/reference by oracle/Makefile into oracle/_ref/).
// This file contains no arithmetic of its own: every function forwards to the
// reference function whose declaration is repeated here (file:line cited), so that
// tests can check oracle/sd3_oracle.c against the reference bit for bit and so
// that tests/golden/make_golden.py can write fixtures.
#include <torch/torch.h>

#include <cstdlib>
#include <cstring>
#include <new>

#include <functional>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

// ---- declarations of reference functions (external linkage in modules.cpp) ----
void layernorm(float* x, float* y, float* mean, float* rstd, float* w, float* bias, float eps, int B, int T, int C);  // modules.cpp:10
void rmsnorm_group(float* x, float* y, float* w, float* rms, float eps, int groups, int B, int T, int C);              // modules.cpp:192
void gelu(float* x, float* y, long long n_elem);                                                                       // modules.cpp:280
void gelu_tanh(float* input, float* output, long long n_elem);                                                         // modules.cpp:293
void silu(float* x, float* y, long long n_elem);                                                                       // modules.cpp:352
void linear(float* x, float* W, float* b, float* y, int B, int C_in, int C_out);                                       // modules.cpp:475
void partial_linear(float* x, float* W, float* b, float* y, int M, int K, int N, int Nmax, int n0);                    // modules.cpp:492
void add(float* input, float* other, float* output, long long size);                                                   // modules.cpp:513
void multihead_attention(float* Q, float* K, float* V, float* output, int B, int num_heads, int T, int L, int head_dim);  // modules.cpp:766
torch::Tensor sinusoidal_embedding(torch::Tensor& timesteps, int emb_dim);                                             // modules.cpp:920
void positional_embedding2D(float* output, int emb_dim, int height, int width, int base_size);                         // modules.cpp:946
void crop_positional_embedding2D(float* pos_embed, float* new_pos_embed, int pos_embed_max_size, int new_height, int new_width, int emb_dim);  // modules.cpp:977
void conv2d(float* input, float* output, float* kernel, float* bias, int B, int kernel_height, int kernel_width, int in_channels,
            int out_channels, int in_height, int in_width, int out_height, int out_width, int stride, int padding);    // modules.cpp:1037
void mlp(float* x, float* output, float* h1, float* W1, float* b1, float* W2, float* b2, int B, int C_in, int C_hid, int C_out,
         std::function<void(float*, float*, long long)> activation);                                                   // modules.cpp:1120
void scale_and_shift(float* input, float* output, float* shift, float* scale, int B, int T, int C);                    // modules.cpp:1207
void gating_mechanism(float* input, float* output, float* gate, int B, int T, int C);                                  // modules.cpp:1223
void concatenate_along_tokens(float* x, float* y, float* output, int B, int Tx, int Ty, int C);                        // modules.cpp:1239
void split_along_tokens(float* input, float* split1, float* split2, int B, int T1, int T2, int C);                     // modules.cpp:1268
std::vector<torch::Tensor> DiT_block_forward(torch::Tensor& temp_embeddings, torch::Tensor& context_embeddings, torch::Tensor& latent_vector,
                                             std::unordered_map<std::string, torch::Tensor>& params, int B, int Tc, int Tx, int emb_dim,
                                             int attn_heads, int mlp_expand, bool use_dual_attention, bool use_qk_norm,
                                             bool discard_context);                                                    // modules.cpp:1508
torch::Tensor DiT_forward(torch::Tensor& pooled_captions, torch::Tensor& captions, torch::Tensor& latent_vector, torch::Tensor& timesteps,
                          std::unordered_map<std::string, torch::Tensor>& params, int num_layers,
                          std::unordered_set<int> dual_attention_layers, int pooled_dim, int captions_dim, int C_in, int emb_dim,
                          int attn_heads, int mlp_expand, int patch_size, int pos_embed_max_size, int base_height,
                          bool use_qk_norm);                                                                           // modules.cpp:1605

// The reference accumulates the patch convolution into a scratch buffer that it allocates with
// new float[] and never clears (modules.cpp:1032 with modules.cpp:1642,1682), so its output depends
// on what the heap held before: two calls in one process can differ by O(1). Its author's test
// passes on fresh zero pages. This library therefore hands every new[] made inside it (the version
// script keeps these two symbols local to the library) zero-filled memory, which makes the compiled
// reference deterministic and equal to the PyTorch model it is tested against.
void* operator new[](std::size_t n) {
    void* p = std::calloc(n ? n : 1, 1);
    if (!p) throw std::bad_alloc();
    return p;
}
void operator delete[](void* p) noexcept { std::free(p); }
void operator delete[](void* p, std::size_t) noexcept { std::free(p); }

namespace {
torch::Tensor wrap(float* p, std::vector<int64_t> shape) { return torch::from_blob(p, shape, torch::kFloat32); }

std::unordered_map<std::string, torch::Tensor> make_params(int n, const char** names, float** ptrs, const long long* numels) {
    std::unordered_map<std::string, torch::Tensor> m;
    for (int i = 0; i < n; i++) m.emplace(std::string(names[i]), wrap(ptrs[i], {(int64_t)numels[i]}));
    return m;
}
}  // namespace

#define REF_API extern "C" __attribute__((visibility("default")))

REF_API void ref_layernorm(float* x, float* y, float eps, int B, int T, int C) { layernorm(x, y, nullptr, nullptr, nullptr, nullptr, eps, B, T, C); }
REF_API void ref_rmsnorm_group(float* x, float* y, float* w, float eps, int groups, int B, int T, int C) { rmsnorm_group(x, y, w, nullptr, eps, groups, B, T, C); }
REF_API void ref_gelu_tanh(float* in, float* out, long long n) { gelu_tanh(in, out, n); }
REF_API void ref_gelu(float* in, float* out, long long n) { gelu(in, out, n); }
REF_API void ref_silu(float* in, float* out, long long n) { silu(in, out, n); }
REF_API void ref_linear(float* x, float* W, float* b, float* y, int B, int Cin, int Cout) { linear(x, W, b, y, B, Cin, Cout); }
REF_API void ref_partial_linear(float* x, float* W, float* b, float* y, int M, int K, int N, int Nmax, int n0) { partial_linear(x, W, b, y, M, K, N, Nmax, n0); }
REF_API void ref_add(float* a, float* b, float* out, long long n) { add(a, b, out, n); }
REF_API void ref_multihead_attention(float* Q, float* K, float* V, float* out, int B, int NH, int T, int L, int HS) { multihead_attention(Q, K, V, out, B, NH, T, L, HS); }
REF_API void ref_sinusoidal_embedding(float* t, float* out, int B, int emb_dim) {
    torch::Tensor tt = wrap(t, {B});
    torch::Tensor o = sinusoidal_embedding(tt, emb_dim);
    std::memcpy(out, o.data_ptr<float>(), sizeof(float) * (size_t)B * emb_dim);
}
REF_API void ref_positional_embedding2D(float* out, int emb_dim, int height, int width, int base_size) { positional_embedding2D(out, emb_dim, height, width, base_size); }
REF_API void ref_crop_positional_embedding2D(float* pe, float* out, int max_size, int h, int w, int emb_dim) { crop_positional_embedding2D(pe, out, max_size, h, w, emb_dim); }
REF_API void ref_conv2d(float* in, float* out, float* kernel, float* bias, int B, int kh, int kw, int cin, int cout, int ih, int iw, int oh, int ow, int stride, int pad) {
    conv2d(in, out, kernel, bias, B, kh, kw, cin, cout, ih, iw, oh, ow, stride, pad);
}
// act: 0 = silu, 1 = gelu_tanh (the two activations the forward path passes to mlp)
REF_API void ref_mlp(float* x, float* out, float* h1, float* W1, float* b1, float* W2, float* b2, int B, int Cin, int Chid, int Cout, int act) {
    if (act == 0) mlp(x, out, h1, W1, b1, W2, b2, B, Cin, Chid, Cout, silu);
    else mlp(x, out, h1, W1, b1, W2, b2, B, Cin, Chid, Cout, gelu_tanh);
}
REF_API void ref_scale_and_shift(float* in, float* out, float* shift, float* scale, int B, int T, int C) { scale_and_shift(in, out, shift, scale, B, T, C); }
REF_API void ref_gating_mechanism(float* in, float* out, float* gate, int B, int T, int C) { gating_mechanism(in, out, gate, B, T, C); }
REF_API void ref_concatenate_along_tokens(float* x, float* y, float* out, int B, int Tx, int Ty, int C) { concatenate_along_tokens(x, y, out, B, Tx, Ty, C); }
REF_API void ref_split_along_tokens(float* in, float* s1, float* s2, int B, int T1, int T2, int C) { split_along_tokens(in, s1, s2, B, T1, T2, C); }

// c and x are updated in place, like the reference does.
REF_API void ref_dit_block(float* y, float* c, float* x, int n_params, const char** names, float** ptrs, const long long* numels, int B, int Tc,
                           int Tx, int emb_dim, int attn_heads, int mlp_expand, int use_dual, int use_qk_norm, int discard_context) {
    auto params = make_params(n_params, names, ptrs, numels);
    torch::Tensor ty = wrap(y, {B, emb_dim}), tc = wrap(c, {B, Tc, emb_dim}), tx = wrap(x, {B, Tx, emb_dim});
    DiT_block_forward(ty, tc, tx, params, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual != 0, use_qk_norm != 0, discard_context != 0);
}

REF_API void ref_dit_forward(float* pooled, float* captions, float* latent, float* timesteps, float* out, int n_params, const char** names,
                             float** ptrs, const long long* numels, int B, int Tc, int H, int W, int num_layers, int n_dual,
                             const int* dual_layers, int pooled_dim, int captions_dim, int C_in, int emb_dim, int attn_heads, int mlp_expand,
                             int patch_size, int pos_embed_max_size, int base_height, int use_qk_norm) {
    auto params = make_params(n_params, names, ptrs, numels);
    std::unordered_set<int> dual(dual_layers, dual_layers + n_dual);
    torch::Tensor tp = wrap(pooled, {B, pooled_dim}), tcap = wrap(captions, {B, Tc, captions_dim}), tl = wrap(latent, {B, C_in, H, W}),
                  tt = wrap(timesteps, {B});
    torch::Tensor o = DiT_forward(tp, tcap, tl, tt, params, num_layers, dual, pooled_dim, captions_dim, C_in, emb_dim, attn_heads, mlp_expand,
                                  patch_size, pos_embed_max_size, base_height, use_qk_norm != 0);
    std::memcpy(out, o.data_ptr<float>(), sizeof(float) * (size_t)o.numel());
}
