// The binding a maintainer of MichelHUANGGit/SD3.c adds in place of cuda/dit.cu: DiT_block_forward_cuda with the reference's
// signature (declared modules.cpp:1783-1787, registered as `DiT_block_cuda` at modules.cpp:1814) implemented over the C ABI
// of include/sd3_hip.h, plus `DiT_cuda` in the same pattern around sd3_dit_forward (argument list of DiT_forward,
// modules.cpp:1605-1613). Built here as a torch extension of its own so that the tests can call it the way
// module_tests/dit_block.py:60-66 calls the reference's.
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "sd3_hip.h"

static sd3_ctx* g_ctx = nullptr;
static int g_precision = SD3_PREC_F32;

// The reference's entry points receive the parameter map on every call. The context lives across calls and the incoming map is
// compared with the one bound by the previous call: an unchanged entry costs a hash lookup and keeps the library's bf16 copy of
// that weight; an entry whose tensor torch has modified in place (version counter) has its copies dropped; a new or moved
// tensor is bound; a name that is gone is unbound. The previous map's tensors are held until then, so that their addresses
// cannot be handed out again for other data in the meantime.
struct Bound {
    torch::Tensor t;
    uint32_t version;
};
static std::unordered_map<std::string, Bound> g_bound;

static void ok(int rc) {
    if (rc != SD3_OK) throw std::runtime_error(sd3_last_error());
}
static void bind_all(std::unordered_map<std::string, torch::Tensor>& params, const torch::Tensor& like) {
    if (!g_ctx) ok(sd3_ctx_create(&g_ctx, like.get_device()));
    ok(sd3_ctx_set_stream(g_ctx, c10::hip::getCurrentHIPStream().stream()));
    for (auto it = g_bound.begin(); it != g_bound.end();) {
        if (params.find(it->first) == params.end()) {
            ok(sd3_weights_unbind(g_ctx, it->first.c_str()));
            it = g_bound.erase(it);
        } else {
            ++it;
        }
    }
    for (auto& kv : params) {  // same names as get_ptr() looks up, modules.cpp:1558-1575
        const torch::Tensor& t = kv.second;
        const float* p = t.data_ptr<float>();
        const uint32_t version = t._version();
        auto old = g_bound.find(kv.first);
        if (old != g_bound.end() && old->second.t.data_ptr<float>() == p && old->second.t.numel() == t.numel()) {
            if (old->second.version != version) ok(sd3_weights_forget(g_ctx, p));  // same memory, new contents
        } else {
            ok(sd3_weights_bind(g_ctx, kv.first.c_str(), p, t.numel()));
        }
        g_bound[kv.first] = Bound{t, version};
    }
}

std::vector<torch::Tensor> DiT_block_forward_cuda(torch::Tensor& temp_embeddings, torch::Tensor& context_embeddings, torch::Tensor& latent_vector,
                                                  std::unordered_map<std::string, torch::Tensor>& params, int B, int Tc, int Tx, int emb_dim,
                                                  int attn_heads, int mlp_expand, bool use_dual_attention, bool use_qk_norm, bool discard_context) {
    bind_all(params, latent_vector);
    const int rc = sd3_dit_block(g_ctx, temp_embeddings.data_ptr<float>(), context_embeddings.data_ptr<float>(), latent_vector.data_ptr<float>(),
                                 /*prefix*/ "", B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm, discard_context, g_precision);
    if (rc != SD3_OK) throw std::runtime_error(sd3_last_error());
    return {context_embeddings, latent_vector};  // updated in place, as modules.cpp:1602 does
}

torch::Tensor DiT_forward_cuda(torch::Tensor& pooled_captions, torch::Tensor& captions, torch::Tensor& latent_vector, torch::Tensor& timesteps,
                               std::unordered_map<std::string, torch::Tensor>& params, int num_layers, std::unordered_set<int> dual_attention_layers,
                               int pooled_dim, int captions_dim, int C_in, int emb_dim, int attn_heads, int mlp_expand, int patch_size,
                               int pos_embed_max_size, int base_height, bool use_qk_norm) {
    bind_all(params, latent_vector);
    std::vector<int> dual(dual_attention_layers.begin(), dual_attention_layers.end());
    torch::Tensor out = torch::empty_like(latent_vector);  // a fresh tensor, as modules.cpp:1633
    const int B = latent_vector.size(0), H = latent_vector.size(2), W = latent_vector.size(3), Tc = captions.size(1);
    const int rc = sd3_dit_forward(g_ctx, pooled_captions.data_ptr<float>(), captions.data_ptr<float>(), latent_vector.data_ptr<float>(),
                                   timesteps.data_ptr<float>(), out.data_ptr<float>(), B, Tc, H, W, num_layers, dual.data(), (int)dual.size(), pooled_dim,
                                   captions_dim, C_in, emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm,
                                   g_precision);
    if (rc != SD3_OK) throw std::runtime_error(sd3_last_error());
    return out;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("DiT_block_cuda", &DiT_block_forward_cuda, "DiT block forward on the GPU (modules.cpp:1814)");
    m.def("DiT_cuda", &DiT_forward_cuda, "DiT forward on the GPU (argument list of modules.cpp:1811)");
    m.def("set_precision", [](const std::string& p) { g_precision = p == "bf16" ? SD3_PREC_BF16 : SD3_PREC_F32; });
    m.def("copies_built", []() {
        long long n = 0;
        if (g_ctx) ok(sd3_weights_copies_built(g_ctx, &n));
        return n;
    }, "derived weight copies the binding's context has built so far");
    m.def("release", []() {
        if (g_ctx) sd3_ctx_destroy(g_ctx);
        g_ctx = nullptr;
        g_bound.clear();
    });
}
