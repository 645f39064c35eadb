// A C++ caller of the boundary, written the way a translation unit of MichelHUANGGit/SD3.c calls its raw-pointer layer
// (modules.cpp:1340-1366 dit_block, :475 linear, :1120 mlp): same function names, same argument lists, through
// sd3.c_amd/csrc/modules_api.hpp. The only difference to the reference's caller (modules.cpp:1577-1583) is that the
// buffers are device memory.
//
//   host_block <case.bin> <out.bin> [bf16]
//
// case.bin : 10 int32 (B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual, use_qk_norm, discard_context, n_tensors), then
//            n_tensors records of (int64 numel, numel float32): y, c, x, then the 30 block weights in the argument order of
//            dit_block; numel 0 stands for a null pointer.
// out.bin  : c, x after the block; linear(x_in, latent_attn_Wout); mlp(x_in, latent_mlp, gelu_tanh) -- raw float32.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "modules_api.hpp"

#define HIP_OK(e)                                                                    \
    do {                                                                             \
        hipError_t e_ = (e);                                                         \
        if (e_ != hipSuccess) {                                                      \
            std::fprintf(stderr, "%s: %s\n", #e, hipGetErrorString(e_));             \
            return 2;                                                                \
        }                                                                            \
    } while (0)

int main(int argc, char** argv) {
    if (argc < 3) return 64;
    FILE* f = std::fopen(argv[1], "rb");
    if (!f) return 66;
    int32_t h[10];
    if (std::fread(h, sizeof(int32_t), 10, f) != 10) return 65;
    const int B = h[0], Tc = h[1], Tx = h[2], C = h[3], NH = h[4], E = h[5], n = h[9];
    const bool dual = h[6], qk = h[7], discard = h[8];
    if (n != 33) return 65;
    std::vector<std::vector<float>> host(n);
    std::vector<float*> d(n, nullptr);
    for (int i = 0; i < n; i++) {
        int64_t numel = 0;
        if (std::fread(&numel, sizeof(numel), 1, f) != 1) return 65;
        host[i].resize(numel);
        if (numel && std::fread(host[i].data(), sizeof(float), numel, f) != (size_t)numel) return 65;
        if (numel) {
            HIP_OK(hipMalloc((void**)&d[i], numel * sizeof(float)));
            HIP_OK(hipMemcpy(d[i], host[i].data(), numel * sizeof(float), hipMemcpyHostToDevice));
        }
    }
    std::fclose(f);
    if (argc > 3 && !std::strcmp(argv[3], "bf16")) sd3::modules_precision() = SD3_PREC_BF16;

    float *x_in = nullptr, *lin = nullptr, *mlp_h = nullptr, *mlp_out = nullptr;
    const size_t mx = (size_t)B * Tx;
    HIP_OK(hipMalloc((void**)&x_in, mx * C * sizeof(float)));
    HIP_OK(hipMemcpy(x_in, d[2], mx * C * sizeof(float), hipMemcpyDeviceToDevice));
    HIP_OK(hipMalloc((void**)&lin, mx * C * sizeof(float)));
    HIP_OK(hipMalloc((void**)&mlp_h, mx * E * C * sizeof(float)));
    HIP_OK(hipMalloc((void**)&mlp_out, mx * C * sizeof(float)));
    float* y = d[0];
    float* c = d[1];
    float* x = d[2];
    float** w = d.data() + 3;
    float* none = nullptr;  // the 16 scratch buffers of the reference: accepted, unused
    try {
        dit_block(y, c, x, w[0], w[1], w[2], w[3], w[4], w[5], w[6], w[7], w[8], w[9], w[10], w[11],      // context stream
                  w[12], w[13], w[14], w[15], w[16], w[17], w[18], w[19],                                  // latent stream
                  w[20], w[21], w[22], w[23], w[24], w[25],                                                // dual branch
                  w[26], w[27], w[28], w[29],                                                              // latent MLP
                  none, none, none, none, none, none, none, none, none, none, none, none, none, none, none, none,
                  B, Tc, Tx, C, NH, E, dual, qk, discard);
        linear(x_in, w[18], w[19], lin, (int)mx, C, C);
        mlp(x_in, mlp_out, mlp_h, w[26], w[27], w[28], w[29], (int)mx, C, E * C, C, gelu_tanh);
    } catch (const std::exception& e) {
        std::fprintf(stderr, "%s\n", e.what());
        return 1;
    }
    HIP_OK(hipDeviceSynchronize());
    FILE* o = std::fopen(argv[2], "wb");
    if (!o) return 73;
    auto dump = [&](const float* p, size_t numel) {
        std::vector<float> buf(numel);
        if (numel && hipMemcpy(buf.data(), p, numel * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess) return false;
        return std::fwrite(buf.data(), sizeof(float), numel, o) == numel;
    };
    const bool ok = dump(c, (size_t)B * Tc * C) && dump(x, mx * C) && dump(lin, mx * C) && dump(mlp_out, mx * C);
    std::fclose(o);
    if (!ok) return 74;

    // Stream lifetime: the same block twice more, each time on a stream that this program creates before the call and destroys
    // after it. When the second call hands the context its new stream the previous one no longer exists, and when the context is
    // destroyed neither does: the library must order its work without touching a dead stream's handle, and give the same bits.
    std::vector<float> first(mx * C), again(mx * C);
    HIP_OK(hipMemcpy(first.data(), x, mx * C * sizeof(float), hipMemcpyDeviceToHost));
    for (int round = 0; round < 2; round++) {
        hipStream_t s = nullptr;
        HIP_OK(hipStreamCreate(&s));
        sd3::modules_stream() = s;
        HIP_OK(hipMemcpyAsync(c, host[1].data(), host[1].size() * sizeof(float), hipMemcpyHostToDevice, s));
        HIP_OK(hipMemcpyAsync(x, host[2].data(), host[2].size() * sizeof(float), hipMemcpyHostToDevice, s));
        try {
            dit_block(y, c, x, w[0], w[1], w[2], w[3], w[4], w[5], w[6], w[7], w[8], w[9], w[10], w[11], w[12], w[13], w[14], w[15], w[16], w[17],
                      w[18], w[19], w[20], w[21], w[22], w[23], w[24], w[25], w[26], w[27], w[28], w[29], none, none, none, none, none, none, none,
                      none, none, none, none, none, none, none, none, none, B, Tc, Tx, C, NH, E, dual, qk, discard);
        } catch (const std::exception& e) {
            std::fprintf(stderr, "stream round %d: %s\n", round, e.what());
            return 1;
        }
        HIP_OK(hipMemcpyAsync(again.data(), x, mx * C * sizeof(float), hipMemcpyDeviceToHost, s));
        HIP_OK(hipStreamSynchronize(s));
        HIP_OK(hipStreamDestroy(s));
        if (std::memcmp(first.data(), again.data(), mx * C * sizeof(float)) != 0) {
            std::fprintf(stderr, "stream round %d: result differs from the first call\n", round);
            return 75;
        }
    }
    if (sd3_ctx_destroy(sd3::modules_ctx()) != SD3_OK) return 76;  // (its last stream is gone by now)
    return 0;
}
