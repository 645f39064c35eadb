// What the bf16 matrix cores sustain on this device when nothing else is in the way: every wavefront of a full grid
// (one 8-wavefront workgroup per compute unit) issues v_mfma_f32_32x32x16_bf16 back to back on operands that never
// leave its registers. No memory, no LDS, no waits: whatever this loop reaches is an upper bound for any kernel built
// on that instruction. The operands are either all zero or random, because the answer depends on it: the device holds
// its power limit by lowering the shader clock, and matrix instructions on random bits draw far more than on zeros.
#include "common.hpp"

namespace sd3 {
namespace {

union ProbeFrag {
    uint4 u;
    bf16x8_t v;
};

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du;
    x ^= x >> 15; x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}
// two bf16 values drawn from N(0, 1) (Box-Muller on two hashed uniforms), the distribution of this model's activations
__device__ __forceinline__ uint32_t probe_pair(uint32_t h) {
    const float u1 = ((h >> 16) + 1.0f) * (1.0f / 65537.0f), u2 = (h & 0xffffu) * (1.0f / 65536.0f);
    const float rad = sqrtf(-2.0f * __logf(u1));
    return pack_bf16x2(rad * __cosf(6.2831853f * u2), rad * __sinf(6.2831853f * u2));
}

__global__ void __launch_bounds__(512) mfma_probe_kernel(float* sink, int iters, int random_operands) {
    ProbeFrag a[4], b[2];
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
#pragma unroll
    for (int i = 0; i < 6; i++) {
        uint4 u = make_uint4(0u, 0u, 0u, 0u);
        if (random_operands) {
            const uint32_t s = t * 24u + i * 4u;
            u = make_uint4(probe_pair(probe_hash(s)), probe_pair(probe_hash(s + 1)), probe_pair(probe_hash(s + 2)), probe_pair(probe_hash(s + 3)));
        }
        if (i < 4) a[i].u = u;
        else b[i - 4].u = u;
    }
    f32x16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i].v, b[j].v, acc[i][j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) s += acc[i][j][r];
    sink[t] = s;
}

}  // namespace
}  // namespace sd3

extern "C" int sd3_probe_mfma_bf16(int random_operands, int iters, double* tflops) {
    using namespace sd3;
    if (!tflops || iters <= 0) return fail(SD3_ERR_INVALID_ARG, "sd3_probe_mfma_bf16: needs a result pointer and iters > 0");
    int dev = 0, cus = 0;
    SD3_HIP_TRY(hipGetDevice(&dev));
    SD3_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (cus <= 0) return fail(SD3_ERR_HIP, "sd3_probe_mfma_bf16: the device reports no compute units");
    float* sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    SD3_HIP_TRY(hipMalloc(&sink, (size_t)cus * 512 * sizeof(float)));
    int rc = SD3_OK;
    float ms = 0.f;
    auto check = [&](hipError_t e, const char* what) {
        if (e != hipSuccess && rc == SD3_OK) rc = fail(SD3_ERR_HIP, "sd3_probe_mfma_bf16: %s: %s", what, hipGetErrorString(e));
    };
    check(hipEventCreate(&e0), "hipEventCreate");
    check(hipEventCreate(&e1), "hipEventCreate");
    if (rc == SD3_OK) {
        // a short untimed run first: the clock governor needs a moment to leave its idle state
        hipLaunchKernelGGL(mfma_probe_kernel, dim3(cus), dim3(512), 0, nullptr, sink, iters / 8 + 1, random_operands);
        check(hipEventRecord(e0, nullptr), "hipEventRecord");
        hipLaunchKernelGGL(mfma_probe_kernel, dim3(cus), dim3(512), 0, nullptr, sink, iters, random_operands);
        check(hipEventRecord(e1, nullptr), "hipEventRecord");
        check(hipEventSynchronize(e1), "hipEventSynchronize");
        check(hipGetLastError(), "launch");
        if (rc == SD3_OK) check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (rc != SD3_OK) return rc;
    // wavefronts x iterations x 8 instructions x (32 x 32 x 16 multiply-adds = 32768 FLOP)
    *tflops = (double)cus * 8.0 * iters * 8.0 * 32768.0 / ((double)ms * 1e-3) / 1e12;
    return SD3_OK;
}
