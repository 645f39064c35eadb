// bf16 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16), fp32 accumulation:
//   out(M,N) = A(M,K) @ Wp^T + epilogue,  A bf16 row-major, Wp bf16 (N,K) row-major (the reference's (K,N) fp32
//   weight transposed and rounded once by pack_weight_bf16), so that both operands are K-contiguous.
// It replaces linear / partial_linear of the reference (modules.cpp:475-511) for the QKV, out-projection and MLP
// layers. Epilogues: bias | bias+GELU-tanh | bias+SiLU | gate*(.)+residual (fp32, in place) | bias + row table.
// Tile 128x128x64 per workgroup of 4 wavefronts (2x2), each wavefront 64x64 = 2x2 MFMA blocks.
#include "common.hpp"

namespace sd3 {
namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int PITCH = BK + 8;  // 144-byte rows: 16 consecutive rows start in 16 different 16-byte bank groups

struct EpiDev {
    const float* bias;
    const float* gate;
    const float* resid;
    const float* table;
    int gate_ld;
    int rows_per_batch;
};

template <int EPI, bool OUT_F32>
__global__ void __launch_bounds__(256) gemm_bf16_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ Wp, void* __restrict__ out_, int ldc,
                                                        int M, int N, int K, EpiDev epi) {
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * PITCH];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * PITCH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lk = lane >> 5;
    const int m_blk = blockIdx.y * BM, n_blk = blockIdx.x * BN;

    // staging: each tile is 128 rows x 128 bytes = 1024 chunks of 16 bytes, 4 per thread; 8 consecutive threads read one row
    const int ld_row = tid >> 3, ld_kc = (tid & 7) * 8;
    uint4 ra[4], rb[4];
    auto load_tiles = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int m = m_blk + ld_row + i * 32;
            ra[i] = (m < M) ? *reinterpret_cast<const uint4*>(A + (long long)m * K + k0 + ld_kc) : make_uint4(0, 0, 0, 0);
            const int n = n_blk + ld_row + i * 32;
            rb[i] = (n < N) ? *reinterpret_cast<const uint4*>(Wp + (long long)n * K + k0 + ld_kc) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_tiles = [&]() {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *reinterpret_cast<uint4*>(&As[(ld_row + i * 32) * PITCH + ld_kc]) = ra[i];
            *reinterpret_cast<uint4*>(&Bs[(ld_row + i * 32) * PITCH + ld_kc]) = rb[i];
        }
    };

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    load_tiles(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        store_tiles();
        __syncthreads();
        if (k0 + BK < K) load_tiles(k0 + BK);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            bf16x8_t a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++) a[i] = *reinterpret_cast<const bf16x8_t*>(&As[(wm * 64 + i * 32 + l32) * PITCH + ks * 16 + lk * 8]);
#pragma unroll
            for (int j = 0; j < 2; j++) b[j] = *reinterpret_cast<const bf16x8_t*>(&Bs[(wn * 64 + j * 32 + l32) * PITCH + ks * 16 + lk * 8]);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // C layout: lane holds column (lane % 32); register r is row 8*(r/4) + 4*(lane/32) + r%4
    float* outf = reinterpret_cast<float*>(out_);
    bf16_t* outh = reinterpret_cast<bf16_t*>(out_);
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = n_blk + wn * 64 + j * 32 + l32;
            if (n >= N) continue;
            const float bias = epi.bias ? epi.bias[n] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m_blk + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lk + (r & 3);
                if (m >= M) continue;
                const long long idx = (long long)m * ldc + n;
                float v = acc[i][j][r] + bias;
                if (EPI == EPI_BIAS_GELU) v = gelu_tanh_f(v);
                else if (EPI == EPI_BIAS_SILU) v = v / (1.0f + __expf(-v));
                else if (EPI == EPI_GATE_RESID) v = epi.resid[idx] + epi.gate[(long long)(m / epi.rows_per_batch) * epi.gate_ld + n] * v;
                else if (EPI == EPI_BIAS_ROWADD) v += epi.table[(long long)(m % epi.rows_per_batch) * epi.gate_ld + n];
                if (OUT_F32) outf[idx] = v;
                else outh[idx] = f32_to_bf16(v);
            }
        }
}

}  // namespace

int gemm_bf16(const bf16_t* A, const bf16_t* Wp, void* out, int out_is_f32, int ldc, int M, int N, int K, int epi, const GemmEpilogueArgs& ea,
              hipStream_t st) {
    if (M <= 0 || N <= 0) return SD3_OK;
    if (K <= 0 || (K % BK) != 0) return fail(SD3_ERR_UNSUPPORTED, "gemm_bf16: K=%d must be a positive multiple of %d", K, BK);
    if ((reinterpret_cast<uintptr_t>(A) & 15) || (reinterpret_cast<uintptr_t>(Wp) & 15))
        return fail(SD3_ERR_INVALID_ARG, "gemm_bf16: operands must be 16-byte aligned");
    EpiDev e{ea.bias, ea.gate, ea.resid, ea.table, ea.gate_ld, ea.rows_per_batch > 0 ? ea.rows_per_batch : 1};
    if (epi == EPI_BIAS_ROWADD) e.gate_ld = N;
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM), block(256);
#define SD3_GEMM_BF16_LAUNCH(E)                                                                                                \
    do {                                                                                                                       \
        if (out_is_f32) hipLaunchKernelGGL((gemm_bf16_kernel<E, true>), grid, block, 0, st, A, Wp, out, ldc, M, N, K, e);      \
        else hipLaunchKernelGGL((gemm_bf16_kernel<E, false>), grid, block, 0, st, A, Wp, out, ldc, M, N, K, e);                \
    } while (0)
    switch (epi) {
        case EPI_BIAS: SD3_GEMM_BF16_LAUNCH(EPI_BIAS); break;
        case EPI_BIAS_GELU: SD3_GEMM_BF16_LAUNCH(EPI_BIAS_GELU); break;
        case EPI_BIAS_SILU: SD3_GEMM_BF16_LAUNCH(EPI_BIAS_SILU); break;
        case EPI_GATE_RESID: SD3_GEMM_BF16_LAUNCH(EPI_GATE_RESID); break;
        case EPI_BIAS_ROWADD: SD3_GEMM_BF16_LAUNCH(EPI_BIAS_ROWADD); break;
        default: return fail(SD3_ERR_INVALID_ARG, "gemm_bf16: unknown epilogue %d", epi);
    }
#undef SD3_GEMM_BF16_LAUNCH
    return launch_status("gemm_bf16");
}

}  // namespace sd3
