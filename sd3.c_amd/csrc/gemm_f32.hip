// fp32 GEMM on the gfx950 fp32 matrix cores (v_mfma_f32_32x32x2_f32), for the fp32 parity path:
//   out(M,N) = A(M,K) @ W(K,N)[:, n0:n0+N] + epilogue
// replacing linear / partial_linear of the reference (modules.cpp:475-511, naive triple loops).
// Tile: 128x128x16 per workgroup of 4 wavefronts (2x2), each wavefront owns 64x64 = 2x2 MFMA blocks.
// Any M, N, K: out-of-range elements are zero-filled on load and masked on store.
#include "common.hpp"

namespace sd3 {

namespace {
constexpr int BM = 128, BN = 128, BK = 16;
constexpr int A_PITCH = BM + 4;  // As[k][m]: 4*(BM+4) = 528 = 16 mod 64 -> the four k-quads of a wave hit disjoint banks on store
constexpr int B_PITCH = BN + 4;

struct EpiDev {
    const float* bias;
    const float* gate;
    const float* resid;
    const float* table;
    int gate_ld;
    int rows_per_batch;
};

template <int EPI>
__device__ __forceinline__ float apply_epilogue(float acc, int m, int n, int n_glob, const EpiDev& e, long long out_idx) {
    float v = acc;
    if (e.bias) v += e.bias[n_glob];
    if (EPI == EPI_BIAS_GELU) v = gelu_tanh_precise(v);
    else if (EPI == EPI_BIAS_SILU) v = silu_precise(v);
    else if (EPI == EPI_GATE_RESID) {
        v *= e.gate[(long long)(m / e.rows_per_batch) * e.gate_ld + n];
        v += e.resid[out_idx];
    } else if (EPI == EPI_BIAS_ROWADD) {
        v += e.table[(long long)(m % e.rows_per_batch) * /*table row stride = N, passed in gate_ld*/ e.gate_ld + n];
    }
    return v;
}

template <int EPI, bool ALIGNED>
__global__ void __launch_bounds__(256) gemm_f32_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw, int n0,
                                                       float* __restrict__ out, int ldc, int M, int N, int K, EpiDev epi) {
    __shared__ float As[BK * A_PITCH];
    __shared__ float Bs[BK * B_PITCH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m_blk = blockIdx.y * BM, n_blk = blockIdx.x * BN;

    // global -> register staging: A tile 128x16 (2 float4 per thread along k), W tile 16x128 (2 float4 per thread along n)
    const int a_row = tid >> 2, a_kq = (tid & 3) * 4;  // rows a_row and a_row+64
    const int b_k = tid >> 5, b_n = (tid & 31) * 4;    // k rows b_k and b_k+8
    float4 ra[2], rb[2];

    auto load_tiles = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int m = m_blk + a_row + i * 64;
            const int k = k0 + a_kq;
            if (ALIGNED) {
                ra[i] = (m < M && k < K) ? *reinterpret_cast<const float4*>(A + (long long)m * lda + k) : make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                float t[4];
#pragma unroll
                for (int j = 0; j < 4; j++) t[j] = (m < M && k + j < K) ? A[(long long)m * lda + k + j] : 0.f;
                ra[i] = make_float4(t[0], t[1], t[2], t[3]);
            }
            const int kk = k0 + b_k + i * 8;
            const int n = n_blk + b_n;
            if (ALIGNED) {
                rb[i] = (kk < K && n < N) ? *reinterpret_cast<const float4*>(W + (long long)kk * ldw + n0 + n) : make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                float t[4];
#pragma unroll
                for (int j = 0; j < 4; j++) t[j] = (kk < K && n + j < N) ? W[(long long)kk * ldw + n0 + n + j] : 0.f;
                rb[i] = make_float4(t[0], t[1], t[2], t[3]);
            }
        }
    };
    auto store_tiles = [&]() {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int m = a_row + i * 64;
            As[(a_kq + 0) * A_PITCH + m] = ra[i].x;
            As[(a_kq + 1) * A_PITCH + m] = ra[i].y;
            As[(a_kq + 2) * A_PITCH + m] = ra[i].z;
            As[(a_kq + 3) * A_PITCH + m] = ra[i].w;
            *reinterpret_cast<float4*>(&Bs[(b_k + i * 8) * B_PITCH + b_n]) = rb[i];
        }
    };

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const int l32 = lane & 31, lk = lane >> 5;
    load_tiles(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        store_tiles();
        __syncthreads();
        if (k0 + BK < K) load_tiles(k0 + BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++) a[i] = As[(kk + lk) * A_PITCH + wm * 64 + i * 32 + l32];
#pragma unroll
            for (int j = 0; j < 2; j++) b[j] = Bs[(kk + lk) * B_PITCH + wn * 64 + j * 32 + l32];
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // C layout of the 32x32 MFMA: lane holds column (lane % 32); register r is row 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int n = n_blk + wn * 64 + j * 32 + l32;
            if (n >= N) continue;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m_blk + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lk + (r & 3);
                if (m < M) {
                    const long long idx = (long long)m * ldc + n;
                    out[idx] = apply_epilogue<EPI>(acc[i][j][r], m, n, n0 + n, epi, idx);
                }
            }
        }
}
}  // namespace

int gemm_f32(const float* A, int lda, const float* W, int ldw, int n0, float* out, int ldc, int M, int N, int K, int epi, const GemmEpilogueArgs& ea,
             hipStream_t st) {
    if (M <= 0 || N <= 0) return SD3_OK;
    if (K <= 0) return fail(SD3_ERR_INVALID_ARG, "gemm_f32: K must be positive");
    EpiDev e{ea.bias, ea.gate, ea.resid, ea.table, ea.gate_ld, ea.rows_per_batch > 0 ? ea.rows_per_batch : 1};
    if (epi == EPI_BIAS_ROWADD) e.gate_ld = N;
    const bool aligned = (lda % 4 == 0) && (ldw % 4 == 0) && (n0 % 4 == 0) && (K % 4 == 0) && (N % 4 == 0) &&
                         ((reinterpret_cast<uintptr_t>(A) & 15) == 0) && ((reinterpret_cast<uintptr_t>(W) & 15) == 0);
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM), block(256);
#define SD3_GEMM_F32_LAUNCH(E)                                                                                                               \
    do {                                                                                                                                     \
        if (aligned) hipLaunchKernelGGL((gemm_f32_kernel<E, true>), grid, block, 0, st, A, lda, W, ldw, n0, out, ldc, M, N, K, e);             \
        else hipLaunchKernelGGL((gemm_f32_kernel<E, false>), grid, block, 0, st, A, lda, W, ldw, n0, out, ldc, M, N, K, e);                    \
    } while (0)
    switch (epi) {
        case EPI_BIAS: SD3_GEMM_F32_LAUNCH(EPI_BIAS); break;
        case EPI_BIAS_GELU: SD3_GEMM_F32_LAUNCH(EPI_BIAS_GELU); break;
        case EPI_BIAS_SILU: SD3_GEMM_F32_LAUNCH(EPI_BIAS_SILU); break;
        case EPI_GATE_RESID: SD3_GEMM_F32_LAUNCH(EPI_GATE_RESID); break;
        case EPI_BIAS_ROWADD: SD3_GEMM_F32_LAUNCH(EPI_BIAS_ROWADD); break;
        default: return fail(SD3_ERR_INVALID_ARG, "gemm_f32: unknown epilogue %d", epi);
    }
#undef SD3_GEMM_F32_LAUNCH
    return launch_status("gemm_f32");
}

}  // namespace sd3
