// Linear layers whose left operand has few rows (the batch; eight per launch): the adaLN modulation projections
// (modules.cpp:1384-1501 compute them one 1536-column chunk at a time with partial_linear), the timestep and
// pooled-text MLPs (modules.cpp:1664-1671). They are pure weight streaming, so one launch covers a whole list
// of weight matrices ("jobs") and reads every weight element exactly once, N-contiguous as the reference stores it.
#include <vector>

#include "common.hpp"

namespace sd3 {

template <typename WT>
struct WLoad;
template <>
struct WLoad<float> {
    static __device__ __forceinline__ void load4(const float* p, float (&w)[4]) {
        float4 v = *reinterpret_cast<const float4*>(p);
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    }
    static __device__ __forceinline__ float load1(const float* p) { return *p; }
};
template <>
struct WLoad<bf16_t> {
    static __device__ __forceinline__ void load4(const bf16_t* p, float (&w)[4]) {
        uint2 v = *reinterpret_cast<const uint2*>(p);
        w[0] = __uint_as_float(v.x << 16); w[1] = __uint_as_float(v.x & 0xffff0000u);
        w[2] = __uint_as_float(v.y << 16); w[3] = __uint_as_float(v.y & 0xffff0000u);
    }
    static __device__ __forceinline__ float load1(const bf16_t* p) { return bf16_to_f32(*p); }
};

// Block = 256 threads = 32 column groups (4 columns each, 128 columns per block) x 8 slices of K.
// x is staged transposed in LDS (xs[k][m]) so that a thread reads its M inputs for one k with wide LDS loads.
// Jobs travel as a kernel argument (no device-side table to keep coherent with the host).
struct SmallLinearJobPack {
    SmallLinearJob j[SMALL_LINEAR_JOBS_PER_LAUNCH];  // 52 x 56 bytes of kernel arguments: the 49 projections of a 24-block forward in one launch
};

template <int M, typename WT, bool VEC>
__global__ void __launch_bounds__(256) small_linear_kernel(const float* __restrict__ x_all, int m_real, int K_all, const SmallLinearJobPack jobs, int act) {
    extern __shared__ float smem[];
    const SmallLinearJob job = jobs.j[blockIdx.y];
    const int col_base = blockIdx.x * 128;
    if (col_base >= job.N) return;
    const float* __restrict__ x = job.x ? job.x : x_all;  // (uniform over the workgroup)
    const int K = job.x ? job.K : K_all;
    const int tid = threadIdx.x;
#pragma unroll
    for (int m = 0; m < M; m++)
        for (int k = tid; k < K; k += 256) smem[k * M + m] = (m < m_real) ? x[(long long)m * K + k] : 0.f;
    __syncthreads();

    const int cl = tid & 31, ks = tid >> 5;
    const int c0 = col_base + cl * 4;
    const int kper = (K + 7) / 8;
    const int kbeg = ks * kper, kend = min(K, kbeg + kper);
    const WT* W = reinterpret_cast<const WT*>(job.W) + job.n0 + c0;
    float acc[M][4];
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[m][j] = 0.f;

    constexpr int UNROLL_K = M <= 2 ? 8 : 4;
    if (c0 < job.N) {
        // weight rows in flight per thread: eight with one or two rows of x (measured: 4 and 16 are slower), four with more rows (registers)
#pragma unroll UNROLL_K
        for (int k = kbeg; k < kend; k++) {
            float w[4];
            if (VEC) {
                WLoad<WT>::load4(W + (long long)k * job.ldw, w);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) w[j] = (c0 + j < job.N) ? WLoad<WT>::load1(W + (long long)k * job.ldw + j) : 0.f;
            }
#pragma unroll
            for (int m = 0; m < M; m++) {
                const float xv = smem[k * M + m];
#pragma unroll
                for (int j = 0; j < 4; j++) acc[m][j] += xv * w[j];
            }
        }
    }
    __syncthreads();  // everyone is done with xs; reuse it for the cross-slice reduction: red[ks][m][128]
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
        for (int j = 0; j < 4; j++) smem[(ks * M + m) * 128 + cl * 4 + j] = acc[m][j];
    __syncthreads();
    for (int e = tid; e < M * 128; e += 256) {
        const int m = e >> 7, c = e & 127;
        const int col = col_base + c;
        if (m < m_real && col < job.N) {
            float s = 0.f;
#pragma unroll
            for (int s8 = 0; s8 < 8; s8++) s += smem[(s8 * M + m) * 128 + c];
            if (job.bias) s += job.bias[job.n0 + col];
            if (act == SD3_ACT_SILU) s = silu_precise(s);
            else if (act == SD3_ACT_GELU_TANH) s = gelu_tanh_precise(s);
            job.out[(long long)m * job.N + col] = s;
        }
    }
}

template <int M>
static void launch_small(const float* x, int m_real, int K, int K_max, const SmallLinearJobPack& jobs, int n_jobs, int max_N, int w_is_bf16, bool vec, int act,
                         hipStream_t st) {
    dim3 grid((max_N + 127) / 128, n_jobs), block(256);
    const int kk = K_max > 1024 ? K_max : 1024;
    const size_t smem = (size_t)kk * M * sizeof(float);
    if (w_is_bf16) {
        if (vec) hipLaunchKernelGGL((small_linear_kernel<M, bf16_t, true>), grid, block, smem, st, x, m_real, K, jobs, act);
        else hipLaunchKernelGGL((small_linear_kernel<M, bf16_t, false>), grid, block, smem, st, x, m_real, K, jobs, act);
    } else {
        if (vec) hipLaunchKernelGGL((small_linear_kernel<M, float, true>), grid, block, smem, st, x, m_real, K, jobs, act);
        else hipLaunchKernelGGL((small_linear_kernel<M, float, false>), grid, block, smem, st, x, m_real, K, jobs, act);
    }
}

int small_linear_batched(const float* x, int M, int K, const SmallLinearJob* jobs_host, int n_jobs, int w_is_bf16, int act, hipStream_t st) {
    if (M <= 0 || n_jobs <= 0) return SD3_OK;
    const int K_launch = K;  // depth of the launch's own x (jobs may bring theirs)
    for (int i = 0; i < n_jobs; i++) {
        if (!jobs_host[i].x && !x) return fail(SD3_ERR_INVALID_ARG, "small_linear: job %d has no left operand", i);
        if (jobs_host[i].x && jobs_host[i].K > K) K = jobs_host[i].K;  // from here on K is the largest depth of the launch (LDS size)
    }
    if (K <= 0 || K > 4096) return fail(SD3_ERR_UNSUPPORTED, "small_linear: K=%d out of range", K);
    // rows per launch: eight, or four when eight transposed rows of x do not fit the 64 KB of LDS a workgroup may use (K > 2048)
    const int group = ((size_t)(K > 1024 ? K : 1024) * 8 * sizeof(float) > 65536) ? 4 : 8;
    if (M > group) {
        // more rows than that (the reference's own block test runs a batch of 16, module_tests/dit_block.py:12): a group at a time, the
        // weights streamed once per group
        std::vector<SmallLinearJob> part(jobs_host, jobs_host + n_jobs);
        for (int m0 = 0; m0 < M; m0 += group) {
            for (int i = 0; i < n_jobs; i++) {
                part[i].out = jobs_host[i].out ? jobs_host[i].out + (long long)m0 * jobs_host[i].N : nullptr;
                part[i].x = jobs_host[i].x ? jobs_host[i].x + (long long)m0 * jobs_host[i].K : nullptr;
            }
            SD3_TRY(small_linear_batched(x ? x + (long long)m0 * K_launch : nullptr, M - m0 < group ? M - m0 : group, K_launch, part.data(), n_jobs, w_is_bf16, act, st));
        }
        return SD3_OK;
    }
    const int esz = w_is_bf16 ? 2 : 4;
    constexpr int PER = SMALL_LINEAR_JOBS_PER_LAUNCH;
    for (int base = 0; base < n_jobs; base += PER) {
        const int n = (n_jobs - base) < PER ? (n_jobs - base) : PER;
        SmallLinearJobPack pack;
        int max_N = 0;
        bool vec = true;
        for (int i = 0; i < n; i++) {
            pack.j[i] = jobs_host[base + i];
            const SmallLinearJob& j = pack.j[i];
            if (j.N > max_N) max_N = j.N;
            if ((j.N % 4) || (j.ldw % 4) || (j.n0 % 4) || ((reinterpret_cast<uintptr_t>(j.W) % (4 * esz)) != 0)) vec = false;
        }
        for (int i = n; i < PER; i++) pack.j[i] = SmallLinearJob{nullptr, nullptr, nullptr, 0, 0, 0, nullptr, 0};
        if (max_N == 0) continue;
        if (M == 1) launch_small<1>(x, M, K_launch, K, pack, n, max_N, w_is_bf16, vec, act, st);
        else if (M == 2) launch_small<2>(x, M, K_launch, K, pack, n, max_N, w_is_bf16, vec, act, st);
        else if (M <= 4) launch_small<4>(x, M, K_launch, K, pack, n, max_N, w_is_bf16, vec, act, st);
        else launch_small<8>(x, M, K_launch, K, pack, n, max_N, w_is_bf16, vec, act, st);
        SD3_TRY(launch_status("small_linear"));
    }
    return SD3_OK;
}

}  // namespace sd3
