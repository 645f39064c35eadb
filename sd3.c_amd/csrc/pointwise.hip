// Memory-bound kernels: LayerNorm(+adaLN modulation), per-head RMSNorm, activations, gating, embeddings,
// patch gather / scatter, casts. All are sized so that one launch streams its tensors once through HBM.
#include "common.hpp"

namespace sd3 {

static constexpr int WAVE = 64;

__device__ __forceinline__ float pos_embed_value(int a, int b, int ch, int C, int height, int width, int base_size);

template <typename T>
__device__ __forceinline__ void store4(T* p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float a, float b, float c, float d) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
}
template <typename T>
__device__ __forceinline__ void store1(T* p, float a);
template <>
__device__ __forceinline__ void store1<float>(float* p, float a) { *p = a; }
template <>
__device__ __forceinline__ void store1<bf16_t>(bf16_t* p, float a) { *p = f32_to_bf16(a); }

// One wavefront per row, the row held in registers (NV float4 per lane), two-pass mean / variance like the
// reference (modules.cpp:22-37), then up to two modulated outputs (modules.cpp:1207-1221 fused in).
template <typename OutT>
struct LnSegDev {
    const float* x;
    OutT* out;
    OutT* out2;
    const float* shift;
    const float* scale;
    const float* shift2;
    const float* scale2;
    int mod_ld, T;
    long long rows;
};
template <typename OutT>
struct LnSegPair {
    LnSegDev<OutT> s[2];  // rows [0, s[0].rows) belong to the first tensor, the rest to the second (the two streams of a block)
};
template <typename OutT, int NV>
__global__ void __launch_bounds__(256) ln_mod_vec_kernel(const LnSegPair<OutT> segs, float eps, int C) {
    const int lane = threadIdx.x & (WAVE - 1);
    // (the wavefront's index as a scalar: the row, the segment it belongs to and every pointer derived from them then live in scalar
    // registers, which keeps the kernel within 64 vector registers, i.e. at 8 wavefronts per SIMD: all rows of the latent stream at once)
    long long row = (long long)blockIdx.x * (blockDim.x / WAVE) + __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int which = row >= segs.s[0].rows ? 1 : 0;
    if (which) row -= segs.s[0].rows;
    const LnSegDev<OutT>& g = segs.s[which];
    if (row >= g.rows) return;
    const int T = g.T, mod_ld = g.mod_ld;
    OutT* __restrict__ out = g.out;
    OutT* __restrict__ out2 = g.out2;
    const int nvec = C >> 2;
    const float4* xr = reinterpret_cast<const float4*>(g.x + row * C);
    float4 v[NV];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int j = lane + i * WAVE;
        v[i] = (j < nvec) ? xr[j] : make_float4(0.f, 0.f, 0.f, 0.f);
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    const float mu = wave_sum(s) / C;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int j = lane + i * WAVE;
        if (j < nvec) {
            float a = v[i].x - mu, b = v[i].y - mu, c = v[i].z - mu, d = v[i].w - mu;
            q += (a * a + b * b) + (c * c + d * d);
        }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / C + eps);
    long long b = 0;  // batch element of the row: with at most 8 of them a few comparisons instead of a 64-bit division
    if (g.rows <= 8LL * T) {
#pragma unroll
        for (int k = 1; k < 8; k++) b += (row >= (long long)k * T) ? 1 : 0;
    } else {
        b = row / T;
    }
    const float4* sh = g.shift ? reinterpret_cast<const float4*>(g.shift + b * mod_ld) : nullptr;
    const float4* sc = g.scale ? reinterpret_cast<const float4*>(g.scale + b * mod_ld) : nullptr;
    const float4* sh2 = g.shift2 ? reinterpret_cast<const float4*>(g.shift2 + b * mod_ld) : nullptr;
    const float4* sc2 = g.scale2 ? reinterpret_cast<const float4*>(g.scale2 + b * mod_ld) : nullptr;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int j = lane + i * WAVE;
        if (j < nvec) {
            float n0 = rstd * (v[i].x - mu), n1 = rstd * (v[i].y - mu), n2 = rstd * (v[i].z - mu), n3 = rstd * (v[i].w - mu);
            if (sc) {
                float4 a = sc[j], c = sh[j];
                store4<OutT>(out + row * C + 4 * j, n0 * (1.0f + a.x) + c.x, n1 * (1.0f + a.y) + c.y, n2 * (1.0f + a.z) + c.z, n3 * (1.0f + a.w) + c.w);
            } else {
                store4<OutT>(out + row * C + 4 * j, n0, n1, n2, n3);
            }
            if (out2) {
                float4 a = sc2[j], c = sh2[j];
                store4<OutT>(out2 + row * C + 4 * j, n0 * (1.0f + a.x) + c.x, n1 * (1.0f + a.y) + c.y, n2 * (1.0f + a.z) + c.z, n3 * (1.0f + a.w) + c.w);
            }
        }
    }
}

// Any C: one wavefront per row, the row re-read from cache for each pass. Also the full reference signature
// (optional affine weight/bias, optional saved mean/rstd; modules.cpp:10-49).
template <typename OutT>
__global__ void __launch_bounds__(256) ln_mod_generic_kernel(const float* __restrict__ x, OutT* __restrict__ out, OutT* __restrict__ out2,
                                                             const float* __restrict__ shift, const float* __restrict__ scale,
                                                             const float* __restrict__ shift2, const float* __restrict__ scale2, int mod_ld,
                                                             const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ mean,
                                                             float* __restrict__ rstd_out, float eps, long long rows, int T, int C) {
    const int lane = threadIdx.x & (WAVE - 1);
    const long long row = (long long)blockIdx.x * (blockDim.x / WAVE) + (threadIdx.x / WAVE);
    if (row >= rows) return;
    const float* xr = x + row * C;
    float s = 0.f;
    for (int j = lane; j < C; j += WAVE) s += xr[j];
    const float mu = wave_sum(s) / C;
    float q = 0.f;
    for (int j = lane; j < C; j += WAVE) {
        float d = xr[j] - mu;
        q += d * d;
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / C + eps);
    if (lane == 0) {
        if (mean) mean[row] = mu;
        if (rstd_out) rstd_out[row] = rstd;
    }
    const long long b = row / T;
    for (int j = lane; j < C; j += WAVE) {
        float n = rstd * (xr[j] - mu);
        float o = n;
        if (w) o *= w[j];
        if (bias) o += bias[j];
        if (scale) o = o * (1.0f + scale[b * mod_ld + j]) + shift[b * mod_ld + j];
        store1<OutT>(out + row * C + j, o);
        if (out2) store1<OutT>(out2 + row * C + j, n * (1.0f + scale2[b * mod_ld + j]) + shift2[b * mod_ld + j]);
    }
}

template <typename OutT>
static bool ln_seg_vectorisable(const LnSegDev<OutT>& g, int C) {
    auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    return (C % 4 == 0) && (C <= 3072) && (g.mod_ld % 4 == 0) && al(g.x) && al(g.out) && al(g.out2) && al(g.shift) && al(g.scale) && al(g.shift2) &&
           al(g.scale2);
}
template <typename OutT>
static int ln_mod_launch_vec(const LnSegPair<OutT>& segs, float eps, int C, hipStream_t st) {
    const int wpb = 4;
    const long long rows = segs.s[0].rows + segs.s[1].rows;
    dim3 grid((unsigned)((rows + wpb - 1) / wpb)), block(wpb * WAVE);
    const int nv = (C / 4 + WAVE - 1) / WAVE;
#define SD3_LN_CASE(N)                                                                       \
    case N:                                                                                  \
        hipLaunchKernelGGL((ln_mod_vec_kernel<OutT, N>), grid, block, 0, st, segs, eps, C); \
        break;
    switch (nv) { SD3_LN_CASE(1) SD3_LN_CASE(2) SD3_LN_CASE(3) SD3_LN_CASE(4) SD3_LN_CASE(5) SD3_LN_CASE(6) SD3_LN_CASE(7) SD3_LN_CASE(8)
                  SD3_LN_CASE(9) SD3_LN_CASE(10) SD3_LN_CASE(11) SD3_LN_CASE(12) }
#undef SD3_LN_CASE
    return launch_status("layernorm_modulate");
}
template <typename OutT>
static int ln_mod_dispatch(const LnSegDev<OutT>& g, float eps, int C, hipStream_t st) {
    if (g.rows == 0) return SD3_OK;
    if (ln_seg_vectorisable(g, C)) {
        LnSegPair<OutT> segs{};
        segs.s[0] = g;
        return ln_mod_launch_vec(segs, eps, C, st);
    }
    const int wpb = 4;
    dim3 grid((unsigned)((g.rows + wpb - 1) / wpb)), block(wpb * WAVE);
    hipLaunchKernelGGL((ln_mod_generic_kernel<OutT>), grid, block, 0, st, g.x, g.out, g.out2, g.shift, g.scale, g.shift2, g.scale2, g.mod_ld, nullptr, nullptr,
                       nullptr, nullptr, eps, g.rows, g.T, C);
    return launch_status("layernorm_modulate");
}
template <typename OutT>
static int ln_mod_pair_t(const LayerNormJob* jobs, int n, float eps, int C, hipStream_t st) {
    LnSegDev<OutT> g[2];
    int m = 0;
    for (int i = 0; i < n; i++) {
        const LayerNormJob& j = jobs[i];
        const long long rows = (long long)j.B * j.T;
        if (rows == 0) continue;
        g[m++] = LnSegDev<OutT>{j.x, (OutT*)j.out, (OutT*)j.out2, j.shift, j.scale, j.shift2, j.scale2, j.mod_ld, j.T, rows};
    }
    if (m == 2 && ln_seg_vectorisable(g[0], C) && ln_seg_vectorisable(g[1], C)) {
        LnSegPair<OutT> segs{};
        segs.s[0] = g[0];
        segs.s[1] = g[1];
        return ln_mod_launch_vec(segs, eps, C, st);  // the few rows of the second tensor ride along instead of paying a launch
    }
    for (int i = 0; i < m; i++) SD3_TRY(ln_mod_dispatch(g[i], eps, C, st));
    return SD3_OK;
}

int layernorm_modulate(const float* x, void* out, void* out2, const float* shift, const float* scale, const float* shift2, const float* scale2,
                       int mod_ld, float eps, int B, int T, int C, int out_bf16, hipStream_t st) {
    const LayerNormJob j{x, out, out2, shift, scale, shift2, scale2, mod_ld, B, T};
    return layernorm_modulate_pair(&j, 1, eps, C, out_bf16, st);
}

int layernorm_modulate_pair(const LayerNormJob* jobs, int n, float eps, int C, int out_bf16, hipStream_t st) {
    if (n < 1 || n > 2) return fail(SD3_ERR_INVALID_ARG, "layernorm_modulate_pair: 1 or 2 tensors (got %d)", n);
    return out_bf16 ? ln_mod_pair_t<bf16_t>(jobs, n, eps, C, st) : ln_mod_pair_t<float>(jobs, n, eps, C, st);
}

int layernorm_full(const float* x, float* y, float* mean, float* rstd, const float* w, const float* bias, float eps, long long rows, int C,
                   hipStream_t st) {
    if (rows == 0) return SD3_OK;
    const int wpb = 4;
    dim3 grid((unsigned)((rows + wpb - 1) / wpb)), block(wpb * WAVE);
    hipLaunchKernelGGL((ln_mod_generic_kernel<float>), grid, block, 0, st, x, y, (float*)nullptr, (const float*)nullptr, (const float*)nullptr,
                       (const float*)nullptr, (const float*)nullptr, 0, w, bias, mean, rstd, eps, rows, 1, C);
    return launch_status("layernorm");
}

// Per-(row, group) RMSNorm over `hs` consecutive values (modules.cpp:154-198); 16 lanes per (row, group). Used by
// the fp32 path and the stand-alone operator (the bf16 path applies the norm inside the attention kernel).
__global__ void __launch_bounds__(256) rmsnorm_rows_kernel(const float* __restrict__ x, float* __restrict__ y, const float* __restrict__ w,
                                                           float* __restrict__ rms, float eps, long long n_groups_total, int groups, int hs, int ld_in,
                                                           int ld_out) {
    const int sub = threadIdx.x & 15;
    const long long g = ((long long)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    if (g >= n_groups_total) return;  // whole 16-lane group exits together
    const long long row = g / groups;
    const int grp = (int)(g % groups);
    const float* xr = x + row * ld_in + (long long)grp * hs;
    float* yr = y + row * ld_out + (long long)grp * hs;
    float s = 0.f;
    for (int j = sub; j < hs; j += 16) s += xr[j] * xr[j];
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) s += __shfl_xor(s, o, 16);
    const float inv = 1.0f / sqrtf(eps + s / hs);
    if (rms && sub == 0) rms[g] = inv;
    for (int j = sub; j < hs; j += 16) {
        float v = xr[j] * inv;
        if (w) v *= w[j];
        yr[j] = v;
    }
}

int rmsnorm_rows(const float* x, float* y, const float* w, float* rms, float eps, long long rows, int groups, int hs, int ld_in, int ld_out,
                 hipStream_t st) {
    const long long total = rows * groups;
    if (total == 0) return SD3_OK;
    const long long threads = total * 16;
    dim3 grid((unsigned)((threads + 255) / 256)), block(256);
    hipLaunchKernelGGL(rmsnorm_rows_kernel, grid, block, 0, st, x, y, w, rms, eps, total, groups, hs, ld_in, ld_out);
    return launch_status("rmsnorm");
}

// ---- elementwise ----
template <int OP>  // 0 silu, 1 gelu_tanh, 2 gelu (erf form, modules.cpp:280-285)
__global__ void __launch_bounds__(256) unary_kernel(const float* __restrict__ in, float* __restrict__ out, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        const float v = in[i];
        out[i] = (OP == 0) ? silu_precise(v) : (OP == 1) ? gelu_tanh_precise(v) : 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
    }
}
static unsigned grid_for(long long n, int per_block = 256, unsigned cap = 256 * 64) {
    long long g = (n + per_block - 1) / per_block;
    return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}
int unary_op(const float* in, float* out, long long n, int act, hipStream_t st) {
    if (n == 0) return SD3_OK;
    if (act == SD3_ACT_SILU) hipLaunchKernelGGL((unary_kernel<0>), dim3(grid_for(n)), dim3(256), 0, st, in, out, n);
    else if (act == SD3_ACT_GELU_ERF) hipLaunchKernelGGL((unary_kernel<2>), dim3(grid_for(n)), dim3(256), 0, st, in, out, n);
    else hipLaunchKernelGGL((unary_kernel<1>), dim3(grid_for(n)), dim3(256), 0, st, in, out, n);
    return launch_status("activation");
}

template <int SILU>
__global__ void __launch_bounds__(256) add_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ out, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        float v = a[i] + b[i];
        out[i] = SILU ? silu_precise(v) : v;
    }
}
int add_op(const float* a, const float* b, float* out, long long n, hipStream_t st) {
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL((add_kernel<0>), dim3(grid_for(n)), dim3(256), 0, st, a, b, out, n);
    return launch_status("add");
}
int add_silu_op(const float* a, const float* b, float* out, long long n, hipStream_t st) {
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL((add_kernel<1>), dim3(grid_for(n)), dim3(256), 0, st, a, b, out, n);
    return launch_status("add_silu");
}

// out = in*(1+scale[b,c]) + shift[b,c]  (scale != null)   or   out = in*gate[b,c]  (scale == null, `shift` is the gate)
__global__ void __launch_bounds__(256) modulate_kernel(const float* __restrict__ in, float* __restrict__ out, const float* __restrict__ shift,
                                                       const float* __restrict__ scale, long long n, long long TC, int C) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        const long long b = i / TC;
        const int c = (int)(i % C);
        const float v = in[i];
        out[i] = scale ? v * (1.0f + scale[b * C + c]) + shift[b * C + c] : v * shift[b * C + c];
    }
}
int modulate_op(const float* in, float* out, const float* shift, const float* scale, int B, int T, int C, hipStream_t st) {
    const long long n = (long long)B * T * C;
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(modulate_kernel, dim3(grid_for(n)), dim3(256), 0, st, in, out, shift, scale, n, (long long)T * C, C);
    return launch_status("scale_and_shift");
}
int gate_op(const float* in, float* out, const float* gate, int B, int T, int C, hipStream_t st) { return modulate_op(in, out, gate, nullptr, B, T, C, st); }

__global__ void __launch_bounds__(256) copy_rows_kernel(const float* __restrict__ in, long long in_bs, float* __restrict__ out, long long out_bs,
                                                        long long n_per_batch) {
    const int b = blockIdx.y;
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n_per_batch; i += stride) out[b * out_bs + i] = in[b * in_bs + i];
}
int copy_rows(const float* in, long long in_bs, float* out, long long out_bs, int B, long long n_per_batch, hipStream_t st) {
    if (B == 0 || n_per_batch == 0) return SD3_OK;
    hipLaunchKernelGGL(copy_rows_kernel, dim3(grid_for(n_per_batch, 256, 4096), B), dim3(256), 0, st, in, in_bs, out, out_bs, n_per_batch);
    return launch_status("copy_rows");
}

__global__ void __launch_bounds__(256) cast_bf16_kernel(const float* __restrict__ in, bf16_t* __restrict__ out, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += stride) out[i] = f32_to_bf16(in[i]);
}
int cast_f32_to_bf16(const float* in, bf16_t* out, long long n, hipStream_t st) {
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(cast_bf16_kernel, dim3(grid_for(n)), dim3(256), 0, st, in, out, n);
    return launch_status("cast_f32_to_bf16");
}

// (K,N) fp32 -> (N,K) bf16 or fp32 through a 32x33 LDS tile so that both sides are coalesced.
template <typename OutT>
__global__ void __launch_bounds__(256) pack_weight_kernel(const float* __restrict__ W, OutT* __restrict__ out, int K, int N) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    const int n0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
    for (int r = ty; r < 32; r += 8) {
        int k = k0 + r, n = n0 + tx;
        tile[r][tx] = (k < K && n < N) ? W[(long long)k * N + n] : 0.f;
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        int n = n0 + r, k = k0 + tx;
        if (n < N && k < K) store1<OutT>(out + (long long)n * K + k, tile[tx][r]);
    }
}
int pack_weight_bf16(const float* W, bf16_t* out, int K, int N, hipStream_t st) {
    if (K == 0 || N == 0) return SD3_OK;
    hipLaunchKernelGGL((pack_weight_kernel<bf16_t>), dim3((N + 31) / 32, (K + 31) / 32), dim3(256), 0, st, W, out, K, N);
    return launch_status("pack_weight_bf16");
}
int transpose_f32(const float* W, float* out, int K, int N, hipStream_t st) {
    if (K == 0 || N == 0) return SD3_OK;
    hipLaunchKernelGGL((pack_weight_kernel<float>), dim3((N + 31) / 32, (K + 31) / 32), dim3(256), 0, st, W, out, K, N);
    return launch_status("transpose_f32");
}

// Stand-alone patch embedding (modules.cpp:1093-1117): one thread per output element, the patch gathered on the fly,
// the position value evaluated in place. The model forward uses im2col + GEMM with a cached table instead.
__global__ void __launch_bounds__(256) patch_embed_direct_kernel(const float* __restrict__ latent, float* __restrict__ out,
                                                                 const float* __restrict__ kernel, const float* __restrict__ bias, int B, int H, int W,
                                                                 int Cin, int C, int p, int hp, int wp, int pos_max, int base_size, long long n) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int ch = (int)(idx % C);
    const long long m = idx / C;
    const int j = (int)(m % wp), i = (int)((m / wp) % hp), b = (int)(m / ((long long)wp * hp));
    float total = 0.f;
    for (int ic = 0; ic < Cin; ic++) {
        float acc = 0.f;
        for (int r = 0; r < p; r++)
            for (int s = 0; s < p; s++)
                acc += kernel[(((long long)ch * Cin + ic) * p + r) * p + s] * latent[(((long long)b * Cin + ic) * H + (i * p + r)) * W + (j * p + s)];
        total += acc;
    }
    const int oh = (pos_max - hp) / 2, ow = (pos_max - wp) / 2;
    out[idx] = (total + bias[ch]) + pos_embed_value(i + oh, j + ow, ch, C, pos_max, pos_max, base_size);
}
int patch_embed_direct(const float* latent, float* out, const float* kernel, const float* bias, int B, int H, int W, int Cin, int C, int p, int pos_max,
                       int base_height, hipStream_t st) {
    const int hp = (H - p) / p + 1, wp = (W - p) / p + 1;
    const long long n = (long long)B * hp * wp * C;
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(patch_embed_direct_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, latent, out, kernel, bias, B, H, W, Cin, C, p, hp,
                       wp, pos_max, base_height / p, n);
    return launch_status("patch_embedding");
}

// ---- embeddings ----
// modules.cpp:920-944: out[b, i] = cos(f_i t_b), out[b, half+i] = sin(f_i t_b), f_i = exp(-ln(1e4) * 2i / dim)
__global__ void timestep_embedding_kernel(const float* __restrict__ t, float* __restrict__ out, int B, int dim) {
    const int half = dim / 2;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= B * half) return;
    const int b = idx / half, i = idx % half;
    const float freq = expf(-logf(10000.0f) * 2 * i / dim);
    const float a = freq * t[b];
    out[(long long)b * dim + i] = cosf(a);
    out[(long long)b * dim + half + i] = sinf(a);
}
int timestep_embedding(const float* t, float* out, int B, int dim, hipStream_t st) {
    const int n = B * (dim / 2);
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(timestep_embedding_kernel, dim3((n + 255) / 256), dim3(256), 0, st, t, out, B, dim);
    return launch_status("sinusoidal_embedding");
}

// modules.cpp:946-975 evaluated in fp64. The reference stores the table with its "w" loop variable as the slow
// index. Entry (a, b): a = slow index (scaled by base/width), b = fast index (scaled by base/height); the four
// channel quarters are [sin b, cos b, sin a, cos a].
__device__ __forceinline__ float pos_embed_value(int a, int b, int ch, int C, int height, int width, int base_size) {
    const int q = C / 4;
    const int part = ch / q, i = ch % q;
    const double freq = 1.0 / pow(10000.0, (double)4 * i / C);
    const double pos = (part < 2) ? (double)(b * base_size) / height : (double)(a * base_size) / width;
    const double ang = pos * freq;
    return (float)((part & 1) ? cos(ang) : sin(ang));
}
__global__ void __launch_bounds__(256) pos_embed_table_kernel(float* __restrict__ out, int C, int height, int width, int base_size, long long n) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int ch = (int)(idx % C);
    const long long p = idx / C;
    const int b = (int)(p % height), a = (int)(p / height);
    out[idx] = pos_embed_value(a, b, ch, C, height, width, base_size);
}
int pos_embed_table(float* out, int C, int height, int width, int base_size, hipStream_t st) {
    const long long n = (long long)height * width * C;
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(pos_embed_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, out, C, height, width, base_size, n);
    return launch_status("positional_embedding2D");
}
// modules.cpp:977-995: out[i, j, :] = table[i + off_h, j + off_w, :] with the table read as [row][col]
__global__ void __launch_bounds__(256) pos_embed_crop_kernel(const float* __restrict__ table, float* __restrict__ out, int max_size, int h, int w, int C,
                                                             long long n) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int ch = (int)(idx % C);
    const long long p = idx / C;
    const int j = (int)(p % w), i = (int)(p / w);
    const int oh = (max_size - h) / 2, ow = (max_size - w) / 2;
    out[idx] = table[((long long)(i + oh) * max_size + (j + ow)) * C + ch];
}
int pos_embed_crop(const float* table, float* out, int max_size, int h, int w, int C, hipStream_t st) {
    const long long n = (long long)h * w * C;
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(pos_embed_crop_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, table, out, max_size, h, w, C, n);
    return launch_status("crop_positional_embedding2D");
}
// Cropped table generated directly: token (i, j) of the h x w grid reads table row (i+off_h), column (j+off_w), i.e.
// slow index a = i+off_h, fast index b = j+off_w of a (max_size x max_size) table.
__global__ void __launch_bounds__(256) pos_embed_cropped_kernel(float* __restrict__ out, int C, int max_size, int base_size, int h, int w, long long n) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int ch = (int)(idx % C);
    const long long p = idx / C;
    const int j = (int)(p % w), i = (int)(p / w);
    const int oh = (max_size - h) / 2, ow = (max_size - w) / 2;
    out[idx] = pos_embed_value(i + oh, j + ow, ch, C, max_size, max_size, base_size);
}
int pos_embed_cropped(float* out, int C, int max_size, int base_size, int h, int w, hipStream_t st) {
    const long long n = (long long)h * w * C;
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(pos_embed_cropped_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, out, C, max_size, base_size, h, w, n);
    return launch_status("pos_embed_cropped");
}

// ---- convolution (stand-alone operator; the model's patch embedding goes through im2col + GEMM) ----
__global__ void __launch_bounds__(256) conv2d_kernel(const float* __restrict__ in, float* __restrict__ out, const float* __restrict__ kernel,
                                                     const float* __restrict__ bias, int B, int kh, int kw, int Cin, int Cout, int ih, int iw, int oh,
                                                     int ow, int stride, int pad, long long n) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int x = (int)(idx % ow);
    const int y = (int)((idx / ow) % oh);
    const int oc = (int)((idx / ((long long)ow * oh)) % Cout);
    const int b = (int)(idx / ((long long)ow * oh * Cout));
    float total = 0.f;
    for (int ic = 0; ic < Cin; ic++) {
        const float* src = in + ((long long)b * Cin + ic) * ih * iw;
        const float* ker = kernel + ((long long)oc * Cin + ic) * kh * kw;
        float acc = 0.f;
        for (int r = 0; r < kh; r++)
            for (int s = 0; s < kw; s++) {
                const int yy = y * stride + r - pad, xx = x * stride + s - pad;
                if (yy >= 0 && yy < ih && xx >= 0 && xx < iw) acc += ker[r * kw + s] * src[(long long)yy * iw + xx];
            }
        total += acc;
    }
    out[idx] = total + bias[oc];
}
int conv2d_direct(const float* in, float* out, const float* kernel, const float* bias, int B, int kh, int kw, int Cin, int Cout, int ih, int iw, int oh,
                  int ow, int stride, int pad, hipStream_t st) {
    const long long n = (long long)B * Cout * oh * ow;
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(conv2d_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, in, out, kernel, bias, B, kh, kw, Cin, Cout, ih, iw, oh, ow,
                       stride, pad, n);
    return launch_status("conv2d");
}

template <typename OutT>
__global__ void __launch_bounds__(256) im2col_kernel(const float* __restrict__ latent, OutT* __restrict__ out, int B, int Cin, int H, int W, int p, int hp,
                                                     int wp, long long n) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int Kc = Cin * p * p;
    const int k = (int)(idx % Kc);
    const long long m = idx / Kc;
    const int s = k % p, r = (k / p) % p, ic = k / (p * p);
    const int j = (int)(m % wp), i = (int)((m / wp) % hp), b = (int)(m / ((long long)wp * hp));
    store1<OutT>(out + idx, latent[(((long long)b * Cin + ic) * H + (i * p + r)) * W + (j * p + s)]);
}
int im2col_patches(const float* latent, void* out, int out_bf16, int B, int Cin, int H, int W, int p, hipStream_t st) {
    const int hp = (H - p) / p + 1, wp = (W - p) / p + 1;
    const long long n = (long long)B * hp * wp * Cin * p * p;
    if (n == 0) return SD3_OK;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (out_bf16) hipLaunchKernelGGL((im2col_kernel<bf16_t>), grid, block, 0, st, latent, (bf16_t*)out, B, Cin, H, W, p, hp, wp, n);
    else hipLaunchKernelGGL((im2col_kernel<float>), grid, block, 0, st, latent, (float*)out, B, Cin, H, W, p, hp, wp, n);
    return launch_status("im2col_patches");
}

// modules.cpp:1730-1752: out[b, ch, hp*p+ph, wp*p+pw] = tokens[b, hp*Wp+wp, (ph*p+pw)*Cin + ch]
// CFG: the batch holds [n unconditional ; n conditional] samples and the kernel writes, for each of the n samples, the
// latent after classifier-free guidance and one Euler step of the flow-matching sampler:
//   out = latent + dsigma * (v_u + guidance * (v_c - v_u))          (no counterpart in the reference, which stops at v)
template <bool CFG>
__global__ void __launch_bounds__(256) unpatchify_kernel(const float* __restrict__ tokens, const float* __restrict__ latent, float* __restrict__ out,
                                                         int B, int Cin, int H, int W, int p, int Hp, int Wp, long long n, float guidance, float dsigma) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int w = (int)(idx % W), h = (int)((idx / W) % H);
    const int ch = (int)((idx / ((long long)W * H)) % Cin), b = (int)(idx / ((long long)W * H * Cin));
    const int hp = h / p, ph = h % p, wq = w / p, pw = w % p;
    const bool inside = hp < Hp && wq < Wp;
    const long long tok = ((long long)hp * Wp + wq) * (p * p * Cin) + (ph * p + pw) * Cin + ch, per_sample = (long long)Hp * Wp * (p * p * Cin);
    if (!CFG) {
        out[idx] = inside ? tokens[(long long)b * per_sample + tok] : 0.f;
    } else {
        const float vu = inside ? tokens[(long long)b * per_sample + tok] : 0.f;
        const float vc = inside ? tokens[(long long)(b + B) * per_sample + tok] : 0.f;
        out[idx] = latent[idx] + dsigma * (vu + guidance * (vc - vu));
    }
}
int unpatchify(const float* tokens, float* out, int B, int Cin, int H, int W, int p, hipStream_t st) {
    const int Hp = (H - p) / p + 1, Wp = (W - p) / p + 1;
    const long long n = (long long)B * Cin * H * W;
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(unpatchify_kernel<false>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, tokens, nullptr, out, B, Cin, H, W, p, Hp, Wp, n, 0.f, 0.f);
    return launch_status("unpatchify");
}
int unpatchify_cfg_euler(const float* tokens, const float* latent, float* out, int n_samples, int Cin, int H, int W, int p, float guidance, float dsigma,
                         hipStream_t st) {
    const int Hp = (H - p) / p + 1, Wp = (W - p) / p + 1;
    const long long n = (long long)n_samples * Cin * H * W;
    if (n == 0) return SD3_OK;
    hipLaunchKernelGGL(unpatchify_kernel<true>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, tokens, latent, out, n_samples, Cin, H, W, p, Hp, Wp, n,
                       guidance, dsigma);
    return launch_status("unpatchify_cfg_euler");
}

}  // namespace sd3

// ---- OCP fp8 (e4m3) quantisation for the fp8 GEMM ----
namespace sd3 {
namespace {
constexpr float FP8_MAX = 448.0f;  // largest finite e4m3 value

__device__ __forceinline__ uint32_t pack_fp8x4(float a, float b, float c, float d) {
    int v = 0;
    v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, v, false);
    v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
    return (uint32_t)v;
}

// one wavefront per row: amax[m] = max_k |A[m][k]|
__global__ void __launch_bounds__(256) row_amax_bf16_kernel(const bf16_t* __restrict__ A, float* __restrict__ amax, int M, int K) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= M) return;
    const uint2* p = reinterpret_cast<const uint2*>(A + (long long)row * K);  // 4 bf16 per load (K % 4 == 0)
    float mx = 0.f;
    for (int i = lane; i < K / 4; i += 64) {
        const uint2 v = p[i];
        mx = fmaxf(mx, fmaxf(fmaxf(fabsf(__uint_as_float(v.x << 16)), fabsf(__uint_as_float(v.x & 0xffff0000u))),
                             fmaxf(fabsf(__uint_as_float(v.y << 16)), fabsf(__uint_as_float(v.y & 0xffff0000u)))));
    }
    mx = wave_max(mx);
    if (lane == 0) amax[row] = mx;
}
// vals[i] <- max over all i (one workgroup; fixed order, so the result does not depend on timing)
__global__ void __launch_bounds__(1024) broadcast_max_kernel(float* __restrict__ vals, int n) {
    __shared__ float part[16];
    float mx = 0.f;
    for (int i = threadIdx.x; i < n; i += 1024) mx = fmaxf(mx, vals[i]);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = 0.f;
    for (int i = 0; i < 16; i++) mx = fmaxf(mx, part[i]);
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += 1024) vals[i] = mx;
}
// aq[m][k] = fp8(A[m][k] / s), s = amax[m] / 448 (1 for an all-zero row); amax[m] is overwritten with s
__global__ void __launch_bounds__(256) quantize_rows_fp8_kernel(const bf16_t* __restrict__ A, uint8_t* __restrict__ aq, float* __restrict__ amax, int M, int K) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= M) return;
    const float mx = amax[row];
    const float s = mx > 0.f ? mx * (1.0f / FP8_MAX) : 1.0f, inv = 1.0f / s;
    const uint2* p = reinterpret_cast<const uint2*>(A + (long long)row * K);
    uint32_t* o = reinterpret_cast<uint32_t*>(aq + (long long)row * K);
    for (int i = lane; i < K / 4; i += 64) {
        const uint2 v = p[i];
        o[i] = pack_fp8x4(__uint_as_float(v.x << 16) * inv, __uint_as_float(v.x & 0xffff0000u) * inv, __uint_as_float(v.y << 16) * inv,
                          __uint_as_float(v.y & 0xffff0000u) * inv);
    }
    __builtin_amdgcn_wave_barrier();  // every lane has read amax[row] before lane 0 replaces it
    if (lane == 0) amax[row] = s;
}
// column n of a (K,N) fp32 weight: amax[n] = max_k |W[k][n]|; one thread per column, rows walked together so reads stay coalesced
__global__ void __launch_bounds__(256) col_amax_f32_kernel(const float* __restrict__ W, float* __restrict__ amax, int K, int N) {
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    float mx = 0.f;
    for (int k = 0; k < K; k++) mx = fmaxf(mx, fabsf(W[(long long)k * N + n]));
    amax[n] = mx;
}
// (K,N) fp32 -> (N,K) fp8 through a 32x33 LDS tile, each column divided by its factor s[n] = amax[n] / 448
__global__ void __launch_bounds__(256) pack_weight_fp8_kernel(const float* __restrict__ W, uint8_t* __restrict__ out, const float* __restrict__ amax, int K,
                                                              int N) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int n0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
    for (int r = ty; r < 32; r += 8) {
        const int k = k0 + r, n = n0 + tx;
        float v = 0.f;
        if (k < K && n < N) {
            const float mx = amax[n];
            v = W[(long long)k * N + n] * (mx > 0.f ? FP8_MAX / mx : 1.0f);
        }
        tile[r][tx] = v;
    }
    __syncthreads();
    // 8 threads per output row (n), 4 consecutive k each
    const int r = threadIdx.x >> 3, k4 = (threadIdx.x & 7) * 4;
    const int n = n0 + r, k = k0 + k4;
    if (n < N && k < K) *reinterpret_cast<uint32_t*>(out + (long long)n * K + k) = pack_fp8x4(tile[k4][r], tile[k4 + 1][r], tile[k4 + 2][r], tile[k4 + 3][r]);
}
__global__ void __launch_bounds__(256) amax_to_scale_kernel(float* __restrict__ v, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) v[i] = v[i] > 0.f ? v[i] * (1.0f / FP8_MAX) : 1.0f;
}
}  // namespace

int quantize_rows_fp8(const bf16_t* A, uint8_t* aq, float* scale, int M, int K, int per_tensor, hipStream_t st) {
    if (M <= 0) return SD3_OK;
    if (K <= 0 || K % 4) return fail(SD3_ERR_UNSUPPORTED, "quantize_rows_fp8: K=%d must be a positive multiple of 4", K);
    hipLaunchKernelGGL(row_amax_bf16_kernel, dim3((M + 3) / 4), dim3(256), 0, st, A, scale, M, K);
    if (per_tensor) hipLaunchKernelGGL(broadcast_max_kernel, dim3(1), dim3(1024), 0, st, scale, M);
    hipLaunchKernelGGL(quantize_rows_fp8_kernel, dim3((M + 3) / 4), dim3(256), 0, st, A, aq, scale, M, K);
    return launch_status("quantize_rows_fp8");
}
int quantize_weight_fp8(const float* W, uint8_t* wq, float* scale, int K, int N, int per_tensor, hipStream_t st) {
    if (K <= 0 || N <= 0) return SD3_OK;
    if (K % 4) return fail(SD3_ERR_UNSUPPORTED, "quantize_weight_fp8: K=%d must be a multiple of 4", K);
    hipLaunchKernelGGL(col_amax_f32_kernel, dim3((N + 255) / 256), dim3(256), 0, st, W, scale, K, N);
    if (per_tensor) hipLaunchKernelGGL(broadcast_max_kernel, dim3(1), dim3(1024), 0, st, scale, N);
    hipLaunchKernelGGL(pack_weight_fp8_kernel, dim3((N + 31) / 32, (K + 31) / 32), dim3(256), 0, st, W, wq, scale, K, N);
    hipLaunchKernelGGL(amax_to_scale_kernel, dim3((N + 255) / 256), dim3(256), 0, st, scale, N);
    return launch_status("quantize_weight_fp8");
}
}  // namespace sd3
