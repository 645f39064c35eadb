// Shared declarations of the HIP library: status/error plumbing, bf16 helpers, kernel launchers.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/sd3_hip.h"

namespace sd3 {

// ---- error plumbing (thread-local message, never exit) ----
int fail(int status, const char* fmt, ...);
void set_error(const char* msg);

#define SD3_HIP_TRY(expr)                                                                                       \
    do {                                                                                                        \
        hipError_t e_ = (expr);                                                                                 \
        if (e_ != hipSuccess) return ::sd3::fail(SD3_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
    } while (0)
#define SD3_TRY(expr)               \
    do {                            \
        int s_ = (expr);            \
        if (s_ != SD3_OK) return s_; \
    } while (0)
#define SD3_REQUIRE(cond, ...)                                           \
    do {                                                                 \
        if (!(cond)) return ::sd3::fail(SD3_ERR_INVALID_ARG, __VA_ARGS__); \
    } while (0)

inline int launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SD3_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
    return SD3_OK;
}

// ---- bf16 as raw 16-bit storage ----
typedef uint16_t bf16_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
// fp32 -> bf16, round to nearest even (the gfx950 v_cvt_pk_bf16_f32 instruction)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    const __bf16 r = (__bf16)f;
    return __builtin_bit_cast(bf16_t, r);
}
__device__ __forceinline__ float bf16_to_f32(bf16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// tanh-GELU in 8 full-rate operations: 0.5 x (1 + tanh(u)) = x * sigmoid(2u) = x / (1 + 2^(-2u log2 e)),
// u = sqrt(2/pi) (x + 0.044715 x^3). Saturates cleanly: the exponential overflows to +inf -> 0, or underflows to 0 -> x.
__device__ __forceinline__ float gelu_tanh_f(float x) {
    const float k1 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;  // -2 sqrt(2/pi) log2(e)
    const float k3 = k1 * 0.044715f;
    const float x2 = x * x;
    const float e = __builtin_amdgcn_exp2f(x * (k3 * x2 + k1));
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float gelu_tanh_precise(float x) {
    const float p = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(p * (x + 0.044715f * x * x * x)));
}
__device__ __forceinline__ float silu_precise(float x) { return x / (1.0f + expf(-x)); }

// the value of another lane of the same row of 16 lanes, chosen by a DPP control word (no trip through the LDS crossbar)
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// ---- epilogues of the GEMM kernels ----
enum Epilogue : int {
    EPI_BIAS = 0,         // out = acc + bias
    EPI_BIAS_GELU = 1,    // out = gelu_tanh(acc + bias)
    EPI_BIAS_SILU = 2,    // out = silu(acc + bias)
    EPI_GATE_RESID = 3,   // out = resid + gate[m / rows_per_batch][n] * (acc + bias)   (out may alias resid)
    EPI_BIAS_ROWADD = 4,  // out = acc + bias + table[m % rows_per_batch][n]
    EPI_QKV_NORM = 5,     // packed q|k|v projection (N = 3C): acc + bias, then per-head RMSNorm (64 columns, eps 1e-6) of the q and k thirds
                          // with weights `gate` (q) and `resid` (k), each 64 floats; C is given in gate_ld
};

struct GemmEpilogueArgs {
    const float* bias = nullptr;   // (N) or null
    const float* gate = nullptr;   // (B, gate_ld) for EPI_GATE_RESID
    int gate_ld = 0;
    const float* resid = nullptr;  // (M, ldc) fp32 for EPI_GATE_RESID
    const float* table = nullptr;  // (rows_per_batch, N) for EPI_BIAS_ROWADD
    int rows_per_batch = 1;
    const float* a_scale = nullptr;  // fp8 GEMM: factor per row of A (M) and per output column (N); null = 1
    const float* w_scale = nullptr;
};

// fp32 GEMM on the fp32 MFMA units: out(M,N) = A(M,K; lda) @ W(K, ldw)[:, n0:n0+N] (+ epilogue); out fp32 with row stride ldc.
int gemm_f32(const float* A, int lda, const float* W, int ldw, int n0, float* out, int ldc, int M, int N, int K, int epi, const GemmEpilogueArgs& ea,
             hipStream_t st);
// bf16 GEMM: A bf16 (M,K) row-major; Wp = packed weight, bf16 (N,K) K-contiguous; out bf16 (out_is_f32 = 0) or fp32.
int gemm_bf16(const bf16_t* A, const bf16_t* Wp, void* out, int out_is_f32, int ldc, int M, int N, int K, int epi, const GemmEpilogueArgs& ea,
              hipStream_t st);
// Up to three independent bf16 GEMMs (same epilogue kind and output type) in one launch.
struct GemmBf16Problem {
    const bf16_t* A;
    const bf16_t* Wp;
    void* out;
    int ldc, M, N, K;
    GemmEpilogueArgs ea;
};
extern std::atomic<long long> g_gemm_bf16_launches;  // kernels launched by the bf16 GEMM so far (for per-launch profile figures)
int gemm_bf16_grouped(const GemmBf16Problem* probs, int n, int out_is_f32, int epi, hipStream_t st);
// The same with OCP fp8 (e4m3) operands: A (M,K) and Wp (N,K) are bytes, K % 128 == 0, and the accumulators are multiplied by
// ea.a_scale[m] * ea.w_scale[n] before the epilogue (epilogues: bias, bias+GELU, gate+residual, q|k|v with qk-norm).
int gemm_fp8_grouped(const GemmBf16Problem* probs, int n, int out_is_f32, int epi, hipStream_t st);
// fp8 quantisation. Rows of a bf16 matrix: aq[m][k] = fp8(A[m][k] / s[m]), s[m] = max_k |A[m][k]| / 448 (one common s with per_tensor).
int quantize_rows_fp8(const bf16_t* A, uint8_t* aq, float* scale, int M, int K, int per_tensor, hipStream_t st);
// A (K,N) fp32 weight -> (N,K) fp8 with one factor per output column n (one common factor with per_tensor)
int quantize_weight_fp8(const float* W, uint8_t* wq, float* scale, int K, int N, int per_tensor, hipStream_t st);
// (K,N) fp32 row-major -> (N,K) bf16 row-major
int pack_weight_bf16(const float* W, bf16_t* out, int K, int N, hipStream_t st);
int cast_f32_to_bf16(const float* in, bf16_t* out, long long n, hipStream_t st);
// (K,N) fp32 -> (N,K) fp32
int transpose_f32(const float* W, float* out, int K, int N, hipStream_t st);
int patch_embed_direct(const float* latent, float* out, const float* kernel, const float* bias, int B, int H, int W, int Cin, int C, int p, int pos_max,
                       int base_height, hipStream_t st);

// LayerNorm without affine over the last axis + optional modulation: out = LN(x)*(1+scale[b])+shift[b]; a second modulated
// output (shift2/scale2/out2) may be produced from the same normalised row. scale/shift rows have stride mod_ld.
// out_bf16 selects bf16 (1) or fp32 (0) outputs.
// LayerNorm (no affine) + optional modulation of one tensor (B, T, C) into one or two outputs; two such jobs with the same C
// and eps (the two streams of a block) can share a launch
struct LayerNormJob {
    const float* x;
    void* out;
    void* out2;
    const float* shift;
    const float* scale;
    const float* shift2;
    const float* scale2;
    int mod_ld, B, T;
};
int layernorm_modulate_pair(const LayerNormJob* jobs, int n, float eps, int C, int out_bf16, hipStream_t st);
int layernorm_modulate(const float* x, void* out, void* out2, const float* shift, const float* scale, const float* shift2, const float* scale2,
                       int mod_ld, float eps, int B, int T, int C, int out_bf16, hipStream_t st);
int layernorm_full(const float* x, float* y, float* mean, float* rstd, const float* w, const float* bias, float eps, long long rows, int C,
                   hipStream_t st);
// RMSNorm over groups of `hs` consecutive values inside rows of stride `ld` (in place allowed): x[r*ld + g*hs + i], g < groups
int rmsnorm_rows(const float* x, float* y, const float* w, float* rms, float eps, long long rows, int groups, int hs, int ld_in, int ld_out,
                 hipStream_t st);
int unary_op(const float* in, float* out, long long n, int act, hipStream_t st);
int add_op(const float* a, const float* b, float* out, long long n, hipStream_t st);
int add_silu_op(const float* a, const float* b, float* out, long long n, hipStream_t st);
int modulate_op(const float* in, float* out, const float* shift, const float* scale, int B, int T, int C, hipStream_t st);  // scale null -> gate with `shift` as gate
int gate_op(const float* in, float* out, const float* gate, int B, int T, int C, hipStream_t st);
int copy_rows(const float* in, long long in_batch_stride, float* out, long long out_batch_stride, int B, long long n_per_batch, hipStream_t st);
int timestep_embedding(const float* t, float* out, int B, int dim, hipStream_t st);
int pos_embed_table(float* out, int C, int height, int width, int base_size, hipStream_t st);
int pos_embed_crop(const float* table, float* out, int max_size, int h, int w, int C, hipStream_t st);
// cropped table written directly (what PatchEmbedding needs): out (h*w, C)
int pos_embed_cropped(float* out, int C, int max_size, int base_size, int h, int w, hipStream_t st);
int conv2d_direct(const float* in, float* out, const float* kernel, const float* bias, int B, int kh, int kw, int Cin, int Cout, int ih, int iw, int oh,
                  int ow, int stride, int pad, hipStream_t st);
// latent (B,Cin,H,W) -> patch rows (B*h*w, Cin*p*p), k index = (ic*p + r)*p + s; fp32 or bf16 output
int im2col_patches(const float* latent, void* out, int out_bf16, int B, int Cin, int H, int W, int p, hipStream_t st);
// tokens (B, h*w, p*p*Cin) -> pixels (B,Cin,H,W)
int unpatchify(const float* tokens, float* out, int B, int Cin, int H, int W, int p, hipStream_t st);
int unpatchify_cfg_euler(const float* tokens, const float* latent, float* out, int n_samples, int Cin, int H, int W, int p, float guidance, float dsigma,
                         hipStream_t st);

// Small-M linear (M <= 8): out(M, N) = act(x(M,K) @ W[:, n0:n0+N] + b[n0:n0+N]); W fp32 (K, ldw) or bf16 (K, ldw), both N-contiguous.
struct SmallLinearJob {
    const void* W;
    const float* bias;
    float* out;
    int N;    // columns of this job
    int ldw;  // row stride of W
    int n0;   // first column
    const float* x = nullptr;  // this job's own left operand (M, K) instead of the launch's, or null
    int K = 0;                 // its depth (with x)
};
constexpr int SMALL_LINEAR_JOBS_PER_LAUNCH = 52;
int small_linear_batched(const float* x, int M, int K, const SmallLinearJob* jobs_host, int n_jobs, int w_is_bf16, int act /* -1 none */,
                         hipStream_t st);

// Attention. Two token segments (segment 0 first in the joint sequence); each has its own q/k/v/out pointers and row strides.
struct AttnSegments {
    const void* q[2];
    const void* k[2];
    const void* v[2];
    void* out[2];
    int ld_qkv[2];  // row stride (elements) of q/k/v
    int ld_out[2];
    int T[2];       // keys/values per batch element in each segment (T[1] may be 0)
    int Tq[2];      // queries per batch element in each segment (equal to T for self-attention)
    const float* rms_q[2];  // bf16 kernel only: fused per-head RMSNorm weights (null = no norm)
    const float* rms_k[2];
};
int attention_f32(const AttnSegments& s, int B, int NH, int HS, hipStream_t st);
int attention_bf16(const AttnSegments& s, int B, int NH, int HS, hipStream_t st);
// Up to three attention problems in one launch. kv_splits[i] > 1 (or null: all 1) splits the keys of set i into that many runs, one
// work item each, whose partial results go through split_ws[i] (attention_bf16_split_workspace_floats floats) and are merged by a
// second, small kernel. attention_bf16_context_splits: the number of splits that pays for the Tc context queries of a joint
// attention next to Tx latent ones, or 0 when the plain one-set launch is the better choice.
int attention_bf16_multi(const AttnSegments* sets, const int* kv_splits, float* const* split_ws, int n, int B, int NH, int HS, hipStream_t st);
int attention_bf16_context_splits(int Tc, int Tx);
size_t attention_bf16_split_workspace_floats(int B, int NH, int Tc, int splits);

}  // namespace sd3
