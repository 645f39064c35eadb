// Joint text+image flash attention for head_dim 64 on the gfx950 bf16 matrix cores (v_mfma_f32_32x32x16_bf16).
//
// One launch does what the reference does in eight calls (modules.cpp:1396-1399, 1420-1432): per-head RMSNorm of q
// and k (applied while the operands are loaded), concatenation of context and latent tokens (never materialised:
// rows of the joint sequence are fetched from the context buffer below T[0] and from the latent buffer above),
// softmax(q k^T / sqrt(64)) v with an online softmax (no T x T matrix), and the split of the result.
// q, k, v are the column thirds of the packed (tokens, 3C) bf16 buffers that the QKV GEMM writes; head h is columns
// [h*64, h*64+64) inside a third, exactly the reference's layout.
//
// Everything is kept transposed so that probabilities stay in registers between the two matrix products:
//   S^T (keys x queries) = K . Q^T     : a lane owns one query column and 16 of every 32 keys
//   O^T (d x queries)   += V^T . P^T   : the lane's S^T registers 8j..8j+7 are, unchanged, the P^T operand of step j
// which needs V^T (d-major) in LDS; V rows are transposed while being staged (two keys packed per 32-bit store).
#include "common.hpp"

namespace sd3 {
namespace {

constexpr int HS = 64;
constexpr int BQ = 128;       // queries per workgroup: 4 wavefronts x 32
constexpr int BKV = 64;       // keys per tile
constexpr int K_PITCH = 72;   // bf16 per K row in LDS (144 B: conflict-free 16-byte reads across 16 rows)
constexpr int V_PITCH = 66;   // bf16 per V^T row (33 words: conflict-free transposing stores and 8-byte reads)

struct SegDev {
    const bf16_t* q[2];
    const bf16_t* k[2];
    const bf16_t* v[2];
    bf16_t* out[2];
    const float* rms_q[2];
    const float* rms_k[2];
    int ld_qkv[2];
    int ld_out[2];
    int T[2];
    int Tq[2];
};

__device__ __forceinline__ void unpack8(const uint4& u, float (&f)[8]) {
    f[0] = __uint_as_float(u.x << 16); f[1] = __uint_as_float(u.x & 0xffff0000u);
    f[2] = __uint_as_float(u.y << 16); f[3] = __uint_as_float(u.y & 0xffff0000u);
    f[4] = __uint_as_float(u.z << 16); f[5] = __uint_as_float(u.z & 0xffff0000u);
    f[6] = __uint_as_float(u.w << 16); f[7] = __uint_as_float(u.w & 0xffff0000u);
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
    return make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7]));
}
union Frag {
    uint4 u;
    bf16x8_t v;
};

__global__ void __launch_bounds__(256) flash_attn_bf16_kernel(SegDev s, float q_scale /* log2(e)/sqrt(64) */, float eps) {
    // K tile (64 x 72) and V^T tile (64 x 66); the same memory later holds the output tile (128 x 72)
    __shared__ __attribute__((aligned(16))) bf16_t smem[BQ * K_PITCH];
    static_assert(BKV * K_PITCH + HS * V_PITCH <= BQ * K_PITCH, "tiles must fit the shared buffer");
    bf16_t* const Ks = smem;
    bf16_t* const Vt = smem + BKV * K_PITCH;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int h = blockIdx.y, b = blockIdx.z;
    const int T0 = s.T[0], T = s.T[0] + s.T[1];
    const int Tq0 = s.Tq[0], TQ = s.Tq[0] + s.Tq[1];

    // ---- Q^T operand: lane = query l32 of this wavefront; k-step ks covers d = 16*ks + 8*lk + (0..7) ----
    const int qt = blockIdx.x * BQ + wave * 32 + l32;
    Frag qf[4];
    {
        const int seg = (qt < Tq0) ? 0 : 1;
        float f[4][8];
        float ss = 0.f;
        if (qt < TQ) {
            const bf16_t* qp = s.q[seg] + ((long long)b * s.Tq[seg] + (seg ? qt - Tq0 : qt)) * s.ld_qkv[seg] + h * HS;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const uint4 u = *reinterpret_cast<const uint4*>(qp + ks * 16 + lk * 8);
                unpack8(u, f[ks]);
#pragma unroll
                for (int e = 0; e < 8; e++) ss += f[ks][e] * f[ks][e];
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < 4; ks++)
#pragma unroll
                for (int e = 0; e < 8; e++) f[ks][e] = 0.f;
        }
        ss += __shfl_xor(ss, 32, 64);  // the other half of the row lives in lane ^ 32
        const float* w = s.rms_q[seg];
        const float mul = w ? q_scale / sqrtf(eps + ss * (1.0f / HS)) : q_scale;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
#pragma unroll
            for (int e = 0; e < 8; e++) f[ks][e] *= w ? mul * w[ks * 16 + lk * 8 + e] : mul;
            qf[ks].u = pack8(f[ks]);
        }
    }

    f32x16_t oacc[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[i][r] = 0.f;
    float m_run = -1e30f, l_run = 0.f;

    // ---- staging roles ----
    // K: 64 rows x 8 chunks of 16 B = 512 chunks, 2 per thread (rows r and r+32); 8 consecutive lanes share a row
    const int k_row = tid >> 3, k_ch = tid & 7;
    // V: thread = (key pair, d-chunk): rows 2*vp and 2*vp+1, d = 8*v_ch..+7; stored transposed, two keys per 32-bit word
    const int v_pair = tid >> 3, v_ch = tid & 7;
    uint4 rk[2], rv[2];
    auto kv_row_ptr = [&](const bf16_t* const* base, int t) -> const bf16_t* {
        const int seg = (t < T0) ? 0 : 1;
        return base[seg] + ((long long)b * s.T[seg] + (seg ? t - T0 : t)) * s.ld_qkv[seg] + h * HS;
    };
    auto load_kv = [&](int t0) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int tk = t0 + k_row + i * 32;
            rk[i] = (tk < T) ? *reinterpret_cast<const uint4*>(kv_row_ptr(s.k, tk) + k_ch * 8) : make_uint4(0, 0, 0, 0);
            const int tv = t0 + 2 * v_pair + i;
            rv[i] = (tv < T) ? *reinterpret_cast<const uint4*>(kv_row_ptr(s.v, tv) + v_ch * 8) : make_uint4(0, 0, 0, 0);
        }
    };
    auto store_kv = [&](int t0) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int tk = t0 + k_row + i * 32;
            const float* w = s.rms_k[(tk < T0) ? 0 : 1];
            uint4 u = rk[i];
            if (w) {
                float f[8];
                unpack8(u, f);
                float ss = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) ss += f[e] * f[e];
                ss += __shfl_xor(ss, 1, 64);
                ss += __shfl_xor(ss, 2, 64);
                ss += __shfl_xor(ss, 4, 64);
                const float inv = 1.0f / sqrtf(eps + ss * (1.0f / HS));
#pragma unroll
                for (int e = 0; e < 8; e++) f[e] *= inv * w[k_ch * 8 + e];
                u = pack8(f);
            }
            *reinterpret_cast<uint4*>(&Ks[(k_row + i * 32) * K_PITCH + k_ch * 8]) = u;
        }
        // V^T[d][2*vp .. 2*vp+1] = (V[2vp][d], V[2vp+1][d])
        const uint32_t a[4] = {rv[0].x, rv[0].y, rv[0].z, rv[0].w};
        const uint32_t c[4] = {rv[1].x, rv[1].y, rv[1].z, rv[1].w};
        uint32_t* vt32 = reinterpret_cast<uint32_t*>(Vt);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t lo = (a[e] & 0xffffu) | (c[e] << 16);          // d = 8*v_ch + 2e
            const uint32_t hi = (a[e] >> 16) | (c[e] & 0xffff0000u);      // d = 8*v_ch + 2e + 1
            vt32[((v_ch * 8 + 2 * e) * V_PITCH) / 2 + v_pair] = lo;
            vt32[((v_ch * 8 + 2 * e + 1) * V_PITCH) / 2 + v_pair] = hi;
        }
    };

    load_kv(0);
    for (int t0 = 0; t0 < T; t0 += BKV) {
        __syncthreads();  // the previous tile has been consumed by every wavefront
        store_kv(t0);
        __syncthreads();
        if (t0 + BKV < T) load_kv(t0 + BKV);  // in flight during the matrix work below

        // ---- S^T = K . Q^T for the two 32-key blocks ----
        f32x16_t sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int r = 0; r < 16; r++) sacc[kb][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(&Ks[(kb * 32 + l32) * K_PITCH + ks * 16 + lk * 8]);
                sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks].v, sacc[kb], 0, 0, 0);
            }
        }
        // ---- online softmax (base 2: log2(e)/8 is folded into q). Register r of block kb is key t0+32kb+8(r/4)+4lk+r%4 ----
        if (t0 + BKV > T) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if (t0 + kb * 32 + 8 * (r >> 2) + 4 * lk + (r & 3) >= T) sacc[kb][r] = -1e30f;
        }
        float tmax = sacc[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) tmax = fmaxf(tmax, sacc[kb][r]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float p = __builtin_amdgcn_exp2f(sacc[kb][r] - m_new);
                sacc[kb][r] = p;
                psum += p;
            }
        l_run = l_run * alpha + psum;
        if (__any(alpha != 1.0f)) {  // once the running maxima have settled no lane needs the rescale
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
        }

        // ---- O^T += V^T . P^T ; step j of block kb contracts keys 32kb + 16j + {4lk..4lk+3, 8+4lk..8+4lk+3} ----
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                Frag pf;
                pf.u = make_uint4(pack_bf16x2(sacc[kb][8 * j + 0], sacc[kb][8 * j + 1]), pack_bf16x2(sacc[kb][8 * j + 2], sacc[kb][8 * j + 3]),
                                  pack_bf16x2(sacc[kb][8 * j + 4], sacc[kb][8 * j + 5]), pack_bf16x2(sacc[kb][8 * j + 6], sacc[kb][8 * j + 7]));
                const int key0 = kb * 32 + 16 * j + 4 * lk;
#pragma unroll
                for (int db = 0; db < 2; db++) {
                    const uint32_t* row = reinterpret_cast<const uint32_t*>(&Vt[(db * 32 + l32) * V_PITCH + key0]);
                    Frag vf;
                    vf.u = make_uint4(row[0], row[1], row[4], row[5]);
                    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf.v, oacc[db], 0, 0, 0);
                }
            }
    }

    // ---- normalise; transpose through LDS (reusing the K tile) so that rows leave as 16-byte stores ----
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = 1.0f / l_tot;
    __syncthreads();
    bf16_t* Ow = smem + wave * 32 * K_PITCH;  // this wavefront's 32 output rows
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int d0 = db * 32 + 8 * g + 4 * lk;
            const uint2 v = make_uint2(pack_bf16x2(oacc[db][4 * g + 0] * inv, oacc[db][4 * g + 1] * inv),
                                       pack_bf16x2(oacc[db][4 * g + 2] * inv, oacc[db][4 * g + 3] * inv));
            *reinterpret_cast<uint2*>(&Ow[l32 * K_PITCH + d0]) = v;
        }
    __syncthreads();
    // 32 rows x 8 chunks per wavefront = 256 chunks, 4 per lane
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = lane + i * 64;
        const int row = c >> 3, ch = c & 7;
        const int t = blockIdx.x * BQ + wave * 32 + row;
        if (t < TQ) {
            const int seg = (t < Tq0) ? 0 : 1;
            if (s.out[seg]) {
                bf16_t* op = s.out[seg] + ((long long)b * s.Tq[seg] + (seg ? t - Tq0 : t)) * s.ld_out[seg] + h * HS + ch * 8;
                *reinterpret_cast<uint4*>(op) = *reinterpret_cast<const uint4*>(&Ow[row * K_PITCH + ch * 8]);
            }
        }
    }
}

}  // namespace

int attention_bf16(const AttnSegments& a, int B, int NH, int hs, hipStream_t st) {
    const int T = a.T[0] + a.T[1], TQ = a.Tq[0] + a.Tq[1];
    if (B <= 0 || NH <= 0 || TQ <= 0) return SD3_OK;
    if (hs != HS) return fail(SD3_ERR_UNSUPPORTED, "attention (bf16): head_dim must be 64 (got %d)", hs);
    if (T <= 0) return fail(SD3_ERR_INVALID_ARG, "attention: no keys");
    SegDev s;
    for (int i = 0; i < 2; i++) {
        s.q[i] = (const bf16_t*)a.q[i]; s.k[i] = (const bf16_t*)a.k[i]; s.v[i] = (const bf16_t*)a.v[i]; s.out[i] = (bf16_t*)a.out[i];
        s.rms_q[i] = a.rms_q[i]; s.rms_k[i] = a.rms_k[i];
        s.ld_qkv[i] = a.ld_qkv[i]; s.ld_out[i] = a.ld_out[i]; s.T[i] = a.T[i]; s.Tq[i] = a.Tq[i];
        if (a.Tq[i] > 0 && !a.q[i]) return fail(SD3_ERR_INVALID_ARG, "attention: null q for segment %d", i);
        if (a.T[i] > 0 && (!a.k[i] || !a.v[i])) return fail(SD3_ERR_INVALID_ARG, "attention: null k/v for segment %d", i);
        if (a.T[i] > 0 || a.Tq[i] > 0) {
            if ((a.ld_qkv[i] % 8) || (a.ld_out[i] % 8) || (reinterpret_cast<uintptr_t>(a.q[i]) & 15) || (reinterpret_cast<uintptr_t>(a.k[i]) & 15) ||
                (reinterpret_cast<uintptr_t>(a.v[i]) & 15) || (reinterpret_cast<uintptr_t>(a.out[i]) & 15))
                return fail(SD3_ERR_INVALID_ARG, "attention (bf16): rows must be 16-byte aligned (segment %d)", i);
        }
    }
    const float q_scale = 1.4426950408889634f / sqrtf((float)HS);
    dim3 grid((TQ + BQ - 1) / BQ, NH, B), block(256);
    hipLaunchKernelGGL(flash_attn_bf16_kernel, grid, block, 0, st, s, q_scale, 1e-6f);
    return launch_status("flash_attention_bf16");
}

}  // namespace sd3
