// fp32 multi-head attention on the fp32 matrix cores, for the fp32 parity path.
// Replaces multihead_attention (modules.cpp:766-831) and, through its two-segment addressing, the token
// concatenation / split around it (modules.cpp:1427-1432): keys/values/queries of the joint sequence are read
// straight from the context buffers (first T[0] tokens) and the latent buffers (next T[1] tokens).
//
// Formulation: everything is kept transposed so that the probabilities never leave registers.
//   S^T (keys x queries) = K . Q^T      -> C-layout: a lane owns ONE query column and 16 keys per 32-key block
//   O^T (d x queries)   += V^T . P^T    -> the lane's own S^T registers are exactly the P^T operand it must supply
// Online softmax statistics are per query = per lane (plus one exchange with lane^32).
#include "common.hpp"

namespace sd3 {
namespace {

constexpr int BQ = 128;   // queries per workgroup (4 wavefronts x 32)

struct SegDev {
    const float* q[2];
    const float* k[2];
    const float* v[2];
    float* out[2];
    int ld_qkv[2];
    int ld_out[2];
    int T[2];   // keys/values per batch element in each segment
    int Tq[2];  // queries per batch element in each segment
};

template <int HSP, bool VEC>
__global__ void __launch_bounds__(256) attn_f32_kernel(SegDev s, int HS, float scale) {
    constexpr int KP = HSP + 1;
    constexpr int BKV = (HSP == 128) ? 32 : 64;  // keys per LDS tile (both tiles must fit 64 KiB of static LDS)
    constexpr int NKB = BKV / 32;
    __shared__ float Ks[BKV * KP];
    __shared__ float Vs[BKV * HSP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int h = blockIdx.y, b = blockIdx.z;
    const int T0 = s.T[0], T = s.T[0] + s.T[1];
    const int Tq0 = s.Tq[0], TQ = s.Tq[0] + s.Tq[1];

    // ---- this lane's query row (as the B operand of S^T = K.Q^T: element [d = 2*kk + lk][q = l32]) ----
    const int qt = blockIdx.x * BQ + wave * 32 + l32;
    float qreg[HSP / 2];
    {
        const int seg = (qt < Tq0) ? 0 : 1;
        const int tl = seg ? qt - Tq0 : qt;
        const float* qp = s.q[seg] + ((long long)b * s.Tq[seg] + tl) * s.ld_qkv[seg] + (long long)h * HS;
#pragma unroll
        for (int kk = 0; kk < HSP / 2; kk++) {
            const int d = 2 * kk + lk;
            qreg[kk] = (qt < TQ && d < HS) ? qp[d] * scale : 0.f;
        }
    }

    f32x16_t oacc[HSP / 32];
#pragma unroll
    for (int i = 0; i < HSP / 32; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[i][r] = 0.f;
    float m_run = -1e30f, l_run = 0.f;  // l_run: partial sum over the keys this lane owns

    for (int t0 = 0; t0 < T; t0 += BKV) {
        __syncthreads();  // previous tile fully consumed
        // ---- stage K and V rows t0..t0+BKV-1 of head h (zero beyond T or beyond HS) ----
        if (VEC) {
            constexpr int VPR = HSP / 4;  // float4 per row
            for (int e = tid; e < BKV * VPR; e += 256) {
                const int row = e / VPR, dv = (e % VPR) * 4;
                const int t = t0 + row;
                float4 kv = make_float4(0.f, 0.f, 0.f, 0.f), vv = kv;
                if (t < T && dv < HS) {
                    const int seg = (t < T0) ? 0 : 1;
                    const long long off = ((long long)b * s.T[seg] + (seg ? t - T0 : t)) * s.ld_qkv[seg] + (long long)h * HS + dv;
                    kv = *reinterpret_cast<const float4*>(s.k[seg] + off);
                    vv = *reinterpret_cast<const float4*>(s.v[seg] + off);
                }
                float* kd = &Ks[row * KP + dv];
                kd[0] = kv.x; kd[1] = kv.y; kd[2] = kv.z; kd[3] = kv.w;
                *reinterpret_cast<float4*>(&Vs[row * HSP + dv]) = vv;
            }
        } else {
            for (int e = tid; e < BKV * HSP; e += 256) {
                const int row = e / HSP, d = e % HSP;
                const int t = t0 + row;
                float kv = 0.f, vv = 0.f;
                if (t < T && d < HS) {
                    const int seg = (t < T0) ? 0 : 1;
                    const long long off = ((long long)b * s.T[seg] + (seg ? t - T0 : t)) * s.ld_qkv[seg] + (long long)h * HS + d;
                    kv = s.k[seg][off];
                    vv = s.v[seg][off];
                }
                Ks[row * KP + d] = kv;
                Vs[row * HSP + d] = vv;
            }
        }
        __syncthreads();

        // ---- S^T for the 32-key blocks of the tile ----
        f32x16_t sacc[NKB];
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) {
#pragma unroll
            for (int r = 0; r < 16; r++) sacc[kb][r] = 0.f;
#pragma unroll
            for (int kk = 0; kk < HSP / 2; kk++) {
                const float a = Ks[(kb * 32 + l32) * KP + 2 * kk + lk];
                sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, qreg[kk], sacc[kb], 0, 0, 0);
            }
        }
        // lane holds keys  t0 + kb*32 + 8*(r/4) + 4*lk + (r%4)  of query column l32
        float tmax = -1e30f;
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = t0 + kb * 32 + 8 * (r >> 2) + 4 * lk + (r & 3);
                if (key >= T) sacc[kb][r] = -1e30f;
                tmax = fmaxf(tmax, sacc[kb][r]);
            }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = expf(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float p = expf(sacc[kb][r] - m_new);
                sacc[kb][r] = p;
                psum += p;
            }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int i = 0; i < HSP / 32; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;

        // ---- O^T += V^T . P^T : step r of block kb contracts key (8*(r/4) + 4*lk + r%4) of each lane half ----
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = kb * 32 + 8 * (r >> 2) + 4 * lk + (r & 3);
#pragma unroll
                for (int i = 0; i < HSP / 32; i++) {
                    const float a = Vs[key * HSP + i * 32 + l32];
                    oacc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, sacc[kb][r], oacc[i], 0, 0, 0);
                }
            }
    }

    // ---- normalise and store: lane owns query qt, rows d = i*32 + 8*(r/4) + 4*lk + r%4 ----
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    if (qt < TQ) {
        const int seg = (qt < Tq0) ? 0 : 1;
        if (s.out[seg]) {
            const int tl = seg ? qt - Tq0 : qt;
            float* op = s.out[seg] + ((long long)b * s.Tq[seg] + tl) * s.ld_out[seg] + (long long)h * HS;
            const float inv = 1.0f / l_tot;
#pragma unroll
            for (int i = 0; i < HSP / 32; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int d = i * 32 + 8 * (r >> 2) + 4 * lk + (r & 3);
                    if (d < HS) op[d] = oacc[i][r] * inv;
                }
        }
    }
}

}  // namespace

int attention_f32(const AttnSegments& a, int B, int NH, int HS, hipStream_t st) {
    const int T = a.T[0] + a.T[1], TQ = a.Tq[0] + a.Tq[1];
    if (B <= 0 || NH <= 0 || TQ <= 0) return SD3_OK;
    if (T <= 0) return fail(SD3_ERR_INVALID_ARG, "attention: no keys");
    if (HS <= 0 || HS > 128) return fail(SD3_ERR_UNSUPPORTED, "attention (fp32): head_dim %d not in 1..128", HS);
    SegDev s;
    bool vec = (HS % 4 == 0);
    for (int i = 0; i < 2; i++) {
        s.q[i] = (const float*)a.q[i]; s.k[i] = (const float*)a.k[i]; s.v[i] = (const float*)a.v[i]; s.out[i] = (float*)a.out[i];
        s.ld_qkv[i] = a.ld_qkv[i]; s.ld_out[i] = a.ld_out[i]; s.T[i] = a.T[i]; s.Tq[i] = a.Tq[i];
        if (a.Tq[i] > 0 && !a.q[i]) return fail(SD3_ERR_INVALID_ARG, "attention: null q for segment %d", i);
        if (a.T[i] > 0) {
            if (!a.k[i] || !a.v[i]) return fail(SD3_ERR_INVALID_ARG, "attention: null k/v for segment %d", i);
            if ((a.ld_qkv[i] % 4) || (reinterpret_cast<uintptr_t>(a.k[i]) & 15) || (reinterpret_cast<uintptr_t>(a.v[i]) & 15)) vec = false;
        }
    }
    const float scale = (float)(1.0 / sqrtf((float)HS));
    dim3 grid((TQ + BQ - 1) / BQ, NH, B), block(256);
    const int hsp = HS <= 32 ? 32 : (HS <= 64 ? 64 : 128);
#define SD3_ATTN_LAUNCH(P)                                                                              \
    do {                                                                                                \
        if (vec) hipLaunchKernelGGL((attn_f32_kernel<P, true>), grid, block, 0, st, s, HS, scale);      \
        else hipLaunchKernelGGL((attn_f32_kernel<P, false>), grid, block, 0, st, s, HS, scale);         \
    } while (0)
    if (hsp == 32) SD3_ATTN_LAUNCH(32);
    else if (hsp == 64) SD3_ATTN_LAUNCH(64);
    else SD3_ATTN_LAUNCH(128);
#undef SD3_ATTN_LAUNCH
    return launch_status("attention_f32");
}

}  // namespace sd3
