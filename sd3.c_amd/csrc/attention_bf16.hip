// Joint text+image flash attention for head_dim 64 on the gfx950 bf16 matrix cores (v_mfma_f32_32x32x16_bf16).
//
// One launch does what the reference does in eight calls (modules.cpp:1396-1399, 1420-1432): per-head RMSNorm of q
// and k (optional: applied while the operands are loaded), concatenation of context and latent tokens (never
// materialised: rows of the joint sequence are fetched from the context buffer below T[0] and from the latent buffer
// above), softmax(q k^T / sqrt(64)) v with an online softmax (no T x T matrix), and the split of the result.
// q, k, v are the column thirds of the packed (tokens, 3C) bf16 buffers that the QKV GEMM writes; head h is columns
// [h*64, h*64+64) inside a third, exactly the reference's layout.
//
// Everything is kept transposed so that probabilities stay in registers between the two matrix products:
//   S^T (keys x queries) = K . Q^T     : a lane owns one query column per 32-query block and 16 of every 32 keys
//   O^T (d x queries)   += V^T . P^T   : the lane's S^T registers 8j..8j+7 are, unchanged, the P^T operand of step j
// which needs V^T (d-major) in LDS; V rows are transposed while being staged (two keys packed per 32-bit store).
// A wavefront owns 64 queries (two 32-query blocks), so every K / V^T fragment read from LDS feeds two matrix
// instructions; a workgroup of 4 wavefronts shares each 64-key tile. K tiles go global -> LDS directly
// (global_load_lds_dwordx4) into 128-byte rows with XOR-swizzled 16-byte chunks; tiles are double-buffered with one
// barrier per tile.
#include <type_traits>

#include "common.hpp"

namespace sd3 {
namespace {

constexpr int HS = 64;
constexpr int NW = 4;            // wavefronts per workgroup
constexpr int QW = 64;           // queries per wavefront
constexpr int BQ = NW * QW;      // queries per workgroup
constexpr int BKV = 64;          // keys per tile
constexpr int K_BYTES = BKV * 128, V_BYTES = BKV * 128, STAGE_BYTES = K_BYTES + V_BYTES;
constexpr int O_PITCH = 72;      // bf16 per staged output row
// Tiles are requested PF tiles ahead of the one being worked on, into a ring of PF + 2 LDS stages (the tile in use, PF on their
// way or landed, and the stage of the tile before, which the newest request overwrites). One tile ahead is enough: with two
// (SD3_ATTN_PREFETCH_2; not with the K rows passing through registers, NORM) and the barrier waiting only for the tile it
// publishes, nothing was gained at any occupancy (measured), so the wait in the middle of a tile is not where time goes.
constexpr int prefetch_tiles(bool norm) {
#ifdef SD3_ATTN_PREFETCH_2
    return norm ? 1 : 2;
#else
    return 1;
#endif
}
constexpr int smem_bytes(bool norm) {
    return ((prefetch_tiles(norm) + 2) * STAGE_BYTES > NW * QW * O_PITCH * 2) ? (prefetch_tiles(norm) + 2) * STAGE_BYTES : NW * QW * O_PITCH * 2;
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;

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
    int NH, nqb;  // heads, query blocks per (batch, head)
    // kv_splits > 1: every (batch, head, query block) becomes kv_splits work items, each over its own run of key tiles, and an item
    // writes what it has accumulated -- unnormalised O (fp32), the softmax reference and the row sum -- for attn_combine_kernel
    int kv_splits;
    float* part_o;   // (items, BQ, 64)
    float* part_ml;  // (items, BQ, 2)
};
// One launch covers up to three independent attention problems ("sets": in a block, the joint attention of the latent queries,
// the extra self-attention, and the few context queries split along the keys): workgroups [0, end[0]) belong to set 0, ...
constexpr int MAX_SETS = 3;
struct AttnSets {
    SegDev set[MAX_SETS];
    int end[MAX_SETS];
};

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

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

// ds_read_b64_tr_b16 works on blocks of 16 lanes: lane i of a block receives, as element j (of 4 bf16), element i%4 of the
// 8 bytes addressed by lane (i/4 + 4j) of the block. Issued as inline assembly: through the compiler's builtin every such
// read is preceded by s_waitcnt vmcnt(0), which would serialise it behind the global->LDS loads of the next tile. The
// compiler does not count these reads, so the results may only be used after one of the waits below has named them.
__device__ __forceinline__ uint2 lds_read_tr16_b64(uint32_t lds_byte_addr, int imm_offset) {
    uint2 r;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(lds_byte_addr), "i"(imm_offset));
    return r;
}
// A plain 16-byte LDS read issued the same way (K fragments in the hand-ordered steps of the fast tiles), and the waits that name
// what has landed: LDS operations return in order, so "at most N outstanding" means all but the newest N have arrived.
__device__ __forceinline__ bf16x8_t lds_read_b128(uint32_t lds_byte_addr, int imm_offset) {
    bf16x8_t r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(lds_byte_addr), "i"(imm_offset));
    return r;
}
template <int N>
__device__ __forceinline__ void lds_wait_k(bf16x8_t (&k)[4]) {
    static_assert(N == 0 || N == 4 || N == 8, "outstanding LDS reads behind the four K fragments");
    if (N == 8) asm volatile("s_waitcnt lgkmcnt(8)" : "+v"(k[0]), "+v"(k[1]), "+v"(k[2]), "+v"(k[3]));
    else if (N == 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(k[0]), "+v"(k[1]), "+v"(k[2]), "+v"(k[3]));
    else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(k[0]), "+v"(k[1]), "+v"(k[2]), "+v"(k[3]));
}
// The transposing reads are issued in two groups of four (first vfr[0..3], then vfr[4..7]). LDS operations complete in order, so
// once at most four are outstanding the first group has landed whatever else the compiler has put in between.
__device__ __forceinline__ void lds_wait_first4(uint2 (&a)[8]) {
    asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]));
}
__device__ __forceinline__ void lds_wait_last4(uint2 (&a)[8]) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]));
}

// NORM: apply the per-head RMSNorm to q and k while loading them (K then goes through registers instead of the
// direct global->LDS path). Without it q and k are taken as they are (already normalised by the QKV GEMM epilogue).
template <bool NORM>
__global__ void __launch_bounds__(NW * 64, 2) flash_attn_bf16_kernel(const AttnSets sets, float q_scale /* log2(e)/sqrt(64) */, float eps) {
    constexpr int PF = prefetch_tiles(NORM);
    __shared__ __attribute__((aligned(1024))) char smem[smem_bytes(NORM)];
    // The barrier in the middle of a tile, which publishes tile t+1 and retires the stage of tile t-1. In front of it a thread's own
    // requests for tile t+1 must have landed -- every thread requests four 16-byte chunks per tile, so that is "all but the newest
    // 4 (PF - 1)" -- and its LDS accesses must be done. A bare barrier between compiler fences: __syncthreads() would wait for
    // every load in flight, the tiles requested further ahead included.
    auto tile_barrier = [&]() {
        __builtin_amdgcn_s_waitcnt(((4 * (PF - 1)) & 15) | (7 << 4) | (0 << 8));  // vmcnt(4 (PF - 1)), lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    const int which = (blockIdx.x >= (unsigned)sets.end[0]) + (blockIdx.x >= (unsigned)sets.end[1]);  // uniform
    const SegDev& s = sets.set[which];
    const int wg_first = which ? sets.end[which - 1] : 0;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: LDS destinations of the direct loads are then scalar
    const int l32 = lane & 31, lk = lane >> 5;
    const int T0 = s.T[0], T = s.T[0] + s.T[1];
    const int Tq0 = s.Tq[0], TQ = s.Tq[0] + s.Tq[1];

    // ---- workgroup -> (batch, head, query block): consecutive workgroup ids go to different XCDs (each with its own L2),
    //      so the workgroups of one XCD get a contiguous run of work items; all query blocks of a head then share K/V in one L2
    int b, h, qblk, split, item;
    {
        const int total = sets.end[which] - wg_first, wg = blockIdx.x - wg_first, xcd = wg % 8, local = wg / 8;
        const int per = (total + 7) / 8, tall = (total % 8) ? (total % 8) : 8;
        item = (xcd < tall) ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
        split = item % s.kv_splits;
        const int t = item / s.kv_splits;
        const int bh = t / s.nqb;
        qblk = t % s.nqb;
        b = bh / s.NH;
        h = bh % s.NH;
    }
    // this item's run of key tiles: [kv0, kv0 + nt * BKV), the whole sequence when kv_splits == 1
    const int nt_all = (T + BKV - 1) / BKV, nt_per = (nt_all + s.kv_splits - 1) / s.kv_splits;
    const int kv0 = split * nt_per * BKV;
    const int nt = min(nt_per, nt_all - split * nt_per);  // >= 1: the host chooses kv_splits so that no item is empty

    // ---- Q^T operands: for block qb the lane is query (q0 + 32 qb + l32); k-step ks covers d = 16 ks + 8 lk + (0..7) ----
    const int q0 = qblk * BQ + wave * QW;
    Frag qf[2][4];
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
        const int qt = q0 + qb * 32 + l32;
        const int seg = (qt < Tq0) ? 0 : 1;
        float f[4][8];
        float ss = 0.f;
        if (qt < TQ) {
            const bf16_t* qp = s.q[seg] + ((long long)b * s.Tq[seg] + (seg ? qt - Tq0 : qt)) * s.ld_qkv[seg] + h * HS;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const uint4 u = *reinterpret_cast<const uint4*>(qp + ks * 16 + lk * 8);
                unpack8(u, f[ks]);
                if (NORM)
#pragma unroll
                    for (int e = 0; e < 8; e++) ss += f[ks][e] * f[ks][e];
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < 4; ks++)
#pragma unroll
                for (int e = 0; e < 8; e++) f[ks][e] = 0.f;
        }
        const float* w = NORM ? s.rms_q[seg] : nullptr;
        float mul = q_scale;
        if (NORM) {
            ss += __shfl_xor(ss, 32, 64);  // the other half of the row lives in lane ^ 32
            if (w) mul = q_scale / sqrtf(eps + ss * (1.0f / HS));
        }
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
#pragma unroll
            for (int e = 0; e < 8; e++) f[ks][e] *= (NORM && w) ? mul * w[ks * 16 + lk * 8 + e] : mul;
            qf[qb][ks].u = pack8(f[ks]);
        }
    }

    f32x16_t oacc[2][2];  // [d block][query block]
    // Softmax reference point m_run per query (any value works as long as numerator and denominator use the same one) and
    // this lane's share l_run of the row sum. The matrix unit subtracts the reference and masks keys beyond the sequence:
    // a score block starts from AUX . NEGM, where AUX[key][k=0] = 1, AUX[key][k=1] = (key beyond the sequence),
    // NEGM[k=0][query] = -m_run (kept representable in bf16), NEGM[k=1][query] = -1e30 and everything else is zero.
    // While the reference is zero and no key of a block is masked that product is zero, and the loop over such tiles
    // ("fast" tiles below) leaves it out.
    float m_run[2], l_run[2];
    const uint32_t NEG_BIG_HI = pack_bf16x2(0.f, -1e30f);  // bf16(-1e30) in the upper half
    Frag negm_f[2];
    // a partial row sum of 16 probabilities above this bound (or infinite) moves the reference
    constexpr float L_BOUND = 1073741824.0f;  // 2^30

    // ---- staging: chunk q = i*256 + tid of a tile lands at LDS byte q*16 of the K (V) area: row q/8, physical 16-byte
    //      chunk q%8. The logical chunk fetched into that slot is XOR-swizzled per row so that the fragment reads below
    //      are conflict-free: K by swz(row) (16-byte reads down a column of rows), V by 2*(row%4) (the transposing read
    //      touches 32 bytes in each of 4 consecutive rows). ----
    auto kv_row_ptr = [&](const bf16_t* const* base, int t) -> const bf16_t* {
        t = min(t, T - 1);  // rows beyond the sequence re-read the last row: finite values, masked out of the softmax
        const int seg = (t < T0) ? 0 : 1;
        return base[seg] + ((long long)b * s.T[seg] + (seg ? t - T0 : t)) * s.ld_qkv[seg] + h * HS;
    };
    uint4 rk[2];
    // Row pointers of this thread's two K chunks and two V chunks. Inside a segment they advance by a constant per tile;
    // they are recomputed from scratch only for the first tile, the tiles around the segment boundary and the last tile.
    const bf16_t* kp[2];
    const bf16_t* vp[2];
    // advance() moves the four row pointers to the tile that starts at key t0 (branches; kept out of the pipeline steps),
    // fetch_tile() issues the loads through them (straight-line; interleaved with a step's matrix instructions)
    // (the two strides are read once, here: inside advance() the set's row stride, a kernel argument selected by `which`, was a
    // scalar memory load and a wait for it in the middle of every tile)
    const long long tile_step0 = (long long)BKV * s.ld_qkv[0], tile_step1 = (long long)BKV * s.ld_qkv[1];
    auto advance = [&](int t0) {
        const bool in0 = (t0 >= kv0 + BKV) && (t0 + BKV <= T0), in1 = (t0 - BKV >= max(T0, kv0)) && (t0 + BKV <= T);
        if (in0 || in1) {
            const long long step = in1 ? tile_step1 : tile_step0;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                kp[i] += step;
                vp[i] += step;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int q = i * 256 + tid, row = q >> 3;
                kp[i] = kv_row_ptr(s.k, t0 + row) + ((q & 7) ^ swz(row)) * 8;
                vp[i] = kv_row_ptr(s.v, t0 + row) + ((q & 7) ^ (2 * (row & 3))) * 8;
            }
        }
    };
    auto fetch_tile = [&](int stage_byte) {
        char* ks_ = smem + stage_byte;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (NORM) rk[i] = *reinterpret_cast<const uint4*>(kp[i]);
            else __builtin_amdgcn_global_load_lds((glb_ptr_t)kp[i], (lds_ptr_t)(ks_ + (i * 256 + wave * 64) * 16), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((glb_ptr_t)vp[i], (lds_ptr_t)(ks_ + K_BYTES + (i * 256 + wave * 64) * 16), 16, 0, 0);
        }
    };
    auto store_k_normed = [&](int t0, int stage_byte) {  // NORM only: K rows pass through registers to be normalised
        char* ks_ = smem + stage_byte;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int q = i * 256 + tid, row = q >> 3, lc = (q & 7) ^ swz(row);
            const float* w = s.rms_k[(min(t0 + row, T - 1) < T0) ? 0 : 1];
            uint4 u = rk[i];
            if (w) {
                float f[8];
                unpack8(u, f);
                float ss = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) ss += f[e] * f[e];
                ss += __shfl_xor(ss, 1, 64);  // the 8 chunks of a row sit in 8 consecutive lanes
                ss += __shfl_xor(ss, 2, 64);
                ss += __shfl_xor(ss, 4, 64);
                const float inv = 1.0f / sqrtf(eps + ss * (1.0f / HS));
#pragma unroll
                for (int e = 0; e < 8; e++) f[e] *= inv * w[lc * 8 + e];
                u = pack8(f);
            }
            *reinterpret_cast<uint4*>(ks_ + q * 16) = u;
        }
    };

    // Loop-invariant LDS byte offsets (relative to the stage) of this lane's operand fragments.
    // K: the four 16-byte chunks (k-steps) of key row l32; 32-key blocks are a constant 32*128 bytes apart.
    // V: with lane n of a 16-lane block pointing at V[key0 + n/4][d0 + 4*(n%4) ..], the transposing read leaves lane i
    // with V[key0 + 0..3][d0 + i]: a column strip, i.e. half of a V^T operand row. The lane's block covers
    // d0 = 32 db + 16 (lane/16 % 2) and key0 = (constant) + 4 lk.
    int koff[4], voff[2];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) koff[ks] = l32 * 128 + (((2 * ks + lk) ^ swz(l32)) * 16);
    {
        const int n = lane & 15, row = 4 * lk + (n >> 2);  // row % 4 == n / 4 for every constant added below (multiples of 8)
#pragma unroll
        for (int db = 0; db < 2; db++) {
            const int chunk = db * 4 + 2 * ((lane >> 4) & 1) + ((n & 3) >> 1);
            voff[db] = K_BYTES + row * 128 + ((chunk ^ (2 * (row & 3))) * 16) + 8 * (n & 1);
        }
    }
    const uint32_t smem_addr = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
    const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // ---- the pipeline. The unit of work is (32 keys) x (32 queries): unit u = (tile t, key half kb, query block qb), in
    //      that order. Step u of the pipeline issues, interleaved in one instruction stream,
    //        matrix unit:  the scores of unit u+1  and  O^T += V^T . P^T of unit u-1
    //        vector unit:  the probabilities (exp2, bf16 rounding, row sums) of unit u
    //      so that neither unit waits for the other inside a wavefront. Tiles live in a ring of three LDS stages: the
    //      loads of tile t+2 are issued right after the barrier that publishes tile t+1, at which point every wavefront
    //      has finished its reads of tile t-1, whose stage they overwrite. ----
    f32x16_t sacc[2];   // sacc[qb]: scores of the unit of query block qb that is in the pipeline
    Frag pf[2][2];      // pf[qb][j]: its probabilities as P^T operands
    bf16x8_t kf[4];     // K fragments of the key half whose scores are being issued
    uint2 vfr[8];       // V^T fragments of the key half whose PV products are being issued: [j][d block][keys 0-3 | 8-11 of the step]
    // AUX rows for keys key_base + l32: one persistent operand whose first register alone changes from unit to unit
    Frag aux;
    int first_masked;  // key_base >= first_masked  <=>  key key_base + l32 lies beyond the sequence
    auto reset = [&]() {  // the state in front of an item's first tile
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[i][j][r] = 0.f;
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            l_run[qb] = 0.f;
#pragma unroll
            for (int j = 0; j < 2; j++) pf[qb][j].u = make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) vfr[i] = make_uint2(0u, 0u);
    };
    // The operands of the general path that say "reference zero". Called in front of an item's first tile and again behind the fast
    // tiles, which use none of this: built from a value the optimiser cannot trace, so that the second call does not simply keep
    // the results of the first in registers across the fast tiles, where registers are what the instruction schedule is short of.
    auto zero_reference = [&]() {
        int lane_o = (int)__lane_id();
        asm volatile("" : "+v"(lane_o));
        first_masked = T - (lane_o & 31);
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            m_run[qb] = 0.f;
            negm_f[qb].u = make_uint4((lane_o >> 5) == 0 ? NEG_BIG_HI : 0u, 0u, 0u, 0u);
        }
        aux.u = make_uint4(0u, 0u, 0u, 0u);
    };
    auto scores = [&](int qb, int key_base) {
        aux.u.x = (key_base >= first_masked) ? 0x3f803f80u : 0x00003f80u;
        sacc[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aux.v, negm_f[qb].v, zero, 0, 0, 0);
        sacc[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[0], qf[qb][0].v, sacc[qb], 0, 0, 0);
#pragma unroll
        for (int ks = 1; ks < 4; ks++) sacc[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qf[qb][ks].v, sacc[qb], 0, 0, 0);
    };
    auto load_k = [&](int stage_byte, int kb) {
#pragma unroll
        for (int ks = 0; ks < 4; ks++) kf[ks] = *reinterpret_cast<const bf16x8_t*>(smem + stage_byte + koff[ks] + kb * 32 * 128);
    };
    // probabilities of one unit -> bf16 P^T operands + this lane's sum of them (of the unrounded values, with plain
    // additions: the bf16 dot-product instructions, one per packed pair, measure about 8 cycles each during which the
    // matrix unit accepts nothing, while additions issue beside it for free)
    auto pack_probs = [&](const f32x16_t& pr, Frag (&out)[2]) -> float {
        float ls0 = 0.f, ls1 = 0.f;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                w[e] = pack_bf16x2(pr[8 * j + 2 * e], pr[8 * j + 2 * e + 1]);
                if (e & 1) ls1 += pr[8 * j + 2 * e] + pr[8 * j + 2 * e + 1];
                else ls0 += pr[8 * j + 2 * e] + pr[8 * j + 2 * e + 1];
            }
            out[j].u = make_uint4(w[0], w[1], w[2], w[3]);
        }
        return ls0 + ls1;
    };
    // O^T += V^T . P^T for query block qb, half j of it: contracts keys 16j + {4lk..4lk+3, 8+4lk..8+4lk+3} of the key half in vfr
    auto pv = [&](int qb, int j) {
#pragma unroll
        for (int db = 0; db < 2; db++) {
            Frag vf;
            vf.u = make_uint4(vfr[(j * 2 + db) * 2].x, vfr[(j * 2 + db) * 2].y, vfr[(j * 2 + db) * 2 + 1].x, vfr[(j * 2 + db) * 2 + 1].y);
            oacc[db][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[qb][j].v, oacc[db][qb], 0, 0, 0);
        }
    };
    // the V^T fragments of half j of key half kb: issued as soon as the products that used the previous contents are issued
    auto load_v = [&](int stage_byte, int kb, int j) {
#pragma unroll
        for (int db = 0; db < 2; db++)
#pragma unroll
            for (int hi = 0; hi < 2; hi++)
                vfr[(j * 2 + db) * 2 + hi] = lds_read_tr16_b64(smem_addr + stage_byte + voff[db], (kb * 32 + 16 * j + 8 * hi) * 128);
    };
    // probabilities of the unit in sacc[qb] -> pf[qb]; returns this lane's row-sum increment
    auto probs = [&](int qb) -> float {
        f32x16_t pr;
#pragma unroll
        for (int r = 0; r < 16; r++) pr[r] = __builtin_amdgcn_exp2f(sacc[qb][r]);
        return pack_probs(pr, pf[qb]);
    };
    // When the reference has to move (forced for the first units: they run with reference 0), the raw scores are
    // recovered from the matrix unit's result, the reference goes to the running maximum, what was accumulated for this
    // query block is rescaled and the probabilities are redone.
    auto settle = [&](int qb, float inc, bool force) {
        if (__any(inc > L_BOUND) || force) {
            const float m_old = m_run[qb];
            float tmax = fmaxf(sacc[qb][0], sacc[qb][1]);
#pragma unroll
            for (int r = 2; r < 16; r += 2) tmax = fmaxf(tmax, fmaxf(sacc[qb][r], sacc[qb][r + 1]));
            // lanes l and l^32 hold the two key halves of the same query and feed the same accumulators: same reference
            // (forced = the first unit of a query block: nothing has been accumulated, the reference is still zero and goes to that unit's
            // maximum wherever that lies, also far below zero, where a reference of zero would turn every probability into nothing)
            const float pair_max = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            const float m_new = force ? pair_max : fmaxf(m_old, m_old + pair_max);
            const uint32_t negm_bits = pack_bf16x2(-m_new, 0.f) & 0xffffu;
            const float m_ref = -__uint_as_float(negm_bits << 16);
            const float alpha = force ? 1.0f : __builtin_amdgcn_exp2f(m_old - m_ref);
            m_run[qb] = m_ref;
            negm_f[qb].u.x = lk == 0 ? (negm_bits | NEG_BIG_HI) : 0u;
            l_run[qb] *= alpha;
#pragma unroll
            for (int db = 0; db < 2; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[db][qb][r] *= alpha;
            f32x16_t pr;
#pragma unroll
            for (int r = 0; r < 16; r++) pr[r] = __builtin_amdgcn_exp2f(sacc[qb][r] + (m_old - m_ref));
            inc = pack_probs(pr, pf[qb]);
        }
        l_run[qb] += inc;
    };
    // one matrix instruction, then a few vector instructions, nine times: the mix of one pipeline step of the general path
    auto interleave = [&]() {
#pragma unroll
        for (int i = 0; i < 9; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        }
    };

    // Stages of tiles t, t+1, t+2
    int st_cur, st_nxt, st_nx2, st_ld;
    auto rotate_stages = [&]() {
        const int tmp = st_cur;
        st_cur = st_nxt;
        if (PF == 2) {
            st_nxt = st_nx2;
            st_nx2 = st_ld;
        } else {
            st_nxt = st_ld;
        }
        st_ld = tmp;
    };
    // One tile of the pipeline on the general path (any key may be masked, the reference may move): four steps.
    auto tile = [&](int t) {
        float inc;
        // ---- step (t, 0, 0): PV of (t-1,1,1), each half followed by the fetch of V of key half 0 into the registers it
        //      frees; scores of (t,0,1); then fetch K of half 1 ----
        pv(1, 0);
        load_v(st_cur, 0, 0);
        scores(1, kv0 + t * BKV);
        load_k(st_cur, 1);
        inc = probs(0);
        pv(1, 1);
        load_v(st_cur, 0, 1);
        interleave();
        settle(0, inc, t == 0);
        // ---- step (t, 0, 1): PV of (t,0,0); scores of (t,1,0) ----
        lds_wait_first4(vfr);
        pv(0, 0);
        scores(0, kv0 + t * BKV + 32);
        inc = probs(1);
        lds_wait_last4(vfr);
        pv(0, 1);
        interleave();
        settle(1, inc, t == 0);
        // ---- step (t, 1, 0): tile t+1 becomes visible and the loads of tile t+2 set off (past the end: the last tile once
        //      more, into a stage nobody reads again); PV of (t,0,1) and fetch of V of key half 1; scores of (t,1,1); then
        //      fetch K of half 0 of tile t+1 (past the last tile: stale LDS, feeding scores that are never used) ----
        if (NORM && t + 1 < nt) store_k_normed(kv0 + (t + 1) * BKV, st_nxt);
        tile_barrier();  // (also in the last tile: the stage the redundant loads go to must not be in use by a slower wavefront)
        if (t + PF + 1 < nt) advance(kv0 + (t + PF + 1) * BKV);
        fetch_tile(st_ld);
        pv(1, 0);
        load_v(st_cur, 1, 0);
        scores(1, kv0 + t * BKV + 32);
        load_k(st_nxt, 0);
        inc = probs(0);
        pv(1, 1);
        load_v(st_cur, 1, 1);
        interleave();
        settle(0, inc, false);
        // ---- step (t, 1, 1): PV of (t,1,0); scores of (t+1,0,0) ----
        lds_wait_first4(vfr);
        pv(0, 0);
        scores(0, kv0 + t * BKV + BKV);
        inc = probs(1);
        lds_wait_last4(vfr);
        pv(0, 1);
        interleave();
        settle(1, inc, false);
        rotate_stages();
    };

    // ---- a fast tile with the instruction order written out. Left to itself the compiler bunches the matrix instructions of a
    //      step (six in a row behind the barrier, thirty vector instructions in a row elsewhere). Here every step is eight slices of
    //      {one matrix instruction; an eighth of the step's vector work: 2 exp2, 1 conversion, 2 additions}, and nothing moves across
    //      a slice boundary. Order inside a step: the four score products first (the K fragments are then free: the next key half
    //      is fetched right behind them and has four slices to arrive), then PV of the first key quarter, then of the second, each
    //      followed in even steps by the fetch of the next V fragments into the registers just read. All LDS reads of these
    //      tiles are issued from assembly and waited for by count; exp2 of a pair of scores is issued one slice ahead of its
    //      conversion. Measured against the compiler's order on one device, 1536 workgroups of 64 tiles: 6 % faster with all-zero
    //      operands, 1.7 % with N(0,1) operands, where the power limit and not the instruction stream sets the pace. (Also tried
    //      on this basis: the row sums as two more matrix instructions per unit, ONES . P^T, instead of 16 additions: 7.5 % faster
    //      on zeros, 3 % slower on N(0,1) operands; the requests for the next tile spread over a step: slower.) ----
    auto fast_step = [&](auto qb_tag, auto loads_tag, auto vkb_tag, int v_stage, auto kkb_tag, int k_stage) {
        constexpr int QB = decltype(qb_tag)::value, PQ = QB ^ 1;     // probabilities of query block QB; scores and PV of the other one
        constexpr bool LOADS = decltype(loads_tag)::value;          // even steps fetch K of the next key half and V of this one
        constexpr int VKB = decltype(vkb_tag)::value, KKB = decltype(kkb_tag)::value;
        // The vector instructions are written as assembly statements, which the compiler keeps in the order given (as plain
        // arithmetic it sinks the conversions to where their results are needed, a step later). What the compiler's hazard
        // handling cannot see through them holds by construction: a score block is read here four or more slices behind the last
        // matrix instruction that wrote it, the operands packed here are read by matrix instructions of the next step, and no
        // exp2 result is used by the instruction right behind it.
        float e[2][2];
        uint32_t w[8];
        auto exps = [&](int c) {
            asm volatile("v_exp_f32 %0, %1" : "=v"(e[c & 1][0]) : "v"(sacc[QB][2 * c]));
            asm volatile("v_exp_f32 %0, %1" : "=v"(e[c & 1][1]) : "v"(sacc[QB][2 * c + 1]));
        };
        auto convert = [&](int c) { asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(w[c]) : "v"(e[c & 1][0]), "v"(e[c & 1][1])); };
        // Sum of pair c and its two partial sums: the same pairs and the same partial sums as pack_probs. A dependent vector
        // instruction right behind its producer costs a wait state, so the sum of a pair joins its partial sum a slice later.
        float pair[2], ls[2];
        auto add_pair = [&](int c) {
            if (c < 2) asm volatile("v_add_f32 %0, %1, %2" : "=v"(ls[c & 1]) : "v"(e[c & 1][0]), "v"(e[c & 1][1]));
            else asm volatile("v_add_f32 %0, %1, %2" : "=v"(pair[c & 1]) : "v"(e[c & 1][0]), "v"(e[c & 1][1]));
        };
        auto join = [&](int c) {
            if (c >= 2) asm volatile("v_add_f32 %0, %0, %1" : "+v"(ls[c & 1]) : "v"(pair[c & 1]));
        };
        if (!LOADS) lds_wait_k<8>(kf);  // the K fragments fetched in the step before (eight V reads may still be on their way)
        // matrix instructions of the step: 0-3 scores; 4, 5 PV of key quarter 0; 6, 7 PV of quarter 1
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (i < 4) {
                sacc[PQ] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i], qf[PQ][i].v, i == 0 ? zero : sacc[PQ], 0, 0, 0);
            } else {
                const int j = (i - 4) >> 1, db = (i - 4) & 1;
                if (!LOADS && i == 4) lds_wait_first4(vfr);
                if (!LOADS && i == 6) lds_wait_last4(vfr);
                Frag vf;
                vf.u = make_uint4(vfr[(j * 2 + db) * 2].x, vfr[(j * 2 + db) * 2].y, vfr[(j * 2 + db) * 2 + 1].x, vfr[(j * 2 + db) * 2 + 1].y);
                oacc[db][PQ] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[PQ][j].v, oacc[db][PQ], 0, 0, 0);
            }
            if (LOADS && i == 3) {
#pragma unroll
                for (int ks = 0; ks < 4; ks++) kf[ks] = lds_read_b128(smem_addr + k_stage + koff[ks], KKB * 32 * 128);
            }
            if (LOADS && (i == 5 || i == 7)) {
                const int j = (i - 4) >> 1;
#pragma unroll
                for (int db = 0; db < 2; db++)
#pragma unroll
                    for (int hi = 0; hi < 2; hi++)
                        vfr[(j * 2 + db) * 2 + hi] = lds_read_tr16_b64(smem_addr + v_stage + voff[db], (VKB * 32 + 16 * j + 8 * hi) * 128);
            }
            if (i == 0) exps(0);
            if (i > 0) convert(i - 1);
            if (i > 1) join(i - 2);
            if (i > 0) add_pair(i - 1);
            if (i < 7) exps(i + 1);
            if (i == 7) {  // the tail of the step's vector work: the last pair and the row-sum update (a short dependent chain)
                convert(7);
                join(6);
                add_pair(7);
                asm volatile("v_nop");
                join(7);
                float both;
                asm volatile("v_add_f32 %0, %1, %2" : "=v"(both) : "v"(ls[0]), "v"(ls[1]));
                asm volatile("v_nop");
                asm volatile("v_add_f32 %0, %0, %1" : "+v"(l_run[QB]) : "v"(both));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        pf[QB][0].u = make_uint4(w[0], w[1], w[2], w[3]);
        pf[QB][1].u = make_uint4(w[4], w[5], w[6], w[7]);
    };
    auto fast_tile = [&](int t) {
        const std::integral_constant<int, 0> I0;
        const std::integral_constant<int, 1> I1;
        const std::integral_constant<bool, true> YES;
        const std::integral_constant<bool, false> NO;
        fast_step(I0, YES, I0, st_cur, I1, st_cur);  // (t,0,0): V of key half 0, K of key half 1
        fast_step(I1, NO, I0, 0, I0, 0);             // (t,0,1)
        tile_barrier();
        if (t + PF + 1 < nt) advance(kv0 + (t + PF + 1) * BKV);
        fetch_tile(st_ld);
        __builtin_amdgcn_sched_barrier(0);
        fast_step(I0, YES, I1, st_cur, I0, st_nxt);  // (t,1,0): V of key half 1, K of key half 0 of tile t+1
        fast_step(I1, NO, I0, 0, I0, 0);             // (t,1,1)
        rotate_stages();
    };

    // Fast tiles: the leading tiles whose units, and the unit whose scores the last of them issues (the first of the next tile), lie
    // wholly inside the sequence. With the reference at zero a probability is 2^score, which is as good as any other reference while
    // the row sums stay inside the range of fp32: every lane's partial row sum must have left the denormal range (a row whose scores
    // are all hugely negative would otherwise be lost) and stay below 2^40 (far from overflow; a row sum of 4250 normalised head
    // vectors with unit weights is below 2^24). Row sums only grow and an infinity stays one, so one look behind the last fast
    // tile is enough (looking inside the loop as well was tried: the extra control flow makes the register allocator spill
    // hundreds of registers). A lane that sees otherwise raises a flag in LDS, a barrier follows, every wavefront reads the
    // flag, and the whole item starts again with every tile going through the general path. Nothing has been written by then,
    // so values that overflowed in the meantime are simply dropped; an input like that pays for the fast tiles in vain.
    __shared__ int unsafe_flag;
    constexpr float L_TINY = 5.421010862427522e-20f /* 2^-64 */, L_HUGE = 1099511627776.0f /* 2^40 */;
    int n_fast = (kv0 + nt * BKV <= T) ? nt : min(nt, (T - kv0 - 32) / BKV);
    if (NORM || n_fast < 4) n_fast = 0;

    for (;;) {
        reset();
        zero_reference();
        if (tid == 0) unsafe_flag = 0;
        // prologue: tiles 0 and 1 on their way, tile 0 visible, scores of the first unit issued
        // (the first key is hidden from the optimiser here: otherwise the address arithmetic of the prologue, which does not
        // change from one attempt to the next, is moved in front of this loop and its results are kept in scratch memory)
        int first_key = kv0;
        asm volatile("" : "+s"(first_key));
        advance(first_key);
        fetch_tile(0);
        if (PF == 1) {
            if (NORM) store_k_normed(kv0, 0);
            if (nt > 1) {
                advance(first_key + BKV);
                fetch_tile(STAGE_BYTES);
                __builtin_amdgcn_s_waitcnt((7 << 4) | (0 << 8) | 4);  // vmcnt(4): all but the four loads of tile 1; lgkmcnt(0)
            } else {
                __builtin_amdgcn_s_waitcnt((7 << 4) | (0 << 8));
            }
            st_cur = 0, st_nxt = STAGE_BYTES, st_nx2 = 0, st_ld = 2 * STAGE_BYTES;
        } else {
            // two more tiles on their way (a sequence shorter than that: its last tile once more, so that the count of requests in
            // flight is the same for every length and "tile t+1 has landed" is a fixed count in the loop)
            if (nt > 1) advance(first_key + BKV);
            fetch_tile(STAGE_BYTES);
            if (nt > 2) advance(first_key + 2 * BKV);
            fetch_tile(2 * STAGE_BYTES);
            __builtin_amdgcn_s_waitcnt((7 << 4) | (0 << 8) | 8);  // vmcnt(8): all but the eight loads of tiles 1 and 2; lgkmcnt(0)
            st_cur = 0, st_nxt = STAGE_BYTES, st_nx2 = 2 * STAGE_BYTES, st_ld = 3 * STAGE_BYTES;
        }
        asm volatile("" ::: "memory");  // (a bare barrier: __syncthreads() would wait for the tiles requested ahead as well)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        load_k(0, 0);
        scores(0, kv0);

        // verdict on the fast tiles so far, the same for every wavefront of the workgroup: flags raised in front of a barrier, read behind it
        auto unsafe = [&]() -> bool {
            const bool bad = !(l_run[0] <= L_HUGE && l_run[1] <= L_HUGE) || l_run[0] < L_TINY || l_run[1] < L_TINY;
            volatile int* flag = &unsafe_flag;
            if (__any(bad)) *flag = 1;
            __syncthreads();
            return __builtin_amdgcn_readfirstlane(*flag) != 0;
        };
        for (int t = 0; t < n_fast; t++) fast_tile(t);
        const bool redo = n_fast > 0 && unsafe();
        if (!redo) {
            if (n_fast > 0) zero_reference();
            for (int t = n_fast; t < nt; t++) tile(t);
            break;
        }
        // start again without fast tiles, once every wavefront is done with the LDS stages and no load into them is in flight
        __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));
        __syncthreads();
        n_fast = 0;
    }
    pv(1, 0);  // PV of the last unit
    pv(1, 1);
    __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));  // the redundant loads issued past the last tile have landed before LDS is reused

    // The lane's coordinates once more, derived behind the loops from a value the optimiser cannot trace back: index arithmetic for
    // the stores below would otherwise be computed up front and carried, through scratch memory, across the loops.
    int lane_e = (int)__lane_id();
    asm volatile("" : "+v"(lane_e));
    const int l32e = lane_e & 31, lke = lane_e >> 5;
    // ---- an item of a split: leave the unnormalised accumulators, the reference and the row sum for the combining kernel ----
    if (s.kv_splits > 1) {
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            const long long prow = (long long)item * BQ + wave * QW + qb * 32 + l32e;
            const float l_tot = l_run[qb] + __shfl_xor(l_run[qb], 32, 64);
            if (lke == 0) *reinterpret_cast<float2*>(s.part_ml + prow * 2) = make_float2(m_run[qb], l_tot);
#pragma unroll
            for (int db = 0; db < 2; db++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    *reinterpret_cast<float4*>(s.part_o + prow * HS + db * 32 + 8 * g + 4 * lke) =
                        make_float4(oacc[db][qb][4 * g + 0], oacc[db][qb][4 * g + 1], oacc[db][qb][4 * g + 2], oacc[db][qb][4 * g + 3]);
        }
        return;
    }
    // ---- normalise; transpose through LDS (each wavefront its own 64-row region) so that rows leave as 16-byte stores ----
    __syncthreads();
    bf16_t* Ow = reinterpret_cast<bf16_t*>(smem) + wave * QW * O_PITCH;
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
        const float l_tot = l_run[qb] + __shfl_xor(l_run[qb], 32, 64);
        const float inv = 1.0f / l_tot;
#pragma unroll
        for (int db = 0; db < 2; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = db * 32 + 8 * g + 4 * lke;
                const uint2 v = make_uint2(pack_bf16x2(oacc[db][qb][4 * g + 0] * inv, oacc[db][qb][4 * g + 1] * inv),
                                           pack_bf16x2(oacc[db][qb][4 * g + 2] * inv, oacc[db][qb][4 * g + 3] * inv));
                *reinterpret_cast<uint2*>(&Ow[(qb * 32 + l32e) * O_PITCH + d0]) = v;
            }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // 64 rows x 8 chunks per wavefront = 512 chunks, 8 per lane_e
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int c = lane_e + i * 64;
        const int row = c >> 3, ch = c & 7;
        const int t = q0 + row;
        if (t < TQ) {
            const int seg = (t < Tq0) ? 0 : 1;
            if (s.out[seg]) {
                bf16_t* op = s.out[seg] + ((long long)b * s.Tq[seg] + (seg ? t - Tq0 : t)) * s.ld_out[seg] + h * HS + ch * 8;
                *reinterpret_cast<uint4*>(op) = *reinterpret_cast<const uint4*>(&Ow[row * O_PITCH + ch * 8]);
            }
        }
    }
}

// Merges the kv_splits partial results of every query of a split set, in split order: with M = max_s m_s,
// out = sum_s O_s 2^(m_s - M) / sum_s l_s 2^(m_s - M). 16 lanes per query row, 4 of the 64 output values each.
__global__ void __launch_bounds__(256) attn_combine_kernel(const SegDev s, int B) {
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    const int sub = (int)(idx & 15);
    const long long r = idx >> 4;  // (batch, head, query block, row in block)
    const long long rows = (long long)B * s.NH * s.nqb * BQ;
    if (r >= rows) return;
    const int row = (int)(r % BQ);
    const long long t = r / BQ;  // (batch, head, query block)
    const int qblk = (int)(t % s.nqb);
    const long long bh = t / s.nqb;
    const int b = (int)(bh / s.NH), h = (int)(bh % s.NH);
    const int q = qblk * BQ + row, Tq0 = s.Tq[0];
    if (q >= s.Tq[0] + s.Tq[1]) return;
    const int seg = (q < Tq0) ? 0 : 1;
    if (!s.out[seg]) return;
    float mmax = -3.0e38f;
    for (int k = 0; k < s.kv_splits; k++) mmax = fmaxf(mmax, s.part_ml[((t * s.kv_splits + k) * BQ + row) * 2]);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float l = 0.f;
    for (int k = 0; k < s.kv_splits; k++) {
        const long long prow = (t * s.kv_splits + k) * BQ + row;
        const float2 ml = *reinterpret_cast<const float2*>(s.part_ml + prow * 2);
        const float w = __builtin_amdgcn_exp2f(ml.x - mmax);
        const float4 o = *reinterpret_cast<const float4*>(s.part_o + prow * HS + sub * 4);
        acc.x = fmaf(o.x, w, acc.x); acc.y = fmaf(o.y, w, acc.y); acc.z = fmaf(o.z, w, acc.z); acc.w = fmaf(o.w, w, acc.w);
        l = fmaf(ml.y, w, l);
    }
    const float inv = 1.0f / l;
    bf16_t* op = s.out[seg] + ((long long)b * s.Tq[seg] + (seg ? q - Tq0 : q)) * s.ld_out[seg] + h * HS + sub * 4;
    *reinterpret_cast<uint2*>(op) = make_uint2(pack_bf16x2(acc.x * inv, acc.y * inv), pack_bf16x2(acc.z * inv, acc.w * inv));
}

int fill_set(const AttnSegments& a, int NH, SegDev& s, bool& norm) {
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
            if (a.rms_q[i] || a.rms_k[i]) norm = true;
        }
    }
    s.NH = NH;
    s.nqb = (a.Tq[0] + a.Tq[1] + BQ - 1) / BQ;
    s.kv_splits = 1;
    s.part_o = nullptr;
    s.part_ml = nullptr;
    return SD3_OK;
}

}  // namespace

// Key splits for the context queries of a joint attention, or 0 when the one-set launch is the better choice. The joint sequence
// of the headline shape has 17 query blocks of 256 per (batch, head), the last one holding the 154 leftover rows: 816 workgroups,
// which run as long as 1024 would (two per compute unit: 512 at a time). With the latent queries alone the count is 768, whose
// last 256 have a compute unit to themselves and finish early; the context queries then go, split four ways along the keys into
// short work items, into the slots those leave free, and a small kernel merges their partial results.
int g_attention_context_splits = -1;  // -1: chosen from the sizes; 0: never split; n >= 2: n splits wherever splitting applies (sd3_tune)
int attention_bf16_context_splits(int Tc, int Tx) {
    const int nt_all = (Tc + Tx + BKV - 1) / BKV;
    if (Tc <= 0 || Tc > BQ || Tx < 4 * BQ || nt_all < 16 || g_attention_context_splits == 0) return 0;
    int S = g_attention_context_splits > 0 ? g_attention_context_splits : 4;
    S = S < 2 ? 2 : (S > 8 ? 8 : S);
    // every split must own at least one key tile: with ceil(nt_all / S) tiles each, the last one starts at (S-1) * that
    while (S > 1 && ((nt_all + S - 1) / S) * (S - 1) >= nt_all) S--;
    return S > 1 ? S : 0;
}
size_t attention_bf16_split_workspace_floats(int B, int NH, int Tc, int splits) {
    const size_t items = (size_t)B * NH * ((Tc + BQ - 1) / BQ) * splits;
    return items * BQ * (HS + 2);
}

int attention_bf16_multi(const AttnSegments* jobs, const int* kv_splits, float* const* split_ws, int n, int B, int NH, int hs, hipStream_t st) {
    if (n < 1 || n > MAX_SETS) return fail(SD3_ERR_INVALID_ARG, "attention: 1 to %d sets per launch (got %d)", MAX_SETS, n);
    if (hs != HS) return fail(SD3_ERR_UNSUPPORTED, "attention (bf16): head_dim must be 64 (got %d)", hs);
    if (B <= 0 || NH <= 0) return SD3_OK;
    AttnSets sets{};
    bool norm = false;
    int m = 0, total = 0;
    for (int i = 0; i < n; i++) {
        const AttnSegments& a = jobs[i];
        const int T = a.T[0] + a.T[1], TQ = a.Tq[0] + a.Tq[1];
        if (TQ <= 0) continue;
        if (T <= 0) return fail(SD3_ERR_INVALID_ARG, "attention: no keys");
        SegDev& s = sets.set[m];
        SD3_TRY(fill_set(a, NH, s, norm));
        const int S = kv_splits ? kv_splits[i] : 1;
        if (S > 1) {
            const int nt_all = (T + BKV - 1) / BKV, per = (nt_all + S - 1) / S;
            if (per * (S - 1) >= nt_all) return fail(SD3_ERR_INVALID_ARG, "attention: %d key splits leave an empty one for %d keys", S, T);
            if (!split_ws || !split_ws[i]) return fail(SD3_ERR_INVALID_ARG, "attention: a split set needs its workspace");
            s.kv_splits = S;
            s.part_o = split_ws[i];
            s.part_ml = split_ws[i] + (size_t)B * NH * s.nqb * S * BQ * HS;
        }
        total += s.nqb * NH * B * s.kv_splits;
        sets.end[m++] = total;
    }
    if (m == 0) return SD3_OK;
    for (int i = m; i < MAX_SETS; i++) sets.end[i] = total;
    const float q_scale = 1.4426950408889634f / sqrtf((float)HS);
    dim3 grid((unsigned)total), block(NW * 64);
    if (norm) hipLaunchKernelGGL(flash_attn_bf16_kernel<true>, grid, block, 0, st, sets, q_scale, 1e-6f);
    else hipLaunchKernelGGL(flash_attn_bf16_kernel<false>, grid, block, 0, st, sets, q_scale, 1e-6f);
    SD3_TRY(launch_status("flash_attention_bf16"));
    for (int i = 0; i < m; i++) {
        const SegDev& s = sets.set[i];
        if (s.kv_splits <= 1) continue;
        const long long threads = (long long)B * NH * s.nqb * BQ * 16;
        hipLaunchKernelGGL(attn_combine_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, s, B);
        SD3_TRY(launch_status("attention_combine"));
    }
    return SD3_OK;
}

int attention_bf16(const AttnSegments& a, int B, int NH, int hs, hipStream_t st) { return attention_bf16_multi(&a, nullptr, nullptr, 1, B, NH, hs, st); }

}  // namespace sd3
