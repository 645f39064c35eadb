// bf16 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16), fp32 accumulation:
//   out(M,N) = A(M,K) @ Wp^T + epilogue,  A bf16 row-major, Wp bf16 (N,K) row-major (the reference's (K,N) fp32
//   weight transposed and rounded once by pack_weight_bf16), so that both operands are K-contiguous.
// It replaces linear / partial_linear of the reference (modules.cpp:475-511) for the QKV, out-projection and MLP
// layers. Epilogues: bias | bias+GELU-tanh | bias+SiLU | gate*(.)+residual (fp32, in place) | bias + row table.
//
// Data path: global -> LDS with direct loads (global_load_lds_dwordx4: no registers, no VALU), a ring of STAGES
// LDS buffers with one workgroup barrier per 64-deep K tile; LDS rows are 128 bytes with the 16-byte chunk index
// XOR-swizzled by a key of the row, which makes both the linear LDS fill and the 16-byte MFMA operand reads conflict-free.
#include "common.hpp"

#include <type_traits>

namespace sd3 {
namespace {

constexpr int BK = 64;  // bf16 elements per K tile = 128 bytes per LDS row

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;

struct EpiDev {
    const float* a_scale;  // fp8 operands: one factor per row of A (null: 1)
    const float* w_scale;  // fp8 operands: one factor per output column (null: 1)
    const float* bias;
    const float* gate;
    const float* resid;
    const float* table;
    int gate_ld;
    int rows_per_batch;
};

// XOR key of an LDS row: rows r..r+7 get 8 different keys (no conflicts on 8-lane / 32-bank groups) and rows r, r+8 get
// keys that differ in bit 0 (no conflicts on 16-lane / 64-bank groups either).
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }
// The key for tiles whose fragments are read in the 16x16x32 layout (lane l: row l % 16, chunk 4 * step + l / 16). A 16-byte LDS
// read is served in four phases of 16 lanes (lanes 0-3, 12-15, 20-23, 24-27; 4-7, 8-11, 16-19, 28-31; the same + 32), so a phase
// holds rows 0-3 and 12-15 with one chunk index and rows 4-11 with the next: even and odd rows lie in different halves of the 64
// banks, and row & 6 gives the four even (odd) rows of either group the keys 0, 2, 4, 6 -- with the chunk indices one apart, all
// eight 16-byte slots of a half. (With swz() that pattern hits every slot twice: the bank-conflict counter read 47 % of the LDS
// cycles; the 32x32 layout, lane l: row l % 32, is conflict-free with swz() and would not be with this key.)
__device__ __forceinline__ int swz16(int row) { return row & 6; }

// s_waitcnt vmcnt(n) with the other counters left unconstrained (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14])
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Workgroup -> output tile. The hardware hands consecutive workgroup ids to the 8 XCDs in turn, and each XCD has its own L2, so
// the workgroups that land on one XCD should share as few A row panels and W column panels as possible. When the tile grid
// divides that way, the XCDs take a 4 x 2 arrangement of rectangular blocks of it (for 32 x 24 tiles: 8 x 12 each, 8 + 12 panels
// through that L2 instead of 4 + 24 with contiguous runs of tile rows), walked in bands of 4 tile rows so that the 32 tiles an XCD
// works on at a time form a 4 x 8 patch. Otherwise every XCD gets a contiguous run of tiles, walked in bands of 2 tile rows
// (measured over 1, 2, 3, 4, 8, 16 on the 24-block forward).
__device__ __forceinline__ void tile_of_workgroup(int wg, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
    constexpr int XCDS = 8, XR = 4, XC = 2, BAND = 4, GROUP_M = 2;
    const int total = tiles_m * tiles_n;
    const int xcd = wg % XCDS, local = wg / XCDS;
    if (tiles_m % (XR * BAND) == 0 && tiles_n % XC == 0) {
        const int bm = tiles_m / XR, bc = tiles_n / XC;  // the XCD's block: bm x bc tiles, exactly total / 8
        const int band = local / (BAND * bc), r = local % (BAND * bc);
        tile_m = (xcd / XC) * bm + band * BAND + r % BAND;
        tile_n = (xcd % XC) * bc + r / BAND;
        return;
    }
    const int per = (total + XCDS - 1) / XCDS, tall = (total % XCDS) ? (total % XCDS) : XCDS;  // `tall` XCDs get `per` tiles, the rest per-1
    const int t = (xcd < tall) ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
    const int in_group = GROUP_M * tiles_n, group = t / in_group, first_m = group * GROUP_M;
    const int gsize = min(tiles_m - first_m, GROUP_M);
    tile_m = first_m + (t % in_group) % gsize;
    tile_n = (t % in_group) / gsize;
}

// LDS bytes of a configuration: the tile ring, or the epilogue staging slabs if those are larger
template <int BM, int BN, int WM, int WN, int STAGES>
constexpr int smem_bytes() {
    constexpr int ring = STAGES * (BM + BN) * 128, epi = WM * WN * 32 * (BN / WN + 4) * 4;
    return ring > epi ? ring : epi;
}

// One launch covers up to three independent problems of the same kind (latent-stream, dual-branch and context-stream
// layer): work items [0, end[0]) belong to problem 0, [end[0], end[1]) to problem 1, [end[1], end[2]) to problem 2.
struct Prob {
    const bf16_t* A;
    const bf16_t* Wp;
    void* out;
    int ldc, M, N, K;
    EpiDev epi;
};
constexpr int MAX_PROBS = 3;
struct ProbSet {
    Prob p[MAX_PROBS];
    int end[MAX_PROBS];  // running totals of tiles
};

// One output tile: K loop + epilogue. `wg` is the tile's position in the XCD-aware order of its problem.
typedef __attribute__((__vector_size__(8 * sizeof(int)))) int i32x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4_t;

// FP8: the operands are OCP e4m3 bytes (A (M,K) and Wp (N,K), both K-contiguous); a 128-byte LDS row then holds 128 k values and
// the matrix instruction is v_mfma_f32_32x32x64_f8f6f4; the accumulators are multiplied by a_scale[m] * w_scale[n] in the epilogue.
template <int BM, int BN, int WM, int WN, int STAGES, int EPI, bool OUT_F32, bool FP8>
__device__ __forceinline__ void gemm_tile(const Prob& pr, const int wg, char* smem) {
    constexpr int ESZ = FP8 ? 1 : 2;                  // bytes per operand element
    const char* __restrict__ A = reinterpret_cast<const char*>(pr.A);
    const char* __restrict__ Wp = reinterpret_cast<const char*>(pr.Wp);
    void* __restrict__ out_ = pr.out;
    const int ldc = pr.ldc, M = pr.M, N = pr.N, K = pr.K;
    const EpiDev epi = pr.epi;
    constexpr int NT = WM * WN * 64;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;      // 32x32 MFMA blocks per wavefront
    constexpr int A_BYTES = BM * 128, STAGE_BYTES = (BM + BN) * 128;
    constexpr int LA = BM * 8 / NT, LB = BN * 8 / NT;        // 16-byte chunks per thread per tile
    static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile rows must divide evenly over the threads");
    static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0 && (BM == 256 || (BM % (WM * 32) == 0 && BN % (WN * 32) == 0)), "wavefront tiles are made of 16x16 (256-row tiles) or 32x32 blocks");

    constexpr bool M16 = (BM == 256) && !FP8;  // 16x16x32 matrix instructions (see below)
    auto key = [](int row) { return M16 ? swz16(row) : swz(row); };
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: LDS destinations of the direct loads are then scalar
    const int wm = wave / WN, wn = wave % WN;
    int tile_m, tile_n;
    tile_of_workgroup(wg, (M + BM - 1) / BM, (N + BN - 1) / BN, tile_m, tile_n);
    const int m_blk = tile_m * BM, n_blk = tile_n * BN;

    // ---- loader: chunk q = i*NT + tid lands at LDS byte q*16 of its tile, i.e. row q/8, physical chunk q%8 ----
    const char* ga[LA];
    const char* gb[LB];
    const long long row_bytes = (long long)K * ESZ;
#pragma unroll
    for (int i = 0; i < LA; i++) {
        const int q = i * NT + tid, row = q >> 3, lc = (q & 7) ^ key(row);
        const int m = min(m_blk + row, M - 1);  // rows beyond M re-read the last row; their results are never stored
        ga[i] = A + (long long)m * row_bytes + lc * 16;
    }
#pragma unroll
    for (int i = 0; i < LB; i++) {
        const int q = i * NT + tid, row = q >> 3, lc = (q & 7) ^ key(row);
        const int n = min(n_blk + row, N - 1);
        gb[i] = Wp + (long long)n * row_bytes + lc * 16;
    }
    auto issue_tile = [&](int kt, int stage) {
        char* sa = smem + stage * STAGE_BYTES + wave * 1024;
        char* sb = sa + A_BYTES;
#pragma unroll
        for (int i = 0; i < LA; i++) __builtin_amdgcn_global_load_lds((glb_ptr_t)(ga[i] + kt * 128), (lds_ptr_t)(sa + i * NT * 16), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < LB; i++) __builtin_amdgcn_global_load_lds((glb_ptr_t)(gb[i] + kt * 128), (lds_ptr_t)(sb + i * NT * 16), 16, 0, 0);
    };

    // Two matrix instructions. 256x256 tiles use v_mfma_f32_16x16x32_bf16: on this device the clock under matrix load is set by
    // the power limit, and measured on random operands the 16x16x32 form sustains 15-24 % more than 32x32x16 at the same nominal
    // rate (half as many accumulator updates per product). 128x128 tiles keep v_mfma_f32_32x32x16_bf16: with four wavefronts per
    // workgroup the finer instruction stream measured 5-15 % slower there. Both forms give bit-identical results.
    constexpr int MI = BM / WM / 16, NJ = BN / WN / 16;      // 16x16 blocks per wavefront
    f32x16_t acc[M16 ? 1 : TM][M16 ? 1 : TN];
    f32x4_t acc16[M16 ? MI : 1][M16 ? NJ : 1];
#pragma unroll
    for (int i = 0; i < (M16 ? 1 : TM); i++)
#pragma unroll
        for (int j = 0; j < (M16 ? 1 : TN); j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
#pragma unroll
    for (int i = 0; i < (M16 ? MI : 1); i++)
#pragma unroll
        for (int j = 0; j < (M16 ? NJ : 1); j++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc16[i][j][r] = 0.f;

    static_assert(STAGES >= 2 && (STAGES - 1) * (LA + LB) < 64, "ring depth: at least two stages, and the loads in flight must fit the 6-bit counter");
    const int nkt = (int)(row_bytes / 128);
    const int l32 = lane & 31, lk = lane >> 5;   // position in a 32x32 block
    const int lr = lane & 15, lg = lane >> 4;    // position in a 16x16 block

    // ---- epilogue set-up ----
    constexpr int WNC = BN / WN;        // columns per wavefront
    constexpr int EP = WNC + 4;         // fp32 pitch of the staging slab
    static_assert(WM * WN * 32 * EP * 4 <= smem_bytes<BM, BN, WM, WN, STAGES>(), "epilogue staging must fit in the LDS allocation");
    constexpr int CPR = WNC / 4;        // float4 chunks per row
    static_assert(WNC % 4 == 0 && CPR <= 64, "a row of the wavefront's slab is made of float4 chunks");
    // rows covered by one pass of the wavefront: the largest power of two with RPI * CPR <= 64 (when CPR does not divide 64, as with
    // 48-column slabs, the lanes beyond RPI * CPR sit the epilogue out)
    constexpr int RPI = CPR > 32 ? 1 : CPR > 16 ? 2 : CPR > 8 ? 4 : CPR > 4 ? 8 : CPR > 2 ? 16 : 32;
    // rows per slab: 32 (measured faster than 16 on the 64-column slabs of the 256x256 tile), 16 for 48-column slabs
    constexpr int SR = (M16 && WNC % 64 != 0) ? 16 : 32;
    constexpr int NSLAB = BM / WM / SR;
    constexpr int NP = SR / RPI;        // rows of a slab per lane
    float* slab = reinterpret_cast<float*>(smem) + wave * 32 * EP;
    float* outf = reinterpret_cast<float*>(out_);
    bf16_t* outh = reinterpret_cast<bf16_t*>(out_);
    const bool lane_on = lane < RPI * CPR;
    const int e_row = lane_on ? lane / CPR : 0, e_col = lane_on ? (lane % CPR) * 4 : 0;
    const int n0 = n_blk + wn * WNC + e_col;
    const bool vec_ok = ((N & 3) == 0) && ((ldc & 3) == 0);
    const bool table_vec = EPI == EPI_BIAS_ROWADD && ((epi.gate_ld & 3) == 0) && ((reinterpret_cast<uintptr_t>(epi.table) & 15) == 0);
    const int nvalid = lane_on ? min(4, N - n0) : 0;  // <= 0 for lanes beyond the last column (and for lanes that sit out)
    // batch index of a row without a division per row: the tile starts in batch b0 and crosses a boundary every rpb rows
    const int rpb = epi.rows_per_batch, b0 = m_blk / rpb;
    // gated layers: the residual rows of the NEXT slab are requested before the current slab goes through LDS, so that
    // their latency is not paid once per slab with nothing else to do
    constexpr bool PREFETCH_RESID = (EPI == EPI_GATE_RESID);
    float4 rnext[PREFETCH_RESID ? NP : 1];
    auto request_resid = [&](int i) {
        if (PREFETCH_RESID && vec_ok)
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int m = m_blk + wm * (BM / WM) + i * SR + p * RPI + e_row;
                if (m < M && nvalid > 0) rnext[p] = *reinterpret_cast<const float4*>(epi.resid + (long long)m * ldc + n0);
            }
    };
    if constexpr (M16) {
        // v_mfma_f32_16x16x32_bf16 operands: lane l holds row (column) l%16 of its block and the 8 consecutive k values 8*(l/16).. of
        // the 32-deep step: one 16-byte chunk of the row's 128-byte LDS line, chunk (4*step + l/16) ^ swz16(row)
        const int sw = swz16(lr);  // (block offsets are multiples of 16 rows, which the key does not see)
        const int a_off = (wm * (BM / WM) + lr) * 128, b_off = A_BYTES + (wn * (BN / WN) + lr) * 128;
        // A fragments: one buffer (the fragment of the next step replaces a[i] as soon as row block i is done), except for the last
        // TAIL row blocks, which have two so that no fragment read is left to issue behind the last matrix instructions of a step
        // (it would be waited for at once); B fragments: two buffers
        // (one such row block for the large tiles: more of them cost registers, which the gated fp32 epilogue then spills)
        constexpr int TAIL = MI >= 6 ? 1 : MI / 2, HEAD = MI - TAIL;
        // Where the direct loads of the next-but-one tile go among the 32 matrix instructions of a tile's last step: one behind every
        // second instruction, from the seventh on (behind the fragment reads of the first row block). Swept on the 24-block forward,
        // ms per step: first slot 0 / 2 / 3 / 4 / 5 / 6 / 7 / 8 / 16 with one load per instruction: +0.43 / +0.2 / +0.03 / 0 / -0.05 /
        // -0.1 / +0.18 / +0.15 / +0.56; from slot 6 every second / third instruction: -0.14 / -0.1.
        constexpr int LOAD_FIRST = 6, LOAD_EVERY = 2;
        static_assert(HEAD >= TAIL && TAIL >= 1, "every tail fragment is fetched behind a head row block");
        bf16x8_t a[HEAD], at[2][TAIL], b[2][NJ];
        auto a_addr = [&](const char* st, int s, int i) { return reinterpret_cast<const bf16x8_t*>(st + a_off + i * 16 * 128 + (((4 * s + lg) ^ sw) * 16)); };
        auto load_b = [&](const char* st, int s, int buf) {
#pragma unroll
            for (int j = 0; j < NJ; j++) b[buf][j] = *reinterpret_cast<const bf16x8_t*>(st + b_off + j * 16 * 128 + (((4 * s + lg) ^ sw) * 16));
        };

        // Every stage is filled up front and exactly one tile is requested per K tile after that (past the end: the last tile
        // once more, into a buffer nobody reads again), so "tile kt+1 has landed" is always "all but the newest STAGES-2 tiles".
#pragma unroll
        for (int s = 0; s < STAGES; s++) issue_tile(min(s, nkt - 1), s);
        wait_vmcnt<(STAGES - 1) * (LA + LB)>();
        // tile 0 is in LDS. A bare barrier between compiler fences: __syncthreads() would add a wait for ALL loads in flight
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        load_b(smem, 0, 0);
#pragma unroll
        for (int i = 0; i < HEAD; i++) a[i] = *a_addr(smem, 0, i);
#pragma unroll
        for (int i = 0; i < TAIL; i++) at[0][i] = *a_addr(smem, 0, HEAD + i);
        __builtin_amdgcn_sched_group_barrier(0x100, MI + NJ, 0);

        constexpr int KS = BK / 32;
        static_assert(KS == 2, "two 32-deep steps per K tile");
        // one 32-deep step on the fragments in a[], at[buf] and b[buf]; with FETCH, the fragments of step ns of stage nst are fetched
        // behind the matrix instructions: the B fragments first, the A fragment of head row block i once that block is done, the tail
        // fragments (into the other buffer) behind the first head blocks
        auto step = [&](int buf, const char* nst, int ns, auto fetch_tag, auto loads_tag) {
            constexpr bool FETCH = decltype(fetch_tag)::value, LOADS = decltype(loads_tag)::value;
            constexpr int NLOADS = LA + LB;
            static_assert(LOAD_FIRST + NLOADS * LOAD_EVERY <= MI * NJ, "the direct loads fit between the matrix instructions of one step");
            if (FETCH) load_b(nst, ns, buf ^ 1);
#pragma unroll
            for (int i = 0; i < MI; i++) {
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    acc16[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(i < HEAD ? a[i] : at[buf][i - HEAD], b[buf][j], acc16[i][j], 0, 0, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (FETCH && i == 0) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                       // B fragment j of the next step
                    if (LOADS && i * NJ + j >= LOAD_FIRST && i * NJ + j < LOAD_FIRST + NLOADS * LOAD_EVERY && (i * NJ + j - LOAD_FIRST) % LOAD_EVERY == 0) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one direct load
                }
                if (FETCH && i < HEAD) {
                    a[i] = *a_addr(nst, ns, i);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    if (i < TAIL) {
                        at[buf ^ 1][i] = *a_addr(nst, ns, HEAD + i);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    }
                }
            }
        };
        // One K tile. The workgroup barrier sits in front of the LAST step of a tile, not behind it: by then every fragment
        // of tile kt is in registers (or on its way: waited for), so its buffer can be handed to the loads of tile kt+STAGES, and the
        // loads' issue and the fragment reads of tile kt+1 are interleaved with the matrix instructions of that last step.
        auto k_tile = [&](const int kt, auto has_next_tag) {
            constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
            const char* st = smem + (kt % STAGES) * STAGE_BYTES;
            step(0, st, 1, std::true_type{}, std::false_type{});
            if (HAS_NEXT) {
                // this thread's loads of tile kt+1 have landed (vmcnt: all but the newest STAGES-2 tiles) and its reads of tile kt are done (lgkmcnt(0))
                constexpr int INFLIGHT = (STAGES - 2) * (LA + LB);
                __builtin_amdgcn_s_waitcnt((INFLIGHT & 15) | (7 << 4) | ((INFLIGHT >> 4) << 14));
                asm volatile("" ::: "memory");  // (the barrier builtin alone does not keep the compiler from moving LDS reads across it)
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                issue_tile(min(kt + STAGES, nkt - 1), kt % STAGES);
                step(1, smem + ((kt + 1) % STAGES) * STAGE_BYTES, 0, std::true_type{}, std::true_type{});
            } else {
                step(1, st, 0, std::false_type{}, std::false_type{});
            }
        };
        for (int kt = 0; kt + 1 < nkt; kt++) k_tile(kt, std::true_type{});
        k_tile(nkt - 1, std::false_type{});
    } else {
        // operand addresses inside a stage: row*128 + (chunk ^ sw)*16 with sw = swz(row) = swz(l32) (block offsets are multiples of 16).
        // bf16: k-step ks (16 deep) takes chunk 2*ks + lk; fp8: k-step ks (64 deep) takes the two chunks 4*ks + 2*lk, +1
        const int sw = swz(l32);
        const int a_off = (wm * (BM / WM) + l32) * 128, b_off = A_BYTES + (wn * (BN / WN) + l32) * 128;
        // operand fragments of k-step ks live in buffer ks&1; those of step ks+1 are fetched from LDS while the matrix cores work on step ks
        using frag_t = std::conditional_t<FP8, i32x8_t, bf16x8_t>;
        frag_t a[2][TM], b[2][TN];
        auto read_frag = [&](const char* row, int ks) -> frag_t {
            if constexpr (FP8) {
                const i32x4_t lo = *reinterpret_cast<const i32x4_t*>(row + (((4 * ks + 2 * lk) ^ sw) * 16));
                const i32x4_t hi = *reinterpret_cast<const i32x4_t*>(row + (((4 * ks + 2 * lk + 1) ^ sw) * 16));
                return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            } else {
                return *reinterpret_cast<const bf16x8_t*>(row + (((2 * ks + lk) ^ sw) * 16));
            }
        };
        auto fetch = [&](const char* st, int ks, int buf) {
#pragma unroll
            for (int i = 0; i < TM; i++) a[buf][i] = read_frag(st + a_off + i * 32 * 128, ks);
#pragma unroll
            for (int j = 0; j < TN; j++) b[buf][j] = read_frag(st + b_off + j * 32 * 128, ks);
        };
        constexpr int DSR = FP8 ? 2 : 1;  // LDS reads per fragment

        // Every stage is filled up front and exactly one tile is requested per K tile after that (past the end: the last tile
        // once more, into a buffer nobody reads again), so "tile kt+1 has landed" is always "all but the newest STAGES-2 tiles".
#pragma unroll
        for (int s = 0; s < STAGES; s++) issue_tile(min(s, nkt - 1), s);
        wait_vmcnt<(STAGES - 1) * (LA + LB)>();
        // tile 0 is in LDS. A bare barrier between compiler fences: __syncthreads() would add a wait for ALL loads in flight
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        fetch(smem, 0, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, DSR * (TM + TN), 0);

        constexpr int KS = FP8 ? 2 : 4;  // k-steps per 128-byte K tile
        // One K tile. The workgroup barrier sits in front of the LAST k-step of a tile, not behind it: by then every fragment
        // of tile kt is in registers (or on its way: waited for), so its buffer can be handed to the loads of tile kt+2, and the
        // loads' issue and the first fragment reads of tile kt+1 are interleaved with the matrix instructions of that last
        // step. With the barrier between tiles instead, the matrix pipeline drains at every tile boundary while all
        // wavefronts of the compute unit wait for the barrier, issue their loads and wait for their first LDS reads.
        auto k_tile = [&](const int kt, auto has_next_tag) {
            constexpr bool HAS_NEXT = decltype(has_next_tag)::value;
            const char* st = smem + (kt % STAGES) * STAGE_BYTES;
            auto mfmas = [&](int buf) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        if constexpr (FP8) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[buf][i], b[buf][j], acc[i][j], 0, 0, 0, 0, 0, 0);
                        else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[buf][i], b[buf][j], acc[i][j], 0, 0, 0);
                    }
            };
            // scheduling pattern of a step: behind each of the first matrix instructions one LDS fragment read of the next step
            // (and, in the last step, one direct global->LDS load of the tile after next), so that their issue and latency are
            // covered by matrix work
#pragma unroll
            for (int ks = 0; ks + 1 < KS; ks++) {
                fetch(st, ks + 1, (ks + 1) & 1);
                mfmas(ks & 1);
#pragma unroll
                for (int x = 0; x < TM + TN; x++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);    // 1 MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, DSR, 0);  // 1 fragment read
                }
                __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
            }
            if (HAS_NEXT) {
                // this thread's loads of tile kt+1 have landed (vmcnt: all but the newest STAGES-2 tiles) and its reads of tile kt are done (lgkmcnt(0))
                constexpr int INFLIGHT = (STAGES - 2) * (LA + LB);
                __builtin_amdgcn_s_waitcnt((INFLIGHT & 15) | (7 << 4) | ((INFLIGHT >> 4) << 14));
                asm volatile("" ::: "memory");  // (the barrier builtin alone does not keep the compiler from moving LDS reads across it)
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                issue_tile(min(kt + STAGES, nkt - 1), kt % STAGES);
                fetch(smem + ((kt + 1) % STAGES) * STAGE_BYTES, 0, 0);
            }
            mfmas((KS - 1) & 1);
            if (HAS_NEXT) {
                constexpr int NLOADS = LA + LB, NM = TM * TN;
                constexpr int LPS = (NLOADS + NM - 1) / NM;   // loads per slot
                static_assert(TM + TN <= NM, "more fragment reads than matrix instructions to hide them behind");
#pragma unroll
                for (int x = 0; x < NM; x++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                              // 1 MFMA
                    if (x < TM + TN) __builtin_amdgcn_sched_group_barrier(0x100, DSR, 0);            // 1 fragment read
                    if (x * LPS < NLOADS) __builtin_amdgcn_sched_group_barrier(0x020, LPS, 0);       // VMEM reads
                }
            }
        };
        for (int kt = 0; kt + 1 < nkt; kt++) k_tile(kt, std::true_type{});
        k_tile(nkt - 1, std::false_type{});
    }

    // ---- epilogue. The MFMA C layouts (32x32: lane = column, register r = row 8*(r/4) + 4*(lane/32) + r%4) would give 2- or
    // 4-byte scattered stores; each wavefront instead transposes one 32-row slab at a time through its private LDS
    // region (the tile ring is free now) and leaves with 16 lanes covering 64 contiguous columns of one row.
    __syncthreads();
    float bias4[4] = {0.f, 0.f, 0.f, 0.f};
    if (epi.bias)
#pragma unroll
        for (int c = 0; c < 4; c++)
            if (c < nvalid) bias4[c] = epi.bias[n0 + c];
    float ws4[4] = {1.f, 1.f, 1.f, 1.f};  // fp8: the output column's factor
    if (FP8 && epi.w_scale)
#pragma unroll
        for (int c = 0; c < 4; c++)
            if (c < nvalid) ws4[c] = epi.w_scale[n0 + c];
    request_resid(0);
#pragma unroll
    for (int i = 0; i < NSLAB; i++) {
        float4 rcur[PREFETCH_RESID ? NP : 1];
        if (PREFETCH_RESID) {
#pragma unroll
            for (int p = 0; p < NP; p++) rcur[p] = rnext[p];
            if (i + 1 < NSLAB) request_resid(i + 1);
        }
        if constexpr (M16) {
            // C layout of a 16x16 block: lane = column l%16, register r = row 4*(l/16) + r
#pragma unroll
            for (int ii = 0; ii < SR / 16; ii++)
#pragma unroll
                for (int j = 0; j < NJ; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++) slab[(16 * ii + 4 * lg + r) * EP + j * 16 + lr] = acc16[(SR / 16) * i + ii][j][r];
        } else {
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) slab[(8 * (r >> 2) + 4 * lk + (r & 3)) * EP + j * 32 + l32] = acc[i][j][r];
        }
        // LDS operations of one wavefront execute in program order, so the reads below see the writes above without a
        // fence (a fence would also make the wavefront wait for its outstanding global stores on every pass)
        __builtin_amdgcn_wave_barrier();
        // all rows of the slab are read into registers of their own before the first store is issued: a store keeps its data
        // registers busy until it has left, so reusing one register set per row would put a full store round trip between rows
        float4 vals[NP];
#pragma unroll
        for (int p = 0; p < NP; p++) vals[p] = *reinterpret_cast<const float4*>(&slab[(p * RPI + e_row) * EP + e_col]);
        float4 res[NP];
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int row = p * RPI + e_row;
            const int m = m_blk + wm * (BM / WM) + i * SR + row;
            if (m < M && nvalid > 0) {
                float4 a4 = vals[p];
                if constexpr (FP8) {
                    const float sa = epi.a_scale ? epi.a_scale[m] : 1.0f;
                    a4.x *= sa * ws4[0]; a4.y *= sa * ws4[1]; a4.z *= sa * ws4[2]; a4.w *= sa * ws4[3];
                }
                float v[4] = {a4.x + bias4[0], a4.y + bias4[1], a4.z + bias4[2], a4.w + bias4[3]};
                const long long idx = (long long)m * ldc + n0;
                if (EPI == EPI_BIAS_GELU) {
#pragma unroll
                    for (int c = 0; c < 4; c++) v[c] = gelu_tanh_f(v[c]);
                } else if (EPI == EPI_BIAS_SILU) {
#pragma unroll
                    for (int c = 0; c < 4; c++) v[c] = v[c] / (1.0f + __expf(-v[c]));
                } else if (EPI == EPI_GATE_RESID) {
                    int bi = b0;
                    for (int nb = (b0 + 1) * rpb; nb <= m; nb += rpb) bi++;  // at most BM/rpb + 1 steps, 0 or 1 in practice
                    const float* g = epi.gate + (long long)bi * epi.gate_ld + n0;
                    if (vec_ok) {
                        const float4 g4 = *reinterpret_cast<const float4*>(g), r4 = rcur[PREFETCH_RESID ? p : 0];
                        v[0] = r4.x + g4.x * v[0]; v[1] = r4.y + g4.y * v[1]; v[2] = r4.z + g4.z * v[2]; v[3] = r4.w + g4.w * v[3];
                    } else {
#pragma unroll
                        for (int c = 0; c < 4; c++)
                            if (c < nvalid) v[c] = epi.resid[idx + c] + g[c] * v[c];
                    }
                } else if (EPI == EPI_BIAS_ROWADD) {
                    const float* t = epi.table + (long long)(m % rpb) * epi.gate_ld + n0;
                    if (vec_ok && table_vec) {
                        const float4 t4 = *reinterpret_cast<const float4*>(t);
                        v[0] += t4.x; v[1] += t4.y; v[2] += t4.z; v[3] += t4.w;
                    } else {
#pragma unroll
                        for (int c = 0; c < 4; c++)
                            if (c < nvalid) v[c] += t[c];
                    }
                }
                if constexpr (EPI == EPI_QKV_NORM && WNC % 64 == 0) {
                    // 16 consecutive lanes hold 64 consecutive columns of this row = one head of one token (modules.cpp:192-198, fused)
                    const int third = n0 / epi.gate_ld;  // 0 = q, 1 = k, 2 = v (uniform over the 16 lanes: C is a multiple of 64)
                    if (third < 2) {
                        // explicit fused multiply-adds: left to the compiler, each unrolled copy of this code may pick a different
                        // product to fuse, and a row's result would depend on where in the tile it sits
                        float ss = fmaf(v[3], v[3], fmaf(v[2], v[2], fmaf(v[1], v[1], v[0] * v[0])));
                        // butterfly over the 16 lanes with data-parallel-primitive moves (no trip through the LDS crossbar): lanes ^1 and ^2
                        // by quad permutes; after those every quad holds one value, so mirroring the half row (i <-> 7-i) and then the
                        // row (i <-> 15-i) pairs the same partial sums as lanes ^4 and ^8 would
                        ss += dpp_move<0xB1>(ss);   // quad_perm [1,0,3,2]
                        ss += dpp_move<0x4E>(ss);   // quad_perm [2,3,0,1]
                        ss += dpp_move<0x141>(ss);  // row_half_mirror
                        ss += dpp_move<0x140>(ss);  // row_mirror
                        // (the hardware's reciprocal square root, 1 ulp: a divide and a square root here cost 0.2 ms per forward,
                        // and the result is rounded to bf16 anyway)
                        const float inv = __builtin_amdgcn_rsqf(1e-6f + ss * (1.0f / 64.0f));
                        const float4 w4 = *reinterpret_cast<const float4*>((third == 0 ? epi.gate : epi.resid) + (n0 & 63));
                        v[0] = (v[0] * inv) * w4.x; v[1] = (v[1] * inv) * w4.y; v[2] = (v[2] * inv) * w4.z; v[3] = (v[3] * inv) * w4.w;
                    }
                }
                res[p] = make_float4(v[0], v[1], v[2], v[3]);
            }
        }
        // ... and all stores of the slab leave back to back
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int m = m_blk + wm * (BM / WM) + i * SR + p * RPI + e_row;
            if (m < M && nvalid > 0) {
                const long long idx = (long long)m * ldc + n0;
                const float v[4] = {res[p].x, res[p].y, res[p].z, res[p].w};
                if (vec_ok) {
                    if (OUT_F32) *reinterpret_cast<float4*>(outf + idx) = make_float4(v[0], v[1], v[2], v[3]);
                    else *reinterpret_cast<uint2*>(outh + idx) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
                } else {
#pragma unroll
                    for (int c = 0; c < 4; c++)
                        if (c < nvalid) {
                            if (OUT_F32) outf[idx + c] = v[c];
                            else outh[idx + c] = f32_to_bf16(v[c]);
                        }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// Persistent kernel: one workgroup per compute unit walks over the tiles of up to three problems. The stores of a finished
// tile drain while the next tile's K loop is already running, instead of holding the compute unit until they retire.
// Workgroup g takes work items g, g + G, g + 2G ... (G = grid size, a multiple of 8), so it stays on its XCD's run of tiles.
template <int BM, int BN, int WM, int WN, int STAGES, int EPI, bool OUT_F32, bool FP8 = false>
__global__ void __launch_bounds__(WM* WN * 64) gemm_bf16_kernel(const ProbSet args) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    for (int w = blockIdx.x; w < args.end[MAX_PROBS - 1]; w += gridDim.x) {
        const int which = (w >= args.end[0]) + (w >= args.end[1]);
        gemm_tile<BM, BN, WM, WN, STAGES, EPI, OUT_F32, FP8>(args.p[which], w - (which ? args.end[which - 1] : 0), smem);
        __syncthreads();  // the staging slabs of this tile's epilogue alias the ring the next tile fills
    }
}

// compute units of the current device (0 after a failed query, which has set the error message)
int compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            fail(SD3_ERR_HIP, "gemm_bf16: cannot query the number of compute units");
            return 0;
        }
        cus = n;
    }
    return cus;
}

template <int BM, int BN, int WM, int WN, int STAGES, int EPI, bool OUT_F32, bool FP8 = false>
int launch_cfg(ProbSet& args, int n, hipStream_t st) {
    auto kern = gemm_bf16_kernel<BM, BN, WM, WN, STAGES, EPI, OUT_F32, FP8>;
    constexpr int smem = smem_bytes<BM, BN, WM, WN, STAGES>();
    static bool attr_done = false;  // raising the dynamic LDS limit is a per-function, per-process setting
    if (smem > 65536 && !attr_done) {
        SD3_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
        attr_done = true;
    }
    if (EPI == EPI_QKV_NORM && (BN / WN) % 64 != 0) return fail(SD3_ERR_UNSUPPORTED, "gemm_bf16: this tile shape cannot fuse the qk-norm");
    int total = 0;
    for (int i = 0; i < MAX_PROBS; i++) {
        if (i < n) total += ((args.p[i].N + BN - 1) / BN) * ((args.p[i].M + BM - 1) / BM);
        args.end[i] = total;
    }
    // as many workgroups as can be resident at once (LDS allows one 256x256 or two 128x128 workgroups per compute unit), rounded
    // down to a multiple of the 8 XCDs
    const int cus = compute_units();
    if (cus <= 0) return SD3_ERR_HIP;
    constexpr int per_cu = (160 * 1024) / smem > 1 ? 2 : 1;
    const int resident = (cus * per_cu / 8 * 8) > 8 ? (cus * per_cu / 8 * 8) : 8;
    dim3 grid(total < resident ? total : resident), block(WM * WN * 64);
    hipLaunchKernelGGL(kern, grid, block, smem, st, args);
    g_gemm_bf16_launches.fetch_add(1, std::memory_order_relaxed);
    return launch_status("gemm_bf16");
}

// fp8 operands: 256x256 tiles (variant 4) or 128x128 tiles with a ring of two stages (anything else)
template <int EPI, bool OUT_F32>
int launch_epi_fp8(int variant, ProbSet& args, int n, hipStream_t st) {
    if (variant == 4) return launch_cfg<256, 256, 2, 4, 2, EPI, OUT_F32, true>(args, n, st);
    return launch_cfg<128, 128, 2, 2, 2, EPI, OUT_F32, true>(args, n, st);
}

template <int EPI, bool OUT_F32>
int launch_epi(int variant, ProbSet& args, int n, hipStream_t st) {
    switch (variant) {
        case 4: return launch_cfg<256, 256, 2, 4, 2, EPI, OUT_F32>(args, n, st);
        case 5: return launch_cfg<256, 192, 2, 4, 2, EPI, OUT_F32>(args, n, st);
        case 1: return launch_cfg<128, 128, 2, 2, 4, EPI, OUT_F32>(args, n, st);
        default: return launch_cfg<128, 128, 2, 2, 2, EPI, OUT_F32>(args, n, st);
    }
}

}  // namespace

std::atomic<long long> g_gemm_bf16_launches{0};
int g_gemm_bf16_row_split = 1;  // 0: never split a problem's rows over two launches (sd3_tune)
int g_gemm_bf16_variant = -1;  // -1: choose by shape; 0 / 4: forced 128x128 / 256x256 tiles (sd3_gemm_bf16_force_tile); 1: 128x128 with a ring of four stages

static int grouped_impl(const GemmBf16Problem* probs, int n, int out_is_f32, int epi, bool fp8, hipStream_t st) {
    if (n < 1 || n > MAX_PROBS) return fail(SD3_ERR_INVALID_ARG, "gemm_bf16_grouped: 1 to %d problems (got %d)", MAX_PROBS, n);
    ProbSet args{};
    int m = 0, max_M = 0;
    for (int i = 0; i < n; i++) {
        const GemmBf16Problem& q = probs[i];
        if (q.M <= 0 || q.N <= 0) continue;  // an empty problem simply contributes no tiles
        const int kmult = fp8 ? 128 : BK;  // one LDS row of a K tile is 128 bytes
        if (q.K <= 0 || (q.K % kmult) != 0) return fail(SD3_ERR_UNSUPPORTED, "gemm_%s: K=%d must be a positive multiple of %d", fp8 ? "fp8" : "bf16", q.K, kmult);
        if ((reinterpret_cast<uintptr_t>(q.A) & 15) || (reinterpret_cast<uintptr_t>(q.Wp) & 15))
            return fail(SD3_ERR_INVALID_ARG, "gemm_bf16: operands must be 16-byte aligned");
        Prob& d = args.p[m++];
        d.A = q.A; d.Wp = q.Wp; d.out = q.out; d.ldc = q.ldc; d.M = q.M; d.N = q.N; d.K = q.K;
        d.epi = EpiDev{fp8 ? q.ea.a_scale : nullptr, fp8 ? q.ea.w_scale : nullptr, q.ea.bias, q.ea.gate, q.ea.resid, q.ea.table, q.ea.gate_ld,
                       q.ea.rows_per_batch > 0 ? q.ea.rows_per_batch : 1};
        if (epi == EPI_BIAS_ROWADD) d.epi.gate_ld = q.N;
        if (epi == EPI_QKV_NORM) {
            if (q.N % 192 || !q.ea.gate || !q.ea.resid || (reinterpret_cast<uintptr_t>(q.ea.gate) & 15) || (reinterpret_cast<uintptr_t>(q.ea.resid) & 15))
                return fail(SD3_ERR_INVALID_ARG, "gemm_bf16: the fused qk-norm needs N = 3C with C a multiple of 64 and two aligned weight vectors");
            d.epi.gate_ld = q.N / 3;
        }
        if (q.M > max_M) max_M = q.M;
    }
    if (m == 0) return SD3_OK;
    auto launch = [&](ProbSet& pp, int count, int v) -> int {
        if (fp8) {
#define SD3_GEMM_FP8_LAUNCH(E) return out_is_f32 ? launch_epi_fp8<E, true>(v, pp, count, st) : launch_epi_fp8<E, false>(v, pp, count, st)
            switch (epi) {
                case EPI_BIAS: SD3_GEMM_FP8_LAUNCH(EPI_BIAS);
                case EPI_BIAS_GELU: SD3_GEMM_FP8_LAUNCH(EPI_BIAS_GELU);
                case EPI_GATE_RESID: SD3_GEMM_FP8_LAUNCH(EPI_GATE_RESID);
                case EPI_QKV_NORM: SD3_GEMM_FP8_LAUNCH(EPI_QKV_NORM);
                default: return fail(SD3_ERR_UNSUPPORTED, "gemm_fp8: epilogue %d is not built for fp8 operands", epi);
            }
#undef SD3_GEMM_FP8_LAUNCH
        }
#define SD3_GEMM_BF16_LAUNCH(E) return out_is_f32 ? launch_epi<E, true>(v, pp, count, st) : launch_epi<E, false>(v, pp, count, st)
        switch (epi) {
            case EPI_BIAS: SD3_GEMM_BF16_LAUNCH(EPI_BIAS);
            case EPI_BIAS_GELU: SD3_GEMM_BF16_LAUNCH(EPI_BIAS_GELU);
            case EPI_BIAS_SILU: SD3_GEMM_BF16_LAUNCH(EPI_BIAS_SILU);
            case EPI_GATE_RESID: SD3_GEMM_BF16_LAUNCH(EPI_GATE_RESID);
            case EPI_BIAS_ROWADD: SD3_GEMM_BF16_LAUNCH(EPI_BIAS_ROWADD);
            case EPI_QKV_NORM: SD3_GEMM_BF16_LAUNCH(EPI_QKV_NORM);
            default: return fail(SD3_ERR_INVALID_ARG, "gemm_bf16: unknown epilogue %d", epi);
        }
#undef SD3_GEMM_BF16_LAUNCH
    };
    if (g_gemm_bf16_variant >= 0) return launch(args, m, fp8 && g_gemm_bf16_variant != 4 ? 0 : g_gemm_bf16_variant);
    // Tile shape and grouping by a small cost model. A persistent launch takes ceil(tiles / resident workgroups) rounds; the unit
    // of cost is one round of 256x256 tiles (8 wavefronts, one workgroup per compute unit). Measured on full rounds, a round of
    // 128x128 tiles (4 wavefronts, two workgroups per unit) takes 0.62 of that for a quarter of the outputs per tile, and a launch
    // of its own for problems with few rows (a short round of small tiles, bound by per-tile overhead) about 0.38.
    const int cus = compute_units();
    if (cus <= 0) return SD3_ERR_HIP;
    constexpr double ROUND128 = 0.62, SMALL_LAUNCH = 0.38;
    auto tiles = [](const Prob& q, int t) { return ((q.M + t - 1) / t) * ((q.N + t - 1) / t); };
    auto rounds = [](long long t, int slots) { return (double)((t + slots - 1) / slots); };
    ProbSet big{}, small{};
    int nb = 0, ns = 0;
    long long big256 = 0, big128 = 0, small256 = 0, small128 = 0;
    for (int i = 0; i < m; i++) {
        if (args.p[i].M < 1024) {
            small.p[ns++] = args.p[i];
            small256 += tiles(args.p[i], 256);
            small128 += tiles(args.p[i], 128);
        } else {
            big.p[nb++] = args.p[i];
            big256 += tiles(args.p[i], 256);
            big128 += tiles(args.p[i], 128);
        }
    }
    // only problems with few rows: small tiles; with no more tiles than compute units one workgroup per unit, so that LDS can hold
    // a ring of four stages
    const int v_small = small128 <= cus ? 1 : 0;
    if (nb == 0) return launch(args, m, v_small);
    const double together256 = rounds(big256 + small256, cus), together128 = ROUND128 * rounds(big128 + small128, 2 * cus);
    double best = together256 <= together128 ? together256 : together128;
    int plan = together256 <= together128 ? 0 : 1;  // 0/1: one launch with 256/128 tiles; 2/3: the small problems first, alone
    if (ns > 0) {
        const double apart256 = rounds(big256, cus) + SMALL_LAUNCH, apart128 = ROUND128 * rounds(big128, 2 * cus) + SMALL_LAUNCH;
        if (apart256 < best) { best = apart256; plan = 2; }
        if (apart128 < best) { best = apart128; plan = 3; }
    }
    // One more plan when the 256x256 tiles of the many-row problems fill R >= 1 rounds and leave a partial one: everything up to the
    // last row tile of the last many-row problem that still fits R rounds as 256x256 tiles, the remaining rows of that problem
    // together with the few-row problems as 128x128 tiles in a second launch (a round of those costs 0.62). Only for epilogues that do
    // not look at the row index (a row split would shift the batch boundaries).
    if (g_gemm_bf16_row_split && nb >= 1 && nb + ns <= MAX_PROBS && !fp8 &&
        (epi == EPI_BIAS || epi == EPI_BIAS_GELU || epi == EPI_BIAS_SILU || epi == EPI_QKV_NORM)) {
        const Prob& q = big.p[nb - 1];
        long long before = 0;  // tiles of the many-row problems in front of the one that is split
        for (int i = 0; i + 1 < nb; i++) before += tiles(big.p[i], 256);
        const int tn = (q.N + 255) / 256, tm = (q.M + 255) / 256;
        const long long R = big256 / cus, avail = R * cus - before;
        const int m1 = (R > 0 && avail > 0) ? (int)(avail / tn) : 0;  // row tiles of q that fit the R full rounds
        if (m1 > 0 && m1 < tm) {
            Prob head = q, tail = q;
            head.M = m1 * 256;
            tail.M = q.M - head.M;
            tail.A = q.A + (long long)head.M * q.K;
            tail.out = (char*)q.out + (long long)head.M * q.ldc * (out_is_f32 ? 4 : 2);
            const double split = rounds(before + tiles(head, 256), cus) + ROUND128 * rounds(tiles(tail, 128) + small128, 2 * cus);
            if (split < best) {
                ProbSet first{}, second{};
                for (int i = 0; i + 1 < nb; i++) first.p[i] = big.p[i];
                first.p[nb - 1] = head;
                second.p[0] = tail;
                for (int i = 0; i < ns; i++) second.p[1 + i] = small.p[i];
                SD3_TRY(launch(first, nb, 4));
                return launch(second, 1 + ns, 0);
            }
        }
    }
    if (plan >= 2) {
        SD3_TRY(launch(small, ns, v_small));
        return launch(big, nb, plan == 2 ? 4 : 0);
    }
    return launch(args, m, plan == 0 ? 4 : 0);
}

int gemm_bf16_grouped(const GemmBf16Problem* probs, int n, int out_is_f32, int epi, hipStream_t st) { return grouped_impl(probs, n, out_is_f32, epi, false, st); }
int gemm_fp8_grouped(const GemmBf16Problem* probs, int n, int out_is_f32, int epi, hipStream_t st) { return grouped_impl(probs, n, out_is_f32, epi, true, st); }

int gemm_bf16(const bf16_t* A, const bf16_t* Wp, void* out, int out_is_f32, int ldc, int M, int N, int K, int epi, const GemmEpilogueArgs& ea,
              hipStream_t st) {
    GemmBf16Problem q{A, Wp, out, ldc, M, N, K, ea};
    return gemm_bf16_grouped(&q, 1, out_is_f32, epi, st);
}

}  // namespace sd3

extern "C" int sd3_gemm_bf16_force_tile(int tile) {
    if (tile != 0 && tile != 128 && tile != 192 && tile != 256)
        return sd3::fail(SD3_ERR_INVALID_ARG, "sd3_gemm_bf16_force_tile: tile must be 0, 128, 192 or 256 (got %d)", tile);
    sd3::g_gemm_bf16_variant = tile == 0 ? -1 : (tile == 256 ? 4 : tile == 192 ? 5 : 0);
    return SD3_OK;
}
