// Host side of the library: context (bound weights, bf16 copies, workspace), the block schedule
// (dit_block, modules.cpp:1340-1505) and the full forward (DiT_forward, modules.cpp:1605-1780) expressed as
// launches of the fused kernels. No arithmetic happens on the host.
#include <cmath>
#include <cstring>
#include <map>
#include <new>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "common.hpp"

namespace sd3 {

// ------------------------------------------------------------------ errors
static thread_local char g_err[512] = "";
void set_error(const char* msg) {
    std::strncpy(g_err, msg, sizeof(g_err) - 1);
    g_err[sizeof(g_err) - 1] = 0;
}
int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}
const char* last_error() { return g_err; }

}  // namespace sd3

using namespace sd3;

namespace sd3 {
extern int g_attention_context_splits;  // attention_bf16.hip
extern int g_gemm_bf16_row_split;       // gemm_bf16.hip
}

// ------------------------------------------------------------------ fixed scratch of the entry point that allocates nothing
// Lives in device memory from the moment the code object is loaded on a device until the process ends; every device has
// its own copy at its own address. Host code never uses the array's name as an address: the address on a device is asked
// for once (static_scratch_of, with that device current) and kept.
static __device__ __align__(256) unsigned char scratch[SD3_STATIC_SCRATCH_BYTES];
static constexpr int MAX_DEVICES = 64;
static void* g_scratch_ptr[MAX_DEVICES] = {};

// the calling thread's current device must be `device`
static int static_scratch_of(int device, void** out) {
    if (device < 0 || device >= MAX_DEVICES) return fail(SD3_ERR_UNSUPPORTED, "device %d: at most %d devices", device, MAX_DEVICES);
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        SD3_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(SD3_ERR_HIP, "hipGetSymbolAddress returned a null address for the fixed scratch array on device %d", device);
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return SD3_OK;
}

// ------------------------------------------------------------------ context
struct PackedWeight {
    void* ptr = nullptr;
    long long K = 0, N = 0;
    int kind = 0;  // 0: bf16 (N,K) transposed for the MFMA GEMM; 1: bf16 (K,N) plain cast for small_linear; 2: fp32 (K,N) transpose of an (N,K) tensor;
                   // 3 / 4: fp8 e4m3 (N,K) followed (at the next 256-byte boundary) by N fp32 factors, one per output column (3) or all equal (4)
};
static inline size_t fp8_scale_offset(long long K, long long N) { return ((size_t)K * N + 255) & ~(size_t)255; }
static inline bool is_bf(int prec) { return prec != SD3_PREC_F32; }
static inline int fp8_kind(int prec) { return prec == SD3_PREC_BF16_FP8 ? 3 : prec == SD3_PREC_BF16_FP8_TENSOR ? 4 : 0; }

struct sd3_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    // Recorded behind the last kernel of every enqueueing call (outside stream capture). Everything that must wait for the
    // context's earlier work between calls -- a change of stream, freeing derived copies, destroying the context -- waits on this
    // event, which the library owns, and never touches the handle of a stream the caller may have destroyed since.
    hipEvent_t order_event = nullptr;
    bool order_pending = false;
    std::unordered_map<std::string, std::pair<const float*, long long>> params;
    std::map<std::pair<const float*, int>, PackedWeight> packed;
    std::map<std::tuple<int, int, int, int, int>, float*> pos_tables;  // (C, max, base, h, w) -> cropped table
    void* ws = nullptr;
    size_t ws_bytes = 0;
    void* static_scratch = nullptr;  // this device's address of the fixed scratch array (resolved when the context is created)
    long long copies_built = 0;  // derived weight copies built so far (sd3_weights_copies_built)
    bool no_alloc = false;  // set for the duration of a call that must not allocate: a missing derived weight copy is then an error
    // optional per-kernel-class timing with HIP events on the context's stream
    bool prof_on = false;
    struct ProfSample {
        hipEvent_t a, b;
        int cls;
        double work;
        long long launches;
    };
    std::vector<ProfSample> prof;
    std::vector<hipEvent_t> event_pool;
};

namespace {

struct DeviceGuard {
    int prev = -1;
    bool ok = false;
    explicit DeviceGuard(int dev) {
        if (hipGetDevice(&prev) == hipSuccess && (prev == dev || hipSetDevice(dev) == hipSuccess)) ok = true;
        else (void)hipGetLastError();
    }
    ~DeviceGuard() {
        int cur = -1;
        if (ok && hipGetDevice(&cur) == hipSuccess && cur != prev) (void)hipSetDevice(prev);
    }
};

struct Bump {
    char* base;
    size_t off = 0, cap;
    Bump(void* b, size_t c) : base((char*)b), cap(c) {}
    template <typename T>
    T* take(size_t n) {
        size_t bytes = (n * sizeof(T) + 255) & ~(size_t)255;
        T* p = base ? reinterpret_cast<T*>(base + off) : nullptr;
        off += bytes;
        return p;
    }
};

// Marks the end of an enqueueing call on the context's stream (see sd3_ctx::order_event). Nothing is recorded while the stream
// is being captured into a graph: the event would become part of the capture, and replays are ordered by the caller.
void record_order(sd3_ctx* ctx) {
    if (!ctx->order_event) return;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->stream, &cap) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    if (cap != hipStreamCaptureStatusNone) return;
    if (hipEventRecord(ctx->order_event, ctx->stream) == hipSuccess) ctx->order_pending = true;
    else (void)hipGetLastError();
}
// Waits on the host until the work of every earlier call has finished (the device of the context must be current).
int wait_idle(sd3_ctx* ctx) {
    if (ctx->order_pending) SD3_HIP_TRY(hipEventSynchronize(ctx->order_event));
    return SD3_OK;
}
struct OrderScope {  // records the order event when an enqueueing entry point returns, on every path
    sd3_ctx* ctx;
    explicit OrderScope(sd3_ctx* c) : ctx(c) {}
    ~OrderScope() { record_order(ctx); }
};

int ensure_workspace(sd3_ctx* ctx, size_t bytes) {
    if (bytes <= ctx->ws_bytes) return SD3_OK;
    if (ctx->ws) {
        SD3_HIP_TRY(hipStreamSynchronize(ctx->stream));
        SD3_HIP_TRY(hipFree(ctx->ws));
        ctx->ws = nullptr;
        ctx->ws_bytes = 0;
    }
    hipError_t e = hipMalloc(&ctx->ws, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(SD3_ERR_OOM, "workspace of %zu bytes: %s", bytes, hipGetErrorString(e));
    }
    ctx->ws_bytes = bytes;
    return SD3_OK;
}

int get_packed(sd3_ctx* ctx, const float* w, long long K, long long N, int kind, const void** out) {
    auto key = std::make_pair(w, kind);
    auto it = ctx->packed.find(key);
    if (it != ctx->packed.end() && it->second.K == K && it->second.N == N) {
        *out = it->second.ptr;
        return SD3_OK;
    }
    if (ctx->no_alloc)
        return fail(SD3_ERR_MISSING_PARAM,
                    "the bf16 copy of a %lld x %lld weight has not been built yet and this entry point allocates nothing: call sd3_weights_prepare "
                    "(or sd3_dit_block once) first, or use SD3_PREC_F32, which reads the bound weights in place", K, N);
    if (it != ctx->packed.end()) {
        SD3_HIP_TRY(hipStreamSynchronize(ctx->stream));
        SD3_HIP_TRY(hipFree(it->second.ptr));
        ctx->packed.erase(it);
    }
    PackedWeight p;
    p.K = K; p.N = N; p.kind = kind;
    const size_t bytes = kind >= 3 ? fp8_scale_offset(K, N) + (size_t)N * sizeof(float) : (size_t)K * N * (kind == 2 ? 4 : 2);
    hipError_t e = hipMalloc(&p.ptr, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(SD3_ERR_OOM, "bf16 weight copy of %zu bytes: %s", bytes, hipGetErrorString(e));
    }
    int rc;
    if (kind == 0) rc = pack_weight_bf16(w, (bf16_t*)p.ptr, (int)K, (int)N, ctx->stream);
    else if (kind == 1) rc = cast_f32_to_bf16(w, (bf16_t*)p.ptr, K * N, ctx->stream);
    else if (kind >= 3) rc = quantize_weight_fp8(w, (uint8_t*)p.ptr, (float*)((char*)p.ptr + fp8_scale_offset(K, N)), (int)K, (int)N, kind == 4, ctx->stream);
    else rc = transpose_f32(w, (float*)p.ptr, (int)N, (int)K, ctx->stream);  // input is (N,K): transpose to (K,N)
    if (rc != SD3_OK) {
        (void)hipFree(p.ptr);
        return rc;
    }
    ctx->packed[key] = p;
    ctx->copies_built++;
    *out = p.ptr;
    return SD3_OK;
}

// Frees every derived copy made from the tensor at `w` (after the work that may still read them has finished).
int drop_packed_of(sd3_ctx* ctx, const float* w) {
    bool synced = false;
    for (int kind = 0; kind < 5; kind++) {
        auto it = ctx->packed.find(std::make_pair(w, kind));
        if (it == ctx->packed.end()) continue;
        if (!synced) {
            DeviceGuard g(ctx->device);
            SD3_TRY(wait_idle(ctx));
            synced = true;
        }
        DeviceGuard g(ctx->device);
        (void)hipFree(it->second.ptr);
        ctx->packed.erase(it);
    }
    return SD3_OK;
}

// Brackets one kernel launch with two events when profiling is on. `work` is the launch's algorithmic work
// (FLOP for the MFMA classes, bytes for the memory-bound ones).
struct ProfScope {
    sd3_ctx* ctx;
    hipEvent_t a = nullptr, b = nullptr;
    int cls;
    double work;
    long long gemm_launches_before;  // one bracketed call may launch more than one GEMM kernel; the class counts kernels
    long long explicit_launches;     // kernels launched inside the bracket when the caller knows the number (0: count GEMM kernels, at least 1)
    ProfScope(sd3_ctx* c, int cls_, double work_, long long launches_ = 0)
        : ctx(c), cls(cls_), work(work_), gemm_launches_before(g_gemm_bf16_launches.load(std::memory_order_relaxed)), explicit_launches(launches_) {
        if (!ctx->prof_on || ctx->no_alloc) return;  // (creating an event allocates)
        auto get = [&]() -> hipEvent_t {
            hipEvent_t e = nullptr;
            if (!ctx->event_pool.empty()) {
                e = ctx->event_pool.back();
                ctx->event_pool.pop_back();
            } else if (hipEventCreate(&e) != hipSuccess) {
                (void)hipGetLastError();
                e = nullptr;
            }
            return e;
        };
        a = get();
        b = get();
        if (a) (void)hipEventRecord(a, ctx->stream);
    }
    ~ProfScope() {
        if (!a || !b) return;
        (void)hipEventRecord(b, ctx->stream);
        const long long kernels = g_gemm_bf16_launches.load(std::memory_order_relaxed) - gemm_launches_before;
        ctx->prof.push_back({a, b, cls, work, explicit_launches > 0 ? explicit_launches : (kernels > 1 ? kernels : 1)});
    }
};

struct Dims {
    int B, Tc, Tx, C, NH, HS, E;  // E = mlp_expand
    bool dual, qk, discard;
};

size_t block_workspace_bytes(const Dims& d, int prec) {
    Bump b(nullptr, 0);
    const size_t es = is_bf(prec) ? 2 : 4;
    const size_t mc = (size_t)d.B * d.Tc, mx = (size_t)d.B * d.Tx;
    auto act = [&](size_t n) { b.take<char>(n * es); };
    if (fp8_kind(prec)) {  // fp8 copies of the MLP inputs and one factor per row
        b.take<char>(mc * d.E * d.C); b.take<char>(mx * d.E * d.C);
        b.take<float>(mc); b.take<float>(mx);
    }
    act(mc * d.C); act(mx * d.C); act(mx * d.C);           // c_hid, x_hid, x_hid2
    act(mc * 3 * d.C); act(mx * 3 * d.C);                  // c_qkv, x_qkv
    if (d.dual) act(mx * 3 * d.C);                         // x_qkv2
    act(mc * d.C); act(mx * d.C);                          // c_att, x_att
    if (is_bf(prec)) {
        if (d.dual) act(mx * d.C);                         // x_att2: both attentions of a dual block run in one launch
        const int S = attention_bf16_context_splits(d.Tc, d.Tx);
        if (S) b.take<float>(attention_bf16_split_workspace_floats(d.B, d.NH, d.Tc, S));
    }
    act(mc * d.E * d.C); act(mx * d.E * d.C);              // c_mlp, x_mlp
    b.take<float>((size_t)d.B * 6 * d.C); b.take<float>((size_t)d.B * 9 * d.C);  // ada_c, ada_x
    return b.off;
}

// One linear layer: out = epilogue(A @ W + b). fp32: W used in place; bf16: the packed copy.
int linear_layer(sd3_ctx* ctx, int prec, const void* A, const float* W, const float* bias, void* out, int out_f32, int ldc, int M, int N, int K, int epi,
                 GemmEpilogueArgs ea) {
    if (!W) return fail(SD3_ERR_MISSING_PARAM, "a weight needed by this configuration is not bound (N=%d K=%d)", N, K);
    ea.bias = bias;
    if (!is_bf(prec)) {
        ProfScope ps(ctx, SD3_PROF_GEMM, 2.0 * M * N * K);
        return gemm_f32((const float*)A, K, W, N, 0, (float*)out, ldc, M, N, K, epi, ea, ctx->stream);
    }
    const void* wp = nullptr;
    SD3_TRY(get_packed(ctx, W, K, N, 0, &wp));
    ProfScope ps(ctx, SD3_PROF_GEMM, 2.0 * M * N * K);
    return gemm_bf16((const bf16_t*)A, (const bf16_t*)wp, out, out_f32, ldc, M, N, K, epi, ea, ctx->stream);
}

// The same layer of the latent stream and of the context stream (different weights and rows, same kind): on the bf16
// path both go into one launch, so that the few context rows ride along instead of paying a launch of their own.
struct LayerCall {
    const void* A;
    const float* W;
    const float* bias;
    void* out;
    int ldc, M, N, K;
    GemmEpilogueArgs ea;
};
int linear_pair(sd3_ctx* ctx, int prec, const LayerCall* calls, int n, int out_f32, int epi) {
    if (!is_bf(prec)) {
        for (int i = 0; i < n; i++) {
            const LayerCall& c = calls[i];
            if (c.M > 0) SD3_TRY(linear_layer(ctx, prec, c.A, c.W, c.bias, c.out, out_f32, c.ldc, c.M, c.N, c.K, epi, c.ea));
        }
        return SD3_OK;
    }
    GemmBf16Problem probs[3];
    if (n > 3) return fail(SD3_ERR_INVALID_ARG, "linear_pair: at most three layers per group");
    int m = 0;
    double flop = 0;
    for (int i = 0; i < n; i++) {
        const LayerCall& c = calls[i];
        if (c.M <= 0) continue;
        if (!c.W) return fail(SD3_ERR_MISSING_PARAM, "a weight needed by this configuration is not bound (N=%d K=%d)", c.N, c.K);
        const void* wp = nullptr;
        SD3_TRY(get_packed(ctx, c.W, c.K, c.N, 0, &wp));
        probs[m] = GemmBf16Problem{(const bf16_t*)c.A, (const bf16_t*)wp, c.out, c.ldc, c.M, c.N, c.K, c.ea};
        probs[m].ea.bias = c.bias;
        flop += 2.0 * c.M * c.N * c.K;
        m++;
    }
    if (m == 0) return SD3_OK;
    ProfScope ps(ctx, SD3_PROF_GEMM, flop);
    return gemm_bf16_grouped(probs, m, out_f32, epi, ctx->stream);
}

int ada_jobs_run(sd3_ctx* ctx, int prec, const float* y, int B, int C, std::vector<SmallLinearJob>& jobs) {
    if (is_bf(prec)) {
        for (auto& j : jobs) {
            const void* wp = nullptr;
            SD3_TRY(get_packed(ctx, (const float*)j.W, C, j.ldw, 1, &wp));
            j.W = wp;
        }
    }
    double bytes = 0;
    for (auto& j : jobs) bytes += (double)C * j.N * (is_bf(prec) ? 2 : 4) + (double)B * j.N * 4;
    ProfScope ps(ctx, SD3_PROF_ADALN, bytes, ((long long)jobs.size() + SMALL_LINEAR_JOBS_PER_LAUNCH - 1) / SMALL_LINEAR_JOBS_PER_LAUNCH);
    return small_linear_batched(y, B, C, jobs.data(), (int)jobs.size(), is_bf(prec), -1, ctx->stream);
}

// LayerNorm + modulation, timed as a memory-bound launch: reads x once (fp32), writes one or two outputs.
int ln_mod(sd3_ctx* ctx, const float* x, void* out, void* out2, const float* shift, const float* scale, const float* shift2, const float* scale2,
           int mod_ld, float eps, int B, int T, int C, int bf) {
    const double n = (double)B * T * C;
    ProfScope ps(ctx, SD3_PROF_LAYERNORM, n * 4 + n * (bf ? 2 : 4) * (out2 ? 2 : 1));
    return layernorm_modulate(x, out, out2, shift, scale, shift2, scale2, mod_ld, eps, B, T, C, bf, ctx->stream);
}

// The LayerNorms of the latent and of the context stream at the same point of the block: one launch
int ln_mod_pair(sd3_ctx* ctx, const LayerNormJob* jobs, int n, float eps, int C, int bf) {
    double bytes = 0;
    for (int i = 0; i < n; i++) {
        const double e = (double)jobs[i].B * jobs[i].T * C;
        bytes += e * 4 + e * (bf ? 2 : 4) * (jobs[i].out2 ? 2 : 1);
    }
    if (bytes == 0) return SD3_OK;
    ProfScope ps(ctx, SD3_PROF_LAYERNORM, bytes);
    return layernorm_modulate_pair(jobs, n, eps, C, bf, ctx->stream);
}

int attention(sd3_ctx* ctx, const AttnSegments& a, int B, int NH, int HS, bool bf) {
    const double Tq = a.Tq[0] + a.Tq[1], Tk = a.T[0] + a.T[1];
    ProfScope ps(ctx, SD3_PROF_ATTENTION, 4.0 * B * NH * Tq * Tk * HS);
    return bf ? attention_bf16(a, B, NH, HS, ctx->stream) : attention_f32(a, B, NH, HS, ctx->stream);
}

// The block. ada_c / ada_x: modulation vectors (B, chunks*C) already computed, or null to compute them here.
int run_block(sd3_ctx* ctx, int prec, const float* y, float* c, float* x, const sd3_block_weights& w, const Dims& d, const float* ada_c,
              const float* ada_x, Bump& ws) {
    hipStream_t st = ctx->stream;
    const int B = d.B, Tc = d.Tc, Tx = d.Tx, C = d.C;
    const int mc = B * Tc, mx = B * Tx;
    const int cch = d.discard ? 2 : 6, xch = d.dual ? 9 : 6;
    const bool bf = is_bf(prec);
    const int f8 = fp8_kind(prec);
    const size_t es = bf ? 2 : 4;
    auto act = [&](size_t n) -> void* { return ws.take<char>(n * es); };
    uint8_t *cq = nullptr, *xq = nullptr;
    float *cs = nullptr, *xs = nullptr;
    if (f8) {
        cq = ws.take<uint8_t>((size_t)mc * d.E * C); xq = ws.take<uint8_t>((size_t)mx * d.E * C);
        cs = ws.take<float>((size_t)mc); xs = ws.take<float>((size_t)mx);
    }
    void* c_hid = act((size_t)mc * C);
    void* x_hid = act((size_t)mx * C);
    void* x_hid2 = act((size_t)mx * C);
    void* c_qkv = act((size_t)mc * 3 * C);
    void* x_qkv = act((size_t)mx * 3 * C);
    void* x_qkv2 = d.dual ? act((size_t)mx * 3 * C) : nullptr;  // q,k,v of the extra self-attention branch
    void* c_att = act((size_t)mc * C);
    void* x_att = act((size_t)mx * C);
    void* x_att2 = x_att;  // output of the extra self-attention (bf16 path: a buffer of its own, the two attentions share a launch)
    float* split_ws = nullptr;
    const int ctx_splits = is_bf(prec) ? attention_bf16_context_splits(Tc, Tx) : 0;
    if (is_bf(prec)) {
        if (d.dual) x_att2 = act((size_t)mx * C);
        if (ctx_splits) split_ws = ws.take<float>(attention_bf16_split_workspace_floats(B, d.NH, Tc, ctx_splits));
    }
    void* c_mlp = act((size_t)mc * d.E * C);
    void* x_mlp = act((size_t)mx * d.E * C);
    float* ada_c_buf = ws.take<float>((size_t)B * 6 * C);
    float* ada_x_buf = ws.take<float>((size_t)B * 9 * C);

    if (!w.c_ada_w || !w.c_ada_b || !w.x_ada_w || !w.x_ada_b) return fail(SD3_ERR_MISSING_PARAM, "adaLN modulation weights are not bound");
    if (!w.c_qkv_w || !w.c_qkv_b || !w.x_qkv_w || !w.x_qkv_b || !w.x_out_w || !w.x_out_b || !w.x_mlp_w1 || !w.x_mlp_b1 || !w.x_mlp_w2 || !w.x_mlp_b2)
        return fail(SD3_ERR_MISSING_PARAM, "attention / MLP weights of the latent or context stream are not bound");
    if (!d.discard && (!w.c_out_w || !w.c_out_b || !w.c_mlp_w1 || !w.c_mlp_b1 || !w.c_mlp_w2 || !w.c_mlp_b2))
        return fail(SD3_ERR_MISSING_PARAM, "context out-projection / MLP weights are not bound (needed unless discard_context)");
    if (d.dual && (!w.x2_qkv_w || !w.x2_qkv_b || !w.x2_out_w || !w.x2_out_b))
        return fail(SD3_ERR_MISSING_PARAM, "latent_dual_* weights are not bound (needed with use_dual_attention)");
    if (d.qk && (!w.c_rms_q || !w.c_rms_k || !w.x_rms_q || !w.x_rms_k || (d.dual && (!w.x2_rms_q || !w.x2_rms_k))))
        return fail(SD3_ERR_MISSING_PARAM, "rmsnorm weights are not bound (needed with use_qk_norm)");

    // modulation vectors: every chunk of both streams in one launch (the reference issues 12-20 partial_linear calls)
    if (!ada_c || !ada_x) {
        std::vector<SmallLinearJob> jobs = {
            {w.c_ada_w, w.c_ada_b, ada_c_buf, cch * C, cch * C, 0},
            {w.x_ada_w, w.x_ada_b, ada_x_buf, xch * C, xch * C, 0},
        };
        SD3_TRY(ada_jobs_run(ctx, prec, y, B, C, jobs));
        ada_c = ada_c_buf;
        ada_x = ada_x_buf;
    }
    const int ldc_ada = cch * C, ldx_ada = xch * C;
    auto cchunk = [&](int k) { return ada_c + (size_t)k * C; };
    auto xchunk = [&](int k) { return ada_x + (size_t)k * C; };
    GemmEpilogueArgs none;

    // ---- both streams up to q,k,v (modules.cpp:1381-1423); with discard_context chunk 0 is the scale, chunk 1 the shift;
    //      the dual branch's input comes from the same normalised latent rows
    const float* c_shift = d.discard ? cchunk(1) : cchunk(0);
    const float* c_scale = d.discard ? cchunk(0) : cchunk(1);
    {
        const LayerNormJob ln1[2] = {{x, x_hid, d.dual ? x_hid2 : nullptr, xchunk(0), xchunk(1), d.dual ? xchunk(6) : nullptr, d.dual ? xchunk(7) : nullptr,
                                      ldx_ada, B, Tx},
                                     {c, c_hid, nullptr, c_shift, c_scale, nullptr, nullptr, ldc_ada, B, Tc}};
        SD3_TRY(ln_mod_pair(ctx, ln1, 2, 1e-6f, C, bf));
    }
    {
        // bf16 path: the per-head RMSNorm of q and k (modules.cpp:1396-1399, 1420-1423) runs in the projection's epilogue, on the
        // fp32 accumulators, so the attention kernel streams K tiles straight into LDS
        GemmEpilogueArgs nx, nc;
        nx.gate = w.x_rms_q; nx.resid = w.x_rms_k;
        nc.gate = w.c_rms_q; nc.resid = w.c_rms_k;
        const bool fused_norm = bf && d.qk;
        GemmEpilogueArgs n2;
        n2.gate = w.x2_rms_q; n2.resid = w.x2_rms_k;
        // the dual branch's projection reads the other output of the same LayerNorm pass: same kind, same launch
        LayerCall qkv[3] = {{x_hid, w.x_qkv_w, w.x_qkv_b, x_qkv, 3 * C, mx, 3 * C, C, fused_norm ? nx : none},
                            {x_hid2, w.x2_qkv_w, w.x2_qkv_b, x_qkv2, 3 * C, d.dual ? mx : 0, 3 * C, C, fused_norm ? n2 : none},
                            {c_hid, w.c_qkv_w, w.c_qkv_b, c_qkv, 3 * C, mc, 3 * C, C, fused_norm ? nc : none}};
        SD3_TRY(linear_pair(ctx, prec, qkv, 3, !bf, fused_norm ? EPI_QKV_NORM : EPI_BIAS));
    }

    // ---- joint attention over [context ; latent] (modules.cpp:1427-1432); fp32 path: qk-norm in place first
    auto seg_ptr = [&](void* base, int third) -> void* { return (char*)base + (size_t)third * C * es; };
    if (!bf && d.qk) {
        SD3_TRY(rmsnorm_rows((float*)c_qkv, (float*)c_qkv, w.c_rms_q, nullptr, 1e-6f, mc, d.NH, d.HS, 3 * C, 3 * C, st));
        SD3_TRY(rmsnorm_rows((float*)seg_ptr(c_qkv, 1), (float*)seg_ptr(c_qkv, 1), w.c_rms_k, nullptr, 1e-6f, mc, d.NH, d.HS, 3 * C, 3 * C, st));
        SD3_TRY(rmsnorm_rows((float*)x_qkv, (float*)x_qkv, w.x_rms_q, nullptr, 1e-6f, mx, d.NH, d.HS, 3 * C, 3 * C, st));
        SD3_TRY(rmsnorm_rows((float*)seg_ptr(x_qkv, 1), (float*)seg_ptr(x_qkv, 1), w.x_rms_k, nullptr, 1e-6f, mx, d.NH, d.HS, 3 * C, 3 * C, st));
    }
    AttnSegments joint{}, dual_set{};
    joint.q[0] = c_qkv; joint.k[0] = seg_ptr(c_qkv, 1); joint.v[0] = seg_ptr(c_qkv, 2); joint.out[0] = d.discard ? nullptr : c_att;
    joint.q[1] = x_qkv; joint.k[1] = seg_ptr(x_qkv, 1); joint.v[1] = seg_ptr(x_qkv, 2); joint.out[1] = x_att;
    joint.ld_qkv[0] = joint.ld_qkv[1] = 3 * C; joint.ld_out[0] = joint.ld_out[1] = C;
    joint.T[0] = joint.Tq[0] = Tc; joint.T[1] = joint.Tq[1] = Tx;
    if (d.dual) {  // extra self-attention over the latent tokens (modules.cpp:1440-1453): independent of the joint one
        dual_set.q[0] = x_qkv2; dual_set.k[0] = seg_ptr(x_qkv2, 1); dual_set.v[0] = seg_ptr(x_qkv2, 2); dual_set.out[0] = x_att2;
        dual_set.ld_qkv[0] = dual_set.ld_qkv[1] = 3 * C; dual_set.ld_out[0] = dual_set.ld_out[1] = C;
        dual_set.T[0] = dual_set.Tq[0] = Tx;
    }
    if (bf) {
        // One launch for everything attention has to do in this block. With few context tokens beside many latent ones the joint
        // attention is taken apart by queries: the latent queries as one set, the context queries as short work items split along
        // the keys (see attention_bf16_context_splits), the extra self-attention as a third set.
        AttnSegments sets[3];
        int splits[3] = {1, 1, 1};
        float* wsp[3] = {nullptr, nullptr, nullptr};
        int n = 0;
        double flop = 0;
        const double Tj = (double)Tc + Tx;
        if (ctx_splits) {
            sets[n] = joint;
            sets[n].Tq[0] = 0; sets[n].out[0] = nullptr;
            n++;
        } else {
            sets[n++] = joint;
        }
        flop += 4.0 * B * d.NH * (d.discard ? (double)Tx : Tj) * Tj * d.HS;  // (a discard_context block computes no context queries)
        if (d.dual) {
            sets[n++] = dual_set;
            flop += 4.0 * B * d.NH * (double)Tx * Tx * d.HS;
        }
        if (ctx_splits && !d.discard) {
            sets[n] = joint;
            sets[n].Tq[1] = 0; sets[n].out[1] = nullptr;
            splits[n] = ctx_splits;
            wsp[n] = split_ws;
            n++;
        }
        ProfScope ps(ctx, SD3_PROF_ATTENTION, flop, 1 + ((ctx_splits && !d.discard) ? 1 : 0));  // (+ the kernel that merges the key splits)
        SD3_TRY(attention_bf16_multi(sets, splits, wsp, n, B, d.NH, d.HS, st));  // q and k arrive normalised
    } else {
        SD3_TRY(attention(ctx, joint, B, d.NH, d.HS, bf));
    }
    // ---- out-projections with the gate and the residual add in the epilogue (modules.cpp:1435-1436, 1459-1462, 1481-1485)
    GemmEpilogueArgs gx, gc;
    gc.rows_per_batch = Tc; gc.gate = cchunk(2); gc.gate_ld = ldc_ada; gc.resid = c;
    gx.rows_per_batch = Tx; gx.gate = xchunk(2); gx.gate_ld = ldx_ada; gx.resid = x;
    {
        LayerCall proj[2] = {{x_att, w.x_out_w, w.x_out_b, x, C, mx, C, C, gx}, {c_att, w.c_out_w, w.c_out_b, c, C, d.discard ? 0 : mc, C, C, gc}};
        SD3_TRY(linear_pair(ctx, prec, proj, 2, 1, EPI_GATE_RESID));
    }

    // ---- extra self-attention over the latent tokens (modules.cpp:1440-1453, 1486)
    if (d.dual) {
        if (!bf && d.qk) {
            SD3_TRY(rmsnorm_rows((float*)x_qkv2, (float*)x_qkv2, w.x2_rms_q, nullptr, 1e-6f, mx, d.NH, d.HS, 3 * C, 3 * C, st));
            SD3_TRY(rmsnorm_rows((float*)seg_ptr(x_qkv2, 1), (float*)seg_ptr(x_qkv2, 1), w.x2_rms_k, nullptr, 1e-6f, mx, d.NH, d.HS, 3 * C, 3 * C, st));
        }
        if (!bf) SD3_TRY(attention(ctx, dual_set, B, d.NH, d.HS, bf));
        GemmEpilogueArgs g2;
        g2.rows_per_batch = Tx; g2.gate = xchunk(8); g2.gate_ld = ldx_ada; g2.resid = x;
        SD3_TRY(linear_layer(ctx, prec, x_att2, w.x2_out_w, w.x2_out_b, x, 1, C, mx, C, C, EPI_GATE_RESID, g2));
    }

    // ---- MLPs of both streams (modules.cpp:1463-1476, 1488-1504)
    const int mcm = d.discard ? 0 : mc;
    {
        const LayerNormJob ln2[2] = {{x, x_hid, nullptr, xchunk(3), xchunk(4), nullptr, nullptr, ldx_ada, B, Tx},
                                     {c, c_hid, nullptr, cchunk(3), cchunk(4), nullptr, nullptr, ldc_ada, B, d.discard ? 0 : Tc}};
        SD3_TRY(ln_mod_pair(ctx, ln2, 2, 1e-6f, C, bf));
    }
    if (f8) {
        // fp8 MLPs: the inputs of both layers are quantised row by row (one factor per token), the weights column by column (one
        // factor per output channel) -- or one factor per tensor on either side -- and the products run on the fp8 matrix instruction
        const int H = d.E * C;
        auto fp8_pair = [&](const void* xa, const void* ca, int K, const float* xw, const float* cw, const float* xb, const float* cb, void* xo, void* co,
                            int N, int out_f32, int epi, const GemmEpilogueArgs& xe, const GemmEpilogueArgs& ce) -> int {
            {
                ProfScope ps(ctx, SD3_PROF_QUANT, (double)(mx + mcm) * K * 3.0, mcm ? 4 : 2);
                SD3_TRY(quantize_rows_fp8((const bf16_t*)xa, xq, xs, mx, K, f8 == 4, st));
                SD3_TRY(quantize_rows_fp8((const bf16_t*)ca, cq, cs, mcm, K, f8 == 4, st));
            }
            GemmBf16Problem probs[2];
            int n = 0;
            double flop = 0;
            const void* wp = nullptr;
            if (!xw) return fail(SD3_ERR_MISSING_PARAM, "a weight needed by this configuration is not bound (N=%d K=%d)", N, K);
            SD3_TRY(get_packed(ctx, xw, K, N, f8, &wp));
            probs[n] = GemmBf16Problem{(const bf16_t*)xq, (const bf16_t*)wp, xo, N, mx, N, K, xe};
            probs[n].ea.bias = xb; probs[n].ea.a_scale = xs; probs[n].ea.w_scale = (const float*)((const char*)wp + fp8_scale_offset(K, N));
            flop += 2.0 * mx * N * K;
            n++;
            if (mcm > 0) {
                if (!cw) return fail(SD3_ERR_MISSING_PARAM, "a weight needed by this configuration is not bound (N=%d K=%d)", N, K);
                SD3_TRY(get_packed(ctx, cw, K, N, f8, &wp));
                probs[n] = GemmBf16Problem{(const bf16_t*)cq, (const bf16_t*)wp, co, N, mcm, N, K, ce};
                probs[n].ea.bias = cb; probs[n].ea.a_scale = cs; probs[n].ea.w_scale = (const float*)((const char*)wp + fp8_scale_offset(K, N));
                flop += 2.0 * mcm * N * K;
                n++;
            }
            ProfScope ps(ctx, SD3_PROF_GEMM_FP8, flop);
            return gemm_fp8_grouped(probs, n, out_f32, epi, st);
        };
        SD3_TRY(fp8_pair(x_hid, c_hid, C, w.x_mlp_w1, w.c_mlp_w1, w.x_mlp_b1, w.c_mlp_b1, x_mlp, c_mlp, H, 0, EPI_BIAS_GELU, none, none));
        gc.gate = cchunk(5);
        gx.gate = xchunk(5);
        SD3_TRY(fp8_pair(x_mlp, c_mlp, H, w.x_mlp_w2, w.c_mlp_w2, w.x_mlp_b2, w.c_mlp_b2, x, c, C, 1, EPI_GATE_RESID, gx, gc));
        return SD3_OK;
    }
    {
        LayerCall up[2] = {{x_hid, w.x_mlp_w1, w.x_mlp_b1, x_mlp, d.E * C, mx, d.E * C, C, none},
                           {c_hid, w.c_mlp_w1, w.c_mlp_b1, c_mlp, d.E * C, mcm, d.E * C, C, none}};
        SD3_TRY(linear_pair(ctx, prec, up, 2, !bf, EPI_BIAS_GELU));
        gc.gate = cchunk(5);
        gx.gate = xchunk(5);
        LayerCall down[2] = {{x_mlp, w.x_mlp_w2, w.x_mlp_b2, x, C, mx, C, d.E * C, gx}, {c_mlp, w.c_mlp_w2, w.c_mlp_b2, c, C, mcm, C, d.E * C, gc}};
        SD3_TRY(linear_pair(ctx, prec, down, 2, 1, EPI_GATE_RESID));
    }
    return SD3_OK;
}

int check_block_dims(const Dims& d, int prec) {
    if (d.B <= 0 || d.Tc < 0 || d.Tx <= 0 || d.C <= 0 || d.NH <= 0 || d.E <= 0)
        return fail(SD3_ERR_INVALID_ARG, "block: sizes must be positive (B=%d Tc=%d Tx=%d emb_dim=%d heads=%d mlp_expand=%d)", d.B, d.Tc, d.Tx, d.C, d.NH, d.E);
    if (d.C % d.NH) return fail(SD3_ERR_INVALID_ARG, "block: emb_dim %d is not divisible by attn_heads %d", d.C, d.NH);
    if (prec < SD3_PREC_F32 || prec > SD3_PREC_BF16_FP8_TENSOR) return fail(SD3_ERR_INVALID_ARG, "unknown precision %d", prec);
    if (is_bf(prec) && (d.HS != 64 || d.C % 64)) return fail(SD3_ERR_UNSUPPORTED, "bf16 path needs head_dim 64 and emb_dim %% 64 == 0");
    if (fp8_kind(prec) && (d.C % 128)) return fail(SD3_ERR_UNSUPPORTED, "fp8 MLPs need emb_dim %% 128 == 0");
    if (prec == SD3_PREC_F32 && d.HS > 128) return fail(SD3_ERR_UNSUPPORTED, "fp32 path needs head_dim <= 128");
    return SD3_OK;
}

const float* find_param(sd3_ctx* ctx, const std::string& name, long long expect_numel, int* status) {
    auto it = ctx->params.find(name);
    if (it == ctx->params.end()) return nullptr;
    if (expect_numel > 0 && it->second.second != expect_numel) {
        *status = fail(SD3_ERR_INVALID_ARG, "parameter %s has %lld elements, expected %lld", name.c_str(), it->second.second, expect_numel);
        return nullptr;
    }
    return it->second.first;
}

int lookup_block_weights(sd3_ctx* ctx, const std::string& prefix, const Dims& d, sd3_block_weights* w) {
    int st = SD3_OK;
    const long long C = d.C, E = d.E;
    const long long cch = d.discard ? 2 : 6, xch = d.dual ? 9 : 6;
    auto g = [&](const char* n, long long numel) { return find_param(ctx, prefix + n, numel, &st); };
    w->c_ada_w = g("context_ada_lnorm.linear.weight", C * cch * C); w->c_ada_b = g("context_ada_lnorm.linear.bias", cch * C);
    w->c_qkv_w = g("context_to_qkv.weight", C * 3 * C); w->c_qkv_b = g("context_to_qkv.bias", 3 * C);
    w->c_rms_q = g("context_rmsnorm_query.weight", d.HS); w->c_rms_k = g("context_rmsnorm_key.weight", d.HS);
    w->c_out_w = g("context_attn_Wout.weight", C * C); w->c_out_b = g("context_attn_Wout.bias", C);
    w->c_mlp_w1 = g("context_mlp.lin1.weight", C * E * C); w->c_mlp_b1 = g("context_mlp.lin1.bias", E * C);
    w->c_mlp_w2 = g("context_mlp.lin2.weight", C * E * C); w->c_mlp_b2 = g("context_mlp.lin2.bias", C);
    w->x_ada_w = g("latent_ada_lnorm.linear.weight", C * xch * C); w->x_ada_b = g("latent_ada_lnorm.linear.bias", xch * C);
    w->x_qkv_w = g("latent_to_qkv.weight", C * 3 * C); w->x_qkv_b = g("latent_to_qkv.bias", 3 * C);
    w->x_rms_q = g("latent_rmsnorm_query.weight", d.HS); w->x_rms_k = g("latent_rmsnorm_key.weight", d.HS);
    w->x_out_w = g("latent_attn_Wout.weight", C * C); w->x_out_b = g("latent_attn_Wout.bias", C);
    w->x2_qkv_w = g("latent_dual_to_qkv.weight", C * 3 * C); w->x2_qkv_b = g("latent_dual_to_qkv.bias", 3 * C);
    w->x2_rms_q = g("latent_dual_rmsnorm_query.weight", d.HS); w->x2_rms_k = g("latent_dual_rmsnorm_key.weight", d.HS);
    w->x2_out_w = g("latent_dual_attn_Wout.weight", C * C); w->x2_out_b = g("latent_dual_attn_Wout.bias", C);
    w->x_mlp_w1 = g("latent_mlp.lin1.weight", C * E * C); w->x_mlp_b1 = g("latent_mlp.lin1.bias", E * C);
    w->x_mlp_w2 = g("latent_mlp.lin2.weight", C * E * C); w->x_mlp_b2 = g("latent_mlp.lin2.bias", C);
    return st;
}


}  // namespace

// ================================================================== C ABI
extern "C" {

const char* sd3_last_error(void) { return sd3::last_error(); }
int sd3_version(void) { return 1; }

#define ST(s) ((hipStream_t)(s))
#define NOTNULL(p) SD3_REQUIRE((p) != nullptr, "%s: null pointer argument '%s'", __func__, #p)

int sd3_layernorm(const float* x, float* y, float* mean, float* rstd, const float* w, const float* bias, float eps, int B, int T, int C, void* stream) {
    SD3_REQUIRE(B >= 0 && T >= 0 && C > 0, "layernorm: bad sizes B=%d T=%d C=%d", B, T, C);
    if ((long long)B * T == 0) return SD3_OK;
    NOTNULL(x); NOTNULL(y);
    return layernorm_full(x, y, mean, rstd, w, bias, eps, (long long)B * T, C, ST(stream));
}
int sd3_rmsnorm(const float* x, float* y, const float* w, float* rms, float eps, int B, int T, int C, void* stream) {
    SD3_REQUIRE(B >= 0 && T >= 0 && C > 0, "rmsnorm: bad sizes B=%d T=%d C=%d", B, T, C);
    if ((long long)B * T == 0) return SD3_OK;
    NOTNULL(x); NOTNULL(y);
    return rmsnorm_rows(x, y, w, rms, eps, (long long)B * T, 1, C, C, C, ST(stream));
}
int sd3_rmsnorm_group(const float* x, float* y, const float* w, float* rms, float eps, int groups, int B, int T, int C, void* stream) {
    SD3_REQUIRE(B >= 0 && T >= 0 && C > 0 && groups > 0, "rmsnorm_group: bad sizes B=%d T=%d C=%d groups=%d", B, T, C, groups);
    SD3_REQUIRE(C % groups == 0, "rmsnorm_group: C=%d is not divisible by groups=%d", C, groups);
    if ((long long)B * T == 0) return SD3_OK;
    NOTNULL(x); NOTNULL(y);
    return rmsnorm_rows(x, y, w, rms, eps, (long long)B * T, groups, C / groups, C, C, ST(stream));
}
int sd3_gelu_tanh(const float* in, float* out, long long n, void* stream) {
    SD3_REQUIRE(n >= 0, "gelu_tanh: negative size");
    if (n == 0) return SD3_OK;
    NOTNULL(in); NOTNULL(out);
    return unary_op(in, out, n, SD3_ACT_GELU_TANH, ST(stream));
}
int sd3_gelu(const float* in, float* out, long long n, void* stream) {
    SD3_REQUIRE(n >= 0, "gelu: negative size");
    if (n == 0) return SD3_OK;
    NOTNULL(in); NOTNULL(out);
    return unary_op(in, out, n, SD3_ACT_GELU_ERF, ST(stream));
}
int sd3_silu(const float* in, float* out, long long n, void* stream) {
    SD3_REQUIRE(n >= 0, "silu: negative size");
    if (n == 0) return SD3_OK;
    NOTNULL(in); NOTNULL(out);
    return unary_op(in, out, n, SD3_ACT_SILU, ST(stream));
}
int sd3_linear(const float* x, const float* W, const float* b, float* y, int B, int C_in, int C_out, void* stream) {
    SD3_REQUIRE(B >= 0 && C_in > 0 && C_out > 0, "linear: bad sizes B=%d C_in=%d C_out=%d", B, C_in, C_out);
    if (B == 0) return SD3_OK;
    NOTNULL(x); NOTNULL(W); NOTNULL(b); NOTNULL(y);
    GemmEpilogueArgs ea;
    ea.bias = b;
    return gemm_f32(x, C_in, W, C_out, 0, y, C_out, B, C_out, C_in, EPI_BIAS, ea, ST(stream));
}
int sd3_partial_linear(const float* x, const float* W, const float* b, float* y, int M, int K, int N, int Nmax, int n0, void* stream) {
    SD3_REQUIRE(M >= 0 && K > 0 && N > 0 && n0 >= 0 && n0 + N <= Nmax, "partial_linear: bad sizes M=%d K=%d N=%d Nmax=%d n0=%d", M, K, N, Nmax, n0);
    if (M == 0) return SD3_OK;
    NOTNULL(x); NOTNULL(W); NOTNULL(b); NOTNULL(y);
    GemmEpilogueArgs ea;
    ea.bias = b;
    return gemm_f32(x, K, W, Nmax, n0, y, N, M, N, K, EPI_BIAS, ea, ST(stream));
}
int sd3_add(const float* a, const float* b, float* out, long long n, void* stream) {
    SD3_REQUIRE(n >= 0, "add: negative size");
    if (n == 0) return SD3_OK;
    NOTNULL(a); NOTNULL(b); NOTNULL(out);
    return add_op(a, b, out, n, ST(stream));
}
int sd3_multihead_attention(const float* Q, const float* K, const float* V, float* out, int B, int num_heads, int T, int L, int head_dim, void* stream) {
    SD3_REQUIRE(B >= 0 && num_heads > 0 && T >= 0 && L > 0 && head_dim > 0, "multihead_attention: bad sizes B=%d heads=%d T=%d L=%d head_dim=%d", B,
                num_heads, T, L, head_dim);
    if (B == 0 || T == 0) return SD3_OK;
    NOTNULL(Q); NOTNULL(K); NOTNULL(V); NOTNULL(out);
    AttnSegments a{};
    const int C = num_heads * head_dim;
    a.q[0] = Q; a.k[0] = K; a.v[0] = V; a.out[0] = out;
    a.ld_qkv[0] = a.ld_qkv[1] = C; a.ld_out[0] = a.ld_out[1] = C;
    a.T[0] = L; a.Tq[0] = T;
    return attention_f32(a, B, num_heads, head_dim, ST(stream));
}
int sd3_sinusoidal_embedding(const float* timesteps, float* out, int B, int emb_dim, void* stream) {
    SD3_REQUIRE(B >= 0 && emb_dim > 0 && emb_dim % 2 == 0, "sinusoidal_embedding: bad sizes B=%d emb_dim=%d", B, emb_dim);
    if (B == 0) return SD3_OK;
    NOTNULL(timesteps); NOTNULL(out);
    return timestep_embedding(timesteps, out, B, emb_dim, ST(stream));
}
int sd3_positional_embedding2D(float* out, int emb_dim, int height, int width, int base_size, void* stream) {
    SD3_REQUIRE(emb_dim > 0 && emb_dim % 4 == 0 && height > 0 && width > 0, "positional_embedding2D: bad sizes emb_dim=%d height=%d width=%d", emb_dim,
                height, width);
    NOTNULL(out);
    return pos_embed_table(out, emb_dim, height, width, base_size, ST(stream));
}
int sd3_crop_positional_embedding2D(const float* pos_embed, float* out, int pos_embed_max_size, int new_height, int new_width, int emb_dim, void* stream) {
    SD3_REQUIRE(new_height > 0 && new_width > 0 && emb_dim > 0 && new_height <= pos_embed_max_size && new_width <= pos_embed_max_size,
                "crop_positional_embedding2D: %dx%d does not fit a table of size %d", new_height, new_width, pos_embed_max_size);
    NOTNULL(pos_embed); NOTNULL(out);
    return pos_embed_crop(pos_embed, out, pos_embed_max_size, new_height, new_width, emb_dim, ST(stream));
}
int sd3_conv2d(const float* in, float* out, const float* kernel, const float* bias, int B, int kernel_height, int kernel_width, int in_channels,
               int out_channels, int in_height, int in_width, int out_height, int out_width, int stride, int padding, void* stream) {
    SD3_REQUIRE(B >= 0 && kernel_height > 0 && kernel_width > 0 && in_channels > 0 && out_channels > 0 && stride > 0 && padding >= 0, "conv2d: bad sizes");
    SD3_REQUIRE(out_height == (in_height + 2 * padding - kernel_height) / stride + 1 && out_width == (in_width + 2 * padding - kernel_width) / stride + 1,
                "conv2d: output size %dx%d does not match the input/kernel/stride/padding", out_height, out_width);
    if (B == 0) return SD3_OK;
    NOTNULL(in); NOTNULL(out); NOTNULL(kernel); NOTNULL(bias);
    return conv2d_direct(in, out, kernel, bias, B, kernel_height, kernel_width, in_channels, out_channels, in_height, in_width, out_height, out_width,
                         stride, padding, ST(stream));
}
int sd3_patch_embedding(const float* latent, float* out, const float* kernel, const float* bias, int B, int H, int W, int C_in, int emb_dim,
                        int patch_size, int pos_embed_max_size, int base_height, void* stream) {
    SD3_REQUIRE(B >= 0 && H > 0 && W > 0 && C_in > 0 && emb_dim > 0 && emb_dim % 4 == 0 && patch_size > 0, "patch_embedding: bad sizes");
    const int hp = (H - patch_size) / patch_size + 1, wp = (W - patch_size) / patch_size + 1;
    SD3_REQUIRE(hp > 0 && wp > 0 && hp <= pos_embed_max_size && wp <= pos_embed_max_size,
                "patch_embedding: a %dx%d patch grid does not fit pos_embed_max_size=%d", hp, wp, pos_embed_max_size);
    if (B == 0) return SD3_OK;
    NOTNULL(latent); NOTNULL(out); NOTNULL(kernel); NOTNULL(bias);
    return patch_embed_direct(latent, out, kernel, bias, B, H, W, C_in, emb_dim, patch_size, pos_embed_max_size, base_height, ST(stream));
}
int sd3_mlp(const float* x, float* out, float* h1, const float* W1, const float* b1, const float* W2, const float* b2, int B, int C_in, int C_hid,
            int C_out, int activation, void* stream) {
    SD3_REQUIRE(B >= 0 && C_in > 0 && C_hid > 0 && C_out > 0, "mlp: bad sizes");
    SD3_REQUIRE(activation == SD3_ACT_SILU || activation == SD3_ACT_GELU_TANH, "mlp: unknown activation %d", activation);
    if (B == 0) return SD3_OK;
    NOTNULL(x); NOTNULL(out); NOTNULL(h1); NOTNULL(W1); NOTNULL(b1); NOTNULL(W2); NOTNULL(b2);
    GemmEpilogueArgs ea;
    ea.bias = b1;
    SD3_TRY(gemm_f32(x, C_in, W1, C_hid, 0, h1, C_hid, B, C_hid, C_in, activation == SD3_ACT_SILU ? EPI_BIAS_SILU : EPI_BIAS_GELU, ea, ST(stream)));
    ea.bias = b2;
    return gemm_f32(h1, C_hid, W2, C_out, 0, out, C_out, B, C_out, C_hid, EPI_BIAS, ea, ST(stream));
}
int sd3_scale_and_shift(const float* in, float* out, const float* shift, const float* scale, int B, int T, int C, void* stream) {
    SD3_REQUIRE(B >= 0 && T >= 0 && C > 0, "scale_and_shift: bad sizes");
    if ((long long)B * T == 0) return SD3_OK;
    NOTNULL(in); NOTNULL(out); NOTNULL(shift); NOTNULL(scale);
    return modulate_op(in, out, shift, scale, B, T, C, ST(stream));
}
int sd3_gating_mechanism(const float* in, float* out, const float* gate, int B, int T, int C, void* stream) {
    SD3_REQUIRE(B >= 0 && T >= 0 && C > 0, "gating_mechanism: bad sizes");
    if ((long long)B * T == 0) return SD3_OK;
    NOTNULL(in); NOTNULL(out); NOTNULL(gate);
    return gate_op(in, out, gate, B, T, C, ST(stream));
}
int sd3_concatenate_along_tokens(const float* x, const float* y, float* out, int B, int Tx, int Ty, int C, void* stream) {
    SD3_REQUIRE(B >= 0 && Tx >= 0 && Ty >= 0 && C > 0, "concatenate_along_tokens: bad sizes");
    if (B == 0) return SD3_OK;
    NOTNULL(out);
    const long long T = (long long)Tx + Ty;
    if (Tx) { NOTNULL(x); SD3_TRY(copy_rows(x, (long long)Tx * C, out, T * C, B, (long long)Tx * C, ST(stream))); }
    if (Ty) { NOTNULL(y); SD3_TRY(copy_rows(y, (long long)Ty * C, out + (long long)Tx * C, T * C, B, (long long)Ty * C, ST(stream))); }
    return SD3_OK;
}
int sd3_split_along_tokens(const float* in, float* split1, float* split2, int B, int T1, int T2, int C, void* stream) {
    SD3_REQUIRE(B >= 0 && T1 >= 0 && T2 >= 0 && C > 0, "split_along_tokens: bad sizes");
    if (B == 0) return SD3_OK;
    NOTNULL(in);
    const long long T = (long long)T1 + T2;
    if (T1) { NOTNULL(split1); SD3_TRY(copy_rows(in, T * C, split1, (long long)T1 * C, B, (long long)T1 * C, ST(stream))); }
    if (T2) { NOTNULL(split2); SD3_TRY(copy_rows(in + (long long)T1 * C, T * C, split2, (long long)T2 * C, B, (long long)T2 * C, ST(stream))); }
    return SD3_OK;
}

// ------------------------------------------------------------------ context
int sd3_ctx_create(sd3_ctx** out, int device) {
    NOTNULL(out);
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        (void)hipGetLastError();
        return fail(SD3_ERR_HIP, "no HIP device available (%s)", e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    }
    SD3_REQUIRE(device >= 0 && device < n, "ctx_create: device %d out of range (0..%d)", device, n - 1);
    sd3_ctx* c = new (std::nothrow) sd3_ctx();
    if (!c) return fail(SD3_ERR_OOM, "ctx_create: out of host memory");
    c->device = device;
    {
        // the address of the fixed scratch array on this device, asked for once per device with that device current
        DeviceGuard g(device);
        int rc = g.ok ? static_scratch_of(device, &c->static_scratch) : fail(SD3_ERR_HIP, "cannot select device %d", device);
        if (rc == SD3_OK && hipEventCreateWithFlags(&c->order_event, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            rc = fail(SD3_ERR_HIP, "ctx_create: cannot create the ordering event on device %d", device);
        }
        if (rc != SD3_OK) {
            delete c;
            return rc;
        }
    }
    *out = c;
    return SD3_OK;
}
int sd3_weights_clear(sd3_ctx* ctx) {
    NOTNULL(ctx);
    DeviceGuard g(ctx->device);
    SD3_TRY(wait_idle(ctx));
    for (auto& kv : ctx->packed) (void)hipFree(kv.second.ptr);
    ctx->packed.clear();
    ctx->params.clear();
    return SD3_OK;
}
int sd3_ctx_destroy(sd3_ctx* ctx) {
    if (!ctx) return SD3_OK;
    {
        DeviceGuard g(ctx->device);
        (void)wait_idle(ctx);
        for (auto& kv : ctx->packed) (void)hipFree(kv.second.ptr);
        for (auto& kv : ctx->pos_tables) (void)hipFree(kv.second);
        if (ctx->ws) (void)hipFree(ctx->ws);
        for (auto& p : ctx->prof) {
            (void)hipEventDestroy(p.a);
            (void)hipEventDestroy(p.b);
        }
        for (auto e : ctx->event_pool) (void)hipEventDestroy(e);
        if (ctx->order_event) (void)hipEventDestroy(ctx->order_event);
        (void)hipGetLastError();
    }
    delete ctx;
    return SD3_OK;
}
int sd3_ctx_set_stream(sd3_ctx* ctx, void* stream) {
    NOTNULL(ctx);
    if (ST(stream) == ctx->stream) return SD3_OK;
    // The workspace, the derived weight copies and the position tables are shared by everything the context enqueues: work
    // already queued on the old stream must finish before work on the new stream touches them.
    // The old stream's handle is not used here (its owner may have destroyed it since the last call): the new stream waits on the
    // event recorded behind that call's last kernel. A stream that is being captured into a graph cannot wait on work outside the
    // capture; its owner has ordered the capture behind earlier work, and orders the graph's replays.
    DeviceGuard g(ctx->device);
    if (!g.ok) return fail(SD3_ERR_HIP, "cannot select device %d", ctx->device);
    if (ctx->order_pending) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        SD3_HIP_TRY(hipStreamIsCapturing(ST(stream), &cap));
        if (cap == hipStreamCaptureStatusNone) SD3_HIP_TRY(hipStreamWaitEvent(ST(stream), ctx->order_event, 0));
    }
    ctx->stream = ST(stream);
    return SD3_OK;
}
int sd3_ctx_synchronize(sd3_ctx* ctx) {
    NOTNULL(ctx);
    DeviceGuard g(ctx->device);
    SD3_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SD3_OK;
}
int sd3_weights_bind(sd3_ctx* ctx, const char* name, const float* ptr, long long numel) {
    NOTNULL(ctx); NOTNULL(name); NOTNULL(ptr);
    SD3_REQUIRE(numel > 0, "weights_bind(%s): numel must be positive", name);
    SD3_REQUIRE((reinterpret_cast<uintptr_t>(ptr) & 3) == 0, "weights_bind(%s): pointer is not 4-byte aligned", name);
    // Binding a name again to the tensor it is already bound to (same address, same size) changes nothing and keeps the derived
    // copies: callers shaped like the reference's entry points hand over the whole parameter map on every call.
    auto old = ctx->params.find(name);
    if (old != ctx->params.end() && old->second.first == ptr && old->second.second == numel) return SD3_OK;
    // Otherwise: derived copies are keyed by the tensor's address, so what was made from the tensor this name was bound to before,
    // or from an earlier tensor that lived at the new address, must not survive the re-binding.
    if (old != ctx->params.end() && old->second.first != ptr) SD3_TRY(drop_packed_of(ctx, old->second.first));
    SD3_TRY(drop_packed_of(ctx, ptr));
    ctx->params[name] = std::make_pair(ptr, numel);
    return SD3_OK;
}
int sd3_weights_unbind(sd3_ctx* ctx, const char* name) {
    NOTNULL(ctx); NOTNULL(name);
    auto it = ctx->params.find(name);
    if (it == ctx->params.end()) return SD3_OK;
    SD3_TRY(drop_packed_of(ctx, it->second.first));
    ctx->params.erase(it);
    return SD3_OK;
}
int sd3_weights_forget(sd3_ctx* ctx, const float* ptr) {
    NOTNULL(ctx); NOTNULL(ptr);
    return drop_packed_of(ctx, ptr);
}
int sd3_weights_copies_built(sd3_ctx* ctx, long long* count) {
    NOTNULL(ctx); NOTNULL(count);
    *count = ctx->copies_built;
    return SD3_OK;
}
int sd3_weights_prepare(sd3_ctx* ctx, int precision) {
    NOTNULL(ctx);
    SD3_REQUIRE(precision >= SD3_PREC_F32 && precision <= SD3_PREC_BF16_FP8_TENSOR, "weights_prepare: unknown precision %d", precision);
    DeviceGuard g(ctx->device);
    if (!g.ok) return fail(SD3_ERR_HIP, "cannot select device %d", ctx->device);
    // drop what exists (the bound tensors may have been changed in place) ...
    OrderScope order(ctx);
    SD3_TRY(wait_idle(ctx));
    for (auto& kv : ctx->packed) (void)hipFree(kv.second.ptr);
    ctx->packed.clear();
    // ... and rebuild every copy the forward of this precision would otherwise build on first use. A linear layer's shape follows
    // from its two bound tensors: `<layer>.bias` has C_out elements and `<layer>.weight` C_in * C_out.
    auto ends_with = [](const std::string& s, const char* suffix) {
        const size_t n = std::strlen(suffix);
        return s.size() >= n && s.compare(s.size() - n, n, suffix) == 0;
    };
    for (auto& kv : ctx->params) {
        const std::string& name = kv.first;
        if (!ends_with(name, ".weight")) continue;
        auto b = ctx->params.find(name.substr(0, name.size() - 6) + "bias");
        if (b == ctx->params.end() || b->second.second <= 0 || kv.second.second % b->second.second) continue;
        const long long N = b->second.second, K = kv.second.second / N;
        const void* unused = nullptr;
        if (name == "to_patch.conv.weight") {  // (C_out, C_in*p*p): bf16 cast for the MFMA GEMM, fp32 transpose for the fp32 one
            if (is_bf(precision)) SD3_TRY(get_packed(ctx, kv.second.first, N, K, 1, &unused));
            else SD3_TRY(get_packed(ctx, kv.second.first, K, N, 2, &unused));
            continue;
        }
        if (!is_bf(precision)) continue;
        if (fp8_kind(precision) && (ends_with(name, "_mlp.lin1.weight") || ends_with(name, "_mlp.lin2.weight")) && K % 128 == 0) {
            SD3_TRY(get_packed(ctx, kv.second.first, K, N, fp8_kind(precision), &unused));
            continue;
        }
        const bool adaln = ends_with(name, "ada_lnorm.linear.weight") || name == "ada_ln_out.linear.weight";
        const bool gemm = ends_with(name, "_to_qkv.weight") || ends_with(name, "_attn_Wout.weight") || ends_with(name, "_mlp.lin1.weight") ||
                          ends_with(name, "_mlp.lin2.weight") || name == "captions_linear.weight" || name == "linear_out.weight";
        if (adaln) SD3_TRY(get_packed(ctx, kv.second.first, K, N, 1, &unused));
        else if (gemm && K % 64 == 0) SD3_TRY(get_packed(ctx, kv.second.first, K, N, 0, &unused));
    }
    return SD3_OK;
}

int sd3_profile_begin(sd3_ctx* ctx) {
    NOTNULL(ctx);
    for (auto& p : ctx->prof) {
        ctx->event_pool.push_back(p.a);
        ctx->event_pool.push_back(p.b);
    }
    ctx->prof.clear();
    ctx->prof_on = true;
    return SD3_OK;
}
int sd3_profile_end(sd3_ctx* ctx, double* ms, double* work, long long* launches) {
    NOTNULL(ctx); NOTNULL(ms); NOTNULL(work); NOTNULL(launches);
    ctx->prof_on = false;
    DeviceGuard g(ctx->device);
    SD3_HIP_TRY(hipStreamSynchronize(ctx->stream));
    for (int i = 0; i < SD3_PROF_CLASSES; i++) {
        ms[i] = 0;
        work[i] = 0;
        launches[i] = 0;
    }
    for (auto& p : ctx->prof) {
        float t = 0.f;
        SD3_HIP_TRY(hipEventElapsedTime(&t, p.a, p.b));
        ms[p.cls] += t;
        work[p.cls] += p.work;
        launches[p.cls] += p.launches;
        ctx->event_pool.push_back(p.a);
        ctx->event_pool.push_back(p.b);
    }
    ctx->prof.clear();
    return SD3_OK;
}

// ------------------------------------------------------------------ block
int sd3_dit_block_w(sd3_ctx* ctx, const float* y, float* c, float* x, const sd3_block_weights* w, int B, int Tc, int Tx, int emb_dim, int attn_heads,
                    int mlp_expand, int use_dual_attention, int use_qk_norm, int discard_context, int precision) {
    NOTNULL(ctx); NOTNULL(y); NOTNULL(x); NOTNULL(w);
    SD3_REQUIRE(attn_heads > 0, "block: attn_heads must be positive");
    Dims d{B, Tc, Tx, emb_dim, attn_heads, emb_dim / attn_heads, mlp_expand, use_dual_attention != 0, use_qk_norm != 0, discard_context != 0};
    SD3_TRY(check_block_dims(d, precision));
    if (Tc > 0) NOTNULL(c);
    DeviceGuard g(ctx->device);
    if (!g.ok) return fail(SD3_ERR_HIP, "cannot select device %d", ctx->device);
    OrderScope order(ctx);
    SD3_TRY(ensure_workspace(ctx, block_workspace_bytes(d, precision)));
    Bump ws(ctx->ws, ctx->ws_bytes);
    return run_block(ctx, precision, y, c, x, *w, d, nullptr, nullptr, ws);
}

int sd3_dit_block(sd3_ctx* ctx, const float* y, float* c, float* x, const char* prefix, int B, int Tc, int Tx, int emb_dim, int attn_heads, int mlp_expand,
                  int use_dual_attention, int use_qk_norm, int discard_context, int precision) {
    NOTNULL(ctx);
    SD3_REQUIRE(attn_heads > 0 && emb_dim > 0, "block: emb_dim and attn_heads must be positive");
    Dims d{B, Tc, Tx, emb_dim, attn_heads, emb_dim / attn_heads, mlp_expand, use_dual_attention != 0, use_qk_norm != 0, discard_context != 0};
    SD3_TRY(check_block_dims(d, precision));
    sd3_block_weights w;
    SD3_TRY(lookup_block_weights(ctx, prefix ? prefix : "", d, &w));
    return sd3_dit_block_w(ctx, y, c, x, &w, B, Tc, Tx, emb_dim, attn_heads, mlp_expand, use_dual_attention, use_qk_norm, discard_context, precision);
}

// The block without any allocation: intermediates live in the fixed scratch array instead of the context's workspace.
// Calls on one device share that array, so two of them must not overlap in time. Nothing in it has to start at zero:
// every intermediate is written in full by the kernel that produces it before another kernel reads it.
int sd3_dit_block_static(sd3_ctx* ctx, const float* y, float* c, float* x, const char* prefix, int B, int Tc, int Tx, int emb_dim, int attn_heads,
                         int mlp_expand, int use_dual_attention, int use_qk_norm, int discard_context, int precision) {
    NOTNULL(ctx); NOTNULL(y); NOTNULL(x);
    SD3_REQUIRE(attn_heads > 0 && emb_dim > 0, "block: emb_dim and attn_heads must be positive");
    Dims d{B, Tc, Tx, emb_dim, attn_heads, emb_dim / attn_heads, mlp_expand, use_dual_attention != 0, use_qk_norm != 0, discard_context != 0};
    SD3_TRY(check_block_dims(d, precision));
    if (Tc > 0) NOTNULL(c);
    const size_t need = block_workspace_bytes(d, precision);
    if (need > (size_t)SD3_STATIC_SCRATCH_BYTES)
        return fail(SD3_ERR_UNSUPPORTED, "dit_block_static: this block needs %zu bytes of intermediates, the fixed scratch array holds %zu; use sd3_dit_block",
                    need, (size_t)SD3_STATIC_SCRATCH_BYTES);
    sd3_block_weights w;
    SD3_TRY(lookup_block_weights(ctx, prefix ? prefix : "", d, &w));
    DeviceGuard g(ctx->device);
    if (!g.ok) return fail(SD3_ERR_HIP, "cannot select device %d", ctx->device);
    if (!ctx->static_scratch) return fail(SD3_ERR_HIP, "dit_block_static: the fixed scratch array has no address on device %d", ctx->device);
    OrderScope order(ctx);  // (records an event that exists since the context was created: no allocation)
    Bump ws(ctx->static_scratch, SD3_STATIC_SCRATCH_BYTES);
    ctx->no_alloc = true;
    const int rc = run_block(ctx, precision, y, c, x, w, d, nullptr, nullptr, ws);
    ctx->no_alloc = false;
    return rc;
}

// ------------------------------------------------------------------ full forward
// guidance step: null for the plain forward (out = velocity of every batch element); otherwise the batch is
// [B/2 unconditional ; B/2 conditional] and out (B/2 samples) = latent + dsigma * (v_u + guidance * (v_c - v_u))
struct CfgEulerStep {
    float guidance, dsigma;
};
static int dit_forward_impl(sd3_ctx* ctx, const float* pooled, const float* captions, const float* latent, const float* timesteps, float* out, int B, int Tc,
                            int H, int W, int num_layers, const int* dual_attention_layers, int n_dual, int pooled_dim, int captions_dim, int C_in,
                            int emb_dim, int attn_heads, int mlp_expand, int patch_size, int pos_embed_max_size, int base_height, int use_qk_norm,
                            int precision, const CfgEulerStep* step) {
    NOTNULL(ctx); NOTNULL(pooled); NOTNULL(captions); NOTNULL(latent); NOTNULL(timesteps); NOTNULL(out);
    SD3_REQUIRE(num_layers > 0 && patch_size > 0 && H >= patch_size && W >= patch_size && C_in > 0 && pooled_dim > 0 && captions_dim > 0 && attn_heads > 0 &&
                    emb_dim > 0 && n_dual >= 0 && (n_dual == 0 || dual_attention_layers),
                "DiT: bad sizes");
    const int C = emb_dim, p = patch_size;
    const int Hp = (H - p) / p + 1, Wp = (W - p) / p + 1, Tx = Hp * Wp, PPC = p * p * C_in, Kp = C_in * p * p;
    SD3_REQUIRE(Hp <= pos_embed_max_size && Wp <= pos_embed_max_size, "DiT: a %dx%d patch grid does not fit pos_embed_max_size=%d", Hp, Wp, pos_embed_max_size);
    SD3_REQUIRE(C % 4 == 0, "DiT: emb_dim must be a multiple of 4");
    Dims dmax{B, Tc, Tx, C, attn_heads, C / attn_heads, mlp_expand, n_dual > 0, use_qk_norm != 0, false};
    SD3_TRY(check_block_dims(dmax, precision));
    const bool bf = is_bf(precision);
    if (bf && ((captions_dim % 64) || (Kp % 64))) return fail(SD3_ERR_UNSUPPORTED, "bf16 path needs captions_dim and C_in*patch^2 to be multiples of 64");
    DeviceGuard g(ctx->device);
    if (!g.ok) return fail(SD3_ERR_HIP, "cannot select device %d", ctx->device);
    OrderScope order(ctx);
    hipStream_t st = ctx->stream;

    std::vector<char> is_dual(num_layers, 0);
    for (int i = 0; i < n_dual; i++)
        if (dual_attention_layers[i] >= 0 && dual_attention_layers[i] < num_layers) is_dual[dual_attention_layers[i]] = 1;

    // ---- weights by name (modules.cpp:1665-1728)
    int pst = SD3_OK;
    auto P = [&](const char* n, long long numel) -> const float* {
        const float* q = find_param(ctx, n, numel, &pst);
        if (!q && pst == SD3_OK) pst = fail(SD3_ERR_MISSING_PARAM, "parameter %s is not bound", n);
        return q;
    };
    const float* t_w0 = P("timestep_mlp.0.weight", 256LL * C); const float* t_b0 = P("timestep_mlp.0.bias", C);
    const float* t_w2 = P("timestep_mlp.2.weight", (long long)C * C); const float* t_b2 = P("timestep_mlp.2.bias", C);
    const float* p_w0 = P("pooled_mlp.0.weight", (long long)pooled_dim * C); const float* p_b0 = P("pooled_mlp.0.bias", C);
    const float* p_w2 = P("pooled_mlp.2.weight", (long long)C * C); const float* p_b2 = P("pooled_mlp.2.bias", C);
    const float* cap_w = P("captions_linear.weight", (long long)captions_dim * C); const float* cap_b = P("captions_linear.bias", C);
    const float* patch_w = P("to_patch.conv.weight", (long long)C * Kp); const float* patch_b = P("to_patch.conv.bias", C);
    const float* ao_w = P("ada_ln_out.linear.weight", 2LL * C * C); const float* ao_b = P("ada_ln_out.linear.bias", 2LL * C);
    const float* out_w = P("linear_out.weight", (long long)C * PPC); const float* out_b = P("linear_out.bias", PPC);
    if (pst != SD3_OK) return pst;
    std::vector<sd3_block_weights> bw(num_layers);
    std::vector<Dims> bd(num_layers, dmax);
    for (int l = 0; l < num_layers; l++) {
        bd[l].dual = is_dual[l] != 0;
        bd[l].discard = (l == num_layers - 1);
        SD3_TRY(lookup_block_weights(ctx, "transformer." + std::to_string(l) + ".", bd[l], &bw[l]));
        if (!bw[l].c_ada_w || !bw[l].c_ada_b || !bw[l].x_ada_w || !bw[l].x_ada_b)
            return fail(SD3_ERR_MISSING_PARAM, "transformer.%d: adaLN modulation weights are not bound", l);
    }

    // ---- workspace
    auto layout = [&](Bump& b, float** temb, float** h1, float** h2, float** yt, float** yp, float** y, float** c, float** x, void** cap_in, void** patches,
                      float** ada_all, float** ada_out, float** tokens) {
        *temb = b.take<float>((size_t)B * 256);
        *h1 = b.take<float>((size_t)B * C);
        *h2 = b.take<float>((size_t)B * C);
        *yt = b.take<float>((size_t)B * C);
        *yp = b.take<float>((size_t)B * C);
        *y = b.take<float>((size_t)B * C);
        *c = b.take<float>((size_t)B * Tc * C);
        *x = b.take<float>((size_t)B * Tx * C);
        *cap_in = bf ? (void*)b.take<bf16_t>((size_t)B * Tc * captions_dim) : nullptr;
        *patches = b.take<char>((size_t)B * Tx * Kp * (bf ? 2 : 4));
        *ada_all = b.take<float>((size_t)B * 15 * C * num_layers);
        *ada_out = b.take<float>((size_t)B * 2 * C);
        *tokens = b.take<float>((size_t)B * Tx * PPC);
    };
    float *temb, *h1, *h2, *yt, *yp, *y, *c, *x, *ada_all, *ada_out, *tokens;
    void *cap_in, *patches;
    Bump probe(nullptr, 0);
    layout(probe, &temb, &h1, &h2, &yt, &yp, &y, &c, &x, &cap_in, &patches, &ada_all, &ada_out, &tokens);
    SD3_TRY(ensure_workspace(ctx, probe.off + block_workspace_bytes(dmax, precision)));
    Bump ws(ctx->ws, ctx->ws_bytes);
    layout(ws, &temb, &h1, &h2, &yt, &yp, &y, &c, &x, &cap_in, &patches, &ada_all, &ada_out, &tokens);
    const size_t block_ws_off = ws.off;

    // ---- y = silu(MLP(t_emb) + MLP(pooled)) (modules.cpp:1663-1675); weights stay fp32 here: 8 MB read once
    SD3_TRY(timestep_embedding(timesteps, temb, B, 256, st));
    {
        // the two MLPs side by side: both first layers in one launch (each job brings its own input), then both second layers
        const SmallLinearJob first[2] = {{t_w0, t_b0, h1, C, C, 0, temb, 256}, {p_w0, p_b0, h2, C, C, 0, pooled, pooled_dim}};
        SD3_TRY(small_linear_batched(nullptr, B, 0, first, 2, 0, SD3_ACT_SILU, st));
        const SmallLinearJob second[2] = {{t_w2, t_b2, yt, C, C, 0, h1, C}, {p_w2, p_b2, yp, C, C, 0, h2, C}};
        SD3_TRY(small_linear_batched(nullptr, B, 0, second, 2, 0, -1, st));
        SD3_TRY(add_silu_op(yt, yp, y, (long long)B * C, st));
    }
    // ---- c = captions @ W + b (modules.cpp:1678)
    {
        GemmEpilogueArgs none;
        const void* a_in = captions;
        if (bf) {
            SD3_TRY(cast_f32_to_bf16(captions, (bf16_t*)cap_in, (long long)B * Tc * captions_dim, st));
            a_in = cap_in;
        }
        if (Tc > 0) SD3_TRY(linear_layer(ctx, precision, a_in, cap_w, cap_b, c, 1, C, B * Tc, C, captions_dim, EPI_BIAS, none));
    }
    // ---- x = patchify-conv(latent) + bias + position table (modules.cpp:1682 -> 1093-1117) as an im2col GEMM
    {
        auto key = std::make_tuple(C, pos_embed_max_size, base_height / p, Hp, Wp);
        float* table = nullptr;
        auto it = ctx->pos_tables.find(key);
        if (it == ctx->pos_tables.end()) {
            hipError_t e = hipMalloc((void**)&table, (size_t)Tx * C * sizeof(float));
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return fail(SD3_ERR_OOM, "position table: %s", hipGetErrorString(e));
            }
            int rc = pos_embed_cropped(table, C, pos_embed_max_size, base_height / p, Hp, Wp, st);
            if (rc != SD3_OK) {
                (void)hipFree(table);
                return rc;
            }
            ctx->pos_tables[key] = table;
        } else {
            table = it->second;
        }
        SD3_TRY(im2col_patches(latent, patches, bf, B, C_in, H, W, p, st));
        GemmEpilogueArgs ea;
        ea.bias = patch_b; ea.table = table; ea.rows_per_batch = Tx;
        if (bf) {
            // the conv weight (C, C_in*p*p) is already (N,K) K-contiguous: its MFMA form is a plain cast
            const void* wp = nullptr;
            SD3_TRY(get_packed(ctx, patch_w, C, Kp, 1, &wp));
            ProfScope ps(ctx, SD3_PROF_GEMM, 2.0 * B * Tx * C * Kp);
            SD3_TRY(gemm_bf16((const bf16_t*)patches, (const bf16_t*)wp, x, 1, C, B * Tx, C, Kp, EPI_BIAS_ROWADD, ea, st));
        } else {
            const void* wt = nullptr;
            SD3_TRY(get_packed(ctx, patch_w, Kp, C, 2, &wt));
            ProfScope ps(ctx, SD3_PROF_GEMM, 2.0 * B * Tx * C * Kp);
            SD3_TRY(gemm_f32((const float*)patches, Kp, (const float*)wt, C, 0, x, C, B * Tx, C, Kp, EPI_BIAS_ROWADD, ea, st));
        }
    }
    // ---- modulation vectors of every block and of the output layer: y does not change across blocks, so all
    //      adaLN projections (0.77 G parameters) are streamed once, up front
    {
        std::vector<SmallLinearJob> jobs;
        for (int l = 0; l < num_layers; l++) {
            const int cch = bd[l].discard ? 2 : 6, xch = bd[l].dual ? 9 : 6;
            float* base = ada_all + (size_t)l * B * 15 * C;
            jobs.push_back({bw[l].c_ada_w, bw[l].c_ada_b, base, cch * C, cch * C, 0});
            jobs.push_back({bw[l].x_ada_w, bw[l].x_ada_b, base + (size_t)B * 6 * C, xch * C, xch * C, 0});
        }
        jobs.push_back({ao_w, ao_b, ada_out, 2 * C, 2 * C, 0});
        SD3_TRY(ada_jobs_run(ctx, precision, y, B, C, jobs));
    }
    // ---- blocks (modules.cpp:1687-1718)
    for (int l = 0; l < num_layers; l++) {
        Bump bws(ctx->ws, ctx->ws_bytes);
        bws.off = block_ws_off;
        const float* base = ada_all + (size_t)l * B * 15 * C;
        SD3_TRY(run_block(ctx, precision, y, c, x, bw[l], bd[l], base, base + (size_t)B * 6 * C, bws));
    }
    // ---- output layer: LN(eps 1e-5), chunk 0 = scale, chunk 1 = shift, projection, tokens -> pixels (modules.cpp:1721-1752)
    {
        Bump bws(ctx->ws, ctx->ws_bytes);
        bws.off = block_ws_off;
        void* x_hid = bws.take<char>((size_t)B * Tx * C * (bf ? 2 : 4));
        SD3_TRY(ln_mod(ctx, x, x_hid, nullptr, ada_out + C, ada_out, nullptr, nullptr, 2 * C, 1e-5f, B, Tx, C, bf));
        GemmEpilogueArgs none;
        SD3_TRY(linear_layer(ctx, precision, x_hid, out_w, out_b, tokens, 1, PPC, B * Tx, PPC, C, EPI_BIAS, none));
        if (step) SD3_TRY(unpatchify_cfg_euler(tokens, latent, out, B / 2, C_in, H, W, p, step->guidance, step->dsigma, st));
        else SD3_TRY(unpatchify(tokens, out, B, C_in, H, W, p, st));
    }
    return SD3_OK;
}

int sd3_dit_forward(sd3_ctx* ctx, const float* pooled, const float* captions, const float* latent, const float* timesteps, float* out, int B, int Tc,
                    int H, int W, int num_layers, const int* dual_attention_layers, int n_dual, int pooled_dim, int captions_dim, int C_in, int emb_dim,
                    int attn_heads, int mlp_expand, int patch_size, int pos_embed_max_size, int base_height, int use_qk_norm, int precision) {
    return dit_forward_impl(ctx, pooled, captions, latent, timesteps, out, B, Tc, H, W, num_layers, dual_attention_layers, n_dual, pooled_dim, captions_dim,
                            C_in, emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm, precision, nullptr);
}

int sd3_dit_forward_cfg_euler(sd3_ctx* ctx, const float* pooled, const float* captions, const float* latent, const float* timesteps, float* latent_out,
                              int B, int Tc, int H, int W, int num_layers, const int* dual_attention_layers, int n_dual, int pooled_dim, int captions_dim,
                              int C_in, int emb_dim, int attn_heads, int mlp_expand, int patch_size, int pos_embed_max_size, int base_height,
                              int use_qk_norm, int precision, float guidance, float dsigma) {
    SD3_REQUIRE(B >= 2 && B % 2 == 0, "DiT guidance step: the batch holds [unconditional ; conditional] halves, so B must be even (got %d)", B);
    const CfgEulerStep step{guidance, dsigma};
    return dit_forward_impl(ctx, pooled, captions, latent, timesteps, latent_out, B, Tc, H, W, num_layers, dual_attention_layers, n_dual, pooled_dim,
                            captions_dim, C_in, emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm, precision, &step);
}

// ------------------------------------------------------------------ bf16 kernels on their own
int sd3_flash_attention_bf16(const void* qkv0, const void* qkv1, void* out0, void* out1, const float* rms_q0, const float* rms_k0, const float* rms_q1,
                             const float* rms_k1, int B, int T0, int T1, int num_heads, int head_dim, void* stream) {
    SD3_REQUIRE(B >= 0 && T0 >= 0 && T1 >= 0 && num_heads > 0 && head_dim > 0, "flash_attention_bf16: bad sizes");
    if (B == 0 || T0 + T1 == 0) return SD3_OK;
    const int C = num_heads * head_dim;
    AttnSegments a{};
    const void* qkv[2] = {qkv0, qkv1};
    void* outs[2] = {out0, out1};
    const float* rq[2] = {rms_q0, rms_q1};
    const float* rk[2] = {rms_k0, rms_k1};
    const int T[2] = {T0, T1};
    for (int i = 0; i < 2; i++) {
        if (T[i] > 0) SD3_REQUIRE(qkv[i] != nullptr, "flash_attention_bf16: null qkv buffer for segment %d", i);
        a.q[i] = qkv[i];
        a.k[i] = qkv[i] ? (const char*)qkv[i] + (size_t)C * 2 : nullptr;
        a.v[i] = qkv[i] ? (const char*)qkv[i] + (size_t)2 * C * 2 : nullptr;
        a.out[i] = outs[i];
        a.ld_qkv[i] = 3 * C; a.ld_out[i] = C;
        a.T[i] = a.Tq[i] = T[i];
        a.rms_q[i] = rq[i]; a.rms_k[i] = rk[i];
    }
    return attention_bf16(a, B, num_heads, head_dim, ST(stream));
}
int sd3_flash_attention_bf16_split(const void* qkv0, const void* qkv1, void* out0, void* out1, int B, int T0, int T1, int num_heads, int head_dim,
                                   int kv_splits, void* workspace, long long workspace_bytes, void* stream) {
    SD3_REQUIRE(B >= 0 && T0 > 0 && T1 > 0 && num_heads > 0 && head_dim > 0 && kv_splits >= 2, "flash_attention_bf16_split: bad sizes");
    if (B == 0) return SD3_OK;
    NOTNULL(qkv0); NOTNULL(qkv1); NOTNULL(out0); NOTNULL(out1); NOTNULL(workspace);
    const long long need = (long long)attention_bf16_split_workspace_floats(B, num_heads, T0, kv_splits) * (long long)sizeof(float);
    SD3_REQUIRE(workspace_bytes >= need, "flash_attention_bf16_split: the workspace holds %lld bytes, %lld are needed", workspace_bytes, need);
    const int C = num_heads * head_dim;
    AttnSegments joint{};
    const void* qkv[2] = {qkv0, qkv1};
    void* outs[2] = {out0, out1};
    const int T[2] = {T0, T1};
    for (int i = 0; i < 2; i++) {
        joint.q[i] = qkv[i];
        joint.k[i] = (const char*)qkv[i] + (size_t)C * 2;
        joint.v[i] = (const char*)qkv[i] + (size_t)2 * C * 2;
        joint.out[i] = outs[i];
        joint.ld_qkv[i] = 3 * C; joint.ld_out[i] = C;
        joint.T[i] = joint.Tq[i] = T[i];
    }
    AttnSegments sets[2] = {joint, joint};
    sets[0].Tq[0] = 0; sets[0].out[0] = nullptr;  // the segment-1 queries, whole key range
    sets[1].Tq[1] = 0; sets[1].out[1] = nullptr;  // the segment-0 queries, split along the keys
    const int splits[2] = {1, kv_splits};
    float* wsp[2] = {nullptr, (float*)workspace};
    return attention_bf16_multi(sets, splits, wsp, 2, B, num_heads, head_dim, ST(stream));
}
int sd3_pack_weight_bf16(const float* W, void* wpacked, int K, int N, void* stream) {
    SD3_REQUIRE(K > 0 && N > 0, "pack_weight_bf16: bad sizes");
    NOTNULL(W); NOTNULL(wpacked);
    return pack_weight_bf16(W, (bf16_t*)wpacked, K, N, ST(stream));
}
int sd3_gemm_bf16(const void* A, const void* wpacked, const float* bias, void* out, int M, int N, int K, int epilogue, void* stream) {
    SD3_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes");
    SD3_REQUIRE(epilogue == EPI_BIAS || epilogue == EPI_BIAS_GELU, "gemm_bf16: epilogue must be 0 (bias) or 1 (bias+GELU)");
    if (M == 0) return SD3_OK;
    NOTNULL(A); NOTNULL(wpacked); NOTNULL(out);
    GemmEpilogueArgs ea;
    ea.bias = bias;
    return gemm_bf16((const bf16_t*)A, (const bf16_t*)wpacked, out, 0, N, M, N, K, epilogue, ea, ST(stream));
}
int sd3_gemm_bf16_grouped(const sd3_gemm_bf16_problem* problems, int n_problems, int epilogue, int out_is_f32, void* stream) {
    NOTNULL(problems);
    SD3_REQUIRE(n_problems >= 1 && n_problems <= 3, "gemm_bf16_grouped: 1 to 3 problems per launch (got %d)", n_problems);
    SD3_REQUIRE(epilogue >= EPI_BIAS && epilogue <= EPI_QKV_NORM, "gemm_bf16_grouped: unknown epilogue %d", epilogue);
    GemmBf16Problem probs[3];
    for (int i = 0; i < n_problems; i++) {
        const sd3_gemm_bf16_problem& q = problems[i];
        SD3_REQUIRE(q.M >= 0 && q.N > 0 && q.K > 0, "gemm_bf16_grouped: bad sizes in problem %d (M=%d N=%d K=%d)", i, q.M, q.N, q.K);
        if (q.M > 0) SD3_REQUIRE(q.A && q.wpacked && q.out, "gemm_bf16_grouped: null operand in problem %d", i);
        GemmEpilogueArgs ea;
        ea.bias = q.bias;
        ea.rows_per_batch = q.rows_per_batch > 0 ? q.rows_per_batch : 1;
        if (epilogue == EPI_GATE_RESID) {
            if (q.M > 0) SD3_REQUIRE(q.gate && q.resid && q.gate_ld >= q.N, "gemm_bf16_grouped: the gated epilogue needs gate (row stride >= N) and resid in problem %d", i);
            SD3_REQUIRE(out_is_f32, "gemm_bf16_grouped: the gated epilogue updates an fp32 residual stream (out_is_f32 must be 1)");
            ea.gate = q.gate; ea.gate_ld = q.gate_ld; ea.resid = q.resid;
        } else if (epilogue == EPI_BIAS_ROWADD) {
            if (q.M > 0) SD3_REQUIRE(q.table, "gemm_bf16_grouped: the row-table epilogue needs a table in problem %d", i);
            ea.table = q.table;
        } else if (epilogue == EPI_QKV_NORM) {
            ea.gate = q.rms_q; ea.resid = q.rms_k;  // (checked by the launcher: both present, 16-byte aligned, N = 3C with C % 64 == 0)
        }
        probs[i] = GemmBf16Problem{(const bf16_t*)q.A, (const bf16_t*)q.wpacked, q.out, q.N, q.M, q.N, q.K, ea};
    }
    return gemm_bf16_grouped(probs, n_problems, out_is_f32, epilogue, ST(stream));
}
int sd3_quantize_weight_fp8(const float* W, void* wq, float* w_scale, int K, int N, int per_tensor, void* stream) {
    SD3_REQUIRE(K > 0 && N > 0, "quantize_weight_fp8: bad sizes");
    NOTNULL(W); NOTNULL(wq); NOTNULL(w_scale);
    return quantize_weight_fp8(W, (uint8_t*)wq, w_scale, K, N, per_tensor != 0, ST(stream));
}
int sd3_quantize_rows_fp8(const void* A, void* aq, float* a_scale, int M, int K, int per_tensor, void* stream) {
    SD3_REQUIRE(M >= 0 && K > 0, "quantize_rows_fp8: bad sizes");
    if (M == 0) return SD3_OK;
    NOTNULL(A); NOTNULL(aq); NOTNULL(a_scale);
    return quantize_rows_fp8((const bf16_t*)A, (uint8_t*)aq, a_scale, M, K, per_tensor != 0, ST(stream));
}
int sd3_gemm_fp8(const void* aq, const float* a_scale, const void* wq, const float* w_scale, const float* bias, void* out, int M, int N, int K, int epilogue,
                 int out_is_f32, void* stream) {
    SD3_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_fp8: bad sizes");
    SD3_REQUIRE(epilogue == EPI_BIAS || epilogue == EPI_BIAS_GELU, "gemm_fp8: epilogue must be 0 (bias) or 1 (bias+GELU)");
    if (M == 0) return SD3_OK;
    NOTNULL(aq); NOTNULL(wq); NOTNULL(out);
    GemmBf16Problem q{(const bf16_t*)aq, (const bf16_t*)wq, out, N, M, N, K, GemmEpilogueArgs{}};
    q.ea.bias = bias; q.ea.a_scale = a_scale; q.ea.w_scale = w_scale;
    return gemm_fp8_grouped(&q, 1, out_is_f32, epilogue, ST(stream));
}
int sd3_tune(const char* name, int value) {
    NOTNULL(name);
    if (!std::strcmp(name, "gemm_bf16_tile")) return sd3_gemm_bf16_force_tile(value);
    if (!std::strcmp(name, "gemm_bf16_row_split")) {
        g_gemm_bf16_row_split = value != 0;
        return SD3_OK;
    }
    if (!std::strcmp(name, "attention_context_splits")) {
        SD3_REQUIRE(value >= -1 && value != 1 && value <= 8, "sd3_tune(%s): -1 (automatic), 0 (off) or 2..8 (got %d)", name, value);
        g_attention_context_splits = value;
        return SD3_OK;
    }
    return fail(SD3_ERR_INVALID_ARG, "sd3_tune: unknown setting '%s'", name);
}
int sd3_cast_f32_to_bf16(const float* in, void* out, long long n, void* stream) {
    SD3_REQUIRE(n >= 0, "cast: negative size");
    if (n == 0) return SD3_OK;
    NOTNULL(in); NOTNULL(out);
    return cast_f32_to_bf16(in, (bf16_t*)out, n, ST(stream));
}

}  // extern "C"
