/* sd3_hip.h -- C ABI of the MI355X (gfx950) implementation of the SD3.5-medium MMDiT-X denoiser forward.
 *
 * Every entry point replaces one function of MichelHUANGGit/SD3.c `modules.cpp` (cited per declaration) and
 * keeps its argument meaning, tensor layouts and in-place behaviour. Differences that hold everywhere:
 *   - all data pointers are DEVICE pointers (HIP global memory), fp32 unless the name says otherwise;
 *   - a trailing `void* stream` is the hipStream_t to enqueue on (NULL = the default stream); calls are
 *     asynchronous with respect to the host;
 *   - the return value is an sd3_status (0 = ok); the library never calls exit() or abort(). The text of the
 *     last failure on the calling thread is returned by sd3_last_error().
 * Linear weights use the reference's layout: (C_in, C_out) row-major, i.e. the transposed PyTorch weight
 * (module_tests/DiT.py:26-31).
 */
#ifndef SD3_HIP_H
#define SD3_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

typedef enum sd3_status {
    SD3_OK = 0,
    SD3_ERR_INVALID_ARG = 1,   /* null pointer, non-positive size, C % heads != 0 ... */
    SD3_ERR_MISSING_PARAM = 2, /* a weight the requested configuration needs was not bound */
    SD3_ERR_UNSUPPORTED = 3,   /* shape outside what the kernels handle (e.g. head_dim > 128) */
    SD3_ERR_HIP = 4,           /* a HIP runtime call failed; see sd3_last_error() */
    SD3_ERR_OOM = 5
} sd3_status;

typedef enum sd3_precision {
    SD3_PREC_F32 = 0, /* fp32 storage and fp32 MFMA arithmetic: matches the CPU reference to <= 1e-4 */
    SD3_PREC_BF16 = 1, /* bf16 operands on the MFMA units, fp32 accumulation, fp32 residual stream */
    /* SD3_PREC_BF16 with the two MLP layers of both streams (half of the block's GEMM work) on the fp8 matrix instruction: OCP e4m3
     * operands, fp32 accumulation; activations quantised per token row and weights per output channel ... */
    SD3_PREC_BF16_FP8 = 2,
    /* ... or with one factor per tensor on both sides (coarser; kept for comparison). Neither is the reference's arithmetic nor
     * the benchmark's: they exist to be measured against the same error criterion as SD3_PREC_BF16. */
    SD3_PREC_BF16_FP8_TENSOR = 3
} sd3_precision;

typedef enum sd3_activation { SD3_ACT_SILU = 0, SD3_ACT_GELU_TANH = 1, SD3_ACT_GELU_ERF = 2 } sd3_activation;

typedef struct sd3_ctx sd3_ctx; /* owns: bound weights table, bf16 weight copies, workspace, stream */

const char* sd3_last_error(void);
int sd3_version(void);

/* ------------------------------------------------------------------ primitive operators (modules.cpp L1) */

/* modules.cpp:10 layernorm(x,y,mean,rstd,w,bias,eps,B,T,C). mean/rstd/w/bias may each be NULL, as in the reference. */
int sd3_layernorm(const float* x, float* y, float* mean, float* rstd, const float* w, const float* bias, float eps, int B, int T, int C, void* stream);
/* modules.cpp:154 rmsnorm(x,y,w,rms,eps,B,T,C); x == y allowed. */
int sd3_rmsnorm(const float* x, float* y, const float* w, float* rms, float eps, int B, int T, int C, void* stream);
/* modules.cpp:192 rmsnorm_group: per-(token, group) RMSNorm over C/groups values with a shared weight of C/groups values. */
int sd3_rmsnorm_group(const float* x, float* y, const float* w, float* rms, float eps, int groups, int B, int T, int C, void* stream);
/* modules.cpp:280 gelu(x, y, n): the erf form 0.5 x (1 + erf(x / sqrt 2)), which the reference's extension exports as `gelu`
 * (modules.cpp:1795). Not used by the forward path (the block MLPs use gelu_tanh). */
int sd3_gelu(const float* in, float* out, long long n, void* stream);
/* modules.cpp:293 gelu_tanh(input, output, n). */
int sd3_gelu_tanh(const float* in, float* out, long long n, void* stream);
/* modules.cpp:352 silu(x, y, n). */
int sd3_silu(const float* in, float* out, long long n, void* stream);
/* modules.cpp:475 linear(x,W,b,y,B,C_in,C_out): y = x @ W + b. */
int sd3_linear(const float* x, const float* W, const float* b, float* y, int B, int C_in, int C_out, void* stream);
/* modules.cpp:492 partial_linear(x,W,b,y,M,K,N,Nmax,n0): y = x @ W[:, n0:n0+N] + b[n0:n0+N]. */
int sd3_partial_linear(const float* x, const float* W, const float* b, float* y, int M, int K, int N, int Nmax, int n0, void* stream);
/* modules.cpp:513 add(input, other, output, size). */
int sd3_add(const float* a, const float* b, float* out, long long n, void* stream);
/* modules.cpp:766 multihead_attention(Q,K,V,output,B,num_heads,T,L,head_dim); layouts (B,T,C)/(B,L,C), head h at
 * columns [h*head_dim,(h+1)*head_dim); output may alias Q. head_dim <= 128. */
int sd3_multihead_attention(const float* Q, const float* K, const float* V, float* out, int B, int num_heads, int T, int L, int head_dim, void* stream);
/* modules.cpp:920 sinusoidal_embedding(timesteps, emb_dim): out (B, emb_dim) = [cos | sin]. */
int sd3_sinusoidal_embedding(const float* timesteps, float* out, int B, int emb_dim, void* stream);
/* modules.cpp:946 positional_embedding2D(output, emb_dim, height, width, base_size); table evaluated in fp64. */
int sd3_positional_embedding2D(float* out, int emb_dim, int height, int width, int base_size, void* stream);
/* modules.cpp:977 crop_positional_embedding2D(pos_embed, new_pos_embed, pos_embed_max_size, new_height, new_width, emb_dim). */
int sd3_crop_positional_embedding2D(const float* pos_embed, float* out, int pos_embed_max_size, int new_height, int new_width, int emb_dim, void* stream);
/* modules.cpp:1037 conv2d(...). Unlike the reference, `output` need not be zeroed by the caller. */
int sd3_conv2d(const float* in, float* out, const float* kernel, const float* bias, int B, int kernel_height, int kernel_width, int in_channels,
               int out_channels, int in_height, int in_width, int out_height, int out_width, int stride, int padding, void* stream);
/* modules.cpp:1093 PatchEmbedding(latent, patches, pos_embed_max, pos_embed, output, kernel, bias, B,H,W,C,emb_dim,patch,pos_max,base_height).
 * The three scratch pointers of the reference are not needed: the kernel gathers patches itself and the
 * position table of the requested grid is generated on the device. */
int sd3_patch_embedding(const float* latent, float* out, const float* kernel, const float* bias, int B, int H, int W, int C_in, int emb_dim,
                        int patch_size, int pos_embed_max_size, int base_height, void* stream);
/* modules.cpp:1120 mlp(x, output, h1, W1,b1,W2,b2, B,C_in,C_hid,C_out, activation); the std::function becomes an sd3_activation. */
int sd3_mlp(const float* x, float* out, float* h1, const float* W1, const float* b1, const float* W2, const float* b2, int B, int C_in, int C_hid,
            int C_out, int activation, void* stream);
/* modules.cpp:1207 scale_and_shift(input, output, shift, scale, B,T,C): out = in*(1+scale[b]) + shift[b]. */
int sd3_scale_and_shift(const float* in, float* out, const float* shift, const float* scale, int B, int T, int C, void* stream);
/* modules.cpp:1223 gating_mechanism(input, output, gate, B,T,C). */
int sd3_gating_mechanism(const float* in, float* out, const float* gate, int B, int T, int C, void* stream);
/* modules.cpp:1239 / 1268 concatenate_along_tokens / split_along_tokens. */
int sd3_concatenate_along_tokens(const float* x, const float* y, float* out, int B, int Tx, int Ty, int C, void* stream);
int sd3_split_along_tokens(const float* in, float* split1, float* split2, int B, int T1, int T2, int C, void* stream);

/* ------------------------------------------------------------------ the block with raw pointers (modules.cpp L2) */

/* Weights of one block in the argument order of dit_block (modules.cpp:1344-1358). Absent entries are NULL and are
 * never dereferenced (last block: no context out-projection / MLP; non-dual blocks: no x2_*; no qk-norm: no *_rms_*). */
typedef struct sd3_block_weights {
    const float *c_ada_w, *c_ada_b, *c_qkv_w, *c_qkv_b, *c_rms_q, *c_rms_k, *c_out_w, *c_out_b, *c_mlp_w1, *c_mlp_b1, *c_mlp_w2, *c_mlp_b2;
    const float *x_ada_w, *x_ada_b, *x_qkv_w, *x_qkv_b, *x_rms_q, *x_rms_k, *x_out_w, *x_out_b;
    const float *x2_qkv_w, *x2_qkv_b, *x2_rms_q, *x2_rms_k, *x2_out_w, *x2_out_b;
    const float *x_mlp_w1, *x_mlp_b1, *x_mlp_w2, *x_mlp_b2;
} sd3_block_weights;

/* modules.cpp:1340 dit_block(y, c, x, <30 weights>, <16 scratch>, B,Tc,Tx,emb_dim,attn_heads,mlp_expand,use_dual,use_qk_norm,discard).
 * c and x are updated in place. The reference's 16 caller-owned scratch buffers are replaced by the context's
 * workspace (the fused kernels use differently shaped intermediates). */
int sd3_dit_block_w(sd3_ctx* ctx, const float* y, float* c, float* x, const sd3_block_weights* w, int B, int Tc, int Tx, int emb_dim,
                    int attn_heads, int mlp_expand, int use_dual_attention, int use_qk_norm, int discard_context, int precision);

/* ------------------------------------------------------------------ context, weights by name (modules.cpp L3) */

int sd3_ctx_create(sd3_ctx** out, int device);
int sd3_ctx_destroy(sd3_ctx* ctx);
/* The stream that the context's calls enqueue on from now on (default: the null stream). The new stream is made to wait for
 * the work of the context's earlier calls (they share the workspace and the derived weight copies) through an event the
 * library records behind each call, so the previous stream may already have been destroyed by its owner. A stream must be
 * alive while a call enqueues on it. Under stream capture no event is recorded or waited on: whoever replays a captured
 * graph orders the replays against the context's other work. */
int sd3_ctx_set_stream(sd3_ctx* ctx, void* stream);
int sd3_ctx_synchronize(sd3_ctx* ctx);

/* One entry of the reference's `name -> tensor` parameter map (modules.cpp:1512,1609). `ptr` is borrowed: it must stay
 * valid and unchanged while bound. Names are the reference's (modules.cpp:1558-1575, 1665-1728).
 * The reference's entry points receive the whole map on every call (modules.cpp:1605-1613, 1783-1787); a caller shaped like
 * them keeps one context and binds the map again each time: binding a name to the tensor it is already bound to (same
 * address, same numel) is free and keeps the derived copies; a different address or size drops what was derived from the
 * old tensor and from whatever lived at the new address before. What the library cannot see is a change of CONTENTS at an
 * unchanged address (an in-place update, or memory that was freed and handed out again for another tensor of the same
 * size): then call sd3_weights_forget(ptr) / sd3_weights_unbind(name) for that tensor, or sd3_weights_prepare for all. */
int sd3_weights_bind(sd3_ctx* ctx, const char* name, const float* ptr, long long numel);
/* Removes one name from the map (no error if it is not bound) and drops what was derived from its tensor. */
int sd3_weights_unbind(sd3_ctx* ctx, const char* name);
/* Drops the derived copies made from the tensor at `ptr` (its contents have changed); names stay bound, the copies are built
 * again on next use. Also serves callers of sd3_dit_block_w, whose weights have no names. */
int sd3_weights_forget(sd3_ctx* ctx, const float* ptr);
int sd3_weights_clear(sd3_ctx* ctx);
/* Number of derived weight copies the context has built since it was created (bf16 / fp8 / transposed copies, one per
 * weight and kind): lets a caller or a test see whether a call re-used the existing copies or built new ones. */
int sd3_weights_copies_built(sd3_ctx* ctx, long long* count);
/* Rebuilds, from the current contents of the bound tensors, every derived copy a forward of `precision` uses (bf16: the
 * K-contiguous bf16 copies of the GEMM weights, the bf16 copies of the adaLN weights and of the patch-conv weight; fp32: the
 * transposed patch-conv weight). Optional before a first forward (copies are otherwise built on first use, inside that
 * forward); REQUIRED after changing a bound tensor in place, which the library cannot see. A layer's shape is taken from
 * its bound `.weight` / `.bias` pair. Re-binding a name with sd3_weights_bind drops the copies of the tensor it replaces. */
int sd3_weights_prepare(sd3_ctx* ctx, int precision);

/* modules.cpp:1508 DiT_block_forward / modules.cpp:1783 DiT_block_forward_cuda: the block with weights looked up by
 * name. `prefix` is "" for the single-block entry points and "transformer.<l>." inside the full model. */
int sd3_dit_block(sd3_ctx* ctx, const float* y, float* c, float* x, const char* prefix, int B, int Tc, int Tx, int emb_dim, int attn_heads,
                  int mlp_expand, int use_dual_attention, int use_qk_norm, int discard_context, int precision);

/* No counterpart in the reference. sd3_dit_block for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same arguments, same kernels, same results, but the
 * block's intermediates live in a fixed array of SD3_STATIC_SCRATCH_BYTES that every device the library runs on holds
 * from load until the process ends, and the call makes no hipMalloc / hipFree / event creation. A block whose
 * intermediates need more (the size grows with B*(Tc+Tx)*emb_dim) is refused with SD3_ERR_UNSUPPORTED. With SD3_PREC_BF16
 * the bf16 copies of the block's weights must exist already (sd3_weights_prepare, or one earlier sd3_dit_block call with
 * the same bindings, builds them); otherwise the call returns SD3_ERR_MISSING_PARAM. All calls on one device share the array: calls that
 * overlap in time on one device (two streams, two contexts, two threads) race. */
#define SD3_STATIC_SCRATCH_BYTES (64u << 20)
int sd3_dit_block_static(sd3_ctx* ctx, const float* y, float* c, float* x, const char* prefix, int B, int Tc, int Tx, int emb_dim, int attn_heads,
                         int mlp_expand, int use_dual_attention, int use_qk_norm, int discard_context, int precision);

/* modules.cpp:1605 DiT_forward(pooled_captions, captions, latent_vector, timesteps, params, num_layers, dual_attention_layers,
 * pooled_dim, captions_dim, C_in, emb_dim, attn_heads, mlp_expand, patch_size, pos_embed_max_size, base_height, use_qk_norm).
 * pooled (B,pooled_dim), captions (B,Tc,captions_dim), latent (B,C_in,H,W), timesteps (B); out (B,C_in,H,W). Inputs are
 * left untouched. The std::unordered_set of dual layers becomes an int array. */
int sd3_dit_forward(sd3_ctx* ctx, const float* pooled, const float* captions, const float* latent, const float* timesteps, float* out, int B,
                    int Tc, int H, int W, int num_layers, const int* dual_attention_layers, int n_dual, int pooled_dim, int captions_dim, int C_in,
                    int emb_dim, int attn_heads, int mlp_expand, int patch_size, int pos_embed_max_size, int base_height, int use_qk_norm,
                    int precision);

/* The sampler step around the denoiser, with no counterpart in the reference (which stops at the velocity): the same
 * forward on a batch laid out [B/2 unconditional ; B/2 conditional] samples (both halves of `latent` hold the same B/2
 * latents), with classifier-free guidance and one Euler step of the flow-matching sampler applied where the tokens go
 * back to pixels:  latent_out[i] = latent[i] + dsigma * (v_u[i] + guidance * (v_c[i] - v_u[i])),  i < B/2,
 * dsigma = sigma_next - sigma. latent_out is (B/2, C_in, H, W) and must not alias latent. */
int sd3_dit_forward_cfg_euler(sd3_ctx* ctx, const float* pooled, const float* captions, const float* latent, const float* timesteps, float* latent_out,
                              int B, int Tc, int H, int W, int num_layers, const int* dual_attention_layers, int n_dual, int pooled_dim, int captions_dim,
                              int C_in, int emb_dim, int attn_heads, int mlp_expand, int patch_size, int pos_embed_max_size, int base_height,
                              int use_qk_norm, int precision, float guidance, float dsigma);

/* Per-kernel-class timing (no counterpart in the reference, which has no profiling). Between begin and end every
 * launch made through `ctx` by sd3_dit_block* / sd3_dit_forward is bracketed by two HIP events on the context's stream.
 * sd3_profile_end synchronises and returns, per class, the summed event time in ms, the summed algorithmic work
 * (FLOP for SD3_PROF_GEMM / SD3_PROF_ATTENTION: 2*M*N*K and 4*B*heads*Tq*Tk*head_dim; bytes for the others: each
 * tensor counted once per read and once per write) and the number of launches. Arrays have SD3_PROF_CLASSES entries. */
enum { SD3_PROF_GEMM = 0, SD3_PROF_ATTENTION = 1, SD3_PROF_LAYERNORM = 2, SD3_PROF_ADALN = 3, SD3_PROF_GEMM_FP8 = 4, SD3_PROF_QUANT = 5, SD3_PROF_CLASSES = 6 };
int sd3_profile_begin(sd3_ctx* ctx);
int sd3_profile_end(sd3_ctx* ctx, double* ms, double* work, long long* launches);

/* ------------------------------------------------------------------ bf16 kernels on their own (no counterpart in the reference,
 * whose GPU file is fp32/TF32 only; exposed so that the MFMA kernels can be tested and timed in isolation) */

/* Joint attention over two token segments without concatenation: segment 0 (context, T0 tokens) then segment 1
 * (latent, T1 tokens), each given as a packed bf16 (B*T_s, 3*C) q|k|v buffer as the QKV GEMM writes it. Per-head
 * RMSNorm (eps 1e-6, weights rms_q[s]/rms_k[s] of head_dim floats, or NULL for none) is applied to q and k while
 * they are loaded. Output: bf16 (B*T_s, C) per segment (out[s] may be NULL to skip writing it). head_dim must be 64.
 * This is the fused form of modules.cpp:1396-1399,1420-1432 (rmsnorm_group x4, concatenate x3, attention, split). */
int sd3_flash_attention_bf16(const void* qkv0, const void* qkv1, void* out0, void* out1, const float* rms_q0, const float* rms_k0,
                             const float* rms_q1, const float* rms_k1, int B, int T0, int T1, int num_heads, int head_dim, void* stream);
/* The same joint attention (without the fused norm) taken apart the way the block does it when segment 0 is short and segment 1
 * long: one launch holds the segment-1 queries over all keys and the segment-0 queries as kv_splits work items each, every item
 * over its own run of keys; a second small kernel merges the partial results of the split (sum_s O_s 2^(m_s-M) / sum_s l_s 2^(m_s-M)).
 * workspace: device memory of at least B * num_heads * ceil(T0/256) * kv_splits * 256 * 66 * 4 bytes. Rows of segment 1 come out
 * bit-identical to sd3_flash_attention_bf16, rows of segment 0 equal up to the rounding of the merge. */
int sd3_flash_attention_bf16_split(const void* qkv0, const void* qkv1, void* out0, void* out1, int B, int T0, int T1, int num_heads, int head_dim,
                                   int kv_splits, void* workspace, long long workspace_bytes, void* stream);
/* out(M,N) = A(M,K) @ W + bias with A bf16 row-major, W given in the reference's fp32 (K,N) layout already packed by
 * sd3_pack_weight_bf16 into `wpacked`; out bf16. K % 64 == 0 and N % 8 == 0 required. epilogue: 0 bias, 1 bias+GELU-tanh. */
int sd3_pack_weight_bf16(const float* W, void* wpacked, int K, int N, void* stream);
int sd3_gemm_bf16(const void* A, const void* wpacked, const float* bias, void* out, int M, int N, int K, int epilogue, void* stream);
/* The same kernel with every epilogue the block uses and up to three independent problems per launch (in a block: the latent,
 * dual-branch and context layer of the same kind). epilogue, applied to acc = A @ W (fp32 accumulation):
 *   0  acc + bias                      (modules.cpp:475-490 linear)
 *   1  gelu_tanh(acc + bias)           (modules.cpp:1120-1127 mlp, first half)
 *   2  silu(acc + bias)
 *   3  resid + gate[m / rows_per_batch] * (acc + bias), fp32, out may equal resid
 *                                      (linear + gating_mechanism + add, modules.cpp:1435-1436, 1223-1236, 513-518)
 *   4  acc + bias + table[m % rows_per_batch]      (PatchEmbedding's position table, modules.cpp:1110-1116)
 *   5  N = 3C packed q|k|v: acc + bias, then per-head RMSNorm (64 columns, eps 1e-6) of the q and k thirds with weights
 *      rms_q / rms_k (partial_linear x3 + rmsnorm_group x2, modules.cpp:1391-1399)
 * out is (M, N) row-major, bf16 or (out_is_f32) fp32. Results do not depend on how problems are grouped. */
typedef struct sd3_gemm_bf16_problem {
    const void* A;       /* bf16 (M, K) row-major */
    const void* wpacked; /* from sd3_pack_weight_bf16 */
    const float* bias;   /* (N) or NULL */
    void* out;
    int M, N, K;
    const float* gate;   /* epilogue 3: (batches, gate_ld) */
    int gate_ld;
    const float* resid;  /* epilogue 3: fp32 (M, N) */
    const float* table;  /* epilogue 4: fp32 (rows_per_batch, N) */
    int rows_per_batch;  /* epilogues 3 and 4 */
    const float* rms_q;  /* epilogue 5: 64 floats each, 16-byte aligned */
    const float* rms_k;
} sd3_gemm_bf16_problem;
int sd3_gemm_bf16_grouped(const sd3_gemm_bf16_problem* problems, int n_problems, int epilogue, int out_is_f32, void* stream);
/* The fp8 form of the same GEMM (OCP e4m3 operands on v_mfma_f32_32x32x64_f8f6f4, fp32 accumulation), with no counterpart in the
 * reference: out = epilogue(a_scale[m] * w_scale[n] * (Aq @ Wq^T) + bias).
 * sd3_quantize_weight_fp8: W fp32 (K,N) in the reference's layout -> wq (N,K) bytes + w_scale (N): w_scale[n] = max_k |W[k][n]| / 448
 * (per_tensor: the same factor, from the whole tensor, for every n). sd3_quantize_rows_fp8: A bf16 (M,K) -> aq (M,K) bytes +
 * a_scale (M), one factor per row (per_tensor: one for all rows). K % 128 == 0. epilogue: 0 bias, 1 bias+GELU-tanh. */
int sd3_quantize_weight_fp8(const float* W, void* wq, float* w_scale, int K, int N, int per_tensor, void* stream);
int sd3_quantize_rows_fp8(const void* A, void* aq, float* a_scale, int M, int K, int per_tensor, void* stream);
int sd3_gemm_fp8(const void* aq, const float* a_scale, const void* wq, const float* w_scale, const float* bias, void* out, int M, int N, int K, int epilogue,
                 int out_is_f32, void* stream);
/* fp32 -> bf16 (round to nearest even) */
int sd3_cast_f32_to_bf16(const float* in, void* out, long long n, void* stream);
/* Tuning hook with no counterpart in the reference: forces the output tile of the bf16 GEMM for every later call in this
 * process. tile = 0: chosen per call from the problem sizes (the default); 128: 128x128 tiles, two workgroups per compute
 * unit; 256: 256x256 tiles, one workgroup per compute unit; 192: 256x192 tiles (not with the fused qk-norm epilogue). Results do
 * not depend on the choice. */
int sd3_gemm_bf16_force_tile(int tile);
/* Process-wide tuning switches by name (no counterpart in the reference); results never depend on them. "gemm_bf16_tile": as
 * sd3_gemm_bf16_force_tile; "attention_context_splits": -1 chosen from the sizes (default), 0 never, 2..8 that many key splits for
 * the context queries of a block's joint attention wherever splitting applies (results of those rows change in the last bf16 bit
 * with the number of splits); "gemm_bf16_row_split": 0 / 1 (default), whether a many-row problem that leaves a partial round of
 * 256x256 tiles may send its last rows to a second launch of 128x128 tiles. Unknown names return SD3_ERR_INVALID_ARG. */
int sd3_tune(const char* name, int value);
/* Measurement aid with no counterpart in the reference: the rate (in TFLOP/s) at which the device's matrix cores run the
 * bf16 instruction the GEMM and attention kernels are built on when every wavefront issues it back to back on operands held
 * in registers (no memory or LDS traffic), with all-zero operands (random_operands = 0) or random ones (1). The two differ
 * widely because the device keeps its power limit by lowering the clock; the second figure is the ceiling for a kernel that
 * works on real data. Runs on the current device's default stream, allocates a small buffer for the duration of the call,
 * and returns after `iters` iterations of 8 instructions per wavefront (40000 take about 15 ms). */
int sd3_probe_mfma_bf16(int random_operands, int iters, double* tflops);

#ifdef __cplusplus
}
#endif
#endif /* SD3_HIP_H */
