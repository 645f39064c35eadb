/* TEST INFRASTRUCTURE ONLY -- a single-threaded fp32 CPU restatement of the forward path of
 * MichelHUANGGit/SD3.c `modules.cpp`. It exists to check the HIP library and to be timed as the CPU
 * baseline. Nothing under the shipped package may include, link or load it.
 *
 * Every function keeps the reference's evaluation order (same loop nest, same accumulator start
 * value, same float/double promotions) so that its results equal the compiled reference bit for bit
 * on the same libm; tests/test_oracle_vs_reference.py checks that wherever oracle/_ref is built, and
 * tests/golden/ holds vectors written from the compiled reference for everywhere else.
 *
 * Pinning status (what fixes each function besides the compiled reference):
 *   orc_layernorm            torch.nn.functional.layer_norm; rows have mean 0 / variance 1
 *   orc_rmsnorm_heads        torch.nn.functional.rms_norm on the (rows, HS) view
 *   orc_gelu_tanh, orc_silu  torch gelu(approximate="tanh"), silu
 *   orc_gelu                 torch gelu(approximate="none") (what module_tests/gelu.py:28 compares with); float64 closed form
 *   orc_linear, orc_partial_linear   x @ W + b in float64
 *   orc_attention            float64 softmax(QK^T/sqrt(HS))V; key-permutation invariance; ones-V
 *   orc_timestep_embedding   closed form cos/sin(t * 10000^(-i/128)) in float64
 *   orc_pos_embed_table/crop closed form in float64 incl. the axis order of modules.cpp:957
 *   orc_conv2d               torch.nn.functional.conv2d
 *   orc_modulate, orc_gate   affine closed forms
 *   orc_dit_block            float64 numpy block written from the op list; zero-gate identity;
 *                            golden vectors from the compiled reference
 *   orc_dit_forward          golden vectors from the compiled reference; un-patchify index identity
 * No function is "parity unpinned".
 */
#ifndef SD3_ORACLE_H
#define SD3_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_ACT_SILU = 0, ORC_ACT_GELU_TANH = 1 };

/* modules.cpp:10-49 with all four optional pointers null. rows = B*T. */
void orc_layernorm(const float* x, float* y, float eps, long rows, int C);
/* modules.cpp:154-198 (rmsnorm_group, in place): rows = B*T*heads, each of HS values, shared weight w[HS] (may be null). */
void orc_rmsnorm_heads(float* x, const float* w, float eps, long rows, int HS);
/* modules.cpp:293-300 */
void orc_gelu_tanh(const float* in, float* out, long n);
/* modules.cpp:280-285: 0.5 x (1 + erf(x / sqrt 2)), what the extension binds as `gelu` (modules.cpp:1795); not used by the forward path */
void orc_gelu(const float* in, float* out, long n);
/* modules.cpp:352-358 */
void orc_silu(const float* in, float* out, long n);
/* modules.cpp:475-490: y(M,N) = x(M,K) @ W(K,N) + b(N) */
void orc_linear(const float* x, const float* W, const float* b, float* y, int M, int K, int N);
/* modules.cpp:492-511: y(M,N) = x(M,K) @ W[:, n0:n0+N] + b[n0:n0+N], W is (K,Nmax) */
void orc_partial_linear(const float* x, const float* W, const float* b, float* y, int M, int K, int N, int Nmax, int n0);
/* modules.cpp:513-518 */
void orc_add(const float* a, const float* b, float* out, long n);
/* modules.cpp:1207-1221: out = in*(1+scale[b,:]) + shift[b,:]  (argument order shift, scale as in the reference) */
void orc_modulate(const float* in, float* out, const float* shift, const float* scale, int B, int T, int C);
/* modules.cpp:1223-1236 */
void orc_gate(const float* in, float* out, const float* gate, int B, int T, int C);
/* modules.cpp:1239-1294 */
void orc_concat_tokens(const float* a, const float* b, float* out, int B, int Ta, int Tb, int C);
void orc_split_tokens(const float* in, float* a, float* b, int B, int Ta, int Tb, int C);
/* modules.cpp:766-831; out may alias Q */
void orc_attention(const float* Q, const float* K, const float* V, float* out, int B, int NH, int T, int L, int HS);
/* modules.cpp:920-944 */
void orc_timestep_embedding(const float* t, float* out, int B, int dim);
/* modules.cpp:946-975 and 977-995 */
void orc_pos_embed_table(float* out, int C, int height, int width, int base_size);
void orc_pos_embed_crop(const float* table, float* out, int max_size, int h, int w, int C);
/* modules.cpp:1037-1062; `out` must be zero on entry, as the reference requires (modules.cpp:1015) */
void orc_conv2d(const float* in, float* out, const float* kernel, const float* bias, int B, int kh, int kw, int Cin, int Cout, int ih, int iw,
                int oh, int ow, int stride, int pad);
/* modules.cpp:1093-1117. Deliberate deviation: the conv scratch is cleared first (the reference
 * passes an uninitialised buffer, modules.cpp:1642,1682). */
void orc_patch_embed(const float* latent, float* out, const float* kernel, const float* bias, int B, int H, int W, int Cin, int C, int patch,
                     int pos_max, int base_height);
/* modules.cpp:1120-1127; out may alias x */
void orc_mlp(const float* x, float* out, float* hidden, const float* W1, const float* b1, const float* W2, const float* b2, int M, int Cin,
             int Chid, int Cout, int act);

/* Weights of one block, in the reference's layout (2-D weights are (C_in, C_out) row-major).
 * Field order = argument order of dit_block, modules.cpp:1344-1358. Absent entries are null. */
typedef struct orc_block_weights {
    const float *c_ada_w, *c_ada_b, *c_qkv_w, *c_qkv_b, *c_rms_q, *c_rms_k, *c_out_w, *c_out_b, *c_mlp_w1, *c_mlp_b1, *c_mlp_w2, *c_mlp_b2;
    const float *x_ada_w, *x_ada_b, *x_qkv_w, *x_qkv_b, *x_rms_q, *x_rms_k, *x_out_w, *x_out_b;
    const float *x2_qkv_w, *x2_qkv_b, *x2_rms_q, *x2_rms_k, *x2_out_w, *x2_out_b;
    const float *x_mlp_w1, *x_mlp_b1, *x_mlp_w2, *x_mlp_b2;
} orc_block_weights;

/* modules.cpp:1340-1505; c and x are updated in place. Returns 0, or -1 if out of memory. */
int orc_dit_block(const float* y, float* c, float* x, const orc_block_weights* w, int B, int Tc, int Tx, int C, int NH, int mlp_expand,
                  int use_dual, int use_qk_norm, int discard_context);

typedef struct orc_dit_weights {
    const float *t_w0, *t_b0, *t_w2, *t_b2;       /* timestep_mlp.{0,2} */
    const float *p_w0, *p_b0, *p_w2, *p_b2;       /* pooled_mlp.{0,2} */
    const float *cap_w, *cap_b;                   /* captions_linear */
    const float *patch_w, *patch_b;               /* to_patch.conv (C, C_in, p, p) */
    const float *ada_out_w, *ada_out_b;           /* ada_ln_out.linear (C, 2C) */
    const float *out_w, *out_b;                   /* linear_out (C, p*p*C_in) */
    const orc_block_weights* blocks;              /* num_layers entries */
} orc_dit_weights;

/* modules.cpp:1605-1780. dual_mask[l] != 0 marks a block with the extra image self-attention. */
int orc_dit_forward(const float* pooled, const float* captions, const float* latent, const float* timesteps, float* out,
                    const orc_dit_weights* w, const unsigned char* dual_mask, int B, int Tc, int H, int W, int num_layers, int pooled_dim,
                    int captions_dim, int C_in, int C, int NH, int mlp_expand, int patch, int pos_max, int base_height, int use_qk_norm);

#ifdef __cplusplus
}
#endif
#endif
