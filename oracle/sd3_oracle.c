/* TEST INFRASTRUCTURE ONLY -- see sd3_oracle.h. Single-threaded fp32 CPU restatement of the forward
 * path of MichelHUANGGit/SD3.c modules.cpp, kept in the reference's evaluation order.
 * Build: gcc -O2 -std=c99 -ffp-contract=off (no fast-math, no FMA contraction). */
#define _GNU_SOURCE
#include "sd3_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* 1/pi rounded to float: the constant M_1_PIf32 that modules.cpp:289 uses. */
static const float ORC_INV_PI_F = 0.318309886183790671537767526745028724f;

/* modules.cpp:10-49 */
void orc_layernorm(const float* x, float* y, float eps, long rows, int C) {
    for (long r = 0; r < rows; r++) {
        const float* xr = x + r * (long)C;
        float* yr = y + r * (long)C;
        float mu = 0.0f;
        for (int i = 0; i < C; i++) mu += xr[i];
        mu /= C;
        float var = 0.0f;
        for (int i = 0; i < C; i++) {
            float d = xr[i] - mu;
            var += d * d;
        }
        var /= C;
        float rstd = 1.0f / sqrtf(var + eps);
        for (int i = 0; i < C; i++) yr[i] = rstd * (xr[i] - mu);
    }
}

/* modules.cpp:154-198, the in-place branch: x *= r, then x *= w, as two roundings. */
void orc_rmsnorm_heads(float* x, const float* w, float eps, long rows, int HS) {
    for (long r = 0; r < rows; r++) {
        float* xr = x + r * (long)HS;
        float ss = 0.0f;
        for (int i = 0; i < HS; i++) ss += xr[i] * xr[i];
        ss /= HS;
        float inv = (float)(1.0 / sqrtf(eps + ss)); /* double division, modules.cpp:171 */
        for (int i = 0; i < HS; i++) {
            xr[i] *= inv;
            if (w) xr[i] *= w[i];
        }
    }
}

/* modules.cpp:293-300: the inner polynomial is float, the outer product is evaluated in double. */
void orc_gelu_tanh(const float* in, float* out, long n) {
    const float k = 0.044715f;
    const float p = sqrtf((float)(2.0 * ORC_INV_PI_F));
    for (long i = 0; i < n; i++) {
        float v = in[i];
        float th = tanhf(p * (v + k * v * v * v));
        out[i] = (float)(0.5 * v * (1.0 + th));
    }
}

/* modules.cpp:280-285 (erf form, the extension's `gelu`): the division and erff are float, the outer product is double. */
void orc_gelu(const float* in, float* out, long n) {
    const float sqrt2 = sqrtf(2.0f);
    for (long i = 0; i < n; i++) out[i] = (float)(0.5 * in[i] * (1.0 + erff(in[i] / sqrt2)));
}

/* modules.cpp:352-358 */
void orc_silu(const float* in, float* out, long n) {
    for (long i = 0; i < n; i++) {
        float sig = (float)(1.0 / (1.0 + expf(-in[i])));
        out[i] = in[i] * sig;
    }
}

/* modules.cpp:475-490: accumulator starts at 0, bias added last. */
void orc_linear(const float* x, const float* W, const float* b, float* y, int M, int K, int N) {
    for (int m = 0; m < M; m++) {
        const float* xm = x + (long)m * K;
        for (int n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int k = 0; k < K; k++) acc += xm[k] * W[(long)k * N + n];
            y[(long)m * N + n] = acc + b[n];
        }
    }
}

/* modules.cpp:492-511: accumulator starts at the bias. */
void orc_partial_linear(const float* x, const float* W, const float* b, float* y, int M, int K, int N, int Nmax, int n0) {
    for (int m = 0; m < M; m++) {
        const float* xm = x + (long)m * K;
        for (int n = 0; n < N; n++) {
            float acc = b[n0 + n];
            for (int k = 0; k < K; k++) acc += xm[k] * W[(long)k * Nmax + n0 + n];
            y[(long)m * N + n] = acc;
        }
    }
}

/* modules.cpp:513-518 */
void orc_add(const float* a, const float* b, float* out, long n) {
    for (long i = 0; i < n; i++) out[i] = a[i] + b[i];
}

/* modules.cpp:1207-1221 */
void orc_modulate(const float* in, float* out, const float* shift, const float* scale, int B, int T, int C) {
    for (int b = 0; b < B; b++)
        for (int t = 0; t < T; t++) {
            long o = ((long)b * T + t) * C;
            for (int i = 0; i < C; i++) out[o + i] = in[o + i] * (1.0f + scale[(long)b * C + i]) + shift[(long)b * C + i];
        }
}

/* modules.cpp:1223-1236 */
void orc_gate(const float* in, float* out, const float* gate, int B, int T, int C) {
    for (int b = 0; b < B; b++)
        for (int t = 0; t < T; t++) {
            long o = ((long)b * T + t) * C;
            for (int i = 0; i < C; i++) out[o + i] = in[o + i] * gate[(long)b * C + i];
        }
}

/* modules.cpp:1239-1266 */
void orc_concat_tokens(const float* a, const float* b, float* out, int B, int Ta, int Tb, int C) {
    for (int s = 0; s < B; s++) {
        float* o = out + (long)s * (Ta + Tb) * C;
        memcpy(o, a + (long)s * Ta * C, sizeof(float) * (size_t)Ta * C);
        memcpy(o + (long)Ta * C, b + (long)s * Tb * C, sizeof(float) * (size_t)Tb * C);
    }
}

/* modules.cpp:1268-1294 */
void orc_split_tokens(const float* in, float* a, float* b, int B, int Ta, int Tb, int C) {
    for (int s = 0; s < B; s++) {
        const float* i = in + (long)s * (Ta + Tb) * C;
        memcpy(a + (long)s * Ta * C, i, sizeof(float) * (size_t)Ta * C);
        memcpy(b + (long)s * Tb * C, i + (long)Ta * C, sizeof(float) * (size_t)Tb * C);
    }
}

/* modules.cpp:766-831: one score row at a time; normalise the row, then row @ V. */
void orc_attention(const float* Q, const float* K, const float* V, float* out, int B, int NH, int T, int L, int HS) {
    float* row = (float*)malloc(sizeof(float) * (size_t)L);
    const float scale = (float)(1.0 / sqrtf((float)HS));
    const long C = (long)NH * HS;
    for (int b = 0; b < B; b++)
        for (int h = 0; h < NH; h++)
            for (int t = 0; t < T; t++) {
                const float* q = Q + ((long)b * T + t) * C + (long)h * HS;
                float mx = -INFINITY;
                for (int l = 0; l < L; l++) {
                    const float* k = K + ((long)b * L + l) * C + (long)h * HS;
                    float dot = 0.0f;
                    for (int d = 0; d < HS; d++) dot += q[d] * k[d];
                    dot *= scale;
                    row[l] = dot;
                    mx = (mx < dot) ? dot : mx;
                }
                float sum = 0.0f;
                for (int l = 0; l < L; l++) {
                    row[l] = expf(row[l] - mx);
                    sum += row[l];
                }
                for (int l = 0; l < L; l++) row[l] /= sum;
                float* o = out + ((long)b * T + t) * C + (long)h * HS;
                for (int d = 0; d < HS; d++) {
                    const float* v = V + (long)b * L * C + (long)h * HS + d;
                    float acc = 0.0f;
                    for (int l = 0; l < L; l++) acc += row[l] * v[(long)l * C];
                    o[d] = acc;
                }
            }
    free(row);
}

/* modules.cpp:920-944: cos half first, then sin half; all float arithmetic. */
void orc_timestep_embedding(const float* t, float* out, int B, int dim) {
    const float ln1e4 = logf(10000.0f);
    const int half = dim / 2;
    for (int b = 0; b < B; b++)
        for (int i = 0; i < half; i++) {
            float freq = expf(-ln1e4 * 2 * i / dim);
            out[(long)b * dim + i] = cosf(freq * t[b]);
            out[(long)b * dim + half + i] = sinf(freq * t[b]);
        }
}

/* modules.cpp:946-975: evaluated in double, width is the slow index of the stored table. */
void orc_pos_embed_table(float* out, int C, int height, int width, int base_size) {
    const int q = C / 4;
    for (int wi = 0; wi < width; wi++) {
        double pw = (double)(wi * base_size) / width;
        for (int hi = 0; hi < height; hi++) {
            double ph = (double)(hi * base_size) / height;
            float* e = out + ((long)wi * height + hi) * C;
            for (int i = 0; i < q; i++) {
                double freq = 1.0 / pow(10000.0f, (double)4 * i / C);
                e[i] = (float)sin(ph * freq);
                e[q + i] = (float)cos(ph * freq);
                e[2 * q + i] = (float)sin(pw * freq);
                e[3 * q + i] = (float)cos(pw * freq);
            }
        }
    }
}

/* modules.cpp:977-995: centre crop of the (max,max,C) table read as [row][col]. */
void orc_pos_embed_crop(const float* table, float* out, int max_size, int h, int w, int C) {
    const int oh = (max_size - h) / 2, ow = (max_size - w) / 2;
    for (int i = 0; i < h; i++)
        for (int j = 0; j < w; j++)
            memcpy(out + ((long)i * w + j) * C, table + ((long)(i + oh) * max_size + (j + ow)) * C, sizeof(float) * (size_t)C);
}

/* modules.cpp:1011-1062: per (b, out channel): for each input channel add a single-channel 2-D
 * correlation into the output plane, then add the bias. */
void orc_conv2d(const float* in, float* out, const float* kernel, const float* bias, int B, int kh, int kw, int Cin, int Cout, int ih, int iw,
                int oh, int ow, int stride, int pad) {
    for (int b = 0; b < B; b++)
        for (int oc = 0; oc < Cout; oc++) {
            float* plane = out + ((long)b * Cout + oc) * oh * ow;
            for (int ic = 0; ic < Cin; ic++) {
                const float* src = in + ((long)b * Cin + ic) * ih * iw;
                const float* ker = kernel + ((long)oc * Cin + ic) * kh * kw;
                for (int y = 0; y < oh; y++)
                    for (int x = 0; x < ow; x++) {
                        float acc = 0.0f;
                        for (int r = 0; r < kh; r++)
                            for (int s = 0; s < kw; s++) {
                                int yy = y * stride + r - pad, xx = x * stride + s - pad;
                                if (yy >= 0 && yy < ih && xx >= 0 && xx < iw) acc += ker[r * kw + s] * src[(long)yy * iw + xx];
                            }
                        plane[(long)y * ow + x] += acc;
                    }
            }
            for (long i = 0; i < (long)oh * ow; i++) plane[i] += bias[oc];
        }
}

/* modules.cpp:1093-1117 */
void orc_patch_embed(const float* latent, float* out, const float* kernel, const float* bias, int B, int H, int W, int Cin, int C, int patch,
                     int pos_max, int base_height) {
    const int h = (H - patch) / patch + 1, w = (W - patch) / patch + 1;
    const long Tx = (long)h * w;
    float* planes = (float*)calloc((size_t)B * C * Tx, sizeof(float));
    float* table = (float*)malloc(sizeof(float) * (size_t)pos_max * pos_max * C);
    float* pos = (float*)malloc(sizeof(float) * (size_t)Tx * C);
    orc_conv2d(latent, planes, kernel, bias, B, patch, patch, Cin, C, H, W, h, w, patch, 0);
    orc_pos_embed_table(table, C, pos_max, pos_max, base_height / patch);
    orc_pos_embed_crop(table, pos, pos_max, h, w, C);
    for (int b = 0; b < B; b++)
        for (long t = 0; t < Tx; t++)
            for (int d = 0; d < C; d++) out[((long)b * Tx + t) * C + d] = planes[((long)b * C + d) * Tx + t] + pos[t * C + d];
    free(planes);
    free(table);
    free(pos);
}

/* modules.cpp:1120-1127 */
void orc_mlp(const float* x, float* out, float* hidden, const float* W1, const float* b1, const float* W2, const float* b2, int M, int Cin,
             int Chid, int Cout, int act) {
    orc_linear(x, W1, b1, hidden, M, Cin, Chid);
    if (act == ORC_ACT_SILU) orc_silu(hidden, hidden, (long)M * Chid);
    else orc_gelu_tanh(hidden, hidden, (long)M * Chid);
    orc_linear(hidden, W2, b2, out, M, Chid, Cout);
}

/* One adaLN chunk: y(B,C) @ W[:, k*C:(k+1)*C] + b -- how the reference gets every modulation vector. */
static void ada_chunk(const float* y, const float* W, const float* b, float* out, int B, int C, int chunks, int k) {
    orc_partial_linear(y, W, b, out, B, C, C, chunks * C, k * C);
}

/* q,k,v = column thirds of one (C,3C) projection, then the per-head RMSNorm of q and k. */
static void qkv_project(const float* in, const float* W, const float* b, const float* rq, const float* rk, float* q, float* k, float* v, long M,
                        int C, int NH, int use_qk_norm) {
    orc_partial_linear(in, W, b, q, (int)M, C, C, 3 * C, 0);
    orc_partial_linear(in, W, b, k, (int)M, C, C, 3 * C, C);
    orc_partial_linear(in, W, b, v, (int)M, C, C, 3 * C, 2 * C);
    if (use_qk_norm) {
        orc_rmsnorm_heads(q, rq, 1e-6f, M * NH, C / NH);
        orc_rmsnorm_heads(k, rk, 1e-6f, M * NH, C / NH);
    }
}

/* modules.cpp:1340-1505 */
int orc_dit_block(const float* y, float* c, float* x, const orc_block_weights* w, int B, int Tc, int Tx, int C, int NH, int mlp_expand,
                  int use_dual, int use_qk_norm, int discard_context) {
    const int T = Tc + Tx, HS = C / NH;
    const int cch = discard_context ? 2 : 6, xch = use_dual ? 9 : 6;
    const long nc = (long)B * Tc * C, nx = (long)B * Tx * C, nt = (long)B * T * C;
    const size_t total = (size_t)(4 * nc + 5 * nx + 3 * nt + 2 * (long)B * C) + (size_t)B * T * mlp_expand * C;
    float* pool = (float*)malloc(sizeof(float) * total);
    if (!pool) return -1;
    float* p = pool;
    float *c_hid = p; p += nc;
    float *cq = p; p += nc;
    float *ck = p; p += nc;
    float *cv = p; p += nc;
    float *x_hid = p; p += nx;
    float *x_dual = p; p += nx;
    float *xq = p; p += nx;
    float *xk = p; p += nx;
    float *xv = p; p += nx;
    float *Q = p; p += nt;
    float *K = p; p += nt;
    float *V = p; p += nt;
    float *m1 = p; p += (long)B * C;
    float *m2 = p; p += (long)B * C;
    float *c_mlp = p; p += (long)B * Tc * mlp_expand * C;
    float *x_mlp = p;

    /* context stream before attention (modules.cpp:1381-1399); with discard_context the two chunks are (scale, shift) */
    orc_layernorm(c, c_hid, 1e-6f, (long)B * Tc, C);
    ada_chunk(y, w->c_ada_w, w->c_ada_b, m1, B, C, cch, 0);
    ada_chunk(y, w->c_ada_w, w->c_ada_b, m2, B, C, cch, 1);
    if (discard_context) orc_modulate(c_hid, c_hid, m2, m1, B, Tc, C);
    else orc_modulate(c_hid, c_hid, m1, m2, B, Tc, C);
    qkv_project(c_hid, w->c_qkv_w, w->c_qkv_b, w->c_rms_q, w->c_rms_k, cq, ck, cv, (long)B * Tc, C, NH, use_qk_norm);

    /* latent stream before attention (modules.cpp:1402-1423) */
    orc_layernorm(x, x_hid, 1e-6f, (long)B * Tx, C);
    if (use_dual) {
        ada_chunk(y, w->x_ada_w, w->x_ada_b, m1, B, C, xch, 6);
        ada_chunk(y, w->x_ada_w, w->x_ada_b, m2, B, C, xch, 7);
        orc_modulate(x_hid, x_dual, m1, m2, B, Tx, C);
    }
    ada_chunk(y, w->x_ada_w, w->x_ada_b, m1, B, C, xch, 0);
    ada_chunk(y, w->x_ada_w, w->x_ada_b, m2, B, C, xch, 1);
    orc_modulate(x_hid, x_hid, m1, m2, B, Tx, C);
    qkv_project(x_hid, w->x_qkv_w, w->x_qkv_b, w->x_rms_q, w->x_rms_k, xq, xk, xv, (long)B * Tx, C, NH, use_qk_norm);

    /* joint attention, context tokens first (modules.cpp:1427-1436) */
    orc_concat_tokens(cq, xq, Q, B, Tc, Tx, C);
    orc_concat_tokens(ck, xk, K, B, Tc, Tx, C);
    orc_concat_tokens(cv, xv, V, B, Tc, Tx, C);
    orc_attention(Q, K, V, Q, B, NH, T, T, HS);
    orc_split_tokens(Q, cq, xq, B, Tc, Tx, C);
    if (!discard_context) orc_linear(cq, w->c_out_w, w->c_out_b, c_hid, B * Tc, C, C);
    orc_linear(xq, w->x_out_w, w->x_out_b, x_hid, B * Tx, C, C);

    /* extra self-attention over image tokens (modules.cpp:1440-1453) */
    if (use_dual) {
        qkv_project(x_dual, w->x2_qkv_w, w->x2_qkv_b, w->x2_rms_q, w->x2_rms_k, xq, xk, xv, (long)B * Tx, C, NH, use_qk_norm);
        orc_attention(xq, xk, xv, xq, B, NH, Tx, Tx, HS);
        orc_linear(xq, w->x2_out_w, w->x2_out_b, x_dual, B * Tx, C, C);
        ada_chunk(y, w->x_ada_w, w->x_ada_b, m1, B, C, xch, 8);
        orc_gate(x_dual, x_dual, m1, B, Tx, C);
    }

    /* context residual + MLP (modules.cpp:1457-1477) */
    if (!discard_context) {
        ada_chunk(y, w->c_ada_w, w->c_ada_b, m1, B, C, cch, 2);
        orc_gate(c_hid, c_hid, m1, B, Tc, C);
        orc_add(c_hid, c, c, nc);
        orc_layernorm(c, c_hid, 1e-6f, (long)B * Tc, C);
        ada_chunk(y, w->c_ada_w, w->c_ada_b, m1, B, C, cch, 3);
        ada_chunk(y, w->c_ada_w, w->c_ada_b, m2, B, C, cch, 4);
        orc_modulate(c_hid, c_hid, m1, m2, B, Tc, C);
        orc_mlp(c_hid, c_hid, c_mlp, w->c_mlp_w1, w->c_mlp_b1, w->c_mlp_w2, w->c_mlp_b2, B * Tc, C, mlp_expand * C, C, ORC_ACT_GELU_TANH);
        ada_chunk(y, w->c_ada_w, w->c_ada_b, m1, B, C, cch, 5);
        orc_gate(c_hid, c_hid, m1, B, Tc, C);
        orc_add(c_hid, c, c, nc);
    }

    /* latent residuals (main branch first, then the extra branch) + MLP (modules.cpp:1481-1504) */
    ada_chunk(y, w->x_ada_w, w->x_ada_b, m1, B, C, xch, 2);
    orc_gate(x_hid, x_hid, m1, B, Tx, C);
    orc_add(x_hid, x, x, nx);
    if (use_dual) orc_add(x_dual, x, x, nx);
    orc_layernorm(x, x_hid, 1e-6f, (long)B * Tx, C);
    ada_chunk(y, w->x_ada_w, w->x_ada_b, m1, B, C, xch, 3);
    ada_chunk(y, w->x_ada_w, w->x_ada_b, m2, B, C, xch, 4);
    orc_modulate(x_hid, x_hid, m1, m2, B, Tx, C);
    orc_mlp(x_hid, x_hid, x_mlp, w->x_mlp_w1, w->x_mlp_b1, w->x_mlp_w2, w->x_mlp_b2, B * Tx, C, mlp_expand * C, C, ORC_ACT_GELU_TANH);
    ada_chunk(y, w->x_ada_w, w->x_ada_b, m1, B, C, xch, 5);
    orc_gate(x_hid, x_hid, m1, B, Tx, C);
    orc_add(x_hid, x, x, nx);

    free(pool);
    return 0;
}

/* modules.cpp:1605-1780 */
int orc_dit_forward(const float* pooled, const float* captions, const float* latent, const float* timesteps, float* out,
                    const orc_dit_weights* w, const unsigned char* dual_mask, int B, int Tc, int H, int W, int num_layers, int pooled_dim,
                    int captions_dim, int C_in, int C, int NH, int mlp_expand, int patch, int pos_max, int base_height, int use_qk_norm) {
    const int Hp = (H - patch) / patch + 1, Wp = (W - patch) / patch + 1;
    const long Tx = (long)Hp * Wp;
    const int PPC = patch * patch * C_in;
    float* temb = (float*)malloc(sizeof(float) * (size_t)B * 256);
    float* y = (float*)malloc(sizeof(float) * (size_t)B * C);
    float* pl = (float*)malloc(sizeof(float) * (size_t)B * C);
    float* hid = (float*)malloc(sizeof(float) * (size_t)B * C);
    float* hid2 = (float*)malloc(sizeof(float) * (size_t)B * C);
    float* c = (float*)malloc(sizeof(float) * (size_t)B * Tc * C);
    float* x = (float*)malloc(sizeof(float) * (size_t)B * Tx * C);
    float* xh = (float*)malloc(sizeof(float) * (size_t)B * Tx * C);
    int rc = 0;
    if (!temb || !y || !pl || !hid || !hid2 || !c || !x || !xh) { rc = -1; goto done; }

    /* conditioning vector y = silu(MLP(t_emb) + MLP(pooled)) (modules.cpp:1663-1675) */
    orc_timestep_embedding(timesteps, temb, B, 256);
    orc_mlp(temb, y, hid, w->t_w0, w->t_b0, w->t_w2, w->t_b2, B, 256, C, C, ORC_ACT_SILU);
    orc_mlp(pooled, pl, hid, w->p_w0, w->p_b0, w->p_w2, w->p_b2, B, pooled_dim, C, C, ORC_ACT_SILU);
    orc_add(y, pl, y, (long)B * C);
    orc_silu(y, y, (long)B * C);

    orc_linear(captions, w->cap_w, w->cap_b, c, B * Tc, captions_dim, C);                               /* modules.cpp:1678 */
    orc_patch_embed(latent, x, w->patch_w, w->patch_b, B, H, W, C_in, C, patch, pos_max, base_height);  /* modules.cpp:1682 */

    for (int l = 0; l < num_layers && rc == 0; l++)                                                     /* modules.cpp:1687-1718 */
        rc = orc_dit_block(y, c, x, &w->blocks[l], B, Tc, (int)Tx, C, NH, mlp_expand, dual_mask[l] != 0, use_qk_norm, l == num_layers - 1);
    if (rc) goto done;

    /* final norm (eps 1e-5), chunk 0 = scale, chunk 1 = shift, projection (modules.cpp:1721-1728) */
    orc_layernorm(x, xh, 1e-5f, (long)B * Tx, C);
    ada_chunk(y, w->ada_out_w, w->ada_out_b, hid, B, C, 2, 0);
    ada_chunk(y, w->ada_out_w, w->ada_out_b, hid2, B, C, 2, 1);
    orc_modulate(xh, xh, hid2, hid, B, (int)Tx, C);
    orc_linear(xh, w->out_w, w->out_b, x, B * (int)Tx, C, PPC);

    /* tokens -> pixels: out[b,ch,hp*p+ph,wp*p+pw] = x[b, hp*Wp+wp, (ph*p+pw)*C_in+ch] (modules.cpp:1730-1752) */
    for (int b = 0; b < B; b++)
        for (int ch = 0; ch < C_in; ch++)
            for (int hp = 0; hp < Hp; hp++)
                for (int wp = 0; wp < Wp; wp++)
                    for (int ph = 0; ph < patch; ph++)
                        for (int pw = 0; pw < patch; pw++)
                            out[(((long)b * C_in + ch) * H + hp * patch + ph) * W + wp * patch + pw] =
                                x[((long)b * Tx + (long)hp * Wp + wp) * PPC + (ph * patch + pw) * C_in + ch];
done:
    free(temb); free(y); free(pl); free(hid); free(hid2); free(c); free(x); free(xh);
    return rc;
}
