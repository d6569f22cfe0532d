/* TEST INFRASTRUCTURE -- NOT PRODUCT CODE.
 *
 * CPU restatement of the reference's int8-simulated network forward, used only as the
 * checker for the HIP evaluator (tests, the smoke check and the bench's CPU baseline).
 * Nothing under brokefish_amd/ may link, load or call this file.
 *
 * What it restates (paths inside the reference tree):
 *   board word decode            brokefish/nn/model.py:251-265, docs/reference/spec.md:38-69
 *   control / rep indices        brokefish/nn/model.py:466-473
 *   embedding sum + order        brokefish/nn/model.py:635-640, docs/reference/spec.md:386-391
 *   pre-norm block structure     brokefish/nn/model.py:303-311, :525 (torch TransformerEncoderLayer,
 *                                norm_first, ReLU, key padding mask on dead slots)
 *   activation quantiser         brokefish/nn/quant.py:246-260
 *   weight quantiser             brokefish/nn/quant.py:263-278
 *   int8 linear + descale        brokefish/nn/quant.py:281-305
 *   which matmuls are int8       brokefish/nn/quant.py:421-440, :466-473 (ffn2 unsigned)
 *   final norm + heads           brokefish/nn/model.py:551-617, :644-645
 *   legal-mask AND + argmax      docs/reference/spec.md:141-143, :537-540;
 *                                brokefish/search/torch_impl.py:200-209 (lowest index on ties)
 *
 * Integer arithmetic (operand bytes, int32 accumulators) is exact and has one answer.
 * Floating point has to pick an order of operations wherever the reference defers to a
 * torch library routine (LayerNorm and attention reductions, exp, tanh).  This file
 * fixes those orders explicitly -- they are the orders the HIP kernel uses -- so the
 * kernel can be compared with it bit for bit.  Every fp32 operation here is a single
 * IEEE-754 operation (build with -ffp-contract=off; fused multiply-adds are spelled
 * fmaf).  The torch restatement in oracle/emulated.py uses library reductions instead
 * and agrees with this file to rounding noise; tests/test_oracle.py pins both.
 *
 * Reduction orders fixed here ("lane order"): channels of a 32-wide tile are visited as
 *   ch(r, g) = 8 * (r / 4) + 4 * g + (r % 4),  r = 0..15, g = 0..1
 *   - row sums: two partial sums, one per g; total = part[0] + part[1].  The softmax
 *     denominator accumulates each sequentially over r; LayerNorm mean / variance form each
 *     from four group sums (a quarter of the tiles each, sequential over tiles then r)
 *     added in group order, ((s0 + s1) + s2) + s3
 *   - dot products (QK^T, PV, heads): one fused-multiply-add chain over tiles, then r,
 *     then g, starting from +0
 *
 * Parity status of each function against the reference's own vectors is listed in
 * tests/test_oracle.py; nothing here is "parity unpinned" except where that file says so.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "bf_oracle.h"

#define T 32
#define ROW_K 256   /* brokefish/nn/quant.py:92 */
#define BLOCK_N 128 /* brokefish/nn/quant.py:82 */

static inline int ch(int r, int g) { return 8 * (r / 4) + 4 * g + (r % 4); }

/* ---- scalar functions shared in spirit with the kernel ---------------------- */

/* exp(x) for x <= 0, flushed to 0 below -87.  One rounding per operation. */
float bfo_exp_neg(float x) {
    if (!(x >= -87.0f)) return 0.0f;
    const float t = x * 1.44269504088896341f;
    const float n = rintf(t);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    const float z = r * r;
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float y = fmaf(p, z, r);
    y = y + 1.0f;
    /* multiply by 2^n exactly: n is in [-126, 0] */
    union { float f; int32_t i; } u;
    u.f = y;
    u.i += ((int32_t)n) << 23;
    return u.f;
}

float bfo_tanh(float x) {
    const float a = fabsf(x);
    float th;
    if (a > 9.0f) {
        th = 1.0f;
    } else {
        const float e = bfo_exp_neg(-2.0f * a);
        th = (1.0f - e) / (1.0f + e);
    }
    return copysignf(th, x);
}

/* ---- quantisers -------------------------------------------------------------- */

/* brokefish/nn/quant.py:263-278: one scale per 128 output rows over the whole K. */
void bfo_quantise_weights_int8(const float* w, int n, int k, int8_t* q, float* scale) {
    for (int b = 0; b < n / BLOCK_N; b++) {
        float amax = 0.0f;
        for (int i = 0; i < BLOCK_N * k; i++) amax = fmaxf(amax, fabsf(w[(size_t)b * BLOCK_N * k + i]));
        const float s = amax > 0.0f ? amax / 127.0f : 1.0f;
        scale[b] = s;
        for (int i = 0; i < BLOCK_N * k; i++) {
            float v = rintf(w[(size_t)b * BLOCK_N * k + i] / s);
            v = fminf(fmaxf(v, -127.0f), 127.0f);
            q[(size_t)b * BLOCK_N * k + i] = (int8_t)v;
        }
    }
}

/* brokefish/nn/quant.py:246-260: one scale per row; q is returned as int16 so the
 * unsigned range [0, 255] fits. */
void bfo_quantise_activations_int8(const float* x, int m, int k, int unsigned_, int16_t* q,
                                   float* scale) {
    for (int i = 0; i < m; i++) {
        const float* row = x + (size_t)i * k;
        float amax = 0.0f;
        for (int j = 0; j < k; j++) {
            const float v = unsigned_ ? fmaxf(row[j], 0.0f) : fabsf(row[j]);
            amax = fmaxf(amax, v);
        }
        const float qmax = unsigned_ ? 255.0f : 127.0f;
        const float s = amax > 0.0f ? amax / qmax : 1.0f;
        scale[i] = s;
        for (int j = 0; j < k; j++) {
            float v = unsigned_ ? fmaxf(row[j], 0.0f) : row[j];
            v = rintf(v / s);
            v = fminf(fmaxf(v, unsigned_ ? 0.0f : -127.0f), qmax);
            q[(size_t)i * k + j] = (int16_t)v;
        }
    }
}

/* brokefish/nn/quant.py:281-305 with pre-quantised weights.
 * x [m,k] fp32, wq [n,k] int8, ws [n/128], bias [n] or NULL -> out [m,n].
 * Optional taps: qa [m,k] int16 operand values, sa [m, k/256] scales,
 * acc [k/256][m][n] exact integer accumulators per 256-chunk. */
void bfo_int8_linear_q(const float* x, int m, int k, const int8_t* wq, const float* ws, int n,
                       const float* bias, int unsigned_, float* out, int16_t* qa_tap,
                       float* sa_tap, int32_t* acc_tap) {
    const int chunks = k / ROW_K;
    int16_t* q = (int16_t*)malloc((size_t)m * ROW_K * sizeof(int16_t));
    float* xs = (float*)malloc((size_t)m * ROW_K * sizeof(float));
    float* sa = (float*)malloc((size_t)m * sizeof(float));
    double* o64 = (double*)calloc((size_t)m * n, sizeof(double));
    for (int c = 0; c < chunks; c++) {
        for (int i = 0; i < m; i++)
            memcpy(xs + (size_t)i * ROW_K, x + (size_t)i * k + (size_t)c * ROW_K, ROW_K * sizeof(float));
        bfo_quantise_activations_int8(xs, m, ROW_K, unsigned_, q, sa);
        for (int i = 0; i < m; i++) {
            if (qa_tap)
                memcpy(qa_tap + (size_t)i * k + (size_t)c * ROW_K, q + (size_t)i * ROW_K, ROW_K * sizeof(int16_t));
            if (sa_tap) sa_tap[(size_t)i * chunks + c] = sa[i];
            for (int j = 0; j < n; j++) {
                int32_t acc = 0;
                const int8_t* wr = wq + (size_t)j * k + (size_t)c * ROW_K;
                const int16_t* qr = q + (size_t)i * ROW_K;
                for (int kk = 0; kk < ROW_K; kk++) acc += (int32_t)qr[kk] * (int32_t)wr[kk];
                if (acc_tap) acc_tap[((size_t)c * m + i) * n + j] = acc;
                o64[(size_t)i * n + j] += (double)acc * (double)sa[i];
            }
        }
    }
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) {
            float v = (float)o64[(size_t)i * n + j] * ws[j / BLOCK_N];
            if (bias) v = v + bias[j];
            out[(size_t)i * n + j] = v;
        }
    free(q); free(xs); free(sa); free(o64);
}

/* Same, quantising the fp32 weight on the fly exactly as the reference does. */
void bfo_int8_linear(const float* x, int m, int k, const float* w, int n, const float* bias,
                     int unsigned_, float* out) {
    int8_t* wq = (int8_t*)malloc((size_t)n * k);
    float* ws = (float*)malloc((size_t)(n / BLOCK_N) * sizeof(float));
    bfo_quantise_weights_int8(w, n, k, wq, ws);
    bfo_int8_linear_q(x, m, k, wq, ws, n, bias, unsigned_, out, NULL, NULL, NULL);
    free(wq); free(ws);
}

/* ---- LayerNorm in lane order -------------------------------------------------- */

/* tile sums of a quarter of the width, added as a balanced tree (1, 2 or 4 tiles) */
static float tree_sum(const float* ts, int n) {
    if (n == 1) return ts[0];
    if (n == 2) return ts[0] + ts[1];
    return (ts[0] + ts[1]) + (ts[2] + ts[3]);
}

static void layernorm_rows(const float* x, int d, const float* gamma, const float* beta,
                           float eps, float* y) {
    for (int t = 0; t < T; t++) {
        const float* row = x + (size_t)t * d;
        /* per lane half g: every 32-wide tile's 16 values form one chain from zero; the tile sums
         * of a quarter of the width are added as a balanced tree (t0 + t1 for two tiles,
         * (t0 + t1) + (t2 + t3) for four); the four quarter sums are added in order; then the
         * two halves */
        const int tq = d / 32 / 4;
        float part[2];
        for (int g = 0; g < 2; g++) {
            float sg[4];
            for (int q = 0; q < 4; q++) {
                float ts[4];
                for (int n = 0; n < tq; n++) {
                    float s = 0.0f;
                    for (int r = 0; r < 16; r++) s = s + row[32 * (q * tq + n) + ch(r, g)];
                    ts[n] = s;
                }
                sg[q] = tree_sum(ts, tq);
            }
            part[g] = ((sg[0] + sg[1]) + sg[2]) + sg[3];
        }
        const float inv_d = 1.0f / (float)d; /* d is a power of two: exact */
        const float mean = (part[0] + part[1]) * inv_d;
        for (int g = 0; g < 2; g++) {
            float sg[4];
            for (int q = 0; q < 4; q++) {
                float ts[4];
                for (int n = 0; n < tq; n++) {
                    float s = 0.0f;
                    for (int r = 0; r < 16; r++) {
                        const float dv = row[32 * (q * tq + n) + ch(r, g)] - mean;
                        s = fmaf(dv, dv, s);
                    }
                    ts[n] = s;
                }
                sg[q] = tree_sum(ts, tq);
            }
            part[g] = ((sg[0] + sg[1]) + sg[2]) + sg[3];
        }
        const float var = (part[0] + part[1]) * inv_d;
        const float rstd = 1.0f / sqrtf(var + eps);
        for (int c = 0; c < d; c++) {
            const float dv = row[c] - mean;
            y[(size_t)t * d + c] = fmaf(dv * rstd, gamma[c], beta[c]);
        }
    }
}

/* ---- the forward ---------------------------------------------------------------- */

struct bfo_model {
    bfo_config cfg;
    /* fp32 parameters, natural (state_dict) layout */
    float *emb[5];
    float *norm1_w, *norm1_b, *norm2_w, *norm2_b; /* [L][d] */
    float *b_qkv, *b_out, *b_ff1, *b_ff2;          /* [L][3d], [L][d], [L][dff], [L][d] */
    int8_t *q_qkv, *q_out, *q_ff1, *q_ff2;         /* quantised weights [L][n][k] */
    float *s_qkv, *s_out, *s_ff1, *s_ff2;          /* [L][n/128] */
    float *normf_w, *normf_b;
    float *head_w; /* [64 + 4 + n_value][d] */
};

static float* dupf(const float* p, size_t n) {
    float* r = (float*)malloc(n * sizeof(float));
    memcpy(r, p, n * sizeof(float));
    return r;
}

/* How many positive floats m (every `stride`-th bit pattern) the kernels' three-instruction
 * quotient by a constant -- q = m * c, r = fma(-q, D, m), q' = fma(r, c, q), c = fl(1 / D) --
 * fails to divide correctly (q' != m / D).  stride 1 covers all 2,139,095,039 of them (0 failures for D = 127 and D = 255, the
 * divisors of the activation scales; about a minute on 8 cores). */
long bfo_check_div_const(float D, unsigned stride) {
    const float c = 1.0f / D;
    long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (unsigned long long u = 1; u < 0x7f800000ull; u += stride) {
        float m;
        const unsigned bits = (unsigned)u;
        memcpy(&m, &bits, 4);
        const float q = m * c;
        const float q2 = fmaf(fmaf(-q, D, m), c, q);
        bad += q2 != m / D;
    }
    return bad;
}

bfo_model* bfo_model_create(const bfo_config* cfg, const bfo_params* p) {
    const int d = cfg->d_model, L = cfg->n_layers, f = cfg->d_ff;
    if (d % 256 || f % 256 || d / cfg->n_heads != 32 || (cfg->n_value != 1 && cfg->n_value != 3) ||
        cfg->value_mode < 0 || cfg->value_mode > 2)
        return NULL;
    bfo_model* m = (bfo_model*)calloc(1, sizeof(bfo_model));
    m->cfg = *cfg;
    const int rows[5] = {64, 12, 4, 101, 3};
    const float* tabs[5] = {p->emb_square, p->emb_type_special, p->emb_color_turn, p->emb_clock, p->emb_rep};
    for (int i = 0; i < 5; i++) m->emb[i] = dupf(tabs[i], (size_t)rows[i] * d);
    m->norm1_w = dupf(p->norm1_w, (size_t)L * d); m->norm1_b = dupf(p->norm1_b, (size_t)L * d);
    m->norm2_w = dupf(p->norm2_w, (size_t)L * d); m->norm2_b = dupf(p->norm2_b, (size_t)L * d);
    m->b_qkv = dupf(p->in_proj_b, (size_t)L * 3 * d); m->b_out = dupf(p->out_proj_b, (size_t)L * d);
    m->b_ff1 = dupf(p->linear1_b, (size_t)L * f); m->b_ff2 = dupf(p->linear2_b, (size_t)L * d);
    m->q_qkv = (int8_t*)malloc((size_t)L * 3 * d * d); m->s_qkv = (float*)malloc((size_t)L * (3 * d / 128) * 4);
    m->q_out = (int8_t*)malloc((size_t)L * d * d);     m->s_out = (float*)malloc((size_t)L * (d / 128) * 4);
    m->q_ff1 = (int8_t*)malloc((size_t)L * f * d);     m->s_ff1 = (float*)malloc((size_t)L * (f / 128) * 4);
    m->q_ff2 = (int8_t*)malloc((size_t)L * d * f);     m->s_ff2 = (float*)malloc((size_t)L * (d / 128) * 4);
    for (int l = 0; l < L; l++) {
        bfo_quantise_weights_int8(p->in_proj_w + (size_t)l * 3 * d * d, 3 * d, d, m->q_qkv + (size_t)l * 3 * d * d, m->s_qkv + (size_t)l * (3 * d / 128));
        bfo_quantise_weights_int8(p->out_proj_w + (size_t)l * d * d, d, d, m->q_out + (size_t)l * d * d, m->s_out + (size_t)l * (d / 128));
        bfo_quantise_weights_int8(p->linear1_w + (size_t)l * f * d, f, d, m->q_ff1 + (size_t)l * f * d, m->s_ff1 + (size_t)l * (f / 128));
        bfo_quantise_weights_int8(p->linear2_w + (size_t)l * d * f, d, f, m->q_ff2 + (size_t)l * d * f, m->s_ff2 + (size_t)l * (d / 128));
    }
    m->normf_w = dupf(p->norm_f_w, d); m->normf_b = dupf(p->norm_f_b, d);
    const int nh = 64 + 4 + cfg->n_value;
    m->head_w = (float*)malloc((size_t)nh * d * sizeof(float));
    memcpy(m->head_w, p->policy_w, (size_t)64 * d * 4);
    memcpy(m->head_w + (size_t)64 * d, p->promo_w, (size_t)4 * d * 4);
    memcpy(m->head_w + (size_t)68 * d, p->value_w, (size_t)cfg->n_value * d * 4);
    return m;
}

void bfo_model_destroy(bfo_model* m) {
    if (!m) return;
    for (int i = 0; i < 5; i++) free(m->emb[i]);
    free(m->norm1_w); free(m->norm1_b); free(m->norm2_w); free(m->norm2_b);
    free(m->b_qkv); free(m->b_out); free(m->b_ff1); free(m->b_ff2);
    free(m->q_qkv); free(m->q_out); free(m->q_ff1); free(m->q_ff2);
    free(m->s_qkv); free(m->s_out); free(m->s_ff1); free(m->s_ff2);
    free(m->normf_w); free(m->normf_b); free(m->head_w);
    free(m);
}

const int8_t* bfo_model_qweight(const bfo_model* m, int which, int layer, const float** scale) {
    const int d = m->cfg.d_model, f = m->cfg.d_ff;
    switch (which) {
    case 0: if (scale) *scale = m->s_qkv + (size_t)layer * (3 * d / 128); return m->q_qkv + (size_t)layer * 3 * d * d;
    case 1: if (scale) *scale = m->s_out + (size_t)layer * (d / 128); return m->q_out + (size_t)layer * d * d;
    case 2: if (scale) *scale = m->s_ff1 + (size_t)layer * (f / 128); return m->q_ff1 + (size_t)layer * f * d;
    case 3: if (scale) *scale = m->s_ff2 + (size_t)layer * (d / 128); return m->q_ff2 + (size_t)layer * d * f;
    }
    return NULL;
}

/* Embedding of one board: x [32][d], alive bitmask. */
static uint32_t embed_board(const bfo_model* m, const uint16_t* words, int16_t control,
                            uint8_t rep, float* x) {
    const int d = m->cfg.d_model;
    const int stm = control < 0;
    int mag = control < 0 ? -(int)control : (int)control;
    int clock = mag - 1;
    if (clock < 0) clock = 0;
    if (clock > 100) clock = 100;
    const int rp = rep > 2 ? 2 : rep;
    uint32_t alive = 0;
    for (int t = 0; t < T; t++) {
        const unsigned w = words[t];
        if (!((w >> 11) & 1)) alive |= 1u << t;
        const int colour = (w >> 10) & 1, special = (w >> 9) & 1, type = (w >> 6) & 7, sq = w & 63;
        int ts = type * 2 + special;
        if (ts > 11) ts = 11; /* types 6, 7 are undefined; never index past the table */
        const int ct = colour * 2 + stm;
        for (int c = 0; c < d; c++) {
            const float per_board = m->emb[3][(size_t)clock * d + c] + m->emb[4][(size_t)rp * d + c];
            float v = m->emb[0][(size_t)sq * d + c];
            v = v + m->emb[1][(size_t)ts * d + c];
            v = v + m->emb[2][(size_t)ct * d + c];
            v = v + per_board;
            x[(size_t)t * d + c] = v;
        }
    }
    return alive;
}

/* Attention for one board: qkv [32][3d] -> o [32][d]; dead keys masked. */
static void attention_board(const float* qkv, int d, int n_heads, uint32_t alive, float* o) {
    const float scale = 0.17677669529663687f; /* 1/sqrt(32) */
    for (int h = 0; h < n_heads; h++) {
        const float* Q = qkv + 32 * h;
        const float* K = qkv + d + 32 * h;
        const float* V = qkv + 2 * d + 32 * h;
        for (int i = 0; i < T; i++) {
            float s[T], p[T];
            float mx = -INFINITY;
            for (int j = 0; j < T; j++) {
                float acc = 0.0f;
                for (int r = 0; r < 16; r++)
                    for (int g = 0; g < 2; g++) {
                        const int c = ch(r, g);
                        acc = fmaf(K[(size_t)j * 3 * d + c], Q[(size_t)i * 3 * d + c], acc);
                    }
                acc = acc * scale;
                if (!((alive >> j) & 1)) acc = -INFINITY;
                s[j] = acc;
                mx = fmaxf(mx, acc);
            }
            float part[2];
            for (int g = 0; g < 2; g++) {
                float l = 0.0f;
                for (int r = 0; r < 16; r++) {
                    const int j = ch(r, g);
                    p[j] = bfo_exp_neg(s[j] - mx);
                    l = l + p[j];
                }
                part[g] = l;
            }
            const float rl = 1.0f / (part[0] + part[1]);
            for (int j = 0; j < T; j++) p[j] = p[j] * rl;
            for (int c = 0; c < 32; c++) {
                float acc = 0.0f;
                for (int r = 0; r < 16; r++)
                    for (int g = 0; g < 2; g++) {
                        const int j = ch(r, g);
                        acc = fmaf(V[(size_t)j * 3 * d + c], p[j], acc);
                    }
                o[(size_t)i * d + 32 * h + c] = acc;
            }
        }
    }
}

/* Copy helpers for the taps. */
static void tap_q(int8_t* dst, const int16_t* q, size_t n, int unsigned_) {
    /* operand bytes as the evaluator holds them: signed s8, or u8 for ffn2 */
    for (size_t i = 0; i < n; i++) dst[i] = (int8_t)(unsigned_ ? (uint8_t)q[i] : (int8_t)q[i]);
}

int bfo_forward(const bfo_model* m, const uint16_t* boards, const int16_t* control,
                const uint8_t* rep, const uint64_t* mask, int n, float* policy, float* promo,
                float* value, int32_t* best_move, const bfo_taps* taps) {
    const int d = m->cfg.d_model, L = m->cfg.n_layers, f = m->cfg.d_ff, H = m->cfg.n_heads;
    const int nv = m->cfg.n_value;
    const float eps = m->cfg.eps;
    const int kc_d = d / ROW_K, kc_f = f / ROW_K;
    int l0 = 0, l1 = L;
    if (taps && (taps->layer_begin || taps->layer_end)) { l0 = taps->layer_begin; l1 = taps->layer_end; }
    if (l0 < 0 || l1 > L || l0 > l1) return -1;
#pragma omp parallel for schedule(dynamic, 1)
    for (int b = 0; b < n; b++) {
        float* x = (float*)malloc((size_t)T * d * 4);
        float* y = (float*)malloc((size_t)T * d * 4);
        float* qkv = (float*)malloc((size_t)T * 3 * d * 4);
        float* o = (float*)malloc((size_t)T * d * 4);
        float* hid = (float*)malloc((size_t)T * f * 4);
        float* tmp = (float*)malloc((size_t)T * d * 4);
        int16_t* qa = (int16_t*)malloc((size_t)T * f * 2);
        float* sa = (float*)malloc((size_t)T * (kc_f > kc_d ? kc_f : kc_d) * 4);
        int32_t* acc = (int32_t*)malloc((size_t)T * (size_t)(3 * d > f ? 3 * d : f) * (kc_f > kc_d ? kc_f : kc_d) * 4);

        const uint32_t alive = embed_board(m, boards + (size_t)b * 32, control[b], rep[b], x);
        if (taps && taps->x_in) memcpy(x, taps->x_in + (size_t)b * T * d, (size_t)T * d * 4);
        if (taps && taps->embed) memcpy(taps->embed + (size_t)b * T * d, x, (size_t)T * d * 4);
        for (int l = l0; l < l1; l++) {
            const size_t bl = (size_t)b * (l1 - l0) + (l - l0);
            /* x += out_proj(attention(in_proj(LN1(x)))) */
            layernorm_rows(x, d, m->norm1_w + (size_t)l * d, m->norm1_b + (size_t)l * d, eps, y);
            bfo_int8_linear_q(y, T, d, m->q_qkv + (size_t)l * 3 * d * d, m->s_qkv + (size_t)l * (3 * d / 128),
                              3 * d, m->b_qkv + (size_t)l * 3 * d, 0, qkv, qa, sa, acc);
            if (taps && taps->qa_qkv) tap_q(taps->qa_qkv + bl * T * d, qa, (size_t)T * d, 0);
            if (taps && taps->acc_qkv) memcpy(taps->acc_qkv + bl * kc_d * T * 3 * d, acc, (size_t)kc_d * T * 3 * d * 4);
            attention_board(qkv, d, H, alive, o);
            bfo_int8_linear_q(o, T, d, m->q_out + (size_t)l * d * d, m->s_out + (size_t)l * (d / 128), d,
                              m->b_out + (size_t)l * d, 0, tmp, qa, sa, acc);
            if (taps && taps->qa_out) tap_q(taps->qa_out + bl * T * d, qa, (size_t)T * d, 0);
            if (taps && taps->acc_out) memcpy(taps->acc_out + bl * kc_d * T * d, acc, (size_t)kc_d * T * d * 4);
            for (int i = 0; i < T * d; i++) x[i] = x[i] + tmp[i];
            /* x += linear2(relu(linear1(LN2(x)))) */
            layernorm_rows(x, d, m->norm2_w + (size_t)l * d, m->norm2_b + (size_t)l * d, eps, y);
            bfo_int8_linear_q(y, T, d, m->q_ff1 + (size_t)l * f * d, m->s_ff1 + (size_t)l * (f / 128), f,
                              m->b_ff1 + (size_t)l * f, 0, hid, qa, sa, acc);
            if (taps && taps->qa_ff1) tap_q(taps->qa_ff1 + bl * T * d, qa, (size_t)T * d, 0);
            if (taps && taps->acc_ff1) memcpy(taps->acc_ff1 + bl * kc_d * T * f, acc, (size_t)kc_d * T * f * 4);
            for (int i = 0; i < T * f; i++) hid[i] = fmaxf(hid[i], 0.0f);
            bfo_int8_linear_q(hid, T, f, m->q_ff2 + (size_t)l * d * f, m->s_ff2 + (size_t)l * (d / 128), d,
                              m->b_ff2 + (size_t)l * d, 1, tmp, qa, sa, acc);
            if (taps && taps->qa_ff2) tap_q(taps->qa_ff2 + bl * T * f, qa, (size_t)T * f, 1);
            if (taps && taps->acc_ff2) memcpy(taps->acc_ff2 + bl * kc_f * T * d, acc, (size_t)kc_f * T * d * 4);
            for (int i = 0; i < T * d; i++) x[i] = x[i] + tmp[i];
            if (taps && taps->resid) memcpy(taps->resid + bl * T * d, x, (size_t)T * d * 4);
        }
        layernorm_rows(x, d, m->normf_w, m->normf_b, eps, y);
        if (taps && taps->normed) memcpy(taps->normed + (size_t)b * T * d, y, (size_t)T * d * 4);
        /* heads: one fma chain per output in lane order */
        float raw[3] = {0, 0, 0};
        const int vmode = m->cfg.value_mode;
        const int king = vmode ? -1 : (control[b] < 0 ? 31 : 15);
        for (int t = 0; t < T; t++)
            for (int oo = 0; oo < 68 + nv; oo++) {
                if (oo >= 68 && t != king) continue;
                const float* w = m->head_w + (size_t)oo * d;
                float a = 0.0f;
                for (int nn = 0; nn < d / 32; nn++)
                    for (int r = 0; r < 16; r++)
                        for (int g = 0; g < 2; g++) {
                            const int c = 32 * nn + ch(r, g);
                            a = fmaf(w[c], y[(size_t)t * d + c], a);
                        }
                if (oo < 64) policy[((size_t)b * T + t) * 64 + oo] = a;
                else if (oo < 68) promo[((size_t)b * T + t) * 4 + (oo - 64)] = a;
                else raw[oo - 68] = a;
            }
        if (vmode) {
            /* pooled heads (brokefish/nn/model.py:576-617): the value row is the mean over the live
             * tokens of the normed stream (1) or norm_f of the mean of the residual stream (2).  The
             * token sum is a butterfly (distances 16, 8, 4, 2, 1), dead tokens count as 0; the row
             * then goes through the value rows like a token; White's frame, so negated for Black. */
            const float* src = vmode == 1 ? y : x;
            float* row = tmp; /* [d], then [T][d] scratch for layernorm_rows */
            int cnt = 0;
            for (int t = 0; t < T; t++) cnt += (alive >> t) & 1;
            const float cdiv = (float)(cnt > 0 ? cnt : 1);
            for (int c = 0; c < d; c++) {
                float v[32];
                for (int t = 0; t < T; t++) v[t] = ((alive >> t) & 1) ? src[(size_t)t * d + c] : 0.0f;
                for (int dist = 16; dist >= 1; dist >>= 1) {
                    float w[32];
                    for (int t = 0; t < T; t++) w[t] = v[t] + v[t ^ dist];
                    memcpy(v, w, sizeof v);
                }
                row[c] = v[0] / cdiv;
            }
            if (vmode == 2) {   /* the same LayerNorm as a token row gets */
                for (int t = 1; t < T; t++) memcpy(row + (size_t)t * d, row, (size_t)d * 4);
                layernorm_rows(row, d, m->normf_w, m->normf_b, eps, o);
                memcpy(row, o, (size_t)d * 4);
            }
            for (int k = 0; k < nv; k++) {
                const float* w = m->head_w + (size_t)(68 + k) * d;
                float a = 0.0f;
                for (int nn = 0; nn < d / 32; nn++)
                    for (int r = 0; r < 16; r++)
                        for (int g = 0; g < 2; g++) {
                            const int c = 32 * nn + ch(r, g);
                            a = fmaf(w[c], row[c], a);
                        }
                raw[k] = a;
            }
        }
        if (nv == 1) {
            value[b] = bfo_tanh(raw[0]);
        } else {
            /* classes 0 = loss, 1 = draw, 2 = win: p(win) - p(loss), brokefish/nn/model.py:156-170 */
            const float mx = fmaxf(fmaxf(raw[0], raw[1]), raw[2]);
            const float e0 = bfo_exp_neg(raw[0] - mx), e1 = bfo_exp_neg(raw[1] - mx), e2 = bfo_exp_neg(raw[2] - mx);
            value[b] = (e2 - e0) / ((e0 + e1) + e2);
        }
        if (vmode && !(control[b] > 0)) value[b] = -value[b];
        if (mask) {
            int best = -1;
            float bv = -INFINITY;
            for (int t = 0; t < T; t++)
                for (int s = 0; s < 64; s++) {
                    float* pv = &policy[((size_t)b * T + t) * 64 + s];
                    if (!((mask[(size_t)b * 32 + t] >> s) & 1)) { *pv = -INFINITY; continue; }
                    if (best < 0 || *pv > bv) { bv = *pv; best = t * 64 + s; }
                }
            if (best_move) best_move[b] = best;
        }
        free(x); free(y); free(qkv); free(o); free(hid); free(tmp); free(qa); free(sa); free(acc);
    }
    return 0;
}
