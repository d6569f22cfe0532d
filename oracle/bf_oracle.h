/* TEST INFRASTRUCTURE -- NOT PRODUCT CODE.  See bf_oracle.c. */
#ifndef BF_ORACLE_H
#define BF_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    int d_model, n_layers, n_heads, d_ff, n_value;
    float eps;
    /* value head (brokefish/nn/model.py:551-617): 0 king row, 1 pooled (mean of the final-normed
     * live tokens), 2 prenorm (final norm of the mean of the live tokens' residual stream) */
    int value_mode;
} bfo_config;

/* fp32 parameters in state_dict layout (brokefish/nn/model.py:297-316); per-layer
 * tensors are stacked on a leading [n_layers] axis. */
typedef struct {
    const float *emb_square, *emb_type_special, *emb_color_turn, *emb_clock, *emb_rep;
    const float *in_proj_w, *in_proj_b;   /* [L,3d,d], [L,3d] */
    const float *out_proj_w, *out_proj_b; /* [L,d,d],  [L,d]  */
    const float *linear1_w, *linear1_b;   /* [L,f,d],  [L,f]  */
    const float *linear2_w, *linear2_b;   /* [L,d,f],  [L,d]  */
    const float *norm1_w, *norm1_b, *norm2_w, *norm2_b; /* [L,d] */
    const float *norm_f_w, *norm_f_b;     /* [d] */
    const float *policy_w, *promo_w, *value_w; /* [64,d], [4,d], [n_value,d] */
} bfo_params;

/* Optional intermediate outputs; any pointer may be NULL.  B = boards, L = layers,
 * kc = K / 256 chunks of the matmul in question.
 *   qa_*   int8 operand bytes exactly as quantised (u8 bit patterns for ffn2)
 *   acc_*  exact integer accumulators, [B, L, kc, 32, Nout] */
typedef struct {
    const float* x_in; /* [B,32,d] residual stream to start from instead of the embedding */
    int layer_begin, layer_end; /* run layers [begin, end); 0,0 means all.  L below = layers run */
    float* embed;      /* [B,32,d] */
    int8_t* qa_qkv;    /* [B,L,32,d] */
    int32_t* acc_qkv;  /* [B,L,kc,32,3d] */
    int8_t* qa_out;    /* [B,L,32,d] */
    int32_t* acc_out;  /* [B,L,kc,32,d] */
    int8_t* qa_ff1;    /* [B,L,32,d] */
    int32_t* acc_ff1;  /* [B,L,kc,32,f] */
    int8_t* qa_ff2;    /* [B,L,32,f] */
    int32_t* acc_ff2;  /* [B,L,kc,32,d] */
    float* resid;      /* [B,L,32,d] residual stream after each layer */
    float* normed;     /* [B,32,d] after norm_f */
} bfo_taps;

typedef struct bfo_model bfo_model;

long bfo_check_div_const(float D, unsigned stride);
float bfo_exp_neg(float x);
float bfo_tanh(float x);
void bfo_quantise_weights_int8(const float* w, int n, int k, int8_t* q, float* scale);
void bfo_quantise_activations_int8(const float* x, int m, int k, int unsigned_, int16_t* q, float* scale);
void bfo_int8_linear_q(const float* x, int m, int k, const int8_t* wq, const float* ws, int n,
                       const float* bias, int unsigned_, float* out, int16_t* qa_tap,
                       float* sa_tap, int32_t* acc_tap);
void bfo_int8_linear(const float* x, int m, int k, const float* w, int n, const float* bias,
                     int unsigned_, float* out);

bfo_model* bfo_model_create(const bfo_config* cfg, const bfo_params* p);
void bfo_model_destroy(bfo_model* m);
/* which: 0 qkv, 1 out, 2 ffn1, 3 ffn2 */
const int8_t* bfo_model_qweight(const bfo_model* m, int which, int layer, const float** scale);

/* boards [n,32] u16, control [n] i16, rep [n] u8, mask [n,32] u64 or NULL.
 * policy [n,32,64], promo [n,32,4], value [n] fp32; with a mask, illegal policy
 * entries become -inf and best_move [n] (may be NULL) receives slot*64+square. */
int bfo_forward(const bfo_model* m, const uint16_t* boards, const int16_t* control,
                const uint8_t* rep, const uint64_t* mask, int n, float* policy, float* promo,
                float* value, int32_t* best_move, const bfo_taps* taps);

#ifdef __cplusplus
}
#endif
#endif
