/*
 * TEST INFRASTRUCTURE - interface of the CPU checker (see mk_oracle.c).
 * Buffers have the layouts of the reference's Globals
 * (megakernels/demos/latency/scheduler.py:38-115): bf16 tensors are passed as
 * uint16_t bit patterns, everything is contiguous, batch size is 1.
 */
#ifndef MK_ORACLE_H
#define MK_ORACLE_H

#include <stdint.h>

typedef struct mk_oracle_globals {
    /* weights, stacked over layers */
    const uint16_t *qkv_proj_weights;     /* [L, (H+2KVH) D, hidden] */
    const uint16_t *attn_ln_weights;      /* [L, hidden] */
    const uint16_t *o_proj_weights;       /* [L, hidden, hidden] */
    const uint16_t *mlp_ln_weights;       /* [L, hidden] */
    const uint16_t *up_proj_weights;      /* [L, inter, hidden] */
    const uint16_t *gate_proj_weights;    /* [L, inter, hidden] */
    const uint16_t *down_proj_weights;    /* [L, hidden, inter] */
    const uint16_t *lm_head_norm_weights; /* [hidden] */
    const uint16_t *lm_head_weights;      /* [vocab, hidden] */
    uint16_t *k_cache;                    /* [L, kv_max_len, KVH, D] */
    uint16_t *v_cache;
    const float *rope_cos;                /* [positions, D] */
    const float *rope_sin;
    /* activations */
    uint16_t *hidden_states;              /* [hidden] */
    uint16_t *post_ln_rope_q;             /* [H D] */
    uint16_t *attn_out;                   /* [H D] */
    float *attn_lse_intermediates;        /* [H, max_partials] */
    float *attn_out_intermediates;        /* [H, max_partials, D] */
    uint16_t *silu_out;                   /* [inter] */
    uint16_t *logits;                     /* [vocab] */
    int32_t *barriers;                    /* [L, 10, H + 2 KVH] */
    /* shapes */
    int32_t num_hidden_layers, num_attention_heads, num_kv_heads, head_dim;
    int32_t hidden_size, intermediate_size, vocab_size;
    int32_t kv_max_len, max_partials;
    int32_t matvec_reduction_size, attn_reduction_size;
    /* scalars */
    int32_t pos_id;
    int32_t skip_attn_reduction;
    int32_t check_barriers;               /* 1: assert predecessor counters exactly, like the reference VM */
    float attn_scale;
    float rms_norm_eps;
} mk_oracle_globals;

/* Runs `count` instructions of 32 int32 words each, in order.  Returns 0, or
 * -1 with a message available from mk_oracle_last_error(). */
int mk_oracle_run(mk_oracle_globals *g, const int32_t *instructions, int count);
const char *mk_oracle_last_error(void);
int mk_oracle_threads(void);
int mk_oracle_argmax_bf16(const uint16_t *v, int n);

float mk_oracle_expf(float x);
float mk_oracle_exp2f(float x);
float mk_oracle_log2f(float x);
uint16_t mk_oracle_f32_to_bf16(float x);
float mk_oracle_dot(const uint16_t *w, const float *x, int K);
/* out[i] = acc[i] + a[i].lo * b[i].lo + a[i].hi * b[i].hi (bf16 pairs), the two-element dot product
 * of exact_math.h */
void mk_oracle_dot2(const uint32_t *a, const uint32_t *b, const float *acc, float *out, size_t n);
/* the same through the clause-by-clause form only (orc_dot2_bf16 takes a shorter way for ordinary operands) */
void mk_oracle_dot2_general(const uint32_t *a, const uint32_t *b, const float *acc, float *out, size_t n);

#endif
