/*
 * oracle.h -- CPU restatement of the reference's LLaMA3 forward pass.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, the host
 * engine, the GPU leg of bench.py) may include, link or call this file.  It is
 * the checker: tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
 * are its only users.
 *
 * Two arithmetic modes share one graph:
 *   ORC_REF16  every inter-kernel activation is rounded to fp16 exactly where
 *              the reference stores a __half, accumulation is fp32 in the
 *              reference's order (ascending k, its reduction trees).
 *   ORC_FP32   same graph, no intermediate rounding, free accumulation order,
 *              OpenMP over rows/heads -- the timed "fp32 forward" CPU baseline.
 *
 *   ORC_REF16_REV  ORC_REF16 with every projection summed over k downwards: the same
 *              arithmetic in another legal fp32 order.  Not a parity target; it
 *              measures how much of a deviation is summation order alone.
 *
 * Every function cites the reference lines it restates (paths under
 * src/ of abhisheknair10/LLM.cu).
 */
#ifndef LLMCU_ORACLE_H
#define LLMCU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_REF16 = 0, ORC_FP32 = 1, ORC_REF16_REV = 2 };

typedef struct {
    int n_layers;
    int d_model;
    int n_heads;
    int n_kv_heads;
    int head_dim;
    int ffn_dim;
    int vocab;
    int max_pos;
    double rms_eps;   /* the reference writes the double literal 1e-5 (inference.cu:351) */
    float rope_theta; /* 500000.0f (inference.cu:673) */
} orc_config;

/* fp16 bit patterns, [out, in] row-major, one pointer per layer. */
typedef struct {
    const uint16_t *embed;   /* [vocab, d]  */
    const uint16_t *lm_head; /* [vocab, d]  */
    const uint16_t *norm;    /* [d]         */
    const uint16_t *const *input_ln; /* [d] */
    const uint16_t *const *post_ln;  /* [d] */
    const uint16_t *const *wq;    /* [Hq*hd, d]  */
    const uint16_t *const *wk;    /* [Hkv*hd, d] */
    const uint16_t *const *wv;    /* [Hkv*hd, d] */
    const uint16_t *const *wo;    /* [d, Hq*hd]  */
    const uint16_t *const *wgate; /* [F, d] */
    const uint16_t *const *wup;   /* [F, d] */
    const uint16_t *const *wdown; /* [d, F] */
} orc_weights;

/* ---- scalar conversions --------------------------------------------- */
uint16_t orc_f32_to_f16_soft(float f);   /* IEEE RNE, NaN -> 0x7FFF */
float    orc_f16_to_f32_soft(uint16_t h);
uint16_t orc_f32_to_f16(float f);        /* F16C when compiled in, else soft */
float    orc_f16_to_f32(uint16_t h);

/* ---- single ops (fp16 bit patterns in and out, ORC_REF16 arithmetic) -- */
void orc_bf16_to_fp16(const uint16_t *src, uint16_t *dst, size_t n);
void orc_embed(const uint16_t *table, const int32_t *ids, int T, int d, uint16_t *out);
int  orc_rmsnorm(const uint16_t *x, const uint16_t *gain, int T, int d, double eps, uint16_t *out);
void orc_add(uint16_t *x, const uint16_t *res, size_t n);
void orc_linear(const uint16_t *x, const uint16_t *w, int T, int N, int K, uint16_t *out);
void orc_linear_swiglu(const uint16_t *x, const uint16_t *wgate, const uint16_t *wup,
                       int T, int N, int K, uint16_t *out);
void orc_rope(uint16_t *buf, int T, int n_heads, int head_dim, int pos0, float theta);
/* causal GQA attention of Tq query rows at absolute positions pos0..pos0+Tq-1
 * over keys/values 0..pos0+Tq-1 (k, v: [pos, Hkv*hd] token-major as in the reference). */
void orc_attention(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                   int Tq, int pos0, int n_heads, int n_kv_heads, int head_dim, uint16_t *out);
/* the reference's three-kernel form: full [H,T,T] fp32 score tensor, masked softmax, P.V */
void orc_attention_materialized(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                                int T, int n_heads, int n_kv_heads, int head_dim, uint16_t *out);
int  orc_argmax_f16(const uint16_t *logits, int n);

/* ---- whole model ------------------------------------------------------ */
typedef struct orc_model orc_model;

orc_model *orc_model_new(const orc_config *cfg, const orc_weights *w, int mode);
void orc_model_free(orc_model *m);
void orc_model_reset(orc_model *m);
int  orc_model_pos(const orc_model *m);
/* Append n_new tokens at the current position using the KV cache; returns the
 * greedy next token (argmax over the fp16-rounded logits of the last row).
 * hidden_out (may be NULL): [n_layers][n_new][d] fp16 bits, X after each layer.
 * logits_out (may be NULL): [vocab] fp16 bits of the last row. */
int orc_model_forward(orc_model *m, const int32_t *tokens, int n_new,
                      uint16_t *hidden_out, uint16_t *logits_out);
/* The reference's own schedule: re-run the whole sequence with no cache
 * (inference.cu:149-193).  ORC_REF16 only; same outputs as above for the
 * full sequence (hidden_out: [n_layers][T][d]). */
int orc_model_forward_recompute(const orc_config *cfg, const orc_weights *w,
                                const int32_t *tokens, int T,
                                uint16_t *hidden_out, uint16_t *logits_out);

int orc_num_threads(void);

/* ---- host sampler (inference.cu:1030-1161) ------------------------------ */
/* glibc's rand() as the reference uses it (never seeded, i.e. srand(1)): the TYPE_3 additive-feedback
 * generator r[i] = r[i-3] + r[i-31], output r[i] >> 1, restated so that the oracle keeps a private
 * stream.  state: 34 + 2 words. */
typedef struct { int32_t r[34]; int f, b; } orc_rand_state;
void orc_rand_seed(orc_rand_state *s, unsigned seed);
int  orc_rand_next(orc_rand_state *s); /* 0 .. 2^31-1 */
/* One call of sample_next_token(): temperature softmax, qsort, top-k (draw discarded, renormalisation
 * kept), top-p.  Consumes two draws when top_k > 0 and top_p > 0. */
int orc_sample(const uint16_t *logits, int vocab, float temperature, int top_k, float top_p, orc_rand_state *s);

#ifdef __cplusplus
}
#endif
#endif
