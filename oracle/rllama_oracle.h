/*
 * rllama_oracle.h -- CPU restatement of rllama's per-token transformer forward path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls
 * this code.  Its callers are the parity tests, the smoke check and the CPU-baseline
 * leg of the benchmark, where it plays the role of "rllama's own CPU path".
 *
 * Every function names the lines of the reference (Noeda/rllama, paths relative to
 * the reference checkout) whose arithmetic it follows: the same fp32 lane order, the
 * same FMA/no-FMA choice, the same f16 rounding points.  It is compiled with
 * -ffp-contract=off so that only the explicit _mm256_fmadd_ps calls fuse, as in the
 * reference (rustc never contracts a*b+c on its own).
 *
 * Pinning status (which independent check covers which function) is listed in the
 * header comment of rllama_oracle.c.
 */
#ifndef RLLAMA_ORACLE_H
#define RLLAMA_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Tensor kinds: the weight names of transformer.rs:297-304, 405-412, 490-503, 595-614
 * and embedding.rs:18. */
enum {
    ORC_TOK_EMB = 0,   /* tok_embeddings.weight          [vocab x dim]  */
    ORC_WQ = 1,        /* layers.i.attention.wq.weight   [dim x dim]    */
    ORC_WK = 2,
    ORC_WV = 3,
    ORC_WO = 4,
    ORC_W1 = 5,        /* layers.i.feed_forward.w1.weight [ffn x dim]   */
    ORC_W2 = 6,        /* layers.i.feed_forward.w2.weight [dim x ffn]   */
    ORC_W3 = 7,        /* layers.i.feed_forward.w3.weight [ffn x dim]   */
    ORC_ATTN_NORM = 8, /* layers.i.attention_norm.weight  [dim]         */
    ORC_FFN_NORM = 9,  /* layers.i.ffn_norm.weight        [dim]         */
    ORC_NORM = 10,     /* norm.weight                     [dim]         */
    ORC_OUTPUT = 11    /* output.weight                   [vocab x dim] */
};

enum { ORC_F16 = 0, ORC_F32 = 1 };

typedef struct {
    int32_t dim;
    int32_t n_layers;
    int32_t n_heads;
    int32_t ffn_hidden;   /* read off w1's stored shape in the reference */
    int32_t vocab_size;
    int32_t max_seq_len;
    double  norm_eps;     /* RMSNorm.eps is f64, cast to f32 at use (transformer.rs:217, 477) */
    int32_t force_f16;    /* DataSettings::force_f16 (transformer.rs:105-108): --f16 */
} orc_params;

typedef struct orc_model orc_model;
typedef struct orc_caches orc_caches;

/* ---- scalar / vector building blocks (exported so tests can pin them) ---- */

/* half::f16::from_f32 / _mm256_cvtps_ph(a, 0): IEEE round-to-nearest-even (simd_support.rs:50-52,
 * tensor.rs:374-375).  Portable bit-manipulation version, and the F16C instruction version. */
uint16_t orc_f32_to_f16_bits(float v);
float    orc_f16_bits_to_f32(uint16_t h);
uint16_t orc_f32_to_f16_hw(float v);
float    orc_f16_to_f32_hw(uint16_t h);
void     orc_f32_to_f16_array(const float *src, uint16_t *dst, size_t n);   /* tensor.rs:2281-2314 */
void     orc_f16_to_f32_array(const uint16_t *src, float *dst, size_t n);   /* tensor.rs:2226-2279 */

/* horizontal_sum_f32x8 (simd_support.rs:97-105): ((a0+a4)+(a1+a5)) + ((a2+a6)+(a3+a7)). */
float orc_hsum8(const float a[8]);

/* dot8: 8 fp32 lanes, lane l accumulates k = l (mod 8) by FMA in increasing k, then hsum8.
 * This is the value every transposed-matmul kernel of the reference produces per output element
 * (tensor.rs:1351-1447 f32 tiled, 1577-1638 f16 tiled, 1870-1902 f32 GEMV, 1957-1979 gather). */
float orc_dot8_f32(const float *a, const float *b, int k);
float orc_dot8_f16(const uint16_t *a, const uint16_t *b, int k);
/* Same value computed with scalar fmaf() instead of AVX2, used to cross-check the intrinsics. */
float orc_dot8_f32_scalar(const float *a, const float *b, int k);

/* Tensor::matrix_mul_transposed (tensor.rs:999-1025 -> 1250-1666):
 * out[r*n_w + c] = dot8(x[r,:], w[c,:]); f16 variant rounds the result to f16 (tensor.rs:1623-1643)
 * and returns the f16 bits.  x: [n_x x k], w: [n_w x k], row-major, dense. */
void orc_matmul_transposed_f32(const float *x, int n_x, const float *w, int n_w, int k, float *out);
void orc_matmul_transposed_f16(const uint16_t *x, int n_x, const uint16_t *w, int n_w, int k, uint16_t *out);
/* Tensor::matrix_mul_inplace f32 (tensor.rs:1050-1115): per element a sequential-k FMA chain.
 * a: [m x k], b: [k x n] -> out [m x n]. */
void orc_matmul_f32_seqk(const float *a, int m, const float *b, int n, int k, float *out);
/* Tensor::vector_matrix_mul (tensor.rs:1923-1983): out[c] = dot8 over rows of b (gather). a: [k], b: [k x n]. */
void orc_vector_matrix_mul_f32(const float *a, const float *b, int k, int n, float *out);

/* RMSNorm::forward (transformer.rs:476-480) on one row. */
void orc_rmsnorm_row(const float *x, const float *w, int d, double eps, float *out);
/* Tensor::softmax (tensor.rs:479-494) on one row: no max subtraction, sequential sum. */
void orc_softmax_row(const float *s, int n, float *out);
/* Tensor::silu_cpu (tensor.rs:822-832). */
float orc_silu(float v);
/* compute_freqs_cis (transformer.rs:858-885): out[(pos*(hd/2)+j)*2 + {0,1}] = (cos, sin) in f64. */
void orc_freqs_cis(int head_dim, int max_seq_len, double theta, double *out);
/* apply_rotary_emb (transformer.rs:823-856) on one [n_heads x head_dim] row, in place. */
void orc_rope_row(float *x, int n_heads, int head_dim, const double *freqs_cis_at_pos);

/* TokenSampler::sample (token_sampler.rs:83-174) with top_k = 1, top_p = 1, repetition_penalty = 1:
 * returns the token id; *prob (may be NULL) receives its probability.  *n_ties (may be NULL)
 * receives how many ids share the top probability (the reference's sort_unstable_by does not
 * define which of them wins; this picks the lowest id). */
int32_t orc_sample_greedy(const float *logits, int vocab, float temperature, float *prob, int32_t *n_ties);
/* token_sampler.rs:83-174 in two halves: the candidate list after the top-k / top-p cuts, and the draw with the uniform variate passed in */
int32_t orc_sample_candidates(const float *logits, int vocab, float temperature, float top_p, int32_t top_k, float repetition_penalty,
                              const int32_t *existing_tokens, int32_t n_existing, int32_t *out_ids, float *out_probs, float *total_p);
int32_t orc_sample_pick(const int32_t *ids, const float *probs, int32_t n, float total_p, float u, float *prob);

/* ---- model level ---- */

void orc_set_threads(int n);   /* rayon pool size analogue (rllama_main.rs:148-157); results do not depend on it */
int  orc_get_threads(void);
/* 1: one-row f32 products (output head; w1/w2/w3 in f32 mode) run on one thread like tensor.rs:1837-1918. Timing only. */
void orc_set_reference_threading(int on);
/* Sensitivity probe (default off): the f16 projections sum their products in another valid fp32 order (not the reference's).
 * Measures how far the reference's own results move under a reordering of its additions. */
void orc_set_alt_order(int on);
/* Second probe (default off): every sum (dot products, RMSNorm's sum of squares, the softmax denominator) accumulated in float64
 * and rounded to f32 once; rounding points, element-wise steps and libm calls unchanged.  NOT the reference's values: the point
 * that the reference and every reordering of its fp32 additions scatter around. */
void orc_set_exact_sums(int on);

orc_model *orc_model_create(const orc_params *p);
void       orc_model_free(orc_model *m);
/* Stores one weight.  src is dense row-major [rows x cols] of src_dtype.  The reference loads every
 * tensor to f32 (tensor.rs:2467, 2538) and then, under force_f16, converts the seven projection
 * matrices to f16 (transformer.rs:508-512, 624-629); norms, embedding and the output head stay f32
 * (transformer.rs:468, 302-308; embedding.rs:41-47). Returns 0 on success. */
int orc_model_set_tensor(orc_model *m, int kind, int layer, const void *src, int rows, int cols, int src_dtype);

orc_caches *orc_caches_create(const orc_model *m);                 /* Transformer::make_caches transformer.rs:328-341 */
orc_caches *orc_caches_true_clone(const orc_caches *c);            /* TransformerCaches::true_clone :207-213 */
void        orc_caches_shift_left(orc_caches *c, int shifts);      /* TransformerCaches::shift_left :201-205 */
void        orc_caches_free(orc_caches *c);
/* Copies cache contents of (layer, head) as f32 [head_dim x max_seq_len] (position along columns). which: 0 = K, 1 = V. */
void        orc_caches_read(const orc_caches *c, int layer, int head, int which, float *out);

/* Transformer::forward (transformer.rs:343-383). logits_out: vocab floats. Returns 0 on success,
 * nonzero where the reference would panic (n > 1 with start_pos > 0: mask shape mismatch, tensor.rs:576-584;
 * start_pos + n > max_seq_len). */
int orc_forward(const orc_model *m, orc_caches *c, const int32_t *tokens, int n, int start_pos, float *logits_out);

/* The same forward cut where the reference's layer split (percentage_to_gpu, transformer.rs:262-279) cuts it, so that a
 * test can run some blocks elsewhere: orc_embed is the gather of :361-367, orc_forward_layers the blocks
 * first_layer..=last_layer on a stream x_in [n x dim] (:368-376), orc_head the final norm and output head on the last
 * row (:378-381).  orc_embed -> orc_forward_layers(0..n_layers-1) -> orc_head is orc_forward bit for bit. */
int orc_embed(const orc_model *m, const int32_t *tokens, int n, float *x_out);
int orc_forward_layers(const orc_model *m, orc_caches *c, const float *x_in, int n, int start_pos, int first_layer, int last_layer, float *x_out);
int orc_head(const orc_model *m, const float *x, int n, float *logits_out);

/* Optional taps for debugging parity: if non-NULL, receives the residual stream [n x dim] after each layer
 * (n_layers * n * dim floats) of the most recent orc_forward call on this thread. */
void orc_set_layer_tap(float *buf);

#ifdef __cplusplus
}
#endif
#endif
