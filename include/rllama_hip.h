/*
 * rllama_hip.h -- C ABI of librllama_hip.so: rllama's per-token transformer forward path on one
 * MI355X (gfx950), weights and KV cache resident in HBM.
 *
 * This is the seam rllama's `opencl` Cargo feature occupies (Cargo.toml:42-44; Tensor.opencl_data,
 * src/tensor.rs:99-102; DataSettings, src/transformer.rs:38-109).  A Rust host binds these symbols
 * from an `extern "C"` block; nothing here needs a C++ or torch type.
 *
 * Conventions
 *   - every function returns 0 on success or a nonzero rlh_status; rlh_last_error() gives the text of
 *     the calling thread's most recent failure (the reference's OpenCLError strings,
 *     src/tensor_opencl_support.rs:77-83, play this role);
 *   - handles are opaque; a handle belongs to the context that made it;
 *   - all calls on one context are serialised by the library (the reference serialises on a
 *     `programs.write()` lock and one in-order queue, src/tensor_opencl_support.rs:120, :322), so
 *     handles may be shared between threads (DataSettings is Send + Sync, src/transformer.rs:52-53).
 *     One piece of state is per model, not per call: the sampled id that rlh_decode_greedy continues
 *     from, so a greedy call on other caches in between (from any thread) makes it refuse;
 *   - host pointers are only read/written during the call unless stated otherwise;
 *   - there is no CPU fallback: without a usable HIP device rlh_init fails and nothing else works.
 *
 * Citations `file:line` are into the reference checkout (Noeda/rllama).
 */
#ifndef RLLAMA_HIP_H
#define RLLAMA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    RLH_OK = 0,
    RLH_ERR_INVALID = 1,      /* bad argument / shape; where the reference panics on a shape assert */
    RLH_ERR_NO_DEVICE = 2,    /* no HIP device / ordinal out of range (OpenCLError::OpenCLDeviceListError) */
    RLH_ERR_HIP = 3,          /* a HIP runtime call failed (OpenCLError::OpenCL) */
    RLH_ERR_OOM = 4,          /* device allocation failed */
    RLH_ERR_STATE = 5,        /* model not fully loaded, caches of another model, sequence too long ... */
    RLH_ERR_UNSUPPORTED = 6   /* arch is not gfx950, or a dtype the reference does not offload either */
} rlh_status;

typedef enum { RLH_F16 = 0, RLH_F32 = 1 } rlh_dtype;   /* TensorDType (src/tensor.rs:50-54) */

/* Weight names: src/transformer.rs:297-304, 405-412, 490-503, 595-614; src/embedding.rs:18 */
typedef enum {
    RLH_TOK_EMB = 0,     /* tok_embeddings.weight            [vocab x dim]  */
    RLH_WQ = 1,          /* layers.i.attention.wq.weight     [dim x dim]    */
    RLH_WK = 2,
    RLH_WV = 3,
    RLH_WO = 4,
    RLH_W1 = 5,          /* layers.i.feed_forward.w1.weight  [ffn x dim]    */
    RLH_W2 = 6,          /* layers.i.feed_forward.w2.weight  [dim x ffn]    */
    RLH_W3 = 7,          /* layers.i.feed_forward.w3.weight  [ffn x dim]    */
    RLH_ATTN_NORM = 8,   /* layers.i.attention_norm.weight   [dim]          */
    RLH_FFN_NORM = 9,    /* layers.i.ffn_norm.weight         [dim]          */
    RLH_NORM = 10,       /* norm.weight                      [dim]          */
    RLH_OUTPUT = 11      /* output.weight                    [vocab x dim]  */
} rlh_tensor_kind;

typedef struct rlh_ctx rlh_ctx;
typedef struct rlh_model rlh_model;
typedef struct rlh_caches rlh_caches;
typedef struct rlh_tensor rlh_tensor;
typedef struct rlh_event rlh_event;

/* ------------------------------------------------------------------------------------------------
 * Context.  Replaces OpenCL::new(verbose, nth_device) (src/tensor_opencl_support.rs:86-128), called
 * from src/rllama_main.rs:182-199.  Fails (no fallback) if the ordinal does not name a gfx950 device.
 * ---------------------------------------------------------------------------------------------- */
int  rlh_init(int device_ordinal, int verbose, rlh_ctx **out);
void rlh_shutdown(rlh_ctx *ctx);
/* OpenCL::flush (src/tensor_opencl_support.rs:130) / Tensor::finish (src/tensor.rs:2198-2206): returns
 * when all work queued on the context has completed. */
int  rlh_sync(rlh_ctx *ctx);
const char *rlh_last_error(void);
/* The library's switches (no reference counterpart: the reference has compile-time features only, Cargo.toml:42-44).
 * rlh_init reads RLLAMA_HIP_<NAME> from the environment once per context; nothing reads the environment afterwards, and
 * this call is the only other way to change a switch: name = NAME without the prefix ("GEMM_DUAL", "ATTN_MERGE", ...),
 * value = what the variable would hold, NULL = back to the default.  Waits for the context's queued work first; applies to
 * every later call on the context.  Unknown names and unusable values are RLH_ERR_INVALID. */
int  rlh_set_option(rlh_ctx *ctx, const char *name, const char *value);
/* Device facts for reports: name (<= cap bytes incl. NUL), compute units, total HBM bytes. */
int  rlh_device_info(rlh_ctx *ctx, char *name, int cap, int *compute_units, uint64_t *hbm_bytes);

/* ------------------------------------------------------------------------------------------------
 * Model.  Replaces Transformer::from_unpickled (src/transformer.rs:242-326) + the per-tensor
 * to_f16()/to_gpu_inplace() calls (src/transformer.rs:508-525, 624-644).
 * ---------------------------------------------------------------------------------------------- */
typedef struct {
    int32_t dim;                /* params.json "dim"        (src/model_params.rs:3-14) */
    int32_t n_layers;           /* "n_layers" */
    int32_t n_heads;            /* "n_heads"; dim % n_heads == 0 (src/transformer.rs:252) */
    int32_t ffn_hidden;         /* rows of w1 as stored; not a params.json field */
    int32_t vocab_size;         /* "vocab_size" */
    int32_t max_seq_len;        /* --max-seq-len (src/rllama_main.rs:247): RoPE table and cache length */
    double  norm_eps;           /* "norm_eps" */
    int32_t force_f16;          /* --f16, DataSettings::force_f16 (src/transformer.rs:105-108): 1 = f16
                                   projection weights, f16 KV cache and the f16 rounding points of
                                   src/transformer.rs:665-668, 537-540, 563-565, 795;
                                   0 = f32 weights, f32 KV cache, no rounding anywhere */
    float   percentage_to_gpu;  /* --percentage-to-gpu; clamped like src/transformer.rs:91-103.  1.0 (the
                                   reference's default): every layer is resident.  Below 1.0 only layers
                                   0..=round(p * (n_layers - 1)) get weights and cache planes on the device
                                   (src/transformer.rs:262-279): see rlh_forward_layers */
} rlh_model_params;

int  rlh_model_create(rlh_ctx *ctx, const rlh_model_params *params, rlh_model **out);
void rlh_model_free(rlh_model *model);
/* Copies one weight from host memory into HBM.  `host` is dense row-major [rows x cols] of src_dtype
 * (f16 = IEEE binary16 bits, as in consolidated.NN/data/<k>; src/tensor.rs:2498-2538).  Norm vectors
 * are [1 x dim].  layer is ignored for TOK_EMB / NORM / OUTPUT.  Under force_f16 an f32 source is
 * rounded to f16 like Tensor::to_f16 (src/tensor.rs:2281-2314).  The host buffer is free on return. */
int  rlh_model_set_tensor(rlh_model *model, int kind, int layer, const void *host, int rows, int cols, int src_dtype);
/* Reads a stored weight back as dst_dtype [rows x cols]: RLH_F32 gives what Tensor::to_f32 of it would hold,
 * RLH_F16 the IEEE binary16 bits (exact for f16 storage, Tensor::to_f16 rounding for f32 storage). */
int  rlh_model_get_tensor(rlh_model *model, int kind, int layer, void *host_out, int rows, int cols, int dst_dtype);
/* Fills every weight on the device from the counter-based generator in synth.h: projection matrices,
 * embedding and head i.i.d. N(0, std^2) rounded to f16, norm weights 1.0.  Bit-identical to
 * rlh_synth_normal_f16 on the host.  (No reference counterpart: the reference only loads files.) */
int  rlh_model_fill_synthetic(rlh_model *model, uint64_t seed, double std);
/* How a multi-token forward (n > 1 at start_pos == 0, src/transformer.rs:343-383) is executed.  0 (default): every
 * projection as one matrix-core GEMM over all n rows and attention as batched GEMMs around a causal softmax
 * (f16 mode: f16 matrix cores with the reference's rounding points; f32 mode: fp32 matrix cores, no rounding points,
 * when dim, ffn_hidden and head_dim are multiples of 32, else mode 1).  1: token by token with the decode kernels.
 * Both give the reference's result up to the order of fp32 additions. */
int  rlh_model_set_prefill_mode(rlh_model *model, int mode);
/* The layer split rule of src/transformer.rs:262-279: last_layer_on_gpu = round(p * (n_layers - 1)).
 * Layers beyond it have no device storage: rlh_model_set_tensor / get_tensor / rlh_caches_read refuse them. */
int  rlh_model_layers_on_gpu(const rlh_model *model, int *last_layer_on_gpu);
/* Bytes of HBM one decode step must read at sequence length T: weights + KV (the roofline's numerator); of the resident
 * layers only, and without the head, for a model split by percentage_to_gpu. */
int  rlh_model_decode_bytes(const rlh_model *model, int T, uint64_t *bytes);

/* ------------------------------------------------------------------------------------------------
 * KV caches.  TransformerCaches / AttentionCache (src/transformer.rs:111-214).
 * ---------------------------------------------------------------------------------------------- */
int  rlh_caches_create(rlh_model *model, rlh_caches **out);                 /* make_caches :328-341 (zero filled) */
int  rlh_caches_true_clone(const rlh_caches *src, rlh_caches **out);        /* true_clone  :207-213 */
int  rlh_caches_shift_left(rlh_caches *caches, int shifts);                 /* shift_left  :201-205 */
void rlh_caches_free(rlh_caches *caches);
/* Test hook: (layer, head) cache contents as f32 [head_dim x max_seq_len], position along columns, the
 * reference's own orientation (src/transformer.rs:143-154).  which: 0 = K, 1 = V. */
int  rlh_caches_read(const rlh_caches *caches, int layer, int head, int which, float *host_out);

/* ------------------------------------------------------------------------------------------------
 * Forward.  Transformer::forward(tokens, start_pos, caches) -> logits[vocab] (src/transformer.rs:343-383).
 * Valid calls are the reference's: any n >= 1 at start_pos == 0, n == 1 at start_pos > 0 (the mask of
 * :350-357 only fits start_pos == 0), start_pos + n <= max_seq_len.  logits_out: vocab floats on the host.
 * ---------------------------------------------------------------------------------------------- */
int  rlh_forward(rlh_model *model, rlh_caches *caches, const int32_t *tokens, int n, int start_pos, float *logits_out);
/* The transformer blocks first_layer..=last_layer alone, for a model split by percentage_to_gpu (the loop body of
 * src/transformer.rs:361-376 over the layers whose DataSettings kept use_opencl, :262-279).  x_in: the n rows of
 * the residual stream entering first_layer, host f32 [n x dim] (for layer 0 the embedding rows, which the
 * reference gathers on the host, src/transformer.rs:344-348, src/embedding.rs:41-58).  x_out: the stream
 * leaving last_layer, same shape (may alias x_in).  The cache planes of those layers are filled at
 * start_pos..start_pos+n.  Everything else of the forward — the host-side blocks, the final norm and the output
 * head, which the reference keeps as host tensors (src/transformer.rs:296-308) — stays with the caller's own code:
 * this library has no host arithmetic.  Same call rules as rlh_forward; also valid on a whole model for any span.
 * rlh_forward* and the generate loops refuse a split model (RLH_ERR_STATE). */
int  rlh_forward_layers(rlh_model *model, rlh_caches *caches, const float *x_in, int n, int start_pos, int first_layer, int last_layer,
                        float *x_out);
/* forward + TokenSampler::sample with top_k = 1, temperature = 1, repetition_penalty = 1
 * (src/token_sampler.rs:83-174; its loops over 0..logits.rows() only ever touch token 0, whose logit
 * becomes 0.0): the argmax runs on the device, only the id crosses PCIe. */
int  rlh_forward_greedy(rlh_model *model, rlh_caches *caches, const int32_t *tokens, int n, int start_pos, int32_t *next_token);
/* The token loop of command_line_inference (src/rllama_main.rs:821-897) at top_k = 1: one forward over
 * the prompt, then one single-token forward per new token, each fed the previous argmax on the device.
 * out_tokens receives n_new ids.  ms_first / ms_per_token (may be NULL) are measured with HIP events
 * on the launch stream and follow src/rllama_main.rs:890-894, 908-917 (first call apart, then the mean
 * over the remaining steps). */
int  rlh_generate_greedy(rlh_model *model, rlh_caches *caches, const int32_t *prompt, int n_prompt, int n_new,
                         int32_t *out_tokens, float *ms_first, float *ms_per_token);

/* Continues the greedy token loop from where rlh_forward_greedy / rlh_generate_greedy / rlh_decode_greedy left
 * it (the last sampled id and its position are still on the device): n_steps further single-token forwards,
 * no host round trip in between.  out_tokens receives n_steps ids; ms_total (may be NULL) is the HIP-event
 * time of the n_steps steps on the launch stream. */
int  rlh_decode_greedy(rlh_model *model, rlh_caches *caches, int n_steps, int32_t *out_tokens, float *ms_total);

/* TokenSampler (src/token_sampler.rs:6-11).  rlh_sampler_default fills in TokenSampler::new()'s values
 * (:20-29: temperature 0.2, top_p 1.0, top_k 1, repetition_penalty 0.8). */
typedef struct rlh_sampler_params {
    float temperature;          /* logits are multiplied by 1 / temperature when it is > 0 (:99-102) */
    float top_p;
    int32_t top_k;
    float repetition_penalty;   /* 1.0 = none */
} rlh_sampler_params;
void rlh_sampler_default(rlh_sampler_params *p);

/* TokenSampler::sample up to the random draw (src/token_sampler.rs:83-159), host arithmetic on host logits (needs no
 * device): the candidates that survive the top-k and top-p cuts, in the order the draw walks them, with their softmax
 * probabilities; *total_p is their mass.  The reference's loops over "rows" of the transposed logits touch only token 0
 * (:105, :113, :121): only token 0 is penalised, and its logit ends up as 0; nothing else has a maximum subtracted.
 * Equal probabilities are ordered by ascending id.  out_ids / out_probs hold `cap` entries; more candidates than
 * that is RLH_ERR_INVALID.  existing_tokens may be NULL when n_existing is 0. */
int  rlh_sample_candidates(const float *logits, int vocab, const rlh_sampler_params *p, const int32_t *existing_tokens, int n_existing,
                           int32_t *out_ids, float *out_probs, int cap, int *n_out, float *total_p);
/* The whole of TokenSampler::sample (:83-174) with the uniform variate passed in: u in [0, 1] stands for
 * rng.gen_range(0.0..=total_p) / total_p.  *prob (may be NULL) = the chosen probability / total_p. */
int  rlh_sample(const float *logits, int vocab, const rlh_sampler_params *p, const int32_t *existing_tokens, int n_existing, float u,
                int32_t *token, float *prob);
/* forward + sample: the body of the reference's token loop (src/rllama_main.rs:846-860).  With top_k == 1 the choice is
 * made by the device argmax (no logits leave the device) and *prob is 1. */
int  rlh_forward_sample(rlh_model *model, rlh_caches *caches, const int32_t *tokens, int n, int start_pos, const rlh_sampler_params *p,
                        const int32_t *existing_tokens, int n_existing, float u, int32_t *token, float *prob);

/* ------------------------------------------------------------------------------------------------
 * Op level.  Mirrors OpenCLTensor (src/tensor_opencl_support.rs:134-405) so that a host Tensor can
 * offload single ops, and so that each kernel can be checked alone.  Tensors are dense row-major.
 * ---------------------------------------------------------------------------------------------- */
/* OpenCL::data_u16_to_gpu (:134-169), generalised to f32.  cols_capacity = row stride of the HOST buffer in
 * elements (src/tensor.rs:192-222); the device copy is dense. */
int  rlh_tensor_upload(rlh_ctx *ctx, const void *host, int rows, int cols, int cols_capacity, int dtype, rlh_tensor **out);
int  rlh_tensor_alloc(rlh_ctx *ctx, int rows, int cols, int dtype, rlh_tensor **out);   /* zero filled */
/* OpenCLTensor::data_u16_from_gpu (:198-212): asynchronous read; *ev (may be NULL = wait inside) must be
 * waited on before `host` is read.  Host row stride = cols_capacity. */
int  rlh_tensor_download(rlh_tensor *t, void *host, int cols_capacity, rlh_event **ev);
void rlh_tensor_free(rlh_tensor *t);
int  rlh_tensor_shape(const rlh_tensor *t, int *rows, int *cols, int *dtype);
int  rlh_event_wait(rlh_event *ev);                               /* OpenCLEvent::wait (:409-411); frees the event */
/* HIP-event timing on the launch stream (for measurements). */
int  rlh_event_record(rlh_ctx *ctx, rlh_event **out);
int  rlh_event_elapsed_ms(rlh_event *start, rlh_event *stop, float *ms);   /* waits for stop */
void rlh_event_free(rlh_event *ev);

int  rlh_copy_inplace(rlh_tensor *dst, const rlh_tensor *src);                       /* :215-232 */
int  rlh_transpose_from(rlh_tensor *dst, const rlh_tensor *src);                     /* :234-256 */
int  rlh_hadamard_product_inplace(rlh_tensor *dst, const rlh_tensor *src);           /* :258-281; f16: result rounded to f16 */
int  rlh_silu_inplace(rlh_tensor *t);                                                /* :283-299 */
/* OpenCLTensor::matrix_mul_inplace_transposed(self, src, other) (:301-405): dst[r, c] = sum_k src[r, k] * other[c, k].
 * src [n x k], other [m x k], dst [n x m].  f16 operands give an f16-rounded dst (as src/tensor.rs:1623-1643);
 * f32 operands give f32.  src and other must share a dtype; dst has it too.  n == 1 takes the GEMV kernel,
 * n > 1 the MFMA GEMM (f16) or the tiled fp32 kernel.  The first call with n > 1 on a context allocates a 64 MiB workspace
 * that stays with the context (partial sums of products cut along K, as inside the forward; rlh_ffn_gate shares it). */
int  rlh_matrix_mul_inplace_transposed(rlh_tensor *dst, const rlh_tensor *src, const rlh_tensor *other);
/* Decode GEMV with the rounding switches of the fused path: y[c] = sum_k x[k] * W[c, k]; x f32 [1 x k]
 * (rounded to f16 first if round_x), W f16 or f32 [m x k], y f32 [1 x m] (rounded to f16 precision if round_y). */
int  rlh_gemv(rlh_tensor *y, const rlh_tensor *w, const rlh_tensor *x, int round_x, int round_y);
/* RMSNorm::forward (src/transformer.rs:476-480) per row; x, y f32 [n x d], w f32 [1 x d]; round_y = f16 rounding point. */
int  rlh_rmsnorm(rlh_tensor *y, const rlh_tensor *x, const rlh_tensor *w, double eps, int round_y);
/* apply_rotary_emb (src/transformer.rs:823-856) on one [n_heads x head_dim] f32 row at position pos, in place. */
int  rlh_rope_inplace(rlh_tensor *x, int n_heads, int head_dim, int pos);

/* The steps of the attention block and of the token loop that the reference runs on the host (its OpenCL backend has no
 * call for them); here they are device kernels of the forward, exported one by one so that each can be checked alone.
 * "Cache planes" are one layer's K and V cache as the forward holds them: two tensors [n_heads * max_seq_len x head_dim]
 * of one dtype (f16 or f32), row h * max_seq_len + t = head h, position t -- the transpose of the reference's per-head
 * [head_dim x max_seq_len] (src/transformer.rs:143-154).  head_dim is 16, 32, 64 or 128. */
/* Tensor::add (src/tensor.rs:573-593) as the residual adds use it (src/transformer.rs:442, 445): dst = a + b, f32. */
int  rlh_add(rlh_tensor *dst, const rlh_tensor *a, const rlh_tensor *b);
/* FeedForward's gate (src/transformer.rs:557-565): dst = silu(gate) * up, formed in f32 (src/tensor.rs:822-832, 722-734);
 * f16 tensors are read as f16, and the f32 product is rounded to f16 (the one rounding point). */
int  rlh_silu_mul(rlh_tensor *dst, const rlh_tensor *gate, const rlh_tensor *up);
/* FeedForward up to its gate for several rows at once, f16 mode (src/transformer.rs:551-565 with seq_len > 1):
 * dst = f16(silu(f16(x * w1^T)) * f16(x * w3^T)); x [n x k], w1 and w3 [m x k], dst [n x m], all f16, k a multiple of 8.
 * Where the shape fills the part, both products run as one matrix-core pass over x with two accumulator sets and the gate
 * never reaches memory; otherwise as two products, the second consuming the first (same bits either way). */
int  rlh_ffn_gate(rlh_tensor *dst, const rlh_tensor *x, const rlh_tensor *w1, const rlh_tensor *w3);
/* One token's cache update (src/transformer.rs:704-761 with seq_len 1): RoPE on q (in place) and on k at position pos,
 * then k and v into the cache planes at pos (rounded to f16 for f16 planes).  q, k, v: f32, n_heads * head_dim elements. */
int  rlh_rope_kvwrite(rlh_tensor *q, const rlh_tensor *k, const rlh_tensor *v, rlh_tensor *cache_k, rlh_tensor *cache_v, int n_heads,
                      int max_seq_len, int pos);
/* Single-query attention over positions 0..T-1 of the cache planes (src/transformer.rs:762-781 with seq_len 1: scores
 * src/tensor.rs:1923-1983, softmax :479-494, P.V :1282-1475): out = softmax(q K^T / sqrt(head_dim)) V per head.
 * q (after RoPE) and out: f32, n_heads * head_dim elements; round_out = the f16 rounding point before wo (:793-796).
 * n_splits: blocks per head the positions are shared between, 1..64; 0 = the forward's own choice for T.
 * The softmax subtracts the running maximum: equal to the reference's exp(s) / sum exp(s) wherever that is finite, and
 * finite where the reference overflows to NaN (scores above ln(FLT_MAX)). */
int  rlh_attn_decode(rlh_tensor *out, const rlh_tensor *q, const rlh_tensor *cache_k, const rlh_tensor *cache_v, int n_heads, int max_seq_len,
                     int T, int n_splits, int round_out);
/* rlh_attn_decode for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and bit-identical
 * results, but the work memory (arrival counters, the position word and the partial triples of a split sequence) is a
 * static device array of 4 MiB + 4.25 KiB inside the library, which every GPU the library runs on holds until the process
 * ends; rlh_init looks its address up once per device.  Nothing is allocated or freed by the call (no hipMalloc, no
 * hipFree, no memset node: the counters are cleared by a small fill kernel).  Limits: n_heads * n_splits * (head_dim + 2)
 * <= 1,048,576 floats (e.g. 64 heads of 128 dims with 64 splits need 532,480), else RLH_ERR_UNSUPPORTED.  All calls on one
 * GPU share the array, which keeps the last call's contents: calls that overlap on one GPU (two contexts on the same
 * device, or a captured graph replayed while another call runs) race. */
int  rlh_attn_decode_noalloc(rlh_tensor *out, const rlh_tensor *q, const rlh_tensor *cache_k, const rlh_tensor *cache_v, int n_heads,
                             int max_seq_len, int T, int n_splits, int round_out);
/* The attention block of a multi-token forward at start_pos 0 between the projections and wo (src/transformer.rs:704-796):
 * RoPE on the q and k columns of qkv, k and v into the cache planes at positions 0..n-1, causal attention per head, heads
 * concatenated and rounded to f16.  qkv: f16 [n x 3 dim] (columns [0, dim) wq's output, [dim, 2 dim) wk's, [2 dim, 3 dim)
 * wv's); out: f16 [n x dim]; f16 cache planes; head_dim 64 or 128 (the one-kernel matrix-core form). */
int  rlh_attn_prefill(rlh_tensor *out, const rlh_tensor *qkv, rlh_tensor *cache_k, rlh_tensor *cache_v, int n_heads, int max_seq_len);
/* TokenSampler::sample with top_k = 1 (src/token_sampler.rs:83-174) on device logits (an f32 vector), as the greedy
 * entry points run it: logits * (1 / temperature) when temperature > 0 (:99-102), token 0's value becomes 0 (:112-123),
 * un-shifted softmax, first of the descending probabilities with NaN last (:124-147).  While the softmax sum is finite that
 * is the largest scaled logit (lowest id among equal ones); once it is not (a scaled logit above ln(FLT_MAX), a NaN, or
 * the sum itself overflowing) every probability is 0 or NaN and the pick is token 0. */
int  rlh_argmax_greedy(const rlh_tensor *logits, float temperature, int32_t *token);

/* ------------------------------------------------------------------------------------------------
 * Measurement aids (no reference counterpart; src/benches/benchmark.rs times the CPU/OpenCL ops with criterion).
 * Both time `iters` back-to-back launches with HIP events on the launch stream.
 * ---------------------------------------------------------------------------------------------- */
/* One kernel of the token step, cycling through the layers so that every launch streams different weights.
 * which: 0 = attention_norm + wq|wk|wv + RoPE + cache write, 1 = single-query attention at sequence length T,
 * 2 = wo + residual, 3 = ffn_norm + w1|w3 + SiLU*gate, 4 = w2 + residual, 5 = final norm + output head.
 * bytes_per_launch (may be NULL): the algorithmic bytes of one launch (weights once + vectors).
 * The launches use the model's token-step state and activation buffers as they are and leave them overwritten (position
 * T - 1, a fixed token id), and which = 0 writes the K / V rows of position T - 1 of every layer of `caches`: use caches
 * made for the measurement.  A greedy loop in progress is ended (rlh_decode_greedy refuses until the next
 * rlh_forward_greedy / rlh_generate_greedy). */
int  rlh_model_time_kernel(rlh_model *model, rlh_caches *caches, int which, int T, int iters, float *us_per_launch,
                           uint64_t *bytes_per_launch);
/* Isolated GEMV y = W x, W [rows x k] of w_dtype, x f32, cycling through n_buffers distinct weight buffers
 * (choose n_buffers * rows * k * elem size well above the 256 MB last-level cache). */
int  rlh_time_gemv(rlh_ctx *ctx, int rows, int k, int w_dtype, int round_x, int round_y, int n_buffers, int iters,
                   float *us_per_launch);

/* Where the fixed cost of a GEMV launch is spent: `launches` back-to-back launches of the isolated product (as rlh_time_gemv,
 * f16 weights, n_buffers distinct matrices) in which every wavefront reads the 100 MHz wall clock at kernel entry, when the
 * activation vector is staged, behind its first and its last burst of weights, and at exit.  out_us receives 8 means over
 * the launches after the first, in microseconds: [0] first wavefront of a launch enters after the last wavefront of the
 * previous launch left (the gap between dependent kernels on the device), [1] last wavefront enters after the first one
 * (dispatch ramp), [2] entry -> x staged (prologue, mean over wavefronts), [3] x staged -> first burst consumed (first-byte
 * latency, mean), [4] first -> last burst consumed (streaming, mean), [5] last burst -> exit (epilogue, mean), [6] first
 * wavefront to leave -> last wavefront to leave (tail skew), [7] first entry -> last exit (the launch as the device sees it). */
int  rlh_probe_gemv_phases(rlh_ctx *ctx, int rows, int k, int n_buffers, int launches, float *out_us);

/* ------------------------------------------------------------------------------------------------
 * Synthetic inputs (host side; usable without a device).  See synth.h.
 * ---------------------------------------------------------------------------------------------- */
void rlh_synth_normal_f16(uint64_t seed, int kind, int layer, uint64_t first_index, uint64_t count, double std, uint16_t *out);
void rlh_synth_tokens(uint64_t seed, uint64_t first_index, uint64_t count, int32_t lo, int32_t hi, int32_t *out);

/* ABI version of this header. */
int  rlh_abi_version(void);
#define RLH_ABI_VERSION 1

#ifdef __cplusplus
}
#endif
#endif
