// kernels.h -- host-side launch interface of the gfx950 kernels (internal to librllama_hip.so).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace rlh {

enum GemvEpilogue {
    kEpiStore = 0,   // y[c] = v
    kEpiRopeKv = 2,  // fused wq|wk|wv: RoPE on q and k, q -> y, k/v -> KV cache at *pos
    kEpiSilu = 3,    // two matrices (w1, w3): y[c] = silu(v1) * v3   (transformer.rs:561-562)
    kEpiStoreArgmax = 4 // y[c] = v, and the greedy pick over all rows (TokenSampler::sample at top_k = 1, temperature 1) in the same
                     // launch: the last workgroup to finish reduces the workgroups' candidates and advances the token-step
                     // state like argmax_advance_kernel (fp32 x only)
};

// Device-resident scalars of the token loop.  Kernels read them from memory so that a recorded
// sequence of launches can be replayed for the next token without new arguments.
struct DecodeState {
    int32_t pos;       // position of the token being processed (start_pos of transformer.rs:343)
    int32_t token;     // its id
    int32_t n_out;     // how many ids the argmax kernel has appended to out_tokens
    int32_t pad;
};

struct GemvParams {
    const void *w;            // [n_rows x k] row-major, f16 or f32
    const void *w_b;          // kEpiSilu: second matrix (w3), same shape
    const float *x;           // [k] f32
    const float *x_add;       // optional [k]: the product's input is x + x_add (the residual adds of
                              // transformer.rs:442, 445 happen in the consumer's prologue)
    float *x_out;             // optional [k]: block 0 stores x + x_add here (must not alias x or x_add)
    const float *norm_w;      // fused RMSNorm weight [k] or nullptr
    float eps;
    float *y;
    int n_rows;
    int k;
    int w_is_f16;             // weight storage
    int x_f16;                // 1: x (after the optional norm) is rounded to f16 before the product
    int round_y;              // 1: product rounded to f16 precision (tensor.rs:1623-1643)
    int stream_weights;       // 1: non-temporal weight loads
    int burst_fixed;          // 1: bursts of 8 loads whatever the row length (default: a length that divides the row where one is built)
    // kEpiRopeKv only
    const void *embed_table;  // optional [vocab x k], f16 or f32: the input row is row state->token of this table, widened to f32
                              // (x is then unused; x_out, if set, receives the row)
    int embed_f16;
    const DecodeState *state;
    int pos1_host;            // position + 1 where the host knows it (spares the kernel a dependent load), 0: read state->pos
    const float2 *freqs;      // [max_seq_len x head_dim/2] (cos, sin) as f32
    void *cache_k;            // this layer's K cache [n_heads x max_seq_len x head_dim]
    void *cache_v;
    int cache_f16;
    int dim;
    int head_dim;
    int max_seq_len;
    unsigned long long *stamps; // measurement launches only (launch_gemv_stamped): kGemvStamps wall-clock readings per wavefront
    // kEpiStoreArgmax only
    float *amax_ws;           // one 16-byte record per workgroup of the launch (gemv_argmax_ws_bytes)
    unsigned *amax_ticket;    // arrival counter, zero before the launch; the kernel leaves it zero
    DecodeState *state_rw;    // receives the pick: token = id, pos += 1, n_out += 1
    int32_t *out_tokens;      // optional: out_tokens[n_out] = id while n_out < out_cap
    int out_cap;
};

hipError_t launch_gemv(const GemvParams &p, int epilogue, hipStream_t s);
// bytes of dynamic LDS launch_gemv will request for a given k (for capability checks)
size_t gemv_lds_bytes(int k, int w_is_f16, int x_f16);
// bytes of GemvParams::amax_ws that any launch can need
size_t gemv_argmax_ws_bytes();
// The plain product (kEpiStore, f16 weights, fp32 x) with every wavefront recording the 100 MHz wall clock at kernel entry,
// when x is staged, behind its first and its last burst, and at exit, into p.stamps [wavefronts of the grid][5]
// (*n_waves receives their number): where the fixed cost of a launch is spent.
hipError_t launch_gemv_stamped(const GemvParams &p, hipStream_t s, int stamps_capacity_waves, int *n_waves);

struct AttnDecodeParams {
    const float *q;           // [n_heads x head_dim] f32 (after RoPE)
    const void *cache_k;      // this layer: [n_heads x max_seq_len x head_dim]
    const void *cache_v;
    int cache_f16;
    const DecodeState *state; // T = state->pos + 1 ...
    int pos_host;             // ... unless the host knows the position (>= 0): saves the kernel a dependent load
    int n_heads;
    int head_dim;
    int max_seq_len;
    int n_splits;             // grid.y: blocks per head, each covering an equal share of the T positions
    float *out;               // [n_heads x head_dim]
    int round_out;            // f16 rounding point before wo (transformer.rs:793-796)
    float *workspace;         // [n_heads x n_splits x (head_dim + 2)] partial (max, sum, weighted V), needed when n_splits > 1
    unsigned *tickets;        // [n_heads] arrival counters, needed when n_splits > 1 and the merge runs inside the kernel;
                              // zero before the launch, and the kernel leaves them zero
    int merge_mode;           // 0: a second small kernel merges the partial results; 2: the last block of a head to finish
                              // merges them (partial results stored and loaded at device scope)
    int chunk_hint;           // upper bound of the positions one block covers (sizes the loads in flight); 0 = unknown
    int lds_stage;            // 1: K / V tiles staged in LDS first (comparison variant; needs pos_host, an f16 cache, head_dim 64 / 128)
};

hipError_t launch_attn_decode(const AttnDecodeParams &p, hipStream_t s);
size_t attn_decode_workspace_floats(int n_heads, int head_dim, int n_splits);
constexpr int kAttnDecodeMaxSplits = 64;

// What becomes of the wq|wk|wv product of a multi-token forward (prefill.hip; as an epilogue: gemm_dma.hip)
struct PrefillRopeParams {
    const void *qkv;        // [n x 3 dim] f16
    const float2 *freqs;    // [max_seq_len x head_dim/2]
    void *q_hi, *q_lo;      // [n_heads][n] rows of head_dim f16, q_stride halves apart
    void *cache_k, *cache_v; // this layer: [n_heads][max_seq_len][head_dim]
    int cache_f16;
    void *v_t;              // [n_heads][head_dim][t_pad] f16
    int n, dim, head_dim, max_seq_len, t_pad;
    int q_stride;
    int vt_swap;            // 1: positions within v_t rows have bits 2 and 3 swapped (the order attn_prefill_kernel reads)
};

// ---- prefill: C = A * B^T on the matrix cores (gemm.hip) ----
enum GemmEpilogue {
    kGemmEpiF16 = 0,        // C f16 = round(acc)                      (projection outputs, tensor.rs:1623-1643)
    kGemmEpiF32 = 1,        // C f32 = acc, or += acc when accumulate  (attention scores / P.V partial products)
    kGemmEpiResAddF32 = 2,  // C f32 = residual + f16r(acc)            (wo and w2 followed by transformer.rs:442 / :445)
    kGemmEpiSiluGateF16 = 3, // C f16 = round(silu(gate) * f16r(acc))  (w3 with w1's f16 output as the gate: transformer.rs:557-565)
    kGemmEpiRopeQkv = 4     // fast path only: the f16-rounded [m x 3 dim] product of wq|wk|wv is not stored; RoPE on its q and k
                            // columns, q as hi + lo halves, k and v into the cache, v transposed (GemmParams::rope; what
                            // rope_kv_prefill_tiled_kernel does with the stored product: transformer.rs:704-761)
};

// Switches of the prompt-path products; all zero = the launchers' own choices.  They come from the context (parsed from the
// environment once, when the context is made; rlh_set_option changes them), never from the environment at launch time.
struct GemmTune {
    int tile_plus1;       // GEMM_TILE=0..3 forces the tile (128x128, 256x128, 256x192, 256x256): stored as tile + 1
    int split_k;          // GEMM_SPLIT_K=N forces N K-pieces for the products that qualify for a cut along K
    int no_split_half;    // GEMM_SPLIT_HALF=0: cut along K only when the tiles cover at most a quarter of the compute units
    int dual_plus1;       // GEMM_DUAL=0..5: w1 and w3 in one pass never (0) / in that form wherever the kernel can run: stored as mode + 1
    int no_dual_cut;      // GEMM_DUAL_CUT=0: the one-pass w1|w3 product always covers all columns
    int no_rope_epilogue; // GEMM_ROPE=0: RoPE, q hi/lo, cache rows and V^T as a kernel of their own on the stored wq|wk|wv product
    int no_finish_norm;   // FINISH_NORM=0: the RMSNorm after a split wo / w2 product as a kernel of its own
    int no_kgroup;        // GEMM_KGROUP=0: 128x128 products stay on the kernel whose wavefronts split the tile
};

struct GemmParams {
    const _Float16 *a;      // [m x k], row stride lda
    const _Float16 *b;      // [n x k], row stride ldb
    void *c;                // [m x n], row stride ldc
    const float *residual;  // kGemmEpiResAddF32: [m x n], row stride ldc
    const _Float16 *gate;   // kGemmEpiSiluGateF16: [m x n], row stride ldc
    const _Float16 *b2;     // kGemmEpiSiluGateF16, fast path, instead of gate: a second [n x k] matrix (row stride ldb); the gate is
                            // f16(a * b^T), computed in the same pass, and C = SiLU(gate) * f16(a * b2^T) (gemm_f16_dual_gate_supported)
    int m, n, k;
    int lda, ldb, ldc;
    int batch;              // grid.z; element strides between batch items:
    size_t stride_a, stride_b, stride_c;
    int accumulate;         // kGemmEpiF32 only
    // fast path only (gemm_dma.hip); 0 = off:
    int k_seg;              // K is made of K / k_seg segments: A's k index runs through all of them, B's wraps (k % k_seg).
                            // Sums sum_s A_s * B^T in one pass (A = [hi | lo] halves of an fp32 operand against one B).
    int causal;             // 1: C tiles that lie entirely above the diagonal (col > row) are skipped, not written
                            // 2: of every segment only k < (last row of the C tile) + 1, rounded up to the K-tile, is used
                            //    (A holds zeros beyond the diagonal: causal probabilities times V)
    int split_k;            // set by the launcher only: grid.z = K ranges of one product (see gemm_dma.hip)
    void *workspace;        // optional, for split-K partial sums: fp32 [pieces][m][n rounded up to 4]; without it products run unsplit
    size_t workspace_bytes;
    int f32_operands;       // 1: a and b point to fp32 data (f32 mode); m, n, k, lda, ldb, strides and k_seg count elements
                            //    all the same.  Needs k % 32 == 0 and the kGemmEpiF32 epilogue.
    // Optional (kGemmEpiResAddF32, fast path): the RMSNorm that follows the residual add (transformer.rs:443 after :442, :432 of
    // the next block after :445).  Where the launcher adds up split-K partial sums anyway, that kernel also writes
    // norm_out = f16(rmsnorm(C row) * norm_w) and sets *norm_done = 1 at launch; otherwise it leaves both alone and the
    // caller runs the norm kernel itself.  Same arithmetic, same order of additions either way.
    const float *norm_w;    // [n]
    _Float16 *norm_out;     // [m x n], row stride n
    float norm_eps;
    int *norm_done;         // host flag
    GemmTune tune;          // the context's switches (zero = defaults)
    PrefillRopeParams rope; // kGemmEpiRopeQkv: the destinations (qkv unused; n = m, 3 dim = n, f16 cache, vt_swap as the reader expects)
};

hipError_t launch_gemm_f16(const GemmParams &p, int epilogue, hipStream_t s);
// fast path (gemm_dma.hip): k % 32 == 0; launch_gemm_f16 picks it when it applies
bool gemm_f16_dma_supported(const GemmParams &p);
hipError_t launch_gemm_f16_dma(const GemmParams &p, int epilogue, hipStream_t s);
// whether the fast path runs w1 and w3 of a feed-forward block (b, b2: both [n x k]) as one pass over A for this shape
bool gemm_f16_dual_gate_supported(const GemmParams &p);
// small output tiles per compute unit (gemm_kgroup.hip): wavefronts split the K-steps instead of the tile; launch_gemm_f16_dma
// hands such products over
bool gemm_f16_kgroup_supported(const GemmParams &p, int epilogue, int tile);
hipError_t launch_gemm_f16_kgroup(const GemmParams &p, int epilogue, int tile, hipStream_t s);
// whether the fast path applies RoPE and writes q / the cache / V^T straight from the wq|wk|wv product for this shape
bool gemm_f16_rope_supported(const GemmParams &p);

// ---- prefill: element-wise kernels around the GEMMs (prefill.hip) ----
// fused causal attention of a multi-token forward (attn_prefill.hip); head_dim 64 or 128, f16 cache
struct AttnPrefillParams {
    const void *q2;          // [n_heads][n] rows [q hi (head_dim) | q lo (head_dim)] f16, after RoPE
    const void *cache_k;     // this layer: [n_heads][max_seq_len][head_dim] f16
    const void *v_t;         // [n_heads][head_dim][t_pad] f16 (V transposed with vt_swap, finite values in the padding)
    void *out;               // [n][dim] f16: head h at columns h * head_dim ..
    int n, n_heads, head_dim, dim, max_seq_len, t_pad;
    float scale;             // 1 / sqrt(head_dim) (transformer.rs:770)
    int order;               // launch order of the query blocks: 0 ascending, 1 descending, 2 descending then ascending
};
bool attn_prefill_supported(int head_dim);
hipError_t launch_attn_prefill(const AttnPrefillParams &p, hipStream_t s);

// f32 mode (prefill_f32.hip): the same steps on fp32 tensors, no rounding points
struct PrefillRopeF32Params {
    const float *qkv;       // [n x 3 dim]
    const float2 *freqs;    // [max_seq_len x head_dim/2]
    float *q;               // [n_heads][n][head_dim], after RoPE
    float *cache_k, *cache_v; // this layer: [n_heads][max_seq_len][head_dim]
    float *v_t;             // [n_heads][head_dim][t_pad]
    int n, dim, head_dim, max_seq_len, t_pad;
};
hipError_t launch_rmsnorm_rows_f32(float *y, const float *x, const float *w, int rows, int d, float eps, hipStream_t s);
hipError_t launch_rope_kv_prefill_f32(const PrefillRopeF32Params &p, hipStream_t s);
// scores [n_heads][n] rows of t_pad floats (raw q.k) -> causal probabilities in place
hipError_t launch_causal_softmax_f32(float *scores, int n_heads, int n, int t_pad, int head_dim, hipStream_t s);
hipError_t launch_silu_mul_f32(const float *g, const float *u, float *m, size_t total, hipStream_t s);

hipError_t launch_embed_rows(const void *table, int table_f16, const int32_t *tokens_dev, int n, int dim, float *x, hipStream_t s);
hipError_t launch_rmsnorm_rows_f16(void *y, const float *x, const float *w, int rows, int d, float eps, hipStream_t s);
hipError_t launch_rope_kv_prefill(const PrefillRopeParams &p, hipStream_t s);
// scores rows are t_pad floats apart, the probability rows (hi and lo alike) p_stride halves
hipError_t launch_causal_softmax(const float *scores, void *p_hi, void *p_lo, int n_heads, int n, int t_pad, int p_stride, int head_dim, hipStream_t s);

hipError_t launch_embed(const void *table, int table_f16, int dim, const DecodeState *state, float *x, hipStream_t s);
// TokenSampler::sample at top_k = 1 (token_sampler.rs:99-147) on logits * scale (scale = 1 / temperature); writes
// state->token, appends to out_tokens[state->n_out++] and advances state->pos.
hipError_t launch_argmax_advance(const float *logits, int vocab, DecodeState *state, int32_t *out_tokens, int out_cap,
                                 hipStream_t s, float scale = 1.0f);
hipError_t launch_set_state(DecodeState *state, int pos, int token, int reset_out, hipStream_t s);
hipError_t launch_reset_out(DecodeState *state, hipStream_t s);
hipError_t launch_advance_pos(DecodeState *state, const int32_t *tokens_dev, int idx, hipStream_t s);

// synthetic fills (synth.h)
hipError_t launch_synth_fill(void *dst, int dst_f16, uint64_t n, uint64_t key, double std, hipStream_t s);
hipError_t launch_fill_f32(float *dst, uint64_t n, float v, hipStream_t s);
hipError_t launch_fill_u32(uint32_t *dst, uint64_t n, uint32_t v, hipStream_t s);

// op level (OpenCLTensor's op set, tensor_opencl_support.rs:215-405)
hipError_t launch_convert(void *dst, int dst_f16, const void *src, int src_f16, uint64_t n, hipStream_t s);
hipError_t launch_transpose(void *dst, const void *src, int rows, int cols, int is_f16, hipStream_t s); // src [rows x cols]
hipError_t launch_hadamard(void *dst, const void *src, uint64_t n, int is_f16, hipStream_t s);
hipError_t launch_silu(void *dst, uint64_t n, int is_f16, hipStream_t s);
hipError_t launch_add_f32(float *dst, const float *a, const float *b, uint64_t n, hipStream_t s); // dst = a + b
hipError_t launch_rmsnorm_rows(float *y, const float *x, const float *w, int rows, int d, float eps, int round_y, hipStream_t s);
hipError_t launch_rope_row(float *x, int n_heads, int head_dim, const float2 *freqs_at_pos, hipStream_t s);
hipError_t launch_silu_mul_f16(const void *g, const void *u, void *m, size_t total, hipStream_t s); // m = f16(silu(g) * u)
// RoPE on q (in place) and k at `pos`, k and v into the cache planes [head][position][head_dim] at `pos`
hipError_t launch_rope_kvwrite(float *q, const float *k, const float *v, void *cache_k, void *cache_v, int cache_f16, int n_heads, int head_dim,
                               int max_seq_len, int pos, const float2 *freqs_at_pos, hipStream_t s);
// KV-cache services (transformer.rs:180-197): shift positions left by `shifts` within each (head) plane
hipError_t launch_cache_shift_left(void *cache, int is_f16, size_t planes, int max_seq_len, int head_dim, int shifts, hipStream_t s);
// test hook: [head_dim x max_seq_len] f32 view of one head's plane
hipError_t launch_cache_read(float *dst, const void *plane, int is_f16, int max_seq_len, int head_dim, hipStream_t s);

} // namespace rlh
