// api.hip -- the C ABI of librllama_hip.so (include/rllama_hip.h): context, HBM-resident model and KV
// caches, the token-step launch sequence, and the op-level entry points.
//
// Structure mirrors what it replaces in the reference (Noeda/rllama): OpenCL (tensor_opencl_support.rs:40-58)
// -> rlh_ctx; Transformer (transformer.rs:17-34) -> rlh_model; TransformerCaches (transformer.rs:111-113)
// -> rlh_caches; OpenCLTensor (tensor_opencl_support.rs:23-38) -> rlh_tensor.
#include "../../include/rllama_hip.h"
#include "api_internal.h"
#include "synth.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <map>
#include <string>
#include <thread>
#include <vector>

using namespace rlh;

// ------------------------------------------------------------------------------------------------
// errors
// ------------------------------------------------------------------------------------------------
static thread_local std::string g_last_error;

namespace rlh {
int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}
int set_error(int code, const char *msg) { return fail(code, "%s", msg); }
} // namespace rlh

extern "C" const char *rlh_last_error(void) { return g_last_error.c_str(); }
extern "C" int rlh_abi_version(void) { return RLH_ABI_VERSION; }

// ------------------------------------------------------------------------------------------------
// objects
// ------------------------------------------------------------------------------------------------
struct Weight {
    void *p = nullptr;
    int rows = 0, cols = 0;
    int f16 = 0;
    bool loaded = false;
    size_t bytes() const { return (size_t)rows * cols * (f16 ? 2 : 4); }
};

struct Layer {
    Weight wqkv; // rows [0,d) wq, [d,2d) wk, [2d,3d) wv: one fused GEMV streams all three
    bool q_loaded = false, k_loaded = false, v_loaded = false;
    Weight wo, w1, w2, w3, attn_norm, ffn_norm;
};

// Work buffers of a multi-token forward (prefill); grown on demand, kept for the next call.
struct PrefillScratch {
    int n_cap = 0;       // rows the buffers are sized for
    int t_pad = 0;       // n_cap rounded up to 128: row stride of scores / probabilities / transposed V
    float *x = nullptr, *h = nullptr, *scores = nullptr;
    // q2: rows [q hi | q lo] of 2 head_dim halves; p2: rows [P hi | P lo] of 2 t_pad halves (one GEMM sums both parts)
    void *xn = nullptr, *qkv = nullptr, *q2 = nullptr, *v_t = nullptr, *p2 = nullptr, *a = nullptr;
    void *g = nullptr, *u = nullptr, *mm = nullptr;
    void *gemm_ws = nullptr; // fp32 partial sums of split-K products (short prompts)
    bool gemm_attention = false; // the buffers of the two-GEMM form of attention (scores, p2) exist
    static constexpr size_t kGemmWsBytes = (size_t)64 << 20;
    void release() {
        void *all[] = {x, h, scores, xn, qkv, q2, v_t, p2, a, g, u, mm, gemm_ws};
        for (void *b : all)
            if (b) (void)hipFree(b);
        *this = PrefillScratch();
    }
};

struct rlh_model {
    rlh_ctx *ctx = nullptr;
    rlh_model_params prm;
    int head_dim = 0;
    int last_layer_on_gpu = 0;
    // Layers 0 .. n_resident - 1 hold weights and cache planes on the device; with percentage_to_gpu < 1 the rest stay with
    // the host (transformer.rs:262-279) and only rlh_forward_layers runs on such a model.
    int n_resident = 0;
    Weight tok_emb, norm, output;
    std::vector<Layer> layers;
    float2 *freqs = nullptr;
    // activations of one token step
    // x: residual stream entering a layer; h: after the attention block; att: attention output; att_o / ffn_o:
    // outputs of wo / w2 (added to the stream in the next kernel's prologue)
    float *x = nullptr, *h = nullptr, *q = nullptr, *att = nullptr, *att_o = nullptr, *mh = nullptr, *ffn_o = nullptr, *logits = nullptr;
    DecodeState *state = nullptr;
    int32_t *out_tokens = nullptr;
    int out_cap = 0;
    int32_t *prompt_dev = nullptr;
    int prompt_cap = 0;
    float *attn_ws = nullptr;
    unsigned *attn_tickets = nullptr; // [n_heads] arrival counters of the in-kernel merge (zero between launches)
    int max_splits = kAttnDecodeMaxSplits;
    bool capturing = false;    // a decode step is being recorded into a HIP graph
    int stream_weights = 1;
    PrefillScratch pf;
    int prefill_mode = 0; // 0: matrix-core prefill where available (f16 mode), 1: token by token
    // the greedy pick inside the output head's launch: one record per workgroup, one arrival counter (zero between launches)
    float *amax_ws = nullptr;
    unsigned *amax_ticket = nullptr;
    // host mirror of the device state after a greedy call: next position to fill, or -1 if the device holds no sampled token
    uint64_t uid = 0;   // unique per created model: a later model at the same address is still another model
    int next_pos = -1;
    rlh_caches *greedy_caches = nullptr;
};

// A run over some of the layers: the stream enters from and leaves to host memory, no embedding, no output head.
struct LayerSpan {
    int first = 0, last = 0;
    const float *x_in = nullptr; // [n x dim] f32, the stream entering layer `first`
    float *x_out = nullptr;      // [n x dim] f32, the stream leaving layer `last`
};

struct rlh_caches {
    rlh_ctx *ctx = nullptr;
    const rlh_model *model = nullptr; // identity only: never dereferenced (the model may be freed first)
    uint64_t model_uid = 0;
    int n_layers = 0, n_heads = 0, head_dim = 0, max_seq_len = 0;
    void *k = nullptr, *v = nullptr;
    size_t bytes_each = 0;
    int f16 = 0;
    // one captured decode step (token step + greedy pick) per attention grid shape, replayed by the greedy loops
    std::map<int, hipGraphExec_t> step_graphs;
    unsigned graphs_tun_version = 0; // the context's switches when the graphs were captured
};

// ------------------------------------------------------------------------------------------------
// switches
// ------------------------------------------------------------------------------------------------
namespace rlh {
bool tunables_set(Tunables &t, const char *name, const char *value) {
    if (!name) return false;
    const Tunables dflt;
    const std::string n(name);
    const bool reset = value == nullptr;
    const int v = reset ? 0 : atoi(value);
    auto flag_off = [&](int &no_field) { no_field = reset ? 0 : (v == 0 ? 1 : 0); return true; }; // NAME=0 switches a default-on feature off
    if (n == "GEMV_BURST") return flag_off(t.gemv_burst_fixed);
    if (n == "ATTN_CHUNK") { t.attn_chunk = reset ? dflt.attn_chunk : v; return reset || v == 0 || v == -1 || v >= 16; }
    if (n == "ATTN_SINGLE_MAX") { t.attn_single_max = reset ? dflt.attn_single_max : v; return reset || v >= 0; }
    if (n == "ATTN_MERGE") { t.attn_merge_mode = reset ? dflt.attn_merge_mode : v; return reset || v == 0 || v == 2; }
    if (n == "ATTN_LDS") { t.attn_lds = reset ? 0 : (v != 0); return true; }
    if (n == "PREFILL_ATTN") { t.prefill_attn_gemm = !reset && !strcmp(value, "gemm"); return reset || !strcmp(value, "gemm") || !strcmp(value, "fused"); }
    if (n == "PREFILL_ATTN_ORDER") { t.prefill_attn_order = reset ? dflt.prefill_attn_order : v; return reset || (v >= 0 && v <= 2); }
    if (n == "DECODE_GRAPH") { t.decode_graph = reset ? 0 : (v != 0); return true; }
    if (n == "DECODE_FOLD") { t.decode_fold = reset ? 1 : (v != 0); return true; }
    if (n == "GEMM_TILE") { t.gemm.tile_plus1 = reset ? 0 : v + 1; return reset || (v >= 0 && v <= 3); }
    if (n == "GEMM_SPLIT_K") { t.gemm.split_k = reset ? 0 : v; return reset || v >= 0; }
    if (n == "GEMM_SPLIT_HALF") return flag_off(t.gemm.no_split_half);
    if (n == "GEMM_DUAL") { t.gemm.dual_plus1 = reset ? 0 : v + 1; return reset || (v >= 0 && v <= 5); }
    if (n == "GEMM_DUAL_CUT") return flag_off(t.gemm.no_dual_cut);
    if (n == "GEMM_ROPE") return flag_off(t.gemm.no_rope_epilogue);
    if (n == "FINISH_NORM") return flag_off(t.gemm.no_finish_norm);
    if (n == "GEMM_KGROUP") return flag_off(t.gemm.no_kgroup);
    return false;
}

void tunables_from_env(Tunables &t) {
    static const char *const names[] = {"GEMV_BURST", "ATTN_CHUNK", "ATTN_SINGLE_MAX", "ATTN_MERGE", "ATTN_LDS", "PREFILL_ATTN", "PREFILL_ATTN_ORDER",
                                        "DECODE_GRAPH", "DECODE_FOLD", "GEMM_TILE", "GEMM_SPLIT_K", "GEMM_SPLIT_HALF", "GEMM_DUAL", "GEMM_DUAL_CUT",
                                        "GEMM_ROPE", "FINISH_NORM", "GEMM_KGROUP"};
    for (const char *name : names) {
        const std::string env = std::string("RLLAMA_HIP_") + name;
        const char *val = getenv(env.c_str());
        if (val != nullptr && !tunables_set(t, name, val)) {
            (void)tunables_set(t, name, nullptr); // an unusable value leaves the default in place
            fprintf(stderr, "rllama_hip: ignoring %s=%s\n", env.c_str(), val);
        }
    }
}
} // namespace rlh

extern "C" int rlh_set_option(rlh_ctx *ctx, const char *name, const char *value) {
    if (!ctx || !name) return fail(RLH_ERR_INVALID, "rlh_set_option: NULL argument");
    CtxLock lock(ctx);
    Tunables t = ctx->tun;
    if (!tunables_set(t, name, value)) return fail(RLH_ERR_INVALID, "rlh_set_option: unknown option or unusable value: %s=%s", name, value ? value : "(default)");
    // work queued under the old setting finishes first: captured decode steps and work buffers depend on some of these
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    ctx->tun = t;
    ctx->tun_version++;
    return RLH_OK;
}

// ------------------------------------------------------------------------------------------------
// context
// ------------------------------------------------------------------------------------------------
extern "C" int rlh_init(int device_ordinal, int verbose, rlh_ctx **out) {
    if (!out) return fail(RLH_ERR_INVALID, "rlh_init: out is NULL");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        return fail(RLH_ERR_NO_DEVICE, "rlh_init: no HIP device (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    }
    if (device_ordinal < 0 || device_ordinal >= count) {
        return fail(RLH_ERR_NO_DEVICE, "rlh_init: device ordinal %d out of range (%d devices)", device_ordinal, count);
    }
    rlh_ctx *c = new rlh_ctx();
    c->device = device_ordinal;
    c->verbose = verbose;
    tunables_from_env(c->tun); // the only place the library reads its environment switches
    if ((e = hipSetDevice(device_ordinal)) != hipSuccess || (e = hipGetDeviceProperties(&c->prop, device_ordinal)) != hipSuccess) {
        delete c;
        return fail(RLH_ERR_HIP, "rlh_init: %s", hipGetErrorString(e));
    }
    if (strncmp(c->prop.gcnArchName, "gfx950", 6) != 0) {
        int rc = fail(RLH_ERR_UNSUPPORTED, "rlh_init: device %d is %s; this library holds gfx950 code only", device_ordinal,
                      c->prop.gcnArchName);
        delete c;
        return rc;
    }
    if ((e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking)) != hipSuccess) {
        delete c;
        return fail(RLH_ERR_HIP, "rlh_init: hipStreamCreate: %s", hipGetErrorString(e));
    }
    if (int rc = noalloc_setup(c); rc != RLH_OK) {
        (void)hipStreamDestroy(c->stream);
        delete c;
        return rc;
    }
    if (verbose) {
        fprintf(stderr, "rllama_hip: device %d %s (%s), %d CUs, %.1f GB HBM\n", device_ordinal, c->prop.name, c->prop.gcnArchName,
                c->prop.multiProcessorCount, (double)c->prop.totalGlobalMem / 1e9);
    }
    *out = c;
    return RLH_OK;
}

extern "C" void rlh_shutdown(rlh_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipStreamDestroy(ctx->stream);
    }
    ops_release(ctx);
    delete ctx;
}

extern "C" int rlh_sync(rlh_ctx *ctx) {
    if (!ctx) return fail(RLH_ERR_INVALID, "rlh_sync: ctx is NULL");
    CtxLock lock(ctx);
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_device_info(rlh_ctx *ctx, char *name, int cap, int *compute_units, uint64_t *hbm_bytes) {
    if (!ctx) return fail(RLH_ERR_INVALID, "rlh_device_info: ctx is NULL");
    if (name && cap > 0) snprintf(name, (size_t)cap, "%s (%s)", ctx->prop.name, ctx->prop.gcnArchName);
    if (compute_units) *compute_units = ctx->prop.multiProcessorCount;
    if (hbm_bytes) *hbm_bytes = (uint64_t)ctx->prop.totalGlobalMem;
    return RLH_OK;
}

// ------------------------------------------------------------------------------------------------
// model
// ------------------------------------------------------------------------------------------------
static void free_weight(Weight &w) {
    if (w.p) (void)hipFree(w.p);
    w.p = nullptr;
}

static int alloc_weight(Weight &w, int rows, int cols, int f16) {
    w.rows = rows;
    w.cols = cols;
    w.f16 = f16;
    HIP_TRY(hipMalloc(&w.p, w.bytes()));
    return RLH_OK;
}

static float clamp_percentage(float p) {
    // DataSettings::percentage_to_gpu (transformer.rs:91-103)
    if (p >= 1.0f) p = 1.0f;
    if (p < 0.0f) p = 0.0f;
    if (std::isnan(p)) p = 0.0f;
    return p;
}

extern "C" int rlh_model_create(rlh_ctx *ctx, const rlh_model_params *prm, rlh_model **out) {
    if (!ctx || !prm || !out) return fail(RLH_ERR_INVALID, "rlh_model_create: NULL argument");
    *out = nullptr;
    if (prm->dim <= 0 || prm->n_layers <= 0 || prm->n_heads <= 0 || prm->ffn_hidden <= 0 || prm->vocab_size <= 0 ||
        prm->max_seq_len <= 0) {
        return fail(RLH_ERR_INVALID, "rlh_model_create: non-positive dimension");
    }
    if (prm->dim % prm->n_heads != 0) return fail(RLH_ERR_INVALID, "rlh_model_create: dim %% n_heads != 0 (transformer.rs:252)");
    const int hd = prm->dim / prm->n_heads;
    if (hd != 16 && hd != 32 && hd != 64 && hd != 128) {
        return fail(RLH_ERR_UNSUPPORTED, "rlh_model_create: head_dim %d (supported: 16, 32, 64, 128)", hd);
    }
    if (prm->dim % 8 != 0 || prm->ffn_hidden % 8 != 0) {
        return fail(RLH_ERR_UNSUPPORTED, "rlh_model_create: dim and ffn_hidden must be multiples of 8 (16-byte weight rows)");
    }
    CtxLock lock(ctx);
    const int wf16 = prm->force_f16 ? 1 : 0;
    const size_t lds_need = gemv_lds_bytes(prm->ffn_hidden > prm->dim ? prm->ffn_hidden : prm->dim, wf16, wf16);
    if (lds_need > (size_t)ctx->prop.sharedMemPerBlock && lds_need > 160 * 1024) {
        return fail(RLH_ERR_UNSUPPORTED, "rlh_model_create: activation vector of %zu bytes does not fit in LDS", lds_need);
    }
    rlh_model *m = new rlh_model();
    static std::atomic<uint64_t> next_uid{1};
    m->uid = next_uid.fetch_add(1);
    m->ctx = ctx;
    m->prm = *prm;
    m->prm.percentage_to_gpu = clamp_percentage(prm->percentage_to_gpu);
    m->head_dim = hd;
    // transformer.rs:266-268
    m->last_layer_on_gpu = (int)std::round(m->prm.percentage_to_gpu * (float)(prm->n_layers - 1));
    m->n_resident = m->last_layer_on_gpu + 1;
    m->layers.resize((size_t)prm->n_layers);
    const int d = prm->dim, F = prm->ffn_hidden, V = prm->vocab_size;
    int rc = RLH_OK;
    auto A = [&](Weight &w, int r, int c, int f16) {
        if (rc == RLH_OK) rc = alloc_weight(w, r, c, f16);
    };
    for (int l = 0; l < m->n_resident; l++) {
        Layer &L = m->layers[(size_t)l];
        A(L.wqkv, 3 * d, d, wf16);
        A(L.wo, d, d, wf16);
        A(L.w1, F, d, wf16);
        A(L.w2, d, F, wf16);
        A(L.w3, F, d, wf16);
        A(L.attn_norm, 1, d, 0);
        A(L.ffn_norm, 1, d, 0);
    }
    A(m->norm, 1, d, 0);
    // tok_emb and output are allocated at set_tensor time in the dtype of their source (the reference keeps
    // both in f32, embedding.rs:41-47 / transformer.rs:302-308; f16 file contents widen exactly).
    m->tok_emb.rows = V;
    m->tok_emb.cols = d;
    m->output.rows = V;
    m->output.cols = d;

    // RoPE table: compute_freqs_cis (transformer.rs:858-885) in f64, cast to f32 as at its use (:836-837)
    if (rc == RLH_OK) {
        std::vector<float2> tab((size_t)prm->max_seq_len * (hd / 2));
        for (int pos = 0; pos < prm->max_seq_len; pos++) {
            for (int j = 0; j < hd / 2; j++) {
                const double freq = 1.0 / std::pow(10000.0, (double)j * 2.0 / (double)hd);
                const double ang = freq * (double)pos;
                tab[(size_t)pos * (hd / 2) + j] = make_float2((float)std::cos(ang), (float)std::sin(ang));
            }
        }
        hipError_t e = hipMalloc((void **)&m->freqs, tab.size() * sizeof(float2));
        if (e == hipSuccess) e = hipMemcpy(m->freqs, tab.data(), tab.size() * sizeof(float2), hipMemcpyHostToDevice);
        if (e != hipSuccess) rc = fail(RLH_ERR_HIP, "rlh_model_create: RoPE table: %s", hipGetErrorString(e));
    }
    auto B = [&](void **p, size_t bytes) {
        if (rc != RLH_OK) return;
        hipError_t e = hipMalloc(p, bytes);
        if (e == hipSuccess) e = hipMemset(*p, 0, bytes);
        if (e != hipSuccess) rc = fail(e == hipErrorOutOfMemory ? RLH_ERR_OOM : RLH_ERR_HIP, "rlh_model_create: %s", hipGetErrorString(e));
    };
    m->out_cap = prm->max_seq_len + 1;
    m->prompt_cap = prm->max_seq_len;
    B((void **)&m->x, sizeof(float) * d);
    B((void **)&m->h, sizeof(float) * d);
    B((void **)&m->q, sizeof(float) * d);
    B((void **)&m->att_o, sizeof(float) * d);
    B((void **)&m->ffn_o, sizeof(float) * d);
    B((void **)&m->att, sizeof(float) * d);
    B((void **)&m->mh, sizeof(float) * F);
    B((void **)&m->logits, sizeof(float) * V);
    B((void **)&m->state, sizeof(DecodeState));
    B((void **)&m->out_tokens, sizeof(int32_t) * m->out_cap);
    B((void **)&m->prompt_dev, sizeof(int32_t) * m->prompt_cap);
    B((void **)&m->attn_ws, sizeof(float) * attn_decode_workspace_floats(prm->n_heads, hd, m->max_splits));
    B((void **)&m->attn_tickets, sizeof(unsigned) * (size_t)prm->n_heads);
    B((void **)&m->amax_ws, gemv_argmax_ws_bytes());
    B((void **)&m->amax_ticket, 256);
    if (rc == RLH_OK && hipDeviceSynchronize() != hipSuccess) rc = fail(RLH_ERR_HIP, "rlh_model_create: hipDeviceSynchronize failed");
    if (rc != RLH_OK) {
        rlh_model_free(m);
        return rc;
    }
    *out = m;
    return RLH_OK;
}

extern "C" void rlh_model_free(rlh_model *m) {
    if (!m) return;
    CtxLock lock(m->ctx);
    (void)hipStreamSynchronize(m->ctx->stream);
    for (auto &L : m->layers) {
        free_weight(L.wqkv);
        free_weight(L.wo);
        free_weight(L.w1);
        free_weight(L.w2);
        free_weight(L.w3);
        free_weight(L.attn_norm);
        free_weight(L.ffn_norm);
    }
    free_weight(m->tok_emb);
    free_weight(m->norm);
    free_weight(m->output);
    m->pf.release();
    void *bufs[] = {m->freqs, m->x, m->h, m->q, m->att, m->att_o, m->mh, m->ffn_o, m->logits, m->state, m->out_tokens, m->prompt_dev, m->attn_ws, m->attn_tickets, m->amax_ws, m->amax_ticket};
    for (void *b : bufs)
        if (b) (void)hipFree(b);
    delete m;
}

struct Slot {
    Weight *w = nullptr;
    size_t row_off = 0; // rows into w (fused wqkv)
    int rows = 0, cols = 0;
    bool *flag = nullptr;
};

static int find_slot(rlh_model *m, int kind, int layer, Slot *s) {
    const int d = m->prm.dim, F = m->prm.ffn_hidden, V = m->prm.vocab_size;
    if (kind >= RLH_WQ && kind <= RLH_FFN_NORM) {
        if (layer < 0 || layer >= m->prm.n_layers) return fail(RLH_ERR_INVALID, "layer %d out of range", layer);
        if (layer >= m->n_resident) {
            return fail(RLH_ERR_STATE, "layer %d stays on the host: percentage_to_gpu %.4f keeps layers 0..%d on the device (transformer.rs:262-279)",
                        layer, (double)m->prm.percentage_to_gpu, m->last_layer_on_gpu);
        }
    }
    Layer *L = (kind >= RLH_WQ && kind <= RLH_FFN_NORM) ? &m->layers[(size_t)layer] : nullptr;
    switch (kind) {
    case RLH_TOK_EMB: *s = Slot{&m->tok_emb, 0, V, d, &m->tok_emb.loaded}; break;
    case RLH_OUTPUT: *s = Slot{&m->output, 0, V, d, &m->output.loaded}; break;
    case RLH_NORM: *s = Slot{&m->norm, 0, 1, d, &m->norm.loaded}; break;
    case RLH_WQ: *s = Slot{&L->wqkv, 0, d, d, &L->q_loaded}; break;
    case RLH_WK: *s = Slot{&L->wqkv, (size_t)d, d, d, &L->k_loaded}; break;
    case RLH_WV: *s = Slot{&L->wqkv, (size_t)2 * d, d, d, &L->v_loaded}; break;
    case RLH_WO: *s = Slot{&L->wo, 0, d, d, &L->wo.loaded}; break;
    case RLH_W1: *s = Slot{&L->w1, 0, F, d, &L->w1.loaded}; break;
    case RLH_W2: *s = Slot{&L->w2, 0, d, F, &L->w2.loaded}; break;
    case RLH_W3: *s = Slot{&L->w3, 0, F, d, &L->w3.loaded}; break;
    case RLH_ATTN_NORM: *s = Slot{&L->attn_norm, 0, 1, d, &L->attn_norm.loaded}; break;
    case RLH_FFN_NORM: *s = Slot{&L->ffn_norm, 0, 1, d, &L->ffn_norm.loaded}; break;
    default: return fail(RLH_ERR_INVALID, "unknown tensor kind %d", kind);
    }
    return RLH_OK;
}

extern "C" int rlh_model_set_tensor(rlh_model *m, int kind, int layer, const void *host, int rows, int cols, int src_dtype) {
    if (!m || !host) return fail(RLH_ERR_INVALID, "rlh_model_set_tensor: NULL argument");
    if (src_dtype != RLH_F16 && src_dtype != RLH_F32) return fail(RLH_ERR_INVALID, "rlh_model_set_tensor: bad src_dtype %d", src_dtype);
    CtxLock lock(m->ctx);
    Slot s;
    int rc = find_slot(m, kind, layer, &s);
    if (rc != RLH_OK) return rc;
    if (rows != s.rows || cols != s.cols) {
        return fail(RLH_ERR_INVALID, "rlh_model_set_tensor: kind %d expects [%d x %d], got [%d x %d]", kind, s.rows, s.cols, rows, cols);
    }
    hipStream_t st = m->ctx->stream;
    if (kind == RLH_TOK_EMB || kind == RLH_OUTPUT) {
        // stored in the source's dtype: lossless either way
        if (s.w->p && s.w->f16 != (src_dtype == RLH_F16)) free_weight(*s.w);
        if (!s.w->p) {
            rc = alloc_weight(*s.w, rows, cols, src_dtype == RLH_F16);
            if (rc != RLH_OK) return rc;
        }
    }
    const size_t n = (size_t)rows * cols;
    const int dst_f16 = s.w->f16;
    char *dst = (char *)s.w->p + s.row_off * (size_t)cols * (dst_f16 ? 2 : 4);
    if ((src_dtype == RLH_F16) == (dst_f16 != 0)) {
        HIP_TRY(hipMemcpyAsync(dst, host, n * (dst_f16 ? 2 : 4), hipMemcpyHostToDevice, st));
        HIP_TRY(hipStreamSynchronize(st));
    } else {
        // widen (f16 file -> f32 tensor, tensor.rs:2467) or narrow (Tensor::to_f16 under --f16, tensor.rs:2281-2314) on the device
        void *tmp = nullptr;
        const size_t sb = n * (src_dtype == RLH_F16 ? 2 : 4);
        HIP_TRY(hipMalloc(&tmp, sb));
        hipError_t e = hipMemcpyAsync(tmp, host, sb, hipMemcpyHostToDevice, st);
        if (e == hipSuccess) e = launch_convert(dst, dst_f16, tmp, src_dtype == RLH_F16, n, st);
        hipError_t e2 = hipStreamSynchronize(st);
        (void)hipFree(tmp);
        HIP_TRY(e);
        HIP_TRY(e2);
    }
    *s.flag = true;
    return RLH_OK;
}

extern "C" int rlh_model_get_tensor(rlh_model *m, int kind, int layer, void *host_out, int rows, int cols, int dst_dtype) {
    if (!m || !host_out) return fail(RLH_ERR_INVALID, "rlh_model_get_tensor: NULL argument");
    if (dst_dtype != RLH_F16 && dst_dtype != RLH_F32) return fail(RLH_ERR_INVALID, "rlh_model_get_tensor: bad dst_dtype %d", dst_dtype);
    CtxLock lock(m->ctx);
    Slot s;
    int rc = find_slot(m, kind, layer, &s);
    if (rc != RLH_OK) return rc;
    if (rows != s.rows || cols != s.cols) return fail(RLH_ERR_INVALID, "rlh_model_get_tensor: shape mismatch");
    if (!*s.flag || !s.w->p) return fail(RLH_ERR_STATE, "rlh_model_get_tensor: tensor not loaded");
    const size_t n = (size_t)rows * cols;
    hipStream_t st = m->ctx->stream;
    const char *src = (const char *)s.w->p + s.row_off * (size_t)cols * (s.w->f16 ? 2 : 4);
    const int want_f16 = dst_dtype == RLH_F16;
    const size_t db = n * (want_f16 ? 2 : 4);
    if ((s.w->f16 != 0) == (want_f16 != 0)) {
        HIP_TRY(hipMemcpyAsync(host_out, src, db, hipMemcpyDeviceToHost, st));
        HIP_TRY(hipStreamSynchronize(st));
        return RLH_OK;
    }
    void *tmp = nullptr;
    HIP_TRY(hipMalloc(&tmp, db));
    hipError_t e = launch_convert(tmp, want_f16, src, s.w->f16, n, st);
    if (e == hipSuccess) e = hipMemcpyAsync(host_out, tmp, db, hipMemcpyDeviceToHost, st);
    hipError_t e2 = hipStreamSynchronize(st);
    (void)hipFree(tmp);
    HIP_TRY(e);
    HIP_TRY(e2);
    return RLH_OK;
}

extern "C" int rlh_model_fill_synthetic(rlh_model *m, uint64_t seed, double std) {
    if (!m) return fail(RLH_ERR_INVALID, "rlh_model_fill_synthetic: NULL model");
    CtxLock lock(m->ctx);
    hipStream_t st = m->ctx->stream;
    const int d = m->prm.dim;
    const bool whole = m->n_resident == m->prm.n_layers; // a split model leaves embedding, final norm and head to the host (transformer.rs:296-308)
    for (Weight *w : {&m->tok_emb, &m->output}) {
        if (whole && !w->p) {
            int rc = alloc_weight(*w, w->rows, w->cols, 1);
            if (rc != RLH_OK) return rc;
        }
    }
    auto fill = [&](Weight &w, size_t row_off, int rows, int kind, int layer) -> hipError_t {
        char *dst = (char *)w.p + row_off * (size_t)w.cols * (w.f16 ? 2 : 4);
        return launch_synth_fill(dst, w.f16, (uint64_t)rows * w.cols, synth_key(seed, SYNTH_STREAM_TENSOR(kind, layer)), std, st);
    };
    if (whole) {
        HIP_TRY(fill(m->tok_emb, 0, m->tok_emb.rows, RLH_TOK_EMB, 0));
        HIP_TRY(fill(m->output, 0, m->output.rows, RLH_OUTPUT, 0));
        m->tok_emb.loaded = m->output.loaded = true;
    }
    HIP_TRY(launch_fill_f32((float *)m->norm.p, (uint64_t)d, 1.0f, st));
    m->norm.loaded = true;
    for (int l = 0; l < m->n_resident; l++) {
        Layer &L = m->layers[(size_t)l];
        HIP_TRY(fill(L.wqkv, 0, d, RLH_WQ, l));
        HIP_TRY(fill(L.wqkv, (size_t)d, d, RLH_WK, l));
        HIP_TRY(fill(L.wqkv, (size_t)2 * d, d, RLH_WV, l));
        HIP_TRY(fill(L.wo, 0, L.wo.rows, RLH_WO, l));
        HIP_TRY(fill(L.w1, 0, L.w1.rows, RLH_W1, l));
        HIP_TRY(fill(L.w2, 0, L.w2.rows, RLH_W2, l));
        HIP_TRY(fill(L.w3, 0, L.w3.rows, RLH_W3, l));
        HIP_TRY(launch_fill_f32((float *)L.attn_norm.p, (uint64_t)d, 1.0f, st));
        HIP_TRY(launch_fill_f32((float *)L.ffn_norm.p, (uint64_t)d, 1.0f, st));
        L.q_loaded = L.k_loaded = L.v_loaded = true;
        L.wo.loaded = L.w1.loaded = L.w2.loaded = L.w3.loaded = L.attn_norm.loaded = L.ffn_norm.loaded = true;
    }
    HIP_TRY(hipStreamSynchronize(st));
    return RLH_OK;
}

extern "C" int rlh_model_set_prefill_mode(rlh_model *m, int mode) {
    if (!m || (mode != 0 && mode != 1)) return fail(RLH_ERR_INVALID, "rlh_model_set_prefill_mode: bad argument");
    m->prefill_mode = mode;
    return RLH_OK;
}

extern "C" int rlh_model_layers_on_gpu(const rlh_model *m, int *last_layer_on_gpu) {
    if (!m || !last_layer_on_gpu) return fail(RLH_ERR_INVALID, "rlh_model_layers_on_gpu: NULL argument");
    *last_layer_on_gpu = m->last_layer_on_gpu;
    return RLH_OK;
}

extern "C" int rlh_model_decode_bytes(const rlh_model *m, int T, uint64_t *bytes) {
    if (!m || !bytes || T < 1) return fail(RLH_ERR_INVALID, "rlh_model_decode_bytes: bad argument");
    const uint64_t d = (uint64_t)m->prm.dim, F = (uint64_t)m->prm.ffn_hidden, V = (uint64_t)m->prm.vocab_size, L = (uint64_t)m->n_resident;
    const uint64_t es = m->prm.force_f16 ? 2 : 4;
    const uint64_t head_es = (m->output.p && !m->output.f16) ? 4 : 2;
    const bool whole = m->n_resident == m->prm.n_layers; // a split model's head is the host's
    uint64_t b = L * (4 * d * d + 3 * d * F) * es + (whole ? V * d * head_es : 0);
    b += L * 2 * (uint64_t)T * d * es; // K and V rows read
    b += L * 2 * d * es;               // K and V row written
    *bytes = b;
    return RLH_OK;
}

static int layers_ready(const rlh_model *m, int first, int last) {
    for (int l = first; l <= last; l++) {
        const Layer &L = m->layers[(size_t)l];
        if (!(L.q_loaded && L.k_loaded && L.v_loaded && L.wo.loaded && L.w1.loaded && L.w2.loaded && L.w3.loaded && L.attn_norm.loaded &&
              L.ffn_norm.loaded))
            return 0;
    }
    return 1;
}

static int model_ready(const rlh_model *m) {
    if (!m->tok_emb.loaded || !m->output.loaded || !m->norm.loaded) return 0;
    return layers_ready(m, 0, m->prm.n_layers - 1);
}

// ------------------------------------------------------------------------------------------------
// caches
// ------------------------------------------------------------------------------------------------
extern "C" int rlh_caches_create(rlh_model *m, rlh_caches **out) {
    if (!m || !out) return fail(RLH_ERR_INVALID, "rlh_caches_create: NULL argument");
    *out = nullptr;
    CtxLock lock(m->ctx);
    rlh_caches *c = new rlh_caches();
    c->ctx = m->ctx;
    c->model = m;
    c->model_uid = m->uid;
    c->n_layers = m->n_resident; // planes of host-side layers live with the host
    c->n_heads = m->prm.n_heads;
    c->head_dim = m->head_dim;
    c->max_seq_len = m->prm.max_seq_len;
    c->f16 = m->prm.force_f16 ? 1 : 0; // transformer.rs:138-142
    c->bytes_each = (size_t)c->n_layers * c->n_heads * c->max_seq_len * c->head_dim * (c->f16 ? 2 : 4);
    hipError_t e = hipMalloc(&c->k, c->bytes_each);
    if (e == hipSuccess) e = hipMalloc(&c->v, c->bytes_each);
    if (e == hipSuccess) e = hipMemsetAsync(c->k, 0, c->bytes_each, c->ctx->stream); // Tensor::zeros
    if (e == hipSuccess) e = hipMemsetAsync(c->v, 0, c->bytes_each, c->ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c->ctx->stream);
    if (e != hipSuccess) {
        if (c->k) (void)hipFree(c->k);
        if (c->v) (void)hipFree(c->v);
        delete c;
        return fail(e == hipErrorOutOfMemory ? RLH_ERR_OOM : RLH_ERR_HIP, "rlh_caches_create: %s", hipGetErrorString(e));
    }
    *out = c;
    return RLH_OK;
}

extern "C" int rlh_caches_true_clone(const rlh_caches *src, rlh_caches **out) {
    if (!src || !out) return fail(RLH_ERR_INVALID, "rlh_caches_true_clone: NULL argument");
    *out = nullptr;
    rlh_ctx *ctx = src->ctx;
    CtxLock lock(ctx);
    rlh_caches *c = new rlh_caches(*src);
    c->k = c->v = nullptr;
    c->step_graphs.clear(); // captured steps hold the source's cache addresses: the clone captures its own
    hipError_t e = hipMalloc(&c->k, c->bytes_each);
    if (e == hipSuccess) e = hipMalloc(&c->v, c->bytes_each);
    if (e == hipSuccess) e = hipMemcpyAsync(c->k, src->k, c->bytes_each, hipMemcpyDeviceToDevice, ctx->stream);
    if (e == hipSuccess) e = hipMemcpyAsync(c->v, src->v, c->bytes_each, hipMemcpyDeviceToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        if (c->k) (void)hipFree(c->k);
        if (c->v) (void)hipFree(c->v);
        delete c;
        return fail(e == hipErrorOutOfMemory ? RLH_ERR_OOM : RLH_ERR_HIP, "rlh_caches_true_clone: %s", hipGetErrorString(e));
    }
    *out = c;
    return RLH_OK;
}

extern "C" int rlh_caches_shift_left(rlh_caches *c, int shifts) {
    if (!c || shifts < 0) return fail(RLH_ERR_INVALID, "rlh_caches_shift_left: bad argument");
    if (shifts == 0) return RLH_OK;
    CtxLock lock(c->ctx);
    const size_t planes = (size_t)c->n_layers * c->n_heads;
    HIP_TRY(launch_cache_shift_left(c->k, c->f16, planes, c->max_seq_len, c->head_dim, shifts, c->ctx->stream));
    HIP_TRY(launch_cache_shift_left(c->v, c->f16, planes, c->max_seq_len, c->head_dim, shifts, c->ctx->stream));
    return RLH_OK;
}

extern "C" void rlh_caches_free(rlh_caches *c) {
    if (!c) return;
    CtxLock lock(c->ctx);
    (void)hipStreamSynchronize(c->ctx->stream);
    for (auto &kv : c->step_graphs) (void)hipGraphExecDestroy(kv.second);
    if (c->k) (void)hipFree(c->k);
    if (c->v) (void)hipFree(c->v);
    delete c;
}

extern "C" int rlh_caches_read(const rlh_caches *c, int layer, int head, int which, float *host_out) {
    if (!c || !host_out) return fail(RLH_ERR_INVALID, "rlh_caches_read: NULL argument");
    if (layer < 0 || layer >= c->n_layers || head < 0 || head >= c->n_heads) return fail(RLH_ERR_INVALID, "rlh_caches_read: index out of range");
    CtxLock lock(c->ctx);
    hipStream_t st = c->ctx->stream;
    const size_t per_plane = (size_t)c->max_seq_len * c->head_dim;
    const size_t off = ((size_t)layer * c->n_heads + head) * per_plane * (c->f16 ? 2 : 4);
    const char *plane = (const char *)(which ? c->v : c->k) + off;
    float *tmp = nullptr;
    HIP_TRY(hipMalloc((void **)&tmp, per_plane * 4));
    hipError_t e = launch_cache_read(tmp, plane, c->f16, c->max_seq_len, c->head_dim, st);
    if (e == hipSuccess) e = hipMemcpyAsync(host_out, tmp, per_plane * 4, hipMemcpyDeviceToHost, st);
    hipError_t e2 = hipStreamSynchronize(st);
    (void)hipFree(tmp);
    HIP_TRY(e);
    HIP_TRY(e2);
    return RLH_OK;
}

// ------------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------------
static int attn_splits(const rlh_model *m, int T) {
    const Tunables &t = m->ctx->tun;
    return attn_splits_rule(T, m->prm.n_heads, m->ctx->prop.multiProcessorCount, t.attn_single_max, t.attn_chunk, m->max_splits);
}

enum StepKernel { kStepQkv = 0, kStepAttn = 1, kStepWo = 2, kStepW13 = 3, kStepW2 = 4, kStepHead = 5 };

// The launch parameters of one matrix-vector kernel of layer l (or of the output head) for the token described by the
// device state; *epi receives its epilogue.  which: kStepQkv, kStepWo, kStepW13, kStepW2, kStepHead.
// from_embedding: layer 0 of a whole token step reads its input row from the embedding table (no launch of its own for it);
// pick: the output head also makes the greedy pick and advances the token-step state.
static void build_gemv_step(rlh_model *m, rlh_caches *c, int l, int which, int first_layer, GemvParams *out, int *epi, bool from_embedding = false,
                            bool pick = false) {
    const rlh_model_params &P = m->prm;
    const int d = P.dim, F = P.ffn_hidden, V = P.vocab_size;
    const int f16 = P.force_f16 ? 1 : 0;
    const float eps = (float)P.norm_eps; // add_scalar(self.eps as f32), transformer.rs:477
    GemvParams g{};
    g.stream_weights = m->stream_weights;
    g.burst_fixed = m->ctx->tun.gemv_burst_fixed;
    g.w_is_f16 = f16;
    g.x_f16 = f16;
    g.round_y = f16;
    g.eps = eps;
    // The stream enters layer l in m->x (l == first_layer: the embedding row, or the row a layer span was handed) or as
    // m->h + m->ffn_o of layer l - 1.
    if (which == kStepHead) {
        // last residual add + final norm + output head: f32 activations, no rounding
        // (transformer.rs:445, 378-381; tensor.rs:1837-1918)
        GemvParams p{};
        p.stream_weights = m->stream_weights;
        p.burst_fixed = m->ctx->tun.gemv_burst_fixed;
        p.w = m->output.p;
        p.w_is_f16 = m->output.f16;
        p.x = m->h;
        p.x_add = m->ffn_o;
        p.x_f16 = 0;
        p.round_y = 0;
        p.norm_w = (const float *)m->norm.p;
        p.eps = eps;
        p.y = m->logits;
        p.n_rows = V;
        p.k = d;
        *epi = kEpiStore;
        if (pick) {
            p.amax_ws = m->amax_ws;
            p.amax_ticket = m->amax_ticket;
            p.state_rw = m->state;
            p.out_tokens = m->out_tokens;
            p.out_cap = m->out_cap;
            *epi = kEpiStoreArgmax;
        }
        *out = p;
        return;
    }
    Layer &L = m->layers[(size_t)l];
    GemvParams p = g;
    switch (which) {
    case kStepQkv: {
        // (previous layer's second residual add, transformer.rs:445) + attention_norm + wq|wk|wv + RoPE + cache
        // write (transformer.rs:432, 665-668, 694-725, 751-761)
        const size_t layer_elems = (size_t)P.n_heads * P.max_seq_len * m->head_dim;
        const size_t ces = c->f16 ? 2 : 4;
        p.w = L.wqkv.p;
        if (l == first_layer && from_embedding) {
            p.embed_table = m->tok_emb.p; // Embedding::get_embedding (embedding.rs:50-52) inside this launch
            p.embed_f16 = m->tok_emb.f16;
            p.x_out = m->x;               // the stream entering the layer, for this layer's first residual add
        } else if (l == first_layer) {
            p.x = m->x;
        } else {
            p.x = m->h;
            p.x_add = m->ffn_o;
            p.x_out = m->x;
        }
        p.norm_w = (const float *)L.attn_norm.p;
        p.y = m->q;
        p.n_rows = 3 * d;
        p.k = d;
        p.state = m->state;
        p.freqs = m->freqs;
        p.cache_k = (char *)c->k + (size_t)l * layer_elems * ces;
        p.cache_v = (char *)c->v + (size_t)l * layer_elems * ces;
        p.cache_f16 = c->f16;
        p.dim = d;
        p.head_dim = m->head_dim;
        p.max_seq_len = P.max_seq_len;
        *epi = kEpiRopeKv;
        break;
    }
    case kStepWo:
        // wo (transformer.rs:783-819); its output joins the stream in the next kernel
        p.w = L.wo.p;
        p.x = m->att;
        p.y = m->att_o;
        p.n_rows = d;
        p.k = d;
        *epi = kEpiStore;
        break;
    case kStepW13:
        // h = x + att_out (transformer.rs:442) + ffn_norm + w1|w3 + SiLU * gate (transformer.rs:443, 537-565)
        p.w = L.w1.p;
        p.w_b = L.w3.p;
        p.x = m->x;
        p.x_add = m->att_o;
        p.x_out = m->h;
        p.norm_w = (const float *)L.ffn_norm.p;
        p.y = m->mh;
        p.n_rows = F;
        p.k = d;
        *epi = kEpiSilu;
        break;
    default: // kStepW2
        // w2 (transformer.rs:568-570); its output joins the stream in the next kernel
        p.w = L.w2.p;
        p.x = m->mh;
        p.y = m->ffn_o;
        p.n_rows = d;
        p.k = F;
        *epi = kEpiStore;
        break;
    }
    *out = p;
}

// Enqueues one of the five kernels of layer l (or the output head) for the token described by the device
// state.  T_host = position + 1 as known to the host (sizes the attention grid).
static int enqueue_step_kernel(rlh_model *m, rlh_caches *c, int l, int which, int T_host, int first_layer = 0, bool from_embedding = false, bool pick = false) {
    hipStream_t st = m->ctx->stream;
    const rlh_model_params &P = m->prm;
    if (which < kStepQkv || which > kStepHead) return fail(RLH_ERR_INVALID, "unknown step kernel %d", which);
    if (which != kStepAttn) {
        GemvParams p;
        int epi = kEpiStore;
        build_gemv_step(m, c, l, which, first_layer, &p, &epi, from_embedding, pick);
        if (which == kStepQkv && !m->capturing) p.pos1_host = T_host; // (a captured step is replayed at later positions: it reads the device state)
        HIP_TRY(launch_gemv(p, epi, st));
        return RLH_OK;
    }
    // scores, softmax, P.V (transformer.rs:762-779) + f16 rounding point before wo (:793-796)
    const size_t layer_elems = (size_t)P.n_heads * P.max_seq_len * m->head_dim;
    const size_t ces = c->f16 ? 2 : 4;
    AttnDecodeParams a{};
    a.q = m->q;
    a.cache_k = (char *)c->k + (size_t)l * layer_elems * ces;
    a.cache_v = (char *)c->v + (size_t)l * layer_elems * ces;
    a.cache_f16 = c->f16;
    a.state = m->state;
    a.pos_host = m->capturing ? -1 : T_host - 1; // a captured step is replayed at later positions: it reads the device state
    a.n_heads = P.n_heads;
    a.head_dim = m->head_dim;
    a.max_seq_len = P.max_seq_len;
    a.n_splits = attn_splits(m, T_host);
    a.out = m->att;
    a.round_out = P.force_f16 ? 1 : 0;
    a.workspace = m->attn_ws;
    a.tickets = m->attn_tickets;
    a.merge_mode = m->ctx->tun.attn_merge_mode;
    a.chunk_hint = (((T_host + a.n_splits - 1) / a.n_splits) + 15) & ~15;
    a.lds_stage = m->ctx->tun.attn_lds && !m->capturing && c->f16 && (m->head_dim == 128 || m->head_dim == 64) && a.merge_mode == 2 &&
                  (size_t)a.chunk_hint * m->head_dim * 4 <= 128 * 1024;
    HIP_TRY(launch_attn_decode(a, st));
    return RLH_OK;
}

// Enqueues one token step (the body of Transformer::forward for a single row, transformer.rs:361-381):
// reads state->token / state->pos on the device.
static int enqueue_token_step(rlh_model *m, rlh_caches *c, int T_host, bool with_head, bool pick = false) {
    // pick (with_head only): the greedy pick and the advance of the token-step state follow the head.  With the context's
    // DECODE_FOLD switch on (default) neither the embedding row nor the pick is a launch of its own.
    const bool fold = m->ctx->tun.decode_fold != 0;
    if (!fold) HIP_TRY(launch_embed(m->tok_emb.p, m->tok_emb.f16, m->prm.dim, m->state, m->x, m->ctx->stream));
    for (int l = 0; l < m->prm.n_layers; l++) {
        for (int which = kStepQkv; which <= kStepW2; which++) {
            int rc = enqueue_step_kernel(m, c, l, which, T_host, 0, fold && l == 0 && which == kStepQkv);
            if (rc != RLH_OK) return rc;
        }
    }
    if (!with_head) return RLH_OK;
    int rc = enqueue_step_kernel(m, c, 0, kStepHead, T_host, 0, false, pick && fold);
    if (rc != RLH_OK) return rc;
    if (pick && !fold) HIP_TRY(launch_argmax_advance(m->logits, m->prm.vocab_size, m->state, m->out_tokens, m->out_cap, m->ctx->stream));
    return RLH_OK;
}

static int ensure_prefill_scratch(rlh_model *m, int n) {
    PrefillScratch &S = m->pf;
    const size_t d = (size_t)m->prm.dim, F = (size_t)m->prm.ffn_hidden, H = (size_t)m->prm.n_heads, hd = (size_t)m->head_dim;
    const size_t es = m->prm.force_f16 ? 2 : 4; // element size of the activations between the GEMMs
    // the [n x n] score / probability matrices exist only in the GEMM form of attention (the one-kernel form keeps them
    // on chip); f32 mode turns the scores into probabilities in place
    const bool gemm_attention = !(es == 2 && !m->ctx->tun.prefill_attn_gemm && attn_prefill_supported((int)hd));
    if (n <= S.n_cap && (S.gemm_attention || !gemm_attention)) return RLH_OK;
    if (n < S.n_cap) n = S.n_cap; // (the form of attention changed: same capacity, with the score buffers)
    HIP_TRY(hipStreamSynchronize(m->ctx->stream));
    S.release();
    const size_t N = (size_t)n, tp = (N + 127) & ~(size_t)127;
    hipError_t e = hipSuccess;
    auto A = [&](void **p, size_t bytes) {
        if (e != hipSuccess) return;
        e = hipMalloc(p, bytes);
        if (e == hipSuccess) e = hipMemsetAsync(*p, 0, bytes, m->ctx->stream); // padding must hold finite values
    };
    A((void **)&S.x, N * d * 4);
    A((void **)&S.h, N * d * 4);
    A((void **)&S.xn, N * d * es);
    A((void **)&S.qkv, N * 3 * d * es);
    A((void **)&S.q2, N * d * 2 * 2); // f16 mode: hi and lo halves; f32 mode: one float
    A((void **)&S.v_t, H * hd * tp * es);
    if (gemm_attention) A((void **)&S.scores, H * N * tp * 4);
    if (gemm_attention && es == 2) A((void **)&S.p2, H * N * tp * 2 * 2);
    A((void **)&S.a, N * d * es);
    A((void **)&S.g, N * F * es);
    if (es == 4) A((void **)&S.u, N * F * es); // f16 mode: w3's epilogue consumes its product on the spot
    A((void **)&S.mm, N * F * es);
    A((void **)&S.gemm_ws, PrefillScratch::kGemmWsBytes);
    if (e == hipSuccess) e = hipStreamSynchronize(m->ctx->stream);
    if (e != hipSuccess) {
        S.release();
        return fail(e == hipErrorOutOfMemory ? RLH_ERR_OOM : RLH_ERR_HIP, "prefill work buffers for %d tokens: %s", n, hipGetErrorString(e));
    }
    S.n_cap = n;
    S.gemm_attention = gemm_attention;
    S.t_pad = (int)tp;
    return RLH_OK;
}

// Multi-token forward at start_pos == 0 in f16 mode: every projection is one matrix-core GEMM over all n rows
// (transformer.rs:694-702, 783-815, 551-570 with seq_len > 1), attention is two batched GEMMs per head around a
// causal softmax (transformer.rs:762-779).  Leaves the last row's logits in m->logits and the KV cache filled.
static int enqueue_prefill(rlh_model *m, rlh_caches *c, const int32_t *tokens, int n, const LayerSpan *span = nullptr) {
    int rc = ensure_prefill_scratch(m, n);
    if (rc != RLH_OK) return rc;
    hipStream_t st = m->ctx->stream;
    const rlh_model_params &P = m->prm;
    PrefillScratch &S = m->pf;
    const int d = P.dim, F = P.ffn_hidden, V = P.vocab_size, H = P.n_heads, hd = m->head_dim;
    const int tp = (n + 127) & ~127; // row stride of this call's scores / probabilities / transposed V (a whole number of key tiles)
    const float eps = (float)P.norm_eps;
    if (span) {
        HIP_TRY(hipMemcpyAsync(S.x, span->x_in, sizeof(float) * (size_t)n * d, hipMemcpyHostToDevice, st));
    } else {
        HIP_TRY(hipMemcpyAsync(m->prompt_dev, tokens, sizeof(int32_t) * (size_t)n, hipMemcpyHostToDevice, st));
        HIP_TRY(launch_set_state(m->state, n - 1, tokens[n - 1], 1, st));
        HIP_TRY(launch_embed_rows(m->tok_emb.p, m->tok_emb.f16, m->prompt_dev, n, d, S.x, st));
    }
    const int l_first = span ? span->first : 0, l_last = span ? span->last : P.n_layers - 1;
    const size_t layer_elems = (size_t)H * P.max_seq_len * hd;
    // norm_w / norm_done: the RMSNorm that follows a residual product, written to S.xn by the product itself where it can
    auto gemm = [&](const void *a, int lda, const void *b, int ldb, void *cc, int ldc, int mm, int nn, int kk, int epi, const float *res,
                    const void *gate = nullptr, const float *norm_w = nullptr, int *norm_done = nullptr) -> int {
        GemmParams g{};
        g.tune = m->ctx->tun.gemm;
        g.a = (const _Float16 *)a;
        g.b = (const _Float16 *)b;
        g.c = cc;
        g.residual = res;
        g.gate = (const _Float16 *)gate;
        g.norm_w = norm_w;
        g.norm_out = (_Float16 *)S.xn;
        g.norm_eps = eps;
        g.norm_done = norm_done;
        g.m = mm;
        g.n = nn;
        g.k = kk;
        g.lda = lda;
        g.ldb = ldb;
        g.ldc = ldc;
        g.batch = 1;
        g.workspace = S.gemm_ws;
        g.workspace_bytes = PrefillScratch::kGemmWsBytes;
        HIP_TRY(launch_gemm_f16(g, epi, st));
        return RLH_OK;
    };
    int normed = 0; // S.xn already holds this layer's attention_norm(S.x): the previous layer's w2 product wrote it
    for (int l = l_first; l <= l_last; l++) {
        Layer &L = m->layers[(size_t)l];
        char *ck = (char *)c->k + (size_t)l * layer_elems * 2;
        char *cv = (char *)c->v + (size_t)l * layer_elems * 2;
        if (!normed) HIP_TRY(launch_rmsnorm_rows_f16(S.xn, S.x, (const float *)L.attn_norm.p, n, d, eps, st));
        PrefillRopeParams rp{};
        rp.qkv = S.qkv;
        rp.freqs = m->freqs;
        rp.q_hi = S.q2;
        rp.q_lo = (char *)S.q2 + (size_t)hd * 2;
        rp.q_stride = 2 * hd;
        rp.cache_k = ck;
        rp.cache_v = cv;
        rp.cache_f16 = 1;
        rp.v_t = S.v_t;
        rp.n = n;
        rp.dim = d;
        rp.head_dim = hd;
        rp.max_seq_len = P.max_seq_len;
        rp.t_pad = tp;
        const bool fused = !m->ctx->tun.prefill_attn_gemm && attn_prefill_supported(hd);
        rp.vt_swap = fused ? 1 : 0;
        {
            // wq|wk|wv; RoPE, the hi + lo halves of q, the cache rows and V^T come straight out of the product's epilogue where
            // the shape allows, else the product is stored and a kernel of its own does the same
            GemmParams g{};
            g.tune = m->ctx->tun.gemm;
        g.tune = m->ctx->tun.gemm;
            g.a = (const _Float16 *)S.xn;
            g.b = (const _Float16 *)L.wqkv.p;
            g.c = S.qkv;
            g.m = n;
            g.n = 3 * d;
            g.k = d;
            g.lda = g.ldb = d;
            g.ldc = 3 * d;
            g.batch = 1;
            g.workspace = S.gemm_ws;
            g.workspace_bytes = PrefillScratch::kGemmWsBytes;
            g.rope = rp;
            if (gemm_f16_rope_supported(g)) {
                HIP_TRY(launch_gemm_f16(g, kGemmEpiRopeQkv, st));
            } else {
                HIP_TRY(launch_gemm_f16(g, kGemmEpiF16, st));
                HIP_TRY(launch_rope_kv_prefill(rp, st));
            }
        }
        if (fused) {
            // scores, mask, softmax and P.V in one kernel; the score matrix never reaches memory
            AttnPrefillParams ap{};
            ap.q2 = S.q2;
            ap.cache_k = ck;
            ap.v_t = S.v_t;
            ap.out = S.a;
            ap.n = n;
            ap.n_heads = H;
            ap.head_dim = hd;
            ap.dim = d;
            ap.max_seq_len = P.max_seq_len;
            ap.t_pad = tp;
            ap.scale = 1.0f / sqrtf((float)hd);
            ap.order = m->ctx->tun.prefill_attn_order;
            HIP_TRY(launch_attn_prefill(ap, st));
        } else {
            // scores[h] = q[h] . K[h]^T summed over the hi and lo parts of q: one pass that skips the tiles above the
            // diagonal where the fast GEMM takes head_dim as a K segment, else one accumulating pass per part
            const bool one_pass = hd % 64 == 0;
            for (int part = 0; part < (one_pass ? 1 : 2); part++) {
                GemmParams g{};
                g.tune = m->ctx->tun.gemm;
            g.tune = m->ctx->tun.gemm;
        g.tune = m->ctx->tun.gemm;
                g.a = (const _Float16 *)S.q2 + (size_t)part * hd;
                g.b = (const _Float16 *)ck;
                g.c = S.scores;
                g.m = n;
                g.n = n;
                g.k = one_pass ? 2 * hd : hd;
                g.k_seg = one_pass ? hd : 0;
                g.causal = one_pass ? 1 : 0;
                g.accumulate = part;
                g.lda = 2 * hd;
                g.ldb = hd;
                g.ldc = tp;
                g.batch = H;
                g.stride_a = (size_t)n * 2 * hd;
                g.stride_b = (size_t)P.max_seq_len * hd;
                g.stride_c = (size_t)n * tp;
                HIP_TRY(launch_gemm_f16(g, kGemmEpiF32, st));
            }
            HIP_TRY(launch_causal_softmax(S.scores, S.p2, (char *)S.p2 + (size_t)tp * 2, H, n, tp, 2 * tp, hd, st));
            {   // out[h] = P[h] . V[h] summed over the hi and lo parts of P, rounded to f16 and written as columns
                // h * hd .. of the [n x dim] input of wo (the concat of heads and the rounding point of transformer.rs:783-796)
                GemmParams g{};
                g.tune = m->ctx->tun.gemm;
            g.tune = m->ctx->tun.gemm;
        g.tune = m->ctx->tun.gemm;
                g.a = (const _Float16 *)S.p2;
                g.b = (const _Float16 *)S.v_t;
                g.c = S.a;
                g.m = n;
                g.n = hd;
                g.k = 2 * tp;
                g.k_seg = tp;
                g.causal = 2;
                g.lda = 2 * tp;
                g.ldb = tp;
                g.ldc = d;
                g.batch = H;
                g.stride_a = (size_t)n * 2 * tp;
                g.stride_b = (size_t)hd * tp;
                g.stride_c = (size_t)hd;
                HIP_TRY(launch_gemm_f16(g, kGemmEpiF16, st));
            }
        }
        normed = 0;
        if ((rc = gemm(S.a, d, L.wo.p, d, S.h, d, n, d, d, kGemmEpiResAddF32, S.x, nullptr, (const float *)L.ffn_norm.p, &normed)) != RLH_OK) return rc; // h = x + wo(att)
        if (!normed) HIP_TRY(launch_rmsnorm_rows_f16(S.xn, S.h, (const float *)L.ffn_norm.p, n, d, eps, st));
        {
            // SiLU(w1 x) * (w3 x) with the f16 rounding points of transformer.rs:557-565: where the shape allows, both products
            // in one pass over xn; otherwise w1's product goes to memory and w3's epilogue consumes it
            GemmParams g{};
            g.tune = m->ctx->tun.gemm;
        g.tune = m->ctx->tun.gemm;
            g.a = (const _Float16 *)S.xn;
            g.b = (const _Float16 *)L.w1.p;
            g.b2 = (const _Float16 *)L.w3.p;
            g.c = S.mm;
            g.m = n;
            g.n = F;
            g.k = d;
            g.lda = g.ldb = d;
            g.ldc = F;
            g.batch = 1;
            g.workspace = S.gemm_ws; // the same policy as rlh_ffn_gate: whether the pass runs is decided with the work memory in place
            g.workspace_bytes = PrefillScratch::kGemmWsBytes;
            if (gemm_f16_dual_gate_supported(g)) {
                HIP_TRY(launch_gemm_f16(g, kGemmEpiSiluGateF16, st));
            } else {
                if ((rc = gemm(S.xn, d, L.w1.p, d, S.g, F, n, F, d, kGemmEpiF16, nullptr)) != RLH_OK) return rc;
                if ((rc = gemm(S.xn, d, L.w3.p, d, S.mm, F, n, F, d, kGemmEpiSiluGateF16, nullptr, S.g)) != RLH_OK) return rc;
            }
        }
        // x = h + w2(...); the next block's attention_norm rides along where it can
        normed = 0;
        const float *next_norm = l < l_last ? (const float *)m->layers[(size_t)l + 1].attn_norm.p : nullptr;
        if ((rc = gemm(S.mm, F, L.w2.p, F, S.x, d, n, d, F, kGemmEpiResAddF32, S.h, nullptr, next_norm, next_norm ? &normed : nullptr)) != RLH_OK) return rc;
    }
    if (span) {
        HIP_TRY(hipMemcpyAsync(span->x_out, S.x, sizeof(float) * (size_t)n * d, hipMemcpyDeviceToHost, st));
        return RLH_OK;
    }
    // final norm + output head on the last row only (transformer.rs:378-381)
    GemvParams p{};
    p.stream_weights = m->stream_weights;
    p.w = m->output.p;
    p.w_is_f16 = m->output.f16;
    p.x = S.x + (size_t)(n - 1) * d;
    p.norm_w = (const float *)m->norm.p;
    p.eps = eps;
    p.y = m->logits;
    p.n_rows = V;
    p.k = d;
    HIP_TRY(launch_gemv(p, kEpiStore, st));
    return RLH_OK;
}

// f32 mode can take the matrix-core path when every K extent is a whole number of 32-float K-tiles
static bool prefill_f32_supported(const rlh_model *m) {
    return m->prm.dim % 32 == 0 && m->prm.ffn_hidden % 32 == 0 && m->head_dim % 32 == 0;
}

// Multi-token forward at start_pos == 0 in f32 mode: the same structure as enqueue_prefill on fp32 operands
// (v_mfma_f32_32x32x2_f32), no rounding points, residual adds as accumulating GEMM epilogues on x in place.
static int enqueue_prefill_f32(rlh_model *m, rlh_caches *c, const int32_t *tokens, int n, const LayerSpan *span = nullptr) {
    int rc = ensure_prefill_scratch(m, n);
    if (rc != RLH_OK) return rc;
    hipStream_t st = m->ctx->stream;
    const rlh_model_params &P = m->prm;
    PrefillScratch &S = m->pf;
    const int d = P.dim, F = P.ffn_hidden, V = P.vocab_size, H = P.n_heads, hd = m->head_dim;
    const int tp = (n + 63) & ~63;
    const float eps = (float)P.norm_eps;
    if (span) {
        HIP_TRY(hipMemcpyAsync(S.x, span->x_in, sizeof(float) * (size_t)n * d, hipMemcpyHostToDevice, st));
    } else {
        HIP_TRY(hipMemcpyAsync(m->prompt_dev, tokens, sizeof(int32_t) * (size_t)n, hipMemcpyHostToDevice, st));
        HIP_TRY(launch_set_state(m->state, n - 1, tokens[n - 1], 1, st));
        HIP_TRY(launch_embed_rows(m->tok_emb.p, m->tok_emb.f16, m->prompt_dev, n, d, S.x, st));
    }
    const int l_first = span ? span->first : 0, l_last = span ? span->last : P.n_layers - 1;
    const size_t layer_elems = (size_t)H * P.max_seq_len * hd;
    auto gemm = [&](const void *a, int lda, const void *b, int ldb, float *cc, int ldc, int mm, int nn, int kk, int accumulate) -> int {
        GemmParams g{};
        g.tune = m->ctx->tun.gemm;
        g.a = (const _Float16 *)a;
        g.b = (const _Float16 *)b;
        g.c = cc;
        g.m = mm;
        g.n = nn;
        g.k = kk;
        g.lda = lda;
        g.ldb = ldb;
        g.ldc = ldc;
        g.batch = 1;
        g.accumulate = accumulate;
        g.f32_operands = 1;
        g.workspace = S.gemm_ws;
        g.workspace_bytes = PrefillScratch::kGemmWsBytes;
        HIP_TRY(launch_gemm_f16(g, kGemmEpiF32, st));
        return RLH_OK;
    };
    float *xn = (float *)S.xn, *qkv = (float *)S.qkv, *q = (float *)S.q2, *v_t = (float *)S.v_t, *att = (float *)S.a;
    float *gg = (float *)S.g, *uu = (float *)S.u, *mm = (float *)S.mm;
    for (int l = l_first; l <= l_last; l++) {
        Layer &L = m->layers[(size_t)l];
        float *ck = (float *)c->k + (size_t)l * layer_elems;
        float *cv = (float *)c->v + (size_t)l * layer_elems;
        HIP_TRY(launch_rmsnorm_rows_f32(xn, S.x, (const float *)L.attn_norm.p, n, d, eps, st));
        if ((rc = gemm(xn, d, L.wqkv.p, d, qkv, 3 * d, n, 3 * d, d, 0)) != RLH_OK) return rc;
        PrefillRopeF32Params rp{};
        rp.qkv = qkv;
        rp.freqs = m->freqs;
        rp.q = q;
        rp.cache_k = ck;
        rp.cache_v = cv;
        rp.v_t = v_t;
        rp.n = n;
        rp.dim = d;
        rp.head_dim = hd;
        rp.max_seq_len = P.max_seq_len;
        rp.t_pad = tp;
        HIP_TRY(launch_rope_kv_prefill_f32(rp, st));
        {   // scores[h] = q[h] . K[h]^T, tiles above the diagonal skipped (transformer.rs:762-770)
            GemmParams g{};
            g.tune = m->ctx->tun.gemm;
        g.tune = m->ctx->tun.gemm;
            g.a = (const _Float16 *)q;
            g.b = (const _Float16 *)ck;
            g.c = S.scores;
            g.m = n;
            g.n = n;
            g.k = hd;
            g.causal = 1;
            g.lda = hd;
            g.ldb = hd;
            g.ldc = tp;
            g.batch = H;
            g.stride_a = (size_t)n * hd;
            g.stride_b = (size_t)P.max_seq_len * hd;
            g.stride_c = (size_t)n * tp;
            g.f32_operands = 1;
            HIP_TRY(launch_gemm_f16(g, kGemmEpiF32, st));
        }
        HIP_TRY(launch_causal_softmax_f32(S.scores, H, n, tp, hd, st));
        {   // out[h] = P[h] . V[h], written as columns h * hd .. of the [n x dim] input of wo (transformer.rs:777-796)
            GemmParams g{};
            g.tune = m->ctx->tun.gemm;
        g.tune = m->ctx->tun.gemm;
            g.a = (const _Float16 *)S.scores;
            g.b = (const _Float16 *)v_t;
            g.c = att;
            g.m = n;
            g.n = hd;
            g.k = tp;
            g.causal = 2;
            g.lda = tp;
            g.ldb = tp;
            g.ldc = d;
            g.batch = H;
            g.stride_a = (size_t)n * tp;
            g.stride_b = (size_t)hd * tp;
            g.stride_c = (size_t)hd;
            g.f32_operands = 1;
            HIP_TRY(launch_gemm_f16(g, kGemmEpiF32, st));
        }
        if ((rc = gemm(att, d, L.wo.p, d, S.x, d, n, d, d, 1)) != RLH_OK) return rc;     // x += wo(att)   (transformer.rs:442)
        HIP_TRY(launch_rmsnorm_rows_f32(xn, S.x, (const float *)L.ffn_norm.p, n, d, eps, st));
        if ((rc = gemm(xn, d, L.w1.p, d, gg, F, n, F, d, 0)) != RLH_OK) return rc;
        if ((rc = gemm(xn, d, L.w3.p, d, uu, F, n, F, d, 0)) != RLH_OK) return rc;
        HIP_TRY(launch_silu_mul_f32(gg, uu, mm, (size_t)n * F, st));
        if ((rc = gemm(mm, F, L.w2.p, F, S.x, d, n, d, F, 1)) != RLH_OK) return rc;      // x += w2(...)   (transformer.rs:445)
    }
    if (span) {
        HIP_TRY(hipMemcpyAsync(span->x_out, S.x, sizeof(float) * (size_t)n * d, hipMemcpyDeviceToHost, st));
        return RLH_OK;
    }
    // final norm + output head on the last row only (transformer.rs:378-381)
    GemvParams p{};
    p.stream_weights = m->stream_weights;
    p.w = m->output.p;
    p.w_is_f16 = m->output.f16;
    p.x = S.x + (size_t)(n - 1) * d;
    p.norm_w = (const float *)m->norm.p;
    p.eps = eps;
    p.y = m->logits;
    p.n_rows = V;
    p.k = d;
    HIP_TRY(launch_gemv(p, kEpiStore, st));
    return RLH_OK;
}

static int check_forward_args(rlh_model *m, rlh_caches *c, const int32_t *tokens, int n, int start_pos, const char *who) {
    if (!m || !c || !tokens) return fail(RLH_ERR_INVALID, "%s: NULL argument", who);
    if (c->model != m || c->model_uid != m->uid) return fail(RLH_ERR_STATE, "%s: caches belong to another model", who);
    if (m->n_resident < m->prm.n_layers) {
        return fail(RLH_ERR_STATE,
                    "%s: percentage_to_gpu %.4f keeps layers %d.. on the host (transformer.rs:262-279): run rlh_forward_layers over 0..%d and the "
                    "remaining blocks, the final norm and the output head with the host's own path",
                    who, (double)m->prm.percentage_to_gpu, m->n_resident, m->last_layer_on_gpu);
    }
    if (!model_ready(m)) return fail(RLH_ERR_STATE, "%s: model has tensors that were never set", who);
    if (n < 1) return fail(RLH_ERR_INVALID, "%s: n must be >= 1", who);
    if (n > 1 && start_pos != 0) {
        return fail(RLH_ERR_INVALID, "%s: n > 1 needs start_pos == 0 (the reference's mask is n x n, transformer.rs:350-357)", who);
    }
    if (start_pos < 0 || start_pos + n > m->prm.max_seq_len) {
        return fail(RLH_ERR_STATE, "%s: start_pos + n = %d exceeds max_seq_len %d", who, start_pos + n, m->prm.max_seq_len);
    }
    for (int i = 0; i < n; i++) {
        if (tokens[i] < 0 || tokens[i] >= m->prm.vocab_size) return fail(RLH_ERR_INVALID, "%s: token id %d out of range", who, tokens[i]);
    }
    return RLH_OK;
}

// Runs the n tokens of one forward call; logits of the last one are left in m->logits.
static int enqueue_forward(rlh_model *m, rlh_caches *c, const int32_t *tokens, int n, int start_pos) {
    hipStream_t st = m->ctx->stream;
    m->next_pos = -1;
    m->greedy_caches = nullptr;
    if (n > 1 && m->prefill_mode == 0) {
        if (m->prm.force_f16) return enqueue_prefill(m, c, tokens, n);
        if (prefill_f32_supported(m)) return enqueue_prefill_f32(m, c, tokens, n);
    }
    HIP_TRY(hipMemcpyAsync(m->prompt_dev, tokens, sizeof(int32_t) * (size_t)n, hipMemcpyHostToDevice, st));
    HIP_TRY(launch_set_state(m->state, start_pos, tokens[0], 1, st));
    for (int i = 0; i < n; i++) {
        int rc = enqueue_token_step(m, c, start_pos + i + 1, i == n - 1);
        if (rc != RLH_OK) return rc;
        if (i + 1 < n) HIP_TRY(launch_advance_pos(m->state, m->prompt_dev, i + 1, st));
    }
    return RLH_OK;
}

extern "C" int rlh_forward(rlh_model *m, rlh_caches *c, const int32_t *tokens, int n, int start_pos, float *logits_out) {
    int rc = check_forward_args(m, c, tokens, n, start_pos, "rlh_forward");
    if (rc != RLH_OK) return rc;
    if (!logits_out) return fail(RLH_ERR_INVALID, "rlh_forward: logits_out is NULL");
    CtxLock lock(m->ctx);
    rc = enqueue_forward(m, c, tokens, n, start_pos);
    if (rc != RLH_OK) return rc;
    HIP_TRY(hipMemcpyAsync(logits_out, m->logits, sizeof(float) * (size_t)m->prm.vocab_size, hipMemcpyDeviceToHost, m->ctx->stream));
    HIP_TRY(hipStreamSynchronize(m->ctx->stream));
    return RLH_OK;
}

// forward + the device pick at top_k = 1 on logits * scale
static int forward_greedy_scaled(rlh_model *m, rlh_caches *c, const int32_t *tokens, int n, int start_pos, int32_t *next_token, float scale) {
    int rc = check_forward_args(m, c, tokens, n, start_pos, "rlh_forward_greedy");
    if (rc != RLH_OK) return rc;
    if (!next_token) return fail(RLH_ERR_INVALID, "rlh_forward_greedy: next_token is NULL");
    CtxLock lock(m->ctx);
    hipStream_t st = m->ctx->stream;
    rc = enqueue_forward(m, c, tokens, n, start_pos);
    if (rc != RLH_OK) return rc;
    HIP_TRY(launch_argmax_advance(m->logits, m->prm.vocab_size, m->state, m->out_tokens, m->out_cap, st, scale));
    HIP_TRY(hipMemcpyAsync(next_token, m->out_tokens, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    HIP_TRY(hipStreamSynchronize(st));
    m->next_pos = start_pos + n;
    m->greedy_caches = c;
    return RLH_OK;
}

extern "C" int rlh_forward_greedy(rlh_model *m, rlh_caches *c, const int32_t *tokens, int n, int start_pos, int32_t *next_token) {
    return forward_greedy_scaled(m, c, tokens, n, start_pos, next_token, 1.0f);
}

extern "C" int rlh_forward_layers(rlh_model *m, rlh_caches *c, const float *x_in, int n, int start_pos, int first_layer, int last_layer,
                                  float *x_out) {
    if (!m || !c || !x_in || !x_out) return fail(RLH_ERR_INVALID, "rlh_forward_layers: NULL argument");
    if (c->model != m || c->model_uid != m->uid) return fail(RLH_ERR_STATE, "rlh_forward_layers: caches belong to another model");
    if (first_layer < 0 || last_layer < first_layer || last_layer >= m->prm.n_layers) {
        return fail(RLH_ERR_INVALID, "rlh_forward_layers: layers %d..%d out of range (model has %d)", first_layer, last_layer, m->prm.n_layers);
    }
    if (last_layer >= m->n_resident) {
        return fail(RLH_ERR_STATE, "rlh_forward_layers: layer %d stays on the host: percentage_to_gpu %.4f keeps layers 0..%d on the device",
                    last_layer, (double)m->prm.percentage_to_gpu, m->last_layer_on_gpu);
    }
    if (!layers_ready(m, first_layer, last_layer)) return fail(RLH_ERR_STATE, "rlh_forward_layers: layers %d..%d have tensors that were never set", first_layer, last_layer);
    if (n < 1) return fail(RLH_ERR_INVALID, "rlh_forward_layers: n must be >= 1");
    if (n > 1 && start_pos != 0) {
        return fail(RLH_ERR_INVALID, "rlh_forward_layers: n > 1 needs start_pos == 0 (the reference's mask is n x n, transformer.rs:350-357)");
    }
    if (start_pos < 0 || start_pos + n > m->prm.max_seq_len) {
        return fail(RLH_ERR_STATE, "rlh_forward_layers: start_pos + n = %d exceeds max_seq_len %d", start_pos + n, m->prm.max_seq_len);
    }
    CtxLock lock(m->ctx);
    hipStream_t st = m->ctx->stream;
    m->next_pos = -1; // the device state no longer describes a sampled token
    m->greedy_caches = nullptr;
    LayerSpan span;
    span.first = first_layer;
    span.last = last_layer;
    span.x_in = x_in;
    span.x_out = x_out;
    int rc = RLH_OK;
    if (n > 1 && m->prefill_mode == 0 && (m->prm.force_f16 || prefill_f32_supported(m))) {
        rc = m->prm.force_f16 ? enqueue_prefill(m, c, nullptr, n, &span) : enqueue_prefill_f32(m, c, nullptr, n, &span);
        if (rc != RLH_OK) return rc;
    } else {
        const int d = m->prm.dim;
        for (int i = 0; i < n; i++) {
            HIP_TRY(launch_set_state(m->state, start_pos + i, 0, 1, st));
            HIP_TRY(hipMemcpyAsync(m->x, x_in + (size_t)i * d, sizeof(float) * (size_t)d, hipMemcpyHostToDevice, st));
            for (int l = first_layer; l <= last_layer; l++) {
                for (int which = kStepQkv; which <= kStepW2; which++) {
                    rc = enqueue_step_kernel(m, c, l, which, start_pos + i + 1, first_layer);
                    if (rc != RLH_OK) return rc;
                }
            }
            // the last block's second residual add (transformer.rs:445), which a following kernel's prologue would have done
            HIP_TRY(launch_add_f32(m->x, m->h, m->ffn_o, (uint64_t)d, st));
            HIP_TRY(hipMemcpyAsync(x_out + (size_t)i * d, m->x, sizeof(float) * (size_t)d, hipMemcpyDeviceToHost, st));
        }
    }
    HIP_TRY(hipStreamSynchronize(st));
    return RLH_OK;
}

extern "C" int rlh_forward_sample(rlh_model *m, rlh_caches *c, const int32_t *tokens, int n, int start_pos, const rlh_sampler_params *sp,
                                  const int32_t *existing_tokens, int n_existing, float u, int32_t *token, float *prob) {
    if (!sp || !token) return fail(RLH_ERR_INVALID, "rlh_forward_sample: NULL argument");
    if (sp->top_k == 1) {
        // one candidate: the draw cannot choose.  Which one it is does not depend on the penalty (it only reaches token 0,
        // whose value is then shifted to 0); the temperature matters only through what it does to the un-shifted softmax
        // (scaled logits beyond ln(FLT_MAX) turn probabilities into NaN), so the device pick runs on the scaled logits
        // (token_sampler.rs:99-147).
        const float scale = sp->temperature > 0.0f ? 1.0f / sp->temperature : 1.0f;
        const int rc = forward_greedy_scaled(m, c, tokens, n, start_pos, token, scale);
        if (rc == RLH_OK && prob) *prob = 1.0f; // v.1 / total_p with a single candidate (:170)
        return rc;
    }
    if (!m) return fail(RLH_ERR_INVALID, "rlh_forward_sample: NULL argument");
    std::vector<float> logits((size_t)m->prm.vocab_size);
    int rc = rlh_forward(m, c, tokens, n, start_pos, logits.data());
    if (rc != RLH_OK) return rc;
    return rlh_sample(logits.data(), m->prm.vocab_size, sp, existing_tokens, n_existing, u, token, prob);
}

// One greedy decode step: the token step for the token in the device state, then argmax + advance.  With
// RLLAMA_HIP_DECODE_GRAPH=1 the step is captured once per attention grid shape (the only launch parameter that depends on
// the host's view of the position) and replayed as a graph.
static int enqueue_decode_step(rlh_model *m, rlh_caches *c, int T_host) {
    const bool use_graph = m->ctx->tun.decode_graph != 0;
    hipStream_t st = m->ctx->stream;
    if (!use_graph) return enqueue_token_step(m, c, T_host, true, true);
    if (c->graphs_tun_version != m->ctx->tun_version) { // captured under other switches
        for (auto &kv : c->step_graphs) (void)hipGraphExecDestroy(kv.second);
        c->step_graphs.clear();
        c->graphs_tun_version = m->ctx->tun_version;
    }
    const int key = attn_splits(m, T_host);
    auto it = c->step_graphs.find(key);
    if (it == c->step_graphs.end()) {
        hipGraph_t graph = nullptr;
        HIP_TRY(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        m->capturing = true;
        int rc = enqueue_token_step(m, c, T_host, true, true);
        m->capturing = false;
        hipError_t e2 = hipStreamEndCapture(st, &graph);
        if (rc != RLH_OK || e2 != hipSuccess) {
            if (graph) (void)hipGraphDestroy(graph);
            if (rc != RLH_OK) return rc;
            HIP_TRY(e2);
        }
        hipGraphExec_t exec = nullptr;
        hipError_t e3 = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        HIP_TRY(e3);
        it = c->step_graphs.emplace(key, exec).first;
    }
    HIP_TRY(hipGraphLaunch(it->second, st));
    return RLH_OK;
}

extern "C" int rlh_generate_greedy(rlh_model *m, rlh_caches *c, const int32_t *prompt, int n_prompt, int n_new, int32_t *out_tokens,
                                   float *ms_first, float *ms_per_token) {
    int rc = check_forward_args(m, c, prompt, n_prompt, 0, "rlh_generate_greedy");
    if (rc != RLH_OK) return rc;
    if (!out_tokens || n_new < 1) return fail(RLH_ERR_INVALID, "rlh_generate_greedy: bad output arguments");
    if (n_prompt + n_new - 1 > m->prm.max_seq_len) {
        return fail(RLH_ERR_STATE, "rlh_generate_greedy: %d prompt + %d new tokens exceed max_seq_len %d", n_prompt, n_new, m->prm.max_seq_len);
    }
    CtxLock lock(m->ctx);
    hipStream_t st = m->ctx->stream;
    hipEvent_t e0 = nullptr, e1 = nullptr, e2 = nullptr;
    auto cleanup = [&]() {
        for (hipEvent_t ev : {e0, e1, e2})
            if (ev) (void)hipEventDestroy(ev);
    };
    hipError_t e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) e = hipEventCreate(&e2);
    if (e == hipSuccess) e = hipEventRecord(e0, st);
    if (e == hipSuccess) {
        rc = enqueue_forward(m, c, prompt, n_prompt, 0);
        if (rc == RLH_OK) e = launch_argmax_advance(m->logits, m->prm.vocab_size, m->state, m->out_tokens, m->out_cap, st);
    }
    if (rc == RLH_OK && e == hipSuccess) e = hipEventRecord(e1, st);
    for (int i = 1; rc == RLH_OK && e == hipSuccess && i < n_new; i++) {
        // the new token sits at position n_prompt + i - 1; attention spans n_prompt + i positions
        rc = enqueue_decode_step(m, c, n_prompt + i);
    }
    if (rc == RLH_OK && e == hipSuccess) e = hipEventRecord(e2, st);
    if (rc == RLH_OK && e == hipSuccess) e = hipMemcpyAsync(out_tokens, m->out_tokens, sizeof(int32_t) * (size_t)n_new, hipMemcpyDeviceToHost, st);
    if (rc == RLH_OK && e == hipSuccess) e = hipStreamSynchronize(st);
    if (rc == RLH_OK && e == hipSuccess) {
        float a = 0.0f, b = 0.0f;
        (void)hipEventElapsedTime(&a, e0, e1);
        (void)hipEventElapsedTime(&b, e1, e2);
        if (ms_first) *ms_first = a;
        if (ms_per_token) *ms_per_token = n_new > 1 ? b / (float)(n_new - 1) : 0.0f;
    }
    cleanup();
    if (rc != RLH_OK) return rc;
    HIP_TRY(e);
    m->next_pos = n_prompt + n_new - 1;
    m->greedy_caches = c;
    return RLH_OK;
}

extern "C" int rlh_decode_greedy(rlh_model *m, rlh_caches *c, int n_steps, int32_t *out_tokens, float *ms_total) {
    if (!m || !c || !out_tokens || n_steps < 1) return fail(RLH_ERR_INVALID, "rlh_decode_greedy: bad argument");
    if (c->model != m || c->model_uid != m->uid) return fail(RLH_ERR_STATE, "rlh_decode_greedy: caches belong to another model");
    if (m->next_pos < 0 || m->greedy_caches != c) {
        return fail(RLH_ERR_STATE, "rlh_decode_greedy: no sampled token on the device for these caches (call rlh_forward_greedy or rlh_generate_greedy first)");
    }
    if (m->next_pos + n_steps > m->prm.max_seq_len) {
        return fail(RLH_ERR_STATE, "rlh_decode_greedy: position %d + %d steps exceed max_seq_len %d", m->next_pos, n_steps, m->prm.max_seq_len);
    }
    if (n_steps > m->out_cap) return fail(RLH_ERR_INVALID, "rlh_decode_greedy: n_steps too large");
    CtxLock lock(m->ctx);
    hipStream_t st = m->ctx->stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    HIP_TRY(hipEventCreate(&e0));
    hipError_t e = hipEventCreate(&e1);
    int rc = RLH_OK;
    // keep pos/token, restart the output list
    if (e == hipSuccess) e = launch_reset_out(m->state, st);
    if (e == hipSuccess) e = hipEventRecord(e0, st);
    for (int i = 0; rc == RLH_OK && e == hipSuccess && i < n_steps; i++) {
        rc = enqueue_decode_step(m, c, m->next_pos + i + 1);
    }
    if (rc == RLH_OK && e == hipSuccess) e = hipEventRecord(e1, st);
    if (rc == RLH_OK && e == hipSuccess) e = hipMemcpyAsync(out_tokens, m->out_tokens, sizeof(int32_t) * (size_t)n_steps, hipMemcpyDeviceToHost, st);
    hipError_t e2 = hipStreamSynchronize(st);
    float ms = 0.0f;
    if (rc == RLH_OK && e == hipSuccess && e2 == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (rc != RLH_OK || e != hipSuccess || e2 != hipSuccess) m->next_pos = -1;
    if (rc != RLH_OK) return rc;
    HIP_TRY(e);
    HIP_TRY(e2);
    if (ms_total) *ms_total = ms;
    m->next_pos += n_steps;
    return RLH_OK;
}

// ------------------------------------------------------------------------------------------------
// measurement aids
// ------------------------------------------------------------------------------------------------
extern "C" int rlh_model_time_kernel(rlh_model *m, rlh_caches *c, int which, int T, int iters, float *us_per_launch, uint64_t *bytes_per_launch) {
    if (!m || !c || !us_per_launch || iters < 1) return fail(RLH_ERR_INVALID, "rlh_model_time_kernel: bad argument");
    if (c->model != m || c->model_uid != m->uid) return fail(RLH_ERR_STATE, "rlh_model_time_kernel: caches belong to another model");
    if (!model_ready(m)) return fail(RLH_ERR_STATE, "rlh_model_time_kernel: model has tensors that were never set");
    if (T < 1 || T > m->prm.max_seq_len || which < kStepQkv || which > kStepHead) return fail(RLH_ERR_INVALID, "rlh_model_time_kernel: bad T or kernel id");
    CtxLock lock(m->ctx);
    hipStream_t st = m->ctx->stream;
    const uint64_t d = (uint64_t)m->prm.dim, F = (uint64_t)m->prm.ffn_hidden, V = (uint64_t)m->prm.vocab_size;
    const uint64_t es = m->prm.force_f16 ? 2 : 4;
    if (bytes_per_launch) {
        // algorithmic bytes: the weights the kernel must read once + its input and output vectors
        switch (which) {
        case kStepQkv: *bytes_per_launch = 3 * d * d * es + d * 4 + d * 4 + d * 4 + 2 * d * es; break;
        case kStepAttn: *bytes_per_launch = 2 * (uint64_t)T * d * es + d * 4 + d * 4; break;
        case kStepWo: *bytes_per_launch = d * d * es + d * 4 + 2 * d * 4; break;
        case kStepW13: *bytes_per_launch = 2 * F * d * es + d * 4 + d * 4 + F * 4; break;
        case kStepW2: *bytes_per_launch = d * F * es + F * 4 + 2 * d * 4; break;
        default: *bytes_per_launch = V * d * (m->output.f16 ? 2 : 4) + d * 4 + d * 4 + V * 4; break;
        }
    }
    // the timed launches run on the model's own token-step state and buffers: whatever greedy loop was in progress is over
    m->next_pos = -1;
    m->greedy_caches = nullptr;
    HIP_TRY(launch_set_state(m->state, T - 1, 3 % m->prm.vocab_size, 1, st));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    HIP_TRY(hipEventCreate(&e0));
    HIP_TRY(hipEventCreate(&e1));
    int rc = RLH_OK;
    const int L = m->prm.n_layers;
    auto one = [&](int i) { return enqueue_step_kernel(m, c, i % L, which, T); };
    for (int i = 0; rc == RLH_OK && i < (L < 4 ? L : 4); i++) rc = one(i); // warm-up
    hipError_t e = hipEventRecord(e0, st);
    for (int i = 0; rc == RLH_OK && e == hipSuccess && i < iters; i++) rc = one(i);
    if (e == hipSuccess) e = hipEventRecord(e1, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != RLH_OK) return rc;
    HIP_TRY(e);
    *us_per_launch = ms * 1000.0f / (float)iters;
    return RLH_OK;
}

extern "C" int rlh_time_gemv(rlh_ctx *ctx, int rows, int k, int w_dtype, int round_x, int round_y, int n_buffers, int iters, float *us_per_launch) {
    if (!ctx || !us_per_launch || rows < 1 || k < 1 || n_buffers < 1 || iters < 1) return fail(RLH_ERR_INVALID, "rlh_time_gemv: bad argument");
    const int f16 = w_dtype == RLH_F16;
    if (k % (f16 ? 8 : 4) != 0) return fail(RLH_ERR_UNSUPPORTED, "rlh_time_gemv: k must be a multiple of %d", f16 ? 8 : 4);
    CtxLock lock(ctx);
    hipStream_t st = ctx->stream;
    const size_t wbytes = (size_t)rows * k * (f16 ? 2 : 4);
    std::vector<void *> bufs((size_t)n_buffers, nullptr);
    float *x = nullptr, *y = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipSuccess;
    for (int i = 0; e == hipSuccess && i < n_buffers; i++) {
        e = hipMalloc(&bufs[(size_t)i], wbytes);
        if (e == hipSuccess) e = launch_synth_fill(bufs[(size_t)i], f16, (uint64_t)rows * k, synth_key(99, (uint64_t)i), 0.02, st);
    }
    if (e == hipSuccess) e = hipMalloc((void **)&x, sizeof(float) * (size_t)k);
    if (e == hipSuccess) e = hipMalloc((void **)&y, sizeof(float) * (size_t)rows);
    if (e == hipSuccess) e = launch_fill_f32(x, (uint64_t)k, 0.5f, st);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    GemvParams p{};
    p.w_is_f16 = f16;
    p.x = x;
    p.x_f16 = round_x ? 1 : 0;
    p.round_y = round_y ? 1 : 0;
    p.y = y;
    p.n_rows = rows;
    p.k = k;
    p.stream_weights = 1;
    p.burst_fixed = ctx->tun.gemv_burst_fixed;
    for (int i = 0; e == hipSuccess && i < n_buffers; i++) {
        p.w = bufs[(size_t)i];
        e = launch_gemv(p, kEpiStore, st);
    }
    if (e == hipSuccess) e = hipEventRecord(e0, st);
    for (int i = 0; e == hipSuccess && i < iters; i++) {
        p.w = bufs[(size_t)(i % n_buffers)];
        e = launch_gemv(p, kEpiStore, st);
    }
    if (e == hipSuccess) e = hipEventRecord(e1, st);
    hipError_t e2 = hipStreamSynchronize(st);
    float ms = 0.0f;
    if (e == hipSuccess && e2 == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    for (void *b : bufs)
        if (b) (void)hipFree(b);
    if (x) (void)hipFree(x);
    if (y) (void)hipFree(y);
    HIP_TRY(e);
    HIP_TRY(e2);
    *us_per_launch = ms * 1000.0f / (float)iters;
    return RLH_OK;
}

extern "C" int rlh_probe_gemv_phases(rlh_ctx *ctx, int rows, int k, int n_buffers, int launches, float *out_us) {
    if (!ctx || !out_us || rows < 1 || k < 8 || k % 8 != 0 || n_buffers < 1 || launches < 2 || launches > 256) return fail(RLH_ERR_INVALID, "rlh_probe_gemv_phases: bad argument");
    CtxLock lock(ctx);
    hipStream_t st = ctx->stream;
    const size_t wbytes = (size_t)rows * k * 2;
    std::vector<void *> bufs((size_t)n_buffers, nullptr);
    float *x = nullptr, *y = nullptr;
    unsigned long long *stamps = nullptr;
    constexpr int kS = 5;
    const size_t max_waves = 2048 + 64;
    hipError_t e = hipSuccess;
    for (int i = 0; e == hipSuccess && i < n_buffers; i++) {
        e = hipMalloc(&bufs[(size_t)i], wbytes);
        if (e == hipSuccess) e = launch_synth_fill(bufs[(size_t)i], 1, (uint64_t)rows * k, synth_key(98, (uint64_t)i), 0.02, st);
    }
    if (e == hipSuccess) e = hipMalloc((void **)&x, sizeof(float) * (size_t)k);
    if (e == hipSuccess) e = hipMalloc((void **)&y, sizeof(float) * (size_t)rows);
    if (e == hipSuccess) e = hipMalloc((void **)&stamps, sizeof(unsigned long long) * (size_t)launches * max_waves * kS);
    if (e == hipSuccess) e = hipMemsetAsync(stamps, 0, sizeof(unsigned long long) * (size_t)launches * max_waves * kS, st);
    if (e == hipSuccess) e = launch_fill_f32(x, (uint64_t)k, 0.5f, st);
    GemvParams p{};
    p.w_is_f16 = 1;
    p.x = x;
    p.y = y;
    p.n_rows = rows;
    p.k = k;
    p.stream_weights = 1;
    int n_waves = 0;
    for (int i = 0; e == hipSuccess && i < launches; i++) {
        p.w = bufs[(size_t)(i % n_buffers)];
        p.stamps = stamps + (size_t)i * max_waves * kS;
        e = launch_gemv_stamped(p, st, (int)max_waves, &n_waves);
    }
    std::vector<unsigned long long> host;
    if (e == hipSuccess) {
        host.resize((size_t)launches * max_waves * kS);
        e = hipMemcpyAsync(host.data(), stamps, host.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost, st);
    }
    hipError_t e2 = hipStreamSynchronize(st);
    for (void *b : bufs)
        if (b) (void)hipFree(b);
    for (void *b : {(void *)x, (void *)y, (void *)stamps})
        if (b) (void)hipFree(b);
    HIP_TRY(e);
    HIP_TRY(e2);
    double acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    unsigned long long prev_last_exit = 0;
    int counted = 0;
    for (int i = 0; i < launches; i++) {
        const unsigned long long *s = host.data() + (size_t)i * max_waves * kS;
        unsigned long long first_in = ~0ull, last_in = 0, first_out = ~0ull, last_out = 0;
        double pro = 0, lat = 0, stream = 0, epi = 0;
        for (int w = 0; w < n_waves; w++) {
            const unsigned long long *t = s + (size_t)w * kS;
            first_in = std::min(first_in, t[0]);
            last_in = std::max(last_in, t[0]);
            first_out = std::min(first_out, t[4]);
            last_out = std::max(last_out, t[4]);
            pro += (double)(t[1] - t[0]);
            lat += (double)(t[2] - t[1]);
            stream += (double)(t[3] - t[2]);
            epi += (double)(t[4] - t[3]);
        }
        if (i > 0) {
            acc[0] += (double)first_in - (double)prev_last_exit;
            acc[1] += (double)(last_in - first_in);
            acc[2] += pro / n_waves;
            acc[3] += lat / n_waves;
            acc[4] += stream / n_waves;
            acc[5] += epi / n_waves;
            acc[6] += (double)(last_out - first_out);
            acc[7] += (double)(last_out - first_in);
            counted++;
        }
        prev_last_exit = last_out;
    }
    for (int j = 0; j < 8; j++) out_us[j] = (float)(acc[j] / counted * 0.01); // 100 MHz ticks -> microseconds
    return RLH_OK;
}

// ------------------------------------------------------------------------------------------------
// synthetic inputs on the host
// ------------------------------------------------------------------------------------------------
extern "C" void rlh_synth_normal_f16(uint64_t seed, int kind, int layer, uint64_t first_index, uint64_t count, double std, uint16_t *out) {
    const uint64_t key = synth_key(seed, SYNTH_STREAM_TENSOR(kind, layer));
    unsigned nt = std::thread::hardware_concurrency();
    if (nt > 16) nt = 16;
    if (nt < 1 || count < (1u << 16)) nt = 1;
    auto work = [=](uint64_t lo, uint64_t hi) {
        uint64_t have = ~0ull; // pair whose deviates are in z0, z1
        double z0 = 0.0, z1 = 0.0;
        for (uint64_t i = lo; i < hi; i++) {
            const uint64_t idx = first_index + i;
            if ((idx >> 1) != have) {
                have = idx >> 1;
                synth_normal_pair(key, have, &z0, &z1);
            }
            out[i] = synth_scale_to_f16((idx & 1u) ? z1 : z0, std);
        }
    };
    if (nt == 1) {
        work(0, count);
        return;
    }
    std::vector<std::thread> pool;
    const uint64_t per = (count + nt - 1) / nt;
    for (unsigned t = 0; t < nt; t++) {
        const uint64_t lo = (uint64_t)t * per, hi = lo + per < count ? lo + per : count;
        if (lo < hi) pool.emplace_back(work, lo, hi);
    }
    for (auto &th : pool) th.join();
}

extern "C" void rlh_synth_tokens(uint64_t seed, uint64_t first_index, uint64_t count, int32_t lo, int32_t hi, int32_t *out) {
    const uint64_t key = synth_key(seed, SYNTH_STREAM_TOKENS);
    for (uint64_t i = 0; i < count; i++) out[i] = synth_token(key, first_index + i, lo, hi);
}
