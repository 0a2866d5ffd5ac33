// api_ops.hip -- the op-level entry points of the C ABI (include/rllama_hip.h): device tensors and the single operations
// on them, mirroring OpenCLTensor (Noeda/rllama, src/tensor_opencl_support.rs:134-405) plus the steps of the forward the
// reference runs on the host (attention, residual add, greedy pick) so that each kernel can be checked alone.
#include "api_internal.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

using namespace rlh;

// ------------------------------------------------------------------------------------------------
// op level
// ------------------------------------------------------------------------------------------------
extern "C" int rlh_tensor_alloc(rlh_ctx *ctx, int rows, int cols, int dtype, rlh_tensor **out) {
    if (!ctx || !out || rows <= 0 || cols <= 0 || (dtype != RLH_F16 && dtype != RLH_F32)) return fail(RLH_ERR_INVALID, "rlh_tensor_alloc: bad argument");
    *out = nullptr;
    CtxLock lock(ctx);
    rlh_tensor *t = new rlh_tensor();
    t->ctx = ctx;
    t->rows = rows;
    t->cols = cols;
    t->dtype = dtype;
    hipError_t e = hipMalloc(&t->p, t->count() * t->esize());
    if (e == hipSuccess) e = hipMemsetAsync(t->p, 0, t->count() * t->esize(), ctx->stream);
    if (e != hipSuccess) {
        if (t->p) (void)hipFree(t->p);
        delete t;
        return fail(e == hipErrorOutOfMemory ? RLH_ERR_OOM : RLH_ERR_HIP, "rlh_tensor_alloc: %s", hipGetErrorString(e));
    }
    *out = t;
    return RLH_OK;
}

extern "C" int rlh_tensor_upload(rlh_ctx *ctx, const void *host, int rows, int cols, int cols_capacity, int dtype, rlh_tensor **out) {
    if (!host || cols_capacity < cols) return fail(RLH_ERR_INVALID, "rlh_tensor_upload: bad argument");
    int rc = rlh_tensor_alloc(ctx, rows, cols, dtype, out);
    if (rc != RLH_OK) return rc;
    CtxLock lock(ctx);
    rlh_tensor *t = *out;
    const size_t es = t->esize();
    hipError_t e = hipMemcpy2DAsync(t->p, (size_t)cols * es, host, (size_t)cols_capacity * es, (size_t)cols * es, (size_t)rows,
                                    hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream); // the host buffer is the caller's again on return
    if (e != hipSuccess) {
        rlh_tensor_free(t);
        *out = nullptr;
        return fail(RLH_ERR_HIP, "rlh_tensor_upload: %s", hipGetErrorString(e));
    }
    return RLH_OK;
}

extern "C" int rlh_tensor_download(rlh_tensor *t, void *host, int cols_capacity, rlh_event **ev) {
    if (!t || !host || cols_capacity < t->cols) return fail(RLH_ERR_INVALID, "rlh_tensor_download: bad argument");
    CtxLock lock(t->ctx);
    const size_t es = t->esize();
    HIP_TRY(hipMemcpy2DAsync(host, (size_t)cols_capacity * es, t->p, (size_t)t->cols * es, (size_t)t->cols * es, (size_t)t->rows,
                             hipMemcpyDeviceToHost, t->ctx->stream));
    if (ev) {
        int rc = rlh_event_record(t->ctx, ev);
        if (rc != RLH_OK) return rc;
    } else {
        HIP_TRY(hipStreamSynchronize(t->ctx->stream));
    }
    return RLH_OK;
}

extern "C" void rlh_tensor_free(rlh_tensor *t) {
    if (!t) return;
    CtxLock lock(t->ctx);
    (void)hipStreamSynchronize(t->ctx->stream);
    if (t->p) (void)hipFree(t->p);
    delete t;
}

extern "C" int rlh_tensor_shape(const rlh_tensor *t, int *rows, int *cols, int *dtype) {
    if (!t) return fail(RLH_ERR_INVALID, "rlh_tensor_shape: NULL tensor");
    if (rows) *rows = t->rows;
    if (cols) *cols = t->cols;
    if (dtype) *dtype = t->dtype;
    return RLH_OK;
}

extern "C" int rlh_event_record(rlh_ctx *ctx, rlh_event **out) {
    if (!ctx || !out) return fail(RLH_ERR_INVALID, "rlh_event_record: NULL argument");
    CtxLock lock(ctx);
    rlh_event *ev = new rlh_event();
    ev->ctx = ctx;
    hipError_t e = hipEventCreate(&ev->ev);
    if (e == hipSuccess) e = hipEventRecord(ev->ev, ctx->stream);
    if (e != hipSuccess) {
        if (ev->ev) (void)hipEventDestroy(ev->ev);
        delete ev;
        return fail(RLH_ERR_HIP, "rlh_event_record: %s", hipGetErrorString(e));
    }
    *out = ev;
    return RLH_OK;
}

extern "C" int rlh_event_wait(rlh_event *ev) {
    if (!ev) return fail(RLH_ERR_INVALID, "rlh_event_wait: NULL event");
    hipError_t e = hipEventSynchronize(ev->ev);
    (void)hipEventDestroy(ev->ev);
    delete ev;
    if (e != hipSuccess) return fail(RLH_ERR_HIP, "rlh_event_wait: %s", hipGetErrorString(e));
    return RLH_OK;
}

extern "C" int rlh_event_elapsed_ms(rlh_event *start, rlh_event *stop, float *ms) {
    if (!start || !stop || !ms) return fail(RLH_ERR_INVALID, "rlh_event_elapsed_ms: NULL argument");
    HIP_TRY(hipEventSynchronize(stop->ev));
    HIP_TRY(hipEventElapsedTime(ms, start->ev, stop->ev));
    return RLH_OK;
}

extern "C" void rlh_event_free(rlh_event *ev) {
    if (!ev) return;
    if (ev->ev) (void)hipEventDestroy(ev->ev);
    delete ev;
}

static int same_shape(const rlh_tensor *a, const rlh_tensor *b) { return a->rows == b->rows && a->cols == b->cols && a->dtype == b->dtype; }

extern "C" int rlh_copy_inplace(rlh_tensor *dst, const rlh_tensor *src) {
    if (!dst || !src || !same_shape(dst, src)) return fail(RLH_ERR_INVALID, "rlh_copy_inplace: shape/dtype mismatch");
    CtxLock lock(dst->ctx);
    // a plain copy kernel (the reference's copy_inplace is a kernel too); also the calibration point for HBM counters
    HIP_TRY(launch_convert(dst->p, dst->dtype == RLH_F16, src->p, src->dtype == RLH_F16, dst->count(), dst->ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_transpose_from(rlh_tensor *dst, const rlh_tensor *src) {
    if (!dst || !src || dst->rows != src->cols || dst->cols != src->rows || dst->dtype != src->dtype) {
        return fail(RLH_ERR_INVALID, "rlh_transpose_from: shape/dtype mismatch");
    }
    CtxLock lock(dst->ctx);
    HIP_TRY(launch_transpose(dst->p, src->p, src->rows, src->cols, src->dtype == RLH_F16, dst->ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_hadamard_product_inplace(rlh_tensor *dst, const rlh_tensor *src) {
    if (!dst || !src || !same_shape(dst, src)) return fail(RLH_ERR_INVALID, "rlh_hadamard_product_inplace: shape/dtype mismatch");
    CtxLock lock(dst->ctx);
    HIP_TRY(launch_hadamard(dst->p, src->p, dst->count(), dst->dtype == RLH_F16, dst->ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_silu_inplace(rlh_tensor *t) {
    if (!t) return fail(RLH_ERR_INVALID, "rlh_silu_inplace: NULL tensor");
    CtxLock lock(t->ctx);
    HIP_TRY(launch_silu(t->p, t->count(), t->dtype == RLH_F16, t->ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_gemv(rlh_tensor *y, const rlh_tensor *w, const rlh_tensor *x, int round_x, int round_y) {
    if (!y || !w || !x) return fail(RLH_ERR_INVALID, "rlh_gemv: NULL argument");
    if (x->dtype != RLH_F32 || y->dtype != RLH_F32) return fail(RLH_ERR_INVALID, "rlh_gemv: x and y must be f32");
    if (x->rows != 1 || y->rows != 1 || x->cols != w->cols || y->cols != w->rows) return fail(RLH_ERR_INVALID, "rlh_gemv: shape mismatch");
    const int vec = w->dtype == RLH_F16 ? 8 : 4;
    if (w->cols % vec != 0) return fail(RLH_ERR_UNSUPPORTED, "rlh_gemv: k must be a multiple of %d", vec);
    CtxLock lock(y->ctx);
    GemvParams p{};
    p.w = w->p;
    p.w_is_f16 = w->dtype == RLH_F16;
    p.x = (const float *)x->p;
    p.x_f16 = round_x ? 1 : 0;
    p.round_y = round_y ? 1 : 0;
    p.y = (float *)y->p;
    p.n_rows = w->rows;
    p.k = w->cols;
    p.stream_weights = 1;
    p.burst_fixed = y->ctx->tun.gemv_burst_fixed;
    HIP_TRY(launch_gemv(p, kEpiStore, y->ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_matrix_mul_inplace_transposed(rlh_tensor *dst, const rlh_tensor *src, const rlh_tensor *other) {
    if (!dst || !src || !other) return fail(RLH_ERR_INVALID, "rlh_matrix_mul_inplace_transposed: NULL argument");
    if (src->cols != other->cols) return fail(RLH_ERR_INVALID, "Invalid matrix multiplication %dx%d vs %dx%d", src->rows, src->cols, other->rows, other->cols);
    if (src->dtype != other->dtype || dst->dtype != src->dtype) return fail(RLH_ERR_INVALID, "Invalid matrix multiplication, different dtypes");
    if (dst->rows != src->rows) return fail(RLH_ERR_INVALID, "Invalid matrix multiplication, different number of rows");
    if (dst->cols != other->rows) return fail(RLH_ERR_INVALID, "Invalid matrix multiplication, different number of cols");
    const int f16 = src->dtype == RLH_F16;
    if (src->cols % (f16 ? 8 : 4) != 0) return fail(RLH_ERR_UNSUPPORTED, "rlh_matrix_mul_inplace_transposed: k must be a multiple of %d", f16 ? 8 : 4);
    CtxLock lock(dst->ctx);
    hipStream_t st = dst->ctx->stream;
    const int n = src->rows, k = src->cols, mrows = other->rows;
    if (n > 1 && (f16 || k % 32 == 0)) {
        // more than one row: the matrix-core GEMM (fp32 operands need whole K-tiles of 32, else the per-row path below)
        GemmParams g{};
        g.tune = dst->ctx->tun.gemm;
        g.a = (const _Float16 *)src->p;
        g.b = (const _Float16 *)other->p;
        g.c = dst->p;
        g.m = n;
        g.n = mrows;
        g.k = k;
        g.lda = k;
        g.ldb = k;
        g.ldc = mrows;
        g.batch = 1;
        g.f32_operands = f16 ? 0 : 1;
        if (!dst->ctx->ops.gemm_ws) HIP_TRY(hipMalloc(&dst->ctx->ops.gemm_ws, kOpGemmWsBytes));
        g.workspace = dst->ctx->ops.gemm_ws;
        g.workspace_bytes = kOpGemmWsBytes;
        HIP_TRY(launch_gemm_f16(g, f16 ? kGemmEpiF16 : kGemmEpiF32, st));
        return RLH_OK;
    }
    float *xf = nullptr, *yf = nullptr;
    HIP_TRY(hipMalloc((void **)&xf, sizeof(float) * (size_t)n * k));
    hipError_t e = hipMalloc((void **)&yf, sizeof(float) * (size_t)n * mrows);
    if (e == hipSuccess) e = launch_convert(xf, 0, src->p, f16, (uint64_t)n * k, st);
    for (int r = 0; e == hipSuccess && r < n; r++) {
        GemvParams p{};
        p.w = other->p;
        p.w_is_f16 = f16;
        p.x = xf + (size_t)r * k;
        p.x_f16 = f16;
        p.round_y = f16;
        p.y = yf + (size_t)r * mrows;
        p.n_rows = mrows;
        p.k = k;
        p.stream_weights = 0;
        e = launch_gemv(p, kEpiStore, st);
    }
    if (e == hipSuccess) e = launch_convert(dst->p, f16, yf, 0, (uint64_t)n * mrows, st);
    hipError_t e2 = hipStreamSynchronize(st);
    if (xf) (void)hipFree(xf);
    if (yf) (void)hipFree(yf);
    HIP_TRY(e);
    HIP_TRY(e2);
    return RLH_OK;
}

extern "C" int rlh_rmsnorm(rlh_tensor *y, const rlh_tensor *x, const rlh_tensor *w, double eps, int round_y) {
    if (!y || !x || !w) return fail(RLH_ERR_INVALID, "rlh_rmsnorm: NULL argument");
    if (x->dtype != RLH_F32 || y->dtype != RLH_F32 || w->dtype != RLH_F32) return fail(RLH_ERR_INVALID, "rlh_rmsnorm: f32 tensors only");
    if (!same_shape(x, y) || w->rows != 1 || w->cols != x->cols) return fail(RLH_ERR_INVALID, "rlh_rmsnorm: shape mismatch");
    CtxLock lock(y->ctx);
    HIP_TRY(launch_rmsnorm_rows((float *)y->p, (const float *)x->p, (const float *)w->p, x->rows, x->cols, (float)eps, round_y, y->ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_rope_inplace(rlh_tensor *x, int n_heads, int head_dim, int pos) {
    if (!x || x->dtype != RLH_F32 || n_heads <= 0 || head_dim <= 0 || (head_dim % 2) != 0 || pos < 0 || x->count() != (size_t)n_heads * head_dim) {
        return fail(RLH_ERR_INVALID, "rlh_rope_inplace: bad argument");
    }
    CtxLock lock(x->ctx);
    std::vector<float2> tab((size_t)head_dim / 2);
    for (int j = 0; j < head_dim / 2; j++) {
        const double freq = 1.0 / std::pow(10000.0, (double)j * 2.0 / (double)head_dim);
        const double ang = freq * (double)pos;
        tab[(size_t)j] = make_float2((float)std::cos(ang), (float)std::sin(ang));
    }
    float2 *dev = nullptr;
    HIP_TRY(hipMalloc((void **)&dev, tab.size() * sizeof(float2)));
    hipError_t e = hipMemcpyAsync(dev, tab.data(), tab.size() * sizeof(float2), hipMemcpyHostToDevice, x->ctx->stream);
    if (e == hipSuccess) e = launch_rope_row((float *)x->p, n_heads, head_dim, dev, x->ctx->stream);
    hipError_t e2 = hipStreamSynchronize(x->ctx->stream);
    (void)hipFree(dev);
    HIP_TRY(e);
    HIP_TRY(e2);
    return RLH_OK;
}


extern "C" int rlh_add(rlh_tensor *dst, const rlh_tensor *a, const rlh_tensor *b) {
    if (!dst || !a || !b || !same_shape(dst, a) || !same_shape(dst, b)) return fail(RLH_ERR_INVALID, "rlh_add: shape/dtype mismatch");
    if (dst->dtype != RLH_F32) return fail(RLH_ERR_UNSUPPORTED, "rlh_add: f32 tensors only (the residual stream is f32, transformer.rs:442)");
    CtxLock lock(dst->ctx);
    HIP_TRY(launch_add_f32((float *)dst->p, (const float *)a->p, (const float *)b->p, dst->count(), dst->ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_silu_mul(rlh_tensor *dst, const rlh_tensor *gate, const rlh_tensor *up) {
    if (!dst || !gate || !up || !same_shape(dst, gate) || !same_shape(dst, up)) return fail(RLH_ERR_INVALID, "rlh_silu_mul: shape/dtype mismatch");
    CtxLock lock(dst->ctx);
    if (dst->dtype == RLH_F16) HIP_TRY(launch_silu_mul_f16(gate->p, up->p, dst->p, dst->count(), dst->ctx->stream));
    else HIP_TRY(launch_silu_mul_f32((const float *)gate->p, (const float *)up->p, (float *)dst->p, dst->count(), dst->ctx->stream));
    return RLH_OK;
}

extern "C" int rlh_ffn_gate(rlh_tensor *dst, const rlh_tensor *x, const rlh_tensor *w1, const rlh_tensor *w3) {
    if (!dst || !x || !w1 || !w3) return fail(RLH_ERR_INVALID, "rlh_ffn_gate: NULL argument");
    if (dst->dtype != RLH_F16 || x->dtype != RLH_F16 || w1->dtype != RLH_F16 || w3->dtype != RLH_F16) return fail(RLH_ERR_UNSUPPORTED, "rlh_ffn_gate: f16 tensors only");
    if (!same_shape(w1, w3) || w1->cols != x->cols || dst->rows != x->rows || dst->cols != w1->rows) {
        return fail(RLH_ERR_INVALID, "rlh_ffn_gate: shapes do not fit (x %dx%d, w1 %dx%d, w3 %dx%d, dst %dx%d)", x->rows, x->cols, w1->rows, w1->cols, w3->rows, w3->cols,
                    dst->rows, dst->cols);
    }
    if (x->cols % 8 != 0) return fail(RLH_ERR_UNSUPPORTED, "rlh_ffn_gate: k must be a multiple of 8");
    CtxLock lock(dst->ctx);
    hipStream_t st = dst->ctx->stream;
    GemmParams g{};
    g.tune = dst->ctx->tun.gemm;
    g.a = (const _Float16 *)x->p;
    g.b = (const _Float16 *)w1->p;
    g.c = dst->p;
    g.m = x->rows;
    g.n = w1->rows;
    g.k = x->cols;
    g.lda = g.ldb = x->cols;
    g.ldc = w1->rows;
    g.batch = 1;
    if (!dst->ctx->ops.gemm_ws) HIP_TRY(hipMalloc(&dst->ctx->ops.gemm_ws, kOpGemmWsBytes));
    g.workspace = dst->ctx->ops.gemm_ws;
    g.workspace_bytes = kOpGemmWsBytes;
    GemmParams both = g;
    both.b2 = (const _Float16 *)w3->p;
    if (gemm_f16_dual_gate_supported(both)) { // both products in one pass over x
        HIP_TRY(launch_gemm_f16(both, kGemmEpiSiluGateF16, st));
        return RLH_OK;
    }
    // w1's product into dst, then w3's with dst as its gate: every element of the gate is read by the lane that overwrites it
    HIP_TRY(launch_gemm_f16(g, kGemmEpiF16, st));
    g.b = (const _Float16 *)w3->p;
    g.gate = (const _Float16 *)dst->p;
    HIP_TRY(launch_gemm_f16(g, kGemmEpiSiluGateF16, st));
    return RLH_OK;
}

// (cos, sin) of compute_freqs_cis (transformer.rs:858-885) for positions first .. first + n - 1, as f32 like :836-837
static std::vector<float2> rope_table(int head_dim, int first, int n) {
    std::vector<float2> tab((size_t)n * (head_dim / 2));
    for (int i = 0; i < n; i++) {
        for (int j = 0; j < head_dim / 2; j++) {
            const double freq = 1.0 / std::pow(10000.0, (double)j * 2.0 / (double)head_dim);
            const double ang = freq * (double)(first + i);
            tab[(size_t)i * (head_dim / 2) + j] = make_float2((float)std::cos(ang), (float)std::sin(ang));
        }
    }
    return tab;
}

// Checks one layer's pair of cache planes [n_heads * max_seq_len x head_dim] and returns head_dim (0 on a mismatch).
static int cache_planes_head_dim(const rlh_tensor *ck, const rlh_tensor *cv, int n_heads, int max_seq_len) {
    if (!ck || !cv || n_heads <= 0 || max_seq_len <= 0 || !same_shape(ck, cv)) return 0;
    if ((int64_t)ck->rows != (int64_t)n_heads * max_seq_len) return 0;
    const int hd = ck->cols;
    return (hd == 16 || hd == 32 || hd == 64 || hd == 128) ? hd : 0;
}

extern "C" int rlh_rope_kvwrite(rlh_tensor *q, const rlh_tensor *k, const rlh_tensor *v, rlh_tensor *cache_k, rlh_tensor *cache_v, int n_heads,
                                int max_seq_len, int pos) {
    const int hd = cache_planes_head_dim(cache_k, cache_v, n_heads, max_seq_len);
    if (!hd) return fail(RLH_ERR_INVALID, "rlh_rope_kvwrite: cache planes must be two [n_heads * max_seq_len x head_dim] tensors of one dtype, head_dim 16/32/64/128");
    if (!q || !k || !v || q->dtype != RLH_F32 || !same_shape(q, k) || !same_shape(q, v) || q->count() != (size_t)n_heads * hd) {
        return fail(RLH_ERR_INVALID, "rlh_rope_kvwrite: q, k, v must be f32 with n_heads * head_dim elements");
    }
    if (pos < 0 || pos >= max_seq_len) return fail(RLH_ERR_STATE, "rlh_rope_kvwrite: position %d outside the cache (max_seq_len %d)", pos, max_seq_len);
    CtxLock lock(q->ctx);
    hipStream_t st = q->ctx->stream;
    const std::vector<float2> tab = rope_table(hd, pos, 1);
    float2 *dev = nullptr;
    HIP_TRY(hipMalloc((void **)&dev, tab.size() * sizeof(float2)));
    hipError_t e = hipMemcpyAsync(dev, tab.data(), tab.size() * sizeof(float2), hipMemcpyHostToDevice, st);
    if (e == hipSuccess)
        e = launch_rope_kvwrite((float *)q->p, (const float *)k->p, (const float *)v->p, cache_k->p, cache_v->p, cache_k->dtype == RLH_F16, n_heads, hd,
                                max_seq_len, pos, dev, st);
    hipError_t e2 = hipStreamSynchronize(st);
    (void)hipFree(dev);
    HIP_TRY(e);
    HIP_TRY(e2);
    return RLH_OK;
}

namespace rlh {
int attn_splits_rule(int T, int n_heads, int compute_units, int single_max, int chunk, int max_splits) {
    // One workgroup per (head, split).  Short sequences stay in one workgroup per head; longer ones are cut so that the part
    // holds about one workgroup per compute unit, in pieces of at least 128 positions (chunk == -1, the default), or into
    // pieces of about `chunk` positions (chunk > 0; chunk == 0: 128).  Measured at 2112 positions of the 13B shape (40 heads):
    // 6 pieces of 352 positions 13.0 - 14.0 us, 17 of 128 14.1 - 14.5 us -- every piece ends at about the same time, and the
    // workgroup that merges loads 6 partial results instead of 17; the 7B shape (32 heads) gets the same pieces up to 1024
    // positions and 8 of 256 instead of 16 of 128 at 2048 (12.25 against 12.35 us).
    constexpr int kAutoChunk = 128;
    if (T <= single_max) return 1;
    int S;
    if (chunk == -1) {
        const int per_head = compute_units / (n_heads > 0 ? n_heads : 1);
        S = (T + 127) / 128;
        if (S > per_head) S = per_head;
    } else {
        const int c = chunk > 0 ? chunk : kAutoChunk;
        S = (T + c - 1) / c;
    }
    if (S < 1) S = 1;
    if (S > max_splits) S = max_splits;
    return S;
}
} // namespace rlh

static int ensure_op_scratch(rlh_ctx *ctx, size_t attn_ws_floats) {
    OpScratch &o = ctx->ops;
    if (!o.state) {
        HIP_TRY(hipMalloc((void **)&o.state, sizeof(DecodeState)));
        HIP_TRY(hipMemset(o.state, 0, sizeof(DecodeState)));
    }
    if (!o.token) HIP_TRY(hipMalloc((void **)&o.token, sizeof(int32_t)));
    if (!o.tickets) {
        HIP_TRY(hipMalloc((void **)&o.tickets, sizeof(unsigned) * kOpMaxHeads));
        HIP_TRY(hipMemset(o.tickets, 0, sizeof(unsigned) * kOpMaxHeads));
    }
    if (attn_ws_floats > o.attn_ws_floats) {
        if (o.attn_ws) {
            HIP_TRY(hipStreamSynchronize(ctx->stream));
            (void)hipFree(o.attn_ws);
            o.attn_ws = nullptr;
            o.attn_ws_floats = 0;
        }
        HIP_TRY(hipMalloc((void **)&o.attn_ws, attn_ws_floats * sizeof(float)));
        o.attn_ws_floats = attn_ws_floats;
    }
    return RLH_OK;
}

namespace rlh {
void ops_release(rlh_ctx *ctx) {
    OpScratch &o = ctx->ops;
    void *all[] = {o.state, o.attn_ws, o.tickets, o.token, o.gemm_ws};
    for (void *b : all)
        if (b) (void)hipFree(b);
    o = OpScratch();
}
} // namespace rlh

// Argument checks of rlh_attn_decode; fills in head_dim and the number of splits.
static int check_attn_decode(const char *who, const rlh_tensor *out, const rlh_tensor *q, const rlh_tensor *ck, const rlh_tensor *cv, int n_heads,
                             int max_seq_len, int T, int *n_splits, int *head_dim) {
    const int hd = cache_planes_head_dim(ck, cv, n_heads, max_seq_len);
    if (!hd) return fail(RLH_ERR_INVALID, "%s: cache planes must be two [n_heads * max_seq_len x head_dim] tensors of one dtype, head_dim 16/32/64/128", who);
    if (!out || !q || q->dtype != RLH_F32 || out->dtype != RLH_F32 || q->count() != (size_t)n_heads * hd || out->count() != (size_t)n_heads * hd) {
        return fail(RLH_ERR_INVALID, "%s: q and out must be f32 with n_heads * head_dim elements", who);
    }
    if (T < 1 || T > max_seq_len) return fail(RLH_ERR_STATE, "%s: sequence length %d outside 1..max_seq_len %d", who, T, max_seq_len);
    if (n_heads > kOpMaxHeads) return fail(RLH_ERR_UNSUPPORTED, "%s: more than %d heads", who, kOpMaxHeads);
    if (*n_splits == 0) {
        const Tunables &t = out->ctx->tun;
        *n_splits = attn_splits_rule(T, n_heads, out->ctx->prop.multiProcessorCount, t.attn_single_max, t.attn_chunk, kAttnDecodeMaxSplits);
    }
    if (*n_splits < 1 || *n_splits > kAttnDecodeMaxSplits) return fail(RLH_ERR_INVALID, "%s: n_splits %d outside 1..%d", who, *n_splits, kAttnDecodeMaxSplits);
    *head_dim = hd;
    return RLH_OK;
}

static hipError_t enqueue_attn_decode(rlh_ctx *ctx, rlh_tensor *out, const rlh_tensor *q, const rlh_tensor *ck, const rlh_tensor *cv, int n_heads, int hd,
                                      int max_seq_len, int T, int n_splits, int round_out, DecodeState *state, float *ws, unsigned *tickets) {
    hipStream_t st = ctx->stream;
    hipError_t e = launch_set_state(state, T - 1, 0, 1, st);
    if (e != hipSuccess) return e;
    // the counters must start at zero whatever an earlier call left behind (a fill kernel, so that callers may capture this)
    e = launch_fill_u32(tickets, (uint64_t)n_heads, 0u, st);
    if (e != hipSuccess) return e;
    AttnDecodeParams a{};
    a.q = (const float *)q->p;
    a.cache_k = ck->p;
    a.cache_v = cv->p;
    a.cache_f16 = ck->dtype == RLH_F16;
    a.state = state;
    a.pos_host = T - 1;
    a.n_heads = n_heads;
    a.head_dim = hd;
    a.max_seq_len = max_seq_len;
    a.n_splits = n_splits;
    a.out = (float *)out->p;
    a.round_out = round_out ? 1 : 0;
    a.workspace = ws;
    a.tickets = tickets;
    a.merge_mode = ctx->tun.attn_merge_mode;
    a.chunk_hint = (((T + n_splits - 1) / n_splits) + 15) & ~15;
    return launch_attn_decode(a, st);
}

extern "C" int rlh_attn_decode(rlh_tensor *out, const rlh_tensor *q, const rlh_tensor *cache_k, const rlh_tensor *cache_v, int n_heads, int max_seq_len,
                               int T, int n_splits, int round_out) {
    int hd = 0;
    int rc = check_attn_decode("rlh_attn_decode", out, q, cache_k, cache_v, n_heads, max_seq_len, T, &n_splits, &hd);
    if (rc != RLH_OK) return rc;
    rlh_ctx *ctx = out->ctx;
    CtxLock lock(ctx);
    rc = ensure_op_scratch(ctx, attn_decode_workspace_floats(n_heads, hd, n_splits));
    if (rc != RLH_OK) return rc;
    HIP_TRY(enqueue_attn_decode(ctx, out, q, cache_k, cache_v, n_heads, hd, max_seq_len, T, n_splits, round_out, ctx->ops.state, ctx->ops.attn_ws,
                                ctx->ops.tickets));
    return RLH_OK;
}

extern "C" int rlh_attn_prefill(rlh_tensor *out, const rlh_tensor *qkv, rlh_tensor *cache_k, rlh_tensor *cache_v, int n_heads, int max_seq_len) {
    const int hd = cache_planes_head_dim(cache_k, cache_v, n_heads, max_seq_len);
    if (!hd || cache_k->dtype != RLH_F16) return fail(RLH_ERR_INVALID, "rlh_attn_prefill: cache planes must be two f16 [n_heads * max_seq_len x head_dim] tensors");
    if (!attn_prefill_supported(hd)) return fail(RLH_ERR_UNSUPPORTED, "rlh_attn_prefill: head_dim %d (the one-kernel form takes 64 and 128)", hd);
    const int d = n_heads * hd;
    if (!out || !qkv || out->dtype != RLH_F16 || qkv->dtype != RLH_F16 || qkv->cols != 3 * d || out->cols != d || out->rows != qkv->rows) {
        return fail(RLH_ERR_INVALID, "rlh_attn_prefill: qkv must be f16 [n x 3 dim] and out f16 [n x dim]");
    }
    const int n = qkv->rows;
    if (n > max_seq_len) return fail(RLH_ERR_STATE, "rlh_attn_prefill: %d rows exceed max_seq_len %d", n, max_seq_len);
    rlh_ctx *ctx = out->ctx;
    CtxLock lock(ctx);
    hipStream_t st = ctx->stream;
    const int tp = (n + 127) & ~127;
    const std::vector<float2> tab = rope_table(hd, 0, n);
    float2 *freqs = nullptr;
    void *q2 = nullptr, *v_t = nullptr;
    const size_t q2_bytes = (size_t)n * d * 2 * 2, vt_bytes = (size_t)n_heads * hd * tp * 2;
    hipError_t e = hipMalloc((void **)&freqs, tab.size() * sizeof(float2));
    if (e == hipSuccess) e = hipMalloc(&q2, q2_bytes);
    if (e == hipSuccess) e = hipMalloc(&v_t, vt_bytes);
    if (e == hipSuccess) e = hipMemsetAsync(v_t, 0, vt_bytes, st); // the padding past n must hold finite values
    if (e == hipSuccess) e = hipMemcpyAsync(freqs, tab.data(), tab.size() * sizeof(float2), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) {
        PrefillRopeParams rp{};
        rp.qkv = qkv->p;
        rp.freqs = freqs;
        rp.q_hi = q2;
        rp.q_lo = (char *)q2 + (size_t)hd * 2;
        rp.q_stride = 2 * hd;
        rp.cache_k = cache_k->p;
        rp.cache_v = cache_v->p;
        rp.cache_f16 = 1;
        rp.v_t = v_t;
        rp.n = n;
        rp.dim = d;
        rp.head_dim = hd;
        rp.max_seq_len = max_seq_len;
        rp.t_pad = tp;
        rp.vt_swap = 1;
        e = launch_rope_kv_prefill(rp, st);
    }
    if (e == hipSuccess) {
        AttnPrefillParams ap{};
        ap.q2 = q2;
        ap.cache_k = cache_k->p;
        ap.v_t = v_t;
        ap.out = out->p;
        ap.n = n;
        ap.n_heads = n_heads;
        ap.head_dim = hd;
        ap.dim = d;
        ap.max_seq_len = max_seq_len;
        ap.t_pad = tp;
        ap.scale = 1.0f / sqrtf((float)hd);
        ap.order = ctx->tun.prefill_attn_order;
        e = launch_attn_prefill(ap, st);
    }
    hipError_t e2 = hipStreamSynchronize(st);
    for (void *b : {(void *)freqs, q2, v_t})
        if (b) (void)hipFree(b);
    HIP_TRY(e);
    HIP_TRY(e2);
    return RLH_OK;
}

extern "C" int rlh_argmax_greedy(const rlh_tensor *logits, float temperature, int32_t *token) {
    if (!logits || !token || logits->dtype != RLH_F32 || (logits->rows != 1 && logits->cols != 1)) {
        return fail(RLH_ERR_INVALID, "rlh_argmax_greedy: logits must be an f32 vector");
    }
    rlh_ctx *ctx = logits->ctx;
    CtxLock lock(ctx);
    int rc = ensure_op_scratch(ctx, 0);
    if (rc != RLH_OK) return rc;
    hipStream_t st = ctx->stream;
    HIP_TRY(launch_set_state(ctx->ops.state, 0, 0, 1, st));
    HIP_TRY(launch_argmax_advance((const float *)logits->p, (int)logits->count(), ctx->ops.state, ctx->ops.token, 1, st,
                                  temperature > 0.0f ? 1.0f / temperature : 1.0f));
    HIP_TRY(hipMemcpyAsync(token, ctx->ops.token, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    HIP_TRY(hipStreamSynchronize(st));
    return RLH_OK;
}

// ------------------------------------------------------------------------------------------------
// rlh_attn_decode without any allocation: the work memory is a static device array
// ------------------------------------------------------------------------------------------------
// Layout of the array: arrival counters [kOpMaxHeads], the position word block, then the partial triples.
constexpr size_t kStaticTicketsBytes = sizeof(unsigned) * kOpMaxHeads;
constexpr size_t kStaticStateOffset = kStaticTicketsBytes;
constexpr size_t kStaticWsOffset = kStaticStateOffset + 256;
constexpr size_t kStaticWsFloats = (size_t)1 << 20; // 4 MiB of partial triples: n_heads * n_splits * (head_dim + 2) floats at most
constexpr size_t kStaticScratchBytes = kStaticWsOffset + kStaticWsFloats * sizeof(float);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace rlh {
// The array's name is only a host-side stand-in; every device holds its own copy at its own address.  This looks the
// address up for the context's device (current when rlh_init calls this) and keeps it in the context.
int noalloc_setup(rlh_ctx *ctx) {
    void *ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
        return fail(RLH_ERR_HIP, "rlh_init: hipGetSymbolAddress(scratch) on device %d: %s", ctx->device, hipGetErrorString(e));
    }
    ctx->noalloc_scratch = ptr;
    return RLH_OK;
}
} // namespace rlh

extern "C" int rlh_attn_decode_noalloc(rlh_tensor *out, const rlh_tensor *q, const rlh_tensor *cache_k, const rlh_tensor *cache_v, int n_heads,
                                       int max_seq_len, int T, int n_splits, int round_out) {
    int hd = 0;
    int rc = check_attn_decode("rlh_attn_decode_noalloc", out, q, cache_k, cache_v, n_heads, max_seq_len, T, &n_splits, &hd);
    if (rc != RLH_OK) return rc;
    const size_t need = attn_decode_workspace_floats(n_heads, hd, n_splits);
    if (need > kStaticWsFloats) {
        return fail(RLH_ERR_UNSUPPORTED,
                    "rlh_attn_decode_noalloc: %d heads x %d splits x (%d + 2) floats = %zu exceed the static work memory of %zu floats; use fewer "
                    "splits or rlh_attn_decode",
                    n_heads, n_splits, hd, need, kStaticWsFloats);
    }
    rlh_ctx *ctx = out->ctx;
    CtxLock lock(ctx);
    unsigned char *base = static_cast<unsigned char *>(ctx->noalloc_scratch); // this device's address of `scratch`, from rlh_init
    if (!base) return fail(RLH_ERR_STATE, "rlh_attn_decode_noalloc: the context holds no address of the static work memory");
    HIP_TRY(enqueue_attn_decode(ctx, out, q, cache_k, cache_v, n_heads, hd, max_seq_len, T, n_splits, round_out,
                                reinterpret_cast<DecodeState *>(base + kStaticStateOffset), reinterpret_cast<float *>(base + kStaticWsOffset),
                                reinterpret_cast<unsigned *>(base)));
    return RLH_OK;
}
