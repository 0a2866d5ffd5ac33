// prefill.hip -- the element-wise kernels around the matrix-core GEMMs of a multi-token forward at
// start_pos == 0 (the only multi-token call the reference supports: its mask is n x n, transformer.rs:350-357).
//
// Rounding points are the reference's (Noeda/rllama): RMSNorm output -> f16 (transformer.rs:665-668, 537-540),
// projection outputs -> f16 (tensor.rs:1623-1643), K and V -> f16 on cache write (transformer.rs:754-761),
// attention output -> f16 (transformer.rs:793-796), SiLU*gate -> f16 (transformer.rs:563-565).  The reference
// keeps q (after RoPE) and the softmax probabilities in fp32; to feed them to the f16 matrix cores without
// losing that, each is split into a high and a low f16 part (v = hi + lo to about 2^-22 relative) and the
// product is accumulated over both parts.
#include "kernels.h"
#include "device_utils.h"

namespace rlh {

// X[r, :] = table[tokens[r], :] widened to f32 (embedding.rs:50-52, transformer.rs:361-367)
template <typename ET>
__global__ void embed_rows_kernel(const ET *table, const int32_t *tokens, int dim, float *x) {
    const int r = blockIdx.x;
    const size_t tok = (size_t)tokens[r];
    for (int i = threadIdx.x; i < dim; i += blockDim.x) x[(size_t)r * dim + i] = (float)table[tok * dim + i];
}

hipError_t launch_embed_rows(const void *table, int table_f16, const int32_t *tokens_dev, int n, int dim, float *x, hipStream_t s) {
    if (table_f16) hipLaunchKernelGGL(embed_rows_kernel<half_t>, dim3(n), dim3(256), 0, s, (const half_t *)table, tokens_dev, dim, x);
    else hipLaunchKernelGGL(embed_rows_kernel<float>, dim3(n), dim3(256), 0, s, (const float *)table, tokens_dev, dim, x);
    return hipGetLastError();
}

// RMSNorm::forward per row (transformer.rs:476-480), output rounded to f16 for the projections that follow.
// One workgroup per row; rows of up to 256 x 4 x kNormVecs floats are read once (16-byte loads, kept in registers).
constexpr int kNormVecs = 8;
__global__ __launch_bounds__(256) void rmsnorm_rows_f16_kernel(half_t *y, const float *x, const float *w, int d, float eps) {
    __shared__ float red[16];
    const float *xr = x + (size_t)blockIdx.x * d;
    half_t *yr = y + (size_t)blockIdx.x * d;
    const int tid = threadIdx.x;
    if ((d & 3) == 0 && d <= 256 * 4 * kNormVecs) {
        const int n4 = d / 4;
        const float4_t *x4 = reinterpret_cast<const float4_t *>(xr);
        const float4_t *w4 = reinterpret_cast<const float4_t *>(w);
        float4_t xv[kNormVecs];
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < kNormVecs; j++) {
            const int i = tid + j * 256;
            xv[j] = i < n4 ? x4[i] : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int e = 0; e < 4; e++) ss = fmaf(xv[j][e], xv[j][e], ss);
        }
        float4_t wn[kNormVecs]; // requested before the row sum, not after it
#pragma unroll
        for (int j = 0; j < kNormVecs; j++) {
            const int i = tid + j * 256;
            wn[j] = i < n4 ? w4[i] : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
        ss = block_sum(ss, red);
        const float rs = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
        for (int j = 0; j < kNormVecs; j++) {
            const int i = tid + j * 256;
            if (i < n4) {
                const float4_t wv = wn[j];
                typedef __attribute__((ext_vector_type(4))) _Float16 half4_t;
                half4_t o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = to_f16((xv[j][e] * rs) * wv[e]);
                *reinterpret_cast<half4_t *>(yr + i * 4) = o;
            }
        }
        return;
    }
    float ss = 0.0f;
    for (int i = tid; i < d; i += blockDim.x) ss = fmaf(xr[i], xr[i], ss);
    ss = block_sum(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)d + eps);
    for (int i = tid; i < d; i += blockDim.x) yr[i] = to_f16((xr[i] * rs) * w[i]);
}

hipError_t launch_rmsnorm_rows_f16(void *y, const float *x, const float *w, int rows, int d, float eps, hipStream_t s) {
    hipLaunchKernelGGL(rmsnorm_rows_f16_kernel, dim3(rows), dim3(256), 0, s, (half_t *)y, x, w, d, eps);
    return hipGetLastError();
}

// qkv [n x 3 dim] f16 (rows = tokens at positions 0..n-1) ->
//   q after RoPE, split hi/lo, head-major [head][n] rows of head_dim, q_stride halves apart
//   K (after RoPE) and V into the cache [head][max_seq_len][head_dim] at positions 0..n-1
//   V transposed [head][head_dim][t_pad] (positions contiguous) as the B operand of P.V
__global__ void rope_kv_prefill_kernel(PrefillRopeParams p) {
    const int half_hd = p.head_dim / 2;
    const int pairs_per_row = p.dim / 2;
    const size_t total = (size_t)p.n * pairs_per_row;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const half_t *qkv = reinterpret_cast<const half_t *>(p.qkv);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int r = (int)(i / pairs_per_row);              // token row = position
        const int pr = (int)(i - (size_t)r * pairs_per_row); // pair within the row
        const int head = pr / half_hd, c = pr - head * half_hd;
        const int j = head * p.head_dim + 2 * c;
        const float2 f = p.freqs[(size_t)r * half_hd + c];
        const half_t *row = qkv + (size_t)r * 3 * p.dim;
        // q
        float a, b;
        rope_pair((float)row[j], (float)row[j + 1], f, a, b);
        const size_t qo = ((size_t)head * p.n + r) * p.q_stride + 2 * c;
        half_t *qhi = reinterpret_cast<half_t *>(p.q_hi), *qlo = reinterpret_cast<half_t *>(p.q_lo);
        const half_t ah = (half_t)a, bh = (half_t)b;
        qhi[qo] = ah;
        qhi[qo + 1] = bh;
        qlo[qo] = (half_t)(a - (float)ah);
        qlo[qo + 1] = (half_t)(b - (float)bh);
        // k
        rope_pair((float)row[p.dim + j], (float)row[p.dim + j + 1], f, a, b);
        const size_t co = ((size_t)head * p.max_seq_len + r) * p.head_dim + 2 * c;
        const float v0 = (float)row[2 * p.dim + j], v1 = (float)row[2 * p.dim + j + 1];
        if (p.cache_f16) {
            half_t *ck = reinterpret_cast<half_t *>(p.cache_k), *cv = reinterpret_cast<half_t *>(p.cache_v);
            ck[co] = (half_t)a; // Tensor::set_f32 on an f16 cache (tensor.rs:373-376)
            ck[co + 1] = (half_t)b;
            cv[co] = (half_t)v0;
            cv[co + 1] = (half_t)v1;
        } else {
            float *ck = reinterpret_cast<float *>(p.cache_k), *cv = reinterpret_cast<float *>(p.cache_v);
            ck[co] = a;
            ck[co + 1] = b;
            cv[co] = v0;
            cv[co + 1] = v1;
        }
        half_t *vt = reinterpret_cast<half_t *>(p.v_t);
        vt[((size_t)head * p.head_dim + 2 * c) * p.t_pad + r] = (half_t)v0;
        vt[((size_t)head * p.head_dim + 2 * c + 1) * p.t_pad + r] = (half_t)v1;
    }
}

// The same for f16 caches, tiled: a workgroup takes 64 positions of one head, moves everything in 16-byte pieces (8 dims = 4
// RoPE pairs of one row per thread and step) and transposes V through LDS so that V^T is written in 128-byte rows too.
constexpr int kRopeTileRows = 64;
__global__ __launch_bounds__(256) void rope_kv_prefill_tiled_kernel(PrefillRopeParams p) {
    typedef __attribute__((ext_vector_type(8))) _Float16 h8;
    constexpr int kPad = kRopeTileRows + 8; // halves per LDS row of the transposed V tile
    __shared__ __attribute__((aligned(16))) half_t vt_tile[128 * kPad];
    const int hd = p.head_dim, half_hd = hd / 2;
    const int head = blockIdx.y, r0 = blockIdx.x * kRopeTileRows;
    const int chunks = hd / 8; // 16-byte pieces per row
    const half_t *qkv = reinterpret_cast<const half_t *>(p.qkv);
    half_t *qhi = reinterpret_cast<half_t *>(p.q_hi), *qlo = reinterpret_cast<half_t *>(p.q_lo);
    half_t *ck = reinterpret_cast<half_t *>(p.cache_k), *cv = reinterpret_cast<half_t *>(p.cache_v);
    for (int c = threadIdx.x; c < kRopeTileRows * chunks; c += blockDim.x) {
        const int rr = c / chunks, ch = c - rr * chunks;
        const int r = r0 + rr;
        const int j = head * hd + ch * 8; // first of this piece's 8 dims within the row of q / k / v
        // position of this row in the transposed V tile
        const int rs = p.vt_swap ? (rr & ~12) | ((rr & 4) << 1) | ((rr & 8) >> 1) : rr;
        h8 v8 = {0, 0, 0, 0, 0, 0, 0, 0};
        if (r < p.n) {
            const half_t *row = qkv + (size_t)r * 3 * p.dim;
            const h8 q8 = *reinterpret_cast<const h8 *>(row + j);
            const h8 k8 = *reinterpret_cast<const h8 *>(row + p.dim + j);
            v8 = *reinterpret_cast<const h8 *>(row + 2 * p.dim + j);
            const float2 *fr = p.freqs + (size_t)r * half_hd + ch * 4;
            h8 qh, ql, kk;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float2 f = fr[e];
                float a, b;
                rope_pair((float)q8[2 * e], (float)q8[2 * e + 1], f, a, b);
                const half_t ah = (half_t)a, bh = (half_t)b;
                qh[2 * e] = ah;
                qh[2 * e + 1] = bh;
                ql[2 * e] = (half_t)(a - (float)ah);
                ql[2 * e + 1] = (half_t)(b - (float)bh);
                rope_pair((float)k8[2 * e], (float)k8[2 * e + 1], f, a, b);
                kk[2 * e] = (half_t)a; // Tensor::set_f32 on an f16 cache (tensor.rs:373-376)
                kk[2 * e + 1] = (half_t)b;
            }
            const size_t qo = ((size_t)head * p.n + r) * p.q_stride + ch * 8;
            *reinterpret_cast<h8 *>(qhi + qo) = qh;
            *reinterpret_cast<h8 *>(qlo + qo) = ql;
            const size_t co = ((size_t)head * p.max_seq_len + r) * hd + ch * 8;
            *reinterpret_cast<h8 *>(ck + co) = kk;
            *reinterpret_cast<h8 *>(cv + co) = v8;
        }
#pragma unroll
        for (int e = 0; e < 8; e++) vt_tile[(ch * 8 + e) * kPad + rs] = v8[e]; // zeros for positions past n: finite padding
    }
    __syncthreads();
    half_t *vt = reinterpret_cast<half_t *>(p.v_t) + (size_t)head * hd * p.t_pad + r0;
    for (int c = threadIdx.x; c < hd * (kRopeTileRows / 8); c += blockDim.x) {
        const int jrow = c / (kRopeTileRows / 8), ch = c - jrow * (kRopeTileRows / 8);
        *reinterpret_cast<h8 *>(vt + (size_t)jrow * p.t_pad + ch * 8) = *reinterpret_cast<const h8 *>(&vt_tile[jrow * kPad + ch * 8]);
    }
}

hipError_t launch_rope_kv_prefill(const PrefillRopeParams &p, hipStream_t s) {
    if (p.cache_f16 && p.head_dim % 8 == 0 && p.head_dim <= 128 && p.t_pad % kRopeTileRows == 0 && p.q_stride % 8 == 0 && p.dim % 8 == 0) {
        const int n_heads = p.dim / p.head_dim;
        hipLaunchKernelGGL(rope_kv_prefill_tiled_kernel, dim3((p.n + kRopeTileRows - 1) / kRopeTileRows, n_heads), dim3(256), 0, s, p);
        return hipGetLastError();
    }
    if (p.vt_swap) return hipErrorInvalidValue; // only the tiled kernel writes the swapped order
    const size_t total = (size_t)p.n * (p.dim / 2);
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    hipLaunchKernelGGL(rope_kv_prefill_kernel, dim3(blocks), dim3(256), 0, s, p);
    return hipGetLastError();
}

// Scores [head][n][t_pad] f32 (raw q.k) -> causal softmax probabilities split hi/lo f16, rows p_stride halves apart.
// scalar_multiply_f32(1/sqrt(hd)), + full_triu mask, softmax (transformer.rs:768-779; tensor.rs:496-508, 479-494);
// evaluated with the row maximum subtracted, which is the same function wherever the reference's is finite.
// One wavefront per row.  Masked columns get probability 0 up to the next multiple of 256 columns (what a
// causal P.V product with row tiles of at most 256 reads); columns past that are left as they are.
constexpr int kSoftmaxRegs = 32; // scores a lane keeps in registers: rows up to 64 * 32 columns are read once
__global__ __launch_bounds__(256) void causal_softmax_kernel(const float *scores, half_t *p_hi, half_t *p_lo, size_t total_rows, int n, int t_pad,
                                                             int p_stride, float scale) {
    const int lane = threadIdx.x & 63;
    const size_t row_id = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6); // over heads * n
    if (row_id >= total_rows) return;                                  // whole wavefronts leave together
    const int r = (int)(row_id % (size_t)n);                           // row r attends to columns 0..r
    const float *srow = scores + row_id * t_pad;
    half_t *hi = p_hi + row_id * p_stride;
    half_t *lo = p_lo + row_id * p_stride;
    const int c_end = min(t_pad, (r + 256) & ~255);
    auto put = [&](int c, float pv) {
        const half_t h = (half_t)pv;
        hi[c] = h;
        lo[c] = (half_t)(pv - (float)h);
    };
    if (r < 64 * kSoftmaxRegs) {
        float v[kSoftmaxRegs];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < kSoftmaxRegs; i++) {
            const int c = lane + 64 * i;
            v[i] = c <= r ? srow[c] * scale : -INFINITY;
            mx = fmaxf(mx, v[i]);
        }
        mx = wave_max(mx);
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < kSoftmaxRegs; i++) {
            v[i] = expf(v[i] - mx); // masked columns: exp(-inf) = 0
            sum += v[i];
        }
        sum = wave_sum(sum);
#pragma unroll
        for (int i = 0; i < kSoftmaxRegs; i++) {
            const int c = lane + 64 * i;
            if (c < c_end) put(c, v[i] / sum);
        }
        return;
    }
    float mx = -INFINITY;
    for (int c = lane; c <= r; c += 64) mx = fmaxf(mx, srow[c] * scale);
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int c = lane; c <= r; c += 64) sum += expf(srow[c] * scale - mx);
    sum = wave_sum(sum);
    for (int c = lane; c < c_end; c += 64) put(c, c <= r ? expf(srow[c] * scale - mx) / sum : 0.0f);
}

hipError_t launch_causal_softmax(const float *scores, void *p_hi, void *p_lo, int n_heads, int n, int t_pad, int p_stride, int head_dim, hipStream_t s) {
    const size_t rows = (size_t)n_heads * n;
    hipLaunchKernelGGL(causal_softmax_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, scores, (half_t *)p_hi, (half_t *)p_lo, rows, n, t_pad,
                       p_stride, 1.0f / sqrtf((float)head_dim)); // transformer.rs:770
    return hipGetLastError();
}

} // namespace rlh
