// prefill_f32.hip -- the element-wise kernels around the fp32 matrix-core GEMMs of a multi-token forward at
// start_pos == 0 in f32 mode (no --f16: fp32 weights, activations and KV cache; Noeda/rllama transformer.rs:343-383 with
// seq_len > 1).  There is no rounding point in this mode: every kernel here reads and writes fp32.
#include "kernels.h"
#include "device_utils.h"

namespace rlh {

// RMSNorm::forward per row (transformer.rs:476-480).  One workgroup per row.
__global__ __launch_bounds__(256) void rmsnorm_rows_f32_kernel(float *y, const float *x, const float *w, int d, float eps) {
    __shared__ float red[16];
    const float *xr = x + (size_t)blockIdx.x * d;
    float *yr = y + (size_t)blockIdx.x * d;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) ss = fmaf(xr[i], xr[i], ss);
    ss = block_sum(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += blockDim.x) yr[i] = (xr[i] * rs) * w[i];
}

hipError_t launch_rmsnorm_rows_f32(float *y, const float *x, const float *w, int rows, int d, float eps, hipStream_t s) {
    hipLaunchKernelGGL(rmsnorm_rows_f32_kernel, dim3(rows), dim3(256), 0, s, y, x, w, d, eps);
    return hipGetLastError();
}

// qkv [n x 3 dim] fp32 (rows = tokens at positions 0..n-1) ->
//   q after RoPE (transformer.rs:823-856), head-major [head][n][head_dim]
//   K (after RoPE) and V into the fp32 cache [head][max_seq_len][head_dim] at positions 0..n-1 (transformer.rs:751-761)
//   V transposed [head][head_dim][t_pad] (the B operand of P.V), zeros at positions n .. t_pad - 1
// One workgroup per (64 positions, head); V^T goes through LDS so that both sides move whole 16-byte pieces.
constexpr int kRopeF32Rows = 64;
__global__ __launch_bounds__(256) void rope_kv_prefill_f32_kernel(PrefillRopeF32Params p) {
    constexpr int kPad = kRopeF32Rows + 4; // floats per LDS row of the transposed V tile
    __shared__ __attribute__((aligned(16))) float vt_tile[128 * kPad];
    const int hd = p.head_dim, half_hd = hd / 2;
    const int head = blockIdx.y, r0 = blockIdx.x * kRopeF32Rows;
    const int chunks = hd / 4; // 16-byte pieces per row
    for (int c = threadIdx.x; c < kRopeF32Rows * chunks; c += blockDim.x) {
        const int rr = c / chunks, ch = c - rr * chunks;
        const int r = r0 + rr;
        const int j = head * hd + ch * 4; // first of this piece's 4 dims within the row of q / k / v
        float4_t v4 = {0.0f, 0.0f, 0.0f, 0.0f};
        if (r < p.n) {
            const float *row = p.qkv + (size_t)r * 3 * p.dim;
            const float4_t q4 = *reinterpret_cast<const float4_t *>(row + j);
            const float4_t k4 = *reinterpret_cast<const float4_t *>(row + p.dim + j);
            v4 = *reinterpret_cast<const float4_t *>(row + 2 * p.dim + j);
            const float2 *fr = p.freqs + (size_t)r * half_hd + ch * 2;
            float4_t qo, ko;
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const float2 f = fr[e];
                float a, b;
                rope_pair(q4[2 * e], q4[2 * e + 1], f, a, b);
                qo[2 * e] = a;
                qo[2 * e + 1] = b;
                rope_pair(k4[2 * e], k4[2 * e + 1], f, a, b);
                ko[2 * e] = a;
                ko[2 * e + 1] = b;
            }
            *reinterpret_cast<float4_t *>(p.q + ((size_t)head * p.n + r) * hd + ch * 4) = qo;
            const size_t co = ((size_t)head * p.max_seq_len + r) * hd + ch * 4;
            *reinterpret_cast<float4_t *>(p.cache_k + co) = ko;
            *reinterpret_cast<float4_t *>(p.cache_v + co) = v4;
        }
#pragma unroll
        for (int e = 0; e < 4; e++) vt_tile[(ch * 4 + e) * kPad + rr] = v4[e]; // zeros for positions past n: finite padding
    }
    __syncthreads();
    float *vt = p.v_t + (size_t)head * hd * p.t_pad + r0;
    for (int c = threadIdx.x; c < hd * (kRopeF32Rows / 4); c += blockDim.x) {
        const int jrow = c / (kRopeF32Rows / 4), ch = c - jrow * (kRopeF32Rows / 4);
        *reinterpret_cast<float4_t *>(vt + (size_t)jrow * p.t_pad + ch * 4) = *reinterpret_cast<const float4_t *>(&vt_tile[jrow * kPad + ch * 4]);
    }
}

hipError_t launch_rope_kv_prefill_f32(const PrefillRopeF32Params &p, hipStream_t s) {
    if (p.head_dim % 4 != 0 || p.head_dim > 128 || p.t_pad % kRopeF32Rows != 0 || p.dim % 4 != 0 || p.n < 1) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rope_kv_prefill_f32_kernel, dim3((p.n + kRopeF32Rows - 1) / kRopeF32Rows, p.dim / p.head_dim), dim3(256), 0, s, p);
    return hipGetLastError();
}

// Scores [head][n][t_pad] fp32 (raw q.k) -> causal softmax probabilities, in place.
// scalar_multiply_f32(1/sqrt(hd)), + full_triu mask, softmax (transformer.rs:768-779; tensor.rs:496-508, 479-494);
// evaluated with the row maximum subtracted, which is the same function wherever the reference's is finite.
// One wavefront per row.  Masked columns get probability 0 up to the next multiple of 256 columns (what a causal P.V
// product with row tiles of at most 256 reads); columns past that are left as they are.
__global__ __launch_bounds__(256) void causal_softmax_f32_kernel(float *scores, size_t total_rows, int n, int t_pad, float scale) {
    const int lane = threadIdx.x & 63;
    const size_t row_id = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6); // over heads * n
    if (row_id >= total_rows) return;                                  // whole wavefronts leave together
    const int r = (int)(row_id % (size_t)n);                           // row r attends to columns 0..r
    float *srow = scores + row_id * t_pad;
    const int c_end = min(t_pad, (r + 256) & ~255);
    float mx = -INFINITY;
    for (int c = lane; c <= r; c += 64) mx = fmaxf(mx, srow[c] * scale);
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int c = lane; c <= r; c += 64) sum += expf(srow[c] * scale - mx);
    sum = wave_sum(sum);
    for (int c = lane; c < c_end; c += 64) srow[c] = c <= r ? expf(srow[c] * scale - mx) / sum : 0.0f;
}

hipError_t launch_causal_softmax_f32(float *scores, int n_heads, int n, int t_pad, int head_dim, hipStream_t s) {
    const size_t rows = (size_t)n_heads * n;
    hipLaunchKernelGGL(causal_softmax_f32_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, scores, rows, n, t_pad,
                       1.0f / sqrtf((float)head_dim)); // transformer.rs:770
    return hipGetLastError();
}

// m = silu(g) * u on fp32 tensors (transformer.rs:557-565; tensor.rs:822-832, 722-734)
__global__ void silu_mul_f32_kernel(const float *g, const float *u, float *m, size_t total) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const float x = g[i];
        m[i] = (x / (1.0f + expf(-x))) * u[i];
    }
}

hipError_t launch_silu_mul_f32(const float *g, const float *u, float *m, size_t total, hipStream_t s) {
    const size_t want = (total + 255) / 256;
    hipLaunchKernelGGL(silu_mul_f32_kernel, dim3((unsigned)(want < 16384 ? (want ? want : 1) : 16384)), dim3(256), 0, s, g, u, m, total);
    return hipGetLastError();
}

} // namespace rlh
