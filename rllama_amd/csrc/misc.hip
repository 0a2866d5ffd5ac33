// misc.hip -- the small gfx950 kernels around the token step (embedding row, greedy pick, device state),
// the synthetic-weight fill, and the op-level element-wise kernels.
#include "kernels.h"
#include "device_utils.h"
#include "synth.h"

namespace rlh {

// ------------------------------------------------------------------------------------------------
// Small kernels of the token loop
// ------------------------------------------------------------------------------------------------
template <typename ET>
__global__ void embed_kernel(const ET *table, int dim, const DecodeState *state, float *x) {
    // Embedding::get_embedding (embedding.rs:50-52): one table row, widened to f32
    const int tok = state->token;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < dim; i += gridDim.x * blockDim.x) {
        x[i] = (float)table[(size_t)tok * dim + i];
    }
}

hipError_t launch_embed(const void *table, int table_f16, int dim, const DecodeState *state, float *x, hipStream_t s) {
    const int threads = 256;
    const int blocks = (dim + threads - 1) / threads;
    if (table_f16) {
        hipLaunchKernelGGL(embed_kernel<half_t>, dim3(blocks), dim3(threads), 0, s, reinterpret_cast<const half_t *>(table), dim, state, x);
    } else {
        hipLaunchKernelGGL(embed_kernel<float>, dim3(blocks), dim3(threads), 0, s, reinterpret_cast<const float *>(table), dim, state, x);
    }
    return hipGetLastError();
}

__global__ __launch_bounds__(1024) void argmax_advance_kernel(const float *logits, int vocab, DecodeState *state,
                                                              int32_t *out_tokens, int out_cap, float scale) {
    // TokenSampler::sample at top_k = 1 (token_sampler.rs:99-147): the max/shift loops run over
    // 0..logits.rows() == 0..1 on the transposed 1 x vocab tensor, so token 0's logit becomes l0 - l0
    // and the rest are untouched; then softmax WITHOUT a maximum subtracted (tensor.rs:479-494), a sort by
    // descending probability with NaN last (:131-145), and the first entry wins.
    //   * While sum(exp(l)) is finite, exp and the division by the sum keep the order of the logits, so the winner is
    //     the largest shifted logit (equal values: the lowest id).
    //   * Once that sum is not finite every probability is 0 or NaN: a logit above ln(FLT_MAX) gives inf / inf = NaN,
    //     everything else x / inf = 0, and a NaN logit turns the sum and with it every probability into NaN.  What wins then
    //     is the lowest id whose probability is not NaN -- token 0, whose shifted logit is exactly 0 -- or, with every
    //     probability NaN, the id the reference's fall-through returns, 0 as well.
    // `scale` is 1 / temperature (:99-102; 1.0 leaves the logits as they are).
    // The sum is only evaluated when it can overflow at all (largest logit above ln(FLT_MAX / vocab)); it is then formed in
    // double, which decides like the reference's sequential f32 sum except within rounding of FLT_MAX itself.
    __shared__ float sval[16];
    __shared__ int sidx[16];
    __shared__ int snan[16];
    __shared__ double ssum[16];
    __shared__ float s_best;
    __shared__ int s_nan;
    const int tid = threadIdx.x;
    float best = -INFINITY;
    int besti = -1;
    int seen_nan = 0;
    auto consider = [&](float v, int i) {
        v = v * scale;
        if (i == 0) v = v - v;
        if (v != v) seen_nan = 1;
        if (v > best || (besti < 0 && v == best)) {
            best = v;
            besti = i;
        }
    };
    if ((vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0) {
        // 16-byte loads, 8 of them in flight per thread before the first comparison: one memory latency per 32 K logits instead
        // of one per element (a thread visits its indices in ascending order, so ties still go to the lowest id)
        const float4_t *l4 = reinterpret_cast<const float4_t *>(logits);
        const int n4 = vocab / 4;
        for (int base = 0; base < n4; base += 8 * 1024) {
            float4_t v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int i4 = base + u * 1024 + tid;
                v[u] = i4 < n4 ? l4[i4] : float4_t{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int i4 = base + u * 1024 + tid;
                if (i4 < n4) {
#pragma unroll
                    for (int e = 0; e < 4; e++) consider(v[u][e], i4 * 4 + e);
                }
            }
        }
    } else {
        for (int i = tid; i < vocab; i += blockDim.x) consider(logits[i], i);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        float ov = __shfl_xor(best, off, kWave);
        int oi = __shfl_xor(besti, off, kWave);
        seen_nan |= __shfl_xor(seen_nan, off, kWave);
        bool take = (oi >= 0) && (besti < 0 || ov > best || (ov == best && oi < besti));
        if (take) {
            best = ov;
            besti = oi;
        }
    }
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int nw = blockDim.x / kWave;
    if (lane == 0) {
        sval[wave] = best;
        sidx[wave] = besti;
        snan[wave] = seen_nan;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < nw; w++) {
            float ov = sval[w];
            int oi = sidx[w];
            seen_nan |= snan[w];
            bool take = (oi >= 0) && (besti < 0 || ov > best || (ov == best && oi < besti));
            if (take) {
                best = ov;
                besti = oi;
            }
        }
        s_best = best;
        s_nan = seen_nan;
    }
    __syncthreads();
    // can sum(exp(l)) overflow f32?  Only if vocab * exp(largest) can: largest > ln(FLT_MAX) - ln(vocab)
    const float kLnFltMax = 88.72283172607422f; // expf overflows above this value
    const bool sum_at_risk = !s_nan && s_best <= kLnFltMax && s_best > kLnFltMax - logf((float)vocab);
    double total = 0.0;
    if (sum_at_risk) { // block-uniform
        double part = 0.0;
        for (int i = tid; i < vocab; i += blockDim.x) {
            const float v = i == 0 ? 0.0f : logits[i] * scale;
            part += exp((double)v);
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) part += __shfl_xor(part, off, kWave);
        if (lane == 0) ssum[wave] = part;
        __syncthreads();
        if (tid == 0)
            for (int w = 0; w < nw; w++) total += ssum[w];
    }
    if (tid == 0) {
        if (besti < 0) besti = 0;                                           // every logit NaN
        if (seen_nan || best > kLnFltMax || total > 3.4028234663852886e38) besti = 0; // sum not finite: see above
        state->token = besti;
        state->pos = state->pos + 1;
        const int k = state->n_out;
        if (out_tokens != nullptr && k < out_cap) out_tokens[k] = besti;
        state->n_out = k + 1;
    }
}

hipError_t launch_argmax_advance(const float *logits, int vocab, DecodeState *state, int32_t *out_tokens, int out_cap,
                                 hipStream_t s, float scale) {
    hipLaunchKernelGGL(argmax_advance_kernel, dim3(1), dim3(1024), 0, s, logits, vocab, state, out_tokens, out_cap, scale);
    return hipGetLastError();
}

__global__ void set_state_kernel(DecodeState *state, int pos, int token, int reset_out) {
    state->pos = pos;
    state->token = token;
    if (reset_out) state->n_out = 0;
}

hipError_t launch_set_state(DecodeState *state, int pos, int token, int reset_out, hipStream_t s) {
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(1), 0, s, state, pos, token, reset_out);
    return hipGetLastError();
}

__global__ void reset_out_kernel(DecodeState *state) { state->n_out = 0; }

hipError_t launch_reset_out(DecodeState *state, hipStream_t s) {
    hipLaunchKernelGGL(reset_out_kernel, dim3(1), dim3(1), 0, s, state);
    return hipGetLastError();
}

__global__ void advance_pos_kernel(DecodeState *state, const int32_t *tokens, int idx) {
    state->pos = state->pos + 1;
    state->token = tokens[idx];
}

hipError_t launch_advance_pos(DecodeState *state, const int32_t *tokens_dev, int idx, hipStream_t s) {
    hipLaunchKernelGGL(advance_pos_kernel, dim3(1), dim3(1), 0, s, state, tokens_dev, idx);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// Synthetic fills
// ------------------------------------------------------------------------------------------------
template <typename ET>
__global__ void synth_fill_kernel(ET *dst, uint64_t n, uint64_t key, double std) {
    // one polar pair (elements 2p, 2p + 1) per thread step
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    const uint64_t n_pairs = (n + 1) / 2;
    for (uint64_t pr = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; pr < n_pairs; pr += stride) {
        double z0, z1;
        synth_normal_pair(key, pr, &z0, &z1);
        const uint64_t i = pr * 2;
        dst[i] = (ET)__builtin_bit_cast(half_t, synth_scale_to_f16(z0, std));
        if (i + 1 < n) dst[i + 1] = (ET)__builtin_bit_cast(half_t, synth_scale_to_f16(z1, std));
    }
}

hipError_t launch_synth_fill(void *dst, int dst_f16, uint64_t n, uint64_t key, double std, hipStream_t s) {
    const int threads = 256;
    uint64_t want = ((n + 1) / 2 + threads - 1) / threads;
    const int blocks = (int)(want < 65536 ? (want ? want : 1) : 65536);
    if (dst_f16) {
        hipLaunchKernelGGL(synth_fill_kernel<half_t>, dim3(blocks), dim3(threads), 0, s, reinterpret_cast<half_t *>(dst), n, key, std);
    } else {
        hipLaunchKernelGGL(synth_fill_kernel<float>, dim3(blocks), dim3(threads), 0, s, reinterpret_cast<float *>(dst), n, key, std);
    }
    return hipGetLastError();
}

template <typename T>
__global__ void fill_kernel(T *dst, uint64_t n, T v) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = v;
}

static int fill_blocks(uint64_t n) {
    uint64_t want = (n + 255) / 256;
    return (int)(want < 16384 ? (want ? want : 1) : 16384);
}

hipError_t launch_fill_f32(float *dst, uint64_t n, float v, hipStream_t s) {
    hipLaunchKernelGGL(fill_kernel<float>, dim3(fill_blocks(n)), dim3(256), 0, s, dst, n, v);
    return hipGetLastError();
}

hipError_t launch_fill_u32(uint32_t *dst, uint64_t n, uint32_t v, hipStream_t s) {
    hipLaunchKernelGGL(fill_kernel<uint32_t>, dim3(fill_blocks(n)), dim3(256), 0, s, dst, n, v);
    return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// Op level
// ------------------------------------------------------------------------------------------------
template <typename DT, typename ST>
__global__ void convert_kernel(DT *dst, const ST *src, uint64_t n) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = (DT)(float)src[i];
}

hipError_t launch_convert(void *dst, int dst_f16, const void *src, int src_f16, uint64_t n, hipStream_t s) {
    dim3 g(fill_blocks(n)), b(256);
    if (dst_f16 && src_f16) hipLaunchKernelGGL((convert_kernel<half_t, half_t>), g, b, 0, s, (half_t *)dst, (const half_t *)src, n);
    else if (dst_f16) hipLaunchKernelGGL((convert_kernel<half_t, float>), g, b, 0, s, (half_t *)dst, (const float *)src, n);
    else if (src_f16) hipLaunchKernelGGL((convert_kernel<float, half_t>), g, b, 0, s, (float *)dst, (const half_t *)src, n);
    else hipLaunchKernelGGL((convert_kernel<float, float>), g, b, 0, s, (float *)dst, (const float *)src, n);
    return hipGetLastError();
}

template <typename T>
__global__ void transpose_kernel(T *dst, const T *src, int rows, int cols) {
    // dst [cols x rows] = src^T; 32x32 tiles through LDS so both sides are coalesced
    __shared__ T tile[32][33];
    const int bx = blockIdx.x * 32, by = blockIdx.y * 32;
    for (int j = threadIdx.y; j < 32; j += blockDim.y) {
        int r = by + j, c = bx + threadIdx.x;
        if (r < rows && c < cols) tile[j][threadIdx.x] = src[(size_t)r * cols + c];
    }
    __syncthreads();
    for (int j = threadIdx.y; j < 32; j += blockDim.y) {
        int r = bx + j, c = by + threadIdx.x; // dst coordinates
        if (r < cols && c < rows) dst[(size_t)r * rows + c] = tile[threadIdx.x][j];
    }
}

hipError_t launch_transpose(void *dst, const void *src, int rows, int cols, int is_f16, hipStream_t s) {
    dim3 g((cols + 31) / 32, (rows + 31) / 32), b(32, 8);
    if (is_f16) hipLaunchKernelGGL(transpose_kernel<half_t>, g, b, 0, s, (half_t *)dst, (const half_t *)src, rows, cols);
    else hipLaunchKernelGGL(transpose_kernel<float>, g, b, 0, s, (float *)dst, (const float *)src, rows, cols);
    return hipGetLastError();
}

template <typename T>
__global__ void hadamard_kernel(T *dst, const T *src, uint64_t n) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        dst[i] = (T)((float)dst[i] * (float)src[i]);
    }
}

hipError_t launch_hadamard(void *dst, const void *src, uint64_t n, int is_f16, hipStream_t s) {
    dim3 g(fill_blocks(n)), b(256);
    if (is_f16) hipLaunchKernelGGL(hadamard_kernel<half_t>, g, b, 0, s, (half_t *)dst, (const half_t *)src, n);
    else hipLaunchKernelGGL(hadamard_kernel<float>, g, b, 0, s, (float *)dst, (const float *)src, n);
    return hipGetLastError();
}

// dst = a + b (Tensor::add, tensor.rs:573-593), f32
__global__ void add_f32_kernel(float *dst, const float *a, const float *b, uint64_t n) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = a[i] + b[i];
}

hipError_t launch_add_f32(float *dst, const float *a, const float *b, uint64_t n, hipStream_t s) {
    dim3 g(fill_blocks(n)), blk(256);
    hipLaunchKernelGGL(add_f32_kernel, g, blk, 0, s, dst, a, b, n);
    return hipGetLastError();
}

template <typename T>
__global__ void silu_kernel(T *dst, uint64_t n) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float v = (float)dst[i];
        dst[i] = (T)(v / (1.0f + expf(-v)));
    }
}

hipError_t launch_silu(void *dst, uint64_t n, int is_f16, hipStream_t s) {
    dim3 g(fill_blocks(n)), b(256);
    if (is_f16) hipLaunchKernelGGL(silu_kernel<half_t>, g, b, 0, s, (half_t *)dst, n);
    else hipLaunchKernelGGL(silu_kernel<float>, g, b, 0, s, (float *)dst, n);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(float *y, const float *x, const float *w, int d, float eps, int round_y) {
    __shared__ float red[16];
    const float *xr = x + (size_t)blockIdx.x * d;
    float *yr = y + (size_t)blockIdx.x * d;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) ss = fmaf(xr[i], xr[i], ss);
    ss = block_sum(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        float v = (xr[i] * rs) * w[i];
        yr[i] = round_y ? f16r(v) : v;
    }
}

hipError_t launch_rmsnorm_rows(float *y, const float *x, const float *w, int rows, int d, float eps, int round_y, hipStream_t s) {
    hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3(rows), dim3(256), 0, s, y, x, w, d, eps, round_y);
    return hipGetLastError();
}

__global__ void rope_row_kernel(float *x, int n_heads, int head_dim, const float2 *freqs) {
    const int half = head_dim / 2;
    const int total = n_heads * half;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        const int h = i / half, c = i - h * half;
        float *pr = x + (size_t)h * head_dim + 2 * c;
        float a, b;
        rope_pair(pr[0], pr[1], freqs[c], a, b);
        pr[0] = a;
        pr[1] = b;
    }
}

hipError_t launch_rope_row(float *x, int n_heads, int head_dim, const float2 *freqs_at_pos, hipStream_t s) {
    const int total = n_heads * (head_dim / 2);
    hipLaunchKernelGGL(rope_row_kernel, dim3((total + 255) / 256), dim3(256), 0, s, x, n_heads, head_dim, freqs_at_pos);
    return hipGetLastError();
}

// m = silu(g) * u on f16 tensors: g and u are f16 values (projection outputs, tensor.rs:1623-1643), the product is formed
// in f32 and rounded once (transformer.rs:557-565)
__global__ void silu_mul_f16_kernel(const half_t *g, const half_t *u, half_t *m, size_t total) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const float x = (float)g[i];
        m[i] = to_f16((x / (1.0f + expf(-x))) * (float)u[i]);
    }
}

hipError_t launch_silu_mul_f16(const void *g, const void *u, void *m, size_t total, hipStream_t s) {
    hipLaunchKernelGGL(silu_mul_f16_kernel, dim3(fill_blocks(total)), dim3(256), 0, s, (const half_t *)g, (const half_t *)u, (half_t *)m, total);
    return hipGetLastError();
}

// One token's attention inputs (transformer.rs:704-761 with seq_len 1): RoPE on q (in place) and on k, then k and v go
// into the cache planes [head][position][head_dim] at `pos`, rounded to f16 where the cache is f16.
template <typename CT>
__global__ void rope_kvwrite_kernel(float *q, const float *k, const float *v, CT *cache_k, CT *cache_v, int n_heads, int head_dim, int max_seq_len,
                                    int pos, const float2 *freqs) {
    const int half = head_dim / 2;
    const int total = n_heads * half;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        const int h = i / half, c = i - h * half;
        const size_t e = (size_t)h * head_dim + 2 * c;
        float a, b;
        rope_pair(q[e], q[e + 1], freqs[c], a, b);
        q[e] = a;
        q[e + 1] = b;
        rope_pair(k[e], k[e + 1], freqs[c], a, b);
        const size_t idx = ((size_t)h * max_seq_len + pos) * head_dim + 2 * c;
        cache_k[idx] = (CT)a; // Tensor::set_f32 on the cache's dtype (tensor.rs:373-376)
        cache_k[idx + 1] = (CT)b;
        cache_v[idx] = (CT)v[e];
        cache_v[idx + 1] = (CT)v[e + 1];
    }
}

hipError_t launch_rope_kvwrite(float *q, const float *k, const float *v, void *cache_k, void *cache_v, int cache_f16, int n_heads, int head_dim,
                               int max_seq_len, int pos, const float2 *freqs_at_pos, hipStream_t s) {
    const int total = n_heads * (head_dim / 2);
    dim3 g((total + 255) / 256), b(256);
    if (cache_f16)
        hipLaunchKernelGGL(rope_kvwrite_kernel<half_t>, g, b, 0, s, q, k, v, (half_t *)cache_k, (half_t *)cache_v, n_heads, head_dim, max_seq_len, pos, freqs_at_pos);
    else
        hipLaunchKernelGGL(rope_kvwrite_kernel<float>, g, b, 0, s, q, k, v, (float *)cache_k, (float *)cache_v, n_heads, head_dim, max_seq_len, pos, freqs_at_pos);
    return hipGetLastError();
}

template <typename T>
__global__ void cache_shift_kernel(T *dst, const T *src, size_t planes, int max_seq_len, int head_dim, int shifts) {
    // AttentionCache::shift_left (transformer.rs:180-197), `shifts` times: position t takes position
    // min(t + shifts, max_seq_len - 1).
    const size_t per_plane = (size_t)max_seq_len * head_dim;
    const size_t total = planes * per_plane;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const size_t plane = i / per_plane;
        const size_t rem = i - plane * per_plane;
        const int t = (int)(rem / head_dim);
        const int j = (int)(rem - (size_t)t * head_dim);
        int ts = t + shifts;
        if (ts > max_seq_len - 1) ts = max_seq_len - 1;
        dst[i] = src[plane * per_plane + (size_t)ts * head_dim + j];
    }
}

hipError_t launch_cache_shift_left(void *cache, int is_f16, size_t planes, int max_seq_len, int head_dim, int shifts, hipStream_t s) {
    const size_t total = planes * (size_t)max_seq_len * head_dim;
    const size_t bytes = total * (is_f16 ? 2 : 4);
    void *tmp = nullptr;
    hipError_t e = hipMalloc(&tmp, bytes);
    if (e != hipSuccess) return e;
    dim3 g(fill_blocks(total)), b(256);
    if (is_f16) hipLaunchKernelGGL(cache_shift_kernel<half_t>, g, b, 0, s, (half_t *)tmp, (const half_t *)cache, planes, max_seq_len, head_dim, shifts);
    else hipLaunchKernelGGL(cache_shift_kernel<float>, g, b, 0, s, (float *)tmp, (const float *)cache, planes, max_seq_len, head_dim, shifts);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpyAsync(cache, tmp, bytes, hipMemcpyDeviceToDevice, s);
    hipError_t e2 = hipStreamSynchronize(s);
    (void)hipFree(tmp);
    return e != hipSuccess ? e : e2;
}

template <typename T>
__global__ void cache_read_kernel(float *dst, const T *plane, int max_seq_len, int head_dim) {
    const int total = max_seq_len * head_dim;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        const int j = i / max_seq_len, t = i - j * max_seq_len; // dst [head_dim x max_seq_len]
        dst[i] = (float)plane[(size_t)t * head_dim + j];
    }
}

hipError_t launch_cache_read(float *dst, const void *plane, int is_f16, int max_seq_len, int head_dim, hipStream_t s) {
    const int total = max_seq_len * head_dim;
    dim3 g((total + 255) / 256), b(256);
    if (is_f16) hipLaunchKernelGGL(cache_read_kernel<half_t>, g, b, 0, s, dst, (const half_t *)plane, max_seq_len, head_dim);
    else hipLaunchKernelGGL(cache_read_kernel<float>, g, b, 0, s, dst, (const float *)plane, max_seq_len, head_dim);
    return hipGetLastError();
}

} // namespace rlh
