// kernels.hip -- hand-written gfx950 (CDNA4, wave64) kernels for rllama's per-token forward path.
//
// Decode (one token) is bound by HBM bandwidth: every weight byte is read once per token.  The GEMV
// kernel therefore streams the weight rows with 16-byte loads per lane (a wave covers 1 KiB of one row
// per load), keeps several independent loads in flight per wave, holds the activation vector in LDS,
// accumulates in fp32 and reduces across the wave with DPP.  RMSNorm, the f16 rounding points, RoPE, the
// KV-cache write, SiLU*gate and the residual adds are fused into its prologue / epilogue so that one
// layer is five launches.
//
// Arithmetic follows the reference's rounding points (Noeda/rllama, paths relative to its checkout):
// f16 rounding of the GEMV inputs (transformer.rs:665-668, 537-540, 563-565, 795), of the GEMV outputs
// (tensor.rs:1623-1643) and of K/V on cache write (transformer.rs:754-761; tensor.rs:373-376);
// everything else in fp32.  Summation order inside a dot product differs from the reference's 8-lane
// order (tensor.rs:1577-1638), which is the only source of numerical difference.
#include "kernels.h"
#include "device_utils.h"
#include "synth.h"

namespace rlh {

// ------------------------------------------------------------------------------------------------
// GEMV
// ------------------------------------------------------------------------------------------------
constexpr int kGemvWaves = 4;
constexpr int kGemvThreads = kGemvWaves * kWave;
constexpr int kGemvUnroll = 4;  // 16-byte loads per row in flight per lane

template <typename WT>
struct WVec;
template <>
struct WVec<half_t> {
    static constexpr int kVec = 8;
    __device__ static __forceinline__ void unpack(const uint4_t &raw, float (&out)[8]) {
        half8_t h = __builtin_bit_cast(half8_t, raw);
#pragma unroll
        for (int i = 0; i < 8; i++) out[i] = (float)h[i];
    }
};
template <>
struct WVec<float> {
    static constexpr int kVec = 4;
    __device__ static __forceinline__ void unpack(const uint4_t &raw, float (&out)[4]) {
        float4_t f = __builtin_bit_cast(float4_t, raw);
#pragma unroll
        for (int i = 0; i < 4; i++) out[i] = f[i];
    }
};

template <typename XT, int kVec>
__device__ __forceinline__ void load_x(const XT *xs, float (&out)[kVec]) {
    if constexpr (sizeof(XT) == 2 && kVec == 8) {
        half8_t h = *reinterpret_cast<const half8_t *>(xs);
#pragma unroll
        for (int i = 0; i < 8; i++) out[i] = (float)h[i];
    } else if constexpr (sizeof(XT) == 2 && kVec == 4) {
        typedef __attribute__((ext_vector_type(4))) _Float16 half4_t;
        half4_t h = *reinterpret_cast<const half4_t *>(xs);
#pragma unroll
        for (int i = 0; i < 4; i++) out[i] = (float)h[i];
    } else if constexpr (sizeof(XT) == 4 && kVec == 8) {
        float4_t a = *reinterpret_cast<const float4_t *>(xs);
        float4_t b = *reinterpret_cast<const float4_t *>(xs + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            out[i] = a[i];
            out[i + 4] = b[i];
        }
    } else {
        float4_t a = *reinterpret_cast<const float4_t *>(xs);
#pragma unroll
        for (int i = 0; i < 4; i++) out[i] = a[i];
    }
}

__host__ __device__ inline int gemv_padded_k(int k, int vec) {
    const int per_chunk = kWave * vec * kGemvUnroll;
    return ((k + per_chunk - 1) / per_chunk) * per_chunk;
}

size_t gemv_lds_bytes(int k, int w_is_f16, int x_f16) {
    return (size_t)gemv_padded_k(k, w_is_f16 ? 8 : 4) * (x_f16 ? 2 : 4);
}

__device__ __forceinline__ void rope_pair(float re, float im, float2 f, float &ore, float &oim) {
    // transformer.rs:844-847: four products and two sums, each rounded to f32 (no FMA)
#pragma clang fp contract(off)
    float p0 = re * f.x;
    float p1 = im * f.y;
    float p2 = re * f.y;
    float p3 = im * f.x;
    ore = p0 - p1;
    oim = p2 + p3;
}

template <typename WT, typename XT, int kEpi, int kRows, bool kStream>
__global__ __launch_bounds__(kGemvThreads) void gemv_kernel(GemvParams p) {
    constexpr int kVec = WVec<WT>::kVec;
    constexpr int kMats = (kEpi == kEpiSilu) ? 2 : 1;
    extern __shared__ uint4_t smem_raw[];
    XT *xs = reinterpret_cast<XT *>(smem_raw);
    __shared__ float red[16];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int K = p.k;
    const int kpad = gemv_padded_k(K, kVec);
    const int n_chunks = kpad / (kWave * kVec * kGemvUnroll);
    const int row0 = (blockIdx.x * kGemvWaves + wave) * kRows;
    const WT *wbase[kMats];
    wbase[0] = reinterpret_cast<const WT *>(p.w);
    if constexpr (kMats == 2) wbase[1] = reinterpret_cast<const WT *>(p.w_b);

    uint4_t wreg[kMats][kRows][kGemvUnroll];
    auto load_chunk = [&](int c) {
#pragma unroll
        for (int u = 0; u < kGemvUnroll; u++) {
            const int kk = ((c * kGemvUnroll + u) * kWave + lane) * kVec;
#pragma unroll
            for (int m = 0; m < kMats; m++) {
#pragma unroll
                for (int r = 0; r < kRows; r++) {
                    const int row = row0 + r;
                    if (kk < K && row < p.n_rows) {
                        wreg[m][r][u] = load16<kStream>(wbase[m] + (size_t)row * K + kk);
                    } else {
                        wreg[m][r][u] = uint4_t{0u, 0u, 0u, 0u};
                    }
                }
            }
        }
    };

    // Weight loads do not depend on the activation: issue the first chunk before staging x.
    load_chunk(0);

    // ---- prologue: stage x in LDS (optionally RMSNorm'ed, optionally rounded to f16) ----
    if (p.norm_w != nullptr) {
        // RMSNorm::forward (transformer.rs:476-480): (x * rsqrt(mean(x^2) + eps)) * w
        float ss = 0.0f;
        for (int i = tid; i < K; i += kGemvThreads) {
            float v = p.x[i];
            ss = fmaf(v, v, ss);
        }
        ss = block_sum(ss, red);
        const float rs = 1.0f / sqrtf(ss / (float)K + p.eps);
        for (int i = tid; i < kpad; i += kGemvThreads) {
            float v = 0.0f;
            if (i < K) v = (p.x[i] * rs) * p.norm_w[i];
            xs[i] = (XT)v;
        }
    } else {
        for (int i = tid; i < kpad; i += kGemvThreads) {
            float v = i < K ? p.x[i] : 0.0f;
            xs[i] = (XT)v;
        }
    }
    __syncthreads();

    // ---- main loop ----
    float acc[kMats][kRows];
#pragma unroll
    for (int m = 0; m < kMats; m++)
#pragma unroll
        for (int r = 0; r < kRows; r++) acc[m][r] = 0.0f;

    for (int c = 0; c < n_chunks; c++) {
        uint4_t cur[kMats][kRows][kGemvUnroll];
#pragma unroll
        for (int m = 0; m < kMats; m++)
#pragma unroll
            for (int r = 0; r < kRows; r++)
#pragma unroll
                for (int u = 0; u < kGemvUnroll; u++) cur[m][r][u] = wreg[m][r][u];
        if (c + 1 < n_chunks) load_chunk(c + 1);
#pragma unroll
        for (int u = 0; u < kGemvUnroll; u++) {
            const int kk = ((c * kGemvUnroll + u) * kWave + lane) * kVec;
            float xv[kVec];
            load_x<XT, kVec>(xs + kk, xv);
#pragma unroll
            for (int m = 0; m < kMats; m++) {
#pragma unroll
                for (int r = 0; r < kRows; r++) {
                    float wv[kVec];
                    WVec<WT>::unpack(cur[m][r][u], wv);
#pragma unroll
                    for (int i = 0; i < kVec; i++) acc[m][r] = fmaf(wv[i], xv[i], acc[m][r]);
                }
            }
        }
    }

    // ---- wave reduction: results become wave-uniform ----
#pragma unroll
    for (int m = 0; m < kMats; m++)
#pragma unroll
        for (int r = 0; r < kRows; r++) {
            float v = wave_sum(acc[m][r]);
            acc[m][r] = p.round_y ? f16r(v) : v;
        }

    if (row0 >= p.n_rows || lane != 0) return;

    // ---- epilogue (lane 0 of each wave) ----
    if constexpr (kEpi == kEpiStore) {
#pragma unroll
        for (int r = 0; r < kRows; r++)
            if (row0 + r < p.n_rows) p.y[row0 + r] = acc[0][r];
    } else if constexpr (kEpi == kEpiResAdd) {
#pragma unroll
        for (int r = 0; r < kRows; r++)
            if (row0 + r < p.n_rows) p.y[row0 + r] = p.y[row0 + r] + acc[0][r];
    } else if constexpr (kEpi == kEpiSilu) {
#pragma unroll
        for (int r = 0; r < kRows; r++) {
            if (row0 + r < p.n_rows) {
                const float g = acc[0][r];
                const float u = acc[1][r];
                const float sg = g / (1.0f + expf(-g)); // tensor.rs:826-827
                const float mval = sg * u;                 // tensor.rs:729
                p.y[row0 + r] = p.x_f16 ? f16r(mval) : mval; // transformer.rs:563-565 (cast to w2's dtype)
            }
        }
    } else { // kEpiRopeKv: rows [0, dim) = wq, [dim, 2 dim) = wk, [2 dim, 3 dim) = wv
        static_assert(kEpi != kEpiRopeKv || (kRows % 2 == 0), "RoPE pairs must sit in one wave");
        const int pos = p.state->pos;
        const int half_hd = p.head_dim / 2;
#pragma unroll
        for (int r = 0; r < kRows; r += 2) {
            const int c = row0 + r;
            if (c + 1 < p.n_rows) {
                const int which = c / p.dim;
                const int j = c - which * p.dim;
                const int head = j / p.head_dim;
                const int jj = j - head * p.head_dim;
                float a = acc[0][r];
                float b = acc[0][r + 1];
                if (which < 2) {
                    const float2 f = p.freqs[(size_t)pos * half_hd + (jj >> 1)];
                    float ra, rb;
                    rope_pair(a, b, f, ra, rb);
                    a = ra;
                    b = rb;
                }
                if (which == 0) {
                    p.y[j] = a;
                    p.y[j + 1] = b;
                } else {
                    void *cache = which == 1 ? p.cache_k : p.cache_v;
                    const size_t idx = ((size_t)head * p.max_seq_len + pos) * p.head_dim + jj;
                    if (p.cache_f16) {
                        half2_t hv;
                        hv[0] = (half_t)a; // Tensor::set_f32 on an f16 cache (tensor.rs:373-376)
                        hv[1] = (half_t)b;
                        *reinterpret_cast<half2_t *>(reinterpret_cast<half_t *>(cache) + idx) = hv;
                    } else {
                        float2 fv = make_float2(a, b);
                        *reinterpret_cast<float2 *>(reinterpret_cast<float *>(cache) + idx) = fv;
                    }
                }
            }
        }
    }
}

template <typename WT, typename XT, int kEpi, int kRows>
static hipError_t launch_gemv_t(const GemvParams &p, hipStream_t s) {
    const int rows_per_block = kGemvWaves * kRows;
    const int blocks = (p.n_rows + rows_per_block - 1) / rows_per_block;
    const size_t lds = (size_t)gemv_padded_k(p.k, WVec<WT>::kVec) * sizeof(XT);
    if (p.stream_weights) {
        auto kern = gemv_kernel<WT, XT, kEpi, kRows, true>;
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGemvThreads), lds, s, p);
    } else {
        auto kern = gemv_kernel<WT, XT, kEpi, kRows, false>;
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGemvThreads), lds, s, p);
    }
    return hipGetLastError();
}

template <int kEpi, int kRows>
static hipError_t launch_gemv_e(const GemvParams &p, hipStream_t s) {
    if (p.w_is_f16) {
        return p.x_f16 ? launch_gemv_t<half_t, half_t, kEpi, kRows>(p, s) : launch_gemv_t<half_t, float, kEpi, kRows>(p, s);
    }
    return p.x_f16 ? launch_gemv_t<float, half_t, kEpi, kRows>(p, s) : launch_gemv_t<float, float, kEpi, kRows>(p, s);
}

hipError_t launch_gemv(const GemvParams &p, int epilogue, hipStream_t s) {
    const int vec = p.w_is_f16 ? 8 : 4;
    if (p.k <= 0 || p.n_rows <= 0 || (p.k % vec) != 0) return hipErrorInvalidValue;
    switch (epilogue) {
    case kEpiStore: return launch_gemv_e<kEpiStore, 2>(p, s);
    case kEpiResAdd: return launch_gemv_e<kEpiResAdd, 2>(p, s);
    case kEpiSilu: return launch_gemv_e<kEpiSilu, 2>(p, s);
    case kEpiRopeKv:
        if ((p.dim % 2) != 0 || (p.head_dim % 2) != 0 || p.n_rows != 3 * p.dim) return hipErrorInvalidValue;
        return launch_gemv_e<kEpiRopeKv, 2>(p, s);
    default: return hipErrorInvalidValue;
    }
}

// ------------------------------------------------------------------------------------------------
// Single-query attention over the KV cache (transformer.rs:727-781 for seq_len == 1).
// Cache layout per layer: [head][position][head_dim], so both the score pass (q . K[t]) and the value
// pass (sum_t p[t] V[t]) read whole 16-byte-per-lane rows.  Grid = (heads, splits over positions);
// softmax is evaluated with the running-max form, which equals the reference's exp(s)/sum(exp(s))
// (tensor.rs:479-494) wherever that is finite.  Partial results of the splits are merged by whichever
// block of a head finishes last.
// ------------------------------------------------------------------------------------------------
constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / kWave;

template <typename CT>
__device__ __forceinline__ void load8(const CT *p, float (&out)[8]) {
    if constexpr (sizeof(CT) == 2) {
        half8_t h = *reinterpret_cast<const half8_t *>(p);
#pragma unroll
        for (int i = 0; i < 8; i++) out[i] = (float)h[i];
    } else {
        float4_t a = *reinterpret_cast<const float4_t *>(p);
        float4_t b = *reinterpret_cast<const float4_t *>(p + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            out[i] = a[i];
            out[i + 4] = b[i];
        }
    }
}

template <typename CT, int kHeadDim>
__global__ __launch_bounds__(kAttnThreads) void attn_decode_kernel(AttnDecodeParams p) {
    constexpr int kLanesPerPos = kHeadDim / 8;         // each lane owns 8 consecutive dims
    constexpr int kPosPerWave = kWave / kLanesPerPos;  // positions handled per wave step
    static_assert(kLanesPerPos >= 1 && kLanesPerPos <= 16, "head_dim must be 8..128 in steps giving a power of two");
    extern __shared__ uint4_t smem_raw[];
    float *scores = reinterpret_cast<float *>(smem_raw);              // [chunk_cap]
    float *partial = scores + p.chunk_cap;                            // [kAttnWaves * kPosPerWave * kHeadDim]
    __shared__ float red[16];
    __shared__ int is_last_s;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int head = blockIdx.x;
    const int split = blockIdx.y;
    const int S = p.n_splits;
    const int T = p.state->pos + 1;
    int chunk = (T + S - 1) / S;
    chunk = (chunk + 15) & ~15;
    const int t0 = split * chunk;
    const int t1 = min(T, t0 + chunk);
    const int n = max(0, t1 - t0);
    const int sub = lane / kLanesPerPos;
    const int dl = lane % kLanesPerPos;
    const float scale = 1.0f / sqrtf((float)kHeadDim); // transformer.rs:770

    const CT *kbase = reinterpret_cast<const CT *>(p.cache_k) + (size_t)head * p.max_seq_len * kHeadDim;
    const CT *vbase = reinterpret_cast<const CT *>(p.cache_v) + (size_t)head * p.max_seq_len * kHeadDim;

    float m_loc = -INFINITY, l_loc = 0.0f, o_val = 0.0f;
    if (n > 0) {
        float qv[8];
#pragma unroll
        for (int i = 0; i < 8; i++) qv[i] = p.q[head * kHeadDim + dl * 8 + i];

        // pass 1: scores
        const int n_groups = (n + kPosPerWave - 1) / kPosPerWave;
        for (int g = wave; g < n_groups; g += kAttnWaves) {
            const int t = t0 + g * kPosPerWave + sub;
            float part = 0.0f;
            if (t < t1) {
                float kv[8];
                load8<CT>(kbase + (size_t)t * kHeadDim + dl * 8, kv);
#pragma unroll
                for (int i = 0; i < 8; i++) part = fmaf(qv[i], kv[i], part);
            }
            part = group_sum<kLanesPerPos>(part);
            if (dl == 0 && t < t1) scores[t - t0] = part * scale;
        }
        __syncthreads();

        // pass 2: softmax numerators
        float mx = -INFINITY;
        for (int i = tid; i < n; i += kAttnThreads) mx = fmaxf(mx, scores[i]);
        m_loc = block_max(mx, red);
        float ls = 0.0f;
        for (int i = tid; i < n; i += kAttnThreads) {
            float e = expf(scores[i] - m_loc);
            scores[i] = e;
            ls += e;
        }
        l_loc = block_sum(ls, red);

        // pass 3: values
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = 0.0f;
        for (int g = wave; g < n_groups; g += kAttnWaves) {
            const int t = t0 + g * kPosPerWave + sub;
            if (t < t1) {
                float vv[8];
                load8<CT>(vbase + (size_t)t * kHeadDim + dl * 8, vv);
                const float pt = scores[t - t0];
#pragma unroll
                for (int i = 0; i < 8; i++) acc[i] = fmaf(pt, vv[i], acc[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; i++) partial[(wave * kPosPerWave + sub) * kHeadDim + dl * 8 + i] = acc[i];
        __syncthreads();
        if (tid < kHeadDim) {
            float o = 0.0f;
#pragma unroll
            for (int w = 0; w < kAttnWaves * kPosPerWave; w++) o += partial[w * kHeadDim + tid];
            o_val = o;
        }
    }

    if (S == 1) {
        if (tid < kHeadDim) {
            float o = o_val / l_loc;
            p.out[head * kHeadDim + tid] = p.round_out ? f16r(o) : o;
        }
        return;
    }

    // ---- merge the splits: last block of this head to arrive does it ----
    float *ws = p.workspace + ((size_t)head * S + split) * (kHeadDim + 2);
    if (tid == 0) {
        ws[0] = m_loc;
        ws[1] = l_loc;
    }
    if (tid < kHeadDim) ws[2 + tid] = o_val;
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        unsigned int prev = atomicAdd(&p.counters[head], 1u);
        is_last_s = (prev == (unsigned int)(S - 1));
    }
    __syncthreads();
    if (!is_last_s) return;
    __threadfence();
    if (tid < kHeadDim) {
        const float *wh = p.workspace + (size_t)head * S * (kHeadDim + 2);
        float M = -INFINITY;
        for (int s2 = 0; s2 < S; s2++) M = fmaxf(M, __builtin_nontemporal_load(wh + (size_t)s2 * (kHeadDim + 2)));
        float L = 0.0f, O = 0.0f;
        for (int s2 = 0; s2 < S; s2++) {
            const float *w2 = wh + (size_t)s2 * (kHeadDim + 2);
            const float ms = __builtin_nontemporal_load(w2);
            const float ls2 = __builtin_nontemporal_load(w2 + 1);
            const float os = __builtin_nontemporal_load(w2 + 2 + tid);
            const float f = (ls2 > 0.0f) ? expf(ms - M) : 0.0f;
            L = fmaf(ls2, f, L);
            O = fmaf(os, f, O);
        }
        float o = O / L;
        p.out[head * kHeadDim + tid] = p.round_out ? f16r(o) : o;
    }
    if (tid == 0) p.counters[head] = 0u; // ready for the next launch (ordered by the stream)
}

template <typename CT>
static hipError_t launch_attn_t(const AttnDecodeParams &p, hipStream_t s) {
    dim3 grid(p.n_heads, p.n_splits);
    const int lanes_per_pos = p.head_dim / 8;
    const int pos_per_wave = kWave / lanes_per_pos;
    const size_t lds = ((size_t)p.chunk_cap + (size_t)kAttnWaves * pos_per_wave * p.head_dim) * sizeof(float);
    switch (p.head_dim) {
    case 128: hipLaunchKernelGGL((attn_decode_kernel<CT, 128>), grid, dim3(kAttnThreads), lds, s, p); break;
    case 64: hipLaunchKernelGGL((attn_decode_kernel<CT, 64>), grid, dim3(kAttnThreads), lds, s, p); break;
    case 32: hipLaunchKernelGGL((attn_decode_kernel<CT, 32>), grid, dim3(kAttnThreads), lds, s, p); break;
    case 16: hipLaunchKernelGGL((attn_decode_kernel<CT, 16>), grid, dim3(kAttnThreads), lds, s, p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_attn_decode(const AttnDecodeParams &p, hipStream_t s) {
    if (p.n_splits < 1 || p.chunk_cap < 16 || (p.chunk_cap % 16) != 0) return hipErrorInvalidValue;
    if (p.n_splits > 1 && (p.workspace == nullptr || p.counters == nullptr)) return hipErrorInvalidValue;
    return p.cache_f16 ? launch_attn_t<half_t>(p, s) : launch_attn_t<float>(p, s);
}

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
                                                              int32_t *out_tokens, int out_cap) {
    // TokenSampler::sample at top_k = 1 (token_sampler.rs:99-147): the max/shift loops run over
    // 0..logits.rows() == 0..1 on the transposed 1 x vocab tensor, so token 0's logit becomes l0 - l0
    // and the rest are untouched; softmax is monotonic, so the winner is the largest shifted logit.
    // NaN never wins (sorted last, :131-145); equal values resolve to the lowest id.
    __shared__ float sval[16];
    __shared__ int sidx[16];
    const int tid = threadIdx.x;
    float best = -INFINITY;
    int besti = -1;
    for (int i = tid; i < vocab; i += blockDim.x) {
        float v = logits[i];
        if (i == 0) v = v - v;
        if (v > best || (besti < 0 && v == best)) {
            best = v;
            besti = i;
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        float ov = __shfl_xor(best, off, kWave);
        int oi = __shfl_xor(besti, off, kWave);
        bool take = (oi >= 0) && (besti < 0 || ov > best || (ov == best && oi < besti));
        if (take) {
            best = ov;
            besti = oi;
        }
    }
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    if (lane == 0) {
        sval[wave] = best;
        sidx[wave] = besti;
    }
    __syncthreads();
    if (tid == 0) {
        const int nw = blockDim.x / kWave;
        for (int w = 1; w < nw; w++) {
            float ov = sval[w];
            int oi = sidx[w];
            bool take = (oi >= 0) && (besti < 0 || ov > best || (ov == best && oi < besti));
            if (take) {
                best = ov;
                besti = oi;
            }
        }
        if (besti < 0) besti = 0; // every logit NaN
        state->token = besti;
        state->pos = state->pos + 1;
        const int k = state->n_out;
        if (out_tokens != nullptr && k < out_cap) out_tokens[k] = besti;
        state->n_out = k + 1;
    }
}

hipError_t launch_argmax_advance(const float *logits, int vocab, DecodeState *state, int32_t *out_tokens, int out_cap,
                                 hipStream_t s) {
    hipLaunchKernelGGL(argmax_advance_kernel, dim3(1), dim3(1024), 0, s, logits, vocab, state, out_tokens, out_cap);
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
