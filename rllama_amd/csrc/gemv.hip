// gemv.hip -- batch-1 decode GEMV for gfx950 (CDNA4, wave64): y = W x with W [n_rows x k] row-major in HBM.
//
// One token step reads every weight byte exactly once, so this kernel is bound by HBM bandwidth and is
// built as a streaming reader:
//   * a wavefront produces one output row at a time with 16-byte loads per lane (one load instruction
//     covers 1 KiB of the row), issued in bursts of 8 independent loads whose addresses differ by
//     compile-time offsets, so the per-load instruction overhead is one VMEM instruction;
//   * rows are interleaved over all wavefronts of the grid (wave w takes rows w, w + W, ...), so that at
//     any moment the grid reads one dense window of the matrix, and the launch is sized so that all
//     wavefronts are resident at once (about 8 per CU);
//   * the activation vector lives in LDS (as f16 where the reference rounds it to f16), products are
//     accumulated in fp32 (v_fma_mix_f32 takes the f16 operands directly) and reduced across the wave
//     with DPP;
//   * what surrounds the product in the reference is fused in: the residual add and RMSNorm that
//     produce x (prologue), and RoPE + KV-cache write, or SiLU*gate, or the f16 rounding of y (epilogue).
//
// Rounding points follow the reference (Noeda/rllama): x -> f16 (transformer.rs:665-668, 537-540, 563-565,
// 795), y -> f16 (tensor.rs:1623-1643), K/V -> f16 on cache write (transformer.rs:754-761).  The order of
// the fp32 additions inside one dot product differs from the reference's 8-lane order (tensor.rs:1577-1638);
// that is the only numerical difference.
#include "kernels.h"
#include "device_utils.h"

namespace rlh {

// Launch shape (overridable at compile time for tuning runs).
#ifndef RLH_GEMV_WAVES
#define RLH_GEMV_WAVES 4
#endif
#ifndef RLH_GEMV_TARGET_WAVES
#define RLH_GEMV_TARGET_WAVES 2048 // 256 CUs x 8 resident wavefronts
#endif
#ifndef RLH_GEMV_BURST
#define RLH_GEMV_BURST 8
#endif
constexpr int kGemvWaves = RLH_GEMV_WAVES;
constexpr int kGemvThreads = kGemvWaves * kWave;
constexpr int kGemvTargetWaves = RLH_GEMV_TARGET_WAVES;

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

// iterations of 64 lanes x vec elements that cover k, and the LDS footprint that goes with them
__host__ __device__ inline int gemv_iters(int k, int vec) { return (k + kWave * vec - 1) / (kWave * vec); }

size_t gemv_lds_bytes(int k, int w_is_f16, int x_f16) {
    const int vec = w_is_f16 ? 8 : 4;
    return (size_t)gemv_iters(k, vec) * kWave * vec * (x_f16 ? 2 : 4);
}

// Sum over the wavefront, valid in lane 63 only (no broadcast).
__device__ __forceinline__ float wave_sum_lane63(float v) {
    v = group_sum<16>(v);
    v = dpp_add<kDppRowBcast15, 0xa>(v);
    v = dpp_add<kDppRowBcast31, 0xc>(v);
    return v;
}

constexpr int kGemvBurst = RLH_GEMV_BURST; // 16-byte loads per lane issued back to back before they are consumed
#ifndef RLH_GEMV_PRELOAD
#define RLH_GEMV_PRELOAD 1
#endif
#ifndef RLH_GEMV_PROLOGUE_VECS
#define RLH_GEMV_PROLOGUE_VECS 8
#endif
constexpr int kGemvPrologueVecs = RLH_GEMV_PROLOGUE_VECS; // float4 loads per thread per prologue batch (one batch covers k <= 1024 * this)

template <typename WT, typename XT, int kEpi, bool kStream>
__global__ __launch_bounds__(kGemvThreads) void gemv_kernel(GemvParams p) {
    constexpr int kVec = WVec<WT>::kVec;
    constexpr int kMats = (kEpi == kEpiSilu) ? 2 : 1;    // w1 and w3 share x and the epilogue
    constexpr int kRows = (kEpi == kEpiRopeKv) ? 2 : 1;  // a RoPE pair (2j, 2j+1) is produced by one wave
    constexpr int kU = kGemvBurst / (kMats * kRows);     // pieces of one row per burst
    constexpr int kPiece = kWave * kVec;                  // elements one wave-wide load covers
    extern __shared__ uint4_t smem_raw[];
    XT *xs = reinterpret_cast<XT *>(smem_raw);
    __shared__ float red[16];
    __shared__ float2 rope_f[64]; // (cos, sin) of this position, head_dim / 2 <= 64 entries

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int K = p.k;
    const int pieces = gemv_iters(K, kVec);      // incl. a partial last piece
    const int pieces_full = K / kPiece;
    const int kpad = pieces * kPiece;

    // The first burst of this wavefront's first row unit does not depend on x: it is issued right behind the prologue's own
    // loads (which stay ahead of it in the in-order return queue), so that its memory latency runs under the norm / staging work.
    const WT *wmat[kMats];
    wmat[0] = reinterpret_cast<const WT *>(p.w);
    if constexpr (kMats == 2) wmat[1] = reinterpret_cast<const WT *>(p.w_b);
    const int unit_first = blockIdx.x * kGemvWaves + wave;
    // (measured: worth 1 % on the w1|w3 product, nothing or a loss on the others, so only that instantiation does it)
    const bool have_pre = RLH_GEMV_PRELOAD && kEpi == kEpiSilu && unit_first < p.n_rows / kRows && kU <= pieces_full;
    uint4_t wpre[kU][kMats][kRows];
    auto preload = [&]() {
        if (have_pre) {
#pragma unroll
            for (int u = 0; u < kU; u++)
#pragma unroll
                for (int m = 0; m < kMats; m++)
#pragma unroll
                    for (int r = 0; r < kRows; r++)
                        wpre[u][m][r] = load16<kStream>(wmat[m] + (size_t)(unit_first * kRows + r) * K + (size_t)u * kPiece + lane * kVec);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- prologue: x = (x_in [+ x_add]) [RMSNorm] [-> f16], staged in LDS, zero padded to kpad ----
    // All global loads of a batch are issued before any is consumed (one exposed memory latency per batch).
    const bool writes_sum = (p.x_out != nullptr) && blockIdx.x == 0;
    const int n4 = K / 4; // k is a multiple of 4
    const float4_t *x4 = reinterpret_cast<const float4_t *>(p.x);
    const float4_t *a4 = reinterpret_cast<const float4_t *>(p.x_add);
    float4_t *o4 = reinterpret_cast<float4_t *>(p.x_out);
    for (int i = K + tid; i < kpad; i += kGemvThreads) xs[i] = (XT)0.0f;
    if (p.norm_w != nullptr && n4 <= kGemvPrologueVecs * kGemvThreads) {
        // RMSNorm::forward (transformer.rs:476-480): (x * rsqrt(mean(x^2) + eps)) * w, x kept in registers
        const float4_t *w4 = reinterpret_cast<const float4_t *>(p.norm_w);
        float4_t xv[kGemvPrologueVecs], wv[kGemvPrologueVecs];
#pragma unroll
        for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = x4[min(tid + j * kGemvThreads, n4 - 1)];
        if (a4 != nullptr) {
#pragma unroll
            for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = xv[j] + a4[min(tid + j * kGemvThreads, n4 - 1)]; // transformer.rs:442 / :445
        }
#pragma unroll
        for (int j = 0; j < kGemvPrologueVecs; j++) wv[j] = w4[min(tid + j * kGemvThreads, n4 - 1)];
        __builtin_amdgcn_sched_barrier(0);
        preload();
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < kGemvPrologueVecs; j++) {
            const int i = tid + j * kGemvThreads;
            if (i < n4) {
                if (writes_sum) o4[i] = xv[j];
#pragma unroll
                for (int e = 0; e < 4; e++) ss = fmaf(xv[j][e], xv[j][e], ss);
            }
        }
        ss = block_sum(ss, red);
        const float rs = 1.0f / sqrtf(ss / (float)K + p.eps);
#pragma unroll
        for (int j = 0; j < kGemvPrologueVecs; j++) {
            const int i = tid + j * kGemvThreads;
            if (i < n4) {
#pragma unroll
                for (int e = 0; e < 4; e++) xs[i * 4 + e] = (XT)((xv[j][e] * rs) * wv[j][e]);
            }
        }
    } else if (p.norm_w != nullptr) {
        // k too large for the register path: two passes over global memory
        preload();
        float ss = 0.0f;
        for (int i = tid; i < K; i += kGemvThreads) {
            float v = p.x[i];
            if (p.x_add != nullptr) v = v + p.x_add[i];
            if (writes_sum) p.x_out[i] = v;
            ss = fmaf(v, v, ss);
        }
        ss = block_sum(ss, red);
        const float rs = 1.0f / sqrtf(ss / (float)K + p.eps);
        for (int i = tid; i < K; i += kGemvThreads) {
            float v = p.x[i];
            if (p.x_add != nullptr) v = v + p.x_add[i];
            xs[i] = (XT)((v * rs) * p.norm_w[i]);
        }
    } else {
        for (int base = 0; base < n4; base += kGemvPrologueVecs * kGemvThreads) {
            float4_t xv[kGemvPrologueVecs];
#pragma unroll
            for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = x4[min(base + tid + j * kGemvThreads, n4 - 1)];
            if (a4 != nullptr) {
#pragma unroll
                for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = xv[j] + a4[min(base + tid + j * kGemvThreads, n4 - 1)];
            }
            if (base == 0) {
                __builtin_amdgcn_sched_barrier(0);
                preload();
            }
#pragma unroll
            for (int j = 0; j < kGemvPrologueVecs; j++) {
                const int i = base + tid + j * kGemvThreads;
                if (i < n4) {
                    if (writes_sum) o4[i] = xv[j];
#pragma unroll
                    for (int e = 0; e < 4; e++) xs[i * 4 + e] = (XT)xv[j][e];
                }
            }
        }
    }
    int pos = 0;
    if constexpr (kEpi == kEpiRopeKv) {
        pos = p.state->pos;
        const int half_hd = p.head_dim / 2;
        if (tid < half_hd) rope_f[tid] = p.freqs[(size_t)pos * half_hd + tid];
    }
    __syncthreads();

    // ---- main loop: row units interleaved over all wavefronts of the grid, so that at any moment the
    //      grid reads one dense window of the matrix ----
    const int n_units = p.n_rows / kRows; // n_rows is a multiple of kRows (checked on the host)
    const int W = gridDim.x * kGemvWaves;

    for (int unit = unit_first; unit < n_units; unit += W) {
        const int row0 = unit * kRows;
        float acc[kMats][kRows];
#pragma unroll
        for (int m = 0; m < kMats; m++)
#pragma unroll
            for (int r = 0; r < kRows; r++) acc[m][r] = 0.0f;

        for (int c = 0; c < pieces; c += kU) {
            uint4_t wv[kU][kMats][kRows];
            if (have_pre && c == 0 && unit == unit_first) {
#pragma unroll
                for (int u = 0; u < kU; u++)
#pragma unroll
                    for (int m = 0; m < kMats; m++)
#pragma unroll
                        for (int r = 0; r < kRows; r++) wv[u][m][r] = wpre[u][m][r];
            } else if (c + kU <= pieces_full) {
                // full burst: addresses differ by compile-time offsets
#pragma unroll
                for (int u = 0; u < kU; u++)
#pragma unroll
                    for (int m = 0; m < kMats; m++)
#pragma unroll
                        for (int r = 0; r < kRows; r++)
                            wv[u][m][r] = load16<kStream>(wmat[m] + (size_t)(row0 + r) * K + (size_t)(c + u) * kPiece + lane * kVec);
            } else {
                // tail burst: pieces past the end are skipped, the partial last piece is clamped to valid
                // weights (they meet zeros of the padded x)
#pragma unroll
                for (int u = 0; u < kU; u++) {
                    const int kk = min((c + u) * kPiece + lane * kVec, K - kVec);
#pragma unroll
                    for (int m = 0; m < kMats; m++)
#pragma unroll
                        for (int r = 0; r < kRows; r++) {
                            if (c + u < pieces) wv[u][m][r] = load16<kStream>(wmat[m] + (size_t)(row0 + r) * K + kk);
                            else wv[u][m][r] = uint4_t{0u, 0u, 0u, 0u};
                        }
                }
            }
#pragma unroll
            for (int u = 0; u < kU; u++) {
                if (c + u < pieces) {
                    float xv[kVec];
                    load_x<XT, kVec>(xs + (c + u) * kPiece + lane * kVec, xv);
#pragma unroll
                    for (int m = 0; m < kMats; m++)
#pragma unroll
                        for (int r = 0; r < kRows; r++) {
                            float wf[kVec];
                            WVec<WT>::unpack(wv[u][m][r], wf);
#pragma unroll
                            for (int i = 0; i < kVec; i++) acc[m][r] = fmaf(wf[i], xv[i], acc[m][r]);
                        }
                }
            }
        }

        // ---- reduce (valid in lane 63) and epilogue ----
        float v[kMats][kRows];
#pragma unroll
        for (int m = 0; m < kMats; m++)
#pragma unroll
            for (int r = 0; r < kRows; r++) {
                v[m][r] = wave_sum_lane63(acc[m][r]);
                if (p.round_y) v[m][r] = f16r(v[m][r]); // tensor.rs:1623-1643
            }
        if (lane == 63) {
            if constexpr (kEpi == kEpiStore) {
                p.y[row0] = v[0][0];
            } else if constexpr (kEpi == kEpiSilu) {
                const float g = v[0][0];
                const float u = v[1][0];
                const float sg = g / (1.0f + expf(-g)); // tensor.rs:826-827
                const float mval = sg * u;              // tensor.rs:729
                p.y[row0] = p.x_f16 ? f16r(mval) : mval; // transformer.rs:563-565 (cast to w2's dtype)
            } else { // kEpiRopeKv: rows [0, dim) = wq, [dim, 2 dim) = wk, [2 dim, 3 dim) = wv
                const int which = row0 / p.dim;
                const int jdx = row0 - which * p.dim;
                const int head = jdx / p.head_dim;
                const int jj = jdx - head * p.head_dim;
                float a = v[0][0], b = v[0][kRows - 1];
                if (which < 2) {
                    float ra, rb;
                    rope_pair(a, b, rope_f[jj >> 1], ra, rb);
                    a = ra;
                    b = rb;
                }
                if (which == 0) {
                    *reinterpret_cast<float2 *>(p.y + jdx) = make_float2(a, b);
                } else {
                    void *cache = which == 1 ? p.cache_k : p.cache_v;
                    const size_t idx = ((size_t)head * p.max_seq_len + pos) * p.head_dim + jj;
                    if (p.cache_f16) {
                        half2_t hv;
                        hv[0] = (half_t)a; // Tensor::set_f32 on an f16 cache (tensor.rs:373-376)
                        hv[1] = (half_t)b;
                        *reinterpret_cast<half2_t *>(reinterpret_cast<half_t *>(cache) + idx) = hv;
                    } else {
                        *reinterpret_cast<float2 *>(reinterpret_cast<float *>(cache) + idx) = make_float2(a, b);
                    }
                }
            }
        }
    }
}

template <typename WT, typename XT, int kEpi>
static hipError_t launch_gemv_t(GemvParams p, hipStream_t s) {
    constexpr int rows_per_unit = (kEpi == kEpiRopeKv) ? 2 : 1;
    const int n_units = p.n_rows / rows_per_unit;
    int n_waves = n_units < kGemvTargetWaves ? n_units : kGemvTargetWaves;
    const int blocks = (n_waves + kGemvWaves - 1) / kGemvWaves;
    const size_t lds = (size_t)gemv_iters(p.k, WVec<WT>::kVec) * kWave * WVec<WT>::kVec * sizeof(XT);
    auto launch = [&](auto kern) -> hipError_t {
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGemvThreads), lds, s, p);
        return hipGetLastError();
    };
    if (p.stream_weights) return launch(gemv_kernel<WT, XT, kEpi, true>);
    return launch(gemv_kernel<WT, XT, kEpi, false>);
}

template <int kEpi>
static hipError_t launch_gemv_e(const GemvParams &p, hipStream_t s) {
    if (p.w_is_f16) {
        return p.x_f16 ? launch_gemv_t<half_t, half_t, kEpi>(p, s) : launch_gemv_t<half_t, float, kEpi>(p, s);
    }
    return p.x_f16 ? launch_gemv_t<float, half_t, kEpi>(p, s) : launch_gemv_t<float, float, kEpi>(p, s);
}

hipError_t launch_gemv(const GemvParams &p, int epilogue, hipStream_t s) {
    const int vec = p.w_is_f16 ? 8 : 4;
    if (p.k < vec || p.n_rows <= 0 || (p.k % vec) != 0) return hipErrorInvalidValue;
    switch (epilogue) {
    case kEpiStore: return launch_gemv_e<kEpiStore>(p, s);
    case kEpiSilu: return launch_gemv_e<kEpiSilu>(p, s);
    case kEpiRopeKv:
        if ((p.dim % 2) != 0 || (p.head_dim % 2) != 0 || p.head_dim > 128 || p.n_rows != 3 * p.dim) return hipErrorInvalidValue;
        return launch_gemv_e<kEpiRopeKv>(p, s);
    default: return hipErrorInvalidValue;
    }
}

} // namespace rlh
