// gemv_device.h -- device code of the batch-1 decode GEMV (gemv.hip has the design notes).
#pragma once

#include "kernels.h"
#include "device_utils.h"

#include <type_traits>
#include <utility>

namespace rlh {

// f(integral_constant<int, 0>), f(integral_constant<int, 1>), ...: a loop whose index is a compile-time constant in every
// iteration (register arrays indexed by it stay in registers)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int kN, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(static_cast<F &&>(f), std::make_integer_sequence<int, kN>{});
}

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
constexpr int kGemvBurst = RLH_GEMV_BURST; // 16-byte loads per lane issued back to back before they are consumed
#ifndef RLH_GEMV_PRELOAD_EPIS
#define RLH_GEMV_PRELOAD_EPIS 0x0d // bit per epilogue (kEpiStore, kEpiRopeKv, kEpiSilu): its first burst is issued by the prologue
#endif
#ifndef RLH_GEMV_AHEAD_EPIS
#define RLH_GEMV_AHEAD_EPIS 0x11 // bit per epilogue (kEpiStore, kEpiStoreArgmax): the next row unit's first burst is requested in
                                 // front of the current unit's reduction and epilogue.  Measured per launch: wo of the 7B shape
                                 // 8.0 -> 7.55 us, of the 13B shape 10.7 -> 10.2, the isolated 11008 x 4096 product 16.0 -> 15.6,
                                 // the head 41.3 -> 40.8; w2 unchanged; wq|wk|wv and w1|w3 unchanged at the 7B shape and 0.4 us
                                 // slower at the 13B shape, so they do not do it.
#endif
#ifndef RLH_GEMV_PROLOGUE_VECS
#define RLH_GEMV_PROLOGUE_VECS 8
#endif
constexpr int kGemvPrologueVecs = RLH_GEMV_PROLOGUE_VECS; // float4 loads per thread per prologue batch (one batch covers k <= 1024 * this)

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

// Sum over the wavefront, valid in lane 63 only (no broadcast).
__device__ __forceinline__ float wave_sum_lane63(float v) {
    v = group_sum<16>(v);
    v = dpp_add<kDppRowBcast15, 0xa>(v);
    v = dpp_add<kDppRowBcast31, 0xc>(v);
    return v;
}

// How the first burst of the first row unit reaches the main loop.
enum GemvPreload {
    kPreNone = 0,   // loaded in the main loop like every other burst
    kPreSelf = 1    // issued by the prologue right behind its own loads (they stay ahead of it in the in-order return queue),
                    // so that its memory latency runs under the norm / staging work
};

// kBurst: 16-byte loads per lane and burst.  Rows that divide into whole bursts stream about 1 us faster per product than rows
// whose last burst is a partial one (7B shape, k = 11008 = 21.5 pieces: 18.4 us with bursts of 8 + 8 + 6, 17.3 us with 11 + 11),
// so the launcher picks a burst length that divides the row where one of the instantiated lengths does.
template <typename WT, int kEpi, int kBurst = kGemvBurst>
struct GemvShape {
    static constexpr int kVec = WVec<WT>::kVec;
    static constexpr int kMats = (kEpi == kEpiSilu) ? 2 : 1;    // w1 and w3 share x and the epilogue
    static constexpr int kRows = (kEpi == kEpiRopeKv) ? 2 : 1;  // a RoPE pair (2j, 2j+1) is produced by one wave
    static constexpr int kU = kBurst / (kMats * kRows);         // pieces of one row per burst
    static constexpr int kPiece = kWave * kVec;                  // elements one wave-wide load covers
};

// Issues the loads of a wavefront's first burst (pieces 0 .. kU - 1 of its first row unit) into wpre and returns true, or
// returns false where that burst does not exist or is not a full one (left to the main loop).  The loads do not depend on x.
template <typename WT, int kEpi, bool kStream, int kBurst = kGemvBurst>
__device__ __forceinline__ bool gemv_issue_first_burst(const GemvParams &p, uint4_t (&wpre)[kBurst]) {
    using S = GemvShape<WT, kEpi, kBurst>;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int K = p.k;
    const int pieces_full = K / S::kPiece;
    const int n_units = p.n_rows / S::kRows;
    const WT *wmat[2] = {reinterpret_cast<const WT *>(p.w), reinterpret_cast<const WT *>(p.w_b)};
    const int unit = blockIdx.x * kGemvWaves + wave;
    if (unit >= n_units || S::kU > pieces_full) return false;
#pragma unroll
    for (int u = 0; u < S::kU; u++)
#pragma unroll
        for (int m = 0; m < S::kMats; m++)
#pragma unroll
            for (int r = 0; r < S::kRows; r++)
                wpre[(u * S::kMats + m) * S::kRows + r] =
                    load16<kStream>(wmat[m] + (size_t)(unit * S::kRows + r) * K + (size_t)u * S::kPiece + lane * S::kVec);
    return true;
}

// A running greedy candidate: the largest value seen and the lowest id that holds it, and whether a NaN was seen
// (TokenSampler::sample at top_k = 1, token_sampler.rs:112-147: token 0's value becomes v - v, the rest are untouched).
struct GreedyBest {
    float best;
    int idx;
    int nan;
};
__device__ __forceinline__ void greedy_consider(GreedyBest &g, float v, int i) {
    if (i == 0) v = v - v;
    if (v != v) g.nan = 1;
    if (v > g.best || (g.idx < 0 && v == g.best)) {
        g.best = v;
        g.idx = i;
    }
}
__device__ __forceinline__ void greedy_merge(GreedyBest &g, float ov, int oi, int onan) {
    g.nan |= onan;
    if (oi >= 0 && (g.idx < 0 || ov > g.best || (ov == g.best && oi < g.idx))) {
        g.best = ov;
        g.idx = oi;
    }
}

// One GEMV over the whole grid: prologue (x staged in LDS), main loop, epilogue.  `smem_raw` is the block's dynamic LDS
// (gemv_lds_bytes); `red` 16 floats and `rope_f` 64 float2 of static LDS.
// kEmbed (kEpiRopeKv only): the input row comes from the embedding table (GemvParams::embed_table) instead of p.x.
// kStamp (measurement builds only): every wavefront records the 100 MHz wall clock at five points into p.stamps.
constexpr int kGemvStamps = 5; // entry, x staged, first burst consumed, last burst consumed, exit
template <typename WT, typename XT, int kEpi, bool kStream, int kPre, int kBurst = kGemvBurst, bool kEmbed = false, bool kStamp = false>
__device__ __forceinline__ void gemv_body(const GemvParams &p, uint4_t *smem_raw, float *red, float2 *rope_f) {
    [[maybe_unused]] unsigned long long stamp[kGemvStamps] = {0, 0, 0, 0, 0};
    if constexpr (kStamp) stamp[0] = wall_clock64();
    using S = GemvShape<WT, kEpi, kBurst>;
    constexpr int kVec = S::kVec, kMats = S::kMats, kRows = S::kRows, kU = S::kU, kPiece = S::kPiece;
    constexpr bool kArgmax = kEpi == kEpiStoreArgmax;
    XT *xs = reinterpret_cast<XT *>(smem_raw);

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int K = p.k;
    const int pieces = gemv_iters(K, kVec);      // incl. a partial last piece
    const int pieces_full = K / kPiece;
    const int kpad = pieces * kPiece;

    const WT *wmat[kMats];
    wmat[0] = reinterpret_cast<const WT *>(p.w);
    if constexpr (kMats == 2) wmat[1] = reinterpret_cast<const WT *>(p.w_b);
    const int unit_first = blockIdx.x * kGemvWaves + wave;
    uint4_t wpre[kBurst];
    bool have_pre = false;
    auto preload = [&]() {
        if constexpr (kPre == kPreSelf) have_pre = gemv_issue_first_burst<WT, kEpi, kStream, kBurst>(p, wpre);
        __builtin_amdgcn_sched_barrier(0);
    };

    // The position and this position's (cos, sin) row are requested first, so that their latencies run under the prologue's
    // (behind it they were two dependent loads in front of the main loop: 1.5 us per launch on the 7B shape).
    int pos = 0;
    [[maybe_unused]] float2 rope_early = make_float2(0.0f, 0.0f);
    // Layer 0 of a token step takes its input row from the embedding table (Embedding::get_embedding, embedding.rs:50-52:
    // one table row, widened to f32), named by the token id in the device state: a launch of its own for 16 KB otherwise.
    [[maybe_unused]] const half_t *emb_h = nullptr;
    [[maybe_unused]] const float *emb_f = nullptr;
    if constexpr (kEmbed) {
        static_assert(kEpi == kEpiRopeKv, "the embedding row feeds the first product of a token step");
        const size_t row = (size_t)p.state->token * (size_t)K;
        if (p.embed_f16) emb_h = reinterpret_cast<const half_t *>(p.embed_table) + row;
        else emb_f = reinterpret_cast<const float *>(p.embed_table) + row;
    }
    if constexpr (kEpi == kEpiRopeKv) {
        pos = p.pos1_host > 0 ? p.pos1_host - 1 : p.state->pos;
        const int half_hd = p.head_dim / 2;
        if (tid < half_hd) rope_early = p.freqs[(size_t)pos * half_hd + tid];
    }
    // one prologue batch of the input vector: kGemvPrologueVecs float4 per thread starting at float4 index `base`; the source is
    // chosen once, outside the unrolled loads, so that all loads of the batch are issued back to back
    auto load_batch = [&](int base, int n4, float4_t (&xv)[kGemvPrologueVecs]) {
        const float4_t *x4 = reinterpret_cast<const float4_t *>(p.x);
        if constexpr (kEmbed) {
            if (emb_h != nullptr) {
                typedef __attribute__((ext_vector_type(4))) _Float16 half4_t;
                half4_t hv[kGemvPrologueVecs];
#pragma unroll
                for (int j = 0; j < kGemvPrologueVecs; j++) hv[j] = *reinterpret_cast<const half4_t *>(emb_h + (size_t)min(base + tid + j * kGemvThreads, n4 - 1) * 4);
#pragma unroll
                for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = float4_t{(float)hv[j][0], (float)hv[j][1], (float)hv[j][2], (float)hv[j][3]};
                return;
            }
            if (emb_f != nullptr) x4 = reinterpret_cast<const float4_t *>(emb_f);
        }
#pragma unroll
        for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = x4[min(base + tid + j * kGemvThreads, n4 - 1)];
    };
    auto load_in1 = [&](int i) -> float {
        if constexpr (kEmbed) {
            if (emb_h != nullptr) return (float)emb_h[i];
            if (emb_f != nullptr) return emb_f[i];
        }
        return p.x[i];
    };

    // ---- prologue: x = (x_in [+ x_add]) [RMSNorm] [-> f16], staged in LDS, zero padded to kpad ----
    // All global loads of a batch are issued before any is consumed (one exposed memory latency per batch).
    const bool writes_sum = (p.x_out != nullptr) && blockIdx.x == 0;
    const int n4 = K / 4; // k is a multiple of 4
    const float4_t *a4 = reinterpret_cast<const float4_t *>(p.x_add);
    float4_t *o4 = reinterpret_cast<float4_t *>(p.x_out);
    for (int i = K + tid; i < kpad; i += kGemvThreads) xs[i] = (XT)0.0f;
    if (p.norm_w != nullptr && n4 <= kGemvPrologueVecs * kGemvThreads) {
        // RMSNorm::forward (transformer.rs:476-480): (x * rsqrt(mean(x^2) + eps)) * w, x kept in registers
        const float4_t *w4 = reinterpret_cast<const float4_t *>(p.norm_w);
        float4_t xv[kGemvPrologueVecs], av[kGemvPrologueVecs], wv[kGemvPrologueVecs];
        load_batch(0, n4, xv);
        if (a4 != nullptr) {
#pragma unroll
            for (int j = 0; j < kGemvPrologueVecs; j++) av[j] = a4[min(tid + j * kGemvThreads, n4 - 1)];
        }
#pragma unroll
        for (int j = 0; j < kGemvPrologueVecs; j++) wv[j] = w4[min(tid + j * kGemvThreads, n4 - 1)];
        if (a4 != nullptr) {
#pragma unroll
            for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = xv[j] + av[j]; // transformer.rs:442 / :445
        }
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
                for (int e = 0; e < 4; e++) xs[i * 4 + e] = (XT)as_f32((xv[j][e] * rs) * wv[j][e]);
            }
        }
    } else if (p.norm_w != nullptr) {
        // k too large for the register path: two passes over global memory
        preload();
        float ss = 0.0f;
        for (int i = tid; i < K; i += kGemvThreads) {
            float v = load_in1(i);
            if (p.x_add != nullptr) v = v + p.x_add[i];
            if (writes_sum) p.x_out[i] = v;
            ss = fmaf(v, v, ss);
        }
        ss = block_sum(ss, red);
        const float rs = 1.0f / sqrtf(ss / (float)K + p.eps);
        for (int i = tid; i < K; i += kGemvThreads) {
            float v = load_in1(i);
            if (p.x_add != nullptr) v = v + p.x_add[i];
            xs[i] = (XT)as_f32((v * rs) * p.norm_w[i]);
        }
    } else {
        for (int base = 0; base < n4; base += kGemvPrologueVecs * kGemvThreads) {
            float4_t xv[kGemvPrologueVecs], av[kGemvPrologueVecs];
            load_batch(base, n4, xv);
            if (a4 != nullptr) {
#pragma unroll
                for (int j = 0; j < kGemvPrologueVecs; j++) av[j] = a4[min(base + tid + j * kGemvThreads, n4 - 1)];
#pragma unroll
                for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = xv[j] + av[j];
            }
            if (base + kGemvPrologueVecs * kGemvThreads >= n4) { // behind the loads of the last batch: x stays ahead of it in the return queue
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
    if constexpr (kEpi == kEpiRopeKv) {
        if (tid < p.head_dim / 2) rope_f[tid] = rope_early;
    }
    __syncthreads();
    if constexpr (kStamp) stamp[1] = wall_clock64();

    // ---- main loop: row units interleaved over all wavefronts of the grid, so that at any moment the
    //      grid reads one dense window of the matrix ----
    const int n_units = p.n_rows / kRows; // n_rows is a multiple of kRows (checked on the host)
    const int W = gridDim.x * kGemvWaves;
    float acc[kMats][kRows];
    [[maybe_unused]] GreedyBest gb{-INFINITY, -1, 0}; // kArgmax: this wavefront's candidate (meaningful in lane 63)
    // the loads of the burst that starts at piece c of row unit `unit`
    auto fetch = [&](int unit, int c, uint4_t (&wv)[kU][kMats][kRows]) {
        const int row0 = unit * kRows;
        if (c + kU <= pieces_full) {
            // full burst: addresses differ by compile-time offsets
#pragma unroll
            for (int u = 0; u < kU; u++)
#pragma unroll
                for (int m = 0; m < kMats; m++)
#pragma unroll
                    for (int r = 0; r < kRows; r++)
                        wv[u][m][r] = load16<kStream>(wmat[m] + (size_t)(row0 + r) * K + (size_t)(c + u) * kPiece + lane * kVec);
        } else if (c + kU <= pieces) {
            // the row ends with this burst in a partial piece: every piece exists, lanes past the end of the row are clamped
            // to valid weights (they meet zeros of the padded x)
#pragma unroll
            for (int u = 0; u < kU; u++) {
                const int kk = min((c + u) * kPiece + lane * kVec, K - kVec);
#pragma unroll
                for (int m = 0; m < kMats; m++)
#pragma unroll
                    for (int r = 0; r < kRows; r++) wv[u][m][r] = load16<kStream>(wmat[m] + (size_t)(row0 + r) * K + kk);
            }
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
    };
    // products of one burst against x from LDS
    auto mac = [&](int c, const uint4_t (&wv)[kU][kMats][kRows]) {
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
    };
    // reduce (valid in lane 63) and epilogue of one row unit
    auto finish = [&](int unit) {
        const int row0 = unit * kRows;
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
            } else if constexpr (kArgmax) {
                // the logits also go to memory; stored at device scope, because the workgroup that draws the last ticket may
                // read them back in this same launch (see the end of this function)
                __hip_atomic_store(p.y + row0, v[0][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                greedy_consider(gb, v[0][0], row0); // a wavefront's rows ascend, so equal values keep the lowest id
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
    };

    // (Measured and not kept: a wavefront requesting the first burst of its last row unit together with the last burst of the
    // unit before, so that the partial last round of units -- 768 of 2048 wavefronts on the 7B shape's 11008 rows -- costs no
    // memory latency of its own: the isolated 11008 x 4096 product 16.45 -> 17.25 us, w1|w3 30.1 -> 30.6 us, and with the code
    // in place but switched off w2 17.1 -> 17.7 us.)
    // The burst the prologue requested (pieces 0 .. kU - 1 of the first row unit) is consumed at the head of that unit.  With
    // kAhead the first burst of the *next* unit is requested before the reduction and epilogue of the current one run, so
    // that those run under its memory latency.
    constexpr bool kAhead = !kStamp && ((RLH_GEMV_AHEAD_EPIS >> kEpi) & 1);
    const bool burst0_full = kU <= pieces_full;
    bool have = false;
    if constexpr (kPre != kPreNone) have = have_pre;
    for (int unit = unit_first; unit < n_units; unit += W) {
#pragma unroll
        for (int m = 0; m < kMats; m++)
#pragma unroll
            for (int r = 0; r < kRows; r++) acc[m][r] = 0.0f;
        int c_first = 0;
        if constexpr (kPre != kPreNone || kAhead) {
            if (have) {
                uint4_t wv[kU][kMats][kRows];
#pragma unroll
                for (int u = 0; u < kU; u++)
#pragma unroll
                    for (int m = 0; m < kMats; m++)
#pragma unroll
                        for (int r = 0; r < kRows; r++) wv[u][m][r] = wpre[(u * kMats + m) * kRows + r];
                mac(0, wv);
                c_first = kU;
                have = false;
            }
        }
        for (int c = c_first; c < pieces; c += kU) {
            uint4_t wv[kU][kMats][kRows];
            fetch(unit, c, wv);
            mac(c, wv);
            if constexpr (kStamp) {
                // (the products depend on the loaded data, and the clock is read behind them)
                asm volatile("" : "+v"(acc[0][0]));
                const unsigned long long now = wall_clock64();
                if (stamp[2] == 0) stamp[2] = now;
                stamp[3] = now;
            }
        }
        if constexpr (kAhead) {
            const int next = unit + W;
            if (next < n_units && burst0_full) {
#pragma unroll
                for (int u = 0; u < kU; u++)
#pragma unroll
                    for (int m = 0; m < kMats; m++)
#pragma unroll
                        for (int r = 0; r < kRows; r++)
                            wpre[(u * kMats + m) * kRows + r] =
                                load16<kStream>(wmat[m] + (size_t)(next * kRows + r) * K + (size_t)u * kPiece + lane * kVec);
                have = true;
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        finish(unit);
    }
    if constexpr (kStamp) {
        stamp[4] = wall_clock64();
        if ((threadIdx.x & (kWave - 1)) == 0 && p.stamps != nullptr) {
            unsigned long long *dst = p.stamps + ((size_t)blockIdx.x * kGemvWaves + threadIdx.x / kWave) * kGemvStamps;
#pragma unroll
            for (int i = 0; i < kGemvStamps; i++) dst[i] = stamp[i];
        }
    }

    if constexpr (kArgmax) {
        // ---- the greedy pick over all rows (TokenSampler::sample at top_k = 1, token_sampler.rs:99-147, as
        //      argmax_advance_kernel runs it at temperature 1) without a launch of its own ----
        // Every workgroup reduces its wavefronts' candidates and publishes one (value, id, NaN seen) record; the workgroup
        // that draws the last ticket reduces the records and advances the token-step state.  The hand-over uses device-scope
        // (write-through) stores that are waited for before the ticket is drawn, and device-scope loads after it.  That a
        // store acknowledged to the wavefront (vmcnt) is visible to a later device-scope load from another compute unit is a
        // property of this part (gfx950: device-scope stores write through the XCD's L2 to memory, device-scope loads miss
        // it), not a guarantee of the HIP memory model for relaxed atomics; rlh_init refuses every other architecture.
        __shared__ float am_val[kGemvWaves];
        __shared__ int am_idx[kGemvWaves];
        __shared__ int am_nan[kGemvWaves];
        __shared__ int am_last;
        if (lane == 63) {
            am_val[wave] = gb.best;
            am_idx[wave] = gb.idx;
            am_nan[wave] = gb.nan;
        }
        __syncthreads();
        if (tid == 0) {
            GreedyBest b{am_val[0], am_idx[0], am_nan[0]};
#pragma unroll
            for (int w = 1; w < kGemvWaves; w++) greedy_merge(b, am_val[w], am_idx[w], am_nan[w]);
            float *rec = p.amax_ws + (size_t)blockIdx.x * 4;
            __hip_atomic_store(rec + 0, b.best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(reinterpret_cast<int *>(rec) + 1, b.idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(reinterpret_cast<int *>(rec) + 2, b.nan, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // every store of this workgroup (its logits and its record) has been acknowledged before its ticket is drawn
        asm volatile("" ::: "memory");
        wait_vmcnt<0>();
        asm volatile("" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const unsigned prev = __hip_atomic_fetch_add(p.amax_ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int last = prev == gridDim.x - 1;
            if (last) __hip_atomic_store(p.amax_ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // ready for the next launch
            am_last = last;
        }
        __syncthreads();
        if (!am_last) return;
        GreedyBest b{-INFINITY, -1, 0};
        for (int blk = tid; blk < (int)gridDim.x; blk += kGemvThreads) { // ascending ids per thread: ties keep the lowest id
            const float *rec = p.amax_ws + (size_t)blk * 4;
            const float ov = __hip_atomic_load(rec + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int oi = __hip_atomic_load(reinterpret_cast<const int *>(rec) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int on = __hip_atomic_load(reinterpret_cast<const int *>(rec) + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            greedy_merge(b, ov, oi, on);
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(b.best, off, kWave);
            const int oi = __shfl_xor(b.idx, off, kWave);
            const int on = __shfl_xor(b.nan, off, kWave);
            greedy_merge(b, ov, oi, on);
        }
        __syncthreads(); // am_* are about to be reused
        if (lane == 0) {
            am_val[wave] = b.best;
            am_idx[wave] = b.idx;
            am_nan[wave] = b.nan;
        }
        __syncthreads();
#pragma unroll
        for (int w = 0; w < kGemvWaves; w++) greedy_merge(b, am_val[w], am_idx[w], am_nan[w]); // every thread ends with the grid's pick
        // Can sum(exp(l)) overflow f32?  Only if vocab * exp(largest) can: largest > ln(FLT_MAX) - ln(vocab).  Then (rare) the
        // sum decides, formed in double over the stored logits like argmax_advance_kernel does.
        const float kLnFltMax = 88.72283172607422f;
        const bool sum_at_risk = !b.nan && b.best <= kLnFltMax && b.best > kLnFltMax - logf((float)p.n_rows);
        double total = 0.0;
        if (sum_at_risk) { // uniform over the workgroup
            __shared__ double am_sum[kGemvWaves];
            double part = 0.0;
            for (int i = tid; i < p.n_rows; i += kGemvThreads) {
                const float v = i == 0 ? 0.0f : __hip_atomic_load(p.y + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                part += exp((double)v);
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) part += __shfl_xor(part, off, kWave);
            if (lane == 0) am_sum[wave] = part;
            __syncthreads();
#pragma unroll
            for (int w = 0; w < kGemvWaves; w++) total += am_sum[w];
        }
        if (tid == 0) {
            int pick = b.idx < 0 ? 0 : b.idx;                                                   // every logit NaN
            if (b.nan || b.best > kLnFltMax || total > 3.4028234663852886e38) pick = 0;        // sum not finite: every probability 0 or NaN
            DecodeState *st = p.state_rw;
            st->token = pick;
            st->pos = st->pos + 1;
            const int k = st->n_out;
            if (p.out_tokens != nullptr && k < p.out_cap) p.out_tokens[k] = pick;
            st->n_out = k + 1;
        }
    }
}

} // namespace rlh
