// gemv_device.h -- device code of the batch-1 decode GEMV (gemv.hip has the design notes), shared by the stand-alone
// kernel (gemv.hip) and the fused layer kernel (decode_fused.hip).
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
#ifndef RLH_GEMV_PRELOAD
#define RLH_GEMV_PRELOAD 1
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

// ---- activations that cross workgroups inside one launch --------------------------------------------------------------
// Between kernels the launch boundary makes every store visible.  Inside the fused layer kernel an activation vector is
// written by some workgroups and read by all of them after a device-wide barrier, and the eight L2 caches of the part are
// not coherent with each other for ordinary accesses: such vectors are stored (kDev) and loaded (kDevLoad) at device scope
// -- write-through stores that are in memory once acknowledged, loads that do not take a stale L2 line.  Measured
// alternatives for the reading side: an acquire fence at device scope followed by ordinary loads costs 9 us per barrier
// (it invalidates the L2 under the weight stream); four-byte device-scope loads cost 3 us per phase (512 workgroups
// fetching the same few KB dword by dword from memory); 16-byte ones about 1 us.
// Device-scope 16-byte loads are written as inline assembly (the compiler offers device scope only for scalar types): a
// batch is issued with act_issue4, then act_wait8 waits for everything outstanding and ties the destination registers to the
// wait, so that no use of them can be scheduled in front of it.  The ordinary form is a plain load and no wait.
template <bool kDev>
__device__ __forceinline__ void act_issue4(float4_t &dst, const float4_t *p) {
    if constexpr (kDev) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(dst) : "v"(p) : "memory");
    else dst = *p;
}
template <bool kDev, int kN>
__device__ __forceinline__ void act_wait(float4_t (&v)[kN]) {
    static_assert(kN == 8, "batches of eight");
    if constexpr (kDev)
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7])::"memory");
}
template <bool kDev>
__device__ __forceinline__ float act_load1(const float *p) {
    if constexpr (kDev) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else return *p;
}
template <bool kDev>
__device__ __forceinline__ void act_store4(float4_t *p, float4_t v) {
    if constexpr (kDev) {
        float *q = reinterpret_cast<float *>(p);
        __hip_atomic_store(q, v[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(q + 1, v[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(q + 2, v[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(q + 3, v[3], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        *p = v;
    }
}
template <bool kDev>
__device__ __forceinline__ void act_store1(float *p, float v) {
    if constexpr (kDev) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}

// How the first burst of the first row unit reaches the main loop.
enum GemvPreload {
    kPreNone = 0,   // loaded in the main loop like every other burst
    kPreSelf = 1,   // issued by the prologue right behind its own loads (they stay ahead of it in the in-order return queue),
                    // so that its memory latency runs under the norm / staging work
    kPreGiven = 2   // issued by the caller before this phase began (the fused kernel issues it before the barrier it waits at)
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

// The bursts of a wavefront in the order its main loop takes them: row units unit_first, unit_first + W, ..., and within a
// unit the pieces 0, kU, 2 kU, ...  This issues the loads of the first kD of them into wpre and returns a mask of those it
// issued (bit d: burst d is in wpre[d]); a burst that does not exist or is not a full one (the ragged end of a row) is left
// to the main loop.  The loads do not depend on x.
template <typename WT, int kEpi, bool kStream, int kD, int kBurst = kGemvBurst>
__device__ __forceinline__ unsigned gemv_issue_bursts(const GemvParams &p, uint4_t (&wpre)[kD][kBurst]) {
    using S = GemvShape<WT, kEpi, kBurst>;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int K = p.k;
    const int pieces = gemv_iters(K, S::kVec);
    const int pieces_full = K / S::kPiece;
    const int n_units = p.n_rows / S::kRows;
    const int W = gridDim.x * kGemvWaves;
    const WT *wmat[2] = {reinterpret_cast<const WT *>(p.w), reinterpret_cast<const WT *>(p.w_b)};
    int unit = blockIdx.x * kGemvWaves + wave, c = 0;
    unsigned mask = 0;
    static_for<kD>([&](auto dc) {
        constexpr int d = decltype(dc)::value;
        if (unit < n_units && c + S::kU <= pieces_full) {
            mask |= 1u << d;
#pragma unroll
            for (int u = 0; u < S::kU; u++)
#pragma unroll
                for (int m = 0; m < S::kMats; m++)
#pragma unroll
                    for (int r = 0; r < S::kRows; r++)
                        wpre[d][(u * S::kMats + m) * S::kRows + r] =
                            load16<kStream>(wmat[m] + (size_t)(unit * S::kRows + r) * K + (size_t)(c + u) * S::kPiece + lane * S::kVec);
        }
        c += S::kU;
        if (c >= pieces) {
            c = 0;
            unit += W;
        }
    });
    return mask;
}

// One GEMV over the whole grid: prologue (x staged in LDS), main loop, epilogue.  `smem_raw` is the block's dynamic LDS
// (gemv_lds_bytes); `red` 16 floats and `rope_f` 64 float2 of static LDS.  kDev: x / x_add are read and y / x_out written at
// device scope (see above).  With kPre == kPreGiven, wpre holds the first kD bursts the caller issued and pre_mask says which.
template <typename WT, typename XT, int kEpi, bool kStream, bool kDev, int kPre, bool kDevLoad = false, int kD = 1, int kBurst = kGemvBurst>
__device__ __forceinline__ void gemv_body(const GemvParams &p, uint4_t *smem_raw, float *red, float2 *rope_f, uint4_t (&wpre)[kD][kBurst],
                                          unsigned pre_mask) {
    using S = GemvShape<WT, kEpi, kBurst>;
    constexpr int kVec = S::kVec, kMats = S::kMats, kRows = S::kRows, kU = S::kU, kPiece = S::kPiece;
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
    auto preload = [&]() {
        if constexpr (kPre == kPreSelf) pre_mask = gemv_issue_bursts<WT, kEpi, kStream, kD, kBurst>(p, wpre);
        __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (kPre == kPreNone) pre_mask = 0;

    // The position and this position's (cos, sin) row are requested first, so that their latencies run under the prologue's
    // (behind it they were two dependent loads in front of the main loop: 1.5 us per launch on the 7B shape).
    int pos = 0;
    [[maybe_unused]] float2 rope_early = make_float2(0.0f, 0.0f);
    if constexpr (kEpi == kEpiRopeKv) {
        pos = p.pos1_host > 0 ? p.pos1_host - 1 : p.state->pos;
        const int half_hd = p.head_dim / 2;
        if (tid < half_hd) rope_early = p.freqs[(size_t)pos * half_hd + tid];
    }

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
        static_assert(kGemvPrologueVecs == 8, "act_wait takes batches of eight");
        float4_t xv[kGemvPrologueVecs], av[kGemvPrologueVecs], wv[kGemvPrologueVecs];
#pragma unroll
        for (int j = 0; j < kGemvPrologueVecs; j++) act_issue4<kDevLoad>(xv[j], x4 + min(tid + j * kGemvThreads, n4 - 1));
        if (a4 != nullptr) {
#pragma unroll
            for (int j = 0; j < kGemvPrologueVecs; j++) act_issue4<kDevLoad>(av[j], a4 + min(tid + j * kGemvThreads, n4 - 1));
        }
#pragma unroll
        for (int j = 0; j < kGemvPrologueVecs; j++) wv[j] = w4[min(tid + j * kGemvThreads, n4 - 1)];
        act_wait<kDevLoad>(xv);
        if (a4 != nullptr) {
            act_wait<kDevLoad>(av);
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
                if (writes_sum) act_store4<kDev>(o4 + i, xv[j]);
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
            float v = act_load1<kDevLoad>(p.x + i);
            if (p.x_add != nullptr) v = v + act_load1<kDevLoad>(p.x_add + i);
            if (writes_sum) act_store1<kDev>(p.x_out + i, v);
            ss = fmaf(v, v, ss);
        }
        ss = block_sum(ss, red);
        const float rs = 1.0f / sqrtf(ss / (float)K + p.eps);
        for (int i = tid; i < K; i += kGemvThreads) {
            float v = act_load1<kDevLoad>(p.x + i);
            if (p.x_add != nullptr) v = v + act_load1<kDevLoad>(p.x_add + i);
            xs[i] = (XT)as_f32((v * rs) * p.norm_w[i]);
        }
    } else {
        for (int base = 0; base < n4; base += kGemvPrologueVecs * kGemvThreads) {
            float4_t xv[kGemvPrologueVecs], av[kGemvPrologueVecs];
#pragma unroll
            for (int j = 0; j < kGemvPrologueVecs; j++) act_issue4<kDevLoad>(xv[j], x4 + min(base + tid + j * kGemvThreads, n4 - 1));
            if (a4 != nullptr) {
#pragma unroll
                for (int j = 0; j < kGemvPrologueVecs; j++) act_issue4<kDevLoad>(av[j], a4 + min(base + tid + j * kGemvThreads, n4 - 1));
            }
            act_wait<kDevLoad>(xv);
            if (a4 != nullptr) {
                act_wait<kDevLoad>(av);
#pragma unroll
                for (int j = 0; j < kGemvPrologueVecs; j++) xv[j] = xv[j] + av[j];
            }
            if (base == 0) {
                __builtin_amdgcn_sched_barrier(0);
                preload();
            }
#pragma unroll
            for (int j = 0; j < kGemvPrologueVecs; j++) {
                const int i = base + tid + j * kGemvThreads;
                if (i < n4) {
                    if (writes_sum) act_store4<kDev>(o4 + i, xv[j]);
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

    // ---- main loop: row units interleaved over all wavefronts of the grid, so that at any moment the
    //      grid reads one dense window of the matrix ----
    const int n_units = p.n_rows / kRows; // n_rows is a multiple of kRows (checked on the host)
    const int W = gridDim.x * kGemvWaves;
    float acc[kMats][kRows];
    auto clear_acc = [&]() {
#pragma unroll
        for (int m = 0; m < kMats; m++)
#pragma unroll
            for (int r = 0; r < kRows; r++) acc[m][r] = 0.0f;
    };
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
    auto take_pre = [&](auto dc, uint4_t (&wv)[kU][kMats][kRows]) {
        constexpr int d = decltype(dc)::value;
#pragma unroll
        for (int u = 0; u < kU; u++)
#pragma unroll
            for (int m = 0; m < kMats; m++)
#pragma unroll
                for (int r = 0; r < kRows; r++) wv[u][m][r] = wpre[d][(u * kMats + m) * kRows + r];
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
                act_store1<kDev>(p.y + row0, v[0][0]);
            } else if constexpr (kEpi == kEpiSilu) {
                const float g = v[0][0];
                const float u = v[1][0];
                const float sg = g / (1.0f + expf(-g)); // tensor.rs:826-827
                const float mval = sg * u;              // tensor.rs:729
                act_store1<kDev>(p.y + row0, p.x_f16 ? f16r(mval) : mval); // transformer.rs:563-565 (cast to w2's dtype)
            } else { // kEpiRopeKv: rows [0, dim) = wq, [dim, 2 dim) = wk, [2 dim, 3 dim) = wv
                // q and the cache rows are read by the attention kernel, a later launch: ordinary stores
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

    if constexpr (kPre == kPreGiven) {
        // The wavefront's bursts as one sequence, the first kD of them possibly already in registers (gemv_issue_bursts walks
        // the same sequence).
        int unit = unit_first, c = 0;
        clear_acc();
        auto advance = [&]() {
            c += kU;
            if (c >= pieces) {
                finish(unit);
                clear_acc();
                c = 0;
                unit += W;
            }
        };
        static_for<kD>([&](auto dc) {
            constexpr int d = decltype(dc)::value;
            if (unit < n_units) {
                uint4_t wv[kU][kMats][kRows];
                if (pre_mask & (1u << d)) take_pre(dc, wv);
                else fetch(unit, c, wv);
                mac(c, wv);
                advance();
            }
        });
        while (unit < n_units) {
            uint4_t wv[kU][kMats][kRows];
            fetch(unit, c, wv);
            mac(c, wv);
            advance();
        }
    } else {
        for (int unit = unit_first; unit < n_units; unit += W) {
            clear_acc();
            for (int c = 0; c < pieces; c += kU) {
                uint4_t wv[kU][kMats][kRows];
                if (kPre != kPreNone && (pre_mask & 1u) && c == 0 && unit == unit_first) take_pre(std::integral_constant<int, 0>{}, wv);
                else fetch(unit, c, wv);
                mac(c, wv);
            }
            finish(unit);
        }
    }
}

} // namespace rlh
