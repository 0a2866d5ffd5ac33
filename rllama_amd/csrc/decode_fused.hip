// decode_fused.hip -- the matrix-vector part of one transformer block of a token step as ONE launch (gfx950).
//
// A token step is a chain of dependent matrix-vector products (Noeda/rllama, transformer.rs:424-446, 536-583, 657-820):
// wo -> (residual, ffn_norm) w1|w3 -> w2 -> (residual, attention_norm of the next block) wq|wk|wv, or the output head after
// the last block.  As separate launches every link costs the fixed price of a kernel boundary (about 3 us during which no
// weight byte moves).  Here the four products are phases of one kernel on one resident grid:
//   * between two phases all workgroups meet at a device-wide barrier (two levels of arrival counters, so that no counter
//     sees more than a few dozen atomics);
//   * the weights of a phase do not depend on the activations, so every wavefront requests the first burst(s) of its first
//     row(s) of the NEXT phase before it waits at the barrier;
//   * activation vectors that cross the barrier are written and read at device scope (gemv_device.h), everything else --
//     the weight stream, q and the cache rows for the attention kernel that follows -- as in the stand-alone kernels.
// The arithmetic of every phase is gemv_body, the same code the stand-alone kernels run: results are bit-identical.
//
// MEASURED, AND NOT THE DEFAULT: on the 7B shape the fused launch takes 82 us against 76 us for the four kernels it
// replaces.  Per-workgroup time stamps show why: the phases themselves run at the streaming rate, but the workgroups of a
// phase finish up to 9 us apart (the memory system does not serve them evenly), the barrier completes 1.5 - 4 us after the
// LAST arrival, and what a wavefront requested ahead when IT arrived has long landed by then -- one, two, three or four
// bursts ahead make no difference -- so the memory system idles about as long as across a kernel boundary, and the
// device-scope hand-over of the activation vector costs more than the L2-cached reads of a fresh kernel.  It is kept behind
// RLLAMA_HIP_FUSED=1 as the reference point for that measurement.
//
// Every wait is bounded by the wall clock: a barrier that does not complete within the limit (a workgroup that never became
// resident) raises the error word, every workgroup leaves, and the host reports the failure.
#include "gemv_device.h"

#include <type_traits>

namespace rlh {

constexpr int kFusedLine = 32;  // counters sit on separate 128-byte lines
#ifndef RLH_FUSED_PREFETCH
#define RLH_FUSED_PREFETCH 1
#endif
constexpr int kFusedPrefetch = RLH_FUSED_PREFETCH; // bursts of the next phase every wavefront requests before it waits at a barrier

__device__ __forceinline__ unsigned bar_load(const unsigned *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void bar_store(unsigned *p, unsigned v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Device-wide barrier of the resident grid, driven by thread 0 of every workgroup.  All counters only ever grow (modulo
// 2^32): barrier number n of the barrier's lifetime is complete when gen == n, group counter g has then seen n * members(g)
// arrivals and the top counter n * groups.  A launch learns n from gen before its first arrival.
struct GridBarrier {
    unsigned *cnt, *top, *gen, *err;
    unsigned done;      // barriers complete so far (lifetime count)
    unsigned groups, grp, members;
    long long limit_ticks;

    __device__ void init(FusedBarrierState *b, long long limit) {
        cnt = b->words;
        top = b->words + kFusedGroups * kFusedLine;
        gen = top + kFusedLine;
        err = gen + kFusedLine;
        groups = gridDim.x < (unsigned)kFusedGroups ? gridDim.x : (unsigned)kFusedGroups;
        grp = blockIdx.x % groups;
        members = gridDim.x / groups + (grp < gridDim.x % groups ? 1u : 0u);
        limit_ticks = limit;
        done = bar_load(gen); // no barrier of this launch can complete before every workgroup has arrived, i.e. has read this
    }
    __device__ void arrive() {
        const unsigned n = done + 1;
        const unsigned prev = __hip_atomic_fetch_add(cnt + grp * kFusedLine, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev + 1u == n * members) {
            const unsigned p2 = __hip_atomic_fetch_add(top, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (p2 + 1u == n * groups) bar_store(gen, n);
        }
    }
    // false: timed out or another workgroup did (the error word is set; the caller leaves the kernel)
    __device__ bool wait() {
        const unsigned n = done + 1;
        const long long t0 = wall_clock64();
        while ((int)(bar_load(gen) - n) < 0) {
            if (bar_load(err) != 0u) return false;
            if (wall_clock64() - t0 > limit_ticks) {
                bar_store(err, 1u);
                return false;
            }
        }
        done = n;
        return true;
    }
};

// kLast: what follows w2 -- 0: the next block's wq|wk|wv (RoPE + cache write), 1: the output head with f16 weights,
// 2: the output head with f32 weights.  P.n_phases = 3 leaves it out (a prompt token that is not the last).
template <typename WT, typename XT, int kLast>
__global__ __launch_bounds__(kGemvThreads) void fused_layer_kernel(FusedLayerParams P) {
    extern __shared__ uint4_t smem_raw[];
    __shared__ float red[16];
    __shared__ float2 rope_f[64];
    __shared__ int s_abort;
    const int tid = threadIdx.x;
    GridBarrier bar;
    if (tid == 0) {
        s_abort = 0;
        bar.init(P.barrier, P.limit_ticks);
    }
    uint4_t wpre[kFusedPrefetch][kGemvBurst];
    unsigned have = gemv_issue_bursts<WT, kEpiStore, true, kFusedPrefetch>(P.wo, wpre);
    __syncthreads();

    // End of a phase: this wavefront's activation stores are acknowledged, the workgroup arrives, the next phase's first
    // burst is requested, and only then does the workgroup wait for the others.
    auto hand_over = [&](auto issue_next) -> bool {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) bar.arrive();
        have = issue_next();
        if (tid == 0 && !bar.wait()) s_abort = 1;
        __syncthreads();
        return s_abort == 0;
    };

    // wo (transformer.rs:783-819)
    gemv_body<WT, XT, kEpiStore, true, true, kPreGiven, true, kFusedPrefetch>(P.wo, smem_raw, red, rope_f, wpre, have);
    if (!hand_over([&]() { return gemv_issue_bursts<WT, kEpiSilu, true, kFusedPrefetch>(P.w13, wpre); })) return;
    // h = x + wo(att), ffn_norm, w1|w3, SiLU * gate (transformer.rs:442-443, 537-565)
    gemv_body<WT, XT, kEpiSilu, true, true, kPreGiven, true, kFusedPrefetch>(P.w13, smem_raw, red, rope_f, wpre, have);
    if (!hand_over([&]() { return gemv_issue_bursts<WT, kEpiStore, true, kFusedPrefetch>(P.w2, wpre); })) return;
    // w2 (transformer.rs:568-570)
    gemv_body<WT, XT, kEpiStore, true, true, kPreGiven, true, kFusedPrefetch>(P.w2, smem_raw, red, rope_f, wpre, have);
    if (P.n_phases < 4) return;
    if constexpr (kLast == 0) {
        if (!hand_over([&]() { return gemv_issue_bursts<WT, kEpiRopeKv, true, kFusedPrefetch>(P.last, wpre); })) return;
        // x = h + w2(...), the next block's attention_norm, wq|wk|wv, RoPE, cache write (transformer.rs:445, 432, 665-761)
        gemv_body<WT, XT, kEpiRopeKv, true, true, kPreGiven, true, kFusedPrefetch>(P.last, smem_raw, red, rope_f, wpre, have);
    } else {
        using HT = typename std::conditional<kLast == 1, half_t, float>::type;
        if (!hand_over([&]() { return gemv_issue_bursts<HT, kEpiStore, true, kFusedPrefetch>(P.last, wpre); })) return;
        // x = h + w2(...), final norm, output head on fp32 activations (transformer.rs:445, 378-381)
        gemv_body<HT, float, kEpiStore, true, true, kPreGiven, true, kFusedPrefetch>(P.last, smem_raw, red, rope_f, wpre, have);
    }
}

template <typename WT, typename XT>
static const void *fused_kernel_ptr(int last_kind) {
    switch (last_kind) {
    case 0: return reinterpret_cast<const void *>(fused_layer_kernel<WT, XT, 0>);
    case 1: return reinterpret_cast<const void *>(fused_layer_kernel<WT, XT, 1>);
    default: return reinterpret_cast<const void *>(fused_layer_kernel<WT, XT, 2>);
    }
}

static size_t phase_lds(const GemvParams &g) { return gemv_lds_bytes(g.k, g.w_is_f16, g.x_f16); }

static size_t fused_lds_bytes(const FusedLayerParams &P) {
    size_t lds = phase_lds(P.wo);
    for (const GemvParams *g : {&P.w13, &P.w2, &P.last}) {
        if (g == &P.last && P.n_phases < 4) continue;
        const size_t b = phase_lds(*g);
        lds = b > lds ? b : lds;
    }
    return lds;
}

static int units_of(const GemvParams &g, int rows_per_unit) { return g.n_rows / rows_per_unit; }

// The grid of the fused kernel: enough workgroups for the longest phase, at most kGemvTargetWaves wavefronts, and never more
// than the device holds resident at once (a workgroup that is not resident would never reach the barrier).
hipError_t fused_layer_grid(const FusedLayerParams &P, int compute_units, int *blocks_out) {
    const int f16 = P.wo.w_is_f16;
    const void *kern = f16 ? fused_kernel_ptr<half_t, half_t>(P.last_kind) : fused_kernel_ptr<float, float>(P.last_kind);
    const size_t lds = fused_lds_bytes(P);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    int per_cu = 0;
    hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, kGemvThreads, lds);
    if (e != hipSuccess) return e;
    int units = units_of(P.wo, 1);
    units = units_of(P.w13, 1) > units ? units_of(P.w13, 1) : units;
    units = units_of(P.w2, 1) > units ? units_of(P.w2, 1) : units;
    if (P.n_phases >= 4) {
        const int u = units_of(P.last, P.last_kind == 0 ? 2 : 1);
        units = u > units ? u : units;
    }
    int waves = units < kGemvTargetWaves ? units : kGemvTargetWaves;
    int blocks = (waves + kGemvWaves - 1) / kGemvWaves;
    const long long resident = (long long)per_cu * compute_units;
    if (resident < 1) return hipErrorInvalidConfiguration;
    if (blocks > resident) blocks = (int)resident;
    *blocks_out = blocks < 1 ? 1 : blocks;
    return hipSuccess;
}

hipError_t launch_fused_layer(const FusedLayerParams &P, int blocks, hipStream_t s) {
    const int f16 = P.wo.w_is_f16;
    if (P.w13.w_is_f16 != f16 || P.w2.w_is_f16 != f16 || P.wo.x_f16 != f16 || P.w13.x_f16 != f16 || P.w2.x_f16 != f16) return hipErrorInvalidValue;
    if (P.n_phases != 3 && P.n_phases != 4) return hipErrorInvalidValue;
    if (P.n_phases == 4) {
        if (P.last_kind == 0 && (P.last.w_is_f16 != f16 || P.last.x_f16 != f16 || (P.last.dim % 2) != 0 || (P.last.head_dim % 2) != 0 ||
                                 P.last.head_dim > 128 || P.last.n_rows != 3 * P.last.dim))
            return hipErrorInvalidValue;
        if (P.last_kind != 0 && (P.last.x_f16 != 0 || P.last.w_is_f16 != (P.last_kind == 1))) return hipErrorInvalidValue;
    }
    for (const GemvParams *g : {&P.wo, &P.w13, &P.w2, &P.last}) {
        if (g == &P.last && P.n_phases < 4) continue;
        const int vec = g->w_is_f16 ? 8 : 4;
        if (g->k < vec || g->n_rows <= 0 || (g->k % vec) != 0) return hipErrorInvalidValue;
    }
    if (P.barrier == nullptr || blocks < 1) return hipErrorInvalidValue;
    const size_t lds = fused_lds_bytes(P);
    const void *kern = f16 ? fused_kernel_ptr<half_t, half_t>(P.last_kind) : fused_kernel_ptr<float, float>(P.last_kind);
    FusedLayerParams args = P;
    void *kargs[] = {&args};
    return hipLaunchKernel(kern, dim3(blocks), dim3(kGemvThreads), kargs, lds, s);
}

} // namespace rlh
