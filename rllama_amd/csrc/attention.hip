// attention.hip -- single-query attention over the HBM-resident KV cache (gfx950, wave64).
//
// What it replaces in the reference (Noeda/rllama, transformer.rs:727-781 with seq_len == 1): per head, the
// whole clipped cache is converted to a fresh f32 tensor, scores = q.K / sqrt(hd) (tensor.rs:1923-1983),
// softmax without max subtraction (tensor.rs:479-494), then P.V (tensor.rs:1282-1475).
//
// Here the cache is laid out [head][position][head_dim], so that one position's K (or V) row is contiguous:
// a lane owns 8 consecutive dims, head_dim / 8 lanes make one position, and a wave covers 64 / (head_dim / 8)
// positions per step with 16-byte loads.  K and V rows of several steps are loaded together before any is
// consumed (independent loads in flight hide the memory latency; a single query leaves nothing to reuse).  Every lane group keeps a running
// (max, sum, weighted V) triple (the max-subtracted form equals the reference's exp(s) / sum exp(s)
// wherever that is finite), so the main loop has no block-wide synchronisation; the groups' triples are
// merged once at the end through LDS.  A sequence is split over several blocks per head (grid.y); every block
// publishes its partial triple to a workspace and takes a ticket, and the block that draws the last ticket of its
// head merges the partial triples (in split order, so the result does not depend on which block that was).
#include "kernels.h"
#include "device_utils.h"

namespace rlh {

constexpr int kAttnMaxSplits = 64;

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

// 8 consecutive cache elements of one lane: one 16-byte word (f16) or two (f32)
template <typename CT>
__device__ __forceinline__ void unpack8(const uint4_t *raw, float (&out)[8]) {
    if constexpr (sizeof(CT) == 2) {
        half8_t h = __builtin_bit_cast(half8_t, raw[0]);
#pragma unroll
        for (int i = 0; i < 8; i++) out[i] = (float)h[i];
    } else {
        float4_t a = __builtin_bit_cast(float4_t, raw[0]);
        float4_t b = __builtin_bit_cast(float4_t, raw[1]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            out[i] = a[i];
            out[i + 4] = b[i];
        }
    }
}

// How the partial triples of a split sequence travel from the blocks that make them to the block that merges them.
enum AttnMergeMode {
    kMergeSeparate = 0, // a second kernel merges (attn_merge_kernel)
    kMergeThrough = 2   // last block of a head merges; the partials are stored and loaded at device scope (write-through /
                        // cache-bypassing accesses), the stores only waited for before the ticket.  (Release / acquire fences
                        // at device scope around the ticket instead were measured at 48 - 146 us for the same launch: each
                        // fence writes back or invalidates a whole L2 under the stream.)
};

template <int kMode>
__device__ __forceinline__ void publish(float *dst, float v) {
    if constexpr (kMode == kMergeThrough) __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *dst = v;
}
template <int kMode>
__device__ __forceinline__ float collect(const float *src) {
    if constexpr (kMode == kMergeThrough) return __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else return *src;
}

// kThreads threads per block, kBatch cache rows of K and of V loaded together per lane before any is consumed.
// kLds: the block's K and V rows are first moved into LDS as whole tiles (direct global -> LDS loads) and consumed from
// there; otherwise they go from memory straight into registers.
template <typename CT, int kHeadDim, int kThreads, int kBatch, int kMode, bool kLds = false>
__global__ __launch_bounds__(kThreads) void attn_decode_kernel(AttnDecodeParams p) {
    constexpr int kAttnThreads = kThreads;
    constexpr int kAttnWaves = kThreads / kWave;
    constexpr int kAttnBatch = kBatch;
    constexpr int kRawPerRow = sizeof(CT) == 2 ? 1 : 2;
    constexpr int kLanesPerPos = kHeadDim / 8;        // each lane owns 8 consecutive dims
    constexpr int kPosPerWave = kWave / kLanesPerPos; // positions per wave step
    constexpr int kSets = kAttnWaves * kPosPerWave;   // lane groups in the block, one partial triple each
    static_assert(kLanesPerPos >= 1 && kLanesPerPos <= 16 && (kLanesPerPos & (kLanesPerPos - 1)) == 0, "head_dim in {8,...,128}, power of two");
    __shared__ float pm[kSets];
    __shared__ float pl[kSets];
    __shared__ float pacc[kSets][kHeadDim];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int head = blockIdx.x;
    const int split = blockIdx.y;
    const int S = gridDim.y;
    const int T = (p.pos_host >= 0 ? p.pos_host : p.state->pos) + 1;
    int chunk = (T + S - 1) / S;
    chunk = (chunk + 15) & ~15;
    const int t0 = split * chunk;
    const int t1 = min(T, t0 + chunk);
    const int sub = lane / kLanesPerPos;
    const int dl = lane % kLanesPerPos;
    const float scale = 1.0f / sqrtf((float)kHeadDim); // transformer.rs:770

    const CT *kbase = reinterpret_cast<const CT *>(p.cache_k) + (size_t)head * p.max_seq_len * kHeadDim + dl * 8;
    const CT *vbase = reinterpret_cast<const CT *>(p.cache_v) + (size_t)head * p.max_seq_len * kHeadDim + dl * 8;

    float qv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) qv[i] = p.q[head * kHeadDim + dl * 8 + i];

    float m_run = -INFINITY, l_run = 0.0f;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = 0.0f;

    // LDS-staged form (f16 caches): the block's rows [t0, t1) of K and of V are contiguous in memory; every wavefront moves
    // 1 KiB pieces of them (each lane names its own 16 bytes, clamped to the last valid row) and the block waits once.
    extern __shared__ uint4_t lds_kv[];
    const int rows_cap = chunk;                                      // the launcher sized the LDS for this many rows
    const uint4_t *lds_k = lds_kv;
    const uint4_t *lds_v = lds_kv + (size_t)rows_cap * kLanesPerPos; // 16-byte words per row = kLanesPerPos
    if constexpr (kLds) {
        static_assert(!kLds || sizeof(CT) == 2, "LDS staging is built for f16 caches");
        const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)lds_kv;
        const int rows = t1 > t0 ? t1 - t0 : 0;
        const int words = rows * kLanesPerPos;           // 16-byte words of one tile
        const int pieces = (words + kWave - 1) / kWave;  // 1 KiB pieces
        const half_t *ksrc = reinterpret_cast<const half_t *>(p.cache_k) + ((size_t)head * p.max_seq_len + t0) * kHeadDim;
        const half_t *vsrc = reinterpret_cast<const half_t *>(p.cache_v) + ((size_t)head * p.max_seq_len + t0) * kHeadDim;
        const int wv = __builtin_amdgcn_readfirstlane(wave);
        for (int pc = wv; pc < pieces; pc += kAttnWaves) {
            const int w = min(pc * kWave + lane, words - 1);
            dma16(ksrc + (size_t)w * 8, lds_base + (unsigned)pc * 1024u);
            dma16(vsrc + (size_t)w * 8, lds_base + (unsigned)(rows_cap * kLanesPerPos * 16) + (unsigned)pc * 1024u);
        }
        wait_vmcnt<0>();
        __syncthreads();
    }

    // this lane group's positions: t0 + (wave + g * kAttnWaves) * kPosPerWave + sub, g = 0, 1, ...
    // kAttnBatch steps are loaded together (2 * kAttnBatch independent 16-byte loads in flight per lane)
    const int stride = kAttnWaves * kPosPerWave;
    const int t_safe = t1 > t0 ? t1 - 1 : 0; // address clamp for lanes past the end (their values are discarded)
    int t = t0 + wave * kPosPerWave + sub;
    // the loop bound is wave-uniform: the wave's first position decides, lanes past t1 are masked
    for (int tw = t0 + wave * kPosPerWave; tw < t1; tw += stride * kAttnBatch, t += stride * kAttnBatch) {
        uint4_t kraw[kAttnBatch][kRawPerRow], vraw[kAttnBatch][kRawPerRow];
#pragma unroll
        for (int u = 0; u < kAttnBatch; u++) {
            const size_t off = (size_t)min(t + u * stride, t_safe) * kHeadDim;
#pragma unroll
            for (int w = 0; w < kRawPerRow; w++) {
                if constexpr (kLds) {
                    const int r = min(t + u * stride, t_safe) - t0;
                    kraw[u][w] = lds_k[r * kLanesPerPos + dl];
                    vraw[u][w] = lds_v[r * kLanesPerPos + dl];
                } else if (kAttnBatch == 8 && !(t + u * stride < t1)) {
                    // The single batch of 8 steps (129 .. 256 positions per block): positions past the end request nothing.
                    // One workgroup per head is bound by what its compute unit can take in, and a clamped load costs as
                    // much of that as a real one: 4.77 -> 4.41 us at 136 positions of the 7B shape, 4.85 -> 4.55 at 160.
                    // (In the looping forms the same test cost 0.1 - 0.3 us per launch, so they keep the clamped loads.)
                    kraw[u][w] = uint4_t{0u, 0u, 0u, 0u};
                    vraw[u][w] = uint4_t{0u, 0u, 0u, 0u};
                } else {
                    kraw[u][w] = *reinterpret_cast<const uint4_t *>(reinterpret_cast<const char *>(kbase + off) + 16 * w);
                    vraw[u][w] = *reinterpret_cast<const uint4_t *>(reinterpret_cast<const char *>(vbase + off) + 16 * w);
                }
            }
        }
        // the scores of the batch first (independent of each other), then one new maximum and one rescale for the batch:
        // one exponential per position and one per batch instead of two per position in a serial chain
        float sc[kAttnBatch];
        float m_new = m_run;
#pragma unroll
        for (int u = 0; u < kAttnBatch; u++) {
            float kc[8];
            unpack8<CT>(kraw[u], kc);
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) part = fmaf(qv[i], kc[i], part);
            sc[u] = t + u * stride < t1 ? group_sum<kLanesPerPos>(part) * scale : -INFINITY;
            m_new = fmaxf(m_new, sc[u]);
        }
        if (m_new > -INFINITY) { // some position of the batch belongs to this lane group (or earlier ones did)
            const float alpha = expf(m_run - m_new); // first batch: exp(-inf) = 0
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] *= alpha;
#pragma unroll
            for (int u = 0; u < kAttnBatch; u++) {
                float vc[8];
                unpack8<CT>(vraw[u], vc);
                const float pe = expf(sc[u] - m_new); // positions past the end: exp(-inf) = 0
                l_run += pe;
#pragma unroll
                for (int i = 0; i < 8; i++) acc[i] = fmaf(pe, vc[i], acc[i]);
            }
            m_run = m_new;
        }
    }

    // ---- merge the lane groups of this block ----
    const int set = wave * kPosPerWave + sub;
    if (dl == 0) {
        pm[set] = m_run;
        pl[set] = l_run;
    }
#pragma unroll
    for (int i = 0; i < 8; i++) pacc[set][dl * 8 + i] = acc[i];
    __syncthreads();
    // one weight exp(m_s - M) per lane group, computed once (not once per output dim) and left in pm
    static_assert(kSets <= kAttnThreads, "one thread per lane group");
    float M = -INFINITY;
    for (int s2 = 0; s2 < kSets; s2++) M = fmaxf(M, pm[s2]);
    float f = 0.0f;
    if (tid < kSets) f = pl[tid] > 0.0f ? expf(pm[tid] - M) : 0.0f;
    __syncthreads(); // everybody has read the maxima
    if (tid < kSets) pm[tid] = f;
    __syncthreads();
    if (tid < kHeadDim) {
        float L = 0.0f, O = 0.0f;
#pragma unroll 8
        for (int s2 = 0; s2 < kSets; s2++) {
            const float f2 = pm[s2];
            L = fmaf(pl[s2], f2, L);
            O = fmaf(pacc[s2][tid], f2, O);
        }
        if (S == 1) {
            const float o = O / L;
            p.out[head * kHeadDim + tid] = p.round_out ? f16r(o) : o; // f16 rounding point before wo (transformer.rs:793-796)
        } else {
            float *ws = p.workspace + ((size_t)head * S + split) * (kHeadDim + 2);
            if (tid == 0) {
                publish<kMode>(ws + 0, M);
                publish<kMode>(ws + 1, L);
            }
            publish<kMode>(ws + 2 + tid, O);
        }
    }
    if constexpr (kMode != kMergeSeparate) {
        if (S == 1) return;
        // ---- the block that draws the last ticket of this head merges the head's partial triples ----
        __shared__ int is_last;
        // The write-through stores have left the wavefront and been acknowledged (vmcnt) before the block's ticket is drawn, and
        // the merging block reads them with device-scope loads after it.  That an acknowledged device-scope store is visible to
        // a later device-scope load from another compute unit is a property of this part (gfx950: such stores write through the
        // XCD's L2 to memory, such loads miss it), not a guarantee of the HIP memory model for relaxed atomics -- there is no
        // release / acquire edge between the blocks.  rlh_init refuses every other architecture.
        asm volatile("" ::: "memory");
        wait_vmcnt<0>();
        asm volatile("" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const unsigned prev = __hip_atomic_fetch_add(p.tickets + head, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int last = prev == (unsigned)(S - 1);
            if (last) __hip_atomic_store(p.tickets + head, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // ready for the next launch
            is_last = last;
        }
        __syncthreads();
        if (!is_last) return;
        // Every wavefront forms the splits' weights for itself (lane s holds split s), and the first partial outputs are
        // requested before those weights are needed: one memory latency for the whole merge, no exchange through LDS.
        const float *wh = p.workspace + (size_t)head * S * (kHeadDim + 2);
        float ms = -INFINITY, ls = 0.0f;
        if (lane < S) {
            ms = collect<kMode>(wh + (size_t)lane * (kHeadDim + 2));
            ls = collect<kMode>(wh + (size_t)lane * (kHeadDim + 2) + 1);
        }
        constexpr int kMergeBatch = 8;
        const int col = tid < kHeadDim ? tid : 0; // threads beyond head_dim compute along and store nothing
        float ob[kMergeBatch];
#pragma unroll
        for (int u = 0; u < kMergeBatch; u++) ob[u] = u < S ? collect<kMode>(wh + (size_t)u * (kHeadDim + 2) + 2 + col) : 0.0f;
        const float Mh = wave_max(ms);
        const float fh = ls > 0.0f ? expf(ms - Mh) : 0.0f;
        const float Lh = wave_sum(ls * fh);
        float O = 0.0f;
        for (int s0 = 0; s0 < S; s0 += kMergeBatch) {
            float cur[kMergeBatch];
#pragma unroll
            for (int u = 0; u < kMergeBatch; u++) cur[u] = ob[u];
            if (s0 + kMergeBatch < S) {
#pragma unroll
                for (int u = 0; u < kMergeBatch; u++) {
                    const int s2 = s0 + kMergeBatch + u;
                    ob[u] = s2 < S ? collect<kMode>(wh + (size_t)s2 * (kHeadDim + 2) + 2 + col) : 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < kMergeBatch; u++) {
                const int s2 = s0 + u; // in split order: the sum does not depend on which block merges
                if (s2 < S) O = fmaf(cur[u], __shfl(fh, s2, kWave), O);
            }
        }
        if (tid < kHeadDim) {
            const float o = O / Lh;
            p.out[head * kHeadDim + tid] = p.round_out ? f16r(o) : o;
        }
    }
}

// Merges the per-split triples of one head as a kernel of its own (kMergeSeparate): grid = heads, block = max(head_dim, 64)
// threads.  The first wavefront turns the (max, sum) pairs into one weight per split (one load per lane, wave
// reductions); then thread j sums the weighted partial outputs of dim j with independent loads.  The in-kernel merge above
// does the same arithmetic in the same order.
__global__ void attn_merge_kernel(const float *workspace, int n_splits, int head_dim, float *out, int round_out) {
    __shared__ float wgt[kAttnMaxSplits];
    __shared__ float l_total;
    const int head = blockIdx.x;
    const int tid = threadIdx.x;
    const float *wh = workspace + (size_t)head * n_splits * (head_dim + 2);
    if (tid < kWave) {
        float ms = -INFINITY, ls = 0.0f;
        if (tid < n_splits) {
            ms = wh[(size_t)tid * (head_dim + 2)];
            ls = wh[(size_t)tid * (head_dim + 2) + 1];
        }
        const float M = wave_max(ms);
        const float f = ls > 0.0f ? expf(ms - M) : 0.0f;
        const float L = wave_sum(ls * f);
        if (tid < n_splits) wgt[tid] = f;
        if (tid == 0) l_total = L;
    }
    __syncthreads();
    if (tid < head_dim) {
        float O = 0.0f;
        int s = 0;
        for (; s + 4 <= n_splits; s += 4) {
            const float o0 = wh[(size_t)(s + 0) * (head_dim + 2) + 2 + tid];
            const float o1 = wh[(size_t)(s + 1) * (head_dim + 2) + 2 + tid];
            const float o2 = wh[(size_t)(s + 2) * (head_dim + 2) + 2 + tid];
            const float o3 = wh[(size_t)(s + 3) * (head_dim + 2) + 2 + tid];
            O = fmaf(o0, wgt[s], O);
            O = fmaf(o1, wgt[s + 1], O);
            O = fmaf(o2, wgt[s + 2], O);
            O = fmaf(o3, wgt[s + 3], O);
        }
        for (; s < n_splits; s++) O = fmaf(wh[(size_t)s * (head_dim + 2) + 2 + tid], wgt[s], O);
        const float o = O / l_total;
        out[head * head_dim + tid] = round_out ? f16r(o) : o;
    }
}

template <typename CT, int kThreads, int kBatch, int kMode>
static hipError_t launch_attn_t(const AttnDecodeParams &p, hipStream_t s) {
    dim3 grid(p.n_heads, p.n_splits);
    switch (p.head_dim) {
    case 128: hipLaunchKernelGGL((attn_decode_kernel<CT, 128, kThreads, kBatch, kMode>), grid, dim3(kThreads), 0, s, p); break;
    case 64: hipLaunchKernelGGL((attn_decode_kernel<CT, 64, kThreads, kBatch, kMode>), grid, dim3(kThreads), 0, s, p); break;
    case 32: hipLaunchKernelGGL((attn_decode_kernel<CT, 32, kThreads, kBatch, kMode>), grid, dim3(kThreads), 0, s, p); break;
    case 16: hipLaunchKernelGGL((attn_decode_kernel<CT, 16, kThreads, kBatch, kMode>), grid, dim3(kThreads), 0, s, p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// LDS-staged variant (kept for comparison): f16 cache, head_dim 64 / 128, write-through merge
static hipError_t launch_attn_lds(const AttnDecodeParams &p, hipStream_t s) {
    const int chunk = p.chunk_hint;
    const size_t lds = (size_t)2 * chunk * p.head_dim * 2;
    dim3 grid(p.n_heads, p.n_splits);
    auto go = [&](auto kern) -> hipError_t {
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, s, p);
        return hipGetLastError();
    };
    if (p.head_dim == 128) return go(attn_decode_kernel<half_t, 128, 512, 4, kMergeThrough, true>);
    return go(attn_decode_kernel<half_t, 64, 512, 4, kMergeThrough, true>);
}

template <typename CT, int kMode>
static hipError_t launch_attn_m(const AttnDecodeParams &p, hipStream_t s) {
    // Block shape by the positions a block covers (an upper bound from the host's view of the sequence length): 512 threads
    // cover 64 * 512 / head_dim positions per step of the loop, and the rows of kBatch steps are in flight together, so up to
    // 8 steps run as one batch (one exposed memory latency); longer chunks loop with batches of 4 (a single batch of 12 steps
    // for chunks of 257 .. 384 positions measured slower than three batches of 4: 6.3 against 5.95 us at 384 positions of the
    // 7B shape).
    const int chunk = p.chunk_hint > 0 ? p.chunk_hint : p.max_seq_len;
    const int per_step = 8 * 512 / p.head_dim;
    if (chunk <= 2 * per_step) return launch_attn_t<CT, 512, 2, kMode>(p, s);
    if (chunk > 4 * per_step && chunk <= 8 * per_step) return launch_attn_t<CT, 512, 8, kMode>(p, s);
    return launch_attn_t<CT, 512, 4, kMode>(p, s);
}

hipError_t launch_attn_decode(const AttnDecodeParams &p, hipStream_t s) {
    if (p.n_splits < 1 || p.n_splits > kAttnMaxSplits) return hipErrorInvalidValue;
    if (p.n_splits > 1 && p.workspace == nullptr) return hipErrorInvalidValue;
    if (p.n_splits > 1 && p.merge_mode != kMergeSeparate && p.tickets == nullptr) return hipErrorInvalidValue;
    if (p.lds_stage) {
        // needs the exact chunk the kernel will compute (host position known), an f16 cache and room in LDS
        if (p.pos_host < 0 || !p.cache_f16 || (p.head_dim != 128 && p.head_dim != 64) || p.merge_mode != kMergeThrough ||
            (size_t)2 * p.chunk_hint * p.head_dim * 2 > 128 * 1024)
            return hipErrorInvalidValue;
        return launch_attn_lds(p, s);
    }
    hipError_t e;
    switch (p.merge_mode) {
    case kMergeSeparate: e = p.cache_f16 ? launch_attn_m<half_t, kMergeSeparate>(p, s) : launch_attn_m<float, kMergeSeparate>(p, s); break;
    case kMergeThrough: e = p.cache_f16 ? launch_attn_m<half_t, kMergeThrough>(p, s) : launch_attn_m<float, kMergeThrough>(p, s); break;
    default: return hipErrorInvalidValue;
    }
    if (e != hipSuccess || p.n_splits == 1 || p.merge_mode != kMergeSeparate) return e;
    hipLaunchKernelGGL(attn_merge_kernel, dim3(p.n_heads), dim3(p.head_dim < kWave ? kWave : p.head_dim), 0, s, p.workspace, p.n_splits, p.head_dim, p.out,
                       p.round_out);
    return hipGetLastError();
}

size_t attn_decode_workspace_floats(int n_heads, int head_dim, int n_splits) { return (size_t)n_heads * n_splits * (head_dim + 2); }

} // namespace rlh
