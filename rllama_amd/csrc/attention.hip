// attention.hip -- single-query attention over the HBM-resident KV cache (gfx950, wave64).
//
// What it replaces in the reference (Noeda/rllama, transformer.rs:727-781 with seq_len == 1): per head, the
// whole clipped cache is converted to a fresh f32 tensor, scores = q.K / sqrt(hd) (tensor.rs:1923-1983),
// softmax without max subtraction (tensor.rs:479-494), then P.V (tensor.rs:1282-1475).
//
// Here the cache is laid out [head][position][head_dim], so that one position's K (or V) row is contiguous:
// a lane owns 8 consecutive dims, head_dim / 8 lanes make one position, and a wave covers 64 / (head_dim / 8)
// positions per step with 16-byte loads.  K and V rows of a step are loaded together and the next step's
// rows are already in flight while the current ones are consumed.  Every lane group keeps a running
// (max, sum, weighted V) triple (the max-subtracted form equals the reference's exp(s) / sum exp(s)
// wherever that is finite), so the main loop has no block-wide synchronisation; the groups' triples are
// merged once at the end through LDS.  Long sequences are split over several blocks per head
// (grid.y); their partial triples go to a workspace and a small second kernel merges them.
#include "kernels.h"
#include "device_utils.h"

namespace rlh {

constexpr int kAttnThreads = 512;
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
    const int T = p.state->pos + 1;
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

    // this lane group's positions: t0 + (wave + g * kAttnWaves) * kPosPerWave + sub, g = 0, 1, ...
    const int stride = kAttnWaves * kPosPerWave;
    int t = t0 + wave * kPosPerWave + sub;
    float kc[8], vc[8], kn[8], vn[8];
    const int t_safe = t1 > t0 ? t1 - 1 : 0; // address clamp for lanes past the end (their values are discarded)
    load8<CT>(kbase + (size_t)min(t, t_safe) * kHeadDim, kc);
    load8<CT>(vbase + (size_t)min(t, t_safe) * kHeadDim, vc);
    // the loop bound is wave-uniform: the wave's first position decides, lanes past t1 are masked by `valid`
    for (int tw = t0 + wave * kPosPerWave; tw < t1; tw += stride, t += stride) {
        const int tn = t + stride;
        load8<CT>(kbase + (size_t)min(tn, t_safe) * kHeadDim, kn);
        load8<CT>(vbase + (size_t)min(tn, t_safe) * kHeadDim, vn);
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) part = fmaf(qv[i], kc[i], part);
        const float s = group_sum<kLanesPerPos>(part) * scale;
        if (t < t1) {
            const float m_new = fmaxf(m_run, s);
            const float alpha = expf(m_run - m_new);
            const float pe = expf(s - m_new);
            l_run = fmaf(l_run, alpha, pe);
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = fmaf(acc[i], alpha, pe * vc[i]);
            m_run = m_new;
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            kc[i] = kn[i];
            vc[i] = vn[i];
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
    if (tid < kHeadDim) {
        float M = -INFINITY;
        for (int s2 = 0; s2 < kSets; s2++) M = fmaxf(M, pm[s2]);
        float L = 0.0f, O = 0.0f;
        for (int s2 = 0; s2 < kSets; s2++) {
            const float ls = pl[s2];
            const float f = ls > 0.0f ? expf(pm[s2] - M) : 0.0f;
            L = fmaf(ls, f, L);
            O = fmaf(pacc[s2][tid], f, O);
        }
        if (S == 1) {
            const float o = O / L;
            p.out[head * kHeadDim + tid] = p.round_out ? f16r(o) : o; // f16 rounding point before wo (transformer.rs:793-796)
        } else {
            float *ws = p.workspace + ((size_t)head * S + split) * (kHeadDim + 2);
            if (tid == 0) {
                ws[0] = M;
                ws[1] = L;
            }
            ws[2 + tid] = O;
        }
    }
}

// Merges the per-split triples of one head: grid = heads, block = head_dim threads.
__global__ void attn_merge_kernel(const float *workspace, int n_splits, int head_dim, float *out, int round_out) {
    const int head = blockIdx.x;
    const int j = threadIdx.x;
    const float *wh = workspace + (size_t)head * n_splits * (head_dim + 2);
    float M = -INFINITY;
    for (int s = 0; s < n_splits; s++) M = fmaxf(M, wh[(size_t)s * (head_dim + 2)]);
    float L = 0.0f, O = 0.0f;
    for (int s = 0; s < n_splits; s++) {
        const float *w = wh + (size_t)s * (head_dim + 2);
        const float ls = w[1];
        const float f = ls > 0.0f ? expf(w[0] - M) : 0.0f;
        L = fmaf(ls, f, L);
        O = fmaf(w[2 + j], f, O);
    }
    const float o = O / L;
    out[head * head_dim + j] = round_out ? f16r(o) : o;
}

template <typename CT>
static hipError_t launch_attn_t(const AttnDecodeParams &p, hipStream_t s) {
    dim3 grid(p.n_heads, p.n_splits);
    switch (p.head_dim) {
    case 128: hipLaunchKernelGGL((attn_decode_kernel<CT, 128>), grid, dim3(kAttnThreads), 0, s, p); break;
    case 64: hipLaunchKernelGGL((attn_decode_kernel<CT, 64>), grid, dim3(kAttnThreads), 0, s, p); break;
    case 32: hipLaunchKernelGGL((attn_decode_kernel<CT, 32>), grid, dim3(kAttnThreads), 0, s, p); break;
    case 16: hipLaunchKernelGGL((attn_decode_kernel<CT, 16>), grid, dim3(kAttnThreads), 0, s, p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_attn_decode(const AttnDecodeParams &p, hipStream_t s) {
    if (p.n_splits < 1) return hipErrorInvalidValue;
    if (p.n_splits > 1 && p.workspace == nullptr) return hipErrorInvalidValue;
    hipError_t e = p.cache_f16 ? launch_attn_t<half_t>(p, s) : launch_attn_t<float>(p, s);
    if (e != hipSuccess || p.n_splits == 1) return e;
    hipLaunchKernelGGL(attn_merge_kernel, dim3(p.n_heads), dim3(p.head_dim), 0, s, p.workspace, p.n_splits, p.head_dim, p.out, p.round_out);
    return hipGetLastError();
}

} // namespace rlh
