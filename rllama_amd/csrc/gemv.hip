// gemv.hip -- batch-1 decode GEMV for gfx950 (CDNA4, wave64): y = W x with W [n_rows x k] row-major in HBM.
//
// One token step reads every weight byte exactly once, so this kernel is bound by HBM bandwidth and is
// built as a streaming reader:
//   * a wavefront produces one output row at a time with 16-byte loads per lane (one load instruction
//     covers 1 KiB of the row), issued in bursts of 8 independent loads (7 to 11 where that divides the row
//     and 8 does not) whose addresses differ by compile-time offsets, so the per-load instruction overhead
//     is one VMEM instruction;
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
#include "gemv_device.h"

#include <cstdlib>
#include <type_traits>

namespace rlh {

size_t gemv_lds_bytes(int k, int w_is_f16, int x_f16) {
    const int vec = w_is_f16 ? 8 : 4;
    return (size_t)gemv_iters(k, vec) * kWave * vec * (x_f16 ? 2 : 4);
}

template <typename WT, typename XT, int kEpi, bool kStream, int kBurst = kGemvBurst, bool kEmbed = false, bool kStamp = false>
__global__ __launch_bounds__(kGemvThreads) void gemv_kernel(GemvParams p) {
    extern __shared__ uint4_t smem_raw[];
    __shared__ float red[16];
    __shared__ float2 rope_f[64]; // (cos, sin) of this position, head_dim / 2 <= 64 entries
    // The first burst of weights is issued right behind the prologue's own loads (behind those of its last batch where x takes
    // more than one), so that its memory latency runs under the norm / staging work while x stays ahead of it in the in-order
    // return queue, and is consumed in front of the main loop.  Measured per launch against the same kernel without it --
    // 7B shape: wq|wk|wv 19.3 -> 18.9 us, wo 8.05 -> 8.0, w2 17.1 -> 16.4, the isolated 11008 x 4096 product 16.3 -> 15.9,
    // 4096 x 11008 17.6 -> 16.9; 13B shape: wq|wk|wv 27.3 -> 27.05, wo 10.8 -> 10.6, w2 24.3 -> 24.15; w1|w3 has done it since
    // it was worth 1.6 % there.  (Issued behind the first of w2's two batches of x it cost 0.4 us instead: the second batch
    // waits behind the burst.  With a test for it inside the main loop the 13B wq|wk|wv lost 0.6 us.)  The output head with the
    // greedy pick gains nothing from it and does not do it.
    // (The stamped measurement build keeps the burst behind the prologue, so that "x staged" and "first burst" stay two phases.)
    constexpr int kPre = (!kStamp && ((RLH_GEMV_PRELOAD_EPIS >> kEpi) & 1)) ? kPreSelf : kPreNone;
    gemv_body<WT, XT, kEpi, kStream, kPre, kBurst, kEmbed, kStamp>(p, smem_raw, red, rope_f);
}

static int gemv_blocks(int n_units) {
    const int n_waves = n_units < kGemvTargetWaves ? n_units : kGemvTargetWaves;
    return (n_waves + kGemvWaves - 1) / kGemvWaves;
}

size_t gemv_argmax_ws_bytes() { return (size_t)gemv_blocks(kGemvTargetWaves) * 16; }

template <typename WT, typename XT, int kEpi>
static hipError_t launch_gemv_t(GemvParams p, hipStream_t s) {
    constexpr int rows_per_unit = (kEpi == kEpiRopeKv) ? 2 : 1;
    const int blocks = gemv_blocks(p.n_rows / rows_per_unit);
    const size_t lds = (size_t)gemv_iters(p.k, WVec<WT>::kVec) * kWave * WVec<WT>::kVec * sizeof(XT);
    auto launch = [&](auto kern) -> hipError_t {
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGemvThreads), lds, s, p);
        return hipGetLastError();
    };
    // f16 weights: a burst length that divides the row into whole bursts, where one of these does (pieces of 512 halves per row,
    // LLaMA shapes: 8 / 10 / 16 for dim 4096 / 5120 / 8192, 21.5 -> 22 / 27 / 35 for ffn 11008 / 13824 / 17920; 13 and 43 --
    // dim 6656, ffn 22016 -- have no divisor here and keep the default with its partial last burst).  Same order of additions
    // per lane whatever the burst length, so the same bits.  Measured: w2 of the 7B shape 18.8 -> 17.3 us, wo of the 13B shape
    // 12.2 -> 11.1 us, w2 of the 13B shape 25.7 -> 25.4 us.
    if constexpr (std::is_same<WT, half_t>::value && (kEpi == kEpiStore || kEpi == kEpiStoreArgmax)) {
        const int pieces = gemv_iters(p.k, WVec<WT>::kVec);
        auto pick = [&](auto burst) -> hipError_t {
            constexpr int kB = decltype(burst)::value;
            if (p.stream_weights) return launch(gemv_kernel<WT, XT, kEpi, true, kB>);
            return launch(gemv_kernel<WT, XT, kEpi, false, kB>);
        };
        // (one matrix, one row per unit only: the 13B shape's wq|wk|wv and w1|w3, 10 pieces per row as 5 + 5 instead of
        // 4 + 4 + 2 for each of two rows, measured 30.1 against 29.2 us and 46.6 against 46.4 us)
        if (!p.burst_fixed && pieces % kGemvBurst != 0) {
            if (pieces % 9 == 0) return pick(std::integral_constant<int, 9>{});
            if (pieces % 10 == 0) return pick(std::integral_constant<int, 10>{});
            if (pieces % 11 == 0) return pick(std::integral_constant<int, 11>{});
            if (pieces % 7 == 0) return pick(std::integral_constant<int, 7>{});
        }
    }
    if constexpr (kEpi == kEpiRopeKv) {
        // layer 0 of a token step: the input row read from the embedding table (an instantiation of its own, so that the other
        // layers' kernel carries none of it)
        if (p.embed_table != nullptr) {
            if (p.stream_weights) return launch(gemv_kernel<WT, XT, kEpi, true, kGemvBurst, true>);
            return launch(gemv_kernel<WT, XT, kEpi, false, kGemvBurst, true>);
        }
    }
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

hipError_t launch_gemv_stamped(const GemvParams &p, hipStream_t s, int stamps_capacity_waves, int *n_waves) {
    if (!p.w_is_f16 || p.x_f16 || p.k < 8 || (p.k % 8) != 0 || p.n_rows <= 0 || p.stamps == nullptr) return hipErrorInvalidValue;
    const int blocks = gemv_blocks(p.n_rows);
    if (blocks * kGemvWaves > stamps_capacity_waves) return hipErrorInvalidValue; // every wavefront writes its stamps: checked before the launch
    if (n_waves) *n_waves = blocks * kGemvWaves;
    const size_t lds = (size_t)gemv_iters(p.k, 8) * kWave * 8 * sizeof(float);
    auto kern = gemv_kernel<half_t, float, kEpiStore, true, kGemvBurst, false, true>;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(kGemvThreads), lds, s, p);
    return hipGetLastError();
}

hipError_t launch_gemv(const GemvParams &p, int epilogue, hipStream_t s) {
    const int vec = p.w_is_f16 ? 8 : 4;
    if (p.k < vec || p.n_rows <= 0 || (p.k % vec) != 0) return hipErrorInvalidValue;
    if (p.embed_table != nullptr && (epilogue != kEpiRopeKv || p.state == nullptr)) return hipErrorInvalidValue;
    switch (epilogue) {
    case kEpiStore: return launch_gemv_e<kEpiStore>(p, s);
    case kEpiSilu: return launch_gemv_e<kEpiSilu>(p, s);
    case kEpiRopeKv:
        if ((p.dim % 2) != 0 || (p.head_dim % 2) != 0 || p.head_dim > 128 || p.n_rows != 3 * p.dim) return hipErrorInvalidValue;
        return launch_gemv_e<kEpiRopeKv>(p, s);
    case kEpiStoreArgmax:
        // the output head: fp32 x, no rounding; the pick needs its work memory and the state it advances
        if (p.x_f16 || p.round_y || !p.amax_ws || !p.amax_ticket || !p.state_rw) return hipErrorInvalidValue;
        return p.w_is_f16 ? launch_gemv_t<half_t, float, kEpiStoreArgmax>(p, s) : launch_gemv_t<float, float, kEpiStoreArgmax>(p, s);
    default: return hipErrorInvalidValue;
    }
}

} // namespace rlh
