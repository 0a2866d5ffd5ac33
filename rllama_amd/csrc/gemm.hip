// gemm.hip -- f16 MFMA GEMM for multi-token prompt prefill on gfx950 (CDNA4):  C = A * B^T
//   A [M x K] f16 row-major (activations, one row per prompt token), B [N x K] f16 row-major (a projection
//   weight exactly as the reference stores it, [out x in]), fp32 accumulation in the matrix cores.
//
// It replaces Tensor::matrix_mul_inplace_transposed's f16 branch (Noeda/rllama tensor.rs:1476-1666) for
// src.rows > 1: every output is sum_k A[r,k] * B[c,k] accumulated in fp32 and (for the projection uses)
// rounded to f16 like tensor.rs:1623-1643.  Only the order of the fp32 additions differs.
//
// Blocking: a workgroup of 4 wavefronts computes a 128 x 128 tile of C; each wavefront owns a 64 x 64
// quadrant = 2 x 2 v_mfma_f32_32x32x16_f16 tiles (64 fp32 accumulator registers per lane).  A and B tiles of
// 128 x 64 halves are staged through LDS (rows padded by 16 bytes so that the 16-byte operand reads of
// 16 consecutive lanes fall into distinct banks) and double buffered: the global loads of K-tile i+1
// are in flight while K-tile i feeds the matrix cores.  Both operands have K contiguous in memory, so an
// MFMA operand (8 consecutive k of one row per lane) is one 16-byte LDS read.
// Batched over grid.z with element strides (used for the per-head products of prefill attention).
#include "kernels.h"
#include "device_utils.h"

#include <cstdlib>

namespace rlh {

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kLdsStride = kBK + 8; // halves per staged row (144 bytes)
constexpr int kGemmThreads = 256;

typedef __attribute__((ext_vector_type(16))) float float16_t;

template <int kEpi>
__global__ __launch_bounds__(kGemmThreads) void gemm_f16_kernel(GemmParams p) {
    __shared__ __attribute__((aligned(16))) half_t As[2][kBM * kLdsStride];
    __shared__ __attribute__((aligned(16))) half_t Bs[2][kBN * kLdsStride];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1; // quadrant of the block tile
    const int bm0 = blockIdx.y * kBM, bn0 = blockIdx.x * kBN;
    const size_t zb = blockIdx.z;
    const half_t *A = p.a + zb * p.stride_a;
    const half_t *B = p.b + zb * p.stride_b;
    const int M = p.m, N = p.n, K = p.k;

    // global -> register staging: 128 rows x 8 chunks of 16 bytes per operand tile, 4 chunks per thread
    uint4_t ra[4], rb[4];
    auto load_tiles = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int q = tid + i * kGemmThreads;
            const int row = q >> 3, ch = q & 7;
            const int kk = k0 + ch * 8;
            const int ar = bm0 + row, br = bn0 + row;
            ra[i] = (ar < M && kk < K) ? *reinterpret_cast<const uint4_t *>(A + (size_t)ar * p.lda + kk) : uint4_t{0u, 0u, 0u, 0u};
            rb[i] = (br < N && kk < K) ? *reinterpret_cast<const uint4_t *>(B + (size_t)br * p.ldb + kk) : uint4_t{0u, 0u, 0u, 0u};
        }
    };
    auto store_tiles = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int q = tid + i * kGemmThreads;
            const int row = q >> 3, ch = q & 7;
            *reinterpret_cast<uint4_t *>(&As[buf][row * kLdsStride + ch * 8]) = ra[i];
            *reinterpret_cast<uint4_t *>(&Bs[buf][row * kLdsStride + ch * 8]) = rb[i];
        }
    };

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int n_kt = (K + kBK - 1) / kBK;
    load_tiles(0);
    store_tiles(0);
    __syncthreads();
    for (int kt = 0; kt < n_kt; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < n_kt) load_tiles((kt + 1) * kBK);
        // operand fragments: lane l supplies row (l % 32), k = 8 * (l / 32) .. + 8 of a 32 x 16 slab
        const int frow = lane & 31, fk = (lane >> 5) * 8;
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ks++) {
            half8_t af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                af[i] = *reinterpret_cast<const half8_t *>(&As[buf][(wm * 64 + i * 32 + frow) * kLdsStride + ks * 16 + fk]);
                bf[i] = *reinterpret_cast<const half8_t *>(&Bs[buf][(wn * 64 + i * 32 + frow) * kLdsStride + ks * 16 + fk]);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < n_kt) store_tiles(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue.  Accumulator register v of a 32 x 32 tile: row 8 * (v / 4) + 4 * (lane / 32) + v % 4, col lane % 32
    const int col_in = lane & 31;
    const int row_in = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int c = bn0 + wn * 64 + j * 32 + col_in;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int r = bm0 + wm * 64 + i * 32 + (v >> 2) * 8 + row_in + (v & 3);
                if (r < M && c < N) {
                    const float val = acc[i][j][v];
                    const size_t off = zb * p.stride_c + (size_t)r * p.ldc + c;
                    if constexpr (kEpi == kGemmEpiF16) {
                        reinterpret_cast<half_t *>(p.c)[off] = (half_t)val; // tensor.rs:1623-1643
                    } else if constexpr (kEpi == kGemmEpiF32) {
                        float *cp = reinterpret_cast<float *>(p.c) + off;
                        *cp = p.accumulate ? (*cp + val) : val;
                    } else if constexpr (kEpi == kGemmEpiSiluGateF16) { // tensor.rs:822-832 on the f16 gate, times the f16-rounded product
                        const float g = (float)p.gate[(size_t)r * p.ldc + c];
                        reinterpret_cast<half_t *>(p.c)[off] = to_f16(silu_fast(g) * f16r(val));
                    } else { // kGemmEpiResAddF32: residual add of transformer.rs:442 / :445 on the f16-rounded product
                        reinterpret_cast<float *>(p.c)[off] = p.residual[(size_t)r * p.ldc + c] + f16r(val);
                    }
                }
            }
        }
    }
}

hipError_t launch_gemm_f16(const GemmParams &p, int epilogue, hipStream_t s) {
    if (p.f32_operands) { // fp32 operands exist on the fast path only
        if (p.m <= 0 || p.n <= 0 || p.batch < 1 || !gemm_f16_dma_supported(p)) return hipErrorInvalidValue;
        return launch_gemm_f16_dma(p, epilogue, s);
    }
    if (p.m <= 0 || p.n <= 0 || p.k <= 0 || (p.k % 8) != 0 || (p.lda % 8) != 0 || (p.ldb % 8) != 0 || p.batch < 1) return hipErrorInvalidValue;
    if (epilogue == kGemmEpiRopeQkv) return gemm_f16_rope_supported(p) ? launch_gemm_f16_dma(p, epilogue, s) : hipErrorInvalidValue; // fast path only
    if (p.b2 != nullptr) return gemm_f16_dual_gate_supported(p) ? launch_gemm_f16_dma(p, epilogue, s) : hipErrorInvalidValue; // fast path only
    if (p.k_seg != 0 || p.causal != 0) return gemm_f16_dma_supported(p) ? launch_gemm_f16_dma(p, epilogue, s) : hipErrorInvalidValue;
    if (gemm_f16_dma_supported(p)) return launch_gemm_f16_dma(p, epilogue, s);
    dim3 grid((p.n + kBN - 1) / kBN, (p.m + kBM - 1) / kBM, p.batch);
    switch (epilogue) {
    case kGemmEpiF16: hipLaunchKernelGGL(gemm_f16_kernel<kGemmEpiF16>, grid, dim3(kGemmThreads), 0, s, p); break;
    case kGemmEpiF32: hipLaunchKernelGGL(gemm_f16_kernel<kGemmEpiF32>, grid, dim3(kGemmThreads), 0, s, p); break;
    case kGemmEpiResAddF32:
        if (p.residual == nullptr || p.batch != 1) return hipErrorInvalidValue;
        hipLaunchKernelGGL(gemm_f16_kernel<kGemmEpiResAddF32>, grid, dim3(kGemmThreads), 0, s, p);
        break;
    case kGemmEpiSiluGateF16:
        if (p.gate == nullptr || p.batch != 1) return hipErrorInvalidValue;
        hipLaunchKernelGGL(gemm_f16_kernel<kGemmEpiSiluGateF16>, grid, dim3(kGemmThreads), 0, s, p);
        break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace rlh
