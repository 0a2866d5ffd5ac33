// gemm_dma.hip -- the fast path of the prefill GEMM  C = A * B^T  (f16 operands, fp32 accumulate) on gfx950.
//
// Same contract as gemm.hip's kernel, restricted to K % 64 == 0.  What differs is how operands reach LDS:
//   * direct global -> LDS loads (global_load_lds_dwordx4: each lane names a global address, the 64 x 16 bytes
//     of a wavefront land contiguously in LDS), so no registers and no ds_write are spent on staging and a
//     load can stay in flight for several K-tiles: four LDS stages, the loads of K-tile t + 2 are issued while
//     K-tile t feeds the matrix cores, one barrier per K-tile;
//   * LDS rows are 128 bytes (64 halves) without padding; the 16-byte chunk c of row r is stored at chunk
//     c ^ ((r >> 1) & 7), which makes the MFMA operand reads (16 consecutive rows, same logical chunk) hit 16
//     distinct bank groups, and is free on the store side because every lane chooses its own global address.
// Workgroup tile 128 x 128, 4 wavefronts of 64 x 64 (2 x 2 v_mfma_f32_32x32x16_f16).
#include "kernels.h"
#include "device_utils.h"

namespace rlh {

constexpr int kDmaBM = 128, kDmaBN = 128, kDmaBK = 64;
constexpr int kDmaStages = 4;
constexpr int kDmaThreads = 256;
constexpr int kDmaStageBytes = (kDmaBM + kDmaBN) * kDmaBK * 2; // 32 KiB
constexpr int kDmaLoadsPerWave = (kDmaBM + kDmaBN) / 8 / 4;    // 1 KiB loads (8 rows) per wavefront and K-tile

typedef __attribute__((ext_vector_type(16))) float float16_t;

template <int kEpi>
__global__ __launch_bounds__(kDmaThreads) void gemm_f16_dma_kernel(GemmParams p) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int bm0 = blockIdx.y * kDmaBM, bn0 = blockIdx.x * kDmaBN;
    const size_t zb = blockIdx.z;
    const half_t *A = p.a + zb * p.stride_a;
    const half_t *B = p.b + zb * p.stride_b;
    const int M = p.m, N = p.n, K = p.k;
    const int n_kt = K / kDmaBK;

    // ---- staging: wavefront w moves row groups (8 rows = 1 KiB of LDS) w*8 .. w*8+7 of the 32 groups of a stage
    //      (groups 0..15 = A rows, 16..31 = B rows).  Lane i of a group: row i / 8, physical chunk i % 8.
    const int l_row = lane >> 3, l_pc = lane & 7;
    const half_t *gsrc[kDmaLoadsPerWave];
#pragma unroll
    for (int i = 0; i < kDmaLoadsPerWave; i++) {
        const int g = wave * kDmaLoadsPerWave + i;
        const bool is_b = g >= kDmaBM / 8;
        const int row = (is_b ? g - kDmaBM / 8 : g) * 8 + l_row;  // row within the tile
        const int lc = l_pc ^ ((row >> 1) & 7);                   // logical chunk this lane fetches
        // rows past the matrix edge are clamped to a valid row; what they produce is never stored
        const int grow = is_b ? min(bn0 + row, N - 1) : min(bm0 + row, M - 1);
        gsrc[i] = (is_b ? B + (size_t)grow * p.ldb : A + (size_t)grow * p.lda) + lc * 8;
    }
    // The loads are written as inline assembly on purpose: through the builtin the compiler tracks them as LDS
    // writes and puts s_waitcnt vmcnt(0) in front of every LDS read, which would wait for the prefetched K-tiles as
    // well; here the waits are placed by hand (vmcnt is decremented in issue order).
    const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)lds_raw;
    const unsigned wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto issue = [&](int kt) {
        const int k0 = min(kt, n_kt - 1) * kDmaBK; // past the end: reload the last tile (keeps the in-flight count constant)
        const unsigned stage = lds_base + (unsigned)(kt % kDmaStages) * kDmaStageBytes + wave_u * (kDmaLoadsPerWave * 1024);
#pragma unroll
        for (int i = 0; i < kDmaLoadsPerWave; i++) {
            const half_t *src = gsrc[i] + k0;
            const unsigned dst = stage + i * 1024; // wave-uniform LDS byte address; lane l lands at dst + 16 l
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(dst) : "memory");
        }
    };

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // operand fragments: lane l supplies row (l % 32), logical chunk 2 * ks + l / 32 of a 32 x 16 slab
    const int frow = lane & 31, fch = lane >> 5;
    int a_off[2], b_off[2], a_sw[2], b_sw[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int ra = wm * 64 + i * 32 + frow, rb = wn * 64 + i * 32 + frow;
        a_off[i] = ra * 128;
        a_sw[i] = (ra >> 1) & 7;
        b_off[i] = kDmaBM * 128 + rb * 128;
        b_sw[i] = (rb >> 1) & 7;
    }

    issue(0);
    issue(1);
    for (int kt = 0; kt < n_kt; kt++) {
        issue(kt + 2);
        // K-tile kt was issued two issue() calls ago: at most 2 * kDmaLoadsPerWave newer loads may still be in flight
        __builtin_amdgcn_s_waitcnt(0x0F70 | ((2 * kDmaLoadsPerWave) & 0xF) | (((2 * kDmaLoadsPerWave) >> 4) << 14));
        __syncthreads();
        const unsigned char *stage = lds_raw + (kt % kDmaStages) * kDmaStageBytes;
#pragma unroll
        for (int ks = 0; ks < kDmaBK / 16; ks++) {
            half8_t af[2], bf[2];
            const int lc = ks * 2 + fch;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                af[i] = *reinterpret_cast<const half8_t *>(stage + a_off[i] + ((lc ^ a_sw[i]) << 4));
                bf[i] = *reinterpret_cast<const half8_t *>(stage + b_off[i] + ((lc ^ b_sw[i]) << 4));
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // drain the clamped tail loads before the block's LDS is released

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
                    } else { // kGemmEpiResAddF32: residual add of transformer.rs:442 / :445 on the f16-rounded product
                        reinterpret_cast<float *>(p.c)[off] = p.residual[(size_t)r * p.ldc + c] + f16r(val);
                    }
                }
            }
        }
    }
}

bool gemm_f16_dma_supported(const GemmParams &p) { return p.k >= kDmaBK && (p.k % kDmaBK) == 0 && (p.lda % 8) == 0 && (p.ldb % 8) == 0; }

hipError_t launch_gemm_f16_dma(const GemmParams &p, int epilogue, hipStream_t s) {
    if (!gemm_f16_dma_supported(p) || p.m <= 0 || p.n <= 0 || p.batch < 1) return hipErrorInvalidValue;
    const size_t lds = (size_t)kDmaStages * kDmaStageBytes;
    dim3 grid((p.n + kDmaBN - 1) / kDmaBN, (p.m + kDmaBM - 1) / kDmaBM, p.batch);
    auto go = [&](auto kern) -> hipError_t {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, grid, dim3(kDmaThreads), lds, s, p);
        return hipGetLastError();
    };
    switch (epilogue) {
    case kGemmEpiF16: return go(gemm_f16_dma_kernel<kGemmEpiF16>);
    case kGemmEpiF32: return go(gemm_f16_dma_kernel<kGemmEpiF32>);
    case kGemmEpiResAddF32:
        if (p.residual == nullptr || p.batch != 1) return hipErrorInvalidValue;
        return go(gemm_f16_dma_kernel<kGemmEpiResAddF32>);
    default: return hipErrorInvalidValue;
    }
}

} // namespace rlh
