// gemm_kgroup.hip -- C = A * B^T (f16 operands, fp32 accumulate) for products whose output gives every compute unit only a
// small tile (wo and w2 of a multi-token forward: 1024 x 4096 outputs = one 128 x 128 tile per compute unit).
//
// What bounds the kernels of gemm_dma.hip is the LDS: per K-tile a workgroup writes the staged operands into LDS once and
// every wavefront reads its operand fragments back, and the sum of both, divided by the MFMA cycles of the K-tile, is what
// the measured MFMA utilisation follows (about 65 bytes per cycle and compute unit come out of the LDS in these loops:
// 128 x 128 with four wavefronts of 64 x 64 moves 96 KB per K-tile for 512 MFMA cycles per SIMD -> 0.34 predicted, 0.32
// measured; 256 x 192 with eight of 64 x 96: 216 KB for 1536 -> 0.45 / 0.50; both products of w1|w3 in one pass: 336 KB
// for 3072 -> 0.58 / 0.60).  The staged bytes are fixed by the tile; the fragment bytes fall with the size of a
// wavefront's own tile.  So here the wavefronts of a workgroup do not split the tile but the K-steps: wavefront g of kKG
// takes K-steps g, g + kKG, ... of every K-tile on a tile kKG times larger than its share (128 x 128 per wavefront: 8
// fragment reads per 16 MFMAs instead of 4 per 4), and the kKG partial sums are added at the end through LDS, each
// wavefront ending up with the rows of the tile it then runs the epilogue on (a reduce-scatter along the 32-row slabs).
// The sum over k is therefore taken in another order than in gemm_dma.hip (kKG interleaved partial sums, added in the
// order of g): deterministic, but not bit-identical to that kernel.
//
// Measured and not kept: K-tiles of 128 halves in two stages of 64 KB (two K-steps per wavefront and K-tile, the second step's
// fragments read under the first step's MFMAs, one barrier per 512 MFMA cycles): 15.75 against 15.15 ms for the 1024-token
// forward of the 7B shape -- one K-tile of look-ahead instead of three costs more than the barriers saved.
//
// Contract: GemmParams with batch 1, no K segments, no causal skipping, k % 64 == 0, lda / ldb % 8 == 0; epilogues
// kGemmEpiF16 and kGemmEpiResAddF32, and kGemmEpiF32 for the pieces of a product cut along K (batch = split_k K ranges as
// grid.z, at least four K-tiles each, partial sums stride_c apart).
#include "kernels.h"
#include "device_utils.h"

#include <cstdlib>
#include <type_traits>

namespace rlh {

typedef __attribute__((ext_vector_type(16))) float float16_t;

// the largest number of column tiles per round of the partial-sum exchange that fits the LDS of the stages
constexpr int kgroup_round_tiles(int n_waves, int kg, int nt, int lds_bytes) {
    int best = 1;
    for (int j = 1; j <= nt; j++)
        if (nt % j == 0 && n_waves * (kg - 1) * j * 16 * 64 * 4 <= lds_bytes) best = j;
    return best;
}

// kWM x kWN wavefront tiles of (32 kIT) x (32 kNT) per K-group, kKG K-groups: kWM kWN kKG wavefronts.
template <int kEpi, int kWM, int kWN, int kKG, int kIT, int kNT, int kStages>
__global__ __launch_bounds__(64 * kWM * kWN * kKG) void gemm_f16_kgroup_kernel(GemmParams p) {
    constexpr int kBK = 64, kKS = kBK / 16, kMy = kKS / kKG;
    static_assert(kKS % kKG == 0 && kIT % kKG == 0, "K-steps and row slabs divide among the K-groups");
    constexpr int kWaves = kWM * kWN * kKG;
    constexpr int kWR = 32 * kIT, kTW = 32 * kNT;
    constexpr int kBM = kWR * kWM, kBN = kTW * kWN;
    constexpr int kRowBytes = kBK * 2, kCpr = kBK / 8, kRowsPerLoad = 64 / kCpr, kSwzDiv = 16 / kCpr;
    constexpr int kStageBytes = (kBM + kBN) * kRowBytes;
    static_assert((kBM / kRowsPerLoad) % kWaves == 0 && (kBN / kRowsPerLoad) % kWaves == 0, "every load of a wavefront stays within one matrix");
    constexpr int kLA = kBM / kRowsPerLoad / kWaves, kLB = kBN / kRowsPerLoad / kWaves, kLoads = kLA + kLB;
    constexpr int kITo = kIT / kKG, kWRo = 32 * kITo; // what a wavefront owns after the partial sums are added
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave % kWN, wm = (wave / kWN) % kWM, g = wave / (kWN * kWM);
    int bx = blockIdx.x, by = blockIdx.y;
    if (gridDim.x % 8 != 0) {
        // workgroups go to the 8 XCDs round-robin in launch order: keep the row tiles of one column tile on one XCD
        const int nx = gridDim.x, ny = gridDim.y;
        const int L = by * nx + bx, per = 8 * ny;
        const int chunk = L / per, j = L - chunk * per;
        const int w = min(8, nx - chunk * 8);
        by = j / w;
        bx = chunk * 8 + (j - by * w);
    }
    const int bm0 = by * kBM, bn0 = bx * kBN;
    const int M = p.m, N = p.n, K = p.k;
    // split_k > 1: grid.z counts K ranges of one product -- range z takes K-tiles [z q + min(z, r), ...) of the K / 64 =
    // split_k q + r tiles, one more for z < r -- and C item z (stride_c apart) gets its partial sum (kGemmEpiF32 only)
    int n_kt = K / kBK, k_skip = 0;
    if (p.split_k > 1) {
        const int total = n_kt, q = total / p.split_k, r = total % p.split_k, z = (int)blockIdx.z;
        n_kt = q + (z < r ? 1 : 0);
        k_skip = (z * q + min(z, r)) * kBK;
    }

    // ---- staging: a stage holds rows 0 .. kBM-1 of A then rows 0 .. kBN-1 of B, 128 bytes each, 16-byte chunk c of row r at
    //      chunk c ^ ((r / 2) % 8).  Addresses: a uniform base per matrix (tile origin + k) plus a 32-bit offset per load.
    const int l_row = lane / kCpr, l_pc = lane % kCpr;
    unsigned voff_a[kLA], voff_b[kLB];
#pragma unroll
    for (int i = 0; i < kLA; i++) {
        const int row = (i * kWaves + wave) * kRowsPerLoad + l_row;
        const int lc = l_pc ^ ((row / kSwzDiv) % kCpr);
        voff_a[i] = (unsigned)(((min(bm0 + row, M - 1) - bm0) * p.lda + lc * 8) * 2); // rows past the edge: a valid row, never stored
    }
#pragma unroll
    for (int i = 0; i < kLB; i++) {
        const int row = (i * kWaves + wave) * kRowsPerLoad + l_row;
        const int lc = l_pc ^ ((row / kSwzDiv) % kCpr);
        voff_b[i] = (unsigned)(((min(bn0 + row, N - 1) - bn0) * p.ldb + lc * 8) * 2);
    }
    const half_t *s_a = p.a + (size_t)bm0 * p.lda + k_skip, *s_b = p.b + (size_t)bn0 * p.ldb + k_skip;
    const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)lds_raw;
    int iss_k = 0;
    auto issue = [&](int kt) { // called for kt = 0, 1, 2, ... in this order
        const unsigned dst = lds_base + (unsigned)(kt % kStages) * kStageBytes + (unsigned)wave * 1024;
#pragma unroll
        for (int i = 0; i < kLA; i++) dma16_base(s_a + iss_k, voff_a[i], dst + i * (kWaves * 1024));
#pragma unroll
        for (int i = 0; i < kLB; i++) dma16_base(s_b + iss_k, voff_b[i], dst + (kLA + i) * (kWaves * 1024));
        if (kt + 1 < n_kt) iss_k += kBK; // past the end the last tile is loaded again (keeps the in-flight count constant)
    };

    float16_t acc[kIT][kNT];
#pragma unroll
    for (int i = 0; i < kIT; i++)
#pragma unroll
        for (int j = 0; j < kNT; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // the rows this wavefront owns in the end, and (residual epilogue) what it will add to them, fetched now so that the
    // latency is gone when the sums are ready; each element is read and later written by the same lane (C may alias it)
    const int col_in = lane & 31, row_in = (lane >> 5) * 4;
    const int row_base = bm0 + wm * kWR + g * kWRo, col_base = bn0 + wn * kTW;
    [[maybe_unused]] float16_t early[kEpi == kGemmEpiResAddF32 ? kITo : 1][kEpi == kGemmEpiResAddF32 ? kNT : 1];
    if constexpr (kEpi == kGemmEpiResAddF32) {
#pragma unroll
        for (int i = 0; i < kITo; i++)
#pragma unroll
            for (int j = 0; j < kNT; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int r = row_base + i * 32 + (v >> 2) * 8 + row_in + (v & 3), c = col_base + j * 32 + col_in;
                    early[i][j][v] = (r < M && c < N) ? p.residual[(size_t)r * p.ldc + c] : 0.0f;
                }
    }

    // operand fragments: lane l supplies row l % 32, logical chunk 2 ks + l / 32 of a 32 x 16 slab; the swizzle term is the
    // same for every slab of a lane (slabs start at multiples of 32 rows)
    const int frow = lane & 31, fch = lane >> 5;
    const int sw = (frow / kSwzDiv) % kCpr;
    const int xa = (wm * kWR + frow) * kRowBytes, xb = (kBM + wn * kTW + frow) * kRowBytes;
    int coff[kMy]; // byte offset of this wavefront's s-th K-step within a row
#pragma unroll
    for (int s = 0; s < kMy; s++) coff[s] = (((s * kKG + g) * 2 + fch) ^ sw) << 4;
    half8_t fa[2][kIT], fb[2][kNT];
    auto read_frags = [&](int set, const unsigned char *stage, int s) {
#pragma unroll
        for (int i = 0; i < kIT; i++) fa[set][i] = *reinterpret_cast<const half8_t *>(stage + xa + i * (32 * kRowBytes) + coff[s]);
#pragma unroll
        for (int j = 0; j < kNT; j++) fb[set][j] = *reinterpret_cast<const half8_t *>(stage + xb + j * (32 * kRowBytes) + coff[s]);
    };
    auto mma = [&](int set, int i, int j) { acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0); };

    // Software pipeline as in gemm_dma.hip: all stages in flight at the start; the fragments of a wavefront's next K-step are
    // read while the MFMAs of the current one run; the K-tile change (wait, barrier, refill, first fragments of the next tile)
    // sits in the middle of the wavefront's last K-step of the tile.  `parity` is the parity of the wavefront's K-step count
    // so far (compile time: the loop over K-tiles is unrolled by two).
#pragma unroll
    for (int t = 0; t < kStages; t++) issue(t);
    wait_vmcnt<(kStages - 1) * kLoads>();
    __syncthreads();
    read_frags(0, lds_raw, 0);
    auto k_tile = [&](int kt, auto parity) {
        const unsigned char *stage = lds_raw + (kt % kStages) * kStageBytes;
#pragma unroll
        for (int s = 0; s < kMy; s++) {
            const int cur = (decltype(parity)::value * kMy + s) & 1, nxt = cur ^ 1;
            if (s + 1 < kMy) {
                read_frags(nxt, stage, s + 1);
#pragma unroll
                for (int j = 0; j < kNT; j++)
#pragma unroll
                    for (int i = 0; i < kIT; i++) mma(cur, i, j);
#pragma unroll
                for (int r = 0; r < kIT + kNT; r++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
                }
                __builtin_amdgcn_sched_group_barrier(0x008, kIT * kNT - (kIT + kNT), 0);
            } else {
#pragma unroll
                for (int j = 0; j < kNT / 2; j++)
#pragma unroll
                    for (int i = 0; i < kIT; i++) mma(cur, i, j);
                __builtin_amdgcn_sched_barrier(0);
                wait_vmcnt<(kStages - 2) * kLoads>();
                __syncthreads(); // K-tile kt + 1 is in LDS for everybody, and nobody reads K-tile kt any more
                issue(kt + kStages);
                read_frags(nxt, lds_raw + ((kt + 1) % kStages) * kStageBytes, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = kNT / 2; j < kNT; j++)
#pragma unroll
                    for (int i = 0; i < kIT; i++) mma(cur, i, j);
            }
        }
    };
    for (int kt = 0; kt < n_kt; kt += 2) {
        k_tile(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < n_kt) {
            k_tile(kt + 1, std::integral_constant<int, 1>{});
        } else if constexpr ((kMy & 1) != 0) {
            // an odd number of K-tiles with an odd number of K-steps each: nothing follows, the fragment sets need no fixing
        }
    }
    wait_vmcnt<0>(); // drain the clamped tail loads before LDS is reused
    __syncthreads();

    // ---- the K-groups' partial sums: wavefront g keeps slabs g kITo .. of its tile and receives them from the other groups.
    //      One round per slab index and half of the column tiles, so that what is in LDS at a time fits the stages.
    float16_t out[kITo][kNT];
    if constexpr (kKG == 1) {
#pragma unroll
        for (int i = 0; i < kITo; i++)
#pragma unroll
            for (int j = 0; j < kNT; j++) out[i][j] = acc[i][j];
    } else {
        constexpr int kJH = kgroup_round_tiles(kWaves, kKG, kNT, kStages * kStageBytes); // column tiles per round
        constexpr int kSlotFloats = kJH * 16 * 64;                          // one wavefront's contribution to one owner
        static_assert((size_t)kWaves * (kKG - 1) * kSlotFloats * 4 <= (size_t)kStages * kStageBytes, "a round of partial sums fits the stages");
        float *xbuf = reinterpret_cast<float *>(lds_raw);
        const int pair = wave % (kWN * kWM);                                // wavefronts of the same tile position
#pragma unroll
        for (int r = 0; r < kITo; r++) {
#pragma unroll
            for (int jh = 0; jh < kNT; jh += kJH) {
                // write: for every other group h, slab h kITo + r of my sums goes to the slot (owner h, sender g)
#pragma unroll
                for (int h = 0; h < kKG; h++) {
                    if (h != g) {
                        const int sender = g < h ? g : g - 1; // 0 .. kKG - 2 among the senders of owner h, in the order of g
                        float *dst = xbuf + ((size_t)((h * (kWN * kWM) + pair) * (kKG - 1) + sender)) * kSlotFloats + lane;
#pragma unroll
                        for (int j = 0; j < kJH; j++)
#pragma unroll
                            for (int v = 0; v < 16; v++) dst[(j * 16 + v) * 64] = acc[h * kITo + r][jh + j][v];
                    }
                }
                __syncthreads();
                // read: my slab g kITo + r plus what the others sent, in the order of their g
#pragma unroll
                for (int h = 0; h < kKG; h++) {
                    if (h == g) {
                        const float *src = xbuf + ((size_t)((h * (kWN * kWM) + pair) * (kKG - 1))) * kSlotFloats + lane;
#pragma unroll
                        for (int j = 0; j < kJH; j++)
#pragma unroll
                            for (int v = 0; v < 16; v++) {
                                // partial sums in the order of the K-groups: groups before g, g itself, groups after g
                                float sum = 0.0f;
                                bool first = true;
#pragma unroll
                                for (int q = 0; q < kKG; q++) {
                                    float term;
                                    if (q == h) term = acc[h * kITo + r][jh + j][v];
                                    else term = src[((q < h ? q : q - 1) * kSlotFloats) + (j * 16 + v) * 64];
                                    sum = first ? term : sum + term;
                                    first = false;
                                }
                                out[r][jh + j][v] = sum;
                            }
                    }
                }
                __syncthreads();
            }
        }
    }

    // ---- epilogue on the wavefront's own rows
    if constexpr (kEpi == kGemmEpiF16) {
        // every wavefront lays its rows out in LDS and stores 16-byte pieces of consecutive columns
        const bool rows16 = (p.ldc % 8) == 0 && (N % 8) == 0 && (reinterpret_cast<uintptr_t>(p.c) % 16) == 0;
        if (rows16) {
            constexpr int kTS = kTW + 8;
            static_assert(kWaves * kWRo * kTS * 2 <= kStages * kStageBytes, "the output tiles reuse the stages");
            constexpr int kChunks = kTW / 8;
            half_t *tile = reinterpret_cast<half_t *>(lds_raw) + wave * (kWRo * kTS);
#pragma unroll
            for (int i = 0; i < kITo; i++)
#pragma unroll
                for (int j = 0; j < kNT; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++) tile[(i * 32 + (v >> 2) * 8 + row_in + (v & 3)) * kTS + j * 32 + col_in] = (half_t)out[i][j][v]; // tensor.rs:1623-1643
            half_t *cbase = reinterpret_cast<half_t *>(p.c);
#pragma unroll
            for (int it = 0; it < kChunks * kWRo / 64; it++) {
                const int idx = it * 64 + lane;
                const int rr = idx / kChunks, ch = idx - rr * kChunks;
                const int r = row_base + rr, c = col_base + ch * 8;
                if (r < M && c < N) *reinterpret_cast<half8_t *>(cbase + (size_t)r * p.ldc + c) = *reinterpret_cast<const half8_t *>(tile + rr * kTS + ch * 8);
            }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < kITo; i++)
#pragma unroll
        for (int j = 0; j < kNT; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int r = row_base + i * 32 + (v >> 2) * 8 + row_in + (v & 3), c = col_base + j * 32 + col_in;
                if (r < M && c < N) {
                    const size_t off = (size_t)r * p.ldc + c;
                    if constexpr (kEpi == kGemmEpiF16) reinterpret_cast<half_t *>(p.c)[off] = (half_t)out[i][j][v];
                    else if constexpr (kEpi == kGemmEpiF32) reinterpret_cast<float *>(p.c)[(size_t)blockIdx.z * p.stride_c + off] = out[i][j][v]; // a piece's partial sum
                    else reinterpret_cast<float *>(p.c)[off] = early[i][j][v] + f16r(out[i][j][v]); // transformer.rs:442 / :445 on the f16-rounded product
                }
            }
}

bool gemm_f16_kgroup_supported(const GemmParams &p, int epilogue, int tile) {
    if (p.tune.no_kgroup) return false;
    // tile: the choice of gemm_dma.hip's model -- 0 / 4: 128 x 128.  (256 x 192 tiles with wavefronts of 128 x 96 on every other
    // K-step -- 192 accumulator registers, A fragments single-buffered -- measured 98.8 against 102.2 us on the plain wq|wk|wv product of the 7B shape
    // and 112.4 against 111 us with RoPE and the cache write in the epilogue: the cycles fall as the LDS bytes do, the clock
    // falls with them (power), and the exchange of the partial sums is added.  Not wired in.)
    if (tile != 0 && tile != 4) return false;
    if (epilogue != kGemmEpiF16 && epilogue != kGemmEpiResAddF32 && epilogue != kGemmEpiF32) return false;
    // (fp32 store: the pieces of a product cut along K, as the launcher of gemm_dma.hip sets them up -- batch = split_k pieces)
    if (epilogue == kGemmEpiF32 ? (p.split_k < 2 || p.batch != p.split_k || p.k / 64 / p.split_k < 4) : (p.split_k > 1 || p.batch != 1)) return false;
    if (p.f32_operands || p.k_seg != 0 || p.causal != 0 || p.b2 != nullptr || p.accumulate) return false;
    if (p.m <= 0 || p.n <= 0 || p.k < 64 || p.k % 64 != 0 || p.lda % 8 != 0 || p.ldb % 8 != 0) return false;
    if (epilogue == kGemmEpiResAddF32 && p.residual == nullptr) return false;
    return true;
}

template <int kEpi, int kWM, int kWN, int kKG, int kIT, int kNT, int kStages>
static hipError_t launch_kgroup(const GemmParams &p, hipStream_t s) {
    constexpr int bm = 32 * kIT * kWM, bn = 32 * kNT * kWN;
    constexpr size_t lds = (size_t)kStages * (bm + bn) * 64 * 2;
    static_assert(lds <= 160 * 1024, "LDS of one compute unit");
    static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_f16_kgroup_kernel<kEpi, kWM, kWN, kKG, kIT, kNT, kStages>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) return attr;
    const dim3 grid((p.n + bn - 1) / bn, (p.m + bm - 1) / bm, p.split_k > 1 ? p.split_k : 1);
    hipLaunchKernelGGL((gemm_f16_kgroup_kernel<kEpi, kWM, kWN, kKG, kIT, kNT, kStages>), grid, dim3(64 * kWM * kWN * kKG), lds, s, p);
    return hipGetLastError();
}

hipError_t launch_gemm_f16_kgroup(const GemmParams &p, int epilogue, int tile, hipStream_t s) {
    if (!gemm_f16_kgroup_supported(p, epilogue, tile)) return hipErrorInvalidValue;
    // 128 x 128 per workgroup: eight wavefronts = two column halves x four K-groups, each wavefront on 128 x 64 for one K-step in
    // four (the whole tile per wavefront -- 256 accumulator registers -- does not survive hipcc's register allocation); four
    // stages of 32 KB
    if (epilogue == kGemmEpiF16) return launch_kgroup<kGemmEpiF16, 1, 2, 4, 4, 2, 4>(p, s);
    if (epilogue == kGemmEpiF32) return launch_kgroup<kGemmEpiF32, 1, 2, 4, 4, 2, 4>(p, s);
    return launch_kgroup<kGemmEpiResAddF32, 1, 2, 4, 4, 2, 4>(p, s);
}

} // namespace rlh
