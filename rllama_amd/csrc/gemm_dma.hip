// gemm_dma.hip -- the fast path of the prefill GEMM  C = A * B^T  (f16 operands, fp32 accumulate) on gfx950.
//
// Same contract as gemm.hip's kernel, restricted to K % 32 == 0.  What differs is how operands reach LDS and how
// large a tile a workgroup owns:
//   * direct global -> LDS loads (global_load_lds_dwordx4: each lane names a global address, the 64 x 16 bytes
//     of a wavefront land contiguously in LDS), so no registers and no ds_write are spent on staging and a
//     load can stay in flight across K-tiles: several LDS stages, the loads of K-tile t + stages - 1 are issued
//     while K-tile t feeds the matrix cores, one barrier per K-tile;
//   * LDS rows are 2 kBK bytes without padding; the 16-byte chunk c of row r is stored at a chunk XOR-ed
//     with a function of r, which makes the MFMA operand reads (16 consecutive rows, same logical chunk) hit 16
//     distinct bank groups, and is free on the store side because every lane chooses its own global address;
//   * the tile is a template parameter.  What bounds this kernel is the L2 -> LDS traffic, which falls with the
//     tile edge: 128 x 128 moves 1 byte per 64 flop, 256 x 256 one per 128 flop.  launch_gemm_f16_dma picks the
//     tile by a small cost model (rounds of workgroups over the compute units x tile efficiency).
// Wavefronts form a (kWavesM x 2) grid; each owns 64 x (32 kNT) of C = 2 x kNT v_mfma_f32_32x32x16_f16 tiles.
// The same kernel runs on fp32 operands (f32 mode, v_mfma_f32_32x32x2_f32) and, for products with few output tiles,
// on K ranges whose partial sums gemm_split_finish_kernel adds up (both further down).
#include "kernels.h"
#include "device_utils.h"
#include "gemm_epilogue.h"

#include <cstdlib>

namespace rlh {

constexpr int kDmaMinBK = 32;

typedef __attribute__((ext_vector_type(16))) float float16_t;

// kWavesM: wavefront rows (tile height 64 kWavesM); kNT: 32-column MFMA tiles per wavefront (tile width 64 kNT);
// kBK: halves of K per tile (32 or 64); kStages: LDS stages (K-tiles in flight).
// kF32: the operands are fp32 (f32 mode: tensor.rs:1282-1475 for src.rows > 1).  Staging moves bytes and is the same
// with a row of kBK / 2 floats; a 16-byte fragment then holds 4 consecutive k of a row and feeds 4
// v_mfma_f32_32x32x2_f32 (k slot of lane half h in the j-th of them: float j of chunk 2 ks + h, for A and B alike).
// kIT: 32-row MFMA tiles per wavefront (2: wavefronts of 64 x 32 kNT; 1: 32 x 32 kNT, for products with at most 32 rows).
// kDual: two products of the same A in one pass -- A * B^T and A * B2^T (w1 and w3 of the feed-forward block,
// transformer.rs:551-565) -- with two accumulator sets per wavefront: a K-tile of A is staged once for both, so the L2 -> LDS
// bytes per flop fall by a further 29 % on the 256 x 192 tile, the gate never goes to memory and comes back, and the
// epilogue writes SiLU(f16(A B^T)) * f16(A B2^T) straight from the accumulators.
template <int kEpi, int kWavesM, int kNT, int kBK, int kStages, bool kF32 = false, int kIT = 2, bool kDual = false>
__global__ __launch_bounds__(128 * kWavesM) void gemm_f16_dma_kernel(GemmParams p) {
    static_assert(!kDual || (kEpi == kGemmEpiSiluGateF16 && !kF32), "two products share the SiLU-gate epilogue only");
    constexpr int kP = kDual ? 2 : 1;                    // products
    constexpr int kE = kF32 ? 2 : 1;                     // halves per operand element: k, lda, ldb, strides count elements
    constexpr int kWaves = 2 * kWavesM;
    constexpr int kWR = 32 * kIT;                        // rows of a wavefront's tile
    constexpr int kBM = kWR * kWavesM, kBN = 64 * kNT;
    constexpr int kCpr = kBK / 8;                        // 16-byte chunks per LDS row
    constexpr int kRowsPerLoad = 64 / kCpr;              // rows one wavefront-wide load covers (1 KiB of LDS)
    constexpr int kSwzDiv = 16 / kCpr;                   // physical chunk = logical chunk ^ ((row / kSwzDiv) % kCpr)
    constexpr int kRowBytes = kBK * 2;
    constexpr int kStageBytes = (kBM + kP * kBN) * kRowBytes;
    constexpr int kGroups = kStageBytes / 1024;          // 1 KiB row groups per stage, dealt round-robin to wavefronts
    constexpr int kLoadsMax = (kGroups + kWaves - 1) / kWaves;
    constexpr int kLoadsMin = kGroups / kWaves;
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    int bx = blockIdx.x, by = blockIdx.y;
    if (gridDim.x % 8 != 0) {
        // Workgroups go to the 8 XCDs round-robin in launch order (x fastest).  With a row of tiles that is not a multiple of
        // 8 wide, the row tiles of one column tile (same B rows) would land on different XCDs and each L2 would fetch that B
        // tile again: renumber in chunks of 8 columns so that they are 8 launches apart and meet in one L2.
        const int nx = gridDim.x, ny = gridDim.y;
        const int L = by * nx + bx, per = 8 * ny;
        const int chunk = L / per, j = L - chunk * per;
        const int w = min(8, nx - chunk * 8);
        by = j / w;
        bx = chunk * 8 + (j - by * w);
    }
    const int bm0 = by * kBM, bn0 = bx * kBN;
    const size_t zb = blockIdx.z;
    const half_t *A = p.a + zb * p.stride_a * kE;
    const half_t *B = p.b + zb * p.stride_b * kE;
    const int M = p.m, N = p.n, K = p.k * kE;          // K, segments and k offsets below are in halves
    // split_k > 1: grid.z counts K ranges of one product, not batch items (strides of a and b are 0 then): range z takes
    // K-tiles [z q + min(z, r), ...) of the K / kBK = split_k q + r tiles, one more for z < r; C item z gets its partial sum
    int split_tiles = -1;
    if (p.split_k > 1) {
        const int total = K / kBK, q = total / p.split_k, r = total % p.split_k, z = (int)blockIdx.z;
        split_tiles = q + (z < r ? 1 : 0);
        const int skip = (z * q + min(z, r)) * kBK;
        A += skip;
        B += skip;
    }
    if (p.causal == 1 && bn0 > bm0 + kBM - 1) return; // the whole tile lies above the diagonal (uniform for the workgroup)
    // K-tiles: n_seg segments of tps tiles each; A's k runs on from segment to segment, B's starts over
    const int seg_len = p.k_seg > 0 ? p.k_seg * kE : K;
    const int seg_used = p.causal == 2 ? min(seg_len, ((bm0 + kBM) * kE + kBK - 1) / kBK * kBK) : seg_len;
    const int tps = seg_used / kBK;
    const int n_kt = split_tiles >= 0 ? split_tiles : (K / seg_len) * tps;

    // ---- staging: a stage holds rows 0 .. kBM-1 of A then rows 0 .. kBN-1 of B, kRowBytes each.  Load i of
    //      wavefront w moves row group i * kWaves + w; lane l of a group: row l / kCpr, physical chunk l % kCpr.
    const int l_row = lane / kCpr, l_pc = lane % kCpr;
    const bool short_wave = kLoadsMax != kLoadsMin && (kLoadsMax - 1) * kWaves + wave >= kGroups; // one load fewer
    const half_t *gsrc[kLoadsMax];
    bool src_is_b[kLoadsMax];
#pragma unroll
    for (int i = 0; i < kLoadsMax; i++) {
        const int g = min(i * kWaves + wave, kGroups - 1);
        const int row2 = g * kRowsPerLoad + l_row;       // 0 .. kBM + kP kBN - 1 over A, then B (, then B2)
        const bool is_b = row2 >= kBM;
        const bool is_b2 = kDual && row2 >= kBM + kBN;
        const int row = is_b2 ? row2 - kBM - kBN : is_b ? row2 - kBM : row2;
        const int lc = l_pc ^ ((row / kSwzDiv) % kCpr);  // logical chunk this lane fetches
        // rows past the matrix edge are clamped to a valid row; what they produce is never stored
        const int grow = is_b ? min(bn0 + row, N - 1) : min(bm0 + row, M - 1);
        const half_t *bsrc = is_b2 ? p.b2 : B;
        gsrc[i] = (is_b ? bsrc + (size_t)grow * p.ldb * kE : A + (size_t)grow * p.lda * kE) + lc * 8;
        src_is_b[i] = is_b;
    }
    const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)lds_raw;
    int iss_t = 0, iss_ka = 0, iss_kb = 0; // the K-tile the next issue() loads: index within its segment, k offsets in A and B
    auto issue = [&](int kt) {             // called for kt = 0, 1, 2, ... in this order
        const unsigned dst = lds_base + (unsigned)(kt % kStages) * kStageBytes + (unsigned)wave * 1024;
#pragma unroll
        for (int i = 0; i < kLoadsMax; i++)
            if (i < kLoadsMin || !short_wave) dma16(gsrc[i] + (src_is_b[i] ? iss_kb : iss_ka), dst + i * (kWaves * 1024));
        if (kt + 1 < n_kt) { // past the end the last tile is loaded again (keeps the in-flight count constant)
            if (++iss_t == tps) {
                iss_t = 0;
                iss_ka += seg_len - (tps - 1) * kBK;
                iss_kb = 0;
            } else {
                iss_ka += kBK;
                iss_kb += kBK;
            }
        }
    };

    constexpr int kNTs = kP * kNT;                       // column tiles of a wavefront over all products (product q: j / kNT)
    float16_t acc[kIT][kNTs];
#pragma unroll
    for (int i = 0; i < kIT; i++)
#pragma unroll
        for (int j = 0; j < kNTs; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // Residual epilogue on small wavefront tiles: what the epilogue adds to is fetched now, before the K loop, so that its
    // latency is gone by the time the accumulators are ready (these ordinary loads are older than every direct-to-LDS
    // load below, so the hand-placed vmcnt waits only get stricter).  Each element is read and later written by the
    // same lane, so C may alias the residual.
    constexpr bool kEarlyResidual = kEpi == kGemmEpiResAddF32 && kNT * kIT <= 4;
    [[maybe_unused]] float16_t early[kEarlyResidual ? kIT : 1][kEarlyResidual ? kNT : 1];
    if constexpr (kEarlyResidual) {
#pragma unroll
        for (int i = 0; i < kIT; i++)
#pragma unroll
            for (int j = 0; j < kNT; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int r = bm0 + wm * kWR + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                    const int c = bn0 + wn * (32 * kNT) + j * 32 + (lane & 31);
                    early[i][j][v] = (r < M && c < N) ? p.residual[(size_t)r * p.ldc + c] : 0.0f;
                }
    }

    // SiLU-gate epilogue: the gate values this lane will need (the 16-byte pieces it handles in the row-wise epilogue below)
    // are fetched now as well, for the same reason.
    [[maybe_unused]] const bool rows16 = (p.ldc % 8) == 0 && (N % 8) == 0 && ((zb * p.stride_c) % 8) == 0 && (reinterpret_cast<uintptr_t>(p.c) % 16) == 0 &&
                                         (kEpi != kGemmEpiSiluGateF16 || kDual || (reinterpret_cast<uintptr_t>(p.gate) % 16) == 0);
    constexpr bool kGatePre = kEpi == kGemmEpiSiluGateF16 && !kDual && kNT * kIT <= 6; // the widest tile has no registers to spare for it
    constexpr int kRowChunks = 32 * kNT / 8;             // 16-byte pieces per row of a wavefront's tile
    constexpr int kGateChunks = kGatePre ? kRowChunks * kWR / 64 : 1;
    [[maybe_unused]] half8_t gate_pre[kGateChunks];
    if constexpr (kGatePre) {
        if (rows16) {
#pragma unroll
            for (int it = 0; it < kGateChunks; it++) {
                const int idx = it * 64 + lane;
                const int rr = idx / kRowChunks, ch = idx - rr * kRowChunks;
                const int r = bm0 + wm * kWR + rr, c = bn0 + wn * (32 * kNT) + ch * 8;
                gate_pre[it] = (r < M && c < N) ? *reinterpret_cast<const half8_t *>(p.gate + (size_t)r * p.ldc + c) : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            }
        }
    }

    // operand fragments: lane l supplies row (l % 32), logical chunk 2 * ks + l / 32 of a 32 x 16 slab
    const int frow = lane & 31, fch = lane >> 5;
    int a_off[kIT], a_sw[kIT], b_off[kNTs], b_sw[kNTs];
#pragma unroll
    for (int i = 0; i < kIT; i++) {
        const int ra = wm * kWR + i * 32 + frow;
        a_off[i] = ra * kRowBytes;
        a_sw[i] = (ra / kSwzDiv) % kCpr;
    }
#pragma unroll
    for (int j = 0; j < kNTs; j++) {
        const int rb = wn * (32 * kNT) + (j % kNT) * 32 + frow; // row within its own matrix (the swizzle counts from there)
        b_off[j] = (kBM + (j / kNT) * kBN + rb) * kRowBytes;
        b_sw[j] = (rb / kSwzDiv) % kCpr;
    }

    // Software pipeline.  LDS: all kStages stages are in flight at the start; at the end of K-tile t the wavefront
    // waits for K-tile t + 1, passes the barrier (now nobody reads stage t % kStages any more) and refills that stage
    // with K-tile t + kStages.  Registers: the operand fragments of K-step s + 1 are read from LDS while the MFMAs
    // of K-step s run (two fragment sets, selected by the parity of the unrolled K-step); the tile change sits in
    // the middle of the last K-step's MFMAs so that the barrier and the LDS latency behind it stay covered.
    constexpr int kKS = kBK / 16;
    constexpr int kSplitJ = kNTs / 2; // column tiles of the last K-step whose MFMAs run before the tile change (0 .. kNT measured alike)
    static_assert(kKS % 2 == 0, "fragment sets alternate by K-step parity");
    half8_t af[2][kIT];
    [[maybe_unused]] half8_t bf[2][kDual ? 1 : kNT];
    auto mma = [&](const half8_t &a, const half8_t &b, float16_t &c) {
        if constexpr (kF32) {
            const float4_t a4 = __builtin_bit_cast(float4_t, a), b4 = __builtin_bit_cast(float4_t, b);
#pragma unroll
            for (int e = 0; e < 4; e++) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[e], b4[e], c, 0, 0, 0);
        } else {
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
        }
    };
    auto read_frags = [&](int set, const unsigned char *stage, int ks) {
        const int lc = ks * 2 + fch;
#pragma unroll
        for (int i = 0; i < kIT; i++) af[set][i] = *reinterpret_cast<const half8_t *>(stage + a_off[i] + ((lc ^ a_sw[i]) << 4));
#pragma unroll
        for (int j = 0; j < (kDual ? 0 : kNT); j++) bf[set][j] = *reinterpret_cast<const half8_t *>(stage + b_off[j] + ((lc ^ b_sw[j]) << 4));
    };
    if constexpr (kDual) {
        // Two products: 192 accumulator registers of the 256 a wavefront has here, so everything else is kept small.  Staging
        // addresses are a uniform base per matrix (tile origin + k, scalar registers) plus one 32-bit offset per load that B and
        // B2 share; B fragments are single-buffered per product -- those of product 1 are read while the MFMAs of product 0 run,
        // those of product 0 for the next K-step (with A's, double-buffered) while product 1's run.
        static_assert((kBM / kRowsPerLoad) % kWaves == 0 && (kBN / kRowsPerLoad) % kWaves == 0, "every load of a wavefront stays within one matrix");
        static_assert(kSwzDiv * kCpr <= 32 && 32 % (kSwzDiv * kCpr) == 0, "one swizzle term for all fragments of a lane");
        constexpr int kLA = kBM / kRowsPerLoad / kWaves, kLB = kBN / kRowsPerLoad / kWaves;
        constexpr int kLoads = kLA + 2 * kLB;
        unsigned voff_a[kLA], voff_b[kLB];
#pragma unroll
        for (int i = 0; i < kLA; i++) {
            const int row = (i * kWaves + wave) * kRowsPerLoad + l_row;
            const int lc = l_pc ^ ((row / kSwzDiv) % kCpr);
            voff_a[i] = (unsigned)(((min(bm0 + row, M - 1) - bm0) * p.lda + lc * 8) * 2);
        }
#pragma unroll
        for (int i = 0; i < kLB; i++) {
            const int row = (i * kWaves + wave) * kRowsPerLoad + l_row;
            const int lc = l_pc ^ ((row / kSwzDiv) % kCpr);
            voff_b[i] = (unsigned)(((min(bn0 + row, N - 1) - bn0) * p.ldb + lc * 8) * 2);
        }
        const half_t *s_a = A + (size_t)bm0 * p.lda, *s_b = B + (size_t)bn0 * p.ldb, *s_b2 = p.b2 + (size_t)bn0 * p.ldb;
        int iss_k = 0;
        auto issue2 = [&](int kt) {
            const unsigned dst = lds_base + (unsigned)(kt % kStages) * kStageBytes + (unsigned)wave * 1024;
#pragma unroll
            for (int i = 0; i < kLA; i++) dma16_base(s_a + iss_k, voff_a[i], dst + i * (kWaves * 1024));
#pragma unroll
            for (int i = 0; i < kLB; i++) dma16_base(s_b + iss_k, voff_b[i], dst + (kLA + i) * (kWaves * 1024));
#pragma unroll
            for (int i = 0; i < kLB; i++) dma16_base(s_b2 + iss_k, voff_b[i], dst + (kLA + kLB + i) * (kWaves * 1024));
            if (kt + 1 < n_kt) iss_k += kBK; // past the end the last tile is loaded again (keeps the in-flight count constant)
        };
        const int sw = (frow / kSwzDiv) % kCpr;
        const int xa = (wm * kWR + frow) * kRowBytes, xb = (kBM + wn * (32 * kNT) + frow) * kRowBytes;
        half8_t b0[kNT], b1[kNT];
        auto read_a = [&](int set, const unsigned char *stage, int ks) {
            const int c = ((ks * 2 + fch) ^ sw) << 4;
#pragma unroll
            for (int i = 0; i < kIT; i++) af[set][i] = *reinterpret_cast<const half8_t *>(stage + xa + i * (32 * kRowBytes) + c);
        };
        auto read_b = [&](half8_t (&b)[kNT], const unsigned char *stage, int ks, int q) {
            const int c = ((ks * 2 + fch) ^ sw) << 4;
#pragma unroll
            for (int j = 0; j < kNT; j++) b[j] = *reinterpret_cast<const half8_t *>(stage + xb + (q * kBN + j * 32) * kRowBytes + c);
        };
#pragma unroll
        for (int t = 0; t < kStages; t++) issue2(t);
        wait_vmcnt<(kStages - 1) * kLoads>();
        __syncthreads();
        read_a(0, lds_raw, 0);
        read_b(b0, lds_raw, 0, 0);
        for (int kt = 0; kt < n_kt; kt++) {
            const unsigned char *stage = lds_raw + (kt % kStages) * kStageBytes;
#pragma unroll
            for (int ks = 0; ks < kKS; ks++) {
                const int cur = ks & 1, nxt = cur ^ 1;
                read_b(b1, stage, ks, 1);
#pragma unroll
                for (int j = 0; j < kNT; j++)
#pragma unroll
                    for (int i = 0; i < kIT; i++) mma(af[cur][i], b0[j], acc[i][j]);
#pragma unroll
                for (int r = 0; r < kNT; r++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // DS read
                }
                if constexpr (kIT * kNT - kNT > 0) __builtin_amdgcn_sched_group_barrier(0x008, kIT * kNT - kNT, 0);
                if (ks + 1 < kKS) {
                    read_a(nxt, stage, ks + 1);
                    read_b(b0, stage, ks + 1, 0);
#pragma unroll
                    for (int j = 0; j < kNT; j++)
#pragma unroll
                        for (int i = 0; i < kIT; i++) mma(af[cur][i], b1[j], acc[i][kNT + j]);
                    constexpr int kMmas2 = kIT * kNT, kReads2 = kIT + kNT, kPairs2 = kMmas2 < kReads2 ? kMmas2 : kReads2;
#pragma unroll
                    for (int r = 0; r < kPairs2; r++) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    }
                    if constexpr (kMmas2 > kPairs2) __builtin_amdgcn_sched_group_barrier(0x008, kMmas2 - kPairs2, 0);
                    if constexpr (kReads2 > kPairs2) __builtin_amdgcn_sched_group_barrier(0x100, kReads2 - kPairs2, 0);
                } else {
                    __builtin_amdgcn_sched_barrier(0);
                    wait_vmcnt<(kStages - 2) * kLoads>();
                    __syncthreads(); // K-tile kt + 1 is in LDS for everybody, and nobody reads K-tile kt any more
                    issue2(kt + kStages);
                    const unsigned char *next = lds_raw + ((kt + 1) % kStages) * kStageBytes;
                    read_a(nxt, next, 0);
                    read_b(b0, next, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = 0; j < kNT; j++)
#pragma unroll
                        for (int i = 0; i < kIT; i++) mma(af[cur][i], b1[j], acc[i][kNT + j]);
                }
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < kStages; t++) issue(t);
        if (short_wave) wait_vmcnt<(kStages - 1) * kLoadsMin>();
        else wait_vmcnt<(kStages - 1) * kLoadsMax>();
        __syncthreads();
        read_frags(0, lds_raw, 0);
        for (int kt = 0; kt < n_kt; kt++) {
            const unsigned char *stage = lds_raw + (kt % kStages) * kStageBytes;
#pragma unroll
            for (int ks = 0; ks < kKS; ks++) {
                const int cur = ks & 1, nxt = cur ^ 1;
                if (ks + 1 < kKS) {
                    read_frags(nxt, stage, ks + 1);
#pragma unroll
                    for (int j = 0; j < kNTs; j++)
#pragma unroll
                        for (int i = 0; i < kIT; i++) mma(af[cur][i], bf[cur][j], acc[i][j]);
                    {   // order within the step: an LDS fragment read of the next step behind each of the first MFMAs of this one,
                        // so that the reads are in flight under the matrix pipe and none is left to wait for when the next step
                        // begins (left to itself the scheduler issues the reads at the end of the step and the MFMAs wait for them)
                        constexpr int kPerMma = kF32 ? 4 : 1; // MFMA instructions per fragment pair
                        constexpr int kMmas = kIT * kNTs, kReads = kIT + kNTs, kPairs = kMmas < kReads ? kMmas : kReads;
#pragma unroll
                        for (int r = 0; r < kPairs; r++) {
                            __builtin_amdgcn_sched_group_barrier(0x008, kPerMma, 0); // MFMA
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);       // DS read
                        }
                        if constexpr (kMmas > kPairs) __builtin_amdgcn_sched_group_barrier(0x008, (kMmas - kPairs) * kPerMma, 0);
                        if constexpr (kReads > kPairs) __builtin_amdgcn_sched_group_barrier(0x100, kReads - kPairs, 0);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < kSplitJ; j++)
#pragma unroll
                        for (int i = 0; i < kIT; i++) mma(af[cur][i], bf[cur][j], acc[i][j]);
                    __builtin_amdgcn_sched_barrier(0);
                    if (short_wave) wait_vmcnt<(kStages - 2) * kLoadsMin>();
                    else wait_vmcnt<(kStages - 2) * kLoadsMax>();
                    __syncthreads(); // K-tile kt + 1 is in LDS for everybody, and nobody reads K-tile kt any more
                    issue(kt + kStages);
                    read_frags(nxt, lds_raw + ((kt + 1) % kStages) * kStageBytes, 0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = kSplitJ; j < kNTs; j++)
#pragma unroll
                        for (int i = 0; i < kIT; i++) mma(af[cur][i], bf[cur][j], acc[i][j]);
                }
            }
        }
    }
    wait_vmcnt<0>(); // drain the clamped tail loads before the block's LDS is released

    // ---- epilogue.  Accumulator register v of a 32 x 32 tile: row 8 * (v / 4) + 4 * (lane / 32) + v % 4, col lane % 32
    const int col_in = lane & 31;
    const int row_in = (lane >> 5) * 4;
    auto out_row = [&](int i, int v) { return bm0 + wm * kWR + i * 32 + (v >> 2) * 8 + row_in + (v & 3); };
    auto out_col = [&](int j) { return bn0 + wn * (32 * kNT) + j * 32 + col_in; };
    // f16 outputs whose rows are 16-byte aligned go through LDS (the stages are free now): every wavefront lays its 64 x 32 kNT
    // tile out as rows, then stores whole 16-byte pieces of consecutive columns (and, with the SiLU gate, reads the gate the
    // same way) instead of one 2-byte element per lane and accumulator register.
    if constexpr (kEpi == kGemmEpiRopeQkv) {
        // The product of wq|wk|wv never reaches memory: every wavefront lays its f16-rounded tile (tensor.rs:1623-1643) out
        // as rows in LDS and then handles it in 16-byte pieces of 8 consecutive columns, each of which lies within q, k or v
        // of one head: RoPE on q and k in fp32 (transformer.rs:823-856), q as hi + lo f16 halves for the attention kernel, k
        // and v rounded into the cache (tensor.rs:373-376), and v once more transposed, 8 positions per piece.
        const PrefillRopeParams &R = p.rope;
        constexpr int kTW = 32 * kNT;
        constexpr int kPad = (kWaves * kWR * (kTW + 8) * 2 <= kStages * kStageBytes) ? 8 : 0;
        constexpr int kTS = kTW + kPad;
        static_assert(kWaves * kWR * kTS * 2 <= kStages * kStageBytes, "the output tiles reuse the stages");
        __syncthreads(); // every wavefront has read its last fragments
        half_t *tile = reinterpret_cast<half_t *>(lds_raw) + wave * (kWR * kTS);
#pragma unroll
        for (int i = 0; i < kIT; i++)
#pragma unroll
            for (int j = 0; j < kNT; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) tile[(i * 32 + (v >> 2) * 8 + row_in + (v & 3)) * kTS + j * 32 + col_in] = (half_t)acc[i][j][v];
        rope_qkv_from_tile<kWR, kTW, kTS>(tile, lane, bm0 + wm * kWR, bn0 + wn * kTW, M, N, R);
        return;
    }
    if constexpr (kEpi == kGemmEpiF16 || kEpi == kGemmEpiSiluGateF16) {
        if (rows16) { // uniform for the launch
            constexpr int kTW = 32 * kNT; // tile width of a wavefront
            constexpr int kPad = (kWaves * kWR * (kTW + 8) * 2 <= kStages * kStageBytes) ? 8 : 0;
            constexpr int kTS = kTW + kPad; // halves per LDS row
            static_assert(kWaves * kWR * kTS * 2 <= kStages * kStageBytes, "the output tiles reuse the stages");
            constexpr int kChunks = kTW / 8;
            __syncthreads(); // every wavefront has read its last fragments
            half_t *tile = reinterpret_cast<half_t *>(lds_raw) + wave * (kWR * kTS);
#pragma unroll
            for (int i = 0; i < kIT; i++)
#pragma unroll
                for (int j = 0; j < kNT; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++)
                    {
                        half_t o = (half_t)acc[i][j][v]; // tensor.rs:1623-1643
                        if constexpr (kDual) o = to_f16(silu_fast(f16r(acc[i][j][v])) * f16r(acc[i][kNT + j][v])); // tensor.rs:822-832 on the f16 gate
                        tile[(i * 32 + (v >> 2) * 8 + row_in + (v & 3)) * kTS + j * 32 + col_in] = o;
                    }
            half_t *cbase = reinterpret_cast<half_t *>(p.c) + zb * p.stride_c;
#pragma unroll
            for (int it = 0; it < kChunks * kWR / 64; it++) {
                const int idx = it * 64 + lane;
                const int rr = idx / kChunks, ch = idx - rr * kChunks;
                const int r = bm0 + wm * kWR + rr, c = bn0 + wn * kTW + ch * 8;
                if (r < M && c < N) {
                    half8_t o = *reinterpret_cast<const half8_t *>(tile + rr * kTS + ch * 8);
                    const size_t off = (size_t)r * p.ldc + c;
                    if constexpr (kEpi == kGemmEpiSiluGateF16 && !kDual) { // tensor.rs:822-832 on the f16 gate, times the f16-rounded product
                        half8_t g8;
                        if constexpr (kGatePre) g8 = gate_pre[it];
                        else g8 = *reinterpret_cast<const half8_t *>(p.gate + off);
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            const float g = (float)g8[e];
                            o[e] = to_f16(silu_fast(g) * (float)o[e]);
                        }
                    }
                    *reinterpret_cast<half8_t *>(cbase + off) = o;
                }
            }
            return;
        }
    }
    // What the epilogue adds to (the residual, or C itself when accumulating) is loaded in batches of one column
    // tile: C may alias the residual, so a load issued between the stores would wait for the store before it.
    [[maybe_unused]] const float *prev_src = nullptr;
    if constexpr (kEpi == kGemmEpiResAddF32) prev_src = p.residual;
    if constexpr (kEpi == kGemmEpiF32) prev_src = p.accumulate ? reinterpret_cast<const float *>(p.c) + zb * p.stride_c : nullptr;
#pragma unroll
    for (int j = 0; j < kNT; j++) {
        const int c = out_col(j);
        [[maybe_unused]] float16_t prev[kIT];
        if constexpr (kEarlyResidual) {
#pragma unroll
            for (int i = 0; i < kIT; i++) prev[i] = early[i][j];
        } else if constexpr (kDual) {
#pragma unroll
            for (int i = 0; i < kIT; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) prev[i][v] = f16r(acc[i][j][v]);
        } else if constexpr (kEpi == kGemmEpiSiluGateF16) {
#pragma unroll
            for (int i = 0; i < kIT; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int r = out_row(i, v);
                    prev[i][v] = (r < M && c < N) ? (float)p.gate[(size_t)r * p.ldc + c] : 0.0f;
                }
        } else if constexpr (kEpi != kGemmEpiF16) {
#pragma unroll
            for (int i = 0; i < kIT; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int r = out_row(i, v);
                    prev[i][v] = (prev_src != nullptr && r < M && c < N) ? prev_src[(size_t)r * p.ldc + c] : 0.0f;
                }
        }
#pragma unroll
        for (int i = 0; i < kIT; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int r = out_row(i, v);
                if (r < M && c < N) {
                    const float val = acc[i][kDual ? kNT + j : j][v];
                    const size_t off = zb * p.stride_c + (size_t)r * p.ldc + c;
                    if constexpr (kEpi == kGemmEpiF16) {
                        reinterpret_cast<half_t *>(p.c)[off] = (half_t)val; // tensor.rs:1623-1643
                    } else if constexpr (kEpi == kGemmEpiF32) {
                        reinterpret_cast<float *>(p.c)[off] = prev[i][v] + val;
                    } else if constexpr (kEpi == kGemmEpiRopeQkv) {
                        (void)val; // returned above
                    } else if constexpr (kEpi == kGemmEpiSiluGateF16) { // tensor.rs:822-832 on the f16 gate, times the f16-rounded product
                        const float g = prev[i][v];
                        reinterpret_cast<half_t *>(p.c)[off] = to_f16(silu_fast(g) * f16r(val));
                    } else { // kGemmEpiResAddF32: residual add of transformer.rs:442 / :445 on the f16-rounded product
                        reinterpret_cast<float *>(p.c)[off] = prev[i][v] + f16r(val);
                    }
                }
            }
        }
    }
}

bool gemm_f16_dma_supported(const GemmParams &p) {
    const int e = p.f32_operands ? 2 : 1; // halves per element
    if (p.k * e < kDmaMinBK || ((p.k * e) % kDmaMinBK) != 0 || ((p.lda * e) % 8) != 0 || ((p.ldb * e) % 8) != 0) return false;
    if (((p.stride_a * e) % 8) != 0 || ((p.stride_b * e) % 8) != 0) return false;
    if (p.k_seg < 0 || (p.k_seg > 0 && ((p.k % p.k_seg) != 0 || ((p.k_seg * e) % 64) != 0))) return false;
    return p.causal >= 0 && p.causal <= 2;
}

template <int kEpi, int kWavesM, int kNT, int kBK, int kStages, bool kF32 = false, int kIT = 2, bool kDual = false>
static hipError_t launch_dma(const GemmParams &p, hipStream_t s) {
    constexpr int bm = 32 * kIT * kWavesM, bn = 64 * kNT;
    constexpr size_t lds = (size_t)kStages * (bm + (kDual ? 2 : 1) * bn) * kBK * 2;
    static_assert(lds <= 160 * 1024, "LDS of one compute unit");
    static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_f16_dma_kernel<kEpi, kWavesM, kNT, kBK, kStages, kF32, kIT, kDual>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) return attr;
    dim3 grid((p.n + bn - 1) / bn, (p.m + bm - 1) / bm, p.batch);
    hipLaunchKernelGGL((gemm_f16_dma_kernel<kEpi, kWavesM, kNT, kBK, kStages, kF32, kIT, kDual>), grid, dim3(128 * kWavesM), lds, s, p);
    return hipGetLastError();
}

// fp32 operands (always K-tiles of 32 floats, fp32 store / accumulate epilogue)
static hipError_t launch_dma_f32(const GemmParams &p, int tile, hipStream_t s) {
    switch (tile) {
    case 0: return launch_dma<kGemmEpiF32, 2, 2, 64, 2, true>(p, s);
    case 4: return launch_dma<kGemmEpiF32, 2, 2, 64, 4, true>(p, s);
    case 1: return launch_dma<kGemmEpiF32, 4, 2, 64, 3, true>(p, s);
    case 2: return launch_dma<kGemmEpiF32, 4, 3, 64, 2, true>(p, s);
    case 3: return launch_dma<kGemmEpiF32, 4, 4, 64, 2, true>(p, s);
    case 5: return launch_dma<kGemmEpiF32, 2, 1, 64, 6, true>(p, s);
    case 6: return launch_dma<kGemmEpiF32, 1, 1, 64, 10, true, 1>(p, s);
    case 7: return launch_dma<kGemmEpiF32, 1, 1, 64, 8, true, 2>(p, s);
    default: return hipErrorInvalidValue;
    }
}

template <int kEpi>
static hipError_t launch_dma_epi(const GemmParams &p, int tile, hipStream_t s) {
    // K tiles of 64 halves move whole 128-byte lines per row and are preferred where K allows (measured inside a 7B prefill:
    // 256 x 192 with K-tile 64 / 2 stages against K-tile 32 / 4 stages is worth 3 % of the whole forward)
    const bool k64 = p.k % 64 == 0 && (p.k_seg == 0 || p.k_seg % 64 == 0);
    switch (tile) {
    case 0: return launch_dma<kEpi, 2, 2, 64, 2>(p, s);  // 128 x 128, 64 KiB of LDS: two workgroups per compute unit
#ifndef RLH_T4_ARGS
#define RLH_T4_ARGS 2, 2, 64, 4
#endif
    case 4: return launch_dma<kEpi, RLH_T4_ARGS>(p, s);  // 128 x 128, 128 KiB: one workgroup per compute unit, three K-tiles ahead
    case 5: return launch_dma<kEpi, 2, 1, 64, 6>(p, s);  // 128 x 64, 144 KiB: few rows, so twice the workgroups stream the weights
    case 6: return launch_dma<kEpi, 1, 1, 64, 10, false, 1>(p, s);  // 32 x 64, 120 KiB: at most 32 rows, nine weight tiles in flight per workgroup
    case 7: return launch_dma<kEpi, 1, 1, 64, 8, false, 2>(p, s);   // 64 x 64, 128 KiB: at most 64 rows
    case 1: return k64 ? launch_dma<kEpi, 4, 2, 64, 3>(p, s) : launch_dma<kEpi, 4, 2, 32, 4>(p, s);  // 256 x 128
    case 2: return k64 ? launch_dma<kEpi, 4, 3, 64, 2>(p, s) : launch_dma<kEpi, 4, 3, 32, 4>(p, s);  // 256 x 192
    case 3: return k64 ? launch_dma<kEpi, 4, 4, 64, 2>(p, s) : launch_dma<kEpi, 4, 4, 32, 4>(p, s);  // 256 x 256
    default: return hipErrorInvalidValue;
    }
}

static int device_compute_units() {
    static const int n_cu = [] {
        int dev = 0, cu = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev);
        return cu > 0 ? cu : 256;
    }();
    return n_cu;
}

// Tile choice: time ~ (rounds of workgroups over the compute units) x (work per workgroup) / (efficiency of the tile);
// larger tiles are more efficient (less L2 -> LDS traffic per flop) but leave compute units idle on small outputs.
static int choose_tile(const GemmParams &p, double *model_time = nullptr) {
    const int forced = p.tune.tile_plus1 - 1; // -1: by the model below
    if (forced >= 1 && forced <= 3) return forced;
    const int k_halves = p.k * (p.f32_operands ? 2 : 1);
    if (forced == 0 && k_halves % 64 == 0) return 0;
    const int n_cu = device_compute_units();
    const int bms[4] = {128, 256, 256, 256}, bns[4] = {128, 128, 192, 256};
    // relative throughput of a busy compute unit, measured on 7B shapes.  (The 128 x 128 tile of the kernel whose wavefronts
    // split the K-steps, gemm_kgroup.hip, is 1.15 in one round of workgroups, but rating it so here sends products to it in
    // two and three rounds, where it loses: 7B shape 1536 / 2048 rows 26.1 / 30.0 ms to the first token against 24.7 / 28.9,
    // 13B shape 1024 rows 35.6 against 31.2.  It takes over only where this model picks the 128 x 128 tile anyway.)
    const double eff[4] = {1.0, 1.05, 1.23, 1.15};
    int best = -1;
    double best_t = 0.0;
    for (int t = 0; t < 4; t++) {
        if (t == 0 && k_halves % 64 != 0) continue;
        const long blocks = (long)((p.n + bns[t] - 1) / bns[t]) * ((p.m + bms[t] - 1) / bms[t]) * p.batch;
        const long rounds = (blocks + n_cu - 1) / n_cu;
        const double time = (double)rounds * bms[t] * bns[t] / eff[t];
        if (best < 0 || time < best_t) { best = t; best_t = time; }
    }
    // fp32 operands run at a sixteenth of the f16 matrix rate, so what counts there is how evenly the tiles fill the compute
    // units, not the staging: the 128 x 64 tile (tile 5) is a candidate too (7B shape in f32 mode, 384 / 512 prompt rows:
    // 86 -> 65 / 87 -> 67 ms to the first token; its busy-unit throughput measured 0.93 of the 128 x 128 tile's)
    // (products with so few tiles that they are cut along K instead keep the 128 x 128 tile that the cut expects)
    const long tiles128 = (long)((p.n + 127) / 128) * ((p.m + 127) / 128);
    if (p.f32_operands && p.batch == 1 && p.k_seg == 0 && p.causal == 0 && p.m > 128 && k_halves % 64 == 0 && tiles128 > n_cu / 4) {
        const long blocks = (long)((p.n + 63) / 64) * ((p.m + 127) / 128);
        const long rounds = (blocks + n_cu - 1) / n_cu;
        const double time = (double)rounds * 128 * 64 / 0.93;
        if (time < best_t) { best = 5; best_t = time; }
    }
    if (model_time != nullptr) *model_time = best_t;
    return best;
}

// Second step of a split-K product: C = epilogue(sum over the split_k partial sums, in the order of the splits).
template <int kEpi>
__global__ void gemm_split_finish_kernel(GemmParams p, const float *partial, int splits) {
    const size_t per = (size_t)p.m * p.n; // the partial sums are [splits][m][n], n a multiple of 4 here
    const int n4 = p.n / 4;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < (size_t)p.m * n4; i += (size_t)gridDim.x * blockDim.x) {
        const int r = (int)(i / n4), c = (int)(i % n4) * 4;
        const size_t off = (size_t)r * p.ldc + c, woff = i * 4;
        float4_t acc = *reinterpret_cast<const float4_t *>(partial + woff);
        for (int z = 1; z < splits; z++) acc += *reinterpret_cast<const float4_t *>(partial + z * per + woff);
        if constexpr (kEpi == kGemmEpiF16) {
            typedef __attribute__((ext_vector_type(4))) _Float16 half4_t;
            half4_t o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = (half_t)acc[e]; // tensor.rs:1623-1643
            *reinterpret_cast<half4_t *>(reinterpret_cast<half_t *>(p.c) + off) = o;
        } else if constexpr (kEpi == kGemmEpiF32) {
            float4_t *dst = reinterpret_cast<float4_t *>(reinterpret_cast<float *>(p.c) + off);
            *dst = p.accumulate ? *dst + acc : acc;
        } else if constexpr (kEpi == kGemmEpiSiluGateF16) {
            typedef __attribute__((ext_vector_type(4))) _Float16 half4_t;
            const half4_t g4 = *reinterpret_cast<const half4_t *>(p.gate + off);
            half4_t o;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float g = (float)g4[e];
                o[e] = to_f16(silu_fast(g) * f16r(acc[e]));
            }
            *reinterpret_cast<half4_t *>(reinterpret_cast<half_t *>(p.c) + off) = o;
        } else {
            const float4_t res = *reinterpret_cast<const float4_t *>(p.residual + off);
            float4_t o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = res[e] + f16r(acc[e]);
            *reinterpret_cast<float4_t *>(reinterpret_cast<float *>(p.c) + off) = o;
        }
    }
}

// The same second step for the residual epilogue with the row RMSNorm that follows it: one workgroup per row of C adds the
// partial sums in the order of the splits, applies the epilogue, keeps the row in registers, and writes the normalised row
// rounded to f16 as well (the loop structure and the order of additions of rmsnorm_rows_f16_kernel, prefill.hip).
constexpr int kFinishNormVecs = 8; // rows of up to 256 x 4 x 8 floats
__global__ __launch_bounds__(256) void gemm_split_finish_norm_kernel(GemmParams p, const float *partial, int splits) {
    __shared__ float red[16];
    const size_t per = (size_t)p.m * p.n;
    const int r = blockIdx.x, tid = threadIdx.x, n4 = p.n / 4;
    const size_t row = (size_t)r * p.ldc, wrow = (size_t)r * p.n;
    const float4_t *w4 = reinterpret_cast<const float4_t *>(p.norm_w);
    float4_t xv[kFinishNormVecs];
    float ss = 0.0f;
    // the pieces outermost, so that a thread's loads of one piece are all in flight together (per element the partial sums are
    // still added in the order of the pieces)
#pragma unroll
    for (int j = 0; j < kFinishNormVecs; j++) {
        const int i = tid + j * 256;
        xv[j] = i < n4 ? *reinterpret_cast<const float4_t *>(partial + wrow + (size_t)i * 4) : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
    float4_t res[kFinishNormVecs];
#pragma unroll
    for (int j = 0; j < kFinishNormVecs; j++) {
        const int i = tid + j * 256;
        res[j] = i < n4 ? *reinterpret_cast<const float4_t *>(p.residual + row + (size_t)i * 4) : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
    for (int z = 1; z < splits; z++) {
        float4_t part[kFinishNormVecs];
#pragma unroll
        for (int j = 0; j < kFinishNormVecs; j++) {
            const int i = tid + j * 256;
            part[j] = i < n4 ? *reinterpret_cast<const float4_t *>(partial + z * per + wrow + (size_t)i * 4) : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int j = 0; j < kFinishNormVecs; j++) xv[j] += part[j];
    }
#pragma unroll
    for (int j = 0; j < kFinishNormVecs; j++) {
        const int i = tid + j * 256;
        if (i < n4) {
#pragma unroll
            for (int e = 0; e < 4; e++) xv[j][e] = res[j][e] + f16r(xv[j][e]);
            *reinterpret_cast<float4_t *>(reinterpret_cast<float *>(p.c) + row + (size_t)i * 4) = xv[j];
        }
#pragma unroll
        for (int e = 0; e < 4; e++) ss = fmaf(xv[j][e], xv[j][e], ss);
    }
    float4_t wn[kFinishNormVecs]; // requested before the row sum, not after it
#pragma unroll
    for (int j = 0; j < kFinishNormVecs; j++) {
        const int i = tid + j * 256;
        wn[j] = i < n4 ? w4[i] : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
    ss = block_sum(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)p.n + p.norm_eps);
    half_t *yr = p.norm_out + (size_t)r * p.n;
#pragma unroll
    for (int j = 0; j < kFinishNormVecs; j++) {
        const int i = tid + j * 256;
        if (i < n4) {
            const float4_t wv = wn[j];
            typedef __attribute__((ext_vector_type(4))) _Float16 half4_t;
            half4_t o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = to_f16((xv[j][e] * rs) * wv[e]);
            *reinterpret_cast<half4_t *>(yr + i * 4) = o;
        }
    }
}

// Products with few output tiles (few prompt rows) leave most compute units without a workgroup, and what bounds them is
// streaming the weights once: the K range is then cut into split_k pieces that run as separate workgroups (more weight bytes
// in flight, every compute unit busy), their fp32 partial sums go to the caller's workspace and a second small kernel adds
// them and applies the epilogue.  Returns 1 for "run as one product".
static int choose_split_k(const GemmParams &p, int tile) {
    if (p.workspace == nullptr || p.batch != 1 || p.k_seg != 0 || p.causal != 0) return 1;
    const int k_halves = p.k * (p.f32_operands ? 2 : 1);
    if (tile != 0 || (p.n % 4) != 0 || (p.ldc % 4) != 0 || k_halves % 64 != 0) return 1;
    const int forced = p.tune.split_k;
    const int n_cu = device_compute_units();
    const long blocks = (long)((p.n + 127) / 128) * ((p.m + 127) / 128);
    const int k_tiles = k_halves / 64;
    // Worth it while the partial sums (pieces x m x n floats, written and read back) stay small beside the weights: products
    // whose tiles cover at most a quarter of the compute units (measured on the 7B shapes: wq|wk|wv / w1 / w3 on their 86 - 96
    // tiles are faster unsplit on the narrower 128 x 64 tile at any row count, wo / w2 on 32 tiles faster split)
    // -- and, with more than one row tile, products whose tiles cover at most half of them: a 128 x 128 tile takes as long
    // with half the compute units idle as with all of them busy, so two pieces on twice the workgroups nearly halve the product
    // (wo / w2 of the 7B shape at 320 / 384 / 512 rows: 10.0 / 10.7 / 11.1 -> 9.1 / 9.4 / 10.2 ms to the first token; three
    // pieces measured the same as two; at 640 rows and more the tiles fill the part and a cut costs)
    const bool half_ok = !p.tune.no_split_half;
    const long max_blocks = p.m > 128 && half_ok ? n_cu / 2 : n_cu / 4;
    if (blocks > max_blocks && forced <= 1) return 1;
    // a single row tile runs its pieces on the 128 x 64 tile: twice the column tiles, half the pieces, half the partial sums
    const long tiles = p.m <= 128 ? (long)((p.n + 63) / 64) : blocks;
    long s = forced > 1 ? forced : (n_cu + tiles - 1) / tiles;
    if (forced <= 1 && blocks > n_cu / 4) s = 2;
    if (s > k_tiles / 4) s = k_tiles / 4;                  // at least 4 K-tiles per piece
    const size_t per = (size_t)p.m * p.n * sizeof(float);
    if (per > 0 && (size_t)s * per > p.workspace_bytes) s = (long)(p.workspace_bytes / per);
    return s < 2 ? 1 : (int)s;
}

template <int kEpi>
static hipError_t launch_split_finish(const GemmParams &p, int splits, hipStream_t s) {
    const size_t work = (size_t)p.m * (p.n / 4);
    const unsigned blocks = (unsigned)((work + 255) / 256 < 4096 ? (work + 255) / 256 : 4096);
    hipLaunchKernelGGL(gemm_split_finish_kernel<kEpi>, dim3(blocks), dim3(256), 0, s, p, (const float *)p.workspace, splits);
    return hipGetLastError();
}

// Two products in one pass pay off where their workgroups fill the compute units about as well as the best single-product
// tile does.  Returns 0 (two launches), 1 (workgroups of 256 x 192 of both products, eight wavefronts, all of the LDS),
// 2 (128 x 192 of both, four wavefronts: prompts of about 300 to 512 rows, where the 128 x 128 tile of a single product needs two
// rounds of workgroups and this form one) or 3 / 4 / 5 (32 / 64 / 128 rows x 64 columns of both: short prompts).  The model is choose_tile's: rounds of workgroups x outputs per workgroup / relative
// throughput of a busy compute unit, with 1.23 x 1.18 measured for the 256-row form (7B and 13B shapes, 256 to 2048 prompt
// rows: faster from 768 rows on except where the last round is nearly empty) and 0.87 for the 128-row form (7B shape: 3 - 4 % of
// the time to the first token at 384 and 512 rows, slower at 256 and 640).
// *cut_cols (optional) receives a number of columns n1 > 0 when the 256-row form should run on the first n1 columns only
// and the remaining columns as two launches: where the workgroups of the pass make whole rounds and a bit (13B shape, 2048
// rows: 576 = 2.25 rounds of 256), the bit costs a whole round, and as two small products it costs a fraction of one.
static int choose_dual(const GemmParams &p, int *cut_cols = nullptr) {
    if (cut_cols != nullptr) *cut_cols = 0;
    const int mode = p.tune.dual_plus1 - 1; // 0: never, 1 ... 5: that form wherever the kernel can run (tests), -1: by shape
    if (mode == 0 || p.f32_operands || !gemm_f16_dma_supported(p) || p.batch != 1 || p.k_seg != 0 || p.causal != 0 || p.k % 64 != 0) return 0;
    if ((p.ldc % 8) != 0 || (p.n % 8) != 0 || (reinterpret_cast<uintptr_t>(p.c) % 16) != 0) return 0;
    if (mode >= 1 && mode <= 5) return mode;
    // Up to 128 rows both products are bound by streaming their weights once, and one launch whose workgroups each take 64
    // rows of w1 and the same 64 of w3 streams them at the rate of the single-row kernel (7B shape: 29.8 / 34.3 / 40.0 us at
    // 16 / 48 / 128 rows against 41.7 / 49.1 / 60.3 us for two launches on 64 rows per workgroup; the single-row pair: 29.9).
    // Beyond one round of such workgroups (65B shape: 344) only the 32-row form still gains (168 against 184 us).
    if (p.m <= 128) {
        const bool one_round = (p.n + 63) / 64 <= device_compute_units();
        if (p.m <= 32) return 3;
        if (one_round) return p.m <= 64 ? 4 : 5;
    }
    double single = 0.0;
    const int tile = choose_tile(p, &single);
    if (tile < 0 || tile > 3 || choose_split_k(p, tile) != 1) return 0;
    const int n_cu = device_compute_units();
    const long cols = (p.n + 191) / 192;
    const long blocks256 = cols * ((p.m + 255) / 256), blocks128 = cols * ((p.m + 127) / 128);
    const double unit256 = 2.0 * 256 * 192 / (1.23 * 1.18);
    double dual256 = (double)((blocks256 + n_cu - 1) / n_cu) * unit256;
    const double dual128 = (double)((blocks128 + n_cu - 1) / n_cu) * 2.0 * 128 * 192 / 0.87;
    // the 256-row form on the columns that make whole rounds, the rest (at most a quarter of a round of its workgroups) as two
    // launches; 3 us per additional launch in the model's unit (6.2e-7 us x K each)
    const bool cut_ok = !p.tune.no_dual_cut;
    const long rows256 = (p.m + 255) / 256, full = blocks256 / n_cu, cols_main = full * n_cu / rows256;
    int n1 = 0;
    // (from two whole rounds on: with one, 7B shape 1280 rows and 13B shape 1024 rows, the cut measured 3 % slower than without)
    if (cut_ok && cut_cols != nullptr && full >= 2 && cols_main >= 1 && cols_main < cols && (cols - cols_main) * rows256 * 4 <= n_cu) {
        GemmParams r = p;
        r.n = p.n - (int)cols_main * 192;
        r.b2 = nullptr;
        double rest = 0.0;
        const int rt = choose_tile(r, &rest);
        const double launch = 3.0 / (6.2e-7 * p.k);
        const double with_cut = (double)full * unit256 + 2.0 * rest + 2.0 * launch;
        if (rt >= 0 && with_cut < dual256) {
            dual256 = with_cut;
            n1 = (int)cols_main * 192;
        }
    }
    const double best = dual256 <= dual128 ? dual256 : dual128;
    // (10 % in favour of the pass: with three row tiles -- 520 to 768 rows -- it runs on 174 workgroups at a higher clock than
    // the model's unit assumes, 145.6 us at the 7B shape against 84.5 + 77.3 us for two launches of 128 x 128 tiles in two rounds)
    if (best >= 2.0 * single * 1.1) return 0;
    if (dual256 <= dual128 && cut_cols != nullptr) *cut_cols = n1;
    return dual256 <= dual128 ? 1 : 2;
}

bool gemm_f16_dual_gate_supported(const GemmParams &p) {
    int n1 = 0;
    return choose_dual(p, &n1) != 0;
}

// The RoPE epilogue needs whole 16-byte pieces everywhere and an unsplit product (a product cut along K has its epilogue in
// the kernel that adds the partial sums; the caller then stores the product and runs the separate kernel).
bool gemm_f16_rope_supported(const GemmParams &p) {
    if (p.tune.no_rope_epilogue) return false;
    const PrefillRopeParams &R = p.rope;
    if (p.f32_operands || !gemm_f16_dma_supported(p) || p.batch != 1 || p.k_seg != 0 || p.causal != 0 || p.b2 != nullptr) return false;
    if (R.dim <= 0 || R.head_dim <= 0 || p.n != 3 * R.dim || R.n != p.m || R.dim % R.head_dim != 0 || R.head_dim % 8 != 0 || !R.cache_f16) return false;
    if (R.q_stride % 8 != 0 || R.t_pad % 8 != 0 || R.t_pad < p.m || p.m > R.max_seq_len) return false;
    for (const void *q : {(const void *)R.q_hi, (const void *)R.q_lo, (const void *)R.cache_k, (const void *)R.cache_v, (const void *)R.v_t})
        if (q == nullptr || (reinterpret_cast<uintptr_t>(q) % 16) != 0) return false;
    if (R.freqs == nullptr || (reinterpret_cast<uintptr_t>(R.freqs) % 8) != 0) return false;
    return choose_split_k(p, choose_tile(p)) == 1;
}

hipError_t launch_gemm_f16_dma(const GemmParams &p_in, int epilogue, hipStream_t s) {
    if (!gemm_f16_dma_supported(p_in) || p_in.m <= 0 || p_in.n <= 0 || p_in.batch < 1) return hipErrorInvalidValue;
    if (epilogue == kGemmEpiResAddF32 && (p_in.residual == nullptr || p_in.batch != 1)) return hipErrorInvalidValue;
    if (epilogue == kGemmEpiRopeQkv && !gemm_f16_rope_supported(p_in)) return hipErrorInvalidValue;
    if (p_in.b2 != nullptr) {
        int n1 = 0;
        const int dual = epilogue == kGemmEpiSiluGateF16 ? choose_dual(p_in, &n1) : 0;
        if (dual == 1 && n1 > 0) {
            GemmParams left = p_in, right = p_in;
            left.n = n1;
            hipError_t e = launch_dma<kGemmEpiSiluGateF16, 4, 3, 64, 2, false, 2, true>(left, s);
            if (e != hipSuccess) return e;
            // the other columns: w1's product into C, then w3's with C as its gate (every element of the gate is read by the
            // lane that overwrites it)
            right.n = p_in.n - n1;
            right.b = p_in.b + (size_t)n1 * p_in.ldb;
            right.b2 = nullptr;
            right.c = reinterpret_cast<half_t *>(p_in.c) + n1;
            e = launch_gemm_f16_dma(right, kGemmEpiF16, s);
            if (e != hipSuccess) return e;
            right.b = p_in.b2 + (size_t)n1 * p_in.ldb;
            right.gate = reinterpret_cast<const half_t *>(right.c);
            return launch_gemm_f16_dma(right, kGemmEpiSiluGateF16, s);
        }
        if (dual == 1) return launch_dma<kGemmEpiSiluGateF16, 4, 3, 64, 2, false, 2, true>(p_in, s); // 256 x 192 of both products, all of the LDS
        if (dual == 2) return launch_dma<kGemmEpiSiluGateF16, 2, 3, 64, 2, false, 2, true>(p_in, s); // 128 x 192 of both, four wavefronts
        if (dual == 3) return launch_dma<kGemmEpiSiluGateF16, 1, 1, 64, 7, false, 1, true>(p_in, s); // 32 x 64 of both, two wavefronts
        if (dual == 4) return launch_dma<kGemmEpiSiluGateF16, 1, 1, 64, 6, false, 2, true>(p_in, s); // 64 x 64 of both, two wavefronts
        if (dual == 5) return launch_dma<kGemmEpiSiluGateF16, 2, 1, 64, 4, false, 2, true>(p_in, s); // 128 x 64 of both, four wavefronts
        return hipErrorInvalidValue;
    }
    if (epilogue == kGemmEpiSiluGateF16 && (p_in.gate == nullptr || p_in.batch != 1 || p_in.f32_operands)) return hipErrorInvalidValue;
    const int splits = choose_split_k(p_in, choose_tile(p_in));
    if (splits > 1) {
        GemmParams q = p_in;            // the partial sums: split_k pieces as grid.z, fp32 store, C item z = workspace slice z
        q.c = p_in.workspace;
        q.residual = nullptr;
        q.accumulate = 0;
        q.split_k = splits;
        q.batch = splits;
        q.stride_a = q.stride_b = 0;
        q.ldc = p_in.n;
        q.stride_c = (size_t)p_in.m * p_in.n;
        q.workspace = nullptr;
        hipError_t e = launch_gemm_f16_dma(q, kGemmEpiF32, s);
        if (e != hipSuccess) return e;
        if (epilogue == kGemmEpiResAddF32 && p_in.norm_w != nullptr && p_in.norm_out != nullptr && p_in.norm_done != nullptr &&
            p_in.n <= 256 * 4 * kFinishNormVecs && !p_in.tune.no_finish_norm) {
            hipLaunchKernelGGL(gemm_split_finish_norm_kernel, dim3(p_in.m), dim3(256), 0, s, p_in, (const float *)p_in.workspace, splits);
            *p_in.norm_done = 1;
            return hipGetLastError();
        }
        switch (epilogue) {
        case kGemmEpiF16: return launch_split_finish<kGemmEpiF16>(p_in, splits, s);
        case kGemmEpiF32: return launch_split_finish<kGemmEpiF32>(p_in, splits, s);
        case kGemmEpiResAddF32: return launch_split_finish<kGemmEpiResAddF32>(p_in, splits, s);
        case kGemmEpiSiluGateF16: return launch_split_finish<kGemmEpiSiluGateF16>(p_in, splits, s);
        default: return hipErrorInvalidValue;
        }
    }
    const GemmParams &p = p_in;
    int tile = choose_tile(p);
    if (tile == 0) {
        // With at most one workgroup per compute unit anyway, the LDS that a second one would need buys a deeper load
        // pipeline instead (measured on the wo / w2 products of a 1024-token 7B prefill: 108 -> 85 us per launch).
        const long blocks = (long)((p.n + 127) / 128) * ((p.m + 127) / 128) * p.batch;
        if (blocks <= device_compute_units()) tile = 4;
        // one row tile and few column tiles (a short prompt): half the tile width, so that twice the workgroups stream the
        // weights; the pieces of a split product use it too
        if (p.m <= 128 && (p.batch == 1 || p.split_k > 1) && (long)((p.n + 127) / 128) * 2 <= device_compute_units() && p.k_seg == 0 && p.causal == 0) tile = p.m <= 32 ? 6 : p.m <= 64 ? 7 : 5;
    }
    // 128 x 128 or 256 x 192 per workgroup it stays: the kernel whose wavefronts split the K-steps instead of the tile
    if (gemm_f16_kgroup_supported(p, epilogue, tile)) return launch_gemm_f16_kgroup(p, epilogue, tile, s);
    if (p.f32_operands) {
        if (epilogue != kGemmEpiF32 || ((p.k * 2) % 64) != 0 || (p.k_seg != 0 && ((p.k_seg * 2) % 64) != 0)) return hipErrorInvalidValue;
        return launch_dma_f32(p, tile, s);
    }
    switch (epilogue) {
    case kGemmEpiF16: return launch_dma_epi<kGemmEpiF16>(p, tile, s);
    case kGemmEpiF32: return launch_dma_epi<kGemmEpiF32>(p, tile, s);
    case kGemmEpiResAddF32:
        if (p.residual == nullptr || p.batch != 1) return hipErrorInvalidValue;
        return launch_dma_epi<kGemmEpiResAddF32>(p, tile, s);
    case kGemmEpiSiluGateF16: return launch_dma_epi<kGemmEpiSiluGateF16>(p, tile, s);
    case kGemmEpiRopeQkv: return launch_dma_epi<kGemmEpiRopeQkv>(p, tile, s);
    default: return hipErrorInvalidValue;
    }
}

} // namespace rlh
