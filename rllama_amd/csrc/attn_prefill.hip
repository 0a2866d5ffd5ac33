// attn_prefill.hip -- causal attention of a multi-token forward at start_pos == 0 on the matrix cores, one kernel:
// scores, mask, softmax and P.V of Noeda/rllama transformer.rs:762-781 (with tensor.rs:496-508 and 479-494) without
// the [n x n] score matrix ever reaching memory.
//
// Numerics.  The reference keeps q (after RoPE) and the probabilities in fp32 and multiplies them with f16 K / V
// widened to fp32.  Here q and P are split into hi + lo f16 halves and both halves go through the MFMA, accumulated in
// fp32, so no rounding point is added; the softmax is evaluated in its streaming form (a reference point m that follows the
// running maximum, running sum l, rescaled accumulator; exponentials through exp2), which is the same function as
// exp(s) / sum exp(s) wherever that is finite.  The output is rounded to f16 where the reference does (transformer.rs:793-796).
//
// Blocking.  Workgroup = 2 KQ wavefronts = 64 queries of one head.  Wavefront (g, h) owns the 32 queries of query group g
// and, of every key tile of 32 KQ keys, the 32 keys of key part h; the parts keep their own (m, l, O) and are merged
// through LDS at the end.  Splitting the keys rather than taking more queries gives every SIMD two wavefronts, so that
// one's softmax arithmetic overlaps the other's MFMAs.  KQ = 2 (four wavefronts, 64-key tiles, two workgroups per compute
// unit) is what runs; KQ = 4 (eight wavefronts, 128-key tiles, one workgroup per compute unit, which keeps two wavefronts
// on every SIMD for the whole life of a heavy query block) measured 1 % slower on whole 7B prompts of 1024 and 2048 tokens
// and is kept as the comparison.  The K tile [keys x hd] and the V^T tile [hd x keys] go from global memory straight into LDS
// (global_load_lds, two stages: the next tile's loads are in flight while the current one is used; one barrier per tile).
//
// Where the time goes (7B shape, 1024 rows, 32 us per launch; timing-only builds): without the exponentials 29 us, without
// the lo-half MFMAs 26.5 us, without refilling the tiles 29.5 us, with none of these and no P.V product 16 us -- per tile and
// wavefront about 120 vector instructions and 17 exponentials stand against 32 MFMAs, and a wavefront issues in program order.
// Starting the next tile's score MFMAs ahead of the softmax arithmetic (two score registers sets, K and V^T tiles in rings of
// their own) changed nothing as long as the compiler kept the MFMAs in one block (32.7 us), and forcing them in between the
// vector instructions with scheduling groups ran out of registers (q hi + lo alone take 64); it is not in the code.
//
// Both products are computed transposed so that every per-query quantity lives in one lane pair:
//   S^T [key x query]  = K (A operand, rows = keys)   x  q (B operand, rows = queries), summed over hd
//   O^T [dim x query] += V^T (A operand, rows = dims)  x  P (B operand, rows = queries), summed over keys
// With v_mfma_f32_32x32x16_f16 the accumulator register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4 and column
// l % 32: the column is the query in both products, so max / sum / rescale need one exchange with lane l ^ 32 and no
// other cross-lane traffic.  The 16 probabilities a lane holds for a 32-key group are exactly what it must supply as the
// B operand of the second product if the k slots of that MFMA are assigned to keys in the accumulator's order: slot i
// of lane half h in 16-key slab s is key 16 s + 8 (i / 4) + 4 h + i % 4.  V^T is stored with the keys of every 16-key
// group in the order 0-3, 8-11, 4-7, 12-15 (bits 2 and 3 of the position swapped, see rope_kv_prefill_tiled_kernel), so
// that the 8 keys of a lane half are one 16-byte piece.
#include "kernels.h"
#include "device_utils.h"

#include <type_traits>

namespace rlh {

typedef __attribute__((ext_vector_type(16))) float float16_t;
typedef __attribute__((ext_vector_type(4))) _Float16 half4_t;

constexpr int kApQueries = 64; // per workgroup

template <int HD, int KQ>
__global__ __launch_bounds__(128 * KQ, KQ == 2 ? 2 : 1) void attn_prefill_kernel(AttnPrefillParams p) {
    constexpr int kApKeys = 32 * KQ;              // per key tile
    constexpr int kWaves = 2 * KQ;
    constexpr int kKS = HD / 16;                  // MFMA K-steps over the head dimension
    constexpr int kDT = HD / 32;                  // 32-row tiles of O^T
    constexpr int kKRowBytes = HD * 2;            // K tile row (one key)
    constexpr int kKChunks = HD / 8;              // 16-byte chunks per K row
    constexpr int kKSwzDiv = 16 / kKChunks;       // K rows per 256 bytes of LDS: rows that start in the same bank
    constexpr int kKTileBytes = kApKeys * kKRowBytes;
    constexpr int kVRowBytes = kApKeys * 2;       // V^T tile row (one dim): 8 or 16 chunks
    constexpr int kVChunks = kApKeys / 8;
    constexpr int kVTileBytes = HD * kVRowBytes;
    constexpr int kStageBytes = kKTileBytes + kVTileBytes;
    constexpr int kKIssues = kKTileBytes / (kWaves * 1024);  // wavefront-wide 1 KiB loads per wavefront and tile
    constexpr int kVIssues = kVTileBytes / (kWaves * 1024);
    constexpr int kMergeFloats = 64 * (kDT * 16 + 2); // one key part's (O, m, l), a float per lane and value
    constexpr int kOutRowHalves = HD + 8;         // padded row of the f16 output tile
    constexpr int kOutOffset = 2 * (KQ - 1) * kMergeFloats * 4;
    static_assert(kOutOffset + 2 * 32 * kOutRowHalves * 2 <= 2 * kStageBytes, "epilogue buffers reuse the tile stages");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qg = wave & 1, kh = wave >> 1;      // query group, key part
    const int col = lane & 31, half = lane >> 5;
    const int n = p.n;
    const int n_qblocks = (n + kApQueries - 1) / kApQueries;
    // Heavy query blocks first.  When every workgroup is resident at once (two per compute unit) the second half of the
    // grid runs upwards from the lightest block, so that workgroups b and b + grid / 2 together hold a constant number of
    // key tiles.
    int qi, head;
    {
        const int b = blockIdx.x;
        const int rank = b / p.n_heads;           // 0 .. n_qblocks - 1 in launch order
        head = b - rank * p.n_heads;
        if (p.order == 0) qi = rank;
        else if (p.order == 1) qi = n_qblocks - 1 - rank;
        else {
            const int top = (n_qblocks + 1) / 2;  // blocks taken from the top, descending
            qi = rank < top ? n_qblocks - 1 - rank : rank - top;
        }
    }
    const int qblock = qi * kApQueries;
    const int q0 = qblock + qg * 32;              // this wavefront's first query
    const int my_q = q0 + col;                    // the query this lane's accumulator column belongs to

    const half_t *kbase = reinterpret_cast<const half_t *>(p.cache_k) + (size_t)head * p.max_seq_len * HD;
    const half_t *vbase = reinterpret_cast<const half_t *>(p.v_t) + (size_t)head * HD * p.t_pad;
    const half_t *qbase = reinterpret_cast<const half_t *>(p.q2) + (size_t)head * n * (2 * HD);

    // q as the B operand: lane supplies query row `col`, k = 16 ks + 8 half .. + 8, hi and lo parts
    half8_t q_hi[kKS], q_lo[kKS];
    {
        const half_t *qrow = qbase + (size_t)min(my_q, n - 1) * (2 * HD); // rows past n are clamped; their results are not stored
#pragma unroll
        for (int ks = 0; ks < kKS; ks++) {
            q_hi[ks] = *reinterpret_cast<const half8_t *>(qrow + ks * 16 + half * 8);
            q_lo[ks] = *reinterpret_cast<const half8_t *>(qrow + HD + ks * 16 + half * 8);
        }
    }

    float16_t o_acc[kDT];
#pragma unroll
    for (int d = 0; d < kDT; d++)
#pragma unroll
        for (int v = 0; v < 16; v++) o_acc[d][v] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    // keys 0 .. qblock + 63 matter to this workgroup (causal)
    const int n_tiles = (qblock + kApQueries + kApKeys - 1) / kApKeys;

    // ---- staging.  Load i of wavefront w fills LDS bytes (4 i + w) * 1024 .. + 1024 of the tile; lane l's 16 bytes are
    //      chunk position l % chunks of row l / chunks, which holds the row's chunk (position ^ f(row)): consecutive
    //      rows put the same logical chunk into different banks, which makes the MFMA operand reads conflict-free.
    const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)lds;
    auto v_swz = [](int row) { return kVChunks == 8 ? (row >> 1) & 7 : row & 15; }; // 16 consecutive rows of V^T: 16 distinct 16-byte bank groups
    int k_row[kKIssues], k_off[kKIssues], v_off[kVIssues];
#pragma unroll
    for (int i = 0; i < kKIssues; i++) {
        const int L = (i * kWaves + wave) * 64 + lane;
        const int row = L / kKChunks, cp = L % kKChunks;
        k_row[i] = row;
        k_off[i] = (cp ^ ((row / kKSwzDiv) & (kKChunks - 1))) * 8;
    }
#pragma unroll
    for (int i = 0; i < kVIssues; i++) {
        const int L = (i * kWaves + wave) * 64 + lane;
        const int row = L / kVChunks, cp = L % kVChunks;
        v_off[i] = row * p.t_pad + (cp ^ v_swz(row)) * 8;
    }
    auto issue = [&](int kt) {
        const unsigned dst = lds_base + (unsigned)(kt & 1) * kStageBytes + (unsigned)wave * 1024;
#pragma unroll
        for (int i = 0; i < kKIssues; i++) {
            const int key = min(kt * kApKeys + k_row[i], p.max_seq_len - 1); // keys past the sequence are masked below
            dma16(kbase + (size_t)key * HD + k_off[i], dst + i * (kWaves * 1024));
        }
#pragma unroll
        for (int i = 0; i < kVIssues; i++) dma16(vbase + (size_t)(kt * kApKeys) + v_off[i], dst + kKTileBytes + i * (kWaves * 1024));
    };

    const float c2 = p.scale * 1.44269504088896340736f;
    // One key tile; `stage` is a compile-time constant at both call sites, so that every LDS address of the tile is the lane's
    // base plus an immediate offset.
    auto tile_step = [&](int kt, auto stage) {
        wait_vmcnt<0>();  // this wavefront's part of tile kt has landed
        __syncthreads();  // ... and everybody's; everybody is done with tile kt - 1, whose stage is loaded next
        if (kt + 1 < n_tiles) issue(kt + 1);
        const int kg = kt * kApKeys + kh * 32; // first key of this wavefront's group
        if (kg > q0) return;                   // (both are multiples of 32) every key lies after every query: all masked
        const unsigned char *lds_k = lds + decltype(stage)::value * kStageBytes, *lds_v = lds_k + kKTileBytes;

        // ---- S^T for the 32-key group
        float16_t s_acc;
#pragma unroll
        for (int v = 0; v < 16; v++) s_acc[v] = 0.0f;
        {
            const int krow = kh * 32 + col;
            const unsigned char *rowp = lds_k + krow * kKRowBytes;
            const int sw = (krow / kKSwzDiv) & (kKChunks - 1);
#pragma unroll
            for (int ks = 0; ks < kKS; ks++) {
                const half8_t kf = *reinterpret_cast<const half8_t *>(rowp + (((ks * 2 + half) ^ sw) << 4));
                s_acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, q_hi[ks], s_acc, 0, 0, 0);
                s_acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, q_lo[ks], s_acc, 0, 0, 0);
            }
        }
        // ---- scale (transformer.rs:768-770), causal mask (tensor.rs:496-508: col >= row + 1 is -inf), streaming softmax.
        //      The work per score is kept small: the maximum is taken on the raw scores (the scale is positive), scale
        //      and log2(e) are folded into one multiplier of an exp2 (exp(scale s - scale m) = exp2(c s - c m), one fused
        //      multiply-add and one v_exp_f32 per score; the argument error is a few 1e-6 relative in the probability),
        //      the mask is applied only on groups that reach the diagonal, and the accumulator is rescaled only when
        //      some row's maximum moved.
        if (kg + 31 > q0) { // some key of the group lies after some query of this wavefront
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int key = kg + (v >> 2) * 8 + half * 4 + (v & 3);
                if (key > my_q) s_acc[v] = -INFINITY;
            }
        }
        float m_tile = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; v++) m_tile = fmaxf(m_tile, s_acc[v]);
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
        // the group holds key kg <= q0 <= my_q, so m_tile is finite.  The reference point m_run of the exponentials follows the
        // running maximum lazily: it moves (and the sums so far are rescaled) only when some row's maximum has grown by more than
        // 8 in the exponent of 2, so probabilities are at most 2^8 -- any reference point gives the same softmax, the hi + lo
        // halves keep their relative precision, and the 64 multiplications of the accumulator leave the common path (with an
        // exact running maximum some row of the 32 finds a new one in nearly every tile)
        const float m_new = fmaxf(m_run, m_tile);
        if (__any((m_new - m_run) * c2 > 8.0f)) { // first group: inf
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c2); // first group: exp2(-inf) = 0
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int d = 0; d < kDT; d++)
#pragma unroll
                for (int v = 0; v < 16; v++) o_acc[d][v] *= alpha;
        }
        const float mc = m_run * c2;
        float l_tile = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float e = __builtin_amdgcn_exp2f(fmaf(s_acc[v], c2, -mc)); // masked: exp2(-inf) = 0
            s_acc[v] = e;
            l_tile += e;
        }
        l_run += l_tile; // this lane's half of the row; the halves are added at the end

        // ---- O^T += V^T . P, probabilities split hi + lo
#pragma unroll
        for (int s = 0; s < 2; s++) {
            // hi = the probability rounded towards zero, lo = the rest (exact in fp32, then rounded): hi + lo carries 22
            // bits whichever way hi is rounded, and the packed conversion makes two halves per instruction
            half8_t p_hi, p_lo;
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const float pa = s_acc[s * 8 + i], pb = s_acc[s * 8 + i + 1];
                const half2_t h = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(pa, pb));
                const half2_t l = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_pkrtz(pa - (float)h[0], pb - (float)h[1]));
                p_hi[i] = h[0];
                p_hi[i + 1] = h[1];
                p_lo[i] = l[0];
                p_lo[i + 1] = l[1];
            }
            const int ch = (kh * 2 + s) * 2 + half; // the chunk of the V^T row that holds this lane half's 8 keys
#pragma unroll
            for (int d = 0; d < kDT; d++) {
                const int vrow = d * 32 + col;
                const half8_t vf = *reinterpret_cast<const half8_t *>(lds_v + vrow * kVRowBytes + ((ch ^ v_swz(vrow)) << 4));
                o_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, p_hi, o_acc[d], 0, 0, 0);
                o_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, p_lo, o_acc[d], 0, 0, 0);
            }
        }
    };
    issue(0);
    for (int kt = 0; kt < n_tiles; kt += 2) {
        tile_step(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < n_tiles) tile_step(kt + 1, std::integral_constant<int, 1>{});
    }

    // ---- merge the key parts: wavefronts (g, 1 ..) hand (O, m, l) to wavefront (g, 0) through LDS
    __syncthreads(); // every wavefront is done with the tiles (all loads were waited for above)
    float *mb = reinterpret_cast<float *>(lds) + qg * ((KQ - 1) * kMergeFloats) + lane;
    if (kh > 0) {
        float *mine = mb + (kh - 1) * kMergeFloats;
#pragma unroll
        for (int d = 0; d < kDT; d++)
#pragma unroll
            for (int v = 0; v < 16; v++) mine[(d * 16 + v) * 64] = o_acc[d][v];
        mine[(kDT * 16) * 64] = m_run;
        mine[(kDT * 16 + 1) * 64] = l_run;
    }
    __syncthreads();
    if (kh > 0) return;
    {
        // m_run is finite (key 0 <= every query); another part's maximum is -inf if it saw no key
        float m = m_run;
#pragma unroll
        for (int j = 0; j < KQ - 1; j++) m = fmaxf(m, mb[j * kMergeFloats + (kDT * 16) * 64]);
        float a[KQ];
        a[0] = __builtin_amdgcn_exp2f((m_run - m) * c2);
        float l_half = l_run * a[0];
#pragma unroll
        for (int j = 0; j < KQ - 1; j++) {
            a[j + 1] = __builtin_amdgcn_exp2f((mb[j * kMergeFloats + (kDT * 16) * 64] - m) * c2);
            l_half += mb[j * kMergeFloats + (kDT * 16 + 1) * 64] * a[j + 1];
        }
        const float l_tot = l_half + __shfl_xor(l_half, 32, 64);
#pragma unroll
        for (int j = 0; j < KQ; j++) a[j] = a[j] / l_tot;
        // normalise, round to f16 (transformer.rs:793-796) and turn O^T into rows of the output through LDS, so that
        // the stores to memory are whole 16-byte pieces of consecutive columns
        half_t *ot = reinterpret_cast<half_t *>(lds + kOutOffset) + qg * (32 * kOutRowHalves);
#pragma unroll
        for (int d = 0; d < kDT; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                half4_t o;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float sum = o_acc[d][g * 4 + i] * a[0];
#pragma unroll
                    for (int j = 0; j < KQ - 1; j++) sum += mb[j * kMergeFloats + (d * 16 + g * 4 + i) * 64] * a[j + 1];
                    o[i] = to_f16(sum);
                }
                *reinterpret_cast<half4_t *>(ot + col * kOutRowHalves + d * 32 + g * 8 + half * 4) = o;
            }
        // rows q0 .. q0 + 31, columns head * HD .. + HD of wo's input
        half_t *obase = reinterpret_cast<half_t *>(p.out) + (size_t)head * HD;
#pragma unroll
        for (int i = 0; i < 32 * kKChunks / 64; i++) {
            const int c = i * 64 + lane;
            const int r = c / kKChunks, ch = c % kKChunks;
            if (q0 + r < n)
                *reinterpret_cast<half8_t *>(obase + (size_t)(q0 + r) * p.dim + ch * 8) = *reinterpret_cast<const half8_t *>(ot + r * kOutRowHalves + ch * 8);
        }
    }
}

bool attn_prefill_supported(int head_dim) { return head_dim == 64 || head_dim == 128; }

hipError_t launch_attn_prefill(const AttnPrefillParams &p, hipStream_t s) {
    // four wavefronts on key tiles of 64; t_pad covers whole key tiles
    if (p.n < 1 || p.n_heads < 1 || (p.t_pad % 64) != 0 || p.t_pad < p.n || (p.dim % 8) != 0 || p.max_seq_len < 1) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((p.n + kApQueries - 1) / kApQueries * p.n_heads));
    if (p.head_dim == 64) hipLaunchKernelGGL((attn_prefill_kernel<64, 2>), grid, dim3(256), 0, s, p);
    else if (p.head_dim == 128) hipLaunchKernelGGL((attn_prefill_kernel<128, 2>), grid, dim3(256), 0, s, p);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

} // namespace rlh
