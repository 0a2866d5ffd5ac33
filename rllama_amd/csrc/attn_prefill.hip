// attn_prefill.hip -- causal attention of a multi-token forward at start_pos == 0 on the matrix cores, one kernel:
// scores, mask, softmax and P.V of Noeda/rllama transformer.rs:762-781 (with tensor.rs:496-508 and 479-494) without
// the [n x n] score matrix ever reaching memory.
//
// Numerics.  The reference keeps q (after RoPE) and the probabilities in fp32 and multiplies them with f16 K / V
// widened to fp32.  Here q and P are split into hi + lo f16 halves and both halves go through the MFMA, accumulated in
// fp32, so no rounding point is added; the softmax is evaluated in its streaming form (running maximum m, running sum l,
// rescaled accumulator; exponentials through exp2), which is the same function as exp(s) / sum exp(s) wherever that is
// finite.  The output is
// rounded to f16 where the reference does (transformer.rs:793-796).
//
// Blocking.  Workgroup = 4 wavefronts = 128 queries of one head; a wavefront owns 32 queries and walks the keys in
// tiles of 64 (K tile [64 x hd] and V^T tile [hd x 64] staged in LDS once for the four wavefronts, next tile's global
// loads in flight while the current one is used).  Both products are computed transposed so that every per-query
// quantity lives in one lane pair:
//   S^T [key x query]  = K (A operand, rows = keys)   x  q (B operand, rows = queries), summed over hd
//   O^T [dim x query] += V^T (A operand, rows = dims)  x  P (B operand, rows = queries), summed over keys
// With v_mfma_f32_32x32x16_f16 the accumulator register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4 and column
// l % 32: the column is the query in both products, so max / sum / rescale need one exchange with lane l ^ 32 and no
// other cross-lane traffic.  The 16 probabilities a lane holds for a 32-key group are exactly what it must supply as the
// B operand of the second product if the k slots of that MFMA are assigned to keys in the accumulator's order; V^T is
// read from LDS in the same order (two 8-byte reads per operand).
#include "kernels.h"
#include "device_utils.h"

namespace rlh {

typedef __attribute__((ext_vector_type(16))) float float16_t;
typedef __attribute__((ext_vector_type(4))) _Float16 half4_t;

constexpr int kApQueries = 128; // per workgroup
constexpr int kApKeys = 64;     // per key tile
constexpr int kApThreads = 256;

template <int HD>
__global__ __launch_bounds__(kApThreads) void attn_prefill_kernel(AttnPrefillParams p) {
    constexpr int kKS = HD / 16;                 // MFMA K-steps over the head dimension
    constexpr int kDT = HD / 32;                 // 32-row tiles of O^T
    constexpr int kKRowBytes = HD * 2;           // K tile row (one key)
    constexpr int kKChunks = HD / 8;             // 16-byte chunks per K row
    constexpr int kKTileBytes = kApKeys * kKRowBytes;
    constexpr int kVRowBytes = kApKeys * 2;      // V^T tile row (one dim): 128 bytes
    constexpr int kVTileBytes = HD * kVRowBytes;
    constexpr int kKLoads = kApKeys * kKChunks / kApThreads; // 16-byte chunks per thread and tile
    constexpr int kVLoads = HD * 8 / kApThreads;
    __shared__ __attribute__((aligned(16))) unsigned char lds[kKTileBytes + kVTileBytes];
    unsigned char *lds_k = lds, *lds_v = lds + kKTileBytes;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int head = blockIdx.y;
    const int qblock = blockIdx.x * kApQueries;
    const int q0 = qblock + wave * 32;           // this wavefront's first query
    const int n = p.n;
    const int my_q = q0 + col;                   // the query this lane's accumulator column belongs to

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

    // keys 0 .. qblock + 127 matter to this workgroup (causal), i.e. key tiles 0 .. n_tiles - 1
    const int last_q = min(qblock + kApQueries, n) - 1;
    const int n_tiles = last_q / kApKeys + 1;

    // global -> register staging of one key tile: K rows [key][hd], V^T rows [dim][key]
    uint4_t kreg[kKLoads], vreg[kVLoads];
    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < kKLoads; i++) {
            const int c = tid + i * kApThreads;
            const int row = c / kKChunks, ch = c % kKChunks;
            const int key = min(kt * kApKeys + row, p.max_seq_len - 1); // keys past the sequence are masked below
            kreg[i] = *reinterpret_cast<const uint4_t *>(kbase + (size_t)key * HD + ch * 8);
        }
#pragma unroll
        for (int i = 0; i < kVLoads; i++) {
            const int c = tid + i * kApThreads;
            const int row = c / 8, ch = c % 8;
            vreg[i] = *reinterpret_cast<const uint4_t *>(vbase + (size_t)row * p.t_pad + kt * kApKeys + ch * 8);
        }
    };
    // LDS placement: 16-byte chunk c of row r goes to chunk c ^ f(r), so that the MFMA operand reads of consecutive
    // rows fall into different banks
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < kKLoads; i++) {
            const int c = tid + i * kApThreads;
            const int row = c / kKChunks, ch = c % kKChunks;
            *reinterpret_cast<uint4_t *>(lds_k + row * kKRowBytes + ((ch ^ (row & (kKChunks - 1))) << 4)) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < kVLoads; i++) {
            const int c = tid + i * kApThreads;
            const int row = c / 8, ch = c % 8;
            // rows with bit 4 set keep the two 8-byte halves of every chunk swapped: a half-wave reads one 8-byte half per
            // row of 32 consecutive rows, and rows r and r + 16 would otherwise meet in the same banks
            const uint4_t vv = (row & 16) ? uint4_t{vreg[i][2], vreg[i][3], vreg[i][0], vreg[i][1]} : vreg[i];
            *reinterpret_cast<uint4_t *>(lds_v + row * kVRowBytes + ((ch ^ ((row >> 1) & 7)) << 4)) = vv;
        }
    };

    load_tile(0);
    for (int kt = 0; kt < n_tiles; kt++) {
        __syncthreads(); // everybody is done with the previous tile
        store_tile();
        __syncthreads();
        if (kt + 1 < n_tiles) load_tile(kt + 1);
        const int key0 = kt * kApKeys;
        if (key0 > q0 + 31) continue; // every key of this tile lies after every query of this wavefront (barriers are above)

        // ---- S^T for the two 32-key groups of the tile
        float16_t s_acc[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
            for (int v = 0; v < 16; v++) s_acc[j][v] = 0.0f;
            if (key0 + j * 32 <= q0 + 31) { // wave-uniform: otherwise the whole group is masked
                const int krow = j * 32 + col;
#pragma unroll
                for (int ks = 0; ks < kKS; ks++) {
                    const int ch = ks * 2 + half;
                    const half8_t kf = *reinterpret_cast<const half8_t *>(lds_k + krow * kKRowBytes + ((ch ^ (krow & (kKChunks - 1))) << 4));
                    s_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, q_hi[ks], s_acc[j], 0, 0, 0);
                    s_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, q_lo[ks], s_acc[j], 0, 0, 0);
                }
            }
        }
        // ---- scale (transformer.rs:768-770), causal mask (tensor.rs:496-508: col >= row + 1 is -inf), streaming softmax.
        //      The vector ALU is what this kernel waits for, so the work per score is kept small: the maximum is taken on
        //      the raw scores (the scale is positive), scale and log2(e) are folded into one multiplier of an exp2
        //      (exp(scale s - scale m) = exp2(c s - c m), one fused multiply-add and one v_exp_f32 per score; the
        //      argument error is a few 1e-6 relative in the probability), the mask is applied only on tiles that reach
        //      the diagonal, and the accumulator is rescaled only when some row's maximum moved.
        if (key0 + kApKeys - 1 > q0) { // some key of the tile lies after some query of this wavefront
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int key = key0 + j * 32 + (v >> 2) * 8 + half * 4 + (v & 3);
                    if (key > my_q) s_acc[j][v] = -INFINITY;
                }
        }
        float m_tile = -INFINITY;
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) m_tile = fmaxf(m_tile, s_acc[j][v]);
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
        // the tile holds at least key0 <= q0 <= my_q, so m_tile is finite
        const float c2 = p.scale * 1.44269504088896340736f;
        const float m_new = fmaxf(m_run, m_tile);
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c2); // first tile: exp2(-inf) = 0
        m_run = m_new;
        const float mc = m_new * c2;
        float l_tile = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float e = __builtin_amdgcn_exp2f(fmaf(s_acc[j][v], c2, -mc)); // masked: exp2(-inf) = 0
                s_acc[j][v] = e;
                l_tile += e;
            }
        l_run = l_run * alpha + l_tile; // this lane's half of the row; the halves are added at the end
        if (!__all(alpha == 1.0f)) {
#pragma unroll
            for (int d = 0; d < kDT; d++)
#pragma unroll
                for (int v = 0; v < 16; v++) o_acc[d][v] *= alpha;
        }

        // ---- O^T += V^T . P, probabilities split hi + lo.  k slot i of lane half h in 16-slot slab s of group j is key
        //      32 j + 16 s + 8 (i / 4) + 4 h + i % 4: the order the accumulator holds them in
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if (key0 + j * 32 > q0 + 31) continue; // all probabilities of the group are zero
#pragma unroll
            for (int s = 0; s < 2; s++) {
                half8_t p_hi, p_lo;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float pv = s_acc[j][s * 8 + i];
                    const half_t h = (half_t)pv;
                    p_hi[i] = h;
                    p_lo[i] = (half_t)(pv - (float)h);
                }
                const int kk = j * 32 + s * 16 + half * 4; // first key (within the tile) of this lane's slots 0..3; slots 4..7: + 8
#pragma unroll
                for (int d = 0; d < kDT; d++) {
                    const int vrow = d * 32 + col;
                    const unsigned char *rowp = lds_v + vrow * kVRowBytes;
                    const int sw = (vrow >> 1) & 7;
                    const int sub = (((kk & 4) << 1)) ^ ((vrow & 16) >> 1); // which 8-byte half of the chunk (halves swapped in rows with bit 4 set)
                    const half4_t a0 = *reinterpret_cast<const half4_t *>(rowp + ((((kk) >> 3) ^ sw) << 4) + sub);
                    const half4_t a1 = *reinterpret_cast<const half4_t *>(rowp + ((((kk + 8) >> 3) ^ sw) << 4) + sub);
                    half8_t vf;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        vf[i] = a0[i];
                        vf[4 + i] = a1[i];
                    }
                    o_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, p_hi, o_acc[d], 0, 0, 0);
                    o_acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, p_lo, o_acc[d], 0, 0, 0);
                }
            }
        }
    }

    // ---- normalise, round to f16 (transformer.rs:793-796) and write row my_q, columns head * HD + dim of wo's input
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    if (my_q < n) {
        half_t *orow = reinterpret_cast<half_t *>(p.out) + (size_t)my_q * p.dim + head * HD;
#pragma unroll
        for (int d = 0; d < kDT; d++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                half4_t o;
#pragma unroll
                for (int i = 0; i < 4; i++) o[i] = (half_t)(o_acc[d][g * 4 + i] / l_tot);
                *reinterpret_cast<half4_t *>(orow + d * 32 + g * 8 + half * 4) = o;
            }
    }
}

bool attn_prefill_supported(int head_dim) { return head_dim == 64 || head_dim == 128; }

hipError_t launch_attn_prefill(const AttnPrefillParams &p, hipStream_t s) {
    if (p.n < 1 || p.n_heads < 1 || (p.t_pad % kApKeys) != 0 || p.t_pad < p.n || (p.dim % 4) != 0) return hipErrorInvalidValue;
    dim3 grid((p.n + kApQueries - 1) / kApQueries, p.n_heads);
    switch (p.head_dim) {
    case 64: hipLaunchKernelGGL(attn_prefill_kernel<64>, grid, dim3(kApThreads), 0, s, p); break;
    case 128: hipLaunchKernelGGL(attn_prefill_kernel<128>, grid, dim3(kApThreads), 0, s, p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace rlh
