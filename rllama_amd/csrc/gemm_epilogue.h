// gemm_epilogue.h -- epilogue steps shared by the prefill GEMM kernels (gemm_dma.hip, gemm_kgroup.hip).
#pragma once

#include "kernels.h"
#include "device_utils.h"

namespace rlh {

// What becomes of a wavefront's [kRows x kTW] piece of the f16-rounded wq|wk|wv product, laid out as rows of kTS halves in
// LDS at `tile` (first row = position wr0, first column wc0 of the [m x 3 dim] product): handled in 16-byte pieces of 8
// consecutive columns, each of which lies within q, k or v of one head -- RoPE on q and k in fp32 (transformer.rs:823-856), q
// as hi + lo f16 halves for the attention kernel, k and v rounded into the cache (tensor.rs:373-376), and v once more
// transposed, 8 positions per piece.
template <int kRows, int kTW, int kTS>
__device__ __forceinline__ void rope_qkv_from_tile(const half_t *tile, int lane, int wr0, int wc0, int M, int N, const PrefillRopeParams &R) {
    constexpr int kChunks = kTW / 8;
    const int d = R.dim, hd = R.head_dim, half_hd = hd / 2;
    half_t *qhi = reinterpret_cast<half_t *>(R.q_hi), *qlo = reinterpret_cast<half_t *>(R.q_lo);
    half_t *ck = reinterpret_cast<half_t *>(R.cache_k), *cv = reinterpret_cast<half_t *>(R.cache_v);
#pragma unroll
    for (int it = 0; it < kChunks * kRows / 64; it++) {
        const int idx = it * 64 + lane;
        const int rr = idx / kChunks, ch = idx - rr * kChunks;
        const int r = wr0 + rr, c = wc0 + ch * 8;
        if (r < M && c < N) {
            const half8_t o = *reinterpret_cast<const half8_t *>(tile + rr * kTS + ch * 8);
            const int part = c / d, cin = c - part * d; // 0 q, 1 k, 2 v
            const int head = cin / hd, d0 = cin - head * hd;
            const size_t co = ((size_t)head * R.max_seq_len + r) * hd + d0;
            if (part == 2) {
                *reinterpret_cast<half8_t *>(cv + co) = o;
            } else {
                const float2 *fr = R.freqs + (size_t)r * half_hd + d0 / 2;
                half8_t hi, lo;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float a, b;
                    rope_pair((float)o[2 * e], (float)o[2 * e + 1], fr[e], a, b);
                    hi[2 * e] = (half_t)a;
                    hi[2 * e + 1] = (half_t)b;
                    lo[2 * e] = (half_t)(a - (float)hi[2 * e]);
                    lo[2 * e + 1] = (half_t)(b - (float)hi[2 * e + 1]);
                }
                if (part == 0) {
                    const size_t qo = ((size_t)head * M + r) * R.q_stride + d0;
                    *reinterpret_cast<half8_t *>(qhi + qo) = hi;
                    *reinterpret_cast<half8_t *>(qlo + qo) = lo;
                } else {
                    *reinterpret_cast<half8_t *>(ck + co) = hi; // the rotated k rounded to f16
                }
            }
        }
    }
    // V^T [dim][t_pad]: 8 consecutive (stored) positions of one column per piece; eight lanes cover the 64 positions of a
    // column, i.e. 128 contiguous bytes.  Rows past m hold copies of the last row (finite), which is what the padding of
    // V^T needs.  With vt_swap the stored order within every 16 positions has bits 2 and 3 of the position exchanged.
    if (wc0 + kTW > 2 * d) {
        half_t *vt = reinterpret_cast<half_t *>(R.v_t);
        constexpr int kPieces = kRows / 8;
#pragma unroll
        for (int it = 0; it < kTW * kPieces / 64; it++) {
            const int idx = it * 64 + lane;
            const int cc = idx / kPieces, j = idx - cc * kPieces;
            const int c = wc0 + cc, pos0 = wr0 + j * 8;
            if (c >= 2 * d && c < N && pos0 < R.t_pad) {
                half8_t o;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int rs = j * 8 + e;
                    const int src = R.vt_swap ? (rs & ~12) | ((rs & 4) << 1) | ((rs & 8) >> 1) : rs;
                    o[e] = tile[src * kTS + cc];
                }
                *reinterpret_cast<half8_t *>(vt + (size_t)(c - 2 * d) * R.t_pad + pos0) = o;
            }
        }
    }
}

} // namespace rlh
