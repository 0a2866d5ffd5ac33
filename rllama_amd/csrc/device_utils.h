// device_utils.h -- wave64 / LDS building blocks shared by the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rlh {

typedef _Float16 half_t;
typedef __attribute__((ext_vector_type(2))) _Float16 half2_t;
typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(4))) float float4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t uint4_t;

constexpr int kWave = 64;

// f32 -> f16 -> f32 with round-to-nearest-even: the reference's rounding points
// (half::f16::from_f32 / _mm256_cvtps_ph(a, 0), simd_support.rs:50-52, tensor.rs:374-375).
// The conversion goes through as_f32: left to itself hipcc folds an f32 multiply (or multiply-add) whose only use is a conversion
// to f16 into v_fma_mixlo_f16, which rounds the exact product once, to f16, where the reference rounds it to f32 first and to
// f16 after; the two differ for about 6 products in 100000 (counted on the part over 2^24 random pairs).  An empty asm
// statement keeps the value a plain f32 register.
__device__ __forceinline__ float as_f32(float v) {
    asm("" : "+v"(v));
    return v;
}
__device__ __forceinline__ half_t to_f16(float v) { return (half_t)as_f32(v); }
__device__ __forceinline__ float f16r(float v) { return (float)to_f16(v); }

// ---- DPP cross-lane moves (GFX9 encodings) -------------------------------------------------
constexpr int kDppQuadPerm1032 = 0xB1;   // lanes i <-> i^1
constexpr int kDppQuadPerm2301 = 0x4E;   // lanes i <-> i^2
constexpr int kDppRowHalfMirror = 0x141; // lane i of each 8 <- lane 7-i
constexpr int kDppRowMirror = 0x140;     // lane i of each 16 <- lane 15-i
constexpr int kDppRowBcast15 = 0x142;    // lane 15 of each row -> next row
constexpr int kDppRowBcast31 = 0x143;    // lane 31 -> rows 2 and 3

template <int kCtrl, int kRowMask = 0xf>
__device__ __forceinline__ float dpp_add(float v) {
    // lanes whose row is masked out, or whose source lane does not exist, receive 0 and keep v
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, kRowMask, 0xf, false);
    return v + __builtin_bit_cast(float, moved);
}

// Sum over groups of kLanes consecutive lanes (kLanes in {2,4,8,16}); every lane of a group gets the sum.
template <int kLanes>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(kLanes == 1 || kLanes == 2 || kLanes == 4 || kLanes == 8 || kLanes == 16, "group size");
    if constexpr (kLanes >= 2) v = dpp_add<kDppQuadPerm1032>(v);
    if constexpr (kLanes >= 4) v = dpp_add<kDppQuadPerm2301>(v);
    if constexpr (kLanes >= 8) v = dpp_add<kDppRowHalfMirror>(v);
    if constexpr (kLanes >= 16) v = dpp_add<kDppRowMirror>(v);
    return v;
}

// Sum over the whole wavefront; the result is wave-uniform (read from lane 63).
__device__ __forceinline__ float wave_sum(float v) {
    v = group_sum<16>(v);
    v = dpp_add<kDppRowBcast15, 0xa>(v);
    v = dpp_add<kDppRowBcast31, 0xc>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Block-wide sum for blocks of up to 16 waves.  `scratch` needs 16 floats.  All threads get the sum.
__device__ __forceinline__ float block_sum(float v, float *scratch) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int nwaves = (blockDim.x + kWave - 1) / kWave;
    v = wave_sum(v);
    __syncthreads(); // scratch may still be read by a previous call
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.0f;
    for (int i = 0; i < nwaves; i++) total += scratch[i];
    return total;
}

__device__ __forceinline__ float block_max(float v, float *scratch) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int nwaves = (blockDim.x + kWave - 1) / kWave;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int i = 1; i < nwaves; i++) total = fmaxf(total, scratch[i]);
    return total;
}

// 16-byte global loads.  Weights are read exactly once per token and exceed every cache level, so the
// streaming variant marks them non-temporal to keep activations and the KV cache resident in L2/MALL.
template <bool kStream>
__device__ __forceinline__ uint4_t load16(const void *p) {
    if constexpr (kStream) {
        return __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p));
    } else {
        return *reinterpret_cast<const uint4_t *>(p);
    }
}

// One interleaved RoPE pair (transformer.rs:844-847): four products and two sums, each rounded to f32 (no FMA).
__device__ __forceinline__ void rope_pair(float re, float im, float2 f, float &ore, float &oim) {
#pragma clang fp contract(off)
    float p0 = re * f.x;
    float p1 = im * f.y;
    float p2 = re * f.y;
    float p3 = im * f.x;
    ore = p0 - p1;
    oim = p2 + p3;
}

// SiLU (tensor.rs:822-832: v / (1 + exp(-v))) through the hardware exp2 and reciprocal: about 3e-7 relative from the
// libm form, i.e. one f16-rounded product in a few thousand lands on the neighbouring f16 value.  Used where the call
// sits in a GEMM epilogue that every wavefront of the chip runs at the same time (there the libm form costs 6 us per launch).
__device__ __forceinline__ float silu_fast(float v) {
    return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v * -1.44269504088896340736f));
}

// One direct-to-LDS load: lane l's 16 bytes at `src` land at LDS byte address dst + 16 l (dst is wave-uniform and
// travels in M0).  Written as inline assembly on purpose: through the builtin the compiler tracks the load as an LDS
// write and puts s_waitcnt vmcnt(0) in front of every LDS read, which would also wait for the prefetched K-tiles;
// here the waits are placed by hand (vmcnt is decremented in issue order).
__device__ __forceinline__ void dma16(const half_t *src, unsigned dst) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(dst) : "memory");
}

// The same with the address as a wave-uniform base (scalar registers) plus a 32-bit byte offset per lane: half the vector
// registers per load address of the form above.
__device__ __forceinline__ void dma16_base(const half_t *base, unsigned byte_off, unsigned dst) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(byte_off), "s"(base), "s"(dst) : "memory");
}

template <int kN>
__device__ __forceinline__ void wait_vmcnt() { // s_waitcnt vmcnt(kN) only (6-bit count: bits 3:0 and 15:14)
    static_assert(kN >= 0 && kN < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (kN & 0xF) | ((kN >> 4) << 14));
}

} // namespace rlh
