// 32x32 MFMA wrappers shared by the kernels (gfx950).
//
// A lane owns 8 contraction slots of an operand fragment: slot t of lane-half h = lane/32,
// for operand row (A) or column (B) lane%32.  A and B use the same slot <-> k assignment in
// hardware, so kernels only have to be consistent between the two operands.  The 32x32
// fp32 accumulator gives lane (n = lane%32, h) the 16 values  D[m][n],
// m = 8*(v/4) + 4*h + v%4  for v = 0..15.
#pragma once

#include "common.hpp"

namespace mta {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

template <typename T> struct alignas(sizeof(T) * 8 > 16 ? 16 : sizeof(T) * 8) frag8 { T v[8]; };

__device__ __forceinline__ void mma32(f32x16 &c, const frag8<bf16_t> &a, const frag8<bf16_t> &b)
{
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ void mma32(f32x16 &c, const frag8<f16_t> &a, const frag8<f16_t> &b)
{
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}
// fp32 operands: eight 32x32x2 steps, slot t of both fragments feeding step t
__device__ __forceinline__ void mma32(f32x16 &c, const frag8<float> &a, const frag8<float> &b)
{
#pragma unroll
    for (int t = 0; t < 8; ++t) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[t], b.v[t], c, 0, 0, 0);
}

// 16x16x32 (16-bit operands only).  Lane (r = lane%16, g = lane/16) owns operand row/column r and
// the 8 slots of k-group g; the fp32 accumulator gives it D[m][n] with n = r, m = 4*g + v, v = 0..3.
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void mma16(f32x4 &c, const frag8<bf16_t> &a, const frag8<bf16_t> &b)
{
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ void mma16(f32x4 &c, const frag8<f16_t> &a, const frag8<f16_t> &b)
{
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

template <typename T> __device__ __forceinline__ frag8<T> zero_frag()
{
    frag8<T> f;
#pragma unroll
    for (int t = 0; t < 8; ++t) f.v[t] = from_float<T>(0.0f);
    return f;
}

// Swizzle of a V block in LDS: row `key` stores its 16-byte chunk c at position c ^ v_swizzle(key).  A transpose read
// touches, per group of 16 lanes, 32 contiguous bytes (8 banks) of each of 4 consecutive keys, and groups are 8 keys
// apart: the keys {0..3, 8..11} (+4, +16) that may be served in one cycle must land in 8 different 8-bank regions.
// D = 128 (a row is all 64 banks): region = chunk pair ^ (key%4 + 4*bit 3 of key).  D = 64 (a row is 32 banks, odd keys
// take the other half): region = chunk pair ^ (bit 1 + 2*bit 3 of key).  (XOR with the plain key index put keys 2k and
// 2k+1 into the same region: every transpose read took a two-way bank conflict.)
template <int D> __device__ __forceinline__ int v_swizzle(int key)
{
    if constexpr (D == 128) return 2 * ((key & 3) | ((key >> 1) & 4));
    else return 2 * (((key >> 1) & 1) | ((key >> 2) & 2));
}

}  // namespace mta
