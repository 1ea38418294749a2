// Shared device/host helpers for the MTA forward kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mta_hip.h"

namespace mta {

// ---- 16-bit storage types (raw bits; arithmetic is always done in fp32) ----------
struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }
__device__ __forceinline__ float to_float(f16_t v) { return (float)v.v; }

// round-to-nearest-even fp32 -> bf16 (NaN kept quiet), as torch does
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
// gfx950 converts fp32 -> bf16 (round to nearest even) in hardware; the compiler emits it for this cast
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return __builtin_bit_cast(bf16_t, (__bf16)v); }
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float v) { return f16_t{(_Float16)v}; }

// two fp32 values rounded to the 16-bit type T and packed into one register (a in the low half): one
// v_cvt_pk_* instruction on gfx950
typedef float mta_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 mta_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 mta_f16x2 __attribute__((ext_vector_type(2)));
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b)
{
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((mta_f32x2){a, b}, mta_bf16x2));
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b)
{
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((mta_f32x2){a, b}, mta_f16x2));
}
// the two halves of such a register, widened back to fp32
template <typename T> __device__ __forceinline__ void unpack2(uint32_t r, float &a, float &b);
template <> __device__ __forceinline__ void unpack2<bf16_t>(uint32_t r, float &a, float &b)
{
    a = __uint_as_float(r << 16);
    b = __uint_as_float(r & 0xffff0000u);
}
template <> __device__ __forceinline__ void unpack2<f16_t>(uint32_t r, float &a, float &b)
{
    const mta_f16x2 h = __builtin_bit_cast(mta_f16x2, r);
    a = (float)h[0];
    b = (float)h[1];
}

// value of the I/O dtype nearest to v, as fp32 (models an intermediate stored in T)
template <typename T> __device__ __forceinline__ float round_to(float v) { return to_float(from_float<T>(v)); }

// read element `idx` of an array whose dtype is only known at run time (weights)
__device__ __forceinline__ float load_any(const void *p, int dtype, int64_t idx)
{
    if (dtype == MTA_F32) return ((const float *)p)[idx];
    if (dtype == MTA_BF16) return to_float(((const bf16_t *)p)[idx]);
    return to_float(((const f16_t *)p)[idx]);
}

template <typename T> struct vec_of;  // elements per 16-byte vector
template <> struct vec_of<float> { static constexpr int n = 4; };
template <> struct vec_of<bf16_t> { static constexpr int n = 8; };
template <> struct vec_of<f16_t> { static constexpr int n = 8; };

template <typename T> struct alignas(16) pack16 { T v[vec_of<T>::n]; };

// ---- host-side helpers --------------------------------------------------------------
// ---- the triangular layout of a causal (S,S) score tensor --------------------------------------------------------
// Only what lies on and below the diagonal is stored.  Row p holds 64*(p/64 + 1) elements (keys 0 .. p and padding up
// to the next multiple of 64: every row starts on a 128-byte boundary and a 64-key block that holds an attended key is
// stored whole); the heads of a group of GL heads are interleaved by rows: row p of the group's first head, row p of its
// second head, ...  A workgroup that reads row p of every head of a group reads one contiguous run of memory, and the
// rows that are in flight at one time lie next to each other, which HBM rewards (a copy of the triangle in this layout
// runs at 6.0-6.3 TB/s where four separate planes with rows of S elements give 5.1).
// tri_rowoff(p): elements of one head ahead of row p;  tri_rowlen(p): elements of row p;  a group occupies
// GL*tri_rowoff(S) elements and element (head i of the group, row p, key q <= p) sits at
// GL*tri_rowoff(p) + i*tri_rowlen(p) + q from the group's start.
__host__ __device__ __forceinline__ int tri_rowlen(int p) { return ((p >> 6) + 1) << 6; }
__host__ __device__ __forceinline__ int64_t tri_rowoff(int p)
{
    const int64_t a = p >> 6;
    return ((a * (a + 1)) << 11) + (int64_t)(p & 63) * ((a + 1) << 6);
}
// element offset of (head i of its group, row p, key 0) from the group's start, in 32 bits (groups of up to 2^31 elements)
__device__ __forceinline__ unsigned tri_row_start(int p, int gl, int i)
{
    const unsigned a = (unsigned)p >> 6, len = (a + 1u) << 6;
    return (unsigned)gl * (((a * (a + 1u)) << 11) + ((unsigned)p & 63u) * len) + (unsigned)i * len;
}

inline int dtype_size(int dt) { return dt == MTA_F32 ? 4 : (dt == MTA_BF16 || dt == MTA_F16) ? 2 : 0; }
inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline int launch_status()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? MTA_OK : (int)e;
}

#define MTA_DISPATCH_IO(dt, ...)                                      \
    do {                                                              \
        if ((dt) == MTA_F32) { using io_t = float; __VA_ARGS__; }     \
        else if ((dt) == MTA_BF16) { using io_t = mta::bf16_t; __VA_ARGS__; } \
        else { using io_t = mta::f16_t; __VA_ARGS__; }                \
    } while (0)

// conv_mix16.hip: depthwise conv + dense mixing of groups of 16 heads on the matrix cores; MTA_ERR_UNSUPPORTED when no
// instance covers the arguments
int conv_mix16_dispatch(const void *x, const void *wc, const void *wm, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                        int S, int causal, int fill_upper, int io_dtype, hipStream_t st);
}  // namespace mta
