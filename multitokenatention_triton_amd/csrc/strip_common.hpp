// Helpers shared by the kernels that stage strips of a score plane in LDS with asynchronous copies and read them from
// inline assembly (conv2d_causal.hip, conv_mix16.hip).
#pragma once

#include "common.hpp"

#include <atomic>
#include <type_traits>
#include <utility>

namespace {
using namespace mta;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Returns its argument, opaquely: what is derived from the result cannot be hoisted out of the (rarely taken) block
// that computes it, so it does not occupy registers in the main loop.
__device__ __forceinline__ int opaque(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}

typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;

// LDS is read and written through these, not through C++ accesses: the compiler cannot tell an access to one half of
// the double buffer from the asynchronous copy in flight into the other half and would wait for the copy first (the copy
// would then never overlap the matrix products).  LDS operations of a wavefront complete in order; lds_wait() waits for
// all of them and ties the loaded values to that point.
__device__ __forceinline__ u32x4 lds_load16(unsigned addr)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
// read and wait in one statement: the value is defined when the statement ends (for values that live across code the
// compiler arranges freely)
__device__ __forceinline__ u32x4 lds_load16_sync(unsigned addr)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
// four such reads (1 KB apart, from byte offset `off`: a compile-time constant below 62464) and the wait, one statement
__device__ __forceinline__ void lds_load4x16_sync(unsigned addr, int off, u32x4 &a, u32x4 &b, u32x4 &c, u32x4 &d)
{
    asm volatile("ds_read_b128 %0, %4 offset:%5\n\t"
                 "ds_read_b128 %1, %4 offset:%6\n\t"
                 "ds_read_b128 %2, %4 offset:%7\n\t"
                 "ds_read_b128 %3, %4 offset:%8\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d)
                 : "v"(addr), "n"(off), "n"(off + 1024), "n"(off + 2048), "n"(off + 3072)
                 : "memory");
}
// the same with a compile-time byte offset in the instruction (no address arithmetic per access)
// (`off` must fold to a constant below 65536: it goes into the instruction's offset field)
__device__ __forceinline__ u32x4 lds_load16_at(unsigned addr, int off)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(off) : "memory");
    return v;
}
__device__ __forceinline__ unsigned lds_load_u16(unsigned addr)
{
    unsigned v;
    asm volatile("ds_read_u16 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
__device__ __forceinline__ void lds_store8_at(unsigned addr, int off, unsigned lo, unsigned hi)
{
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 v = {lo, hi};
    asm volatile("ds_write_b64 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(off) : "memory");
}
__device__ __forceinline__ void lds_store16(unsigned addr, u32x4 v)
{
    asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }
__device__ __forceinline__ void lds_wait(u32x4 &a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a) : : "memory"); }
// workgroup barrier without the memory fence __syncthreads() carries (which would wait for the copy in flight)
__device__ __forceinline__ void wg_barrier() { asm volatile("s_barrier" : : : "memory"); }

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), in order
template <int... I, typename F> __device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

inline int device_cu_count()
{
    // (atomic slots: concurrent first calls on a device both query and both store the same value, without a data race)
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

}  // namespace
