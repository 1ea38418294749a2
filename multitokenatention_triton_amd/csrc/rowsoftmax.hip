// Fused  head-mix -> causal row softmax -> head-mix  over an (N,C,P,Q) score tensor.
//
// One workgroup owns one query row p of one mixing group (G heads) of one batch
// entry.  The G x Q row segment is read once (only q <= p when causal), mixed with
// w1 in fp32, kept in registers through the max / sum reductions, normalised, mixed
// with w2 and written once.  This is one pass over the tensor where the unfused
// pipeline makes three or four, and it removes the fp32 copy of the score tensor
// that a float softmax of a 16-bit tensor would materialise.
//
// Rounding points of the unfused pipeline in a 16-bit dtype are reproduced: the
// mixed scores and the probabilities are rounded to the I/O dtype before they are
// used again.
#include <stdlib.h>

#include <type_traits>

#include "common.hpp"

constexpr int RS_OCC = 5;  // wavefronts per SIMD the G*NV = 8 instances (e.g. 4 heads x 4096 keys) are compiled for

namespace mta {
// rowsoftmax_dense16.hip: the same pass for groups of 16 heads, both mixes on the matrix cores
int mix16_softmax_launch(const void *x, const void *w1, const void *w2, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                         int causal, int fill_upper, int io_dtype, int w_dtype, hipStream_t st, int tri_in = 0, int tri_out = 0,
                         const float *key_bias = nullptr, const int *row_lo = nullptr);
}  // namespace mta

namespace {
using namespace mta;

template <typename T, int VEC> struct alignas(sizeof(T) * VEC) vecN { T v[VEC]; };

// a and b rounded to the I/O dtype (one packed convert for the 16-bit types)
template <typename T> __device__ __forceinline__ void round_pair(float &a, float &b)
{
    if constexpr (sizeof(T) == 2) {
        unpack2<T>(pack2<T>(a, b), a, b);
    }
}
// a.lo*b.lo + a.hi*b.hi + c for two packed pairs of the 16-bit type T, accumulated in fp32 (one v_dot2c instruction)
template <typename T> __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
{
    if constexpr (sizeof(T) != 2) {
        return c;
    } else if constexpr (std::is_same<T, bf16_t>::value) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(mta_bf16x2, a), __builtin_bit_cast(mta_bf16x2, b), c, false);
    } else {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(mta_f16x2, a), __builtin_bit_cast(mta_f16x2, b), c, false);
    }
}

// VEC fp32 values -> a vector of the I/O dtype
template <typename T, int VEC> __device__ __forceinline__ void pack_vec(const float (&f)[VEC], vecN<T, VEC> &out)
{
    if constexpr (sizeof(T) == 2 && VEC % 2 == 0) {
        uint32_t r[VEC / 2];
#pragma unroll
        for (int u = 0; u < VEC / 2; ++u) r[u] = pack2<T>(f[2 * u], f[2 * u + 1]);
        __builtin_memcpy(&out, r, sizeof(out));
    } else {
#pragma unroll
        for (int u = 0; u < VEC; ++u) out.v[u] = from_float<T>(f[u]);
    }
}

// the tensor is streamed: every element is read once and written once
template <typename V> __device__ __forceinline__ V load_stream(const V *src)
{
    if constexpr (sizeof(V) == 16) {
        typedef unsigned int u4 __attribute__((ext_vector_type(4)));
        return __builtin_bit_cast(V, __builtin_nontemporal_load(reinterpret_cast<const u4 *>(src)));
    } else {
        return *src;
    }
}
template <typename V> __device__ __forceinline__ void store_stream(V *dst, const V &v)
{
    if constexpr (sizeof(V) == 16) {
        typedef unsigned int u4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(__builtin_bit_cast(u4, v), reinterpret_cast<u4 *>(dst));
    } else {
        *dst = v;
    }
}

template <int NT> __device__ __forceinline__ float block_max(float v, float *red)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    constexpr int NW = NT / 64;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) r = fmaxf(r, red[i]);
    __syncthreads();
    return r;
}

template <int NT> __device__ __forceinline__ float block_sum(float v, float *red)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    constexpr int NW = NT / 64;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) r += red[i];
    __syncthreads();
    return r;
}

// Register-resident row: Q <= NT*VEC*NV.
// (KB: with a key bias and / or a first visible key per query row.  An instantiation of its own, compiled without the
// occupancy target: the bias vector costs the registers that target leaves none of.)
template <typename T, int G, int NV, int VEC, int NT, bool KB>
__global__ __launch_bounds__(NT, (!KB && NT == 256 && G * NV == 8) ? RS_OCC : 1) void mix_softmax_mix(const T *__restrict__ x, const void *__restrict__ w1,
                                                      const void *__restrict__ w2, const float *__restrict__ kb,
                                                      T *__restrict__ y, int C, int P, int Q, int causal,
                                                      int w_dtype, int fill_upper, const int *__restrict__ row_lo)
{
    __shared__ float w1s[G * G];
    __shared__ float w2s[G * G];
    __shared__ uint32_t w2p[G * (G / 2) + 1];  // w2 as packed pairs of the I/O dtype: (w2[o][2j], w2[o][2j+1])
    __shared__ float red[2][(NT / 64) * G];  // [0] maxima, [1] sums: no barrier needed between the two uses
    const int tid = threadIdx.x;
    const int groups = C / G;
    int64_t b = blockIdx.x;
    const int p = (int)(b % P); b /= P;
    const int g = (int)(b % groups);
    const int64_t n = b / groups;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base = (n * C + (int64_t)g * G) * plane + (int64_t)p * Q;
    const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;  // last attended key
    using V = vecN<T, VEC>;

    // All row loads are issued first, unconditionally within a wavefront (a lane beyond the attended keys re-reads
    // the row start), so that they overlap each other and the weight fetch below.  Pass k of wavefront w covers
    // keys [(k*NT + 64w)*VEC, +64*VEC); a pass wholly beyond the attended keys (a wavefront-uniform condition) is
    // skipped everywhere below: the arithmetic follows the triangle, not the square.
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    auto dead = [&](int k) { return (k * NT + wave * 64) * VEC > last; };
    // band mask: the keys ahead of the row's first visible one are hidden; a pass wholly ahead of it is neither read nor
    // computed (its outputs are +0)
    int lo = 0;
    if constexpr (KB) {
        if (row_lo) lo = row_lo[n * P + p];
    }
    auto hid = [&](int k) { return KB && (k * NT + wave * 64 + 64) * VEC <= lo; };
    auto gone = [&](int k) { return dead(k) || hid(k); };
    V xin[NV][G];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        if (gone(k)) continue;
        const int q = (k * NT + tid) * VEC;
        const int qs = (q <= last) ? q : 0;
#pragma unroll
        for (int i = 0; i < G; ++i) xin[k][i] = load_stream(reinterpret_cast<const V *>(x + base + i * plane + qs));
    }
    for (int t = tid; t < G * G; t += NT) {
        const int64_t widx = (int64_t)(g * G + t / G) * C + g * G + t % G;
        w1s[t] = w1 ? load_any(w1, w_dtype, widx) : (t / G == t % G ? 1.0f : 0.0f);
        w2s[t] = w2 ? load_any(w2, w_dtype, widx) : (t / G == t % G ? 1.0f : 0.0f);
    }
    // 16-bit I/O with weights of the same dtype: the second mix runs on packed dot products.  The probabilities are
    // rounded to the I/O dtype in pairs of heads (the rounding the unfused pipeline applies to them) and each output is
    // G/2 v_dot2c instructions instead of G fused multiply-adds plus unpacking.
    constexpr bool DOT_OK = sizeof(T) == 2 && G % 2 == 0;
    const bool use_dot = DOT_OK && w2 && w_dtype == (std::is_same<T, bf16_t>::value ? MTA_BF16 : MTA_F16);
    if constexpr (DOT_OK) {
        if (use_dot) {
            for (int t = tid; t < G * (G / 2); t += NT) {
                const int o = t / (G / 2), j = t % (G / 2);
                const int64_t widx = (int64_t)(g * G + o) * C + g * G + 2 * j;
                w2p[t] = pack2<T>(load_any(w2, w_dtype, widx), load_any(w2, w_dtype, widx + 1));
            }
        }
    }
    __syncthreads();

    float s[G][NV][VEC];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        if (gone(k)) continue;
        const int q = (k * NT + tid) * VEC;
#pragma unroll
        for (int o = 0; o < G; ++o) {
#pragma unroll
            for (int u = 0; u < VEC; ++u) {
                float acc;
                if (w1) {
                    acc = 0.0f;
#pragma unroll
                    for (int i = 0; i < G; ++i) acc = fmaf(w1s[o * G + i], to_float(xin[k][i].v[u]), acc);
                } else {
                    acc = to_float(xin[k][o].v[u]);
                }
                s[o][k][u] = acc;
            }
            if (w1) {
                if constexpr (VEC % 2 == 0) {
#pragma unroll
                    for (int u = 0; u < VEC; u += 2) round_pair<T>(s[o][k][u], s[o][k][u + 1]);
                } else {
#pragma unroll
                    for (int u = 0; u < VEC; ++u) s[o][k][u] = round_to<T>(s[o][k][u]);
                }
            }
        }
        if constexpr (KB) {
            if (kb) {  // additive key bias of this batch entry (0 / -inf for a key mask), added in the I/O dtype
                const int qs = (q <= last) ? q : 0;
                float kbv[VEC];
#pragma unroll
                for (int u = 0; u < VEC; ++u) kbv[u] = kb[n * Q + qs + u];
#pragma unroll
                for (int o = 0; o < G; ++o) {
#pragma unroll
                    for (int u = 0; u < VEC; ++u) s[o][k][u] += kbv[u];
                    if constexpr (VEC % 2 == 0) {
#pragma unroll
                        for (int u = 0; u < VEC; u += 2) round_pair<T>(s[o][k][u], s[o][k][u + 1]);
                    } else {
#pragma unroll
                        for (int u = 0; u < VEC; ++u) s[o][k][u] = round_to<T>(s[o][k][u]);
                    }
                }
            }
            if (row_lo) {  // band mask: the keys ahead of the row's first visible one are hidden
                if (q < lo) {
#pragma unroll
                    for (int o = 0; o < G; ++o)
#pragma unroll
                        for (int u = 0; u < VEC; ++u)
                            if (q + u < lo) s[o][k][u] = -INFINITY;
                }
            }
        }
        if (q + VEC - 1 > last) {  // the vector that straddles the last attended key, and those beyond it
#pragma unroll
            for (int o = 0; o < G; ++o)
#pragma unroll
                for (int u = 0; u < VEC; ++u)
                    if (q + u > last) s[o][k][u] = -INFINITY;
        }
    }

    // row maxima and sums of all G heads are reduced together: two barriers per reduction, not 2*G
    constexpr int NW = NT / 64;
    float m[G], inv[G];
#pragma unroll
    for (int o = 0; o < G; ++o) {
        float v = -INFINITY;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (gone(k)) continue;
#pragma unroll
            for (int u = 0; u < VEC; ++u) v = fmaxf(v, s[o][k][u]);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
        if (lane == 0) red[0][wave * G + o] = v;
    }
    __syncthreads();
#pragma unroll
    for (int o = 0; o < G; ++o) {
        float v = red[0][o];
#pragma unroll
        for (int i = 1; i < NW; ++i) v = fmaxf(v, red[0][i * G + o]);
        m[o] = v;
    }
#pragma unroll
    for (int o = 0; o < G; ++o) {
        float sum = 0.0f;
        // exp(s - m) = exp2(s*log2(e) - m*log2(e)): one fused multiply-add and one v_exp per element (m is finite
        // unless a key bias hides every attended key of the row, which gives NaN as a softmax of all -inf does;
        // s = -inf gives 0)
        constexpr float LOG2E = 1.4426950408889634f;
        const float mneg = -m[o] * LOG2E;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (gone(k)) continue;
#pragma unroll
            for (int u = 0; u < VEC; ++u) {
                const float e = __builtin_amdgcn_exp2f(fmaf(s[o][k][u], LOG2E, mneg));
                s[o][k][u] = e;
                sum += e;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
        if (lane == 0) red[1][wave * G + o] = sum;
    }
    __syncthreads();
#pragma unroll
    for (int o = 0; o < G; ++o) {
        float v = red[1][o];
#pragma unroll
        for (int i = 1; i < NW; ++i) v += red[1][i * G + o];
        inv[o] = 1.0f / v;
    }
#pragma unroll
    for (int o = 0; o < G; ++o)
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (gone(k)) continue;
#pragma unroll
            for (int u = 0; u < VEC; ++u) s[o][k][u] *= inv[o];
            if (use_dot) continue;  // rounded below, when the heads are packed in pairs
            if constexpr (VEC % 2 == 0) {
#pragma unroll
                for (int u = 0; u < VEC; u += 2) round_pair<T>(s[o][k][u], s[o][k][u + 1]);
            } else {
#pragma unroll
                for (int u = 0; u < VEC; ++u) s[o][k][u] = round_to<T>(s[o][k][u]);
            }
        }

#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int q = (k * NT + tid) * VEC;
        if (hid(k) && !dead(k)) {  // pass wholly ahead of the row's first visible key: +0
            if (q < Q) {
                V z;
#pragma unroll
                for (int u = 0; u < VEC; ++u) z.v[u] = from_float<T>(0.0f);
#pragma unroll
                for (int o = 0; o < G; ++o) store_stream(reinterpret_cast<V *>(y + base + o * plane + q), z);
            }
            continue;
        }
        if (dead(k)) {  // pass wholly above the diagonal: +0 only on request
            if (fill_upper && q < Q) {
                V z;
#pragma unroll
                for (int u = 0; u < VEC; ++u) z.v[u] = from_float<T>(0.0f);
#pragma unroll
                for (int o = 0; o < G; ++o) store_stream(reinterpret_cast<V *>(y + base + o * plane + q), z);
            }
            continue;
        }
        if (q >= Q || (!fill_upper && q > last)) continue;  // vectors wholly above the diagonal: +0 only on request
        uint32_t pp[DOT_OK ? G / 2 : 1][VEC];  // probabilities of heads (2j, 2j+1), rounded and packed
        if constexpr (DOT_OK) {
            if (use_dot) {
#pragma unroll
                for (int j = 0; j < G / 2; ++j)
#pragma unroll
                    for (int u = 0; u < VEC; ++u) pp[j][u] = pack2<T>(s[2 * j][k][u], s[2 * j + 1][k][u]);
            }
        }
#pragma unroll
        for (int o = 0; o < G; ++o) {
            float of[VEC];
            if constexpr (DOT_OK) {
                if (use_dot) {
#pragma unroll
                    for (int u = 0; u < VEC; ++u) {
                        float acc = 0.0f;
#pragma unroll
                        for (int j = 0; j < G / 2; ++j) acc = dot2<T>(w2p[o * (G / 2) + j], pp[j][u], acc);
                        of[u] = acc;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < VEC; ++u) {
                if (use_dot) break;
                float acc;
                if (w2) {
                    acc = 0.0f;
#pragma unroll
                    for (int i = 0; i < G; ++i) acc = fmaf(w2s[o * G + i], s[i][k][u], acc);
                } else {
                    acc = s[o][k][u];
                }
                of[u] = acc;
            }
            if (q + VEC - 1 > last) {
#pragma unroll
                for (int u = 0; u < VEC; ++u)
                    if (q + u > last) of[u] = 0.0f;
            }
            V out;
            pack_vec<T, VEC>(of, out);
            store_stream(reinterpret_cast<V *>(y + base + o * plane + q), out);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// 16-bit data with weights of the same dtype (or none), even group size, rows of at most 256*8*NV keys: the same
// computation with roughly a fifth fewer vector-ALU instructions - on this kernel the SIMDs' issue slots, not the
// memory system, are the first limit (about 14 instructions per element in the kernel above).
//   * both mixes run on packed dot products (v_dot2c: two multiply-adds per instruction).  For the first mix the loaded
//     vectors (8 keys of one head) are re-paired with byte permutes into (head 2j, head 2j+1) pairs of one key.
//   * the mixed scores are kept rounded and packed (they are rounded to the I/O dtype anyway); the row maximum is
//     taken before the rounding, which commutes with it (rounding is monotonic).
//   * the weights are 2G*G/2 packed pairs read through wavefront-uniform addresses (scalar registers).
//   * the number of live 2048-key passes of a wavefront (keys at or below the diagonal) selects one of NV+1 straight
//     instantiations of each phase: no per-pass tests inside.
//   * wavefront reductions use DPP within rows of 16 lanes.
typedef unsigned int rs_u4 __attribute__((ext_vector_type(4)));

// max(a, b, c) in one instruction (the compiler only forms it when it can rule out signalling NaNs).  Only for
// operands produced by ordinary vector-ALU instructions or loads.
__device__ __forceinline__ float max3(float a, float b, float c)
{
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// max(a, b) without the compiler's canonicalisation of the inputs (no NaNs reach these reductions)
__device__ __forceinline__ float max_raw(float a, float b)
{
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// One DPP step of a reduction inside rows of 16 lanes (the operand permuted on the way into the ALU; the two wait states
// a DPP read of a just-written register needs are part of the asm).
#define MTA_RS_DPP_STEP(op, ctrl) asm("s_nop 1\n\t" op "_dpp %0, %1, %1 " ctrl " row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v)); v = r;
// The same for operands that dot-product instructions may just have written: a different vector-ALU instruction
// may read such a register only three wait states later, and the compiler, which inserts those for its own
// instructions, cannot see into the assembly.
__device__ __forceinline__ float max3_after_dot(float a, float b, float c)
{
    float r;
    asm("s_nop 2\n\tv_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

typedef unsigned int rs_u2 __attribute__((ext_vector_type(2)));
template <bool IS_MAX> __device__ __forceinline__ float rs_op(float a, float b) { return IS_MAX ? max_raw(a, b) : a + b; }

// The G per-lane values v[0..G) (one per head), each reduced over the wavefront, all at once: an exchange of the two
// halves of the wavefront leaves head 2j's result-so-far in the lower and head 2j+1's in the upper 32 lanes of one
// register, an exchange of rows of 16 lanes folds two such registers into one (rows 0..3 then hold heads 4j, 4j+2, 4j+1,
// 4j+3), and four DPP steps finish inside the rows.  The first lane of each row writes dst[head*NW + wave].
template <bool IS_MAX, int G, int NW> __device__ __forceinline__ void heads_reduce_store(const float (&val)[G], float *dst, int wave, int lane)
{
    static_assert(G == 2 || G == 4 || G == 8, "head groups of the packed kernel");
    float c[G / 2];
#pragma unroll
    for (int j = 0; j < G / 2; ++j) {
        const rs_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(val[2 * j]), __float_as_uint(val[2 * j + 1]), false, false);
        c[j] = rs_op<IS_MAX>(__uint_as_float(r[0]), __uint_as_float(r[1]));
    }
    constexpr int ND = G >= 4 ? G / 4 : 1;
    float d[ND];
#pragma unroll
    for (int j = 0; j < ND; ++j) {
        const float a = c[G >= 4 ? 2 * j : 0], b = c[G >= 4 ? 2 * j + 1 : 0];
        const rs_u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
        d[j] = rs_op<IS_MAX>(__uint_as_float(r[0]), __uint_as_float(r[1]));
    }
    const int row = lane >> 4;
#pragma unroll
    for (int j = 0; j < ND; ++j) {
        float v = d[j], r;
        if constexpr (IS_MAX) {
            MTA_RS_DPP_STEP("v_max_f32", "quad_perm:[1,0,3,2]")
            MTA_RS_DPP_STEP("v_max_f32", "quad_perm:[2,3,0,1]")
            MTA_RS_DPP_STEP("v_max_f32", "row_half_mirror")
            MTA_RS_DPP_STEP("v_max_f32", "row_mirror")
        } else {
            MTA_RS_DPP_STEP("v_add_f32", "quad_perm:[1,0,3,2]")
            MTA_RS_DPP_STEP("v_add_f32", "quad_perm:[2,3,0,1]")
            MTA_RS_DPP_STEP("v_add_f32", "row_half_mirror")
            MTA_RS_DPP_STEP("v_add_f32", "row_mirror")
        }
        // rows 0..3 hold heads (G >= 4) 4j + {0, 2, 1, 3}; (G == 2) {0, 0, 1, 1}
        const int head = G >= 4 ? 4 * j + ((row & 1) << 1) + (row >> 1) : (row >> 1);
        if ((lane & 15) == 0 && (G >= 4 || (row & 1) == 0)) dst[head * NW + wave] = v;
    }
}

// What the wavefronts flw .. nlw-1 left in src[head*NW + wave], combined per head, the same in every lane: lane l takes
// entry l, NW neighbouring lanes fold with DPP steps, and one lane per head is read out as a wavefront-uniform value.
template <bool IS_MAX, int G, int NW> __device__ __forceinline__ void heads_combine(const float *src, int nlw, int lane, float (&out)[G], int flw = 0)
{
    static_assert(NW * G <= 64 && (NW == 4 || NW == 8), "one entry per lane");
    const float neutral = IS_MAX ? -INFINITY : 0.0f;
    const float got = src[lane & (NW * G - 1)];
    float v = ((lane & (NW - 1)) < nlw && (lane & (NW - 1)) >= flw) ? got : neutral, r;
    if constexpr (IS_MAX) {
        MTA_RS_DPP_STEP("v_max_f32", "quad_perm:[1,0,3,2]")
        MTA_RS_DPP_STEP("v_max_f32", "quad_perm:[2,3,0,1]")
        if constexpr (NW == 8) { MTA_RS_DPP_STEP("v_max_f32", "row_half_mirror") }
    } else {
        MTA_RS_DPP_STEP("v_add_f32", "quad_perm:[1,0,3,2]")
        MTA_RS_DPP_STEP("v_add_f32", "quad_perm:[2,3,0,1]")
        if constexpr (NW == 8) { MTA_RS_DPP_STEP("v_add_f32", "row_half_mirror") }
    }
#pragma unroll
    for (int o = 0; o < G; ++o) out[o] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), o * NW));
}
#undef MTA_RS_DPP_STEP

// BAND (one pass per wavefront only): row_lo[n, p] is the first key row p sees; a wavefront whose slice lies wholly ahead
// of it stores +0 and ends, like those above the diagonal, and the slice that holds it masks the keys ahead of it.
// KBIAS: key_bias[n, q] (fp32, a value of the I/O dtype) is added to the mixed, rounded scores and the sum rounded again:
// the reference's `scores + mask` for a mask that is one value per (batch entry, key).
template <typename T, int G, int NV, bool HAS1, bool HAS2, int NT, int OCC, bool BAND = false, bool KBIAS = false>
__global__ __launch_bounds__(NT, OCC) void mix_softmax_mix_packed(
    const T *__restrict__ x, const T *__restrict__ w1, const T *__restrict__ w2, T *__restrict__ y, int C, int P, int Q,
    int causal, int fill_upper, const int *__restrict__ row_lo, int tri, const float *__restrict__ key_bias)
{
    constexpr int VEC = 8, NW = NT / 64, H2 = G / 2;
    static_assert(sizeof(T) == 2 && G % 2 == 0, "packed pairs of a 16-bit type");
    static_assert(!BAND || NV == 1, "the band mask is built for one pass per wavefront");
    __shared__ float red[2][NW * G];  // [0] maxima, [1] sums
    const int lane = threadIdx.x & 63;
    const unsigned groups = (unsigned)(C / G);
    unsigned b = blockIdx.x;
    const int p = (int)(b % (unsigned)P); b /= (unsigned)P;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int tid = threadIdx.x;
    const int g = (int)(b % groups);
    const int64_t n = b / groups;
    int64_t plane = (int64_t)P * Q;
    int64_t base = (n * C + (int64_t)g * G) * plane + (int64_t)p * Q;
    if (tri) {  // triangular layout (square, causal, nothing stored above the diagonal): the group's rows p lie side by side
        plane = tri_rowlen(p);
        base = (n * groups + g) * (G * tri_rowoff(P)) + G * tri_rowoff(p);
    }
    const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;  // last attended key

    // live passes of this wavefront: pass k covers keys [(k*NT + 64*wave)*VEC, +64*VEC)
    int nlive = 0;
#pragma unroll
    for (int k = 0; k < NV; ++k) nlive += ((k * NT + wave * 64) * VEC <= last) ? 1 : 0;
    // Slices wholly above the diagonal: nothing to read and nothing to contribute.  Their wavefronts end here, ahead of
    // the workgroup barriers (a barrier waits for the surviving wavefronts only), and free their registers for the next
    // workgroup; the others reduce over the first `nlw` slices.
    const int nlw = last / (64 * VEC) + 1 < NW ? last / (64 * VEC) + 1 : NW;
    int lo = 0, flw = 0;  // band mask: first visible key, and the wavefront whose slice holds it
    if constexpr (BAND) {
        lo = row_lo[n * P + p];
        lo = lo < 0 ? 0 : lo;
        flw = lo / (64 * VEC) < nlw - 1 ? lo / (64 * VEC) : nlw - 1;  // (a row that sees no key: NaN from the last slice)
        if (wave < flw) {  // slice wholly ahead of the first visible key (and below the diagonal): +0
            const int q = tid * VEC;
            const rs_u4 z = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int o = 0; o < G; ++o) __builtin_nontemporal_store(z, reinterpret_cast<rs_u4 *>(y + base + o * plane + q));
            return;
        }
    }
    if (nlive == 0) {
        if (fill_upper) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int q = (k * NT + tid) * VEC;
                if (q >= Q) continue;
                const rs_u4 z = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int o = 0; o < G; ++o) __builtin_nontemporal_store(z, reinterpret_cast<rs_u4 *>(y + base + o * plane + q));
            }
        }
        return;
    }

    // packed weights, (w[o][2j], w[o][2j+1]); identical for all lanes
    uint32_t w1p[G][H2], w2p[G][H2];
#pragma unroll
    for (int o = 0; o < G; ++o)
#pragma unroll
        for (int j = 0; j < H2; ++j) {
            const int64_t widx = (int64_t)(g * G + o) * C + g * G + 2 * j;
            w1p[o][j] = HAS1 ? *reinterpret_cast<const uint32_t *>(w1 + widx) : 0u;
            w2p[o][j] = HAS2 ? *reinterpret_cast<const uint32_t *>(w2 + widx) : 0u;
        }

    // One straight instantiation per (number of live passes L, whether the last of them straddles the last attended
    // key): masks exist only in the EDGE instantiations and only for pass L-1 (an earlier pass lies wholly below the
    // diagonal).  The two workgroup barriers sit inside the instantiations - every wavefront passes exactly two.
    auto run = [&](auto live_tag, auto edge_tag) __attribute__((always_inline)) {
        constexpr int L = decltype(live_tag)::value;
        constexpr bool EDGE = decltype(edge_tag)::value;
        constexpr int LL = L > 0 ? L : 1;
        uint32_t sp[G][LL][VEC / 2];  // mixed scores, rounded, two keys per register
        float m[G], inv[G];

        // ---- load, first mix, running maximum, round and pack ----
        {
            rs_u4 xin[LL][G];
#pragma unroll
            for (int k = 0; k < L; ++k) {
                const int q = (k * NT + tid) * VEC;
                const int qs = (!EDGE || k < L - 1 || q <= last) ? q : 0;  // beyond the attended keys: re-read the row start
#pragma unroll
                for (int i = 0; i < G; ++i)
                    xin[k][i] = __builtin_nontemporal_load(reinterpret_cast<const rs_u4 *>(x + base + i * plane + qs));
            }
#pragma unroll
            for (int o = 0; o < G; ++o) m[o] = -INFINITY;
#pragma unroll
            for (int k = 0; k < L; ++k) {
                const int q = (k * NT + tid) * VEC;
                float kbv[KBIAS ? VEC : 1];
                if constexpr (KBIAS) {
                    typedef float rs_f4 __attribute__((ext_vector_type(4)));
                    const int qs = (!EDGE || k < L - 1 || q <= last) ? q : 0;  // (as for x: beyond the attended keys, the row start)
                    const rs_f4 b0 = *reinterpret_cast<const rs_f4 *>(key_bias + n * Q + qs);
                    const rs_f4 b1 = *reinterpret_cast<const rs_f4 *>(key_bias + n * Q + qs + 4);
#pragma unroll
                    for (int u = 0; u < 4; ++u) { kbv[u] = b0[u]; kbv[4 + u] = b1[u]; }
                }
#pragma unroll
                for (int d = 0; d < VEC / 2; ++d) {
                    float a[G][2];
                    if constexpr (HAS1) {
                        uint32_t lo[H2], hi[H2];  // (head 2j, head 2j+1) of key 2d and of key 2d+1
#pragma unroll
                        for (int j = 0; j < H2; ++j) {
                            lo[j] = __builtin_amdgcn_perm(xin[k][2 * j + 1][d], xin[k][2 * j][d], 0x05040100u);
                            hi[j] = __builtin_amdgcn_perm(xin[k][2 * j + 1][d], xin[k][2 * j][d], 0x07060302u);
                        }
#pragma unroll
                        for (int o = 0; o < G; ++o) {
                            a[o][0] = 0.0f;
                            a[o][1] = 0.0f;
#pragma unroll
                            for (int j = 0; j < H2; ++j) {
                                a[o][0] = dot2<T>(lo[j], w1p[o][j], a[o][0]);
                                a[o][1] = dot2<T>(hi[j], w1p[o][j], a[o][1]);
                            }
                        }
                    } else {
#pragma unroll
                        for (int o = 0; o < G; ++o) unpack2<T>(xin[k][o][d], a[o][0], a[o][1]);
                    }
                    if constexpr (KBIAS) {
#pragma unroll
                        for (int o = 0; o < G; ++o) {
                            if constexpr (HAS1) round_pair<T>(a[o][0], a[o][1]);  // (the mixed scores as the unfused chain stores them)
                            a[o][0] += kbv[2 * d];
                            a[o][1] += kbv[2 * d + 1];
                        }
                    }
                    if (EDGE && k == L - 1) {
#pragma unroll
                        for (int o = 0; o < G; ++o) {
                            if (q + 2 * d > last) a[o][0] = -INFINITY;
                            if (q + 2 * d + 1 > last) a[o][1] = -INFINITY;
                        }
                    }
                    if constexpr (BAND) {
#pragma unroll
                        for (int o = 0; o < G; ++o) {
                            if (q + 2 * d < lo) a[o][0] = -INFINITY;
                            if (q + 2 * d + 1 < lo) a[o][1] = -INFINITY;
                        }
                    }
#pragma unroll
                    for (int o = 0; o < G; ++o) {
                        m[o] = (HAS1 && !KBIAS) ? max3_after_dot(m[o], a[o][0], a[o][1]) : max3(m[o], a[o][0], a[o][1]);
                        sp[o][k][d] = (HAS1 || BAND || KBIAS || (EDGE && k == L - 1)) ? pack2<T>(a[o][0], a[o][1]) : xin[k][o][d];
                    }
                }
            }
        }
        heads_reduce_store<true, G, NW>(m, red[0], wave, lane);
        __syncthreads();
        heads_combine<true, G, NW>(red[0], nlw, lane, m, flw);
        if constexpr (HAS1 || KBIAS) {
            // the maximum of the rounded scores is the rounded maximum (the row's first key is always attended: finite)
#pragma unroll
            for (int o = 0; o < G; o += 2) round_pair<T>(m[o], m[o + 1]);
        }

        // ---- exp(s - max) = exp2(s*log2(e) - max*log2(e)), running sum ----
        float e[G][LL][VEC];
        constexpr float LOG2E = 1.4426950408889634f;
#pragma unroll
        for (int o = 0; o < G; ++o) {
            const float mneg = -m[o] * LOG2E;
            float &acc = inv[o];
            acc = 0.0f;
#pragma unroll
            for (int k = 0; k < L; ++k)
#pragma unroll
                for (int d = 0; d < VEC / 2; ++d) {
                    float s0, s1;
                    unpack2<T>(sp[o][k][d], s0, s1);
                    e[o][k][2 * d] = __builtin_amdgcn_exp2f(fmaf(s0, LOG2E, mneg));
                    e[o][k][2 * d + 1] = __builtin_amdgcn_exp2f(fmaf(s1, LOG2E, mneg));
                    acc += e[o][k][2 * d];
                    acc += e[o][k][2 * d + 1];
                }
        }
        heads_reduce_store<false, G, NW>(inv, red[1], wave, lane);
        __syncthreads();
        heads_combine<false, G, NW>(red[1], nlw, lane, inv, flw);
#pragma unroll
        for (int o = 0; o < G; ++o) {  // 1/sum: the hardware reciprocal and one Newton step (within an ulp of the quotient)
            const float r = __builtin_amdgcn_rcpf(inv[o]);
            inv[o] = fmaf(fmaf(-inv[o], r, 1.0f), r, r);
        }

        // ---- normalise, round in pairs of heads, second mix, store ----
#pragma unroll
        for (int k = 0; k < L; ++k) {
            const int q = (k * NT + tid) * VEC;
            if (EDGE && k == L - 1 && (q >= Q || (!fill_upper && q > last))) continue;  // wholly above: +0 only on request
            uint32_t out[G][VEC / 2];
            if constexpr (HAS2) {
#pragma unroll
                for (int d = 0; d < VEC / 2; ++d) {
                    uint32_t pp[H2][2];  // probabilities of heads (2j, 2j+1) at keys 2d and 2d+1, rounded
#pragma unroll
                    for (int j = 0; j < H2; ++j)
#pragma unroll
                        for (int h = 0; h < 2; ++h)
                            pp[j][h] = pack2<T>(e[2 * j][k][2 * d + h] * inv[2 * j], e[2 * j + 1][k][2 * d + h] * inv[2 * j + 1]);
#pragma unroll
                    for (int o = 0; o < G; ++o) {
                        float r0 = 0.0f, r1 = 0.0f;
#pragma unroll
                        for (int j = 0; j < H2; ++j) {
                            r0 = dot2<T>(w2p[o][j], pp[j][0], r0);
                            r1 = dot2<T>(w2p[o][j], pp[j][1], r1);
                        }
                        out[o][d] = pack2<T>(r0, r1);
                    }
                }
            } else {
#pragma unroll
                for (int o = 0; o < G; ++o)
#pragma unroll
                    for (int d = 0; d < VEC / 2; ++d)
                        out[o][d] = pack2<T>(e[o][k][2 * d] * inv[o], e[o][k][2 * d + 1] * inv[o]);
            }
            if (EDGE && k == L - 1) {  // +0 beyond the last attended key
#pragma unroll
                for (int o = 0; o < G; ++o)
#pragma unroll
                    for (int d = 0; d < VEC / 2; ++d) {
                        if (q + 2 * d > last) out[o][d] &= 0xffff0000u;
                        if (q + 2 * d + 1 > last) out[o][d] &= 0x0000ffffu;
                    }
            }
#pragma unroll
            for (int o = 0; o < G; ++o) {
                const rs_u4 v = {out[o][0], out[o][1], out[o][2], out[o][3]};
                __builtin_nontemporal_store(v, reinterpret_cast<rs_u4 *>(y + base + o * plane + q));
            }
        }
        if (fill_upper) {  // passes wholly above the diagonal
#pragma unroll
            for (int k = L; k < NV; ++k) {
                const int q = (k * NT + tid) * VEC;
                if (q >= Q) continue;
                const rs_u4 z = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int o = 0; o < G; ++o) __builtin_nontemporal_store(z, reinterpret_cast<rs_u4 *>(y + base + o * plane + q));
            }
        }
    };
    // does the last live pass reach beyond the last attended key?
    const bool edge = ((nlive - 1) * NT + wave * 64 + 64) * VEC - 1 > last;
    static_assert(NV <= 4, "live-pass dispatch");
    using std::integral_constant;
    if (edge) {
        if (nlive == 1) run(integral_constant<int, 1>{}, std::true_type{});
        if constexpr (NV >= 2) { if (nlive == 2) run(integral_constant<int, 2>{}, std::true_type{}); }
        if constexpr (NV >= 3) { if (nlive == 3) run(integral_constant<int, 3>{}, std::true_type{}); }
        if constexpr (NV >= 4) { if (nlive == 4) run(integral_constant<int, 4>{}, std::true_type{}); }
    } else {
        if (nlive == 1) run(integral_constant<int, 1>{}, std::false_type{});
        if constexpr (NV >= 2) { if (nlive == 2) run(integral_constant<int, 2>{}, std::false_type{}); }
        if constexpr (NV >= 3) { if (nlive == 3) run(integral_constant<int, 3>{}, std::false_type{}); }
        if constexpr (NV >= 4) { if (nlive == 4) run(integral_constant<int, 4>{}, std::false_type{}); }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// No weights, 16-bit data, rows of at most 2048 keys: a wavefront per row (up to 4 vectors of 8 keys per lane), no LDS
// and no barrier; a workgroup of four wavefronts takes SR_ROWS consecutive rows of one plane.  With a workgroup per row,
// a launch over 128 heads x 2048 rows starts 262144 workgroups that move 4 KB each, and that is what its time is.
constexpr int SR_ROWS = 32, SR_NV = 4;
template <typename T>
__global__ __launch_bounds__(256) void softmax_rows_wave(const T *__restrict__ x, T *__restrict__ y, int P, int Q, int causal,
                                                         int fill_upper, int blocks_per_plane)
{
    constexpr int VEC = 8;
    constexpr float LOG2E = 1.4426950408889634f;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t plane = blockIdx.x / (unsigned)blocks_per_plane;
    const int p0 = (int)(blockIdx.x % (unsigned)blocks_per_plane) * SR_ROWS;
    for (int p = p0 + wave; p < p0 + SR_ROWS && p < P; p += 4) {
        const T *xr = x + (plane * P + p) * (int64_t)Q;
        T *yr = y + (plane * P + p) * (int64_t)Q;
        const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;  // last attended key
        rs_u4 xin[SR_NV];
#pragma unroll
        for (int k = 0; k < SR_NV; ++k) {
            if (k * 64 * VEC > last) break;  // (wavefront-uniform) wholly beyond the attended keys
            const int q = (k * 64 + lane) * VEC;
            xin[k] = __builtin_nontemporal_load(reinterpret_cast<const rs_u4 *>(xr + (q <= last ? q : 0)));  // (beyond: the row start)
        }
        float sv[SR_NV][VEC];
        float m = -INFINITY;
#pragma unroll
        for (int k = 0; k < SR_NV; ++k) {
            if (k * 64 * VEC > last) break;
            const int q = (k * 64 + lane) * VEC;
#pragma unroll
            for (int d = 0; d < VEC / 2; ++d) {
                unpack2<T>(xin[k][d], sv[k][2 * d], sv[k][2 * d + 1]);
                if (q + 2 * d > last) sv[k][2 * d] = -INFINITY;
                if (q + 2 * d + 1 > last) sv[k][2 * d + 1] = -INFINITY;
                m = fmaxf(m, fmaxf(sv[k][2 * d], sv[k][2 * d + 1]));
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
        const float mneg = -m * LOG2E;
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < SR_NV; ++k) {
            if (k * 64 * VEC > last) break;
#pragma unroll
            for (int u = 0; u < VEC; ++u) {
                sv[k][u] = __builtin_amdgcn_exp2f(fmaf(sv[k][u], LOG2E, mneg));  // (-inf -> 0)
                sum += sv[k][u];
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
        const float rc = __builtin_amdgcn_rcpf(sum);  // 1/sum: the hardware reciprocal and one Newton step
        const float inv = fmaf(fmaf(-sum, rc, 1.0f), rc, rc);
#pragma unroll
        for (int k = 0; k < SR_NV; ++k) {
            const int q = (k * 64 + lane) * VEC;
            if (q >= Q) break;
            if (q > last) {  // wholly above the diagonal: +0 on request
                if (fill_upper) __builtin_nontemporal_store(rs_u4{0u, 0u, 0u, 0u}, reinterpret_cast<rs_u4 *>(yr + q));
                continue;
            }
            // (keys beyond the last attended one carry probability 0 and come out as +0)
            const rs_u4 out = {pack2<T>(sv[k][0] * inv, sv[k][1] * inv), pack2<T>(sv[k][2] * inv, sv[k][3] * inv),
                               pack2<T>(sv[k][4] * inv, sv[k][5] * inv), pack2<T>(sv[k][6] * inv, sv[k][7] * inv)};
            __builtin_nontemporal_store(out, reinterpret_cast<rs_u4 *>(yr + q));
        }
    }
}

// Any row length / any group size: three sweeps over the row, inputs re-read (and re-mixed)
// in each; scalar accesses.  Correctness fallback for ragged or very long rows.
template <typename T, int NT>
__global__ __launch_bounds__(NT) void mix_softmax_mix_any(const T *__restrict__ x, const void *__restrict__ w1,
                                                          const void *__restrict__ w2, const float *__restrict__ kb,
                                                          T *__restrict__ y, int C, int G, int P, int Q, int causal,
                                                          int w_dtype, int fill_upper, const int *__restrict__ row_lo)
{
    __shared__ float red[NT / 64];
    extern __shared__ float stats[];  // [G] max, [G] 1/sum
    const int tid = threadIdx.x;
    const int groups = C / G;
    int64_t b = blockIdx.x;
    const int p = (int)(b % P); b /= P;
    const int g = (int)(b % groups);
    const int64_t n = b / groups;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base = (n * C + (int64_t)g * G) * plane + (int64_t)p * Q;
    const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;

    const int lo = row_lo ? row_lo[n * P + p] : 0;  // first visible key of the row (band mask)
    auto mixed = [&](int o, int q) -> float {
        if (q < lo) return -INFINITY;
        float acc;
        if (!w1) {
            acc = to_float(x[base + o * plane + q]);
        } else {
            acc = 0.0f;
            for (int i = 0; i < G; ++i)
                acc = fmaf(load_any(w1, w_dtype, (int64_t)(g * G + o) * C + g * G + i), to_float(x[base + i * plane + q]), acc);
            acc = round_to<T>(acc);
        }
        return kb ? round_to<T>(acc + kb[n * Q + q]) : acc;
    };
    for (int o = 0; o < G; ++o) {
        float m = -INFINITY;
        for (int q = tid; q <= last; q += NT) m = fmaxf(m, mixed(o, q));
        m = block_max<NT>(m, red);
        float sum = 0.0f;
        for (int q = tid; q <= last; q += NT) sum += __expf(mixed(o, q) - m);
        sum = block_sum<NT>(sum, red);
        if (tid == 0) { stats[o] = m; stats[G + o] = 1.0f / sum; }
    }
    __syncthreads();
    const int q_end = fill_upper ? Q : last + 1;
    for (int q = tid; q < q_end; q += NT) {
        for (int o = 0; o < G; ++o) {
            float acc = 0.0f;
            if (q <= last) {
                if (w2) {
                    for (int i = 0; i < G; ++i) {
                        const float pr = round_to<T>(__expf(mixed(i, q) - stats[i]) * stats[G + i]);
                        acc = fmaf(load_any(w2, w_dtype, (int64_t)(g * G + o) * C + g * G + i), pr, acc);
                    }
                } else {
                    acc = round_to<T>(__expf(mixed(o, q) - stats[o]) * stats[G + o]);
                }
            }
            y[base + o * plane + q] = from_float<T>(acc);
        }
    }
}

template <typename T, int G, int NV, int NT = 256>
int launch_fixed(const void *x, const void *w1, const void *w2, const float *kb, const int *row_lo, void *y, int64_t N, int64_t C,
                 int64_t P, int64_t Q, int causal, int w_dtype, int fill_upper, hipStream_t st)
{
    constexpr int VEC = vec_of<T>::n;
    const int64_t blocks = N * (C / G) * P;
    if (kb || row_lo)
        hipLaunchKernelGGL((mix_softmax_mix<T, G, NV, VEC, NT, true>), dim3((unsigned)blocks), dim3(NT), 0, st, (const T *)x,
                           w1, w2, kb, (T *)y, (int)C, (int)P, (int)Q, causal, w_dtype, fill_upper, row_lo);
    else
        hipLaunchKernelGGL((mix_softmax_mix<T, G, NV, VEC, NT, false>), dim3((unsigned)blocks), dim3(NT), 0, st, (const T *)x,
                           w1, w2, kb, (T *)y, (int)C, (int)P, (int)Q, causal, w_dtype, fill_upper, row_lo);
    return launch_status();
}

template <typename T>
int dispatch(const void *x, const void *w1, const void *w2, const float *kb_in, const int *row_lo, void *y, int64_t N, int64_t C,
             int64_t P, int64_t Q, int G, int causal, int w_dtype, int fill_upper, hipStream_t st, int tri_in = 0, int tri_out = 0)
{
    const int tri = tri_in && tri_out;  // (the packed kernels: both tensors in the triangular layout, or neither)
    // (the kernels without a key bias are the ones without a band mask too: `kb` below stands for "either")
    const float *kb = kb_in;
    const bool plain = !kb_in && !row_lo;
    constexpr int VEC = vec_of<T>::n;
    const bool vec_ok = (Q % VEC == 0) && aligned_to(x, 16) && aligned_to(y, 16);
    const int64_t nv = (Q + 256 * VEC - 1) / (256 * VEC);
    if constexpr (sizeof(T) == 2) {
        // 16-bit data, weights of the same dtype: the packed kernel (MTA_SOFTMAX_NO_PACKED=1 in the environment keeps
        // the general one, for comparisons)
        static const bool no_packed = [] { const char *e_ = getenv("MTA_SOFTMAX_NO_PACKED"); return e_ && e_[0] == '1'; }();
        const int io_code = std::is_same<T, bf16_t>::value ? MTA_BF16 : MTA_F16;
        if (G == 16 && !no_packed && (!kb || aligned_to(kb, 4))) {
            const int rc = mix16_softmax_launch(x, w1, w2, y, N, C, P, Q, causal, fill_upper, io_code, w_dtype, st, tri_in, tri_out,
                                                kb, row_lo);
            if (rc != MTA_ERR_UNSUPPORTED) return rc;
        }
        if (tri_in != tri_out) return MTA_ERR_UNSUPPORTED;
        const bool packed_ok = vec_ok && !no_packed && w_dtype == io_code && (w1 || w2) && (!w1 || aligned_to(w1, 4)) &&
                               (!w2 || aligned_to(w2, 4)) && C % 2 == 0 && Q <= 256 * VEC * 4;
        // key bias without a band mask: the packed kernel's KBIAS instances, one per group size (the one for the longest
        // rows; with 4 heads and one weight the 512-thread shape)
        if (packed_ok && kb && !row_lo && aligned_to(kb, 16)) {
#define MTA_RSK_LAUNCH(g, v, h1, h2, nt, occ)                                                                          \
    {                                                                                                                  \
        hipLaunchKernelGGL((mix_softmax_mix_packed<T, g, v, h1, h2, nt, occ, false, true>),                            \
                           dim3((unsigned)(N * (C / g) * P)), dim3(nt), 0, st, (const T *)x, (const T *)w1,            \
                           (const T *)w2, (T *)y, (int)C, (int)P, (int)Q, causal, fill_upper, nullptr, tri, kb);      \
        return launch_status();                                                                                        \
    }
#define MTA_RSK_CASE(g, v, nt, occ)                                                                                    \
    if (G == g && Q <= (int64_t)(nt) * VEC * (v)) {                                                                    \
        if (w1 && w2) MTA_RSK_LAUNCH(g, v, true, true, nt, occ)                                                        \
        if (w1) MTA_RSK_LAUNCH(g, v, true, false, nt, occ)                                                             \
        MTA_RSK_LAUNCH(g, v, false, true, nt, occ)                                                                     \
    }
            MTA_RSK_CASE(2, 4, 256, RS_OCC)
            if (!(w1 && w2)) MTA_RSK_CASE(4, 1, 512, 8)
            MTA_RSK_CASE(4, 2, 256, RS_OCC) MTA_RSK_CASE(8, 1, 256, 4)  // (8 heads: a register budget without spills)
#undef MTA_RSK_CASE
#undef MTA_RSK_LAUNCH
        }
        // band mask without a key bias, one weight, rows that one pass per wavefront covers: the packed kernel's BAND
        // instances (causal by construction)
        if (packed_ok && row_lo && !kb && causal && !(w1 && w2)) {
#define MTA_RSB_LAUNCH(g, h1, h2, nt, occ)                                                                             \
    {                                                                                                                  \
        hipLaunchKernelGGL((mix_softmax_mix_packed<T, g, 1, h1, h2, nt, occ, true>), dim3((unsigned)(N * (C / g) * P)), \
                           dim3(nt), 0, st, (const T *)x, (const T *)w1, (const T *)w2, (T *)y, (int)C, (int)P,        \
                           (int)Q, causal, fill_upper, row_lo, tri, nullptr);                                          \
        return launch_status();                                                                                        \
    }
#define MTA_RSB_CASE(g, nt, occ)                                                                                       \
    if (G == g && Q <= (int64_t)(nt) * VEC) {                                                                          \
        if (w1) MTA_RSB_LAUNCH(g, true, false, nt, occ)                                                                \
        MTA_RSB_LAUNCH(g, false, true, nt, occ)                                                                        \
    }
            MTA_RSB_CASE(2, 256, 1) MTA_RSB_CASE(4, 256, 1) MTA_RSB_CASE(4, 512, 8) MTA_RSB_CASE(8, 256, RS_OCC)
#undef MTA_RSB_CASE
#undef MTA_RSB_LAUNCH
        }
        if (packed_ok && plain) {
#define MTA_RSP_LAUNCH(g, v, h1, h2, nt, occ)                                                                          \
    {                                                                                                                  \
        hipLaunchKernelGGL((mix_softmax_mix_packed<T, g, v, h1, h2, nt, occ>), dim3((unsigned)(N * (C / g) * P)),      \
                           dim3(nt), 0, st, (const T *)x, (const T *)w1, (const T *)w2, (T *)y, (int)C, (int)P,        \
                           (int)Q, causal, fill_upper, nullptr, tri, nullptr);                                         \
        return launch_status();                                                                                        \
    }
#define MTA_RSP_CASE(g, v, nt, occ)                                                                                    \
    if (G == g && Q <= (int64_t)(nt) * VEC * (v)) {                                                                    \
        if (w1 && w2) MTA_RSP_LAUNCH(g, v, true, true, nt, occ)                                                        \
        if (w1) MTA_RSP_LAUNCH(g, v, true, false, nt, occ)                                                             \
        MTA_RSP_LAUNCH(g, v, false, true, nt, occ)                                                                     \
    }
            MTA_RSP_CASE(2, 1, 256, 1) MTA_RSP_CASE(2, 2, 256, 1) MTA_RSP_CASE(2, 4, 256, RS_OCC) MTA_RSP_CASE(4, 1, 256, 1)
            // 4 heads x up to 4096 keys: with one weight, 8 wavefronts of one pass each (63 registers: 8 wavefronts per
            // SIMD; measured 2 % faster than 4 wavefronts of two passes); with both weights the latter is 4 % faster
            if (!(w1 && w2)) MTA_RSP_CASE(4, 1, 512, 8)
            MTA_RSP_CASE(4, 2, 256, RS_OCC) MTA_RSP_CASE(8, 1, 256, RS_OCC)
#undef MTA_RSP_CASE
#undef MTA_RSP_LAUNCH
        }
    }
    if (tri_in || tri_out) return MTA_ERR_UNSUPPORTED;  // (only the kernels above know the triangular layout)
    if constexpr (sizeof(T) == 2) {
        // no weights, short rows: a wavefront per row (MTA_SOFTMAX_NO_WAVE_ROWS=1 keeps a workgroup per row, for comparisons)
        static const bool no_wave = [] { const char *e_ = getenv("MTA_SOFTMAX_NO_WAVE_ROWS"); return e_ && e_[0] == '1'; }();
        if (G == 1 && !w1 && !w2 && plain && vec_ok && Q <= 64 * VEC * SR_NV && !no_wave) {
            const int64_t bpp = (P + SR_ROWS - 1) / SR_ROWS;
            if (N * C * bpp <= 0x7fffffffLL) {
                hipLaunchKernelGGL((softmax_rows_wave<T>), dim3((unsigned)(N * C * bpp)), dim3(256), 0, st, (const T *)x,
                                   (T *)y, (int)P, (int)Q, causal, fill_upper, (int)bpp);
                return launch_status();
            }
        }
    }
    if (vec_ok) {
#define MTA_RS_CASE(g, v)                                                                   \
    if (G == g && nv <= v) return launch_fixed<T, g, v>(x, w1, w2, kb, row_lo, y, N, C, P, Q, causal, w_dtype, fill_upper, st);
        MTA_RS_CASE(1, 1) MTA_RS_CASE(1, 2) MTA_RS_CASE(1, 4) MTA_RS_CASE(1, 8)
        MTA_RS_CASE(2, 1) MTA_RS_CASE(2, 2) MTA_RS_CASE(2, 4)
        MTA_RS_CASE(4, 1) MTA_RS_CASE(4, 2) MTA_RS_CASE(4, 4)
        MTA_RS_CASE(8, 1) MTA_RS_CASE(8, 2)
#undef MTA_RS_CASE
    }
    constexpr int NT = 256;
    const int64_t blocks = N * (C / G) * P;
    hipLaunchKernelGGL((mix_softmax_mix_any<T, NT>), dim3((unsigned)blocks), dim3(NT), sizeof(float) * 2 * G, st,
                       (const T *)x, w1, w2, kb, (T *)y, (int)C, G, (int)P, (int)Q, causal, w_dtype, fill_upper, row_lo);
    return launch_status();
}
}  // namespace

extern "C" int mta_headmix_softmax_band_fwd(const void *x, const void *w1, const void *w2, const void *key_bias,
                                            const void *first_visible, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                                            int group_size, int causal, int fill_upper, int io_dtype, int w_dtype, void *stream)
{
    if (!x || !y) return MTA_ERR_NULL;
    if ((key_bias && !aligned_to(key_bias, 4)) || (first_visible && !aligned_to(first_visible, 4))) return MTA_ERR_ALIGN;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || P <= 0 || Q <= 0 || P > (1 << 24) || Q > (1 << 24) || C > 4096) return MTA_ERR_SHAPE;
    if (group_size < 0 || (group_size > 0 && C % group_size != 0)) return MTA_ERR_GROUP;
    if (!aligned_to(x, dtype_size(io_dtype)) || !aligned_to(y, dtype_size(io_dtype)) ||
        (w1 && !aligned_to(w1, dtype_size(w_dtype))) || (w2 && !aligned_to(w2, dtype_size(w_dtype))))
        return MTA_ERR_ALIGN;
    int G = group_size > 0 ? group_size : (int)C;
    if (!w1 && !w2) G = 1;
    if (N * (C / G) * P > 0x7fffffffLL) return MTA_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    MTA_DISPATCH_IO(io_dtype, return dispatch<io_t>(x, w1, w2, (const float *)key_bias, (const int *)first_visible, y, N, C, P, Q,
                                                    G, causal, w_dtype, fill_upper || !causal, st));
    return MTA_ERR_DTYPE;
}

// The same pass over a causal square score tensor in the triangular layout (see tri_rowoff in common.hpp), groups of
// `group_size` heads interleaved by rows; nothing above the diagonal exists.  out_planes = 0: the output in the same
// layout (groups of 2, 4, 8 or 16 heads); 1: the output as (N,C,S,S) planes with nothing written above the diagonal
// (groups of 16).  16-bit data with weights of the same dtype only (MTA_ERR_UNSUPPORTED otherwise).
extern "C" int mta_headmix_softmax_tri_fwd(const void *x, const void *w1, const void *w2, const void *key_bias,
                                           const void *first_visible, void *y, int64_t N, int64_t C, int64_t S,
                                           int group_size, int out_planes, int io_dtype, int w_dtype, void *stream)
{
    if (!x || !y) return MTA_ERR_NULL;
    if ((first_visible && !aligned_to(first_visible, 4)) || (key_bias && !aligned_to(key_bias, 4))) return MTA_ERR_ALIGN;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || S <= 0 || S > (1 << 24) || C > 4096) return MTA_ERR_SHAPE;
    if (group_size <= 0 || C % group_size != 0) return MTA_ERR_GROUP;
    if (!aligned_to(x, 16) || !aligned_to(y, 16)) return MTA_ERR_ALIGN;
    if (N * (C / group_size) * S > 0x7fffffffLL) return MTA_ERR_SHAPE;
    if (io_dtype == MTA_F32 || (!w1 && !w2)) return MTA_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (io_dtype == MTA_BF16)
        return dispatch<bf16_t>(x, w1, w2, (const float *)key_bias, (const int *)first_visible, y, N, C, S, S, group_size, 1, w_dtype, 0, st, 1, !out_planes);
    return dispatch<f16_t>(x, w1, w2, (const float *)key_bias, (const int *)first_visible, y, N, C, S, S, group_size, 1, w_dtype, 0, st, 1, !out_planes);
}

// Whether mta_headmix_softmax_tri_fwd has a kernel for these sizes (the cases of `dispatch` that know the layout: the
// packed kernel's instances, with a band mask those for one weight and one pass per wavefront).  Nothing is launched.
extern "C" int mta_headmix_softmax_tri_supported(int64_t C, int64_t S, int group_size, int out_planes, int io_dtype,
                                                 int w_dtype, int has_w1, int has_w2, int band, int key_bias)
{
    if (io_dtype != MTA_BF16 && io_dtype != MTA_F16) return 0;
    if (w_dtype != io_dtype || (!has_w1 && !has_w2) || group_size <= 0 || C <= 0 || C % group_size != 0 || S <= 0 || S % 8 != 0)
        return 0;
    const char *e = getenv("MTA_SOFTMAX_NO_PACKED");
    if (e && e[0] == '1') return 0;
    if (group_size == 16) {  // the matrix-core kernel's row lists (rowsoftmax_dense16.hip)
        const char *e2 = getenv("MTA_MIX16_NO_ROW_LISTS");
        return S <= 4096 && S * S <= (1LL << 27) && !(e2 && e2[0] == '1');
    }
    if (out_planes || (band && key_bias)) return 0;
    if (band && has_w1 && has_w2) return 0;
    const int g = group_size;
    const int64_t cap = band ? (g == 4 ? 4096 : (g == 2 || g == 8) ? 2048 : 0) : (g == 2 ? 8192 : g == 4 ? 4096 : g == 8 ? 2048 : 0);
    return S <= cap ? 1 : 0;
}

extern "C" int mta_headmix_softmax_bias_fwd(const void *x, const void *w1, const void *w2, const void *key_bias,
                                            void *y, int64_t N, int64_t C, int64_t P, int64_t Q, int group_size,
                                            int causal, int fill_upper, int io_dtype, int w_dtype, void *stream)
{
    return mta_headmix_softmax_band_fwd(x, w1, w2, key_bias, nullptr, y, N, C, P, Q, group_size, causal, fill_upper, io_dtype,
                                        w_dtype, stream);
}

extern "C" int mta_headmix_softmax_fwd(const void *x, const void *w1, const void *w2, void *y, int64_t N,
                                       int64_t C, int64_t P, int64_t Q, int group_size, int causal,
                                       int fill_upper, int io_dtype, int w_dtype, void *stream)
{
    return mta_headmix_softmax_bias_fwd(x, w1, w2, nullptr, y, N, C, P, Q, group_size, causal, fill_upper, io_dtype, w_dtype,
                                        stream);
}
