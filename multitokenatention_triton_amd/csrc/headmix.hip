// Head mixing over axis 1 of an (N,C,P,Q) score tensor, without a transpose.
//
//   y[n,o,p,q] = sum_i w[o,i] * x[n,i,p,q]
//
// Heads are P*Q elements apart, keys are contiguous.  Each lane owns one 16-byte
// vector of consecutive keys q at a fixed (n,p) and walks the heads of its mixing
// group, so every global access is a fully coalesced 16-byte-per-lane row segment
// and the small GxG contraction happens inside the lane (no cross-lane traffic).
// Causal: vectors wholly above the diagonal are never read and receive the fill
// value; the vector that straddles the diagonal is masked per element.
#include <stdlib.h>

#include "common.hpp"
#include "mfma.hpp"

namespace {
using namespace mta;

constexpr int NT = 256;

template <typename T, int VEC> struct alignas(sizeof(T) * VEC) vecN { T v[VEC]; };

// inputs are read once and outputs written once by this kernel: move them as streaming (non-temporal) data
template <typename V> __device__ __forceinline__ V load_stream(const V *src)
{
    if constexpr (sizeof(V) == 16) {
        typedef unsigned int u4 __attribute__((ext_vector_type(4)));
        return __builtin_bit_cast(V, __builtin_nontemporal_load(reinterpret_cast<const u4 *>(src)));
    }
    return *src;
}
template <typename V> __device__ __forceinline__ void store_stream(V *dst, const V &v)
{
    if constexpr (sizeof(V) == 16) {
        typedef unsigned int u4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(__builtin_bit_cast(u4, v), reinterpret_cast<u4 *>(dst));
        return;
    }
    *dst = v;
}

// element (o, i) of the mixing matrix the kernels apply: w[o][i], or w[i][o] when `wt` (the transposed matrix is what
// the gradient with respect to the input is mixed with)
__device__ __forceinline__ int64_t w_index(int o, int i, int C, int wt) { return wt ? (int64_t)i * C + o : (int64_t)o * C + i; }

// Workgroups go to the 8 XCDs round-robin by index.  With the key chunk as the fastest-varying part of the index and
// a chunk count that divides 8 (or is a multiple of it), an XCD would always see the same chunks - and under the causal
// mask the chunks near the start of a row carry all the work.  Rotating the chunk by the row spreads every chunk over
// every XCD.  Returns the chunk of workgroup `id` and leaves the row (id / qchunks) in `id`; a bijection within each row.
// All index arithmetic is 32-bit and unsigned (the host rejects grids beyond 2^31 workgroups): a workgroup's share is
// small enough for 64-bit divisions in its prologue to show.
__device__ __forceinline__ int rotated_chunk(unsigned &id, unsigned qchunks)
{
    if (qchunks == 1) return 0;
    const unsigned row = id / qchunks, qc = id - row * qchunks;
    const unsigned rot = (qchunks % 8 == 0) ? row : (unsigned)(((uint64_t)row * qchunks) >> 3);
    id = row;
    return (int)((qc + rot) % qchunks);
}

// G heads mixed inside one lane, G known at compile time.  A workgroup covers one query row of one key chunk: on this
// part the fewer independent streams a wavefront holds, the higher the delivered bandwidth.
template <typename T, int G, int VEC>
__global__ __launch_bounds__(NT) void headmix_fixed(const T *__restrict__ x, const void *__restrict__ w,
                                                    T *__restrict__ y, int C, int P, int Q, int causal,
                                                    float fill, int w_dtype, int wt, int qchunks)
{
    __shared__ float wsm[G * G];
    const int tid = threadIdx.x;
    const int groups = C / G;
    unsigned b = blockIdx.x;
    const int qc = rotated_chunk(b, qchunks);
    const int p = (int)(b % (unsigned)P); b /= (unsigned)P;
    const int g = (int)(b % (unsigned)groups);
    const int64_t n = b / (unsigned)groups;
    const int q = (qc * NT + tid) * VEC;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base = (n * C + (int64_t)g * G) * plane + (int64_t)p * Q + q;
    using V = vecN<T, VEC>;
    const T fill_t = from_float<T>(fill);
    V fillv;
#pragma unroll
    for (int u = 0; u < VEC; ++u) fillv.v[u] = fill_t;
    // (causal == 2: causal, and what lies above the diagonal is the caller's to define - vectors wholly above it are
    // not written)
    if (causal && qc * NT * VEC > p) {  // chunk wholly above the diagonal: fill only, nothing read
        if (q < Q && causal != 2) {
#pragma unroll
            for (int o = 0; o < G; ++o) store_stream(reinterpret_cast<V *>(y + base + o * plane), fillv);
        }
        return;
    }
    // Issue all of this lane's loads first (unconditionally: a lane past the row end or above the
    // diagonal re-reads the row start), then fetch the weights, so that the latencies overlap.
    V xin[G];
    {
        const bool live = q < Q && !(causal && q > p);
        const int64_t lb = base - (live ? 0 : q);
#pragma unroll
        for (int i = 0; i < G; ++i) xin[i] = load_stream(reinterpret_cast<const V *>(x + lb + i * plane));
    }
    for (int t = tid; t < G * G; t += NT) wsm[t] = load_any(w, w_dtype, w_index(g * G + t / G, g * G + t % G, C, wt));
    __syncthreads();
    if (q >= Q) return;
    if (causal && q > p) {
        if (causal != 2) {
#pragma unroll
            for (int o = 0; o < G; ++o) store_stream(reinterpret_cast<V *>(y + base + o * plane), fillv);
        }
        return;
    }
#pragma unroll
    for (int o = 0; o < G; ++o) {
        float acc[VEC];
#pragma unroll
        for (int u = 0; u < VEC; ++u) acc[u] = 0.0f;
#pragma unroll
        for (int i = 0; i < G; ++i) {
            const float wv = wsm[o * G + i];
#pragma unroll
            for (int u = 0; u < VEC; ++u) acc[u] = fmaf(wv, to_float(xin[i].v[u]), acc[u]);
        }
        V out;
#pragma unroll
        for (int u = 0; u < VEC; ++u) out.v[u] = (causal && q + u > p) ? fill_t : from_float<T>(acc[u]);
        store_stream(reinterpret_cast<V *>(y + base + o * plane), out);
    }
}

// Dense mixing of 32 heads on the matrix cores (16-bit I/O, weights of the same dtype).
//
//   y[o, q] = sum_i w[o, i] * x[i, q]        one v_mfma_f32_16x16x32 per 16 output heads x 16 keys: the contraction
//                                            covers all 32 input heads at once
//
// A wavefront owns 128 keys of one (batch, query row) and needs no LDS.  Lane (ln, kg) fetches keys 8ln .. 8ln+7 of the
// heads 8kg .. 8kg+7 with eight 16-byte loads (an instruction covers 4 heads x 256 contiguous bytes), transposes that
// 8 x 8 block inside its own registers (one byte-permute per dword) into the x operands of eight products - product j
// maps the lane's column to key 8ln + j - and keeps w (output heads 0-15, 16-31) in registers as the other operand.
// After the eight products the lane holds keys 8ln .. 8ln+7 of output heads 4kg + v: 16-byte stores, again
// 4 heads x 256 contiguous bytes per instruction.  Columns are independent, so keys beyond the diagonal may carry any
// data (their lanes re-read the row start); their outputs get the fill.
constexpr int DM_WAVES = 4, DM_KEYS = 128;

template <typename T>
__global__ __launch_bounds__(64 * DM_WAVES, 4) void headmix_dense32(const T *__restrict__ x, const T *__restrict__ w,
                                                               T *__restrict__ y, int C, int P, int Q, int causal,
                                                               float fill, int wt, int qchunks)
{
    constexpr int HG = 32;  // heads mixed together
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, ln = lane & 15, kg = lane >> 4;
    const int groups = C / HG;
    unsigned b = blockIdx.x;
    const int qc = rotated_chunk(b, qchunks);
    const int p = (int)(b % (unsigned)P); b /= (unsigned)P;
    const int g = (int)(b % (unsigned)groups);
    const int64_t n = b / (unsigned)groups;
    const int q0 = (qc * DM_WAVES + wave) * DM_KEYS;
    if (q0 >= Q) return;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base = (n * C + (int64_t)g * HG) * plane + (int64_t)p * Q;  // head g*32, row p, key 0
    const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;              // last key that is mixed
    const uint32_t fill2 = pack2<T>(fill, fill);
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    const int key = q0 + ln * 8;

    if (q0 > last) {  // wholly beyond the diagonal: fill only (causal == 2: not even that)
        const u4 fv = {fill2, fill2, fill2, fill2};
        if (key < Q && causal != 2) {
#pragma unroll
            for (int t = 0; t < 8; ++t)
                __builtin_nontemporal_store(fv, reinterpret_cast<u4 *>(y + base + (kg * 8 + t) * plane + key));
        }
        return;
    }

    const T *xp = x + base + (int64_t)(kg * 8) * plane + (key <= last ? key : 0);
    u4 xv[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) xv[t] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(xp + t * plane));

    // w fragments: lane (output head ln of block ob, group kg) holds w[o][8kg .. 8kg+7]
    frag8<T> wf[2];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
        if (!wt) {
            wf[ob] = *reinterpret_cast<const frag8<T> *>(w + (int64_t)(g * HG + ob * 16 + ln) * C + g * HG + kg * 8);
        } else {  // the transposed matrix: a column of w, gathered element by element (once per wavefront)
#pragma unroll
            for (int t = 0; t < 8; ++t) wf[ob].v[t] = w[(int64_t)(g * HG + kg * 8 + t) * C + g * HG + ob * 16 + ln];
        }
    }

    f32x4 acc[8][2];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        u4 xt;  // heads 8kg .. 8kg+7 of key 8ln + j
#pragma unroll
        for (int u = 0; u < 4; ++u)
            xt[u] = __builtin_amdgcn_perm(xv[2 * u + 1][j >> 1], xv[2 * u][j >> 1], (j & 1) ? 0x07060302u : 0x05040100u);
        const frag8<T> xf = __builtin_bit_cast(frag8<T>, xt);
#pragma unroll
        for (int ob = 0; ob < 2; ++ob) {
            acc[j][ob] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            mma16(acc[j][ob], wf[ob], xf);
        }
    }
    if (key >= Q || (causal == 2 && key > last)) return;
    // acc[j][ob][v]: output head 16ob + 4kg + v, key 8ln + j
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            u4 o;
#pragma unroll
            for (int u = 0; u < 4; ++u) o[u] = pack2<T>(acc[2 * u][ob][v], acc[2 * u + 1][ob][v]);
            if (key + 7 > last) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (key + 2 * u > last) o[u] = (o[u] & 0xffff0000u) | (fill2 & 0x0000ffffu);
                    if (key + 2 * u + 1 > last) o[u] = (o[u] & 0x0000ffffu) | (fill2 & 0xffff0000u);
                }
            }
            __builtin_nontemporal_store(o, reinterpret_cast<u4 *>(y + base + (int64_t)(ob * 16 + kg * 4 + v) * plane + key));
        }
    }
}

// Dense mixing of HG = 64 or 128 heads on the matrix cores: the same scheme with the contraction run over HG/32 blocks
// of 32 input heads, one after the other.  A wavefront again owns 128 keys of one (batch, query row) and four blocks of
// 16 output heads (32 accumulators of 4 registers: what fits); with 128 heads two wavefronts share a key chunk, one per
// half of the output heads, and each reads all 128 input rows (the second read hits the cache).  The weight fragments of
// an input block are fetched ahead of its eight input vectors, straight from memory (the matrix is at most 32 KB and
// stays in cache).
template <typename T, int HG>
__global__ __launch_bounds__(64 * DM_WAVES, 2) void headmix_dense_wide(const T *__restrict__ x, const T *__restrict__ w,
                                                                  T *__restrict__ y, int C, int P, int Q, int causal,
                                                                  float fill, int wt, int qchunks)
{
    static_assert(HG == 64 || HG == 128, "blocks of 32 input heads, four blocks of 16 output heads per wavefront");
    constexpr int IB = HG / 32;               // blocks of 32 input heads
    constexpr int OW = 4;                     // blocks of 16 output heads per wavefront
    constexpr int SPLIT = HG / (16 * OW);     // wavefronts that share a key chunk (1 or 2)
    constexpr int CHUNKS = DM_WAVES / SPLIT;  // key chunks per workgroup
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, ln = lane & 15, kg = lane >> 4;
    const int groups = C / HG;
    unsigned b = blockIdx.x;
    const int qc = rotated_chunk(b, qchunks);
    const int p = (int)(b % (unsigned)P); b /= (unsigned)P;
    const int g = (int)(b % (unsigned)groups);
    const int64_t n = b / (unsigned)groups;
    const int q0 = (qc * CHUNKS + wave / SPLIT) * DM_KEYS;
    const int ob0 = (wave % SPLIT) * OW;      // first block of output heads of this wavefront
    if (q0 >= Q) return;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base = (n * C + (int64_t)g * HG) * plane + (int64_t)p * Q;  // head g*HG, row p, key 0
    const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;              // last key that is mixed
    const uint32_t fill2 = pack2<T>(fill, fill);
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    const int key = q0 + ln * 8;

    if (q0 > last) {  // wholly beyond the diagonal: fill only (causal == 2: not even that)
        const u4 fv = {fill2, fill2, fill2, fill2};
        if (key < Q && causal != 2) {
#pragma unroll
            for (int t = 0; t < 16; ++t)  // this lane's share of the wavefront's 64 output heads: 16kg .. 16kg+15
                __builtin_nontemporal_store(fv, reinterpret_cast<u4 *>(y + base + (int64_t)(ob0 * 16 + kg * 16 + t) * plane + key));
        }
        return;
    }

    f32x4 acc[8][OW];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int ob = 0; ob < OW; ++ob) acc[j][ob] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const T *xp = x + base + (int64_t)(kg * 8) * plane + (key <= last ? key : 0);
#pragma unroll 1
    for (int ib = 0; ib < IB; ++ib) {
        // w fragments of this input block: lane (output head ln of block ob, group kg) holds w[o][32ib + 8kg .. + 7]
        frag8<T> wf[OW];
#pragma unroll
        for (int ob = 0; ob < OW; ++ob) {
            const int o = g * HG + (ob0 + ob) * 16 + ln, i0 = g * HG + ib * 32 + kg * 8;
            if (!wt) {
                wf[ob] = *reinterpret_cast<const frag8<T> *>(w + (int64_t)o * C + i0);
            } else {  // the transposed matrix: a column of w, gathered element by element
#pragma unroll
                for (int t = 0; t < 8; ++t) wf[ob].v[t] = w[(int64_t)(i0 + t) * C + o];
            }
        }
        u4 xv[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)
            xv[t] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(xp + (int64_t)(ib * 32 + t) * plane));
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            u4 xt;  // heads 32ib + 8kg .. + 7 of key 8ln + j
#pragma unroll
            for (int u = 0; u < 4; ++u)
                xt[u] = __builtin_amdgcn_perm(xv[2 * u + 1][j >> 1], xv[2 * u][j >> 1], (j & 1) ? 0x07060302u : 0x05040100u);
            const frag8<T> xf = __builtin_bit_cast(frag8<T>, xt);
#pragma unroll
            for (int ob = 0; ob < OW; ++ob) mma16(acc[j][ob], wf[ob], xf);
        }
    }
    if (key >= Q || (causal == 2 && key > last)) return;
    // acc[j][ob][v]: output head 16(ob0 + ob) + 4kg + v, key 8ln + j
#pragma unroll
    for (int ob = 0; ob < OW; ++ob) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            u4 o;
#pragma unroll
            for (int u = 0; u < 4; ++u) o[u] = pack2<T>(acc[2 * u][ob][v], acc[2 * u + 1][ob][v]);
            if (key + 7 > last) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (key + 2 * u > last) o[u] = (o[u] & 0xffff0000u) | (fill2 & 0x0000ffffu);
                    if (key + 2 * u + 1 > last) o[u] = (o[u] & 0x0000ffffu) | (fill2 & 0xffff0000u);
                }
            }
            __builtin_nontemporal_store(o, reinterpret_cast<u4 *>(y + base + (int64_t)((ob0 + ob) * 16 + kg * 4 + v) * plane + key));
        }
    }
}

// The same for 16 heads: the contraction of a 16x16x16 product covers the 16 input heads; lane (ln, kg) fetches keys
// 8ln .. 8ln+7 of the heads 4kg .. 4kg+3 (four 16-byte loads), forms the column of key 8ln + j with two byte permutes,
// and after eight products holds keys 8ln .. 8ln+7 of the output heads 4kg + v.
typedef short hm_s4 __attribute__((ext_vector_type(4)));
typedef _Float16 hm_h4 __attribute__((ext_vector_type(4)));
typedef unsigned int hm_u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ f32x4 hm_mma16(bf16_t, hm_u2 a, hm_u2 b)
{
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(hm_s4, a), __builtin_bit_cast(hm_s4, b),
                                                     f32x4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
}
__device__ __forceinline__ f32x4 hm_mma16(f16_t, hm_u2 a, hm_u2 b)
{
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(hm_h4, a), __builtin_bit_cast(hm_h4, b),
                                                 f32x4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
}

template <typename T>
__global__ __launch_bounds__(64 * DM_WAVES, 4) void headmix_dense16(const T *__restrict__ x, const T *__restrict__ w,
                                                               T *__restrict__ y, int C, int P, int Q, int causal,
                                                               float fill, int wt, int qchunks)
{
    constexpr int HG = 16;  // heads mixed together
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, ln = lane & 15, kg = lane >> 4;
    const int groups = C / HG;
    unsigned b = blockIdx.x;
    const int qc = rotated_chunk(b, qchunks);
    const int p = (int)(b % (unsigned)P); b /= (unsigned)P;
    const int g = (int)(b % (unsigned)groups);
    const int64_t n = b / (unsigned)groups;
    const int q0 = (qc * DM_WAVES + wave) * DM_KEYS;
    if (q0 >= Q) return;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base = (n * C + (int64_t)g * HG) * plane + (int64_t)p * Q;  // head g*16, row p, key 0
    const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;              // last key that is mixed
    const uint32_t fill2 = pack2<T>(fill, fill);
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    const int key = q0 + ln * 8;

    if (q0 > last) {  // wholly beyond the diagonal: fill only (causal == 2: not even that)
        const u4 fv = {fill2, fill2, fill2, fill2};
        if (key < Q && causal != 2) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
                __builtin_nontemporal_store(fv, reinterpret_cast<u4 *>(y + base + (kg * 4 + t) * plane + key));
        }
        return;
    }

    const T *xp = x + base + (int64_t)(kg * 4) * plane + (key <= last ? key : 0);
    u4 xv[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) xv[t] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(xp + t * plane));

    // w fragment: lane (output head ln, group kg) holds w[o][4kg .. 4kg+3]
    hm_u2 wf;
    if (!wt) {
        wf = *reinterpret_cast<const hm_u2 *>(w + (int64_t)(g * HG + ln) * C + g * HG + kg * 4);
    } else {  // the transposed matrix: a column of w, gathered element by element (once per wavefront)
        struct alignas(8) quad { T v[4]; } col;
#pragma unroll
        for (int t = 0; t < 4; ++t) col.v[t] = w[(int64_t)(g * HG + kg * 4 + t) * C + g * HG + ln];
        wf = __builtin_bit_cast(hm_u2, col);
    }

    f32x4 acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const unsigned sel = (j & 1) ? 0x07060302u : 0x05040100u;
        const hm_u2 col = {__builtin_amdgcn_perm(xv[1][j >> 1], xv[0][j >> 1], sel),
                           __builtin_amdgcn_perm(xv[3][j >> 1], xv[2][j >> 1], sel)};  // heads 4kg .. 4kg+3 of key 8ln + j
        acc[j] = hm_mma16(T{}, wf, col);
    }
    if (key >= Q || (causal == 2 && key > last)) return;
    // acc[j][v]: output head 4kg + v, key 8ln + j
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        u4 o;
#pragma unroll
        for (int u = 0; u < 4; ++u) o[u] = pack2<T>(acc[2 * u][v], acc[2 * u + 1][v]);
        if (key + 7 > last) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (key + 2 * u > last) o[u] = (o[u] & 0xffff0000u) | (fill2 & 0x0000ffffu);
                if (key + 2 * u + 1 > last) o[u] = (o[u] & 0x0000ffffu) | (fill2 & 0xffff0000u);
            }
        }
        __builtin_nontemporal_store(o, reinterpret_cast<u4 *>(y + base + (int64_t)(kg * 4 + v) * plane + key));
    }
}

// Any group size: one (output head, vector) per lane-iteration, inputs re-read per output head.
template <typename T, int VEC>
__global__ __launch_bounds__(NT) void headmix_any(const T *__restrict__ x, const void *__restrict__ w,
                                                  T *__restrict__ y, int C, int G, int P, int Q, int causal,
                                                  float fill, int w_dtype, int wt, int qchunks)
{
    const int tid = threadIdx.x;
    const int groups = C / G;
    unsigned b = blockIdx.x;
    const int qc = rotated_chunk(b, qchunks);
    const int p = (int)(b % (unsigned)P); b /= (unsigned)P;
    const int g = (int)(b % (unsigned)groups);
    const int64_t n = b / (unsigned)groups;
    const int q = (qc * NT + tid) * VEC;
    if (q >= Q) return;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base = (n * C + (int64_t)g * G) * plane + (int64_t)p * Q + q;
    using V = vecN<T, VEC>;
    const T fill_t = from_float<T>(fill);
    for (int o = 0; o < G; ++o) {
        float acc[VEC];
#pragma unroll
        for (int u = 0; u < VEC; ++u) acc[u] = 0.0f;
        if (!(causal && q > p)) {
            for (int i = 0; i < G; ++i) {
                const float wv = load_any(w, w_dtype, w_index(g * G + o, g * G + i, C, wt));
                const V xv = *reinterpret_cast<const V *>(x + base + i * plane);
#pragma unroll
                for (int u = 0; u < VEC; ++u) acc[u] = fmaf(wv, to_float(xv.v[u]), acc[u]);
            }
        }
        V out;
#pragma unroll
        for (int u = 0; u < VEC; ++u) out.v[u] = (causal && q + u > p) ? fill_t : from_float<T>(acc[u]);
        *reinterpret_cast<V *>(y + base + o * plane) = out;
    }
}

template <typename T, int VEC>
int launch(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t P, int64_t Q, int G, int causal,
           float fill, int w_dtype, int wt, bool w_same_dtype, hipStream_t st)
{
    if constexpr (VEC == 8) {
        // 16 or 32 heads mixed densely, 16-bit data and weights of the same dtype: matrix cores
        // (MTA_HEADMIX_NO_MFMA=1 in the environment keeps the vector-ALU kernel, for comparisons)
        static const bool no_mfma = [] { const char *e = getenv("MTA_HEADMIX_NO_MFMA"); return e && e[0] == '1'; }();
        if (G == 16 && !no_mfma && w_same_dtype && aligned_to(w, 8) && C % 4 == 0) {
            const int qch = (int)((Q + DM_WAVES * DM_KEYS - 1) / (DM_WAVES * DM_KEYS));
            const int64_t blocks = N * (C / 16) * P * qch;
            if (blocks > 0x7fffffffLL) return MTA_ERR_SHAPE;
            hipLaunchKernelGGL((headmix_dense16<T>), dim3((unsigned)blocks), dim3(64 * DM_WAVES), 0, st, (const T *)x,
                               (const T *)w, (T *)y, (int)C, (int)P, (int)Q, causal, fill, wt, qch);
            return launch_status();
        }
        if (G == 32 && !no_mfma && w_same_dtype && aligned_to(w, 16) && C % 8 == 0) {
            const int qch = (int)((Q + DM_WAVES * DM_KEYS - 1) / (DM_WAVES * DM_KEYS));
            const int64_t blocks = N * (C / 32) * P * qch;
            if (blocks > 0x7fffffffLL) return MTA_ERR_SHAPE;
            hipLaunchKernelGGL((headmix_dense32<T>), dim3((unsigned)blocks), dim3(64 * DM_WAVES), 0, st, (const T *)x,
                               (const T *)w, (T *)y, (int)C, (int)P, (int)Q, causal, fill, wt, qch);
            return launch_status();
        }
        if ((G == 64 || G == 128) && !no_mfma && w_same_dtype && aligned_to(w, 16) && C % 8 == 0) {
            const int chunks = G == 64 ? DM_WAVES : DM_WAVES / 2;  // key chunks per workgroup
            const int qch = (int)((Q + chunks * DM_KEYS - 1) / (chunks * DM_KEYS));
            const int64_t blocks = N * (C / G) * P * qch;
            if (blocks > 0x7fffffffLL) return MTA_ERR_SHAPE;
            if (G == 64)
                hipLaunchKernelGGL((headmix_dense_wide<T, 64>), dim3((unsigned)blocks), dim3(64 * DM_WAVES), 0, st, (const T *)x,
                                   (const T *)w, (T *)y, (int)C, (int)P, (int)Q, causal, fill, wt, qch);
            else
                hipLaunchKernelGGL((headmix_dense_wide<T, 128>), dim3((unsigned)blocks), dim3(64 * DM_WAVES), 0, st, (const T *)x,
                                   (const T *)w, (T *)y, (int)C, (int)P, (int)Q, causal, fill, wt, qch);
            return launch_status();
        }
    }
    const int qchunks = (int)((Q + (int64_t)NT * VEC - 1) / ((int64_t)NT * VEC));
#define MTA_HM_CASE(g)                                                                                         \
    if (G == g) {                                                                                              \
        const int64_t blocks = N * (C / G) * P * qchunks;                                                      \
        if (blocks > 0x7fffffffLL) return MTA_ERR_SHAPE;                                                       \
        hipLaunchKernelGGL((headmix_fixed<T, g, VEC>), dim3((unsigned)blocks), dim3(NT), 0, st, (const T *)x, w, \
                           (T *)y, (int)C, (int)P, (int)Q, causal, fill, w_dtype, wt, qchunks);                 \
        return launch_status();                                                                                \
    }
    MTA_HM_CASE(1)
    MTA_HM_CASE(2)
    MTA_HM_CASE(4)
    MTA_HM_CASE(8)
    MTA_HM_CASE(16)
    MTA_HM_CASE(32)
#undef MTA_HM_CASE
    const int64_t blocks = N * (C / G) * P * qchunks;
    if (blocks > 0x7fffffffLL) return MTA_ERR_SHAPE;
    hipLaunchKernelGGL((headmix_any<T, VEC>), dim3((unsigned)blocks), dim3(NT), 0, st, (const T *)x, w, (T *)y, (int)C, G,
                       (int)P, (int)Q, causal, fill, w_dtype, wt, qchunks);
    return launch_status();
}

int headmix_entry(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t P, int64_t Q, int group_size,
                  int causal, float fill, int io_dtype, int w_dtype, int wt, void *stream)
{
    if (!x || !w || !y) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || P <= 0 || Q <= 0 || P > (1 << 24) || Q > (1 << 24) || C > 4096) return MTA_ERR_SHAPE;
    if (group_size < 0 || (group_size > 0 && C % group_size != 0)) return MTA_ERR_GROUP;
    if (!aligned_to(x, dtype_size(io_dtype)) || !aligned_to(y, dtype_size(io_dtype)) ||
        !aligned_to(w, dtype_size(w_dtype)))
        return MTA_ERR_ALIGN;
    const int G = group_size > 0 ? group_size : (int)C;
    hipStream_t st = (hipStream_t)stream;
    MTA_DISPATCH_IO(io_dtype, {
        constexpr int VEC = vec_of<io_t>::n;
        const bool vec_ok = (Q % VEC == 0) && aligned_to(x, 16) && aligned_to(y, 16);
        const bool same = w_dtype == io_dtype;
        return vec_ok ? launch<io_t, VEC>(x, w, y, N, C, P, Q, G, causal, fill, w_dtype, wt, same, st)
                      : launch<io_t, 1>(x, w, y, N, C, P, Q, G, causal, fill, w_dtype, wt, same, st);
    });
    return MTA_ERR_DTYPE;
}
}  // namespace

extern "C" int mta_headmix_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t P,
                               int64_t Q, int group_size, int causal, float fill, int io_dtype, int w_dtype,
                               void *stream)
{
    return headmix_entry(x, w, y, N, C, P, Q, group_size, causal == MTA_CAUSAL_LOWER_ONLY ? 2 : (causal ? 1 : 0), fill,
                         io_dtype, w_dtype, 0, stream);
}

extern "C" int mta_headmix_tril_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                                    int group_size, int io_dtype, int w_dtype, void *stream)
{
    return headmix_entry(x, w, y, N, C, P, Q, group_size, 2, 0.0f, io_dtype, w_dtype, 0, stream);
}

// dx[n,i,p,q] = sum_o w[o,i] dy[n,o,p,q]: the forward kernels with the transposed matrix; above the diagonal the
// gradient is +0 (those inputs were never read)
extern "C" int mta_headmix_bwd_input(const void *dy, const void *w, void *dx, int64_t N, int64_t C, int64_t P,
                                     int64_t Q, int group_size, int causal, int io_dtype, int w_dtype, void *stream)
{
    return headmix_entry(dy, w, dx, N, C, P, Q, group_size, causal == MTA_CAUSAL_LOWER_ONLY ? 2 : (causal ? 1 : 0), 0.0f,
                         io_dtype, w_dtype, 1, stream);
}
