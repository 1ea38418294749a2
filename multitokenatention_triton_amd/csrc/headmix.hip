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

#ifndef MTA_HM_THREADS
#define MTA_HM_THREADS 256
#endif
constexpr int NT = MTA_HM_THREADS;
#ifndef MTA_HM_NT
#define MTA_HM_NT 1
#endif
#ifndef MTA_HM_NTL
#define MTA_HM_NTL 1
#endif
#ifndef MTA_HM_WREG
#define MTA_HM_WREG 0
#endif
#ifndef MTA_HM_ROWS
#define MTA_HM_ROWS 1
#endif

template <typename T, int VEC> struct alignas(sizeof(T) * VEC) vecN { T v[VEC]; };

// outputs are written once and not read again by this kernel: store them as streaming (non-temporal) data
template <typename V> __device__ __forceinline__ V load_stream(const V *src)
{
#if MTA_HM_NTL
    if constexpr (sizeof(V) == 16) {
        typedef unsigned int u4 __attribute__((ext_vector_type(4)));
        return __builtin_bit_cast(V, __builtin_nontemporal_load(reinterpret_cast<const u4 *>(src)));
    }
#endif
    return *src;
}
template <typename V> __device__ __forceinline__ void store_stream(V *dst, const V &v)
{
#if MTA_HM_NT
    if constexpr (sizeof(V) == 16) {
        typedef unsigned int u4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(__builtin_bit_cast(u4, v), reinterpret_cast<u4 *>(dst));
        return;
    }
#endif
    *dst = v;
}

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

// G heads mixed inside one lane, G known at compile time.  A workgroup covers ROWS consecutive
// query rows of one key chunk, so a lane has ROWS*G independent 16-byte loads in flight.
template <typename T, int G, int VEC, int ROWS>
__global__ __launch_bounds__(NT) void headmix_fixed(const T *__restrict__ x, const void *__restrict__ w,
                                                    T *__restrict__ y, int C, int P, int Q, int causal,
                                                    float fill, int w_dtype, int qchunks, int pblocks)
{
#if MTA_HM_WREG
    constexpr bool WREG = G <= 8;
#else
    constexpr bool WREG = false;
#endif
    __shared__ float wsm[WREG ? 1 : G * G];
    const int tid = threadIdx.x;
    const int groups = C / G;
    unsigned b = blockIdx.x;
    const int qc = rotated_chunk(b, qchunks);
    const int p0 = (int)(b % (unsigned)pblocks) * ROWS; b /= (unsigned)pblocks;
    const int g = (int)(b % (unsigned)groups);
    const int64_t n = b / (unsigned)groups;
    const int q = (qc * NT + tid) * VEC;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base0 = (n * C + (int64_t)g * G) * plane + q;
    using V = vecN<T, VEC>;
    const T fill_t = from_float<T>(fill);
    V fillv;
#pragma unroll
    for (int u = 0; u < VEC; ++u) fillv.v[u] = fill_t;
    const int plast = (p0 + ROWS - 1 < P - 1) ? p0 + ROWS - 1 : P - 1;
    if (causal && qc * NT * VEC > plast) {  // chunk wholly above the diagonal for all rows: fill only, nothing read
        if (q < Q) {
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
                if (p0 + r < P) {
#pragma unroll
                    for (int o = 0; o < G; ++o) store_stream(reinterpret_cast<V *>(y + base0 + (int64_t)(p0 + r) * Q + o * plane), fillv);
                }
        }
        return;
    }
    // Issue all of this lane's loads first (unconditionally: a lane past the row end or above the
    // diagonal re-reads the row start), then fetch the weights, so that the latencies overlap.
    V xin[ROWS][G];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int p = (p0 + r < P) ? p0 + r : P - 1;
        const bool live = q < Q && !(causal && q > p);
        const int64_t lb = base0 + (int64_t)p * Q - (live ? 0 : q);
#pragma unroll
        for (int i = 0; i < G; ++i) xin[r][i] = load_stream(reinterpret_cast<const V *>(x + lb + i * plane));
    }
    float wr[WREG ? G * G : 1];
    if constexpr (WREG) {  // wave-uniform addresses: the weights arrive through the scalar unit
#pragma unroll
        for (int t = 0; t < G * G; ++t) wr[t] = load_any(w, w_dtype, (int64_t)(g * G + t / G) * C + g * G + t % G);
    } else {
        for (int t = tid; t < G * G; t += NT)
            wsm[t] = load_any(w, w_dtype, (int64_t)(g * G + t / G) * C + g * G + t % G);
        __syncthreads();
    }
    if (q >= Q) return;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int p = p0 + r;
        if (p >= P) break;
        const int64_t base = base0 + (int64_t)p * Q;
        if (causal && q > p) {
#pragma unroll
            for (int o = 0; o < G; ++o) store_stream(reinterpret_cast<V *>(y + base + o * plane), fillv);
            continue;
        }
#pragma unroll
        for (int o = 0; o < G; ++o) {
            float acc[VEC];
#pragma unroll
            for (int u = 0; u < VEC; ++u) acc[u] = 0.0f;
#pragma unroll
            for (int i = 0; i < G; ++i) {
                const float wv = WREG ? wr[o * G + i] : wsm[o * G + i];
#pragma unroll
                for (int u = 0; u < VEC; ++u) acc[u] = fmaf(wv, to_float(xin[r][i].v[u]), acc[u]);
            }
            V out;
#pragma unroll
            for (int u = 0; u < VEC; ++u) out.v[u] = (causal && q + u > p) ? fill_t : from_float<T>(acc[u]);
            store_stream(reinterpret_cast<V *>(y + base + o * plane), out);
        }
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
#ifndef MTA_HM_DM_WAVES
#define MTA_HM_DM_WAVES 4
#endif
constexpr int DM_WAVES = MTA_HM_DM_WAVES, DM_KEYS = 128;

template <typename T>
__global__ __launch_bounds__(64 * DM_WAVES, 4) void headmix_dense32(const T *__restrict__ x, const T *__restrict__ w,
                                                               T *__restrict__ y, int C, int P, int Q, int causal,
                                                               float fill, int qchunks)
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

    if (q0 > last) {  // wholly beyond the diagonal: fill only
        const u4 fv = {fill2, fill2, fill2, fill2};
        if (key < Q) {
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
    for (int ob = 0; ob < 2; ++ob)
        wf[ob] = *reinterpret_cast<const frag8<T> *>(w + (int64_t)(g * HG + ob * 16 + ln) * C + g * HG + kg * 8);

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
    if (key >= Q) return;
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

// Any group size: one (output head, vector) per lane-iteration, inputs re-read per output head.
template <typename T, int VEC>
__global__ __launch_bounds__(NT) void headmix_any(const T *__restrict__ x, const void *__restrict__ w,
                                                  T *__restrict__ y, int C, int G, int P, int Q, int causal,
                                                  float fill, int w_dtype, int qchunks)
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
                const float wv = load_any(w, w_dtype, (int64_t)(g * G + o) * C + g * G + i);
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
           float fill, int w_dtype, bool w_same_dtype, hipStream_t st)
{
    if constexpr (VEC == 8) {
        // 32 heads mixed densely, 16-bit data and weights of the same dtype: matrix cores (MTA_HEADMIX_NO_MFMA=1 in the
        // environment keeps the vector-ALU kernel, for comparisons)
        static const bool no_mfma = [] { const char *e = getenv("MTA_HEADMIX_NO_MFMA"); return e && e[0] == '1'; }();
        if (G == 32 && !no_mfma && w_same_dtype && aligned_to(w, 16) && C % 8 == 0) {
            const int qch = (int)((Q + DM_WAVES * DM_KEYS - 1) / (DM_WAVES * DM_KEYS));
            const int64_t blocks = N * (C / 32) * P * qch;
            if (blocks > 0x7fffffffLL) return MTA_ERR_SHAPE;
            hipLaunchKernelGGL((headmix_dense32<T>), dim3((unsigned)blocks), dim3(64 * DM_WAVES), 0, st, (const T *)x,
                               (const T *)w, (T *)y, (int)C, (int)P, (int)Q, causal, fill, qch);
            return launch_status();
        }
    }
    const int qchunks = (int)((Q + (int64_t)NT * VEC - 1) / ((int64_t)NT * VEC));
#define MTA_HM_CASE(g, rows)                                                                                       \
    if (G == g) {                                                                                                  \
        const int pblocks = (int)((P + rows - 1) / rows);                                                          \
        const int64_t blocks = N * (C / G) * pblocks * qchunks;                                                    \
        if (blocks > 0x7fffffffLL) return MTA_ERR_SHAPE;                                                           \
        hipLaunchKernelGGL((headmix_fixed<T, g, VEC, rows>), dim3((unsigned)blocks), dim3(NT), 0, st, (const T *)x, w, \
                           (T *)y, (int)C, (int)P, (int)Q, causal, fill, w_dtype, qchunks, pblocks);               \
        return launch_status();                                                                                    \
    }
    MTA_HM_CASE(1, MTA_HM_ROWS)
    MTA_HM_CASE(2, MTA_HM_ROWS)
    MTA_HM_CASE(4, MTA_HM_ROWS)
    MTA_HM_CASE(8, MTA_HM_ROWS)
    MTA_HM_CASE(16, 1)
    MTA_HM_CASE(32, 1)
#undef MTA_HM_CASE
    const int64_t blocks = N * (C / G) * P * qchunks;
    if (blocks > 0x7fffffffLL) return MTA_ERR_SHAPE;
    hipLaunchKernelGGL((headmix_any<T, VEC>), dim3((unsigned)blocks), dim3(NT), 0, st, (const T *)x, w, (T *)y, (int)C, G,
                       (int)P, (int)Q, causal, fill, w_dtype, qchunks);
    return launch_status();
}
}  // namespace

extern "C" int mta_headmix_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t P,
                               int64_t Q, int group_size, int causal, float fill, int io_dtype, int w_dtype,
                               void *stream)
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
        return vec_ok ? launch<io_t, VEC>(x, w, y, N, C, P, Q, G, causal, fill, w_dtype, same, st)
                      : launch<io_t, 1>(x, w, y, N, C, P, Q, G, causal, fill, w_dtype, same, st);
    });
    return MTA_ERR_DTYPE;
}
