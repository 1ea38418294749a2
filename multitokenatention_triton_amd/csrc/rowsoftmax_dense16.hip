// mix(w1) -> row softmax -> mix(w2) in one pass for mixing groups of 16 heads (a dense 16-head weight), 16-bit data.
//
// One workgroup of 4, 8 or 16 wavefronts per (batch, group, query row), by the length of the row; a row of 16 heads x
// up to 4096 keys stays in registers as fp32 (64 values per lane).  Both mixes run on the matrix cores: out[o][key] = sum_h w[o][h] x[h][key] is a
// 16x16x16 product with the weight as the A operand and, as the B operand, the 16 heads of 16 keys - lane (c = lane%16,
// g = lane/16) loads 16 bytes (keys 8c..8c+7) of each of the heads 4g..4g+3 and forms the column of key 8c+j from them
// with two byte permutes; product j of a tile leaves it out[4g+v][8c+j], v = 0..3: again four heads of one key, which is
// what the second mix takes as its operand without any exchange between lanes.  The 16 lanes that share g hold the same
// four heads: row maxima and sums fold inside DPP rows, then across the wavefronts through LDS.
// Rounding points are those of the unfused chain: mixed scores, probabilities and mixed probabilities are rounded to the
// I/O dtype.
#include "common.hpp"
#include "mfma.hpp"

namespace {
using namespace mta;

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef short m16_s4 __attribute__((ext_vector_type(4)));
typedef _Float16 m16_h4 __attribute__((ext_vector_type(4)));

constexpr int M16_NW = 16;    // wavefronts per workgroup, at most
constexpr int M16_TPW = 2;    // tiles per wavefront
constexpr int M16_TK = 128;   // keys per tile: 16 lanes x 8
constexpr int M16_HG = 16;    // heads mixed together
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ f32x4 mma_16x16x16(bf16_t, u32x2_t a, u32x2_t b)
{
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(m16_s4, a), __builtin_bit_cast(m16_s4, b),
                                                     f32x4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mma_16x16x16(f16_t, u32x2_t a, u32x2_t b)
{
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(m16_h4, a), __builtin_bit_cast(m16_h4, b),
                                                 f32x4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
}

template <bool IS_MAX> __device__ __forceinline__ float fold_op(float a, float b) { return IS_MAX ? fmaxf(a, b) : a + b; }
template <bool IS_MAX, int CTRL> __device__ __forceinline__ float dpp_fold(float v)
{
    const int moved = __builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, false);
    return fold_op<IS_MAX>(v, __uint_as_float((unsigned)moved));
}
// over the 16 lanes of a DPP row, result in all of them
template <bool IS_MAX> __device__ __forceinline__ float row_fold(float v)
{
    v = dpp_fold<IS_MAX, 0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_fold<IS_MAX, 0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_fold<IS_MAX, 0x141>(v);  // row_half_mirror
    v = dpp_fold<IS_MAX, 0x140>(v);  // row_mirror
    return v;
}

// Rows p0 .. p0+PR-1 of every (batch, group), NW wavefronts per row: a causal row p needs (p+1)/128 tiles, and a row
// that fits the tiles of 4 or 8 wavefronts runs in a workgroup of that size - four or two of them per CU instead of one
// (a row's workgroup walks "load, reduce, barrier, exponentials, reduce, barrier, store" alone).
template <typename T, bool HAS1, bool HAS2, int NW>
__global__ __launch_bounds__(64 * NW, 4) void mix16_softmax_kernel(const T *__restrict__ x, const T *__restrict__ w1,
                                                                   const T *__restrict__ w2, T *__restrict__ y, int C, int P,
                                                                   int Q, int causal, int fill_upper, int p0, int PR)
{
    constexpr int TPW = M16_TPW, HG = M16_HG;
    __shared__ __align__(16) float red[2][HG * NW];  // [0] maxima, [1] sums; entry head*NW + wavefront
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    const int ln = lane & 15, kg = lane >> 4;
    const unsigned groups = (unsigned)(C / HG);
    unsigned b = blockIdx.x;
    const int p = p0 + (int)(b % (unsigned)PR); b /= (unsigned)PR;
    const int g = (int)(b % groups);
    const int64_t n = b / groups;
    const int64_t plane = (int64_t)P * Q;
    const int64_t base = (n * C + (int64_t)g * HG) * plane + (int64_t)p * Q;  // head 16g, row p, key 0
    const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;               // last attended key

    // weight fragments: lane (output head ln, group kg) holds w[o][4kg .. 4kg+3]
    u32x2_t wf1 = {0u, 0u}, wf2 = {0u, 0u};
    if constexpr (HAS1) wf1 = *reinterpret_cast<const u32x2_t *>(w1 + (int64_t)(g * HG + ln) * C + g * HG + kg * 4);
    if constexpr (HAS2) wf2 = *reinterpret_cast<const u32x2_t *>(w2 + (int64_t)(g * HG + ln) * C + g * HG + kg * 4);

    // s[i][j][v]: head 4kg+v, key (i*NW + wave)*128 + 8ln + j (mixed and rounded scores, then exponentials)
    float s[TPW][8][4];
    float m[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
        const int q0 = (i * NW + wave) * M16_TK;
        const int key = q0 + ln * 8;
        if (q0 > last) {  // (wavefront-uniform) wholly beyond the attended keys
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) s[i][j][v] = -INFINITY;
            continue;
        }
        // beyond the attended keys a lane re-reads the row start; its values are masked below
        const T *xp = x + base + (int64_t)(kg * 4) * plane + (key <= last ? key : 0);
        u32x4_t xv[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) xv[t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(xp + t * plane));
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if constexpr (HAS1) {
                const unsigned sel = (j & 1) ? 0x07060302u : 0x05040100u;
                const u32x2_t col = {__builtin_amdgcn_perm(xv[1][j >> 1], xv[0][j >> 1], sel),
                                     __builtin_amdgcn_perm(xv[3][j >> 1], xv[2][j >> 1], sel)};  // heads 4kg..4kg+3 of key j
                const f32x4 a = mma_16x16x16(T{}, wf1, col);
                float r0 = a[0], r1 = a[1], r2 = a[2], r3 = a[3];
                unpack2<T>(pack2<T>(r0, r1), r0, r1);  // rounded to the I/O dtype
                unpack2<T>(pack2<T>(r2, r3), r2, r3);
                s[i][j][0] = r0; s[i][j][1] = r1; s[i][j][2] = r2; s[i][j][3] = r3;
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float lo, hi;
                    unpack2<T>(xv[v][j >> 1], lo, hi);
                    s[i][j][v] = (j & 1) ? hi : lo;
                }
            }
        }
        if (q0 + M16_TK - 1 > last) {  // (wavefront-uniform) the tile straddles the last attended key
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (key + j > last) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) s[i][j][v] = -INFINITY;
                }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) m[v] = fmaxf(m[v], s[i][j][v]);
    }

    // ---- row maxima: inside the DPP row, then across the wavefronts ----
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        m[v] = row_fold<true>(m[v]);
        if (ln == 0) red[0][(kg * 4 + v) * NW + wave] = m[v];
    }
    __syncthreads();
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const f32x4 *src = reinterpret_cast<const f32x4 *>(&red[0][(kg * 4 + v) * NW]);
        float r = -INFINITY;
#pragma unroll
        for (int c = 0; c < NW / 4; ++c) {
            const f32x4 q4 = src[c];
            r = fmaxf(fmaxf(r, fmaxf(q4[0], q4[1])), fmaxf(q4[2], q4[3]));
        }
        m[v] = r;  // finite: the row's first key is always attended
    }

    // ---- exponentials and their sums ----
    float inv[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const float mneg = -m[v] * LOG2E;
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                s[i][j][v] = __builtin_amdgcn_exp2f(fmaf(s[i][j][v], LOG2E, mneg));  // (-inf -> 0)
                acc += s[i][j][v];
            }
        acc = row_fold<false>(acc);
        if (ln == 0) red[1][(kg * 4 + v) * NW + wave] = acc;
    }
    __syncthreads();
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const f32x4 *src = reinterpret_cast<const f32x4 *>(&red[1][(kg * 4 + v) * NW]);
        float r = 0.0f;
#pragma unroll
        for (int c = 0; c < NW / 4; ++c) {
            const f32x4 q4 = src[c];
            r += (q4[0] + q4[1]) + (q4[2] + q4[3]);
        }
        const float rc = __builtin_amdgcn_rcpf(r);  // 1/sum: the hardware reciprocal and one Newton step
        inv[v] = fmaf(fmaf(-r, rc, 1.0f), rc, rc);
    }

    // ---- normalise, round, second mix, store ----
    if (NW < M16_NW && fill_upper) {  // keys beyond the tiles of this instance: wholly above the diagonal
        const u32x4_t z = {0u, 0u, 0u, 0u};
        for (int key = (TPW * NW + wave) * M16_TK + ln * 8; key < Q; key += NW * M16_TK) {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                __builtin_nontemporal_store(z, reinterpret_cast<u32x4_t *>(y + base + (int64_t)(kg * 4 + v) * plane + key));
        }
    }
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
        const int q0 = (i * NW + wave) * M16_TK;
        const int key = q0 + ln * 8;
        if (key >= Q) continue;
        if (key > last) {  // wholly above the diagonal: +0 only on request
            if (fill_upper) {
                const u32x4_t z = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    __builtin_nontemporal_store(z, reinterpret_cast<u32x4_t *>(y + base + (int64_t)(kg * 4 + v) * plane + key));
            }
            continue;
        }
        float o[8][4];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if constexpr (HAS2) {
                const u32x2_t col = {pack2<T>(s[i][j][0] * inv[0], s[i][j][1] * inv[1]),
                                     pack2<T>(s[i][j][2] * inv[2], s[i][j][3] * inv[3])};  // rounded probabilities
                const f32x4 a = mma_16x16x16(T{}, wf2, col);
#pragma unroll
                for (int v = 0; v < 4; ++v) o[j][v] = a[v];
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v) o[j][v] = s[i][j][v] * inv[v];
            }
        }
        // (keys beyond the last attended one carry probability 0 and come out as +0)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const u32x4_t out = {pack2<T>(o[0][v], o[1][v]), pack2<T>(o[2][v], o[3][v]), pack2<T>(o[4][v], o[5][v]),
                                 pack2<T>(o[6][v], o[7][v])};
            __builtin_nontemporal_store(out, reinterpret_cast<u32x4_t *>(y + base + (int64_t)(kg * 4 + v) * plane + key));
        }
    }
}
}  // namespace

namespace mta {
// Launches the kernel when it applies (16-bit I/O, weights of the same dtype, groups of 16 heads, Q % 8 == 0,
// Q <= 4096, 16-byte aligned tensors, 8-byte aligned weights); returns MTA_ERR_UNSUPPORTED otherwise.
int mix16_softmax_launch(const void *x, const void *w1, const void *w2, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                         int causal, int fill_upper, int io_dtype, int w_dtype, hipStream_t st)
{
    if (io_dtype == MTA_F32 || w_dtype != io_dtype || (!w1 && !w2) || C % M16_HG != 0 || Q % 8 != 0 ||
        Q > (int64_t)M16_NW * M16_TPW * M16_TK)
        return MTA_ERR_UNSUPPORTED;
    if (!aligned_to(x, 16) || !aligned_to(y, 16) || (w1 && !aligned_to(w1, 8)) || (w2 && !aligned_to(w2, 8)))
        return MTA_ERR_UNSUPPORTED;
    if (N * (C / M16_HG) * P > 0x7fffffffLL) return MTA_ERR_SHAPE;
    // rows by the number of wavefronts their attended keys need: [0, r4) take 4, [r4, r8) take 8, the rest 16
    const int64_t k4 = 4 * M16_TPW * M16_TK, k8 = 8 * M16_TPW * M16_TK;
    const int64_t r4 = !causal ? (Q <= k4 ? P : 0) : (P < k4 ? P : k4);
    const int64_t r8 = !causal ? (Q <= k8 ? P : 0) : (P < k8 ? P : k8);
#define MTA_M16_LAUNCH(T, h1, h2, nw, first, rows)                                                                      \
    if ((rows) > 0)                                                                                                     \
    hipLaunchKernelGGL((mix16_softmax_kernel<T, h1, h2, nw>), dim3((unsigned)(N * (C / M16_HG) * (rows))), dim3(64 * nw), \
                       0, st, (const T *)x, (const T *)w1, (const T *)w2, (T *)y, (int)C, (int)P, (int)Q, causal,       \
                       fill_upper, (int)(first), (int)(rows))
#define MTA_M16_ALL(T, h1, h2)                                    \
    MTA_M16_LAUNCH(T, h1, h2, 4, 0, r4);                          \
    MTA_M16_LAUNCH(T, h1, h2, 8, r4, (r8 > r4 ? r8 - r4 : 0));    \
    MTA_M16_LAUNCH(T, h1, h2, 16, (r8 > r4 ? r8 : r4), P - (r8 > r4 ? r8 : r4))
#define MTA_M16_CASES(T)                                          \
    if (w1 && w2) { MTA_M16_ALL(T, true, true); }                 \
    else if (w1) { MTA_M16_ALL(T, true, false); }                 \
    else { MTA_M16_ALL(T, false, true); }
    if (io_dtype == MTA_BF16) { MTA_M16_CASES(bf16_t) }
    else { MTA_M16_CASES(f16_t) }
#undef MTA_M16_CASES
#undef MTA_M16_ALL
#undef MTA_M16_LAUNCH
    return launch_status();
}
}  // namespace mta
