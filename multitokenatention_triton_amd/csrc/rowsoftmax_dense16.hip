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
#include <cstdlib>

#include "common.hpp"
#include "mfma.hpp"
#include "strip_common.hpp"

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

// Lists of rows per workgroup.  A workgroup that walks "load, reduce, barrier, exponentials, reduce, barrier, store"
// alone on its CU leaves the memory pipe idle while it computes and the vector units idle while it loads, so here a
// workgroup of 16 wavefronts takes a list of steps of one (batch, group) - a step is one row of more than 2048 attended
// keys (16 wavefronts), two rows of more than 1024 (8 each) or four shorter ones (4 each), longest rows first - and the
// next step's input is copied global -> LDS asynchronously while the current rows are reduced and stored: every lane
// copies the 8 vectors it will read itself (1 KB per wavefront and instruction, 128 KB per step), so the staging memory
// needs no barrier, only the wavefront's own count of outstanding memory instructions - the copies of a row are followed
// by the stores of the row before it, 4 per tile that stores, which the wait leaves in flight.
// Rows [0, r4) take 4 wavefronts, [r4, r8) take 8, [r8, P) take 16.
// MASKED instances: key_bias (fp32 (N,Q), or NULL) is added to the mixed, rounded scores and the sum rounded again (the
// reference's `scores + mask` for one value per key; the batch entry's bias row waits in LDS); row_lo (int32 (N,P), or
// NULL) is the first key a row sees (band mask): the keys ahead of it count as -inf, and a tile that lies wholly ahead of
// it is neither copied nor computed - it is stored as +0.
template <typename T, bool HAS1, bool HAS2, bool MASKED = false>
__global__ __launch_bounds__(64 * M16_NW, 1) void mix16_softmax_rows_kernel(const T *__restrict__ x, const T *__restrict__ w1,
                                                                           const T *__restrict__ w2, T *__restrict__ y, int C,
                                                                           int P, int Q, int causal, int fill_upper, int r4,
                                                                           int r8, int wpg, int tri_in, int tri_out,
                                                                           const float *__restrict__ key_bias,
                                                                           const int *__restrict__ row_lo)
{
    constexpr int NW = M16_NW, TPW = M16_TPW, HG = M16_HG;
    __shared__ __align__(16) float kbias[MASKED ? NW * TPW * M16_TK : 4];  // (MASKED) the batch entry's key bias
    __shared__ __align__(16) u32x4_t stage[NW * TPW * 4 * 64];  // [wavefront][tile][head of the lane's four][lane]
    __shared__ __align__(16) float red[2][HG * NW];             // [0] maxima, [1] sums; entry (row*16 + head)*NWR + wavefront
    __shared__ __align__(8) u32x2_t wts[2][64];                 // the lanes' weight fragments
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    const unsigned groups = (unsigned)(C / HG);
    const int j_wg = (int)(blockIdx.x % (unsigned)wpg);
    const unsigned ng = blockIdx.x / (unsigned)wpg;
    const int g = (int)(ng % groups);
    const int64_t n = ng / groups;
    const unsigned plane = (unsigned)P * (unsigned)Q;  // (16 planes of 16-bit values within 4 GB: checked by the launch)
    const int64_t base0 = (n * C + (int64_t)g * HG) * (int64_t)plane;  // head 16g, row 0, key 0
    // (tri_in / tri_out: that tensor is in the triangular layout - causal, square, groups of 16 heads interleaved by rows,
    // nothing above the diagonal: row p of the group starts 16*tri_rowoff(p) elements into the group, head i a row length on)
    const int64_t tbase0 = (n * groups + g) * (HG * tri_rowoff(P));
    // the steps of a (batch, group), longest rows first, and the k-th of this workgroup: its workgroups take the steps in
    // turn, back and forth, so that each gets short and long rows alike
    const int n16 = P - r8, n8 = (r8 - r4 + 1) >> 1, nsteps = n16 + n8 + ((r4 + 3) >> 2);
    auto step_at = [&](int k) { return k * wpg + ((k & 1) ? wpg - 1 - j_wg : j_wg); };
    // step t for this wavefront: log2 of the wavefronts per row, the row (negative: none)
    auto row_of = [&](int t, int &lg) {
        if (t >= nsteps) { lg = 4; return -1; }
        if (t < n16) { lg = 4; return P - 1 - t; }
        if (t < n16 + n8) {
            lg = 3;
            const int p = r8 - 1 - (2 * (t - n16) + (wave >> 3));
            return p >= r4 ? p : -1;
        }
        lg = 2;
        return r4 - 1 - (4 * (t - n16 - n8) + (wave >> 2));
    };

    // weight fragments: lane (output head ln, group kg) holds w[o][4kg .. 4kg+3]; kept in LDS between their uses
    if (wave == 0) {
        const int64_t wo = (int64_t)(g * HG + (lane & 15)) * C + g * HG + (lane >> 4) * 4;
        if constexpr (HAS1) wts[0][lane] = *reinterpret_cast<const u32x2_t *>(w1 + wo);
        if constexpr (HAS2) wts[1][lane] = *reinterpret_cast<const u32x2_t *>(w2 + wo);
    }
    if constexpr (MASKED) {
        if (key_bias)
            for (int q = (int)threadIdx.x; q < Q; q += 64 * NW) kbias[q] = key_bias[n * Q + q];
    }
    __syncthreads();  // (also: nothing is in flight when the loop starts counting)
    // first visible key of row p (0 without a band mask)
    auto lo_of = [&](int p) {
        int lo = 0;
        if constexpr (MASKED) {
            if (row_lo && p >= 0) lo = row_lo[n * P + p];
        }
        return lo < 0 ? 0 : lo;
    };

    // (ln, kg: the lane's key octet and head quad, handed in by the loop: see there)
    auto issue = [&](int p, int lg, int ln, int kg) {
        const int wr = wave & ((1 << lg) - 1);
        const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;
        // (uniform base + 32-bit lane offset)
        const char *xrow = reinterpret_cast<const char *>(tri_in ? x + tbase0 + HG * tri_rowoff(p) : x + base0 + (int64_t)p * Q);
        const unsigned xplane = tri_in ? (unsigned)tri_rowlen(p) : plane;
        const int lo = lo_of(p);
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int q0 = ((i << lg) + wr) * M16_TK;
            if (q0 > last || q0 + M16_TK <= lo) continue;  // (wavefront-uniform) nothing attended / nothing visible in the tile
            const int key = q0 + ln * 8;
            // beyond the attended keys a lane re-reads the row start; its values are masked
            const unsigned off = ((unsigned)(kg * 4) * xplane + (unsigned)(key <= last ? key : 0)) * (unsigned)sizeof(T);
#pragma unroll
            for (int t = 0; t < 4; ++t)
                __builtin_amdgcn_global_load_lds((glb_void_t *)(xrow + (off + (unsigned)t * xplane * (unsigned)sizeof(T))),
                                                 (lds_void_t *)(stage + ((wave * TPW + i) * 4 + t) * 64), 16, 0, 0);
        }
    };
    const unsigned stage_wave = (unsigned)(uintptr_t)(lds_void_t *)stage + (unsigned)(wave * TPW * 4 * 64) * 16u;

    if (step_at(0) >= nsteps) return;
    int lg, lgn;
    int p = row_of(step_at(0), lg);
    if (p >= 0) issue(p, lg, lane & 15, lane >> 4);
    int nst = 0;  // store instructions of the row before, issued after this row's copies
    for (int k = 0;; ++k) {
        const int pn = row_of(step_at(k + 1), lgn);
        const bool more = step_at(k + 1) < nsteps;  // (the same answer in every wavefront)
        const bool active = p >= 0;                 // (the last step of a kind may not have a row for everybody)
        const int nwr = 1 << lg, sub = wave >> lg, wr = wave & (nwr - 1);  // which of the rows, which wavefront of that row
        // what depends on the lane number is derived anew for every row: kept across the loop, the key numbers and
        // address offsets of all tiles would occupy the registers the row's values need
        const int lane_o = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, (unsigned)opaque(0)));  // (the lane number)
        const int ln = lane_o & 15, kg = lane_o >> 4;
        const unsigned stage_lds = stage_wave + (unsigned)lane_o * 16u;
        char *const yrow = reinterpret_cast<char *>(tri_out ? y + tbase0 + HG * tri_rowoff(p > 0 ? p : 0) : y + base0 + (int64_t)p * Q);
        const unsigned yplane = tri_out ? (unsigned)tri_rowlen(p > 0 ? p : 0) : plane;
        const int last = !active ? -1 : causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;
        const int lo = lo_of(p);
        if (nst == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else if (nst == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

        // s[i][j][v]: head 4kg+v, key (i*nwr + wr)*128 + 8ln + j (mixed and rounded scores, then exponentials)
        float s[TPW][8][4];
        float m[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        {
        u32x2_t wf1 = {0u, 0u};
        if constexpr (HAS1) wf1 = wts[0][lane_o];
        static_for<TPW>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int q0 = ((i << lg) + wr) * M16_TK;
            const int key = q0 + ln * 8;
            if (q0 > last || q0 + M16_TK <= lo) return;  // (wavefront-uniform) no attended or no visible key: s[i] stays unused
            u32x4_t xv[4];
            lds_load4x16_sync(stage_lds, i * 4096, xv[0], xv[1], xv[2], xv[3]);
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
            if constexpr (MASKED) {
                if (key_bias) {  // (wavefront-uniform) the sum in the I/O dtype, as the unfused chain stores it
                    const int kq = key <= last ? key : 0;
                    const f32x4 kb0 = *reinterpret_cast<const f32x4 *>(&kbias[kq]), kb1 = *reinterpret_cast<const f32x4 *>(&kbias[kq + 4]);
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float kb = j < 4 ? kb0[j & 3] : kb1[j & 3];
                        float r0 = s[i][j][0] + kb, r1 = s[i][j][1] + kb, r2 = s[i][j][2] + kb, r3 = s[i][j][3] + kb;
                        unpack2<T>(pack2<T>(r0, r1), r0, r1);
                        unpack2<T>(pack2<T>(r2, r3), r2, r3);
                        s[i][j][0] = r0; s[i][j][1] = r1; s[i][j][2] = r2; s[i][j][3] = r3;
                    }
                }
                if (q0 < lo) {  // (wavefront-uniform) the tile holds the row's first visible key
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (key + j < lo) {
#pragma unroll
                            for (int v = 0; v < 4; ++v) s[i][j][v] = -INFINITY;
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
        });
        }
        // this row's staging vectors are in registers: the next row's copies may overwrite them
        if (pn >= 0) issue(pn, lgn, ln, kg);

        // ---- row maxima: inside the DPP row, then across the row's wavefronts ----
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            m[v] = row_fold<true>(m[v]);
            if (ln == 0) red[0][(((sub * HG + kg * 4 + v)) << lg) + wr] = m[v];
        }
        lds_wait();
        wg_barrier();  // (no memory fence: the copies stay in flight)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const f32x4 *src = reinterpret_cast<const f32x4 *>(&red[0][(sub * HG + kg * 4 + v) << lg]);
            float r = -INFINITY;
#pragma unroll
            for (int c = 0; c < NW / 4; ++c) {
                if (c * 4 >= nwr) break;  // (wavefront-uniform)
                const f32x4 q4 = src[c];
                r = fmaxf(fmaxf(r, fmaxf(q4[0], q4[1])), fmaxf(q4[2], q4[3]));
            }
            m[v] = r;  // finite: the row's first key is always attended
        }

        // ---- exponentials and their sums ----
        float inv[4];
        {
            float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int v = 0; v < 4; ++v) m[v] = -m[v] * LOG2E;
#pragma unroll
            for (int i = 0; i < TPW; ++i) {
                if (((i << lg) + wr) * M16_TK > last || ((i << lg) + wr + 1) * M16_TK <= lo) continue;  // (wavefront-uniform) no attended / visible key in this tile
#pragma unroll
                for (int j = 0; j < 8; ++j)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        s[i][j][v] = __builtin_amdgcn_exp2f(fmaf(s[i][j][v], LOG2E, m[v]));  // (-inf -> 0)
                        acc[v] += s[i][j][v];
                    }
            }
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float a = row_fold<false>(acc[v]);
                if (ln == 0) red[1][((sub * HG + kg * 4 + v) << lg) + wr] = a;
            }
        }
        lds_wait();
        wg_barrier();
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const f32x4 *src = reinterpret_cast<const f32x4 *>(&red[1][(sub * HG + kg * 4 + v) << lg]);
            float r = 0.0f;
#pragma unroll
            for (int c = 0; c < NW / 4; ++c) {
                if (c * 4 >= nwr) break;  // (wavefront-uniform)
                const f32x4 q4 = src[c];
                r += (q4[0] + q4[1]) + (q4[2] + q4[3]);
            }
            const float rc = __builtin_amdgcn_rcpf(r);  // 1/sum: the hardware reciprocal and one Newton step
            inv[v] = fmaf(fmaf(-r, rc, 1.0f), rc, rc);
        }

        // ---- normalise, round, second mix, store: four store instructions per tile that stores anything ----
        nst = 0;
        u32x2_t wf2 = {0u, 0u};
        if constexpr (HAS2) wf2 = wts[1][lane_o];
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int q0 = ((i << lg) + wr) * M16_TK;
            const int key = q0 + ln * 8;
            if (!active || q0 >= Q || (q0 > last && !fill_upper)) continue;  // (wavefront-uniform; lane 0 of the others stores)
            nst += 4;
            if (q0 > last || q0 + M16_TK <= lo) {  // (wavefront-uniform) wholly above the diagonal, stored on request, or wholly hidden: +0
                if (key < Q) {
                    const u32x4_t z = {0u, 0u, 0u, 0u};
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        __builtin_nontemporal_store(z, reinterpret_cast<u32x4_t *>(yrow + ((unsigned)(kg * 4 + v) * yplane + (unsigned)key) * (unsigned)sizeof(T)));
                }
                continue;
            }
            // (keys beyond the last attended one carry probability 0 and come out as +0; above the diagonal they are
            // stored on request only)  Two keys at a time, packed at once: few registers between product and store.
            u32x4_t out[4];
#pragma unroll
            for (int jp = 0; jp < 4; ++jp) {
                float o[2][4];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int j = jp * 2 + h;
                    if constexpr (HAS2) {
                        const u32x2_t col = {pack2<T>(s[i][j][0] * inv[0], s[i][j][1] * inv[1]),
                                             pack2<T>(s[i][j][2] * inv[2], s[i][j][3] * inv[3])};  // rounded probabilities
                        const f32x4 a = mma_16x16x16(T{}, wf2, col);
#pragma unroll
                        for (int v = 0; v < 4; ++v) o[h][v] = a[v];
                    } else {
#pragma unroll
                        for (int v = 0; v < 4; ++v) o[h][v] = s[i][j][v] * inv[v];
                    }
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) out[v][jp] = pack2<T>(o[0][v], o[1][v]);
            }
            if (key < Q && (fill_upper || key <= last)) {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    __builtin_nontemporal_store(out[v], reinterpret_cast<u32x4_t *>(yrow + ((unsigned)(kg * 4 + v) * yplane + (unsigned)key) * (unsigned)sizeof(T)));
            }
        }
        // keys beyond the tiles of this instance lie wholly above the diagonal: +0 on request (plain vector stores; the
        // count above leaves them to the wait of the row after, which then waits for a few copies more than it must)
        if (lg < 4 && fill_upper && active) {
            const u32x4_t z = {0u, 0u, 0u, 0u};
            for (int key = (TPW * nwr + wr) * M16_TK + ln * 8; key < Q; key += nwr * M16_TK) {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    __builtin_nontemporal_store(z, reinterpret_cast<u32x4_t *>(yrow + ((unsigned)(kg * 4 + v) * yplane + (unsigned)key) * (unsigned)sizeof(T)));
            }
        }
        p = pn;
        lg = lgn;
        if (!more) break;
        // (red[0] is next written after the second barrier above and red[1] after the next first one: by then every
        // wavefront has read what this row left there)
    }
}
}  // namespace

namespace mta {
// Launches the kernel when it applies (16-bit I/O, weights of the same dtype, groups of 16 heads, Q % 8 == 0,
// Q <= 4096, 16-byte aligned tensors, 8-byte aligned weights); returns MTA_ERR_UNSUPPORTED otherwise.
int mix16_softmax_launch(const void *x, const void *w1, const void *w2, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                         int causal, int fill_upper, int io_dtype, int w_dtype, hipStream_t st, int tri_in, int tri_out,
                         const float *key_bias, const int *row_lo)
{
    const bool masked = key_bias || row_lo;
    if (row_lo && !causal) return MTA_ERR_UNSUPPORTED;
    if (io_dtype == MTA_F32 || w_dtype != io_dtype || (!w1 && !w2) || C % M16_HG != 0 || Q % 8 != 0 ||
        Q > (int64_t)M16_NW * M16_TPW * M16_TK)
        return MTA_ERR_UNSUPPORTED;
    if (!aligned_to(x, 16) || !aligned_to(y, 16) || (w1 && !aligned_to(w1, 8)) || (w2 && !aligned_to(w2, 8)))
        return MTA_ERR_UNSUPPORTED;
    if (N * (C / M16_HG) * P > 0x7fffffffLL) return MTA_ERR_SHAPE;
    const bool small_planes = P * Q <= (1LL << 27);  // the row-list kernel's 32-bit offsets inside a group of 16 planes
    // rows by the number of wavefronts their attended keys need: [0, r4) take 4, [r4, r8) take 8, the rest 16
    static const bool no_rows = [] { const char *e = getenv("MTA_MIX16_NO_ROW_LISTS"); return e && e[0] == '1'; }();  // test switch
    const int64_t k4 = 4 * M16_TPW * M16_TK, k8 = 8 * M16_TPW * M16_TK;
    const int64_t r4 = !causal ? (Q <= k4 ? P : 0) : (P < k4 ? P : k4);
    const int64_t r8x = !causal ? (Q <= k8 ? P : 0) : (P < k8 ? P : k8), r8 = r8x > r4 ? r8x : r4;
#define MTA_M16_LAUNCH(T, h1, h2, nw, first, rows)                                                                      \
    if ((rows) > 0)                                                                                                     \
    hipLaunchKernelGGL((mix16_softmax_kernel<T, h1, h2, nw>), dim3((unsigned)(N * (C / M16_HG) * (rows))), dim3(64 * nw), \
                       0, st, (const T *)x, (const T *)w1, (const T *)w2, (T *)y, (int)C, (int)P, (int)Q, causal,       \
                       fill_upper, (int)(first), (int)(rows))
    // one launch of row lists, about one workgroup per CU; or a launch per kind of row, a workgroup per row
#define MTA_M16_ALL(T, h1, h2)                                                                                          \
    if (no_rows || !small_planes) {                                                                                     \
        if (tri_in || tri_out || masked) return MTA_ERR_UNSUPPORTED;                                                    \
        MTA_M16_LAUNCH(T, h1, h2, 4, 0, r4);                                                                            \
        MTA_M16_LAUNCH(T, h1, h2, 8, r4, r8 - r4);                                                                      \
        MTA_M16_LAUNCH(T, h1, h2, 16, r8, P - r8);                                                                      \
    } else {                                                                                                            \
        const int64_t steps = (P - r8) + (r8 - r4 + 1) / 2 + (r4 + 3) / 4;                                              \
        int64_t wpg = device_cu_count() / (N * (C / M16_HG));                                                           \
        wpg = wpg < 1 ? 1 : (wpg > steps ? steps : wpg);                                                                \
        if (masked)                                                                                                     \
            hipLaunchKernelGGL((mix16_softmax_rows_kernel<T, h1, h2, true>), dim3((unsigned)(N * (C / M16_HG) * wpg)),  \
                               dim3(64 * M16_NW), 0, st, (const T *)x, (const T *)w1, (const T *)w2, (T *)y, (int)C,    \
                               (int)P, (int)Q, causal, fill_upper, (int)r4, (int)r8, (int)wpg, tri_in, tri_out,         \
                               key_bias, row_lo);                                                                       \
        else                                                                                                            \
            hipLaunchKernelGGL((mix16_softmax_rows_kernel<T, h1, h2>), dim3((unsigned)(N * (C / M16_HG) * wpg)),        \
                               dim3(64 * M16_NW), 0, st, (const T *)x, (const T *)w1, (const T *)w2, (T *)y, (int)C,    \
                               (int)P, (int)Q, causal, fill_upper, (int)r4, (int)r8, (int)wpg, tri_in, tri_out,         \
                               nullptr, nullptr);                                                                       \
    }
#define MTA_M16_CASES(T)                                          \
    if (w1 && w2) { MTA_M16_ALL(T, true, true) }                  \
    else if (w1) { MTA_M16_ALL(T, true, false) }                  \
    else { MTA_M16_ALL(T, false, true) }
    if (io_dtype == MTA_BF16) { MTA_M16_CASES(bf16_t) }
    else { MTA_M16_CASES(f16_t) }
#undef MTA_M16_CASES
#undef MTA_M16_ALL
#undef MTA_M16_LAUNCH
    return launch_status();
}
}  // namespace mta
