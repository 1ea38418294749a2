// Gradient of the depthwise causal conv with respect to its (C,R,S) kernel:
//
//   dw[c,i,j] = sum_{n,p,q} xm[n,c, p+i-(R-1), q+j-(S-1)/2] * dym[n,c,p,q]
//
// xm = x with out-of-range taps and (causal) col>row read as 0, dym = dy with (causal) q>p read as 0 -- the masks of
// the forward pass.  Accumulation is fp32 and hierarchical: a lane keeps its R*S sums in registers over all the
// tiles it visits, a workgroup reduces them once at the end and writes one partial kernel to a scratch buffer, and a
// second small kernel adds the partials of each channel in a fixed order (the result does not depend on timing; the
// reference accumulates in fp64 with atomics, convolution_2d_trit.py:236-295).
//
// Work split: the persistent workgroups are divided among the channels; the workgroups of a channel walk that
// channel's (batch, 32x64 tile) list with a stride.  Tiles wholly above the diagonal are skipped.
//
// 16-bit tensors whose rows are a multiple of 8 keys take the matrix cores (conv2d_bwd_weight_mfma): for a fixed
// key offset j the sums over q of dy[p,q] * x[p',q+j-pad] for 16 rows p and 16 rows p' are one 16x16 product with the
// keys as contraction index, and the taps (i,j) are the entries p'-p = i-(R-1) of it.  Every 16-row block of dy meets
// the two 16-row blocks of x that hold its R-1 rows of halo, and all blocks add into the same 2*S accumulators, since
// only p'-p matters.  The operand of offset j is the lane's 24-key window of x shifted by j keys in registers.
#include <atomic>

#include "common.hpp"
#include "mfma.hpp"

namespace {
using namespace mta;

constexpr int NT = 256;
constexpr int TM = 32;  // tile rows   (thread t: row t/8)
constexpr int TN = 64;  // tile cols   (thread t: cols 8*(t%8) .. +7)

// sum over the wavefront, result in every lane
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
    return v;
}

// stage the (TM+R-1) x (TN+S-1) halo tile of x as fp32 with the forward pass's masks applied
template <typename T>
__device__ __forceinline__ void stage_x(const T *xp, float *tile, int LD, int H, int W, int p0, int q0, int R, int S,
                                        int causal, int tid)
{
    const int pad_h = R - 1, pad_w = (S - 1) / 2;
    const int rows = TM + R - 1, cols = TN + S - 1;
    for (int rr = tid / 64; rr < rows; rr += NT / 64) {
        const int h = p0 - pad_h + rr;
        const bool row_ok = h >= 0 && h < H;
        for (int cc = tid % 64; cc < cols; cc += 64) {
            const int k = q0 - pad_w + cc;
            float v = 0.0f;
            if (row_ok && k >= 0 && k < W && (!causal || k <= h)) v = to_float(xp[(int64_t)h * W + k]);
            tile[rr * LD + cc] = v;
        }
    }
}

// (channel, first item, item stride) of a workgroup; items of a channel = batch * tiles
struct split_t { int channel, sub, bpc; };
__device__ __forceinline__ split_t split_of(int block, int C, int bpc)
{
    return split_t{block / bpc, block % bpc, bpc};
}

// Kernel size known at compile time: all R*S sums of a lane live in registers.
template <typename T, int R, int S>
__global__ __launch_bounds__(NT) void conv2d_bwd_weight_fixed(const T *__restrict__ x, const T *__restrict__ dy,
                                                              float *__restrict__ partial, int N, int C, int H, int W,
                                                              int causal, int tiles_m, int tiles_n, int bpc, int vec_ok)
{
    constexpr int LD = TN + S;  // S-1 halo columns + 1 pad
    __shared__ float tile[(TM + R - 1) * LD];
    __shared__ float red[NT / 64][R * S];
    const int tid = threadIdx.x;
    const split_t sp = split_of(blockIdx.x, C, bpc);
    const int c = sp.channel;
    const int tr = tid >> 3, tc = (tid & 7) * 8;

    float acc[R][S];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int j = 0; j < S; ++j) acc[i][j] = 0.0f;

    const int tiles = tiles_m * tiles_n;
    const int64_t items = (int64_t)N * tiles;
    for (int64_t it = sp.sub; it < items; it += sp.bpc) {
        const int n = (int)(it / tiles), t = (int)(it % tiles);
        const int tm = t / tiles_n, tn = t % tiles_n;
        const int p0 = tm * TM, q0 = tn * TN;
        if (causal && q0 > p0 + TM - 1) continue;  // dy is masked to zero on the whole tile (uniform per workgroup)
        const int64_t plane = ((int64_t)n * C + c) * H * W;
        __syncthreads();  // the previous tile's readers are done
        stage_x<T>(x + plane, tile, LD, H, W, p0, q0, R, S, causal, tid);
        // this lane's 8 gradient values
        float g[8];
        const int p = p0 + tr, q = q0 + tc;
        if (vec_ok && p < H && q + 8 <= W) {  // eight contiguous values, 16-byte aligned
            const T *src = dy + plane + (int64_t)p * W + q;
            T raw[8];
            if constexpr (sizeof(T) == 2) {
                *reinterpret_cast<pack16<T> *>(raw) = *reinterpret_cast<const pack16<T> *>(src);
            } else {
                *reinterpret_cast<pack16<T> *>(raw) = *reinterpret_cast<const pack16<T> *>(src);
                *reinterpret_cast<pack16<T> *>(raw + 4) = *reinterpret_cast<const pack16<T> *>(src + 4);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) g[u] = (causal && q + u > p) ? 0.0f : to_float(raw[u]);
        } else {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const bool ok = p < H && q + u < W && !(causal && q + u > p);
                g[u] = ok ? to_float(dy[plane + (int64_t)p * W + q + u]) : 0.0f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < R; ++i) {
            float win[S + 7];
            const float *src = tile + (tr + i) * LD + tc;
#pragma unroll
            for (int u = 0; u < S + 7; ++u) win[u] = src[u];
#pragma unroll
            for (int j = 0; j < S; ++j) {
                float a = acc[i][j];
#pragma unroll
                for (int u = 0; u < 8; ++u) a = fmaf(g[u], win[u + j], a);
                acc[i][j] = a;
            }
        }
    }
    // workgroup reduction, once
    const int wave = tid >> 6, lane = tid & 63;
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int j = 0; j < S; ++j) {
            const float s = wave_sum(acc[i][j]);
            if (lane == 0) red[wave][i * S + j] = s;
        }
    __syncthreads();
    for (int t = tid; t < R * S; t += NT) {
        float s = 0.0f;
#pragma unroll
        for (int wv = 0; wv < NT / 64; ++wv) s += red[wv][t];
        partial[((int64_t)c * bpc + sp.sub) * (R * S) + t] = s;
    }
}

// ---- matrix-core kernel -------------------------------------------------------------------------------------------
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
constexpr int MB = 2;            // 16-row blocks of dy per work item (against MB + 1 blocks of x)
constexpr int HV = 2;            // 32-key halves per step: a step takes whole 128-byte lines of its rows, the two
                                 // halves of a line in load instructions issued back to back
constexpr int MROWS = 16 * MB;   // rows of dy per work item
constexpr int KSTEP = 32 * HV;   // keys per step

// Eight consecutive keys k0..k0+7 (k0 a multiple of 8, possibly -8) of row h.  The forward pass's masks -- 0 outside the
// plane and, under the causal rule, for keys beyond the row index -- are applied in two parts: piece_ok() picks the
// address (a piece that is masked as a whole loads the start of the plane instead, so that every load is unconditional
// and the compiler can keep a whole step's loads in flight), mask_piece() zeroes what must read as 0 once the data is
// there.  `edge` = the step may straddle the diagonal (wavefront-uniform).
__device__ __forceinline__ bool piece_ok(int h, int k0, int H, int W, int causal)
{
    return (unsigned)h < (unsigned)H && (unsigned)k0 < (unsigned)W && !(causal && k0 > h);
}

__device__ __forceinline__ u4 mask_piece(u4 v, int h, int k0, int H, int W, int causal, bool edge)
{
    const unsigned keep = piece_ok(h, k0, H, W, causal) ? 0xffffffffu : 0u;
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] &= keep;
    if (edge) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = k0 + 2 * u;
            v[u] &= (e <= h ? 0x0000ffffu : 0u) | (e + 1 <= h ? 0xffff0000u : 0u);
        }
    }
    return v;
}

// One step of a wavefront covers 32 keys: lane (r, g) loads the eight keys kb + 8g .. +7 of its rows -- MB 16-row blocks
// of dy and the MB + 1 blocks of x around them -- and nothing else.  The products pair the dy keys of the lane group to
// the LEFT (k-8 .. k-1, k = kb + 8g) with the 24-key window k-16 .. k+7 of x, whose first two thirds are the pieces of
// the two lane groups to the left as well: those come over ds_bpermute (for the first groups of a step, from the step
// before, which stays in registers), not from memory.  With every lane loading its whole window itself (three pieces
// per block of x: 11 loads per step instead of 5) the kernel's time followed the number of load instructions.
struct step_pieces {
    u4 dy[MB][HV];
    u4 x[MB + 1][HV];
};

// The rows a lane reads in a work item, as element offsets into the plane (which the host keeps below 2^31 elements):
// x rows p0 - 16 + 16 nb + r and dy rows p0 + 16 mb + r, both from key 8g on.  The offset of a row outside the plane
// wraps around and is never used.
struct lane_rows {
    unsigned x[MB + 1];
    unsigned dy[MB];
};

template <typename T> __device__ __forceinline__ u4 load16(const T *plane, unsigned off)
{
    return *reinterpret_cast<const u4 *>(plane + (size_t)off);
}

// `inner` (wavefront-uniform): every piece of the step lies inside the plane and on or below the diagonal.  kb may be
// -32 (the step ahead of a row's first, whose pieces all read as 0).
template <typename T>
__device__ __forceinline__ void load_step(step_pieces &o, const T *xp, const T *dyp, const lane_rows &rows, int p0, int kb,
                                          int r, int g, int H, int W, int causal, bool inner)
{
    if (inner) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int hv = 0; hv < HV; ++hv) o.dy[mb][hv] = load16(dyp, rows.dy[mb] + kb + 32 * hv);
#pragma unroll
        for (int nb = 0; nb < MB + 1; ++nb)
#pragma unroll
            for (int hv = 0; hv < HV; ++hv) o.x[nb][hv] = load16(xp, rows.x[nb] + kb + 32 * hv);
    } else {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int hv = 0; hv < HV; ++hv) {
                const int k = kb + 32 * hv + 8 * g;
                o.dy[mb][hv] = load16(dyp, piece_ok(p0 + 16 * mb + r, k, H, W, causal) ? rows.dy[mb] + kb + 32 * hv : 0u);
            }
#pragma unroll
        for (int nb = 0; nb < MB + 1; ++nb)
#pragma unroll
            for (int hv = 0; hv < HV; ++hv) {
                const int k = kb + 32 * hv + 8 * g;
                o.x[nb][hv] = load16(xp, piece_ok(p0 - 16 + 16 * nb + r, k, H, W, causal) ? rows.x[nb] + kb + 32 * hv : 0u);
            }
    }
}

__device__ __forceinline__ void mask_step(step_pieces &o, int p0, int kb, int r, int g, int H, int W, int causal)
{
    // rows of this item start at p0 - 16, the step's last key is kb + KSTEP - 1
    const bool edge = causal && kb + KSTEP - 1 > p0 - 16;
#pragma unroll
    for (int hv = 0; hv < HV; ++hv) {
        const int k = kb + 32 * hv + 8 * g;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) o.dy[mb][hv] = mask_piece(o.dy[mb][hv], p0 + 16 * mb + r, k, H, W, causal, edge);
#pragma unroll
        for (int nb = 0; nb < MB + 1; ++nb)
            o.x[nb][hv] = mask_piece(o.x[nb][hv], p0 - 16 + 16 * nb + r, k, H, W, causal, edge);
    }
}

// the piece that lane (r, g - back) holds in `cur`, or, for the first `back` lane groups, lane (r, g - back + 4) in `prev`
__device__ __forceinline__ u4 piece_from_left(const u4 &prev, const u4 &cur, int lane, int back)
{
    const bool from_prev = lane >= 64 - 16 * back;  // as a source: these lanes are read by the first groups of this step
    const int src = ((lane - 16 * back) & 63) * 4;
    u4 v;
#pragma unroll
    for (int d = 0; d < 4; ++d)
        v[d] = (unsigned)__builtin_amdgcn_ds_bpermute(src, (int)(from_prev ? prev[d] : cur[d]));
    return v;
}

// The 2*MB*S products of a step: block mb of dy against blocks mb and mb+1 of x, every key offset j.  The operand of
// offset j is the 24-key window of x from key 8 + j - pad on (a byte shift of two registers for odd starts).
template <typename T, int S>
__device__ __forceinline__ void accumulate_step(f32x4 (&acc)[2][S], const step_pieces &prev, const step_pieces &cur, int lane)
{
    constexpr int PW = (S - 1) / 2;
#pragma unroll
    for (int hv = 0; hv < HV; ++hv) {
        // what lies to the left of this half's first lane groups: the last half of the step before, or this step's
        // half before this one
        frag8<T> a[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const u4 &before = hv == 0 ? prev.dy[mb][HV - 1] : cur.dy[mb][hv > 0 ? hv - 1 : 0];
            a[mb] = __builtin_bit_cast(frag8<T>, piece_from_left(before, cur.dy[mb][hv], lane, 1));
        }
#pragma unroll
        for (int nb = 0; nb < MB + 1; ++nb) {
            const u4 &before = hv == 0 ? prev.x[nb][HV - 1] : cur.x[nb][hv > 0 ? hv - 1 : 0];
            const u4 ll = piece_from_left(before, cur.x[nb][hv], lane, 2), l = piece_from_left(before, cur.x[nb][hv], lane, 1);
            unsigned w[12];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                w[u] = ll[u];
                w[4 + u] = l[u];
                w[8 + u] = cur.x[nb][hv][u];
            }
#pragma unroll
            for (int j = 0; j < S; ++j) {
                const int st = 8 + j - PW;  // compile-time after unrolling
                u4 bv;
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    bv[d] = (st & 1) ? __builtin_amdgcn_alignbyte(w[(st + 1) / 2 + d], w[(st - 1) / 2 + d], 2) : w[st / 2 + d];
                const frag8<T> b = __builtin_bit_cast(frag8<T>, bv);
                if (nb <= MB - 1) mma16(acc[0][j], a[nb < MB ? nb : 0], b);
                if (nb >= 1) mma16(acc[1][j], a[nb - 1 >= 0 ? nb - 1 : 0], b);
            }
        }
    }
}

template <typename T, int R, int S>
__global__ __launch_bounds__(NT) void conv2d_bwd_weight_mfma(const T *__restrict__ x, const T *__restrict__ dy,
                                                             float *__restrict__ partial, int N, int C, int H, int W,
                                                             int causal, int tiles_m, int nseg, int bpc)
{
    static_assert(R <= 17 && S <= 16 && (S - 1) / 2 <= 8, "window of 24 keys, two 16-row blocks of halo");
    __shared__ float tile[2 * S][16][17];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int c = blockIdx.x / bpc, sub = blockIdx.x % bpc;

    // acc[half][j]: D[m][n] = sum over keys of dy[p0m + m, q] * x[p0m - 16 + 16*half + n, q + j - PW]
    f32x4 acc[2][S];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < S; ++j) acc[h][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // Items in order of falling length (under the causal rule a row block further down has more keys), dealt to the
    // channel's wavefronts forwards and backwards in turn, so that every wavefront gets about the same number of steps.
    const int items = N * tiles_m * nseg;  // the host keeps this below 2^31
    const int nwv = bpc * (NT / 64), wv = sub * (NT / 64) + wave, per_tm = N * nseg;
    for (int k = 0; k * nwv < items; ++k) {
        const int it = k * nwv + ((k & 1) ? nwv - 1 - wv : wv);
        if (it >= items) continue;
        const int tm = tiles_m - 1 - it / per_tm, rem = it % per_tm;
        const int n = rem / nseg, sg = rem % nseg;
        const int p0 = tm * MROWS;
        int kend = W;  // dy is zero beyond the diagonal: keys from p0 + MROWS on add nothing
        if (causal && p0 + MROWS < W) kend = p0 + MROWS;
        // a step pairs the dy keys kb-8 .. kb+KSTEP-9 with their windows of x: the row's keys end at kend-1
        const int nsteps = (kend + 8 + KSTEP - 1) / KSTEP, per = (nsteps + nseg - 1) / nseg;
        const int t0 = sg * per, t1 = (t0 + per < nsteps) ? t0 + per : nsteps;
        if (t0 >= t1) continue;
        const int64_t plane = ((int64_t)n * C + c) * H * W;
        const T *xp = x + plane, *dyp = dy + plane;
        lane_rows rows;
#pragma unroll
        for (int nb = 0; nb < MB + 1; ++nb) rows.x[nb] = (unsigned)((p0 - 16 + 16 * nb + r) * W + 8 * g);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) rows.dy[mb] = (unsigned)((p0 + 16 * mb + r) * W + 8 * g);
        // steps whose pieces all lie inside the plane and on or below the diagonal need neither selects nor masks: rows
        // p0-16 .. p0+MROWS-1 inside the plane, keys kb .. kb+KSTEP-1 inside it and (causal) not beyond row p0-16
        const bool rows_in = p0 >= 16 && p0 + MROWS <= H;
        const int in_plane = W - KSTEP, below = p0 - 16 - (KSTEP - 1);
        const int last_inner = causal ? (below < in_plane ? below : in_plane) : in_plane;  // largest such kb
        auto inner = [&](int t) { return rows_in && t >= 0 && KSTEP * t <= last_inner; };
        // Three sets of pieces take turns as (step before, this step, next step): the next step's loads stay in flight
        // through this step's products, and the step before supplies the left neighbours of this step's first lane
        // groups.  The last step fetches itself again, so that the loads in flight never depend on a branch; the step
        // ahead of the segment's first is fetched for its pieces only.
        step_pieces sa, sb, sc;
        load_step(sa, xp, dyp, rows, p0, KSTEP * (t0 - 1), r, g, H, W, causal, inner(t0 - 1));
        load_step(sb, xp, dyp, rows, p0, KSTEP * t0, r, g, H, W, causal, inner(t0));
        if (!inner(t0 - 1)) mask_step(sa, p0, KSTEP * (t0 - 1), r, g, H, W, causal);
        int t = t0;
#define MTA_CBW_STEP(PV, CU, NX)                                                                        \
        {                                                                                               \
            const int tn = t + 1 < t1 ? t + 1 : t;                                                      \
            load_step(NX, xp, dyp, rows, p0, KSTEP * tn, r, g, H, W, causal, inner(tn));                \
            if (!inner(t)) mask_step(CU, p0, KSTEP * t, r, g, H, W, causal);                            \
            accumulate_step<T, S>(acc, PV, CU, lane);                                                   \
        }
        for (;;) {
            MTA_CBW_STEP(sa, sb, sc)
            if (++t >= t1) break;
            MTA_CBW_STEP(sb, sc, sa)
            if (++t >= t1) break;
            MTA_CBW_STEP(sc, sa, sb)
            if (++t >= t1) break;
        }
#undef MTA_CBW_STEP
    }

    // tap (i,j) = sum over m of D_j[m][m + i - (R-1)] taken from the half that holds that column; the four wavefronts
    // pass through the LDS tile one after the other and every tap is added up in a fixed order
    float s = 0.0f;
    const int ti = tid / S, tj = tid % S;
    for (int wv = 0; wv < NT / 64; ++wv) {
        __syncthreads();
        if (wave == wv) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < S; ++j)
#pragma unroll
                    for (int v = 0; v < 4; ++v) tile[h * S + j][4 * g + v][r] = acc[h][j][v];
        }
        __syncthreads();
        if (tid < R * S) {
            for (int m = 0; m < 16; ++m) {
                const int n1 = m + ti - (R - 1);
                s += n1 >= 0 ? tile[S + tj][m][n1] : tile[tj][m][n1 + 16];
            }
        }
    }
    if (tid < R * S) partial[((int64_t)c * bpc + sub) * (R * S) + tid] = s;
}

// Any kernel size: x halo tile and dy tile in LDS, the R*S running sums in LDS too; thread t owns taps t, t+256, ...
// (nothing is unrolled over the taps: the fixed-size kernel above is the fast path).
template <typename T>
__global__ __launch_bounds__(NT) void conv2d_bwd_weight_any(const T *__restrict__ x, const T *__restrict__ dy,
                                                            float *__restrict__ partial, int N, int C, int H, int W,
                                                            int R, int S, int causal, int tiles_m, int tiles_n, int bpc)
{
    extern __shared__ float smem[];
    const int LD = TN + S;
    const int RS = R * S;
    float *tile = smem;                            // (TM+R-1) x LD
    float *gt = tile + (TM + R - 1) * LD;          // TM x TN gradient tile
    float *sums = gt + TM * TN;                    // R*S
    const int tid = threadIdx.x;
    const split_t sp = split_of(blockIdx.x, C, bpc);
    const int c = sp.channel;
    for (int tap = tid; tap < RS; tap += NT) sums[tap] = 0.0f;

    const int tiles = tiles_m * tiles_n;
    const int64_t items = (int64_t)N * tiles;
    for (int64_t it = sp.sub; it < items; it += sp.bpc) {
        const int n = (int)(it / tiles), t = (int)(it % tiles);
        const int tm = t / tiles_n, tn = t % tiles_n;
        const int p0 = tm * TM, q0 = tn * TN;
        if (causal && q0 > p0 + TM - 1) continue;
        const int64_t plane = ((int64_t)n * C + c) * H * W;
        __syncthreads();
        stage_x<T>(x + plane, tile, LD, H, W, p0, q0, R, S, causal, tid);
        for (int e = tid; e < TM * TN; e += NT) {
            const int p = p0 + e / TN, q = q0 + e % TN;
            const bool ok = p < H && q < W && !(causal && q > p);
            gt[e] = ok ? to_float(dy[plane + (int64_t)p * W + q]) : 0.0f;
        }
        __syncthreads();
#pragma unroll 1
        for (int tap = tid; tap < RS; tap += NT) {
            const int i = tap / S, j = tap % S;
            float s = 0.0f;
#pragma unroll 1
            for (int r = 0; r < TM; ++r) {
                const float *xr = tile + (r + i) * LD + j;
                const float *gr = gt + r * TN;
#pragma unroll 8
                for (int col = 0; col < TN; ++col) s = fmaf(gr[col], xr[col], s);
            }
            sums[tap] += s;  // only the owner thread touches this entry
        }
    }
    for (int tap = tid; tap < RS; tap += NT) partial[((int64_t)c * bpc + sp.sub) * RS + tap] = sums[tap];
}

// dw[c][t] = sum over the channel's partial kernels, in a fixed order
__global__ __launch_bounds__(NT) void reduce_partials(const float *__restrict__ partial, float *__restrict__ dw, int total,
                                                      int RS, int bpc)
{
    const int e = blockIdx.x * NT + threadIdx.x;  // (c, tap)
    if (e >= total) return;
    const int c = e / RS, t = e % RS;
    float s = 0.0f;
    for (int b = 0; b < bpc; ++b) s += partial[((int64_t)c * bpc + b) * RS + t];
    dw[e] = s;
}

// workgroups per channel: enough persistent workgroups to fill the device, at most `cap` partial kernels in total
inline int blocks_per_channel(int64_t N, int64_t C, int64_t H, int64_t W, int64_t cap)
{
    const int64_t tiles = ((H + TM - 1) / TM) * ((W + TN - 1) / TN);
    int64_t bpc = (1024 + C - 1) / C;            // about four workgroups per CU in total
    if (bpc > N * tiles) bpc = N * tiles;
    if (bpc * C > cap) bpc = cap / C;
    return (int)(bpc < 1 ? 1 : bpc);
}

constexpr int64_t MAX_PARTIALS = 2048;  // partial kernels per launch, over all channels

int check_args(const void *x, const void *dy, const void *dw, int64_t N, int64_t C, int64_t H, int64_t W, int R, int S,
               int io_dtype)
{
    if (!x || !dy || !dw) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || H > (1 << 24) || W > (1 << 24) || N * C > 65535) return MTA_ERR_SHAPE;
    if (C > MAX_PARTIALS) return MTA_ERR_SHAPE;
    if (R < 1 || S < 1 || R > MTA_MAX_KERNEL_R || S > MTA_MAX_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
    if (!aligned_to(x, dtype_size(io_dtype)) || !aligned_to(dy, dtype_size(io_dtype)) || !aligned_to(dw, 4))
        return MTA_ERR_ALIGN;
    if (((H + TM - 1) / TM) * ((W + TN - 1) / TN) > 0x7fffffffLL) return MTA_ERR_SHAPE;
    return MTA_OK;
}

template <typename T>
int launch(const void *x, const void *dy, float *dw, float *partial, int bpc, int64_t N, int64_t C, int64_t H, int64_t W,
           int R, int S, int causal, hipStream_t st)
{
    const int tiles_m = (int)((H + TM - 1) / TM), tiles_n = (int)((W + TN - 1) / TN);
    const int vec_ok = (W % 8 == 0 && aligned_to(dy, 16)) ? 1 : 0;
    dim3 grid((unsigned)(C * bpc));
    if constexpr (sizeof(T) == 2) {
        // 16-bit tensors with rows of whole 16-byte vectors: matrix cores (MTA_CONV_FORCE_VALU=1 in the environment keeps
        // the fp32-FMA kernel, for comparisons).  Two workgroups per CU; the key range of a row block is cut into
        // segments until every wavefront has about two items.
        static const bool force_valu = [] { const char *e = getenv("MTA_CONV_FORCE_VALU"); return e && e[0] == '1'; }();
        if (!force_valu && vec_ok && aligned_to(x, 16) && R <= 17 && (H + MROWS + 16) * W < 0x7fffffffLL) {
            const int rows_m = (int)((H + MROWS - 1) / MROWS);
            int bm = (int)((512 + C - 1) / C);
            if (bm > bpc) bm = bpc;
            int64_t nseg = ((int64_t)8 * bm + N * rows_m - 1) / (N * rows_m);
            const int64_t seg_cap = W / 256 > 1 ? W / 256 : 1;
            if (nseg > seg_cap) nseg = seg_cap;
            if (nseg > 8) nseg = 8;
            if (bm > N * rows_m * nseg) bm = (int)(N * rows_m * nseg);
            if (N * rows_m * nseg > 0x3fffffffLL) return MTA_ERR_SHAPE;  // the kernel counts items in 32 bits
#define MTA_CONV_CASE(r, s)                                                                                          \
    if (R == r && S == s) {                                                                                          \
        hipLaunchKernelGGL((conv2d_bwd_weight_mfma<T, r, s>), dim3((unsigned)(C * bm)), dim3(NT), 0, st,              \
                           (const T *)x, (const T *)dy, partial, (int)N, (int)C, (int)H, (int)W, causal, rows_m,      \
                           (int)nseg, bm);                                                                           \
        bpc = bm;                                                                                                    \
        goto reduce;                                                                                                 \
    }
            MTA_CONV_CASE(3, 3)
            MTA_CONV_CASE(3, 5)
            MTA_CONV_CASE(5, 5)
            MTA_CONV_CASE(5, 7)
            MTA_CONV_CASE(6, 11)
            MTA_CONV_CASE(7, 7)
            MTA_CONV_CASE(7, 9)
            MTA_CONV_CASE(11, 15)
#undef MTA_CONV_CASE
        }
    }
#define MTA_CONV_CASE(r, s)                                                                                          \
    if (R == r && S == s) {                                                                                          \
        hipLaunchKernelGGL((conv2d_bwd_weight_fixed<T, r, s>), grid, dim3(NT), 0, st, (const T *)x, (const T *)dy,    \
                           partial, (int)N, (int)C, (int)H, (int)W, causal, tiles_m, tiles_n, bpc, vec_ok);           \
        goto reduce;                                                                                                 \
    }
    MTA_CONV_CASE(3, 3)
    MTA_CONV_CASE(3, 5)
    MTA_CONV_CASE(5, 5)
    MTA_CONV_CASE(5, 7)
    MTA_CONV_CASE(6, 11)
    MTA_CONV_CASE(7, 7)
    MTA_CONV_CASE(7, 9)
#undef MTA_CONV_CASE
    {
        const size_t lds = sizeof(float) * ((size_t)(TM + R - 1) * (TN + S) + (size_t)TM * TN + (size_t)R * S);
        auto kern = conv2d_bwd_weight_any<T>;
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
        }
        hipLaunchKernelGGL(kern, grid, dim3(NT), lds, st, (const T *)x, (const T *)dy, partial, (int)N, (int)C, (int)H,
                           (int)W, R, S, causal, tiles_m, tiles_n, bpc);
    }
reduce:
    {
        const int rc = launch_status();
        if (rc != MTA_OK) return rc;
        const int total = (int)(C * R * S);
        hipLaunchKernelGGL(reduce_partials, dim3((unsigned)((total + NT - 1) / NT)), dim3(NT), 0, st, partial, dw, total,
                           R * S, bpc);
        return launch_status();
    }
}

// ---- scratch buffer of the entry point that allocates nothing -----------------------------------------------------
// One array per device, alive until the process ends.  In host code the array's name is only a handle: the address the
// kernels get is the one hipGetSymbolAddress returns for the current device, looked up once per device and kept.  Every
// call on a device shares that device's array: calls that overlap on one device (two streams, two threads) race.  The
// kernels write every partial sum they later read, so nothing has to be cleared between calls.
constexpr int64_t STATIC_FLOATS = 256 * 1024;  // 1 MiB: e.g. 2048 partial kernels of up to 128 taps
static __device__ __align__(256) float scratch[STATIC_FLOATS];

float *static_scratch(int *err)
{
    // (atomic slots: two host threads making their first call on a device may both look the address up and both store
    // it - the same value - without a data race)
    static std::atomic<float *> ptr[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { *err = (int)e; return nullptr; }
    if (dev < 0 || dev >= 64) { *err = MTA_ERR_DEVICE; return nullptr; }
    float *p = ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) { *err = (int)e; return nullptr; }
        ptr[dev].store(p, std::memory_order_release);
    }
    *err = MTA_OK;
    return p;
}
}  // namespace

extern "C" int64_t mta_conv2d_bwd_weight_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int R, int S)
{
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || R < 1 || S < 1 || C > MAX_PARTIALS) return 0;
    return (int64_t)blocks_per_channel(N, C, H, W, MAX_PARTIALS) * C * R * S * (int64_t)sizeof(float);
}

extern "C" int mta_conv2d_bwd_weight(const void *x, const void *dy, void *dw, void *workspace, int64_t workspace_bytes,
                                     int64_t N, int64_t C, int64_t H, int64_t W, int R, int S, int causal, int io_dtype,
                                     void *stream)
{
    const int rc = check_args(x, dy, dw, N, C, H, W, R, S, io_dtype);
    if (rc != MTA_OK) return rc;
    if (!workspace) return MTA_ERR_NULL;
    if (!aligned_to(workspace, 16)) return MTA_ERR_ALIGN;
    const int bpc = blocks_per_channel(N, C, H, W, MAX_PARTIALS);
    if (workspace_bytes < (int64_t)bpc * C * R * S * (int64_t)sizeof(float)) return MTA_ERR_WORKSPACE;
    MTA_DISPATCH_IO(io_dtype, return launch<io_t>(x, dy, (float *)dw, (float *)workspace, bpc, N, C, H, W, R, S, causal,
                                                  (hipStream_t)stream));
    return MTA_ERR_DTYPE;
}


extern "C" int mta_conv2d_bwd_weight_noalloc(const void *x, const void *dy, void *dw, int64_t N, int64_t C, int64_t H,
                                             int64_t W, int R, int S, int causal, int io_dtype, void *stream)
{
    int rc = check_args(x, dy, dw, N, C, H, W, R, S, io_dtype);
    if (rc != MTA_OK) return rc;
    // as many partial kernels as the fixed array holds
    const int64_t cap = STATIC_FLOATS / ((int64_t)R * S);
    if (cap < C) return MTA_ERR_WORKSPACE;  // C*R*S floats do not fit: one partial kernel per channel is the minimum
    const int bpc = blocks_per_channel(N, C, H, W, cap < MAX_PARTIALS ? cap : MAX_PARTIALS);
    float *ws = static_scratch(&rc);
    if (!ws) return rc;
    MTA_DISPATCH_IO(io_dtype, return launch<io_t>(x, dy, (float *)dw, ws, bpc, N, C, H, W, R, S, causal,
                                                  (hipStream_t)stream));
    return MTA_ERR_DTYPE;
}
