// Depthwise causal 2-D convolution over the (N,C,H,W) score tensor.
//
//   y[n,c,p,q] = sum_{i<R,j<S} w[c,i,j] * xm[n,c,p+i-(R-1), q+j-(S-1)/2]
//
// One workgroup owns a TM x TN output tile of one (n,c) plane.  It stages the
// (TM+R-1) x (TN+S-1) query x key halo tile in LDS once (bounds and the causal
// col<=row rule are applied while staging, so the tap loop is mask-free), skips
// tiles that lie entirely above the diagonal (they only receive their +0 fill), and
// applies the causal output rule on store.
//
// Two compute paths:
//   conv2d_valu  fp32 FMAs from an fp32 LDS tile; any I/O and weight dtype; each lane
//                slides a register window along the key axis (8 outputs per lane).
//   conv2d_mfma  16-bit I/O with weights of the same dtype.  The 6x11 conv costs 66 FMAs
//                per output, which on the vector ALU takes longer than moving the tensor
//                through HBM.  Each kernel row is therefore applied as a banded (Toeplitz)
//                matrix product on the matrix cores:
//                    out^T[q, p] += T_i^T[q, k] * X^T[k, p+i-(R-1)]      i = 0..R-1
//                with T_i[k, q] = w[i, k-q-shift] held in registers for the whole kernel
//                and X^T fragments read straight from the row-major LDS tile (a lane reads
//                16 contiguous bytes of one query row).  ~4x the multiply-adds, on a unit
//                with ~16x the rate: the kernel becomes HBM-bound.  Products of 16-bit
//                values are exact in fp32 and accumulation is fp32, as in the VALU path.
#include "common.hpp"
#include "mfma.hpp"

#include <stdlib.h>

namespace {
using namespace mta;

constexpr int NT = 256;

// ------------------------------------------------------------------------------------
// VALU path
// ------------------------------------------------------------------------------------
constexpr int V_TM = 32;  // tile rows   (thread t: row t/8)
constexpr int V_TN = 64;  // tile cols   (thread t: cols 8*(t%8) .. +7)

template <typename T>
__device__ __forceinline__ void store_row8(T *yp, int64_t W, int H, int p, int q, const float *acc,
                                           bool causal)
{
    if (p >= H) return;
    T *dst = yp + (int64_t)p * W + q;
    if (q + 8 <= W && (reinterpret_cast<uintptr_t>(dst) % (8 * sizeof(T))) == 0) {
        struct alignas(8 * sizeof(T)) chunk { T v[8]; } c;
#pragma unroll
        for (int u = 0; u < 8; ++u) c.v[u] = from_float<T>((causal && q + u > p) ? 0.0f : acc[u]);
        *reinterpret_cast<chunk *>(dst) = c;
    } else {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (q + u < W) dst[u] = from_float<T>((causal && q + u > p) ? 0.0f : acc[u]);
    }
}

template <typename T, int R_T, int S_T>
__global__ __launch_bounds__(NT) void conv2d_valu(const T *__restrict__ x, const void *__restrict__ w,
                                                  T *__restrict__ y, int C, int H, int W, int R_rt,
                                                  int S_rt, int causal, float in_scale, int use_scale,
                                                  int w_dtype, int tiles_n)
{
    const int R = R_T > 0 ? R_T : R_rt;
    const int S = S_T > 0 ? S_T : S_rt;
    const int pad_h = R - 1, pad_w = (S - 1) / 2;
    const int LD = V_TN + S;  // S-1 halo columns + 1 pad
    extern __shared__ float smem[];
    float *wsm = smem;                        // R*S weights of this channel
    float *tile = smem + ((R * S + 3) & ~3);  // (V_TM+R-1) x LD

    const int tid = threadIdx.x;
    const int64_t plane = blockIdx.y;
    const int c = (int)(plane % C);
    const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const int p0 = tm * V_TM, q0 = tn * V_TN;
    const T *xp = x + plane * (int64_t)H * W;
    T *yp = y + plane * (int64_t)H * W;
    const int tr = tid >> 3, tc = (tid & 7) * 8;

    float acc[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc[u] = 0.0f;

    if (causal && q0 > p0 + V_TM - 1) {  // wholly above the diagonal: fill only
        store_row8<T>(yp, W, H, p0 + tr, q0 + tc, acc, true);
        return;
    }

    for (int t = tid; t < R * S; t += NT) wsm[t] = load_any(w, w_dtype, (int64_t)c * R * S + t);

    const int rows = V_TM + R - 1, cols = V_TN + S - 1;
    for (int rr = tid / 64; rr < rows; rr += NT / 64) {
        const int h = p0 - pad_h + rr;
        const bool row_ok = h >= 0 && h < H;
        for (int cc = tid % 64; cc < cols; cc += 64) {
            const int k = q0 - pad_w + cc;
            float v = 0.0f;
            if (row_ok && k >= 0 && k < W && (!causal || k <= h)) {
                v = to_float(xp[(int64_t)h * W + k]);
                if (use_scale) v = round_to<T>(v * in_scale);
            }
            tile[rr * LD + cc] = v;
        }
    }
    __syncthreads();

    if constexpr (R_T > 0 && S_T > 0) {
#pragma unroll
        for (int i = 0; i < R_T; ++i) {
            float win[S_T + 7];
            const float *src = tile + (tr + i) * LD + tc;
#pragma unroll
            for (int u = 0; u < S_T + 7; ++u) win[u] = src[u];
#pragma unroll
            for (int j = 0; j < S_T; ++j) {
                const float wv = wsm[i * S_T + j];
#pragma unroll
                for (int u = 0; u < 8; ++u) acc[u] = fmaf(wv, win[u + j], acc[u]);
            }
        }
    } else {
        for (int i = 0; i < R; ++i) {
            const float *src = tile + (tr + i) * LD + tc;
            for (int j = 0; j < S; ++j) {
                const float wv = wsm[i * S + j];
#pragma unroll
                for (int u = 0; u < 8; ++u) acc[u] = fmaf(wv, src[u + j], acc[u]);
            }
        }
    }
    store_row8<T>(yp, W, H, p0 + tr, q0 + tc, acc, causal != 0);
}

template <typename T, int R_T, int S_T>
int launch_valu(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                int S, int causal, float in_scale, int use_scale, int w_dtype, hipStream_t st)
{
    const int tiles_m = (int)((H + V_TM - 1) / V_TM), tiles_n = (int)((W + V_TN - 1) / V_TN);
    const size_t lds = sizeof(float) * (((R * S + 3) & ~3) + (size_t)(V_TM + R - 1) * (V_TN + S));
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)(N * C));
    hipLaunchKernelGGL((conv2d_valu<T, R_T, S_T>), grid, dim3(NT), lds, st, (const T *)x, w, (T *)y, (int)C,
                       (int)H, (int)W, R, S, causal, in_scale, use_scale, w_dtype, tiles_n);
    return launch_status();
}

template <typename T>
int dispatch_valu(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                  int S, int causal, float in_scale, int use_scale, int w_dtype, hipStream_t st)
{
#define MTA_CONV_CASE(r, s)                                                                               \
    if (R == r && S == s)                                                                                 \
        return launch_valu<T, r, s>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st);
    MTA_CONV_CASE(3, 3)
    MTA_CONV_CASE(3, 5)
    MTA_CONV_CASE(5, 5)
    MTA_CONV_CASE(5, 7)
    MTA_CONV_CASE(6, 11)
    MTA_CONV_CASE(7, 7)
    MTA_CONV_CASE(7, 9)
    MTA_CONV_CASE(11, 15)
#undef MTA_CONV_CASE
    return launch_valu<T, 0, 0>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st);
}

// ------------------------------------------------------------------------------------
// MFMA (Toeplitz) path
// ------------------------------------------------------------------------------------
#ifndef MTA_CONV_WAVES_PER_SIMD
#define MTA_CONV_WAVES_PER_SIMD 2
#endif
constexpr int M_WT = 64;   // one wavefront per workgroup
constexpr int M_TM = 32;   // strip rows   (one accumulator column per lane%32)
constexpr int M_TN = 128;  // strip cols   (4 sub-tiles of 32 keys)

template <int R, int S> struct mfma_geom {
    static constexpr int PADW = (S - 1) / 2;
    static constexpr int HL = (PADW + 7) & ~7;                 // left halo, rounded so 16-byte loads stay aligned
    static constexpr int SHIFT = HL - PADW;                    // first tap's offset inside a sub-tile's window
    static constexpr int NCH = (SHIFT + 32 + S - 1 + 15) / 16; // 16-key chunks per 32-output window
    static constexpr int TW = M_TN - 32 + 16 * NCH;            // staged columns
    static constexpr int LD = TW + ((24 - TW % 16) % 16);      // row stride = 8 (mod 16) elements: conflict-free b128 reads
    static constexpr int ROWS = M_TM + R - 1;
};

// logical output column (0..31) held by accumulator row m.  Accumulator register v of lane-half
// h is row m = 8*(v/4) + 4*h + v%4; this choice makes it column 16*(v/8) + 8*h + v%8, so one
// 16-byte store per lane covers 8 consecutive keys and the two halves of a row sit side by side.
__device__ __forceinline__ int toeplitz_q_of_m(int m)
{
    return 16 * (m >> 4) + 8 * ((m >> 2) & 1) + 4 * ((m >> 3) & 1) + (m & 3);
}

// work item -> (plane, strip row tm (32 rows), strip col tn (128 keys)).
// `mirror` (causal, square): only strips that touch the lower triangle are enumerated, by 128x128
// block in row-major lower-triangular order, 4 strips per block; each strip of an off-diagonal
// block also zero-fills a quarter of the block's mirror image above the diagonal.
__device__ __forceinline__ void decode_item(int64_t idx, int ipp, int tiles_n, int mirror, int64_t &plane, int &tm, int &tn)
{
    plane = idx / ipp;
    const int t = (int)(idx % ipp);
    if (mirror) {
        const int blk = t >> 2;
        int bm = (int)((sqrtf(8.0f * (float)blk + 1.0f) - 1.0f) * 0.5f);
        while ((bm + 1) * (bm + 2) / 2 <= blk) ++bm;
        while (bm * (bm + 1) / 2 > blk) --bm;
        tn = blk - bm * (bm + 1) / 2;
        tm = bm * 4 + (t & 3);
    } else {
        tm = t / tiles_n;
        tn = t % tiles_n;
    }
}

template <typename T>
__device__ __forceinline__ void zero_fill_strip(T *yp, int H, int W, int p0, int q0, int lane)
{
    constexpr int VEC = 8;
    pack16<T> z;
#pragma unroll
    for (int u = 0; u < VEC; ++u) z.v[u] = from_float<T>(0.0f);
#pragma unroll
    for (int e = lane; e < M_TM * (M_TN / VEC); e += M_WT) {
        const int r = e / (M_TN / VEC), col = q0 + (e % (M_TN / VEC)) * VEC;
        if (p0 + r < H && col < W) *reinterpret_cast<pack16<T> *>(yp + (int64_t)(p0 + r) * W + col) = z;
    }
}

// Persistent single-wavefront workgroups: each walks a contiguous run of 32x128 strips (so the
// Toeplitz fragments are rebuilt only when the channel changes).  No workgroup barrier is ever
// needed; latency is hidden by the other wavefronts resident on the CU, each in its own phase
// (loading / matrix cores / storing) with its own 11 KB LDS strip.
template <typename T, int R, int S, bool SCALED>
__global__ __launch_bounds__(M_WT, MTA_CONV_WAVES_PER_SIMD) void conv2d_mfma(
    const T *__restrict__ x, const T *__restrict__ w, T *__restrict__ y, int C, int H, int W, int causal, float in_scale,
    int tiles_n, int ipp, int64_t total, int64_t per_xcd, int nw, int mirror)
{
    using G = mfma_geom<R, S>;
    constexpr int LD = G::LD, NCH = G::NCH, VEC = 8;
    constexpr int VPR = G::TW / VEC;                            // 16-byte vectors per staged row
    constexpr int STAGE_IT = (G::ROWS * VPR + M_WT - 1) / M_WT; // vectors per lane
    // weights of the current channel, each kernel row zero-padded on both sides so that the
    // Toeplitz fragments can be gathered without range checks
    constexpr int WZ_OFF = G::SHIFT + 32, WZ_LD = WZ_OFF + 16 * NCH + 2;
    __shared__ __align__(16) T tile[G::ROWS * LD];
    __shared__ T wz[R * WZ_LD];
    using V16 = pack16<T>;

    // XCD-aware split: workgroup ids are dealt round-robin to the 8 XCDs; each XCD gets one
    // contiguous chunk of the item list (whole planes, mostly), so halo re-reads stay in its L2.
    const int64_t c0 = (int64_t)(blockIdx.x & 7) * per_xcd;
    const int64_t c1 = (c0 + per_xcd < total) ? c0 + per_xcd : total;
    const int64_t per_wg = (c1 - c0 + nw - 1) / nw;
    const int64_t first = c0 + (int64_t)(blockIdx.x >> 3) * per_wg;
    const int64_t last = (first + per_wg < c1) ? first + per_wg : c1;
    if (c0 >= total || first >= last) return;

    const int lane = threadIdx.x, ln = lane & 31, hf = lane >> 5;
    frag8<T> tz[R][NCH];
    int cur_channel = -1;

    // per-lane staging geometry, fixed for the whole kernel: slot `it` of this lane is row rr, vector vc
    // of the halo strip; goff/loff are its element offsets from the strip origin in global memory / LDS
    int goff[STAGE_IT], loff[STAGE_IT];
#pragma unroll
    for (int it = 0; it < STAGE_IT; ++it) {
        const int e = it * M_WT + lane;
        const bool in = e < G::ROWS * VPR;
        const int rr = in ? e / VPR : 0, vc = in ? e % VPR : 0;
        goff[it] = rr * W + vc * VEC;
        loff[it] = in ? rr * LD + vc * VEC : -1;
    }
    const int soff = ln * W + hf * 8;  // this lane's output offset from the strip's first output

    for (int64_t idx = first; idx < last; ++idx) {
        int64_t plane;
        int tm, tn;
        decode_item(idx, ipp, tiles_n, mirror, plane, tm, tn);
        const int p0 = tm * M_TM, q0 = tn * M_TN;
        const T *xp = x + plane * (int64_t)H * W;
        T *yp = y + plane * (int64_t)H * W;
        if (causal && q0 > p0 + M_TM - 1) {  // wholly above the diagonal (only reachable when !mirror)
            zero_fill_strip<T>(yp, H, W, p0, q0, lane);
            continue;
        }
        const int channel = (int)(plane % C);
        if (channel != cur_channel) {
            for (int e = lane; e < R * WZ_LD; e += M_WT) {
                const int i = e / WZ_LD, j = e % WZ_LD - WZ_OFF;
                const bool ok = j >= 0 && j < S;
                const T wv = w[channel * R * S + (ok ? i * S + j : 0)];
                wz[e] = ok ? wv : from_float<T>(0.0f);
            }
        }
        // interior strip: the whole halo strip is inside the tensor and on or below the diagonal,
        // so staging and stores need no masks at all (the common case; decided per wavefront)
        const int h0 = p0 - (R - 1), k0 = q0 - G::HL;
        const bool interior = h0 >= 0 && p0 + M_TM <= H && k0 >= 0 && k0 + G::TW <= W &&
                              (!causal || k0 + G::TW - 1 <= h0);

        // ---- stage rows h0.., cols k0.. into LDS.  Loads are unconditional and issued back to back
        // (an invalid slot re-reads a valid address); masks are applied on the way to LDS.
        {
            V16 stage[STAGE_IT];
            if (interior) {
                const T *base = xp + (int64_t)h0 * W + k0;
#pragma unroll
                for (int it = 0; it < STAGE_IT; ++it) stage[it] = *reinterpret_cast<const V16 *>(base + goff[it]);
#pragma unroll
                for (int it = 0; it < STAGE_IT; ++it) {
                    V16 v = stage[it];
                    if (SCALED) {
#pragma unroll
                        for (int u = 0; u < VEC; ++u) v.v[u] = from_float<T>(to_float(v.v[u]) * in_scale);
                    }
                    if (it < STAGE_IT - 1 || loff[it] >= 0) *reinterpret_cast<V16 *>(tile + loff[it]) = v;
                }
            } else {
#pragma unroll
                for (int it = 0; it < STAGE_IT; ++it) {
                    const int e = it * M_WT + lane;
                    const int rr = e / VPR, vc = e % VPR;
                    const int h = h0 + rr, col = k0 + vc * VEC;
                    const bool ok = e < G::ROWS * VPR && h >= 0 && h < H && col >= 0 && col < W && !(causal && col > h);
                    const int64_t off = ok ? (int64_t)h * W + col : 0;
                    stage[it] = *reinterpret_cast<const V16 *>(xp + off);
                }
#pragma unroll
                for (int it = 0; it < STAGE_IT; ++it) {
                    const int e = it * M_WT + lane;
                    const int rr = e / VPR, vc = e % VPR;
                    const int h = h0 + rr, col = k0 + vc * VEC;
                    const bool ok = h >= 0 && h < H && col >= 0 && col < W && !(causal && col > h);
                    V16 v = stage[it];
                    if (SCALED) {
#pragma unroll
                        for (int u = 0; u < VEC; ++u) v.v[u] = from_float<T>(to_float(v.v[u]) * in_scale);
                    }
                    if (!ok) {
#pragma unroll
                        for (int u = 0; u < VEC; ++u) v.v[u] = from_float<T>(0.0f);
                    } else if (causal && col + VEC - 1 > h) {  // the one vector of a row that straddles the diagonal
#pragma unroll
                        for (int u = 0; u < VEC; ++u)
                            if (col + u > h) v.v[u] = from_float<T>(0.0f);
                    }
                    if (e < G::ROWS * VPR) *reinterpret_cast<V16 *>(tile + rr * LD + vc * VEC) = v;
                }
            }
        }
        __syncthreads();  // one wavefront: orders the LDS writes above before the reads below

        if (channel != cur_channel) {  // Toeplitz fragments T_i^T of this lane's accumulator row
            cur_channel = channel;
            const int qm = toeplitz_q_of_m(ln);
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int ch = 0; ch < NCH; ++ch) {
                    const T *src = wz + i * WZ_LD + WZ_OFF + ch * 16 + hf * 8 - G::SHIFT - qm;  // tap j = k-SHIFT-q
#pragma unroll
                    for (int t = 0; t < 8; ++t) tz[i][ch].v[t] = src[t];
                    __builtin_amdgcn_sched_barrier(0);  // keep the gathers of one fragment together (register pressure)
                }
        }

        // ---- out^T: 32 rows x 4 sub-tiles of 32 keys, one sub-tile at a time (16 accumulators live) ----
        const int prow = p0 + ln;  // this lane's query row
        T *ybase = yp + (int64_t)p0 * W + q0;
#pragma unroll
        for (int st = 0; st < M_TN / 32; ++st) {
            f32x16 acc;
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
            if (!(causal && q0 + st * 32 > p0 + M_TM - 1)) {  // else: sub-tile wholly above the diagonal, stays +0
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const T *rowp = tile + (ln + i) * LD + hf * 8 + st * 32;
#pragma unroll
                    for (int ch = 0; ch < NCH; ++ch)
                        mma32(acc, tz[i][ch], *reinterpret_cast<const frag8<T> *>(rowp + ch * 16));
                }
            }
            // accumulator registers 8a..8a+7 of lane (row, half) are 8 consecutive keys
            if (interior) {
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    V16 out;
#pragma unroll
                    for (int u = 0; u < 8; ++u) out.v[u] = from_float<T>(acc[a * 8 + u]);
                    *reinterpret_cast<V16 *>(ybase + soff + st * 32 + a * 16) = out;
                }
            } else if (prow < H) {
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    const int q = q0 + st * 32 + a * 16 + hf * 8;
                    if (q >= W) continue;
                    V16 out;
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        out.v[u] = from_float<T>((causal && q + u > prow) ? 0.0f : acc[a * 8 + u]);
                    *reinterpret_cast<V16 *>(yp + (int64_t)prow * W + q) = out;
                }
            }
        }
        __syncthreads();  // LDS reads done before the next item's staging overwrites the strip

        if (mirror && tn < (tm >> 2))  // a quarter of the 128x128 block's image above the diagonal
            zero_fill_strip<T>(yp, H, W, q0 + (tm & 3) * M_TM, (tm >> 2) * M_TN, lane);
    }
}

inline int device_cu_count()
{
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

template <typename T, int R, int S>
int launch_mfma(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int causal,
                float in_scale, int use_scale, hipStream_t st)
{
    const int tiles_m = (int)((H + M_TM - 1) / M_TM), tiles_n = (int)((W + M_TN - 1) / M_TN);
    // mirror enumeration needs a square grid of whole 128x128 blocks' worth of strips
    const int blocks = (int)((H + M_TN - 1) / M_TN);
    const int mirror = (causal && H == W) ? 1 : 0;
    const int64_t ipp64 = mirror ? (int64_t)blocks * (blocks + 1) / 2 * 4 : (int64_t)tiles_m * tiles_n;
    if (ipp64 > (1 << 24)) return MTA_ERR_SHAPE;  // decode_item's float sqrt is exact well beyond this
    const int ipp = (int)ipp64;
    const int64_t total = N * C * ipp64;
    const int64_t per_xcd = (total + 7) / 8;
    int nw = device_cu_count() * 4 * MTA_CONV_WAVES_PER_SIMD / 8;  // persistent workgroups per XCD
    if (nw < 1) nw = 1;
    if (per_xcd < nw) nw = (int)per_xcd;
    dim3 grid((unsigned)(nw * 8));
    if (use_scale)
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, true>), grid, dim3(M_WT), 0, st, (const T *)x, (const T *)w, (T *)y, (int)C,
                           (int)H, (int)W, causal, in_scale, tiles_n, ipp, total, per_xcd, nw, mirror);
    else
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, false>), grid, dim3(M_WT), 0, st, (const T *)x, (const T *)w, (T *)y, (int)C,
                           (int)H, (int)W, causal, in_scale, tiles_n, ipp, total, per_xcd, nw, mirror);
    return launch_status();
}

// returns 1 when no MFMA instantiation covers (R,S) -- the caller then takes the VALU path
template <typename T>
int dispatch_mfma(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R, int S,
                  int causal, float in_scale, int use_scale, hipStream_t st)
{
#define MTA_CONV_CASE(r, s) \
    if (R == r && S == s) return launch_mfma<T, r, s>(x, w, y, N, C, H, W, causal, in_scale, use_scale, st);
    MTA_CONV_CASE(3, 3)
    MTA_CONV_CASE(3, 5)
    MTA_CONV_CASE(5, 5)
    MTA_CONV_CASE(5, 7)
    MTA_CONV_CASE(6, 11)
    MTA_CONV_CASE(7, 7)
    MTA_CONV_CASE(7, 9)
#undef MTA_CONV_CASE
    return 1;
}
template <>
int dispatch_mfma<float>(const void *, const void *, void *, int64_t, int64_t, int64_t, int64_t, int, int, int, float,
                         int, hipStream_t)
{
    return 1;
}

int conv2d_entry(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                 int S, int causal, float in_scale, int use_scale, int io_dtype, int w_dtype, void *stream)
{
    // MTA_CONV_FORCE_VALU=1 in the environment keeps 16-bit inputs on the fp32-FMA kernel (for comparisons)
    static const bool force_valu = [] { const char *e = getenv("MTA_CONV_FORCE_VALU"); return e && e[0] == '1'; }();
    if (!x || !w || !y) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0) return MTA_ERR_SHAPE;
    if (H > (1 << 24) || W > (1 << 24) || N * C > 0x7fffffffLL / 2) return MTA_ERR_SHAPE;
    if (R < 1 || S < 1 || R > MTA_MAX_KERNEL_R || S > MTA_MAX_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
    if (!aligned_to(x, dtype_size(io_dtype)) || !aligned_to(y, dtype_size(io_dtype)) ||
        !aligned_to(w, dtype_size(w_dtype)))
        return MTA_ERR_ALIGN;
    const int64_t tiles = ((H + V_TM - 1) / V_TM) * ((W + V_TN - 1) / V_TN);
    if (tiles > 0x7fffffffLL || N * C > 65535) return MTA_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    const bool mfma_ok = io_dtype != MTA_F32 && w_dtype == io_dtype && W % 8 == 0 && aligned_to(x, 16) &&
                         aligned_to(y, 16) && !force_valu;
    MTA_DISPATCH_IO(io_dtype, {
        if (mfma_ok) {
            const int rc = dispatch_mfma<io_t>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, st);
            if (rc != 1) return rc;
        }
        return dispatch_valu<io_t>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st);
    });
    return MTA_ERR_DTYPE;
}
}  // namespace

extern "C" int mta_conv2d_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H,
                              int64_t W, int R, int S, int causal, int io_dtype, int w_dtype, void *stream)
{
    return conv2d_entry(x, w, y, N, C, H, W, R, S, causal, 1.0f, 0, io_dtype, w_dtype, stream);
}

extern "C" int mta_conv2d_scaled_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H,
                                     int64_t W, int R, int S, int causal, float in_scale, int io_dtype,
                                     int w_dtype, void *stream)
{
    return conv2d_entry(x, w, y, N, C, H, W, R, S, causal, in_scale, 1, io_dtype, w_dtype, stream);
}
