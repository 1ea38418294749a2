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

// BWD: the gradient with respect to the input,
//   dx[h,w] = sum_{i,j} w[i,j] * dym[h-i+(R-1), w-j+(S-1)/2]        (dym = dy with q>p read as 0 when causal)
// which is the same tile computation with the kernel reversed in both axes, the row halo below the tile instead of
// above it and the key halos swapped; dx is +0 above the diagonal (those inputs were never read).
template <typename T, int R_T, int S_T, bool BWD>
__global__ __launch_bounds__(NT) void conv2d_valu(const T *__restrict__ x, const void *__restrict__ w,
                                                  T *__restrict__ y, int C, int H, int W, int R_rt,
                                                  int S_rt, int causal, float in_scale, int use_scale,
                                                  int w_dtype, int tiles_n)
{
    const int R = R_T > 0 ? R_T : R_rt;
    const int S = S_T > 0 ? S_T : S_rt;
    const int pad_h = BWD ? 0 : R - 1, pad_w = BWD ? S - 1 - (S - 1) / 2 : (S - 1) / 2;
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

    for (int t = tid; t < R * S; t += NT) wsm[t] = load_any(w, w_dtype, (int64_t)c * R * S + (BWD ? R * S - 1 - t : t));

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

template <typename T, int R_T, int S_T, bool BWD>
int launch_valu(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                int S, int causal, float in_scale, int use_scale, int w_dtype, hipStream_t st)
{
    const int tiles_m = (int)((H + V_TM - 1) / V_TM), tiles_n = (int)((W + V_TN - 1) / V_TN);
    const size_t lds = sizeof(float) * (((R * S + 3) & ~3) + (size_t)(V_TM + R - 1) * (V_TN + S));
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)(N * C));
    hipLaunchKernelGGL((conv2d_valu<T, R_T, S_T, BWD>), grid, dim3(NT), lds, st, (const T *)x, w, (T *)y, (int)C,
                       (int)H, (int)W, R, S, causal, in_scale, use_scale, w_dtype, tiles_n);
    return launch_status();
}

template <typename T, bool BWD>
int dispatch_valu(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                  int S, int causal, float in_scale, int use_scale, int w_dtype, hipStream_t st)
{
#define MTA_CONV_CASE(r, s)                                                                               \
    if (R == r && S == s)                                                                                 \
        return launch_valu<T, r, s, BWD>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st);
    MTA_CONV_CASE(3, 3)
    MTA_CONV_CASE(3, 5)
    MTA_CONV_CASE(5, 5)
    MTA_CONV_CASE(5, 7)
    MTA_CONV_CASE(6, 11)
    MTA_CONV_CASE(7, 7)
    MTA_CONV_CASE(7, 9)
    MTA_CONV_CASE(11, 15)
#undef MTA_CONV_CASE
    return launch_valu<T, 0, 0, BWD>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st);
}

// ------------------------------------------------------------------------------------
// MFMA (Toeplitz) path
// ------------------------------------------------------------------------------------
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// The output is written once and not read again by this kernel: non-temporal stores keep it from displacing the input
// rows that neighbouring strips re-read (halos) in the L2.
#define MTA_CONV_STORE(ptr, val) __builtin_nontemporal_store((val), (ptr))

constexpr int M_NW = 2;            // wavefronts per workgroup; each owns one 16-row block of the workgroup's strip
constexpr int M_WT = 64 * M_NW;    // threads per workgroup
constexpr int M_TM = 16 * M_NW;    // strip rows
constexpr int M_TN = 128;          // strip cols: 8 column blocks of 16
constexpr int M_SPB = M_TN / M_TM;  // strips per 128x128 block
constexpr int M_WG_PER_CU = 4;     // persistent workgroups per CU (two 12 KB strip buffers each); 3, 5 and 6 measured slower
static_assert(M_TN % M_TM == 0 && (M_SPB & (M_SPB - 1)) == 0, "strip geometry");

// 16 outputs + S-1 taps (+ alignment shift) must fit the 32-key contraction of one 16x16x32 MFMA
template <int R, int S> struct mfma_geom {
    static constexpr int PADW = (S - 1) / 2;
    static constexpr int HL = (PADW + 7) & ~7;             // left halo, rounded so 16-byte loads stay aligned
    static constexpr int SHIFT = HL - PADW;                // first tap's offset inside a block's 32-key window
    static constexpr bool fits = SHIFT + 16 + S - 1 <= 32;
    static constexpr int TW = M_TN - 16 + 32;              // staged columns
    static constexpr int LD = TW + ((24 - TW % 16) % 16);  // row stride = 8 (mod 16) elements: conflict-free b128 reads
    static constexpr int ROWS = M_TM + R - 1;
};

// position t of a work item inside its plane -> (strip row tm (M_TM rows), strip col tn (128 keys)).
// `mirror` (causal, square): only strips that touch the lower triangle are enumerated, by 128x128
// block in row-major lower-triangular order, M_SPB strips per block; each strip of an off-diagonal
// block also zero-fills its share (1/M_SPB) of the block's mirror image above the diagonal.
__device__ __forceinline__ void decode_item(int t, int tiles_n, int mirror, int &tm, int &tn)
{
    if (mirror) {
        const int blk = t / M_SPB;
        int bm = (int)((sqrtf(8.0f * (float)blk + 1.0f) - 1.0f) * 0.5f);
        while ((bm + 1) * (bm + 2) / 2 <= blk) ++bm;
        while (bm * (bm + 1) / 2 > blk) --bm;
        tn = blk - bm * (bm + 1) / 2;
        tm = bm * M_SPB + (t % M_SPB);
    } else {
        tm = t / tiles_n;
        tn = t % tiles_n;
    }
}

// Returns its argument, opaquely: what is derived from the result cannot be hoisted out of the (rarely taken) block
// that computes it, so it does not occupy registers in the main loop.
__device__ __forceinline__ int opaque(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// +0 over an M_TM x M_TN region, all threads of the workgroup.  FULL: the region lies inside the tensor; the stores are
// then unconditional (exactly M_TM*M_TN/8/M_WT vector-memory instructions per lane)
template <typename T, bool FULL = false>
__device__ __forceinline__ void zero_fill_strip(T *yp, int H, int W, int p0, int q0, int tid)
{
    constexpr int VEC = 8;
    pack16<T> z;
#pragma unroll
    for (int u = 0; u < VEC; ++u) z.v[u] = from_float<T>(0.0f);
    tid = opaque(tid);
    // thread t covers rows t/16 + 8k, vector t%16: a uniform base, one 32-bit per-lane byte offset, uniform row steps
    static_assert(M_WT == 128 && M_TN / VEC == 16, "region rows per pass");
    char *base = reinterpret_cast<char *>(yp + (int64_t)p0 * W + q0);
    const int r0 = tid >> 4, cv = (tid & 15) * VEC;
    const unsigned off = (unsigned)(r0 * W + cv) * (unsigned)sizeof(T);
    const int64_t rstep = (int64_t)(M_WT / 16) * W * (int64_t)sizeof(T);
#pragma unroll
    for (int k = 0; k < M_TM / (M_WT / 16); ++k) {
        if (FULL || (p0 + r0 + k * (M_WT / 16) < H && q0 + cv < W))
            MTA_CONV_STORE(reinterpret_cast<u32x4 *>(base + k * rstep + off), __builtin_bit_cast(u32x4, z));
    }
}

// The part of a square causal output above the diagonal's 128x128 blocks, written as +0 by workgroups of their own
// (mirror == 3): row p of a plane gets keys (p / M_TN + 1) * M_TN .. W-1, a contiguous run.  Workgroup `fid` of `nfill`
// takes rows fid, fid + nfill, ... of all planes.
template <typename T>
__device__ __forceinline__ void fill_above_blocks(T *y, int64_t planes, int H, int W, int fid, int nfill, int tid)
{
    constexpr int VEC = 8;
    pack16<T> z;
#pragma unroll
    for (int u = 0; u < VEC; ++u) z.v[u] = from_float<T>(0.0f);
    const int64_t rows = planes * H;
    for (int64_t rr = fid; rr < rows; rr += nfill) {
        const int p = (int)(rr % H);
        T *row = y + rr * W;
        for (int q = (p / M_TN + 1) * M_TN + tid * VEC; q < W; q += M_WT * VEC)
            MTA_CONV_STORE(reinterpret_cast<u32x4 *>(row + q), __builtin_bit_cast(u32x4, z));
    }
}

typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;

// The staged strips are read and written through these, not through C++ accesses: the compiler cannot tell an access
// to one half of the double buffer from the asynchronous copy in flight into the other half and would wait for the
// copy first (the copy would then never overlap the matrix products).  LDS operations of a wavefront complete in
// order; lds_wait() waits for all of them and ties the loaded values to that point.
__device__ __forceinline__ u32x4 lds_load16(unsigned addr)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
// the same with a compile-time byte offset in the instruction (no address arithmetic per access)
// (`off` must fold to a constant below 65536: it goes into the instruction's offset field)
__device__ __forceinline__ u32x4 lds_load16_at(unsigned addr, int off)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(off) : "memory");
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
__device__ __forceinline__ void lds_store8(unsigned addr, unsigned lo, unsigned hi)
{
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 v = {lo, hi};
    asm volatile("ds_write_b64 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }
__device__ __forceinline__ void lds_wait(u32x4 &a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a) : : "memory"); }
// workgroup barrier without the memory fence __syncthreads() carries (which would wait for the copy in flight)
__device__ __forceinline__ void wg_barrier() { asm volatile("s_barrier" : : : "memory"); }

// Persistent two-wavefront workgroups: each walks a run of M_TM x 128 strips dealt round-robin within its XCD's share
// of the item list.  Wavefront w owns row block w (16 rows) of the strip: it issues half of the staging copies, computes
// its row block and stores it.  The wavefronts meet at one barrier per strip (the strip has landed; the previous
// strip's buffer may be overwritten); latency is hidden by the other workgroups resident on the CU, each in its own
// phase (loading / matrix cores / storing) with its own two 11.6 KB LDS strip buffers.
//
// Per 16x16 output block and kernel row i:  out^T[q, p] += T_i^T[q, k] X^T[k, p+i-(R-1)], one
// v_mfma_f32_16x16x32 whose 32-key contraction window holds the 16 outputs' taps.  A operand =
// Toeplitz fragment (4 VGPRs per kernel row, kept while the channel is unchanged), B operand = 16 contiguous
// bytes of one staged row per lane.  A wavefront sustains about one such 1 KB LDS operand per 35 cycles whatever the
// addresses, against 16 cycles for the product: the products of a strip are therefore split over two wavefronts (on
// two SIMDs).  Results go back through LDS rows that only the owning wavefront reads (row block 0: the strip's first
// 16 staged rows; row block w > 0: the last 16 staged rows of its window) so that the global stores are whole
// 256-byte row segments.
//
// Staging.  A strip whose halo lies wholly inside the tensor and on or below the diagonal (the
// common case, decided per workgroup) is copied global -> LDS by global_load_lds_dwordx4: no
// registers, no masks, no LDS store instructions.  The LDS row stride is 19 16-byte slots (18 of
// data + 1 of padding), so thread t of copy `it` simply owns slot it*128+t.  Diagonal and border strips
// are copied the same way and fixed up in LDS; the rare strips whose copy could leave the tensor go
// through registers, where bounds and the causal col<=row rule are applied.
//
// SCALED: every strip is staged through registers, where x*in_scale is rounded to the I/O dtype before it
// reaches LDS (what a separate elementwise scale pass would have produced).
//
// BWD: the gradient with respect to the input (see conv2d_valu): kernel rows reversed in both axes, the R-1 halo rows
// below the strip instead of above it.  Key sizes are odd here, so the key halos are the same on both sides.
template <typename T, int R, int S, bool SCALED, bool BWD>
__global__ __launch_bounds__(M_WT, 2) void conv2d_mfma(
    const T *__restrict__ x, const T *__restrict__ w, T *__restrict__ y, int C, int H, int W, int causal, float in_scale,
    int tiles_n, int ipp, int64_t total, int64_t per_xcd, int nw, int mirror, int nfill)
{
    // mirror == 3: the image above the diagonal is written by nfill workgroups of their own, which the device runs
    // beside the persistent ones (they hold no registers or LDS traffic to speak of)
    if (mirror == 3 && (int)blockIdx.x >= nw * 8) {
        fill_above_blocks<T>(y, total / ipp, H, W, (int)blockIdx.x - nw * 8, nfill, (int)threadIdx.x);
        return;
    }
    using G = mfma_geom<R, S>;
    static_assert(!BWD || (S % 2 == 1 && !SCALED), "the backward instance assumes symmetric key halos and no scale");
    constexpr int TOP = BWD ? 0 : R - 1;                    // halo rows above the strip (the others lie below it)
    constexpr int LD = G::LD, VEC = 8;
    constexpr int VPR = G::TW / VEC;                        // data vectors per staged row (18)
    constexpr int SPR = LD / VEC;                           // 16-byte slots per LDS row (19)
    constexpr int SLOTS = G::ROWS * SPR;
    constexpr int STAGE_IT = (SLOTS + M_WT - 1) / M_WT;     // copies per strip and lane
    static_assert(SPR == VPR + 1, "one padding slot per row");
    // weights of the current channel, each kernel row zero-padded on both sides so that the
    // Toeplitz fragments can be gathered without range checks
    constexpr int WZ_OFF = G::SHIFT + 16, WZ_LD = WZ_OFF + 32;
    constexpr int BUF = STAGE_IT * M_WT * VEC;               // elements per LDS strip buffer
    __shared__ __align__(16) T tiles[2 * BUF];               // double buffer: strip n is computed while strip n+1 lands
    __shared__ T wz[2][R * WZ_LD];                           // by strip parity: a wavefront may run one strip ahead
    using V16 = pack16<T>;

    // XCD-aware split: workgroup ids are dealt round-robin to the 8 XCDs; each XCD gets one
    // contiguous chunk of the item list (whole planes, mostly), so halo re-reads stay in its L2.
    const int64_t c0 = (int64_t)(blockIdx.x & 7) * per_xcd;
    const int64_t c1 = (c0 + per_xcd < total) ? c0 + per_xcd : total;
    // within the chunk the items are dealt round-robin to the XCD's workgroups, so that at any moment
    // they sweep the same few hundred rows together (DRAM pages are consumed whole, as by a linear copy)
    const int64_t first = c0 + (int64_t)(blockIdx.x >> 3);
    const int64_t last = c1;
    const int step = nw;
    if (c0 >= total || first >= last) return;
    const int n_items = (int)((last - first + step - 1) / step);
    const int64_t HW = (int64_t)H * W;

    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 15, kg = lane >> 4;
    // (the wavefront index through readfirstlane: everything derived from it is then scalar)
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    frag8<T> tz[R];
    int cur_channel = -1;

    // per-thread geometry of the staging copies, fixed for the whole kernel: slot it*M_WT+tid is row srow,
    // vector svc of the strip; padding slots and slots past the strip re-read a neighbouring valid vector
    unsigned goff[STAGE_IT];  // byte offsets from the strip's first staged element (uniform base + 32-bit lane offset)
#pragma unroll
    for (int it = 0; it < STAGE_IT; ++it) {
        const int slot = it * M_WT + tid;
        int rr = slot / SPR, vc = slot % SPR;
        if (rr >= G::ROWS) { rr = 0; vc = 0; }
        if (vc >= VPR) vc = VPR - 1;
        goff[it] = (unsigned)(rr * W + vc * VEC) * (unsigned)sizeof(T);
    }

    // a strip is `interior` when its whole halo lies inside the tensor and on or below the diagonal
    auto is_interior = [&](int p0_, int q0_) {
        if (SCALED) return false;
        const int h0 = p0_ - TOP, k0 = q0_ - G::HL;
        return h0 >= 0 && h0 + G::ROWS <= H && k0 >= 0 && k0 + G::TW <= W && (!causal || k0 + G::TW - 1 <= h0);
    };
    // A strip is `copyable` when the same copy can be issued for it without faulting: its rows lie inside the plane
    // and the bytes its slots address (left halo of the first column strip = tail of the previous row, right halo of
    // the last one = head of the next row) lie inside the tensor.  What such a copy brings in from outside the plane
    // or from above the diagonal is zeroed in LDS afterwards (diagonal and border strips: a quarter of all strips,
    // which would otherwise load synchronously through registers).
    // (a plane is named by the offset of its first element, `pbase`: kept up to date by additions, no 64-bit divisions)
    const int64_t total_elems = (int64_t)(total / ipp) * HW;  // planes * H * W
    auto is_copyable = [&](int64_t pbase_, int p0_, int q0_) {
        if (SCALED) return false;
        const int h0 = p0_ - TOP, k0 = q0_ - G::HL;
        if (h0 < 0 || h0 + G::ROWS > H) return false;
        const int64_t e0 = pbase_ + (int64_t)h0 * W + k0;
        return e0 >= 0 && e0 + (int64_t)(G::ROWS - 1) * W + G::TW <= total_elems;
    };
    // asynchronous copy of an interior or copyable strip into LDS buffer `buf` (this wavefront's half of the slots)
    auto prefetch = [&](int64_t pbase_, int p0_, int q0_, T *buf) {
        const char *base = reinterpret_cast<const char *>(x + pbase_ + (int64_t)(p0_ - TOP) * W + (q0_ - G::HL));
#pragma unroll
        for (int it = 0; it < STAGE_IT; ++it)
            __builtin_amdgcn_global_load_lds((glb_void_t *)(base + goff[it]),
                                             (lds_void_t *)(buf + (it * M_WT + wave * 64) * VEC), 16, 0, 0);
    };

    // The (zero-padded) kernel rows of a strip's channel are fetched one strip ahead into WPL registers per lane and
    // written to `wz` at the top of that strip's iteration: the items of a plane are dealt out over all workgroups of
    // an XCD, so a workgroup changes channel every few strips, and a fetch at the point of use would expose a full
    // memory latency each time.  The loads are issued from inline assembly, before the strip's copy, and are covered
    // by the wait for that copy at the top of the next iteration: seen by the compiler, they would make it wait for
    // every outstanding memory operation - the previous strip's stores included - before the values' first use.
    // (The build fails if this kernel spills registers: a spill between the load and that wait would save a value
    // that has not arrived yet.)
    constexpr int WPL = (R * WZ_LD + M_WT - 1) / M_WT;
    static_assert(sizeof(T) == 2, "16-bit loads");
    unsigned wnext[WPL];
    unsigned woff[WPL];   // byte offset of this lane's tap inside a channel's kernel (0 where the slot is padding)
    unsigned wvalid = 0;  // bit it: slot it*M_WT+tid of the padded kernel rows holds a tap
#pragma unroll
    for (int it = 0; it < WPL; ++it) {
        const int e = it * M_WT + tid;
        const int i = e / WZ_LD, j = e % WZ_LD - WZ_OFF;
        const bool ok = e < R * WZ_LD && j >= 0 && j < S;
        woff[it] = ok ? (unsigned)(BWD ? (R - 1 - i) * S + (S - 1 - j) : i * S + j) * (unsigned)sizeof(T) : 0u;
        wvalid |= ok ? (1u << it) : 0u;
    }
    auto fetch_weights = [&](int channel_) {
        const char *wc = reinterpret_cast<const char *>(w + channel_ * R * S);
#pragma unroll
        for (int it = 0; it < WPL; ++it)
            asm volatile("global_load_ushort %0, %1, %2" : "=v"(wnext[it]) : "v"(woff[it]), "s"(wc) : "memory");
    };
    // current and next work item: position inside the plane, plane (as element offset) and channel
    int t_nx;
    int64_t pbase_nx;
    int chan_nx;
    {
        const int64_t plane0 = first / ipp;
        t_nx = (int)(first - plane0 * ipp);
        pbase_nx = plane0 * HW;
        chan_nx = (int)(plane0 % C);
    }
    int tm, tn;
    decode_item(t_nx, tiles_n, mirror, tm, tn);
    fetch_weights(chan_nx);
    if (is_copyable(pbase_nx, tm * M_TM, tn * M_TN)) prefetch(pbase_nx, tm * M_TM, tn * M_TN, tiles);

    int younger = -1;                      // stores certainly issued after the copy in flight (-1: unknown)
    const bool fill_full = H % M_TN == 0;  // mirror images of whole 128x128 blocks lie inside the (square) tensor
    int parity = 0;
    for (int item = 0; item < n_items; ++item, parity ^= 1) {
        T *tile = tiles + parity * BUF;
        T *other = tiles + (parity ^ 1) * BUF;
        T *wzp = wz[parity];
        const int p0 = tm * M_TM, q0 = tn * M_TN;
        const int ctm = tm, ctn = tn;
        const int64_t pbase = pbase_nx;
        const T *xp = x + pbase;
        T *yp = y + pbase;
        const int channel = chan_nx;
        const bool above = causal && q0 > p0 + M_TM - 1;  // wholly above the diagonal (only reachable when !mirror)
        const bool interior = is_interior(p0, q0);
        const bool copyable = interior || is_copyable(pbase, p0, q0);
        const int h0 = p0 - TOP, k0 = q0 - G::HL;
        // (opaque: the addresses derived from it are then formed where they are used instead of being kept, dozens of
        // them, in registers across the loop)
        const unsigned tile_lds = (unsigned)opaque((int)(unsigned)(uintptr_t)(lds_void_t *)tile);

        // This wavefront's half of the strip's copy (if any) has landed.  Vector-memory operations complete in issue
        // order, and the only ones this wavefront issued after that copy are the previous strip's stores: when their
        // number is known exactly (`younger`), they may stay in flight.
        {
            constexpr int ST = M_TM * (M_TN / VEC) / M_WT;  // stores per strip and lane, and per mirror share
            if (younger == 2 * ST) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * ST) : "memory");
            else if (younger == ST) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(ST) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
        }
        younger = 0;

        // this strip's kernel rows, fetched during the previous iteration, go to LDS (every strip: see fetch_weights)
#pragma unroll
        for (int it = 0; it < WPL; ++it) {
            asm volatile("" : "+v"(wnext[it]));  // (the value is defined from the wait above on)
            const int e = it * M_WT + tid;
            if (e < R * WZ_LD) wzp[e] = ((wvalid >> it) & 1u) ? __builtin_bit_cast(T, (unsigned short)wnext[it]) : from_float<T>(0.0f);
        }

        if (!above && copyable && !interior) {
            // the copy has landed: zero what lies outside the plane or above the diagonal (whole vectors, except the one
            // vector of a row that straddles the diagonal)
            const int tid_ = opaque(tid);
            const u32x4 zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * M_WT + tid_;
                const int rr = slot / SPR, vc = slot % SPR;
                const int h = h0 + rr, col = k0 + vc * VEC;
                const bool ok = rr < G::ROWS && vc < VPR && col >= 0 && col < W && !(causal && col > h);
                const unsigned addr = tile_lds + (unsigned)slot * 16u;
                if (!ok) {
                    lds_store16(addr, zero4);
                } else if (causal && col + VEC - 1 > h) {
                    u32x4 raw = lds_load16(addr);
                    lds_wait(raw);
                    V16 v = __builtin_bit_cast(V16, raw);
#pragma unroll
                    for (int u = 0; u < VEC; ++u)
                        if (col + u > h) v.v[u] = from_float<T>(0.0f);
                    lds_store16(addr, __builtin_bit_cast(u32x4, v));
                }
            }
        } else if (!above && !interior) {
            // edge strip: through registers.  Loads are unconditional and issued back to back (an invalid
            // slot re-reads a valid address); what a slot really holds is decided on the way to LDS
            V16 stage[STAGE_IT];
            const int tid_ = opaque(tid);
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * M_WT + tid_;
                const int rr = slot / SPR, vc = slot % SPR;
                const int h = h0 + rr, col = k0 + vc * VEC;
                const bool ok = rr < G::ROWS && vc < VPR && h >= 0 && h < H && col >= 0 && col < W && !(causal && col > h);
                stage[it] = *reinterpret_cast<const V16 *>(xp + (ok ? (int64_t)h * W + col : 0));
            }
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * M_WT + tid_;
                const int rr = slot / SPR, vc = slot % SPR;
                const int h = h0 + rr, col = k0 + vc * VEC;
                const bool ok = rr < G::ROWS && vc < VPR && h >= 0 && h < H && col >= 0 && col < W && !(causal && col > h);
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
                lds_store16(tile_lds + (unsigned)slot * 16u, __builtin_bit_cast(u32x4, v));
            }
        }
        lds_wait();    // this wavefront's LDS stores above are complete
        wg_barrier();  // the strip and its kernel rows are in LDS; every wavefront is done with the previous strip

        // put the next strip's copy in flight (into the buffer the previous iteration has just released)
        if (item + 1 < n_items) {
            t_nx += step;
            while (t_nx >= ipp) {  // (at most once, unless a plane holds fewer items than there are workgroups)
                t_nx -= ipp;
                pbase_nx += HW;
                chan_nx = chan_nx + 1 == C ? 0 : chan_nx + 1;
            }
            decode_item(t_nx, tiles_n, mirror, tm, tn);
            fetch_weights(chan_nx);  // (before the copy: the loop-top wait counts what is younger than the copy)
            if (is_copyable(pbase_nx, tm * M_TM, tn * M_TN)) prefetch(pbase_nx, tm * M_TM, tn * M_TN, other);
        }
        if (above) {
            zero_fill_strip<T>(yp, H, W, p0, q0, tid);
            younger = -1;
            continue;
        }

        if (channel != cur_channel) {  // Toeplitz fragments T_i^T for this lane's accumulator row
            cur_channel = channel;
#pragma unroll
            for (int i = 0; i < R; ++i) {  // row m = ln, slots k = 8*kg + t, tap j = k-SHIFT-m
                const T *src = wzp + i * WZ_LD + WZ_OFF + kg * 8 - G::SHIFT - ln;
#pragma unroll
                for (int t = 0; t < 8; ++t) tz[i].v[t] = src[t];
            }
        }

        // ---- this wavefront's row block: 8 column blocks of 16x16 outputs on 16x16x32 MFMAs (one per kernel row: the
        // 32-key window holds the 16 outputs' taps).  Lane (row ln, group kg) holds keys 4*kg..4*kg+3 of each block.
        const int rb0 = wave * 16;                                   // first strip row of the block
        const int res0 = wave == 0 ? 0 : wave * 16 + R - 1;          // staged rows that receive the results
        {
            f32x4 acc[M_TN / 16];
            const unsigned xa = tile_lds + (unsigned)((rb0 + ln) * LD + kg * 8) * sizeof(T);
            // Column blocks in pairs.  A wavefront issues in order, so a run of LDS reads followed by a run of
            // products leaves the matrix cores idle during the first and the LDS idle during the second; here one read
            // of the next pair's operands is issued per product of this pair, and a product waits only for its
            // own operand, issued 2R reads earlier (LDS operations complete in order: lgkmcnt(2R) at every
            // step).  Source order is pinned (the scheduler would regroup reads and products).  Blocks above the
            // diagonal are computed like the others and masked below.
            constexpr int NPAIR = M_TN / 32, NLD = 2 * R;
            static_assert(NLD <= 15, "lgkmcnt field");
            u32x4 xf[2][2][R];
            auto xoff = [&](int pr, int c2, int i) { return (int)((i * LD + (pr * 2 + c2) * 16) * sizeof(T)); };
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c2 = 0; c2 < 2; ++c2) xf[0][c2][i] = lds_load16_at(xa, xoff(0, c2, i));
#pragma unroll
            for (int pr = 0; pr < NPAIR; ++pr) {
                acc[2 * pr] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                acc[2 * pr + 1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int i = 0; i < R; ++i)
#pragma unroll
                    for (int c2 = 0; c2 < 2; ++c2) {
                        u32x4 &cur = xf[pr & 1][c2][i];
                        if (pr + 1 < NPAIR) {
                            xf[(pr + 1) & 1][c2][i] = lds_load16_at(xa, xoff(pr + 1, c2, i));
                            asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(cur) : "n"(NLD) : "memory");
                        } else {  // last pair: only this pair's later reads are newer
                            asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(cur) : "n"(NLD - 1 - (2 * i + c2)) : "memory");
                        }
                        mma16(acc[2 * pr + c2], tz[i], __builtin_bit_cast(frag8<T>, cur));
                        __builtin_amdgcn_sched_barrier(0);
                    }
            }
            // results into the staged rows res0.. (read by this wavefront only, and no longer needed by it)
            const int prow = p0 + rb0 + ln;
            const unsigned ra = tile_lds + (unsigned)((res0 + ln) * LD + kg * 4) * sizeof(T);
#pragma unroll
            for (int cb = 0; cb < M_TN / 16; ++cb) {
                const int q = q0 + cb * 16 + kg * 4;
                uint32_t lo = pack2<T>(acc[cb][0], acc[cb][1]), hi = pack2<T>(acc[cb][2], acc[cb][3]);
                if (!interior && causal && q + 3 > prow) {
                    if (q > prow) lo &= 0xffff0000u;
                    if (q + 1 > prow) lo &= 0x0000ffffu;
                    if (q + 2 > prow) hi &= 0xffff0000u;
                    if (q + 3 > prow) hi &= 0x0000ffffu;
                }
                lds_store8_at(ra, (int)(cb * 16 * sizeof(T)), lo, hi);
            }
        }
        // ---- coalesced stores of this wavefront's 16 rows: 16 lanes cover one 256-byte output row (the LDS writes
        // above precede these reads in the wavefront's LDS queue) ----
        {
            // (uniform row base + one 32-bit per-lane byte offset: no 64-bit address arithmetic per store)
            char *ybase = reinterpret_cast<char *>(yp + (int64_t)(p0 + rb0) * W + q0);
            const int lane_o = opaque(lane);  // (row offsets formed here, not kept in registers across the loop)
            const int r_l = lane_o >> 4, cv = (lane_o & 15) * VEC;
            const unsigned yoff = (unsigned)(r_l * W + cv) * (unsigned)sizeof(T);
            const int64_t ystep = (int64_t)4 * W * (int64_t)sizeof(T);
            constexpr int OUT_IT = 16 * (M_TN / VEC) / 64;
            static_assert(OUT_IT == 4, "four row groups per wavefront");
            u32x4 v[4];
            const unsigned va = tile_lds + (unsigned)((res0 + r_l) * LD + cv) * sizeof(T);
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = lds_load16_at(va, (int)(k * 4 * LD * sizeof(T)));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : : "memory");
            if (interior) {  // unconditional: exactly OUT_IT vector-memory instructions
#pragma unroll
                for (int k = 0; k < 4; ++k) MTA_CONV_STORE(reinterpret_cast<u32x4 *>(ybase + k * ystep + yoff), v[k]);
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int r = k * 4 + r_l;
                    if (p0 + rb0 + r < H && q0 + cv < W) MTA_CONV_STORE(reinterpret_cast<u32x4 *>(ybase + k * ystep + yoff), v[k]);
                }
            }
            younger = interior ? OUT_IT : -1;
        }
        // (mirror == 2: the caller does not want the image written)
        if (mirror == 1 && ctn < ctm / M_SPB) {  // this strip's share of the 128x128 block's image above the diagonal
            if (fill_full) {
                zero_fill_strip<T, true>(yp, H, W, q0 + (ctm % M_SPB) * M_TM, (ctm / M_SPB) * M_TN, tid);
                if (younger > 0) younger += M_TM * (M_TN / VEC) / M_WT;
            } else {
                zero_fill_strip<T>(yp, H, W, q0 + (ctm % M_SPB) * M_TM, (ctm / M_SPB) * M_TN, tid);
                younger = -1;
            }
        }
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

template <typename T, int R, int S, bool BWD>
int launch_mfma(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int causal,
                float in_scale, int use_scale, hipStream_t st)
{
    const int tiles_m = (int)((H + M_TM - 1) / M_TM), tiles_n = (int)((W + M_TN - 1) / M_TN);
    // mirror enumeration needs a square grid of whole 128x128 blocks' worth of strips
    const int blocks = (int)((H + M_TN - 1) / M_TN);
    // (MTA_CONV_INLINE_FILL=1 in the environment: the strips' own workgroups write the image, for comparisons)
    static const bool inline_fill = [] { const char *e = getenv("MTA_CONV_INLINE_FILL"); return e && e[0] == '1'; }();
    const int mirror = (causal && H == W) ? (causal == 2 ? 2 : ((inline_fill || W % 8 != 0 || blocks < 2) ? 1 : 3)) : 0;
    const int64_t ipp64 = mirror ? (int64_t)blocks * (blocks + 1) / 2 * M_SPB : (int64_t)tiles_m * tiles_n;
    if (ipp64 > (1 << 24)) return MTA_ERR_SHAPE;  // decode_item's float sqrt is exact well beyond this
    const int ipp = (int)ipp64;
    const int64_t total = N * C * ipp64;
    const int64_t per_xcd = (total + 7) / 8;
    int nw = device_cu_count() * M_WG_PER_CU / 8;  // persistent workgroups per XCD
    if (nw < 1) nw = 1;
    if (per_xcd < nw) nw = (int)per_xcd;
    const int nfill = mirror == 3 ? device_cu_count() * 2 : 0;  // two more workgroups per CU fit beside the persistent four
    dim3 grid((unsigned)(nw * 8 + nfill));
    if constexpr (BWD) {
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, false, true>), grid, dim3(M_WT), 0, st, (const T *)x, (const T *)w, (T *)y,
                           (int)C, (int)H, (int)W, causal, in_scale, tiles_n, ipp, total, per_xcd, nw, mirror, nfill);
    } else if (use_scale) {
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, true, false>), grid, dim3(M_WT), 0, st, (const T *)x, (const T *)w, (T *)y,
                           (int)C, (int)H, (int)W, causal, in_scale, tiles_n, ipp, total, per_xcd, nw, mirror, nfill);
    } else {
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, false, false>), grid, dim3(M_WT), 0, st, (const T *)x, (const T *)w, (T *)y,
                           (int)C, (int)H, (int)W, causal, in_scale, tiles_n, ipp, total, per_xcd, nw, mirror, nfill);
    }
    return launch_status();
}

// returns 1 when no MFMA instantiation covers (R,S) -- the caller then takes the VALU path
template <typename T, bool BWD>
int dispatch_mfma(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R, int S,
                  int causal, float in_scale, int use_scale, hipStream_t st)
{
    if constexpr (sizeof(T) != 2) return 1;
    else {
#define MTA_CONV_CASE(r, s)                                       \
    static_assert(mfma_geom<r, s>::fits, "window exceeds 32 keys"); \
    if (R == r && S == s) return launch_mfma<T, r, s, BWD>(x, w, y, N, C, H, W, causal, in_scale, use_scale, st);
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
}

template <bool BWD>
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
            const int rc = dispatch_mfma<io_t, BWD>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, st);
            if (rc != 1) return rc;
        }
        return dispatch_valu<io_t, BWD>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st);
    });
    return MTA_ERR_DTYPE;
}
// the `causal` argument of the entry points: 0 = no mask, 2 = causal with the output above the diagonal left to the
// caller (MTA_CAUSAL_LOWER_ONLY), anything else = causal with +0 written there
inline int causal_mode(int causal) { return causal == MTA_CAUSAL_LOWER_ONLY ? 2 : (causal ? 1 : 0); }
}  // namespace

extern "C" int mta_conv2d_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H,
                              int64_t W, int R, int S, int causal, int io_dtype, int w_dtype, void *stream)
{
    return conv2d_entry<false>(x, w, y, N, C, H, W, R, S, causal_mode(causal), 1.0f, 0, io_dtype, w_dtype, stream);
}

// (causal == 2 inside this file: causal, and the kernel that enumerates the lower triangle's strips only - the
// matrix-core one on square tensors - does not write their images above the diagonal; every other path fills as usual)
extern "C" int mta_conv2d_tril_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W,
                                   int R, int S, int io_dtype, int w_dtype, void *stream)
{
    return conv2d_entry<false>(x, w, y, N, C, H, W, R, S, 2, 1.0f, 0, io_dtype, w_dtype, stream);
}

extern "C" int mta_conv2d_bwd_input(const void *dy, const void *w, void *dx, int64_t N, int64_t C, int64_t H,
                                    int64_t W, int R, int S, int causal, int io_dtype, int w_dtype, void *stream)
{
    return conv2d_entry<true>(dy, w, dx, N, C, H, W, R, S, causal_mode(causal), 1.0f, 0, io_dtype, w_dtype, stream);
}

extern "C" int mta_conv2d_scaled_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H,
                                     int64_t W, int R, int S, int causal, float in_scale, int io_dtype,
                                     int w_dtype, void *stream)
{
    return conv2d_entry<false>(x, w, y, N, C, H, W, R, S, causal_mode(causal), in_scale, 1, io_dtype, w_dtype, stream);
}
