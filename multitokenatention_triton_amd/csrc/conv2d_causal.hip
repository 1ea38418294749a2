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
#define MTA_CONV_WAVES_PER_SIMD 2  // register budget: 256 VGPRs per lane (the Toeplitz fragments take 72)
#endif
#ifndef MTA_CONV_WG_PER_CU
#define MTA_CONV_WG_PER_CU 2       // persistent workgroups per CU (4 wavefronts each); LDS: 75 KB per workgroup
#endif
#ifndef MTA_CONV_RING
#define MTA_CONV_RING 6            // staged strips per workgroup: one in use, RING-1 copies in flight
#endif
#ifndef MTA_CONV_NT_STORE
#define MTA_CONV_NT_STORE 0
#endif
constexpr int M_NW = 4;          // wavefronts per workgroup: one 32-key sub-tile of the strip each
constexpr int M_NT = 64 * M_NW;
constexpr int M_TM = 32;         // strip rows
constexpr int M_TN = 32 * M_NW;  // strip cols
constexpr int M_RING = MTA_CONV_RING;

// 32 outputs + S-1 taps (+ alignment shift) must fit three 16-key chunks (three 32x32x16 MFMAs per kernel row)
template <int R, int S> struct mfma_geom {
    static constexpr int PADW = (S - 1) / 2;
    static constexpr int HL = (PADW + 7) & ~7;             // left halo, rounded so 16-byte loads stay aligned
    static constexpr int SHIFT = HL - PADW;                // first tap's offset inside a sub-tile's 48-key window
    static constexpr bool fits = SHIFT + 32 + S - 1 <= 48;
    static constexpr int TW = M_TN + 16;                   // staged columns
    static constexpr int LD = TW + ((24 - TW % 16) % 16);  // row stride = 8 (mod 16) elements: conflict-free b128 reads
    static constexpr int ROWS = M_TM + R - 1;
};

// item t of a plane -> strip row tm (32 rows), strip col tn (128 keys).
// `mirror` (causal, square): only strips that touch the lower triangle are enumerated, by 128x128
// block in row-major lower-triangular order, 4 strips per block; each strip of an off-diagonal
// block also zero-fills a quarter of the block's mirror image above the diagonal.
__device__ __forceinline__ void decode_item(int t, int tiles_n, int mirror, int &tm, int &tn)
{
    if (mirror) {
        const int blk = t >> 2;
        // row bm of the triangle: bm(bm+1)/2 <= blk < (bm+1)(bm+2)/2.  The float estimate is off by at most one
        // (blk < 2^22); straight-line corrections, no loops
        int bm = (int)((sqrtf(8.0f * (float)blk + 1.0f) - 1.0f) * 0.5f);
        bm += ((bm + 1) * (bm + 2) / 2 <= blk) ? 1 : 0;
        bm -= (bm * (bm + 1) / 2 > blk) ? 1 : 0;
        tn = blk - bm * (bm + 1) / 2;
        tm = bm * 4 + (t & 3);
    } else {
        tm = t / tiles_n;
        tn = t % tiles_n;
    }
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;

__device__ __forceinline__ void store_out(void *dst, u32x4 v)
{
#if MTA_CONV_NT_STORE
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(dst));
#else
    *reinterpret_cast<u32x4 *>(dst) = v;
#endif
}

// 32 x 128 elements of +0 at (p0, q0): two 16-byte stores per lane.  FULL: the region lies inside the tensor
// (the stores are then unconditional: exactly two vector-memory instructions per wavefront)
template <typename T, bool FULL>
__device__ __forceinline__ void zero_fill_strip(T *yp, int H, int W, int p0, int q0, int tid)
{
    constexpr int VEC = 8;
    const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int it = 0; it < M_TM * (M_TN / VEC) / M_NT; ++it) {
        const int e = it * M_NT + tid, r = e / (M_TN / VEC), col = q0 + (e % (M_TN / VEC)) * VEC;
        if (FULL || (p0 + r < H && col < W)) store_out(yp + (int64_t)(p0 + r) * W + col, z);
    }
}

// The staged strips are read and patched through these, not through C++ loads: the compiler cannot tell a read
// of one ring slot from the asynchronous copy in flight into another and would wait for all copies first.
// The LDS counter is waited for by lds_wait(), which also ties the values to that point.
__device__ __forceinline__ u32x4 lds_load16(unsigned addr)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
__device__ __forceinline__ void lds_store16(unsigned addr, u32x4 v)
{
    asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ void lds_wait(u32x4 &a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a) : : "memory"); }
__device__ __forceinline__ void lds_wait(u32x4 &a, u32x4 &b, u32x4 &c)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c) : : "memory");
}
__device__ __forceinline__ void lds_wait(u32x4 (&a)[6])
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]) : : "memory");
}
// LDS operations of this wavefront complete, then workgroup barrier; vector-memory operations stay in flight
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory"); }
// wait until at most `keep` (a lower bound of the number of younger ones) vector-memory operations are outstanding
__device__ __forceinline__ void vm_wait(int keep)
{
    if (keep >= 24) asm volatile("s_waitcnt vmcnt(24)" : : : "memory");
    else if (keep >= 20) asm volatile("s_waitcnt vmcnt(20)" : : : "memory");
    else if (keep >= 17) asm volatile("s_waitcnt vmcnt(17)" : : : "memory");
    else if (keep >= 14) asm volatile("s_waitcnt vmcnt(14)" : : : "memory");
    else if (keep >= 12) asm volatile("s_waitcnt vmcnt(12)" : : : "memory");
    else if (keep >= 10) asm volatile("s_waitcnt vmcnt(10)" : : : "memory");
    else if (keep >= 8) asm volatile("s_waitcnt vmcnt(8)" : : : "memory");
    else if (keep >= 6) asm volatile("s_waitcnt vmcnt(6)" : : : "memory");
    else if (keep >= 5) asm volatile("s_waitcnt vmcnt(5)" : : : "memory");
    else if (keep >= 3) asm volatile("s_waitcnt vmcnt(3)" : : : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
}

// Persistent workgroups of 4 wavefronts walk a list of 32x128 strips.  The kernel is bound by memory latency, not
// by arithmetic: what counts is the number of bytes in flight per CU.  Every workgroup therefore keeps RING-1
// strip copies in flight while it works on one, and never waits for its stores.
//
// Staging.  Every strip (rows p0-(R-1) .. p0+31, columns q0-HL .. q0+135) is copied global -> LDS by
// global_load_lds_dwordx4, RING-1 strips ahead of the computation, into a ring of LDS buffers: no registers, no
// LDS store instructions.  The LDS row stride is 19 16-byte slots (18 of data + 1 of padding), lane t of copy `it`
// owns slot it*256+t.  A strip whose halo lies wholly inside the tensor and on or below the diagonal needs nothing
// more.  For the others the copy reads from clamped (valid) addresses and, once it has landed, each lane rewrites
// its own slots in LDS: +0 where the slot lies outside the tensor or above the diagonal, a per-element mask in
// the one vector of a row that straddles the diagonal.  SCALED: the same pass replaces every value by
// x*in_scale rounded to the I/O dtype (what a separate elementwise scale pass would have produced).
//
// Waiting.  Vector-memory operations of a wavefront complete in issue order, so "the copy of strip n has landed"
// is "at most k operations are outstanding", k = the number of operations issued after that copy.  The kernel
// counts the operations it is certain to have issued (3 per copy, the unconditional stores of interior strips)
// and waits with that k: later copies and all stores stay in flight.
//
// Compute.  Wavefront s owns output columns 32s..32s+31 of the strip.  Per kernel row i:
//     out^T[q, p] += T_i^T[q, k] X^T[k, p+i-(R-1)]
// as three v_mfma_f32_32x32x16 over the 48-key window of the sub-tile.  A operand = Toeplitz fragment (16 bytes
// of the channel's zero-padded weight row, kept in registers while the channel stays the same), B operand = 16
// contiguous bytes of one staged row per lane.
// A lane ends up with 2 x 8 consecutive keys of one query row and stores them straight to global memory (the 4
// wavefronts of a workgroup complete each row's 256-byte segment; L2 merges the 32-byte pieces).
template <typename T, int R, int S, bool SCALED>
__global__ __launch_bounds__(M_NT, MTA_CONV_WAVES_PER_SIMD) void conv2d_mfma(
    const T *__restrict__ x, const T *__restrict__ w, T *__restrict__ y, int C, int H, int W, int causal, float in_scale,
    int tiles_n, int ipp, int64_t total, int64_t per_xcd, int nw, int mirror)
{
    using G = mfma_geom<R, S>;
    constexpr int LD = G::LD, VEC = 8;
    constexpr int VPR = G::TW / VEC;                        // data vectors per staged row (18)
    constexpr int SPR = LD / VEC;                           // 16-byte slots per LDS row (19)
    constexpr int SLOTS = G::ROWS * SPR;
    constexpr int STAGE_IT = (SLOTS + M_NT - 1) / M_NT;     // copies per lane per strip
    static_assert(SPR == VPR + 1, "one padding slot per row");
    constexpr int NCH = 3;                                  // 16-key chunks per 32-output window
    // weights of the current channel, each kernel row zero-padded on both sides so that the
    // Toeplitz fragments can be gathered without range checks
    constexpr int WZ_OFF = G::SHIFT + 32, WZ_LD = WZ_OFF + 16 * NCH;
    constexpr int WZ_IT = (R * WZ_LD + M_NT - 1) / M_NT;
    constexpr int BUF = STAGE_IT * M_NT * VEC;  // elements per LDS strip buffer
    __shared__ __align__(16) T tiles[M_RING * BUF];
    __shared__ __align__(16) T wz[WZ_IT * M_NT];  // R rows of WZ_LD, rounded up to whole passes of the workgroup

    // XCD-aware split: workgroup ids are dealt round-robin to the 8 XCDs; each XCD gets one
    // contiguous chunk of the item list (whole planes, mostly), so halo re-reads stay in its L2.
    const int64_t c0 = (int64_t)(blockIdx.x & 7) * per_xcd;
    const int64_t c1 = (c0 + per_xcd < total) ? c0 + per_xcd : total;
    // within the chunk the items are dealt round-robin to the XCD's workgroups, so that at any moment
    // they sweep the same few hundred rows together (DRAM pages are consumed whole, as by a linear copy)
    const int64_t first = c0 + (int64_t)(blockIdx.x >> 3);
    if (c0 >= total || first >= c1) return;
    const int n_items = (int)((c1 - first + nw - 1) / nw);  // items of this workgroup

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ln = lane & 31, kg = lane >> 5;
    const unsigned tiles_lds = (unsigned)(uintptr_t)(lds_void_t *)tiles;
    const unsigned wz_lds = (unsigned)(uintptr_t)(lds_void_t *)wz;
    // Toeplitz fragments T_i^T for this lane's accumulator row are 8 consecutive elements of the zero-padded weight
    // row i in LDS.  Accumulator register v of lane-half kg is row m = 8*(v/4) + 4*kg + v%4 of the MFMA; giving
    // that row the output column 16*(v/8) + 8*kg + v%8 makes every 8 registers of a lane 8 consecutive keys
    const int qm = 16 * (ln >> 4) + 8 * ((ln >> 2) & 1) + 4 * ((ln >> 3) & 1) + (ln & 3);
    const unsigned wsrc = wz_lds + (unsigned)(WZ_OFF + kg * 8 - G::SHIFT - qm) * sizeof(T);  // tap j = k - SHIFT - q
    const unsigned xsrc = (unsigned)(ln * LD + wave * 32 + kg * 8) * sizeof(T);               // + slot base

    // per-lane geometry of the staging copies, fixed for the whole kernel: slot it*256+tid is row srow,
    // vector svc of the strip; padding slots and slots past the strip re-read a neighbouring valid vector
    int goff[STAGE_IT];
#pragma unroll
    for (int it = 0; it < STAGE_IT; ++it) {
        const int slot = it * M_NT + tid;
        int rr = slot / SPR, vc = slot % SPR;
        if (rr >= G::ROWS) { rr = 0; vc = 0; }
        if (vc >= VPR) vc = VPR - 1;
        goff[it] = rr * W + vc * VEC;
    }

    // a strip is `interior` when its whole halo lies inside the tensor and on or below the diagonal
    auto is_interior = [&](int p0_, int q0_) {
        const int h0 = p0_ - (R - 1), k0 = q0_ - G::HL;
        return h0 >= 0 && p0_ + M_TM <= H && k0 >= 0 && k0 + G::TW <= W && (!causal || k0 + G::TW - 1 <= h0);
    };
    const auto is_above = [&](int tm_, int tn_) { return causal && tn_ * M_TN > tm_ * M_TM + M_TM - 1; };
    // asynchronous copy of a strip into ring slot `rs`: STAGE_IT vector-memory instructions
    auto prefetch = [&](int64_t plane_, int p0_, int q0_, int rs) {
        const T *xp_ = x + plane_ * (int64_t)H * W;
        T *dst = tiles + rs * BUF + wave * 64 * VEC;
        if (is_interior(p0_, q0_)) {
            const T *base = xp_ + (int64_t)(p0_ - (R - 1)) * W + (q0_ - G::HL);
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it)
                __builtin_amdgcn_global_load_lds((glb_void_t *)(base + goff[it]), (lds_void_t *)(dst + it * M_NT * VEC), 16, 0, 0);
        } else {  // clamped addresses: what the out-of-range slots receive is replaced before it is used
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * M_NT + tid;
                int h = p0_ - (R - 1) + slot / SPR, col = q0_ - G::HL + (slot % SPR) * VEC;
                h = h < 0 ? 0 : (h > H - 1 ? H - 1 : h);
                col = col < 0 ? 0 : (col > W - VEC ? W - VEC : col);
                __builtin_amdgcn_global_load_lds((glb_void_t *)(xp_ + (int64_t)h * W + col),
                                                 (lds_void_t *)(dst + it * M_NT * VEC), 16, 0, 0);
            }
        }
    };

    // the item whose copy is issued next (RING-1 items ahead of the one being computed)
    int64_t pf_plane = first / ipp;
    int pf_t = (int)(first % ipp);
    int pf_left = n_items;  // copies still to issue
    auto issue_next = [&](int rs) -> int {  // returns the number of vector-memory instructions issued (all lanes alike)
        if (pf_left <= 0) return 0;
        int tm_, tn_;
        decode_item(pf_t, tiles_n, mirror, tm_, tn_);
        const bool skip = is_above(tm_, tn_);  // nothing is read for a strip wholly above the diagonal
        if (!skip) prefetch(pf_plane, tm_ * M_TM, tn_ * M_TN, rs);
        --pf_left;
        pf_t += nw;
        pf_plane += (unsigned)pf_t / (unsigned)ipp;
        pf_t = (int)((unsigned)pf_t % (unsigned)ipp);
        return skip ? 0 : STAGE_IT;
    };
    // the item being computed
    int64_t plane = pf_plane;
    int t_item = pf_t;

    // vector-memory instructions certainly issued k iterations ago (index 0 = the current iteration): vb[k] = by
    // that iteration's copy, va[k] = after the copy (stores)
    int vb[M_RING], va[M_RING];
#pragma unroll
    for (int k = 0; k < M_RING; ++k) vb[k] = va[k] = 0;
#pragma unroll
    for (int k = M_RING - 2; k >= 0; --k) vb[k] = issue_next(M_RING - 2 - k);  // strips 0 .. RING-2 -> slots 0 .. RING-2

    int cur_channel = -1;
    u32x4 tz[R][NCH];  // Toeplitz fragments of the current channel
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) tz[i][ch] = u32x4{0u, 0u, 0u, 0u};
    const bool fill_full = H % M_TN == 0;  // mirror images of whole 128x128 blocks lie inside the (square) tensor
    int rs = 0;                            // ring slot of the current strip
    for (int n = 0; n < n_items; ++n) {
        int tm, tn;
        decode_item(t_item, tiles_n, mirror, tm, tn);
        const int p0 = tm * M_TM, q0 = tn * M_TN;
        T *yp = y + plane * (int64_t)H * W;
        const int channel = (int)(plane % C);
        const bool above = is_above(tm, tn);  // wholly above the diagonal (only reachable when !mirror)
        const bool interior = is_interior(p0, q0);
        const int h0 = p0 - (R - 1), k0 = q0 - G::HL;
        const unsigned tile_lds = tiles_lds + (unsigned)(rs * BUF) * sizeof(T);

#pragma unroll
        for (int k = M_RING - 1; k >= 1; --k) { vb[k] = vb[k - 1]; va[k] = va[k - 1]; }
        vb[0] = va[0] = 0;
        // this lane's share of the current strip's copy (issued RING-1 iterations ago) has landed: everything
        // issued after it may stay outstanding
        {
            int keep = va[M_RING - 1];
#pragma unroll
            for (int k = 1; k < M_RING - 1; ++k) keep += vb[k] + va[k];
            vm_wait(keep);
        }
        // ... and everybody else's; the previous strip's matrix products (LDS reads of its slot) are complete
        lds_barrier();

        // refill the slot the previous strip has just released
        vb[0] = issue_next(rs == 0 ? M_RING - 1 : rs - 1);

        // advance to the next item now (the rest of the iteration uses p0, q0, yp, channel)
        {
            t_item += nw;
            plane += (unsigned)t_item / (unsigned)ipp;
            t_item = (int)((unsigned)t_item % (unsigned)ipp);
        }
        rs = rs == M_RING - 1 ? 0 : rs + 1;

        if (above) {
            zero_fill_strip<T, false>(yp, H, W, p0, q0, tid);
            continue;
        }
        const bool new_channel = channel != cur_channel;
        if (new_channel) {
            // weights of the new channel -> wz.  All loads first, so that their latencies overlap; every lane
            // consumes every value it loaded (nothing stays pending for the compiler to wait for later).  The wait
            // for these loads drains the copies in flight too: once per channel.
            cur_channel = channel;
            T wv[WZ_IT];
#pragma unroll
            for (int k = 0; k < WZ_IT; ++k) {
                const int e = k * M_NT + tid, i = e / WZ_LD, j = e % WZ_LD - WZ_OFF;
                const bool ok = e < R * WZ_LD && j >= 0 && j < S;
                wv[k] = w[channel * R * S + (ok ? i * S + j : 0)];
            }
#pragma unroll
            for (int k = 0; k < WZ_IT; ++k) {
                const int e = k * M_NT + tid, j = e % WZ_LD - WZ_OFF;
                wz[e] = (e < R * WZ_LD && j >= 0 && j < S) ? wv[k] : from_float<T>(0.0f);
            }
        }
        if (SCALED || !interior) {
            // each lane rewrites its own slots: zeros outside the tensor and above the diagonal, scaled values
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * M_NT + tid;
                const int rr = slot / SPR, vc = slot % SPR;
                const int h = h0 + rr, col = k0 + vc * VEC;
                const bool ok = rr < G::ROWS && vc < VPR && h >= 0 && h < H && col >= 0 && col < W && !(causal && col > h);
                const bool partial = ok && causal && col + VEC - 1 > h;  // the vector that straddles the diagonal
                if (!SCALED && ok && !partial) continue;
                const unsigned addr = tile_lds + (unsigned)slot * 16u;
                u32x4 raw = {0u, 0u, 0u, 0u};
                if (ok) {
                    raw = lds_load16(addr);
                    lds_wait(raw);
                    pack16<T> v = __builtin_bit_cast(pack16<T>, raw);
#pragma unroll
                    for (int u = 0; u < VEC; ++u) {
                        if (SCALED) v.v[u] = from_float<T>(to_float(v.v[u]) * in_scale);
                        if (partial && col + u > h) v.v[u] = from_float<T>(0.0f);
                    }
                    raw = __builtin_bit_cast(u32x4, v);
                }
                lds_store16(addr, raw);
            }
        }
        if (SCALED || !interior || new_channel) lds_barrier();  // (workgroup-uniform condition)
        if (new_channel) {
            // 16 bytes at a 2-byte aligned LDS address per fragment: slow reads, once per channel
#pragma unroll
            for (int i = 0; i < R; ++i) {
#pragma unroll
                for (int ch = 0; ch < NCH; ++ch) tz[i][ch] = lds_load16(wsrc + (unsigned)(i * WZ_LD + ch * 16) * sizeof(T));
                lds_wait(tz[i][0], tz[i][1], tz[i][2]);
            }
        }

        // ---- this wavefront's 32 rows x 32 keys on 32x32x16 MFMAs, two kernel rows per batch of LDS reads ----
        const int c_sub = wave * 32;
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
        if (interior || !causal || q0 + c_sub <= p0 + M_TM - 1) {  // else: wholly above the diagonal
            const unsigned xa = tile_lds + xsrc;
#pragma unroll
            for (int i0 = 0; i0 < R; i0 += 2) {
                u32x4 xf[6];
#pragma unroll
                for (int k = 0; k < 6; ++k) {
                    const int i = i0 + k / NCH, ch = k % NCH;
                    xf[k] = i < R ? lds_load16(xa + (unsigned)(i * LD + ch * 16) * sizeof(T)) : u32x4{0u, 0u, 0u, 0u};
                }
                lds_wait(xf);
#pragma unroll
                for (int k = 0; k < 6; ++k)
                    if (i0 + k / NCH < R)
                        mma32(acc, __builtin_bit_cast(frag8<T>, tz[i0 + k / NCH][k % NCH]), __builtin_bit_cast(frag8<T>, xf[k]));
            }
        }
        // ---- lane (row ln, half kg) holds keys c_sub + 16a + 8kg .. +7 of its row: two 16-byte stores ----
        {
            const int prow = p0 + ln;
            T *yrow = yp + (int64_t)prow * W + q0 + c_sub + kg * 8;
            u32x4 o[2];
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const int q = q0 + c_sub + a * 16 + kg * 8;
#pragma unroll
                for (int u = 0; u < 4; ++u) o[a][u] = pack2<T>(acc[a * 8 + 2 * u], acc[a * 8 + 2 * u + 1]);
                if (!interior && causal && q + 7 > prow) {
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (q + 2 * u > prow) o[a][u] &= 0xffff0000u;
                        if (q + 2 * u + 1 > prow) o[a][u] &= 0x0000ffffu;
                    }
                }
            }
            if (interior) {
                store_out(yrow, o[0]);
                store_out(yrow + 16, o[1]);
                va[0] += 2;
            } else {
#pragma unroll
                for (int a = 0; a < 2; ++a)
                    if (prow < H && q0 + c_sub + a * 16 + kg * 8 < W) store_out(yrow + a * 16, o[a]);
            }
        }
        if (mirror && tn < (tm >> 2)) {  // a quarter of the 128x128 block's image above the diagonal
            if (fill_full) {
                zero_fill_strip<T, true>(yp, H, W, q0 + (tm & 3) * M_TM, (tm >> 2) * M_TN, tid);
                va[0] += M_TM * (M_TN / VEC) / M_NT;
            } else {
                zero_fill_strip<T, false>(yp, H, W, q0 + (tm & 3) * M_TM, (tm >> 2) * M_TN, tid);
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
    int nw = device_cu_count() * MTA_CONV_WG_PER_CU / 8;  // persistent workgroups per XCD
    if (nw < 1) nw = 1;
    if (per_xcd < nw) nw = (int)per_xcd;
    dim3 grid((unsigned)(nw * 8));
    if (use_scale)
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, true>), grid, dim3(M_NT), 0, st, (const T *)x, (const T *)w, (T *)y, (int)C,
                           (int)H, (int)W, causal, in_scale, tiles_n, ipp, total, per_xcd, nw, mirror);
    else
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, false>), grid, dim3(M_NT), 0, st, (const T *)x, (const T *)w, (T *)y, (int)C,
                           (int)H, (int)W, causal, in_scale, tiles_n, ipp, total, per_xcd, nw, mirror);
    return launch_status();
}

// returns 1 when no MFMA instantiation covers (R,S) -- the caller then takes the VALU path
template <typename T>
int dispatch_mfma(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R, int S,
                  int causal, float in_scale, int use_scale, hipStream_t st)
{
#define MTA_CONV_CASE(r, s)                                       \
    static_assert(mfma_geom<r, s>::fits, "window exceeds 48 keys"); \
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
