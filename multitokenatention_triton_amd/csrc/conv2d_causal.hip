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
#include "strip_common.hpp"

#include <stdlib.h>

#include <atomic>
#include <type_traits>
#include <utility>

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
    if (lds > 160 * 1024) return MTA_ERR_KERNEL_SIZE;
    if (lds > 48 * 1024) {  // per device, so set on every such launch (a cheap host-side call)
        hipError_t e = hipFuncSetAttribute((const void *)conv2d_valu<T, R_T, S_T, BWD>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
    }
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
// The output is written once and not read again by this kernel: non-temporal stores keep it from displacing the input
// rows that neighbouring strips re-read (halos) in the L2.
#define MTA_CONV_STORE(ptr, val) __builtin_nontemporal_store((val), (ptr))

constexpr int M_NW = 4;            // wavefronts per workgroup: (16-row block, 128-key half) of the workgroup's strip each
constexpr int M_WT = 64 * M_NW;    // threads per workgroup
constexpr int M_TM = 32;           // strip rows
constexpr int M_TN = 256;          // strip cols: two halves of 8 column blocks of 16
constexpr int M_HALF = M_TN / 2;   // keys per wavefront
constexpr int M_RPB = M_TN / M_TM;  // row strips per M_TN x M_TN block of the lower triangle
// persistent workgroups per CU: four where two strip buffers take a quarter of the LDS (kernels of up to 6 rows: 37 staged
// rows of 544 bytes are 1258 slots, five copy rounds, 20 KB), else three; kernels of more than 7 rows keep that many more
// Toeplitz fragments in registers and are compiled for two
template <int R> constexpr int wg_per_cu() { return R > 7 ? 2 : (R > 6 ? 3 : 4); }
static_assert(M_NW == 4 && M_TM == 32 && M_TN % M_TM == 0 && M_RPB % 2 == 0, "strip geometry");

// 16 outputs + S-1 taps (+ alignment shift) must fit the 32-key contraction of one 16x16x32 MFMA
template <int R, int S> struct mfma_geom {
    static constexpr int PADW = (S - 1) / 2;
    static constexpr int HL = (PADW + 7) & ~7;             // left halo, rounded so 16-byte loads stay aligned
    static constexpr int SHIFT = HL - PADW;                // first tap's offset inside a block's 32-key window
    static constexpr bool fits = SHIFT + 16 + S - 1 <= 32;
    static constexpr int TW = M_TN - 16 + 32;              // staged columns
    // Row stride in LDS.  A fragment read takes 16 bytes per lane from 16 consecutive rows (lane group kg at byte offset
    // 16 kg); the LDS serves lanes 0-7 together with lanes 24-31 (8-15 with 16-23, ...), i.e. rows 0-7 at one offset with
    // rows 8-15 at the next: with a stride of 2 (mod 8) 16-byte slots those sixteen accesses fall on sixteen different
    // slots of the 256-byte bank line (3 (mod 8), one padding slot after the 34 of data, put rows 3 and 8 on the same one).
    static constexpr int LD = TW;
    static_assert((LD / 8) % 8 == 2, "row stride of the staged strip");
    static constexpr int ROWS = M_TM + R - 1;
    // results of the wavefronts that own key half `h` go back to LDS columns h * RES_OFF .. + M_HALF - 1, which no
    // wavefront of the other half reads as input (half 0 reads columns 0 .. M_HALF+15, half 1 columns M_HALF ..)
    static constexpr int RES_OFF = M_HALF + 16;
    static_assert(RES_OFF + M_HALF <= LD, "result columns of the second half");
};

// Position t of a work item inside its plane -> (strip row tm (M_TM rows), strip col tn (M_TN keys)).
// `tri` (causal, square, lower triangle only): the strips that touch the lower triangle, row strip by row strip from
// the top, each from the left up to the diagonal: row strip tm has tm / M_RPB + 1 of them, so M_RPB/2 * b * (b+1) items
// precede block row b.  Otherwise: all strips, row-major.
__device__ __forceinline__ void decode_item(int t, int tiles_n, int tri, int &tm, int &tn)
{
    if (tri) {
        constexpr int HB = M_RPB / 2;
        int b = (int)((sqrtf((float)t / (float)HB + 0.25f) - 0.5f));
        while (HB * (b + 1) * (b + 2) <= t) ++b;
        while (HB * b * (b + 1) > t) --b;
        const int rem = t - HB * b * (b + 1);
        tm = b * M_RPB + rem / (b + 1);
        tn = rem % (b + 1);
    } else {
        tm = t / tiles_n;
        tn = t % tiles_n;
    }
}

// +0 over an M_TM x M_TN region, all threads of the workgroup.  FULL: the region lies inside the tensor; the stores are
// then unconditional (exactly M_TM*M_TN/8/M_WT vector-memory instructions per lane)
template <typename T, bool FULL = false>
__device__ __forceinline__ void zero_fill_strip(T *yp, int H, int W, int p0, int q0, int tid)
{
    constexpr int VEC = 8, VPRW = M_TN / VEC, RPP = M_WT / VPRW;  // vectors per row, rows per pass
    pack16<T> z;
#pragma unroll
    for (int u = 0; u < VEC; ++u) z.v[u] = from_float<T>(0.0f);
    tid = opaque(tid);
    // thread t covers rows t/VPRW + RPP*k, vector t%VPRW: a uniform base, one 32-bit per-lane byte offset, uniform row steps
    static_assert(M_WT % VPRW == 0 && M_TM % RPP == 0, "region rows per pass");
    char *base = reinterpret_cast<char *>(yp + (int64_t)p0 * W + q0);
    const int r0 = tid / VPRW, cv = (tid % VPRW) * VEC;
    const unsigned off = (unsigned)(r0 * W + cv) * (unsigned)sizeof(T);
    const int64_t rstep = (int64_t)RPP * W * (int64_t)sizeof(T);
#pragma unroll
    for (int k = 0; k < M_TM / RPP; ++k) {
        if (FULL || (p0 + r0 + k * RPP < H && q0 + cv < W))
            MTA_CONV_STORE(reinterpret_cast<u32x4 *>(base + k * rstep + off), __builtin_bit_cast(u32x4, z));
    }
}

// Persistent four-wavefront workgroups: each walks a run of M_TM x M_TN strips dealt round-robin within its XCD's share
// of the item list.  Wavefront w owns row block w & 1 (16 rows) and key half w >> 1 (128 keys) of the strip: it issues a
// quarter of the staging copies and computes its 16 x 128 outputs.  The wavefronts meet at two barriers per strip (the
// strip has landed and the previous strip's buffer may be overwritten; the results are in LDS); latency is hidden by the
// other workgroups resident on the CU, each in its own phase (loading / matrix cores / storing) with its own two LDS
// strip buffers of (M_TM + R - 1) rows x 272 keys.
//
// Item order.  Strips are taken row strip by row strip, each from the left, so that an XCD's workgroups sweep whole
// rows of the output together, zero strips included: under the causal rule a strip wholly above the diagonal is an
// item like the others, whose workgroup stores +0 over it (no copy, no products).  Written this way - every row of the
// output completed within a short time, 512 contiguous bytes per row and strip - the tensor moves through memory a tenth
// faster than with 32 x 128 strips taken block by block and the part above the diagonal filled by workgroups of their
// own.  Odd planes are walked backwards, so that a workgroup's share alternates between the cheap strips above the
// diagonal and the others.  MTA_CAUSAL_LOWER_ONLY on a square tensor enumerates the strips that touch the lower
// triangle only.
//
// Per 16x16 output block and kernel row i:  out^T[q, p] += T_i^T[q, k] X^T[k, p+i-(R-1)], one
// v_mfma_f32_16x16x32 whose 32-key contraction window holds the 16 outputs' taps.  A operand =
// Toeplitz fragment (4 VGPRs per kernel row, kept while the channel is unchanged), B operand = 16 contiguous
// bytes of one staged row per lane.  A wavefront sustains about one such 1 KB LDS operand per 35 cycles whatever the
// addresses, against 16 cycles for the product: the products of a strip are therefore split over four wavefronts (on
// four SIMDs).  Results go back through LDS rows that are no longer needed as input (row block 0: the strip's first 16
// staged rows; row block 1: the last 16 staged rows of its window; see mfma_geom::RES_OFF for the columns); after a
// barrier wavefront w stores strip rows 8w .. 8w+7 whole, two 512-byte rows per instruction.
//
// Staging.  A strip whose halo lies wholly inside the tensor and on or below the diagonal (the common case, decided per
// workgroup) is copied global -> LDS by global_load_lds_dwordx4: no registers, no masks, no LDS store instructions.
// The LDS row stride is 34 16-byte slots (see mfma_geom::LD), and thread t of copy round `it` owns slot it*256+t.  Any
// other strip is copied slot by slot under a predicate - a slot inside the plane and on or below the diagonal is
// copied, any other is written as zeros while the buffer waits for its data - and after landing only the one vector
// per row that straddles the diagonal is masked in LDS.  Nothing is read from outside the tensor.
//
// Kernel rows.  The channel's R*S taps are copied global -> LDS the same way, one strip ahead, as the dwords that hold
// them (from the 4-byte aligned address at or below the first tap: such a dword holds at least one tap, so it lies in
// mapped memory); the copy is older than the strip's, so the wait for the strip covers it, and no register carries a
// value that is still in flight.  The Toeplitz fragments are gathered from there when the channel changes.
//
// SCALED: every strip is staged through registers, where x*in_scale is rounded to the I/O dtype before it
// reaches LDS (what a separate elementwise scale pass would have produced).
//
// BWD: the gradient with respect to the input (see conv2d_valu): kernel rows reversed in both axes, the R-1 halo rows
// below the strip instead of above it.  Key sizes are odd here, so the key halos are the same on both sides.
template <typename T, int R, int S, bool SCALED, bool BWD>
__global__ __launch_bounds__(M_WT, wg_per_cu<R>()) void conv2d_mfma(
    const T *__restrict__ x, const T *__restrict__ w, T *__restrict__ y, int C, int H, int W, int causal, float in_scale,
    int tiles_n, int ipp, int64_t total, int64_t per_xcd, int nw, int tri)
{
    using G = mfma_geom<R, S>;
    static_assert(!BWD || (S % 2 == 1 && !SCALED), "the backward instance assumes symmetric key halos and no scale");
    static_assert(sizeof(T) == 2, "16-bit data");
    constexpr int TOP = BWD ? 0 : R - 1;                    // halo rows above the strip (the others lie below it)
    constexpr int LD = G::LD, VEC = 8;
    constexpr int VPR = G::TW / VEC;                        // data vectors per staged row (34)
    constexpr int SPR = LD / VEC;                           // 16-byte slots per LDS row (35)
    constexpr int SLOTS = G::ROWS * SPR;
    constexpr int STAGE_IT = (SLOTS + M_WT - 1) / M_WT;     // copies per strip and lane (the last round may be partial)
    static_assert(SPR == VPR, "no padding slots");
    // the channel's kernel as it lies in memory (see above) travels with its strip: behind the strip's last slot
    constexpr int WRAW_DW = (R * S + 2) / 2;                 // dwords that cover R*S taps starting in either half of the first
    constexpr int WRAW_IT = (WRAW_DW + 63) / 64;
    constexpr int WRAW_SLOT = (SLOTS + 3) & ~3;              // (64-byte aligned)
    constexpr int NEED_SLOTS = WRAW_SLOT + WRAW_IT * 16;     // (a copy instruction of the kernel rows covers 16 slots)
    constexpr int BUF_SLOTS = NEED_SLOTS > STAGE_IT * M_WT ? (NEED_SLOTS + 3) / 4 * 4 : STAGE_IT * M_WT;
    constexpr int BUF = BUF_SLOTS * VEC;                     // elements per LDS strip buffer
    __shared__ __align__(16) T tiles[2 * BUF];               // double buffer: strip n is computed while strip n+1 lands
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
    const int rb0 = (wave & 1) * 16;         // first strip row of this wavefront's row block
    const int ch = wave >> 1;                // its key half
    frag8<T> tz[R];
    int cur_channel = -1;
    const bool reflect = causal != 0 && !tri;  // odd planes backwards

    // per-thread geometry of the staging copies, fixed for the whole kernel: slot it*M_WT+tid is row srow,
    // vector svc of the strip; padding slots re-read a neighbouring valid vector
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
    // (a plane is named by the offset of its first element, `pbase`: kept up to date by additions, no 64-bit divisions)
    // 0: a strip to convolve, 1: wholly above the diagonal, +0 to be stored, 2: wholly above it, nothing to do
    auto kind_of = [&](int p0_, int q0_) { return (causal && q0_ > p0_ + M_TM - 1) ? (causal == 2 ? 2 : 1) : 0; };
    // Asynchronous copy of a strip into LDS buffer `buf` (this wavefront's quarter of the slots).  Interior strip: every
    // slot is copied.  Any other strip: a slot is copied only if it lies inside the plane and on or below the diagonal;
    // the others - what lies outside the plane (borders), above the diagonal (which is then not read from memory at
    // all), and the padding slots - are written as zeros right here, while the buffer is still waiting for its data.
    // What remains to be done once the copy has landed is the one vector of a row that straddles the diagonal.
    auto slot_valid = [&](int slot, int h0_, int k0_) {
        const int rr = slot / SPR, vc = slot % SPR;
        const int h = h0_ + rr, col = k0_ + vc * VEC;
        return rr < G::ROWS && vc < VPR && h >= 0 && h < H && col >= 0 && col < W && !(causal && col > h);
    };
    auto prefetch = [&](int64_t pbase_, int p0_, int q0_, T *buf, bool interior_) {
        const char *base = reinterpret_cast<const char *>(x) +
                           (pbase_ + (int64_t)(p0_ - TOP) * W + (q0_ - G::HL)) * (int64_t)sizeof(T);
        if (interior_) {
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it)
                if ((it + 1) * M_WT <= SLOTS || it * M_WT + tid < SLOTS)
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(base + goff[it]),
                                                     (lds_void_t *)(buf + (it * M_WT + wave * 64) * VEC), 16, 0, 0);
        } else {
            const int tid_ = opaque(tid);
            const int h0_ = p0_ - TOP, k0_ = q0_ - G::HL;
            const unsigned buf_lds = (unsigned)(uintptr_t)(lds_void_t *)buf;
            const u32x4 zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * M_WT + tid_;
                if (slot_valid(slot, h0_, k0_))
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(base + goff[it]),
                                                     (lds_void_t *)(buf + (it * M_WT + wave * 64) * VEC), 16, 0, 0);
                else if (slot < SLOTS)
                    lds_store16(buf_lds + (unsigned)slot * 16u, zero4);
            }
        }
    };
    // asynchronous copy of a channel's kernel into the spare slots of strip buffer `par` (first wavefront); the taps start
    // wshift(channel) 16-bit elements into them
    auto wshift = [&](int channel_) { return (int)((reinterpret_cast<uintptr_t>(w + (int64_t)channel_ * (R * S)) >> 1) & 1u); };
    auto fetch_weights = [&](int channel_, int par) {
        if (wave != 0) return;
        const uintptr_t a0 = reinterpret_cast<uintptr_t>(w + (int64_t)channel_ * (R * S));
        const char *base = reinterpret_cast<const char *>(a0 & ~(uintptr_t)3);
        const int ndw = ((int)((a0 >> 1) & 1u) + R * S + 1) / 2;  // dwords that hold a tap (at most WRAW_DW)
#pragma unroll
        for (int k = 0; k < WRAW_IT; ++k)
            if (k * 64 + lane < ndw)
                __builtin_amdgcn_global_load_lds((glb_void_t *)(base + (k * 64 + lane) * 4),
                                                 (lds_void_t *)(tiles + par * BUF + (WRAW_SLOT + k * 16) * VEC), 4, 0, 0);
    };
    // current and next work item: position inside the plane, plane (as element offset, and its parity) and channel
    int t_nx;
    int64_t pbase_nx;
    int chan_nx, podd_nx;
    {
        const int64_t plane0 = first / ipp;
        t_nx = (int)(first - plane0 * ipp);
        pbase_nx = plane0 * HW;
        chan_nx = (int)(plane0 % C);
        podd_nx = (int)(plane0 & 1);
    }
    int tm, tn;
    decode_item((reflect && podd_nx) ? ipp - 1 - t_nx : t_nx, tiles_n, tri, tm, tn);
    if (kind_of(tm * M_TM, tn * M_TN) == 0) {
        fetch_weights(chan_nx, 0);
        if (!SCALED) prefetch(pbase_nx, tm * M_TM, tn * M_TN, tiles, is_interior(tm * M_TM, tn * M_TN));
    }

    constexpr int ST = 16 * (M_HALF / VEC) / 64;  // stores per strip and lane (a wavefront's 16 x 128 outputs) ...
    static_assert(ST == M_TM * (M_TN / VEC) / M_WT, "... and per zero strip");
    int younger = -1;                      // stores certainly issued after the copy in flight (-1: unknown)
    int parity = 0;
    for (int item = 0; item < n_items; ++item, parity ^= 1) {
        T *tile = tiles + parity * BUF;
        T *other = tiles + (parity ^ 1) * BUF;
        const int p0 = tm * M_TM, q0 = tn * M_TN;
        const int64_t pbase = pbase_nx;
        const T *xp = x + pbase;
        T *yp = y + pbase;
        const int channel = chan_nx;
        const int kind = kind_of(p0, q0);
        const bool interior = kind == 0 && is_interior(p0, q0);
        const int h0 = p0 - TOP, k0 = q0 - G::HL;
        // the strip's outputs all lie inside the tensor: its stores are unconditional then, and their number is known
        const bool full_out = p0 + M_TM <= H && q0 + M_TN <= W;
        // (opaque: the addresses derived from it are then formed where they are used instead of being kept, dozens of
        // them, in registers across the loop)
        const unsigned tile_lds = (unsigned)opaque((int)(unsigned)(uintptr_t)(lds_void_t *)tile);

        // This wavefront's part of the strip's copy (if any) and of its kernel rows has landed.  Vector-memory operations
        // complete in issue order, and the only ones this wavefront issued after that copy are the previous strip's
        // stores: when their number is known exactly (`younger`), they may stay in flight.
        if (younger == ST) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(ST) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
        younger = 0;

        if (!SCALED && kind == 0 && !interior && causal && k0 + G::TW - 1 > h0) {
            // the copy has landed: in the one vector of a row that straddles the diagonal, zero the keys beyond it (all
            // reads first, one wait, then the writes)
            const int tid_ = opaque(tid);
            constexpr int GRP = 3;  // slots per batch (each holds four registers between its read and its write)
#pragma unroll
            for (int g0 = 0; g0 < STAGE_IT; g0 += GRP) {
                u32x4 raw[GRP];
#pragma unroll
                for (int it = g0; it < g0 + GRP && it < STAGE_IT; ++it) {
                    const int slot = it * M_WT + tid_;
                    const int h = h0 + slot / SPR, col = k0 + (slot % SPR) * VEC;
                    if (slot_valid(slot, h0, k0) && col + VEC - 1 > h) raw[it - g0] = lds_load16(tile_lds + (unsigned)slot * 16u);
                }
                lds_wait();
#pragma unroll
                for (int it = g0; it < g0 + GRP && it < STAGE_IT; ++it) {
                    const int slot = it * M_WT + tid_;
                    const int h = h0 + slot / SPR, col = k0 + (slot % SPR) * VEC;
                    if (slot_valid(slot, h0, k0) && col + VEC - 1 > h) {
                        asm volatile("" : "+v"(raw[it - g0]));  // (the value is defined from the wait above on)
                        V16 v = __builtin_bit_cast(V16, raw[it - g0]);
#pragma unroll
                        for (int u = 0; u < VEC; ++u)
                            if (col + u > h) v.v[u] = from_float<T>(0.0f);
                        lds_store16(tile_lds + (unsigned)slot * 16u, __builtin_bit_cast(u32x4, v));
                    }
                }
            }
        } else if (SCALED && kind == 0) {
            // through registers.  Loads are unconditional and issued back to back (an invalid
            // slot re-reads a valid address); what a slot really holds is decided on the way to LDS
            V16 stage[STAGE_IT];
            const int tid_ = opaque(tid);
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * M_WT + tid_;
                const int rr = slot / SPR, vc = slot % SPR;
                const int h = h0 + rr, col = k0 + vc * VEC;
                stage[it] = *reinterpret_cast<const V16 *>(xp + (slot_valid(slot, h0, k0) ? (int64_t)h * W + col : 0));
            }
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * M_WT + tid_;
                const int rr = slot / SPR, vc = slot % SPR;
                const int h = h0 + rr, col = k0 + vc * VEC;
                const bool ok = slot_valid(slot, h0, k0);
                V16 v = stage[it];
#pragma unroll
                for (int u = 0; u < VEC; ++u) v.v[u] = from_float<T>(to_float(v.v[u]) * in_scale);
                if (!ok) {
#pragma unroll
                    for (int u = 0; u < VEC; ++u) v.v[u] = from_float<T>(0.0f);
                } else if (causal && col + VEC - 1 > h) {  // the one vector of a row that straddles the diagonal
#pragma unroll
                    for (int u = 0; u < VEC; ++u)
                        if (col + u > h) v.v[u] = from_float<T>(0.0f);
                }
                if (slot < SLOTS) lds_store16(tile_lds + (unsigned)slot * 16u, __builtin_bit_cast(u32x4, v));
            }
        }
        lds_wait();    // this wavefront's LDS stores above are complete
        wg_barrier();  // the strip and its kernel rows are in LDS; every wavefront is done with the previous strip

        if (kind == 0 && channel != cur_channel) {  // Toeplitz fragments T_i^T for this lane's accumulator row
            cur_channel = channel;
            const int lane_ = opaque(lane);
            const int ln_ = lane_ & 15, kg_ = lane_ >> 4;
            const unsigned wa = tile_lds + (unsigned)(WRAW_SLOT * 16) + 2u * (unsigned)wshift(channel);
#pragma unroll
            for (int i = 0; i < R; ++i) {  // row m = ln, slots k = 8*kg + t, tap j = k-SHIFT-m
                unsigned tap[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const int j = kg_ * 8 + t - G::SHIFT - ln_;
                    const bool ok = j >= 0 && j < S;
                    const int idx = BWD ? (R - 1 - i) * S + (S - 1 - j) : i * S + j;
                    tap[t] = lds_load_u16(wa + 2u * (unsigned)(ok ? idx : 0));
                }
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(tap[0]), "+v"(tap[1]), "+v"(tap[2]), "+v"(tap[3]), "+v"(tap[4]), "+v"(tap[5]), "+v"(tap[6]), "+v"(tap[7])
                             :
                             : "memory");
                unsigned pk[4];
#pragma unroll
                for (int t = 0; t < 8; t += 2) {
                    const int j = kg_ * 8 + t - G::SHIFT - ln_;
                    const unsigned lo = (j >= 0 && j < S) ? tap[t] : 0u, hi = (j + 1 >= 0 && j + 1 < S) ? tap[t + 1] : 0u;
                    pk[t / 2] = lo | (hi << 16);
                }
                tz[i] = __builtin_bit_cast(frag8<T>, u32x4{pk[0], pk[1], pk[2], pk[3]});
            }
        }

        // put the next strip's copy in flight (into the buffer the previous iteration has just released)
        if (item + 1 < n_items) {
            t_nx += step;
            while (t_nx >= ipp) {  // (at most once, unless a plane holds fewer items than there are workgroups)
                t_nx -= ipp;
                pbase_nx += HW;
                chan_nx = chan_nx + 1 == C ? 0 : chan_nx + 1;
                podd_nx ^= 1;
            }
            decode_item((reflect && podd_nx) ? ipp - 1 - t_nx : t_nx, tiles_n, tri, tm, tn);
            if (kind_of(tm * M_TM, tn * M_TN) == 0) {
                fetch_weights(chan_nx, parity ^ 1);  // (before the copy: the loop-top wait counts what is younger than the copy)
                if (!SCALED) prefetch(pbase_nx, tm * M_TM, tn * M_TN, other, is_interior(tm * M_TM, tn * M_TN));
            }
        }
        if (kind != 0) {
            if (kind == 1) {
                if (full_out) {
                    zero_fill_strip<T, true>(yp, H, W, p0, q0, tid);
                    younger = ST;
                } else {
                    zero_fill_strip<T>(yp, H, W, p0, q0, tid);
                    younger = -1;
                }
            }
            continue;
        }

        // ---- this wavefront's 16 x 128 outputs: 8 column blocks of 16x16 on 16x16x32 MFMAs (one per kernel row: the
        // 32-key window holds the 16 outputs' taps).  Lane (row ln, group kg) holds keys 4*kg..4*kg+3 of each block.
        const int res0 = rb0 == 0 ? 0 : rb0 + R - 1;                 // staged rows that receive the results
        const int qw = q0 + ch * M_HALF;                             // first key of this wavefront's outputs
        {
            constexpr int NCB = M_HALF / 16;
            f32x4 acc[NCB];
            const unsigned xa = tile_lds + (unsigned)((rb0 + ln) * LD + ch * M_HALF + kg * 8) * sizeof(T);
            // Column blocks in pairs, kernel row by kernel row (two independent accumulation chains).  A wavefront issues
            // in order, so a run of LDS reads followed by a run of products leaves the matrix cores idle during the first
            // and the LDS idle during the second: the operand of product n + NLD is read right before product n is issued,
            // into a ring of registers, and a product waits only for its own operand (LDS operations complete in order:
            // exactly the reads issued after it may be outstanding).  Source order is pinned (the scheduler would regroup
            // reads and products).  Blocks above the diagonal are computed like the others and masked below.
            // (operands in flight: 12, or 6 where four workgroups per CU leave a wavefront 128 registers)
            constexpr int NLD_MAX = wg_per_cu<R>() >= 4 ? 6 : 12;
            constexpr int NPROD = NCB * R, NLD = 2 * R < NLD_MAX ? 2 * R : NLD_MAX, NSLOT = NLD + 1;
            static_assert(NLD <= 15 && NPROD > NLD, "lgkmcnt field; pipeline deeper than the work");
            u32x4 ring[NSLOT];
            // product n: column block 2*(n / 2R) + n % 2, kernel row (n % 2R) / 2
            auto issue = [&](auto ic) __attribute__((always_inline)) {
                constexpr int n = decltype(ic)::value;
                constexpr int cb = 2 * (n / (2 * R)) + n % 2, i = (n % (2 * R)) / 2;
                ring[n % NSLOT] = lds_load16_at(xa, (int)((i * LD + cb * 16) * sizeof(T)));
            };
            static_for<NLD>(issue);
            static_for<NPROD>([&](auto ic) __attribute__((always_inline)) {
                constexpr int n = decltype(ic)::value;
                constexpr int cb = 2 * (n / (2 * R)) + n % 2, i = (n % (2 * R)) / 2;
                if constexpr (n + NLD < NPROD) issue(std::integral_constant<int, n + NLD>{});
                constexpr int newer = (n + NLD < NPROD ? n + NLD : NPROD - 1) - n;
                asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(ring[n % NSLOT]) : "n"(newer) : "memory");
                if constexpr (i == 0) acc[cb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                mma16(acc[cb], tz[i], __builtin_bit_cast(frag8<T>, ring[n % NSLOT]));
                __builtin_amdgcn_sched_barrier(0);
            });
            // results into the staged rows res0.. (read by this wavefront only, and no longer needed by it)
            const int prow = p0 + rb0 + ln;
            const unsigned ra = tile_lds + (unsigned)((res0 + ln) * LD + ch * G::RES_OFF + kg * 4) * sizeof(T);
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const int q = qw + cb * 16 + kg * 4;
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
        // ---- coalesced stores.  The four wavefronts' results lie in LDS; after a barrier wavefront w stores rows 8w .. 8w+7
        // of the strip in full, two 512-byte rows per instruction (the halves of a row come from two wavefronts' results):
        // whole rows in one instruction move a few percent faster through memory than 256-byte pieces of four rows ----
        lds_wait();
        wg_barrier();
        {
            // (uniform row base + one 32-bit per-lane byte offset: no 64-bit address arithmetic per store)
            const int sr0 = wave * 8;                                   // first strip row this wavefront stores
            const int sres = sr0 < 16 ? sr0 : sr0 + R - 1;              // ... and where its results lie (see res0)
            char *ybase = reinterpret_cast<char *>(yp + (int64_t)(p0 + sr0) * W + q0);
            const int lane_o = opaque(lane);  // (row offsets formed here, not kept in registers across the loop)
            const int r_l = lane_o >> 5, hf = (lane_o >> 4) & 1, cv = (lane_o & 15) * VEC;
            const unsigned yoff = (unsigned)(r_l * W + hf * M_HALF + cv) * (unsigned)sizeof(T);
            const int64_t ystep = (int64_t)2 * W * (int64_t)sizeof(T);
            static_assert(ST == 4, "four row pairs per wavefront");
            u32x4 v[4];
            const unsigned va = tile_lds + (unsigned)((sres + r_l) * LD + hf * G::RES_OFF + cv) * sizeof(T);
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = lds_load16_at(va, (int)(k * 2 * LD * sizeof(T)));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : : "memory");
            if (full_out) {  // unconditional: exactly ST vector-memory instructions
#pragma unroll
                for (int k = 0; k < 4; ++k) MTA_CONV_STORE(reinterpret_cast<u32x4 *>(ybase + k * ystep + yoff), v[k]);
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int r = k * 2 + r_l;
                    if (p0 + sr0 + r < H && q0 + hf * M_HALF + cv < W) MTA_CONV_STORE(reinterpret_cast<u32x4 *>(ybase + k * ystep + yoff), v[k]);
                }
            }
            younger = full_out ? ST : -1;
        }
    }
}

template <typename T, int R, int S, bool BWD>
int launch_mfma(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int causal,
                float in_scale, int use_scale, hipStream_t st)
{
    const int64_t tiles_m = (H + M_TM - 1) / M_TM, tiles_n = (W + M_TN - 1) / M_TN;
    // causal, square, and the caller wants nothing written above the diagonal: only the strips that touch the lower triangle
    const int tri = (causal == 2 && H == W) ? 1 : 0;
    const int64_t nbf = tiles_m / M_RPB, kl = tiles_m % M_RPB;
    const int64_t ipp64 = tri ? (M_RPB / 2) * nbf * (nbf + 1) + kl * (nbf + 1) : tiles_m * tiles_n;
    if (ipp64 > (1 << 24)) return MTA_ERR_SHAPE;  // decode_item's float sqrt is exact well beyond this
    const int ipp = (int)ipp64;
    const int64_t total = N * C * ipp64;
    const int64_t per_xcd = (total + 7) / 8;
    // persistent workgroups per XCD: as many as fit when only the strips of the lower triangle are walked; with the zero
    // strips in the list three per CU move the tensor fastest (measured at (2,16,2048,2048): 84 us against 85.5 with four)
    const int wgs = tri ? wg_per_cu<R>() : (wg_per_cu<R>() < 3 ? wg_per_cu<R>() : 3);
    int nw = device_cu_count() * wgs / 8;
    if (nw < 1) nw = 1;
    if (per_xcd < nw) nw = (int)per_xcd;
    dim3 grid((unsigned)(nw * 8));
    if constexpr (BWD) {
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, false, true>), grid, dim3(M_WT), 0, st, (const T *)x, (const T *)w, (T *)y,
                           (int)C, (int)H, (int)W, causal, in_scale, (int)tiles_n, ipp, total, per_xcd, nw, tri);
    } else if (use_scale) {
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, true, false>), grid, dim3(M_WT), 0, st, (const T *)x, (const T *)w, (T *)y,
                           (int)C, (int)H, (int)W, causal, in_scale, (int)tiles_n, ipp, total, per_xcd, nw, tri);
    } else {
        hipLaunchKernelGGL((conv2d_mfma<T, R, S, false, false>), grid, dim3(M_WT), 0, st, (const T *)x, (const T *)w, (T *)y,
                           (int)C, (int)H, (int)W, causal, in_scale, (int)tiles_n, ipp, total, per_xcd, nw, tri);
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
    MTA_CONV_CASE(11, 15)
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
