// Depthwise causal conv, then dense mixing of a group of 16 heads, in one pass, both on the matrix cores (16-bit data):
//
//   c[n,h,p,q] = round( sum_{i<R,j<S} wc[h,i,j] * xm[n,h,p+i-(R-1), q+j-(S-1)/2] )      (xm: x, 0 where q > p)
//   y[n,o,p,q] = sum_h wm[o,h] * c[n,h,p,q]                                            (0 where q > p)
//
// What the operator-by-operator pipeline writes to memory and reads back between the two stages - c, a whole
// (N,C,H,W) tensor - stays in registers here.
//
// A workgroup of four wavefronts owns a 32 x 64 tile of positions for all 16 heads of a mixing group; wavefront w owns
// row block w & 1 (16 rows) and key half w >> 1 (32 keys = two 16 x 16 blocks).  Head by head, the tile's window
// ((32+R-1) rows x 80 keys) is copied global -> LDS asynchronously one head ahead (two buffers, one barrier per head)
// and convolved as in conv2d_mfma: per block and kernel row one v_mfma_f32_16x16x32 of a Toeplitz fragment with 16
// contiguous bytes of a staged row per lane.  The rounded results of all 16 heads stay in the lane that computed them
// (64 registers).
//
// Toeplitz fragments change with every head.  A lane's fragment of kernel row i is eight consecutive taps starting at
// an offset that depends on the lane only through e = 8*(lane/16) - lane%16, and is non-zero for S+7 values of e: the
// workgroup expands the group's kernels once into a table of those 16-byte vectors in LDS ((S+7) per head and kernel
// row), and a change of head costs R 16-byte LDS reads per lane (lanes whose fragment is zero keep their zeros).
//
// Mixing.  After the conv a lane (row p = lane%16, group kg) holds keys 4kg .. 4kg+3 of a block for all 16 heads; the
// contraction of v_mfma_f32_16x16x16 wants the heads spread over the lane groups instead.  Two exchanges between rows
// of lanes (v_permlane32_swap, v_permlane16_swap) transpose (head quad) x (key quad): afterwards lane group g holds heads
// 4g .. 4g+3 for all 16 keys of the block, and per key one product with the 16 x 16 weight gives the lane 4 output heads.
// The outputs go through LDS (swizzled, 16 KB, one output head of every lane group per round) so that the global
// stores are whole 128-byte rows.
#include "common.hpp"
#include "mfma.hpp"
#include "strip_common.hpp"

#include <stdlib.h>

#include <algorithm>
#include <vector>

namespace {
using namespace mta;

// 16 bytes of zeros in device memory: what a lane copies into a window slot that lies outside the plane or above the
// diagonal (never written)
__device__ __align__(16) unsigned int xm_zero16[4];

constexpr int X_NW = 4;            // wavefronts per workgroup
constexpr int X_WT = 64 * X_NW;    // threads per workgroup
constexpr int X_TM = 32;           // tile rows
constexpr int X_TN = 64;           // tile keys
constexpr int X_HALF = X_TN / 2;   // keys per wavefront
constexpr int X_NCB = X_HALF / 16; // 16 x 16 blocks per wavefront
constexpr int X_HG = 16;           // heads mixed together
constexpr int X_RPB = X_TN / X_TM; // tile rows per X_TN x X_TN block of the lower triangle
static_assert(X_RPB == 2 && X_NCB == 2, "tile geometry");

template <int R, int S> struct xgeom {
    static constexpr int PADW = (S - 1) / 2;
    static constexpr int HL = (PADW + 7) & ~7;   // left halo, rounded so that 16-byte copies stay aligned
    static constexpr int SHIFT = HL - PADW;      // first tap's offset inside a block's 32-key window
    static constexpr bool fits = SHIFT + 16 + S - 1 <= 32;
    static constexpr int TW = X_TN - 16 + 32;    // staged keys
    static constexpr int LD = TW;                // row stride in LDS: 10 16-byte slots, 2 (mod 8): conflict-free fragment reads
    static_assert((LD / 8) % 8 == 2, "row stride of the staged window");
    static constexpr int ROWS = X_TM + R - 1;
    static constexpr int NVEC = S + 7;           // non-zero Toeplitz vectors per head and kernel row
    static constexpr int E0 = SHIFT - 7;         // e of the first of them
};

typedef unsigned int xm_u2 __attribute__((ext_vector_type(2)));
typedef short xm_s4 __attribute__((ext_vector_type(4)));
typedef _Float16 xm_h4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4 xm_mma16(bf16_t, xm_u2 a, xm_u2 b)
{
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(xm_s4, a), __builtin_bit_cast(xm_s4, b),
                                                     f32x4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
}
__device__ __forceinline__ f32x4 xm_mma16(f16_t, xm_u2 a, xm_u2 b)
{
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(xm_h4, a), __builtin_bit_cast(xm_h4, b),
                                                 f32x4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
}

__device__ __forceinline__ void lds_store2(unsigned addr, unsigned v)
{
    asm volatile("ds_write_b16 %0, %1" : : "v"(addr), "v"(v) : "memory");
}

// Position t inside a plane group -> tile (tm, tn).  tri: the tiles that touch the lower triangle of a square plane, tile
// row by tile row, each from the left up to the diagonal (tile row tm has tm / X_RPB + 1 of them); else all, row-major.
__device__ __forceinline__ void decode_tile(int t, int tiles_n, int tri, int &tm, int &tn)
{
    if (tri) {
        int b = (int)(sqrtf((float)t + 0.25f) - 0.5f);  // X_RPB/2 * b * (b+1) = b(b+1) items precede block row b
        while ((b + 1) * (b + 2) <= t) ++b;
        while (b * (b + 1) > t) --b;
        const int rem = t - b * (b + 1);
        tm = b * X_RPB + rem / (b + 1);
        tn = rem % (b + 1);
    } else {
        tm = t / tiles_n;
        tn = t % tiles_n;
    }
}

// first item of each XCD's share of the item list (start[8]: the number of items)
struct xm_split { int64_t start[9]; };
constexpr int X_ROT = 19;  // by how many workgroups the dealing of an XCD's items is rotated from round to round

template <int R> constexpr int x_occ() { return 2; }  // persistent workgroups per CU

template <typename T, int R, int S>
__global__ __launch_bounds__(X_WT, x_occ<R>()) void conv_mix16_mfma(const T *__restrict__ x, const T *__restrict__ wc,
                                                                   const T *__restrict__ wm, T *__restrict__ y, int C, int H,
                                                                   int W, int causal, int fill_upper, int tiles_n, int ipp,
                                                                   xm_split split, int nw, int tri)
{
    using G = xgeom<R, S>;
    static_assert(sizeof(T) == 2, "16-bit data");
    constexpr int TOP = R - 1, LD = G::LD, VEC = 8, SPR = LD / VEC;
    constexpr int SLOTS = G::ROWS * SPR;
    constexpr int STAGE_IT = (SLOTS + X_WT - 1) / X_WT;
    constexpr int BUF = ((SLOTS + 3) & ~3) * VEC;                // elements per window buffer
    // The slots of a window are copied in STAGE_IT rounds: full rounds of one slot per thread, then the remainder spread
    // evenly over the four wavefronts (their first REM_W lanes), so that every wavefront issues the same number of copy
    // instructions per window - the number the waits below count.
    constexpr int REM = SLOTS - (STAGE_IT - 1) * X_WT;           // slots of the last round
    constexpr int REM_W = (REM + X_NW - 1) / X_NW;               // ... per wavefront
    static_assert(REM - (X_NW - 1) * REM_W > 0 && REM_W <= 64, "every wavefront takes part in the last round");
    constexpr int NBUF = 4;                                      // window buffers: window n + NBUF - 1 is copied during window n
    static_assert(X_HG % NBUF == 0, "a head's buffer is the same in every item");
    constexpr int TAB_VECS = X_HG * R * G::NVEC;                 // 16-byte vectors of the fragment table
    constexpr int STG_BYTES = 4 * X_TM * X_TN * (int)sizeof(T);  // output staging: 4 heads x 32 rows x 128 bytes
    constexpr int RAW_BYTES = X_HG * R * S * (int)sizeof(T);
    constexpr int NRAW = RAW_BYTES / 16;
    static_assert(RAW_BYTES % 16 == 0 && NRAW <= X_WT, "the kernels of a group are whole 16-byte vectors, one per thread");
    constexpr unsigned RAW_OFF = 16;                             // where the raw kernels lie in the staging area while the table is built
    static_assert(RAW_BYTES + 32 <= STG_BYTES, "the raw kernels and what is read around them lie in the staging area");
    constexpr int NST = 16;                                      // store instructions per wavefront and item
    static_assert((NBUF - 2) * STAGE_IT + NST <= 63, "vmcnt field");
    __shared__ __align__(16) T tiles[NBUF * BUF];
    __shared__ __align__(16) u32x4 table[TAB_VECS + 1];          // (+ one vector of zeros)
    __shared__ __align__(16) unsigned char stage[STG_BYTES];

    // XCD-aware: workgroup ids are dealt round-robin to the 8 XCDs; each XCD takes a contiguous run of the item list (of
    // about equal cost, cut by the host), and within it the items are dealt to the XCD's workgroups round by round
    // (neighbouring tiles are in flight together), each round rotated against the one before: the tiles at the diagonal,
    // which cost more, recur with the length of a tile row and would else keep falling to the same workgroups
    const int64_t c0 = split.start[blockIdx.x & 7], c1 = split.start[(blockIdx.x & 7) + 1];
    const int wg_j = (int)(blockIdx.x >> 3);
    auto item_index = [&](int k) { return c0 + (int64_t)k * nw + (wg_j + k * X_ROT) % nw; };
    const int n_rounds = (int)((c1 - c0 + nw - 1) / nw);
    if (n_rounds <= 0) return;
    const int n_items = n_rounds - 1 + (item_index(n_rounds - 1) < c1 ? 1 : 0);
    if (n_items <= 0) return;
    const int64_t first = item_index(0);
    const int groups = C / X_HG;
    const int64_t HW = (int64_t)H * W;

    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rb0 = (wave & 1) * 16, kh = wave >> 1;
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));

    // an item: tile (p0, q0) of plane group pg = (batch entry, mixing group)
    //   pbase: element offset of head 0 of the group;  kind: 0 to compute, 1 wholly above the diagonal and +0 to be
    //   stored, 2 wholly above it and nothing to do;  interior: the whole window lies inside the plane and on or below
    //   the diagonal
    auto item_of = [&](int64_t idx, int64_t &pbase_, int &g_, int &p0_, int &q0_, int &kind_, bool &interior_) {
        const int64_t pg = idx / ipp;
        const int t = (int)(idx - pg * ipp);
        const int64_t n = pg / groups;
        g_ = (int)(pg - n * groups);
        pbase_ = (n * C + (int64_t)g_ * X_HG) * HW;
        int tm, tn;
        decode_tile(t, tiles_n, tri, tm, tn);
        p0_ = tm * X_TM;
        q0_ = tn * X_TN;
        kind_ = (causal && q0_ > p0_ + X_TM - 1) ? (fill_upper ? 1 : 2) : 0;
        const int h0 = p0_ - TOP, k0 = q0_ - G::HL;
        interior_ = h0 >= 0 && h0 + G::ROWS <= H && k0 >= 0 && k0 + G::TW <= W && (!causal || k0 + G::TW - 1 <= h0);
    };

    // slot of this thread in round i (SLOTS and beyond: none), and the first slot of its wavefront in that round
    auto slot_of = [&](int i, int t) {
        if (i < STAGE_IT - 1) return i * X_WT + t;
        const int w = t >> 6, l = t & 63;
        const int lim = REM - w * REM_W < REM_W ? REM - w * REM_W : REM_W;
        return l < lim ? i * X_WT + w * REM_W + l : SLOTS;
    };
    auto wave_slot0 = [&](int i) { return i < STAGE_IT - 1 ? i * X_WT + wave * 64 : i * X_WT + wave * REM_W; };
    unsigned goff[STAGE_IT];
#pragma unroll
    for (int it = 0; it < STAGE_IT; ++it) {
        const int slot = slot_of(it, tid);
        int rr = slot / SPR, vc = slot % SPR;
        if (rr >= G::ROWS) { rr = 0; vc = 0; }
        goff[it] = (unsigned)(rr * W + vc * VEC) * (unsigned)sizeof(T);
    }

    auto slot_valid = [&](int slot, int h0, int k0) {
        const int rr = slot / SPR, vc = slot % SPR;
        const int h = h0 + rr, col = k0 + vc * VEC;
        return rr < G::ROWS && h >= 0 && h < H && col >= 0 && col < W && !(causal && col > h);
    };
    // Asynchronous copy of head `head`'s window into `buf`: STAGE_IT instructions per wavefront whatever the tile (their
    // number is what the waits count).  Interior tile: every slot is copied.  Any other tile: a slot inside the plane and
    // on or below the diagonal is copied; for any other slot the lane copies 16 bytes of zeros instead (nothing is read
    // from outside the plane or above the diagonal).  What remains to be done once the copy has landed is the one vector
    // of a row that straddles the diagonal.
    auto prefetch = [&](int64_t pbase_, int p0_, int q0_, bool interior_, int head, T *buf) {
        const int h0 = p0_ - TOP, k0 = q0_ - G::HL;
        const char *base = reinterpret_cast<const char *>(x + pbase_ + head * HW + (int64_t)h0 * W + k0);
        if (interior_) {
#pragma unroll
            for (int i = 0; i < STAGE_IT; ++i)
                if (slot_of(i, tid) < SLOTS)  // (some lanes of every wavefront: STAGE_IT instructions per wavefront)
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(base + goff[i]),
                                                     (lds_void_t *)(buf + wave_slot0(i) * VEC), 16, 0, 0);
        } else {
            const int tid_ = opaque(tid);
            const char *dummy = reinterpret_cast<const char *>(xm_zero16);
#pragma unroll
            for (int i = 0; i < STAGE_IT; ++i) {
                const int slot = slot_of(i, tid_);
                const char *src = slot_valid(slot, h0, k0) ? base + goff[i] : dummy;
                if (slot < SLOTS)
                    __builtin_amdgcn_global_load_lds((glb_void_t *)src, (lds_void_t *)(buf + wave_slot0(i) * VEC), 16, 0, 0);
            }
        }
    };

    const unsigned stage_lds = (unsigned)(uintptr_t)(lds_void_t *)stage;
    const unsigned table_lds = (unsigned)(uintptr_t)(lds_void_t *)table;
    // The table of Toeplitz vectors of mixing group g: the group's kernels as they lie in memory go to LDS (one 16-byte
    // vector per thread, into the staging area), then vector (h, i, ve) = taps j = ve + t - 7, t = 0..7, of kernel row i
    // of head h (0 outside the row).  All threads; no copy of a window may be in flight into LDS that this disturbs (none
    // is: windows and table are different arrays), and the staging area must be idle.
    auto build_table = [&](int g) {
        wg_barrier();  // every wavefront is done with the staging area and with the previous group's table
        u32x4 rawv = {0u, 0u, 0u, 0u};
        if (tid < NRAW) rawv = *reinterpret_cast<const u32x4 *>(wc + (int64_t)g * X_HG * (R * S) + tid * VEC);
        if (tid < NRAW) lds_store16(stage_lds + RAW_OFF + 16u * (unsigned)tid, rawv);
        lds_wait();
        wg_barrier();
        for (int v = tid; v < TAB_VECS; v += X_WT) {
            const int hi = v / G::NVEC, ve = v - hi * G::NVEC;
            // (taps ve-7 .. ve of the row, read where they would lie: the 16 bytes ahead of the kernels and what follows
            // them are part of the staging area, and what is read outside the row is not used)
            unsigned tap[8];
            asm volatile("ds_read_u16 %0, %8\n\tds_read_u16 %1, %8 offset:2\n\tds_read_u16 %2, %8 offset:4\n\t"
                         "ds_read_u16 %3, %8 offset:6\n\tds_read_u16 %4, %8 offset:8\n\tds_read_u16 %5, %8 offset:10\n\t"
                         "ds_read_u16 %6, %8 offset:12\n\tds_read_u16 %7, %8 offset:14\n\ts_waitcnt lgkmcnt(0)"
                         : "=&v"(tap[0]), "=&v"(tap[1]), "=&v"(tap[2]), "=&v"(tap[3]), "=&v"(tap[4]), "=&v"(tap[5]), "=&v"(tap[6]), "=&v"(tap[7])
                         : "v"(stage_lds + RAW_OFF + 2u * (unsigned)(hi * S + ve) - 14u)
                         : "memory");
            unsigned pk[4];
#pragma unroll
            for (int t = 0; t < 8; t += 2) {
                const int j = ve + t - 7;
                const unsigned lo = (j >= 0 && j < S) ? tap[t] : 0u, hi2 = (j + 1 >= 0 && j + 1 < S) ? tap[t + 1] : 0u;
                pk[t / 2] = lo | (hi2 << 16);
            }
            lds_store16(table_lds + 16u * (unsigned)v, u32x4{pk[0], pk[1], pk[2], pk[3]});
        }
        if (tid == 0) lds_store16(table_lds + 16u * (unsigned)TAB_VECS, u32x4{0u, 0u, 0u, 0u});
        lds_wait();
        wg_barrier();  // the table is complete; the staging area is free again
    };

    // this lane's Toeplitz vector: e = 8kg - ln; lanes outside the band read the vector of zeros
    const int e_rel = kg * 8 - ln - G::E0;
    const bool band = e_rel >= 0 && e_rel < G::NVEC;
    const unsigned tab_lane = table_lds + 16u * (unsigned)(band ? e_rel : 0);
    const unsigned tab_zero = table_lds + 16u * (unsigned)TAB_VECS;

    int64_t c_pbase, n_pbase;
    int c_g, c_p0, c_q0, c_kind, n_g, n_p0, n_q0, n_kind;
    bool c_interior, n_interior;
    item_of(first, c_pbase, c_g, c_p0, c_q0, c_kind, c_interior);
    bool pre_issued = false;  // the first NBUF-1 windows of `cur` were put in flight during the previous item
    int prev_st = 0;          // stores this wavefront issued at the end of the previous item (-1: unknown)
    int cur_g = -1;
    xm_u2 wf = {0u, 0u};

    for (int item = 0; item < n_items; ++item) {
        const bool has_next = item + 1 < n_items;
        n_pbase = c_pbase; n_g = c_g; n_p0 = c_p0; n_q0 = c_q0; n_kind = c_kind; n_interior = c_interior;
        if (has_next) item_of(item_index(item + 1), n_pbase, n_g, n_p0, n_q0, n_kind, n_interior);
        const bool next_ok = has_next && n_kind == 0;
        T *yg = y + c_pbase;
        const int p0 = c_p0, q0 = c_q0;
        auto advance = [&]() { c_pbase = n_pbase; c_g = n_g; c_p0 = n_p0; c_q0 = n_q0; c_kind = n_kind; c_interior = n_interior; };

        if (c_kind != 0) {  // wholly above the diagonal: +0 on request, for all 16 heads
            if (c_kind == 1) {
                const u4 z = {0u, 0u, 0u, 0u};
                const int r = tid >> 3, cv = (tid & 7) * VEC;
                if (p0 + r < H && q0 + cv < W) {
#pragma unroll
                    for (int h = 0; h < X_HG; ++h) __builtin_nontemporal_store(z, reinterpret_cast<u4 *>(yg + h * HW + (int64_t)(p0 + r) * W + q0 + cv));
                }
                prev_st = -1;
            }
            advance();
            pre_issued = false;
            continue;
        }

        if (!pre_issued) {
#pragma unroll
            for (int b = 0; b < NBUF - 1; ++b) prefetch(c_pbase, p0, q0, c_interior, b, tiles + b * BUF);
        }
        if (c_g != cur_g) {
            cur_g = c_g;
            build_table(cur_g);
            // weight fragment of the mixing: lane (output head ln, group kg) holds wm[o][4kg .. 4kg+3]
            wf = *reinterpret_cast<const xm_u2 *>(wm + (int64_t)(cur_g * X_HG + ln) * C + cur_g * X_HG + kg * 4);
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(wf) : : "memory");  // (rare: everything in flight is waited for here)
            prev_st = -1;
        }
        const int h0 = p0 - TOP, k0 = q0 - G::HL;
        const bool interior = c_interior;

        // Wait until this wavefront's copies of window w have landed, w counted from this item's head 0 (X_HG: head 0 of the
        // next item), at a point where the windows up to w + NBUF - 2 have been issued.  Vector-memory operations complete
        // in issue order: what was issued after that window's copy - the next NBUF-2 windows and, when the window was put
        // in flight during the previous item, that item's stores - may stay in flight where its number is known.
        auto wait_window = [&](auto wc) __attribute__((always_inline)) {
            constexpr int w = decltype(wc)::value;
            constexpr int in_item = w >= X_HG ? NBUF - 2 : (w + NBUF - 2 < X_HG - 1 ? w + NBUF - 2 : X_HG - 1) - w;
            constexpr int full = (NBUF - 2) * STAGE_IT, part = in_item * STAGE_IT;
            const bool with_st = pre_issued && w <= NBUF - 2;  // the window is older than the last item's stores
            if (with_st && prev_st < 0) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
            else if (with_st && prev_st > 0) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(full + NST) : "memory");
            else if (next_ok || part == full) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(full) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" : : "n"(part) : "memory");
        };
        // A window that the diagonal passes through: in the one vector of a row that straddles the diagonal, the keys
        // beyond it are zeroed in LDS once the copy has landed (each thread in the slots it copied itself): for head h+1's
        // window after head h's matrix products.
        auto needs_fix = [&](int p0_, int q0_, bool interior_) { return !interior_ && causal && q0_ - G::HL + G::TW - 1 > p0_ - TOP; };
        auto fix_window = [&](int p0_, int q0_, unsigned buf_lds) __attribute__((always_inline)) {
            const int tid_ = opaque(tid), h0_ = p0_ - TOP, k0_ = q0_ - G::HL;
            u32x4 raw[STAGE_IT];
            // (every lane reads - one that has nothing to fix, the buffer's first slot - and read and wait are one
            // statement: the values are defined wherever the compiler may touch the registers)
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = slot_of(it, tid_);
                const int hh = h0_ + slot / SPR, col = k0_ + (slot % SPR) * VEC;
                const bool need = slot_valid(slot, h0_, k0_) && col + VEC - 1 > hh;
                raw[it] = lds_load16_sync(buf_lds + (need ? (unsigned)slot * 16u : 0u));
            }
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = slot_of(it, tid_);
                const int hh = h0_ + slot / SPR, col = k0_ + (slot % SPR) * VEC;
                if (slot_valid(slot, h0_, k0_) && col + VEC - 1 > hh) {
                    pack16<T> v = __builtin_bit_cast(pack16<T>, raw[it]);
#pragma unroll
                    for (int u = 0; u < VEC; ++u)
                        if (col + u > hh) v.v[u] = from_float<T>(0.0f);
                    lds_store16(buf_lds + (unsigned)slot * 16u, __builtin_bit_cast(u32x4, v));
                }
            }
        };
        const bool fix_cur = needs_fix(p0, q0, interior), fix_nxt = next_ok && needs_fix(n_p0, n_q0, n_interior);
        if (fix_cur && !pre_issued) {  // head 0's window of an item whose windows were not in flight before: right here
            wait_window(std::integral_constant<int, 0>{});
            fix_window(p0, q0, (unsigned)(uintptr_t)(lds_void_t *)tiles);
        }

        u32x4 tz[R];
        uint32_t cres[X_HG][X_NCB][2];  // rounded conv results: head, block, (keys 4kg, 4kg+1), (keys 4kg+2, 4kg+3) of row ln

        static_for<X_HG>([&](auto hc) __attribute__((always_inline)) {
            constexpr int h = decltype(hc)::value;
            T *tile = tiles + (h % NBUF) * BUF;
            T *other = tiles + ((h + NBUF - 1) % NBUF) * BUF;  // the previous window's buffer, free after the barrier below
            const unsigned tile_lds = (unsigned)opaque((int)(unsigned)(uintptr_t)(lds_void_t *)tile);
            wait_window(hc);  // this wavefront's part of head h's window has landed
            lds_wait();
            wg_barrier();  // head h's window is in LDS; every wavefront is done with the previous window
            if constexpr (h + NBUF - 1 < X_HG) prefetch(c_pbase, p0, q0, interior, h + NBUF - 1, other);
            else if (next_ok) prefetch(n_pbase, n_p0, n_q0, n_interior, h + NBUF - 1 - X_HG, other);
            // the next window (head h+1's, or head 0's of the next item), where the diagonal passes through it
            const bool fix_w1 = h + 1 < X_HG ? fix_cur : fix_nxt;
            const unsigned w1_lds = (unsigned)opaque((int)(unsigned)(uintptr_t)(lds_void_t *)(tiles + ((h + 1) % NBUF) * BUF));

            // Toeplitz fragments of head h (addresses formed here: kept, all 16 R of them would fill the register file)
            {
                const unsigned tl = (unsigned)opaque((int)tab_lane), tzr = (unsigned)opaque((int)tab_zero);
#pragma unroll
                for (int i = 0; i < R; ++i)
                    tz[i] = lds_load16(band ? tl + (unsigned)((h * R + i) * G::NVEC * 16) : tzr);
            }

            f32x4 acc[X_NCB];
            const unsigned xa = tile_lds + (unsigned)((rb0 + ln) * LD + kh * X_HALF + kg * 8) * sizeof(T);
            constexpr int NPROD = X_NCB * R, NLD = (NPROD - 1) < 8 ? (NPROD - 1) : 8, NSLOT = NLD + 1;
            u32x4 ring[NSLOT];
            auto issue = [&](auto ic) __attribute__((always_inline)) {
                constexpr int nn = decltype(ic)::value;
                constexpr int cb = nn % X_NCB, i = nn / X_NCB;
                ring[nn % NSLOT] = lds_load16_at(xa, (int)((i * LD + cb * 16) * sizeof(T)));
            };
            static_for<NLD>(issue);
            // the fragments are older than the NLD operand reads just issued
#pragma unroll
            for (int i = 0; i < R; ++i) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(tz[i]) : "n"(NLD) : "memory");
            static_for<NPROD>([&](auto ic) __attribute__((always_inline)) {
                constexpr int nn = decltype(ic)::value;
                constexpr int cb = nn % X_NCB, i = nn / X_NCB;
                if constexpr (nn + NLD < NPROD) issue(std::integral_constant<int, nn + NLD>{});
                constexpr int newer = (nn + NLD < NPROD ? nn + NLD : NPROD - 1) - nn;
                asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(ring[nn % NSLOT]) : "n"(newer) : "memory");
                if constexpr (i == 0) acc[cb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                mma16(acc[cb], __builtin_bit_cast(frag8<T>, tz[i]), __builtin_bit_cast(frag8<T>, ring[nn % NSLOT]));
                __builtin_amdgcn_sched_barrier(0);
            });
#pragma unroll
            for (int cb = 0; cb < X_NCB; ++cb) {
                cres[h][cb][0] = pack2<T>(acc[cb][0], acc[cb][1]);
                cres[h][cb][1] = pack2<T>(acc[cb][2], acc[cb][3]);
            }
            if (fix_w1) {  // (after this head's products: the window has had their time to land)
                wait_window(std::integral_constant<int, h + 1>{});
                if constexpr (h + 1 < X_HG) fix_window(p0, q0, w1_lds);
                else fix_window(n_p0, n_q0, w1_lds);
            }
        });

        // ---- mixing ----
        const int prow = p0 + rb0 + ln;
        const bool cross = causal && q0 + X_TN - 1 > p0;  // the tile crosses the diagonal
        uint32_t outp[X_NCB][4][8];  // block, output head 4kg + v, key pairs (2u, 2u+1) of the block
#pragma unroll
        for (int cb = 0; cb < X_NCB; ++cb) {
            // (head quad) x (key quad) transposition across the four lane groups
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const int v = r >> 1, part = r & 1;
                typedef unsigned int u2 __attribute__((ext_vector_type(2)));
                u2 s;
                s = __builtin_amdgcn_permlane32_swap(cres[0 + v][cb][part], cres[8 + v][cb][part], false, false);
                cres[0 + v][cb][part] = s[0]; cres[8 + v][cb][part] = s[1];
                s = __builtin_amdgcn_permlane32_swap(cres[4 + v][cb][part], cres[12 + v][cb][part], false, false);
                cres[4 + v][cb][part] = s[0]; cres[12 + v][cb][part] = s[1];
                s = __builtin_amdgcn_permlane16_swap(cres[0 + v][cb][part], cres[4 + v][cb][part], false, false);
                cres[0 + v][cb][part] = s[0]; cres[4 + v][cb][part] = s[1];
                s = __builtin_amdgcn_permlane16_swap(cres[8 + v][cb][part], cres[12 + v][cb][part], false, false);
                cres[8 + v][cb][part] = s[0]; cres[12 + v][cb][part] = s[1];
            }
            // cres[4kq + v][cb][part] now: head 4kg + v, keys 4kq + 2 part, +1 of the block
            f32x4 macc[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int kq = j >> 2, t = j & 3, part = t >> 1;
                const unsigned sel = (t & 1) ? 0x07060302u : 0x05040100u;
                const xm_u2 col = {__builtin_amdgcn_perm(cres[4 * kq + 1][cb][part], cres[4 * kq + 0][cb][part], sel),
                                   __builtin_amdgcn_perm(cres[4 * kq + 3][cb][part], cres[4 * kq + 2][cb][part], sel)};
                macc[j] = xm_mma16(T{}, wf, col);
            }
            const int qb = q0 + kh * X_HALF + cb * 16;
#pragma unroll
            for (int v = 0; v < 4; ++v)
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    uint32_t o = pack2<T>(macc[2 * u][v], macc[2 * u + 1][v]);
                    if (cross) {
                        if (qb + 2 * u > prow) o &= 0xffff0000u;
                        if (qb + 2 * u + 1 > prow) o &= 0x0000ffffu;
                    }
                    outp[cb][v][u] = o;
                }
        }

        // ---- stores through LDS: round v carries output head 4*og + v of every lane group og ----
        // staging: [og][row 0..31][8 slots of 16 bytes], slot index XOR ((row >> 1) & 7)
        const int srow = rb0 + ln;
        const unsigned wbase = stage_lds + (unsigned)((kg * X_TM + srow) * (X_TN * (int)sizeof(T)));
        const int wsw = (srow >> 1) & 7;
        const int r_l = lane >> 3, c_l = lane & 7;  // reader: row r_l + 8k, slot c_l, lane group `wave`
        // the tile's outputs all lie inside the plane and are all wanted: unconditional stores, NST per wavefront
        const bool full_out = p0 + X_TM <= H && q0 + X_TN <= W && (!cross || fill_upper);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            if (v > 0) wg_barrier();  // the previous round's reads are done
#pragma unroll
            for (int cb = 0; cb < X_NCB; ++cb)
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    const int slot = kh * 4 + cb * 2 + k;
                    lds_store16(wbase + 16u * (unsigned)(slot ^ wsw),
                                u32x4{outp[cb][v][4 * k], outp[cb][v][4 * k + 1], outp[cb][v][4 * k + 2], outp[cb][v][4 * k + 3]});
                }
            lds_wait();
            wg_barrier();
            u32x4 val[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int row = k * 8 + r_l;
                val[k] = lds_load16(stage_lds + (unsigned)((wave * X_TM + row) * (X_TN * (int)sizeof(T))) +
                                    16u * (unsigned)(c_l ^ ((row >> 1) & 7)));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(val[0]), "+v"(val[1]), "+v"(val[2]), "+v"(val[3]) : : "memory");
            T *yh = yg + (int64_t)(wave * 4 + v) * HW;
            if (full_out) {
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    __builtin_nontemporal_store(val[k], reinterpret_cast<u32x4 *>(yh + (int64_t)(p0 + k * 8 + r_l) * W + q0 + c_l * VEC));
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int row = p0 + k * 8 + r_l, col = q0 + c_l * VEC;
                    if (row < H && col < W && (!causal || fill_upper || col <= row))
                        __builtin_nontemporal_store(val[k], reinterpret_cast<u32x4 *>(yh + (int64_t)row * W + col));
                }
            }
        }
        prev_st = full_out ? NST : -1;
        pre_issued = next_ok;
        advance();
        // (the next item's first barrier orders this item's last staging reads before its first staging writes: the
        // staging area is next written after sixteen more barriers)
    }
}

// The item list cut into eight runs of about equal cost.  Cost of a tile: 1; 1.7 where the diagonal passes through its
// window (those are fixed up in LDS head by head); a tile wholly above the diagonal 0.35 when it is filled with +0 and
// next to nothing when it is only skipped.  Per tile row the tiles come in that order.
template <int R, int S>
xm_split make_split(int64_t npg, int64_t tiles_m, int64_t tiles_n, int causal, int fill_upper, int tri, int64_t ipp)
{
    using G = xgeom<R, S>;
    const double c_fix = 1.7, c_zero = fill_upper ? 0.35 : 0.02;
    auto counts = [&](int64_t tm, int64_t &n_plain, int64_t &n_fix, int64_t &n_zero) {
        const int64_t p0 = tm * X_TM;
        const int64_t n0 = causal ? std::min<int64_t>(tiles_n, (p0 + X_TM - 1) / X_TN + 1) : tiles_n;
        int64_t nf = 0;
        if (causal) {  // q0 - HL + TW - 1 > p0 - (R-1)
            const int64_t lim = p0 - (R - 1) + G::HL - G::TW + 1;
            const int64_t first_fix = lim < 0 ? 0 : lim / X_TN + 1;
            nf = std::max<int64_t>(0, n0 - first_fix);
        }
        n_fix = nf;
        n_plain = n0 - nf;
        n_zero = tri ? 0 : tiles_n - n0;
    };
    std::vector<double> cum((size_t)tiles_m + 1, 0.0);
    for (int64_t tm = 0; tm < tiles_m; ++tm) {
        int64_t a, f, z;
        counts(tm, a, f, z);
        cum[(size_t)tm + 1] = cum[(size_t)tm] + (double)a + c_fix * (double)f + c_zero * (double)z;
    }
    const double cost_pg = cum[(size_t)tiles_m], total_cost = cost_pg * (double)npg;
    const int64_t total = npg * ipp;
    xm_split sp;
    sp.start[0] = 0;
    for (int k = 1; k < 8; ++k) {
        const double target = total_cost * k / 8.0;
        int64_t pg = cost_pg > 0 ? (int64_t)(target / cost_pg) : 0;
        if (pg >= npg) pg = npg - 1;
        double rem = target - (double)pg * cost_pg;
        int64_t tm = (int64_t)(std::upper_bound(cum.begin(), cum.end(), rem) - cum.begin()) - 1;
        tm = std::max<int64_t>(0, std::min<int64_t>(tm, tiles_m - 1));
        int64_t a, f, z;
        counts(tm, a, f, z);
        double r = rem - cum[(size_t)tm];
        int64_t off;
        if (r < (double)a) off = (int64_t)r;
        else if (r - (double)a < c_fix * (double)f) off = a + (int64_t)((r - (double)a) / c_fix);
        else off = a + f + (int64_t)((r - (double)a - c_fix * (double)f) / c_zero);
        const int64_t in_row = a + f + z;
        off = std::max<int64_t>(0, std::min<int64_t>(off, in_row));
        const int64_t b = tm / X_RPB;
        const int64_t before = tri ? b * (b + 1) + (tm % X_RPB) * (b + 1) : tm * tiles_n;
        sp.start[k] = std::max(sp.start[k - 1], std::min(total, pg * ipp + before + off));
    }
    sp.start[8] = total;
    return sp;
}

template <typename T, int R, int S>
int launch_x(const void *x, const void *wc, const void *wm, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int causal,
             int fill_upper, hipStream_t st)
{
    const int64_t tiles_m = (H + X_TM - 1) / X_TM, tiles_n = (W + X_TN - 1) / X_TN;
    const int tri = (causal && !fill_upper && H == W) ? 1 : 0;
    const int64_t nbf = tiles_m / X_RPB, kl = tiles_m % X_RPB;
    const int64_t ipp64 = tri ? nbf * (nbf + 1) + kl * (nbf + 1) : tiles_m * tiles_n;
    if (ipp64 > (1 << 24)) return MTA_ERR_SHAPE;
    const int64_t npg = N * (C / X_HG);
    const xm_split sp = make_split<R, S>(npg, tiles_m, tiles_n, causal, fill_upper, tri, ipp64);
    int64_t longest = 0;
    for (int k = 0; k < 8; ++k) longest = std::max(longest, sp.start[k + 1] - sp.start[k]);
    int nw = device_cu_count() * x_occ<R>() / 8;
    if (nw < 1) nw = 1;
    if (longest < nw) nw = (int)std::max<int64_t>(longest, 1);
    hipLaunchKernelGGL((conv_mix16_mfma<T, R, S>), dim3((unsigned)(nw * 8)), dim3(X_WT), 0, st, (const T *)x, (const T *)wc,
                       (const T *)wm, (T *)y, (int)C, (int)H, (int)W, causal, fill_upper, (int)tiles_n, (int)ipp64, sp, nw, tri);
    return launch_status();
}
}  // namespace

namespace mta {
// Returns MTA_ERR_UNSUPPORTED when no instance covers the arguments (the caller then takes another kernel).
int conv_mix16_dispatch(const void *x, const void *wc, const void *wm, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                        int S, int causal, int fill_upper, int io_dtype, hipStream_t st)
{
    // MTA_CONV_MIX16_OFF=1 in the environment keeps groups of 16 heads on the other kernels (for comparisons)
    static const bool off = [] { const char *e = getenv("MTA_CONV_MIX16_OFF"); return e && e[0] == '1'; }();
    if (off || io_dtype == MTA_F32 || C % X_HG != 0 || W % 8 != 0 || !aligned_to(x, 16) || !aligned_to(y, 16) ||
        !aligned_to(wm, 8) || !aligned_to(wc, 16))
        return MTA_ERR_UNSUPPORTED;
#define MTA_XM_CASE(r, s)                                                                                            \
    static_assert(xgeom<r, s>::fits, "window exceeds 32 keys");                                                        \
    if (R == r && S == s) {                                                                                          \
        if (io_dtype == MTA_BF16) return launch_x<bf16_t, r, s>(x, wc, wm, y, N, C, H, W, causal, fill_upper, st);    \
        return launch_x<f16_t, r, s>(x, wc, wm, y, N, C, H, W, causal, fill_upper, st);                               \
    }
    MTA_XM_CASE(3, 3)
    MTA_XM_CASE(5, 5)
    MTA_XM_CASE(7, 7)
#undef MTA_XM_CASE
    return MTA_ERR_UNSUPPORTED;
}
}  // namespace mta
