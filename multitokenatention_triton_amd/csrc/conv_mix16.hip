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

namespace {
using namespace mta;

constexpr int X_NW = 4;            // wavefronts per workgroup
constexpr int X_WT = 64 * X_NW;    // threads per workgroup
constexpr int X_TM = 32;           // tile rows
constexpr int X_TN = 64;           // tile keys
constexpr int X_HALF = X_TN / 2;   // keys per wavefront
constexpr int X_NCB = X_HALF / 16; // 16 x 16 blocks per wavefront
constexpr int X_HG = 16;           // heads mixed together
constexpr int X_RPB = X_TN / X_TM; // tile rows per X_TN x X_TN block of the lower triangle
constexpr int X_OCC = 2;           // workgroups per CU the kernel is compiled for
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

template <typename T, int R, int S>
__global__ __launch_bounds__(X_WT, R <= 3 ? 3 : X_OCC) void conv_mix16_mfma(const T *__restrict__ x, const T *__restrict__ wc,
                                                               const T *__restrict__ wm, T *__restrict__ y, int C, int H,
                                                               int W, int causal, int fill_upper, int tiles_n, int ipp,
                                                               int64_t total, int64_t per_xcd, int tri)
{
    using G = xgeom<R, S>;
    static_assert(sizeof(T) == 2, "16-bit data");
    constexpr int TOP = R - 1, LD = G::LD, VEC = 8, SPR = LD / VEC;
    constexpr int SLOTS = G::ROWS * SPR;
    constexpr int STAGE_IT = (SLOTS + X_WT - 1) / X_WT;
    constexpr int BUF = ((SLOTS + 63) & ~63) * VEC;              // elements per window buffer (whole copy instructions)
    // window buffers: head h + NBUF - 1 is copied during head h (seven where that leaves room for three workgroups per CU)
    constexpr int NBUF = R <= 3 ? 7 : 8;
    constexpr int TAB_VECS = X_HG * R * G::NVEC;                 // 16-byte vectors of the fragment table
    constexpr int STG_BYTES = 4 * X_TM * X_TN * (int)sizeof(T);  // output staging: 4 heads x 32 rows x 128 bytes
    constexpr int RAW_BYTES = (X_HG * R * S * (int)sizeof(T) + 15) & ~15;
    static_assert(STG_BYTES <= NBUF * BUF * (int)sizeof(T), "the outputs are staged in the window buffers, which are free by then");
    __shared__ __align__(16) T tiles[NBUF * BUF];
    __shared__ __align__(16) u32x4 table[TAB_VECS + 1];          // (+ one vector of zeros)
    __shared__ __align__(16) unsigned char rawk[RAW_BYTES];      // the group's kernels as they lie in memory

    // XCD-aware: workgroup ids are dealt round-robin to the 8 XCDs; each XCD takes a contiguous run of the item list
    const int64_t idx = (int64_t)(blockIdx.x & 7) * per_xcd + (int64_t)(blockIdx.x >> 3);
    if ((int64_t)(blockIdx.x >> 3) >= per_xcd || idx >= total) return;
    const int groups = C / X_HG;
    const int64_t pg = idx / ipp;
    const int t_item = (int)(idx - pg * ipp);
    const int64_t n = pg / groups;
    const int g = (int)(pg - n * groups);
    int tm, tn;
    decode_tile(t_item, tiles_n, tri, tm, tn);
    const int p0 = tm * X_TM, q0 = tn * X_TN;
    const int64_t HW = (int64_t)H * W;
    const T *xg = x + (n * C + (int64_t)g * X_HG) * HW;   // head 0 of the group
    T *yg = y + (n * C + (int64_t)g * X_HG) * HW;

    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rb0 = (wave & 1) * 16, kh = wave >> 1;
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));

    if (causal && q0 > p0 + X_TM - 1) {  // wholly above the diagonal: +0 on request, for all 16 heads
        if (!fill_upper) return;
        const u4 z = {0u, 0u, 0u, 0u};
        const int r = tid >> 3, cv = (tid & 7) * VEC;
        if (p0 + r < H && q0 + cv < W) {
#pragma unroll
            for (int h = 0; h < X_HG; ++h) __builtin_nontemporal_store(z, reinterpret_cast<u4 *>(yg + h * HW + (int64_t)(p0 + r) * W + q0 + cv));
        }
        return;
    }

    const int h0 = p0 - TOP, k0 = q0 - G::HL;
    const bool interior = h0 >= 0 && h0 + G::ROWS <= H && k0 >= 0 && k0 + G::TW <= W && (!causal || k0 + G::TW - 1 <= h0);
    unsigned goff[STAGE_IT];
#pragma unroll
    for (int it = 0; it < STAGE_IT; ++it) {
        const int slot = it * X_WT + tid;
        int rr = slot / SPR, vc = slot % SPR;
        if (rr >= G::ROWS) { rr = 0; vc = 0; }
        goff[it] = (unsigned)(rr * W + vc * VEC) * (unsigned)sizeof(T);
    }
    auto slot_valid = [&](int slot) {
        const int rr = slot / SPR, vc = slot % SPR;
        const int h = h0 + rr, col = k0 + vc * VEC;
        return rr < G::ROWS && h >= 0 && h < H && col >= 0 && col < W && !(causal && col > h);
    };
    // asynchronous copy of head `head`'s window into `buf`: a slot inside the plane and on or below the diagonal is
    // copied, any other is written as zeros right here (nothing is read from outside the plane or above the diagonal)
    auto prefetch = [&](int head, T *buf) {
        const char *base = reinterpret_cast<const char *>(xg + head * HW + (int64_t)h0 * W + k0);
        if (interior) {
            // (whole instructions, issued under wavefront-uniform conditions: their number is what the waits count; a
            // lane beyond the window's last slot copies the window's first vector into the buffer's padding)
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it)
                if (it * X_WT + wave * 64 < SLOTS)
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(base + goff[it]),
                                                     (lds_void_t *)(buf + (it * X_WT + wave * 64) * VEC), 16, 0, 0);
        } else {
            const int tid_ = opaque(tid);
            const unsigned buf_lds = (unsigned)(uintptr_t)(lds_void_t *)buf;
            const u32x4 zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * X_WT + tid_;
                if (slot_valid(slot))
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(base + goff[it]),
                                                     (lds_void_t *)(buf + (it * X_WT + wave * 64) * VEC), 16, 0, 0);
                else if (slot < SLOTS)
                    lds_store16(buf_lds + (unsigned)slot * 16u, zero4);
            }
        }
    };

    // the group's kernels as they lie in memory: one 16-byte load per thread, issued ahead of the window copies
    constexpr int NRAW = RAW_BYTES / 16;
    static_assert(X_HG * R * S * (int)sizeof(T) % 16 == 0 && NRAW <= X_WT, "the kernels of a group are whole 16-byte vectors");
    u32x4 rawv = {0u, 0u, 0u, 0u};
    if (tid < NRAW) rawv = *reinterpret_cast<const u32x4 *>(wc + (int64_t)g * X_HG * (R * S) + tid * VEC);
#pragma unroll
    for (int b = 0; b < NBUF - 1; ++b) prefetch(b, tiles + b * BUF);
    // copy instructions of this wavefront per window (interior tiles)
    int n_copy = 0;
#pragma unroll
    for (int it = 0; it < STAGE_IT; ++it) n_copy += (it * X_WT + wave * 64 < SLOTS) ? 1 : 0;

    // ---- the group's kernels as they lie in memory -> LDS (staging area), then the table of Toeplitz vectors ----
    const unsigned stage_lds = (unsigned)(uintptr_t)(lds_void_t *)tiles;
    const unsigned raw_lds = (unsigned)(uintptr_t)(lds_void_t *)rawk;
    const unsigned table_lds = (unsigned)(uintptr_t)(lds_void_t *)table;
    {
        if (tid < NRAW) lds_store16(raw_lds + 16u * (unsigned)tid, rawv);
        lds_wait();
        wg_barrier();
        // vector (h, i, ve): taps j = ve + t - 7, t = 0..7, of kernel row i of head h (0 outside the row)
        for (int v = tid; v < TAB_VECS; v += X_WT) {
            const int hi = v / G::NVEC, ve = v - hi * G::NVEC;
            unsigned tap[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int j = ve + t - 7;
                tap[t] = lds_load_u16(raw_lds + 2u * (unsigned)(hi * S + ((j >= 0 && j < S) ? j : 0)));
            }
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+v"(tap[0]), "+v"(tap[1]), "+v"(tap[2]), "+v"(tap[3]), "+v"(tap[4]), "+v"(tap[5]), "+v"(tap[6]), "+v"(tap[7])
                         :
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
        wg_barrier();  // the table is complete
    }

    // this lane's Toeplitz vector: e = 8kg - ln; lanes outside the band read the vector of zeros
    const int e_rel = kg * 8 - ln - G::E0;
    const bool band = e_rel >= 0 && e_rel < G::NVEC;
    const unsigned tab_lane = table_lds + 16u * (unsigned)(band ? e_rel : 0);
    const unsigned tab_zero = table_lds + 16u * (unsigned)TAB_VECS;
    u32x4 tz[R];
    // weight fragment of the mixing: lane (output head ln, group kg) holds wm[o][4kg .. 4kg+3]
    const xm_u2 wf = *reinterpret_cast<const xm_u2 *>(wm + (int64_t)(g * X_HG + ln) * C + g * X_HG + kg * 4);

    uint32_t cres[X_HG][X_NCB][2];  // rounded conv results: head, block, (keys 4kg, 4kg+1), (keys 4kg+2, 4kg+3) of row ln

    static_for<X_HG>([&](auto hc) __attribute__((always_inline)) {
        constexpr int h = decltype(hc)::value;
        T *tile = tiles + (h % NBUF) * BUF;
        T *other = tiles + ((h + NBUF - 1) % NBUF) * BUF;  // head h-1's buffer, free after the barrier below
        const unsigned tile_lds = (unsigned)opaque((int)(unsigned)(uintptr_t)(lds_void_t *)tile);
        // This wavefront's part of head h's window has landed.  Copies complete in issue order; the windows of the heads
        // h+1 .. h+NBUF-2 may stay in flight when their number of instructions is known (interior tiles).
        {
            constexpr int ahead = (h + NBUF - 2 < X_HG - 1 ? h + NBUF - 2 : X_HG - 1) - h;
            static_assert(STAGE_IT * (NBUF - 2) <= 63, "vmcnt field");
            if (!interior || ahead == 0) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
            else if (n_copy == STAGE_IT) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(ahead * STAGE_IT) : "memory");
            else if (n_copy == STAGE_IT - 1) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(ahead * (STAGE_IT - 1)) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
        }
        if (!interior && causal && k0 + G::TW - 1 > h0) {
            // in the one vector of a row that straddles the diagonal, zero the keys beyond it
            const int tid_ = opaque(tid);
            u32x4 raw[STAGE_IT];
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * X_WT + tid_;
                const int hh = h0 + slot / SPR, col = k0 + (slot % SPR) * VEC;
                if (slot_valid(slot) && col + VEC - 1 > hh) raw[it] = lds_load16(tile_lds + (unsigned)slot * 16u);
            }
            lds_wait();
#pragma unroll
            for (int it = 0; it < STAGE_IT; ++it) {
                const int slot = it * X_WT + tid_;
                const int hh = h0 + slot / SPR, col = k0 + (slot % SPR) * VEC;
                if (slot_valid(slot) && col + VEC - 1 > hh) {
                    asm volatile("" : "+v"(raw[it]));
                    pack16<T> v = __builtin_bit_cast(pack16<T>, raw[it]);
#pragma unroll
                    for (int u = 0; u < VEC; ++u)
                        if (col + u > hh) v.v[u] = from_float<T>(0.0f);
                    lds_store16(tile_lds + (unsigned)slot * 16u, __builtin_bit_cast(u32x4, v));
                }
            }
        }
        lds_wait();
        wg_barrier();  // head h's window is in LDS; every wavefront is done with head h-1's
        if constexpr (h + NBUF - 1 < X_HG) prefetch(h + NBUF - 1, other);

        // Toeplitz fragments of head h
#pragma unroll
        for (int i = 0; i < R; ++i)
            tz[i] = lds_load16(band ? tab_lane + (unsigned)((h * R + i) * G::NVEC * 16) : tab_zero);

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
    wg_barrier();  // every wavefront is done with the last window: the buffers now stage the outputs
    // staging: [og][row 0..31][8 slots of 16 bytes], slot index XOR ((row >> 1) & 7)
    const int srow = rb0 + ln;
    const unsigned wbase = stage_lds + (unsigned)((kg * X_TM + srow) * (X_TN * (int)sizeof(T)));
    const int wsw = (srow >> 1) & 7;
    const int r_l = lane >> 3, c_l = lane & 7;  // reader: row r_l + 8k, slot c_l, lane group `wave`
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
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int row = p0 + k * 8 + r_l, col = q0 + c_l * VEC;
            if (row < H && col < W && (!causal || fill_upper || col <= row))
                __builtin_nontemporal_store(val[k], reinterpret_cast<u32x4 *>(yh + (int64_t)row * W + col));
        }
    }
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
    const int64_t total = N * (C / X_HG) * ipp64;
    const int64_t per_xcd = (total + 7) / 8;
    if (per_xcd * 8 > 0x7fffffffLL) return MTA_ERR_SHAPE;
    hipLaunchKernelGGL((conv_mix16_mfma<T, R, S>), dim3((unsigned)(per_xcd * 8)), dim3(X_WT), 0, st, (const T *)x, (const T *)wc,
                       (const T *)wm, (T *)y, (int)C, (int)H, (int)W, causal, fill_upper, (int)tiles_n, (int)ipp64, total, per_xcd,
                       tri);
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
