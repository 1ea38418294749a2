// O = P V for the MTA pipeline:  P is the (B,H,S,S) post-softmax tensor, V is (B,H,S,D), O is (B,H,S,D).
//
// When causal, only keys q <= p of P are read: nothing above the diagonal is touched (it may be
// uninitialised memory), which halves the traffic of the plain batched GEMM this replaces.
// HBM-bound: the P triangle is streamed once, V blocks are re-read from L2.
//
// P_WAVES wavefronts own a block of 32 query rows each; a wavefront owns two blocks of 16 rows.  O^T += V^T P^T on
// 16x16x32 MFMAs: lane (r = lane%16, g = lane/16) owns query row r of a block and supplies P^T
// fragments straight from global memory (16 contiguous bytes = 8 keys of its row, loaded one key
// block ahead), V blocks of 64 keys are copied global -> LDS asynchronously (double buffered,
// 16-byte chunks XOR-swizzled by key) and V^T fragments come out of them through the LDS transpose
// read: within 16 lanes, lane c supplies the address of 4 head-dim values of key c/4 and lane i
// receives head-dim value i of 4 consecutive keys.
#include <type_traits>

#include <cstdlib>

#include "common.hpp"
#include "mfma.hpp"
#include "strip_common.hpp"

namespace {
using namespace mta;

typedef short v4s_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s_t lds_v4s_t;

constexpr int P_WAVES = 4;          // wavefronts per workgroup (8, i.e. half the V re-reads, measured no faster)
constexpr int P_NT = 64 * P_WAVES;
constexpr int P_BQ = 32 * P_WAVES;  // query rows per block: 32 per wavefront
constexpr int P_OCC = 2;            // workgroups per CU the kernel is compiled for
constexpr int P_BK = 64;  // keys per iteration (128 measured no faster): each lane reads P_BK/4 contiguous bytes of its row per
                                 // iteration, back to back, so that DRAM pages are used in long runs
constexpr int P_KS = P_BK / 32;  // 32-key contraction steps per iteration

// SPLIT = 2: two such groups of wavefronts in a workgroup share the query rows and take the even and the odd key
// blocks; the second group's sums reach the first through LDS at the end.  For grids that put one workgroup on a CU
// (few heads): twice the loads in flight for the same bytes.
template <typename T, int D, int SPLIT>
__global__ __launch_bounds__(P_NT * SPLIT, SPLIT == 2 ? 1 : P_OCC) void causal_pv_kernel(
    const T *__restrict__ P, const T *__restrict__ V, T *__restrict__ O, int S, int causal, int nqb, int64_t total_wg,
    int64_t per_xcd, const int *__restrict__ band_lo, int H, int tri_gl)
{
    constexpr int CPR = D / 8;               // 16-byte chunks per V row
    constexpr int TILE = P_BK * D;           // elements per V block
    constexpr int ROUNDS = (TILE / 8 + P_NT - 1) / P_NT;
    constexpr int DB = D / 16;
    static_assert(SPLIT == 1 || (size_t)SPLIT * TILE * sizeof(T) == (size_t)DB * P_NT * 16, "the sums of one row block fit one V buffer pair");
    // Double buffer as two separate arrays, and a loop body instantiated once per array: the compiler then sees that
    // the LDS reads of one block never touch the asynchronous copy in flight into the other.  With one array it
    // cannot, and waits for the copy (and for every load issued before it) ahead of the first LDS read.
    __shared__ __align__(16) T v_a_all[SPLIT * TILE];
    __shared__ __align__(16) T v_b_all[SPLIT * TILE];

    const int grp = SPLIT == 2 ? (int)(threadIdx.x >> 8) : 0;  // which key blocks: j % SPLIT == grp
    T *const v_a = v_a_all + grp * TILE;
    T *const v_b = v_b_all + grp * TILE;
    const int tid = threadIdx.x & (P_NT - 1);
    const int wave = tid >> 6, lane = tid & 63, ln = lane & 15, kg = lane >> 4;
    // XCD-aware order: XCD x (workgroup id % 8) takes the x-th eighth of the (batch*head, query block) list, so
    // the workgroups that share one head's V run on one L2; within a head the longest query blocks come first
    const int64_t lid = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (lid >= total_wg) return;
    // A workgroup takes two blocks of query rows of one (batch, head): block nqb-1-pi and block pi.  With causal
    // rows the first has the most keys and the second the fewest: every workgroup gets the same amount of work
    // (the whole grid is resident at once, so the longest workgroup would otherwise set the kernel's duration).
    const int npairs = (nqb + 1) / 2;
    const int pi = (int)(lid % npairs);
    const int64_t bh = lid / npairs;
    // (tri_gl > 0: P in the triangular layout, groups of tri_gl heads interleaved by rows)
    const T *Pp = tri_gl > 0 ? P + (bh / tri_gl) * (tri_gl * tri_rowoff(S)) : P + bh * (int64_t)S * S;
    const T *Vp = V + bh * (int64_t)S * D;
    T *Op = O + bh * (int64_t)S * D;
  for (int half = 0; half < 2; ++half) {
    const int qb = half == 0 ? nqb - 1 - pi : pi;
    if (half == 1 && qb == nqb - 1 - pi) break;  // odd number of blocks: the middle one is alone
    const int q0 = qb * P_BQ;
    if (half == 1) __syncthreads();  // the V buffers are reused: everybody has finished reading them

    auto issue_v = [&](int j, T *dst) {
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int slot = r * P_NT + tid;
            if (TILE / 8 % P_NT != 0 && slot >= TILE / 8) break;
            const int row = slot / CPR, c = (slot % CPR) ^ v_swizzle<D>(row);
            int vr = j * P_BK + row;
            vr = vr >= S ? S - 1 : vr;
            __builtin_amdgcn_global_load_lds((glb_void_t *)(Vp + (int64_t)vr * D + c * 8),
                                             (lds_void_t *)(dst + (r * P_NT + wave * 64) * 8), 16, 0, 0);
        }
    };

    int prow[2];
    const T *prow_ptr[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        prow[rb] = q0 + wave * 32 + rb * 16 + ln;
        const int pc = prow[rb] < S ? prow[rb] : S - 1;
        prow_ptr[rb] = tri_gl > 0 ? Pp + tri_gl * tri_rowoff(pc) + (int)(bh % tri_gl) * tri_rowlen(pc) + kg * 8
                                  : Pp + (int64_t)pc * S + kg * 8;
    }
    // P^T fragments of key block j: slots t = 0..7 of k-step ks are keys j*64 + 32ks + 8kg + t; out-of-range
    // vectors re-read the row start, the values are masked when used
    auto load_p = [&](int j, frag8<T> (&pf)[2][P_KS]) {
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int ks = 0; ks < P_KS; ++ks) {
                const int key = j * P_BK + ks * 32 + kg * 8;
                const bool ok = key < S && !(causal && key > prow[rb]);
                // (non-temporal: P is streamed, every element is read once)
                typedef unsigned int u4 __attribute__((ext_vector_type(4)));
                pf[rb][ks] = __builtin_bit_cast(frag8<T>, __builtin_nontemporal_load(reinterpret_cast<const u4 *>(
                                                              prow_ptr[rb] + (ok ? j * P_BK + ks * 32 : -kg * 8))));
            }
    };

    const int q_last = (q0 + P_BQ - 1 < S - 1) ? q0 + P_BQ - 1 : S - 1;
    const int j_end = causal ? q_last / P_BK : (S - 1) / P_BK;
    // band mask (band_lo[b, p]: first key row p sees, P is 0 ahead of it): the key blocks ahead of the first key any row
    // of this query block sees are not visited (every wavefront reduces all the rows: the same answer in each)
    int j0 = 0;
    if (band_lo) {
        const int64_t brow = (bh / H) * (int64_t)S;
        int fmin = S;
        for (int r = lane; r < P_BQ; r += 64) {
            if (q0 + r < S) {
                const int f = band_lo[brow + q0 + r];
                fmin = f < fmin ? f : fmin;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const int o = __shfl_xor(fmin, off);
            fmin = o < fmin ? o : fmin;
        }
        fmin = __builtin_amdgcn_readfirstlane(fmin);
        j0 = (fmin > 0 ? fmin : 0) / P_BK;
        if (j0 > j_end) j0 = j_end;
    }
    // this group's key blocks: jg, jg + SPLIT, ... (by the block's own parity, whatever the first block is: a band mask
    // that skips blocks of zeros leaves every sum as it is, bit for bit)
    const int jg = SPLIT == 2 ? j0 + ((j0 & 1) != grp) : j0;
    const int nsteps = (j_end - j0) / SPLIT + 1;  // of the group that starts at j0: the other one idles in its last step
    if (jg <= j_end) issue_v(jg, v_a);
    // P fragments are fetched one key block ahead, alternately into two register sets
    frag8<T> p_a[2][P_KS], p_b[2][P_KS];
    load_p(jg, p_a);

    f32x4 oacc[2][DB];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int db = 0; db < DB; ++db) oacc[rb][db] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    auto step = [&](int j, const T *Vb, T *Vn, frag8<T> (&pcur)[2][P_KS], frag8<T> (&pnext)[2][P_KS]) __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(0);  // V block j and the P fragments have arrived
        __syncthreads();                // for every wavefront; reads of the other buffer are finished
        if (SPLIT == 2 && j > j_end) return;  // (the other group's last block: this one only meets it at the barrier)
        if (j + SPLIT <= j_end) {
            issue_v(j + SPLIT, Vn);
            load_p(j + SPLIT, pnext);
        }
        // mask the fragments of this block: keys beyond the row (causal) or the sequence count as 0
        frag8<T> pf[2][P_KS];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int ks = 0; ks < P_KS; ++ks) {
                const int key0 = j * P_BK + ks * 32 + kg * 8;
                pf[rb][ks] = pcur[rb][ks];
                const int lim = causal ? (prow[rb] < S - 1 ? prow[rb] : S - 1) : S - 1;
                if (key0 + 7 > lim) {
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        if (key0 + t > lim) pf[rb][ks].v[t] = from_float<T>(0.0f);
                }
            }
        // V^T fragments of block blk = ks*DB + db are read from LDS while the matrix cores work on block blk-1 (left to
        // itself the compiler issues read, wait, product, read, wait, ... : an LDS latency per group of products)
        auto load_vf = [&](int blk, frag8<T> &dst) {
            const int ks = blk / DB, db = blk % DB;
            const int key_a = ks * 32 + kg * 8 + (ln >> 2);  // slots 0..3: keys 8kg+(0..3); slots 4..7: +4
            const int key_b = key_a + 4;
            const int ch = db * 2 + ((ln & 3) >> 1);
            const int sub = (ln & 1) * 4;
            const T *pa = Vb + key_a * D + ((ch ^ v_swizzle<D>(key_a)) * 8) + sub;
            const T *pb = Vb + key_b * D + ((ch ^ v_swizzle<D>(key_b)) * 8) + sub;
            struct { v4s_t a, b; } both = {__builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)pa),
                                           __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)pb)};
            dst = __builtin_bit_cast(frag8<T>, both);
        };
        frag8<T> vf[2];
        load_vf(0, vf[0]);
#pragma unroll
        for (int blk = 0; blk < P_KS * DB; ++blk) {
            const int ks = blk / DB, db = blk % DB;
            if (blk + 1 < P_KS * DB) load_vf(blk + 1, vf[(blk + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);  // (the instruction scheduler would move the reads back behind the products)
            mma16(oacc[0][db], vf[blk & 1], pf[0][ks]);
            mma16(oacc[1][db], vf[blk & 1], pf[1][ks]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for (int i = 0, j = jg;; j += SPLIT) {
        step(j, v_a, v_b, p_a, p_b);
        if (++i >= nsteps) break;
        j += SPLIT;
        step(j, v_b, v_a, p_b, p_a);
        if (++i >= nsteps) break;
    }

    if constexpr (SPLIT == 2) {
        // the second group's sums travel through the V buffers (rows' first block in one, second in the other)
        typedef __attribute__((address_space(3))) f32x4 lds_f4;
        __syncthreads();  // nobody reads V any more
        if (grp == 1) {
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                reinterpret_cast<f32x4 *>(v_a_all)[db * P_NT + tid] = oacc[0][db];
                reinterpret_cast<f32x4 *>(v_b_all)[db * P_NT + tid] = oacc[1][db];
            }
        }
        __syncthreads();
        if (grp == 1) continue;  // (the barrier ahead of the second row block is met at the top of the loop)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            oacc[0][db] += reinterpret_cast<const f32x4 *>(v_a_all)[db * P_NT + tid];
            oacc[1][db] += reinterpret_cast<const f32x4 *>(v_b_all)[db * P_NT + tid];
        }
    }
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        if (prow[rb] >= S) continue;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            struct alignas(8) quad { T v[4]; } out;
#pragma unroll
            for (int v = 0; v < 4; ++v) out.v[v] = from_float<T>(oacc[rb][db][v]);
            *reinterpret_cast<quad *>(Op + (int64_t)prow[rb] * D + db * 16 + kg * 4) = out;
        }
    }
  }
}

// ---- the transposed product --------------------------------------------------------------------------------------
// O[k, :] = sum over p of P[p, k] X[p, :], p >= k only when causal: the gradients that the two matrix products of the
// attention leave on their right-hand operands (dV = P^T dO, dK = G^T Q), whose left factor is only defined - and only
// read - on and below the diagonal.
//
// A workgroup owns 128 keys (output rows; 32 per wavefront, two blocks of 16) and walks the query rows from its first
// key downwards in blocks of 64.  O^T += X^T P on 16x16x32 MFMAs with the query rows as contraction index: both
// operands are copied global -> LDS asynchronously as row-major blocks (64 rows of X, 64 rows x 128 keys of P; double
// buffered, 16-byte chunks XOR-swizzled by row) and both fragments come out of them through the LDS transpose read,
// which hands a lane four consecutive rows of one column: X^T with the head dim as operand row, P with the key as
// operand column.  P is streamed from memory once; the X blocks are re-read from L2 by every key block above them.
constexpr int T_KB = 32 * P_WAVES;  // keys per workgroup
constexpr int T_PB = 64;            // query rows per step
constexpr int T_KS = T_PB / 32;

template <typename T, int D>
__global__ __launch_bounds__(P_NT, P_OCC) void causal_ptx_kernel(const T *__restrict__ P, const T *__restrict__ X,
                                                                 T *__restrict__ O, int S, int causal, int nkb, int64_t total_wg,
                                                                 int64_t per_xcd)
{
    constexpr int XT = T_PB * D, PT = T_PB * T_KB;  // elements per X block / P tile
    constexpr int XC = D / 8, PC = T_KB / 8;        // 16-byte chunks per row
    constexpr int XR = XT / 8 / P_NT, PR = PT / 8 / P_NT;
    static_assert(XT / 8 % P_NT == 0 && PT / 8 % P_NT == 0, "whole copy rounds");
    constexpr int DB = D / 16;
    __shared__ __align__(16) T x_a[XT];
    __shared__ __align__(16) T x_b[XT];
    __shared__ __align__(16) T p_a[PT];
    __shared__ __align__(16) T p_b[PT];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, ln = lane & 15, kg = lane >> 4;
    const int64_t lid = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (lid >= total_wg) return;
    // two key blocks per workgroup, pi and nkb-1-pi: under the causal rule the first has the most query rows and the
    // second the fewest, so that every workgroup gets the same amount of work
    const int npairs = (nkb + 1) / 2;
    const int pi = (int)(lid % npairs);
    const int64_t bh = lid / npairs;
    const T *Pp = P + bh * (int64_t)S * S;
    const T *Xp = X + bh * (int64_t)S * D;
    T *Op = O + bh * (int64_t)S * D;
  for (int half = 0; half < 2; ++half) {
    const int kb = half == 0 ? pi : nkb - 1 - pi;
    if (half == 1 && kb == pi) break;  // odd number of blocks: the middle one is alone
    const int k0 = kb * T_KB;
    if (half == 1) __syncthreads();    // the buffers are reused: everybody has finished reading them

    // block j = query rows 64j ..; rows past the sequence re-read the last row, keys past it the block's first chunk:
    // what they bring in is masked (rows) or belongs to output rows that are not stored (keys)
    auto issue = [&](int j, T *xdst, T *pdst) {
#pragma unroll
        for (int r = 0; r < XR; ++r) {
            const int slot = r * P_NT + tid;
            const int row = slot / XC, c = (slot % XC) ^ v_swizzle<D>(row);
            int pr = j * T_PB + row;
            pr = pr >= S ? S - 1 : pr;
            __builtin_amdgcn_global_load_lds((glb_void_t *)(Xp + (int64_t)pr * D + c * 8),
                                             (lds_void_t *)(xdst + (r * P_NT + wave * 64) * 8), 16, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < PR; ++r) {
            const int slot = r * P_NT + tid;
            const int row = slot / PC;
            int c = (slot % PC) ^ v_swizzle<T_KB>(row);
            if (k0 + c * 8 >= S) c = 0;
            int pr = j * T_PB + row;
            pr = pr >= S ? S - 1 : pr;
            __builtin_amdgcn_global_load_lds((glb_void_t *)(Pp + (int64_t)pr * S + k0 + c * 8),
                                             (lds_void_t *)(pdst + (r * P_NT + wave * 64) * 8), 16, 0, 0);
        }
    };
    // operand fragment out of a row-major block of LD columns: contraction slots t = 0..7 of step ks are the block's rows
    // 32ks + 8kg + t, the operand's row / column is column 16*blk + ln of the block
    auto frag_of = [&](const T *tile, auto ldc, int ks, int blk) {
        constexpr int LD = decltype(ldc)::value;
        const int row_a = ks * 32 + kg * 8 + (ln >> 2), row_b = row_a + 4;
        const int ch = blk * 2 + ((ln & 3) >> 1);
        const int sub = (ln & 1) * 4;
        const T *pa = tile + row_a * LD + ((ch ^ v_swizzle<LD>(row_a)) * 8) + sub;
        const T *pb = tile + row_b * LD + ((ch ^ v_swizzle<LD>(row_b)) * 8) + sub;
        struct { v4s_t a, b; } both = {__builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)pa),
                                       __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)pb)};
        return __builtin_bit_cast(frag8<T>, both);
    };

    // this lane's two output rows (keys)
    int krow[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) krow[rb] = k0 + (wave * 2 + rb) * 16 + ln;
    const int j_start = causal ? k0 / T_PB : 0, j_end = (S - 1) / T_PB;
    f32x4 oacc[2][DB];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int db = 0; db < DB; ++db) oacc[rb][db] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    issue(j_start, x_a, p_a);

    auto step = [&](int j, const T *Xb, const T *Pb, T *Xn, T *Pn) __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(0);  // block j has arrived
        __syncthreads();                // for every wavefront; reads of the other buffers are finished
        if (j < j_end) issue(j + 1, Xn, Pn);
        // P fragments of this wavefront's two key blocks; query rows above the key (causal: P is undefined there) or
        // past the sequence count as 0
        frag8<T> pf[2][T_KS];
        const int pbase = j * T_PB;
        const bool edge = pbase + T_PB > S || (causal && pbase < k0 + T_KB - 1);  // (wavefront-uniform)
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int ks = 0; ks < T_KS; ++ks) {
                pf[rb][ks] = frag_of(Pb, std::integral_constant<int, T_KB>{}, ks, wave * 2 + rb);
                if (edge) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const int p = pbase + ks * 32 + kg * 8 + t;
                        if (p >= S || (causal && p < krow[rb])) pf[rb][ks].v[t] = from_float<T>(0.0f);
                    }
                }
            }
        frag8<T> xf[2];
        xf[0] = frag_of(Xb, std::integral_constant<int, D>{}, 0, 0);
#pragma unroll
        for (int blk = 0; blk < T_KS * DB; ++blk) {
            const int ks = blk / DB, db = blk % DB;
            if (blk + 1 < T_KS * DB) xf[(blk + 1) & 1] = frag_of(Xb, std::integral_constant<int, D>{}, (blk + 1) / DB, (blk + 1) % DB);
            __builtin_amdgcn_sched_barrier(0);  // (the instruction scheduler would move the reads back behind the products)
            mma16(oacc[0][db], xf[blk & 1], pf[0][ks]);
            mma16(oacc[1][db], xf[blk & 1], pf[1][ks]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for (int j = j_start;;) {
        step(j, x_a, p_a, x_b, p_b);
        if (++j > j_end) break;
        step(j, x_b, p_b, x_a, p_a);
        if (++j > j_end) break;
    }

#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        if (krow[rb] >= S) continue;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            struct alignas(8) quad { T v[4]; } out;
#pragma unroll
            for (int v = 0; v < 4; ++v) out.v[v] = from_float<T>(oacc[rb][db][v]);
            *reinterpret_cast<quad *>(Op + (int64_t)krow[rb] * D + db * 16 + kg * 4) = out;
        }
    }
  }
}

template <typename T, int D>
int launch_t(const void *p, const void *x, void *o, int64_t B, int64_t H, int64_t S, int causal, hipStream_t st)
{
    const int nkb = (int)((S + T_KB - 1) / T_KB);
    const int64_t total_wg = B * H * ((nkb + 1) / 2), per_xcd = (total_wg + 7) / 8;
    if (per_xcd * 8 > 0x7fffffffLL) return MTA_ERR_SHAPE;
    dim3 grid((unsigned)(per_xcd * 8));
    auto kern = causal_ptx_kernel<T, D>;
    hipLaunchKernelGGL(kern, grid, dim3(P_NT), 0, st, (const T *)p, (const T *)x, (T *)o, (int)S, causal, nkb, total_wg,
                       per_xcd);
    return launch_status();
}

template <typename T, int D>
int launch(const void *p, const void *v, void *o, int64_t B, int64_t H, int64_t S, int causal, hipStream_t st,
           const int *band_lo = nullptr, int tri_gl = 0)
{
    const int nqb = (int)((S + P_BQ - 1) / P_BQ);
    const int64_t total_wg = B * H * ((nqb + 1) / 2), per_xcd = (total_wg + 7) / 8;
    if (per_xcd * 8 > 0x7fffffffLL) return MTA_ERR_SHAPE;
    dim3 grid((unsigned)(per_xcd * 8));
    // a grid of at most one workgroup per CU runs the two-group instance (key blocks split between them)
    static const int force = [] { const char *e = getenv("MTA_PV_SPLIT"); return e ? atoi(e) : 0; }();  // 1 / 2: test switch
    const bool split = force ? force == 2 : total_wg <= device_cu_count();
    if (split) {
        auto kern = causal_pv_kernel<T, D, 2>;
        hipLaunchKernelGGL(kern, grid, dim3(P_NT * 2), 0, st, (const T *)p, (const T *)v, (T *)o, (int)S, causal, nqb,
                           total_wg, per_xcd, band_lo, (int)H, tri_gl);
    } else {
        auto kern = causal_pv_kernel<T, D, 1>;
        hipLaunchKernelGGL(kern, grid, dim3(P_NT), 0, st, (const T *)p, (const T *)v, (T *)o, (int)S, causal, nqb,
                           total_wg, per_xcd, band_lo, (int)H, tri_gl);
    }
    return launch_status();
}
}  // namespace

// first_visible (int32, (B,S); NULL = none): P[b,h,p,k] is 0 for k < first_visible[b,p] (what the softmax stage leaves
// under a band mask); the key blocks ahead of a query block's first visible key are not read.  Implies causal.
extern "C" int mta_causal_pv_band_fwd(const void *p, const void *v, const void *first_visible, void *o, int64_t B, int64_t H,
                                      int64_t S, int64_t D, int causal, int io_dtype, void *stream)
{
    if (!p || !v || !o) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype)) return MTA_ERR_DTYPE;
    if (B <= 0 || H <= 0 || S <= 0 || S > (1 << 24) || B * H > 65535) return MTA_ERR_SHAPE;
    if (D != 64 && D != 128) return MTA_ERR_HEAD_DIM;
    if (!aligned_to(p, 16) || !aligned_to(v, 16) || !aligned_to(o, 16) || (first_visible && !aligned_to(first_visible, 4)))
        return MTA_ERR_ALIGN;
    if (io_dtype == MTA_F32 || S % 8 != 0 || (first_visible && !causal)) return MTA_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const int *lo = (const int *)first_visible;
    if (io_dtype == MTA_BF16)
        return D == 64 ? launch<bf16_t, 64>(p, v, o, B, H, S, causal, st, lo) : launch<bf16_t, 128>(p, v, o, B, H, S, causal, st, lo);
    return D == 64 ? launch<f16_t, 64>(p, v, o, B, H, S, causal, st, lo) : launch<f16_t, 128>(p, v, o, B, H, S, causal, st, lo);
}

// P in the triangular layout (see tri_rowoff in common.hpp), groups of `group` heads interleaved by rows; causal.
extern "C" int mta_causal_pv_tri_fwd(const void *p, const void *v, const void *first_visible, void *o, int64_t B, int64_t H,
                                     int64_t S, int64_t D, int group, int io_dtype, void *stream)
{
    if (!p || !v || !o) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype)) return MTA_ERR_DTYPE;
    if (B <= 0 || H <= 0 || S <= 0 || S > (1 << 24) || B * H > 65535) return MTA_ERR_SHAPE;
    if (group <= 0 || H % group != 0) return MTA_ERR_GROUP;
    if (D != 64 && D != 128) return MTA_ERR_HEAD_DIM;
    if (!aligned_to(p, 16) || !aligned_to(v, 16) || !aligned_to(o, 16) || (first_visible && !aligned_to(first_visible, 4)))
        return MTA_ERR_ALIGN;
    if (io_dtype == MTA_F32 || S % 8 != 0) return MTA_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const int *lo = (const int *)first_visible;
    if (io_dtype == MTA_BF16)
        return D == 64 ? launch<bf16_t, 64>(p, v, o, B, H, S, 1, st, lo, group) : launch<bf16_t, 128>(p, v, o, B, H, S, 1, st, lo, group);
    return D == 64 ? launch<f16_t, 64>(p, v, o, B, H, S, 1, st, lo, group) : launch<f16_t, 128>(p, v, o, B, H, S, 1, st, lo, group);
}

extern "C" int mta_causal_pv_fwd(const void *p, const void *v, void *o, int64_t B, int64_t H, int64_t S, int64_t D,
                                 int causal, int io_dtype, void *stream)
{
    return mta_causal_pv_band_fwd(p, v, nullptr, o, B, H, S, D, causal, io_dtype, stream);
}

extern "C" int mta_causal_ptx_fwd(const void *p, const void *x, void *o, int64_t B, int64_t H, int64_t S, int64_t D,
                                  int causal, int io_dtype, void *stream)
{
    if (!p || !x || !o) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype)) return MTA_ERR_DTYPE;
    if (B <= 0 || H <= 0 || S <= 0 || S > (1 << 24) || B * H > 65535) return MTA_ERR_SHAPE;
    if (D != 64 && D != 128) return MTA_ERR_HEAD_DIM;
    if (!aligned_to(p, 16) || !aligned_to(x, 16) || !aligned_to(o, 16)) return MTA_ERR_ALIGN;
    if (io_dtype == MTA_F32 || S % 8 != 0) return MTA_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (io_dtype == MTA_BF16)
        return D == 64 ? launch_t<bf16_t, 64>(p, x, o, B, H, S, causal, st) : launch_t<bf16_t, 128>(p, x, o, B, H, S, causal, st);
    return D == 64 ? launch_t<f16_t, 64>(p, x, o, B, H, S, causal, st) : launch_t<f16_t, 128>(p, x, o, B, H, S, causal, st);
}
