// Fused conv-attention forward:  O = softmax( mask( conv( mask0(Q K^T) ) ) * scale ) V
//
// One workgroup (4 wavefronts) owns a block of query rows of one (batch, head) and
// streams over the keys left to right.  No S x S tensor touches global memory: score
// tiles live in LDS, the conv reads them there, probabilities stay in registers.
//
// Orientation.  Every matrix product is issued "transposed" so that a lane always
// owns one query row:
//     S^T = K Q^T     A = K tile (LDS),        B = Q^T (registers, loaded once)
//     O^T = V^T P^T   A = V^T tile (LDS),      B = P^T (registers, straight from softmax)
// With the 32x32 MFMA accumulator layout (lane = column, 16 rows per lane) this puts the
// 16 keys of a score block that belong to one query row into one lane, so the softmax
// row reductions are in-lane plus one exchange with lane^32, the running max / sum and
// the O rescale are per-lane scalars, and P needs no LDS round trip: the MFMA contraction
// index may be permuted freely as long as both operands agree, so V^T is stored in LDS in
// the key order in which the accumulator layout hands out P.
//
// Tile geometry.  The score tile has 128 rows: HR = roundup(R-1, 8) halo rows above the
// block (recomputed, their outputs are discarded) + BQ = 128-HR output rows.  Keys are
// consumed in blocks of 64.  The conv's key halo is NOT recomputed: the last HC =
// roundup(Sk-1, 8) score columns of the previous block stay in LDS, and the conv /
// softmax / PV of a block lag the scores by the right-hand pad so that every tap is
// already there.  One extra leading key block (mostly out-of-range keys) primes that halo.
#include <algorithm>

#include <type_traits>
#include <utility>

#include "common.hpp"
#include "mfma.hpp"

#include <stdlib.h>

namespace {
using namespace mta;

constexpr int NT = 256;  // 4 wavefronts
constexpr int SR = 128;  // score-tile rows (32 per wavefront)
constexpr int BK = 64;   // keys per iteration

// position of key offset k16 (0..15) inside its 16-key group of the V^T tile: the order in
// which a lane's accumulator registers enumerate the keys of a 32x32 block (see header).
__device__ __forceinline__ int vt_pos16(int k16) { return ((k16 >> 2) & 1) * 8 + (k16 >> 3) * 4 + (k16 & 3); }

template <typename T> struct lds_pad { static constexpr int n = 16 / sizeof(T); };  // 16 bytes of padding per row

template <typename T, int D>
__global__ __launch_bounds__(NT) void conv_attn_fwd_kernel(const T *__restrict__ Q, const T *__restrict__ K,
                                                           const T *__restrict__ V, const void *__restrict__ Wt,
                                                           T *__restrict__ O, float *__restrict__ Lse, int S, int R,
                                                           int Sk, int causal, float scale, int w_dtype, int H, int nqb)
{
    constexpr int VEC = vec_of<T>::n;           // elements per 16-byte vector
    constexpr int PAD = lds_pad<T>::n;
    constexpr int KLD = D + PAD;                // K tile row stride
    constexpr int VLD = BK + PAD;               // V^T tile row stride
    constexpr int KS = D / 16;                  // contraction steps over the head dim
    constexpr int DB = D / 32;                  // 32-wide blocks of the head dim
    constexpr int KV_IT = BK * D / VEC / NT;    // 16-byte vectors per thread per K (or V) tile

    const int HR = (R - 1 + 7) & ~7;
    const int HC = (Sk - 1 + 7) & ~7;
    const int BQ = SR - HR;
    const int pw = (Sk - 1) / 2, pwr = Sk - 1 - pw;
    const int SLD = HC + BK + PAD;              // score tile row stride

    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *Ks = reinterpret_cast<T *>(smem_raw);
    T *Vt = Ks + BK * KLD;
    T *Sc = Vt + D * VLD;
    float *Ws = reinterpret_cast<float *>(Sc + SR * SLD);

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, ln = lane & 31, hf = lane >> 5;
    const int qb = nqb - 1 - (int)blockIdx.x;   // longest blocks first
    const int64_t bh = blockIdx.y;
    const int head = (int)(bh % H);
    const int q0 = qb * BQ;
    const int tr = wave * 32 + ln;              // this lane's row in the score tile
    const int p = q0 - HR + tr;                 // ... and its query row
    const T *Qp = Q + bh * (int64_t)S * D;
    const T *Kp = K + bh * (int64_t)S * D;
    const T *Vp = V + bh * (int64_t)S * D;
    T *Op = O + bh * (int64_t)S * D;

    for (int t = tid; t < R * Sk; t += NT) Ws[t] = load_any(Wt, w_dtype, (int64_t)head * R * Sk + t);

    // Q^T fragments of this lane's row, kept for the whole kernel
    frag8<T> qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        if (p >= 0 && p < S) {
            qf[ks] = *reinterpret_cast<const frag8<T> *>(Qp + (int64_t)p * D + ks * 16 + hf * 8);
        } else {
            qf[ks] = zero_frag<T>();
        }
    }

    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[db][v] = 0.0f;
    float m_i = -INFINITY, l_i = 0.0f;

    const int q_last = (q0 + BQ - 1 < S - 1) ? q0 + BQ - 1 : S - 1;
    const int j_end = causal ? q_last / BK : (S - 1) / BK;
    const int j_start = pwr > 0 ? -1 : 0;
    const int tail_vecs = SR * (HC / VEC);      // 16-byte vectors in the retained score columns
    constexpr int TAIL_IT = SR * 64 / VEC / NT; // upper bound (HC <= 64)

    using V16 = pack16<T>;
    for (int j = j_start; j <= j_end; ++j) {
        const int cb = j * BK + pwr;            // first key of the new score block
        // ---- global loads of the K block (keys cb..) and the V block (keys j*BK..) -------
        V16 kreg[KV_IT], vreg[KV_IT];
#pragma unroll
        for (int it = 0; it < KV_IT; ++it) {
            const int idx = it * NT + tid;
            const int row = idx / (D / VEC), vc = idx % (D / VEC);
            // unconditional loads (an out-of-range key re-reads key 0) so that they are issued back to back;
            // out-of-range rows are zeroed when they are written to LDS
            const int kr = cb + row;
            const int vr = j * BK + row;
            kreg[it] = *reinterpret_cast<const V16 *>(Kp + (int64_t)((kr >= 0 && kr < S) ? kr : 0) * D + vc * VEC);
            vreg[it] = *reinterpret_cast<const V16 *>(Vp + (int64_t)((vr >= 0 && vr < S) ? vr : 0) * D + vc * VEC);
        }
        // ---- retained score columns: read the tail of the previous tile ----------------------
        V16 tailreg[TAIL_IT];
#pragma unroll
        for (int it = 0; it < TAIL_IT; ++it) {
            const int idx = it * NT + tid;
            if (idx < tail_vecs) {
                const int row = idx / (HC / VEC), vc = idx % (HC / VEC);
                tailreg[it] = *reinterpret_cast<const V16 *>(Sc + row * SLD + BK + vc * VEC);
            }
        }
        __syncthreads();  // everyone is done reading the previous K, V^T and score tiles
#pragma unroll
        for (int it = 0; it < TAIL_IT; ++it) {
            const int idx = it * NT + tid;
            if (idx < tail_vecs) {
                const int row = idx / (HC / VEC), vc = idx % (HC / VEC);
                *reinterpret_cast<V16 *>(Sc + row * SLD + vc * VEC) = tailreg[it];
            }
        }
#pragma unroll
        for (int it = 0; it < KV_IT; ++it) {
            const int idx = it * NT + tid;
            const int row = idx / (D / VEC), vc = idx % (D / VEC);
            const int kr = cb + row, vr = j * BK + row;
            const bool k_ok = kr >= 0 && kr < S, v_ok = vr >= 0 && vr < S;
            V16 kv = kreg[it];
            if (!k_ok) {
#pragma unroll
                for (int u = 0; u < VEC; ++u) kv.v[u] = from_float<T>(0.0f);
            }
            *reinterpret_cast<V16 *>(Ks + row * KLD + vc * VEC) = kv;
            const int pos = (row & ~15) + vt_pos16(row & 15);
#pragma unroll
            for (int u = 0; u < VEC; ++u) Vt[(vc * VEC + u) * VLD + pos] = v_ok ? vreg[it].v[u] : from_float<T>(0.0f);
        }
        __syncthreads();

        // ---- S^T = K Q^T for this wavefront's 32 rows; causal zero; to LDS in the I/O dtype ----
#pragma unroll
        for (int kb = 0; kb < BK / 32; ++kb) {
            f32x16 sacc;
#pragma unroll
            for (int v = 0; v < 16; ++v) sacc[v] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const frag8<T> kf = *reinterpret_cast<const frag8<T> *>(Ks + (kb * 32 + ln) * KLD + ks * 16 + hf * 8);
                mma32(sacc, kf, qf[ks]);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                struct alignas(sizeof(T) * 4) quad { T v[4]; } out;
                const int xo = kb * 32 + g * 8 + hf * 4;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int col = cb + xo + r;
                    out.v[r] = from_float<T>((causal && col > p) ? 0.0f : sacc[g * 4 + r]);
                }
                *reinterpret_cast<quad *>(Sc + tr * SLD + HC + xo) = out;
            }
        }
        __syncthreads();
        if (j < 0) continue;

        // ---- conv over the LDS score tile (fp32 FMAs), scale, mask ---------------------------------
        float s[BK / 32][4][4];
        float mloc = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < BK / 32; ++kb)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int xo = kb * 32 + g * 8 + hf * 4;
                const int xb = HC - (Sk - 1) + xo;
                float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
                for (int i = 0; i < R; ++i) {
                    const int srow = tr - (R - 1) + i;
                    if (srow < 0) continue;
                    const T *src = Sc + srow * SLD + xb;
                    float w0 = to_float(src[0]), w1 = to_float(src[1]), w2 = to_float(src[2]);
                    for (int jj = 0; jj < Sk; ++jj) {
                        const float w3 = to_float(src[jj + 3]);
                        const float wv = Ws[i * Sk + jj];
                        a0 = fmaf(wv, w0, a0);
                        a1 = fmaf(wv, w1, a1);
                        a2 = fmaf(wv, w2, a2);
                        a3 = fmaf(wv, w3, a3);
                        w0 = w1; w1 = w2; w2 = w3;
                    }
                }
                const float av[4] = {a0, a1, a2, a3};
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int col = j * BK + xo + r;
                    const bool ok = col < S && (!causal || col <= p);
                    const float val = round_to<T>(round_to<T>(av[r]) * scale);
                    s[kb][g][r] = ok ? val : -INFINITY;
                    mloc = fmaxf(mloc, s[kb][g][r]);
                }
            }

        // ---- online softmax: this row is split over lanes ln and ln+32 -----------------------------
        const float mrow = fmaxf(mloc, __shfl_xor(mloc, 32));
        const float m_new = fmaxf(m_i, mrow);
        const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = __expf(m_i - m_use);
        m_i = m_new;
        float lsum = 0.0f;
        frag8<T> pf[BK / 32][2];
#pragma unroll
        for (int kb = 0; kb < BK / 32; ++kb)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float e = __expf(s[kb][g][r] - m_use);
                    const T et = from_float<T>(e);
                    lsum += to_float(et);
                    pf[kb][g >> 1].v[(g & 1) * 4 + r] = et;
                }
        l_i = l_i * alpha + lsum;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[db][v] *= alpha;

        // ---- O^T += V^T P^T -----------------------------------------------------------------------
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int kb = 0; kb < BK / 32; ++kb)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const frag8<T> vf =
                        *reinterpret_cast<const frag8<T> *>(Vt + (db * 32 + ln) * VLD + kb * 32 + ks * 16 + hf * 8);
                    mma32(oacc[db], vf, pf[kb][ks]);
                }
    }

    // ---- normalise and store this lane's row (halo rows are dropped) -----------------------------------
    const float l_row = l_i + __shfl_xor(l_i, 32);
    if (tr >= HR && p < S) {
        const float inv = 1.0f / l_row;
        if (Lse != nullptr && hf == 0) Lse[bh * (int64_t)S + p] = m_i + __logf(l_row);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                struct alignas(sizeof(T) * 4) quad { T v[4]; } out;
#pragma unroll
                for (int r = 0; r < 4; ++r) out.v[r] = from_float<T>(oacc[db][g * 4 + r] * inv);
                *reinterpret_cast<quad *>(Op + (int64_t)p * D + db * 32 + g * 8 + hf * 4) = out;
            }
    }
}

// =======================================================================================
// 16-bit fast path: everything on 16x16x32 MFMAs, conv included.
//
//  * 8 wavefronts own 256 score rows (HR halo rows + 256-HR output rows); a wavefront owns two
//    blocks of 16 rows.  Lane (r = lane%16, g = lane/16) owns query row r of a block; the
//    16x16 accumulator layout gives it keys 4g..4g+3 of every 16-key block, so a query row is
//    spread over 4 lanes and row reductions cost two lane exchanges.
//  * K and V blocks (64 keys) are copied global -> LDS asynchronously (global_load_lds), double
//    buffered, row-major, 16-byte chunks XOR-swizzled by the key index instead of padded.
//  * S^T = K Q^T -> causal/range zero -> LDS score tile (I/O dtype) -> conv as Toeplitz MFMAs
//    (out^T = T_i^T X^T per kernel row, the fragments of T_i^T live in registers) -> online
//    softmax in registers -> O^T += V^T P^T, where the V^T fragments come straight out of the
//    row-major V block through the LDS transpose read (ds_read_b64_tr_b16): within 16 lanes,
//    lane c supplies the address of 4 head-dim values of key c/4 and lane i receives head-dim
//    value i of 4 consecutive keys.
// =======================================================================================
typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;
typedef short v4s_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v4s_t lds_v4s_t;

// The workgroup has NW wavefronts and owns 32*NW score rows: 8 for the attention kernel (one workgroup per CU,
// K and V blocks shared by 256 rows), 4 for the scores-only kernel (three workgroups per CU, which overlap each
// other's barriers and memory latency).
// The attention kernel reads the LDS operands of the next group of matrix products before it issues the current group;
// the instruction scheduler largely undoes that (it moves reads down towards their use, which saves registers).  Pinning
// the source order there was measured and is slower (1.60 -> 1.72 ms at the benchmark shape, 12-14 spilled registers).
// The scores-only kernel pins its conv phase by hand instead (reads issued from assembly, see below).
constexpr int F_BK = 64;   // keys per iteration
constexpr int QK_OCC = 3;     // wavefronts per SIMD the scores-only kernel is compiled for (three workgroups per CU)
constexpr int QK_CHUNK = 32;  // key blocks per work item of the scores-only kernel when no item table is built
// with an item table: long and short items (key blocks), and the share of a query block's key range that goes into short
// ones (MTA_QK_CHUNK_LONG / MTA_QK_CHUNK_SHORT / MTA_QK_SHORT_PERCENT in the environment override them, for comparisons)
// (measured at B2 H16 S4096 D128: 32/32/0 237 us, 16/16/0 231, 64/16/50 238, 48/24/50 228, 52/26/50 227, 48/24/35 243)
constexpr int QK_CHUNK_LONG = 48, QK_CHUNK_SHORT = 24, QK_SHORT_PERCENT = 50;
constexpr int F_SLD = 80;  // score-tile row stride (elements): exactly the retained columns + one key block.  A wider
                           // row costs the scores-only kernel its third workgroup per CU, and with this one a fragment
                           // read (16 consecutive rows x 64 bytes) is free of bank conflicts as it is: the LDS serves
                           // lanes 0-7 together with lanes 24-31 (8-15 with 16-23, ...), and rows 160 bytes apart put
                           // those on the even and the odd 16-byte positions (measured; 144 or 176 bytes halve the rate)

// LDS accesses issued from assembly: the compiler neither reorders them nor waits for the asynchronous copy in flight
// ahead of them (it cannot tell a read of the score tile from the copy's target), and the wait points are placed by
// hand.  LDS operations of a wavefront complete in order, so "at most n operations outstanding" names the oldest ones
// as complete; a loaded value is tied to the wait that covers it through an in/out operand.
__device__ __forceinline__ unsigned lds_addr(const void *p) { return (unsigned)(uintptr_t)(lds_void_t *)p; }
__device__ __forceinline__ u32x4_t lds_read16_at(unsigned addr, int off)
{
    u32x4_t v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(off) : "memory");
    return v;
}
__device__ __forceinline__ void lds_write8_at(unsigned addr, int off, uint32_t lo, uint32_t hi)
{
    const u32x2_t v = {lo, hi};
    asm volatile("ds_write_b64 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(off) : "memory");
}
__device__ __forceinline__ void lds_write16_at(unsigned addr, int off, u32x4_t v)
{
    asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(addr), "v"(v), "n"(off) : "memory");
}
template <int N> __device__ __forceinline__ void lds_wait_upto(u32x4_t &v)
{
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(N) : "memory");
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), in order
template <int... I, typename F> __device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}
// The scores-only kernel writes the scores of 16-key blocks cb-1 and cb (cb odd, both row blocks: two writes) right
// after step (cb+1)*KS + LAG - 1 of its score phase; the last pair after the loop.  Number of those writes issued at the
// end of a step in [lo, hi).
constexpr int score_writes_between(int lo, int hi, int KS, int NCB, int LAG)
{
    int c = 0;
    for (int cb = 1; cb + 1 < NCB; cb += 2) {
        const int s = (cb + 1) * KS + LAG - 1;
        if (s >= lo && s < hi) c += 2;
    }
    return c;
}

// a.lo*b.lo + a.hi*b.hi + c for two packed pairs of the 16-bit type T, accumulated in fp32
template <typename T> __device__ __forceinline__ float dot2_io(uint32_t a, uint32_t b, float c)
{
    if constexpr (std::is_same<T, bf16_t>::value) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(mta_bf16x2, a), __builtin_bit_cast(mta_bf16x2, b), c, false);
    } else {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(mta_f16x2, a), __builtin_bit_cast(mta_f16x2, b), c, false);
    }
}

// max / sum over the four lane groups (lanes l, l^16, l^32, l^48) that share a query row, in every lane: two
// exchanges between whole rows of lanes on the vector ALU (no LDS permute, so the LDS counter stays ours to count)
__device__ __forceinline__ float max_across_groups(float v)
{
    u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_across_groups(float v)
{
    u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Inside a rarely taken, wavefront-uniform `if`: keeps it a branch.  Without it the compiler turns the masks of the
// diagonal key blocks into selects that every key block executes (a third of the attention kernel's vector
// instructions).
#define MTA_KEEP_BRANCH() asm volatile("" ::: "memory")

// Returns its argument, opaquely: what is derived from the result cannot be hoisted out of the block that computes it.
__device__ __forceinline__ int opaque_lane(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// Swizzle of a V block for the attention kernel's transpose reads, whose 16-lane groups are 4 keys apart (keys
// 4kg + 0..3): the 8 consecutive keys that may be served in one cycle must land in 8 different 8-bank regions.
// D = 128: region = chunk pair ^ key%8.  D = 64 (a row is half the banks, odd keys take the other half):
// region = chunk pair ^ (key/2)%4.
template <int D> __device__ __forceinline__ int v_swizzle4(int key)
{
    if constexpr (D == 128) return 2 * (key & 7);
    else return 2 * ((key >> 1) & 3);
}

template <int R, int SK, int NW> struct fused_geom {
    static constexpr int F_SR = 32 * NW;
    static constexpr int HR = (R - 1 + 7) & ~7;    // halo rows above the block (recomputed)
    static constexpr int HC = (SK - 1 + 7) & ~7;   // score columns kept from the previous key block
    static constexpr int BQ = F_SR - HR;           // output rows per workgroup
    static constexpr int PW = (SK - 1) / 2, PWR = SK - 1 - PW;
    static constexpr int SHIFT = HC - (SK - 1);    // first tap's offset in a block's 32-key window
    static constexpr bool fits = SHIFT + 16 + SK - 1 <= 32 && HC + F_BK <= 80;
    static constexpr int WZ_OFF = SHIFT + 16, WZ_LD = WZ_OFF + 32;
};

// A head's work items (query block, range of key blocks) in the order they are to be started: longest first, so that the
// long items all start early and the short ones fill the end of the grid.  Built on the host for every launch (a
// counting sort over at most ITEM_TABLE_MAX items) and passed by value as a kernel argument; n = 0: no table, the kernel
// cuts every query block's key range into chunks of jc_len blocks and walks the query blocks from the last to the first.
// The chunks need not be equal: the first part of a query block's key range goes into long items (one extra key block
// per item rebuilds the retained score columns, and an item costs a few microseconds to set up), the rest into short
// ones, which are started last and even out the end of the grid.
constexpr int ITEM_TABLE_MAX = 768;
struct item_table {
    int n;
    uint32_t e[ITEM_TABLE_MAX];  // query block (11 bits) | first key block << 11 (11 bits) | key blocks << 22
};

// SCORES_ONLY: stop after the conv and write  conv(mask0(scale * Q K^T))  as an (S,S) plane per (batch, head)
// (`O` is then the score tensor, V is unused).  Only q <= p is written when causal, plus +0 above the
// diagonal when `fill_upper` is set.
// BAND (scores-only kernel): a mask of the form "key k of query row p is visible iff band_lo[b, p] <= k <= p" - the
// scores of the hidden keys enter the conv as 0, as the reference's masked_fill ahead of its conv leaves them
// (mta_attention_triton.py:70-73).
template <typename T, int D, int R, int SK, bool SCORES_ONLY, int NW, bool BAND = false>
__global__ __launch_bounds__(64 * NW, SCORES_ONLY ? ((R > 7 || (BAND && R >= 7)) ? 2 : QK_OCC) : 2) void conv_attn_fwd_mfma(const T *__restrict__ Q, const T *__restrict__ K,
                                                             const T *__restrict__ V, const T *__restrict__ Wt,
                                                             T *__restrict__ O, float *__restrict__ Lse, int S, int causal,
                                                             float scale, int H, int nqb, int fill_upper, int64_t total_wg,
                                                             int64_t per_xcd, int jc_len, int items_per_bh, int hpx,
                                                             item_table tbl, const int *__restrict__ band_lo, int tri_gl)
{
    static_assert(!BAND || SCORES_ONLY, "the band mask belongs to the scores-only kernel");
    using G = fused_geom<R, SK, NW>;
    constexpr int F_NT = 64 * NW, F_SR = 32 * NW;
    constexpr int CPR = D / 8;                     // 16-byte chunks per K/V row
    constexpr int TILE = F_BK * D;                 // elements per K or V block
    constexpr int ROUNDS = TILE / 8 / F_NT;        // copy instructions per block per lane
    constexpr int KS = D / 32;                     // contraction steps over the head dim
    constexpr int DB = D / 16;                     // 16-wide blocks of the head dim
    constexpr int NCB = F_BK / 16;                 // 16-key blocks per iteration
    static_assert(ROUNDS >= 1, "block smaller than one copy round");

    // Every buffer is an array of its own, and the key-block loop body is instantiated once per K/V buffer: the
    // compiler then sees that LDS reads never touch the asynchronous copy in flight into the other buffer.  With one
    // block of dynamic LDS it cannot, and waits for the copy ahead of the first LDS read that follows its issue.
    // The scores-only kernel double-buffers K in B0 / B1.  The attention kernel rotates K and V through three
    // buffers: in an iteration K(j) sits in one, V(j) in another; K(j+1) is copied into the third from the top of the
    // iteration on, and V(j+1) into K(j)'s buffer once the score phase is over (the barrier in the middle of the
    // iteration).  Three 16 KB buffers and the score tile are 68 KB: two workgroups per CU, which overlap each
    // other's vector-ALU and matrix-core phases (a single workgroup's wavefronts meet at two barriers per key block
    // and are all in the same phase at the same time).
    __shared__ __align__(16) T B0[TILE];
    __shared__ __align__(16) T B1[TILE];
    __shared__ __align__(16) T B2[SCORES_ONLY ? 8 : TILE];
    __shared__ __align__(16) T Sc[F_SR * F_SLD];                          // score tile
    // zero-padded kernel rows, only needed until the Toeplitz fragments are built: they borrow a buffer that
    // receives its first copy after that (LDS is granted in 1280-byte units; the array's own 648 bytes were the
    // difference between two and three workgroups per CU for the scores-only kernel)
    static_assert(R * G::WZ_LD <= TILE, "kernel rows do not fit the borrowed buffer");
    T *const wz = SCORES_ONLY ? B1 : B2;

    const int tid = threadIdx.x;
    // (the wavefront index through readfirstlane: everything derived from it is then scalar, branches included)
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, ln = lane & 15, kg = lane >> 4;
    // XCD-aware order: workgroup ids are dealt round-robin to the 8 XCDs, so XCD x takes the x-th eighth of the
    // (batch*head, query block) list: the workgroups sharing one head's K and V run on one L2.  Within a head
    // the longest (last) query blocks come first.
    // When the (batch, head) pairs divide evenly over the XCDs (hpx > 0 of them each), the items of an XCD's heads are
    // taken rank by rank - the longest item of each head, then the second longest of each, ... - so that the long items
    // all start early and the short ones fill the end of the grid (workgroups start in index order as slots free up).
    int64_t lid = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (lid >= total_wg) return;
    if (hpx > 0) {
        const int64_t pos = blockIdx.x >> 3;
        lid = ((int64_t)(blockIdx.x & 7) * hpx + pos % hpx) * items_per_bh + pos / hpx;
    }
    // Work item = (batch*head, query block, chunk of jc_len key blocks).  The scores-only kernel splits the key
    // range of a query block (its output columns are independent; a chunk starts one key block early to rebuild
    // the retained halo columns), so that items are short and equal and the grid runs in several even rounds;
    // the attention kernel accumulates over all keys and gets jc_len = all of them.
    const int64_t bh = lid / items_per_bh;
    int item = (int)(lid % items_per_bh), qb = nqb - 1, jc = 0;
    int tbl_lo = -1, tbl_len = 0;
    if (tbl.n > 0) {
        const unsigned e = tbl.e[item];
        qb = (int)(e & 2047u);
        tbl_lo = (int)((e >> 11) & 2047u);
        tbl_len = (int)(e >> 22);
    } else {
        for (; qb > 0; --qb) {  // longest query blocks first
            const int ql = (qb * G::BQ + G::BQ - 1 < S - 1) ? qb * G::BQ + G::BQ - 1 : S - 1;
            const int nch = ((causal ? ql / F_BK : (S - 1) / F_BK) + jc_len) / jc_len;
            if (item < nch) break;
            item -= nch;
        }
        jc = item;
    }
    const int head = (int)(bh % H);
    const int q0 = qb * G::BQ;
    const T *Qp = Q + bh * (int64_t)S * D;
    const T *Kp = K + bh * (int64_t)S * D;
    const T *Vp = SCORES_ONLY ? Kp : V + bh * (int64_t)S * D;
    // (scores only, tri_gl > 0: the scores go out in the triangular layout, groups of tri_gl heads interleaved by rows;
    // nothing above the diagonal is stored then)
    const bool tri = SCORES_ONLY && tri_gl > 0;
    T *Op = tri ? O + (bh / (tri ? tri_gl : 1)) * ((tri ? tri_gl : 1) * tri_rowoff(S)) : O + bh * (int64_t)S * (SCORES_ONLY ? S : D);
    const int tri_i = tri ? (int)(bh % tri_gl) : 0;

    // asynchronous copy of key block j into buffer `buf`: K rows cb.., V rows j*BK..; out-of-range keys
    // re-read a valid row (their scores are zeroed / their probabilities are 0 later)
    // slot r*512+tid of a block is row kv_row[r], 16-byte chunk kv_c of that row (fixed per lane)
    // (a round advances the row by F_NT/CPR, a multiple of CPR: the swizzled chunk is the same in every round)
    static_assert((F_NT / CPR) % CPR == 0 && F_NT % CPR == 0, "copy rounds must keep the swizzle phase");
    const int kv_row0 = tid / CPR;
    const int kv_off0 = kv_row0 * D + ((tid % CPR) ^ (kv_row0 & (CPR - 1))) * 8;
    // V blocks use the swizzle that keeps the transpose reads free of bank conflicts (it only depends on key bits
    // below 4, which a copy round does not change either)
    static_assert((F_NT / CPR) % 16 == 0, "copy rounds must keep the V swizzle phase");
    const int v_off0 = kv_row0 * D + ((tid % CPR) ^ v_swizzle4<D>(kv_row0)) * 8;
    auto issue_k = [&](int j, T *Kdst) {
        const int cb = j * F_BK + G::PWR;
        const bool inside = cb >= 0 && cb + F_BK <= S;  // no key needs clamping
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int kv_row = kv_row0 + r * (F_NT / CPR), kv_off = kv_off0 + r * (F_NT / CPR) * D;
            int koff = cb * D + kv_off;
            if (!inside) {
                int kr = cb + kv_row;
                kr = kr < 0 ? 0 : (kr >= S ? S - 1 : kr);
                koff = kv_off + (kr - kv_row) * D;
            }
            __builtin_amdgcn_global_load_lds((glb_void_t *)(Kp + koff),
                                             (lds_void_t *)(Kdst + (r * F_NT + wave * 64) * 8), 16, 0, 0);
        }
    };
    auto issue_v = [&](int j, T *Vdst) {
        const bool inside = j >= 0 && (j + 1) * F_BK <= S;
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int kv_row = kv_row0 + r * (F_NT / CPR), v_off = v_off0 + r * (F_NT / CPR) * D;
            int voff = j * F_BK * D + v_off;
            if (!inside) {
                int vr = j * F_BK + kv_row;
                vr = vr < 0 ? 0 : (vr >= S ? S - 1 : vr);
                voff = v_off + (vr - kv_row) * D;
            }
            __builtin_amdgcn_global_load_lds((glb_void_t *)(Vp + voff),
                                             (lds_void_t *)(Vdst + (r * F_NT + wave * 64) * 8), 16, 0, 0);
        }
    };

    const int q_last = (q0 + G::BQ - 1 < S - 1) ? q0 + G::BQ - 1 : S - 1;
    const int j_last = causal ? q_last / F_BK : (S - 1) / F_BK;  // last key block of the query block
    int j_lo = tbl_lo >= 0 ? tbl_lo : jc * jc_len;                // first key block whose outputs this item produces
    const int j_len = tbl_lo >= 0 ? tbl_len : jc_len;
    const int j_end = (j_lo + j_len - 1 < j_last) ? j_lo + j_len - 1 : j_last;
    if constexpr (BAND) {
        // Key blocks that lie wholly ahead of the first key any row of this query block sees are skipped: no visible
        // position takes a tap from them, and what they would hold is hidden from every row (left unwritten).  Every
        // wavefront reduces all the rows (the same answer in each: no exchange).
        const int64_t brow = (bh / H) * (int64_t)S;
        int fmin = S;
        for (int r = lane; r < G::BQ + G::HR; r += 64) {
            const int p = q0 - G::HR + r;
            if (p >= 0 && p < S) {
                const int f = band_lo[brow + p];
                fmin = f < fmin ? f : fmin;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const int o = __shfl_xor(fmin, off);
            fmin = o < fmin ? o : fmin;
        }
        fmin = __builtin_amdgcn_readfirstlane(fmin);
        const int j_first = (fmin > 0 ? fmin : 0) / F_BK;
        if (j_first > j_lo) j_lo = j_first;
        if (j_lo > j_end) return;
    }
    // one key block earlier only fills the retained score columns (before the first one: the right pad, if any)
    const int j_start = j_lo > 0 ? j_lo - 1 : (G::PWR > 0 ? -1 : 0);
    issue_k(j_start, B0);
    if (!SCORES_ONLY) issue_v(j_start, B1);

    // zero the score tile once (columns past HC+BK are read by the last window but never written)
    for (int e = tid; e < F_SR * F_SLD / 8; e += F_NT) {
        pack16<T> z;
#pragma unroll
        for (int u = 0; u < 8; ++u) z.v[u] = from_float<T>(0.0f);
        *reinterpret_cast<pack16<T> *>(Sc + e * 8) = z;
    }
    for (int e = tid; e < R * G::WZ_LD; e += F_NT) {
        const int i = e / G::WZ_LD, jj = e % G::WZ_LD - G::WZ_OFF;
        const bool ok = jj >= 0 && jj < SK;
        const T wv = Wt[head * R * SK + (ok ? i * SK + jj : 0)];
        wz[e] = ok ? wv : from_float<T>(0.0f);
    }

    // this lane's two query rows
    int trow[2], prow[2];
    frag8<T> qf[2][KS];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        trow[rb] = wave * 32 + rb * 16 + ln;
        prow[rb] = q0 - G::HR + trow[rb];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int pc = prow[rb] < 0 ? 0 : (prow[rb] >= S ? S - 1 : prow[rb]);
            qf[rb][ks] = *reinterpret_cast<const frag8<T> *>(Qp + (int64_t)pc * D + ks * 32 + kg * 8);
            if (prow[rb] < 0 || prow[rb] >= S) qf[rb][ks] = zero_frag<T>();  // rows outside the sequence are conv padding
        }
    }
    // band mask: first visible key of this lane's two rows, and the largest of them over the wavefront's 32 rows (a key
    // block that starts at or beyond it is visible to all of them)
    int flo[2] = {0, 0}, fmax_w = 0;
    if constexpr (BAND) {
        const int64_t brow = (bh / H) * (int64_t)S;
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) flo[rb] = (prow[rb] >= 0 && prow[rb] < S) ? band_lo[brow + prow[rb]] : 0;
        int m = flo[0] > flo[1] ? flo[0] : flo[1];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const int o = __shfl_xor(m, off);
            m = o > m ? o : m;
        }
        fmax_w = __builtin_amdgcn_readfirstlane(m);
    }
    __syncthreads();

    // Toeplitz fragments T_i^T: accumulator row m = ln, slots k = 8*kg + t, tap = k - SHIFT - m
    frag8<T> tz[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const T *src = wz + i * G::WZ_LD + G::WZ_OFF + kg * 8 - G::SHIFT - ln;
#pragma unroll
        for (int t = 0; t < 8; ++t) tz[i].v[t] = src[t];
    }

    f32x4 oacc[2][DB];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int db = 0; db < DB; ++db) oacc[rb][db] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_i[2] = {-INFINITY, -INFINITY}, l_i[2] = {0.0f, 0.0f};

    // retained columns: each thread moves one 16-byte vector per round (HC/8 vectors per row)
    constexpr int TAIL_VECS = F_SR * (G::HC / 8);
    constexpr int TAIL_IT = (TAIL_VECS + F_NT - 1) / F_NT;

    int tail_off[TAIL_IT > 0 ? TAIL_IT : 1];  // element offset of this thread's retained vector(s) in the tile's head
#pragma unroll
    for (int it = 0; it < TAIL_IT; ++it) {
        constexpr int VPRW = G::HC / 8 > 0 ? G::HC / 8 : 1;
        const int idx = it * F_NT + tid;
        tail_off[it] = idx < TAIL_VECS ? (idx / VPRW) * F_SLD + (idx % VPRW) * 8 : -1;
    }
    // the two 16-row blocks of this wavefront span rows pmin..pmin+31 of the sequence
    const int pmin = q0 - G::HR + wave * 32;
    // Rows of the conv (and of everything after it: softmax, P V, the stores).  The first wavefront's rows are taken
    // R-1 further down than the rows it computes scores for: its conv windows then start at tile row 0 instead of
    // above the tile, every fragment address is the same affine function of (row block, kernel row), and what it
    // leaves out are halo rows nobody stores.  Its last R-1 rows belong to the second wavefront too and are not
    // stored from here.
    const int cshift = wave == 0 ? R - 1 : 0;
    int cprow[2];
    bool row_stored[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        const int tr_ = trow[rb] + cshift;
        cprow[rb] = prow[rb] + cshift;
        row_stored[rb] = tr_ >= G::HR && tr_ < wave * 32 + 32 && cprow[rb] < S;
    }

    // PLAIN: the key block (its scores and its conv outputs) lies inside the sequence and on or below the diagonal
    // for all 32 rows of this wavefront: no masks and no per-sub-block tests (most blocks of a long sequence)
    auto block = [&](auto plain_tag, int j, const T *Kb, const T *Vb, T *Kn, T *Vn) __attribute__((always_inline)) {
        constexpr bool PLAIN = decltype(plain_tag)::value;
        const int cbase = j * F_BK + G::PWR;  // first key of the new score block
        // (a vector type, read by every lane: a struct read under a lane condition travels through scratch memory)
        u32x4_t tailreg[TAIL_IT > 0 ? TAIL_IT : 1];
#pragma unroll
        for (int it = 0; it < TAIL_IT; ++it)
            tailreg[it] = *reinterpret_cast<const u32x4_t *>(Sc + (tail_off[it] >= 0 ? tail_off[it] : 0) + F_BK);
        __builtin_amdgcn_s_waitcnt(0);  // this wavefront's part of block j has landed in LDS
        __syncthreads();                // ... and everybody's; all reads of the previous tiles are done
        // (Leaving the previous iteration's result stores in flight here - vmcnt(number of stores) instead of 0 - was
        // measured: no gain.)
#pragma unroll
        for (int it = 0; it < TAIL_IT; ++it)
            if (tail_off[it] >= 0) *reinterpret_cast<u32x4_t *>(Sc + tail_off[it]) = tailreg[it];
        if (j < j_end) issue_k(j + 1, Kn);  // lands while this block is being worked on

        // ---- S^T = K Q^T, zero above the diagonal / outside the sequence, to the score tile ----
        {
            // Pipelined like the conv phase below: K fragments are read from assembly KLD steps (one or two 16-key
            // blocks) ahead into a ring of registers, a step being one fragment and the two products it feeds (both row
            // blocks); a block's scores are rounded, scaled, masked and written LAG steps into the next block.
            constexpr int NSTEP = NCB * KS, KLD = SCORES_ONLY ? 2 * KS : KS, KSLOT = KLD + 1, LAG = 2;  // (attention kernel: one block ahead; two spill)
            static_assert(NSTEP > KLD && KS >= LAG && NCB % 2 == 0, "pipeline deeper than the work; blocks are written in pairs");
            unsigned ka[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                ka[ks] = lds_addr(Kb) + (unsigned)((ln * D + (((ks * 4 + kg) ^ (ln & (CPR - 1))) * 8)) * (int)sizeof(T));
            const unsigned wa = lds_addr(Sc) + (unsigned)((trow[0] * F_SLD + G::HC + (kg & 1) * 16 + (kg >> 1) * 8) * (int)sizeof(T));
            u32x4_t kring[KSLOT];
            f32x4 sacc[2][2];
            uint32_t held[2][2];
            auto kissue = [&](auto ic) __attribute__((always_inline)) {
                constexpr int n = decltype(ic)::value;
                kring[n % KSLOT] = lds_read16_at(ka[n % KS], (n / KS) * 16 * D * (int)sizeof(T));
            };
            auto epilogue = [&](auto cbc) __attribute__((always_inline)) {
                constexpr int cb = decltype(cbc)::value;
                // key block wholly inside the sequence and on or below the diagonal for all 32 rows: no masks
                const bool s_plain = PLAIN || (cbase + cb * 16 >= 0 && cbase + cb * 16 + 16 <= S && (!causal || cbase + cb * 16 + 15 <= pmin) &&
                                               (!BAND || cbase + cb * 16 >= fmax_w));
#pragma unroll
                for (int rb = 0; rb < 2; ++rb) {
                    const f32x4 a = sacc[cb & 1][rb];
                    uint32_t lo = pack2<T>(a[0], a[1]), hi = pack2<T>(a[2], a[3]);
                    if (SCORES_ONLY) {  // MTA scales the scores before the conv, in the I/O dtype: round, scale, round again
                        float a0, a1, a2, a3;
                        unpack2<T>(lo, a0, a1);
                        unpack2<T>(hi, a2, a3);
                        lo = pack2<T>(a0 * scale, a1 * scale);
                        hi = pack2<T>(a2 * scale, a3 * scale);
                    }
                    if (!s_plain) {
                        MTA_KEEP_BRANCH();
                        const int col = cbase + cb * 16 + kg * 4;
                        const int lim = causal ? (prow[rb] < S - 1 ? prow[rb] : S - 1) : S - 1;  // last key kept
                        const int first = BAND ? (flo[rb] > 0 ? flo[rb] : 0) : 0;  // first key kept
                        if (col < first || col > lim) lo &= 0xffff0000u;
                        if (col + 1 < first || col + 1 > lim) lo &= 0x0000ffffu;
                        if (col + 2 < first || col + 2 > lim) hi &= 0xffff0000u;
                        if (col + 3 < first || col + 3 > lim) hi &= 0x0000ffffu;
                    }
                    // Two 16-key blocks go to the tile together.  A lane holds keys 4kg..4kg+3 of each; after the
                    // exchange between neighbouring lane groups (even groups give their second block's part and take
                    // the neighbour's first block's part) it holds 8 consecutive keys of one block: one 16-byte write
                    // per lane and block pair instead of two 8-byte ones, which conflicted four ways in the banks.
                    if constexpr ((cb & 1) == 0) {
                        held[rb][0] = lo;
                        held[rb][1] = hi;
                    } else {
                        const u32x2_t s0 = __builtin_amdgcn_permlane16_swap(held[rb][0], lo, false, false);
                        const u32x2_t s1 = __builtin_amdgcn_permlane16_swap(held[rb][1], hi, false, false);
                        lds_write16_at(wa, (rb * 16 * F_SLD + (cb - 1) * 16) * (int)sizeof(T), u32x4_t{s0[0], s1[0], s0[1], s1[1]});
                    }
                }
            };
            static_for<KLD>(kissue);
            static_for<NSTEP>([&](auto ic) __attribute__((always_inline)) {
                constexpr int n = decltype(ic)::value;
                constexpr int cb = n / KS, ks = n % KS;
                if constexpr (n + KLD < NSTEP) kissue(std::integral_constant<int, n + KLD>{});
                // LDS operations younger than read n: the reads issued after it and the score writes issued since
                constexpr int younger = (n + KLD < NSTEP ? n + KLD : NSTEP - 1) - n + score_writes_between(n > KLD ? n - KLD : 0, n, KS, NCB, LAG);
                lds_wait_upto<(younger < 15 ? younger : 15)>(kring[n % KSLOT]);
                if constexpr (ks == 0) {
                    sacc[cb & 1][0] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                    sacc[cb & 1][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                }
                mma16(sacc[cb & 1][0], __builtin_bit_cast(frag8<T>, kring[n % KSLOT]), qf[0][ks]);
                mma16(sacc[cb & 1][1], __builtin_bit_cast(frag8<T>, kring[n % KSLOT]), qf[1][ks]);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (cb >= 1 && ks == LAG - 1) {
                    epilogue(std::integral_constant<int, cb - 1>{});
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            epilogue(std::integral_constant<int, NCB - 1>{});
        }
        // score tile complete for everybody.  Only the LDS counter is waited for: a fence would also wait for the
        // copy of the next key block, in flight since the top of the iteration
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        // (attention kernel: nobody reads K(j) any more, the next V block may land in its buffer)
        if (!SCORES_ONLY && j < j_end) issue_v(j + 1, Vn);
        if (j < j_lo) return;

        // ---- conv (Toeplitz MFMAs over the score tile) -> global (scores only) / -> online softmax ----
        // One product needs one fresh 1 KB score fragment from LDS, and a wavefront that waits for each fragment
        // where it is used spends four times the products' own time here.  The reads are therefore issued NLD
        // products ahead, from assembly (see lds_read16_at), into a ring of registers; every product is preceded by
        // a wait that leaves exactly the younger operations outstanding.  The result of an output block is taken up
        // LAG products into the next block, when it is long complete.
        constexpr int NB = 2 * NCB, NREAD = NB * R;
        // score fragments in flight (scores only: 8 and 12 measure the same, 15 spills; the attention kernel, at the
        // 256-register limit, spills from 6 on)
        constexpr int NLD = SCORES_ONLY ? 8 : 4;
        constexpr int NSLOT = NLD + 1;
        constexpr int LAG = 2;
        static_assert(NREAD > NLD && R >= LAG && NLD <= 15, "pipeline deeper than the work or than the counter");
        const unsigned xa = lds_addr(Sc) + (unsigned)(((trow[0] + cshift - (R - 1)) * F_SLD + kg * 8) * (int)sizeof(T));
        u32x4_t ring[NSLOT];
        f32x4 cacc[2];
        auto issue = [&](auto ic) __attribute__((always_inline)) {
            constexpr int n = decltype(ic)::value;
            constexpr int blk = n / R, i = n % R;
            ring[n % NSLOT] = lds_read16_at(xa, (((blk / NCB) * 16 + i) * F_SLD + (blk % NCB) * 16) * (int)sizeof(T));
        };
        // what happens to output block b = rb*NCB + cb (rows crow[rb], keys j*64 + 16cb ..) once it is complete
        uint32_t held[2];           // scores only: the even block of a pair, packed
        float sv[NCB][4], mloc;     // attention: the row block's scaled logits and their running maximum
        frag8<T> pf[2][2];          // attention: probabilities, in the operand layout of the P V products
        auto finish = [&](auto bc) __attribute__((always_inline)) {
            constexpr int b = decltype(bc)::value;
            constexpr int rb = b / NCB, cb = b % NCB;
            const f32x4 a = cacc[b & 1];
            const int p_ = cprow[rb];
            if constexpr (SCORES_ONLY) {
                // Blocks leave in pairs, like the scores above: after the exchange a lane holds 8 consecutive keys of
                // one of the two blocks and stores them itself, 16 rows x 64 bytes per instruction; no staging through LDS.
                // (Ordinary stores: a 128-byte line is completed by two instructions a few hundred cycles apart, and the L2
                // merges them.  Marked non-temporal, each 64-byte half went to memory on its own and the write counter
                // read 1.38 times the bytes; the price of the merge is that the scores displace some of the head's K blocks
                // from the L2 - fetches 79 -> 196 MB per launch at the benchmark shape, 825 -> 736 MB in total, 4 % faster.)
                uint32_t lo = pack2<T>(a[0], a[1]), hi = pack2<T>(a[2], a[3]);
                if (!PLAIN && causal && j * F_BK + cb * 16 + 15 > pmin) {  // block touches the diagonal for some row
                    const int col = j * F_BK + cb * 16 + kg * 4;
                    if (col > p_) lo &= 0xffff0000u;
                    if (col + 1 > p_) lo &= 0x0000ffffu;
                    if (col + 2 > p_) hi &= 0xffff0000u;
                    if (col + 3 > p_) hi &= 0x0000ffffu;
                }
                if constexpr ((cb & 1) == 0) {
                    held[0] = lo;
                    held[1] = hi;
                } else {
                    const u32x2_t s0 = __builtin_amdgcn_permlane16_swap(held[0], lo, false, false);
                    const u32x2_t s1 = __builtin_amdgcn_permlane16_swap(held[1], hi, false, false);
                    // (column from a laundered lane index: the address is then formed here, 64-bit adds and all, instead
                    // of being kept in registers across the key-block loop - the kernel is at its register limit)
                    const int kg_o = opaque_lane(kg);
                    const int col = j * F_BK + (cb - 1 + (kg_o & 1)) * 16 + (kg_o >> 1) * 8;
                    if (row_stored[rb] && (PLAIN || (col < S && (!causal || fill_upper || col <= p_)))) {
                        // (triangular layout: the row's start from a laundered row number, for the same reason)
                        T *dst = tri ? Op + (tri_row_start(opaque_lane(p_), tri_gl, tri_i) + (unsigned)col) : Op + (int64_t)p_ * S + col;
                        *reinterpret_cast<u32x4_t *>(dst) = u32x4_t{s0[0], s1[0], s0[1], s1[1]};
                    }
                }
            } else {
                // conv output and scaled logits are rounded to the I/O dtype, as the unfused pipeline stores them
                float v4[4];
                unpack2<T>(pack2<T>(a[0], a[1]), v4[0], v4[1]);
                unpack2<T>(pack2<T>(a[2], a[3]), v4[2], v4[3]);
                unpack2<T>(pack2<T>(v4[0] * scale, v4[1] * scale), v4[0], v4[1]);
                unpack2<T>(pack2<T>(v4[2] * scale, v4[3] * scale), v4[2], v4[3]);
                const bool c_plain = PLAIN || (j * F_BK + cb * 16 + 16 <= S && (!causal || j * F_BK + cb * 16 + 15 <= pmin));
                if constexpr (cb == 0) mloc = -INFINITY;
                if (!c_plain) {
                    MTA_KEEP_BRANCH();
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int col = j * F_BK + cb * 16 + kg * 4 + v;
                        if (!(col < S && !(causal && col > p_))) v4[v] = -INFINITY;
                    }
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    sv[cb][v] = v4[v];
                    mloc = fmaxf(mloc, v4[v]);
                }
                if constexpr (cb == NCB - 1) {  // the row block is complete: online softmax (a row lives in 4 lanes)
                    mloc = max_across_groups(mloc);
                    const float m_new = fmaxf(m_i[rb], mloc);
                    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
                    // exp(x - m) = exp2(x*log2(e) - m*log2(e)): one multiply-add and one v_exp per element
                    constexpr float LOG2E = 1.4426950408889634f;
                    const float mneg = -m_use * LOG2E;
                    const float alpha = __builtin_amdgcn_exp2f(fmaf(m_i[rb], LOG2E, mneg));
                    m_i[rb] = m_new;
                    float lsum = 0.0f;
                    const uint32_t ones = pack2<T>(1.0f, 1.0f);
#pragma unroll
                    for (int c = 0; c < NCB; ++c) {
                        float e[4];
#pragma unroll
                        for (int v = 0; v < 4; ++v) e[v] = __builtin_amdgcn_exp2f(fmaf(sv[c][v], LOG2E, mneg));
                        const uint32_t lo = pack2<T>(e[0], e[1]), hi = pack2<T>(e[2], e[3]);
                        // the row sum runs over the rounded probabilities (what the P V products see): a packed dot
                        // product with (1, 1) adds a pair in one instruction
                        lsum = dot2_io<T>(lo, ones, lsum);
                        lsum = dot2_io<T>(hi, ones, lsum);
                        uint32_t *dst = reinterpret_cast<uint32_t *>(&pf[rb][c >> 1]) + (c & 1) * 2;
                        dst[0] = lo;
                        dst[1] = hi;
                    }
                    l_i[rb] = l_i[rb] * alpha + lsum;
                    // (once the running maxima have settled, alpha is 1 in every lane for most key blocks: the 4*DB
                    // multiplications are skipped for the wavefront then)
                    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
                        for (int db = 0; db < DB; ++db) oacc[rb][db] *= alpha;
                    }
                }
            }
        };
        static_for<NLD>(issue);
        static_for<NREAD>([&](auto ic) __attribute__((always_inline)) {
            constexpr int n = decltype(ic)::value;
            constexpr int blk = n / R, i = n % R;
            if constexpr (n + NLD < NREAD) issue(std::integral_constant<int, n + NLD>{});
            // LDS operations younger than read n: exactly the reads issued after it
            constexpr int younger = (n + NLD < NREAD ? n + NLD : NREAD - 1) - n;
            lds_wait_upto<younger>(ring[n % NSLOT]);
            if constexpr (i == 0) cacc[blk & 1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            mma16(cacc[blk & 1], tz[i], __builtin_bit_cast(frag8<T>, ring[n % NSLOT]));
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (blk >= 1 && i == LAG - 1) {
                finish(std::integral_constant<int, blk - 1>{});
                __builtin_amdgcn_sched_barrier(0);
            }
        });
        finish(std::integral_constant<int, NB - 1>{});
        if constexpr (SCORES_ONLY) return;

        // ---- O^T += V^T P^T ; V^T fragments via the LDS transpose read of the row-major V block ----
        {
            // slots 0..3: keys 32ks+4kg+(0..3); slots 4..7: keys 32ks+16+4kg+(0..3) -- the order of pf
            frag8<T> vf[2];
            auto load_vf = [&](int blk, frag8<T> &dst) {  // blk = ks * DB + db
                const int ks = blk / DB, db = blk % DB;
                const int key_a = ks * 32 + kg * 4 + (ln >> 2), key_b = key_a + 16;
                const int ch = db * 2 + ((ln & 3) >> 1);  // 16-byte chunk holding head dims 16db+4(ln%4)..
                const int sub = (ln & 1) * 4;             // element offset inside the chunk
                const T *pa = Vb + key_a * D + ((ch ^ v_swizzle4<D>(key_a)) * 8) + sub;
                const T *pb = Vb + key_b * D + ((ch ^ v_swizzle4<D>(key_b)) * 8) + sub;
                struct { v4s_t a, b; } both = {__builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)pa),
                                               __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)pb)};
                dst = __builtin_bit_cast(frag8<T>, both);
            };
            load_vf(0, vf[0]);
#pragma unroll
            for (int blk = 0; blk < 2 * DB; ++blk) {
                const int ks = blk / DB, db = blk % DB;
                if (blk + 1 < 2 * DB) load_vf(blk + 1, vf[(blk + 1) & 1]);
                mma16(oacc[0][db], vf[blk & 1], pf[0][ks]);
                mma16(oacc[1][db], vf[blk & 1], pf[1][ks]);
            }
        }
    };
    auto plain = [&](int j) {  // (scores-only kernel: a second body per buffer rotation makes the attention kernel spill)
        const int cbase = j * F_BK + G::PWR;
        return SCORES_ONLY && j >= 0 && cbase + F_BK <= S && (!causal || cbase + F_BK - 1 <= pmin) && (!BAND || cbase >= fmax_w);
    };
    if constexpr (SCORES_ONLY) {
        for (int j = j_start;;) {  // block(tag, j, K(j), V(j), where K(j+1) goes, where V(j+1) goes)
            if (plain(j)) block(std::true_type{}, j, B0, B0, B1, B1);
            else block(std::false_type{}, j, B0, B0, B1, B1);
            if (++j > j_end) break;
            if (plain(j)) block(std::true_type{}, j, B1, B1, B0, B0);
            else block(std::false_type{}, j, B1, B1, B0, B0);
            if (++j > j_end) break;
        }
    } else {
        for (int j = j_start;;) {
            block(std::false_type{}, j, B0, B1, B2, B0);
            if (++j > j_end) break;
            block(std::false_type{}, j, B2, B0, B1, B2);
            if (++j > j_end) break;
            block(std::false_type{}, j, B1, B2, B0, B1);
            if (++j > j_end) break;
        }
    }

    if constexpr (SCORES_ONLY) {
        // +0 for the key blocks to the right of the last one visited (all above the diagonal)
        if (causal && fill_upper && j_end == j_last) {
            pack16<T> z;
#pragma unroll
            for (int u = 0; u < 8; ++u) z.v[u] = from_float<T>(0.0f);
            const int c_first = (j_end + 1) * F_BK;
            const int vec_per_row = (S - c_first + 7) / 8;
            for (int r = wave; r < G::BQ; r += F_NT / 64) {
                const int p_ = q0 + r;
                if (p_ >= S) break;
                for (int vc = lane; vc < vec_per_row; vc += 64) {
                    const int col = c_first + vc * 8;
                    if (col < S) *reinterpret_cast<pack16<T> *>(Op + (int64_t)p_ * S + col) = z;
                }
            }
        }
        return;
    }
    // ---- normalise and store (halo rows are dropped) ----
    // (row and column from a lane index counted afresh: the store addresses are then formed here, after the key-block
    // loop, and nothing has to be kept - or spilled - across the loop for them)
    const int lane_e = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const int ln_o = lane_e & 15, kg_o = lane_e >> 4;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        const float l_row = sum_across_groups(l_i[rb]);
        const int tr_ = wave * 32 + rb * 16 + ln_o + cshift, p_ = q0 - G::HR + tr_;
        if (tr_ >= G::HR && tr_ < wave * 32 + 32 && p_ < S) {
            const float inv = 1.0f / l_row;
            if (Lse != nullptr && kg_o == 0) Lse[bh * (int64_t)S + p_] = m_i[rb] + __logf(l_row);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const uint32_t lo = pack2<T>(oacc[rb][db][0] * inv, oacc[rb][db][1] * inv);
                const uint32_t hi = pack2<T>(oacc[rb][db][2] * inv, oacc[rb][db][3] * inv);
                *reinterpret_cast<uint2 *>(Op + (int64_t)p_ * D + db * 16 + kg_o * 4) = make_uint2(lo, hi);
            }
        }
    }
}

template <typename T, int D, int R, int SK, bool SCORES_ONLY, bool BAND = false>
int launch_mfma(const void *q, const void *k, const void *v, const void *w, void *o, float *lse, int64_t B, int64_t H,
                int64_t S, int causal, float scale, int fill_upper, hipStream_t st, const int *band_lo = nullptr, int tri_gl = 0)
{
    constexpr int NW = 4;
    constexpr int F_NT = 64 * NW;
    using G = fused_geom<R, SK, NW>;
    static_assert(G::fits, "conv window exceeds the 32-key MFMA contraction");
    const int nqb = (int)((S + G::BQ - 1) / G::BQ);
    auto kern = conv_attn_fwd_mfma<T, D, R, SK, SCORES_ONLY, NW, BAND>;
    // key blocks per work item: all of them for the attention kernel; QK_CHUNK for the scores-only kernel
    const int jc_len = SCORES_ONLY ? QK_CHUNK : (int)((S + F_BK - 1) / F_BK) + 1;
    int64_t items_per_bh = 0;
    for (int qb = 0; qb < nqb; ++qb) {
        const int64_t ql = std::min<int64_t>((int64_t)qb * G::BQ + G::BQ - 1, S - 1);
        items_per_bh += ((causal ? ql / F_BK : (S - 1) / F_BK) + jc_len) / jc_len;
    }
    // the items of a head, longest first (the number of key blocks an item visits, as the kernel computes it)
    item_table tbl;
    tbl.n = 0;
    if (SCORES_ONLY && nqb <= 2047 && (S + F_BK - 1) / F_BK <= 2047) {
        constexpr int MAXLEN = 1023;
        static thread_local int count[MAXLEN + 2];
        static thread_local uint32_t items[ITEM_TABLE_MAX];
        static thread_local int lens[ITEM_TABLE_MAX];
        // long chunks for the first part of a query block's key range, short ones for the last QK_SHORT_SHARE of it
        static const int big = [] { const char *e = getenv("MTA_QK_CHUNK_LONG"); return e ? atoi(e) : QK_CHUNK_LONG; }();
        static const int small = [] { const char *e = getenv("MTA_QK_CHUNK_SHORT"); return e ? atoi(e) : QK_CHUNK_SHORT; }();
        static const int share = [] { const char *e = getenv("MTA_QK_SHORT_PERCENT"); return e ? atoi(e) : QK_SHORT_PERCENT; }();
        int n = 0;
        bool ok = big >= 1 && small >= 1 && big <= MAXLEN && small <= MAXLEN && share >= 0 && share <= 100;
        for (int qb = 0; qb < nqb && ok; ++qb) {
            const int64_t ql = std::min<int64_t>((int64_t)qb * G::BQ + G::BQ - 1, S - 1);
            const int nk = (int)(causal ? ql / F_BK : (S - 1) / F_BK) + 1;  // key blocks 0 .. j_last
            const int nshort = std::min(nk, (nk * share / 100 + small / 2) / small * small);
            const int nlong = nk - nshort;
            for (int j0 = 0; j0 < nk && ok;) {
                const int len = j0 < nlong ? std::min(big, nlong - j0) : std::min(small, nk - j0);
                if (n >= ITEM_TABLE_MAX) { ok = false; break; }
                // what the kernel visits: one key block earlier rebuilds the retained columns (ahead of the first: the right pad)
                lens[n] = len + ((j0 > 0 || G::PWR > 0) ? 1 : 0);
                items[n++] = (uint32_t)qb | ((uint32_t)j0 << 11) | ((uint32_t)len << 22);
                j0 += len;
            }
        }
        if (ok && n > 1) {
            std::fill(count, count + MAXLEN + 2, 0);
            for (int i = 0; i < n; ++i) ++count[lens[i]];
            int pos = 0;
            for (int len = MAXLEN + 1; len >= 0; --len) {  // positions: longer items first
                const int c = count[len];
                count[len] = pos;
                pos += c;
            }
            for (int i = n - 1; i >= 0; --i) tbl.e[count[lens[i]]++] = items[i];  // among equal lengths later query blocks first
            tbl.n = n;
            items_per_bh = n;
        }
    }
    const int64_t total_wg = B * H * items_per_bh, per_xcd = (total_wg + 7) / 8;
    if (per_xcd * 8 > 0x7fffffffLL || items_per_bh > 0x7fffffffLL) return MTA_ERR_SHAPE;
    dim3 grid((unsigned)(per_xcd * 8));
    hipLaunchKernelGGL(kern, grid, dim3(F_NT), 0, st, (const T *)q, (const T *)k, (const T *)v, (const T *)w, (T *)o,
                       lse, (int)S, causal, scale, (int)H, nqb, fill_upper, total_wg, per_xcd, jc_len, (int)items_per_bh,
                       (B * H) % 8 == 0 ? (int)(B * H / 8) : 0, tbl, band_lo, tri_gl);
    return launch_status();
}

// returns 1 when no instantiation covers the kernel size (the caller then uses the general kernel)
template <typename T, int D, bool SCORES_ONLY, bool BAND = false>
int dispatch_mfma(const void *q, const void *k, const void *v, const void *w, void *o, float *lse, int64_t B, int64_t H,
                  int64_t S, int R, int Sk, int causal, float scale, int fill_upper, hipStream_t st, const int *band_lo = nullptr,
                  int tri_gl = 0)
{
    if constexpr (sizeof(T) == 2) {
#define MTA_FUSED_CASE(r, s) \
    if (R == r && Sk == s) return launch_mfma<T, D, r, s, SCORES_ONLY, BAND>(q, k, v, w, o, lse, B, H, S, causal, scale, fill_upper, st, band_lo, tri_gl);
        MTA_FUSED_CASE(3, 3)
        MTA_FUSED_CASE(5, 5)
        MTA_FUSED_CASE(5, 7)
        MTA_FUSED_CASE(6, 11)
        MTA_FUSED_CASE(7, 7)
        // (the 44 registers of its Toeplitz fragments leave the scores kernel two workgroups per CU; the attention
        // kernel, at the register limit with 6 kernel rows, has no such instance and takes the general kernel)
        if constexpr (SCORES_ONLY) { MTA_FUSED_CASE(11, 15) }
#undef MTA_FUSED_CASE
    }
    return 1;
}

template <typename T, int D>
int launch(const void *q, const void *k, const void *v, const void *w, void *o, float *lse, int64_t B, int64_t H,
           int64_t S, int R, int Sk, int causal, float scale, int w_dtype, hipStream_t st)
{
    constexpr int PAD = lds_pad<T>::n;
    const int HR = (R - 1 + 7) & ~7, HC = (Sk - 1 + 7) & ~7;
    const int BQ = SR - HR;
    const int nqb = (int)((S + BQ - 1) / BQ);
    const size_t lds = sizeof(T) * ((size_t)BK * (D + PAD) + (size_t)D * (BK + PAD) + (size_t)SR * (HC + BK + PAD)) +
                       sizeof(float) * (size_t)R * Sk;
    auto kern = conv_attn_fwd_kernel<T, D>;
    if (lds > 160 * 1024) return MTA_ERR_KERNEL_SIZE;
    if (lds > 48 * 1024) {  // per device, so set on every such launch (a cheap host-side call)
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    dim3 grid((unsigned)nqb, (unsigned)(B * H));
    hipLaunchKernelGGL(kern, grid, dim3(NT), lds, st, (const T *)q, (const T *)k, (const T *)v, w, (T *)o, lse, (int)S,
                       R, Sk, causal, scale, w_dtype, (int)H, nqb);
    return launch_status();
}
}  // namespace

extern "C" int mta_conv_attn_fwd_lse(const void *q, const void *k, const void *v, const void *w, void *o, void *lse_out,
                                     int64_t B, int64_t H, int64_t S, int64_t D, int R, int Sk, int causal, float scale,
                                     int io_dtype, int w_dtype, void *stream)
{
    if (!q || !k || !v || !w || !o) return MTA_ERR_NULL;
    float *lse = (float *)lse_out;
    if (lse && !aligned_to(lse, 4)) return MTA_ERR_ALIGN;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (B <= 0 || H <= 0 || S <= 0 || S > (1 << 24) || B * H > 65535) return MTA_ERR_SHAPE;
    if (R < 1 || Sk < 1 || R > MTA_MAX_FUSED_KERNEL_R || Sk > MTA_MAX_FUSED_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
    if (D != 64 && D != 128) return MTA_ERR_HEAD_DIM;
    if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(v, 16) || !aligned_to(o, 16) ||
        !aligned_to(w, dtype_size(w_dtype)))
        return MTA_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    // MTA_FUSED_FORCE_GENERAL=1 in the environment keeps 16-bit inputs on the general kernel (for comparisons)
    static const bool force_general = [] { const char *e = getenv("MTA_FUSED_FORCE_GENERAL"); return e && e[0] == '1'; }();
    const bool fast_ok = io_dtype != MTA_F32 && w_dtype == io_dtype && !force_general;
    MTA_DISPATCH_IO(io_dtype, {
        if (fast_ok) {
            const int rc = D == 64 ? dispatch_mfma<io_t, 64, false>(q, k, v, w, o, lse, B, H, S, R, Sk, causal, scale, 0, st)
                                   : dispatch_mfma<io_t, 128, false>(q, k, v, w, o, lse, B, H, S, R, Sk, causal, scale, 0, st);
            if (rc != 1) return rc;
        }
        if (D == 64) return launch<io_t, 64>(q, k, v, w, o, lse, B, H, S, R, Sk, causal, scale, w_dtype, st);
        return launch<io_t, 128>(q, k, v, w, o, lse, B, H, S, R, Sk, causal, scale, w_dtype, st);
    });
    return MTA_ERR_DTYPE;
}

extern "C" int mta_conv_attn_fwd(const void *q, const void *k, const void *v, const void *w, void *o, int64_t B,
                                 int64_t H, int64_t S, int64_t D, int R, int Sk, int causal, float scale,
                                 int io_dtype, int w_dtype, void *stream)
{
    return mta_conv_attn_fwd_lse(q, k, v, w, o, nullptr, B, H, S, D, R, Sk, causal, scale, io_dtype, w_dtype, stream);
}

// kernel sizes with a scores-only instance (the cases of dispatch_mfma<.., true>)
static bool scores_instance(int R, int Sk)
{
    return (R == 3 && Sk == 3) || (R == 5 && Sk == 5) || (R == 5 && Sk == 7) || (R == 6 && Sk == 11) || (R == 7 && Sk == 7) ||
           (R == 11 && Sk == 15);
}

extern "C" int mta_qk_conv_supported(int64_t S, int64_t D, int R, int Sk, int io_dtype, int w_dtype)
{
    return (io_dtype == MTA_BF16 || io_dtype == MTA_F16) && w_dtype == io_dtype && S > 0 && S % 8 == 0 && (D == 64 || D == 128) &&
                   scores_instance(R, Sk)
               ? 1
               : 0;
}

extern "C" int mta_qk_conv_fwd(const void *q, const void *k, const void *w, void *s_out, int64_t B, int64_t H, int64_t S,
                               int64_t D, int R, int Sk, int causal, float scale, int fill_upper, int io_dtype,
                               int w_dtype, void *stream)
{
    if (!q || !k || !w || !s_out) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (B <= 0 || H <= 0 || S <= 0 || S > (1 << 24) || B * H > 65535) return MTA_ERR_SHAPE;
    if (R < 1 || Sk < 1 || R > MTA_MAX_FUSED_KERNEL_R || Sk > MTA_MAX_FUSED_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
    if (D != 64 && D != 128) return MTA_ERR_HEAD_DIM;
    if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(s_out, 16) || !aligned_to(w, dtype_size(w_dtype)))
        return MTA_ERR_ALIGN;
    if (io_dtype == MTA_F32 || w_dtype != io_dtype || S % 8 != 0) return MTA_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    int rc = 1;
    MTA_DISPATCH_IO(io_dtype, {
        rc = D == 64 ? dispatch_mfma<io_t, 64, true>(q, k, nullptr, w, s_out, nullptr, B, H, S, R, Sk, causal, scale, fill_upper, st)
                     : dispatch_mfma<io_t, 128, true>(q, k, nullptr, w, s_out, nullptr, B, H, S, R, Sk, causal, scale, fill_upper, st);
    });
    // (mta_qk_conv_supported must agree with the dispatch: a kernel size it names always has an instance)
    if (rc == 1 && scores_instance(R, Sk)) return MTA_ERR_KERNEL_SIZE;
    return rc == 1 ? MTA_ERR_UNSUPPORTED : rc;
}

// mta_qk_conv_fwd (causal) / mta_qk_conv_band_fwd (first_visible not NULL) with the scores stored in the triangular
// layout (see tri_rowoff in common.hpp), groups of `group` heads interleaved by rows: B*H*tri_rowoff(S) elements, nothing
// above the diagonal.
extern "C" int mta_qk_conv_tri_fwd(const void *q, const void *k, const void *w, const void *first_visible, void *s_out,
                                   int64_t B, int64_t H, int64_t S, int64_t D, int R, int Sk, float scale, int group,
                                   int io_dtype, int w_dtype, void *stream)
{
    if (!q || !k || !w || !s_out) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (B <= 0 || H <= 0 || S <= 0 || S > (1 << 24) || B * H > 65535) return MTA_ERR_SHAPE;
    if (group <= 0 || H % group != 0) return MTA_ERR_GROUP;
    if (R < 1 || Sk < 1 || R > MTA_MAX_FUSED_KERNEL_R || Sk > MTA_MAX_FUSED_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
    if (D != 64 && D != 128) return MTA_ERR_HEAD_DIM;
    if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(s_out, 16) || !aligned_to(w, dtype_size(w_dtype)) ||
        (first_visible && !aligned_to(first_visible, 4)))
        return MTA_ERR_ALIGN;
    if (io_dtype == MTA_F32 || w_dtype != io_dtype || S % 8 != 0) return MTA_ERR_UNSUPPORTED;
    if ((int64_t)group * tri_rowoff((int)S) > 0x7fffffffLL) return MTA_ERR_UNSUPPORTED;  // (32-bit offsets inside a group)
    hipStream_t st = (hipStream_t)stream;
    const int *lo = (const int *)first_visible;
    int rc = 1;
    MTA_DISPATCH_IO(io_dtype, {
        if (lo)
            rc = D == 64 ? dispatch_mfma<io_t, 64, true, true>(q, k, nullptr, w, s_out, nullptr, B, H, S, R, Sk, 1, scale, 0, st, lo, group)
                         : dispatch_mfma<io_t, 128, true, true>(q, k, nullptr, w, s_out, nullptr, B, H, S, R, Sk, 1, scale, 0, st, lo, group);
        else
            rc = D == 64 ? dispatch_mfma<io_t, 64, true>(q, k, nullptr, w, s_out, nullptr, B, H, S, R, Sk, 1, scale, 0, st, nullptr, group)
                         : dispatch_mfma<io_t, 128, true>(q, k, nullptr, w, s_out, nullptr, B, H, S, R, Sk, 1, scale, 0, st, nullptr, group);
    });
    if (rc == 1 && scores_instance(R, Sk)) return MTA_ERR_KERNEL_SIZE;
    return rc == 1 ? MTA_ERR_UNSUPPORTED : rc;
}

// mta_qk_conv_fwd under a band mask: key k of query row p of batch entry b is visible iff first_visible[b, p] <= k <= p
// (int32, (B, S)); the scores of hidden keys enter the conv as 0.  Causal by construction.
extern "C" int mta_qk_conv_band_fwd(const void *q, const void *k, const void *w, const void *first_visible, void *s_out,
                                    int64_t B, int64_t H, int64_t S, int64_t D, int R, int Sk, float scale, int fill_upper,
                                    int io_dtype, int w_dtype, void *stream)
{
    if (!q || !k || !w || !s_out || !first_visible) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (B <= 0 || H <= 0 || S <= 0 || S > (1 << 24) || B * H > 65535) return MTA_ERR_SHAPE;
    if (R < 1 || Sk < 1 || R > MTA_MAX_FUSED_KERNEL_R || Sk > MTA_MAX_FUSED_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
    if (D != 64 && D != 128) return MTA_ERR_HEAD_DIM;
    if (!aligned_to(q, 16) || !aligned_to(k, 16) || !aligned_to(s_out, 16) || !aligned_to(w, dtype_size(w_dtype)) ||
        !aligned_to(first_visible, 4))
        return MTA_ERR_ALIGN;
    if (io_dtype == MTA_F32 || w_dtype != io_dtype || S % 8 != 0) return MTA_ERR_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const int *lo = (const int *)first_visible;
    int rc = 1;
    MTA_DISPATCH_IO(io_dtype, {
        rc = D == 64 ? dispatch_mfma<io_t, 64, true, true>(q, k, nullptr, w, s_out, nullptr, B, H, S, R, Sk, 1, scale, fill_upper, st, lo)
                     : dispatch_mfma<io_t, 128, true, true>(q, k, nullptr, w, s_out, nullptr, B, H, S, R, Sk, 1, scale, fill_upper, st, lo);
    });
    if (rc == 1 && scores_instance(R, Sk)) return MTA_ERR_KERNEL_SIZE;
    return rc == 1 ? MTA_ERR_UNSUPPORTED : rc;
}
