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
                                                           T *__restrict__ O, int S, int R, int Sk, int causal,
                                                           float scale, int w_dtype, int H, int nqb)
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
typedef __attribute__((address_space(3))) v4s_t lds_v4s_t;

constexpr int F_NT = 512;  // 8 wavefronts
constexpr int F_SR = 256;  // score-tile rows
constexpr int F_BK = 64;   // keys per iteration
constexpr int F_SLD = 88;  // score-tile row stride (elements): 44 dwords, conflict-free 16-byte reads over 16 rows

template <int R, int SK> struct fused_geom {
    static constexpr int HR = (R - 1 + 7) & ~7;    // halo rows above the block (recomputed)
    static constexpr int HC = (SK - 1 + 7) & ~7;   // score columns kept from the previous key block
    static constexpr int BQ = F_SR - HR;           // output rows per workgroup
    static constexpr int PW = (SK - 1) / 2, PWR = SK - 1 - PW;
    static constexpr int SHIFT = HC - (SK - 1);    // first tap's offset in a block's 32-key window
    static constexpr bool fits = SHIFT + 16 + SK - 1 <= 32 && HC + F_BK <= 80;
    static constexpr int WZ_OFF = SHIFT + 16, WZ_LD = WZ_OFF + 32;
};

template <typename T, int D, int R, int SK>
__global__ __launch_bounds__(F_NT, 2) void conv_attn_fwd_mfma(const T *__restrict__ Q, const T *__restrict__ K,
                                                             const T *__restrict__ V, const T *__restrict__ Wt,
                                                             T *__restrict__ O, int S, int causal, float scale, int H,
                                                             int nqb)
{
    using G = fused_geom<R, SK>;
    constexpr int CPR = D / 8;                     // 16-byte chunks per K/V row
    constexpr int TILE = F_BK * D;                 // elements per K or V block
    constexpr int ROUNDS = TILE / 8 / F_NT;        // copy instructions per block per lane
    constexpr int KS = D / 32;                     // contraction steps over the head dim
    constexpr int DB = D / 16;                     // 16-wide blocks of the head dim
    constexpr int NCB = F_BK / 16;                 // 16-key blocks per iteration
    static_assert(ROUNDS >= 1, "block smaller than one copy round");

    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *Kt = reinterpret_cast<T *>(smem_raw);       // [2][TILE]
    T *Vt = Kt + 2 * TILE;                         // [2][TILE]
    T *Sc = Vt + 2 * TILE;                         // [F_SR][F_SLD]
    T *wz = Sc + F_SR * F_SLD;                     // [R][WZ_LD] zero-padded kernel rows

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, ln = lane & 15, kg = lane >> 4;
    const int qb = nqb - 1 - (int)blockIdx.x;      // longest blocks first
    const int64_t bh = blockIdx.y;
    const int head = (int)(bh % H);
    const int q0 = qb * G::BQ;
    const T *Qp = Q + bh * (int64_t)S * D;
    const T *Kp = K + bh * (int64_t)S * D;
    const T *Vp = V + bh * (int64_t)S * D;
    T *Op = O + bh * (int64_t)S * D;

    // asynchronous copy of key block j into buffer `buf`: K rows cb.., V rows j*BK..; out-of-range keys
    // re-read a valid row (their scores are zeroed / their probabilities are 0 later)
    auto issue_kv = [&](int j, int buf) {
        const int cb = j * F_BK + G::PWR;
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int slot = r * F_NT + tid;
            const int row = slot / CPR, c = (slot % CPR) ^ (row & (CPR - 1));
            int kr = cb + row;
            kr = kr < 0 ? 0 : (kr >= S ? S - 1 : kr);
            int vr = j * F_BK + row;
            vr = vr < 0 ? 0 : (vr >= S ? S - 1 : vr);
            __builtin_amdgcn_global_load_lds((glb_void_t *)(Kp + (int64_t)kr * D + c * 8),
                                             (lds_void_t *)(Kt + buf * TILE + (r * F_NT + wave * 64) * 8), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((glb_void_t *)(Vp + (int64_t)vr * D + c * 8),
                                             (lds_void_t *)(Vt + buf * TILE + (r * F_NT + wave * 64) * 8), 16, 0, 0);
        }
    };

    const int q_last = (q0 + G::BQ - 1 < S - 1) ? q0 + G::BQ - 1 : S - 1;
    const int j_end = causal ? q_last / F_BK : (S - 1) / F_BK;
    constexpr int j_start = G::PWR > 0 ? -1 : 0;
    issue_kv(j_start, 0);

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

    int buf = 0;
    for (int j = j_start; j <= j_end; ++j, buf ^= 1) {
        const int cbase = j * F_BK + G::PWR;  // first key of the new score block
        pack16<T> tailreg[TAIL_IT > 0 ? TAIL_IT : 1];
#pragma unroll
        for (int it = 0; it < TAIL_IT; ++it) {
            const int idx = it * F_NT + tid;
            const int row = idx / (G::HC / 8 > 0 ? G::HC / 8 : 1), vc = idx % (G::HC / 8 > 0 ? G::HC / 8 : 1);
            if (idx < TAIL_VECS) tailreg[it] = *reinterpret_cast<const pack16<T> *>(Sc + row * F_SLD + F_BK + vc * 8);
        }
        __builtin_amdgcn_s_waitcnt(0);  // this wavefront's part of block j has landed in LDS
        __syncthreads();                // ... and everybody's; all reads of the previous tiles are done
#pragma unroll
        for (int it = 0; it < TAIL_IT; ++it) {
            const int idx = it * F_NT + tid;
            const int row = idx / (G::HC / 8 > 0 ? G::HC / 8 : 1), vc = idx % (G::HC / 8 > 0 ? G::HC / 8 : 1);
            if (idx < TAIL_VECS) *reinterpret_cast<pack16<T> *>(Sc + row * F_SLD + vc * 8) = tailreg[it];
        }
        if (j < j_end) issue_kv(j + 1, buf ^ 1);  // lands while this block is being worked on

        // ---- S^T = K Q^T, zero above the diagonal / outside the sequence, to the score tile ----
        const T *Kb = Kt + buf * TILE;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            f32x4 sacc[2] = {f32x4{0.0f, 0.0f, 0.0f, 0.0f}, f32x4{0.0f, 0.0f, 0.0f, 0.0f}};
            const int krow = cb * 16 + ln;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int c = (ks * 4 + kg) ^ (krow & (CPR - 1));
                const frag8<T> kf = *reinterpret_cast<const frag8<T> *>(Kb + krow * D + c * 8);
                mma16(sacc[0], kf, qf[0][ks]);
                mma16(sacc[1], kf, qf[1][ks]);
            }
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                struct alignas(8) quad { T v[4]; } out;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int col = cbase + cb * 16 + kg * 4 + v;
                    const bool keep = col >= 0 && col < S && !(causal && col > prow[rb]);
                    out.v[v] = from_float<T>(keep ? sacc[rb][v] : 0.0f);
                }
                *reinterpret_cast<quad *>(Sc + trow[rb] * F_SLD + G::HC + cb * 16 + kg * 4) = out;
            }
        }
        __syncthreads();
        if (j < 0) continue;

        // ---- conv (Toeplitz MFMAs over the score tile), scale, mask, online softmax ----
        frag8<T> pf[2][2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            float sv[NCB][4];
            float mloc = -INFINITY;
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                f32x4 cacc = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    int srow = trow[rb] - (R - 1) + i;
                    srow = srow < 0 ? 0 : srow;  // only halo rows (discarded) can reach above the tile
                    mma16(cacc, tz[i], *reinterpret_cast<const frag8<T> *>(Sc + srow * F_SLD + cb * 16 + kg * 8));
                }
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int col = j * F_BK + cb * 16 + kg * 4 + v;
                    const bool ok = col < S && !(causal && col > prow[rb]);
                    const float val = round_to<T>(round_to<T>(cacc[v]) * scale);
                    sv[cb][v] = ok ? val : -INFINITY;
                    mloc = fmaxf(mloc, sv[cb][v]);
                }
            }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 16));
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
            const float m_new = fmaxf(m_i[rb], mloc);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = __expf(m_i[rb] - m_use);
            m_i[rb] = m_new;
            float lsum = 0.0f;
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const T et = from_float<T>(__expf(sv[cb][v] - m_use));
                    lsum += to_float(et);
                    pf[rb][cb >> 1].v[(cb & 1) * 4 + v] = et;
                }
            l_i[rb] = l_i[rb] * alpha + lsum;
#pragma unroll
            for (int db = 0; db < DB; ++db) oacc[rb][db] *= alpha;
        }

        // ---- O^T += V^T P^T ; V^T fragments via the LDS transpose read of the row-major V block ----
        const T *Vb = Vt + buf * TILE;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            // slots 0..3: keys 32ks+4kg+(0..3); slots 4..7: keys 32ks+16+4kg+(0..3) -- the order of pf
            const int key_a = ks * 32 + kg * 4 + (ln >> 2);
            const int key_b = key_a + 16;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int ch = db * 2 + ((ln & 3) >> 1);           // 16-byte chunk holding head dims 16db+4(ln%4)..
                const int sub = (ln & 1) * 4;                      // element offset inside the chunk
                const T *pa = Vb + key_a * D + ((ch ^ (key_a & (CPR - 1))) * 8) + sub;
                const T *pb = Vb + key_b * D + ((ch ^ (key_b & (CPR - 1))) * 8) + sub;
                const v4s_t va = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)pa);
                const v4s_t vb = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)pb);
                struct { v4s_t a, b; } both = {va, vb};
                const frag8<T> vf = __builtin_bit_cast(frag8<T>, both);
                mma16(oacc[0][db], vf, pf[0][ks]);
                mma16(oacc[1][db], vf, pf[1][ks]);
            }
        }
    }

    // ---- normalise and store (halo rows are dropped) ----
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        float l_row = l_i[rb];
        l_row += __shfl_xor(l_row, 16);
        l_row += __shfl_xor(l_row, 32);
        if (trow[rb] >= G::HR && prow[rb] < S) {
            const float inv = 1.0f / l_row;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                struct alignas(8) quad { T v[4]; } out;
#pragma unroll
                for (int v = 0; v < 4; ++v) out.v[v] = from_float<T>(oacc[rb][db][v] * inv);
                *reinterpret_cast<quad *>(Op + (int64_t)prow[rb] * D + db * 16 + kg * 4) = out;
            }
        }
    }
}

template <typename T, int D, int R, int SK>
int launch_mfma(const void *q, const void *k, const void *v, const void *w, void *o, int64_t B, int64_t H, int64_t S,
                int causal, float scale, hipStream_t st)
{
    using G = fused_geom<R, SK>;
    static_assert(G::fits, "conv window exceeds the 32-key MFMA contraction");
    const int nqb = (int)((S + G::BQ - 1) / G::BQ);
    const size_t lds = sizeof(T) * ((size_t)4 * F_BK * D + (size_t)F_SR * F_SLD + (size_t)R * G::WZ_LD);
    auto kern = conv_attn_fwd_mfma<T, D, R, SK>;
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    dim3 grid((unsigned)nqb, (unsigned)(B * H));
    hipLaunchKernelGGL(kern, grid, dim3(F_NT), lds, st, (const T *)q, (const T *)k, (const T *)v, (const T *)w, (T *)o,
                       (int)S, causal, scale, (int)H, nqb);
    return launch_status();
}

// returns 1 when no instantiation covers the kernel size (the caller then uses the general kernel)
template <typename T, int D>
int dispatch_mfma(const void *q, const void *k, const void *v, const void *w, void *o, int64_t B, int64_t H, int64_t S,
                  int R, int Sk, int causal, float scale, hipStream_t st)
{
#define MTA_FUSED_CASE(r, s) \
    if (R == r && Sk == s) return launch_mfma<T, D, r, s>(q, k, v, w, o, B, H, S, causal, scale, st);
    MTA_FUSED_CASE(3, 3)
    MTA_FUSED_CASE(5, 5)
    MTA_FUSED_CASE(5, 7)
    MTA_FUSED_CASE(6, 11)
    MTA_FUSED_CASE(7, 7)
#undef MTA_FUSED_CASE
    return 1;
}
template <> int dispatch_mfma<float, 64>(const void *, const void *, const void *, const void *, void *, int64_t, int64_t,
                                         int64_t, int, int, int, float, hipStream_t) { return 1; }
template <> int dispatch_mfma<float, 128>(const void *, const void *, const void *, const void *, void *, int64_t, int64_t,
                                          int64_t, int, int, int, float, hipStream_t) { return 1; }

template <typename T, int D>
int launch(const void *q, const void *k, const void *v, const void *w, void *o, int64_t B, int64_t H, int64_t S,
           int R, int Sk, int causal, float scale, int w_dtype, hipStream_t st)
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
    hipLaunchKernelGGL(kern, grid, dim3(NT), lds, st, (const T *)q, (const T *)k, (const T *)v, w, (T *)o, (int)S, R, Sk,
                       causal, scale, w_dtype, (int)H, nqb);
    return launch_status();
}
}  // namespace

extern "C" int mta_conv_attn_fwd(const void *q, const void *k, const void *v, const void *w, void *o, int64_t B,
                                 int64_t H, int64_t S, int64_t D, int R, int Sk, int causal, float scale,
                                 int io_dtype, int w_dtype, void *stream)
{
    if (!q || !k || !v || !w || !o) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (B <= 0 || H <= 0 || S <= 0 || S > (1 << 24) || B * H > 65535) return MTA_ERR_SHAPE;
    if (R < 1 || Sk < 1 || R > MTA_MAX_KERNEL_R || Sk > MTA_MAX_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
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
            const int rc = D == 64 ? dispatch_mfma<io_t, 64>(q, k, v, w, o, B, H, S, R, Sk, causal, scale, st)
                                   : dispatch_mfma<io_t, 128>(q, k, v, w, o, B, H, S, R, Sk, causal, scale, st);
            if (rc != 1) return rc;
        }
        if (D == 64) return launch<io_t, 64>(q, k, v, w, o, B, H, S, R, Sk, causal, scale, w_dtype, st);
        return launch<io_t, 128>(q, k, v, w, o, B, H, S, R, Sk, causal, scale, w_dtype, st);
    });
    return MTA_ERR_DTYPE;
}
