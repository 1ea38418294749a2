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
    MTA_DISPATCH_IO(io_dtype, {
        if (D == 64) return launch<io_t, 64>(q, k, v, w, o, B, H, S, R, Sk, causal, scale, w_dtype, st);
        return launch<io_t, 128>(q, k, v, w, o, B, H, S, R, Sk, causal, scale, w_dtype, st);
    });
    return MTA_ERR_DTYPE;
}
