// Gradient of the head mixing with respect to its (C,C) weight:
//
//   dw[o,i] = sum_{n,p,q} dy[n,o,p,q] * x[n,i,p,q]          (causal: only q <= p take part)
//
// i.e. dW = dY X^T with the contraction running over every attended position of the (N,*,P,Q) tensors.  Both tensors
// are read exactly once.  Accumulation is fp32 and hierarchical (registers over a persistent wavefront's share, one
// partial matrix per workgroup in a scratch buffer, a second kernel adds the partials in a fixed order); the
// reference accumulates with fp32 tl.dot and fp64 atomics (triton_linear_head.py:193-278).
//
// 16-bit tensors with C = 16 or 32 take the matrix cores: A = dY (rows = output heads), B = X (columns = input heads),
// 32 positions per v_mfma_f32_16x16x32.  Which position feeds which contraction slot is free as long as both
// operands agree; product t of a 128-position chunk takes positions 32t..32t+31, lane (head r, group g) the eight from
// 32t + 8g on: a wavefront's load instruction covers 64 contiguous bytes of each of 16 heads.
// Everything else (fp32, other head counts, rows that are not a multiple of 8 keys) takes a generic LDS kernel.
#include "common.hpp"
#include "mfma.hpp"

namespace {
using namespace mta;

constexpr int NT = 256;
// positions per wavefront step of the MFMA kernel: 512 contiguous bytes of every head's row with 16 heads, 256 with 32
// (registers)
template <int NB> constexpr int chunk_of() { return NB == 1 ? 256 : 128; }

// Rows are visited in an order that interleaves short and long ones (0, P-1, 1, P-2, ...), so that under the causal
// mask a pair of consecutive rows always carries P+1 positions.
__device__ __forceinline__ int interleaved_row(int j, int P) { return (j & 1) ? P - 1 - (j >> 1) : (j >> 1); }

typedef unsigned int u4 __attribute__((ext_vector_type(4)));

// One 128-position chunk of one query row: where it starts and where the row's attended positions end.
struct hm_unit {
    int64_t rowbase;
    int q0, last;
};

// The chunk's operands of a lane: for product t the eight positions from q0 + 32t + 8g on, of head 16a + r.
template <int NB> struct hm_operands {
    u4 dy[NB][chunk_of<NB>() / 32], x[NB][chunk_of<NB>() / 32];
};

template <typename T, int NB>
__device__ __forceinline__ void hm_load(hm_operands<NB> &o, const T *x, const T *dy, const hm_unit &u, int64_t plane, int r,
                                        int g)
{
    const int q = u.q0 + 8 * g;
    // every load is unconditional: a vector wholly beyond `last` re-reads the row start and is zeroed before use
#pragma unroll
    for (int a = 0; a < NB; ++a) {
#pragma unroll
        for (int t = 0; t < chunk_of<NB>() / 32; ++t) {
            const int qq = (q + 32 * t <= u.last) ? q + 32 * t : 0;
            o.dy[a][t] = *reinterpret_cast<const u4 *>(dy + u.rowbase + (int64_t)(a * 16 + r) * plane + qq);
        }
#pragma unroll
        for (int t = 0; t < chunk_of<NB>() / 32; ++t) {
            const int qq = (q + 32 * t <= u.last) ? q + 32 * t : 0;
            o.x[a][t] = *reinterpret_cast<const u4 *>(x + u.rowbase + (int64_t)(a * 16 + r) * plane + qq);
        }
    }
}

template <typename T, int NB>
__device__ __forceinline__ void hm_consume(f32x4 (&acc)[NB][NB], hm_operands<NB> &o, const hm_unit &u, int g)
{
    if (u.q0 + chunk_of<NB>() - 1 > u.last) {  // the chunk straddles the end of the row: zero what lies beyond it, in both
                                      // operands (what x holds there need not even be finite)
        const int q = u.q0 + 8 * g;
#pragma unroll
        for (int t = 0; t < chunk_of<NB>() / 32; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int e = q + 32 * t + 2 * v;
                const unsigned keep = (e <= u.last ? 0x0000ffffu : 0u) | (e + 1 <= u.last ? 0xffff0000u : 0u);
#pragma unroll
                for (int a = 0; a < NB; ++a) {
                    o.dy[a][t][v] &= keep;
                    o.x[a][t][v] &= keep;
                }
            }
    }
#pragma unroll
    for (int t = 0; t < chunk_of<NB>() / 32; ++t)
#pragma unroll
        for (int a = 0; a < NB; ++a)
#pragma unroll
            for (int b = 0; b < NB; ++b)
                mma16(acc[a][b], __builtin_bit_cast(frag8<T>, o.dy[a][t]), __builtin_bit_cast(frag8<T>, o.x[b][t]));
}

template <typename T, int NB>  // NB = C / 16
__global__ __launch_bounds__(NT) void headmix_bwd_weight_mfma(const T *__restrict__ x, const T *__restrict__ dy,
                                                              float *__restrict__ partial, int N, int P, int Q, int causal)
{
    constexpr int C = 16 * NB;
    __shared__ float red[NT / 64][C * C];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int64_t plane = (int64_t)P * Q;
    f32x4 acc[NB][NB];
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[a][b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    const int64_t rows = (int64_t)N * P;
    const int64_t nwaves = (int64_t)gridDim.x * (NT / 64), wid = (int64_t)blockIdx.x * (NT / 64) + wave;
    // A wavefront takes pairs of rows (2k, 2k+1) of the interleaved order, k = wid, wid + nwaves, ...; j counts its
    // rows.  The chunks of all its rows form one sequence, and the loads of a chunk are issued before the products of
    // the chunk ahead of it (two operand sets take turns).  (Four wavefronts sharing a row chunk by chunk measured
    // slower: short rows leave most of them without work.)
    int64_t j = 0;
    int q0 = 0;
    auto unit_at = [&](hm_unit &u) -> bool {
        const int64_t rid = 2 * (wid + (j >> 1) * nwaves) + (j & 1);
        if (rid >= rows) return false;
        const int n = (int)(rid / P), p = interleaved_row((int)(rid % P), P);
        u.last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;  // last position of the row that takes part
        u.rowbase = (int64_t)n * C * plane + (int64_t)p * Q;
        u.q0 = q0;
        return true;
    };
    auto advance = [&](const hm_unit &u) {
        q0 += chunk_of<NB>();
        if (q0 > u.last) {
            q0 = 0;
            ++j;
        }
    };
    hm_unit ua, ub;
    hm_operands<NB> oa, ob;
    bool ha = unit_at(ua);
    if (ha) hm_load<T, NB>(oa, x, dy, ua, plane, r, g);
    while (ha) {
        advance(ua);
        const bool hb = unit_at(ub);
        if (!hb) ub = ua;  // nothing follows: fetch the same chunk again, so that the loads in flight never depend on a branch
        hm_load<T, NB>(ob, x, dy, ub, plane, r, g);
        hm_consume<T, NB>(acc, oa, ua, g);
        if (!hb) break;
        advance(ub);
        ha = unit_at(ua);
        if (!ha) ua = ub;
        hm_load<T, NB>(oa, x, dy, ua, plane, r, g);
        hm_consume<T, NB>(acc, ob, ub, g);
    }
    // acc[a][b][v] = dw[16a + 4g + v][16b + r]
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][(a * 16 + 4 * g + v) * C + b * 16 + r] = acc[a][b][v];
    __syncthreads();
    for (int e = threadIdx.x; e < C * C; e += NT) {
        float s = 0.0f;
#pragma unroll
        for (int wv = 0; wv < NT / 64; ++wv) s += red[wv][e];
        partial[(int64_t)blockIdx.x * (C * C) + e] = s;
    }
}

// Any dtype and head count up to 128: a workgroup stages KC positions of every head of both tensors in LDS (fp32,
// masked positions as 0) and keeps the C*C running sums in LDS as well; thread t owns pairs t, t+256, ...
constexpr int KC = 32;
template <typename T>
__global__ __launch_bounds__(NT) void headmix_bwd_weight_any(const T *__restrict__ x, const T *__restrict__ dy,
                                                             float *__restrict__ partial, int N, int C, int P, int Q,
                                                             int causal)
{
    extern __shared__ float smem[];
    float *xs = smem;                // C x (KC+1)
    float *gs = xs + C * (KC + 1);   // C x (KC+1)
    float *sums = gs + C * (KC + 1); // C x C
    const int tid = threadIdx.x;
    const int CC = C * C;
    const int64_t plane = (int64_t)P * Q;
    for (int pair = tid; pair < CC; pair += NT) sums[pair] = 0.0f;
    const int qchunks = (Q + KC - 1) / KC;
    const int64_t items = (int64_t)N * P * qchunks;
    for (int64_t it = blockIdx.x; it < items; it += gridDim.x) {
        const int qc = (int)(it % qchunks);
        const int64_t rid = it / qchunks;
        const int n = (int)(rid / P), p = interleaved_row((int)(rid % P), P);
        const int q0 = qc * KC;
        const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;
        if (q0 > last) continue;
        __syncthreads();
        for (int e = tid; e < C * KC; e += NT) {
            const int h = e / KC, k = e % KC;
            const bool ok = q0 + k <= last;
            const int64_t idx = ((int64_t)n * C + h) * plane + (int64_t)p * Q + q0 + k;
            xs[h * (KC + 1) + k] = ok ? to_float(x[idx]) : 0.0f;
            gs[h * (KC + 1) + k] = ok ? to_float(dy[idx]) : 0.0f;
        }
        __syncthreads();
#pragma unroll 1
        for (int pair = tid; pair < CC; pair += NT) {
            const float *go = gs + (pair / C) * (KC + 1), *xi = xs + (pair % C) * (KC + 1);
            float s = 0.0f;
#pragma unroll
            for (int k = 0; k < KC; ++k) s = fmaf(go[k], xi[k], s);
            sums[pair] += s;  // only the owner thread touches this entry
        }
    }
    for (int pair = tid; pair < CC; pair += NT) partial[(int64_t)blockIdx.x * CC + pair] = sums[pair];
}

// dw[e] = sum of the partial matrices' entries e, in a fixed order: 64 entries per workgroup, the partial matrices dealt
// to 16 wavefronts (each adds its share in index order), the 16 sums added in wavefront order
constexpr int RED_SLICES = 16;
__global__ __launch_bounds__(64 * RED_SLICES) void reduce_partials(const float *__restrict__ partial,
                                                                   float *__restrict__ dw, int CC, int nparts)
{
    __shared__ float red[RED_SLICES][64];
    const int le = threadIdx.x & 63, sl = threadIdx.x >> 6;
    const int e = blockIdx.x * 64 + le;
    float s = 0.0f;
    if (e < CC) {
#pragma unroll 8
        for (int b = sl; b < nparts; b += RED_SLICES) s += partial[(int64_t)b * CC + e];
    }
    red[sl][le] = s;
    __syncthreads();
    if (sl == 0 && e < CC) {
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < RED_SLICES; ++k) t += red[k][le];
        dw[e] = t;
    }
}

constexpr int64_t MAX_WS_BYTES = 8 << 20;  // partial matrices never take more than this

// persistent workgroups (= partial matrices) for a problem
inline int num_blocks(int64_t N, int64_t C, int64_t P, int64_t Q)
{
    int64_t nb = 1024;
    const int64_t pairs = (N * P + 1) / 2;
    if (nb > pairs) nb = pairs;
    const int64_t cap = MAX_WS_BYTES / (C * C * (int64_t)sizeof(float));
    if (nb > cap) nb = cap;
    return (int)(nb < 1 ? 1 : nb);
}
}  // namespace

extern "C" int64_t mta_headmix_bwd_weight_workspace(int64_t N, int64_t C, int64_t P, int64_t Q)
{
    if (N <= 0 || C <= 0 || P <= 0 || Q <= 0 || C > 128) return 0;
    return (int64_t)num_blocks(N, C, P, Q) * C * C * (int64_t)sizeof(float);
}

extern "C" int mta_headmix_bwd_weight(const void *x, const void *dy, void *dw, void *workspace, int64_t workspace_bytes,
                                      int64_t N, int64_t C, int64_t P, int64_t Q, int causal, int io_dtype, void *stream)
{
    if (!x || !dy || !dw || !workspace) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || P <= 0 || Q <= 0 || P > (1 << 24) || Q > (1 << 24) || N * P > 0x7fffffffLL) return MTA_ERR_SHAPE;
    if (C > 128) return MTA_ERR_SHAPE;
    if (!aligned_to(x, dtype_size(io_dtype)) || !aligned_to(dy, dtype_size(io_dtype)) || !aligned_to(dw, 4) ||
        !aligned_to(workspace, 16))
        return MTA_ERR_ALIGN;
    const int nb = num_blocks(N, C, P, Q);
    if (workspace_bytes < (int64_t)nb * C * C * (int64_t)sizeof(float)) return MTA_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    float *partial = (float *)workspace;
    const bool mfma_ok = io_dtype != MTA_F32 && (C == 16 || C == 32) && Q % 8 == 0 && aligned_to(x, 16) && aligned_to(dy, 16);
    MTA_DISPATCH_IO(io_dtype, {
        if constexpr (sizeof(io_t) == 2) {
            if (mfma_ok) {
                if (C == 16)
                    hipLaunchKernelGGL((headmix_bwd_weight_mfma<io_t, 1>), dim3(nb), dim3(NT), 0, st, (const io_t *)x,
                                       (const io_t *)dy, partial, (int)N, (int)P, (int)Q, causal);
                else
                    hipLaunchKernelGGL((headmix_bwd_weight_mfma<io_t, 2>), dim3(nb), dim3(NT), 0, st, (const io_t *)x,
                                       (const io_t *)dy, partial, (int)N, (int)P, (int)Q, causal);
            }
        }
        if (!(sizeof(io_t) == 2 && mfma_ok)) {
            const size_t lds = sizeof(float) * (2 * (size_t)C * (KC + 1) + (size_t)C * C);
            auto kern = headmix_bwd_weight_any<io_t>;
            if (lds > 48 * 1024) {  // per device, so set on every such launch (a cheap host-side call)
                hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
                if (e != hipSuccess) return (int)e;
            }
            hipLaunchKernelGGL(kern, dim3(nb), dim3(NT), lds, st, (const io_t *)x,
                               (const io_t *)dy, partial, (int)N, (int)C, (int)P, (int)Q, causal);
        }
    });
    int rc = launch_status();
    if (rc != MTA_OK) return rc;
    const int CC = (int)(C * C);
    hipLaunchKernelGGL(reduce_partials, dim3((unsigned)((CC + 63) / 64)), dim3(64 * RED_SLICES), 0, st, partial, (float *)dw,
                       CC, nb);
    return launch_status();
}
