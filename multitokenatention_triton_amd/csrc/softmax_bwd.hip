// Gradient of the row softmax of the score tensor, from the stored probabilities:
//
//   dx[q] = p[q] * (dp[q] - sum_k p[k] * dp[k])         over the keys q of one query row; causal: only q <= row index
//
// The reference takes this gradient from torch's autograd through F.softmax(scores.float(), dim=-1).type_as(xq)
// (mta_attention_triton.py:79), i.e. from fp32 copies of the probabilities and of the incoming gradient; here p and dp
// are read once in the score dtype, the arithmetic is fp32, and neither an fp32 copy nor the product p * dp (which
// torch's kernel writes out first) reaches memory.  Above the diagonal nothing is read; dx there is +0 (fill_upper) or
// left alone for a consumer that never reads it.
//
// One workgroup per row.  16-bit rows of whole 16-byte vectors up to 8192 keys stay in registers between the sum and
// the result (one read of p and dp); everything else takes two sweeps over the row.
#include "common.hpp"

namespace {
using namespace mta;

constexpr int NT = 256;

// sum over the workgroup, result in every thread (one barrier; `red` holds one float per wavefront)
__device__ __forceinline__ float block_sum(float v, float *red)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) s += red[w];
    return s;
}

typedef unsigned int u4 __attribute__((ext_vector_type(4)));

// NV = 16-byte vectors per thread: rows of up to NV * 2048 keys
template <typename T, int NV>
__global__ __launch_bounds__(NT) void softmax_bwd_rows16(const T *__restrict__ p, const T *__restrict__ dp,
                                                         T *__restrict__ dx, int P, int Q, int causal, int fill_upper)
{
    __shared__ float red[NT / 64];
    const int64_t row = blockIdx.x;
    const int pr = (int)(row % P);
    const int last = causal ? (pr < Q - 1 ? pr : Q - 1) : Q - 1;  // last key that takes part
    const T *prow = p + row * Q, *grow = dp + row * Q;
    T *xrow = dx + row * Q;
    const int tid = threadIdx.x;

    // every load is unconditional: a vector wholly beyond `last` re-reads the row start and is ignored
    u4 pv[NV], gv[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int q0 = (v * NT + tid) * 8;
        const int qq = q0 <= last ? q0 : 0;
        pv[v] = *reinterpret_cast<const u4 *>(prow + qq);
        gv[v] = *reinterpret_cast<const u4 *>(grow + qq);
    }
    float pf[NV][8], gf[NV][8];
    float dot = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int q0 = (v * NT + tid) * 8;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            unpack2<T>(pv[v][u], pf[v][2 * u], pf[v][2 * u + 1]);
            unpack2<T>(gv[v][u], gf[v][2 * u], gf[v][2 * u + 1]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const bool in = q0 + e <= last;  // what lies beyond need not even be finite
            pf[v][e] = in ? pf[v][e] : 0.0f;
            gf[v][e] = in ? gf[v][e] : 0.0f;
            dot = fmaf(pf[v][e], gf[v][e], dot);
        }
    }
    dot = block_sum(dot, red);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int q0 = (v * NT + tid) * 8;
        if (q0 >= Q) continue;
        if (q0 > last && !fill_upper) continue;
        float r[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = q0 + e <= last ? pf[v][e] * (gf[v][e] - dot) : 0.0f;  // +0 beyond the row's end
        u4 out;
#pragma unroll
        for (int u = 0; u < 4; ++u) out[u] = pack2<T>(r[2 * u], r[2 * u + 1]);
        *reinterpret_cast<u4 *>(xrow + q0) = out;
    }
}

// Any dtype, alignment and row length: two sweeps.
template <typename T>
__global__ __launch_bounds__(NT) void softmax_bwd_rows_any(const T *__restrict__ p, const T *__restrict__ dp,
                                                           T *__restrict__ dx, int P, int Q, int causal, int fill_upper)
{
    __shared__ float red[NT / 64];
    const int64_t row = blockIdx.x;
    const int pr = (int)(row % P);
    const int last = causal ? (pr < Q - 1 ? pr : Q - 1) : Q - 1;
    const T *prow = p + row * Q, *grow = dp + row * Q;
    T *xrow = dx + row * Q;
    float dot = 0.0f;
    for (int q = threadIdx.x; q <= last; q += NT) dot = fmaf(to_float(prow[q]), to_float(grow[q]), dot);
    dot = block_sum(dot, red);
    for (int q = threadIdx.x; q <= last; q += NT) xrow[q] = from_float<T>(to_float(prow[q]) * (to_float(grow[q]) - dot));
    if (fill_upper)
        for (int q = last + 1 + threadIdx.x; q < Q; q += NT) xrow[q] = from_float<T>(0.0f);
}
}  // namespace

extern "C" int mta_softmax_bwd(const void *p, const void *dp, void *dx, int64_t N, int64_t C, int64_t P, int64_t Q,
                               int causal, int fill_upper, int io_dtype, void *stream)
{
    if (!p || !dp || !dx) return MTA_ERR_NULL;
    const size_t es = dtype_size(io_dtype);
    if (!es) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || P <= 0 || Q <= 0 || P > (1 << 24) || Q > (1 << 24)) return MTA_ERR_SHAPE;
    const int64_t rows = N * C * P;
    if (rows > 0x7fffffffLL) return MTA_ERR_SHAPE;
    if (!aligned_to(p, es) || !aligned_to(dp, es) || !aligned_to(dx, es)) return MTA_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = es == 2 && Q % 8 == 0 && Q <= 8192 && aligned_to(p, 16) && aligned_to(dp, 16) && aligned_to(dx, 16);
    MTA_DISPATCH_IO(io_dtype, {
        if constexpr (sizeof(io_t) == 2) {
            if (vec) {
                if (Q <= 2048)
                    hipLaunchKernelGGL((softmax_bwd_rows16<io_t, 1>), dim3((unsigned)rows), dim3(NT), 0, st, (const io_t *)p,
                                       (const io_t *)dp, (io_t *)dx, (int)P, (int)Q, causal, fill_upper);
                else if (Q <= 4096)
                    hipLaunchKernelGGL((softmax_bwd_rows16<io_t, 2>), dim3((unsigned)rows), dim3(NT), 0, st, (const io_t *)p,
                                       (const io_t *)dp, (io_t *)dx, (int)P, (int)Q, causal, fill_upper);
                else
                    hipLaunchKernelGGL((softmax_bwd_rows16<io_t, 4>), dim3((unsigned)rows), dim3(NT), 0, st, (const io_t *)p,
                                       (const io_t *)dp, (io_t *)dx, (int)P, (int)Q, causal, fill_upper);
                return launch_status();
            }
        }
        hipLaunchKernelGGL((softmax_bwd_rows_any<io_t>), dim3((unsigned)rows), dim3(NT), 0, st, (const io_t *)p,
                           (const io_t *)dp, (io_t *)dx, (int)P, (int)Q, causal, fill_upper);
        return launch_status();
    });
    return MTA_ERR_DTYPE;
}
