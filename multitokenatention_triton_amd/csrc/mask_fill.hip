// y[n,c,p,q] = visible[n,c,p,q] ? x[n,c,p,q] : fill,  fill = 0 or -inf: the elementwise steps the reference takes around
// its operators under a mask tensor of arbitrary content - `masked_fill(mask == -inf, 0)` ahead of the two convs,
// `scores + mask` ahead of the softmax (for a 0 / -inf mask that is a select of -inf), `torch.where(mask == -inf, 0.0,
// scores)` behind the post-softmax conv (mta_attention_triton.py:72-73, 77-78, 81-83) - as one pass each that reads the
// mask as a byte per position instead of building (B,H,S,S) tensors in the score dtype and a boolean copy of them.
// `visible` is uint8, non-zero = attend, one plane for all batch entries and / or all heads or one each.  With the causal
// rule only keys q <= p are touched (the operators on either side neither read nor need the rest).  May run in place.
#include "common.hpp"

namespace {
using namespace mta;

typedef unsigned int mf_u4 __attribute__((ext_vector_type(4)));
typedef unsigned int mf_u2 __attribute__((ext_vector_type(2)));
template <typename T, int VEC> struct alignas(sizeof(T) * VEC) mf_vec { T v[VEC]; };
constexpr int MF_NT = 256;
constexpr int MF_ROWS = 32;  // consecutive rows of one plane per workgroup, a wavefront a row at a time

// EB: bytes per element (2 or 4); rows of Q elements, Q % 8 == 0; fill: the element's bit pattern (16-bit: in both halves)
template <int EB>
__global__ __launch_bounds__(MF_NT) void mask_fill_kernel(const unsigned char *__restrict__ x, unsigned char *__restrict__ y,
                                                          const unsigned char *__restrict__ visible, int C, int P, int Q,
                                                          int mask_n, int mask_c, int causal, unsigned fill,
                                                          int blocks_per_plane)
{
    constexpr int VEC = 16 / EB;  // elements per 16-byte vector
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned plane = blockIdx.x / (unsigned)blocks_per_plane;  // n*C + c
    const int p0 = (int)(blockIdx.x % (unsigned)blocks_per_plane) * MF_ROWS;
    const unsigned n = plane / (unsigned)C, c = plane % (unsigned)C;
    const int64_t mplane = (int64_t)(mask_n > 1 ? n : 0) * mask_c + (mask_c > 1 ? c : 0);
    for (int p = p0 + wave; p < p0 + MF_ROWS && p < P; p += MF_NT / 64) {
        const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;  // last key touched
        const int64_t row = ((int64_t)plane * P + p) * Q;
        const unsigned char *m = visible + (mplane * P + p) * Q;
        for (int q0 = lane * VEC; q0 <= last; q0 += 64 * VEC) {
            mf_u4 t = *reinterpret_cast<const mf_u4 *>(x + (row + q0) * EB);
            unsigned mb[2];
            if constexpr (VEC == 8) {
                const mf_u2 mm = *reinterpret_cast<const mf_u2 *>(m + q0);
                mb[0] = mm[0];
                mb[1] = mm[1];
            } else {
                mb[0] = *reinterpret_cast<const unsigned *>(m + q0);
                mb[1] = 0;
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                // (a key beyond the row's last one, in the vector that straddles the diagonal, stays as it is)
                const bool keep = ((mb[e >> 2] >> ((e & 3) * 8)) & 0xffu) != 0 || q0 + e > last;
                if (!keep) {
                    if constexpr (EB == 2) t[e >> 1] = (e & 1) ? ((t[e >> 1] & 0x0000ffffu) | (fill & 0xffff0000u))
                                                               : ((t[e >> 1] & 0xffff0000u) | (fill & 0x0000ffffu));
                    else t[e] = fill;
                }
            }
            *reinterpret_cast<mf_u4 *>(y + (row + q0) * EB) = t;
        }
    }
}
// y = x + mask in the I/O dtype (the sum formed in fp32 and rounded once, as torch adds two 16-bit tensors): the
// reference's `scores = scores + mask` (mta_attention_triton.py:77-78) for an additive mask with finite values, the mask a
// tensor of the scores' dtype, one plane for all batch entries and / or heads or one each.
template <typename T>
__global__ __launch_bounds__(MF_NT) void mask_add_kernel(const T *__restrict__ x, T *__restrict__ y, const T *__restrict__ mask,
                                                         int C, int P, int Q, int mask_n, int mask_c, int causal,
                                                         int blocks_per_plane)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned plane = blockIdx.x / (unsigned)blocks_per_plane;  // n*C + c
    const int p0 = (int)(blockIdx.x % (unsigned)blocks_per_plane) * MF_ROWS;
    const unsigned n = plane / (unsigned)C, c = plane % (unsigned)C;
    const int64_t mplane = (int64_t)(mask_n > 1 ? n : 0) * mask_c + (mask_c > 1 ? c : 0);
    for (int p = p0 + wave; p < p0 + MF_ROWS && p < P; p += MF_NT / 64) {
        const int last = causal ? (p < Q - 1 ? p : Q - 1) : Q - 1;
        const T *xr = x + ((int64_t)plane * P + p) * Q;
        T *yr = y + ((int64_t)plane * P + p) * Q;
        const T *mr = mask + (mplane * P + p) * Q;
        for (int q0 = lane * VEC; q0 <= last; q0 += 64 * VEC) {
            mf_vec<T, VEC> a = *reinterpret_cast<const mf_vec<T, VEC> *>(xr + q0);
            const mf_vec<T, VEC> m = *reinterpret_cast<const mf_vec<T, VEC> *>(mr + q0);
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                if (q0 + e <= last) a.v[e] = from_float<T>(to_float(a.v[e]) + to_float(m.v[e]));
            *reinterpret_cast<mf_vec<T, VEC> *>(yr + q0) = a;
        }
    }
}
}  // namespace

extern "C" int mta_mask_add_fwd(const void *x, const void *mask, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                                int mask_batch, int mask_heads, int causal, int io_dtype, void *stream)
{
    if (!x || !mask || !y) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || P <= 0 || Q <= 0 || Q > (1 << 24) || P > (1 << 24) || N * C > 0x7fffffffLL / ((P + MF_ROWS - 1) / MF_ROWS))
        return MTA_ERR_SHAPE;
    if ((mask_batch != 1 && mask_batch != N) || (mask_heads != 1 && mask_heads != C)) return MTA_ERR_SHAPE;
    if (!aligned_to(x, 16) || !aligned_to(y, 16) || !aligned_to(mask, 16)) return MTA_ERR_ALIGN;
    if (Q % 8 != 0) return MTA_ERR_UNSUPPORTED;
    const int64_t bpp = (P + MF_ROWS - 1) / MF_ROWS;
    const dim3 grid((unsigned)(N * C * bpp));
    hipStream_t st = (hipStream_t)stream;
#define MTA_MASK_ADD(T)                                                                                              \
    hipLaunchKernelGGL(mask_add_kernel<T>, grid, dim3(MF_NT), 0, st, (const T *)x, (T *)y, (const T *)mask, (int)C, (int)P, \
                       (int)Q, mask_batch, mask_heads, causal, (int)bpp)
    if (io_dtype == MTA_F32) MTA_MASK_ADD(float);
    else if (io_dtype == MTA_BF16) MTA_MASK_ADD(bf16_t);
    else MTA_MASK_ADD(f16_t);
#undef MTA_MASK_ADD
    return launch_status();
}

extern "C" int mta_mask_fill_fwd(const void *x, const void *visible, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                                 int mask_batch, int mask_heads, int neg_inf, int causal, int io_dtype, void *stream)
{
    if (!x || !visible || !y) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || P <= 0 || Q <= 0 || Q > (1 << 24) || P > (1 << 24) || N * C > 0x7fffffffLL / ((P + MF_ROWS - 1) / MF_ROWS))
        return MTA_ERR_SHAPE;
    if ((mask_batch != 1 && mask_batch != N) || (mask_heads != 1 && mask_heads != C)) return MTA_ERR_SHAPE;
    if (!aligned_to(x, 16) || !aligned_to(y, 16) || !aligned_to(visible, 8)) return MTA_ERR_ALIGN;
    if (Q % 8 != 0) return MTA_ERR_UNSUPPORTED;
    const int64_t bpp = (P + MF_ROWS - 1) / MF_ROWS;
    const dim3 grid((unsigned)(N * C * bpp));
    hipStream_t st = (hipStream_t)stream;
    if (io_dtype == MTA_F32) {
        hipLaunchKernelGGL(mask_fill_kernel<4>, grid, dim3(MF_NT), 0, st, (const unsigned char *)x, (unsigned char *)y,
                           (const unsigned char *)visible, (int)C, (int)P, (int)Q, mask_batch, mask_heads, causal,
                           neg_inf ? 0xff800000u : 0u, (int)bpp);
    } else {
        const unsigned ninf = io_dtype == MTA_BF16 ? 0xff80ff80u : 0xfc00fc00u;
        hipLaunchKernelGGL(mask_fill_kernel<2>, grid, dim3(MF_NT), 0, st, (const unsigned char *)x, (unsigned char *)y,
                           (const unsigned char *)visible, (int)C, (int)P, (int)Q, mask_batch, mask_heads, causal,
                           neg_inf ? ninf : 0u, (int)bpp);
    }
    return launch_status();
}
