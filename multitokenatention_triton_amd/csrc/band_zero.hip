// x[n,c,p,q] = 0 for q < first_visible[n,p]: what the reference's `torch.where(mask == -inf, 0.0, scores)` behind its
// post-softmax conv (mta_attention_triton.py:82-83) does below the diagonal under a band mask (row p sees the keys
// first_visible[n,p] .. p).  The conv spreads probability into the columns a row does not see; this takes it out again
// before the heads are mixed.  Only the hidden stretch of each row is touched, and only written: whole 16-byte vectors
// are stored, the one vector that holds the first visible key is read, cleared in part and written back.
#include "common.hpp"

namespace {
using namespace mta;

typedef unsigned int bz_u4 __attribute__((ext_vector_type(4)));
constexpr int BZ_NT = 256;

// a workgroup takes BZ_ROWS consecutive rows of one plane, a wavefront a row at a time; 16-bit elements, rows of S
// elements, S % 8 == 0
constexpr int BZ_ROWS = 32;
__global__ __launch_bounds__(BZ_NT) void band_zero_kernel(unsigned short *__restrict__ x, const int *__restrict__ first, int C,
                                                          int S, int blocks_per_plane)
{
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned plane = blockIdx.x / (unsigned)blocks_per_plane;  // n*C + c
    const int p0 = (int)(blockIdx.x % (unsigned)blocks_per_plane) * BZ_ROWS;
    const int64_t n = plane / (unsigned)C;
    const bz_u4 z = {0u, 0u, 0u, 0u};
    for (int p = p0 + wave; p < p0 + BZ_ROWS && p < S; p += BZ_NT / 64) {
        int lo = first[n * S + p];
        lo = lo < 0 ? 0 : (lo > p + 1 ? p + 1 : lo);  // (a row that sees nothing: everything up to the diagonal)
        unsigned short *row = x + ((int64_t)plane * S + p) * S;
        const int full = lo >> 3;  // whole vectors of 8 hidden keys
        for (int v = lane; v < full; v += 64) *reinterpret_cast<bz_u4 *>(row + v * 8) = z;
        const int rest = lo & 7;
        if (rest && lane == 0) {
            bz_u4 t = *reinterpret_cast<const bz_u4 *>(row + full * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (e < rest) t[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
            *reinterpret_cast<bz_u4 *>(row + full * 8) = t;
        }
    }
}
}  // namespace

extern "C" int mta_band_zero_fwd(void *x, const void *first_visible, int64_t N, int64_t C, int64_t S, int io_dtype, void *stream)
{
    if (!x || !first_visible) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || S <= 0 || S > (1 << 24) || N * C * S > 0x7fffffffLL) return MTA_ERR_SHAPE;
    if (!aligned_to(x, 16) || !aligned_to(first_visible, 4)) return MTA_ERR_ALIGN;
    if (io_dtype == MTA_F32 || S % 8 != 0) return MTA_ERR_UNSUPPORTED;
    const int64_t bpp = (S + BZ_ROWS - 1) / BZ_ROWS;
    hipLaunchKernelGGL(band_zero_kernel, dim3((unsigned)(N * C * bpp)), dim3(BZ_NT), 0, (hipStream_t)stream,
                       (unsigned short *)x, (const int *)first_visible, (int)C, (int)S, (int)bpp);
    return launch_status();
}
