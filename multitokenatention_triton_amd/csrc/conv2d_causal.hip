// Depthwise causal 2-D convolution over the (N,C,H,W) score tensor.
//
//   y[n,c,p,q] = sum_{i<R,j<S} w[c,i,j] * xm[n,c,p+i-(R-1), q+j-(S-1)/2]
//
// One workgroup owns a TM x TN output tile of one (n,c) plane.  It stages the
// (TM+R-1) x (TN+S-1) query x key halo tile in LDS once (bounds and the causal
// col<=row rule are applied while staging, so the tap loop is mask-free), skips
// tiles that lie entirely above the diagonal (they only receive their +0 fill), and
// applies the causal output rule on store.
//
// Two compute paths:
//   conv2d_valu  fp32 FMAs from an fp32 LDS tile; any I/O and weight dtype; each lane
//                slides a register window along the key axis (8 outputs per lane).
//   conv2d_mfma  (16-bit I/O with weights of the same dtype) see below.
#include "common.hpp"

namespace {
using namespace mta;

constexpr int NT = 256;

// ------------------------------------------------------------------------------------
// VALU path
// ------------------------------------------------------------------------------------
constexpr int V_TM = 32;  // tile rows   (thread t: row t/8)
constexpr int V_TN = 64;  // tile cols   (thread t: cols 8*(t%8) .. +7)

template <typename T>
__device__ __forceinline__ void store_row8(T *yp, int64_t W, int H, int p, int q, const float *acc,
                                           bool causal)
{
    if (p >= H) return;
    T *dst = yp + (int64_t)p * W + q;
    if (q + 8 <= W && (reinterpret_cast<uintptr_t>(dst) % (8 * sizeof(T))) == 0) {
        struct alignas(8 * sizeof(T)) chunk { T v[8]; } c;
#pragma unroll
        for (int u = 0; u < 8; ++u) c.v[u] = from_float<T>((causal && q + u > p) ? 0.0f : acc[u]);
        *reinterpret_cast<chunk *>(dst) = c;
    } else {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (q + u < W) dst[u] = from_float<T>((causal && q + u > p) ? 0.0f : acc[u]);
    }
}

template <typename T, int R_T, int S_T>
__global__ __launch_bounds__(NT) void conv2d_valu(const T *__restrict__ x, const void *__restrict__ w,
                                                  T *__restrict__ y, int C, int H, int W, int R_rt,
                                                  int S_rt, int causal, float in_scale, int use_scale,
                                                  int w_dtype, int tiles_n)
{
    const int R = R_T > 0 ? R_T : R_rt;
    const int S = S_T > 0 ? S_T : S_rt;
    const int pad_h = R - 1, pad_w = (S - 1) / 2;
    const int LD = V_TN + S;  // S-1 halo columns + 1 pad
    extern __shared__ float smem[];
    float *wsm = smem;                        // R*S weights of this channel
    float *tile = smem + ((R * S + 3) & ~3);  // (V_TM+R-1) x LD

    const int tid = threadIdx.x;
    const int64_t plane = blockIdx.y;
    const int c = (int)(plane % C);
    const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const int p0 = tm * V_TM, q0 = tn * V_TN;
    const T *xp = x + plane * (int64_t)H * W;
    T *yp = y + plane * (int64_t)H * W;
    const int tr = tid >> 3, tc = (tid & 7) * 8;

    float acc[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc[u] = 0.0f;

    if (causal && q0 > p0 + V_TM - 1) {  // wholly above the diagonal: fill only
        store_row8<T>(yp, W, H, p0 + tr, q0 + tc, acc, true);
        return;
    }

    for (int t = tid; t < R * S; t += NT) wsm[t] = load_any(w, w_dtype, (int64_t)c * R * S + t);

    const int rows = V_TM + R - 1, cols = V_TN + S - 1;
    for (int rr = tid / 64; rr < rows; rr += NT / 64) {
        const int h = p0 - pad_h + rr;
        const bool row_ok = h >= 0 && h < H;
        for (int cc = tid % 64; cc < cols; cc += 64) {
            const int k = q0 - pad_w + cc;
            float v = 0.0f;
            if (row_ok && k >= 0 && k < W && (!causal || k <= h)) {
                v = to_float(xp[(int64_t)h * W + k]);
                if (use_scale) v = round_to<T>(v * in_scale);
            }
            tile[rr * LD + cc] = v;
        }
    }
    __syncthreads();

    if constexpr (R_T > 0 && S_T > 0) {
#pragma unroll
        for (int i = 0; i < R_T; ++i) {
            float win[S_T + 7];
            const float *src = tile + (tr + i) * LD + tc;
#pragma unroll
            for (int u = 0; u < S_T + 7; ++u) win[u] = src[u];
#pragma unroll
            for (int j = 0; j < S_T; ++j) {
                const float wv = wsm[i * S_T + j];
#pragma unroll
                for (int u = 0; u < 8; ++u) acc[u] = fmaf(wv, win[u + j], acc[u]);
            }
        }
    } else {
        for (int i = 0; i < R; ++i) {
            const float *src = tile + (tr + i) * LD + tc;
            for (int j = 0; j < S; ++j) {
                const float wv = wsm[i * S + j];
#pragma unroll
                for (int u = 0; u < 8; ++u) acc[u] = fmaf(wv, src[u + j], acc[u]);
            }
        }
    }
    store_row8<T>(yp, W, H, p0 + tr, q0 + tc, acc, causal != 0);
}

template <typename T, int R_T, int S_T>
int launch_valu(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                int S, int causal, float in_scale, int use_scale, int w_dtype, hipStream_t st)
{
    const int tiles_m = (int)((H + V_TM - 1) / V_TM), tiles_n = (int)((W + V_TN - 1) / V_TN);
    const size_t lds = sizeof(float) * (((R * S + 3) & ~3) + (size_t)(V_TM + R - 1) * (V_TN + S));
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)(N * C));
    hipLaunchKernelGGL((conv2d_valu<T, R_T, S_T>), grid, dim3(NT), lds, st, (const T *)x, w, (T *)y, (int)C,
                       (int)H, (int)W, R, S, causal, in_scale, use_scale, w_dtype, tiles_n);
    return launch_status();
}

template <typename T>
int dispatch_valu(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                  int S, int causal, float in_scale, int use_scale, int w_dtype, hipStream_t st)
{
#define MTA_CONV_CASE(r, s)                                                                               \
    if (R == r && S == s)                                                                                 \
        return launch_valu<T, r, s>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st);
    MTA_CONV_CASE(3, 3)
    MTA_CONV_CASE(3, 5)
    MTA_CONV_CASE(5, 5)
    MTA_CONV_CASE(5, 7)
    MTA_CONV_CASE(6, 11)
    MTA_CONV_CASE(7, 7)
    MTA_CONV_CASE(7, 9)
    MTA_CONV_CASE(11, 15)
#undef MTA_CONV_CASE
    return launch_valu<T, 0, 0>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st);
}

int conv2d_entry(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
                 int S, int causal, float in_scale, int use_scale, int io_dtype, int w_dtype, void *stream)
{
    if (!x || !w || !y) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype) || !dtype_size(w_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0) return MTA_ERR_SHAPE;
    if (H > (1 << 24) || W > (1 << 24) || N * C > 0x7fffffffLL / 2) return MTA_ERR_SHAPE;
    if (R < 1 || S < 1 || R > MTA_MAX_KERNEL_R || S > MTA_MAX_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
    if (!aligned_to(x, dtype_size(io_dtype)) || !aligned_to(y, dtype_size(io_dtype)) ||
        !aligned_to(w, dtype_size(w_dtype)))
        return MTA_ERR_ALIGN;
    const int64_t tiles = ((H + V_TM - 1) / V_TM) * ((W + V_TN - 1) / V_TN);
    if (tiles > 0x7fffffffLL || N * C > 65535) return MTA_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    MTA_DISPATCH_IO(io_dtype,
                    return dispatch_valu<io_t>(x, w, y, N, C, H, W, R, S, causal, in_scale, use_scale, w_dtype, st));
    return MTA_ERR_DTYPE;
}
}  // namespace

extern "C" int mta_conv2d_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H,
                              int64_t W, int R, int S, int causal, int io_dtype, int w_dtype, void *stream)
{
    return conv2d_entry(x, w, y, N, C, H, W, R, S, causal, 1.0f, 0, io_dtype, w_dtype, stream);
}

extern "C" int mta_conv2d_scaled_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H,
                                     int64_t W, int R, int S, int causal, float in_scale, int io_dtype,
                                     int w_dtype, void *stream)
{
    return conv2d_entry(x, w, y, N, C, H, W, R, S, causal, in_scale, 1, io_dtype, w_dtype, stream);
}
