// Depthwise causal conv followed by head mixing, in one pass over an (N,C,H,W) tensor:
//
//     t[h]   = round( conv2d(x[h], w_conv[h]) )            causal: taps with col > row read as 0, outputs q > p are +0
//     y[o]   = round( sum_h w_mix[o,h] * t[h] )            over the heads of o's mixing group
//
// which is what mta_conv_after_sm_triton -> wposm_triton compute on the probabilities
// (mta_attention_triton.py:81-85; conv_fwd_kernel, convolution_2d_trit.py:52-135; linear_head_kernel_forward,
// triton_linear_head.py:76-139) with the conv result never leaving the chip: one read and one write of the tensor
// instead of two of each.
//
// A workgroup owns a 32 x 64 tile of positions for all G heads of one mixing group.  It walks the group's heads:
// stage the head's (32+R-1) x (64+S-1) input window in LDS as fp32 (the causal input rule and the borders are
// applied on the way in), convolve - a lane owns 8 consecutive keys of one row, as in the stand-alone conv - round
// to the I/O dtype, and add the head's contribution to the G x 8 output accumulators of the lane.  For 16-bit data
// with mix weights of the same dtype the heads are taken in pairs and the mixing runs on packed dot products (two
// multiply-adds per instruction; the pair is packed from the rounded conv results, which is the rounding the
// unfused pipeline applies to them).
#include <type_traits>

#include "common.hpp"

namespace {
using namespace mta;

constexpr int CH_NT = 256;
constexpr int CH_TM = 32;  // tile rows
constexpr int CH_TN = 64;  // tile keys

template <typename T> __device__ __forceinline__ float dot2_io(uint32_t a, uint32_t b, float c)
{
    if constexpr (std::is_same<T, bf16_t>::value) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(mta_bf16x2, a), __builtin_bit_cast(mta_bf16x2, b), c, false);
    } else if constexpr (std::is_same<T, f16_t>::value) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(mta_f16x2, a), __builtin_bit_cast(mta_f16x2, b), c, false);
    } else {
        return c;
    }
}

// DOT: mix on packed dot products (16-bit data, mix weights of the same dtype, even group size)
template <typename T, int G, int R_T, int S_T, bool DOT>
__global__ __launch_bounds__(CH_NT) void conv_headmix_kernel(const T *__restrict__ x, const void *__restrict__ wc,
                                                            const void *__restrict__ wm, T *__restrict__ y, int C, int H,
                                                            int W, int R_rt, int S_rt, int causal, int fill_upper,
                                                            int wc_dtype, int wm_dtype, int tiles_n)
{
    const int R = R_T > 0 ? R_T : R_rt;
    const int S = S_T > 0 ? S_T : S_rt;
    const int pad_h = R - 1, pad_w = (S - 1) / 2;
    extern __shared__ float smem[];
    float *wms = smem;                              // G*G mix weights of this group, [o][h]
    float *wcs = wms + G * G;                       // G*R*S conv weights of the group's heads
    float *tile = wcs + ((G * R * S + 3) & ~3);     // two windows of (CH_TM+R-1) x LD
    // mix weights as packed pairs of the I/O dtype, (w[o][2j], w[o][2j+1])
    static_assert(!DOT || (sizeof(T) == 2 && G % 2 == 0), "packed pairs of a 16-bit type");
    __shared__ uint32_t wmp[DOT ? G * (G / 2) : 1];

    const int tid = threadIdx.x;
    const int groups = C / G;
    const int64_t n = blockIdx.y / groups;
    const int g = (int)(blockIdx.y % groups);
    const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const int p0 = tm * CH_TM, q0 = tn * CH_TN;
    const int64_t plane = (int64_t)H * W;
    const T *xg = x + (n * C + (int64_t)g * G) * plane;
    T *yg = y + (n * C + (int64_t)g * G) * plane;
    const int tr = tid >> 3, tc = (tid & 7) * 8;
    const int p = p0 + tr, q = q0 + tc;
    const bool vec_ok = (W % 8 == 0) && ((reinterpret_cast<uintptr_t>(y) & 15) == 0);

    auto store8 = [&](int o, const float (&v)[8]) {
        if (p >= H || q >= W) return;
        T *dst = yg + o * plane + (int64_t)p * W + q;
        if (vec_ok) {
            pack16<T> out;
            if constexpr (sizeof(T) == 2) {
                uint32_t r[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) r[u] = pack2<T>(v[2 * u], v[2 * u + 1]);
                __builtin_memcpy(&out, r, 16);
                typedef unsigned int u4 __attribute__((ext_vector_type(4)));
                __builtin_nontemporal_store(__builtin_bit_cast(u4, out), reinterpret_cast<u4 *>(dst));
            } else {
#pragma unroll
                for (int u = 0; u < 4; ++u) out.v[u] = from_float<T>(v[u]);
                *reinterpret_cast<pack16<T> *>(dst) = out;
#pragma unroll
                for (int u = 0; u < 4; ++u) out.v[u] = from_float<T>(v[4 + u]);
                *reinterpret_cast<pack16<T> *>(dst + 4) = out;
            }
        } else {
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (q + u < W) dst[u] = from_float<T>(v[u]);
        }
    };

    if (causal && q0 > p0 + CH_TM - 1) {  // wholly above the diagonal: +0 on request, nothing else
        if (fill_upper) {
            const float z[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int o = 0; o < G; ++o) store8(o, z);
        }
        return;
    }

    for (int t = tid; t < G * G; t += CH_NT)
        wms[t] = load_any(wm, wm_dtype, (int64_t)(g * G + t / G) * C + g * G + t % G);
    for (int t = tid; t < G * R * S; t += CH_NT) wcs[t] = load_any(wc, wc_dtype, (int64_t)g * G * R * S + t);
    if constexpr (DOT) {
        for (int t = tid; t < G * (G / 2); t += CH_NT) {
            const int o = t / (G / 2), j = t % (G / 2);
            const int64_t widx = (int64_t)(g * G + o) * C + g * G + 2 * j;
            wmp[t] = pack2<T>(load_any(wm, wm_dtype, widx), load_any(wm, wm_dtype, widx + 1));
        }
    }

    float out[G][8];
#pragma unroll
    for (int o = 0; o < G; ++o)
#pragma unroll
        for (int u = 0; u < 8; ++u) out[o][u] = 0.0f;

    // Staging.  Kernel sizes with an instantiation of their own, on tensors whose rows are whole 16-byte vectors: the
    // window starts at a vector boundary left of the halo, each lane fetches its vectors of head h+1 into registers
    // before it convolves head h and writes them to the other LDS window afterwards (one barrier per head, the fetch
    // overlaps the arithmetic).  Anything else: element by element into a single window, two barriers per head.
    constexpr int VEC = vec_of<T>::n;
    constexpr bool PRE = R_T > 0 && S_T > 0;
    constexpr int HL = PRE ? ((S_T - 1) / 2 + VEC - 1) / VEC * VEC : 0;
    constexpr int HRT = PRE ? ((S_T - 1 - (S_T - 1) / 2) + VEC - 1) / VEC * VEC : 0;
    constexpr int SW = HL + CH_TN + HRT, VPR = SW / VEC;  // staged columns, vectors per staged row
    constexpr int ROWS_T = CH_TM + (R_T > 0 ? R_T : 1) - 1, NVECS = ROWS_T * VPR, SLOTS = (NVECS + CH_NT - 1) / CH_NT;
    const bool vec_in = PRE && (W % VEC == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    const int LD = vec_in ? SW + 1 : CH_TN + S;   // (odd: the 8 rows x 8 key groups of a wavefront read 64 different banks)
    const int c0 = vec_in ? HL - pad_w : 0;       // window column of the first tap of the lane with tc = 0
    const int rows = CH_TM + R - 1, cols = CH_TN + S - 1;
    float *tile1 = tile + rows * LD;

    auto stage_scalar = [&](int h, float *dst) {
        const T *xp = xg + h * plane;
        for (int rr = tid / 64; rr < rows; rr += CH_NT / 64) {
            const int hh = p0 - pad_h + rr;
            const bool row_ok = hh >= 0 && hh < H;
            for (int cc = tid % 64; cc < cols; cc += 64) {
                const int k = q0 - pad_w + cc;
                float v = 0.0f;
                if (row_ok && k >= 0 && k < W && (!causal || k <= hh)) v = to_float(xp[(int64_t)hh * W + k]);
                dst[rr * LD + cc] = v;
            }
        }
    };
    auto fetch = [&](int h, pack16<T> (&pre)[SLOTS]) __attribute__((always_inline)) {
        const T *xp = xg + h * plane;
#pragma unroll
        for (int sl = 0; sl < SLOTS; ++sl) {
            const int idx = sl * CH_NT + tid;
            const int rr = idx / VPR, vc = idx % VPR;
            const int hh = p0 - pad_h + rr, k0 = q0 - HL + vc * VEC;
            const bool ok = idx < NVECS && hh >= 0 && hh < H && k0 >= 0 && k0 < W && (!causal || k0 <= hh);
            // (a vector outside the plane or wholly above the diagonal re-reads the plane's first vector: the
            // load stays unconditional, its value is dropped below)
            pre[sl] = *reinterpret_cast<const pack16<T> *>(xp + (ok ? (int64_t)hh * W + k0 : 0));
        }
    };
    auto deposit = [&](const pack16<T> (&pre)[SLOTS], float *dst) __attribute__((always_inline)) {
#pragma unroll
        for (int sl = 0; sl < SLOTS; ++sl) {
            const int idx = sl * CH_NT + tid;
            if (idx >= NVECS) continue;
            const int rr = idx / VPR, vc = idx % VPR;
            const int hh = p0 - pad_h + rr, k0 = q0 - HL + vc * VEC;
            const bool ok = hh >= 0 && hh < H && k0 >= 0 && k0 < W;
#pragma unroll
            for (int u = 0; u < VEC; ++u)
                dst[rr * LD + vc * VEC + u] = (ok && (!causal || k0 + u <= hh)) ? to_float(pre[sl].v[u]) : 0.0f;
        }
    };
    // rounded conv result of head h for this lane's 8 positions, from the staged window `tl`
    auto conv_head = [&](const float *tl, int h, float (&acc)[8]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 8; ++u) acc[u] = 0.0f;
        const float *wch = wcs + h * R * S;
        if constexpr (R_T > 0 && S_T > 0) {
#pragma unroll
            for (int i = 0; i < R_T; ++i) {
                float win[S_T + 7];
                const float *src = tl + (tr + i) * LD + tc + c0;
#pragma unroll
                for (int u = 0; u < S_T + 7; ++u) win[u] = src[u];
#pragma unroll
                for (int j = 0; j < S_T; ++j) {
                    const float wv = wch[i * S_T + j];
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc[u] = fmaf(wv, win[u + j], acc[u]);
                }
            }
        } else {
            for (int i = 0; i < R; ++i) {
                const float *src = tl + (tr + i) * LD + tc + c0;
                for (int j = 0; j < S; ++j) {
                    const float wv = wch[i * S + j];
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc[u] = fmaf(wv, src[u + j], acc[u]);
                }
            }
        }
        // the conv's causal output rule, then its rounding to the I/O dtype
#pragma unroll
        for (int u = 0; u < 8; ++u) acc[u] = (causal && q + u > p) ? 0.0f : round_to<T>(acc[u]);
    };
    // head h's contribution to the outputs (packed-dot path: heads enter in pairs)
    uint32_t pp[8];
    auto mix_in = [&](int h, const float (&acc)[8]) __attribute__((always_inline)) {
        if constexpr (DOT) {
            if ((h & 1) == 0) {
#pragma unroll
                for (int u = 0; u < 8; ++u) pp[u] = pack2<T>(acc[u], 0.0f) & 0xffffu;  // (exact: already rounded)
            } else {
#pragma unroll
                for (int u = 0; u < 8; ++u) pp[u] |= pack2<T>(0.0f, acc[u]) & 0xffff0000u;
#pragma unroll
                for (int o = 0; o < G; ++o) {
                    const uint32_t wv = wmp[o * (G / 2) + (h >> 1)];
#pragma unroll
                    for (int u = 0; u < 8; ++u) out[o][u] = dot2_io<T>(wv, pp[u], out[o][u]);
                }
            }
        } else {
#pragma unroll
            for (int o = 0; o < G; ++o) {
                const float wv = wms[o * G + h];
#pragma unroll
                for (int u = 0; u < 8; ++u) out[o][u] = fmaf(wv, acc[u], out[o][u]);
            }
        }
    };
    if (vec_in) {
        pack16<T> pre[SLOTS];
        fetch(0, pre);
        deposit(pre, tile);
        __syncthreads();  // (also covers the weights)
#pragma unroll 1
        for (int h = 0; h < G; ++h) {
            if (h + 1 < G) fetch(h + 1, pre);
            float acc[8];
            conv_head((h & 1) ? tile1 : tile, h, acc);
            mix_in(h, acc);
            if (h + 1 < G) deposit(pre, (h & 1) ? tile : tile1);  // last read a head ago, ahead of the barrier below
            __syncthreads();
        }
    } else {
#pragma unroll 1
        for (int h = 0; h < G; ++h) {
            __syncthreads();  // everybody is done with the previous head's window
            stage_scalar(h, tile);
            __syncthreads();
            float acc[8];
            conv_head(tile, h, acc);
            mix_in(h, acc);
        }
    }
#pragma unroll
    for (int o = 0; o < G; ++o) {
        if (causal) {
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (q + u > p) out[o][u] = 0.0f;
        }
        if (!causal || fill_upper || q <= p) store8(o, out[o]);
    }
}

template <typename T, int G, int R_T, int S_T>
int launch(const void *x, const void *wc, const void *wm, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
           int S, int causal, int fill_upper, int wc_dtype, int wm_dtype, hipStream_t st)
{
    const int tiles_m = (int)((H + CH_TM - 1) / CH_TM), tiles_n = (int)((W + CH_TN - 1) / CH_TN);
    // two windows of (32+R-1) rows; a row is at most 64 keys + both halos rounded up to whole vectors + 1
    const size_t row = (size_t)CH_TN + 2 * ((S + 7) / 8 * 8) + 1;
    const size_t lds = sizeof(float) * ((size_t)G * G + ((G * R * S + 3) & ~3) + 2 * (size_t)(CH_TM + R - 1) * row);
    if (lds > 64 * 1024) return MTA_ERR_UNSUPPORTED;
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)(N * (C / G)));
    constexpr bool DOT_OK = sizeof(T) == 2 && G % 2 == 0;
    const bool use_dot = DOT_OK && wm_dtype == (std::is_same<T, bf16_t>::value ? MTA_BF16 : MTA_F16);
    if constexpr (DOT_OK) {
        if (use_dot) {
            hipLaunchKernelGGL((conv_headmix_kernel<T, G, R_T, S_T, true>), grid, dim3(CH_NT), lds, st, (const T *)x, wc, wm,
                               (T *)y, (int)C, (int)H, (int)W, R, S, causal, fill_upper, wc_dtype, wm_dtype, tiles_n);
            return launch_status();
        }
    }
    hipLaunchKernelGGL((conv_headmix_kernel<T, G, R_T, S_T, false>), grid, dim3(CH_NT), lds, st, (const T *)x, wc, wm,
                       (T *)y, (int)C, (int)H, (int)W, R, S, causal, fill_upper, wc_dtype, wm_dtype, tiles_n);
    return launch_status();
}

template <typename T, int G>
int dispatch_size(const void *x, const void *wc, const void *wm, void *y, int64_t N, int64_t C, int64_t H, int64_t W,
                  int R, int S, int causal, int fill_upper, int wc_dtype, int wm_dtype, hipStream_t st)
{
#define MTA_CH_CASE(r, s) \
    if (R == r && S == s) return launch<T, G, r, s>(x, wc, wm, y, N, C, H, W, R, S, causal, fill_upper, wc_dtype, wm_dtype, st);
    MTA_CH_CASE(3, 3)
    MTA_CH_CASE(7, 7)
#undef MTA_CH_CASE
    return launch<T, G, 0, 0>(x, wc, wm, y, N, C, H, W, R, S, causal, fill_upper, wc_dtype, wm_dtype, st);
}

template <typename T>
int dispatch(const void *x, const void *wc, const void *wm, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R,
             int S, int G, int causal, int fill_upper, int wc_dtype, int wm_dtype, hipStream_t st)
{
#define MTA_CH_GROUP(g) \
    if (G == g) return dispatch_size<T, g>(x, wc, wm, y, N, C, H, W, R, S, causal, fill_upper, wc_dtype, wm_dtype, st);
    MTA_CH_GROUP(1)
    MTA_CH_GROUP(2)
    MTA_CH_GROUP(4)
    MTA_CH_GROUP(8)
    MTA_CH_GROUP(16)
#undef MTA_CH_GROUP
    return MTA_ERR_UNSUPPORTED;
}
}  // namespace

extern "C" int mta_conv2d_headmix_fwd(const void *x, const void *w_conv, const void *w_mix, void *y, int64_t N, int64_t C,
                                      int64_t H, int64_t W, int R, int S, int group_size, int causal, int fill_upper,
                                      int io_dtype, int wconv_dtype, int wmix_dtype, void *stream)
{
    if (!x || !w_conv || !w_mix || !y) return MTA_ERR_NULL;
    if (!dtype_size(io_dtype) || !dtype_size(wconv_dtype) || !dtype_size(wmix_dtype)) return MTA_ERR_DTYPE;
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || H > (1 << 24) || W > (1 << 24) || C > 4096) return MTA_ERR_SHAPE;
    if (R < 1 || S < 1 || R > MTA_MAX_FUSED_KERNEL_R || S > MTA_MAX_FUSED_KERNEL_S) return MTA_ERR_KERNEL_SIZE;
    if (group_size < 0 || (group_size > 0 && C % group_size != 0)) return MTA_ERR_GROUP;
    if (!aligned_to(x, dtype_size(io_dtype)) || !aligned_to(y, dtype_size(io_dtype)) ||
        !aligned_to(w_conv, dtype_size(wconv_dtype)) || !aligned_to(w_mix, dtype_size(wmix_dtype)))
        return MTA_ERR_ALIGN;
    const int G = group_size > 0 ? group_size : (int)C;
    hipStream_t st = (hipStream_t)stream;
    // groups of 16 heads, 16-bit data and weights of the same dtype: conv and mixing both on the matrix cores
    if (G == 16 && io_dtype != MTA_F32 && wconv_dtype == io_dtype && wmix_dtype == io_dtype) {
        const int rc = conv_mix16_dispatch(x, w_conv, w_mix, y, N, C, H, W, R, S, causal, causal ? fill_upper : 1, io_dtype, st);
        if (rc != MTA_ERR_UNSUPPORTED) return rc;
    }
    const int64_t tiles = ((H + CH_TM - 1) / CH_TM) * ((W + CH_TN - 1) / CH_TN);
    if (tiles > 0x7fffffffLL || N * (C / G) > 65535) return MTA_ERR_SHAPE;
    MTA_DISPATCH_IO(io_dtype, return dispatch<io_t>(x, w_conv, w_mix, y, N, C, H, W, R, S, G, causal, causal ? fill_upper : 1,
                                                    wconv_dtype, wmix_dtype, st));
    return MTA_ERR_DTYPE;
}
