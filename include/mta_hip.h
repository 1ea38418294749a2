/* C ABI of libmta_hip.so: Multi-Token-Attention forward kernels for AMD MI355X (gfx950).
 *
 * The reference (Gusanidas/multitokenatention_triton) has no FFI: its operators are
 * Triton kernels launched from torch.autograd.Function.forward.  Each entry point
 * below replaces one such launch site (cited per function) and is what a ctypes /
 * cffi / pybind binding in the reference's operator files would call.
 *
 * Conventions
 *  - All tensors are dense, row-major ("contiguous NCHW"), device pointers.
 *  - The caller allocates and owns every buffer.  The library allocates nothing,
 *    keeps no pointer after return, and fully defines the output (fill values
 *    included), so outputs may be uninitialised memory.
 *  - Work is only enqueued on `stream` (a hipStream_t; NULL = the null stream); no
 *    entry point synchronises.
 *  - Return value: 0 = ok; negative = MTA_ERR_* (argument rejected, nothing
 *    launched); positive = hipError_t reported by the launch.
 *  - dtype codes: MTA_F32, MTA_BF16, MTA_F16.  Accumulation is always fp32.
 */
#ifndef MTA_HIP_H
#define MTA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MTA_ABI_VERSION 10

enum mta_dtype { MTA_F32 = 0, MTA_BF16 = 1, MTA_F16 = 2 };

enum mta_error {
    MTA_OK = 0,
    MTA_ERR_NULL = -1,        /* a required pointer is NULL */
    MTA_ERR_DTYPE = -2,       /* unknown dtype code */
    MTA_ERR_SHAPE = -3,       /* a size is <= 0 or exceeds what the kernel indexes */
    MTA_ERR_KERNEL_SIZE = -4, /* conv kernel R or S outside the supported range */
    MTA_ERR_GROUP = -5,       /* group_size does not divide the head count */
    MTA_ERR_ALIGN = -6,       /* pointer not aligned to its element size */
    MTA_ERR_HEAD_DIM = -7,    /* head dim unsupported by the fused kernel */
    MTA_ERR_DEVICE = -8,      /* no usable gfx950 device / device query failed */
    MTA_ERR_UNSUPPORTED = -9, /* valid arguments, but this entry point has no kernel for the combination */
    MTA_ERR_WORKSPACE = -10   /* workspace smaller than the matching *_workspace() call reports */
};

/* Largest conv kernel the entry points accept. */
/* `causal` of mta_conv2d_fwd, mta_conv2d_scaled_fwd, mta_conv2d_bwd_input, mta_headmix_fwd and mta_headmix_bwd_input:
 * 0 = no mask; MTA_CAUSAL_LOWER_ONLY = causal, for a consumer that never reads above the diagonal (what lies there
 * in the output is left alone, except where a vector or tile straddles the diagonal: +0.0 / fill); any other value =
 * causal with the output above the diagonal written (+0.0 / fill).  The other entry points read `causal` as a flag. */
#define MTA_CAUSAL_LOWER_ONLY 2

/* Largest conv kernel (rows x keys) of the conv operator and its gradients (mta_conv2d_*): beyond the sizes with a
 * matrix-core or unrolled instance they run on the general fp32-FMA kernels, whose staged tile must fit the LDS.  The
 * reference's published rows go up to 77 x 77 (benchmark_seq_len_results.jsonl:140-180). */
#define MTA_MAX_KERNEL_R 80
#define MTA_MAX_KERNEL_S 95
/* ... and of the kernels that keep score tiles in LDS next to K and V blocks (mta_conv_attn_fwd*, mta_qk_conv_fwd,
 * mta_conv2d_headmix_fwd) */
#define MTA_MAX_FUSED_KERNEL_R 32
#define MTA_MAX_FUSED_KERNEL_S 63

int mta_abi_version(void);
const char *mta_strerror(int code);

/* Depthwise (groups = channels) 2-D cross-correlation over an (N,C,H,W) score tensor:
 *   y[n,c,p,q] = sum_{i<R, j<S} w[c,i,j] * xm[n,c, p+i-(R-1), q+j-(S-1)/2]
 * xm = x with out-of-range taps read as 0 and, when causal, taps with col>row read
 * as 0.  When causal every output with q>p is written as +0.0.
 * Replaces Conv2dTritonFunction.forward + conv_fwd_kernel
 * (convolution_2d_trit.py:302-333, 52-135).  w is (C,R,S). */
int mta_conv2d_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H,
                   int64_t W, int R, int S, int causal, int io_dtype, int w_dtype, void *stream);

/* mta_conv2d_fwd with causal = 1 for a consumer that never reads above the diagonal (mta_headmix_*, mta_causal_pv_fwd):
 * what lies there in y is unspecified - left alone on square tensors that take the matrix-core kernel, +0.0 otherwise.
 * A third of the bytes of a causal conv are that fill.  Same citation as mta_conv2d_fwd; the reference zero-fills
 * (convolution_2d_trit.py:313) whoever reads the result. */
int mta_conv2d_tril_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H, int64_t W, int R, int S,
                        int io_dtype, int w_dtype, void *stream);

/* Same op with the input multiplied by `in_scale` as it is read (products are formed
 * in fp32 and, for 16-bit I/O, rounded to the I/O dtype before the taps, which is what
 * a separate elementwise scale in that dtype would produce).  Lets the caller fold
 * the 1/sqrt(D) of mta_attention_triton.py:69-71 into the conv's staging pass. */
int mta_conv2d_scaled_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t H,
                          int64_t W, int R, int S, int causal, float in_scale, int io_dtype,
                          int w_dtype, void *stream);

/* Head mixing over axis 1 of an (N,C,P,Q) tensor, no transpose:
 *   y[n,o,p,q] = sum_i w[o,i] * x[n,i,p,q]          (w is (C,C), row = output head)
 * When causal every q>p is written as `fill` (0 or -inf) and never read.
 * group_size = 0: w is dense.  group_size = G > 0: the caller promises w is zero
 * outside its GxG diagonal blocks; only the blocks are read.
 * Replaces TritonLinearHeadFunction.forward + linear_head_kernel_forward
 * (triton_linear_head.py:283-319, 76-139). */
int mta_headmix_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t P,
                    int64_t Q, int group_size, int causal, float fill, int io_dtype, int w_dtype,
                    void *stream);

/* mta_headmix_fwd with causal = 1 for a consumer that never reads above the diagonal: vectors of y wholly above it
 * are not written (elements above it that share a 16-byte vector with the diagonal are written as +0.0).  Same citation
 * as mta_headmix_fwd; the reference pre-fills the output (triton_linear_head.py:294-297). */
int mta_headmix_tril_fwd(const void *x, const void *w, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                         int group_size, int io_dtype, int w_dtype, void *stream);

/* Gradient of the row softmax over the keys of an (N,C,P,Q) tensor, from the stored probabilities:
 *   dx[q] = p[q] * (dp[q] - sum_k p[k] * dp[k])      fp32 arithmetic, p / dp / dx in the I/O dtype
 * causal: keys q > row index take no part and are never read; dx there is written as +0.0 when
 * fill_upper != 0 and left alone otherwise.
 * Replaces torch's autograd through F.softmax(scores.float(), dim=-1).type_as(xq)
 * (mta_attention_triton.py:79), which keeps an fp32 copy of the probabilities and writes the product
 * p * dp before it reduces it; with p stored in 16 bits the result differs from that path by the
 * rounding of p. */
int mta_softmax_bwd(const void *p, const void *dp, void *dx, int64_t N, int64_t C, int64_t P, int64_t Q,
                    int causal, int fill_upper, int io_dtype, void *stream);

/* Fused head mixing + row softmax + head mixing over (N,C,P,Q), one pass:
 *   s[o] = w1 ? sum_i w1[o,i] x[i] : x[o]      (fp32, rounded to the I/O dtype;
 *                                               causal: q>p takes no part)
 *   p[o] = softmax over q of s[o]              (fp32, rounded to the I/O dtype)
 *   y[o] = w2 ? sum_i w2[o,i] p[i] : p[o]      (causal: q>p written as +0.0 when fill_upper != 0,
 *                                               unspecified when fill_upper == 0 (left alone, or zero
 *                                               where a tile straddles the diagonal) -- for a consumer
 *                                               such as mta_causal_pv_fwd that never reads it)
 * w1 and/or w2 may be NULL (identity); both NULL is a plain causal row softmax.
 * group_size as in mta_headmix_fwd and applies to both weights.
 * Replaces the wpsm_triton -> F.softmax(scores.float()).type_as(xq) -> wposm_triton
 * chain of mta_attention_triton.py:75-85 (the last link only when the post-softmax
 * conv between them is the identity; otherwise pass w2 = NULL). */
int mta_headmix_softmax_fwd(const void *x, const void *w1, const void *w2, void *y, int64_t N,
                            int64_t C, int64_t P, int64_t Q, int group_size, int causal,
                            int fill_upper, int io_dtype, int w_dtype, void *stream);

/* The same with an additive bias per (batch entry, key) on the mixed scores, ahead of the softmax:
 *   s[o] = round(s[o] + key_bias[n, q])        key_bias is fp32, (N,Q), 0 = keep, -inf = key hidden, or any
 *                                              finite value; NULL = none (identical to the entry point above).
 * This is the `scores = scores + mask` of mta_attention_triton.py:77-78 for the masks the reference builds from a
 * 2-D key mask (mta_attention_triton.py:118-122): causal rule plus one value per key, without the (B,H,S,S) mask
 * tensor.  A row whose attended keys are all hidden comes out as NaN, as the softmax of a row of -inf does. */
int mta_headmix_softmax_bias_fwd(const void *x, const void *w1, const void *w2, const void *key_bias, void *y,
                                 int64_t N, int64_t C, int64_t P, int64_t Q, int group_size, int causal,
                                 int fill_upper, int io_dtype, int w_dtype, void *stream);

/* The same under a band mask: first_visible is int32, (N,P); key q of query row p of batch entry n is hidden (its
 * mixed score becomes -inf ahead of the softmax) when q < first_visible[n, p]; NULL = no band (identical to the entry
 * point above).  With the causal rule this is the `scores + mask` of mta_attention_triton.py:77-78 for every mask of
 * the form "row p sees the keys first_visible[p] .. p" - sliding windows, packed documents - without the (B,H,S,S)
 * mask tensor.  key_bias may be given as well.  A row without a visible key comes out as NaN. */
int mta_headmix_softmax_band_fwd(const void *x, const void *w1, const void *w2, const void *key_bias,
                                 const void *first_visible, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                                 int group_size, int causal, int fill_upper, int io_dtype, int w_dtype, void *stream);

/* Depthwise causal conv followed by head mixing, the conv result never written:
 *   t[h] = round(conv2d(x[h], w_conv[h]))                     as mta_conv2d_fwd
 *   y[o] = round(sum_h w_mix[o,h] t[h])                        as mta_headmix_fwd with fill 0
 * x, y are (N,C,H,W); w_conv is (C,R,S); w_mix is (C,C) row = output head; group_size as in mta_headmix_fwd
 * (supported mixing groups: 1, 2, 4, 8, 16 heads; others return MTA_ERR_UNSUPPORTED and the two separate entry
 * points apply).  causal: q>p is written as +0.0 when fill_upper != 0 and left unspecified otherwise.
 * Replaces mta_conv_after_sm_triton -> wposm_triton of mta_attention_triton.py:81-85 (conv_fwd_kernel,
 * convolution_2d_trit.py:52-135, then linear_head_kernel_forward, triton_linear_head.py:76-139): one read and one
 * write of the probabilities instead of two of each. */
int mta_conv2d_headmix_fwd(const void *x, const void *w_conv, const void *w_mix, void *y, int64_t N, int64_t C,
                           int64_t H, int64_t W, int R, int S, int group_size, int causal, int fill_upper,
                           int io_dtype, int wconv_dtype, int wmix_dtype, void *stream);

/* Fused conv-attention forward:
 *   O = softmax( mask( conv( mask0(Q K^T) ) ) * scale ) V        per (batch, head)
 * q,k,v,o are (B,H,S,D); w is (H,R,Sk).  mask0 zeroes col>row before the conv, mask
 * sets col>row to -inf after it (both only when causal).  No S x S tensor is
 * written.  Replaces TritonAttention.forward + _attn_fwd + qk_conv_fwd_kernel
 * (conv_attention_triton.py:362-452, 167-356; qk_conv_kernel.py:11-184); the
 * reference's second output (the QK scratch) has no counterpart. */
int mta_conv_attn_fwd(const void *q, const void *k, const void *v, const void *w, void *o,
                      int64_t B, int64_t H, int64_t S, int64_t D, int R, int Sk, int causal,
                      float scale, int io_dtype, int w_dtype, void *stream);

/* mta_conv_attn_fwd that also writes, when lse != NULL, the row-wise log-sum-exp of the masked, scaled conv scores
 *   lse[b,h,p] = log sum_q exp( scale * conv(mask0(Q K^T))[p,q] )     (natural log, fp32, (B,H,S))
 * the per-row statistic a backward pass needs to rebuild the probabilities.  It is the `M` tensor of
 * TritonAttention.forward (conv_attention_triton.py:352-355, 402-404; m_i + log(l_i)). */
int mta_conv_attn_fwd_lse(const void *q, const void *k, const void *v, const void *w, void *o, void *lse,
                          int64_t B, int64_t H, int64_t S, int64_t D, int R, int Sk, int causal, float scale,
                          int io_dtype, int w_dtype, void *stream);

/* First half of the fused path, for the MTA pipeline (which must mix heads before its softmax):
 *   s_out[b,h] = conv( mask0(scale * Q K^T) )           an (S,S) plane per (batch, head)
 * (Q K^T is rounded to the I/O dtype, scaled and rounded again before the conv, as the unfused
 * pipeline does)
 * q,k are (B,H,S,D), w is (H,R,Sk), s_out is (B,H,S,S).  Replaces matmul -> *rsqrt(d) -> conv_fwd_kernel of
 * mta_attention_triton.py:69-73 without ever writing the raw scores.  When causal only q <= p is
 * defined; fill_upper != 0 also writes +0.0 everywhere above the diagonal (needed only if a consumer reads
 * it), otherwise what lies there is unspecified (left alone, or zero where a tile straddles the diagonal).
 * 16-bit I/O with weights of the same dtype, D in {64,128}, S % 8 == 0 and the kernel sizes that have a
 * matrix-core instantiation; anything else returns MTA_ERR_UNSUPPORTED and the caller takes the
 * unfused route. */
int mta_qk_conv_fwd(const void *q, const void *k, const void *w, void *s_out, int64_t B, int64_t H,
                    int64_t S, int64_t D, int R, int Sk, int causal, float scale, int fill_upper,
                    int io_dtype, int w_dtype, void *stream);

/* 1 when mta_qk_conv_fwd has a kernel for these sizes and dtypes, 0 when it would return MTA_ERR_UNSUPPORTED: lets the
 * caller choose between the one-kernel stage and matmul -> conv (mta_attention_triton.py:69-73) before it launches
 * anything.  Host-side only; needs no GPU. */
int mta_qk_conv_supported(int64_t S, int64_t D, int R, int Sk, int io_dtype, int w_dtype);

/* mta_qk_conv_fwd under a band mask (causal by construction): first_visible is int32, (B,S); the score of key k of
 * query row p enters the conv as 0 unless first_visible[b, p] <= k <= p - the `scores.masked_fill(mask == -inf, 0)`
 * ahead of the conv of mta_attention_triton.py:70-73 for masks of that form.  What is defined are the outputs at visible
 * positions; elsewhere below the diagonal the output is unspecified (key blocks ahead of the first key any row of a query
 * block sees are not even visited).  Same conditions and return codes as mta_qk_conv_fwd (mta_qk_conv_supported answers
 * for both). */
int mta_qk_conv_band_fwd(const void *q, const void *k, const void *w, const void *first_visible, void *s_out, int64_t B,
                         int64_t H, int64_t S, int64_t D, int R, int Sk, float scale, int fill_upper, int io_dtype,
                         int w_dtype, void *stream);

/* O = P V with P (B,H,S,S), V (B,H,S,D), O (B,H,S,D).  When causal only keys q <= p of P are read
 * (what lies above the diagonal may be uninitialised).  Replaces torch.matmul(scores, xv) of
 * mta_attention_triton.py:89 and halves its traffic.  16-bit I/O, D in {64,128}, S % 8 == 0; anything
 * else returns MTA_ERR_UNSUPPORTED. */
int mta_causal_pv_fwd(const void *p, const void *v, void *o, int64_t B, int64_t H, int64_t S, int64_t D,
                      int causal, int io_dtype, void *stream);

/* The same under a band mask: first_visible is int32, (B,S), or NULL; P[b,h,p,k] must be 0 for k < first_visible[b,p]
 * (what mta_headmix_softmax_band_fwd leaves there), and the key blocks ahead of the first key any row of a block of 128
 * query rows sees are not read.  Requires causal when first_visible is given. */
int mta_causal_pv_band_fwd(const void *p, const void *v, const void *first_visible, void *o, int64_t B, int64_t H,
                           int64_t S, int64_t D, int causal, int io_dtype, void *stream);

/* x[n,c,p,q] = 0 for q < first_visible[n,p], in place; x is (N,C,S,S), first_visible int32 (N,S).  The reference's
 * `scores = torch.where(mask == float("-inf"), 0.0, scores)` behind its post-softmax conv (mta_attention_triton.py:82-83)
 * for a band mask, below the diagonal (above it nothing is touched: the causal kernels on either side neither read nor
 * need it).  16-bit I/O, S % 8 == 0; MTA_ERR_UNSUPPORTED otherwise. */
int mta_band_zero_fwd(void *x, const void *first_visible, int64_t N, int64_t C, int64_t S, int io_dtype, void *stream);

/* y[n,c,p,q] = visible[n,c,p,q] ? x[n,c,p,q] : (neg_inf ? -inf : 0) for a mask tensor of arbitrary content: the
 * reference's `scores_masked[mask == float("-inf")] = 0` ahead of its two convs, its `scores = scores + mask` ahead of the
 * softmax for a 0 / -inf mask (neg_inf = 1) and its `torch.where(mask == float("-inf"), 0.0, scores)` behind the
 * post-softmax conv (mta_attention_triton.py:72-73, 77-78, 81-83), one pass each.  x, y: (N,C,P,Q), y may be x;
 * visible: uint8, non-zero = attend, (mask_batch, mask_heads, P, Q) with mask_batch 1 or N and mask_heads 1 or C
 * (broadcast), 8-byte aligned.  causal != 0: only keys q <= p are read and written.  Q % 8 == 0; MTA_ERR_UNSUPPORTED
 * otherwise. */
int mta_mask_fill_fwd(const void *x, const void *visible, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                      int mask_batch, int mask_heads, int neg_inf, int causal, int io_dtype, void *stream);

/* y = x + mask, rounded once to the I/O dtype: the reference's `scores = scores + mask` (mta_attention_triton.py:77-78)
 * for an additive mask with finite values.  mask: the scores' dtype, (mask_batch, mask_heads, P, Q) with mask_batch 1 or N
 * and mask_heads 1 or C (broadcast), 16-byte aligned; y may be x.  causal != 0: only keys q <= p are read and written.
 * Q % 8 == 0; MTA_ERR_UNSUPPORTED otherwise. */
int mta_mask_add_fwd(const void *x, const void *mask, void *y, int64_t N, int64_t C, int64_t P, int64_t Q,
                     int mask_batch, int mask_heads, int causal, int io_dtype, void *stream);

/* ---- The three stages of the causal forward (mta_attention_triton.py:68-89 without a post-softmax conv) over
 * score tensors in a TRIANGULAR LAYOUT.  The (B,H,S,S) tensors between the three kernels never leave the library's
 * caller, so their layout is free; this one stores what lies on and below the diagonal only and puts the rows that one
 * workgroup of the softmax stage reads side by side:
 *   row p holds len(p) = 64*(p/64 + 1) elements (keys 0..p, then padding of unspecified content);
 *   off(p) = 2048*a*(a+1) + (p%64)*64*(a+1), a = p/64, elements of one head lie ahead of row p;  T = off(S);
 *   the heads are taken in groups of `group` consecutive heads (H % group == 0) and a group's rows are interleaved:
 *   element (b, h, p, q <= p) sits at  ((b*H + h)/group)*group*T + group*off(p) + (h%group)*len(p) + q.
 * The tensor has B*H*T elements (about half of B*H*S*S).  Same values as the entry points they mirror; they have no
 * counterpart in the reference, whose kernels exchange full (B,H,S,S) tensors.  16-bit I/O only.
 *   mta_qk_conv_tri_fwd:         mta_qk_conv_fwd (causal) / mta_qk_conv_band_fwd (first_visible not NULL), output layout;
 *                                group*T must stay below 2^31.
 *   mta_headmix_softmax_tri_fwd: mta_headmix_softmax_fwd (causal, fill_upper = 0) / mta_headmix_softmax_bias_fwd (key_bias
 *                                not NULL; fp32 (N,S), 16-byte aligned) / mta_headmix_softmax_band_fwd, layout of
 *                                the input and, with out_planes = 0, of the output; the layout's group = group_size
 *                                (2, 4, 8 or 16); out_planes = 1 (groups of 16 only): the output as
 *                                (N,C,S,S) planes, nothing written above the diagonal; weights of the I/O dtype.
 *   mta_causal_pv_tri_fwd:       mta_causal_pv_band_fwd (causal), layout of P. */
int mta_qk_conv_tri_fwd(const void *q, const void *k, const void *w, const void *first_visible, void *s_out, int64_t B,
                        int64_t H, int64_t S, int64_t D, int R, int Sk, float scale, int group, int io_dtype, int w_dtype,
                        void *stream);
int mta_headmix_softmax_tri_fwd(const void *x, const void *w1, const void *w2, const void *key_bias, const void *first_visible,
                                void *y, int64_t N, int64_t C, int64_t S, int group_size, int out_planes, int io_dtype,
                                int w_dtype, void *stream);
int mta_causal_pv_tri_fwd(const void *p, const void *v, const void *first_visible, void *o, int64_t B, int64_t H, int64_t S,
                          int64_t D, int group, int io_dtype, void *stream);
/* 1 when mta_headmix_softmax_tri_fwd has a kernel for these sizes and dtypes (has_w1 / has_w2: which weights are given;
 * band: with first_visible; key_bias: with a key bias), else 0.  A host-side question: nothing is launched. */
int mta_headmix_softmax_tri_supported(int64_t C, int64_t S, int group_size, int out_planes, int io_dtype, int w_dtype,
                                      int has_w1, int has_w2, int band, int key_bias);

/* The transposed product, O[k,:] = sum_p P[p,k] X[p,:] with P (B,H,S,S), X and O (B,H,S,D); when causal only query rows
 * p >= k take part and nothing of P above the diagonal is read.  These are the gradients the two matrix products of the
 * attention leave on their right-hand operands, dV = P^T dO (mta_attention_triton.py:89) and dK = G^T Q (:69, G the
 * gradient of the raw scores), which the reference leaves to torch's autograd as full-square GEMMs.  Same conditions as
 * mta_causal_pv_fwd. */
int mta_causal_ptx_fwd(const void *p, const void *x, void *o, int64_t B, int64_t H, int64_t S, int64_t D,
                       int causal, int io_dtype, void *stream);

/* ---- backward of the two standalone operators -------------------------------------------------------------
 * Gradients flow through the same masks as the forward pass: with `causal`, entries of dy above the diagonal are
 * never read (the forward wrote a constant there) and gradients with respect to inputs above the diagonal are +0
 * (the forward never read them).  Weight gradients are written as fp32 whatever the I/O dtype, fully defined
 * (not accumulated into), and are bit-reproducible from run to run: partial sums are kept in fp32 registers,
 * written once per workgroup to `workspace` and added in a fixed order by a second kernel (the reference
 * accumulates in fp64 with atomics).  `workspace` is device memory of at least the size the matching
 * *_workspace() call returns for the same sizes (0 = sizes rejected); its contents before and after are garbage. */

/* dx[n,c,h,w] = sum_{i,j} w[c,i,j] * dym[n,c, h-i+(R-1), w-j+(S-1)/2], dym = dy with out-of-range and (causal)
 * q>p entries read as 0.  Replaces conv_bwd_input_kernel + the grad_input half of Conv2dTritonFunction.backward
 * (convolution_2d_trit.py:143-223, 344-358). */
int mta_conv2d_bwd_input(const void *dy, const void *w, void *dx, int64_t N, int64_t C, int64_t H, int64_t W,
                         int R, int S, int causal, int io_dtype, int w_dtype, void *stream);

/* dw[c,i,j] = sum_{n,p,q} xm[n,c, p+i-(R-1), q+j-(S-1)/2] * dym[n,c,p,q]; dw is (C,R,S) fp32.  Replaces
 * conv_bwd_weight_kernel + the grad_weight half of Conv2dTritonFunction.backward
 * (convolution_2d_trit.py:225-295, 360-376). */
int64_t mta_conv2d_bwd_weight_workspace(int64_t N, int64_t C, int64_t H, int64_t W, int R, int S);
int mta_conv2d_bwd_weight(const void *x, const void *dy, void *dw, void *workspace, int64_t workspace_bytes,
                          int64_t N, int64_t C, int64_t H, int64_t W, int R, int S, int causal, int io_dtype,
                          void *stream);

/* mta_conv2d_bwd_weight for callers that cannot allocate device memory or pass a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same kernels
 * and same result; the partial sums live in a 1 MiB array that the library holds statically on each device it runs
 * on.  Needs C*R*S*4 bytes <= 1 MiB (else MTA_ERR_WORKSPACE, nothing launched); with fewer partial kernels than
 * mta_conv2d_bwd_weight would use (large kernels) the sums are added in a different order.  Calls that overlap on
 * one device share that array and race: serialise them (one stream). */
int mta_conv2d_bwd_weight_noalloc(const void *x, const void *dy, void *dw, int64_t N, int64_t C, int64_t H, int64_t W,
                                  int R, int S, int causal, int io_dtype, void *stream);

/* dx[n,i,p,q] = sum_o w[o,i] * dy[n,o,p,q].  group_size as in mta_headmix_fwd.  Replaces
 * linear_head_kernel_backward_input (triton_linear_head.py:144-196, 330-348); the reference leaves dx above the
 * diagonal uninitialised (torch.empty_like), here it is +0. */
int mta_headmix_bwd_input(const void *dy, const void *w, void *dx, int64_t N, int64_t C, int64_t P, int64_t Q,
                          int group_size, int causal, int io_dtype, int w_dtype, void *stream);

/* dw[o,i] = sum_{n,p,q} dy[n,o,p,q] * x[n,i,p,q] (causal: q <= p only); dw is the dense (C,C) matrix in fp32,
 * C <= 128.  Replaces linear_head_kernel_backward_weight (triton_linear_head.py:199-278, 350-368). */
int64_t mta_headmix_bwd_weight_workspace(int64_t N, int64_t C, int64_t P, int64_t Q);
int mta_headmix_bwd_weight(const void *x, const void *dy, void *dw, void *workspace, int64_t workspace_bytes,
                           int64_t N, int64_t C, int64_t P, int64_t Q, int causal, int io_dtype, void *stream);

/* Structure of the small MTA parameters, evaluated on the device (one workgroup, a few microseconds).  The
 * reference has no counterpart: its glue (mta_attention_triton.py:69-89) always runs every stage.  The glue
 * of this build asks these when the caller requests that identity stages be skipped and block-diagonal head
 * weights be applied block by block.
 * mta_probe_head_weight: w is (H,H); out[0] = 1 when w is exactly the identity, out[1] = the smallest G
 * dividing H such that w is zero outside its GxG diagonal blocks (H if none smaller).
 * mta_probe_conv_kernel: w is (C,R,S); out[0] = 1 when every channel is 1.0 at [R-1, S/2] and 0 elsewhere and
 * S is odd (the conv then passes its masked input through).
 * `out` is device memory (2 resp. 1 int32), written on `stream`. */
int mta_probe_head_weight(const void *w, int64_t H, int w_dtype, int32_t *out, void *stream);
int mta_probe_conv_kernel(const void *w, int64_t C, int R, int S, int w_dtype, int32_t *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MTA_HIP_H */
