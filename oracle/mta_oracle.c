/* Brute-force C restatement of the Multi-Token-Attention forward path.
 * TEST INFRASTRUCTURE ONLY: built into oracle/libmta_oracle.so and loaded by
 * tests/, smoke() and bench.py's cpu_baseline leg; never by the product package.
 *
 * Plain nested loops, double accumulation, float in/out, no library calls except
 * exp().  Its job is to pin oracle/mta_oracle.py (which uses torch library routines)
 * on small shapes, so that a wrong pad side, a flipped kernel, a transposed head
 * weight or a misplaced scale in either restatement shows up as a mismatch.
 *
 * Reference lines restated:
 *   conv            mta_attention_pytorch.py:85-112, convolution_2d_trit.py:96-117,126-133,310-311
 *   head mixing     mta_attention_pytorch.py:68,76, triton_linear_head.py:89-95,111-113,135-139,294-297
 *   MTA forward     mta_attention_pytorch.py:58-83
 *   conv attention  conv_attention_pytorch.py:33-92
 *   backward        convolution_2d_trit.py:143-295, triton_linear_head.py:144-278
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

/* out[n,c,p,q] = sum_{i<R,j<S} w[c,i,j] * xm[n,c,p+i-(R-1), q+j-(S-1)/2]
 * xm = x with out-of-range -> 0 and (causal) col>row -> 0; causal outputs q>p are +0. */
void oracle_conv2d(const float *x, const float *w, float *y, int64_t N, int64_t C, int64_t H,
                   int64_t W, int R, int S, int causal)
{
    const int pad_h = R - 1, pad_w = (S - 1) / 2;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c) {
            const float *xp = x + (n * C + c) * H * W;
            float *yp = y + (n * C + c) * H * W;
            const float *wp = w + c * R * S;
            for (int64_t p = 0; p < H; ++p)
                for (int64_t q = 0; q < W; ++q) {
                    if (causal && q > p) { yp[p * W + q] = 0.0f; continue; }
                    double acc = 0.0;
                    for (int i = 0; i < R; ++i) {
                        int64_t h = p + i - pad_h;
                        if (h < 0 || h >= H) continue;
                        for (int j = 0; j < S; ++j) {
                            int64_t k = q + j - pad_w;
                            if (k < 0 || k >= W) continue;
                            if (causal && k > h) continue;
                            acc += (double)wp[i * S + j] * (double)xp[h * W + k];
                        }
                    }
                    yp[p * W + q] = (float)acc;
                }
        }
}

/* y[n,o,p,q] = sum_i Wt[o,i] x[n,i,p,q]; causal: q>p holds `fill`. */
void oracle_headmix(const float *x, const float *wt, float *y, int64_t N, int64_t C, int64_t P,
                    int64_t Q, int causal, float fill)
{
    for (int64_t n = 0; n < N; ++n)
        for (int64_t o = 0; o < C; ++o)
            for (int64_t p = 0; p < P; ++p)
                for (int64_t q = 0; q < Q; ++q) {
                    float *dst = y + ((n * C + o) * P + p) * Q + q;
                    if (causal && q > p) { *dst = fill; continue; }
                    double acc = 0.0;
                    for (int64_t i = 0; i < C; ++i)
                        acc += (double)wt[o * C + i] * (double)x[((n * C + i) * P + p) * Q + q];
                    *dst = (float)acc;
                }
}

/* Backward of the conv, restated from the reference's own backward kernels (not derived from the forward above):
 * conv_bwd_input_kernel (convolution_2d_trit.py:143-223):
 *   dx[h,w] = sum_{i,j} w[i,j] * dy[h-i+pad_h, w-j+pad_w], dy read as 0 out of range and (causal) where col>row;
 *   (causal) dx stays 0 where w>h.
 * conv_bwd_weight_kernel (convolution_2d_trit.py:225-295):
 *   dw[i,j] = sum_{n,p,q} x[p+i-pad_h, q+j-pad_w] * dy[p,q], both read as 0 out of range and (causal) where col>row. */
void oracle_conv2d_bwd(const float *x, const float *w, const float *dy, float *dx, double *dw, int64_t N,
                       int64_t C, int64_t H, int64_t W, int R, int S, int causal)
{
    const int pad_h = R - 1, pad_w = (S - 1) / 2;
    for (int64_t c = 0; c < C; ++c)
        for (int t = 0; t < R * S; ++t) dw[c * R * S + t] = 0.0;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c) {
            const float *xp = x + (n * C + c) * H * W, *gp = dy + (n * C + c) * H * W;
            float *dxp = dx + (n * C + c) * H * W;
            const float *wp = w + c * R * S;
            for (int64_t h = 0; h < H; ++h)
                for (int64_t k = 0; k < W; ++k) {
                    double acc = 0.0;
                    if (!(causal && k > h))
                        for (int i = 0; i < R; ++i) {
                            int64_t oh = h - i + pad_h;
                            if (oh < 0 || oh >= H) continue;
                            for (int j = 0; j < S; ++j) {
                                int64_t ow = k - j + pad_w;
                                if (ow < 0 || ow >= W) continue;
                                if (causal && ow > oh) continue;
                                acc += (double)wp[i * S + j] * (double)gp[oh * W + ow];
                            }
                        }
                    dxp[h * W + k] = (float)acc;
                }
            for (int i = 0; i < R; ++i)
                for (int j = 0; j < S; ++j) {
                    double acc = 0.0;
                    for (int64_t p = 0; p < H; ++p)
                        for (int64_t q = 0; q < W; ++q) {
                            if (causal && q > p) continue;
                            int64_t ih = p + i - pad_h, iw = q + j - pad_w;
                            if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                            if (causal && iw > ih) continue;
                            acc += (double)xp[ih * W + iw] * (double)gp[p * W + q];
                        }
                    dw[c * R * S + i * S + j] += acc;
                }
        }
}

/* Backward of the head mixing, restated from linear_head_kernel_backward_input / _weight
 * (triton_linear_head.py:144-278): dx[n,i,p,q] = sum_o dy[n,o,p,q] w[o,i]; dw[o,i] = sum_{n,p,q} dy[n,o,p,q] x[n,i,p,q];
 * with causal only q <= p take part (dx is left untouched above the diagonal there; 0 here). */
void oracle_headmix_bwd(const float *x, const float *wt, const float *dy, float *dx, double *dw, int64_t N, int64_t C,
                        int64_t P, int64_t Q, int causal)
{
    for (int64_t e = 0; e < C * C; ++e) dw[e] = 0.0;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t p = 0; p < P; ++p)
            for (int64_t q = 0; q < Q; ++q) {
                const int live = !(causal && q > p);
                for (int64_t i = 0; i < C; ++i) {
                    double acc = 0.0;
                    if (live)
                        for (int64_t o = 0; o < C; ++o)
                            acc += (double)dy[((n * C + o) * P + p) * Q + q] * (double)wt[o * C + i];
                    dx[((n * C + i) * P + p) * Q + q] = (float)acc;
                }
                if (live)
                    for (int64_t o = 0; o < C; ++o)
                        for (int64_t i = 0; i < C; ++i)
                            dw[o * C + i] += (double)dy[((n * C + o) * P + p) * Q + q] * (double)x[((n * C + i) * P + p) * Q + q];
            }
}

static void conv_plane_d(const double *x, const float *w, double *y, int64_t S, int R, int Sk)
{
    /* depthwise conv of one S x S plane held in double (blocked entries already zeroed by the
     * caller); output NOT masked */
    const int pad_h = R - 1, pad_w = (Sk - 1) / 2;
    for (int64_t p = 0; p < S; ++p)
        for (int64_t q = 0; q < S; ++q) {
            double acc = 0.0;
            for (int i = 0; i < R; ++i) {
                int64_t h = p + i - pad_h;
                if (h < 0) continue;
                for (int j = 0; j < Sk; ++j) {
                    int64_t k = q + j - pad_w;
                    if (k < 0 || k >= S) continue;
                    acc += (double)w[i * Sk + j] * x[h * S + k];
                }
            }
            y[p * S + q] = acc;
        }
}

/* MTA forward (pad_key="both", dropout 0), all in double.
 * q,k,v: (B,H,S,D); w_pre: (H,R1,S1); wpsm,wposm: (H,H) row = output head;
 * w_post: (H,R2,S2); out: (B,S,H,D).
 * mask: NULL = plain causal, else an additive (B,H,S,S) mask of 0 / -inf entries (what
 * _update_mask of mta_attention_pytorch.py:114-137 hands to forward): blocked scores are
 * zeroed before each conv (:89), -inf is added before the softmax (:69), blocked
 * probabilities are zeroed after the second conv (:74).  A query row with every key
 * blocked gives NaN, as torch's softmax does.
 * Returns 0, or -1 when out of memory. */
int oracle_mta_forward(const float *q, const float *k, const float *v, const float *w_pre,
                       const float *wpsm, const float *w_post, const float *wposm,
                       const float *mask, float *out,
                       int64_t B, int64_t H, int64_t S, int64_t D, int R1, int S1, int R2, int S2)
{
    const int64_t plane = S * S;
    double *a = (double *)malloc(sizeof(double) * H * plane);
    double *b = (double *)malloc(sizeof(double) * H * plane);
    unsigned char *blk = (unsigned char *)malloc((size_t)(H * plane));
    if (!a || !b || !blk) { free(a); free(b); free(blk); return -1; }
    const double scale = 1.0 / sqrt((double)D);
    for (int64_t n = 0; n < B; ++n) {
        for (int64_t h = 0; h < H; ++h)
            for (int64_t p = 0; p < S; ++p)
                for (int64_t c = 0; c < S; ++c)
                    blk[h * plane + p * S + c] =
                        mask ? (unsigned char)(mask[((n * H + h) * S + p) * S + c] == -INFINITY)
                             : (unsigned char)(c > p);
        /* s0 = q k^T * scale, zero where blocked (the conv's input mask) */
        for (int64_t h = 0; h < H; ++h)
            for (int64_t p = 0; p < S; ++p)
                for (int64_t c = 0; c < S; ++c) {
                    double acc = 0.0;
                    if (!blk[h * plane + p * S + c])
                        for (int64_t d = 0; d < D; ++d)
                            acc += (double)q[((n * H + h) * S + p) * D + d] *
                                   (double)k[((n * H + h) * S + c) * D + d];
                    a[h * plane + p * S + c] = acc * scale;
                }
        /* s1 = conv_pre(s0) */
        for (int64_t h = 0; h < H; ++h)
            conv_plane_d(a + h * plane, w_pre + h * R1 * S1, b + h * plane, S, R1, S1);
        /* s2 = wpsm . s1 over heads, then + mask, softmax over keys */
        for (int64_t p = 0; p < S; ++p)
            for (int64_t o = 0; o < H; ++o) {
                const unsigned char *bl = blk + o * plane + p * S;
                double mx = -INFINITY;
                for (int64_t c = 0; c < S; ++c) {
                    if (bl[c]) continue;
                    double acc = 0.0;
                    for (int64_t i = 0; i < H; ++i)
                        acc += (double)wpsm[o * H + i] * b[i * plane + p * S + c];
                    a[o * plane + p * S + c] = acc;
                    if (acc > mx) mx = acc;
                }
                double den = 0.0;
                for (int64_t c = 0; c < S; ++c) {
                    if (bl[c]) continue;
                    double e = exp(a[o * plane + p * S + c] - mx);
                    a[o * plane + p * S + c] = e;
                    den += e;
                }
                for (int64_t c = 0; c < S; ++c)
                    a[o * plane + p * S + c] = bl[c] ? 0.0 : a[o * plane + p * S + c] / den;
            }
        /* p1 = conv_post(p0) (p0 is already 0 where blocked), then zero where blocked */
        for (int64_t h = 0; h < H; ++h) {
            conv_plane_d(a + h * plane, w_post + h * R2 * S2, b + h * plane, S, R2, S2);
            for (int64_t p = 0; p < S; ++p)
                for (int64_t c = 0; c < S; ++c)
                    if (blk[h * plane + p * S + c]) b[h * plane + p * S + c] = 0.0;
        }
        /* p2 = wposm . p1 ; out = p2 v, stored (B,S,H,D) */
        for (int64_t o = 0; o < H; ++o)
            for (int64_t p = 0; p < S; ++p) {
                for (int64_t c = 0; c < S; ++c) {
                    double acc = 0.0;
                    for (int64_t i = 0; i < H; ++i)
                        acc += (double)wposm[o * H + i] * b[i * plane + p * S + c];
                    a[o * plane + p * S + c] = acc;
                }
                for (int64_t d = 0; d < D; ++d) {
                    double acc = 0.0;
                    for (int64_t c = 0; c < S; ++c)
                        acc += a[o * plane + p * S + c] * (double)v[((n * H + o) * S + c) * D + d];
                    out[((n * S + p) * H + o) * D + d] = (float)acc;
                }
            }
    }
    free(a);
    free(b);
    free(blk);
    return 0;
}

/* O = softmax(mask(conv(mask0(Q K^T))) * scale) V, (B,H,S,D) -> (B,H,S,D). */
int oracle_conv_attention(const float *q, const float *k, const float *v, const float *w,
                          float *o, int64_t B, int64_t H, int64_t S, int64_t D, int R, int Sk,
                          int causal, float scale)
{
    const int64_t plane = S * S;
    double *a = (double *)malloc(sizeof(double) * plane);
    double *b = (double *)malloc(sizeof(double) * plane);
    if (!a || !b) { free(a); free(b); return -1; }
    const int pad_h = R - 1, pad_w = (Sk - 1) / 2;
    for (int64_t n = 0; n < B; ++n)
        for (int64_t h = 0; h < H; ++h) {
            const float *qp = q + (n * H + h) * S * D, *kp = k + (n * H + h) * S * D;
            const float *vp = v + (n * H + h) * S * D, *wp = w + h * R * Sk;
            float *op = o + (n * H + h) * S * D;
            for (int64_t p = 0; p < S; ++p)
                for (int64_t c = 0; c < S; ++c) {
                    double acc = 0.0;
                    if (!causal || c <= p)
                        for (int64_t d = 0; d < D; ++d) acc += (double)qp[p * D + d] * (double)kp[c * D + d];
                    a[p * S + c] = acc;
                }
            for (int64_t p = 0; p < S; ++p)
                for (int64_t c = 0; c < S; ++c) {
                    double acc = 0.0;
                    for (int i = 0; i < R; ++i) {
                        int64_t hh = p + i - pad_h;
                        if (hh < 0) continue;
                        for (int j = 0; j < Sk; ++j) {
                            int64_t kk = c + j - pad_w;
                            if (kk < 0 || kk >= S) continue;
                            acc += (double)wp[i * Sk + j] * a[hh * S + kk];
                        }
                    }
                    b[p * S + c] = acc;
                }
            for (int64_t p = 0; p < S; ++p) {
                const int64_t last = causal ? p : S - 1;
                double mx = -INFINITY, den = 0.0;
                for (int64_t c = 0; c <= last; ++c) {
                    b[p * S + c] *= (double)scale;
                    if (b[p * S + c] > mx) mx = b[p * S + c];
                }
                for (int64_t c = 0; c <= last; ++c) {
                    b[p * S + c] = exp(b[p * S + c] - mx);
                    den += b[p * S + c];
                }
                for (int64_t d = 0; d < D; ++d) {
                    double acc = 0.0;
                    for (int64_t c = 0; c <= last; ++c) acc += b[p * S + c] * (double)vp[c * D + d];
                    op[p * D + d] = (float)(acc / den);
                }
            }
        }
    free(a);
    free(b);
    return 0;
}
