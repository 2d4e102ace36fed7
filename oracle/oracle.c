/*
 * CPU oracle for the OriginDL hot path — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 * See oracle.h for scope, pinning status and who may load this.
 * Each function cites the reference file:line whose loop order and rounding it restates
 * (paths relative to the reference checkout).
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ===================================================================================== GEMM */

/* src/mat/origin/cpu/math/matmul.cpp:27-41 — i, j, then k ascending; float accumulator starting at 0. */
void orc_matmul_rows(const float *a, const float *b, float *c_rows, int64_t row0, int64_t row1, int64_t n, int64_t k)
{
    for (int64_t i = row0; i < row1; ++i)
    {
        for (int64_t j = 0; j < n; ++j)
        {
            float sum = 0.0f;
            for (int64_t kk = 0; kk < k; ++kk)
            {
                sum += a[i * k + kk] * b[kk * n + j];
            }
            c_rows[(i - row0) * n + j] = sum;
        }
    }
}

void orc_matmul(const float *a, const float *b, float *c, int64_t m, int64_t n, int64_t k)
{
    orc_matmul_rows(a, b, c, 0, m, n, k);
}

/* matmul.cpp:55-76 (B shared) and 91-109 (B batched) */
/* the same loops over doubles: the reference's matmul is a template over the element type (matmul.cpp:27-41) */
void orc_matmul_f64(const double *a, const double *b, double *c, int64_t m, int64_t n, int64_t k)
{
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j)
        {
            double sum = 0.0;
            for (int64_t p = 0; p < k; ++p)
                sum += a[i * k + p] * b[p * n + j];
            c[i * n + j] = sum;
        }
}

void orc_matmul_batched(const float *a, const float *b, float *c, int64_t batch, int64_t m, int64_t n, int64_t k,
                        int b_is_batched)
{
    for (int64_t bt = 0; bt < batch; ++bt)
    {
        orc_matmul(a + bt * m * k, b_is_batched ? b + bt * k * n : b, c + bt * m * n, m, n, k);
    }
}

/* operation_templates.h:374-390 (outer==1) and 401-416 (last two dims of a higher-rank tensor) */
void orc_transpose(const float *src, float *dst, int64_t outer, int64_t rows, int64_t cols)
{
    for (int64_t o = 0; o < outer; ++o)
    {
        for (int64_t i = 0; i < rows; ++i)
        {
            for (int64_t j = 0; j < cols; ++j)
            {
                dst[o * rows * cols + j * rows + i] = src[o * rows * cols + i * cols + j];
            }
        }
    }
}

/* src/operators/math/mat_mul.cpp:171-177 */
void orc_matmul_backward(const float *x, const float *w, const float *gy, float *gx, float *gw, int64_t m, int64_t k,
                         int64_t n)
{
    float *wT = (float *)malloc(sizeof(float) * (size_t)(k * n));
    float *xT = (float *)malloc(sizeof(float) * (size_t)(m * k));
    orc_transpose(w, wT, 1, k, n); /* w[K,N] -> wT[N,K] */
    orc_transpose(x, xT, 1, m, k); /* x[M,K] -> xT[K,M] */
    orc_matmul(gy, wT, gx, m, k, n); /* gx[M,K] = gy[M,N] . wT[N,K] */
    orc_matmul(xT, gy, gw, k, n, m); /* gw[K,N] = xT[K,M] . gy[M,N] */
    free(wT);
    free(xT);
}

/* ============================================================================== convolution */

int64_t orc_conv_outsize(int64_t in, int64_t k, int64_t s, int64_t p)
{
    /* include/origin/utils/conv_utils.h: C integer division (truncation toward zero) */
    return (in + p * 2 - k) / s + 1;
}

/* conv2d.cpp:91-114 — explicit zero-padded copy */
static float *pad_image(const float *img, int64_t N, int64_t C, int64_t H, int64_t W, int PH, int PW)
{
    int64_t pH = H + 2 * PH, pW = W + 2 * PW;
    float *p = (float *)calloc((size_t)(N * C * pH * pW), sizeof(float));
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t h = 0; h < H; ++h)
                for (int64_t w = 0; w < W; ++w)
                    p[((n * C + c) * pH + h + PH) * pW + w + PW] = img[((n * C + c) * H + h) * W + w];
    return p;
}

int orc_im2col(const float *img, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
               int PW, int to_matrix, float *col)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG; /* conv2d.cpp:69-75 */
    int64_t pH = H + 2 * PH, pW = W + 2 * PW;
    float *p = pad_image(img, N, C, H, W, PH, PW);
    memset(col, 0, sizeof(float) * (size_t)(N * C * KH * KW * OH * OW));
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int kh = 0; kh < KH; ++kh)
                for (int kw = 0; kw < KW; ++kw)
                    for (int64_t oh = 0; oh < OH; ++oh)
                        for (int64_t ow = 0; ow < OW; ++ow)
                        {
                            int64_t hi = kh + SH * oh, wi = kw + SW * ow;
                            if (hi < pH && wi < pW) /* conv2d.cpp:146, 186 */
                            {
                                float v = p[((n * C + c) * pH + hi) * pW + wi];
                                if (to_matrix) /* conv2d.cpp:116-162 */
                                    col[((n * OH + oh) * OW + ow) * (C * KH * KW) + (c * KH + kh) * KW + kw] = v;
                                else /* conv2d.cpp:164-206 */
                                    col[((((n * C + c) * KH + kh) * KW + kw) * OH + oh) * OW + ow] = v;
                            }
                        }
    free(p);
    return ORC_OK;
}

int orc_col2im(const float *col, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
               int PW, int to_matrix, float *img)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG;
    int64_t pH = H + 2 * PH, pW = W + 2 * PW;
    float *p = (float *)calloc((size_t)(N * C * pH * pW), sizeof(float));
    /* conv2d.cpp:320-349 — accumulation order n, c, kh, kw, oh, ow ascending */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int kh = 0; kh < KH; ++kh)
                for (int kw = 0; kw < KW; ++kw)
                    for (int64_t oh = 0; oh < OH; ++oh)
                        for (int64_t ow = 0; ow < OW; ++ow)
                        {
                            int64_t hi = kh + SH * oh, wi = kw + SW * ow;
                            if (hi < pH && wi < pW)
                            {
                                float v = to_matrix
                                              ? col[((n * OH + oh) * OW + ow) * (C * KH * KW) + (c * KH + kh) * KW + kw]
                                              : col[((((n * C + c) * KH + kh) * KW + kw) * OH + oh) * OW + ow];
                                p[((n * C + c) * pH + hi) * pW + wi] += v;
                            }
                        }
    /* conv2d.cpp:352-369 — strip the padding */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t h = 0; h < H; ++h)
                for (int64_t w = 0; w < W; ++w)
                    img[((n * C + c) * H + h) * W + w] = p[((n * C + c) * pH + h + PH) * pW + w + PW];
    free(p);
    return ORC_OK;
}

int orc_conv2d(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
               int KH, int KW, int SH, int SW, int PH, int PW, float *y)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG; /* conv2d.cpp:438-444 */
    int64_t M = N * OH * OW, K = C * KH * KW;
    float *col = (float *)malloc(sizeof(float) * (size_t)(M * K));
    float *wT = (float *)malloc(sizeof(float) * (size_t)(K * OC));
    float *yf = (float *)malloc(sizeof(float) * (size_t)(M * OC));
    orc_im2col(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, col); /* conv2d.cpp:460 */
    orc_transpose(w, wT, 1, OC, K);                             /* 463-464: W[OC,K] -> W_T[K,OC] */
    orc_matmul(col, wT, yf, M, OC, K);                          /* 469 */
    if (b) /* 472-479: bias broadcast to [M,OC] then one float add per element */
        for (int64_t i = 0; i < M; ++i)
            for (int64_t oc = 0; oc < OC; ++oc)
                yf[i * OC + oc] = yf[i * OC + oc] + b[oc];
    /* 489-509: NHWC -> NCHW */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t oc = 0; oc < OC; ++oc)
            for (int64_t oh = 0; oh < OH; ++oh)
                for (int64_t ow = 0; ow < OW; ++ow)
                    y[((n * OC + oc) * OH + oh) * OW + ow] = yf[((n * OH + oh) * OW + ow) * OC + oc];
    free(col);
    free(wT);
    free(yf);
    return ORC_OK;
}

int orc_conv2d_backward(const float *gy, const float *x, const float *w, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *gx, float *gw, float *gb)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG;
    int64_t M = N * OH * OW, K = C * KH * KW;
    /* conv2d.cpp:548 — gy's NCHW buffer is *viewed* as a row-major [M, OC] matrix, no permutation. */
    const float *gy2d = gy;
    float *gyT = (float *)malloc(sizeof(float) * (size_t)(M * OC));
    float *col = (float *)malloc(sizeof(float) * (size_t)(M * K));
    orc_transpose(gy2d, gyT, 1, M, OC);                         /* 550: [M,OC] -> [OC,M] */
    orc_im2col(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, col); /* 554 */
    orc_matmul(gyT, col, gw, OC, K, M);                         /* 559: gW[OC,K] */
    if (gb)
    {
        /* 571-575: gy.sum(2) -> [N,OC,OW]; .sum(2) -> [N,OC]; .sum(0) -> [OC], on the true NCHW gy */
        float *s1 = (float *)malloc(sizeof(float) * (size_t)(N * OC * OW));
        float *s2 = (float *)malloc(sizeof(float) * (size_t)(N * OC));
        orc_sum_axis(gy, N * OC, OH, OW, s1);
        orc_sum_axis(s1, N * OC, OW, 1, s2);
        orc_sum_axis(s2, 1, N, OC, gb);
        free(s1);
        free(s2);
    }
    /* 584-596: gx_col[M,K] = gy2d[M,OC] . W2d[OC,K]; gx = col2im(gx_col) */
    orc_matmul(gy2d, w, col, M, K, OC);
    orc_col2im(col, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, gx);
    free(gyT);
    free(col);
    return ORC_OK;
}

/* ================================================================== reductions / broadcast */

/* operation_templates.h:270-333: for each output (o, i): sequential sum over the axis, ascending. */
void orc_sum_axis(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst)
{
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t i = 0; i < inner; ++i)
        {
            float s = 0.0f;
            for (int64_t a = 0; a < axis; ++a)
                s += src[(o * axis + a) * inner + i];
            dst[o * inner + i] = s;
        }
}

/* operation_templates.h:342-357; sum.cpp:82-90 (T == float: the cast through float is the identity) */
float orc_sum_all(const float *src, int64_t n)
{
    float s = 0.0f;
    for (int64_t i = 0; i < n; ++i)
        s += src[i];
    return s;
}

/* max.cpp:58-117: starts from lowest(), std::max(max_val, v) keeps max_val unless max_val < v */
void orc_max_axis(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst)
{
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t i = 0; i < inner; ++i)
        {
            float m = -3.402823466e+38f;
            for (int64_t a = 0; a < axis; ++a)
            {
                float v = src[(o * axis + a) * inner + i];
                m = (m < v) ? v : m;
            }
            dst[o * inner + i] = m;
        }
}

/* max.cpp:25-40 */
float orc_max_all(const float *src, int64_t n)
{
    float m = src[0];
    for (int64_t i = 1; i < n; ++i)
        m = (m < src[i]) ? src[i] : m;
    return m;
}

static int64_t prod(const int64_t *s, int n)
{
    int64_t p = 1;
    for (int i = 0; i < n; ++i)
        p *= s[i];
    return p;
}

/* sum_to.cpp:11-76 */
int orc_sum_to(const float *src, const int64_t *sshape, int sn, const int64_t *tshape, int tn, float *dst)
{
    int64_t se = prod(sshape, sn), te = prod(tshape, tn);
    int same = (sn == tn);
    for (int i = 0; same && i < sn; ++i)
        same = (sshape[i] == tshape[i]);
    if (same) /* 14-18 */
    {
        memcpy(dst, src, sizeof(float) * (size_t)se);
        return ORC_OK;
    }
    if (te > se) /* 24-28 */
        return ORC_ERR_RUNTIME;
    int sum_dims[16];
    int nd = 0;
    int mind = sn < tn ? sn : tn;
    for (int i = 0; i < mind; ++i) /* 36-42: compared from the LEFT */
        if (tshape[i] == 1 && sshape[i] > 1)
            sum_dims[nd++] = i;
    for (int i = tn; i < sn; ++i) /* 46-52: surplus trailing source dims */
        sum_dims[nd++] = i;
    /* 58: descending order (the list above is already ascending) */
    int64_t cur_shape[16];
    int cn = sn;
    memcpy(cur_shape, sshape, sizeof(int64_t) * (size_t)sn);
    float *cur = (float *)malloc(sizeof(float) * (size_t)(se > 0 ? se : 1));
    memcpy(cur, src, sizeof(float) * (size_t)se);
    for (int d = nd - 1; d >= 0; --d)
    {
        int ax = sum_dims[d];
        int64_t outer = prod(cur_shape, ax), axis = cur_shape[ax], inner = prod(cur_shape + ax + 1, cn - ax - 1);
        float *next = (float *)malloc(sizeof(float) * (size_t)(outer * inner > 0 ? outer * inner : 1));
        orc_sum_axis(cur, outer, axis, inner, next); /* 60-63: keepdim=false */
        free(cur);
        cur = next;
        for (int i = ax; i < cn - 1; ++i)
            cur_shape[i] = cur_shape[i + 1];
        --cn;
    }
    /* 66-71: reshape to the target; reshape throws when the element counts differ */
    int64_t ce = prod(cur_shape, cn);
    if (ce != te)
    {
        free(cur);
        return ORC_ERR_INVALID_ARG;
    }
    memcpy(dst, cur, sizeof(float) * (size_t)te);
    free(cur);
    return ORC_OK;
}

/* operation_templates.h:433-493: right-aligned; a source dim of size 1 is read at index 0 */
void orc_broadcast_to(const float *src, const int64_t *sshape, int sn, const int64_t *dshape, int dn, float *dst)
{
    int64_t sstr[16], total = prod(dshape, dn);
    int64_t st = 1;
    for (int i = sn - 1; i >= 0; --i)
    {
        sstr[i] = st;
        st *= sshape[i];
    }
    for (int64_t di = 0; di < total; ++di)
    {
        int64_t t = di, si = 0;
        for (int i = 0; i < dn; ++i)
        {
            int dd = dn - 1 - i, sd = sn - 1 - i;
            int64_t ix = t % dshape[dd];
            t /= dshape[dd];
            if (sd >= 0)
                si += (sshape[sd] == 1 ? 0 : ix) * sstr[sd];
        }
        dst[di] = src[si];
    }
}

/* ============================================================ softmax / cross entropy */

/* softmax.cpp:37-74: max(axis) -> x - max -> exp -> sum(axis) (sequential) -> divide */
void orc_softmax(const float *x, int64_t outer, int64_t axis, int64_t inner, float *y)
{
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t i = 0; i < inner; ++i)
        {
            float m = -3.402823466e+38f;
            for (int64_t a = 0; a < axis; ++a)
            {
                float v = x[(o * axis + a) * inner + i];
                m = (m < v) ? v : m;
            }
            float s = 0.0f;
            for (int64_t a = 0; a < axis; ++a)
            {
                float e = expf(x[(o * axis + a) * inner + i] - m);
                y[(o * axis + a) * inner + i] = e;
                s += e;
            }
            for (int64_t a = 0; a < axis; ++a)
                y[(o * axis + a) * inner + i] = y[(o * axis + a) * inner + i] / s;
        }
}

static int64_t label_at(const void *idx, int is64, int64_t i)
{
    return is64 ? ((const int64_t *)idx)[i] : (int64_t)((const int32_t *)idx)[i];
}

/* gather.cpp:21-88: out[i] = in[i*C + idx[i]]; an out-of-range index throws invalid_argument (64-67, 78-81) */
int orc_gather(const float *in, const void *idx, int is64, int64_t N, int64_t C, float *out)
{
    for (int64_t i = 0; i < N; ++i)
    {
        int64_t t = label_at(idx, is64, i);
        if (t < 0 || t >= C)
            return ORC_ERR_INVALID_ARG;
        out[i] = in[i * C + t];
    }
    return ORC_OK;
}

/* gather.cpp:91-158: zero fill, then 1.0 where the index is in range; out-of-range is silently skipped */
int orc_one_hot(const void *idx, int is64, int64_t N, int64_t C, float *out)
{
    if (C <= 0)
        return ORC_ERR_INVALID_ARG;
    for (int64_t i = 0; i < N * C; ++i)
        out[i] = 0.0f;
    for (int64_t i = 0; i < N; ++i)
    {
        int64_t t = label_at(idx, is64, i);
        if (t >= 0 && t < C)
            out[i * C + t] = 1.0f;
    }
    return ORC_OK;
}

/* softmax_cross_entropy.cpp:54-73 */
int orc_softmax_ce_loss(const float *x, const void *t, int is64, int64_t N, int64_t C, float *loss)
{
    float *p = (float *)malloc(sizeof(float) * (size_t)(N * C > 0 ? N * C : 1));
    float *sel = (float *)malloc(sizeof(float) * (size_t)(N > 0 ? N : 1));
    orc_softmax(x, N, C, 1, p);
    int rc = orc_gather(p, t, is64, N, C, sel);
    if (rc == ORC_OK)
    {
        for (int64_t i = 0; i < N; ++i)
            sel[i] = logf(sel[i] + 1e-8f); /* 63-65 */
        float s = orc_sum_all(sel, N);     /* 67-69 */
        *loss = -s / (float)N;             /* 70 */
    }
    free(p);
    free(sel);
    return rc;
}

/* softmax_cross_entropy.cpp:92-106 */
int orc_softmax_ce_grad(const float *x, const void *t, int is64, int64_t N, int64_t C, float gy, float *gx)
{
    float *oh = (float *)malloc(sizeof(float) * (size_t)(N * C > 0 ? N * C : 1));
    orc_softmax(x, N, C, 1, gx);
    int rc = orc_one_hot(t, is64, N, C, oh);
    float scale = gy / (float)N;
    for (int64_t i = 0; i < N * C; ++i)
        gx[i] = (gx[i] - oh[i]) * scale;
    free(oh);
    return rc;
}

/* ============================================================================== pooling */

int orc_max_pool2d(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                   int PW, float *y, uint64_t *idx)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG; /* max_pool2d.cpp:71-77 */
    float *col = (float *)malloc(sizeof(float) * (size_t)(N * C * KH * KW * OH * OW));
    orc_im2col(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 0, col); /* 80: 6-D layout, zero padding */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t oh = 0; oh < OH; ++oh)
                for (int64_t ow = 0; ow < OW; ++ow)
                {
                    int64_t base = ((n * C + c) * KH * KW) * OH * OW + oh * OW + ow;
                    float mv = col[base]; /* 110-113: start from window element (0,0) */
                    uint64_t mi = 0;
                    for (int kh = 0; kh < KH; ++kh)
                        for (int kw = 0; kw < KW; ++kw)
                        {
                            float v = col[base + (int64_t)(kh * KW + kw) * OH * OW];
                            if (v > mv) /* 126: strict, so the first maximum wins */
                            {
                                mv = v;
                                mi = (uint64_t)(kh * KW + kw);
                            }
                        }
                    int64_t r = ((n * C + c) * OH + oh) * OW + ow;
                    y[r] = mv;
                    if (idx)
                        idx[r] = mi;
                }
    free(col);
    return ORC_OK;
}

int orc_max_pool2d_backward(const float *gy, const uint64_t *idx, int64_t N, int64_t C, int64_t H, int64_t W, int KH,
                            int KW, int SH, int SW, int PH, int PW, float *gx)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG;
    float *gcol = (float *)calloc((size_t)(N * C * KH * KW * OH * OW), sizeof(float)); /* 185-191 */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t oh = 0; oh < OH; ++oh)
                for (int64_t ow = 0; ow < OW; ++ow)
                {
                    int64_t r = ((n * C + c) * OH + oh) * OW + ow;
                    int kh = (int)idx[r] / KW, kw = (int)idx[r] % KW; /* 203-205 */
                    gcol[((((n * C + c) * KH + kh) * KW + kw) * OH + oh) * OW + ow] = gy[r];
                }
    int rc = orc_col2im(gcol, N, C, H, W, KH, KW, SH, SW, PH, PW, 0, gx); /* 220 */
    free(gcol);
    return rc;
}

/* ============================================================================== metrics */

void orc_argmax_rows(const float *y, int64_t N, int64_t C, int64_t *out)
{
    for (int64_t i = 0; i < N; ++i) /* metrics.cpp:42-53 */
    {
        int64_t mi = 0;
        float mv = y[i * C];
        for (int64_t j = 1; j < C; ++j)
            if (y[i * C + j] > mv)
            {
                mv = y[i * C + j];
                mi = j;
            }
        out[i] = mi;
    }
}

float orc_accuracy(const float *y, const int32_t *t, int64_t N, int64_t C)
{
    int64_t *am = (int64_t *)malloc(sizeof(int64_t) * (size_t)(N > 0 ? N : 1));
    orc_argmax_rows(y, N, C, am);
    int64_t correct = 0;
    for (int64_t i = 0; i < N; ++i) /* metrics.cpp:55-60 */
        if (t[i] >= 0 && t[i] < (int32_t)C && (int64_t)t[i] == am[i])
            ++correct;
    free(am);
    return (float)correct / (float)N; /* 64 */
}

/* ============================================================================ elementwise */

static float binop(int op, float a, float b)
{
    switch (op)
    {
        case 0: return a + b;
        case 1: return a - b;
        case 2: return a * b;
        case 3: return a / b;
        default: return (a > b) ? 1.0f : 0.0f; /* operation_templates.h:233-240: mask in the input dtype */
    }
}

/* add.cpp:56-93 and siblings: same shape, or exactly one single-element operand */
int orc_binary(int op, const float *a, int64_t na, const float *b, int64_t nb, float *out)
{
    if (na == nb)
        for (int64_t i = 0; i < na; ++i)
            out[i] = binop(op, a[i], b[i]);
    else if (nb == 1)
        for (int64_t i = 0; i < na; ++i)
            out[i] = binop(op, a[i], b[0]);
    else if (na == 1)
        for (int64_t i = 0; i < nb; ++i)
            out[i] = binop(op, a[0], b[i]);
    else
        return ORC_ERR_RUNTIME;
    return ORC_OK;
}

void orc_unary(int op, const float *a, int64_t n, float *out)
{
    for (int64_t i = 0; i < n; ++i)
    {
        float v = a[i];
        switch (op)
        {
            case 0: out[i] = v > 0.0f ? v : 0.0f; break; /* activation/relu.cpp */
            case 1: out[i] = expf(v); break;             /* math/exp.cpp */
            case 2: out[i] = logf(v); break;             /* math/log.cpp */
            case 3: out[i] = -v; break;                  /* math/negate.cpp */
            case 4: out[i] = v * v; break;               /* math/square.cpp */
            case 5: out[i] = sqrtf(v); break;            /* math/sqrt.cpp */
            case 6: out[i] = 1.0f / (1.0f + expf(-v)); break; /* device_common/operation_templates.h:168-175 */
            default: /* activation/silu.cpp:49-56 */
            {
                const float sg = 1.0f / (1.0f + expf(-v));
                out[i] = v * sg;
                break;
            }
        }
    }
}

/* math/pow.cpp:35-43: powf for a float32 exponent */
void orc_pow_scalar(const float *a, int64_t n, float e, float *out)
{
    for (int64_t i = 0; i < n; ++i)
        out[i] = powf(a[i], e);
}

/* ========================================================================== batch normalisation */

/* normalization/batch_norm.cpp:31-258. x[N][C][P] (P = H*W; P = 1 is the two-dimensional [N][C] form). Training:
 * per channel, a sequential float sum over (n, p) / count, then the sequential sum of squared differences from that
 * mean / count. Evaluation: mean and var are copies of the running statistics. x_norm may be NULL. */
int orc_batch_norm_forward(const float *x, const float *gamma, const float *beta, const float *running_mean,
                           const float *running_var, int training, float eps, int64_t N, int64_t C, int64_t P, float *y,
                           float *mean, float *var, float *x_norm)
{
    if (N < 0 || C <= 0 || P <= 0)
        return ORC_ERR_INVALID_ARG;
    const int64_t count = N * P;
    for (int64_t c = 0; c < C; ++c)
    {
        if (training)
        {
            float sum = 0.f;
            for (int64_t n = 0; n < N; ++n)
                for (int64_t p = 0; p < P; ++p)
                    sum += x[(n * C + c) * P + p];
            if (count > 0)
                mean[c] = sum / (float)count;
            float sq = 0.f;
            for (int64_t n = 0; n < N; ++n)
                for (int64_t p = 0; p < P; ++p)
                {
                    const float d = x[(n * C + c) * P + p] - mean[c];
                    sq += d * d;
                }
            if (count > 0)
                var[c] = sq / (float)count;
        }
        else
        {
            mean[c] = running_mean[c];
            var[c] = running_var[c];
        }
    }
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
        {
            const float sd = sqrtf(var[c] + eps);
            for (int64_t p = 0; p < P; ++p)
            {
                const int64_t i = (n * C + c) * P + p;
                const float xn = (x[i] - mean[c]) / sd;
                if (x_norm)
                    x_norm[i] = xn;
                const float t = gamma[c] * xn;
                y[i] = t + beta[c];
            }
        }
    return ORC_OK;
}

/* normalization/batch_norm.cpp:279-418 */
int orc_batch_norm_backward(const float *gy, const float *gamma, const float *saved_var, const float *saved_x_norm,
                            float eps, int64_t N, int64_t C, int64_t P, float *gx, float *dgamma, float *dbeta)
{
    if (N < 0 || C <= 0 || P <= 0)
        return ORC_ERR_INVALID_ARG;
    const int64_t count = N * P;
    for (int64_t c = 0; c < C; ++c)
    {
        float sum_gy = 0.f, sum_gy_xn = 0.f;
        for (int64_t n = 0; n < N; ++n)
            for (int64_t p = 0; p < P; ++p)
            {
                const int64_t i = (n * C + c) * P + p;
                sum_gy += gy[i];
                const float t = gy[i] * saved_x_norm[i];
                sum_gy_xn += t;
            }
        const float mean_gy = count > 0 ? sum_gy / (float)count : 0.f;
        const float mean_gy_xn = count > 0 ? sum_gy_xn / (float)count : 0.f;
        const float sd = sqrtf(saved_var[c] + eps);
        dgamma[c] = sum_gy_xn;
        dbeta[c] = sum_gy;
        const float scale = gamma[c] / sd;
        for (int64_t n = 0; n < N; ++n)
            for (int64_t p = 0; p < P; ++p)
            {
                const int64_t i = (n * C + c) * P + p;
                const float t = saved_x_norm[i] * mean_gy_xn;
                gx[i] = scale * ((gy[i] - mean_gy) - t);
            }
    }
    return ORC_OK;
}

/* ========================================================================== detector forward path */

/* nn/upsample.cpp:22-75: nearest neighbour, ih = oh / scale_h, iw = ow / scale_w */
int orc_upsample_nearest(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW, int scale_h,
                         int scale_w, float *y)
{
    if (scale_h <= 0 || scale_w <= 0 || (OH - 1) / scale_h >= H || (OW - 1) / scale_w >= W)
        return ORC_ERR_INVALID_ARG;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t oh = 0; oh < OH; ++oh)
                for (int64_t ow = 0; ow < OW; ++ow)
                    y[((n * C + c) * OH + oh) * OW + ow] = x[((n * C + c) * H + oh / scale_h) * W + ow / scale_w];
    return ORC_OK;
}

/* shape/cat.cpp:20-140: every input viewed as [M, C_i, N]; chunk m of input i lands at out[m][off_i .. off_i + C_i) */
int orc_cat(const float *const *inputs, const int64_t *axis_sizes, int count, int64_t outer, int64_t inner, float *out)
{
    int64_t total = 0, off = 0;
    if (count < 1)
        return ORC_ERR_RUNTIME;
    for (int i = 0; i < count; ++i)
        total += axis_sizes[i];
    for (int i = 0; i < count; ++i)
    {
        const int64_t chunk = axis_sizes[i] * inner;
        for (int64_t m = 0; m < outer; ++m)
            memcpy(out + m * total * inner + off * inner, inputs[i] + m * chunk, sizeof(float) * (size_t)chunk);
        off += axis_sizes[i];
    }
    return ORC_OK;
}

/* custom/yolo_detect.cpp:28-166. conv 1x1 (conv2d.cpp:404-512 through orc_conv2d), reshape [N,A,CI,H,W], permute to
 * [N,A,H,W,CI], sigmoid as -x, exp, 1 + ., 1 / ., then xy = (2s + grid) * stride, wh = pow(2s, 2) * anchor. */
int orc_yolo_detect_forward(const float *x, const float *conv_w, const float *conv_b, const float *grid, int64_t grid_elems,
                            const float *anchor_grid, int64_t anchor_elems, int64_t anchor_H, int64_t anchor_W, int64_t N,
                            int64_t C, int64_t H, int64_t W, float stride, int num_anchors, int num_classes, float *out)
{
    const int64_t CI = num_classes + 5, A = num_anchors, OC = A * CI, HW = H * W;
    float *conv = (float *)malloc(sizeof(float) * (size_t)(N * OC * HW > 0 ? N * OC * HW : 1));
    int rc = orc_conv2d(x, conv_w, conv_b, N, C, H, W, OC, 1, 1, 1, 1, 0, 0, conv);
    if (rc != ORC_OK)
    {
        free(conv);
        return rc;
    }
    for (int64_t b = 0; b < N; ++b)
        for (int64_t i = 0; i < A * HW; ++i)
        {
            const int64_t a = i / HW, sp = i % HW, h = sp / W, w = sp % W;
            float *o = out + (b * A * HW + i) * CI;
            for (int64_t c = 0; c < CI; ++c)
            {
                const float v = conv[((b * A + a) * CI + c) * HW + sp];
                const float e = expf(-v);
                const float d = 1.0f + e;
                o[c] = 1.0f / d;
            }
            {
                const int64_t gb = a * HW * 2 + h * W * 2 + w * 2;
                const float gx = gb < grid_elems ? grid[gb] : 0.0f, gy = gb + 1 < grid_elems ? grid[gb + 1] : 0.0f;
                const int64_t sh = (anchor_H > 0 && H > anchor_H) ? H / anchor_H : 1;
                const int64_t sw = (anchor_W > 0 && W > anchor_W) ? W / anchor_W : 1;
                int64_t ah = h / sh, aw = w / sw;
                if (ah > anchor_H - 1) ah = anchor_H - 1;
                if (aw > anchor_W - 1) aw = anchor_W - 1;
                const int64_t ab = a * anchor_H * anchor_W * 2 + ah * anchor_W * 2 + aw * 2;
                const float anw = ab < anchor_elems ? anchor_grid[ab] : 1.0f;
                const float anh = ab + 1 < anchor_elems ? anchor_grid[ab + 1] : 1.0f;
                const float s0 = o[0], s1 = o[1], s2 = o[2], s3 = o[3];
                float t;
                t = s0 * 2.0f; t = t + gx; o[0] = t * stride;
                t = s1 * 2.0f; t = t + gy; o[1] = t * stride;
                o[2] = powf(s2 * 2.0f, 2.0f) * anw;
                o[3] = powf(s3 * 2.0f, 2.0f) * anh;
            }
        }
    free(conv);
    return ORC_OK;
}

/* ========================================================================== training steps */

static float *fmalloc(int64_t n)
{
    return (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
}

/* nn/layers/linear.cpp:90-104: mat_mul, broadcast_to(bias[1,out] -> [N,out]), add */
static void linear_forward(const float *x, const float *W, const float *b, int64_t N, int64_t in, int64_t out, float *y)
{
    orc_matmul(x, W, y, N, out, in);
    for (int64_t i = 0; i < N; ++i)
        for (int64_t j = 0; j < out; ++j)
            y[i * out + j] = y[i * out + j] + b[j];
}

/* Add::backward passes gy to both inputs (operators/math/add.cpp:29-55); BroadcastTo::backward =
 * sum_to(gy, [1,out]) (operators/math/broadcast_to.cpp:29-46); MatMul::backward (mat_mul.cpp:171-177). */
static void linear_backward(const float *x, const float *W, const float *gy, int64_t N, int64_t in, int64_t out,
                            float *gx, float *gW, float *gb)
{
    int64_t ss[2] = {N, out}, ts[2] = {1, out};
    orc_sum_to(gy, ss, 2, ts, 2, gb);
    orc_matmul_backward(x, W, gy, gx, gW, N, in, out);
}

/* hooks.h:40-65 then adam.cpp:19-114, every step rounded to float as the reference's Mat ops do */
static void adam_update(float *p, const float *g_in, float *m, float *v, int64_t n, int t, float lr, float b1, float b2,
                        float eps, float wd)
{
    float one_m_b1 = 1.0f - b1, one_m_b2 = 1.0f - b2;
    float b1p = powf(b1, (float)t), b2p = powf(b2, (float)t);
    float mhs = 1.0f / (1.0f - b1p), vhs = 1.0f / (1.0f - b2p);
    for (int64_t i = 0; i < n; ++i)
    {
        float g = g_in[i];
        if (wd != 0.0f)
        {
            float term = p[i] * wd; /* hooks.h:52 */
            g = g + term;           /* accumulate_grad -> add_inplace */
        }
        float mm = m[i] * b1;
        float gg = g * one_m_b1;
        m[i] = mm + gg; /* adam.cpp:55 */
        float g2 = g * g;
        float vv = v[i] * b2;
        float g2s = g2 * one_m_b2;
        v[i] = vv + g2s; /* adam.cpp:60-61 */
        float mh = m[i] * mhs;
        float vh = v[i] * vhs;
        float sq = powf(vh, 0.5f); /* adam.cpp:95 */
        float den = sq + eps;
        float upd = mh / den;
        float step = upd * lr;
        p[i] = p[i] - step; /* adam.cpp:110 */
    }
}

int orc_mlp_train_step(const float *x, const void *t, int is64, int64_t N, int64_t D, int64_t Hd, int64_t C, float *W1,
                       float *b1, float *W2, float *b2, float *mW1, float *vW1, float *mb1, float *vb1, float *mW2,
                       float *vW2, float *mb2, float *vb2, int step_t, float lr, float beta1, float beta2, float eps,
                       float wd, float *loss, float *gW1, float *gb1, float *gW2, float *gb2, float *logits)
{
    float *a1 = fmalloc(N * Hd), *mask = fmalloc(N * Hd), *r1 = fmalloc(N * Hd), *a2 = fmalloc(N * C);
    float *g2 = fmalloc(N * C), *gr1 = fmalloc(N * Hd), *ga1 = fmalloc(N * Hd), *gx = fmalloc(N * D);
    float zero = 0.0f;
    int rc;
    /* nn/models/mlp.cpp:43-61 */
    linear_forward(x, W1, b1, N, D, Hd, a1);
    orc_binary(4, a1, N * Hd, &zero, 1, mask); /* activation/relu.cpp:23-29 */
    orc_unary(0, a1, N * Hd, r1);
    linear_forward(r1, W2, b2, N, Hd, C, a2);
    if (logits)
        memcpy(logits, a2, sizeof(float) * (size_t)(N * C));
    rc = orc_softmax_ce_loss(a2, t, is64, N, C, loss);
    if (rc == ORC_OK)
    {
        /* core/tensor_impl.cpp:94-99 seeds the loss gradient with ones */
        orc_softmax_ce_grad(a2, t, is64, N, C, 1.0f, g2);
        linear_backward(r1, W2, g2, N, Hd, C, gr1, gW2, gb2);
        orc_binary(2, gr1, N * Hd, mask, N * Hd, ga1); /* relu.cpp:37-54 */
        linear_backward(x, W1, ga1, N, D, Hd, gx, gW1, gb1);
        /* optim/optimizer.cpp:19-53: hooks over all params, then step_one per param */
        adam_update(W1, gW1, mW1, vW1, D * Hd, step_t, lr, beta1, beta2, eps, wd);
        adam_update(b1, gb1, mb1, vb1, Hd, step_t, lr, beta1, beta2, eps, wd);
        adam_update(W2, gW2, mW2, vW2, Hd * C, step_t, lr, beta1, beta2, eps, wd);
        adam_update(b2, gb2, mb2, vb2, C, step_t, lr, beta1, beta2, eps, wd);
    }
    free(a1); free(mask); free(r1); free(a2); free(g2); free(gr1); free(ga1); free(gx);
    return rc;
}

/* sgd.cpp:18-75 with momentum == 0 and weight_decay == 0: param = param - grad * lr */
static void sgd_update(float *p, const float *g, int64_t n, float lr)
{
    for (int64_t i = 0; i < n; ++i)
    {
        float step = g[i] * lr;
        p[i] = p[i] - step;
    }
}

int orc_cnn_train_step(const float *x, const void *t, int is64, int64_t N, int64_t S, int64_t C1, int64_t C2,
                       int64_t Hd, int64_t Cc, float *Wc1, float *bc1, float *Wc2, float *bc2, float *Wl1, float *bl1,
                       float *Wl2, float *bl2, float lr, float *loss, uint64_t *idx1, uint64_t *idx2, float *gWc1,
                       float *gbc1, float *gWc2, float *gbc2, float *gWl1, float *gbl1, float *gWl2, float *gbl2,
                       float *logits)
{
    int64_t S2 = S / 2, S4 = S2 / 2, F = C2 * S4 * S4;
    float zero = 0.0f;
    float *y1 = fmalloc(N * C1 * S * S), *m1 = fmalloc(N * C1 * S * S), *r1 = fmalloc(N * C1 * S * S);
    float *p1 = fmalloc(N * C1 * S2 * S2);
    float *y2 = fmalloc(N * C2 * S2 * S2), *m2 = fmalloc(N * C2 * S2 * S2), *r2 = fmalloc(N * C2 * S2 * S2);
    float *p2 = fmalloc(N * F);
    float *a3 = fmalloc(N * Hd), *m3 = fmalloc(N * Hd), *r3 = fmalloc(N * Hd), *a4 = fmalloc(N * Cc);
    float *g4 = fmalloc(N * Cc), *gr3 = fmalloc(N * Hd), *ga3 = fmalloc(N * Hd), *gp2 = fmalloc(N * F);
    float *gr2 = fmalloc(N * C2 * S2 * S2), *gy2 = fmalloc(N * C2 * S2 * S2), *gp1 = fmalloc(N * C1 * S2 * S2);
    float *gr1 = fmalloc(N * C1 * S * S), *gy1 = fmalloc(N * C1 * S * S), *gx = fmalloc(N * S * S);
    int rc;

    orc_conv2d(x, Wc1, bc1, N, 1, S, S, C1, 3, 3, 1, 1, 1, 1, y1);
    orc_binary(4, y1, N * C1 * S * S, &zero, 1, m1);
    orc_unary(0, y1, N * C1 * S * S, r1);
    orc_max_pool2d(r1, N, C1, S, S, 2, 2, 2, 2, 0, 0, p1, idx1);
    orc_conv2d(p1, Wc2, bc2, N, C1, S2, S2, C2, 3, 3, 1, 1, 1, 1, y2);
    orc_binary(4, y2, N * C2 * S2 * S2, &zero, 1, m2);
    orc_unary(0, y2, N * C2 * S2 * S2, r2);
    orc_max_pool2d(r2, N, C2, S2, S2, 2, 2, 2, 2, 0, 0, p2, idx2);
    /* flatten = zero-copy reshape [N, C2*S4*S4] (operators/shape/flatten.cpp) */
    linear_forward(p2, Wl1, bl1, N, F, Hd, a3);
    orc_binary(4, a3, N * Hd, &zero, 1, m3);
    orc_unary(0, a3, N * Hd, r3);
    linear_forward(r3, Wl2, bl2, N, Hd, Cc, a4);
    if (logits)
        memcpy(logits, a4, sizeof(float) * (size_t)(N * Cc));
    rc = orc_softmax_ce_loss(a4, t, is64, N, Cc, loss);
    if (rc == ORC_OK)
    {
        orc_softmax_ce_grad(a4, t, is64, N, Cc, 1.0f, g4);
        linear_backward(r3, Wl2, g4, N, Hd, Cc, gr3, gWl2, gbl2);
        orc_binary(2, gr3, N * Hd, m3, N * Hd, ga3);
        linear_backward(p2, Wl1, ga3, N, F, Hd, gp2, gWl1, gbl1);
        orc_max_pool2d_backward(gp2, idx2, N, C2, S2, S2, 2, 2, 2, 2, 0, 0, gr2);
        orc_binary(2, gr2, N * C2 * S2 * S2, m2, N * C2 * S2 * S2, gy2);
        orc_conv2d_backward(gy2, p1, Wc2, N, C1, S2, S2, C2, 3, 3, 1, 1, 1, 1, gp1, gWc2, gbc2);
        orc_max_pool2d_backward(gp1, idx1, N, C1, S, S, 2, 2, 2, 2, 0, 0, gr1);
        orc_binary(2, gr1, N * C1 * S * S, m1, N * C1 * S * S, gy1);
        orc_conv2d_backward(gy1, x, Wc1, N, 1, S, S, C1, 3, 3, 1, 1, 1, 1, gx, gWc1, gbc1);
        sgd_update(Wc1, gWc1, C1 * 9, lr);
        sgd_update(bc1, gbc1, C1, lr);
        sgd_update(Wc2, gWc2, C2 * C1 * 9, lr);
        sgd_update(bc2, gbc2, C2, lr);
        sgd_update(Wl1, gWl1, F * Hd, lr);
        sgd_update(bl1, gbl1, Hd, lr);
        sgd_update(Wl2, gWl2, Hd * Cc, lr);
        sgd_update(bl2, gbl2, Cc, lr);
    }
    free(y1); free(m1); free(r1); free(p1); free(y2); free(m2); free(r2); free(p2);
    free(a3); free(m3); free(r3); free(a4); free(g4); free(gr3); free(ga3); free(gp2);
    free(gr2); free(gy2); free(gp1); free(gr1); free(gy1); free(gx);
    return rc;
}

/* ============================================================== convolution on float64 tensors */
/* The reference's device convolution dispatches over the element type (src/mat/origin/cuda/conv/conv2d.cu:412-664) and
 * runs the algorithm of conv2d.cpp:404-599 in that type: the functions above over doubles, loop for loop. The compiled
 * reference cannot pin these — its CPU im2col copies a float buffer into the double result (conv2d.cpp:87, 159), so a
 * double convolution on the CPU returns garbage. They are pinned by the reference tests' known answers with integer
 * data, by bit-equality with the float functions above on data both types hold exactly, and by numpy restatements of
 * the mathematics (tests/test_oracle.py). */
static double *pad_image_f64(const double *img, int64_t N, int64_t C, int64_t H, int64_t W, int PH, int PW)
{
    int64_t pH = H + 2 * PH, pW = W + 2 * PW;
    double *p = (double *)calloc((size_t)(N * C * pH * pW), sizeof(double));
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t h = 0; h < H; ++h)
                for (int64_t w = 0; w < W; ++w)
                    p[((n * C + c) * pH + h + PH) * pW + w + PW] = img[((n * C + c) * H + h) * W + w];
    return p;
}

int orc_im2col_f64(const double *img, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
               int PW, int to_matrix, double *col)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG; /* conv2d.cpp:69-75 */
    int64_t pH = H + 2 * PH, pW = W + 2 * PW;
    double *p = pad_image_f64(img, N, C, H, W, PH, PW);
    memset(col, 0, sizeof(double) * (size_t)(N * C * KH * KW * OH * OW));
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int kh = 0; kh < KH; ++kh)
                for (int kw = 0; kw < KW; ++kw)
                    for (int64_t oh = 0; oh < OH; ++oh)
                        for (int64_t ow = 0; ow < OW; ++ow)
                        {
                            int64_t hi = kh + SH * oh, wi = kw + SW * ow;
                            if (hi < pH && wi < pW) /* conv2d.cpp:146, 186 */
                            {
                                double v = p[((n * C + c) * pH + hi) * pW + wi];
                                if (to_matrix) /* conv2d.cpp:116-162 */
                                    col[((n * OH + oh) * OW + ow) * (C * KH * KW) + (c * KH + kh) * KW + kw] = v;
                                else /* conv2d.cpp:164-206 */
                                    col[((((n * C + c) * KH + kh) * KW + kw) * OH + oh) * OW + ow] = v;
                            }
                        }
    free(p);
    return ORC_OK;
}

int orc_col2im_f64(const double *col, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
               int PW, int to_matrix, double *img)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG;
    int64_t pH = H + 2 * PH, pW = W + 2 * PW;
    double *p = (double *)calloc((size_t)(N * C * pH * pW), sizeof(double));
    /* conv2d.cpp:320-349 — accumulation order n, c, kh, kw, oh, ow ascending */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int kh = 0; kh < KH; ++kh)
                for (int kw = 0; kw < KW; ++kw)
                    for (int64_t oh = 0; oh < OH; ++oh)
                        for (int64_t ow = 0; ow < OW; ++ow)
                        {
                            int64_t hi = kh + SH * oh, wi = kw + SW * ow;
                            if (hi < pH && wi < pW)
                            {
                                double v = to_matrix
                                              ? col[((n * OH + oh) * OW + ow) * (C * KH * KW) + (c * KH + kh) * KW + kw]
                                              : col[((((n * C + c) * KH + kh) * KW + kw) * OH + oh) * OW + ow];
                                p[((n * C + c) * pH + hi) * pW + wi] += v;
                            }
                        }
    /* conv2d.cpp:352-369 — strip the padding */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c)
            for (int64_t h = 0; h < H; ++h)
                for (int64_t w = 0; w < W; ++w)
                    img[((n * C + c) * H + h) * W + w] = p[((n * C + c) * pH + h + PH) * pW + w + PW];
    free(p);
    return ORC_OK;
}

void orc_transpose_f64(const double *src, double *dst, int64_t outer, int64_t rows, int64_t cols)
{
    for (int64_t o = 0; o < outer; ++o)
    {
        for (int64_t i = 0; i < rows; ++i)
        {
            for (int64_t j = 0; j < cols; ++j)
            {
                dst[o * rows * cols + j * rows + i] = src[o * rows * cols + i * cols + j];
            }
        }
    }
}

void orc_sum_axis_f64(const double *src, int64_t outer, int64_t axis, int64_t inner, double *dst)
{
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t i = 0; i < inner; ++i)
        {
            double s = 0.0f;
            for (int64_t a = 0; a < axis; ++a)
                s += src[(o * axis + a) * inner + i];
            dst[o * inner + i] = s;
        }
}

int orc_conv2d_f64(const double *x, const double *w, const double *b, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
               int KH, int KW, int SH, int SW, int PH, int PW, double *y)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG; /* conv2d.cpp:438-444 */
    int64_t M = N * OH * OW, K = C * KH * KW;
    double *col = (double *)malloc(sizeof(double) * (size_t)(M * K));
    double *wT = (double *)malloc(sizeof(double) * (size_t)(K * OC));
    double *yf = (double *)malloc(sizeof(double) * (size_t)(M * OC));
    orc_im2col_f64(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, col); /* conv2d.cpp:460 */
    orc_transpose_f64(w, wT, 1, OC, K);                             /* 463-464: W[OC,K] -> W_T[K,OC] */
    orc_matmul_f64(col, wT, yf, M, OC, K);                          /* 469 */
    if (b) /* 472-479: bias broadcast to [M,OC] then one double add per element */
        for (int64_t i = 0; i < M; ++i)
            for (int64_t oc = 0; oc < OC; ++oc)
                yf[i * OC + oc] = yf[i * OC + oc] + b[oc];
    /* 489-509: NHWC -> NCHW */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t oc = 0; oc < OC; ++oc)
            for (int64_t oh = 0; oh < OH; ++oh)
                for (int64_t ow = 0; ow < OW; ++ow)
                    y[((n * OC + oc) * OH + oh) * OW + ow] = yf[((n * OH + oh) * OW + ow) * OC + oc];
    free(col);
    free(wT);
    free(yf);
    return ORC_OK;
}

int orc_conv2d_backward_f64(const double *gy, const double *x, const double *w, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, double *gx, double *gw, double *gb)
{
    int64_t OH = orc_conv_outsize(H, KH, SH, PH), OW = orc_conv_outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return ORC_ERR_INVALID_ARG;
    int64_t M = N * OH * OW, K = C * KH * KW;
    /* conv2d.cpp:548 — gy's NCHW buffer is *viewed* as a row-major [M, OC] matrix, no permutation. */
    const double *gy2d = gy;
    double *gyT = (double *)malloc(sizeof(double) * (size_t)(M * OC));
    double *col = (double *)malloc(sizeof(double) * (size_t)(M * K));
    orc_transpose_f64(gy2d, gyT, 1, M, OC);                         /* 550: [M,OC] -> [OC,M] */
    orc_im2col_f64(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, col); /* 554 */
    orc_matmul_f64(gyT, col, gw, OC, K, M);                         /* 559: gW[OC,K] */
    if (gb)
    {
        /* 571-575: gy.sum(2) -> [N,OC,OW]; .sum(2) -> [N,OC]; .sum(0) -> [OC], on the true NCHW gy */
        double *s1 = (double *)malloc(sizeof(double) * (size_t)(N * OC * OW));
        double *s2 = (double *)malloc(sizeof(double) * (size_t)(N * OC));
        orc_sum_axis_f64(gy, N * OC, OH, OW, s1);
        orc_sum_axis_f64(s1, N * OC, OW, 1, s2);
        orc_sum_axis_f64(s2, 1, N, OC, gb);
        free(s1);
        free(s2);
    }
    /* 584-596: gx_col[M,K] = gy2d[M,OC] . W2d[OC,K]; gx = col2im(gx_col) */
    orc_matmul_f64(gy2d, w, col, M, K, OC);
    orc_col2im_f64(col, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, gx);
    free(gyT);
    free(col);
    return ORC_OK;
}
