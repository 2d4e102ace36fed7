// Convolution on float64 tensors. The reference's device convolution dispatches over the element type
// (src/mat/origin/cuda/conv/conv2d.cu:412-664) and is the CPU algorithm in that type
// (src/mat/origin/cpu/conv/conv2d.cpp:404-599): forward = im2col, one product with the filters, bias, NCHW; backward =
// gW from gy's NCHW buffer read as a row-major [N*OH*OW, OC] matrix exactly as it lies (conv2d.cpp:548) times the col
// matrix, gx as that matrix times the filters scattered back by col2im, gb the per-channel sum of gy.
//
// This is the same sequence, with the products on the FP64 matrix cores (odl_hip_dgemm) and plain one-thread-per-element
// kernels around them — float64 is not what the benchmarked path computes in, so none of the float32 kernels' tiling
// is repeated here. The forward runs one product per image, W[OC,K] . col_n[P,K]^T, whose output is the image's NCHW
// block already. The filter gradient has an output of OC x K elements and a reduction as long as the batch has pixels:
// the reduction is cut into runs of rows, one product each (a batch of products for the matrix cores), and the partial
// gradients are added in run order.
#include "odl_common.h"

#include <algorithm>

extern "C" int odl_hip_dgemm(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const double *A, int64_t lda,
                             const double *B, int64_t ldb, double *C, int64_t ldc, int64_t batch, int64_t stride_a,
                             int64_t stride_b, int64_t stride_c, void *stream);
extern "C" int odl_hip_sum_axis_dtype(int dtype, const void *src, int64_t outer, int64_t axis, int64_t inner, int through_float,
                                      void *dst, void *workspace, size_t workspace_bytes, void *stream);
extern "C" size_t odl_hip_sum_axis_dtype_workspace_bytes(int dtype, int64_t outer, int64_t axis, int64_t inner);

namespace
{
constexpr int kBlock = 256;
constexpr int kF64 = 1;  // the reference's DataType::kFloat64

struct Geom
{
    int64_t N, C, H, W, OH, OW;
    int KH, KW, SH, SW, PH, PW;
};

inline int64_t outsize(int64_t in, int k, int s, int p)
{
    return (in + 2 * (int64_t)p - k) / s + 1;  // include/origin/utils/conv_utils.h
}

inline size_t align256(size_t b)
{
    return (b + 255) & ~(size_t)255;
}

// MATRIX: col[(n,oh,ow)][(c,kh,kw)]; else col[n][c][kh][kw][oh][ow] (src/mat/origin/cpu/conv/conv2d.cpp:39-200). One
// thread per col element; outside the image the element is zero.
template <bool MATRIX>
__global__ __launch_bounds__(kBlock) void im2col_f64_kernel(const double *__restrict__ img, double *__restrict__ col, Geom g)
{
    const int64_t total = g.N * g.C * g.KH * g.KW * g.OH * g.OW;
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= total)
        return;
    int64_t r = t, n, c, oh, ow;
    int kh, kw;
    if (MATRIX)
    {
        kw = (int)(r % g.KW), r /= g.KW;
        kh = (int)(r % g.KH), r /= g.KH;
        c = r % g.C, r /= g.C;
        ow = r % g.OW, r /= g.OW;
        oh = r % g.OH, n = r / g.OH;
    }
    else
    {
        ow = r % g.OW, r /= g.OW;
        oh = r % g.OH, r /= g.OH;
        kw = (int)(r % g.KW), r /= g.KW;
        kh = (int)(r % g.KH), r /= g.KH;
        c = r % g.C, n = r / g.C;
    }
    const int64_t h = oh * g.SH + kh - g.PH, w = ow * g.SW + kw - g.PW;
    col[t] = (h >= 0 && h < g.H && w >= 0 && w < g.W) ? img[((n * g.C + c) * g.H + h) * g.W + w] : 0.0;
}

// One thread per image pixel; its taps are added in ascending (kh, kw) starting from +0.0, the order in which the
// reference's scatter loop reaches the pixel (conv2d.cpp:316-349): no atomics, the same sum on every run.
template <bool MATRIX>
__global__ __launch_bounds__(kBlock) void col2im_f64_kernel(const double *__restrict__ col, double *__restrict__ img, Geom g)
{
    const int64_t total = g.N * g.C * g.H * g.W;
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= total)
        return;
    const int64_t w = t % g.W, h = (t / g.W) % g.H;
    const int64_t nc = t / (g.W * g.H), n = nc / g.C, c = nc - n * g.C;
    const int64_t K = g.C * g.KH * g.KW;
    double acc = 0.0;
    for (int kh = 0; kh < g.KH; ++kh)
    {
        const int64_t hp = h + g.PH - kh;
        if (hp < 0 || hp % g.SH != 0 || hp / g.SH >= g.OH)
            continue;
        const int64_t oh = hp / g.SH;
        for (int kw = 0; kw < g.KW; ++kw)
        {
            const int64_t wp = w + g.PW - kw;
            if (wp < 0 || wp % g.SW != 0 || wp / g.SW >= g.OW)
                continue;
            const int64_t ow = wp / g.SW;
            acc += MATRIX ? col[((n * g.OH + oh) * g.OW + ow) * K + (c * g.KH + kh) * g.KW + kw]
                          : col[(((nc * g.KH + kh) * g.KW + kw) * g.OH + oh) * g.OW + ow];
        }
    }
    img[t] = acc;
}

// y[n][oc][p] += b[oc]
__global__ __launch_bounds__(kBlock) void bias_rows_f64_kernel(double *__restrict__ y, const double *__restrict__ b, int64_t OC,
                                                               int64_t P, int64_t total)
{
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t < total)
        y[t] = y[t] + b[(t / P) % OC];
}

int make_geom(Geom &g, const char *who, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH, int PW)
{
    ODL_REQUIRE(N >= 0 && C > 0 && H > 0 && W > 0, "%s: bad image extents", who);
    ODL_REQUIRE(KH > 0 && KW > 0 && SH > 0 && SW > 0 && PH >= 0 && PW >= 0, "%s: bad window, stride or padding", who);
    g = Geom{N, C, H, W, outsize(H, KH, SH, PH), outsize(W, KW, SW, PW), KH, KW, SH, SW, PH, PW};
    ODL_REQUIRE(g.OH > 0 && g.OW > 0, "%s: the window does not fit the padded image", who);
    ODL_REQUIRE(N * C * KH * KW * g.OH * g.OW < (1ll << 40) && N * C * H * W < (1ll << 40), "%s: extents too large", who);
    return ODL_OK;
}

inline dim3 blocks_for(int64_t total)
{
    return dim3((unsigned)odl::ceil_div(total, kBlock));
}

// the reduction of the filter gradient is cut into this many runs of col rows
struct RunPlan
{
    int64_t runs, rows;  // `runs` runs of `rows` rows; the last may be shorter
};

RunPlan plan_runs(int64_t M)
{
    int64_t runs = std::min<int64_t>(64, std::max<int64_t>(1, M / 2048));
    const int64_t rows = odl::ceil_div(M, runs);
    runs = odl::ceil_div(M, rows);
    return RunPlan{runs, rows};
}

struct BwdLayout
{
    size_t col, part, tmp, red;
    size_t total() const { return col + part + tmp + red; }
};

BwdLayout backward_layout(int64_t N, int64_t OC, int64_t M, int64_t K, int64_t P)
{
    BwdLayout l{};
    const RunPlan r = plan_runs(M);
    l.col = align256((size_t)(M * K) * sizeof(double));
    l.part = r.runs > 1 ? align256((size_t)(r.runs * OC * K) * sizeof(double)) : 0;
    l.tmp = align256((size_t)(N * OC) * sizeof(double));
    l.red = align256(std::max({odl_hip_sum_axis_dtype_workspace_bytes(kF64, 1, r.runs, OC * K),
                               odl_hip_sum_axis_dtype_workspace_bytes(kF64, N * OC, P, 1),
                               odl_hip_sum_axis_dtype_workspace_bytes(kF64, 1, N, OC)}));
    return l;
}
}  // namespace

extern "C" {

int odl_hip_im2col_f64(const double *img, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                       int PW, int to_matrix, double *col, void *stream)
{
    ODL_REQUIRE_DEVICE();
    Geom g;
    const int rc = make_geom(g, "im2col", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    const int64_t total = N * C * KH * KW * g.OH * g.OW;
    if (total == 0)
        return ODL_OK;
    ODL_REQUIRE(img && col, "im2col: null operand");
    if (to_matrix)
        hipLaunchKernelGGL(im2col_f64_kernel<true>, blocks_for(total), dim3(kBlock), 0, odl::as_stream(stream), img, col, g);
    else
        hipLaunchKernelGGL(im2col_f64_kernel<false>, blocks_for(total), dim3(kBlock), 0, odl::as_stream(stream), img, col, g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_col2im_f64(const double *col, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                       int PW, int to_matrix, double *img, void *stream)
{
    ODL_REQUIRE_DEVICE();
    Geom g;
    const int rc = make_geom(g, "col2im", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    const int64_t total = N * C * H * W;
    if (total == 0)
        return ODL_OK;
    ODL_REQUIRE(img && col, "col2im: null operand");
    if (to_matrix)
        hipLaunchKernelGGL(col2im_f64_kernel<true>, blocks_for(total), dim3(kBlock), 0, odl::as_stream(stream), col, img, g);
    else
        hipLaunchKernelGGL(col2im_f64_kernel<false>, blocks_for(total), dim3(kBlock), 0, odl::as_stream(stream), col, img, g);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

size_t odl_hip_conv2d_f64_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                                          int SW, int PH, int PW)
{
    (void)OC;
    if (N < 0 || C <= 0 || KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0)
        return 0;
    const int64_t OH = outsize(H, KH, SH, PH), OW = outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return 0;
    return align256((size_t)(N * OH * OW * C * KH * KW) * sizeof(double));
}

int odl_hip_conv2d_f64(const double *x, const double *w, const double *b, int64_t N, int64_t C, int64_t H, int64_t W,
                       int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, double *y, void *workspace,
                       size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    Geom g;
    int rc = make_geom(g, "conv2d", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(OC > 0, "conv2d: OC must be positive");
    const int64_t P = g.OH * g.OW, K = C * KH * KW;
    if (N == 0)
        return ODL_OK;
    ODL_REQUIRE(x && w && y, "conv2d: null operand");
    const size_t need = align256((size_t)(N * P * K) * sizeof(double));
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need, "conv2d: needs a workspace of %zu bytes, got %zu", need,
                workspace_bytes);
    double *col = static_cast<double *>(workspace);
    rc = odl_hip_im2col_f64(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, col, stream);
    if (rc != ODL_OK)
        return rc;
    // y[n] [OC, P] = W [OC, K] . col_n [P, K]^T for every image n: the product's output is the image's NCHW block
    for (int64_t n0 = 0; n0 < N; n0 += 32768)  // (a batch of products is a grid dimension)
    {
        rc = odl_hip_dgemm(0, 1, OC, P, K, w, K, col + n0 * P * K, K, y + n0 * OC * P, P, std::min<int64_t>(N - n0, 32768), 0,
                           P * K, OC * P, stream);
        if (rc != ODL_OK)
            return rc;
    }
    if (b)
    {
        const int64_t total = N * OC * P;
        hipLaunchKernelGGL(bias_rows_f64_kernel, blocks_for(total), dim3(kBlock), 0, odl::as_stream(stream), y, b, OC, P, total);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}

size_t odl_hip_conv2d_backward_f64_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                                                   int SH, int SW, int PH, int PW)
{
    if (N <= 0 || C <= 0 || OC <= 0 || KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0)
        return 0;
    const int64_t OH = outsize(H, KH, SH, PH), OW = outsize(W, KW, SW, PW);
    if (OH <= 0 || OW <= 0)
        return 0;
    return backward_layout(N, OC, N * OH * OW, C * KH * KW, OH * OW).total();
}

int odl_hip_conv2d_backward_f64(const double *gy, const double *x, const double *w, int64_t N, int64_t C, int64_t H, int64_t W,
                                int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, double *gx, double *gw, double *gb,
                                void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    Geom g;
    int rc = make_geom(g, "conv2d_backward", N, C, H, W, KH, KW, SH, SW, PH, PW);
    if (rc != ODL_OK)
        return rc;
    ODL_REQUIRE(OC > 0, "conv2d_backward: OC must be positive");
    const int64_t P = g.OH * g.OW, M = N * P, K = C * KH * KW;
    if (M == 0)
        return ODL_OK;
    ODL_REQUIRE(gy && x && w, "conv2d_backward: null operand");
    const BwdLayout l = backward_layout(N, OC, M, K, P);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= l.total(), "conv2d_backward: needs a workspace of %zu bytes, got %zu",
                l.total(), workspace_bytes);
    char *ws = static_cast<char *>(workspace);
    double *col = reinterpret_cast<double *>(ws);
    double *part = reinterpret_cast<double *>(ws + l.col);
    double *tmp = reinterpret_cast<double *>(ws + l.col + l.part);
    void *red = ws + l.col + l.part + l.tmp;

    if (gw)
    {
        rc = odl_hip_im2col_f64(x, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, col, stream);
        if (rc != ODL_OK)
            return rc;
        // gW [OC, K] = gy2d [M, OC]^T . col [M, K], gy2d = gy's buffer read as [M, OC]; runs of rows, added in run order
        const RunPlan r = plan_runs(M);
        if (r.runs == 1)
            rc = odl_hip_dgemm(1, 0, OC, K, M, gy, OC, col, K, gw, K, 1, 0, 0, 0, stream);
        else
        {
            const int64_t full = M / r.rows, rest = M - full * r.rows;
            rc = odl_hip_dgemm(1, 0, OC, K, r.rows, gy, OC, col, K, part, K, full, r.rows * OC, r.rows * K, OC * K, stream);
            if (rc == ODL_OK && rest > 0)
                rc = odl_hip_dgemm(1, 0, OC, K, rest, gy + full * r.rows * OC, OC, col + full * r.rows * K, K,
                                   part + full * OC * K, K, 1, 0, 0, 0, stream);
            if (rc == ODL_OK)
                rc = odl_hip_sum_axis_dtype(kF64, part, 1, r.runs, OC * K, 0, gw, red, l.red, stream);
        }
        if (rc != ODL_OK)
            return rc;
    }
    if (gb)
    {
        // gb[oc] = sum over n and the plane of gy[n][oc][:] (conv2d.cpp:566-580): the planes first, then the images
        rc = odl_hip_sum_axis_dtype(kF64, gy, N * OC, P, 1, 0, tmp, red, l.red, stream);
        if (rc == ODL_OK)
            rc = odl_hip_sum_axis_dtype(kF64, tmp, 1, N, OC, 0, gb, red, l.red, stream);
        if (rc != ODL_OK)
            return rc;
    }
    if (gx)
    {
        // gx_col [M, K] = gy2d [M, OC] . W2d [OC, K], then the gather back to the image
        rc = odl_hip_dgemm(0, 0, M, K, OC, gy, OC, w, K, col, K, 1, 0, 0, 0, stream);
        if (rc == ODL_OK)
            rc = odl_hip_col2im_f64(col, N, C, H, W, KH, KW, SH, SW, PH, PW, 1, gx, stream);
        if (rc != ODL_OK)
            return rc;
    }
    return ODL_OK;
}

}  // extern "C"
