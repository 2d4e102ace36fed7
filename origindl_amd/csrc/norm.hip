// Batch normalisation over [N, C, P] (P = H*W, or 1 for the two-dimensional [N, C] form): Mat::batch_norm_forward /
// batch_norm / batch_norm_backward (src/mat/origin/cpu/normalization/batch_norm.cpp:31-258, 279-418).
// Bandwidth-bound streams. A channel's N*P elements are treated as one flat range cut into equal chunks, one
// workgroup per (chunk, channel); partial sums go through a small workspace and are added in a fixed order, so the
// results do not depend on scheduling. Forward in training mode is three passes over x (sum -> mean, squared
// differences from that mean -> biased variance, normalise), exactly the two-pass statistics of the reference;
// backward is two passes (the two channel sums, then the input gradient). The per-element arithmetic follows the
// reference expression by expression: x_norm = (x - mean) / sqrt(var + eps), y = gamma * x_norm + beta,
// gx = (gamma / std) * (gy - mean_gy - x_norm * mean_gy_xnorm).
#include "odl_common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace
{
constexpr int kBlock = 256;

struct BnGeom
{
    unsigned C, P;
    unsigned total;  // N * P, elements of one channel
    unsigned chunk;  // elements of one channel per workgroup (a multiple of 4)
    unsigned ns;     // workgroups per channel
    odl::FastDiv by_plane;  // by P / 4 (16-byte path) or by P
};

__device__ inline float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

// sum over the workgroup, valid in every thread
__device__ inline float block_sum_all(float v)
{
    __shared__ float part[kBlock / 64];
    v = wave_sum(v);
    __syncthreads();  // readers of an earlier call are done with `part`
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < kBlock / 64; ++i)
        s += part[i];
    return s;
}

// visits this workgroup's chunk of channel c: f(offset into the tensor, slot 0..3); with V4 an offset names four
// consecutive floats of one image plane
template <bool V4, typename F>
__device__ inline void visit_chunk(const BnGeom &g, F &&f)
{
    constexpr unsigned E = V4 ? 4 : 1;
    const unsigned c = blockIdx.y;
    const unsigned beg = blockIdx.x * g.chunk;
    const unsigned end = (beg + g.chunk < g.total) ? beg + g.chunk : g.total;
    const unsigned plane = g.P / E;
    for (unsigned u0 = beg / E + threadIdx.x; u0 < end / E; u0 += 4 * kBlock)
    {
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const unsigned u = u0 + j * kBlock;
            if (u < end / E)
            {
                const unsigned n = odl::fastdiv(u, g.by_plane), v = u - n * plane;
                f(((int64_t)n * g.C + c) * g.P + (int64_t)v * E, j);
            }
        }
    }
}

// the channel's total from its per-workgroup partials, added in workgroup order by every thread alike
__device__ inline float channel_total(const float *part, unsigned c, unsigned ns, unsigned stride, unsigned which)
{
    float s = 0.f;
    for (unsigned i = 0; i < ns; ++i)
        s += part[((int64_t)c * ns + i) * stride + which];
    return s;
}

template <bool V4>
__global__ __launch_bounds__(kBlock) void bn_sum_kernel(const float *__restrict__ x, float *__restrict__ part, BnGeom g)
{
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    visit_chunk<V4>(g, [&](int64_t off, int j) {
        if (V4)
        {
            const f32x4 q = *reinterpret_cast<const f32x4 *>(x + off);
            acc[j] += (q[0] + q[1]) + (q[2] + q[3]);
        }
        else
            acc[j] += x[off];
    });
    const float s = block_sum_all((acc[0] + acc[1]) + (acc[2] + acc[3]));
    if (threadIdx.x == 0)
        part[(int64_t)blockIdx.y * g.ns + blockIdx.x] = s;
}

template <bool V4>
__global__ __launch_bounds__(kBlock) void bn_sqdiff_kernel(const float *__restrict__ x, const float *__restrict__ sums,
                                                            float *__restrict__ part, float *__restrict__ mean_out,
                                                            BnGeom g, float count)
{
    const float mean = channel_total(sums, blockIdx.y, g.ns, 1, 0) / count;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    visit_chunk<V4>(g, [&](int64_t off, int j) {
        if (V4)
        {
            const f32x4 q = *reinterpret_cast<const f32x4 *>(x + off);
            const float d0 = q[0] - mean, d1 = q[1] - mean, d2 = q[2] - mean, d3 = q[3] - mean;
            acc[j] += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
        }
        else
        {
            const float d = x[off] - mean;
            acc[j] += d * d;
        }
    });
    const float s = block_sum_all((acc[0] + acc[1]) + (acc[2] + acc[3]));
    if (threadIdx.x == 0)
    {
        part[(int64_t)blockIdx.y * g.ns + blockIdx.x] = s;
        if (blockIdx.x == 0)
            mean_out[blockIdx.y] = mean;
    }
}

// mean / variance either from the batch (sqsums != nullptr: variance = its total / count, mean as already stored) or
// from the running statistics; writes the statistics used, x_norm (when asked for) and y
template <bool V4, bool RELU>
__global__ __launch_bounds__(kBlock) void bn_apply_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                           const float *__restrict__ beta,
                                                           const float *__restrict__ mean_src,
                                                           const float *__restrict__ var_src,
                                                           const float *__restrict__ sqsums, float *__restrict__ mean_out,
                                                           float *__restrict__ var_out, float *__restrict__ y,
                                                           float *__restrict__ x_norm, BnGeom g, float count, float eps)
{
    const unsigned c = blockIdx.y;
    const float mean = mean_src[c];
    const float var = sqsums ? channel_total(sqsums, c, g.ns, 1, 0) / count : var_src[c];
    if (blockIdx.x == 0 && threadIdx.x == 0)
    {
        var_out[c] = var;
        if (mean_out != mean_src)
            mean_out[c] = mean;
    }
    const float stdv = sqrtf(var + eps);
    const float ga = gamma[c], be = beta[c];
    visit_chunk<V4>(g, [&](int64_t off, int) {
        if (V4)
        {
            const f32x4 q = *reinterpret_cast<const f32x4 *>(x + off);
            f32x4 xn, o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                xn[i] = (q[i] - mean) / stdv;
                o[i] = ga * xn[i] + be;
                if (RELU)
                    o[i] = odl::apply_act(o[i], 1);
            }
            if (x_norm)
                *reinterpret_cast<f32x4 *>(x_norm + off) = xn;
            *reinterpret_cast<f32x4 *>(y + off) = o;
        }
        else
        {
            const float xn = (x[off] - mean) / stdv;
            if (x_norm)
                x_norm[off] = xn;
            const float o = ga * xn + be;
            y[off] = RELU ? odl::apply_act(o, 1) : o;
        }
    });
}

// FROM_X: `xn` holds x itself and the normalised value is formed here, (x - mean) / sqrt(var + eps) — the expression
// the forward pass used, so the same float — instead of being read back from a saved copy.
//
// RELU: the layer's output went through a ReLU before anything else saw it, and `gy` is the gradient of THAT output.
// The ReLU's mask is formed again from the expression the forward pass evaluated, gamma * xn + beta > 0, and gy is
// multiplied by 1 or 0 as the separate ReLU backward would (relu.cpp:45-52), so both kernels see the masked gradient
// without it ever being stored.
template <bool V4, bool FROM_X, bool RELU>
__global__ __launch_bounds__(kBlock) void bn_bwd_sums_kernel(const float *__restrict__ gy, const float *__restrict__ xn,
                                                              const float *__restrict__ gamma,
                                                              const float *__restrict__ beta,
                                                              const float *__restrict__ mean,
                                                              const float *__restrict__ var, float eps,
                                                              float *__restrict__ part, BnGeom g)
{
    const float mu = FROM_X ? mean[blockIdx.y] : 0.f;
    const float sd = FROM_X ? sqrtf(var[blockIdx.y] + eps) : 1.f;
    const float ga = RELU ? gamma[blockIdx.y] : 0.f, be = RELU ? beta[blockIdx.y] : 0.f;
    float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
    visit_chunk<V4>(g, [&](int64_t off, int j) {
        if (V4)
        {
            f32x4 q = *reinterpret_cast<const f32x4 *>(gy + off);
            f32x4 r = *reinterpret_cast<const f32x4 *>(xn + off);
            if (FROM_X)
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    r[i] = (r[i] - mu) / sd;
            }
            if (RELU)
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    q[i] = q[i] * (ga * r[i] + be > 0.f ? 1.f : 0.f);
            }
            a[j] += (q[0] + q[1]) + (q[2] + q[3]);
            b[j] += (q[0] * r[0] + q[1] * r[1]) + (q[2] * r[2] + q[3] * r[3]);
        }
        else
        {
            const float r = FROM_X ? (xn[off] - mu) / sd : xn[off];
            const float q = RELU ? gy[off] * (ga * r + be > 0.f ? 1.f : 0.f) : gy[off];
            a[j] += q;
            b[j] += q * r;
        }
    });
    const float sa = block_sum_all((a[0] + a[1]) + (a[2] + a[3]));
    const float sb = block_sum_all((b[0] + b[1]) + (b[2] + b[3]));
    if (threadIdx.x == 0)
    {
        float *p = part + ((int64_t)blockIdx.y * g.ns + blockIdx.x) * 2;
        p[0] = sa, p[1] = sb;
    }
}

template <bool V4, bool FROM_X, bool RELU>
__global__ __launch_bounds__(kBlock) void bn_bwd_apply_kernel(const float *__restrict__ gy, const float *__restrict__ xn,
                                                               const float *__restrict__ gamma,
                                                               const float *__restrict__ beta,
                                                               const float *__restrict__ mean,
                                                               const float *__restrict__ var,
                                                               const float *__restrict__ part, float *__restrict__ gx,
                                                               float *__restrict__ dgamma, float *__restrict__ dbeta,
                                                               BnGeom g, float count, float eps)
{
    const unsigned c = blockIdx.y;
    const float mu = FROM_X ? mean[c] : 0.f;
    const float sd = sqrtf(var[c] + eps);
    const float sum_gy = channel_total(part, c, g.ns, 2, 0), sum_gy_xn = channel_total(part, c, g.ns, 2, 1);
    if (blockIdx.x == 0 && threadIdx.x == 0)
        dgamma[c] = sum_gy_xn, dbeta[c] = sum_gy;
    const float mean_gy = sum_gy / count, mean_gy_xn = sum_gy_xn / count;
    const float scale = gamma[c] / sd;
    const float ga = gamma[c], be = RELU ? beta[c] : 0.f;
    visit_chunk<V4>(g, [&](int64_t off, int) {
        if (V4)
        {
            f32x4 q = *reinterpret_cast<const f32x4 *>(gy + off);
            f32x4 r = *reinterpret_cast<const f32x4 *>(xn + off);
            f32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                if (FROM_X)
                    r[i] = (r[i] - mu) / sd;
                if (RELU)
                    q[i] = q[i] * (ga * r[i] + be > 0.f ? 1.f : 0.f);
                const float t = r[i] * mean_gy_xn;
                o[i] = scale * ((q[i] - mean_gy) - t);
            }
            *reinterpret_cast<f32x4 *>(gx + off) = o;
        }
        else
        {
            const float r = FROM_X ? (xn[off] - mu) / sd : xn[off];
            const float q = RELU ? gy[off] * (ga * r + be > 0.f ? 1.f : 0.f) : gy[off];
            const float t = r * mean_gy_xn;
            gx[off] = scale * ((q - mean_gy) - t);
        }
    });
}

template <bool VEC>
__global__ __launch_bounds__(kBlock) void axpby_kernel(float a, const float *__restrict__ x, float b,
                                                        const float *__restrict__ y, float *__restrict__ out, int64_t n)
{
    const int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * (VEC ? 4 : 1);
    if (i >= n)
        return;
    if (VEC)
    {
        const f32x4 p = *reinterpret_cast<const f32x4 *>(x + i), q = *reinterpret_cast<const f32x4 *>(y + i);
        f32x4 o;
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            const float u = a * p[k], v = b * q[k];
            o[k] = u + v;
        }
        *reinterpret_cast<f32x4 *>(out + i) = o;
    }
    else
    {
        const float u = a * x[i], v = b * y[i];
        out[i] = u + v;
    }
}

bool plan_bn(int64_t N, int64_t C, int64_t P, BnGeom &g)
{
    const int64_t total = N * P;
    if (N < 0 || C <= 0 || P <= 0 || total >= (1ll << 31) || C >= 65536)
        return false;
    int64_t want = odl::ceil_div(2048, C);  // about eight workgroups per CU over all channels
    int64_t chunk = odl::ceil_div(total > 0 ? total : 1, want);
    if (chunk < 2048)
        chunk = 2048;
    chunk = odl::ceil_div(chunk, 4) * 4;
    const int64_t ns = odl::ceil_div(total > 0 ? total : 1, chunk);
    if (ns >= 65536)
        return false;
    g = BnGeom{(unsigned)C, (unsigned)P, (unsigned)total, (unsigned)chunk, (unsigned)ns, odl::FastDiv{0, 0, 0}};
    return true;
}

inline bool aligned16(const void *p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}
}  // namespace

extern "C" {

size_t odl_hip_batch_norm_workspace_bytes(int64_t N, int64_t C, int64_t P)
{
    BnGeom g;
    if (!plan_bn(N, C, P, g))
        return 0;
    return (size_t)C * g.ns * 2 * sizeof(float);
}

static int bn_forward_launch(const float *x, const float *gamma, const float *beta, const float *running_mean,
                             const float *running_var, int training, float eps, int64_t N, int64_t C, int64_t P, float *y,
                             float *mean, float *var, float *x_norm, bool relu, void *workspace, size_t workspace_bytes,
                             void *stream)
{
    ODL_REQUIRE_DEVICE();
    BnGeom g;
    ODL_REQUIRE(plan_bn(N, C, P, g), "batch_norm: bad shape (N=%lld, C=%lld, P=%lld)", (long long)N, (long long)C,
                (long long)P);
    ODL_REQUIRE(x && gamma && beta && y && mean && var, "batch_norm: null operand");
    ODL_REQUIRE(training || (running_mean && running_var), "batch_norm: evaluation mode needs the running statistics");
    if (N == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    const bool v4 = P % 4 == 0 && aligned16(x) && aligned16(y) && (x_norm == nullptr || aligned16(x_norm));
    g.by_plane = odl::make_fastdiv((unsigned)(v4 ? P / 4 : P));
    const dim3 grid(g.ns, g.C), block(kBlock);
    const float count = (float)(N * P);
    float *sums = nullptr, *sqsums = nullptr;
    if (training)
    {
        const size_t need = (size_t)C * g.ns * 2 * sizeof(float);
        ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need, "batch_norm: workspace of %zu bytes required, got %zu",
                    need, workspace_bytes);
        sums = static_cast<float *>(workspace), sqsums = sums + (size_t)C * g.ns;
        if (v4)
        {
            hipLaunchKernelGGL((bn_sum_kernel<true>), grid, block, 0, st, x, sums, g);
            hipLaunchKernelGGL((bn_sqdiff_kernel<true>), grid, block, 0, st, x, sums, sqsums, mean, g, count);
        }
        else
        {
            hipLaunchKernelGGL((bn_sum_kernel<false>), grid, block, 0, st, x, sums, g);
            hipLaunchKernelGGL((bn_sqdiff_kernel<false>), grid, block, 0, st, x, sums, sqsums, mean, g, count);
        }
        ODL_LAUNCH_CHECK();
    }
    const float *mean_src = training ? mean : running_mean;
#define ODL_BN_APPLY(V4, RELU)                                                                                       \
    hipLaunchKernelGGL((bn_apply_kernel<V4, RELU>), grid, block, 0, st, x, gamma, beta, mean_src, running_var, sqsums, \
                       mean, var, y, x_norm, g, count, eps)
    if (v4 && relu)
        ODL_BN_APPLY(true, true);
    else if (v4)
        ODL_BN_APPLY(true, false);
    else if (relu)
        ODL_BN_APPLY(false, true);
    else
        ODL_BN_APPLY(false, false);
#undef ODL_BN_APPLY
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_batch_norm_forward(const float *x, const float *gamma, const float *beta, const float *running_mean,
                               const float *running_var, int training, float eps, int64_t N, int64_t C, int64_t P,
                               float *y, float *mean, float *var, float *x_norm, void *workspace,
                               size_t workspace_bytes, void *stream)
{
    return bn_forward_launch(x, gamma, beta, running_mean, running_var, training, eps, N, C, P, y, mean, var, x_norm,
                             false, workspace, workspace_bytes, stream);
}

int odl_hip_batch_norm_relu_forward(const float *x, const float *gamma, const float *beta, const float *running_mean,
                                    const float *running_var, int training, float eps, int64_t N, int64_t C, int64_t P,
                                    float *y, float *mean, float *var, void *workspace, size_t workspace_bytes,
                                    void *stream)
{
    return bn_forward_launch(x, gamma, beta, running_mean, running_var, training, eps, N, C, P, y, mean, var, nullptr,
                             true, workspace, workspace_bytes, stream);
}

static int bn_backward_launch(const float *gy, const float *gamma, const float *beta_for_relu, const float *saved_mean,
                              const float *saved_var, const float *xn_or_x, bool from_x, float eps, int64_t N, int64_t C, int64_t P, float *gx,
                              float *dgamma, float *dbeta, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    BnGeom g;
    ODL_REQUIRE(plan_bn(N, C, P, g), "batch_norm_backward: bad shape (N=%lld, C=%lld, P=%lld)", (long long)N,
                (long long)C, (long long)P);
    ODL_REQUIRE(gy && gamma && saved_var && xn_or_x && gx && dgamma && dbeta && (!from_x || saved_mean),
                "batch_norm_backward: null operand");
    hipStream_t st = odl::as_stream(stream);
    if (N == 0)  // nothing to sum: the parameter gradients are zero (batch_norm.cpp:337-339)
    {
        int rc = odl::fill_launch(dgamma, C, 0.f, st);
        return rc != ODL_OK ? rc : odl::fill_launch(dbeta, C, 0.f, st);
    }
    const size_t need = (size_t)C * g.ns * 2 * sizeof(float);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need,
                "batch_norm_backward: workspace of %zu bytes required, got %zu", need, workspace_bytes);
    float *part = static_cast<float *>(workspace);
    const bool v4 = P % 4 == 0 && aligned16(gy) && aligned16(xn_or_x) && aligned16(gx);
    g.by_plane = odl::make_fastdiv((unsigned)(v4 ? P / 4 : P));
    const dim3 grid(g.ns, g.C), block(kBlock);
    const float count = (float)(N * P);
#define ODL_BN_BWD(V4, FX, RELU)                                                                                    \
    hipLaunchKernelGGL((bn_bwd_sums_kernel<V4, FX, RELU>), grid, block, 0, st, gy, xn_or_x, gamma, beta_for_relu,       \
                       saved_mean, saved_var, eps, part, g);                                                        \
    hipLaunchKernelGGL((bn_bwd_apply_kernel<V4, FX, RELU>), grid, block, 0, st, gy, xn_or_x, gamma, beta_for_relu,      \
                       saved_mean, saved_var, part, gx, dgamma, dbeta, g, count, eps)
    if (beta_for_relu)  // the fused layer keeps x, never x_norm
    {
        if (v4)
        {
            ODL_BN_BWD(true, true, true);
        }
        else
        {
            ODL_BN_BWD(false, true, true);
        }
    }
    else if (v4 && from_x)
    {
        ODL_BN_BWD(true, true, false);
    }
    else if (v4)
    {
        ODL_BN_BWD(true, false, false);
    }
    else if (from_x)
    {
        ODL_BN_BWD(false, true, false);
    }
    else
    {
        ODL_BN_BWD(false, false, false);
    }
#undef ODL_BN_BWD
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_batch_norm_backward(const float *gy, const float *gamma, const float *saved_var, const float *saved_x_norm,
                                float eps, int64_t N, int64_t C, int64_t P, float *gx, float *dgamma, float *dbeta,
                                void *workspace, size_t workspace_bytes, void *stream)
{
    return bn_backward_launch(gy, gamma, nullptr, nullptr, saved_var, saved_x_norm, false, eps, N, C, P, gx, dgamma, dbeta,
                              workspace, workspace_bytes, stream);
}

int odl_hip_batch_norm_backward_from_x(const float *gy, const float *x, const float *gamma, const float *saved_mean,
                                       const float *saved_var, float eps, int64_t N, int64_t C, int64_t P, float *gx,
                                       float *dgamma, float *dbeta, void *workspace, size_t workspace_bytes,
                                       void *stream)
{
    return bn_backward_launch(gy, gamma, nullptr, saved_mean, saved_var, x, true, eps, N, C, P, gx, dgamma, dbeta, workspace,
                              workspace_bytes, stream);
}

int odl_hip_batch_norm_relu_backward_from_x(const float *gy, const float *x, const float *gamma, const float *beta,
                                            const float *saved_mean, const float *saved_var, float eps, int64_t N,
                                            int64_t C, int64_t P, float *gx, float *dgamma, float *dbeta,
                                            void *workspace, size_t workspace_bytes, void *stream)
{
    if (!beta)
        return odl::fail(ODL_ERR_INVALID_ARG, "batch_norm_relu_backward: null operand");
    return bn_backward_launch(gy, gamma, beta, saved_mean, saved_var, x, true, eps, N, C, P, gx, dgamma, dbeta, workspace,
                              workspace_bytes, stream);
}

// ---- float64 (src/mat/origin/cuda/normalization/batch_norm.cu:497-560 runs the same algorithm on doubles). Not a hot
// path: one workgroup per channel walks the channel's N*P elements three times (sum, squared deviations, apply), the
// sums reduced in a fixed order.
}  // extern "C"

namespace
{
__device__ inline double block_sum_f64(double v, double *sh)
{
    for (int off = 32; off > 0; off >>= 1)
        v += __shfl_down(v, off, 64);
    if ((threadIdx.x & 63) == 0)
        sh[threadIdx.x >> 6] = v;
    __syncthreads();
    double s = 0.0;
    for (int i = 0; i < kBlock / 64; ++i)
        s += sh[i];
    __syncthreads();
    return s;  // the same value in every thread
}

__global__ __launch_bounds__(kBlock) void bn_forward_f64_kernel(const double *__restrict__ x, const double *__restrict__ gamma,
                                                                const double *__restrict__ beta,
                                                                const double *__restrict__ running_mean,
                                                                const double *__restrict__ running_var, int training,
                                                                double eps, int64_t N, int64_t C, int64_t P,
                                                                double *__restrict__ y, double *__restrict__ mean_out,
                                                                double *__restrict__ var_out, double *__restrict__ x_norm)
{
    __shared__ double sh[kBlock / 64];
    const int64_t c = blockIdx.x, total = N * P;
    auto at = [&](int64_t i) { return ((i / P) * C + c) * P + i % P; };
    double mean, var;
    if (training)
    {
        double acc = 0.0;
        for (int64_t i = threadIdx.x; i < total; i += kBlock)
            acc += x[at(i)];
        mean = block_sum_f64(acc, sh) / (double)total;
        acc = 0.0;
        for (int64_t i = threadIdx.x; i < total; i += kBlock)
        {
            const double d = x[at(i)] - mean;
            acc += d * d;
        }
        var = block_sum_f64(acc, sh) / (double)total;
    }
    else
        mean = running_mean[c], var = running_var[c];
    if (threadIdx.x == 0)
        mean_out[c] = mean, var_out[c] = var;
    const double stdv = sqrt(var + eps), ga = gamma[c], be = beta[c];
    for (int64_t i = threadIdx.x; i < total; i += kBlock)
    {
        const int64_t off = at(i);
        const double xn = (x[off] - mean) / stdv;
        if (x_norm)
            x_norm[off] = xn;
        y[off] = ga * xn + be;
    }
}

__global__ __launch_bounds__(kBlock) void bn_backward_f64_kernel(const double *__restrict__ gy, const double *__restrict__ xn_or_x,
                                                                 int from_x, const double *__restrict__ gamma,
                                                                 const double *__restrict__ mean,
                                                                 const double *__restrict__ var, double eps, int64_t N,
                                                                 int64_t C, int64_t P, double *__restrict__ gx,
                                                                 double *__restrict__ dgamma, double *__restrict__ dbeta)
{
    __shared__ double sh[kBlock / 64];
    const int64_t c = blockIdx.x, total = N * P;
    auto at = [&](int64_t i) { return ((i / P) * C + c) * P + i % P; };
    const double mu = from_x ? mean[c] : 0.0, sd = sqrt(var[c] + eps);
    auto norm = [&](int64_t off) { return from_x ? (xn_or_x[off] - mu) / sd : xn_or_x[off]; };
    double a = 0.0, b = 0.0;
    for (int64_t i = threadIdx.x; i < total; i += kBlock)
    {
        const int64_t off = at(i);
        a += gy[off];
        b += gy[off] * norm(off);
    }
    const double sum_gy = block_sum_f64(a, sh), sum_gy_xn = block_sum_f64(b, sh);
    if (threadIdx.x == 0)
        dgamma[c] = sum_gy_xn, dbeta[c] = sum_gy;
    const double mean_gy = sum_gy / (double)total, mean_gy_xn = sum_gy_xn / (double)total, scale = gamma[c] / sd;
    for (int64_t i = threadIdx.x; i < total; i += kBlock)
    {
        const int64_t off = at(i);
        gx[off] = scale * ((gy[off] - mean_gy) - norm(off) * mean_gy_xn);
    }
}
}  // namespace

extern "C" {

int odl_hip_batch_norm_forward_f64(const double *x, const double *gamma, const double *beta, const double *running_mean,
                                   const double *running_var, int training, double eps, int64_t N, int64_t C, int64_t P,
                                   double *y, double *mean, double *var, double *x_norm, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && C > 0 && P > 0 && C < (1ll << 31), "batch_norm: bad shape (N=%lld, C=%lld, P=%lld)", (long long)N,
                (long long)C, (long long)P);
    ODL_REQUIRE(x && gamma && beta && y && mean && var, "batch_norm: null operand");
    ODL_REQUIRE(training || (running_mean && running_var), "batch_norm: evaluation mode needs the running statistics");
    if (N == 0)
        return ODL_OK;
    hipLaunchKernelGGL(bn_forward_f64_kernel, dim3((unsigned)C), dim3(kBlock), 0, odl::as_stream(stream), x, gamma, beta,
                       running_mean, running_var, training, eps, N, C, P, y, mean, var, x_norm);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_batch_norm_backward_f64(const double *gy, const double *x_norm_or_x, int from_x, const double *gamma,
                                    const double *saved_mean, const double *saved_var, double eps, int64_t N, int64_t C,
                                    int64_t P, double *gx, double *dgamma, double *dbeta, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N > 0 && C > 0 && P > 0 && C < (1ll << 31), "batch_norm_backward: bad shape (N=%lld, C=%lld, P=%lld)",
                (long long)N, (long long)C, (long long)P);
    ODL_REQUIRE(gy && gamma && saved_var && x_norm_or_x && gx && dgamma && dbeta && (!from_x || saved_mean),
                "batch_norm_backward: null operand");
    hipLaunchKernelGGL(bn_backward_f64_kernel, dim3((unsigned)C), dim3(kBlock), 0, odl::as_stream(stream), gy, x_norm_or_x,
                       from_x, gamma, saved_mean, saved_var, eps, N, C, P, gx, dgamma, dbeta);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_axpby(float a, const float *x, float b, const float *y, int64_t n, float *out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(n >= 0, "axpby: negative length");
    if (n == 0)
        return ODL_OK;
    ODL_REQUIRE(x && y && out, "axpby: null operand");
    hipStream_t st = odl::as_stream(stream);
    if (n % 4 == 0 && aligned16(x) && aligned16(y) && aligned16(out))
        hipLaunchKernelGGL((axpby_kernel<true>), dim3((unsigned)odl::ceil_div(n / 4, kBlock)), dim3(kBlock), 0, st, a, x, b,
                           y, out, n);
    else
        hipLaunchKernelGGL((axpby_kernel<false>), dim3((unsigned)odl::ceil_div(n, kBlock)), dim3(kBlock), 0, st, a, x, b, y,
                           out, n);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

}  // extern "C"
