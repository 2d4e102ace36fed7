// Softmax, gather / one-hot and the fused softmax-cross-entropy forward and gradient, plus the host-argmax
// metric done on the device. The reference builds softmax from eight separate Mat ops with materialised
// broadcasts and syncs twice inside the loss (src/operators/activation/softmax.cpp:14-76,
// src/operators/loss/softmax_cross_entropy.cpp:17-111); here a row of logits is read once by one wave,
// reduced with wave64 shuffles and written once.
#include <cfloat>
#include <vector>

#include "odl_common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace
{
constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;

__device__ inline float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

__device__ inline float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        const float u = __shfl_xor(v, o, 64);
        v = (v < u) ? u : v;
    }
    return v;
}

__device__ inline int64_t label_at(const void *idx, int is64, int64_t i)
{
    return is64 ? static_cast<const int64_t *>(idx)[i] : (int64_t) static_cast<const int32_t *>(idx)[i];
}

// row statistics of one contiguous row handled by one wave: max, then sum of exp(x - max)
__device__ inline void row_stats(const float *row, int64_t C, int lane, float &mx, float &sum)
{
    float m = -FLT_MAX;
    for (int64_t j = lane; j < C; j += 64)
        m = (m < row[j]) ? row[j] : m;
    m = wave_max(m);
    float s = 0.f;
    for (int64_t j = lane; j < C; j += 64)
        s += expf(row[j] - m);
    mx = m;
    sum = wave_sum(s);
}

__global__ void softmax_rows_kernel(const float *__restrict__ x, float *__restrict__ y, int64_t N, int64_t C)
{
    const int64_t row = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (row >= N)
        return;
    const int lane = threadIdx.x & 63;
    float m, s;
    row_stats(x + row * C, C, lane, m, s);
    for (int64_t j = lane; j < C; j += 64)
        y[row * C + j] = expf(x[row * C + j] - m) / s;
}

// Rows whose length is a multiple of 4 and whose bases are 16-byte aligned: a wave keeps its row in registers (QUADS
// float4 per lane, rows of up to 256*QUADS values), so the row is read once and written once.
template <int QUADS>
__global__ __launch_bounds__(kBlock) void softmax_rows_vec_kernel(const float *__restrict__ x, float *__restrict__ y, int64_t N,
                                                                   int64_t C)
{
    const int64_t row = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (row >= N)
        return;
    const int lane = threadIdx.x & 63;
    const f32x4 *xr = reinterpret_cast<const f32x4 *>(x + row * C);
    f32x4 *yr = reinterpret_cast<f32x4 *>(y + row * C);
    const int64_t cq = C / 4;
    f32x4 v[QUADS];
    float m = -FLT_MAX;
#pragma unroll
    for (int u = 0; u < QUADS; ++u)
    {
        const int64_t q = lane + 64 * u;
        if (q < cq)
            v[u] = xr[q];
        else
            v[u] = f32x4{-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
#pragma unroll
        for (int e = 0; e < 4; ++e)
            m = (m < v[u][e]) ? v[u][e] : m;
    }
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < QUADS; ++u)
    {
        const bool in = lane + 64 * u < cq;
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            v[u][e] = in ? expf(v[u][e] - m) : 0.f;
            s += v[u][e];
        }
    }
    s = wave_sum(s);
#pragma unroll
    for (int u = 0; u < QUADS; ++u)
    {
        const int64_t q = lane + 64 * u;
        if (q < cq)
        {
            f32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                o[e] = v[u][e] / s;
            yr[q] = o;
        }
    }
}

// softmax along the middle axis of [outer, axis, inner], one thread per (outer, inner) pair
__global__ void softmax_strided_kernel(const float *__restrict__ x, float *__restrict__ y, int64_t outer, int64_t axis,
                                       int64_t inner)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= outer * inner)
        return;
    const int64_t o = t / inner, i = t % inner;
    const float *p = x + o * axis * inner + i;
    float *q = y + o * axis * inner + i;
    float m = -FLT_MAX;
#pragma unroll 8
    for (int64_t a = 0; a < axis; ++a)
        m = (m < p[a * inner]) ? p[a * inner] : m;
    float s = 0.f;
#pragma unroll 8
    for (int64_t a = 0; a < axis; ++a)
        s += expf(p[a * inner] - m);
#pragma unroll 8
    for (int64_t a = 0; a < axis; ++a)
        q[a * inner] = expf(p[a * inner] - m) / s;
}

__global__ void gather_kernel(const float *__restrict__ in, const void *idx, int is64, int64_t N, int64_t C,
                              float *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N)
        return;
    const int64_t t = label_at(idx, is64, i);
    out[i] = (t >= 0 && t < C) ? in[i * C + t] : 0.f;
}

// the same for elements of another size (a copy: the element type does not matter beyond its width)
template <typename U>
__global__ void gather_words_kernel(const U *__restrict__ in, const void *idx, int is64, int64_t N, int64_t C, U *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N)
        return;
    const int64_t t = label_at(idx, is64, i);
    out[i] = (t >= 0 && t < C) ? in[i * C + t] : (U)0;
}

__global__ void one_hot_kernel(const void *idx, int is64, int64_t N, int64_t C, float *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= N * C)
        return;
    const int64_t i = e / C, j = e % C;
    out[e] = (label_at(idx, is64, i) == j) ? 1.f : 0.f;  // out-of-range labels match no column (gather.cpp:134)
}

// rows of a multiple of four classes, 16-byte aligned output: one 16-byte store per thread, the label read once per quad
__global__ void one_hot_quads_kernel(const void *idx, int is64, unsigned quads, unsigned cq, odl::FastDiv d_cq,
                                     float *__restrict__ out)
{
    const unsigned q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= quads)
        return;
    const unsigned i = odl::fastdiv(q, d_cq), j = (q - i * cq) * 4u;
    const int64_t d = label_at(idx, is64, i) - (int64_t)j;  // the quad's element that is set, if 0 <= d < 4
    reinterpret_cast<f32x4 *>(out)[q] = f32x4{d == 0 ? 1.f : 0.f, d == 1 ? 1.f : 0.f, d == 2 ? 1.f : 0.f, d == 3 ? 1.f : 0.f};
}

// logp[i] = log(softmax(x)[i, t_i] + 1e-8); flag[0] |= 1 when a label is out of range
__global__ void ce_row_logp_kernel(const float *__restrict__ x, const void *t, int is64, int64_t N, int64_t C,
                                   float *__restrict__ logp, int *flag)
{
    const int64_t row = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (row >= N)
        return;
    const int lane = threadIdx.x & 63;
    float m, s;
    row_stats(x + row * C, C, lane, m, s);
    if (lane == 0)
    {
        const int64_t lab = label_at(t, is64, row);
        if (lab < 0 || lab >= C)
        {
            atomicOr(flag, 1);
            logp[row] = 0.f;
        }
        else
        {
            const float p = expf(x[row * C + lab] - m) / s;
            logp[row] = logf(p + 1e-8f);
        }
    }
}

// The same with the row in registers (lengths that are multiples of 4, 16-byte aligned base, up to 256*QUADS classes):
// one read of x instead of two.
template <int QUADS>
__global__ __launch_bounds__(kBlock) void ce_row_logp_vec_kernel(const float *__restrict__ x, const void *t, int is64, int64_t N,
                                                                  int64_t C, float *__restrict__ logp, int *flag)
{
    const int64_t row = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (row >= N)
        return;
    const int lane = threadIdx.x & 63;
    const f32x4 *xr = reinterpret_cast<const f32x4 *>(x + row * C);
    const int64_t cq = C / 4;
    f32x4 v[QUADS];
    float m = -FLT_MAX;
#pragma unroll
    for (int u = 0; u < QUADS; ++u)
    {
        const int64_t q = lane + 64 * u;
        if (q < cq)
            v[u] = xr[q];
        else
            v[u] = f32x4{-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
#pragma unroll
        for (int e = 0; e < 4; ++e)
            m = (m < v[u][e]) ? v[u][e] : m;
    }
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < QUADS; ++u)
    {
        const bool in = lane + 64 * u < cq;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            s += in ? expf(v[u][e] - m) : 0.f;
    }
    s = wave_sum(s);
    if (lane == 0)
    {
        const int64_t lab = label_at(t, is64, row);
        if (lab < 0 || lab >= C)
        {
            atomicOr(flag, 1);
            logp[row] = 0.f;
        }
        else
        {
            const float p = expf(x[row * C + lab] - m) / s;
            logp[row] = logf(p + 1e-8f);
        }
    }
}

// out[0] = -(sum of logp) / N   (softmax_cross_entropy.cpp:67-70); one workgroup
// mirror (may be null): pinned host memory that receives the loss word and the flag word behind it as well
__global__ void ce_finish_kernel(const float *__restrict__ logp, int64_t N, float *out, unsigned int *mirror)
{
    __shared__ float part[1024 / 64];
    float acc = 0.f;
    for (int64_t i = threadIdx.x; i < N; i += blockDim.x)
        acc += logp[i];
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        float s = 0.f;
        for (unsigned i = 0; i < blockDim.x / 64; ++i)
            s += part[i];
        const float loss = -s / (float)N;
        out[0] = loss;
        if (mirror)
        {
            mirror[0] = __float_as_uint(loss);
            mirror[1] = reinterpret_cast<const unsigned int *>(out)[1];  // set by the kernel that ran before this one
        }
    }
}

// The whole loss of a small batch of short rows in ONE launch (the three-launch schedule above is bound by launch latency
// there): one workgroup, a thread per row — max, sum of exponentials and the label's probability in the order the
// reference's loops take them (src/operators/loss/softmax_cross_entropy.cpp:30-70) — then the block sum of ce_finish_kernel.
// Writes both words: out2[0] = loss, out2[1] = 1 when a label is out of range.
__global__ __launch_bounds__(1024) void ce_loss_small_kernel(const float *__restrict__ x, const void *t, int is64, int N,
                                                             int C, unsigned int *out2, unsigned int *mirror)
{
    __shared__ float part[1024 / 64];
    __shared__ int bad;
    if (threadIdx.x == 0)
        bad = 0;
    __syncthreads();
    float acc = 0.f;
    for (int row = threadIdx.x; row < N; row += 1024)
    {
        const float *xr = x + (int64_t)row * C;
        float m = -FLT_MAX;
        for (int j = 0; j < C; ++j)
            m = (m < xr[j]) ? xr[j] : m;
        float s = 0.f;
        for (int j = 0; j < C; ++j)
            s += expf(xr[j] - m);
        const int64_t lab = label_at(t, is64, row);
        if (lab < 0 || lab >= C)
            bad = 1;  // every writer stores the same value
        else
        {
            const float p = expf(xr[lab] - m) / s;
            acc += logf(p + 1e-8f);
        }
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        float s = 0.f;
        for (int i = 0; i < 1024 / 64; ++i)
            s += part[i];
        const float loss = -s / (float)N;
        out2[0] = __float_as_uint(loss);
        out2[1] = bad ? 1u : 0u;
        if (mirror)
            mirror[0] = __float_as_uint(loss), mirror[1] = bad ? 1u : 0u;
    }
}

// The same launch with the gradient for an upstream gradient of one written beside the loss — what backward() asks for
// right after (its seed is the constant 1), so that it needs no launch of its own. Per row the gradient is the float
// ce_grad_kernel<1> would write: that kernel spreads a row over a wave's lanes and adds the exponentials by a butterfly
// (lane l adds lane l ^ 32, then ^ 16, ...), which is a tree of sums a thread can walk alone — lanes past the row hold
// zeros, and adding zero is exact. CMAX: the power of two the classes fit in (the tree's empty upper levels are skipped).
template <int CMAX>
__global__ __launch_bounds__(1024) void ce_loss_grad_small_kernel(const float *__restrict__ x, const void *t, int is64, int N,
                                                                  int C, unsigned int *out2, unsigned int *mirror,
                                                                  float *__restrict__ gx, float scale)
{
    __shared__ float part[1024 / 64];
    __shared__ int bad;
    if (threadIdx.x == 0)
        bad = 0;
    __syncthreads();
    float acc = 0.f;
    for (int row = threadIdx.x; row < N; row += 1024)
    {
        const float *xr = x + (int64_t)row * C;
        float m = -FLT_MAX;
        for (int j = 0; j < C; ++j)
            m = (m < xr[j]) ? xr[j] : m;
        float e[CMAX];
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < CMAX; ++j)
        {
            e[j] = 0.f;
            if (j < C)  // (the same in every thread)
            {
                e[j] = expf(xr[j] - m);
                s += e[j];
            }
        }
        const int64_t lab = label_at(t, is64, row);
        if (lab < 0 || lab >= C)
            bad = 1;  // every writer stores the same value
        else
        {
            const float p = expf(xr[lab] - m) / s;
            acc += logf(p + 1e-8f);
        }
        // the wave's sum of the exponentials
        float tree[CMAX];
#pragma unroll
        for (int j = 0; j < CMAX; ++j)
            tree[j] = e[j];
#pragma unroll
        for (int o = CMAX / 2; o > 0; o >>= 1)
#pragma unroll
            for (int l = 0; l < o; ++l)
                tree[l] = tree[l] + tree[l + o];
        const float sw = tree[0];
        float *gr = gx + (int64_t)row * C;
#pragma unroll
        for (int j = 0; j < CMAX; ++j)
            if (j < C)
                gr[j] = (e[j] / sw - ((j == lab) ? 1.f : 0.f)) * scale;
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        float s = 0.f;
        for (int i = 0; i < 1024 / 64; ++i)
            s += part[i];
        const float loss = -s / (float)N;
        out2[0] = __float_as_uint(loss);
        out2[1] = bad ? 1u : 0u;
        if (mirror)
            mirror[0] = __float_as_uint(loss), mirror[1] = bad ? 1u : 0u;
    }
}

// gx = (softmax(x) - one_hot(t)) * scale, one wave per row. Rows of up to 64*REGS classes stay in registers
// between the max, the sum and the write, so the logits are read from memory once; longer rows re-read them.
template <int REGS>
__global__ __launch_bounds__(kBlock) void ce_grad_kernel(const float *__restrict__ x, const void *t, int is64, int64_t N,
                                                          int64_t C, float scale_in, const float *__restrict__ gy_dev,
    float *__restrict__ gx)
{
    // the upstream gradient either as a host scalar already divided by N, or still in device memory
    const float scale = gy_dev ? gy_dev[0] / (float)N : scale_in;
    const int64_t row = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (row >= N)
        return;
    const int lane = threadIdx.x & 63;
    const float *xr = x + row * C;
    float *gr = gx + row * C;
    const int64_t lab = label_at(t, is64, row);
    if (REGS > 0)
    {
        float v[REGS > 0 ? REGS : 1];
        float m = -FLT_MAX;
#pragma unroll
        for (int u = 0; u < REGS; ++u)
        {
            const int64_t j = lane + 64 * u;
            v[u] = (j < C) ? xr[j] : -FLT_MAX;
            m = (m < v[u]) ? v[u] : m;
        }
        m = wave_max(m);
        float s = 0.f;
#pragma unroll
        for (int u = 0; u < REGS; ++u)
        {
            const int64_t j = lane + 64 * u;
            v[u] = (j < C) ? expf(v[u] - m) : 0.f;
            s += v[u];
        }
        s = wave_sum(s);
#pragma unroll
        for (int u = 0; u < REGS; ++u)
        {
            const int64_t j = lane + 64 * u;
            if (j < C)
                gr[j] = (v[u] / s - ((j == lab) ? 1.f : 0.f)) * scale;
        }
    }
    else
    {
        float m, s;
        row_stats(xr, C, lane, m, s);
        for (int64_t j = lane; j < C; j += 64)
        {
            const float p = expf(xr[j] - m) / s;
            gr[j] = (p - ((j == lab) ? 1.f : 0.f)) * scale;
        }
    }
}

// Same, for rows whose length is a multiple of 4 and whose base is 16-byte aligned: every lane moves 16 bytes
// per access (QUADS float4 per lane, rows of up to 256*QUADS classes).
template <int QUADS>
__global__ __launch_bounds__(kBlock) void ce_grad_vec_kernel(const float *__restrict__ x, const void *t, int is64,
                                                              int64_t N, int64_t C, float scale_in, const float *__restrict__ gy_dev,
    float *__restrict__ gx)
{
    // the upstream gradient either as a host scalar already divided by N, or still in device memory
    const float scale = gy_dev ? gy_dev[0] / (float)N : scale_in;
    const int64_t row = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (row >= N)
        return;
    const int lane = threadIdx.x & 63;
    const f32x4 *xr = reinterpret_cast<const f32x4 *>(x + row * C);
    f32x4 *gr = reinterpret_cast<f32x4 *>(gx + row * C);
    const int64_t lab = label_at(t, is64, row);
    const int64_t cq = C / 4;
    f32x4 v[QUADS];
    float m = -FLT_MAX;
#pragma unroll
    for (int u = 0; u < QUADS; ++u)
    {
        const int64_t q = lane + 64 * u;
        if (q < cq)
            v[u] = xr[q];
        else
            v[u] = f32x4{-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
#pragma unroll
        for (int e = 0; e < 4; ++e)
            m = (m < v[u][e]) ? v[u][e] : m;
    }
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < QUADS; ++u)
    {
        const bool in = lane + 64 * u < cq;
#pragma unroll
        for (int e = 0; e < 4; ++e)
        {
            v[u][e] = in ? expf(v[u][e] - m) : 0.f;
            s += v[u][e];
        }
    }
    s = wave_sum(s);
#pragma unroll
    for (int u = 0; u < QUADS; ++u)
    {
        const int64_t q = lane + 64 * u;
        if (q < cq)
        {
            f32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                o[e] = (v[u][e] / s - ((4 * q + e == lab) ? 1.f : 0.f)) * scale;
            gr[q] = o;
        }
    }
}

// first maximum of each row (strict >), sequential like src/utils/metrics.cpp:42-53
__global__ void argmax_rows_kernel(const float *__restrict__ y, int64_t N, int64_t C, int64_t *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N)
        return;
    const float *p = y + i * C;
    int64_t mi = 0;
    float mv = p[0];
    for (int64_t j = 1; j < C; ++j)
        if (p[j] > mv)
        {
            mv = p[j];
            mi = j;
        }
    out[i] = mi;
}

// The same answer for wide rows with a wave per row: every lane scans its strided share in ascending order (a NaN is
// never greater than anything, as in the sequential scan), the lanes' (value, index) pairs meet by "greater value, or
// equal value at the smaller index"; a row that starts with a NaN keeps index 0 like the sequential scan, where nothing
// compares greater than it.
template <bool VEC>
__device__ inline int64_t wave_first_argmax(const float *p, int64_t C, int lane)
{
    // (the row's first element decides the NaN case below: its load goes out with the others, not behind the reduction)
    const float first = p[0];
    float mv = 0.f;
    unsigned mi = 0;  // a row has fewer than 2^32 classes: 32-bit positions halve the cross-lane traffic of the reduction
    bool has = false;
    if (VEC)
    {
        // 16 bytes per lane and load, four loads in flight; a lane still meets its elements in ascending order
        const f32x4 *pv = reinterpret_cast<const f32x4 *>(p);
        const unsigned cq = (unsigned)(C / 4);
        for (unsigned q0 = (unsigned)lane; q0 < cq; q0 += 256)
        {
            f32x4 v[4];
#pragma unroll
            for (unsigned u = 0; u < 4; ++u)
                if (q0 + 64 * u < cq)
                    v[u] = pv[q0 + 64 * u];
#pragma unroll
            for (unsigned u = 0; u < 4; ++u)
                if (q0 + 64 * u < cq)
                {
#pragma unroll
                    for (unsigned e = 0; e < 4; ++e)
                        if (v[u][e] == v[u][e] && (!has || v[u][e] > mv))
                            mv = v[u][e], mi = 4 * (q0 + 64 * u) + e, has = true;
                }
        }
    }
    else
    {
        for (unsigned j = (unsigned)lane; j < (unsigned)C; j += 64)
        {
            const float v = p[j];
            if (v == v && (!has || v > mv))
                mv = v, mi = j, has = true;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        const float ov = __shfl_xor(mv, o, 64);
        const unsigned oi = (unsigned)__shfl_xor((int)mi, o, 64);
        const int oh = __shfl_xor((int)has, o, 64);
        if (oh && (!has || ov > mv || (ov == mv && oi < mi)))
            mv = ov, mi = oi, has = true;
    }
    return (has && first == first) ? (int64_t)mi : 0;
}

template <bool VEC>
__global__ void argmax_rows_wave_kernel(const float *__restrict__ y, int64_t N, int64_t C, int64_t *__restrict__ out)
{
    const int64_t row = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (row >= N)
        return;
    const int lane = threadIdx.x & 63;
    const int64_t mi = wave_first_argmax<VEC>(y + row * C, C, lane);
    if (lane == 0)
        out[row] = mi;
}

template <bool VEC>
__global__ void accuracy_count_wave_kernel(const float *__restrict__ y, const int32_t *__restrict__ t, int64_t N, int64_t C,
                                           unsigned int *count)
{
    const int64_t row = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
    if (row >= N)
        return;
    const int lane = threadIdx.x & 63;
    const int64_t mi = wave_first_argmax<VEC>(y + row * C, C, lane);
    const int32_t lab = t[row];
    if (lane == 0 && lab >= 0 && lab < (int32_t)C && (int64_t)lab == mi)
        atomicAdd(count, 1u);
}

__global__ void accuracy_count_kernel(const float *__restrict__ y, const int32_t *__restrict__ t, int64_t N, int64_t C,
                                      unsigned int *count)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N)
        return;
    const float *p = y + i * C;
    int64_t mi = 0;
    float mv = p[0];
    for (int64_t j = 1; j < C; ++j)
        if (p[j] > mv)
        {
            mv = p[j];
            mi = j;
        }
    const int32_t lab = t[i];
    if (lab >= 0 && lab < (int32_t)C && (int64_t)lab == mi)  // metrics.cpp:56-59
        atomicAdd(count, 1u);
}

__global__ void zero_words_kernel(unsigned int *p, int n)
{
    if ((int)threadIdx.x < n)
        p[threadIdx.x] = 0u;
}

inline size_t align256(size_t b)
{
    return (b + 255) & ~(size_t)255;
}
}  // namespace

extern "C" size_t odl_hip_dtype_size(int dtype);

extern "C" {

int odl_hip_softmax(const float *x, int64_t outer, int64_t axis, int64_t inner, float *y, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, "softmax: negative extent");
    if (outer * axis * inner == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    const bool vec = axis % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    const dim3 rows_grid((unsigned)odl::ceil_div(outer, kWaves));
    if (inner == 1 && vec && axis > 64 && axis <= 2048)
    {
        if (axis <= 256)
            hipLaunchKernelGGL(softmax_rows_vec_kernel<1>, rows_grid, dim3(kBlock), 0, st, x, y, outer, axis);
        else if (axis <= 512)
            hipLaunchKernelGGL(softmax_rows_vec_kernel<2>, rows_grid, dim3(kBlock), 0, st, x, y, outer, axis);
        else if (axis <= 1024)
            hipLaunchKernelGGL(softmax_rows_vec_kernel<4>, rows_grid, dim3(kBlock), 0, st, x, y, outer, axis);
        else
            hipLaunchKernelGGL(softmax_rows_vec_kernel<8>, rows_grid, dim3(kBlock), 0, st, x, y, outer, axis);
    }
    else if (inner == 1)
        hipLaunchKernelGGL(softmax_rows_kernel, rows_grid, dim3(kBlock), 0, st, x, y, outer, axis);
    else
        hipLaunchKernelGGL(softmax_strided_kernel, dim3((unsigned)odl::ceil_div(outer * inner, kBlock)), dim3(kBlock), 0,
                           st, x, y, outer, axis, inner);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

// the labels are validated on the host before the launch, so that an out-of-range label can be reported the way the
// reference reports it (gather.cpp:64-67; the CUDA backend does the same D2H copy)
static int gather_check_labels(const void *idx, int idx_is_i64, int64_t N, int64_t C, hipStream_t st)
{
    const size_t esz = idx_is_i64 ? 8 : 4;
    std::vector<char> host((size_t)N * esz);
    ODL_HIP_CHECK(hipMemcpyAsync(host.data(), idx, host.size(), hipMemcpyDeviceToHost, st));
    ODL_HIP_CHECK(hipStreamSynchronize(st));
    for (int64_t i = 0; i < N; ++i)
    {
        const int64_t t = idx_is_i64 ? reinterpret_cast<const int64_t *>(host.data())[i]
                                     : (int64_t) reinterpret_cast<const int32_t *>(host.data())[i];
        if (t < 0 || t >= C)
            return odl::fail(ODL_ERR_INVALID_ARG, "gather: index %lld out of range [0, %lld)", (long long)t,
                             (long long)C);
    }
    return ODL_OK;
}

int odl_hip_gather(const float *in, const void *idx, int idx_is_i64, int64_t N, int64_t C, float *out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && C >= 0, "gather: negative extent");
    if (N == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    const int rc = gather_check_labels(idx, idx_is_i64, N, C, st);
    if (rc != ODL_OK)
        return rc;
    hipLaunchKernelGGL(gather_kernel, dim3((unsigned)odl::ceil_div(N, kBlock)), dim3(kBlock), 0, st, in, idx, idx_is_i64,
                       N, C, out);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_gather_dtype(int dtype, const void *in, const void *idx, int idx_is_i64, int64_t N, int64_t C, void *out, void *stream)
{
    if (dtype == 0)
        return odl_hip_gather(static_cast<const float *>(in), idx, idx_is_i64, N, C, static_cast<float *>(out), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && C >= 0, "gather: negative extent");
    const size_t esz = odl_hip_dtype_size(dtype);
    ODL_REQUIRE(esz > 0, "gather: unknown element type code %d", dtype);
    if (N == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    const int rc = gather_check_labels(idx, idx_is_i64, N, C, st);
    if (rc != ODL_OK)
        return rc;
    const dim3 grid((unsigned)odl::ceil_div(N, kBlock)), block(kBlock);
    if (esz == 8)
        hipLaunchKernelGGL(gather_words_kernel<uint64_t>, grid, block, 0, st, static_cast<const uint64_t *>(in), idx, idx_is_i64, N,
                           C, static_cast<uint64_t *>(out));
    else if (esz == 4)
        hipLaunchKernelGGL(gather_words_kernel<uint32_t>, grid, block, 0, st, static_cast<const uint32_t *>(in), idx, idx_is_i64, N,
                           C, static_cast<uint32_t *>(out));
    else
        hipLaunchKernelGGL(gather_words_kernel<uint8_t>, grid, block, 0, st, static_cast<const uint8_t *>(in), idx, idx_is_i64, N, C,
                           static_cast<uint8_t *>(out));
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_one_hot(const void *idx, int idx_is_i64, int64_t N, int64_t C, float *out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0, "one_hot: negative extent");
    ODL_REQUIRE(C > 0, "one_hot: num_classes must be positive, but got %lld", (long long)C);
    if (N == 0)
        return ODL_OK;
    if (C % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 && N * C < (1ll << 33) && N < (1ll << 31))
    {
        const unsigned quads = (unsigned)(N * C / 4), cq = (unsigned)(C / 4);
        hipLaunchKernelGGL(one_hot_quads_kernel, dim3((unsigned)odl::ceil_div(quads, kBlock)), dim3(kBlock), 0,
                           odl::as_stream(stream), idx, idx_is_i64, quads, cq, odl::make_fastdiv(cq), out);
    }
    else
        hipLaunchKernelGGL(one_hot_kernel, dim3((unsigned)odl::ceil_div(N * C, kBlock)), dim3(kBlock), 0,
                           odl::as_stream(stream), idx, idx_is_i64, N, C, out);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

size_t odl_hip_softmax_ce_loss_workspace_bytes(int64_t N)
{
    return align256((size_t)(N > 0 ? N : 0) * sizeof(float)) + 256;
}

// loss and out-of-range flag into two device words: [0] loss (float), [1] flag (int, nonzero = a bad label)
static int ce_loss_launch(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C, unsigned int *out2,
                          unsigned int *mirror, void *workspace, size_t workspace_bytes, hipStream_t st,
                          float *unit_gx = nullptr)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N > 0 && C > 0, "softmax_cross_entropy: empty input");
    const size_t need = odl_hip_softmax_ce_loss_workspace_bytes(N);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need,
                "softmax_cross_entropy: workspace of %zu bytes required, got %zu", need, workspace_bytes);
    if (N <= 2048 && C <= 64 && unit_gx)
    {
        const float scale = 1.0f / (float)N;  // an upstream gradient of 1 over N, as ce_grad_launch forms it
        if (C <= 16)
            hipLaunchKernelGGL(ce_loss_grad_small_kernel<16>, dim3(1), dim3(1024), 0, st, x, t, idx_is_i64, (int)N, (int)C, out2,
                               mirror, unit_gx, scale);
        else if (C <= 32)
            hipLaunchKernelGGL(ce_loss_grad_small_kernel<32>, dim3(1), dim3(1024), 0, st, x, t, idx_is_i64, (int)N, (int)C, out2,
                               mirror, unit_gx, scale);
        else
            hipLaunchKernelGGL(ce_loss_grad_small_kernel<64>, dim3(1), dim3(1024), 0, st, x, t, idx_is_i64, (int)N, (int)C, out2,
                               mirror, unit_gx, scale);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    }
    ODL_REQUIRE(unit_gx == nullptr, "softmax_cross_entropy: no one-launch loss and gradient for %lld rows of %lld classes",
                (long long)N, (long long)C);
    if (N <= 2048 && C <= 64)
    {
        hipLaunchKernelGGL(ce_loss_small_kernel, dim3(1), dim3(1024), 0, st, x, t, idx_is_i64, (int)N, (int)C, out2,
                           mirror);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    }
    float *logp = static_cast<float *>(workspace);
    hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, st, out2, 2);
    ODL_LAUNCH_CHECK();
    const dim3 rows_grid((unsigned)odl::ceil_div(N, kWaves));
    int *flag = reinterpret_cast<int *>(out2 + 1);
    if (C % 4 == 0 && C > 64 && C <= 2048 && (reinterpret_cast<uintptr_t>(x) & 15) == 0)
    {
        if (C <= 256)
            hipLaunchKernelGGL(ce_row_logp_vec_kernel<1>, rows_grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, logp, flag);
        else if (C <= 512)
            hipLaunchKernelGGL(ce_row_logp_vec_kernel<2>, rows_grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, logp, flag);
        else if (C <= 1024)
            hipLaunchKernelGGL(ce_row_logp_vec_kernel<4>, rows_grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, logp, flag);
        else
            hipLaunchKernelGGL(ce_row_logp_vec_kernel<8>, rows_grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, logp, flag);
    }
    else
        hipLaunchKernelGGL(ce_row_logp_kernel, rows_grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, logp, flag);
    ODL_LAUNCH_CHECK();
    hipLaunchKernelGGL(ce_finish_kernel, dim3(1), dim3(1024), 0, st, logp, N, reinterpret_cast<float *>(out2),
                       mirror);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_softmax_ce_loss_device(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C,
                                   float *device_loss2, void *host_mirror2, void *workspace, size_t workspace_bytes,
                                   void *stream)
{
    ODL_REQUIRE(device_loss2 != nullptr, "softmax_cross_entropy: null output");
    return ce_loss_launch(x, t, idx_is_i64, N, C, reinterpret_cast<unsigned int *>(device_loss2),
                          static_cast<unsigned int *>(host_mirror2), workspace,
                          workspace_bytes, odl::as_stream(stream));
}

int odl_hip_softmax_ce_loss_grad_ok(int64_t N, int64_t C)
{
    return (N > 0 && N <= 2048 && C > 0 && C <= 64) ? 1 : 0;
}

int odl_hip_softmax_ce_loss_grad_device(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C,
                                        float *device_loss2, void *host_mirror2, float *unit_gx, void *workspace,
                                        size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE(device_loss2 != nullptr && unit_gx != nullptr, "softmax_cross_entropy: null output");
    return ce_loss_launch(x, t, idx_is_i64, N, C, reinterpret_cast<unsigned int *>(device_loss2),
                          static_cast<unsigned int *>(host_mirror2), workspace, workspace_bytes, odl::as_stream(stream), unit_gx);
}

int odl_hip_softmax_ce_loss(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C, float *host_loss,
                            void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE(host_loss != nullptr, "softmax_cross_entropy: null output");
    hipStream_t st = odl::as_stream(stream);
    const size_t need = odl_hip_softmax_ce_loss_workspace_bytes(N > 0 ? N : 1);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need,
                "softmax_cross_entropy: workspace of %zu bytes required, got %zu", need, workspace_bytes);
    // tail of the workspace: [0] loss (float), [1] out-of-range flag (int)
    unsigned int *tail = reinterpret_cast<unsigned int *>(static_cast<char *>(workspace) + need - 256);
    const int rc = ce_loss_launch(x, t, idx_is_i64, N, C, tail, nullptr, workspace, workspace_bytes, st);
    if (rc != ODL_OK)
        return rc;
    unsigned int host_tail[2] = {0, 0};
    ODL_HIP_CHECK(hipMemcpyAsync(host_tail, tail, sizeof(host_tail), hipMemcpyDeviceToHost, st));
    ODL_HIP_CHECK(hipStreamSynchronize(st));
    if (host_tail[1] != 0)
        return odl::fail(ODL_ERR_INVALID_ARG, "gather: index out of range [0, %lld)", (long long)C);
    float loss;
    __builtin_memcpy(&loss, &host_tail[0], sizeof(float));
    *host_loss = loss;
    return ODL_OK;
}

static int ce_grad_launch(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C, float gy,
                          const float *gy_dev, float *gx, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N > 0 && C > 0, "softmax_cross_entropy backward: empty input");
    const float scale = gy / (float)N;  // softmax_cross_entropy.cpp:105-106
    const dim3 grid((unsigned)odl::ceil_div(N, kWaves));
    hipStream_t st = odl::as_stream(stream);
    const bool vec = C % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gx)) & 15) == 0;
    if (vec && C > 64 && C <= 1024)
    {
        if (C <= 256)
            hipLaunchKernelGGL(ce_grad_vec_kernel<1>, grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, scale, gy_dev, gx);
        else if (C <= 512)
            hipLaunchKernelGGL(ce_grad_vec_kernel<2>, grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, scale, gy_dev, gx);
        else
            hipLaunchKernelGGL(ce_grad_vec_kernel<4>, grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, scale, gy_dev, gx);
    }
    else if (C <= 64)
        hipLaunchKernelGGL(ce_grad_kernel<1>, grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, scale, gy_dev, gx);
    else if (C <= 256)
        hipLaunchKernelGGL(ce_grad_kernel<4>, grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, scale, gy_dev, gx);
    else if (C <= 1024)
        hipLaunchKernelGGL(ce_grad_kernel<16>, grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, scale, gy_dev, gx);
    else
        hipLaunchKernelGGL(ce_grad_kernel<0>, grid, dim3(kBlock), 0, st, x, t, idx_is_i64, N, C, scale, gy_dev, gx);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_softmax_ce_grad(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C, float gy, float *gx,
                            void *stream)
{
    return ce_grad_launch(x, t, idx_is_i64, N, C, gy, nullptr, gx, stream);
}

int odl_hip_softmax_ce_grad_device(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C,
                                   const float *device_gy, float *gx, void *stream)
{
    ODL_REQUIRE(device_gy != nullptr, "softmax_cross_entropy backward: null upstream gradient");
    return ce_grad_launch(x, t, idx_is_i64, N, C, 0.0f, device_gy, gx, stream);
}

int odl_hip_argmax_rows(const float *y, int64_t N, int64_t C, int64_t *out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && C > 0, "argmax: bad shape");
    if (N == 0)
        return ODL_OK;
    const bool vec = C % 4 == 0 && C >= 256 && C < (1ll << 31) && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    if (vec)
        hipLaunchKernelGGL(argmax_rows_wave_kernel<true>, dim3((unsigned)odl::ceil_div(N, kWaves)), dim3(kBlock), 0,
                           odl::as_stream(stream), y, N, C, out);
    else if (C >= 32 && C < (1ll << 31))  // a wave per row once a row is worth 64 lanes; a thread per row for a handful of classes
        hipLaunchKernelGGL(argmax_rows_wave_kernel<false>, dim3((unsigned)odl::ceil_div(N, kWaves)), dim3(kBlock), 0,
                           odl::as_stream(stream), y, N, C, out);
    else
        hipLaunchKernelGGL(argmax_rows_kernel, dim3((unsigned)odl::ceil_div(N, kBlock)), dim3(kBlock), 0,
                           odl::as_stream(stream), y, N, C, out);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

size_t odl_hip_accuracy_workspace_bytes(int64_t)
{
    return 256;
}

int odl_hip_accuracy(const float *y, const int32_t *t, int64_t N, int64_t C, float *host_acc, void *workspace,
                     size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N > 0 && C > 0, "accuracy: empty input");
    ODL_REQUIRE(host_acc != nullptr, "accuracy: null output");
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= 256, "accuracy: workspace of 256 bytes required");
    hipStream_t st = odl::as_stream(stream);
    unsigned int *count = static_cast<unsigned int *>(workspace);
    hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(64), 0, st, count, 1);
    ODL_LAUNCH_CHECK();
    if (C % 4 == 0 && C >= 256 && C < (1ll << 31) && (reinterpret_cast<uintptr_t>(y) & 15) == 0)
        hipLaunchKernelGGL(accuracy_count_wave_kernel<true>, dim3((unsigned)odl::ceil_div(N, kWaves)), dim3(kBlock), 0, st, y,
                           t, N, C, count);
    else if (C >= 32 && C < (1ll << 31))
        hipLaunchKernelGGL(accuracy_count_wave_kernel<false>, dim3((unsigned)odl::ceil_div(N, kWaves)), dim3(kBlock), 0, st, y,
                           t, N, C, count);
    else
        hipLaunchKernelGGL(accuracy_count_kernel, dim3((unsigned)odl::ceil_div(N, kBlock)), dim3(kBlock), 0, st, y, t, N, C,
                           count);
    ODL_LAUNCH_CHECK();
    unsigned int host_count = 0;
    ODL_HIP_CHECK(hipMemcpyAsync(&host_count, count, sizeof(host_count), hipMemcpyDeviceToHost, st));
    ODL_HIP_CHECK(hipStreamSynchronize(st));
    *host_acc = (float)host_count / (float)N;  // metrics.cpp:64
    return ODL_OK;
}

}  // extern "C"
