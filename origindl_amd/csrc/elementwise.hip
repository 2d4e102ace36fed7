// Elementwise plumbing between the hot kernels: add/sub/mul/div (same shape or single-element broadcast, the
// only cases the reference supports, src/mat/origin/cpu/math/add.cpp:56-93), the > mask, relu/exp/log/neg/
// square/sqrt, pow with a scalar exponent, and fills. 16 bytes per lane when the buffers allow it.
// Built with floating-point contraction off: every arithmetic step rounds like the reference's separate ops.
#include "odl_common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace
{
constexpr int kBlock = 256;

template <int OP>
__device__ inline float bin(float a, float b)
{
    if (OP == 0) return a + b;
    if (OP == 1) return a - b;
    if (OP == 2) return a * b;
    if (OP == 3) return a / b;
    // comparisons give a 0/1 mask in the operands' own type (operation_templates.h:177-240)
    if (OP == 4) return (a > b) ? 1.f : 0.f;
    if (OP == 5) return (a == b) ? 1.f : 0.f;
    if (OP == 6) return (a != b) ? 1.f : 0.f;
    if (OP == 7) return (a < b) ? 1.f : 0.f;
    if (OP == 8) return (a <= b) ? 1.f : 0.f;
    if (OP == 9) return (a >= b) ? 1.f : 0.f;
    // backward halves of the activations, a = upstream gradient:
    if (OP == 10)  // sigmoid: b = y = sigmoid(x); gy*y*(1-y) (cpu/activation/sigmoid.cpp:93)
    {
        const float t = a * b;
        return t * (1.0f - b);
    }
    if (OP == 12)  // relu: b = x; gy * (x > 0 ? 1 : 0), a product as in the reference (relu.cpp:23-29, 45-52)
        return a * ((b > 0.f) ? 1.f : 0.f);
    // silu: b = x; gy*(s + x*s*(1-s)) with s = sigmoid(x) (cpu/activation/silu.cpp:87-90)
    const float sg = 1.0f / (1.0f + expf(-b));
    const float xs = b * sg;
    const float g = sg + xs * (1.0f - sg);
    return a * g;
}

template <int OP>
__device__ inline float un(float v)
{
    if (OP == 0) return v > 0.f ? v : 0.f;
    if (OP == 1) return expf(v);
    if (OP == 2) return logf(v);
    if (OP == 3) return -v;
    if (OP == 4) return v * v;
    if (OP == 5) return sqrtf(v);
    // sigmoid as 1/(1+exp(-x)) (operation_templates.h:168-175) and silu as x times that (cpu/activation/silu.cpp:49-56)
    const float s = 1.0f / (1.0f + expf(-v));
    return OP == 6 ? s : v * s;
}

// MODE 0: a[i] op b[i]; 1: a[i] op b[0]; 2: a[0] op b[i]. Each thread handles 4 consecutive elements.
template <int OP, int MODE, bool VEC>
__global__ void binary_kernel(const float *a, const float *b, float *out, int64_t n)
{
    const int64_t i0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i0 >= n)
        return;
    float av[4], bv[4], ov[4];
    const bool full = VEC && (i0 + 4 <= n);
    if (full)
    {
        if (MODE != 2)
        {
            const f32x4 q = *reinterpret_cast<const f32x4 *>(a + i0);
            av[0] = q[0], av[1] = q[1], av[2] = q[2], av[3] = q[3];
        }
        if (MODE != 1)
        {
            const f32x4 q = *reinterpret_cast<const f32x4 *>(b + i0);
            bv[0] = q[0], bv[1] = q[1], bv[2] = q[2], bv[3] = q[3];
        }
    }
    else
    {
        for (int e = 0; e < 4; ++e)
        {
            const bool in = i0 + e < n;
            if (MODE != 2)
                av[e] = in ? a[i0 + e] : 0.f;
            if (MODE != 1)
                bv[e] = in ? b[i0 + e] : 1.f;
        }
    }
    if (MODE == 1)
        bv[0] = bv[1] = bv[2] = bv[3] = b[0];
    if (MODE == 2)
        av[0] = av[1] = av[2] = av[3] = a[0];
#pragma unroll
    for (int e = 0; e < 4; ++e)
        ov[e] = bin<OP>(av[e], bv[e]);
    if (full)
    {
        f32x4 q = {ov[0], ov[1], ov[2], ov[3]};
        *reinterpret_cast<f32x4 *>(out + i0) = q;
    }
    else
        for (int e = 0; e < 4 && i0 + e < n; ++e)
            out[i0 + e] = ov[e];
}

// 16 bytes per lane when the buffers are 16-byte aligned; the tail and unaligned buffers go one float at a time
template <int OP, bool VEC>
__global__ void unary_kernel(const float *a, float *out, int64_t n)
{
    if (VEC)
    {
        const int64_t i0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
        if (i0 + 4 <= n)
        {
            const f32x4 q = *reinterpret_cast<const f32x4 *>(a + i0);
            f32x4 r = {un<OP>(q[0]), un<OP>(q[1]), un<OP>(q[2]), un<OP>(q[3])};
            *reinterpret_cast<f32x4 *>(out + i0) = r;
        }
        else
            for (int64_t i = i0; i < n; ++i)
                out[i] = un<OP>(a[i]);
    }
    else
    {
        const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (i < n)
            out[i] = un<OP>(a[i]);
    }
}

__global__ void pow_kernel(const float *a, float *out, int64_t n, float e)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        out[i] = powf(a[i], e);
}

// One Adam step per element, as the same sequence of separately rounded float operations that the reference's
// optimizer issues as whole-tensor ops (src/optim/adam.cpp:52-113): this file is compiled without contraction,
// so m*b1 + g*(1-b1) is two products and a sum, and the square root is powf(v_hat, 0.5f) as there.
struct AdamScalars
{
    float beta1, one_minus_beta1, beta2, one_minus_beta2, m_hat_scale, v_hat_scale, eps, lr;
    float root;  // 0.5, passed at run time so that the call stays the powf the unfused pow kernel makes
};

__device__ inline void adam_one(float p, float g, float &m, float &v, float &p_out, const AdamScalars &a)
{
    const float mn = m * a.beta1 + g * a.one_minus_beta1;
    const float gg = g * g;
    const float vn = v * a.beta2 + gg * a.one_minus_beta2;
    const float m_hat = mn * a.m_hat_scale;
    const float v_hat = vn * a.v_hat_scale;
    const float denom = powf(v_hat, a.root) + a.eps;
    const float update = m_hat / denom;
    p_out = p - update * a.lr;
    m = mn, v = vn;
}

// `scales` (optional): the two bias-correction factors in device memory, for a step recorded once and replayed with
// a different step count each time
template <bool VEC>
__global__ void adam_step_kernel(const float *p, const float *g, float *m, float *v, float *p_out, int64_t n, AdamScalars a,
                                 const float *__restrict__ scales)
{
    if (scales)
        a.m_hat_scale = scales[0], a.v_hat_scale = scales[1];
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (VEC)
    {
        const int64_t i = 4 * t;
        if (i + 3 < n)
        {
            f32x4 pv = *reinterpret_cast<const f32x4 *>(p + i), gv = *reinterpret_cast<const f32x4 *>(g + i);
            f32x4 mv = *reinterpret_cast<f32x4 *>(m + i), vv = *reinterpret_cast<f32x4 *>(v + i), ov;
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                float mj = mv[j], vj = vv[j], oj;
                adam_one(pv[j], gv[j], mj, vj, oj, a);
                mv[j] = mj, vv[j] = vj, ov[j] = oj;
            }
            *reinterpret_cast<f32x4 *>(m + i) = mv;
            *reinterpret_cast<f32x4 *>(v + i) = vv;
            *reinterpret_cast<f32x4 *>(p_out + i) = ov;
        }
        else
            for (int64_t k = i; k < n; ++k)
                adam_one(p[k], g[k], m[k], v[k], p_out[k], a);
    }
    else if (t < n)
        adam_one(p[t], g[t], m[t], v[t], p_out[t], a);
}

// p_out = p - g * lr, two separately rounded steps (src/optim/sgd.cpp:18-75 without momentum or weight decay)
__global__ void sgd_step_kernel(const float *p, const float *g, float *p_out, int64_t n, float lr)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
    {
        const float step = g[i] * lr;
        p_out[i] = p[i] - step;
    }
}

// ---- one launch over several tensors (all the parameters of a model): the launch count of an optimizer step stops
// growing with the number of parameters, most of which are biases of a few hundred floats
constexpr int kMultiMax = 24;                   // tensors per launch; longer lists go out in several launches
constexpr int kMultiChunk = kBlock * 4;         // elements per workgroup
struct MultiArgs
{
    const float *a[kMultiMax];      // adam, sgd: parameter; axpy: x
    const float *b[kMultiMax];      // adam, sgd: gradient
    float *m[kMultiMax];            // adam: first moment
    float *v[kMultiMax];            // adam: second moment
    float *out[kMultiMax];          // adam, sgd: updated parameter; axpy: y (updated in place)
    const float *scales[kMultiMax]; // adam: the two bias-correction factors in device memory, or null
    float m_hat_scale[kMultiMax], v_hat_scale[kMultiMax];
    int64_t n[kMultiMax];
    unsigned first_block[kMultiMax + 1];  // workgroups [first_block[t], first_block[t+1]) belong to tensor t
    int count;
};

// OP 0: Adam step, 1: SGD step, 2: out += alpha * a — per element the same float operations as the one-tensor kernels.
// OP 3 / 4: the Adam / SGD step with the WeightDecay hook in front of it in the same pass: g += alpha * p (the product
// rounded, then the sum: what OP 2 does) is written back to g, and the step uses that g.
template <int OPX>
__global__ __launch_bounds__(kBlock) void multi_tensor_kernel(MultiArgs q, AdamScalars s, float alpha)
{
    constexpr bool DECAY = OPX >= 3;
    constexpr int OP = OPX == 3 ? 0 : (OPX == 4 ? 1 : OPX);
    int t = 0;
    while (t + 1 < q.count && blockIdx.x >= q.first_block[t + 1])  // the same in every lane
        ++t;
    const int64_t n = q.n[t];
    const int64_t i = ((int64_t)(blockIdx.x - q.first_block[t]) * kBlock + threadIdx.x) * 4;
    if (i >= n)
        return;
    const float *a = q.a[t], *b = q.b[t];
    float *m = q.m[t], *v = q.v[t], *out = q.out[t];
    if (OP == 0)
    {
        s.m_hat_scale = q.m_hat_scale[t], s.v_hat_scale = q.v_hat_scale[t];
        if (q.scales[t])
            s.m_hat_scale = q.scales[t][0], s.v_hat_scale = q.scales[t][1];
    }
    auto aligned = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    const bool vec = i + 3 < n && aligned(a) && aligned(out) && (OP == 2 || aligned(b)) && (OP != 0 || (aligned(m) && aligned(v)));
    if (vec)
    {
        const f32x4 av = *reinterpret_cast<const f32x4 *>(a + i);
        f32x4 ov;
        if (OP == 0)
        {
            f32x4 gv = *reinterpret_cast<const f32x4 *>(b + i);
            if (DECAY)
            {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    const float step = alpha * av[j];
                    gv[j] = gv[j] + step;
                }
                *reinterpret_cast<f32x4 *>(const_cast<float *>(b) + i) = gv;
            }
            f32x4 mv = *reinterpret_cast<f32x4 *>(m + i), vv = *reinterpret_cast<f32x4 *>(v + i);
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                float mj = mv[j], vj = vv[j], oj;
                adam_one(av[j], gv[j], mj, vj, oj, s);
                mv[j] = mj, vv[j] = vj, ov[j] = oj;
            }
            *reinterpret_cast<f32x4 *>(m + i) = mv;
            *reinterpret_cast<f32x4 *>(v + i) = vv;
        }
        else if (OP == 1)
        {
            f32x4 gv = *reinterpret_cast<const f32x4 *>(b + i);
            if (DECAY)
            {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    const float step = alpha * av[j];
                    gv[j] = gv[j] + step;
                }
                *reinterpret_cast<f32x4 *>(const_cast<float *>(b) + i) = gv;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                const float step = gv[j] * s.lr;
                ov[j] = av[j] - step;
            }
        }
        else
        {
            const f32x4 yv = *reinterpret_cast<const f32x4 *>(out + i);
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                const float step = alpha * av[j];
                ov[j] = yv[j] + step;
            }
        }
        *reinterpret_cast<f32x4 *>(out + i) = ov;
        return;
    }
    for (int64_t k = i; k < n && k < i + 4; ++k)
    {
        float gk = OP == 2 ? 0.f : b[k];
        if (DECAY)
        {
            const float step = alpha * a[k];
            gk = gk + step;
            const_cast<float *>(b)[k] = gk;
        }
        if (OP == 0)
            adam_one(a[k], gk, m[k], v[k], out[k], s);
        else if (OP == 1)
        {
            const float step = gk * s.lr;
            out[k] = a[k] - step;
        }
        else
        {
            const float step = alpha * a[k];
            out[k] = out[k] + step;
        }
    }
}

__global__ void fill_kernel(float *dst, int64_t n, float v)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        dst[i] = v;
}

__global__ void fill_bytes_kernel(unsigned char *dst, size_t n, unsigned char v)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        dst[i] = v;
}

template <int OP>
int launch_binary(const float *a, int64_t na, const float *b, int64_t nb, float *out, hipStream_t st)
{
    const int64_t n = na > nb ? na : nb;
    const int mode = (na == nb) ? 0 : (nb == 1 ? 1 : 2);
    auto aligned = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool vec = aligned(out) && (mode == 2 || aligned(a)) && (mode == 1 || aligned(b));
    const dim3 grid((unsigned)odl::ceil_div(odl::ceil_div(n, 4), kBlock));
#define ODL_BIN_CASE(M, V)                                                                          \
    if (mode == M && vec == V)                                                                      \
        hipLaunchKernelGGL((binary_kernel<OP, M, V>), grid, dim3(kBlock), 0, st, a, b, out, n);
    ODL_BIN_CASE(0, true)
    ODL_BIN_CASE(0, false)
    ODL_BIN_CASE(1, true)
    ODL_BIN_CASE(1, false)
    ODL_BIN_CASE(2, true)
    ODL_BIN_CASE(2, false)
#undef ODL_BIN_CASE
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
}  // namespace

namespace odl
{
int fill_launch(float *dst, int64_t n, float value, hipStream_t st)
{
    if (n <= 0)
        return ODL_OK;
    hipLaunchKernelGGL(fill_kernel, dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, st, dst, n, value);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

// byte fill as a kernel: a memset node inside a captured graph is avoided on purpose
int fill_bytes_launch(void *dst, int value, size_t bytes, hipStream_t st)
{
    if (bytes == 0)
        return ODL_OK;
    const unsigned char b = (unsigned char)value;
    if (reinterpret_cast<uintptr_t>(dst) % 4 == 0 && bytes % 4 == 0)
    {
        const unsigned int w = b * 0x01010101u;
        float f;
        __builtin_memcpy(&f, &w, 4);
        return fill_launch(static_cast<float *>(dst), (int64_t)(bytes / 4), f, st);
    }
    hipLaunchKernelGGL(fill_bytes_kernel, dim3((unsigned)ceil_div((int64_t)bytes, kBlock)), dim3(kBlock), 0, st,
                       static_cast<unsigned char *>(dst), bytes, b);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}
// the list goes out kMultiMax tensors at a time; empty tensors are skipped
template <int OPX>
int multi_launch(const char *what, int count, const float *const *a, const float *const *b, float *const *m,
                        float *const *v, float *const *out, const float *const *scales, const float *m_hat,
                        const float *v_hat, const int64_t *n, const AdamScalars &s, float alpha, void *stream)
{
    constexpr int OP = OPX == 3 ? 0 : (OPX == 4 ? 1 : OPX);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(count >= 0, "%s: negative count", what);
    if (count == 0)
        return ODL_OK;
    ODL_REQUIRE(a && out && n && (OP == 2 || b) && (OP != 0 || (m && v && (scales || (m_hat && v_hat)))),
                "%s: null argument list", what);
    MultiArgs q;
    int used = 0;
    uint64_t blocks = 0;
    auto flush = [&]() -> int {
        if (used == 0)
            return ODL_OK;
        q.count = used;
        q.first_block[used] = (unsigned)blocks;
        hipLaunchKernelGGL((multi_tensor_kernel<OPX>), dim3((unsigned)blocks), dim3(kBlock), 0, odl::as_stream(stream), q, s,
                           alpha);
        ODL_LAUNCH_CHECK();
        used = 0, blocks = 0;
        return ODL_OK;
    };
    for (int i = 0; i < count; ++i)
    {
        ODL_REQUIRE(n[i] >= 0, "%s: tensor %d has a negative size", what, i);
        if (n[i] == 0)
            continue;
        ODL_REQUIRE(a[i] && out[i] && (OP == 2 || b[i]) && (OP != 0 || (m[i] && v[i])), "%s: tensor %d has a null operand",
                    what, i);
        const uint64_t nb = (uint64_t)odl::ceil_div(n[i], kMultiChunk);
        ODL_REQUIRE(nb < (1ull << 31), "%s: tensor %d is too large", what, i);
        if (used == kMultiMax || blocks + nb >= (1ull << 31))
        {
            const int rc = flush();
            if (rc != ODL_OK)
                return rc;
        }
        q.a[used] = a[i], q.b[used] = b ? b[i] : nullptr, q.m[used] = m ? m[i] : nullptr, q.v[used] = v ? v[i] : nullptr;
        q.out[used] = out[i], q.scales[used] = scales ? scales[i] : nullptr;
        q.m_hat_scale[used] = m_hat ? m_hat[i] : 0.0f, q.v_hat_scale[used] = v_hat ? v_hat[i] : 0.0f;
        ODL_REQUIRE(OP != 0 || q.scales[used] || (m_hat && v_hat), "%s: tensor %d has no bias-correction factors", what, i);
        q.n[used] = n[i];
        q.first_block[used] = (unsigned)blocks;
        blocks += nb;
        ++used;
    }
    return flush();
}

}  // namespace odl

extern "C" {

int odl_hip_binary(int op, const float *a, int64_t na, const float *b, int64_t nb, float *out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(op >= 0 && op <= 12, "binary: unknown op %d", op);
    ODL_REQUIRE(na >= 0 && nb >= 0, "binary: negative extent");
    if (!(na == nb || na == 1 || nb == 1))
        return odl::fail(ODL_ERR_RUNTIME, "Complex broadcasting not yet implemented (%lld vs %lld elements)",
                         (long long)na, (long long)nb);
    if (na == 0 || nb == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    switch (op)
    {
        case 0: return launch_binary<0>(a, na, b, nb, out, st);
        case 1: return launch_binary<1>(a, na, b, nb, out, st);
        case 2: return launch_binary<2>(a, na, b, nb, out, st);
        case 3: return launch_binary<3>(a, na, b, nb, out, st);
        case 4: return launch_binary<4>(a, na, b, nb, out, st);
        case 5: return launch_binary<5>(a, na, b, nb, out, st);
        case 6: return launch_binary<6>(a, na, b, nb, out, st);
        case 7: return launch_binary<7>(a, na, b, nb, out, st);
        case 8: return launch_binary<8>(a, na, b, nb, out, st);
        case 9: return launch_binary<9>(a, na, b, nb, out, st);
        case 10: return launch_binary<10>(a, na, b, nb, out, st);
        case 11: return launch_binary<11>(a, na, b, nb, out, st);
        default: return launch_binary<12>(a, na, b, nb, out, st);
    }
}

int odl_hip_unary(int op, const float *a, int64_t n, float *out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(op >= 0 && op <= 7, "unary: unknown op %d", op);
    if (n <= 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    const bool vec = (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(out)) % 16 == 0;
    const dim3 grid((unsigned)odl::ceil_div(vec ? odl::ceil_div(n, 4) : n, kBlock));
#define ODL_UN_CASE(OP)                                                                          \
    case OP:                                                                                     \
        if (vec)                                                                                 \
            hipLaunchKernelGGL((unary_kernel<OP, true>), grid, dim3(kBlock), 0, st, a, out, n);  \
        else                                                                                     \
            hipLaunchKernelGGL((unary_kernel<OP, false>), grid, dim3(kBlock), 0, st, a, out, n); \
        break;
    switch (op)
    {
        ODL_UN_CASE(0)
        ODL_UN_CASE(1)
        ODL_UN_CASE(2)
        ODL_UN_CASE(3)
        ODL_UN_CASE(4)
        ODL_UN_CASE(5)
        ODL_UN_CASE(6)
        default:
        ODL_UN_CASE(7)
    }
#undef ODL_UN_CASE
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_pow_scalar(const float *a, int64_t n, float exponent, float *out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    if (n <= 0)
        return ODL_OK;
    hipLaunchKernelGGL(pow_kernel, dim3((unsigned)odl::ceil_div(n, kBlock)), dim3(kBlock), 0, odl::as_stream(stream), a,
                       out, n, exponent);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

static int adam_launch(const float *p, const float *g, float *m, float *v, int64_t n, float beta1, float beta2,
                       float m_hat_scale, float v_hat_scale, const float *scales, float eps, float lr, float *p_out,
                       void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(n >= 0, "adam_step: negative size");
    if (n == 0)
        return ODL_OK;
    ODL_REQUIRE(p && g && m && v && p_out, "adam_step: null operand");
    const AdamScalars a{beta1, 1.0f - beta1, beta2, 1.0f - beta2, m_hat_scale, v_hat_scale, eps, lr, 0.5f};
    auto aligned = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
    hipStream_t st = odl::as_stream(stream);
    if (aligned(p) && aligned(g) && aligned(m) && aligned(v) && aligned(p_out))
        hipLaunchKernelGGL((adam_step_kernel<true>), dim3((unsigned)odl::ceil_div(odl::ceil_div(n, 4), kBlock)),
                           dim3(kBlock), 0, st, p, g, m, v, p_out, n, a, scales);
    else
        hipLaunchKernelGGL((adam_step_kernel<false>), dim3((unsigned)odl::ceil_div(n, kBlock)), dim3(kBlock), 0, st, p, g,
                           m, v, p_out, n, a, scales);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_adam_step(const float *p, const float *g, float *m, float *v, int64_t n, float beta1, float beta2,
                      float m_hat_scale, float v_hat_scale, float eps, float lr, float *p_out, void *stream)
{
    return adam_launch(p, g, m, v, n, beta1, beta2, m_hat_scale, v_hat_scale, nullptr, eps, lr, p_out, stream);
}

int odl_hip_adam_step_device_scales(const float *p, const float *g, float *m, float *v, int64_t n, float beta1,
                                    float beta2, const float *device_scales, float eps, float lr, float *p_out,
                                    void *stream)
{
    ODL_REQUIRE(device_scales != nullptr, "adam_step: null scales");
    return adam_launch(p, g, m, v, n, beta1, beta2, 0.0f, 0.0f, device_scales, eps, lr, p_out, stream);
}

int odl_hip_adam_step_multi(int count, const float *const *p, const float *const *g, float *const *m, float *const *v,
                            const int64_t *n, float beta1, float beta2, const float *m_hat_scale, const float *v_hat_scale,
                            const float *const *device_scales, float eps, float lr, float *const *p_out, void *stream)
{
    const AdamScalars s{beta1, 1.0f - beta1, beta2, 1.0f - beta2, 0.0f, 0.0f, eps, lr, 0.5f};
    return odl::multi_launch<0>("adam_step_multi", count, p, g, m, v, p_out, device_scales, m_hat_scale, v_hat_scale, n, s, 0.0f,
                           stream);
}

int odl_hip_sgd_step_multi(int count, const float *const *p, const float *const *g, const int64_t *n, float lr,
                           float *const *p_out, void *stream)
{
    const AdamScalars s{0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, lr, 0.5f};
    return odl::multi_launch<1>("sgd_step_multi", count, p, g, nullptr, nullptr, p_out, nullptr, nullptr, nullptr, n, s, 0.0f,
                           stream);
}

int odl_hip_adam_step_multi_decay(int count, const float *const *p, float *const *g, float *const *m, float *const *v,
                                  const int64_t *n, float weight_decay, float beta1, float beta2, const float *m_hat_scale,
                                  const float *v_hat_scale, const float *const *device_scales, float eps, float lr,
                                  float *const *p_out, void *stream)
{
    const AdamScalars s{beta1, 1.0f - beta1, beta2, 1.0f - beta2, 0.0f, 0.0f, eps, lr, 0.5f};
    return odl::multi_launch<3>("adam_step_multi_decay", count, p, g, m, v, p_out, device_scales, m_hat_scale, v_hat_scale, n,
                                s, weight_decay, stream);
}

int odl_hip_sgd_step_multi_decay(int count, const float *const *p, float *const *g, const int64_t *n, float weight_decay,
                                 float lr, float *const *p_out, void *stream)
{
    const AdamScalars s{0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, lr, 0.5f};
    return odl::multi_launch<4>("sgd_step_multi_decay", count, p, g, nullptr, nullptr, p_out, nullptr, nullptr, nullptr, n, s,
                                weight_decay, stream);
}

int odl_hip_axpy_multi(int count, float alpha, const float *const *x, float *const *y, const int64_t *n, void *stream)
{
    const AdamScalars s{};
    return odl::multi_launch<2>("axpy_multi", count, x, nullptr, nullptr, nullptr, y, nullptr, nullptr, nullptr, n, s, alpha,
                           stream);
}

int odl_hip_sgd_step(const float *p, const float *g, int64_t n, float lr, float *p_out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(n >= 0, "sgd_step: negative size");
    if (n == 0)
        return ODL_OK;
    ODL_REQUIRE(p && g && p_out, "sgd_step: null operand");
    hipLaunchKernelGGL(sgd_step_kernel, dim3((unsigned)odl::ceil_div(n, kBlock)), dim3(kBlock), 0, odl::as_stream(stream),
                       p, g, p_out, n, lr);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_fill(float *dst, int64_t n, float value, void *stream)
{
    ODL_REQUIRE_DEVICE();
    return odl::fill_launch(dst, n, value, odl::as_stream(stream));
}

}  // extern "C"
