// Shared helpers of the gfx950 backend: status codes, thread-local error text, launch checks.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/odl_hip.h"

namespace odl
{
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);
// true when the current device is a gfx950 part; the kernels in this library are built for nothing else
int require_device();

// Compute units and XCDs (one L2 each) of the current device, read once per device from its properties: a whole
// MI355X has 256 and 8, a partition of it fewer. Without a visible device the whole chip's figures are returned, so
// that the workspace-size queries answer on any machine.
struct Chip
{
    int cus, xcds;
};
Chip chip();
inline int device_cus()
{
    return chip().cus;
}

// small fills as kernels (a memset node inside a captured graph is avoided on purpose)
int fill_launch(float *dst, int64_t n, float value, hipStream_t st);
int fill_bytes_launch(void *dst, int value, size_t bytes, hipStream_t st);

// dst[o][c][r] = src[o][r][c] for elements of 1, 4 or 8 bytes (LDS tiles, lanes along the contiguous side of both)
int transpose_launch(const void *src, void *dst, int elem_bytes, int64_t outer, int64_t rows, int64_t cols, hipStream_t st);

inline hipStream_t as_stream(void *s)
{
    return reinterpret_cast<hipStream_t>(s);
}

inline int64_t ceil_div(int64_t a, int64_t b)
{
    return (a + b - 1) / b;
}

// Division of a 32-bit unsigned number by a divisor fixed at launch: one multiply-high, a subtract, two shifts and
// an add, exact for every 32-bit dividend (the round-up method: mul = floor(2^32 * (2^s - d) / d) + 1 with
// s = ceil(log2 d)). A divisor of 1 has mul = 0 and no shifts.
struct FastDiv
{
    unsigned mul, sh1, sh2;
};

inline FastDiv make_fastdiv(unsigned d)
{
    if (d <= 1)
        return FastDiv{0u, 0u, 0u};
    unsigned s = 0;
    while ((1ull << s) < d)
        ++s;
    return FastDiv{(unsigned)((((1ull << 32) * ((1ull << s) - d)) / d) + 1), 1u, s - 1};
}

__device__ inline unsigned fastdiv(unsigned m, const FastDiv &f)
{
    const unsigned t = __umulhi(m, f.mul);
    return (t + ((m - t) >> f.sh1)) >> f.sh2;
}

// A detect stage whose 1x1 convolution writes decoded rows: what decodes them (grid, anchor grid, stride; CI = classes
// + 5 channels per anchor) and where they go (rows[n * rows_image_stride + (anchor * H * W + pixel) * CI + channel]).
struct DetectRows
{
    const float *grid, *anchor_grid;
    float *rows;
    int64_t grid_elems, anchor_elems, rows_image_stride;
    float stride;
    int CI, anchor_H, anchor_W;
};
// One to four 1x1 convolutions in one launch (conv_direct.hip); with det, member s's outputs are decoded into det[s].rows
// instead of stored to y[s] (y and y_bs are then not read).
int conv_direct_group(int count, const float *const *x, const int64_t *x_bs, const float *const *packed, const float *const *b,
                      float *const *y, const int64_t *y_bs, int64_t N, const int64_t *C, const int64_t *H, const int64_t *W,
                      const int64_t *OC, int act, hipStream_t st, const DetectRows *det = nullptr);
bool conv_direct_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW,
                    int64_t OH, int64_t OW);

// the activations a convolution's epilogue can apply (0 none, 1 relu, 2 silu); the expressions are those of the
// standalone unary kernels
__device__ inline float apply_act(float v, int act)
{
    if (act == 1)
        return v > 0.f ? v : 0.f;
    if (act == 2)
    {
        const float s = 1.0f / (1.0f + expf(-v));
        return v * s;
    }
    return v;
}
}  // namespace odl

#define ODL_HIP_CHECK(expr)                                                                          \
    do                                                                                               \
    {                                                                                                \
        hipError_t e__ = (expr);                                                                     \
        if (e__ != hipSuccess)                                                                       \
            return odl::fail(ODL_ERR_RUNTIME, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e__), \
                             __FILE__, __LINE__);                                                    \
    } while (0)

// after a kernel launch: surfaces launch-configuration errors without synchronising
#define ODL_LAUNCH_CHECK() ODL_HIP_CHECK(hipGetLastError())

#define ODL_REQUIRE(cond, ...)                                   \
    do                                                           \
    {                                                            \
        if (!(cond))                                             \
            return odl::fail(ODL_ERR_INVALID_ARG, __VA_ARGS__);  \
    } while (0)

#define ODL_REQUIRE_DEVICE()             \
    do                                   \
    {                                    \
        int rc__ = odl::require_device(); \
        if (rc__ != ODL_OK)              \
            return rc__;                 \
    } while (0)
