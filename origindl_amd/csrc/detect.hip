// Forward-only operators of the detector path: nearest-neighbour upsampling, concatenation, and the YOLO detect
// head (1x1 convolution, then sigmoid and box decoding in one pass over the convolution's output).
//   upsample  src/mat/origin/cpu/nn/upsample.cpp:22-75        y[n,c,oh,ow] = x[n,c,oh/scale_h,ow/scale_w]
//   cat       src/mat/origin/cpu/shape/cat.cpp:20-140         [M, C_i, N] blocks copied side by side along C
//   detect    src/mat/origin/cpu/custom/yolo_detect.cpp:28-166
// All three are streams over HBM; index arithmetic is 32-bit where the sizes allow.
#include "odl_common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

extern "C" int odl_hip_conv2d(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                              int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *y, void *workspace,
                              size_t workspace_bytes, void *stream);
extern "C" size_t odl_hip_conv2d_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                                                 int SH, int SW, int PH, int PW);

namespace
{
constexpr int kBlock = 256;

// one thread per output pixel; consecutive threads along ow
__global__ __launch_bounds__(kBlock) void upsample_nearest_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                  unsigned planes, int H, int W, int OH, int OW, int sh,
                                                                  int sw)
{
    const unsigned oplane = (unsigned)(OH * OW);
    const unsigned t = blockIdx.x * (unsigned)kBlock + threadIdx.x;
    if (t >= planes * oplane)
        return;
    const unsigned nc = t / oplane, r = t - nc * oplane;
    const int oh = (int)(r / (unsigned)OW), ow = (int)r - oh * OW;
    y[t] = x[(int64_t)nc * H * W + (oh / sh) * W + ow / sw];
}

// The same with four consecutive output pixels per thread (output rows of a multiple of four pixels, 16-byte aligned
// base): one 16-byte store, the index arithmetic once per quad; the repeated source pixels come out of the cache.
__global__ __launch_bounds__(kBlock) void upsample_nearest_quads_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                        unsigned quads, int H, int W, int OH, int OW, int sh,
                                                                        int sw, odl::FastDiv d_qrow, odl::FastDiv d_oh)
{
    const unsigned t = blockIdx.x * (unsigned)kBlock + threadIdx.x;
    if (t >= quads)
        return;
    const unsigned qrow = (unsigned)OW / 4u;
    const unsigned line = odl::fastdiv(t, d_qrow), q = t - line * qrow;  // line = nc * OH + oh
    const unsigned nc = odl::fastdiv(line, d_oh), oh = line - nc * (unsigned)OH;
    const float *row = x + ((int64_t)nc * H + (int)oh / sh) * W;
    const int ow = 4 * (int)q;
    f32x4 v;
    if (sw == 2)
    {
        const float a = row[ow / 2], b = row[ow / 2 + 1];
        v = f32x4{a, a, b, b};
    }
    else
        v = f32x4{row[ow / sw], row[(ow + 1) / sw], row[(ow + 2) / sw], row[(ow + 3) / sw]};
    reinterpret_cast<f32x4 *>(y)[t] = v;
}

// upsample_nearest_quads_kernel for tensors whose images lie x_bs / y_bs floats apart (channel runs of wider tensors)
__global__ __launch_bounds__(kBlock) void upsample_nearest_view_kernel(const float *__restrict__ x, int64_t x_bs,
                                                                       float *__restrict__ y, int64_t y_bs, unsigned quads,
                                                                       int C, int H, int W, int OH, int OW, int sh, int sw,
                                                                       odl::FastDiv d_qrow, odl::FastDiv d_oh, odl::FastDiv d_c)
{
    const unsigned t = blockIdx.x * (unsigned)kBlock + threadIdx.x;
    if (t >= quads)
        return;
    const unsigned qrow = (unsigned)OW / 4u;
    const unsigned line = odl::fastdiv(t, d_qrow), q = t - line * qrow;  // line = (n * C + c) * OH + oh
    const unsigned nc = odl::fastdiv(line, d_oh), oh = line - nc * (unsigned)OH;
    const unsigned n = odl::fastdiv(nc, d_c), c = nc - n * (unsigned)C;
    const float *row = x + (int64_t)n * x_bs + ((int64_t)c * H + (int)oh / sh) * W;
    const int ow = 4 * (int)q;
    const f32x4 v{row[ow / sw], row[(ow + 1) / sw], row[(ow + 2) / sw], row[(ow + 3) / sw]};
    *reinterpret_cast<f32x4 *>(y + (int64_t)n * y_bs + ((int64_t)c * OH + oh) * OW + ow) = v;
}

// dst[m*dst_stride + dst_off + j] = src[m*src_stride + src_off + j] for j < chunk: `outer` contiguous runs;
// grid (run pieces, m). Concatenation scatters whole inputs (src_stride = chunk, src_off = 0); its backward, split,
// gathers a slice (dst_stride = chunk, dst_off = 0).
template <bool VEC>
__global__ __launch_bounds__(kBlock) void cat_copy_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                          int64_t chunk, int64_t src_stride, int64_t src_off,
                                                          int64_t dst_stride, int64_t dst_off)
{
    const int64_t m = blockIdx.y;
    const float *s = src + m * src_stride + src_off;
    float *d = dst + m * dst_stride + dst_off;
    const int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * (VEC ? 4 : 1);
    if (VEC)
    {
        if (i + 3 < chunk)
            *reinterpret_cast<f32x4 *>(d + i) = *reinterpret_cast<const f32x4 *>(s + i);
        else
            for (int64_t k = i; k < chunk; ++k)
                d[k] = s[k];
    }
    else if (i < chunk)
        d[i] = s[i];
}

// Concatenation of up to kCatInputs inputs in one launch: dst[m][col0 + j] for j < cols, where the columns are the inputs'
// chunks one after the other (end[i] = columns up to and including input i). Chunks, strides and bases are multiples of
// four floats, so a 16-byte piece lies in one input. A workgroup moves 16 KB of one destination row, four loads in
// flight per thread.
constexpr int kCatInputs = 8;
struct CatArgs
{
    const float *src[kCatInputs];
    int64_t end[kCatInputs];
    int count;
};

__global__ __launch_bounds__(kBlock) void cat_rows_kernel(const CatArgs a, float *__restrict__ dst, int64_t cols,
                                                          int64_t dst_stride, int64_t dst_off)
{
    const int64_t m = blockIdx.y;
    float *d = dst + m * dst_stride + dst_off;
    const int64_t j0 = (int64_t)blockIdx.x * (16 * kBlock) + 4 * threadIdx.x;
    f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
    {
        const int64_t j = j0 + (int64_t)u * 4 * kBlock;
        if (j < cols)
        {
            int i = 0;
            int64_t start = 0;
#pragma unroll
            for (int k = 0; k + 1 < kCatInputs; ++k)
                if (k + 1 < a.count && j >= a.end[k])
                    i = k + 1, start = a.end[k];
            v[u] = *reinterpret_cast<const f32x4 *>(a.src[i] + m * (a.end[i] - start) + (j - start));
        }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
    {
        const int64_t j = j0 + (int64_t)u * 4 * kBlock;
        if (j < cols)
            *reinterpret_cast<f32x4 *>(d + j) = v[u];
    }
}

// gx[nc][h][w] = sum over the scale_h x scale_w block of gy it was copied to, rows then columns ascending — the order
// in which the reference's loop over gy reaches that input pixel (nn/upsample.cpp:113-131)
__global__ __launch_bounds__(kBlock) void upsample_nearest_bwd_kernel(const float *__restrict__ gy, float *__restrict__ gx,
                                                                      unsigned planes, int H, int W, int OH, int OW, int sh,
                                                                      int sw)
{
    const unsigned plane = (unsigned)(H * W);
    const unsigned t = blockIdx.x * (unsigned)kBlock + threadIdx.x;
    if (t >= planes * plane)
        return;
    const unsigned nc = t / plane, r = t - nc * plane;
    const int h = (int)(r / (unsigned)W), w = (int)r - h * W;
    const float *p = gy + (int64_t)nc * OH * OW;
    float acc = 0.f;
    for (int i = 0; i < sh; ++i)
    {
        const int oh = h * sh + i;
        if (oh >= OH)
            break;
        for (int j = 0; j < sw; ++j)
        {
            const int ow = w * sw + j;
            if (ow < OW)
                acc += p[oh * OW + ow];
        }
    }
    gx[t] = acc;
}

// conv[b][a*CI + c][h][w] -> out[b][(a*H + h)*W + w][c], sigmoid, then the box transform on c = 0..3.
// A workgroup turns a tile of 64 spatial positions x CI channels through LDS: reads run along w, writes along c.
struct DetectGeom
{
    int A, CI, H, W;
    int anchor_H, anchor_W;
    int64_t grid_elems, anchor_elems;
    float stride;
    int64_t out_bs;  // floats from one image's rows of this stage to the next image's
};

// (sixteen waves a workgroup: the kernel is a chain of a load, 85 x 64 sigmoids and a store, and the chain is as long as
// one lane's share of the sigmoids)
constexpr int kDecodeThreads = 1024;
__device__ __forceinline__ void yolo_decode_tile(const float *__restrict__ conv, const float *__restrict__ grid,
                                                 const float *__restrict__ anchor_grid, float *__restrict__ out,
                                                 const DetectGeom &g, int ptiles, unsigned vb)
{
    extern __shared__ float sh_det[];  // [64][CI | 1]
    const int LS = g.CI | 1;
    const int HW = g.H * g.W;
    const int pt = (int)(vb % (unsigned)ptiles);
    vb /= (unsigned)ptiles;
    const int a = (int)(vb % (unsigned)g.A);
    const int b = (int)(vb / (unsigned)g.A);
    const int p0 = pt * 64;
    const int np = (HW - p0 < 64) ? HW - p0 : 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float *src = conv + ((int64_t)(b * g.A + a) * g.CI) * HW + p0;
    // the grid or anchor value of the thread's box channel (used after the first barrier), asked for before anything else:
    // behind the barrier it was a trip to memory of its own in a kernel that is little else than such trips
    float box_operand = 0.0f;
    {
        const int pl = threadIdx.x >> 2, c = threadIdx.x & 3;
        if (pl < np && c < g.CI)
        {
            const int p = p0 + pl;
            const int h = p / g.W, w = p - h * g.W;
            if (c < 2)
            {
                const int64_t gi = ((int64_t)a * HW + (int64_t)h * g.W + w) * 2 + c;
                box_operand = gi < g.grid_elems ? grid[gi] : 0.0f;
            }
            else
            {
                const int sh_ = (g.anchor_H > 0 && g.H > g.anchor_H) ? g.H / g.anchor_H : 1;
                const int sw_ = (g.anchor_W > 0 && g.W > g.anchor_W) ? g.W / g.anchor_W : 1;
                int ah = h / sh_, aw = w / sw_;
                ah = ah < g.anchor_H - 1 ? ah : g.anchor_H - 1;
                aw = aw < g.anchor_W - 1 ? aw : g.anchor_W - 1;
                const int64_t ai = ((int64_t)a * g.anchor_H * g.anchor_W + (int64_t)ah * g.anchor_W + aw) * 2 + (c - 2);
                box_operand = ai < g.anchor_elems ? anchor_grid[ai] : 1.0f;
            }
        }
    }
    // a wave takes every sixteenth channel; eight of them in flight at a time: the loads of a batch are issued together,
    // then its sigmoids (85 channels: one batch a wave, one trip to memory, six sigmoids a lane)
    constexpr int kBatch = 8, kWaves = kDecodeThreads / 64;
    for (int c0 = wave; c0 < g.CI; c0 += kBatch * kWaves)
    {
        float v[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
        {
            const int c = c0 + j * kWaves;
            v[j] = (c < g.CI && lane < np) ? src[(int64_t)c * HW + lane] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
        {
            const int c = c0 + j * kWaves;
            if (c < g.CI && lane < np)
                sh_det[lane * LS + c] = 1.0f / (1.0f + expf(-v[j]));  // the reference's -x, exp, 1 + ., 1 / . steps
        }
    }
    __syncthreads();
    // the four box channels of each pixel: one thread each (64 pixels x 4 = the whole workgroup), so the grid and
    // anchor loads are issued once, outside the streaming loop below
    {
        const int pl = threadIdx.x >> 2, c = threadIdx.x & 3;
        if (pl < np && c < g.CI)
        {
            float v = sh_det[pl * LS + c];
            if (c < 2)
            {
                const float t = v * 2.0f;
                v = (t + box_operand) * g.stride;
            }
            else
            {
                const float t = v * 2.0f;
                v = (t * t) * box_operand;  // pow(2s, 2) * anchor
            }
            sh_det[pl * LS + c] = v;
        }
    }
    __syncthreads();
    // [pixel][channel] rows out of LDS, consecutive lanes along the output
    float *dst = out + (int64_t)b * g.out_bs + ((int64_t)a * HW + p0) * g.CI;
    for (int pl = wave; pl < np; pl += kDecodeThreads / 64)
#pragma unroll 2
        for (int c = lane; c < g.CI; c += 64)
            dst[pl * g.CI + c] = sh_det[pl * LS + c];
}

__global__ __launch_bounds__(kDecodeThreads) void yolo_decode_kernel(const float *__restrict__ conv, const float *__restrict__ grid,
                                                             const float *__restrict__ anchor_grid,
                                                             float *__restrict__ out, DetectGeom g, int ptiles)
{
    yolo_decode_tile(conv, grid, anchor_grid, out, g, ptiles, blockIdx.x);
}

// Up to kMaxStages stages of one detect head in one launch: workgroups [first[s], first[s + 1]) are stage s's, each doing
// what yolo_decode_kernel's workgroup of the same number within the stage does.
constexpr int kMaxStages = 4;
struct DetectStages
{
    const float *conv[kMaxStages], *grid[kMaxStages], *anchor_grid[kMaxStages];
    float *out[kMaxStages];
    DetectGeom g[kMaxStages];
    int ptiles[kMaxStages];
    unsigned first[kMaxStages + 1];
};

__global__ __launch_bounds__(kDecodeThreads) void yolo_decode_stages_kernel(DetectStages d, int stages)
{
    int s = 0;
    for (int j = 1; j < stages; ++j)
        s = blockIdx.x >= d.first[j] ? j : s;
    yolo_decode_tile(d.conv[s], d.grid[s], d.anchor_grid[s], d.out[s], d.g[s], d.ptiles[s], blockIdx.x - d.first[s]);
}
}  // namespace

extern "C" {

int odl_hip_upsample_nearest(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
                             int scale_h, int scale_w, float *y, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && C >= 0 && H > 0 && W > 0 && OH > 0 && OW > 0, "upsample: bad shape");
    ODL_REQUIRE(scale_h > 0 && scale_w > 0, "upsample: scale must be positive");
    // the reference indexes x[oh/scale_h][ow/scale_w] without a bound; here the source pixel must exist
    ODL_REQUIRE((OH - 1) / scale_h < H && (OW - 1) / scale_w < W,
                "upsample: output (%lld,%lld) reaches past input (%lld,%lld) at scale (%d,%d)", (long long)OH,
                (long long)OW, (long long)H, (long long)W, scale_h, scale_w);
    const int64_t total = N * C * OH * OW;
    if (total == 0)
        return ODL_OK;
    ODL_REQUIRE(total < (1ll << 32) - kBlock && H * W < (1ll << 31) && OH * OW < (1ll << 31), "upsample: too large");
    if (OW % 4 == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 && N * C * OH < (1ll << 31))
    {
        const unsigned quads = (unsigned)(total / 4);
        hipLaunchKernelGGL(upsample_nearest_quads_kernel, dim3((unsigned)odl::ceil_div(quads, kBlock)), dim3(kBlock), 0,
                           odl::as_stream(stream), x, y, quads, (int)H, (int)W, (int)OH, (int)OW, scale_h, scale_w,
                           odl::make_fastdiv((unsigned)(OW / 4)), odl::make_fastdiv((unsigned)OH));
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    }
    hipLaunchKernelGGL(upsample_nearest_kernel, dim3((unsigned)odl::ceil_div(total, kBlock)), dim3(kBlock), 0,
                       odl::as_stream(stream), x, y, (unsigned)(N * C), (int)H, (int)W, (int)OH, (int)OW, scale_h,
                       scale_w);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_cat(const float *const *host_inputs, const int64_t *host_axis_sizes, int count, int64_t outer, int64_t inner,
                float *out, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(count >= 1, "cat: requires at least 1 input");
    ODL_REQUIRE(host_inputs && host_axis_sizes && out, "cat: null argument");
    ODL_REQUIRE(outer >= 0 && inner >= 0 && outer < 65536 * 32768ll, "cat: bad outer/inner extents");
    int64_t total_axis = 0;
    for (int i = 0; i < count; ++i)
    {
        ODL_REQUIRE(host_axis_sizes[i] >= 0, "cat: negative axis size");
        total_axis += host_axis_sizes[i];
    }
    hipStream_t st = odl::as_stream(stream);
    int64_t off = 0;
    // every input in 16-byte pieces: one launch for up to kCatInputs of them
    bool all_vec = outer > 0 && outer < 65536 && (total_axis * inner) % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    for (int i = 0; i < count && all_vec; ++i)
        all_vec = (host_axis_sizes[i] * inner) % 4 == 0 &&
                  (host_axis_sizes[i] * inner == 0 || (host_inputs[i] && reinterpret_cast<uintptr_t>(host_inputs[i]) % 16 == 0));
    if (all_vec && count >= 2)
    {
        const int64_t dst_stride = total_axis * inner;
        int i = 0;
        while (i < count)
        {
            CatArgs a{};
            int64_t cols = 0;
            const int64_t dst_off = off * inner;
            while (i < count && a.count < kCatInputs)
            {
                const int64_t chunk = host_axis_sizes[i] * inner;
                if (chunk > 0)
                {
                    cols += chunk;
                    a.src[a.count] = host_inputs[i], a.end[a.count] = cols;
                    ++a.count;
                }
                off += host_axis_sizes[i];
                ++i;
            }
            if (cols == 0)
                continue;
            for (int k = a.count; k < kCatInputs; ++k)
                a.src[k] = a.src[a.count - 1], a.end[k] = cols;
            ODL_REQUIRE(odl::ceil_div(cols, 16 * kBlock) < (1ll << 31), "cat: rows too long");
            hipLaunchKernelGGL(cat_rows_kernel, dim3((unsigned)odl::ceil_div(cols, 16 * kBlock), (unsigned)outer), dim3(kBlock), 0, st,
                               a, out, cols, dst_stride, dst_off);
            ODL_LAUNCH_CHECK();
        }
        return ODL_OK;
    }
    for (int i = 0; i < count; ++i)
    {
        const int64_t chunk = host_axis_sizes[i] * inner;
        if (chunk > 0 && outer > 0)
        {
            ODL_REQUIRE(host_inputs[i] != nullptr, "cat: input %d is null", i);
            const int64_t dst_stride = total_axis * inner, dst_off = off * inner;
            const bool vec = chunk % 4 == 0 && dst_stride % 4 == 0 && dst_off % 4 == 0 &&
                             reinterpret_cast<uintptr_t>(host_inputs[i]) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
            // grid.y carries the outer index in slabs of at most 65535
            for (int64_t m0 = 0; m0 < outer; m0 += 65535)
            {
                const int64_t ms = outer - m0 < 65535 ? outer - m0 : 65535;
                const float *s = host_inputs[i] + m0 * chunk;
                float *d = out + m0 * dst_stride;
                if (vec)
                    hipLaunchKernelGGL((cat_copy_kernel<true>), dim3((unsigned)odl::ceil_div(chunk / 4, kBlock), (unsigned)ms),
                                       dim3(kBlock), 0, st, s, d, chunk, chunk, (int64_t)0, dst_stride, dst_off);
                else
                    hipLaunchKernelGGL((cat_copy_kernel<false>), dim3((unsigned)odl::ceil_div(chunk, kBlock), (unsigned)ms),
                                       dim3(kBlock), 0, st, s, d, chunk, chunk, (int64_t)0, dst_stride, dst_off);
                ODL_LAUNCH_CHECK();
            }
        }
        off += host_axis_sizes[i];
    }
    return ODL_OK;
}

int odl_hip_slice_axis(const float *src, int64_t outer, int64_t axis_size, int64_t inner, int64_t offset, int64_t length,
                       float *dst, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(outer >= 0 && axis_size >= 0 && inner >= 0 && outer < 65536 * 32768ll, "slice: bad extents");
    ODL_REQUIRE(offset >= 0 && length >= 0 && offset + length <= axis_size, "slice: [%lld, %lld) lies outside an axis of %lld",
                (long long)offset, (long long)(offset + length), (long long)axis_size);
    const int64_t chunk = length * inner;
    if (chunk == 0 || outer == 0)
        return ODL_OK;
    ODL_REQUIRE(src && dst, "slice: null operand");
    hipStream_t st = odl::as_stream(stream);
    const int64_t src_stride = axis_size * inner, src_off = offset * inner;
    const bool vec = chunk % 4 == 0 && src_stride % 4 == 0 && src_off % 4 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(dst) % 16 == 0;
    for (int64_t m0 = 0; m0 < outer; m0 += 65535)
    {
        const int64_t ms = outer - m0 < 65535 ? outer - m0 : 65535;
        const float *s = src + m0 * src_stride;
        float *d = dst + m0 * chunk;
        if (vec)
            hipLaunchKernelGGL((cat_copy_kernel<true>), dim3((unsigned)odl::ceil_div(chunk / 4, kBlock), (unsigned)ms), dim3(kBlock),
                               0, st, s, d, chunk, src_stride, src_off, chunk, (int64_t)0);
        else
            hipLaunchKernelGGL((cat_copy_kernel<false>), dim3((unsigned)odl::ceil_div(chunk, kBlock), (unsigned)ms), dim3(kBlock), 0,
                               st, s, d, chunk, src_stride, src_off, chunk, (int64_t)0);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}

int odl_hip_upsample_nearest_backward(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
                                      int scale_h, int scale_w, float *gx, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && C >= 0 && H > 0 && W > 0 && OH > 0 && OW > 0, "upsample backward: bad shape");
    ODL_REQUIRE(scale_h > 0 && scale_w > 0, "upsample backward: scale must be positive");
    ODL_REQUIRE((OH - 1) / scale_h < H && (OW - 1) / scale_w < W, "upsample backward: gradient (%lld,%lld) reaches past input (%lld,%lld)",
                (long long)OH, (long long)OW, (long long)H, (long long)W);
    const int64_t total = N * C * H * W;
    if (total == 0)
        return ODL_OK;
    ODL_REQUIRE(total < (1ll << 32) - kBlock && H * W < (1ll << 31) && OH * OW < (1ll << 31), "upsample backward: too large");
    hipLaunchKernelGGL(upsample_nearest_bwd_kernel, dim3((unsigned)odl::ceil_div(total, kBlock)), dim3(kBlock), 0,
                       odl::as_stream(stream), gy, gx, (unsigned)(N * C), (int)H, (int)W, (int)OH, (int)OW, scale_h, scale_w);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_upsample_nearest_view(const float *x, int64_t x_image_stride, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH,
                                  int64_t OW, int scale_h, int scale_w, float *y, int64_t y_image_stride, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(x && y && N >= 0 && C > 0 && H > 0 && W > 0 && OH > 0 && OW > 0, "upsample: bad shape or null operand");
    ODL_REQUIRE(scale_h > 0 && scale_w > 0, "upsample: scale must be positive");
    ODL_REQUIRE((OH - 1) / scale_h < H && (OW - 1) / scale_w < W,
                "upsample: output (%lld,%lld) reaches past input (%lld,%lld) at scale (%d,%d)", (long long)OH,
                (long long)OW, (long long)H, (long long)W, scale_h, scale_w);
    const int64_t xs = x_image_stride ? x_image_stride : C * H * W, ys = y_image_stride ? y_image_stride : C * OH * OW;
    ODL_REQUIRE(xs >= C * H * W && ys >= C * OH * OW, "upsample: an image stride is shorter than the image");
    ODL_REQUIRE(OW % 4 == 0 && ys % 4 == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0,
                "upsample_view: output rows must be a multiple of four floats and 16-byte aligned");
    const int64_t total = N * C * OH * OW;
    if (total == 0)
        return ODL_OK;
    ODL_REQUIRE(total < (1ll << 32) - kBlock && H * W < (1ll << 31) && OH * OW < (1ll << 31) && N * C * OH < (1ll << 31),
                "upsample: too large");
    const unsigned quads = (unsigned)(total / 4);
    hipLaunchKernelGGL(upsample_nearest_view_kernel, dim3((unsigned)odl::ceil_div(quads, kBlock)), dim3(kBlock), 0,
                       odl::as_stream(stream), x, xs, y, ys, quads, (int)C, (int)H, (int)W, (int)OH, (int)OW, scale_h, scale_w,
                       odl::make_fastdiv((unsigned)(OW / 4)), odl::make_fastdiv((unsigned)OH), odl::make_fastdiv((unsigned)C));
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_copy_images(const float *src, int64_t src_image_stride, float *dst, int64_t dst_image_stride, int64_t N,
                        int64_t count, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && count >= 0 && src_image_stride >= count && dst_image_stride >= count, "copy_images: bad extents");
    if (N == 0 || count == 0)
        return ODL_OK;
    ODL_REQUIRE(src && dst, "copy_images: null operand");
    hipStream_t st = odl::as_stream(stream);
    const bool vec = count % 4 == 0 && src_image_stride % 4 == 0 && dst_image_stride % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0;
    for (int64_t m0 = 0; m0 < N; m0 += 65535)
    {
        const int64_t ms = N - m0 < 65535 ? N - m0 : 65535;
        const float *s = src + m0 * src_image_stride;
        float *d = dst + m0 * dst_image_stride;
        if (vec)
            hipLaunchKernelGGL((cat_copy_kernel<true>), dim3((unsigned)odl::ceil_div(count / 4, kBlock), (unsigned)ms), dim3(kBlock),
                               0, st, s, d, count, src_image_stride, (int64_t)0, dst_image_stride, (int64_t)0);
        else
            hipLaunchKernelGGL((cat_copy_kernel<false>), dim3((unsigned)odl::ceil_div(count, kBlock), (unsigned)ms), dim3(kBlock), 0,
                               st, s, d, count, src_image_stride, (int64_t)0, dst_image_stride, (int64_t)0);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}

int odl_hip_yolo_decode(const float *conv, const float *grid, int64_t grid_elems, const float *anchor_grid, int64_t anchor_elems,
                        int64_t anchor_H, int64_t anchor_W, int64_t N, int64_t H, int64_t W, float stride, int num_anchors,
                        int num_classes, float *out, int64_t out_image_stride, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && H > 0 && W > 0 && num_anchors > 0 && num_classes >= 0, "yolo_decode: bad shape");
    ODL_REQUIRE(conv && grid && anchor_grid && out, "yolo_decode: null operand");
    ODL_REQUIRE(grid_elems >= 0 && anchor_elems >= 0 && anchor_H > 0 && anchor_W > 0, "yolo_decode: bad grid sizes");
    if (N == 0)
        return ODL_OK;
    const int CI = num_classes + 5;
    ODL_REQUIRE(N * num_anchors * odl::ceil_div(H * W, 64) < (1ll << 31) && H * W < (1ll << 30) && CI < 8192, "yolo_decode: too large");
    const int64_t os = out_image_stride ? out_image_stride : (int64_t)num_anchors * H * W * CI;
    ODL_REQUIRE(os >= (int64_t)num_anchors * H * W * CI, "yolo_decode: the output image stride is shorter than a stage's rows");
    const int ptiles = (int)odl::ceil_div(H * W, 64);
    const DetectGeom g{num_anchors, CI, (int)H, (int)W, (int)anchor_H, (int)anchor_W, grid_elems, anchor_elems, stride, os};
    const size_t lds = (size_t)64 * (CI | 1) * sizeof(float);
    hipLaunchKernelGGL(yolo_decode_kernel, dim3((unsigned)(N * num_anchors * ptiles)), dim3(kDecodeThreads), lds, odl::as_stream(stream),
                       conv, grid, anchor_grid, out, g, ptiles);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_yolo_decode_stages(int stages, const float *const *host_conv, const float *const *host_grid, const int64_t *host_grid_elems,
                               const float *const *host_anchor_grid, const int64_t *host_anchor_elems, const int64_t *host_anchor_H,
                               const int64_t *host_anchor_W, int64_t N, const int64_t *host_H, const int64_t *host_W,
                               const float *host_stride, int num_anchors, int num_classes, float *const *host_out,
                               int64_t out_image_stride, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(stages >= 1 && stages <= kMaxStages, "yolo_decode_stages: 1 to %d stages, got %d", kMaxStages, stages);
    ODL_REQUIRE(host_conv && host_grid && host_grid_elems && host_anchor_grid && host_anchor_elems && host_anchor_H && host_anchor_W &&
                    host_H && host_W && host_stride && host_out,
                "yolo_decode_stages: null argument");
    ODL_REQUIRE(N >= 0 && num_anchors > 0 && num_classes >= 0, "yolo_decode_stages: bad shape");
    const int CI = num_classes + 5;
    ODL_REQUIRE(CI < 8192, "yolo_decode_stages: too large");
    DetectStages d{};
    int64_t blocks = 0;
    for (int s = 0; s < stages; ++s)
    {
        const int64_t H = host_H[s], W = host_W[s];
        ODL_REQUIRE(H > 0 && W > 0 && H * W < (1ll << 30), "yolo_decode_stages: bad shape of stage %d", s);
        ODL_REQUIRE(host_conv[s] && host_grid[s] && host_anchor_grid[s] && host_out[s], "yolo_decode_stages: null operand of stage %d", s);
        ODL_REQUIRE(host_grid_elems[s] >= 0 && host_anchor_elems[s] >= 0 && host_anchor_H[s] > 0 && host_anchor_W[s] > 0,
                    "yolo_decode_stages: bad grid sizes of stage %d", s);
        const int64_t rows = (int64_t)num_anchors * H * W * CI;
        const int64_t os = out_image_stride ? out_image_stride : rows;
        ODL_REQUIRE(os >= rows, "yolo_decode_stages: the output image stride is shorter than the rows of stage %d", s);
        d.conv[s] = host_conv[s], d.grid[s] = host_grid[s], d.anchor_grid[s] = host_anchor_grid[s], d.out[s] = host_out[s];
        d.ptiles[s] = (int)odl::ceil_div(H * W, 64);
        d.g[s] = DetectGeom{num_anchors, CI, (int)H, (int)W, (int)host_anchor_H[s], (int)host_anchor_W[s], host_grid_elems[s],
                            host_anchor_elems[s], host_stride[s], os};
        d.first[s] = (unsigned)blocks;
        blocks += N * num_anchors * d.ptiles[s];
        ODL_REQUIRE(blocks < (1ll << 31), "yolo_decode_stages: too large");
    }
    for (int s = stages; s <= kMaxStages; ++s)
        d.first[s] = (unsigned)blocks;
    if (blocks == 0)
        return ODL_OK;
    const size_t lds = (size_t)64 * (CI | 1) * sizeof(float);
    hipLaunchKernelGGL(yolo_decode_stages_kernel, dim3((unsigned)blocks), dim3(kDecodeThreads), lds, odl::as_stream(stream), d, stages);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_yolo_detect_stages_ok(int stages, int64_t N, const int64_t *host_C, const int64_t *host_H, const int64_t *host_W,
                                  int num_anchors, int num_classes)
{
    if (stages < 1 || stages > kMaxStages || N <= 0 || num_anchors <= 0 || num_classes < 0 || !host_C || !host_H || !host_W)
        return 0;
    const int64_t OC = (int64_t)num_anchors * (num_classes + 5);
    for (int s = 0; s < stages; ++s)
        if (host_C[s] <= 0 || host_H[s] <= 0 || host_W[s] <= 0 ||
            !odl::conv_direct_ok(N, host_C[s], host_H[s], host_W[s], OC, 1, 1, 1, 1, 0, 0, host_H[s], host_W[s]))
            return 0;
    return 1;
}

int odl_hip_yolo_detect_stages_forward(int stages, const float *const *host_x, const int64_t *host_x_image_stride,
                                       const float *const *host_packed, const float *const *host_b, const float *const *host_grid,
                                       const int64_t *host_grid_elems, const float *const *host_anchor_grid,
                                       const int64_t *host_anchor_elems, const int64_t *host_anchor_H, const int64_t *host_anchor_W,
                                       int64_t N, const int64_t *host_C, const int64_t *host_H, const int64_t *host_W,
                                       const float *host_stride, int num_anchors, int num_classes, float *const *host_out,
                                       int64_t out_image_stride, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(stages >= 1 && stages <= kMaxStages, "yolo_detect_stages_forward: 1 to %d stages, got %d", kMaxStages, stages);
    ODL_REQUIRE(host_x && host_x_image_stride && host_packed && host_grid && host_grid_elems && host_anchor_grid && host_anchor_elems &&
                    host_anchor_H && host_anchor_W && host_C && host_H && host_W && host_stride && host_out,
                "yolo_detect_stages_forward: null argument");
    ODL_REQUIRE(N >= 0 && num_anchors > 0 && num_classes >= 0, "yolo_detect_stages_forward: bad shape");
    if (N == 0)
        return ODL_OK;
    ODL_REQUIRE(odl_hip_yolo_detect_stages_ok(stages, N, host_C, host_H, host_W, num_anchors, num_classes),
                "yolo_detect_stages_forward: shape not covered (ask odl_hip_yolo_detect_stages_ok first)");
    const int CI = num_classes + 5;
    odl::DetectRows det[kMaxStages];
    int64_t OC[kMaxStages];
    for (int s = 0; s < stages; ++s)
    {
        ODL_REQUIRE(host_x[s] && host_packed[s] && host_grid[s] && host_anchor_grid[s] && host_out[s],
                    "yolo_detect_stages_forward: null operand of stage %d", s);
        ODL_REQUIRE(host_grid_elems[s] >= 0 && host_anchor_elems[s] >= 0 && host_anchor_H[s] > 0 && host_anchor_W[s] > 0,
                    "yolo_detect_stages_forward: bad grid sizes of stage %d", s);
        const int64_t rows = (int64_t)num_anchors * host_H[s] * host_W[s] * CI;
        const int64_t os = out_image_stride ? out_image_stride : rows;
        ODL_REQUIRE(os >= rows, "yolo_detect_stages_forward: the output image stride is shorter than the rows of stage %d", s);
        ODL_REQUIRE(host_x_image_stride[s] == 0 || (host_x_image_stride[s] >= host_C[s] * host_H[s] * host_W[s] && host_x_image_stride[s] < (1ll << 40)),
                    "yolo_detect_stages_forward: bad input image stride of stage %d", s);
        det[s] = odl::DetectRows{host_grid[s], host_anchor_grid[s], host_out[s], host_grid_elems[s], host_anchor_elems[s], os,
                                 host_stride[s], CI, (int)host_anchor_H[s], (int)host_anchor_W[s]};
        OC[s] = (int64_t)num_anchors * CI;
    }
    return odl::conv_direct_group(stages, host_x, host_x_image_stride, host_packed, host_b, nullptr, nullptr, N, host_C, host_H, host_W,
                                  OC, 0, odl::as_stream(stream), det);
}

size_t odl_hip_yolo_detect_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int num_anchors, int num_classes)
{
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || num_anchors <= 0 || num_classes < 0)
        return 0;
    const int64_t OC = (int64_t)num_anchors * (num_classes + 5);
    const size_t conv_out = ((size_t)(N * OC * H * W) * sizeof(float) + 255) & ~(size_t)255;
    return conv_out + odl_hip_conv2d_workspace_bytes(N, C, H, W, OC, 1, 1, 1, 1, 0, 0);
}

int odl_hip_yolo_detect_forward(const float *x, const float *conv_w, const float *conv_b, const float *grid,
                                int64_t grid_elems, const float *anchor_grid, int64_t anchor_elems, int64_t anchor_H,
                                int64_t anchor_W, int64_t N, int64_t C, int64_t H, int64_t W, float stride, int num_anchors,
                                int num_classes, float *out, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && C > 0 && H > 0 && W > 0, "yolo_detect_forward: input must be 4D (N, C, H, W)");
    ODL_REQUIRE(num_anchors > 0 && num_classes >= 0, "yolo_detect_forward: bad anchor/class counts");
    ODL_REQUIRE(x && conv_w && grid && anchor_grid && out, "yolo_detect_forward: null operand");
    ODL_REQUIRE(grid_elems >= 0 && anchor_elems >= 0 && anchor_H > 0 && anchor_W > 0, "yolo_detect_forward: bad grid sizes");
    if (N == 0)
        return ODL_OK;
    const int CI = num_classes + 5;
    const int64_t OC = (int64_t)num_anchors * CI;
    ODL_REQUIRE(N * num_anchors * odl::ceil_div(H * W, 64) < (1ll << 31) && H * W < (1ll << 30) && CI < 8192,
                "yolo_detect_forward: too large");
    const size_t conv_bytes = ((size_t)(N * OC * H * W) * sizeof(float) + 255) & ~(size_t)255;
    const size_t need = odl_hip_yolo_detect_workspace_bytes(N, C, H, W, num_anchors, num_classes);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need, "yolo_detect_forward: workspace of %zu bytes required, got %zu",
                need, workspace_bytes);
    float *conv = static_cast<float *>(workspace);
    int rc = odl_hip_conv2d(x, conv_w, conv_b, N, C, H, W, OC, 1, 1, 1, 1, 0, 0, conv, static_cast<char *>(workspace) + conv_bytes,
                            workspace_bytes - conv_bytes, stream);
    if (rc != ODL_OK)
        return rc;
    const int ptiles = (int)odl::ceil_div(H * W, 64);
    const DetectGeom g{num_anchors, CI, (int)H, (int)W, (int)anchor_H, (int)anchor_W, grid_elems, anchor_elems, stride,
                       (int64_t)num_anchors * H * W * CI};
    const size_t lds = (size_t)64 * (CI | 1) * sizeof(float);
    hipLaunchKernelGGL(yolo_decode_kernel, dim3((unsigned)(N * num_anchors * ptiles)), dim3(kDecodeThreads), lds,
                       odl::as_stream(stream), conv, grid, anchor_grid, out, g, ptiles);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

// Mat::cat / Mat::split in the other element types (the reference dispatches both over the element type,
// src/mat/origin/cuda/shape/{cat,split}.cu): pure copies, so elements of 4 or 8 bytes go through the float32 kernels as
// one or two words each; 1-byte elements take a byte kernel.
}  // extern "C"

extern "C" size_t odl_hip_dtype_size(int dtype);

namespace
{
// dst[m*dst_stride + dst_off + j] = src[m*src_stride + src_off + j] for j < chunk, in bytes; grid (pieces, m)
__global__ __launch_bounds__(kBlock) void copy_runs_bytes_kernel(const unsigned char *__restrict__ src, unsigned char *__restrict__ dst,
                                                                 int64_t chunk, int64_t src_stride, int64_t src_off,
                                                                 int64_t dst_stride, int64_t dst_off)
{
    const int64_t m = blockIdx.y;
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j < chunk)
        dst[m * dst_stride + dst_off + j] = src[m * src_stride + src_off + j];
}

int copy_runs_bytes(const unsigned char *src, unsigned char *dst, int64_t outer, int64_t chunk, int64_t src_stride, int64_t src_off,
                    int64_t dst_stride, int64_t dst_off, hipStream_t st)
{
    for (int64_t m0 = 0; m0 < outer; m0 += 65535)
    {
        const int64_t ms = outer - m0 < 65535 ? outer - m0 : 65535;
        hipLaunchKernelGGL(copy_runs_bytes_kernel, dim3((unsigned)odl::ceil_div(chunk, kBlock), (unsigned)ms), dim3(kBlock), 0, st,
                           src + m0 * src_stride, dst + m0 * dst_stride, chunk, src_stride, src_off, dst_stride, dst_off);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}
}  // namespace

extern "C" {

int odl_hip_cat_dtype(int dtype, const void *const *host_inputs, const int64_t *host_axis_sizes, int count, int64_t outer,
                      int64_t inner, void *out, void *stream)
{
    const size_t esz = odl_hip_dtype_size(dtype);
    if (esz == 0)
        return odl::fail(ODL_ERR_INVALID_ARG, "cat: unknown element type code %d", dtype);
    if (esz % 4 == 0)
        return odl_hip_cat(reinterpret_cast<const float *const *>(host_inputs), host_axis_sizes, count, outer,
                           inner * (int64_t)(esz / 4), static_cast<float *>(out), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(count >= 1, "cat: requires at least 1 input");
    ODL_REQUIRE(host_inputs && host_axis_sizes && out, "cat: null argument");
    ODL_REQUIRE(outer >= 0 && inner >= 0 && outer < 65536 * 32768ll, "cat: bad outer/inner extents");
    int64_t total_axis = 0;
    for (int i = 0; i < count; ++i)
    {
        ODL_REQUIRE(host_axis_sizes[i] >= 0, "cat: negative axis size");
        total_axis += host_axis_sizes[i];
    }
    int64_t off = 0;
    for (int i = 0; i < count; ++i)
    {
        const int64_t chunk = host_axis_sizes[i] * inner;
        if (chunk > 0 && outer > 0)
        {
            ODL_REQUIRE(host_inputs[i] != nullptr, "cat: input %d is null", i);
            const int rc = copy_runs_bytes(static_cast<const unsigned char *>(host_inputs[i]), static_cast<unsigned char *>(out), outer,
                                           chunk, chunk, 0, total_axis * inner, off * inner, odl::as_stream(stream));
            if (rc != ODL_OK)
                return rc;
        }
        off += host_axis_sizes[i];
    }
    return ODL_OK;
}

int odl_hip_slice_axis_dtype(int dtype, const void *src, int64_t outer, int64_t axis_size, int64_t inner, int64_t offset,
                             int64_t length, void *dst, void *stream)
{
    const size_t esz = odl_hip_dtype_size(dtype);
    if (esz == 0)
        return odl::fail(ODL_ERR_INVALID_ARG, "slice: unknown element type code %d", dtype);
    if (esz % 4 == 0)
        return odl_hip_slice_axis(static_cast<const float *>(src), outer, axis_size, inner * (int64_t)(esz / 4), offset, length,
                                  static_cast<float *>(dst), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(outer >= 0 && axis_size >= 0 && inner >= 0 && outer < 65536 * 32768ll, "slice: bad extents");
    ODL_REQUIRE(offset >= 0 && length >= 0 && offset + length <= axis_size, "slice: [%lld, %lld) lies outside an axis of %lld",
                (long long)offset, (long long)(offset + length), (long long)axis_size);
    const int64_t chunk = length * inner;
    if (chunk == 0 || outer == 0)
        return ODL_OK;
    ODL_REQUIRE(src && dst, "slice: null operand");
    return copy_runs_bytes(static_cast<const unsigned char *>(src), static_cast<unsigned char *>(dst), outer, chunk, axis_size * inner,
                           offset * inner, chunk, 0, odl::as_stream(stream));
}

// Mat::upsample / upsample_backward in the other element types (src/mat/origin/cuda/nn/upsample.cu:176, 224 dispatch over
// the type): the forward is a copy and goes by element width; the backward adds the scale_h x scale_w block of gy that
// an input pixel was copied to, rows then columns ascending, in the element type (integers wrap).
}  // extern "C"

namespace
{
template <typename U>
__global__ __launch_bounds__(kBlock) void upsample_nearest_words_kernel(const U *__restrict__ x, U *__restrict__ y, int64_t total,
                                                                        int64_t H, int64_t W, int64_t OH, int64_t OW, int sh, int sw)
{
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= total)
        return;
    const int64_t ow = t % OW, oh = (t / OW) % OH, nc = t / (OW * OH);
    y[t] = x[(nc * H + oh / sh) * W + ow / sw];
}

template <typename T>
__global__ __launch_bounds__(kBlock) void upsample_nearest_bwd_any_kernel(const T *__restrict__ gy, T *__restrict__ gx, int64_t total,
                                                                          int64_t H, int64_t W, int64_t OH, int64_t OW, int sh, int sw)
{
    const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= total)
        return;
    const int64_t w = t % W, h = (t / W) % H, nc = t / (W * H);
    T acc = (T)0;
    for (int64_t oh = h * sh; oh < (h + 1) * sh && oh < OH; ++oh)
        for (int64_t ow = w * sw; ow < (w + 1) * sw && ow < OW; ++ow)
        {
            const T v = gy[(nc * OH + oh) * OW + ow];
            if (sizeof(T) < 4)
                acc = (T)((unsigned)acc + (unsigned)v);  // 8-bit integers wrap like the wider ones
            else
                acc = acc + v;
        }
    gx[t] = acc;
}
}  // namespace

extern "C" {

int odl_hip_upsample_nearest_dtype(int dtype, const void *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
                                   int scale_h, int scale_w, void *y, void *stream)
{
    if (dtype == 0)
        return odl_hip_upsample_nearest(static_cast<const float *>(x), N, C, H, W, OH, OW, scale_h, scale_w, static_cast<float *>(y),
                                        stream);
    ODL_REQUIRE_DEVICE();
    const size_t esz = odl_hip_dtype_size(dtype);
    ODL_REQUIRE(esz > 0, "upsample: unknown element type code %d", dtype);
    ODL_REQUIRE(N >= 0 && C >= 0 && H > 0 && W > 0 && OH > 0 && OW > 0, "upsample: bad shape");
    ODL_REQUIRE(scale_h > 0 && scale_w > 0, "upsample: scale must be positive");
    ODL_REQUIRE((OH - 1) / scale_h < H && (OW - 1) / scale_w < W,
                "upsample: output (%lld,%lld) reaches past input (%lld,%lld) at scale (%d,%d)", (long long)OH, (long long)OW,
                (long long)H, (long long)W, scale_h, scale_w);
    const int64_t total = N * C * OH * OW;
    if (total == 0)
        return ODL_OK;
    const dim3 grid((unsigned)odl::ceil_div(total, kBlock)), block(kBlock);
    hipStream_t st = odl::as_stream(stream);
    if (esz == 8)
        hipLaunchKernelGGL(upsample_nearest_words_kernel<uint64_t>, grid, block, 0, st, static_cast<const uint64_t *>(x),
                           static_cast<uint64_t *>(y), total, H, W, OH, OW, scale_h, scale_w);
    else if (esz == 4)
        hipLaunchKernelGGL(upsample_nearest_words_kernel<uint32_t>, grid, block, 0, st, static_cast<const uint32_t *>(x),
                           static_cast<uint32_t *>(y), total, H, W, OH, OW, scale_h, scale_w);
    else
        hipLaunchKernelGGL(upsample_nearest_words_kernel<uint8_t>, grid, block, 0, st, static_cast<const uint8_t *>(x),
                           static_cast<uint8_t *>(y), total, H, W, OH, OW, scale_h, scale_w);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_upsample_nearest_backward_dtype(int dtype, const void *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH,
                                            int64_t OW, int scale_h, int scale_w, void *gx, void *stream)
{
    if (dtype == 0)
        return odl_hip_upsample_nearest_backward(static_cast<const float *>(gy), N, C, H, W, OH, OW, scale_h, scale_w,
                                                 static_cast<float *>(gx), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(N >= 0 && C >= 0 && H > 0 && W > 0 && OH > 0 && OW > 0, "upsample_backward: bad shape");
    ODL_REQUIRE(scale_h > 0 && scale_w > 0, "upsample_backward: scale must be positive");
    const int64_t total = N * C * H * W;
    if (total == 0)
        return ODL_OK;
    const dim3 grid((unsigned)odl::ceil_div(total, kBlock)), block(kBlock);
    hipStream_t st = odl::as_stream(stream);
#define ODL_UPS_BWD(T)                                                                                                        \
    hipLaunchKernelGGL(upsample_nearest_bwd_any_kernel<T>, grid, block, 0, st, static_cast<const T *>(gy), static_cast<T *>(gx), \
                       total, H, W, OH, OW, scale_h, scale_w)
    switch (dtype)
    {
        case 1: ODL_UPS_BWD(double); break;
        case 2: ODL_UPS_BWD(int8_t); break;
        case 3: ODL_UPS_BWD(int32_t); break;
        case 4: ODL_UPS_BWD(int64_t); break;
        case 5: ODL_UPS_BWD(uint8_t); break;
        default: return odl::fail(ODL_ERR_INVALID_ARG, "upsample_backward: unknown element type code %d", dtype);
    }
#undef ODL_UPS_BWD
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

}  // extern "C"
