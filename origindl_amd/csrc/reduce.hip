// Reductions and broadcast of the backend: Mat::sum / sum_to / max / broadcast_to and the conv bias gradient.
// All of them are bandwidth-bound streams over HBM: loads are coalesced (16 bytes per lane where the layout
// allows), partial sums are combined with wave64 shuffles and one LDS hop, and long reductions are split over
// enough workgroups to fill 256 CUs, the partials being summed by a second small kernel in a fixed order —
// results do not depend on scheduling (no float atomics anywhere).
// Behaviour matched: src/mat/origin/cpu/math/{sum,sum_to,max,broadcast}.cpp and
// include/origin/mat/origin/device_common/operation_templates.h:259-495.
#include <algorithm>
#include <cfloat>
#include <cstdint>

#include "odl_common.h"
#include "reduce_small.h"

#include <mutex>

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace
{
constexpr int kBlock = 256;

inline size_t align256(size_t b)
{
    return (b + 255) & ~(size_t)255;
}

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

// sum over the whole workgroup (kBlock threads); the result is valid in thread 0
__device__ inline float block_sum(float v)
{
    __shared__ float part[kBlock / 64];
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
    if (threadIdx.x == 0)
        for (int i = 0; i < kBlock / 64; ++i)
            s += part[i];
    __syncthreads();
    return s;
}

// ---- rows: src[rows][len] (len contiguous) -> dst[rows]; grid (splits, rows); dst index = row*splits + split
__global__ void row_sum_block_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t len,
                                     int64_t chunk)
{
    const int64_t row = blockIdx.y;
    const int64_t beg = (int64_t)blockIdx.x * chunk;
    const int64_t end = (beg + chunk < len) ? beg + chunk : len;
    const float *p = src + row * len;
    float acc = 0.f;
    // 16-byte loads once the pointer is aligned; head and tail one float at a time
    int64_t i = beg + threadIdx.x;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(p + beg);
    int64_t head = ((16 - (addr & 15)) & 15) / 4;
    if (head > end - beg)
        head = end - beg;
    if ((int64_t)threadIdx.x < head)
        acc += p[i];
    const int64_t vbeg = beg + head;
    const int64_t nvec = (end - vbeg) / 4;
    const f32x4 *pv = reinterpret_cast<const f32x4 *>(p + vbeg);
    f32x4 a4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
    for (int64_t v = threadIdx.x; v < nvec; v += kBlock)  // (unrolled: eight loads on their way, the additions in the same order)
        a4 += pv[v];
    acc += (a4[0] + a4[1]) + (a4[2] + a4[3]);
    for (int64_t t = vbeg + nvec * 4 + threadIdx.x; t < end; t += kBlock)
        acc += p[t];
    const float s = block_sum(acc);
    if (threadIdx.x == 0)
        dst[row * gridDim.x + blockIdx.x] = s;
}

// one wave per row, for many short rows
__global__ void row_sum_wave_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t rows, int64_t len)
{
    const int64_t row = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    const float *p = src + row * len;
    float acc = 0.f;
#pragma unroll 8
    for (int64_t i = threadIdx.x & 63; i < len; i += 64)
        acc += p[i];
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0)
        dst[row] = acc;
}

// ---- columns: src[outer][axis][inner] -> dst[split][outer][inner]
// One thread owns VEC adjacent columns (a workgroup covers 256*VEC contiguous floats of every row it reads) and
// walks its slice of the axis with eight independent loads in flight.
template <int VEC>
__global__ __launch_bounds__(kBlock) void col_sum_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                          int64_t outer, int64_t axis, int64_t inner, int64_t chunk)
{
    const int64_t iq = inner / VEC;  // VEC == 4 only when inner % 4 == 0
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= outer * iq)
        return;
    const int64_t o = t / iq, i = (t % iq) * VEC;
    const int64_t beg = (int64_t)blockIdx.y * chunk;
    const int64_t end = (beg + chunk < axis) ? beg + chunk : axis;
    const float *p = src + (o * axis) * inner + i;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e)
        acc[e] = 0.f;
    int64_t a = beg;
    for (; a + 8 <= end; a += 8)
    {
        float v[8][VEC];
#pragma unroll
        for (int u = 0; u < 8; ++u)
        {
            if (VEC == 4)
            {
                const f32x4 q = *reinterpret_cast<const f32x4 *>(p + (a + u) * inner);
                v[u][0] = q[0], v[u][1 % VEC] = q[1], v[u][2 % VEC] = q[2], v[u][3 % VEC] = q[3];
            }
            else
                v[u][0] = p[(a + u) * inner];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                acc[e] += v[u][e];
    }
    for (; a < end; ++a)
#pragma unroll
        for (int e = 0; e < VEC; ++e)
            acc[e] += p[a * inner + e];
    float *d = dst + ((int64_t)blockIdx.y * outer + o) * inner + i;
#pragma unroll
    for (int e = 0; e < VEC; ++e)
        d[e] = acc[e];
}

// ---- columns of a small tensor in ONE launch (a bias gradient of a few MB is bound by launch latency, not by HBM: the
// two-pass schedule above costs two launches and the gap between them). A workgroup owns CW*VEC adjacent columns of one
// `outer` slice; its 256 threads are CW column lanes x (256/CW) row groups, group g adds rows g, g+G, ... (eight loads
// in flight), the group sums meet in LDS and are added in group order.
template <int VEC, int CW>
__global__ __launch_bounds__(kBlock) void col_sum_small_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                                int64_t axis, int64_t inner)
{
    // (the two halves live in reduce_small.h: the classifier layers' backward launch runs them as one of its jobs)
    __shared__ typename odl::ColSumSmall<VEC, CW>::Sums sh;
    odl::ColSumSmall<VEC, CW>::accumulate(src, axis, inner, blockIdx.x, blockIdx.y, threadIdx.x, sh);
    __syncthreads();
    odl::ColSumSmall<VEC, CW>::finish(dst, inner, blockIdx.x, blockIdx.y, threadIdx.x, sh);
}

// dst[i] = sum over s of part[s*n + i]. 64 columns x 16 slice groups per workgroup: group g adds slices
// g, g+16, ... (coalesced along i), the group sums meet in LDS and are added in group order — a fixed order.
constexpr int kFoldGroups = 16;
__global__ __launch_bounds__(64 * kFoldGroups) void fold_partials_kernel(const float *__restrict__ part,
                                                                          float *__restrict__ dst, int64_t n, int splits)
{
    __shared__ float sh[kFoldGroups][64];
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int64_t i = (int64_t)blockIdx.x * 64 + lane;
    float acc = 0.f;
    if (i < n)
    {
        int z = grp;
        for (; z + 3 * kFoldGroups < splits; z += 4 * kFoldGroups)
        {
            const float v0 = part[(int64_t)z * n + i], v1 = part[(int64_t)(z + kFoldGroups) * n + i];
            const float v2 = part[(int64_t)(z + 2 * kFoldGroups) * n + i];
            const float v3 = part[(int64_t)(z + 3 * kFoldGroups) * n + i];
            acc += v0;
            acc += v1;
            acc += v2;
            acc += v3;
        }
        for (; z < splits; z += kFoldGroups)
            acc += part[(int64_t)z * n + i];
    }
    sh[grp][lane] = acc;
    __syncthreads();
    if (grp == 0 && i < n)
    {
        float s = sh[0][lane];
#pragma unroll
        for (int k = 1; k < kFoldGroups; ++k)
            s += sh[k][lane];
        dst[i] = s;
    }
}

// ---- conv bias gradient: gy[N][OC][P] -> part[oc][nsplit]; grid (nsplit, OC). A channel's N*P elements are one
// flat range cut into nsplit equal chunks, so every thread has work whatever the size of one image plane; each
// thread keeps four independent running sums (four loads in flight) that are added in a fixed order.
struct ChannelSumPlan
{
    int64_t chunk;  // elements of one channel per workgroup (a multiple of 4)
    int64_t ns;     // workgroups per channel
};

__host__ inline ChannelSumPlan plan_channel_sum(int64_t N, int64_t OC, int64_t P)
{
    const int64_t total = (N > 0 ? N : 0) * (P > 0 ? P : 0);
    int64_t want = odl::ceil_div(2048, OC > 0 ? OC : 1);  // about eight workgroups per CU over all channels
    int64_t chunk = odl::ceil_div(total > 0 ? total : 1, want);
    if (chunk < 2048)
        chunk = 2048;
    chunk = odl::ceil_div(chunk, 4) * 4;
    // a channel short enough for one workgroup (a few loads per thread) is summed in a single launch
    if (total <= 16 * 1024 && OC >= 64)
        chunk = odl::ceil_div(total > 0 ? total : 1, 4) * 4;
    ChannelSumPlan p{chunk, odl::ceil_div(total > 0 ? total : 1, chunk)};
    return p;
}

// one workgroup per channel when the single launch is the cheaper schedule: channels for at least half the compute
// units, or fewer channels (32 and up) of at most 400 KB each, which one compute unit reads in the time the second
// launch of the two-pass schedule would take; planes of whole quads
__host__ inline bool channel_sum_whole(int64_t N, int64_t OC, int64_t P)
{
    const int64_t per_channel = N * P;
    if (P % 4 != 0 || per_channel >= (1ll << 31))
        return false;
    return (OC * 2 >= odl::device_cus() && per_channel >= 32 * 1024) ||
           (OC >= 32 && per_channel >= 16 * 1024 && per_channel <= 100 * 1024);
}

template <bool V4>
__global__ __launch_bounds__(kBlock) void nchw_channel_sum_kernel(const float *__restrict__ gy, float *__restrict__ part,
                                                                   unsigned total, unsigned P, unsigned OC,
                                                                   unsigned chunk, odl::FastDiv by_plane)
{
    constexpr unsigned E = V4 ? 4 : 1;  // elements per load; V4 needs P % 4 == 0 and a 16-byte aligned gy
    const unsigned oc = blockIdx.y;
    const unsigned beg = blockIdx.x * chunk;
    const unsigned end = (beg + chunk < total) ? beg + chunk : total;
    const unsigned plane = P / E;  // loads per image plane
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (unsigned u0 = beg / E + threadIdx.x; u0 < end / E; u0 += 4 * kBlock)
    {
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const unsigned u = u0 + j * kBlock;
            if (u < end / E)
            {
                const unsigned n = odl::fastdiv(u, by_plane), v = u - n * plane;
                const float *p = gy + ((int64_t)n * OC + oc) * P + (int64_t)v * E;
                if (V4)
                {
                    const f32x4 q = *reinterpret_cast<const f32x4 *>(p);
                    acc[j] += (q[0] + q[1]) + (q[2] + q[3]);
                }
                else
                    acc[j] += *p;
            }
        }
    }
    const float s = block_sum((acc[0] + acc[1]) + (acc[2] + acc[3]));
    if (threadIdx.x == 0)
        part[(int64_t)oc * gridDim.x + blockIdx.x] = s;  // with one workgroup per channel `part` is the result itself
}

// The same sum with ONE workgroup of 1024 threads per channel, for tensors with enough channels to occupy half the chip
// or more: no partial sums, no second launch (which costs about as long as reading a quarter of C1's gradient). Each
// thread keeps eight 16-byte loads in flight — a lone workgroup per compute unit has to cover the memory latency by
// itself — and the running sums are added in a fixed order.
__global__ __launch_bounds__(1024) void nchw_channel_sum_whole_kernel(const float *__restrict__ gy, float *__restrict__ gb,
                                                                      unsigned total, unsigned P, unsigned OC,
                                                                      odl::FastDiv by_plane)
{
    constexpr unsigned U = 8;
    __shared__ float part[1024 / 64];
    const unsigned oc = blockIdx.x;
    const unsigned plane = P / 4, quads = total / 4;
    float acc[U];
#pragma unroll
    for (unsigned j = 0; j < U; ++j)
        acc[j] = 0.f;
    for (unsigned u0 = threadIdx.x; u0 < quads; u0 += U * 1024)
    {
        f32x4 q[U];
#pragma unroll
        for (unsigned j = 0; j < U; ++j)
        {
            const unsigned u = u0 + j * 1024;
            q[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (u < quads)
            {
                const unsigned n = odl::fastdiv(u, by_plane), v = u - n * plane;
                q[j] = *reinterpret_cast<const f32x4 *>(gy + ((int64_t)n * OC + oc) * P + (int64_t)v * 4);
            }
        }
#pragma unroll
        for (unsigned j = 0; j < U; ++j)
            acc[j] += (q[j][0] + q[j][1]) + (q[j][2] + q[j][3]);
    }
    float v = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        float s = 0.f;
        for (int i = 0; i < 1024 / 64; ++i)
            s += part[i];
        gb[oc] = s;
    }
}

// ---- max
__global__ void row_max_wave_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t rows, int64_t len)
{
    const int64_t row = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    const float *p = src + row * len;
    float m = -FLT_MAX;  // std::numeric_limits<float>::lowest(), max.cpp:96
#pragma unroll 8
    for (int64_t i = threadIdx.x & 63; i < len; i += 64)
        m = (m < p[i]) ? p[i] : m;
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0)
        dst[row] = m;
}

__global__ void col_max_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t outer, int64_t axis,
                               int64_t inner)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= outer * inner)
        return;
    const int64_t o = t / inner, i = t % inner;
    const float *p = src + o * axis * inner + i;
    float m = -FLT_MAX;
    for (int64_t a = 0; a < axis; ++a)
        m = (m < p[a * inner]) ? p[a * inner] : m;
    dst[t] = m;
}

// Merging a partial maximum into a float in memory with integer atomics: the bit patterns of non-negative floats order
// like signed integers, those of negative floats in reverse like unsigned ones. A partial maximum is never a NaN here
// (the scans skip them, as `m < v` does). Equal zeros of different sign end as +0.0f whatever their order.
__device__ inline void atomic_max_float(float *addr, float v)
{
    if (!(__float_as_uint(v) >> 31))
        atomicMax(reinterpret_cast<int *>(addr), __float_as_int(v));
    else
        atomicMin(reinterpret_cast<unsigned *>(addr), __float_as_uint(v));
}

// Maximum over the middle axis of [outer, axis, inner] for long axes: lanes along `inner`, a workgroup scans one chunk
// of the axis for 256 columns; with one chunk the result is stored, with several it is merged into a destination that
// col_max_fill_kernel has set to the starting value.
__global__ __launch_bounds__(256) void col_max_chunk_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t axis,
                                                             int64_t inner, unsigned tiles_i, unsigned chunks, int64_t chunk_len)
{
    unsigned b = blockIdx.x;
    const unsigned ti = b % tiles_i;
    b /= tiles_i;
    const unsigned ch = b % chunks, o = b / chunks;
    const int64_t i = (int64_t)ti * 256 + threadIdx.x;
    if (i >= inner)
        return;
    const int64_t a0 = (int64_t)ch * chunk_len, a1 = a0 + chunk_len < axis ? a0 + chunk_len : axis;
    const float *p = src + ((int64_t)o * axis + a0) * inner + i;
    float m = -FLT_MAX;
#pragma unroll 8
    for (int64_t a = a0; a < a1; ++a, p += inner)
    {
        const float v = *p;
        m = (m < v) ? v : m;
    }
    if (chunks == 1)
        dst[(int64_t)o * inner + i] = m;
    else
        atomic_max_float(dst + (int64_t)o * inner + i, m);
}

// The same for columns in fours (inner % 4 == 0, 16-byte aligned rows): a wave reads 1 KB of a row per load and the
// sixteen waves of a workgroup take every sixteenth row of the chunk; the waves' maxima meet in LDS and one merge per
// column and workgroup goes to memory — the merges of one column are served one after the other by the L2, so their
// number per column (the number of chunks), not the scan, was most of the kernel above on a long axis.
constexpr int kMaxWaves = 16;
__global__ __launch_bounds__(64 * kMaxWaves) void col_max_chunk4_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t axis,
                                                              int64_t inner, unsigned tiles_i, unsigned chunks, int64_t chunk_len)
{
    __shared__ f32x4 part[kMaxWaves - 1][64];
    unsigned b = blockIdx.x;
    const unsigned ti = b % tiles_i;
    b /= tiles_i;
    const unsigned ch = b % chunks, o = b / chunks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t i = (int64_t)ti * 256 + 4 * lane;
    const bool live = i < inner;
    const int64_t a0 = (int64_t)ch * chunk_len, a1 = a0 + chunk_len < axis ? a0 + chunk_len : axis;
    f32x4 m = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
    if (live)
    {
        const float *p = src + ((int64_t)o * axis + a0 + wave) * inner + i;
        const int64_t step = kMaxWaves * inner;
        int64_t a = a0 + wave;
        for (; a + 7 * kMaxWaves < a1; a += 8 * kMaxWaves, p += 8 * step)
        {
            f32x4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = *reinterpret_cast<const f32x4 *>(p + u * step);
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    m[e] = (m[e] < v[u][e]) ? v[u][e] : m[e];
        }
        for (; a < a1; a += kMaxWaves, p += step)
        {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(p);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                m[e] = (m[e] < v[e]) ? v[e] : m[e];
        }
    }
    if (wave > 0)
        part[wave - 1][lane] = m;
    __syncthreads();
    if (wave > 0 || !live)
        return;
#pragma unroll
    for (int w = 0; w < kMaxWaves - 1; ++w)
    {
        const f32x4 v = part[w][lane];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            m[e] = (m[e] < v[e]) ? v[e] : m[e];
    }
    float *d = dst + (int64_t)o * inner + i;
    if (chunks == 1)
        *reinterpret_cast<f32x4 *>(d) = m;
    else
    {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            atomic_max_float(d + e, m[e]);
    }
}

__global__ void max_fill_kernel(float *__restrict__ dst, int64_t n, const float *first)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n)
    {
        // max over an axis starts from lowest(); the whole-tensor maximum from the first element, and stays a NaN if that
        // is one (nothing compares greater): the canonical NaN's bits lose to no merge
        float v = -FLT_MAX;
        if (first)
            v = (first[0] == first[0]) ? first[0] : __uint_as_float(0x7fc00000u);
        dst[t] = v;
    }
}

// whole-tensor maximum over many workgroups: 16-byte loads where the base allows, partial maxima merged as above
__global__ __launch_bounds__(256) void max_all_part_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t n)
{
    __shared__ float part[256 / 64];
    float m = src[0];  // max.cpp:30-35 starts from the first element; scanning it again changes nothing
    const int64_t stride = (int64_t)gridDim.x * 256;
    if ((reinterpret_cast<uintptr_t>(src) & 15) == 0)
    {
        const f32x4 *pv = reinterpret_cast<const f32x4 *>(src);
        const int64_t nq = n / 4;
        for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < nq; q += stride)
        {
            const f32x4 v = pv[q];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                m = (m < v[e]) ? v[e] : m;
        }
        for (int64_t i = nq * 4 + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
            m = (m < src[i]) ? src[i] : m;
    }
    else
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
            m = (m < src[i]) ? src[i] : m;
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int i = 1; i < 256 / 64; ++i)
            m = (m < part[i]) ? part[i] : m;
        if (m == m)  // a NaN first element: the destination already holds the answer
            atomic_max_float(dst, m);
    }
}

__global__ void max_all_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t n)
{
    __shared__ float part[1024 / 64];
    float m = src[0];  // max.cpp:30-35 starts from the first element
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x)
        m = (m < src[i]) ? src[i] : m;
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (unsigned i = 1; i < blockDim.x / 64; ++i)
            m = (m < part[i]) ? part[i] : m;
        dst[0] = m;
    }
}

// ---- broadcast: right-aligned, a source dim of size 1 reads index 0
struct BcastDims
{
    int nd;
    int64_t dshape[8];
    int64_t sstride[8];  // 0 where the source dim is 1 or absent
};

__global__ void broadcast_kernel(const float *__restrict__ src, float *__restrict__ dst, int64_t total, BcastDims d)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    int64_t r = t, si = 0;
    for (int k = d.nd - 1; k >= 0; --k)
    {
        si += (r % d.dshape[k]) * d.sstride[k];
        r /= d.dshape[k];
    }
    dst[t] = src[si];
}

// The same over merged dimensions, four consecutive outputs per thread: neighbouring target dimensions that are both
// copied or both repeated count as one, the innermost merged extent is a multiple of 4, all counts fit 32 bits. A repeated
// innermost dimension splats one source value, a copied one loads 16 bytes.
struct BcastQuads
{
    int nd;
    unsigned dshape[8];  // merged target extents, the innermost in quads
    odl::FastDiv div[8];
    unsigned sstride[8];  // in elements; 0 where the source is repeated
};

__global__ __launch_bounds__(256) void broadcast_quads_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                               unsigned quads, BcastQuads d)
{
    const unsigned t = blockIdx.x * 256u + threadIdx.x;
    if (t >= quads)
        return;
    const int last = d.nd - 1;
    unsigned r = odl::fastdiv(t, d.div[last]);
    unsigned si = (t - r * d.dshape[last]) * 4u * d.sstride[last];
    for (int k = last - 1; k >= 0; --k)
    {
        const unsigned q = odl::fastdiv(r, d.div[k]);
        si += (r - q * d.dshape[k]) * d.sstride[k];
        r = q;
    }
    f32x4 v;
    if (d.sstride[last])
        v = *reinterpret_cast<const f32x4 *>(src + si);
    else
    {
        const float x = src[si];
        v = f32x4{x, x, x, x};
    }
    reinterpret_cast<f32x4 *>(dst)[t] = v;
}

int64_t prod(const int64_t *s, int n)
{
    int64_t p = 1;
    for (int i = 0; i < n; ++i)
        p *= s[i];
    return p;
}

// how a [outer, axis, inner] sum is scheduled
struct SumPlan
{
    bool rows;      // inner == 1
    bool wave_rows; // many short rows: one wave each, no workspace
    int splits;
    int64_t chunk;
    size_t ws_bytes;
};

using odl::small_cols;  // (reduce_small.h)

SumPlan plan_sum(int64_t outer, int64_t axis, int64_t inner)
{
    SumPlan p{};
    p.rows = (inner == 1);
    if (p.rows)
    {
        if (outer >= 1024 || axis <= 2048)
        {
            p.wave_rows = true;
            p.splits = 1;
            return p;
        }
        int64_t s = odl::ceil_div(1024, outer);
        const int64_t max_s = odl::ceil_div(axis, 4096);
        if (s > max_s)
            s = max_s;
        if (s < 1)
            s = 1;
        p.chunk = odl::ceil_div(odl::ceil_div(axis, s), 4) * 4;
        p.splits = (int)odl::ceil_div(axis, p.chunk);
        p.ws_bytes = p.splits > 1 ? (size_t)(outer * p.splits) * sizeof(float) : 0;
        return p;
    }
    if (small_cols(outer, axis, inner))
    {
        p.splits = 1;
        p.chunk = axis;
        return p;
    }
    const int64_t vec = (inner % 4 == 0) ? 4 : 1;
    const int64_t col_blocks = odl::ceil_div(outer * (inner / vec), kBlock);
    // ~2048 workgroups (8 per CU) is where this access pattern streams fastest on 256 CUs
    int64_t s = odl::ceil_div(2048, col_blocks);
    if (s > axis / 16)
        s = axis / 16;
    if (s < 1)
        s = 1;
    if (s > 512)
        s = 512;
    p.chunk = odl::ceil_div(odl::ceil_div(axis, s), 8) * 8;
    p.splits = (int)odl::ceil_div(axis, p.chunk > 0 ? p.chunk : 1);
    if (p.splits < 1)
        p.splits = 1;
    p.ws_bytes = p.splits > 1 ? (size_t)p.splits * outer * inner * sizeof(float) : 0;
    return p;
}

int sum_axis_launch(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst, void *workspace,
                    size_t workspace_bytes, hipStream_t st)
{
    const int64_t nout = outer * inner;
    if (nout == 0)
        return ODL_OK;
    if (axis == 0)
    {
        return odl::fill_launch(dst, nout, 0.f, st);
    }
    SumPlan p = plan_sum(outer, axis, inner);
    if (p.splits > 1 && (workspace == nullptr || workspace_bytes < p.ws_bytes))
        return odl::fail(ODL_ERR_INVALID_ARG, "sum: workspace of %zu bytes required, got %zu", p.ws_bytes,
                         workspace_bytes);
    if (p.rows)
    {
        if (p.wave_rows)
        {
            hipLaunchKernelGGL(row_sum_wave_kernel, dim3((unsigned)odl::ceil_div(outer, kBlock / 64)), dim3(kBlock), 0,
                               st, src, dst, outer, axis);
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        }
        ODL_REQUIRE(outer < 65536, "sum: too many rows for the split schedule");
        float *part = p.splits > 1 ? static_cast<float *>(workspace) : dst;
        hipLaunchKernelGGL(row_sum_block_kernel, dim3((unsigned)p.splits, (unsigned)outer), dim3(kBlock), 0, st, src,
                           part, axis, p.chunk);
        ODL_LAUNCH_CHECK();
        if (p.splits > 1)
        {
            hipLaunchKernelGGL(row_sum_wave_kernel, dim3((unsigned)odl::ceil_div(outer, kBlock / 64)), dim3(kBlock), 0,
                               st, part, dst, outer, (int64_t)p.splits);
            ODL_LAUNCH_CHECK();
        }
        return ODL_OK;
    }
    const bool v4 = (inner % 4 == 0) && (reinterpret_cast<uintptr_t>(src) % 16 == 0);
    if (small_cols(outer, axis, inner))
    {
        if (v4)
            hipLaunchKernelGGL((col_sum_small_kernel<4, 8>), dim3((unsigned)odl::ceil_div(inner, 32), (unsigned)outer),
                               dim3(kBlock), 0, st, src, dst, axis, inner);
        else
            hipLaunchKernelGGL((col_sum_small_kernel<1, 16>), dim3((unsigned)odl::ceil_div(inner, 16), (unsigned)outer),
                               dim3(kBlock), 0, st, src, dst, axis, inner);
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    }
    const int64_t cols = outer * (v4 ? inner / 4 : inner);
    float *part = p.splits > 1 ? static_cast<float *>(workspace) : dst;
    const dim3 grid((unsigned)odl::ceil_div(cols, kBlock), (unsigned)p.splits);
    if (v4)
        hipLaunchKernelGGL(col_sum_kernel<4>, grid, dim3(kBlock), 0, st, src, part, outer, axis, inner, p.chunk);
    else
        hipLaunchKernelGGL(col_sum_kernel<1>, grid, dim3(kBlock), 0, st, src, part, outer, axis, inner, p.chunk);
    ODL_LAUNCH_CHECK();
    if (p.splits > 1)
    {
        hipLaunchKernelGGL(fold_partials_kernel, dim3((unsigned)odl::ceil_div(nout, 64)), dim3(64 * kFoldGroups), 0, st,
                           part, dst, nout, p.splits);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}

// sum_to.cpp:36-72: which dims are reduced (LEFT-aligned), and the [outer,axis,inner] passes that do it,
// one per maximal run of adjacent reduced dims, last run first so earlier extents stay valid.
struct SumToPlan
{
    int rc;  // ODL_OK, or the error the reference would throw
    bool copy;
    int npass;
    int64_t outer[8], axis[8], inner[8];
    size_t ws_bytes;  // two ping-pong intermediates + the largest per-pass workspace
    size_t inter_bytes;
    size_t pass_ws;
};

SumToPlan plan_sum_to(const int64_t *ss, int sn, const int64_t *ts, int tn)
{
    SumToPlan p{};
    p.rc = ODL_OK;
    if (sn > 8 || tn > 8 || sn < 0 || tn < 0)
    {
        p.rc = ODL_ERR_INVALID_ARG;
        return p;
    }
    bool same = (sn == tn);
    for (int i = 0; same && i < sn; ++i)
        same = (ss[i] == ts[i]);
    if (same)
    {
        p.copy = true;
        return p;
    }
    const int64_t se = prod(ss, sn), te = prod(ts, tn);
    if (te > se)
    {
        p.rc = ODL_ERR_RUNTIME;  // sum_to.cpp:24-28
        return p;
    }
    bool red[8] = {false};
    const int mind = sn < tn ? sn : tn;
    for (int i = 0; i < mind; ++i)
        red[i] = (ts[i] == 1 && ss[i] > 1);
    for (int i = tn; i < sn; ++i)
        red[i] = true;
    int64_t kept = 1;
    for (int i = 0; i < sn; ++i)
        if (!red[i])
            kept *= ss[i];
    if (kept != te)
    {
        p.rc = ODL_ERR_INVALID_ARG;  // the final reshape throws
        return p;
    }
    int64_t cur[8];
    for (int i = 0; i < sn; ++i)
        cur[i] = ss[i];
    int i = sn - 1;
    size_t inter = 0;
    while (i >= 0)
    {
        if (!red[i])
        {
            --i;
            continue;
        }
        int j = i;
        while (j - 1 >= 0 && red[j - 1])
            --j;
        const int q = p.npass++;
        p.outer[q] = prod(cur, j);
        p.axis[q]  = prod(cur + j, i - j + 1);
        p.inner[q] = prod(cur + i + 1, sn - i - 1);
        for (int d = j; d <= i; ++d)
            cur[d] = 1;
        const size_t w = plan_sum(p.outer[q], p.axis[q], p.inner[q]).ws_bytes;
        if (w > p.pass_ws)
            p.pass_ws = w;
        const size_t ob = (size_t)(p.outer[q] * p.inner[q]) * sizeof(float);
        if (ob > inter)
            inter = ob;
        i = j - 1;
    }
    p.inter_bytes = p.npass > 1 ? align256(inter) : 0;
    p.ws_bytes = 2 * p.inter_bytes + align256(p.pass_ws);
    return p;
}
}  // namespace

namespace odl
{
size_t sum_nchw_channels_workspace(int64_t N, int64_t OC, int64_t P)
{
    return (size_t)((OC > 0 ? OC : 0) * plan_channel_sum(N, OC, P).ns) * sizeof(float);
}

int sum_nchw_channels_launch(const float *gy, int64_t N, int64_t OC, int64_t P, float *gb, void *workspace,
                             size_t workspace_bytes, hipStream_t st)
{
    if (OC == 0)
        return ODL_OK;
    ODL_REQUIRE(N >= 0 && OC > 0 && OC < 65536 && P >= 0, "conv bias gradient: bad shape");
    ODL_REQUIRE(N * P < (1ll << 31), "conv bias gradient: more than 2^31 elements per channel");
    if (channel_sum_whole(N, OC, P) && reinterpret_cast<uintptr_t>(gy) % 16 == 0)
    {
        hipLaunchKernelGGL(nchw_channel_sum_whole_kernel, dim3((unsigned)OC), dim3(1024), 0, st, gy, gb, (unsigned)(N * P),
                           (unsigned)P, (unsigned)OC, odl::make_fastdiv((unsigned)(P / 4)));
        ODL_LAUNCH_CHECK();
        return ODL_OK;
    }
    const ChannelSumPlan pl = plan_channel_sum(N, OC, P);
    ODL_REQUIRE(pl.ns < 65536, "conv bias gradient: too many workgroups per channel");
    const size_t need = (size_t)(OC * pl.ns) * sizeof(float);
    ODL_REQUIRE(pl.ns == 1 || (workspace != nullptr && workspace_bytes >= need),
                "conv bias gradient: workspace of %zu bytes required, got %zu", need, workspace_bytes);
    float *part = pl.ns == 1 ? gb : static_cast<float *>(workspace);
    const bool v4 = P % 4 == 0 && reinterpret_cast<uintptr_t>(gy) % 16 == 0;
    const dim3 grid((unsigned)pl.ns, (unsigned)OC), block(kBlock);
    if (v4)
        hipLaunchKernelGGL((nchw_channel_sum_kernel<true>), grid, block, 0, st, gy, part, (unsigned)(N * P), (unsigned)P,
                           (unsigned)OC, (unsigned)pl.chunk, odl::make_fastdiv((unsigned)(P / 4)));
    else
        hipLaunchKernelGGL((nchw_channel_sum_kernel<false>), grid, block, 0, st, gy, part, (unsigned)(N * P), (unsigned)P,
                           (unsigned)OC, (unsigned)pl.chunk, odl::make_fastdiv((unsigned)(P > 0 ? P : 1)));
    ODL_LAUNCH_CHECK();
    if (pl.ns > 1)
    {
        hipLaunchKernelGGL(row_sum_wave_kernel, dim3((unsigned)ceil_div(OC, kBlock / 64)), dim3(kBlock), 0, st, part, gb,
                           OC, pl.ns);
        ODL_LAUNCH_CHECK();
    }
    return ODL_OK;
}
}  // namespace odl

extern "C" {

size_t odl_hip_sum_axis_workspace_bytes(int64_t outer, int64_t axis, int64_t inner)
{
    if (outer <= 0 || axis <= 0 || inner <= 0)
        return 0;
    return plan_sum(outer, axis, inner).ws_bytes;
}

int odl_hip_sum_axis(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst, void *workspace,
                     size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, "sum: negative extent");
    return sum_axis_launch(src, outer, axis, inner, dst, workspace, workspace_bytes, odl::as_stream(stream));
}

// ---- the same reduction for callers that cannot allocate (and so cannot bring a workspace): the partial sums go to
// an array that is part of the library's device image. Every device holds its own copy at its own address; the name
// `scratch` is only the host-side handle of that symbol, so launches get the address hipGetSymbolAddress reports.
}  // extern "C"

namespace
{
constexpr size_t kScratchBytes = (size_t)8 << 20;
// (kept in the device image although no kernel names it: kernels receive its address as an argument)
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kScratchBytes];

std::mutex g_scratch_mutex;
void *g_scratch_ptr[64] = {nullptr};  // per device, resolved on the first call with that device current

int scratch_of_current_device(hipStream_t st, void **out)
{
    int dev = -1;
    ODL_HIP_CHECK(hipGetDevice(&dev));
    ODL_REQUIRE(dev >= 0 && dev < 64, "sum_axis_noalloc: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr)
    {
        // resolving the symbol may load the device image: not something to do while a stream is recording
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        ODL_HIP_CHECK(hipStreamIsCapturing(st, &cap));
        if (cap != hipStreamCaptureStatusNone)
            return odl::fail(ODL_ERR_RUNTIME, "sum_axis_noalloc: the first call on a device must come outside stream capture");
        void *ptr = nullptr;
        ODL_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr)
            return odl::fail(ODL_ERR_RUNTIME, "sum_axis_noalloc: the scratch array has no device address");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return ODL_OK;
}
}  // namespace

extern "C" {
size_t odl_hip_sum_axis_noalloc_max_bytes(void)
{
    return kScratchBytes;
}

int odl_hip_sum_axis_noalloc(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, "sum: negative extent");
    const size_t need = (outer > 0 && axis > 0 && inner > 0) ? plan_sum(outer, axis, inner).ws_bytes : 0;
    if (need > kScratchBytes)
        return odl::fail(ODL_ERR_INVALID_ARG,
                         "sum_axis_noalloc: [%lld, %lld, %lld] needs %zu bytes of partial sums, the built-in scratch holds %zu; "
                         "use odl_hip_sum_axis with a workspace",
                         (long long)outer, (long long)axis, (long long)inner, need, kScratchBytes);
    void *ws = nullptr;
    if (need > 0)
    {
        const int rc = scratch_of_current_device(odl::as_stream(stream), &ws);
        if (rc != ODL_OK)
            return rc;
    }
    // every partial the fold reads is written by the pass before it in the same call: nothing has to start at zero
    return sum_axis_launch(src, outer, axis, inner, dst, ws, need, odl::as_stream(stream));
}

size_t odl_hip_sum_all_workspace_bytes(int64_t n)
{
    return odl_hip_sum_axis_workspace_bytes(1, n, 1);
}

int odl_hip_sum_all(const float *src, int64_t n, float *dst, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(n >= 0, "sum: negative extent");
    return sum_axis_launch(src, 1, n, 1, dst, workspace, workspace_bytes, odl::as_stream(stream));
}

int odl_hip_max_axis(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, "max: negative extent");
    if (outer * inner == 0)
        return ODL_OK;
    hipStream_t st = odl::as_stream(stream);
    if (inner == 1)
        hipLaunchKernelGGL(row_max_wave_kernel, dim3((unsigned)odl::ceil_div(outer, kBlock / 64)), dim3(kBlock), 0, st,
                           src, dst, outer, axis);
    else if (axis >= 64 && outer * inner < (int64_t)64 * 256 * odl::device_cus() && outer < (1 << 20))
    {
        // too few columns to fill the chip with a thread each: chunks of the axis per workgroup
        const int64_t tiles_i = odl::ceil_div(inner, 256);
        const bool quads = inner % 4 == 0 && (reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % 16 == 0;
        // workgroups of 256 threads, eight per compute unit; of 1024 threads (columns in fours), two
        int64_t chunks = odl::ceil_div((int64_t)(quads ? 2 : 8) * odl::device_cus(), outer * tiles_i);
        if (chunks > axis / 32)
            chunks = axis / 32;
        if (chunks < 1)
            chunks = 1;
        const int64_t chunk_len = odl::ceil_div(axis, chunks);
        chunks = odl::ceil_div(axis, chunk_len);
        ODL_REQUIRE(outer * chunks * tiles_i < (1ll << 31), "max: too many workgroups");
        if (chunks > 1)
        {
            hipLaunchKernelGGL(max_fill_kernel, dim3((unsigned)odl::ceil_div(outer * inner, kBlock)), dim3(kBlock), 0, st, dst,
                               outer * inner, (const float *)nullptr);
            ODL_LAUNCH_CHECK();
        }
        if (quads)
            hipLaunchKernelGGL(col_max_chunk4_kernel, dim3((unsigned)(outer * chunks * tiles_i)), dim3(64 * kMaxWaves), 0, st, src, dst,
                               axis, inner, (unsigned)tiles_i, (unsigned)chunks, chunk_len);
        else
            hipLaunchKernelGGL(col_max_chunk_kernel, dim3((unsigned)(outer * chunks * tiles_i)), dim3(256), 0, st, src, dst,
                               axis, inner, (unsigned)tiles_i, (unsigned)chunks, chunk_len);
    }
    else
        hipLaunchKernelGGL(col_max_kernel, dim3((unsigned)odl::ceil_div(outer * inner, kBlock)), dim3(kBlock), 0, st,
                           src, dst, outer, axis, inner);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

int odl_hip_max_all(const float *src, int64_t n, float *dst, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(n > 0, "max: empty input");
    if (n < (1 << 16))
        hipLaunchKernelGGL(max_all_kernel, dim3(1), dim3(1024), 0, odl::as_stream(stream), src, dst, n);
    else
    {
        hipLaunchKernelGGL(max_fill_kernel, dim3(1), dim3(64), 0, odl::as_stream(stream), dst, (int64_t)1, src);
        ODL_LAUNCH_CHECK();
        int64_t wgs = odl::ceil_div(n, 256 * 16);
        if (wgs > (int64_t)8 * odl::device_cus())
            wgs = (int64_t)8 * odl::device_cus();
        hipLaunchKernelGGL(max_all_part_kernel, dim3((unsigned)wgs), dim3(256), 0, odl::as_stream(stream), src, dst, n);
    }
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

size_t odl_hip_sum_to_workspace_bytes(const int64_t *host_src_shape, int src_ndim, const int64_t *host_dst_shape,
                                      int dst_ndim)
{
    const SumToPlan p = plan_sum_to(host_src_shape, src_ndim, host_dst_shape, dst_ndim);
    return p.rc == ODL_OK ? p.ws_bytes : 0;
}

int odl_hip_sum_to(const float *src, const int64_t *host_src_shape, int src_ndim, const int64_t *host_dst_shape,
                   int dst_ndim, float *dst, void *workspace, size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    hipStream_t st = odl::as_stream(stream);
    const SumToPlan p = plan_sum_to(host_src_shape, src_ndim, host_dst_shape, dst_ndim);
    if (p.rc == ODL_ERR_RUNTIME)
        return odl::fail(ODL_ERR_RUNTIME, "sum_to: Target shape cannot have more elements than source tensor");
    if (p.rc != ODL_OK)
        return odl::fail(p.rc, "sum_to: source shape cannot be reduced to the target shape (left-aligned rule)");
    if (p.copy)
    {
        const int64_t n = prod(host_src_shape, src_ndim);
        if (n && dst != src)
            ODL_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)n * sizeof(float), hipMemcpyDeviceToDevice, st));
        return ODL_OK;
    }
    if (p.npass == 0)  // only size-1 dims differ: a reshape
    {
        const int64_t n = prod(host_src_shape, src_ndim);
        if (n && dst != src)
            ODL_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)n * sizeof(float), hipMemcpyDeviceToDevice, st));
        return ODL_OK;
    }
    ODL_REQUIRE(p.ws_bytes == 0 || (workspace != nullptr && workspace_bytes >= p.ws_bytes),
                "sum_to: workspace of %zu bytes required, got %zu", p.ws_bytes, workspace_bytes);
    char *ws = static_cast<char *>(workspace);
    float *inter[2] = {reinterpret_cast<float *>(ws), reinterpret_cast<float *>(ws + p.inter_bytes)};
    void *pass_ws = ws + 2 * p.inter_bytes;
    const float *cur = src;
    for (int q = 0; q < p.npass; ++q)
    {
        float *out = (q == p.npass - 1) ? dst : inter[q & 1];
        int rc = sum_axis_launch(cur, p.outer[q], p.axis[q], p.inner[q], out, pass_ws, p.pass_ws, st);
        if (rc != ODL_OK)
            return rc;
        cur = out;
    }
    return ODL_OK;
}

size_t odl_hip_sum_nchw_channels_workspace_bytes(int64_t N, int64_t OC, int64_t P)
{
    return odl::sum_nchw_channels_workspace(N, OC, P);
}

int odl_hip_sum_nchw_channels(const float *gy, int64_t N, int64_t OC, int64_t P, float *gb, void *workspace,
                              size_t workspace_bytes, void *stream)
{
    ODL_REQUIRE_DEVICE();
    return odl::sum_nchw_channels_launch(gy, N, OC, P, gb, workspace, workspace_bytes, odl::as_stream(stream));
}

int odl_hip_broadcast_to(const float *src, const int64_t *host_src_shape, int src_ndim, const int64_t *host_dst_shape,
                         int dst_ndim, float *dst, void *stream)
{
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(src_ndim >= 0 && dst_ndim >= 0 && src_ndim <= 8 && dst_ndim <= 8, "broadcast_to: at most 8 dims");
    ODL_REQUIRE(src_ndim <= dst_ndim, "broadcast_to: source has more dims than the target");
    BcastDims d{};
    d.nd = dst_ndim;
    int64_t st = 1;
    for (int i = 0; i < dst_ndim; ++i)
    {
        const int dd = dst_ndim - 1 - i, sd = src_ndim - 1 - i;
        d.dshape[dd] = host_dst_shape[dd];
        d.sstride[dd] = 0;
        if (sd >= 0)
        {
            const int64_t ssz = host_src_shape[sd];
            ODL_REQUIRE(ssz == 1 || ssz == host_dst_shape[dd], "broadcast_to: dim %d of size %lld cannot become %lld", sd,
                        (long long)ssz, (long long)host_dst_shape[dd]);
            d.sstride[dd] = (ssz == 1) ? 0 : st;
            st *= ssz;
        }
    }
    const int64_t total = prod(host_dst_shape, dst_ndim);
    if (total == 0)
        return ODL_OK;
    {
        // merged dimensions, innermost first in the scan: extents of 1 dropped, neighbours of the same kind multiplied
        BcastQuads q{};
        int64_t mshape[8], mstride[8];
        int m = 0;
        for (int k = 0; k < dst_ndim; ++k)
        {
            if (d.dshape[k] == 1)
                continue;
            const bool rep = d.sstride[k] == 0;
            if (m > 0 && ((rep && mstride[m - 1] == 0) || (!rep && mstride[m - 1] == d.dshape[k] * d.sstride[k])))
                mshape[m - 1] *= d.dshape[k], mstride[m - 1] = d.sstride[k];
            else
                mshape[m] = d.dshape[k], mstride[m] = d.sstride[k], ++m;
        }
        const bool aligned = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
        bool ok = m >= 1 && total < (1ll << 32) && mshape[m - 1] % 4 == 0 && aligned;
        for (int k = 0; ok && k < m; ++k)
            ok = mshape[k] < (1ll << 31) && mstride[k] < (1ll << 31) && (k == m - 1 || mstride[k] % 4 == 0);
        if (ok)
        {
            q.nd = m;
            for (int k = 0; k < m; ++k)
            {
                q.dshape[k] = (unsigned)(k == m - 1 ? mshape[k] / 4 : mshape[k]);
                q.div[k] = odl::make_fastdiv(q.dshape[k]);
                q.sstride[k] = (unsigned)mstride[k];
            }
            const unsigned quads = (unsigned)(total / 4);
            hipLaunchKernelGGL(broadcast_quads_kernel, dim3((unsigned)odl::ceil_div(quads, 256)), dim3(256), 0,
                               odl::as_stream(stream), src, dst, quads, q);
            ODL_LAUNCH_CHECK();
            return ODL_OK;
        }
    }
    hipLaunchKernelGGL(broadcast_kernel, dim3((unsigned)odl::ceil_div(total, kBlock)), dim3(kBlock), 0,
                       odl::as_stream(stream), src, dst, total, d);
    ODL_LAUNCH_CHECK();
    return ODL_OK;
}

}  // extern "C"

// ------------------------------------------------------------------ the same operators in the other element types
// The reference dispatches max, broadcast_to and sum_to over its six element types
// (src/mat/origin/cuda/math/{max,broadcast_to,sum_to}.cu through device_common/type_dispatcher.h). float32 takes the
// kernels above; the other types take the plain forms below (one thread per output element).
extern "C" size_t odl_hip_dtype_size(int dtype);
extern "C" int odl_hip_sum_axis_dtype(int dtype, const void *src, int64_t outer, int64_t axis, int64_t inner, int through_float,
                                      void *dst, void *workspace, size_t workspace_bytes, void *stream);
extern "C" size_t odl_hip_sum_axis_dtype_workspace_bytes(int dtype, int64_t outer, int64_t axis, int64_t inner);

namespace
{
// std::numeric_limits<T>::lowest()
template <typename T>
__device__ inline T lowest_of();
template <>
__device__ inline double lowest_of<double>()
{
    return -DBL_MAX;
}
template <>
__device__ inline int8_t lowest_of<int8_t>()
{
    return INT8_MIN;
}
template <>
__device__ inline int32_t lowest_of<int32_t>()
{
    return INT32_MIN;
}
template <>
__device__ inline int64_t lowest_of<int64_t>()
{
    return INT64_MIN;
}
template <>
__device__ inline uint8_t lowest_of<uint8_t>()
{
    return 0;
}

// max.cpp:58-117: every output starts from lowest() and takes v where `m < v`
template <typename T>
__global__ void max_axis_any_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t outer, int64_t axis, int64_t inner)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= outer * inner)
        return;
    const int64_t o = t / inner, i = t - o * inner;
    const T *p = src + o * axis * inner + i;
    T m = lowest_of<T>();
    for (int64_t a = 0; a < axis; ++a)
    {
        const T v = p[a * inner];
        m = (m < v) ? v : m;
    }
    dst[t] = m;
}

// max.cpp:25-40: the whole tensor, starting from its first element (a NaN there stays: nothing compares greater). One
// workgroup; its threads' maxima are merged in thread order.
template <typename T>
__global__ __launch_bounds__(1024) void max_all_any_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t n)
{
    __shared__ T part[1024];
    T m = src[0];
    for (int64_t i = threadIdx.x; i < n; i += 1024)
    {
        const T v = src[i];
        m = (m < v) ? v : m;
    }
    part[threadIdx.x] = m;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        for (int i = 1; i < 1024; ++i)
            m = (m < part[i]) ? part[i] : m;
        dst[0] = m;
    }
}

template <typename T>
__global__ void broadcast_any_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t total, BcastDims d)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total)
        return;
    int64_t r = t, si = 0;
    for (int k = d.nd - 1; k >= 0; --k)
    {
        si += (r % d.dshape[k]) * d.sstride[k];
        r /= d.dshape[k];
    }
    dst[t] = src[si];
}

// f(T{}) for the element type of a code (include/origin/mat/basic_types.h:19-27), float32 excluded
template <typename F>
int with_other_type(int dt, const char *who, F &&f)
{
    switch (dt)
    {
        case 1: return f(double{});
        case 2: return f(int8_t{});
        case 3: return f(int32_t{});
        case 4: return f(int64_t{});
        case 5: return f(uint8_t{});
        default: return odl::fail(ODL_ERR_INVALID_ARG, "%s: unknown element type code %d", who, dt);
    }
}
}  // namespace

extern "C" {

int odl_hip_max_axis_dtype(int dtype, const void *src, int64_t outer, int64_t axis, int64_t inner, void *dst, void *stream)
{
    if (dtype == 0)
        return odl_hip_max_axis(static_cast<const float *>(src), outer, axis, inner, static_cast<float *>(dst), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(outer >= 0 && axis >= 0 && inner >= 0, "max: negative extent");
    if (outer * inner == 0)
        return ODL_OK;
    return with_other_type(dtype, "max", [&](auto tag) {
        using T = decltype(tag);
        hipLaunchKernelGGL(max_axis_any_kernel<T>, dim3((unsigned)odl::ceil_div(outer * inner, kBlock)), dim3(kBlock), 0,
                           odl::as_stream(stream), static_cast<const T *>(src), static_cast<T *>(dst), outer, axis, inner);
        ODL_LAUNCH_CHECK();
        return (int)ODL_OK;
    });
}

int odl_hip_max_all_dtype(int dtype, const void *src, int64_t n, void *dst, void *stream)
{
    if (dtype == 0)
        return odl_hip_max_all(static_cast<const float *>(src), n, static_cast<float *>(dst), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(n > 0, "max: empty input");
    return with_other_type(dtype, "max", [&](auto tag) {
        using T = decltype(tag);
        hipLaunchKernelGGL(max_all_any_kernel<T>, dim3(1), dim3(1024), 0, odl::as_stream(stream), static_cast<const T *>(src),
                           static_cast<T *>(dst), n);
        ODL_LAUNCH_CHECK();
        return (int)ODL_OK;
    });
}

int odl_hip_broadcast_to_dtype(int dtype, const void *src, const int64_t *host_src_shape, int src_ndim,
                               const int64_t *host_dst_shape, int dst_ndim, void *dst, void *stream)
{
    if (dtype == 0)
        return odl_hip_broadcast_to(static_cast<const float *>(src), host_src_shape, src_ndim, host_dst_shape, dst_ndim,
                                    static_cast<float *>(dst), stream);
    ODL_REQUIRE_DEVICE();
    ODL_REQUIRE(src_ndim >= 0 && dst_ndim >= 0 && src_ndim <= 8 && dst_ndim <= 8, "broadcast_to: at most 8 dims");
    ODL_REQUIRE(src_ndim <= dst_ndim, "broadcast_to: source has more dims than the target");
    BcastDims d{};
    d.nd = dst_ndim;
    int64_t st = 1;
    for (int i = 0; i < dst_ndim; ++i)
    {
        const int dd = dst_ndim - 1 - i, sd = src_ndim - 1 - i;
        d.dshape[dd] = host_dst_shape[dd];
        d.sstride[dd] = 0;
        if (sd >= 0)
        {
            const int64_t ssz = host_src_shape[sd];
            ODL_REQUIRE(ssz == 1 || ssz == host_dst_shape[dd], "broadcast_to: dim %d of size %lld cannot become %lld", sd,
                        (long long)ssz, (long long)host_dst_shape[dd]);
            d.sstride[dd] = (ssz == 1) ? 0 : st;
            st *= ssz;
        }
    }
    const int64_t total = prod(host_dst_shape, dst_ndim);
    if (total == 0)
        return ODL_OK;
    return with_other_type(dtype, "broadcast_to", [&](auto tag) {
        using T = decltype(tag);
        hipLaunchKernelGGL(broadcast_any_kernel<T>, dim3((unsigned)odl::ceil_div(total, kBlock)), dim3(kBlock), 0,
                           odl::as_stream(stream), static_cast<const T *>(src), static_cast<T *>(dst), total, d);
        ODL_LAUNCH_CHECK();
        return (int)ODL_OK;
    });
}

size_t odl_hip_sum_to_dtype_workspace_bytes(int dtype, const int64_t *host_src_shape, int src_ndim, const int64_t *host_dst_shape,
                                            int dst_ndim)
{
    if (dtype == 0)
        return odl_hip_sum_to_workspace_bytes(host_src_shape, src_ndim, host_dst_shape, dst_ndim);
    const SumToPlan p = plan_sum_to(host_src_shape, src_ndim, host_dst_shape, dst_ndim);
    if (p.rc != ODL_OK || p.copy || p.npass == 0)
        return 0;
    size_t inter = 0, pass = 0;
    for (int q = 0; q < p.npass; ++q)
    {
        inter = std::max(inter, (size_t)(p.outer[q] * p.inner[q]) * odl_hip_dtype_size(dtype));
        pass = std::max(pass, odl_hip_sum_axis_dtype_workspace_bytes(dtype, p.outer[q], p.axis[q], p.inner[q]));
    }
    inter = (inter + 255) & ~(size_t)255;
    return 2 * inter + ((pass + 255) & ~(size_t)255);
}

int odl_hip_sum_to_dtype(int dtype, const void *src, const int64_t *host_src_shape, int src_ndim, const int64_t *host_dst_shape,
                         int dst_ndim, void *dst, void *workspace, size_t workspace_bytes, void *stream)
{
    if (dtype == 0)
        return odl_hip_sum_to(static_cast<const float *>(src), host_src_shape, src_ndim, host_dst_shape, dst_ndim,
                              static_cast<float *>(dst), workspace, workspace_bytes, stream);
    ODL_REQUIRE_DEVICE();
    const size_t esz = odl_hip_dtype_size(dtype);
    ODL_REQUIRE(esz > 0, "sum_to: unknown element type code %d", dtype);
    hipStream_t st = odl::as_stream(stream);
    const SumToPlan p = plan_sum_to(host_src_shape, src_ndim, host_dst_shape, dst_ndim);
    if (p.rc == ODL_ERR_RUNTIME)
        return odl::fail(ODL_ERR_RUNTIME, "sum_to: Target shape cannot have more elements than source tensor");
    if (p.rc != ODL_OK)
        return odl::fail(p.rc, "sum_to: source shape cannot be reduced to the target shape (left-aligned rule)");
    if (p.copy || p.npass == 0)  // equal shapes, or only size-1 dims differ: a copy
    {
        const int64_t n = prod(host_src_shape, src_ndim);
        if (n && dst != src)
            ODL_HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)n * esz, hipMemcpyDeviceToDevice, st));
        return ODL_OK;
    }
    const size_t need = odl_hip_sum_to_dtype_workspace_bytes(dtype, host_src_shape, src_ndim, host_dst_shape, dst_ndim);
    ODL_REQUIRE(workspace != nullptr && workspace_bytes >= need, "sum_to: workspace of %zu bytes required, got %zu", need,
                workspace_bytes);
    size_t inter = 0, pass = 0;
    for (int q = 0; q < p.npass; ++q)
    {
        inter = std::max(inter, (size_t)(p.outer[q] * p.inner[q]) * esz);
        pass = std::max(pass, odl_hip_sum_axis_dtype_workspace_bytes(dtype, p.outer[q], p.axis[q], p.inner[q]));
    }
    inter = (inter + 255) & ~(size_t)255;
    char *ws = static_cast<char *>(workspace);
    void *buf[2] = {ws, ws + inter};
    void *pass_ws = ws + 2 * inter;
    const void *cur = src;
    for (int q = 0; q < p.npass; ++q)
    {
        void *out = (q == p.npass - 1) ? dst : buf[q & 1];
        const int rc = odl_hip_sum_axis_dtype(dtype, cur, p.outer[q], p.axis[q], p.inner[q], 0, out, pass_ws, pass, stream);
        if (rc != ODL_OK)
            return rc;
        cur = out;
    }
    return ODL_OK;
}

}  // extern "C"
