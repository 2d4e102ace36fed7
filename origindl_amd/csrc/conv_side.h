// The small independent jobs around the three products of a convolution's backward pass, as device functions that one
// launch can run side by side (each in its own workgroups of 1024 threads): the sum of the weight gradient's partial
// tiles, the bias gradient, and the filter copy the input-gradient kernel stages from. Launched one after the other they
// are three latencies of a few microseconds each, with start-up gaps between them; together they take as long as the
// longest of them.
#pragma once
#include "odl_common.h"

namespace odl
{
typedef float side_f32x4 __attribute__((ext_vector_type(4)));

// ---- weight gradient: gW = part[0] + part[1] + ... in slice order, moved from the tiles' [tile][64 oc][3 taps x 64
// channels] layout to gW[oc][c][kh][kw] (conv_wgrad.hip)
struct SideFold
{
    const float *part;
    float *gw;
    int slices, n4, tiles_oc, CK;  // n4: 16-byte columns of one slice; CK = C*9
};

// `block`: number of the workgroup inside the job; 256 columns per workgroup, four threads per column, each adding every
// fourth slice in order; their sums are then added in thread order: a fixed order, the same on every run.
__device__ inline void side_fold(const SideFold &f, unsigned block, side_f32x4 *sums /* [1024] in LDS */)
{
    const int t = threadIdx.x, col = t & 255, sub = t >> 8;
    const int i = (int)block * 256 + col;
    side_f32x4 s = {0.f, 0.f, 0.f, 0.f};
    if (i < f.n4)
        for (int z = sub; z < f.slices; z += 4)
            s += reinterpret_cast<const side_f32x4 *>(f.part)[(int64_t)z * f.n4 + i];
    sums[t] = s;
    __syncthreads();
    if (sub == 0 && i < f.n4)
    {
        const side_f32x4 v = ((sums[col] + sums[256 + col]) + sums[512 + col]) + sums[768 + col];
        // 16-byte column i = (tile, oc row, 4 of the tile's 192 columns); columns are kw*64 + channel
        const int q4 = i % 48, row = (i / 48) % 64, tile = i / (48 * 64);
        const int rt = tile % f.tiles_oc, rest = tile / f.tiles_oc, kh = rest % 3, cb = rest / 3;
        const int kw = q4 / 16, c = cb * 64 + 4 * (q4 % 16);
        float *o = f.gw + (int64_t)(rt * 64 + row) * f.CK + c * 9 + kh * 3 + kw;
        o[0] = v[0], o[9] = v[1], o[18] = v[2], o[27] = v[3];
    }
}

// ---- bias gradient: gb[oc] = sum over n and the plane of gy[n][oc][:] (src/mat/origin/cpu/conv/conv2d.cpp:566-580),
// one workgroup per channel, eight 16-byte loads in flight per thread, the running sums added in a fixed order.
// P % 4 == 0, gy 16-byte aligned, N*P < 2^31.
struct SideBias
{
    const float *gy;
    float *gb;
    unsigned total, P, OC;  // total = N*P elements per channel
    FastDiv by_plane;       // by P/4
};

__device__ inline void side_bias(const SideBias &b, unsigned oc, float *part /* [16] in LDS */)
{
    constexpr unsigned U = 8;
    const unsigned plane = b.P / 4, quads = b.total / 4;
    float acc[U];
#pragma unroll
    for (unsigned j = 0; j < U; ++j)
        acc[j] = 0.f;
    for (unsigned u0 = threadIdx.x; u0 < quads; u0 += U * 1024)
    {
        side_f32x4 q[U];
#pragma unroll
        for (unsigned j = 0; j < U; ++j)
        {
            const unsigned u = u0 + j * 1024;
            q[j] = side_f32x4{0.f, 0.f, 0.f, 0.f};
            if (u < quads)
            {
                const unsigned n = fastdiv(u, b.by_plane), v = u - n * plane;
                q[j] = *reinterpret_cast<const side_f32x4 *>(b.gy + ((int64_t)n * b.OC + oc) * b.P + (int64_t)v * 4);
            }
        }
#pragma unroll
        for (unsigned j = 0; j < U; ++j)
            acc[j] += (q[j][0] + q[j][1]) + (q[j][2] + q[j][3]);
    }
    float v = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        float s = 0.f;
        for (int i = 0; i < 1024 / 64; ++i)
            s += part[i];
        b.gb[oc] = s;
    }
}

// ---- the zero-padded filter copy the LDS-patch kernels stage from (conv_patch.hip):
// wp[(m*nslab + slab)*144 + tap*16 + cc] = w[m][slab*16 + cc][tap], or with the filter flipped and its first two
// dimensions exchanged for the input gradient
struct SidePack
{
    const float *w;
    float *wp;
    int Cin, M, Mpad, flipped;
};

__device__ inline void side_pack(const SidePack &p, unsigned block, unsigned blocks)
{
    const int total = p.Cin * 9 * p.Mpad, nslab = p.Cin / 16;
    for (int idx = (int)(block * blockDim.x + threadIdx.x); idx < total; idx += (int)(blocks * blockDim.x))
    {
        const int rem = idx % (9 * 16), rest = idx / (9 * 16);
        const int slab = rest % nslab, m = rest / nslab;
        const int tap = rem / 16, ch = slab * 16 + rem % 16;
        float v = 0.f;
        if (m < p.M)
            v = p.flipped ? p.w[((int64_t)ch * p.M + m) * 9 + 8 - tap] : p.w[((int64_t)m * p.Cin + ch) * 9 + tap];
        p.wp[idx] = v;
    }
}
}  // namespace odl
