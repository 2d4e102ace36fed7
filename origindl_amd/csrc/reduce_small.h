// Column sums of a small tensor in one launch — the halves of reduce.hip's col_sum_small_kernel as device functions, so
// that another launch can run the same sum as one of its jobs (the bias gradient beside a classifier layer's two matrix
// gradients, gemm_skinny.hip) and give the same bits as Mat::sum_to would in a launch of its own
// (src/mat/origin/cpu/math/sum_to.cpp via Linear's backward, src/nn/layers/linear.cpp:88-104).
//
// A workgroup's first 256 threads own CW*VEC adjacent columns of one `outer` slice: CW column lanes x (256/CW) row
// groups, group g adds rows g, g+G, ... (eight loads in flight), the group sums meet in LDS and are added in group order.
#pragma once
#include "odl_common.h"

namespace odl
{
// column sums small enough to be bound by launch latency: one launch
inline bool small_cols(int64_t outer, int64_t axis, int64_t inner)
{
    return inner > 1 && axis >= 16 && outer <= 1024 && outer * axis * inner <= (1 << 20);
}

template <int VEC, int CW>
struct ColSumSmall
{
    static constexpr int kThreads = 256, G = kThreads / CW;
    typedef float Sums[G][CW * VEC + 1];
    typedef float vec4 __attribute__((ext_vector_type(4)));

    // threads 0..255 of the workgroup (tid); bx: which CW*VEC columns, o: which outer slice
    __device__ static void accumulate(const float *__restrict__ src, int64_t axis, int64_t inner, unsigned bx, int64_t o,
                                      unsigned tid, Sums &sh)
    {
        const int lane = tid % CW, grp = tid / CW;
        const int64_t col = ((int64_t)bx * CW + lane) * VEC;
        const bool live = col < inner;
        const float *p = src + (o * axis) * inner + col;
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e)
            acc[e] = 0.f;
        if (live)
        {
            int64_t a = grp;
            for (; a + 7 * G < axis; a += 8 * G)
            {
                float v[8][VEC];
#pragma unroll
                for (int u = 0; u < 8; ++u)
                {
                    if (VEC == 4)
                    {
                        const vec4 q = *reinterpret_cast<const vec4 *>(p + (a + u * G) * inner);
                        v[u][0] = q[0], v[u][1 % VEC] = q[1], v[u][2 % VEC] = q[2], v[u][3 % VEC] = q[3];
                    }
                    else
                        v[u][0] = p[(a + u * G) * inner];
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        acc[e] += v[u][e];
            }
            for (; a < axis; a += G)
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    acc[e] += p[a * inner + e];
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e)
            sh[grp][lane * VEC + e] = acc[e];
    }

    // after a barrier
    __device__ static void finish(float *__restrict__ dst, int64_t inner, unsigned bx, int64_t o, unsigned tid, const Sums &sh)
    {
        if (tid < CW * VEC)
        {
            const int64_t c = (int64_t)bx * CW * VEC + tid;
            if (c < inner)
            {
                float t = sh[0][tid];
#pragma unroll 4
                for (int g = 1; g < G; ++g)
                    t += sh[g][tid];
                dst[o * inner + c] = t;
            }
        }
    }
};
}  // namespace odl
