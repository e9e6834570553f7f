// Second pass of a split-K product: P = sum over slices of the partial products.
#ifndef ROCM_SGEMM_AMD_SPLITK_REDUCE_HPP
#define ROCM_SGEMM_AMD_SPLITK_REDUCE_HPP

#include <hip/hip_runtime.h>

#include "tile_order.hpp"

namespace rocm_sgemm
{
namespace kernel
{

// alpha / beta of the final write: out = alpha * sum + beta * old, old not read when beta == 0.
struct output_scale
{
    float alpha, beta;
    __device__ __forceinline__ float operator()(float sum, const float* old) const
    {
        if(alpha == 1.0f && beta == 0.0f) return sum;
        const float t = alpha * sum;
        return beta == 0.0f ? t : __builtin_fmaf(beta, *old, t);
    }
};

// Sums the split_k partial products of batch blockIdx.y in slice order (fixed order => run-to-run
// deterministic).  Partials are packed rows x cols matrices, [batch][slice]; the output has row
// stride ldp and batch stride stride_p.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(float* __restrict__ P,
                                                            const float* __restrict__ partial,
                                                            int          rows,
                                                            int          cols,
                                                            int          ldp,
                                                            long long    stride_p,
                                                            int          split_k,
                                                            output_scale scale)
{
    const size_t count  = static_cast<size_t>(rows) * cols;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    const float* part   = partial + static_cast<size_t>(blockIdx.y) * split_k * count;
    float*       out    = P + blockIdx.y * stride_p;
    for(size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < count;
        idx += stride)
    {
        float s = part[idx];
        for(int k = 1; k < split_k; ++k)
        {
            s += part[static_cast<size_t>(k) * count + idx];
        }
        float* dst = ldp == cols ? out + idx : out + (idx / cols) * ldp + idx % cols;
        *dst       = scale(s, dst);
    }
}

// Same sum, four adjacent elements per thread with 128-bit accesses: for outputs whose rows are
// 16-byte aligned (cols, ldp and stride_p multiples of 4, aligned base).  With nine slices or
// more the loads of eight are issued before the first add; with fewer the plain loop is as fast
// (eight 4 MB partials into a 4 MB output: 7.3 us = 5 TB/s, bound by bandwidth; a variant that
// batched the loads for every slice count measured 8.2 us).
__global__ __launch_bounds__(256) void splitk_reduce_vec4_kernel(float* __restrict__ P,
                                                                 const float* __restrict__ partial,
                                                                 int          rows,
                                                                 int          cols,
                                                                 int          ldp,
                                                                 long long    stride_p,
                                                                 int          split_k,
                                                                 output_scale scale)
{
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const size_t count  = static_cast<size_t>(rows) * cols;
    const size_t quads  = count / 4;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    const float* part   = partial + static_cast<size_t>(blockIdx.y) * split_k * count;
    float*       out    = P + blockIdx.y * stride_p;
    for(size_t q = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; q < quads; q += stride)
    {
        const size_t idx = q * 4;
        f32x4        s   = *reinterpret_cast<const f32x4*>(part + idx);
        int          k   = 1;
        for(; k + 8 <= split_k; k += 8)
        {
            f32x4 v[8];
#pragma unroll
            for(int u = 0; u < 8; ++u)
                v[u] = *reinterpret_cast<const f32x4*>(part + static_cast<size_t>(k + u) * count + idx);
#pragma unroll
            for(int u = 0; u < 8; ++u)
                s += v[u]; // slice order, as in the scalar kernel
        }
        for(; k < split_k; ++k)
        {
            s += *reinterpret_cast<const f32x4*>(part + static_cast<size_t>(k) * count + idx);
        }
        float* dst = out + (idx / cols) * ldp + idx % cols;
        f32x4  o;
        o.x = scale(s.x, dst);
        o.y = scale(s.y, dst + 1);
        o.z = scale(s.z, dst + 2);
        o.w = scale(s.w, dst + 3);
        *reinterpret_cast<f32x4*>(dst) = o;
    }
}

// Second pass of a stream-K tail: tail tile u (blockIdx.x) owns K-tiles [u * k_tiles,
// (u + 1) * k_tiles) of the tail's run space; workgroup g of the first pass covered
// [g * per, (g + 1) * per) and left the partial tile of its segment s at partial[(2 g + s) * bm * bn],
// s = 0 for the tile its run starts in, 1 for the next.  The segments of a tile are summed in
// workgroup order (deterministic) and written into the output matrix, clipped at its edges.
// Workgroup (x = tail tile, y = strip of the tile).
__global__ __launch_bounds__(256) void tail_reduce_kernel(float* __restrict__ P,
                                                          const float* __restrict__ partial,
                                                          int rows,
                                                          int cols,
                                                          int ldp,
                                                          int grid_m,
                                                          int grid_n,
                                                          int group_m,
                                                          int tail_begin,
                                                          int k_tiles,
                                                          int per,
                                                          int bm,
                                                          int bn,
                                                          output_scale scale)
{
    const int                u  = blockIdx.x;
    const detail::tile_coord tc = detail::map_workgroup(tail_begin + u, grid_m, grid_n, group_m);
    const int                m0 = tc.tile_m * bm, n0 = tc.tile_n * bn;
    const int                quads = bm * bn / 4; // bn is a multiple of 4
    const size_t             tile  = static_cast<size_t>(bm) * bn;
    const int                g_first = (u * k_tiles) / per;
    const int                g_last  = ((u + 1) * k_tiles - 1) / per;
    typedef float            f32x4 __attribute__((ext_vector_type(4)));
    for(int q = blockIdx.y * blockDim.x + threadIdx.x; q < quads; q += gridDim.y * blockDim.x)
    {
        const int i = (q * 4) / bn, j = (q * 4) % bn;
        f32x4     s = {0.0f, 0.0f, 0.0f, 0.0f};
        for(int g = g_first; g <= g_last; ++g)
        {
            const int    seg  = (g * per) / k_tiles == u ? 0 : 1;
            const float* part = partial + (static_cast<size_t>(g) * 2 + seg) * tile;
            const f32x4  v    = *reinterpret_cast<const f32x4*>(part + static_cast<size_t>(q) * 4);
            s                 = g == g_first ? v : s + v;
        }
        const int row = m0 + i, col = n0 + j;
        if(row < rows)
        {
            float* out = P + static_cast<size_t>(row) * ldp + col;
            if(col < cols) out[0] = scale(s.x, out);
            if(col + 1 < cols) out[1] = scale(s.y, out + 1);
            if(col + 2 < cols) out[2] = scale(s.z, out + 2);
            if(col + 3 < cols) out[3] = scale(s.w, out + 3);
        }
    }
}

} // namespace kernel
} // namespace rocm_sgemm

#endif
