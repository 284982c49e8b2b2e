// One-pass per-row mean and variance of a [rows, R] fp32 matrix whose rows are
// contiguous: the statistics half of batch normalisation.
//
// The graph computes mean = sum(x)/R and variance = mean((x - mean)^2)
// (ngraph/op_graph/op_graph.py:4007-4009, 4252-4266), which reads x twice.
// Here each workgroup accumulates sum(x - p) and sum((x - p)^2) around a pivot p
// (the row's first element) over one segment of a row, and a second tiny kernel
// merges the segments in a fixed order:  mean = p + S1/R,  var = S2/R - (S1/R)^2.
// Shifting by p keeps the subtraction in `var` from cancelling when |mean| is
// large against the spread.  Segments make rows x segments >> 256 workgroups
// even for a few hundred rows; the fixed merge order keeps results reproducible.
#pragma once
#include <hip/hip_runtime.h>

namespace ngh {

constexpr int kMomBlock = 256;
constexpr int kMomUnroll = 4;     // float4 loads in flight per lane

typedef float mom_f4 __attribute__((ext_vector_type(4)));

template <bool NT>
__device__ __forceinline__ float4 mom_load(const float4* p) {
    if constexpr (NT) {
        const mom_f4 v = __builtin_nontemporal_load(reinterpret_cast<const mom_f4*>(p));
        return make_float4(v.x, v.y, v.z, v.w);
    } else {
        return *p;
    }
}

template <bool NT>
__global__ __launch_bounds__(kMomBlock) void moments_partial_kernel(
    const float* __restrict__ x, long long row_stride, unsigned R4, unsigned n_seg, unsigned seg_chunks,
    float2* __restrict__ partial) {
    const unsigned row = blockIdx.x / n_seg;
    const unsigned seg = blockIdx.x - row * n_seg;
    const float* xr = x + (long long)row * row_stride;
    const float pivot = xr[0];
    const float4* x4 = reinterpret_cast<const float4*>(xr);
    const unsigned c_begin = seg * seg_chunks;
    const unsigned c_end = min(R4, c_begin + seg_chunks);
    float s1[kMomUnroll], s2[kMomUnroll];
#pragma unroll
    for (int u = 0; u < kMomUnroll; ++u) s1[u] = s2[u] = 0.0f;
    unsigned c = c_begin + threadIdx.x;
    for (; c + (kMomUnroll - 1) * kMomBlock < c_end; c += kMomUnroll * kMomBlock) {
        float4 v[kMomUnroll];
#pragma unroll
        for (int u = 0; u < kMomUnroll; ++u) v[u] = mom_load<NT>(x4 + c + u * kMomBlock);
#pragma unroll
        for (int u = 0; u < kMomUnroll; ++u) {
            const float a = v[u].x - pivot, b = v[u].y - pivot, cc = v[u].z - pivot, d = v[u].w - pivot;
            s1[u] += (a + b) + (cc + d);
            s2[u] += (a * a + b * b) + (cc * cc + d * d);
        }
    }
    for (; c < c_end; c += kMomBlock) {
        const float4 v = mom_load<NT>(x4 + c);
        const float a = v.x - pivot, b = v.y - pivot, cc = v.z - pivot, d = v.w - pivot;
        s1[0] += (a + b) + (cc + d);
        s2[0] += (a * a + b * b) + (cc * cc + d * d);
    }
    float t1 = (s1[0] + s1[1]) + (s1[2] + s1[3]);
    float t2 = (s2[0] + s2[1]) + (s2[2] + s2[3]);
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) {
        t1 += __shfl_xor(t1, m, 64);
        t2 += __shfl_xor(t2, m, 64);
    }
    __shared__ float2 sh[kMomBlock / 64];
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = make_float2(t1, t2);
    __syncthreads();
    if (threadIdx.x == 0) {
        float2 a = sh[0];
        for (int w = 1; w < kMomBlock / 64; ++w) { a.x += sh[w].x; a.y += sh[w].y; }
        partial[blockIdx.x] = a;
    }
}

// One wavefront per row: lanes take segments, butterfly, lane 0 writes.
__global__ __launch_bounds__(64) void moments_finish_kernel(
    const float* __restrict__ x, long long row_stride, unsigned R, unsigned tail_begin, unsigned n_seg,
    const float2* __restrict__ partial, float* __restrict__ mean, float* __restrict__ var) {
    const unsigned row = blockIdx.x;
    const float* xr = x + (long long)row * row_stride;
    const float pivot = xr[0];
    float t1 = 0.0f, t2 = 0.0f;
    for (unsigned g = threadIdx.x; g < n_seg; g += 64) {
        const float2 p = partial[row * n_seg + g];
        t1 += p.x;
        t2 += p.y;
    }
    // elements past the last whole float4 (R % 4) are added here
    for (unsigned i = tail_begin + threadIdx.x; i < R; i += 64) {
        const float a = xr[i] - pivot;
        t1 += a;
        t2 += a * a;
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) {
        t1 += __shfl_xor(t1, m, 64);
        t2 += __shfl_xor(t2, m, 64);
    }
    if (threadIdx.x == 0) {
        const float inv = 1.0f / (float)R;
        const float d = t1 * inv;
        mean[row] = pivot + d;
        var[row] = fmaxf(t2 * inv - d * d, 0.0f);
    }
}

}  // namespace ngh
