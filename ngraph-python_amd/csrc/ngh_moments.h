// One-pass per-row mean and variance of a [rows, R] fp32 matrix whose rows are
// contiguous: the statistics half of batch normalisation.
//
// The graph computes mean = sum(x)/R and variance = mean((x - mean)^2)
// (ngraph/op_graph/op_graph.py:4007-4009, 4252-4266), which reads x twice.
// Here each workgroup accumulates sum(x - p) and sum((x - p)^2) around a pivot p
// (the row's first element) over one segment of a row, and the last workgroup of the
// row to finish (or a small second launch) merges the segments in a fixed order:  mean = p + S1/R,
// var = S2/R - (S1/R)^2.  Optionally it also writes 1/sqrt(var + eps), the factor the
// normalisation multiplies by (frontends/neon/layer.py:1255), which saves the graph a
// kernel launch for a few hundred elements.
// Shifting by p keeps the subtraction in `var` from cancelling when |mean| is
// large against the spread.  Segments make rows x segments >> 256 workgroups
// even for a few hundred rows; the fixed merge order keeps results reproducible.
#pragma once
#include <hip/hip_runtime.h>

namespace ngh {

constexpr int kMomBlock = 256;
constexpr int kMomUnroll = 4;     // float4 loads in flight per lane

// Four floats at any 4-byte-aligned address: rows need not start on 16-byte boundaries (the
// device takes unaligned 16-byte accesses at a cost of 2-3 % of the read rate).
typedef float mom_f4 __attribute__((ext_vector_type(4), aligned(4)));

template <bool NT>
__device__ __forceinline__ float4 mom_load(const float4* p) {
    const mom_f4* q = reinterpret_cast<const mom_f4*>(p);
    mom_f4 v;
    if constexpr (NT) v = __builtin_nontemporal_load(q);
    else v = *q;
    return make_float4(v.x, v.y, v.z, v.w);
}

// Hand-over of the row's partial sums, `mode`:
//  2  (the default) every workgroup stores its partial sum and the kernel ends; a second, small
//     launch (moments_merge_kernel) merges each row.  The kernel boundary orders the two, so
//     nothing here leans on more than the language's memory model promises.
//  0, 1  one launch: the workgroups of a row take a ticket when their partial sums are written;
//     the one that draws the last ticket merges the row and resets the row's counter for the
//     next launch (0: relaxed atomics ordered by a data dependency, which relies on the
//     hardware; 1: release tickets and an acquire fence).
// All three merge in segment order with the same arithmetic (moments_merge_row): the result does
// not depend on the mode, nor on which workgroup came last.
__device__ __forceinline__ void moments_merge_row(const float* __restrict__ xr, float pivot, unsigned R, unsigned R4,
                                                  unsigned n_seg, const float2* __restrict__ row_partial, unsigned lane,
                                                  unsigned row, float* __restrict__ mean, float* __restrict__ var,
                                                  float* __restrict__ rstd, float eps) {
    float t1 = 0.0f, t2 = 0.0f;
    for (unsigned g = lane; g < n_seg; g += 64) {
        const unsigned long long p = __hip_atomic_load(
            reinterpret_cast<const unsigned long long*>(row_partial) + g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        t1 += __uint_as_float((unsigned)p);
        t2 += __uint_as_float((unsigned)(p >> 32));
    }
    // elements past the last whole float4 (R % 4) are added here
    for (unsigned i = R4 * 4 + lane; i < R; i += 64) {
        const float a = xr[i] - pivot;
        t1 += a;
        t2 += a * a;
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) {
        t1 += __shfl_xor(t1, m, 64);
        t2 += __shfl_xor(t2, m, 64);
    }
    if (lane == 0) {
        const float inv = 1.0f / (float)R;
        const float d = t1 * inv;
        const float v = fmaxf(t2 * inv - d * d, 0.0f);
        mean[row] = pivot + d;
        var[row] = v;
        if (rstd) rstd[row] = 1.0f / sqrtf(v + eps);
    }
}

template <bool NT>
__global__ __launch_bounds__(kMomBlock) void moments_kernel(
    const float* __restrict__ x, long long row_stride, unsigned R, unsigned R4, unsigned n_seg,
    unsigned seg_chunks, float2* __restrict__ partial, unsigned* __restrict__ row_tickets,
    float* __restrict__ mean, float* __restrict__ var, float* __restrict__ rstd, float eps, int mode) {
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
    __shared__ unsigned ticket;
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = make_float2(t1, t2);
    __syncthreads();
    if (threadIdx.x == 0) {
        float2 a = sh[0];
        for (int w = 1; w < kMomBlock / 64; ++w) { a.x += sh[w].x; a.y += sh[w].y; }
        const unsigned long long bits =
            (unsigned long long)__float_as_uint(a.x) | ((unsigned long long)__float_as_uint(a.y) << 32);
        if (mode == 2) {
            __hip_atomic_store(reinterpret_cast<unsigned long long*>(partial) + blockIdx.x, bits, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        } else if (mode == 1) {
            // By the memory model: the partial is stored, the ticket is a release read-modify-write
            // at device scope, and whoever draws the last ticket issues an acquire fence: it has
            // then acquired every earlier increment's release (a release sequence runs through
            // the increments), so the partials of the row are visible to it.
            __hip_atomic_store(reinterpret_cast<unsigned long long*>(partial) + blockIdx.x, bits, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            ticket = __hip_atomic_fetch_add(row_tickets + row, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            if (ticket == n_seg - 1) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // only the merger acquires
        } else {
            // Without fences, relying on the hardware: publish the partial and take the ticket
            // with device-scope read-modify-write atomics only.  They are performed at the
            // device's point of coherence, and the ticket is issued after the exchange has
            // returned (its increment depends on the returned value), so whoever draws the last
            // ticket can read every partial of the row there.  The language's memory model does
            // not promise this ordering; gfx950 delivers it.
            const unsigned long long old = __hip_atomic_exchange(
                reinterpret_cast<unsigned long long*>(partial) + blockIdx.x, bits, __ATOMIC_RELAXED,
                __HIP_MEMORY_SCOPE_AGENT);
            unsigned one = 1u;
            asm volatile("" : "+v"(one) : "v"((unsigned)old));   // orders the ticket after the exchange
            ticket = __hip_atomic_fetch_add(row_tickets + row, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (mode == 2) return;
    __syncthreads();
    if (ticket != n_seg - 1 || threadIdx.x >= 64) return;
    // last workgroup of the row, first wavefront
    moments_merge_row(xr, pivot, R, R4, n_seg, partial + (size_t)row * n_seg, threadIdx.x, row, mean, var, rstd, eps);
    if (threadIdx.x == 0)
        __hip_atomic_store(row_tickets + row, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The second launch of hand-over mode 2: a wavefront per row merges the row's partial sums.
__global__ __launch_bounds__(kMomBlock) void moments_merge_kernel(
    const float* __restrict__ x, long long row_stride, unsigned R, unsigned R4, unsigned rows, unsigned n_seg,
    const float2* __restrict__ partial, float* __restrict__ mean, float* __restrict__ var, float* __restrict__ rstd,
    float eps) {
    const unsigned row = blockIdx.x * (kMomBlock / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* xr = x + (long long)row * row_stride;
    moments_merge_row(xr, xr[0], R, R4, n_seg, partial + (size_t)row * n_seg, threadIdx.x & 63, row, mean, var, rstd, eps);
}

// Many short rows (layer normalisation: tens of thousands of rows of a few thousand elements):
// L lanes per row (a power of two up to a wavefront), 256 / L rows per workgroup.  Same sums
// around the same pivot as above, folded by a butterfly inside the L lanes: no partial sums in
// memory, no tickets, no barrier.
template <bool NT>
__global__ __launch_bounds__(kMomBlock) void moments_rows_kernel(
    const float* __restrict__ x, long long row_stride, unsigned R, unsigned R4, unsigned rows, unsigned L,
    float* __restrict__ mean, float* __restrict__ var, float* __restrict__ rstd, float eps) {
    const unsigned row = blockIdx.x * (kMomBlock / L) + threadIdx.x / L;
    const unsigned pos = threadIdx.x & (L - 1);
    const bool live = row < rows;                       // (idle lanes still take part in the butterfly)
    const float* xr = x + (long long)(live ? row : 0) * row_stride;
    const float pivot = xr[0];
    const float4* x4 = reinterpret_cast<const float4*>(xr);
    float s1[kMomUnroll], s2[kMomUnroll];
#pragma unroll
    for (int u = 0; u < kMomUnroll; ++u) s1[u] = s2[u] = 0.0f;
    // (a lane's last turn may hold fewer than kMomUnroll chunks: the missing ones count as the
    // pivot, which adds nothing -- every lane of a row leaves the loop in the same turn)
    for (unsigned c = pos; live && c < R4; c += kMomUnroll * L) {
        float4 v[kMomUnroll];
#pragma unroll
        for (int u = 0; u < kMomUnroll; ++u)
            v[u] = (c + u * L < R4) ? mom_load<NT>(x4 + c + u * L) : make_float4(pivot, pivot, pivot, pivot);
#pragma unroll
        for (int u = 0; u < kMomUnroll; ++u) {
            const float a = v[u].x - pivot, b = v[u].y - pivot, cc = v[u].z - pivot, d = v[u].w - pivot;
            s1[u] += (a + b) + (cc + d);
            s2[u] += (a * a + b * b) + (cc * cc + d * d);
        }
    }
    if (live)
        for (unsigned i = R4 * 4 + pos; i < R; i += L) {     // elements past the last whole float4
            const float a = xr[i] - pivot;
            s1[0] += a;
            s2[0] += a * a;
        }
    float t1 = (s1[0] + s1[1]) + (s1[2] + s1[3]);
    float t2 = (s2[0] + s2[1]) + (s2[2] + s2[3]);
    for (unsigned m = L >> 1; m > 0; m >>= 1) {
        t1 += __shfl_xor(t1, (int)m, 64);
        t2 += __shfl_xor(t2, (int)m, 64);
    }
    if (live && pos == 0) {
        const float inv = 1.0f / (float)R;
        const float d = t1 * inv;
        const float v = fmaxf(t2 * inv - d * d, 0.0f);
        mean[row] = pivot + d;
        var[row] = v;
        if (rstd) rstd[row] = 1.0f / sqrtf(v + eps);
    }
}

}  // namespace ngh
