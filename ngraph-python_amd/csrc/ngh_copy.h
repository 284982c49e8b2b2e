// Fill and N-d strided copy (dimshuffle) kernels.
//
// Replaces the generated copy_transpose / copy_oned kernels of
// ngraph/transformers/gpu/kernels/cuda/copy_transpose.py:89-282 used by
// DimShuffleKernel (ngraph/transformers/gpu/tensor_ops.py:137-204) and by
// strided host I/O (ngraph/transformers/gputransform.py:873-909).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ngh {

constexpr int kCopyMaxRank = 8;
constexpr int kCopyBlock = 256;

template <typename T>
__global__ __launch_bounds__(kCopyBlock) void fill_kernel(T* p, T value, size_t n) {
    const size_t step = (size_t)gridDim.x * kCopyBlock;
    for (size_t i = (size_t)blockIdx.x * kCopyBlock + threadIdx.x; i < n; i += step) p[i] = value;
}

struct CopyArgs {
    int       rank;
    unsigned  total;
    long long shape[kCopyMaxRank];
    long long ds[kCopyMaxRank];   // destination element strides
    long long ss[kCopyMaxRank];   // source element strides
};

// Generic path: thread per element, destination-major order (the last axis
// of the view varies fastest across lanes).
template <typename T>
__global__ __launch_bounds__(kCopyBlock) void copy_nd_kernel(T* dst, const T* src, const CopyArgs a) {
    const unsigned step = gridDim.x * kCopyBlock;
    for (unsigned q = blockIdx.x * kCopyBlock + threadIdx.x; q < a.total; q += step) {
        unsigned rem = q;
        long long so = 0, dof = 0;
        for (int ax = a.rank - 1; ax >= 0; --ax) {
            const unsigned d = (unsigned)a.shape[ax];
            const unsigned i = rem % d;
            rem /= d;
            so += (long long)i * a.ss[ax];
            dof += (long long)i * a.ds[ax];
        }
        dst[dof] = src[so];
    }
}

// 2-D transpose path: the view is [batch.., rows, cols] where the source is
// contiguous along `rows` (ss[r-2] == 1) and the destination along `cols`
// (ds[r-1] == 1).  A 64x64 tile goes through LDS (row padded to 65 words) so
// both the global read and the global write are coalesced.
constexpr int kCopyTile = 64;

template <typename T>
__global__ __launch_bounds__(kCopyBlock) void copy_tr_kernel(T* dst, const T* src, const CopyArgs a,
                                                             unsigned tiles_r, unsigned tiles_c) {
    __shared__ T tile[kCopyTile][kCopyTile + 1];
    const int r_ax = a.rank - 2, c_ax = a.rank - 1;
    const unsigned R = (unsigned)a.shape[r_ax], C = (unsigned)a.shape[c_ax];
    unsigned b = blockIdx.x;
    const unsigned tc = b % tiles_c; b /= tiles_c;
    const unsigned tr = b % tiles_r; b /= tiles_r;
    long long so = 0, dof = 0;
    for (int ax = r_ax - 1; ax >= 0; --ax) {
        const unsigned d = (unsigned)a.shape[ax];
        const unsigned i = b % d;
        b /= d;
        so += (long long)i * a.ss[ax];
        dof += (long long)i * a.ds[ax];
    }
    const unsigned tx = threadIdx.x & 63, ty = threadIdx.x >> 6;   // 64 x 4
    // read: lanes along rows (source-contiguous)
    for (unsigned j = ty; j < kCopyTile; j += 4) {
        const unsigned r = tr * kCopyTile + tx, c = tc * kCopyTile + j;
        if (r < R && c < C) tile[j][tx] = src[so + (long long)r * a.ss[r_ax] + (long long)c * a.ss[c_ax]];
    }
    __syncthreads();
    // write: lanes along cols (destination-contiguous)
    for (unsigned j = ty; j < kCopyTile; j += 4) {
        const unsigned r = tr * kCopyTile + j, c = tc * kCopyTile + tx;
        if (r < R && c < C) dst[dof + (long long)r * a.ds[r_ax] + (long long)c * a.ds[c_ax]] = tile[tx][j];
    }
}

template <typename T>
inline hipError_t launch_copy_t(hipStream_t stream, int cus, void* dst, const void* src, const CopyArgs& a) {
    if (a.rank >= 2 && a.ss[a.rank - 2] == 1 && a.ds[a.rank - 1] == 1 && a.ss[a.rank - 1] != 1 &&
        a.shape[a.rank - 2] >= 16 && a.shape[a.rank - 1] >= 16) {
        const unsigned tiles_r = (unsigned)((a.shape[a.rank - 2] + kCopyTile - 1) / kCopyTile);
        const unsigned tiles_c = (unsigned)((a.shape[a.rank - 1] + kCopyTile - 1) / kCopyTile);
        unsigned long long blocks = (unsigned long long)tiles_r * tiles_c;
        for (int ax = 0; ax < a.rank - 2; ++ax) blocks *= (unsigned long long)a.shape[ax];
        if (blocks < (1ULL << 31)) {
            hipLaunchKernelGGL(copy_tr_kernel<T>, dim3((unsigned)blocks), dim3(kCopyBlock), 0, stream, (T*)dst,
                               (const T*)src, a, tiles_r, tiles_c);
            return hipGetLastError();
        }
    }
    unsigned blocks = (a.total + kCopyBlock - 1) / kCopyBlock;
    blocks = blocks < (unsigned)(cus * 16) ? blocks : (unsigned)(cus * 16);
    hipLaunchKernelGGL(copy_nd_kernel<T>, dim3(blocks), dim3(kCopyBlock), 0, stream, (T*)dst, (const T*)src, a);
    return hipGetLastError();
}

inline hipError_t launch_copy(hipStream_t stream, int cus, void* dst, const void* src, const CopyArgs& a,
                              int itemsize) {
    return itemsize == 2 ? launch_copy_t<uint16_t>(stream, cus, dst, src, a)
                         : launch_copy_t<uint32_t>(stream, cus, dst, src, a);
}

}  // namespace ngh
