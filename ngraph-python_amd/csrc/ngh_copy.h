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
    int       diagonal;   // transpose kernels: deal the tiles along diagonals (see copy_diagonal)
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

// When both strided strides are multiples of 4 KiB, tiles are dealt along diagonals: consecutive
// workgroups differ in both tile coordinates.  The tiles of one tile row then start a multiple of
// a large power of two apart on the strided side and fall on the same few memory channels; in
// row-major order the workgroups resident at one time would all read (or all write) through
// those few channels (8192 x 8192 fp32: 131 us row-major, 102 us along diagonals).  With other
// strides row-major order is the faster one by a few per cent.
__device__ __forceinline__ unsigned copy_diagonal(unsigned row, unsigned col, unsigned n_rows, int diagonal) {
    return diagonal ? (row + col) % n_rows : row;
}
inline int copy_wants_diagonal(long long stride_a, long long stride_b, int itemsize) {
    return (stride_a * itemsize) % 4096 == 0 && (stride_b * itemsize) % 4096 == 0;
}

template <typename T>
__global__ __launch_bounds__(kCopyBlock) void copy_tr_kernel(T* dst, const T* src, const CopyArgs a,
                                                             unsigned tiles_r, unsigned tiles_c) {
    __shared__ T tile[kCopyTile][kCopyTile + 1];
    const int r_ax = a.rank - 2, c_ax = a.rank - 1;
    const unsigned R = (unsigned)a.shape[r_ax], C = (unsigned)a.shape[c_ax];
    unsigned b = blockIdx.x;
    const unsigned tc = b % tiles_c; b /= tiles_c;
    const unsigned tr = copy_diagonal(b % tiles_r, tc, tiles_r, a.diagonal); b /= tiles_r;
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

// Rows that are contiguous in both views: 16-byte accesses, one chunk per lane.
template <typename T>
__global__ __launch_bounds__(kCopyBlock) void copy_vec_kernel(T* dst, const T* src, const CopyArgs a,
                                                              unsigned n_chunks, unsigned chunks_per_row) {
    constexpr int V = 16 / (int)sizeof(T);
    const unsigned step = gridDim.x * kCopyBlock;
    for (unsigned q = blockIdx.x * kCopyBlock + threadIdx.x; q < n_chunks; q += step) {
        unsigned rem = q / chunks_per_row;
        const unsigned c = q - rem * chunks_per_row;
        long long so = (long long)c * V, dof = (long long)c * V;
        for (int ax = a.rank - 2; ax >= 0; --ax) {
            const unsigned d = (unsigned)a.shape[ax];
            const unsigned i = rem % d;
            rem /= d;
            so += (long long)i * a.ss[ax];
            dof += (long long)i * a.ds[ax];
        }
        *reinterpret_cast<uint4*>(dst + dof) = *reinterpret_cast<const uint4*>(src + so);
    }
}

// Transpose of 4-byte elements with 16-byte accesses on both sides: a lane reads four
// consecutive source rows-elements (float4 along the source-contiguous axis), scatters them
// into the padded tile, and after the barrier gathers four tile elements that are consecutive
// along the destination-contiguous axis.  Needs R, C and the strides to be multiples of 4.
// TILE x TILE elements per workgroup: 64 (contiguous runs of 256 bytes on both sides) or 128
// (512 bytes, 65 KiB of LDS) for matrices with enough tiles of that size to fill the chip.
template <int TILE>
__global__ __launch_bounds__(kCopyBlock) void copy_tr4_kernel(uint32_t* dst, const uint32_t* src, const CopyArgs a,
                                                              unsigned tiles_r, unsigned tiles_c) {
    constexpr int kChunks = TILE / 4;                      // float4 chunks along a tile edge
    constexpr int kLines = kCopyBlock / kChunks;           // tile lines the workgroup covers per turn
    constexpr int kTurns = TILE / kLines;
    __shared__ uint32_t tile[TILE][TILE + 1];              // [c_local][r_local]
    const int r_ax = a.rank - 2, c_ax = a.rank - 1;
    const unsigned R = (unsigned)a.shape[r_ax], C = (unsigned)a.shape[c_ax];
    unsigned b = blockIdx.x;
    const unsigned tc = b % tiles_c; b /= tiles_c;
    const unsigned tr = copy_diagonal(b % tiles_r, tc, tiles_r, a.diagonal); b /= tiles_r;
    long long so = 0, dof = 0;
    for (int ax = r_ax - 1; ax >= 0; --ax) {
        const unsigned d = (unsigned)a.shape[ax];
        const unsigned i = b % d;
        b /= d;
        so += (long long)i * a.ss[ax];
        dof += (long long)i * a.ds[ax];
    }
    const unsigned cx = threadIdx.x % kChunks, j = threadIdx.x / kChunks;
    uint4 v[kTurns];
#pragma unroll
    for (int i = 0; i < kTurns; ++i) {
        const unsigned c = tc * TILE + j + kLines * i, r = tr * TILE + cx * 4;
        v[i] = make_uint4(0, 0, 0, 0);
        if (r < R && c < C) v[i] = *reinterpret_cast<const uint4*>(src + so + (long long)c * a.ss[c_ax] + r);
    }
#pragma unroll
    for (int i = 0; i < kTurns; ++i) {
        uint32_t* row = tile[j + kLines * i] + cx * 4;
        row[0] = v[i].x; row[1] = v[i].y; row[2] = v[i].z; row[3] = v[i].w;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kTurns; ++i) {
        const unsigned rl = j + kLines * i;
        const unsigned r = tr * TILE + rl, c = tc * TILE + cx * 4;
        if (r < R && c < C) {
            const uint4 w = make_uint4(tile[cx * 4][rl], tile[cx * 4 + 1][rl], tile[cx * 4 + 2][rl], tile[cx * 4 + 3][rl]);
            *reinterpret_cast<uint4*>(dst + dof + (long long)r * a.ds[r_ax] + c) = w;
        }
    }
}

inline bool copy_aligned(const void* dst, const void* src, const CopyArgs& a, int skip0, int skip1, int V) {
    if (((uintptr_t)dst | (uintptr_t)src) & 15) return false;
    for (int ax = 0; ax < a.rank; ++ax) {
        if (ax == skip0 || ax == skip1) continue;
        if (a.ss[ax] % V || a.ds[ax] % V) return false;
    }
    return true;
}

template <typename T>
inline hipError_t launch_copy_t(hipStream_t stream, int cus, void* dst, const void* src, const CopyArgs& plain) {
    const CopyArgs& a = plain;
    constexpr int V = 16 / (int)sizeof(T);
    const int last = a.rank - 1;
    if (a.rank >= 1 && a.ss[last] == 1 && a.ds[last] == 1 && a.shape[last] % V == 0 &&
        copy_aligned(dst, src, a, last, -1, V)) {
        const unsigned cpr = (unsigned)(a.shape[last] / V);
        const unsigned n_chunks = a.total / V;
        unsigned blocks = (n_chunks + kCopyBlock - 1) / kCopyBlock;
        blocks = blocks < (unsigned)(cus * 64) ? blocks : (unsigned)(cus * 64);
        hipLaunchKernelGGL(copy_vec_kernel<T>, dim3(blocks), dim3(kCopyBlock), 0, stream, (T*)dst, (const T*)src, a,
                           n_chunks, cpr);
        return hipGetLastError();
    }
    if (a.rank >= 2 && a.ss[a.rank - 2] == 1 && a.ds[a.rank - 1] == 1 && a.ss[a.rank - 1] != 1 &&
        a.shape[a.rank - 2] >= 16 && a.shape[a.rank - 1] >= 16) {
        const unsigned tiles_r = (unsigned)((a.shape[a.rank - 2] + kCopyTile - 1) / kCopyTile);
        const unsigned tiles_c = (unsigned)((a.shape[a.rank - 1] + kCopyTile - 1) / kCopyTile);
        unsigned long long blocks = (unsigned long long)tiles_r * tiles_c;
        for (int ax = 0; ax < a.rank - 2; ++ax) blocks *= (unsigned long long)a.shape[ax];
        if (blocks < (1ULL << 31)) {
            CopyArgs a = plain;
            a.diagonal = copy_wants_diagonal(a.ss[a.rank - 1], a.ds[a.rank - 2], (int)sizeof(T));
            if constexpr (sizeof(T) == 4) {
                // 16-byte accesses: the source is read along r, the destination written along c
                if (a.shape[a.rank - 2] % 4 == 0 && a.shape[a.rank - 1] % 4 == 0 &&
                    a.ss[a.rank - 1] % 4 == 0 && a.ds[a.rank - 2] % 4 == 0 &&
                    copy_aligned(dst, src, a, a.rank - 2, a.rank - 1, 4)) {
                    const unsigned big_r = (unsigned)((a.shape[a.rank - 2] + 127) / 128);
                    const unsigned big_c = (unsigned)((a.shape[a.rank - 1] + 127) / 128);
                    const unsigned long long big_blocks = blocks / ((unsigned long long)tiles_r * tiles_c) * big_r * big_c;
                    // (measured: 8192 x 8192 102 -> 95 us, 16384 x 4096 108 -> 102 us; strides off the 4 KiB grid lose a few per cent)
                    if (a.diagonal && big_blocks >= (unsigned long long)cus * 8)
                        hipLaunchKernelGGL(copy_tr4_kernel<128>, dim3((unsigned)big_blocks), dim3(kCopyBlock), 0, stream,
                                           (uint32_t*)dst, (const uint32_t*)src, a, big_r, big_c);
                    else
                        hipLaunchKernelGGL(copy_tr4_kernel<64>, dim3((unsigned)blocks), dim3(kCopyBlock), 0, stream,
                                           (uint32_t*)dst, (const uint32_t*)src, a, tiles_r, tiles_c);
                    return hipGetLastError();
                }
            }
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
    return itemsize == 1   ? launch_copy_t<uint8_t>(stream, cus, dst, src, a)
           : itemsize == 2 ? launch_copy_t<uint16_t>(stream, cus, dst, src, a)
                           : launch_copy_t<uint32_t>(stream, cus, dst, src, a);
}

}  // namespace ngh
