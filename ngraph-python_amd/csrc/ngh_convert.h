// float / half tensor -> flex16 mantissas, truncating, with max|mantissa|: the converter the
// reference runs behind its dense flex kernels, whose raw fp32 (or fp16) scratch output it
// turns into a flex tensor (ngraph/transformers/gpu/flex_conv.py:745-791 `convert`:
// `short result = (short)(cvt(value) * scale); max_val = max(iabs(result), max_val);
// ... atomicMax(flex_data, max_val)`).
//
// Here: mantissa = trunc(value * scale) toward zero.  Outside the int16 range, where the
// reference's float -> short cast is undefined, the mantissa saturates at -32768 / 32767
// (what a saturating conversion instruction does, and what the flex fill does,
// tensor_ops.py:690-707); NaN gives 0.  max|mantissa| is taken as int32, so -32768 counts as
// 32768 (the reference's iabs on a short wraps it back to -32768 and loses it).
// Eight elements per lane: 16-byte stores, 2 x 16-byte (fp32) or 16-byte (fp16) loads.
#pragma once
#include "ngh_device.h"

namespace ngh {

constexpr int kCvtBlock = 256;

template <int SRC>
__device__ __forceinline__ float cvt_load1(const void* in, unsigned long long i) {
    if constexpr (SRC == NGH_F32) return reinterpret_cast<const float*>(in)[i];
    else return __half2float(reinterpret_cast<const __half*>(in)[i]);
}

template <int SRC, bool VEC>
__global__ __launch_bounds__(kCvtBlock) void convert_flex16_kernel(short* __restrict__ out, const void* __restrict__ in,
                                                                   unsigned long long n, float mul,
                                                                   const float* __restrict__ dscale,
                                                                   int* __restrict__ partial) {
    const float m = dscale ? 1.0f / *dscale : mul;
    int fmax = 0;
    const unsigned long long step = (unsigned long long)gridDim.x * kCvtBlock;
    unsigned long long done = 0;
    if constexpr (VEC) {
        const unsigned long long n8 = n / 8;
        for (unsigned long long q = (unsigned long long)blockIdx.x * kCvtBlock + threadIdx.x; q < n8; q += step) {
            float v[8];
            if constexpr (SRC == NGH_F32) {
                const float4 a = reinterpret_cast<const float4*>(in)[2 * q], b = reinterpret_cast<const float4*>(in)[2 * q + 1];
                v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
            } else {
                const uint4 raw = reinterpret_cast<const uint4*>(in)[q];
                const unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    unsigned u = w[j];
                    const float2 f = __half22float2(*reinterpret_cast<__half2*>(&u));
                    v[2 * j] = f.x; v[2 * j + 1] = f.y;
                }
            }
            unsigned w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int q0 = flex_quantize_trunc(v[2 * j] * m), q1 = flex_quantize_trunc(v[2 * j + 1] * m);
                fmax = max(fmax, max(iabs(q0), iabs(q1)));
                w[j] = ((unsigned)q0 & 0xffffu) | ((unsigned)q1 << 16);
            }
            reinterpret_cast<uint4*>(out)[q] = make_uint4(w[0], w[1], w[2], w[3]);
        }
        done = n8 * 8;
    }
    // what is left (everything, without 16-byte alignment): one element per lane
    for (unsigned long long i = done + (unsigned long long)blockIdx.x * kCvtBlock + threadIdx.x; i < n; i += step) {
        const int q = flex_quantize_trunc(cvt_load1<SRC>(in, i) * m);
        fmax = max(fmax, iabs(q));
        out[i] = (short)q;
    }
    __shared__ int lds_slot[kCvtBlock / 64];
    block_stat_max(fmax, partial, lds_slot);
}

}  // namespace ngh
