// Device-side building blocks shared by every fused kernel: the per-element
// arithmetic of each opcode, storage-type conversion on load/store (fp32,
// flex16, int32, fp16), and the register files the op programs run on.
//
// Semantics follow the NumPy float32 calls the CPU transformer issues
// (ngraph/transformers/cputransform.py:512-761) for the op set the GPU
// transformer dispatches (ngraph/transformers/gputransform.py:124-275,
// templates in ngraph/transformers/gpu/float_ew2.py:31-108).
#pragma once
#if !defined(__HIPCC_RTC__)
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#else
// Compiled in process (hiprtc): the HIP device headers are built in, host headers do not exist;
// the fixed-width names the kernel headers use are spelled out here.
typedef signed char int8_t;
typedef unsigned char uint8_t;
typedef short int16_t;
typedef unsigned short uint16_t;
typedef int int32_t;
typedef unsigned int uint32_t;
typedef long long int64_t;
typedef unsigned long long uint64_t;
typedef unsigned long uintptr_t;
#endif
#include "ngraph_hip.h"

namespace ngh {

// ---------------------------------------------------------------------------
// Kernel-side view of one stage of a fused spec.  Axes are already permuted by
// the host planner so that axis 2 is the one lanes run along.
// ---------------------------------------------------------------------------
struct KTensor {
    char*        p;
    long long    s[3];       // element strides along kernel axes 0,1,2
    int          dtype;
    float        scale;
    int*         stats;
    const float* dscale;
    int          stat_slot;  // which per-thread max|mantissa| accumulator, -1 = none
    int          stage_slot; // tiled skeleton: which LDS tile carries this operand, -1 = direct access
    unsigned     take_extent;  // table operand of NGH_OP_TAKE: length of the looked-up axis
    int          pad_;
};

// One statistics slot of a launch with deferred statistics (see ngh_flex.h).
struct FlexLazySlot {
    const ngh_flex_state*     in;         // page holding the record as of the previous write
    ngh_flex_state*           out;        // page this launch leaves the record in
    const unsigned long long* words_in;   // group words of the previous write, NULL = nothing pending
    unsigned long long*       words_out;
    unsigned                  tag_in, tag_out;
    int                       count_in;   // the previous write's `count`
    int                       in_place;
};

struct KArgs {
    long long shape[3];
    int       n_tensors, op_begin, op_end, n_regs;
    int       n_red;
    int       red_out[NGH_MAX_REDUCTIONS];
    int       red_axis;      // kernel axis the reductions run along (0 or 2), -1 = none
    int       iota_map[3];   // kernel axis holding spec axis k (for NGH_OP_IOTA)
    int       n_stat_slots;
    int       n_store_stat_slots;   // the first of them belong to tensors a STORE op writes, the rest to reduction results
    int       n_staged;      // tiled skeleton: operands staged through LDS tiles
    int       tile_diagonal; // tiled skeleton: deal the tiles along diagonals (strides that are multiples of 4 KiB)
    int       ragged;        // rows along kernel axis 2 are not whole aligned vectors: a row's last chunk is short
    unsigned  rng_seed, rng_counter;   // NGH_OP_RNG_*
    int       probe;         // NGH_SPEC_PROBE: record max|value| bits instead of storing
    int*      stat_ptr[4];   // device word of each per-thread accumulator
    int*      stat_partial[4];  // per-workgroup scratch the streaming kernels write instead
    // in-kernel exponent management (pre-built streaming kernels only); flex_state[0] == NULL = off
    ngh_flex_state* flex_state[4];  // per statistics slot: the stored tensor's record
    int       flex_in_place[4];     // the kernel also reads the tensor
    int       flex_count;
    unsigned* tickets;              // arrival counters, zero between launches
    int*      group_max;            // per slot and group: merged max|mantissa|, zero between launches
    int          flex_lazy;         // != 0: deferred statistics, lazy[] is set instead of flex_state[];
                                    // the value is the number of compute units
    FlexLazySlot lazy[4];
    int          lazy_blocks_per_cu;
    int          ordered_arrival;   // last-arrival hand-offs use release / acquire tickets
    KTensor   t[NGH_MAX_TENSORS];
    float     consts[NGH_MAX_CONSTS];
    ngh_op    ops[NGH_MAX_OPS];
};

// ---------------------------------------------------------------------------
// Per-element arithmetic.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float np_sign(float x) {
    // np.sign: -1, 0, +1, NaN for NaN (cputransform.py:727-729)
    return (x > 0.0f) ? 1.0f : ((x < 0.0f) ? -1.0f : ((x == 0.0f) ? 0.0f : x));
}

__device__ __forceinline__ float np_maximum(float a, float b) {
    // np.maximum / np.max propagate NaN (cputransform.py:670-676)
    return (a >= b || a != a) ? a : b;
}
__device__ __forceinline__ float np_minimum(float a, float b) {
    return (a <= b || a != a) ? a : b;
}

// NumPy's float divmod (npy_divmod): floor_divide and mod share it
// (cputransform.py:603-609 emit np.floor_divide / np.mod).
__device__ __forceinline__ void np_divmod(float a, float b, float& floordiv, float& mod) {
    if (b == 0.0f) {
        floordiv = a / b;
        mod = fmodf(a, b);
        return;
    }
    mod = fmodf(a, b);
    float div = (a - mod) / b;
    if (mod != 0.0f) {
        if ((b < 0.0f) != (mod < 0.0f)) {
            mod += b;
            div -= 1.0f;
        }
    } else {
        mod = copysignf(0.0f, b);
    }
    if (div != 0.0f) {
        floordiv = floorf(div);
        if (div - floordiv > 0.5f) floordiv += 1.0f;
    } else {
        floordiv = copysignf(0.0f, a / b);
    }
}

__device__ __forceinline__ float op_unary(int opc, float x) {
    switch (opc) {
        case NGH_OP_ASSIGN:  return x;
        case NGH_OP_NEG:     return -x;
        case NGH_OP_ABS:     return fabsf(x);
        case NGH_OP_SQRT:    return sqrtf(x);
        case NGH_OP_SQR:     return x * x;
        case NGH_OP_EXP:     return expf(x);
        case NGH_OP_LOG:     return logf(x);
        case NGH_OP_RCP:     return 1.0f / x;
        case NGH_OP_EXP2:    return exp2f(x);
        case NGH_OP_LOG2:    return log2f(x);
        case NGH_OP_SIG:     return 1.0f / (1.0f + expf(-x));     // float_ew2.py:43
        case NGH_OP_TANH:    return tanhf(x);
        case NGH_OP_SAFELOG: return (x > 0.0f) ? logf(x) : -50.0f; // float_ew2.py:48
        case NGH_OP_SGN:     return np_sign(x);
        case NGH_OP_SIN:     return sinf(x);
        case NGH_OP_COS:     return cosf(x);
        // integer ops: the register's bits read as int32 / uint32
        case NGH_OP_I2F:     return (float)__float_as_int(x);
        case NGH_OP_U2F:     return (float)__float_as_uint(x);
        case NGH_OP_INEG:    return __uint_as_float(0u - __float_as_uint(x));
        case NGH_OP_IABS: {
            const int i = __float_as_int(x);
            return __uint_as_float(i < 0 ? 0u - (unsigned)i : (unsigned)i);
        }
        default:             return x;
    }
}

__device__ __forceinline__ float op_binary(int opc, float x, float y) {
    switch (opc) {
        case NGH_OP_ADD: return x + y;
        case NGH_OP_SUB: return x - y;
        case NGH_OP_MUL: return x * y;
        case NGH_OP_DIV: return x / y;
        case NGH_OP_INT_DIV: { float q, m; np_divmod(x, y, q, m); return q; }
        case NGH_OP_MOD:     { float q, m; np_divmod(x, y, q, m); return m; }
        case NGH_OP_EQ: return (x == y) ? 1.0f : 0.0f;
        case NGH_OP_NE: return (x != y) ? 1.0f : 0.0f;
        case NGH_OP_LT: return (x <  y) ? 1.0f : 0.0f;
        case NGH_OP_LE: return (x <= y) ? 1.0f : 0.0f;
        case NGH_OP_GT: return (x >  y) ? 1.0f : 0.0f;
        case NGH_OP_GE: return (x >= y) ? 1.0f : 0.0f;
        case NGH_OP_POW: return powf(x, y);
        case NGH_OP_MINIMUM: return np_minimum(x, y);
        case NGH_OP_MAXIMUM: return np_maximum(x, y);
        default: break;
    }
    // integer ops: both registers' bits read as int32 / uint32 (unsigned arithmetic wraps)
    const unsigned ux = __float_as_uint(x), uy = __float_as_uint(y);
    const int ix = (int)ux, iy = (int)uy;
    switch (opc) {
        case NGH_OP_IADD: return __uint_as_float(ux + uy);
        case NGH_OP_ISUB: return __uint_as_float(ux - uy);
        case NGH_OP_IMUL: return __uint_as_float(ux * uy);
        case NGH_OP_IMIN: return __int_as_float(ix < iy ? ix : iy);
        case NGH_OP_IMAX: return __int_as_float(ix > iy ? ix : iy);
        case NGH_OP_UMIN: return __uint_as_float(ux < uy ? ux : uy);
        case NGH_OP_UMAX: return __uint_as_float(ux > uy ? ux : uy);
        case NGH_OP_IEQ: return (ix == iy) ? 1.0f : 0.0f;
        case NGH_OP_INE: return (ix != iy) ? 1.0f : 0.0f;
        case NGH_OP_ILT: return (ix <  iy) ? 1.0f : 0.0f;
        case NGH_OP_ILE: return (ix <= iy) ? 1.0f : 0.0f;
        case NGH_OP_IGT: return (ix >  iy) ? 1.0f : 0.0f;
        case NGH_OP_IGE: return (ix >= iy) ? 1.0f : 0.0f;
        case NGH_OP_ULT: return (ux <  uy) ? 1.0f : 0.0f;
        case NGH_OP_ULE: return (ux <= uy) ? 1.0f : 0.0f;
        case NGH_OP_UGT: return (ux >  uy) ? 1.0f : 0.0f;
        case NGH_OP_UGE: return (ux >= uy) ? 1.0f : 0.0f;
        default: return x;
    }
}

__host__ __device__ constexpr bool is_unary(int opc) {
    return (opc >= NGH_OP_ASSIGN && opc <= NGH_OP_COS) || (opc >= NGH_OP_I2F && opc <= NGH_OP_IABS);
}
__host__ __device__ constexpr bool is_binary(int opc) {
    return (opc >= NGH_OP_ADD && opc <= NGH_OP_MAXIMUM) || (opc >= NGH_OP_IADD && opc <= NGH_OP_UGE);
}
__host__ __device__ constexpr bool is_reduce(int opc) { return opc >= NGH_OP_RED_SUM && opc <= NGH_OP_RED_ARGMIN; }
// (ops that cost about as much as a handful of additions: transcendentals, division, power)
__host__ __device__ constexpr bool is_slow_op(int opc) {
    return (opc >= NGH_OP_EXP && opc <= NGH_OP_COS && opc != NGH_OP_RCP && opc != NGH_OP_SGN) || opc == NGH_OP_POW ||
           opc == NGH_OP_DIV;
}

// ---------------------------------------------------------------------------
// flex16 conversion (float_ew2.py:96-97, 261-277): load = scale * mantissa;
// store = cvt.rni.s16.f32(scale * value): round to nearest even, saturate to
// [-32768, 32767], NaN -> 0; statistics = max |stored mantissa| as int32.
// ---------------------------------------------------------------------------
// The device's float -> int32 conversion as the instruction defines it: toward zero, values out
// of range (infinities included) saturate, NaN gives 0.  A C cast leaves those cases undefined,
// so code that relies on them asks for the instruction itself.
__device__ __forceinline__ int cvt_i32_saturating(float v) {
    int q;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(q) : "v"(v));
    return q;
}

__device__ __forceinline__ int flex_quantize(float v) {
    const int q = cvt_i32_saturating(rintf(v));   // round-half-even in the default mode; NaN -> 0
    return min(max(q, -32768), 32767);
}

// ---------------------------------------------------------------------------
// Philox-4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11):
// a counter-based generator, so an element's number depends only on (key, counter).
// ---------------------------------------------------------------------------
struct Philox4 { unsigned x[4]; };

__device__ __forceinline__ Philox4 philox4x32_10(unsigned c0, unsigned c1, unsigned c2, unsigned c3,
                                                 unsigned k0, unsigned k1) {
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        const unsigned lo0 = 0xD2511F53u * c0, hi0 = __umulhi(0xD2511F53u, c0);
        const unsigned lo1 = 0xCD9E8D57u * c2, hi1 = __umulhi(0xCD9E8D57u, c2);
        const unsigned n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    Philox4 r;
    r.x[0] = c0; r.x[1] = c1; r.x[2] = c2; r.x[3] = c3;
    return r;
}

// uniform in [0, 1) with 24 random bits; standard normal by Box-Muller
__device__ __forceinline__ float rng_uniform01(unsigned bits) { return (float)(bits >> 8) * (1.0f / 16777216.0f); }
__device__ __forceinline__ float rng_normal(unsigned b0, unsigned b1) {
    const float u1 = ((float)(b0 >> 8) + 1.0f) * (1.0f / 16777216.0f);       // (0, 1]
    const float u2 = rng_uniform01(b1);
    return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
}

// the fill rule: int(value / scale) cut toward zero, clipped (tensor_ops.py:690-707)
__device__ __forceinline__ int flex_quantize_trunc(float v) {
    return min(max(cvt_i32_saturating(v), -32768), 32767);          // (the conversion cuts toward zero; NaN -> 0)
}

__device__ __forceinline__ int iabs(int x) { return x < 0 ? -x : x; }

// bit pattern of |v| (ordered like the value for non-negative floats); NaN counts as 0
__device__ __forceinline__ int probe_bits(float v) {
    return (v != v) ? 0 : (__float_as_int(v) & 0x7fffffff);
}

// ---------------------------------------------------------------------------
// Element access by storage type.
// ---------------------------------------------------------------------------
// A word that is always there to be read.  A kernel's prologue fetches the scales of its flex
// operands through pointers that may be NULL; "load if not NULL" is a branch, and a branch per
// operand makes the fetches a chain of round trips, one after the other, ahead of the kernel's
// first load of data.  Loading from this word instead of from NULL keeps them unconditional
// and in flight together.
static __device__ float ngh_safe_word = 1.0f;

__device__ __forceinline__ float tensor_scale(const KTensor& t) {
    const float* p = t.dscale ? t.dscale : &ngh_safe_word;
    const float v = *p;
    return t.dscale ? v : t.scale;
}

__device__ __forceinline__ float load1(const KTensor& t, long long off, float scale) {
    switch (t.dtype) {
        case NGH_F32:    return reinterpret_cast<const float*>(t.p)[off];
        case NGH_FLEX16: return scale * (float)reinterpret_cast<const short*>(t.p)[off];
        case NGH_I32:    return (float)reinterpret_cast<const int*>(t.p)[off];
        case NGH_F16:    return __half2float(reinterpret_cast<const __half*>(t.p)[off]);
        case NGH_U32:    return (float)reinterpret_cast<const unsigned*>(t.p)[off];
        case NGH_I16:    return (float)reinterpret_cast<const short*>(t.p)[off];
        case NGH_I8:     return (float)reinterpret_cast<const signed char*>(t.p)[off];
        case NGH_U8:     return (float)reinterpret_cast<const unsigned char*>(t.p)[off];
        default:         return 0.0f;
    }
}

// float -> integer storage: toward zero, saturating at the type's range, NaN -> 0
// (what the hardware conversion does for 32-bit results; narrower types clamp first).
__device__ __forceinline__ int to_int_sat(float v, float lo, float hi) {
    return (int)fminf(fmaxf(v, lo), hi);
}

__device__ __forceinline__ void store1(const KTensor& t, long long off, float v, float scale, int& fmax) {
    switch (t.dtype) {
        case NGH_F32: reinterpret_cast<float*>(t.p)[off] = v; break;
        case NGH_FLEX16: {
            int q = flex_quantize(scale * v);
            reinterpret_cast<short*>(t.p)[off] = (short)q;
            fmax = max(fmax, iabs(q));
        } break;
        case NGH_I32: reinterpret_cast<int*>(t.p)[off] = (int)v; break;
        case NGH_F16: reinterpret_cast<__half*>(t.p)[off] = __float2half(v); break;
        case NGH_U32: reinterpret_cast<unsigned*>(t.p)[off] = (unsigned)v; break;
        case NGH_I16: reinterpret_cast<short*>(t.p)[off] = (short)to_int_sat(v, -32768.0f, 32767.0f); break;
        case NGH_I8:  reinterpret_cast<signed char*>(t.p)[off] = (signed char)to_int_sat(v, -128.0f, 127.0f); break;
        case NGH_U8:  reinterpret_cast<unsigned char*>(t.p)[off] = (unsigned char)to_int_sat(v, 0.0f, 255.0f); break;
        default: break;
    }
}

// 4 consecutive elements; `off` is a multiple of 4 and the base is aligned.
__device__ __forceinline__ void load4(const KTensor& t, long long off, float scale, float (&v)[4]) {
    switch (t.dtype) {
        case NGH_F32: {
            float4 x = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(t.p) + off);
            v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
        } break;
        case NGH_FLEX16: {
            short4 x = *reinterpret_cast<const short4*>(reinterpret_cast<const short*>(t.p) + off);
            v[0] = scale * (float)x.x; v[1] = scale * (float)x.y;
            v[2] = scale * (float)x.z; v[3] = scale * (float)x.w;
        } break;
        case NGH_I32: {
            int4 x = *reinterpret_cast<const int4*>(reinterpret_cast<const int*>(t.p) + off);
            v[0] = (float)x.x; v[1] = (float)x.y; v[2] = (float)x.z; v[3] = (float)x.w;
        } break;
        case NGH_F16: {
            const __half2* h = reinterpret_cast<const __half2*>(reinterpret_cast<const __half*>(t.p) + off);
            uint2 raw = *reinterpret_cast<const uint2*>(h);
            __half2 a = *reinterpret_cast<__half2*>(&raw.x), b = *reinterpret_cast<__half2*>(&raw.y);
            float2 fa = __half22float2(a), fb = __half22float2(b);
            v[0] = fa.x; v[1] = fa.y; v[2] = fb.x; v[3] = fb.y;
        } break;
        case NGH_U32: {
            uint4 x = *reinterpret_cast<const uint4*>(reinterpret_cast<const unsigned*>(t.p) + off);
            v[0] = (float)x.x; v[1] = (float)x.y; v[2] = (float)x.z; v[3] = (float)x.w;
        } break;
        case NGH_I16: {
            short4 x = *reinterpret_cast<const short4*>(reinterpret_cast<const short*>(t.p) + off);
            v[0] = (float)x.x; v[1] = (float)x.y; v[2] = (float)x.z; v[3] = (float)x.w;
        } break;
        case NGH_I8: {
            const unsigned w = *reinterpret_cast<const unsigned*>(t.p + off);
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = (float)(signed char)((w >> (8 * j)) & 0xffu);
        } break;
        case NGH_U8: {
            const unsigned w = *reinterpret_cast<const unsigned*>(t.p + off);
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = (float)((w >> (8 * j)) & 0xffu);
        } break;
        default: v[0] = v[1] = v[2] = v[3] = 0.0f;
    }
}

__device__ __forceinline__ void store4(const KTensor& t, long long off, float scale, const float (&v)[4], int& fmax) {
    switch (t.dtype) {
        case NGH_F32:
            *reinterpret_cast<float4*>(reinterpret_cast<float*>(t.p) + off) = make_float4(v[0], v[1], v[2], v[3]);
            break;
        case NGH_FLEX16: {
            int q0 = flex_quantize(scale * v[0]), q1 = flex_quantize(scale * v[1]);
            int q2 = flex_quantize(scale * v[2]), q3 = flex_quantize(scale * v[3]);
            short4 x; x.x = (short)q0; x.y = (short)q1; x.z = (short)q2; x.w = (short)q3;
            *reinterpret_cast<short4*>(reinterpret_cast<short*>(t.p) + off) = x;
            fmax = max(max(fmax, max(iabs(q0), iabs(q1))), max(iabs(q2), iabs(q3)));
        } break;
        case NGH_I32:
            *reinterpret_cast<int4*>(reinterpret_cast<int*>(t.p) + off) =
                make_int4((int)v[0], (int)v[1], (int)v[2], (int)v[3]);
            break;
        case NGH_F16: {
            __half2 a = __floats2half2_rn(v[0], v[1]), b = __floats2half2_rn(v[2], v[3]);
            uint2 raw; raw.x = *reinterpret_cast<unsigned*>(&a); raw.y = *reinterpret_cast<unsigned*>(&b);
            *reinterpret_cast<uint2*>(reinterpret_cast<__half*>(t.p) + off) = raw;
        } break;
        case NGH_U32:
            *reinterpret_cast<uint4*>(reinterpret_cast<unsigned*>(t.p) + off) =
                make_uint4((unsigned)v[0], (unsigned)v[1], (unsigned)v[2], (unsigned)v[3]);
            break;
        case NGH_I16: {
            short4 x;
            x.x = (short)to_int_sat(v[0], -32768.0f, 32767.0f); x.y = (short)to_int_sat(v[1], -32768.0f, 32767.0f);
            x.z = (short)to_int_sat(v[2], -32768.0f, 32767.0f); x.w = (short)to_int_sat(v[3], -32768.0f, 32767.0f);
            *reinterpret_cast<short4*>(reinterpret_cast<short*>(t.p) + off) = x;
        } break;
        case NGH_I8: {
            unsigned w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) w |= ((unsigned)to_int_sat(v[j], -128.0f, 127.0f) & 0xffu) << (8 * j);
            *reinterpret_cast<unsigned*>(t.p + off) = w;
        } break;
        case NGH_U8: {
            unsigned w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) w |= ((unsigned)to_int_sat(v[j], 0.0f, 255.0f) & 0xffu) << (8 * j);
            *reinterpret_cast<unsigned*>(t.p + off) = w;
        } break;
        default: break;
    }
}

// V consecutive elements (V = 4, 8 or 16).  16-bit elements travel eight to a 16-byte
// access, which is what keeps enough bytes in flight per lane for 2-byte storage types.
template <int V>
__device__ __forceinline__ void loadv(const KTensor& t, long long off, float scale, float (&v)[V]) {
    static_assert(V == 4 || V == 8 || V == 16, "vector width");
    if constexpr (V == 4) {
        load4(t, off, scale, v);
    } else {
        if (t.dtype == NGH_FLEX16 || t.dtype == NGH_F16) {
#pragma unroll
            for (int g = 0; g < V / 8; ++g) {
                const uint4 raw = *reinterpret_cast<const uint4*>(t.p + (off + 8 * g) * 2);
                const unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (t.dtype == NGH_FLEX16) {
                        v[8 * g + 2 * j] = scale * (float)(short)(w[j] & 0xffffu);
                        v[8 * g + 2 * j + 1] = scale * (float)(short)(w[j] >> 16);
                    } else {
                        unsigned u = w[j];
                        const float2 f = __half22float2(*reinterpret_cast<__half2*>(&u));
                        v[8 * g + 2 * j] = f.x;
                        v[8 * g + 2 * j + 1] = f.y;
                    }
                }
            }
        } else {
#pragma unroll
            for (int g = 0; g < V / 4; ++g) {
                float a[4];
                load4(t, off + 4 * g, scale, a);
#pragma unroll
                for (int j = 0; j < 4; ++j) v[4 * g + j] = a[j];
            }
        }
    }
}

template <int V>
__device__ __forceinline__ void storev(const KTensor& t, long long off, float scale, const float (&v)[V], int& fmax) {
    static_assert(V == 4 || V == 8 || V == 16, "vector width");
    if constexpr (V == 4) {
        store4(t, off, scale, v, fmax);
    } else {
        if (t.dtype == NGH_FLEX16 || t.dtype == NGH_F16) {
#pragma unroll
            for (int g = 0; g < V / 8; ++g) {
                unsigned w[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (t.dtype == NGH_FLEX16) {
                        const int q0 = flex_quantize(scale * v[8 * g + 2 * j]);
                        const int q1 = flex_quantize(scale * v[8 * g + 2 * j + 1]);
                        fmax = max(fmax, max(iabs(q0), iabs(q1)));
                        w[j] = ((unsigned)q0 & 0xffffu) | ((unsigned)q1 << 16);
                    } else {
                        __half2 h = __floats2half2_rn(v[8 * g + 2 * j], v[8 * g + 2 * j + 1]);
                        w[j] = *reinterpret_cast<unsigned*>(&h);
                    }
                }
                *reinterpret_cast<uint4*>(t.p + (off + 8 * g) * 2) = make_uint4(w[0], w[1], w[2], w[3]);
            }
        } else {
#pragma unroll
            for (int g = 0; g < V / 4; ++g) {
                const float a[4] = {v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3]};
                store4(t, off + 4 * g, scale, a, fmax);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Register file of the op interpreter.  The program is only known at run
// time, so register numbers are run-time values; a per-lane array indexed that
// way would live in scratch memory.  The file is kept in LDS instead, laid
// out [register][vector element][thread] so lanes of a wavefront hit
// consecutive banks.
// ---------------------------------------------------------------------------
template <int V>
struct LdsRegs {
    float* base;   // &lds[thread]
    int    nthr;   // threads per workgroup
    __device__ __forceinline__ float get(int r, int v) const { return base[(r * V + v) * nthr]; }
    __device__ __forceinline__ void  set(int r, int v, float x) { base[(r * V + v) * nthr] = x; }
};

// ---------------------------------------------------------------------------
// Reduction accumulators (float_ew2.py:70-108: inits 0 / 1 / -FLT_MAX /
// FLT_MAX; argmax/argmin carry (value, index)).  Ties resolve to the lowest
// index, as np.argmax / np.argmin do (cputransform.py:521-527).
// ---------------------------------------------------------------------------
struct Acc {
    float v;
    int   i;
};

__device__ __forceinline__ Acc acc_init(int opc) {
    Acc a; a.i = 0;
    switch (opc) {
        case NGH_OP_RED_SUM:    a.v = 0.0f; break;
        case NGH_OP_RED_PROD:   a.v = 1.0f; break;
        case NGH_OP_RED_MAX:    a.v = -__builtin_inff(); break;
        case NGH_OP_RED_MIN:    a.v =  __builtin_inff(); break;
        case NGH_OP_RED_ARGMAX: a.v = -__builtin_inff(); a.i = 0x7fffffff; break;
        case NGH_OP_RED_ARGMIN: a.v =  __builtin_inff(); a.i = 0x7fffffff; break;
        default: a.v = 0.0f;
    }
    return a;
}

__device__ __forceinline__ Acc acc_merge(int opc, Acc a, Acc b) {
    switch (opc) {
        case NGH_OP_RED_SUM:  a.v = a.v + b.v; break;
        case NGH_OP_RED_PROD: a.v = a.v * b.v; break;
        case NGH_OP_RED_MAX:  a.v = np_maximum(a.v, b.v); break;
        case NGH_OP_RED_MIN:  a.v = np_minimum(a.v, b.v); break;
        case NGH_OP_RED_ARGMAX: {
            bool a_nan = a.v != a.v, b_nan = b.v != b.v;
            bool take_b = (a_nan || b_nan) ? (b_nan && (!a_nan || b.i < a.i))
                                           : (b.v > a.v || (b.v == a.v && b.i < a.i));
            if (take_b) a = b;
        } break;
        case NGH_OP_RED_ARGMIN: {
            bool a_nan = a.v != a.v, b_nan = b.v != b.v;
            bool take_b = (a_nan || b_nan) ? (b_nan && (!a_nan || b.i < a.i))
                                           : (b.v < a.v || (b.v == a.v && b.i < a.i));
            if (take_b) a = b;
        } break;
        default: break;
    }
    return a;
}

__device__ __forceinline__ float acc_result(int opc, Acc a) {
    return (opc == NGH_OP_RED_ARGMAX || opc == NGH_OP_RED_ARGMIN) ? (float)a.i : a.v;
}

__device__ __forceinline__ Acc acc_shfl_xor(Acc a, int mask) {
    Acc b;
    b.v = __shfl_xor(a.v, mask, 64);
    b.i = __shfl_xor(a.i, mask, 64);
    return b;
}

// Reduce a per-thread max|mantissa| over the workgroup and leave it in this workgroup's slot
// of a scratch array; a one-workgroup fold kernel launched right after merges the slots
// into the tensor's statistics word.  No atomics in the streaming kernel: thousands of
// workgroups finishing together and hitting one word with atomicMax cost more than the
// kernel's memory traffic (measured: 22 us -> 38 us for the 16 M element flex kernel).
__device__ __forceinline__ void block_stat_max(int m, int* partial, int* lds_slot /* [nwaves], one per call */) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) m = max(m, __shfl_xor(m, s, 64));
    const int wave = threadIdx.x >> 6, nwaves = (blockDim.x * blockDim.y + 63) >> 6;
    if ((threadIdx.x & 63) == 0) lds_slot[wave] = m;
    __syncthreads();
    if (threadIdx.x == 0 && partial != nullptr) {
        for (int w = 1; w < nwaves; ++w) m = max(m, lds_slot[w]);
        partial[blockIdx.x] = m;
    }
}

__global__ __launch_bounds__(256) void stats_fold_kernel(const int* __restrict__ partial, unsigned n,
                                                         int* __restrict__ word) {
    __shared__ int sh[4];
    int m = 0;
    // eight loads at a time: one workgroup folds up to tens of thousands of partial maxima, and a
    // load per round trip would make this tiny kernel take longer than the kernel it follows
    unsigned i = threadIdx.x;
    for (; i + 7 * 256 < n; i += 8 * 256) {
        int v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = partial[i + j * 256];
#pragma unroll
        for (int j = 0; j < 8; ++j) m = max(m, v[j]);
    }
    for (; i < n; i += 256) m = max(m, partial[i]);
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) m = max(m, __shfl_xor(m, s, 64));
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = max(max(sh[0], sh[1]), max(sh[2], sh[3]));
        if (m > 0) atomicMax(word, m);
    }
}

__device__ __forceinline__ int wave_max_int(int x) {
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) x = max(x, __shfl_xor(x, m, 64));
    return x;
}

}  // namespace ngh
