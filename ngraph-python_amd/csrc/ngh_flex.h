// Device-resident flex exponent management.
//
// The reference reads every output tensor's max|mantissa| back to the host after each
// kernel and updates the scale in Python before the next launch
// (ngraph/transformers/flexgputransform.py:347-366): one host round trip per kernel.
// Here each flex tensor owns a small state record in device memory; kernels read their
// scales from it and merge statistics into it, and two one-wavefront kernels apply the
// exponent policy on the device, so a sequence of flex kernels runs without the host.
//
// The arithmetic below is written as explicit sequential double-precision steps because the
// host mirror (ngraph_hip/flex/hipflex.py, _policy_step) executes the same steps in the same
// order; the two must stay line-for-line equivalent.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ngraph_hip.h"

namespace ngh {

constexpr int kFlexPclip = 32767;
constexpr int kFlexMinDec = 0, kFlexMaxDec = 31;
constexpr int kFlexMaxIds = 8;

struct FlexIds {
    int n;
    int id[kFlexMaxIds];
    int in_place[kFlexMaxIds];   // tensor is also read by the kernel: keep its scale
};

// largest dec in [0, 31] at which |v| fits 15 bits; -1 = leave unchanged (v is 0 or NaN)
__device__ __forceinline__ int flex_fit_dec(double v) {
    v = fabs(v);
    if (v == 0.0 || v != v) return -1;
    if (isinf(v)) return kFlexMinDec;
    int e;
    frexp(v, &e);                       // v = m * 2^e, 0.5 <= m < 1  =>  floor(log2 v) = e - 1
    int dec = 14 - (e - 1);
    return dec < kFlexMinDec ? kFlexMinDec : (dec > kFlexMaxDec ? kFlexMaxDec : dec);
}

__device__ __forceinline__ float flex_scale_of(int dec) { return ldexpf(1.0f, -dec); }

// The exponent a kernel writes a tensor with: the policy's choice once the tensor has been
// written before, unless the kernel also reads it (an in-place update keeps its scale).
__device__ __forceinline__ int flex_write_dec(const ngh_flex_state& s, int in_place) {
    return (!in_place && s.initialized && s.next_dec >= 0) ? s.next_dec : s.dec;
}

// After a write with s.dec / s.scale: record max|mantissa| and choose the next exponent.
__device__ inline void flex_policy_record(ngh_flex_state& s, int maxabs, int count) {
    s.last_maxabs = maxabs;
    s.last_count = count;
    s.initialized = 1;
    const double value = (double)maxabs * (double)s.scale;
    int pos = s.hist_pos;
    if (maxabs >= kFlexPclip) {
        s.history[pos] = 2.0 * value;
        s.hist_pos = (pos + 1) % NGH_FLEX_HISTORY;
        if (s.hist_len < NGH_FLEX_HISTORY) s.hist_len += 1;
        const int d = s.dec - 2;
        s.next_dec = d < kFlexMinDec ? kFlexMinDec : d;
        return;
    }
    s.history[pos] = value;
    s.hist_pos = (pos + 1) % NGH_FLEX_HISTORY;
    if (s.hist_len < NGH_FLEX_HISTORY) s.hist_len += 1;
    const int n = s.hist_len;
    double mx = s.history[0], sum = 0.0;
    for (int j = 0; j < n; ++j) {
        const double h = s.history[j];
        mx = h > mx ? h : mx;
        sum = sum + h;
    }
    const double mean = sum / (double)n;
    double ss = 0.0;
    for (int j = 0; j < n; ++j) {
        const double d = s.history[j] - mean;
        ss = ss + d * d;
    }
    const double sd = sqrt(ss / (double)n);
    const int dec = flex_fit_dec(mx + 3.0 * sd);
    s.next_dec = dec < 0 ? s.dec : dec;
}

// Before a kernel: outputs that are fully overwritten take the exponent the policy chose;
// every output's statistics word is cleared.
__global__ void flex_prepare_kernel(ngh_flex_state* st, const FlexIds ids) {
    const int i = threadIdx.x;
    if (i >= ids.n) return;
    ngh_flex_state& s = st[ids.id[i]];
    const int dec = flex_write_dec(s, ids.in_place[i]);
    if (dec != s.dec) {
        s.dec = dec;
        s.scale = flex_scale_of(dec);
    }
    s.stats = 0;
}

// After a kernel: record max|mantissa| and choose the next exponent.
__global__ void flex_update_kernel(ngh_flex_state* st, const FlexIds ids, int count) {
    const int i = threadIdx.x;
    if (i >= ids.n) return;
    ngh_flex_state& s = st[ids.id[i]];
    flex_policy_record(s, s.stats, count);
}

// ---------------------------------------------------------------------------
// Both steps inside the streaming kernel itself (one launch per managed kernel).
//
// Every workgroup derives the write exponent from the record exactly as flex_prepare_kernel
// would, so no launch has to precede the kernel; the record is only changed by the workgroup
// that finishes last.  Workgroups merge their max|mantissa| into one of kFlexGroups words per
// statistics slot (index = blockIdx.x % kFlexGroups, so no word is hit by more than
// 1/kFlexGroups of the grid) and then take a ticket of their group; a group's last arrival
// takes a ticket of the grid; the grid's last arrival folds the group words and applies the
// policy.  Only device-scope read-modify-write atomics carry the data, each issued after the
// previous one has returned, so an arrival is counted only after its maximum is in place.
// Counters and group words are left at zero for the next launch.
// ---------------------------------------------------------------------------
constexpr int kFlexGroups = 64;
constexpr int kFlexPad = 32;            // ints between two counters: one 128-byte line each
constexpr int kFlexTicketWords = (kFlexGroups + 1) * kFlexPad;
constexpr int kFlexGroupMaxWords = 4 * kFlexGroups * kFlexPad;

template <int NS>
__device__ __forceinline__ void flex_epilogue(ngh_flex_state* const (&state)[4], const int (&in_place)[4],
                                              int count, unsigned* tickets, int* group_max,
                                              const int (&fmax)[4], int (*lds)[4] /* [NS][waves] */) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int m[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        m[s] = fmax[s];
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) m[s] = max(m[s], __shfl_xor(m[s], d, 64));
        if (lane == 0) lds[s][wave] = m[s];
    }
    __syncthreads();
    if (wave != 0) return;
    const unsigned g = blockIdx.x % kFlexGroups;
    const unsigned groups = gridDim.x < (unsigned)kFlexGroups ? gridDim.x : (unsigned)kFlexGroups;
    int last = 0;
    if (lane == 0) {
        unsigned dep = 0;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int bm = max(max(lds[s][0], lds[s][1]), max(lds[s][2], lds[s][3]));
            dep |= (unsigned)__hip_atomic_fetch_max(group_max + (s * kFlexGroups + g) * kFlexPad, bm,
                                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        unsigned one = 1u;
        asm volatile("" : "+v"(one) : "v"(dep));          // the ticket waits for the maxima
        const unsigned members = (gridDim.x - g + kFlexGroups - 1) / kFlexGroups;
        const unsigned t = __hip_atomic_fetch_add(tickets + g * kFlexPad, one, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT);
        if (t == members - 1) {
            __hip_atomic_store(tickets + g * kFlexPad, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned t2 = __hip_atomic_fetch_add(tickets + kFlexGroups * kFlexPad, 1u, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
            if (t2 == groups - 1) {
                __hip_atomic_store(tickets + kFlexGroups * kFlexPad, 0u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
                last = 1;
            }
        }
    }
    last = __shfl(last, 0, 64);
    if (!last) return;
    // the grid's last workgroup, first wavefront: lane g folds group g
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        int gm = 0;
        if ((unsigned)lane < groups) {
            int* w = group_max + (s * kFlexGroups + lane) * kFlexPad;
            gm = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(w, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) gm = max(gm, __shfl_xor(gm, d, 64));
        if (lane == 0) {
            ngh_flex_state& st = *state[s];
            const int dec = flex_write_dec(st, in_place[s]);
            st.dec = dec;
            st.scale = flex_scale_of(dec);
            st.stats = gm;
            flex_policy_record(st, gm, count);
        }
    }
}

}  // namespace ngh
