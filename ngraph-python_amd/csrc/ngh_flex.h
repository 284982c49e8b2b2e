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

// Before a kernel: outputs that are fully overwritten take the exponent the policy chose;
// every output's statistics word is cleared.
__global__ void flex_prepare_kernel(ngh_flex_state* st, const FlexIds ids) {
    const int i = threadIdx.x;
    if (i >= ids.n) return;
    ngh_flex_state& s = st[ids.id[i]];
    if (!ids.in_place[i] && s.initialized && s.next_dec >= 0) {
        s.dec = s.next_dec;
        s.scale = flex_scale_of(s.dec);
    }
    s.stats = 0;
}

// After a kernel: record max|mantissa| and choose the next exponent.
__global__ void flex_update_kernel(ngh_flex_state* st, const FlexIds ids, int count) {
    const int i = threadIdx.x;
    if (i >= ids.n) return;
    ngh_flex_state& s = st[ids.id[i]];
    const int maxabs = s.stats;
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

}  // namespace ngh
