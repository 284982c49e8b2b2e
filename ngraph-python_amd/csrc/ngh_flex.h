// Device-resident flex exponent management.
//
// The reference reads every output tensor's max|mantissa| back to the host after each
// kernel and updates the scale in Python before the next launch
// (ngraph/transformers/flexgputransform.py:347-366): one host round trip per kernel.
// Here each flex tensor owns a small state record in device memory; kernels read their
// scales from it and merge statistics into it, and two one-wavefront kernels apply the
// exponent policy on the device, so a sequence of flex kernels runs without the host.
//
// The policy arithmetic is a sequence of double-precision steps, each rounded once, because the
// host mirror (ngraph_hip/flex/hipflex.py, _policy_step) executes the same steps in the same
// order; the two must stay equivalent (the library is built with -ffp-contract=off).
#pragma once
#include "ngh_device.h"

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

// stand-in record for unconditional prologue loads (see ngh_safe_word)
static __device__ ngh_flex_state ngh_safe_state = {};

// The exponent a kernel writes a tensor with: the policy's choice once the tensor has been
// written before, unless the kernel also reads it (an in-place update keeps its scale).
__device__ __forceinline__ int flex_write_dec(const ngh_flex_state& s, int in_place) {
    return (!in_place && s.initialized && s.next_dec >= 0) ? s.next_dec : s.dec;
}

// The record's scalar fields, as a kernel holds them while it works on a record.
struct FlexFields {
    int   stats, dec, next_dec, initialized;
    float scale;
    int   hist_len, hist_pos, last_maxabs, last_count;
};

// Entry j of a value held one per lane, as a wavefront-uniform number (j is the same in
// every lane).
__device__ __forceinline__ double flex_lane_value(double v, int j) {
    const int lo = __builtin_amdgcn_readlane(__double2loint(v), j);
    const int hi = __builtin_amdgcn_readlane(__double2hiint(v), j);
    return __hiloint2double(hi, lo);
}

// After a write with f.dec / f.scale: record max|mantissa| and choose the next exponent.
// One wavefront with all 64 lanes active works on a record: every lane holds the same fields,
// lane j (j < NGH_FLEX_HISTORY) holds entry j of the ring of recent maxima in `h`.  The sums
// run over the entries in index order, one rounding per step, exactly as the host mirror's
// loops do; only the per-entry work (subtracting the mean, squaring) is done by all lanes at
// once.
__device__ __forceinline__ void flex_policy_step(FlexFields& f, double& h, int maxabs, int count) {
    const int lane = threadIdx.x & 63;
    const int dec_now = f.dec;
    const double value = (double)maxabs * (double)f.scale;
    const int pos = f.hist_pos;
    const bool clipped = maxabs >= kFlexPclip;
    if (lane == pos) h = clipped ? 2.0 * value : value;
    const int n = f.hist_len < NGH_FLEX_HISTORY ? f.hist_len + 1 : NGH_FLEX_HISTORY;
    int next_dec;
    if (clipped) {
        const int d = dec_now - 2;
        next_dec = d < kFlexMinDec ? kFlexMinDec : d;
    } else {
        // Rolled loops on purpose: this code runs once per launch with a cold instruction cache,
        // and fetching a long unrolled sequence costs more than executing it.
        double mx = flex_lane_value(h, 0), sum = 0.0;
#pragma unroll 1
        for (int j = 0; j < n; ++j) {
            const double hj = flex_lane_value(h, j);
            mx = hj > mx ? hj : mx;
            sum = sum + hj;
        }
        const double mean = sum / (double)n;
        const double d = h - mean;
        const double dd = d * d;
        double ss = 0.0;
#pragma unroll 1
        for (int j = 0; j < n; ++j) ss = ss + flex_lane_value(dd, j);
        const double sd = sqrt(ss / (double)n);
        const int dec = flex_fit_dec(mx + 3.0 * sd);
        next_dec = dec < 0 ? dec_now : dec;
    }
    f.last_maxabs = maxabs;
    f.last_count = count;
    f.initialized = 1;
    f.hist_pos = (pos + 1) % NGH_FLEX_HISTORY;
    f.hist_len = n;
    f.next_dec = next_dec;
}

__device__ __forceinline__ FlexFields flex_fields_of(const ngh_flex_state& s) {
    FlexFields f;
    f.stats = s.stats; f.dec = s.dec; f.next_dec = s.next_dec; f.initialized = s.initialized;
    f.scale = s.scale; f.hist_len = s.hist_len; f.hist_pos = s.hist_pos;
    f.last_maxabs = s.last_maxabs; f.last_count = s.last_count;
    return f;
}

__device__ __forceinline__ void flex_fields_to(ngh_flex_state& s, const FlexFields& f) {
    s.stats = f.stats; s.dec = f.dec; s.next_dec = f.next_dec; s.initialized = f.initialized;
    s.scale = f.scale; s.hist_len = f.hist_len; s.hist_pos = f.hist_pos;
    s.last_maxabs = f.last_maxabs; s.last_count = f.last_count;
}

// A record as one wavefront holds it.
struct FlexInWave {
    FlexFields f;
    double     h;       // lane j < NGH_FLEX_HISTORY: ring entry j
};

__device__ __forceinline__ FlexInWave flex_wave_load(const ngh_flex_state& s) {
    FlexInWave r;
    r.f = flex_fields_of(s);
    r.h = s.history[threadIdx.x & (NGH_FLEX_HISTORY - 1)];
    return r;
}

__device__ __forceinline__ void flex_wave_store(ngh_flex_state& s, const FlexInWave& r) {
    const int lane = threadIdx.x & 63;
    if (lane == 0) flex_fields_to(s, r.f);
    if (lane < NGH_FLEX_HISTORY) s.history[lane] = r.h;
}

// whole wavefront: policy step on a record in memory
__device__ __forceinline__ void flex_policy_record(ngh_flex_state& s, int maxabs, int count) {
    FlexInWave r = flex_wave_load(s);
    flex_policy_step(r.f, r.h, maxabs, count);
    flex_wave_store(s, r);
}

__device__ __forceinline__ int flex_write_dec(const FlexFields& f, int in_place) {
    return (!in_place && f.initialized && f.next_dec >= 0) ? f.next_dec : f.dec;
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

// After a kernel: record max|mantissa| and choose the next exponent.  One wavefront per id.
__global__ __launch_bounds__(64) void flex_update_kernel(ngh_flex_state* st, const FlexIds ids, int count) {
    if ((int)blockIdx.x >= ids.n) return;
    ngh_flex_state& s = st[ids.id[blockIdx.x]];
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

// The last arrival's part: fold the group words of slots first, first + step, ... and apply the
// policy to their records (one wavefront, all lanes).
template <int NS>
__device__ __forceinline__ void flex_epilogue_finish(ngh_flex_state* const (&state)[4], const int (&in_place)[4],
                                                     int count, int* group_max, unsigned groups, int lane,
                                                     int first, int step) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        if (s < first || (s - first) % step) continue;
        int gm = 0;
        if ((unsigned)lane < groups) {
            int* w = group_max + (s * kFlexGroups + lane) * kFlexPad;
            gm = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(w, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) gm = max(gm, __shfl_xor(gm, d, 64));
        FlexInWave r = flex_wave_load(*state[s]);
        const int dec = flex_write_dec(r.f, in_place[s]);
        r.f.dec = dec;
        r.f.scale = flex_scale_of(dec);
        r.f.stats = gm;
        flex_policy_step(r.f, r.h, gm, count);
        flex_wave_store(*state[s], r);
    }
}

// A workgroup's arrival (whole workgroup calls; what it returns is meaningful in the first
// wavefront only: is this workgroup the grid's last arrival?)
template <int NS>
__device__ __forceinline__ int flex_epilogue_arrive(unsigned* tickets, int* group_max, const int (&fmax)[4],
                                                    int (*lds)[4] /* [NS][waves] */, int ordered, unsigned& groups) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    groups = gridDim.x < (unsigned)kFlexGroups ? gridDim.x : (unsigned)kFlexGroups;
    int m[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        m[s] = fmax[s];
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) m[s] = max(m[s], __shfl_xor(m[s], d, 64));
        if (lane == 0) lds[s][wave] = m[s];
    }
    __syncthreads();
    if (wave != 0) return 0;
    const unsigned g = blockIdx.x % kFlexGroups;
    int last = 0;
    if (lane == 0) {
        unsigned dep = 0;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int bm = max(max(lds[s][0], lds[s][1]), max(lds[s][2], lds[s][3]));
            dep |= (unsigned)__hip_atomic_fetch_max(group_max + (s * kFlexGroups + g) * kFlexPad, bm,
                                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // `ordered`: the two tickets are release operations and the last arrival issues an acquire
        // fence, as the memory model asks of a hand-off between workgroups; else they are relaxed and ordered behind the maxima by a
        // data dependency alone, which the hardware honours (see moments_kernel)
        unsigned one = 1u;
        asm volatile("" : "+v"(one) : "v"(dep));          // the ticket waits for the maxima
        const unsigned members = (gridDim.x - g + kFlexGroups - 1) / kFlexGroups;
        const unsigned t = ordered ? __hip_atomic_fetch_add(tickets + g * kFlexPad, one, __ATOMIC_RELEASE,
                                                            __HIP_MEMORY_SCOPE_AGENT)
                                   : __hip_atomic_fetch_add(tickets + g * kFlexPad, one, __ATOMIC_RELAXED,
                                                            __HIP_MEMORY_SCOPE_AGENT);
        if (t == members - 1) {
            __hip_atomic_store(tickets + g * kFlexPad, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (ordered) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // the group's maxima are in
            const unsigned t2 = ordered ? __hip_atomic_fetch_add(tickets + kFlexGroups * kFlexPad, 1u, __ATOMIC_RELEASE,
                                                                 __HIP_MEMORY_SCOPE_AGENT)
                                        : __hip_atomic_fetch_add(tickets + kFlexGroups * kFlexPad, 1u, __ATOMIC_RELAXED,
                                                                 __HIP_MEMORY_SCOPE_AGENT);
            if (t2 == groups - 1) {
                if (ordered) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // every group's maxima are in
                __hip_atomic_store(tickets + kFlexGroups * kFlexPad, 0u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
                last = 1;
            }
        }
    }
    return __shfl(last, 0, 64);
}

template <int NS>
__device__ __forceinline__ void flex_epilogue(ngh_flex_state* const (&state)[4], const int (&in_place)[4],
                                              int count, unsigned* tickets, int* group_max,
                                              const int (&fmax)[4], int (*lds)[4] /* [NS][waves] */,
                                              int ordered) {
    unsigned groups;
    const int last = flex_epilogue_arrive<NS>(tickets, group_max, fmax, lds, ordered, groups);
    if ((threadIdx.x >> 6) != 0 || !last) return;
    // the grid's last workgroup, first wavefront: lane g folds group g
    flex_epilogue_finish<NS>(state, in_place, count, group_max, groups, threadIdx.x & 63, 0, 1);
}

// The same with the last workgroup's wavefronts taking a record each (the policy step of a
// record takes one wavefront a few microseconds, after everything else of the launch is done):
// every wavefront waits to learn whether its workgroup came last.  For kernels that write
// several flex tensors and whose workgroups are about to end anyway.
template <int NS>
__device__ __forceinline__ void flex_epilogue_wide(ngh_flex_state* const (&state)[4], const int (&in_place)[4],
                                                   int count, unsigned* tickets, int* group_max,
                                                   const int (&fmax)[4], int (*lds)[4] /* [NS][waves] */,
                                                   int ordered) {
    __shared__ int came_last;
    unsigned groups;
    const int last = flex_epilogue_arrive<NS>(tickets, group_max, fmax, lds, ordered, groups);
    if (threadIdx.x == 0) came_last = last;
    __syncthreads();
    if (!came_last) return;
    if (ordered) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    flex_epilogue_finish<NS>(state, in_place, count, group_max, groups, threadIdx.x & 63, (int)(threadIdx.x >> 6),
                             (int)(blockDim.x >> 6));
}


// ---------------------------------------------------------------------------
// Deferred statistics: no work at all after the last store.
//
// flex_epilogue's chain of dependent atomics runs after the slowest workgroup has finished
// streaming, so it adds to every launch.  Here a workgroup only sends its max|mantissa| to one
// of kFlexGroups words with an atomic that returns nothing, and the fold and the policy step
// are done by whoever needs the record next: the prologue of the next kernel that writes the
// tensor (every workgroup computes the same new record in registers, workgroup 0 stores it),
// or flex_settle_kernel when something else is about to look at the record.
//
// A record therefore has two pages (the ABI's record, and a shadow) and two sets of group
// words.  A launch reads one page and one set and writes the other page and the other set, so
// no workgroup of a launch reads anything another workgroup of the same launch writes.  Words
// carry the write's sequence number in their upper half: a word left by an older write
// compares lower and reads as "no contribution", so the sets never need clearing.
// ---------------------------------------------------------------------------
constexpr int kFlexWordPad = 16;                                  // 64-bit words per 128-byte line
constexpr int kFlexWordsPerSet = kFlexGroups * kFlexWordPad;
constexpr int kFlexWordsPerRecord = 2 * kFlexWordsPerSet;

// What a wavefront holds of a record between asking for it and needing it.
struct FlexLazyLoaded {
    FlexInWave         r;
    unsigned long long word;    // this lane's group word of the pending write
};

// Issue the loads of a record and of the pending group words (one word per lane).
__device__ __forceinline__ void flex_lazy_fetch(const FlexLazySlot& a, FlexLazyLoaded& l) {
    l.r = flex_wave_load(*a.in);
    // the words were written by the previous kernel's atomics and by nobody in this launch: an
    // ordinary (cacheable) load sees them, and thousands of workgroups asking do not all go to
    // memory
    l.word = a.words_in ? a.words_in[(threadIdx.x & 63) * kFlexWordPad] : 0ull;
}

// Fold what is pending into the record (whole wavefront).
__device__ __forceinline__ void flex_lazy_fold(const FlexLazySlot& a, FlexLazyLoaded& l) {
    if (!a.words_in) return;
    int gm = ((unsigned)(l.word >> 32) == a.tag_in) ? (int)(unsigned)(l.word & 0xffffffffull) : 0;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) gm = max(gm, __shfl_xor(gm, d, 64));
    l.r.f.stats = gm;
    flex_policy_step(l.r.f, l.r.h, gm, a.count_in);
}

// The rest of a streaming kernel's prologue (whole wavefront): fold, choose the exponent of this
// write, leave the record in the other page if `store`, return the scale the kernel writes with.
__device__ __forceinline__ float flex_lazy_finish(const FlexLazySlot& a, FlexLazyLoaded& l, bool store) {
    flex_lazy_fold(a, l);
    const int dec = flex_write_dec(l.r.f, a.in_place);
    l.r.f.dec = dec;
    l.r.f.scale = flex_scale_of(dec);
    if (store) flex_wave_store(*a.out, l.r);
    return l.r.f.scale;
}

template <int NS>
__device__ __forceinline__ void flex_lazy_epilogue(const FlexLazySlot* slots, const int (&fmax)[4],
                                                   int (*lds)[4] /* [NS][waves] */) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        int m = fmax[s];
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) m = max(m, __shfl_xor(m, d, 64));
        if (lane == 0) lds[s][wave] = m;
    }
    __syncthreads();
    if (threadIdx.x >= NS) return;
    const int s = threadIdx.x;
    const int bm = max(max(lds[s][0], lds[s][1]), max(lds[s][2], lds[s][3]));
    const unsigned long long v = ((unsigned long long)slots[s].tag_out << 32) | (unsigned)bm;
    (void)__hip_atomic_fetch_max(slots[s].words_out + (blockIdx.x % kFlexGroups) * kFlexWordPad, v,
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Bring records back to their plain form: fold what is pending and leave the result in the
// ABI's record.  One wavefront per entry.
struct FlexSettleArgs {
    int          n;
    FlexLazySlot slot[kFlexMaxIds];       // out = the ABI's record
};

__global__ __launch_bounds__(64) void flex_settle_kernel(const FlexSettleArgs args) {
    if ((int)blockIdx.x >= args.n) return;
    const FlexLazySlot& a = args.slot[blockIdx.x];
    FlexLazyLoaded l;
    flex_lazy_fetch(a, l);
    flex_lazy_fold(a, l);
    flex_wave_store(*a.out, l.r);
}

}  // namespace ngh
