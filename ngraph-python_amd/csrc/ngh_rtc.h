// Op programs compiled in process and loaded as code objects.
//
// The reference compiles the kernels of a computation with NVRTC inside the process and
// launches them through the driver API (ngraph/transformers/gpu/float_ew2.py:1553-1653:
// CudaSourceFile.compile, SourceModule.get_function, prepared_async_call).  The program
// libraries of ngh_programs_load are shared objects that hipcc built from the same headers, host
// launchers included, which needs hipcc on the machine.  This file is the other way in: the host
// side compiles the same generated source with hiprtc, device code only, and hands over the code
// object and the lowered names of the kernels a program may launch; the launchers here make the
// choices the templated ones in ngh_special.h make (cache policy, ragged rows, deferred
// statistics, tile size, chunks or rows per lane) and launch with hipModuleLaunchKernel.
// Host code only.
#pragma once
#include <atomic>
#include <string>
#include <vector>

#include "ngh_table.h"

namespace ngh {

// Kernel slots per family, in the order ngh_program_kernels lists their name expressions:
//   0  ew_static_kernel<P, cp> cp = 0..3 | ew_ragged_static_kernel<P, cp> | ew_static_lazy_kernel<P, cp>
//   1  red_row_static_kernel<P, cp, false> | <P, cp, true> | red_rows_small_static_kernel<P, false> | <P, true>
//   2  red_col_static_kernel<P, cp>
//   3  ew_tiled_static_kernel<P, 16> | <P, 32> | ew_tiled4_static_kernel<P>
//   4  row_chain_static_kernel<cp, U, stages...> for (cp, U) = (0, 4), (0, 8), (2, 4), (2, 8)
//   5  col_chain_static_kernel<cp, NC, stages...> for cp = 0, 2 and NC = 0, 8, 12
// A slot whose kernel the program cannot have (no ragged form, no elementwise store and hence no
// non-temporal-store variants, no statistics slots) stays empty.
constexpr int kRtcMaxKernels = 12;

struct RtcProgram {
    hipModule_t   module = nullptr;
    hipFunction_t fn[kRtcMaxKernels] = {};
    // resident workgroups per compute unit of the deferred-statistics kernels, 0 until asked
    // (contexts on several threads may launch the same program)
    std::atomic<int> lazy_fit[kCachePolicies];
    bool          ragged_ok = false, stores = false, quad_ok = false, stat_slots = false;
    // what the table entry points to
    char          name[64] = {};
    ngh_op        ops[NGH_MAX_OPS] = {};
    int           dtypes[NGH_MAX_TENSORS] = {};
    unsigned char bcast[NGH_MAX_TENSORS] = {}, rowshared[NGH_MAX_TENSORS] = {};
    signed char   staged[NGH_MAX_TENSORS] = {};
    int           red_out[NGH_MAX_REDUCTIONS] = {};
    StaticEntry   stages[NGH_MAX_STAGES] = {};                // a chain's stages
    RtcProgram() { for (auto& f : lazy_fit) f.store(0); }
};

inline bool desc_ok(const ngh_program_desc& d) {
    return d.family >= 0 && d.family <= 5 && (d.V == 1 || d.V == 4 || d.V == 8) && d.n_ops >= 0 && d.n_ops <= NGH_MAX_OPS && d.n_tensors >= 0 &&
           d.n_tensors <= NGH_MAX_TENSORS && d.n_red >= 0 && d.n_red <= NGH_MAX_REDUCTIONS && d.n_stages >= 0 &&
           d.n_stages <= NGH_MAX_STAGES && d.type_name[sizeof(d.type_name) - 1] == 0 && d.name[sizeof(d.name) - 1] == 0;
}

inline bool desc_stores(const ngh_program_desc& d) {
    for (int i = 0; i < d.n_ops; ++i)
        if (d.ops[i].opcode == NGH_OP_STORE || d.ops[i].opcode == NGH_OP_STORE_TRUNC) return true;
    return false;
}

inline bool desc_ragged_ok(const ngh_program_desc& d) {
    return program_ragged_ok(d.V, d.ops, d.n_ops, d.dtypes, d.bcast);
}

// The name expressions of the kernels program `d` (with its stages, for a chain) may launch, one
// per slot, "" for an empty slot.
inline std::vector<std::string> rtc_kernel_names(const ngh_program_desc& d, const ngh_program_desc* stages) {
    std::vector<std::string> names(kRtcMaxKernels);
    const std::string T = std::string("ngh::") + d.type_name;
    auto num = [](int v) { return std::to_string(v); };
    const bool stores = desc_stores(d), ragged = desc_ragged_ok(d);
    switch (d.family) {
        case 0:
            for (int cp = 0; cp < kCachePolicies; ++cp) {
                names[cp] = "ngh::ew_static_kernel<" + T + ", " + num(cp) + ">";
                if (ragged) names[4 + cp] = "ngh::ew_ragged_static_kernel<" + T + ", " + num(cp) + ">";
                if (d.n_stat_slots > 0) names[8 + cp] = "ngh::ew_static_lazy_kernel<" + T + ", " + num(cp) + ">";
            }
            break;
        case 1:
            for (int cp = 0; cp < kCachePolicies; ++cp) {
                if (!stores && (cp & kCpNtStore)) continue;
                names[cp] = "ngh::red_row_static_kernel<" + T + ", " + num(cp) + ", false>";
                if (ragged) names[4 + cp] = "ngh::red_row_static_kernel<" + T + ", " + num(cp) + ", true>";
            }
            names[8] = "ngh::red_rows_small_static_kernel<" + T + ", false>";
            if (ragged) names[9] = "ngh::red_rows_small_static_kernel<" + T + ", true>";
            break;
        case 2:
            for (int cp = 0; cp < kCachePolicies; ++cp) {
                if (!stores && (cp & kCpNtStore)) continue;
                names[cp] = "ngh::red_col_static_kernel<" + T + ", " + num(cp) + ">";
            }
            break;
        case 3:
            names[0] = "ngh::ew_tiled_static_kernel<" + T + ", 16>";
            names[1] = "ngh::ew_tiled_static_kernel<" + T + ", 32>";
            if (program_quad_ok(d.ops, d.n_ops)) names[2] = "ngh::ew_tiled4_static_kernel<" + T + ">";
            break;
        case 4:
        case 5: {
            std::string list;
            for (int j = 0; j < d.n_stages; ++j) list += std::string(", ngh::") + stages[j].type_name;
            int slot = 0;
            for (int cp = 0; cp <= kCpNtStore; cp += kCpNtStore) {
                if (d.family == 4) {
                    for (int U = kChainAhead / 2; U <= kChainAhead; U *= 2)
                        names[slot++] = "ngh::row_chain_static_kernel<" + num(cp) + ", " + num(U) + list + ">";
                } else {
                    for (int NC : {0, kColCached, kColCachedWide})
                        names[slot++] = "ngh::col_chain_static_kernel<" + num(cp) + ", " + num(NC) + list + ">";
                }
            }
            break;
        }
    }
    return names;
}

inline void rtc_fill_entry(StaticEntry& e, RtcProgram& r, const ngh_program_desc& d) {
    snprintf(r.name, sizeof(r.name), "%s", d.name);
    for (int i = 0; i < d.n_ops; ++i) r.ops[i] = d.ops[i];
    for (int i = 0; i < d.n_tensors; ++i) {
        r.dtypes[i] = d.dtypes[i];
        r.bcast[i] = d.bcast[i];
        r.rowshared[i] = d.rowshared[i];
        r.staged[i] = d.staged[i];
    }
    for (int i = 0; i < d.n_red; ++i) r.red_out[i] = d.red_out[i];
    e = StaticEntry{};
    e.name = r.name;
    e.family = d.family;
    e.V = d.V;
    e.n_ops = d.n_ops;
    e.ops = r.ops;
    e.n_tensors = d.n_tensors;
    e.dtypes = r.dtypes;
    e.bcast = r.bcast;
    e.n_red = d.n_red;
    e.red_out = r.red_out;
    e.staged = r.staged;
    e.rowshared = r.rowshared;
}

// ------------------------------------------------------------------------------------ launchers
inline hipError_t rtc_launch_kernel(hipFunction_t f, unsigned blocks, hipStream_t stream, void** args) {
    if (!f) return hipErrorInvalidDeviceFunction;      // (a slot the program was said not to need)
    return hipModuleLaunchKernel(f, blocks, 1, 1, kBlock, 1, 1, 0, stream, args, nullptr);
}

// family 0 (launch_static in ngh_special.h)
inline hipError_t rtc_launch_ew(const StaticEntry& e, hipStream_t stream, unsigned blocks, const KArgs& k,
                                unsigned n_chunks, unsigned cpr, int cache_policy) {
    RtcProgram& r = *const_cast<RtcProgram*>(e.rtc);
    const int cp = cache_policy & (kCachePolicies - 1);
    void* args[] = {(void*)&k, &n_chunks, &cpr};
    if (r.stat_slots && k.flex_lazy) {
        hipFunction_t f = r.fn[8 + cp];
        int fit = r.lazy_fit[cp].load(std::memory_order_relaxed);
        if (f && fit == 0) {
            if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&fit, f, kBlock, 0) != hipSuccess || fit < 1) {
                (void)hipGetLastError();
                fit = 1;
            }
            r.lazy_fit[cp].store(fit, std::memory_order_relaxed);
        }
        if (fit < 1) fit = 1;
        const unsigned per_cu = k.lazy_blocks_per_cu < 0 ? (unsigned)(-k.lazy_blocks_per_cu)
                              : (unsigned)std::max(1, std::min(k.lazy_blocks_per_cu, fit > 6 ? fit - 2 : fit));
        blocks = std::min(blocks, (unsigned)k.flex_lazy * per_cu);
        return rtc_launch_kernel(f, blocks, stream, args);
    }
    if (r.ragged_ok && k.ragged) return rtc_launch_kernel(r.fn[4 + cp], blocks, stream, args);
    return rtc_launch_kernel(r.fn[cp], blocks, stream, args);
}

// families 1, 2 (launch_static_red)
inline hipError_t rtc_launch_red(const StaticEntry& e, hipStream_t stream, unsigned blocks, const KArgs& k,
                                 unsigned n_first, unsigned n_seg, unsigned seg_len, unsigned TX, RedWs ws,
                                 int cache_policy) {
    const RtcProgram& r = *e.rtc;
    const int cp = cache_policy & (r.stores ? 3 : kCpNtLoad);
    if (e.family == 1) {
        const bool ragged = r.ragged_ok && k.ragged;
        if (TX != 0) {
            // short rows: n_first outputs, TX lanes per row
            void* args[] = {(void*)&k, &n_first, &TX};
            return rtc_launch_kernel(r.fn[ragged ? 9 : 8], blocks, stream, args);
        }
        void* args[] = {(void*)&k, &n_first, &n_seg, &seg_len, &ws};
        return rtc_launch_kernel(r.fn[(ragged ? 4 : 0) + cp], blocks, stream, args);
    }
    void* args[] = {(void*)&k, &n_first, &n_seg, &seg_len, &TX, &ws};
    return rtc_launch_kernel(r.fn[cp], blocks, stream, args);
}

// family 3 (launch_static_tiled)
inline hipError_t rtc_launch_tiled(const StaticEntry& e, hipStream_t stream, unsigned blocks, const KArgs& k,
                                   unsigned tiles_a, unsigned tiles_b, unsigned n_tiles, int tile) {
    const RtcProgram& r = *e.rtc;
    void* args[] = {(void*)&k, &tiles_a, &tiles_b, &n_tiles};
    if (tile == kTile4) return rtc_launch_kernel(r.fn[2], blocks, stream, args);
    return rtc_launch_kernel(r.fn[tile == 16 ? 0 : 1], blocks, stream, args);
}

// families 4, 5 (launch_static_chain, launch_static_col_chain)
inline hipError_t rtc_launch_chain(const StaticEntry& e, hipStream_t stream, unsigned blocks, const KArgs& k,
                                   unsigned n_out, unsigned T, int cache_policy) {
    const RtcProgram& r = *e.rtc;
    const bool nt = (cache_policy & kCpNtStore) != 0;
    void* args[] = {(void*)&k, &n_out, &T};
    if (e.family == 4) {
        const bool half = (unsigned long long)(k.shape[2] + 3) / 4 <= (unsigned long long)T * (kChainAhead / 2);
        return rtc_launch_kernel(r.fn[(nt ? 2 : 0) + (half ? 0 : 1)], blocks, stream, args);
    }
    const unsigned RY = T == kBlock ? 1u : kBlock / T;
    const unsigned long long rows_per_lane = ((unsigned long long)k.shape[0] + RY - 1) / RY;
    const int kept = rows_per_lane <= (unsigned long long)kColCached ? 1
                   : (T == kBlock && rows_per_lane <= (unsigned long long)kColCachedWide) ? 2 : 0;
    return rtc_launch_kernel(r.fn[(nt ? 3 : 0) + kept], blocks, stream, args);
}

}  // namespace ngh
