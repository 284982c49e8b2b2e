// The table of compiled op programs: the ones built into the library (ngh_programs.inc) and the
// ones loaded at run time (ngh_programs_load: a shared object hipcc built; ngh_programs_load_code:
// a code object hiprtc built inside the process, ngh_rtc.h).
//
// Counterpart of the reference's kernel cache (ngraph/transformers/gpu/float_ew2.py:1486-1529
// _ops_to_hash, :1560-1567 compiled-kernel lookup): there a structural hash of the op list finds
// a kernel that NVRTC already compiled for this process, here a structural comparison finds a
// kernel compiled with the library, or later by the host side (ngraph_hip/runtime/jit.py).
// Anything without an entry runs on the interpreter.
#pragma once
#include <atomic>
#include <cstdint>
#include <mutex>

#include "ngh_special.h"

namespace ngh {

#include "ngh_programs.inc"

// Entries of loaded program libraries.  Append-only and in place: a slot is filled, then
// published by the count (release / acquire), so readers need no lock and an index, once handed
// out, stays valid for the life of the process; the libraries stay loaded.
constexpr int kMaxLoadedPrograms = 4096;
struct LoadedPrograms {
    std::mutex       lock;                       // writers only
    StaticEntry      entries[kMaxLoadedPrograms];
    uint64_t         hash[kMaxLoadedPrograms];   // of what match_special compares: a quick reject
    std::atomic<int> count{0};
};
inline LoadedPrograms& loaded_programs() {
    static LoadedPrograms table;
    return table;
}

inline uint64_t mix_hash(uint64_t h, uint64_t v) {
    h ^= v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
    return h;
}
inline uint64_t program_hash(int family, int V, int n_ops, const ngh_op* ops, int n_tensors, int n_red) {
    uint64_t h = mix_hash(mix_hash(mix_hash(mix_hash((uint64_t)family, (uint64_t)V), (uint64_t)n_ops),
                                   (uint64_t)n_tensors), (uint64_t)n_red);
    for (int j = 0; j < n_ops; ++j)
        h = mix_hash(h, ((uint64_t)(uint32_t)ops[j].opcode << 48) ^ ((uint64_t)(uint32_t)ops[j].dst << 32) ^
                            ((uint64_t)(uint32_t)ops[j].a << 16) ^ (uint64_t)(uint32_t)ops[j].b);
    return h;
}

inline const StaticEntry& special_entry(int i) {
    return i < kStaticCount ? kStaticTable[i] : loaded_programs().entries[i - kStaticCount];
}

inline const char* special_name(int i) { return special_entry(i).name; }

inline bool entry_matches(const StaticEntry& e, int family, int V, const KArgs& k) {
    const int n_ops = k.op_end - k.op_begin;
    if (e.family != family || e.V != V || e.n_ops != n_ops || e.n_tensors != k.n_tensors || e.n_red != k.n_red)
        return false;
    bool same = true;
    for (int r = 0; r < e.n_red && same; ++r) same = e.red_out[r] == k.red_out[r];
    for (int j = 0; j < n_ops && same; ++j) {
        const ngh_op &a = e.ops[j], &b = k.ops[k.op_begin + j];
        same = a.opcode == b.opcode && a.dst == b.dst && a.a == b.a && a.b == b.b;
    }
    for (int t = 0; t < k.n_tensors && same; ++t)
        same = e.dtypes[t] == k.t[t].dtype && (e.bcast[t] != 0) == (k.t[t].s[2] == 0) &&
               (family != 3 || e.staged[t] == k.t[t].stage_slot);
    return same;
}

// family: 0 streaming elementwise (V >= 4: vector access; V == 1: one element per lane, any
// strides), 1 / 2 reductions, 3 tiled elementwise
inline int match_special(int family, int V, const KArgs& k, long long /*tail*/) {
    if (family > 3 || (family == 0 && ((V != 1 && V < 4) || k.n_red != 0))) return -1;
    for (int i = 0; i < kStaticCount; ++i)
        if (entry_matches(kStaticTable[i], family, V, k)) return i;
    LoadedPrograms& L = loaded_programs();
    const int n = L.count.load(std::memory_order_acquire);
    if (n == 0) return -1;
    const uint64_t h = program_hash(family, V, k.op_end - k.op_begin, k.ops + k.op_begin, k.n_tensors, k.n_red);
    for (int i = 0; i < n; ++i)
        if (L.hash[i] == h && entry_matches(L.entries[i], family, V, k)) return kStaticCount + i;
    return -1;
}

// A chain (family 4) whose stages are the programs of `ks` (argument blocks of the spec's stages
// in row order: kernel axis 2 = the reduced axis; families[i] = 1 for a stage with reductions,
// 0 for an elementwise one), or -1.
// `family` 5: a column chain (argument blocks in the spec's own axis order: kernel axis 0 = the
// reduced, strided axis; families[i] = 2 for a stage with reductions); its entries mark the
// operands that are the same for every row (stride 0 along kernel axis 0).
inline int match_chain(const KArgs* ks, const int* families, int n, int family = 4) {
    auto matches = [&](const StaticEntry& e) {
        if (e.family != family || e.chain_len != n) return false;
        for (int i = 0; i < n; ++i) {
            if (!entry_matches(e.chain[i], families[i], 4, ks[i])) return false;
            for (int t = 0; t < ks[i].n_tensors; ++t) {
                const bool shared = family == 5 ? ks[i].t[t].s[0] == 0 : (ks[i].t[t].s[0] == 0 && ks[i].t[t].s[1] == 0);
                if ((e.chain[i].rowshared[t] != 0) != shared) return false;
            }
        }
        return true;
    };
    for (int i = 0; i < kStaticCount; ++i)
        if (matches(kStaticTable[i])) return i;
    LoadedPrograms& L = loaded_programs();
    const int count = L.count.load(std::memory_order_acquire);
    for (int i = 0; i < count; ++i)
        if (matches(L.entries[i])) return kStaticCount + i;
    return -1;
}

// Same program (what match_special compares), whatever the name.
inline bool same_program(const StaticEntry& a, const StaticEntry& b) {
    if (a.family != b.family || a.V != b.V || a.n_ops != b.n_ops || a.n_tensors != b.n_tensors || a.n_red != b.n_red)
        return false;
    if (a.family == 4 || a.family == 5) {
        if (a.chain_len != b.chain_len) return false;
        for (int i = 0; i < a.chain_len; ++i) {
            if (!same_program(a.chain[i], b.chain[i])) return false;
            for (int t = 0; t < a.chain[i].n_tensors; ++t)
                if ((a.chain[i].rowshared[t] != 0) != (b.chain[i].rowshared[t] != 0)) return false;
        }
        return true;
    }
    for (int r = 0; r < a.n_red; ++r) if (a.red_out[r] != b.red_out[r]) return false;
    for (int j = 0; j < a.n_ops; ++j)
        if (a.ops[j].opcode != b.ops[j].opcode || a.ops[j].dst != b.ops[j].dst || a.ops[j].a != b.ops[j].a ||
            a.ops[j].b != b.ops[j].b)
            return false;
    for (int t = 0; t < a.n_tensors; ++t)
        if (a.dtypes[t] != b.dtypes[t] || (a.bcast[t] != 0) != (b.bcast[t] != 0) ||
            (a.family == 3 && a.staged[t] != b.staged[t]))
            return false;
    return true;
}

// Add the entries of a loaded library that the table does not hold yet; returns how many were
// new, or -1 when the table is full.
inline int add_loaded_programs(const StaticEntry* entries, int n) {
    LoadedPrograms& L = loaded_programs();
    std::lock_guard<std::mutex> guard(L.lock);
    int added = 0;
    for (int i = 0; i < n; ++i) {
        const int have = L.count.load(std::memory_order_relaxed);
        bool known = false;
        for (int j = 0; j < kStaticCount && !known; ++j) known = same_program(kStaticTable[j], entries[i]);
        for (int j = 0; j < have && !known; ++j) known = same_program(L.entries[j], entries[i]);
        if (known) continue;
        if (have == kMaxLoadedPrograms) return -1;
        L.entries[have] = entries[i];
        L.hash[have] = program_hash(entries[i].family, entries[i].V, entries[i].n_ops, entries[i].ops,
                                    entries[i].n_tensors, entries[i].n_red);
        L.count.store(have + 1, std::memory_order_release);
        ++added;
    }
    return added;
}

inline unsigned streaming_blocks(int cus, int blocks_per_cu, unsigned n_chunks) {
    unsigned blocks = (n_chunks + kBlock - 1) / kBlock;
    const unsigned cap = (unsigned)(cus * blocks_per_cu);
    return blocks > cap ? cap : blocks;
}

// the launchers of programs whose kernels live in a code object loaded at run time (ngh_rtc.h)
inline hipError_t rtc_launch_ew(const StaticEntry& e, hipStream_t stream, unsigned blocks, const KArgs& k,
                                unsigned n_chunks, unsigned cpr, int cache_policy);
inline hipError_t rtc_launch_red(const StaticEntry& e, hipStream_t stream, unsigned blocks, const KArgs& k,
                                 unsigned n_first, unsigned n_seg, unsigned seg_len, unsigned TX, RedWs ws,
                                 int cache_policy);
inline hipError_t rtc_launch_tiled(const StaticEntry& e, hipStream_t stream, unsigned blocks, const KArgs& k,
                                   unsigned tiles_a, unsigned tiles_b, unsigned n_tiles, int tile);
inline hipError_t rtc_launch_chain(const StaticEntry& e, hipStream_t stream, unsigned blocks, const KArgs& k,
                                   unsigned n_out, unsigned T, int cache_policy);

inline hipError_t launch_special_tiled(int i, hipStream_t stream, unsigned blocks, const KArgs& k, unsigned tiles_a,
                                       unsigned tiles_b, unsigned n_tiles, int tile) {
    const StaticEntry& e = special_entry(i);
    if (e.rtc) return rtc_launch_tiled(e, stream, blocks, k, tiles_a, tiles_b, n_tiles, tile);
    e.launch_tiled(stream, blocks, k, tiles_a, tiles_b, n_tiles, tile);
    return hipGetLastError();
}

inline hipError_t launch_special_red(int i, hipStream_t stream, unsigned blocks, const KArgs& k, unsigned n_first,
                                     unsigned n_seg, unsigned seg_len, unsigned TX, RedWs ws, int cache_policy) {
    const StaticEntry& e = special_entry(i);
    if (e.rtc) return rtc_launch_red(e, stream, blocks, k, n_first, n_seg, seg_len, TX, ws, cache_policy);
    e.launch_red(stream, blocks, k, n_first, n_seg, seg_len, TX, ws, cache_policy);
    return hipGetLastError();
}

inline hipError_t launch_special_chain(int i, hipStream_t stream, unsigned blocks, const KArgs& k, unsigned n_out,
                                       unsigned TR, int cache_policy) {
    const StaticEntry& e = special_entry(i);
    if (e.rtc) return rtc_launch_chain(e, stream, blocks, k, n_out, TR, cache_policy);
    e.launch_chain(stream, blocks, k, n_out, TR, cache_policy);
    return hipGetLastError();
}

inline hipError_t launch_special(int i, hipStream_t stream, unsigned blocks, const KArgs& k,
                                 unsigned n_chunks, unsigned chunks_per_row, int cache_policy) {
    if (n_chunks == 0) return hipSuccess;
    const StaticEntry& e = special_entry(i);
    if (e.rtc) return rtc_launch_ew(e, stream, blocks, k, n_chunks, chunks_per_row, cache_policy);
    e.launch(stream, blocks, k, n_chunks, chunks_per_row, cache_policy);
    return hipGetLastError();
}

}  // namespace ngh
