// libngraph_hip.so -- C ABI implementation: context, device memory, the
// planner that maps one stage of a fused spec onto a kernel skeleton, and the
// launches.  See include/ngraph_hip.h for the contract of every entry point.
#include <hip/hip_runtime.h>
#include <dlfcn.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "ngraph_hip.h"
#include "ngh_device.h"
#include "ngh_interp.h"
#include "ngh_copy.h"
#include "ngh_table.h"
#include "ngh_rtc.h"
#include "ngh_moments.h"
#include "ngh_flex.h"
#include "ngh_convert.h"
#include "ngh_hostio.h"

using namespace ngh;

// ---------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------
namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                    \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess)                                                            \
            return fail(e_ == hipErrorOutOfMemory ? NGH_E_NOMEM : NGH_E_RUNTIME,         \
                        "%s failed: %s", #expr, hipGetErrorString(e_));                  \
    } while (0)

#define NGH_TRY(expr)                \
    do {                             \
        int rc_ = (expr);            \
        if (rc_ != NGH_OK) return rc_; \
    } while (0)

int itemsize_of(int dtype) {
    switch (dtype) {
        case NGH_F32: case NGH_I32: case NGH_U32: return 4;
        case NGH_FLEX16: case NGH_F16: case NGH_I16: return 2;
        case NGH_I8: case NGH_U8: return 1;
        default: return 0;
    }
}

int env_int(const char* name, int dflt) {
    const char* s = getenv(name);
    return (s && *s) ? atoi(s) : dflt;
}

}  // namespace

// Scratch of ngh_moments_f32_noalloc, the entry point for callers that cannot allocate: the
// per-segment partial sums (one 8-byte word per row and segment) and the per-row arrival
// counters that ngh_moments_f32 keeps in context-owned allocations.  Every device the library
// runs on holds one copy until the process ends; its address on a device is looked up once,
// in ngh_init, with that device current, and only that address is ever handed to a kernel.
constexpr size_t kNoAllocPartials = 65536;   // rows x segments of one call
constexpr size_t kNoAllocRows = 65536;       // rows of one call
constexpr size_t kNoAllocScratchBytes = kNoAllocPartials * sizeof(unsigned long long) + kNoAllocRows * sizeof(unsigned);
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
constexpr int kMaxDevices = 64;
static void* g_scratch_of_device[kMaxDevices] = {nullptr};

// Host-side bookkeeping of deferred statistics (ngh_flex.h): where each record of a table
// allocated by ngh_flex_states_alloc currently lives and whether a fold is outstanding.
struct FlexRecordHost {
    uint8_t  page = 0;      // 0 = the ABI's record, 1 = the shadow page
    uint8_t  pending = 0;   // group words of write `seq` have not been folded in yet
    uint32_t seq = 0;       // number of deferred writes so far (tag of the latest one)
    int32_t  count = 0;     // that write's `count`
    bool unsettled() const { return page != 0 || pending != 0; }
};

struct FlexTable {
    ngh_flex_state*     base = nullptr;
    int32_t             n = 0;
    ngh_flex_state*     shadow = nullptr;   // second page of every record
    unsigned long long* words = nullptr;    // per record: 2 sets of kFlexGroups padded words
    std::vector<FlexRecordHost> rec;
    ngh_flex_state* page(int32_t id, int which) const { return (which ? shadow : base) + id; }
    unsigned long long* set(int32_t id, uint32_t seq) const {
        return words + ((size_t)id * 2 + (seq & 1u)) * ngh::kFlexWordsPerSet;
    }
};

struct ngh_context {
    std::vector<FlexTable> flex_tables;
    int         flex_unsettled = 0;  // records not in their plain form
    int         device = 0;
    int         cus = 0;
    void*       noalloc_scratch = nullptr;   // this device's copy of `scratch`
    hipStream_t stream = nullptr;
    hipEvent_t  ev0 = nullptr, ev1 = nullptr;
    ngh::HostStaging staging;        // pinned ring + copy threads for large host <-> device copies
    int         copy_threads = 8;    // 0: leave large copies to the runtime's own staging
    size_t      staging_slot_bytes = 16u << 20;
    size_t      staged_min_bytes = 4u << 20;   // smaller copies are not worth the threads
    void*       io_tmp = nullptr;    // device scratch for strided host I/O (ngh_io_scratch)
    size_t      io_tmp_bytes = 0;
    void*       ws = nullptr;        // partial results of split reductions
    size_t      ws_bytes = 0;
    unsigned*   tickets = nullptr;   // zero between launches: per-row / per-launch arrival counters
    size_t      n_tickets = 0;
    int*        stat_ws = nullptr;   // per-workgroup max|mantissa| of streaming kernels
    unsigned    stat_ws_blocks = 0;  // capacity per statistics slot
    int         ew_blocks_per_cu = 64;
    int         force_interp = 0;    // never pick a specialised kernel
    int         red_wgs_per_cu = 8;  // workgroups per CU a split reduction along the contiguous axis aims for
    int         red_col_wgs_per_cu = 2;  // ... and one across it
    // launches captured into a HIP graph (ngh_graph_*)
    hipStream_t main_stream = nullptr;    // the context's stream while a capture redirects ctx->stream
    hipStream_t side_stream = nullptr;    // carries the launches of a side branch during a capture
    hipEvent_t  fork_ev = nullptr, join_ev = nullptr;
    bool        capturing = false, side_open = false;
    int         chain_wgs_per_cu = 0;     // row chains: at most this many workgroups per compute unit, each taking several turns (0: one workgroup per group of rows)
    int         col_chain_wgs_per_cu = 2; // workgroups per compute unit a column chain narrows its workgroups for
    int         row_wave_chunks = 0;     // rows of up to this many chunks are reduced by one wavefront each
    int         tile4 = 1;               // tiled elementwise programs may take 64 x 64 tiles with 16-byte accesses
    int         no_tiles = 0;        // never use the LDS-tiled elementwise skeleton
    int         no_pairs = 0;        // never run two independent specs as one launch
    int         no_chain = 0;        // never run the stages of a spec as one row-chain kernel
    int         wide_min_rows = 2;   // column reductions: rows from which a whole workgroup lies along the columns
    int         no_ragged = 0;       // never run compiled programs 4-wide over rows that are not whole aligned vectors
    int         flex_self_managed = 2;  // ngh_launch_fused_flex: 0 = prepare / kernel / update launches,
                                     // 1 = policy at the end of the kernel, 2 = statistics deferred to the next user
                                     // for stages up to stream_bytes and 1 beyond, 3 = always deferred
    int         cache_policy = -1;   // -1: from the operands' cache hints; 0..3 forces bit 0 = non-temporal
                                     // loads, bit 1 = non-temporal stores in pre-built kernels
    long long   stream_bytes = 192ll << 20;  // hints act on stages touching at least this much memory
    int         moments_wgs_per_cu = 8;
    int         ordered_arrival = 2; // grid-wide hand-offs.  2 (default): the moments kernel ends after writing its
                                     // partial sums and a second small launch merges them (ordered by the kernel
                                     // boundary; +1 us on a 31 us kernel).  One launch with last-arrival tickets:
                                     // 1 = release tickets + acquire fence (what the memory model asks for;
                                     // measured 2.6x slower on the moments kernel: a device-scope release per
                                     // workgroup), 0 = relaxed tickets behind a data dependency (relies on gfx950)
    int         flex_lazy_blocks_per_cu = 6;  // grid of a launch with deferred statistics
    char        name[256] = "";
    uint64_t    total_bytes = 0;
};

// ---------------------------------------------------------------------------
// spec validation (host only; also run before every launch so a malformed
// spec can never reach a kernel)
// ---------------------------------------------------------------------------
namespace {

constexpr long long kMaxStageElems = 1LL << 33;
constexpr unsigned kExactIntegers = 1u << 24;     // integers an fp32 register holds exactly
constexpr long long kSmallReduction = 1LL << 19;   // elements: below this a reduction stays one launch
constexpr int kFlexMaxLazyRecords = 4096;   // tables up to this size get pages and words for deferred statistics

int validate(const ngh_fused_spec* sp) {
    if (!sp) return fail(NGH_E_INVALID, "spec is NULL");
    if (sp->abi_version != NGH_ABI_VERSION)
        return fail(NGH_E_INVALID, "spec abi_version %d, library %d", sp->abi_version, NGH_ABI_VERSION);
    if (sp->rank < 1 || sp->rank > NGH_MAX_AXES) return fail(NGH_E_INVALID, "rank %d out of 1..3", sp->rank);
    long long total = 1;
    for (int a = 0; a < NGH_MAX_AXES; ++a) {
        if (sp->shape[a] < 0) return fail(NGH_E_INVALID, "negative shape on axis %d", a);
        if (a >= sp->rank && sp->shape[a] != 1) return fail(NGH_E_INVALID, "axis %d beyond rank must have length 1", a);
        if (sp->shape[a] > kMaxStageElems || (sp->shape[a] > 0 && total > kMaxStageElems / sp->shape[a]))
            return fail(NGH_E_UNSUPPORTED, "iteration space exceeds 2^33 elements");
        total *= sp->shape[a];
    }
    if (sp->n_tensors < 0 || sp->n_tensors > NGH_MAX_TENSORS) return fail(NGH_E_INVALID, "n_tensors %d", sp->n_tensors);
    if (sp->n_ops < 0 || sp->n_ops > NGH_MAX_OPS) return fail(NGH_E_INVALID, "n_ops %d", sp->n_ops);
    if (sp->n_consts < 0 || sp->n_consts > NGH_MAX_CONSTS) return fail(NGH_E_INVALID, "n_consts %d", sp->n_consts);
    if (sp->n_regs < 0 || sp->n_regs > NGH_MAX_REGS) return fail(NGH_E_INVALID, "n_regs %d", sp->n_regs);
    if (sp->n_stages < 1 || sp->n_stages > NGH_MAX_STAGES) return fail(NGH_E_INVALID, "n_stages %d", sp->n_stages);
    for (int t = 0; t < sp->n_tensors; ++t) {
        const ngh_tensor& T = sp->tensors[t];
        if (itemsize_of(T.dtype) == 0) return fail(NGH_E_INVALID, "tensor %d: unknown dtype %d", t, T.dtype);
        if (total > 0 && T.dev == nullptr) return fail(NGH_E_INVALID, "tensor %d: NULL device pointer", t);
        if (((uintptr_t)T.dev) % itemsize_of(T.dtype)) return fail(NGH_E_INVALID, "tensor %d: misaligned pointer", t);
        __int128 reach = 0;      // byte offset of the last element the view can name
        for (int a = 0; a < NGH_MAX_AXES; ++a) {
            if (T.strides[a] < 0) return fail(NGH_E_UNSUPPORTED, "tensor %d: negative stride", t);
            if (sp->shape[a] > 1) reach += (__int128)(sp->shape[a] - 1) * T.strides[a];
        }
        if (reach * itemsize_of(T.dtype) >= ((__int128)1 << 47))
            return fail(NGH_E_UNSUPPORTED, "tensor %d: view spans more than 2^47 bytes", t);
    }
    int next = 0;
    for (int s = 0; s < sp->n_stages; ++s) {
        const ngh_stage& S = sp->stages[s];
        if (S.op_begin != next || S.op_end < S.op_begin || S.op_end > sp->n_ops)
            return fail(NGH_E_INVALID, "stage %d: op range [%d,%d) does not follow %d", s, S.op_begin, S.op_end, next);
        next = S.op_end;
        if (S.n_reductions < 0 || S.n_reductions > NGH_MAX_REDUCTIONS)
            return fail(NGH_E_INVALID, "stage %d: n_reductions %d", s, S.n_reductions);
        bool defined[NGH_MAX_REGS] = {false};
        bool along0[NGH_MAX_REGS] = {false};     // the value varies along axis 0
        int n_red_seen = 0;
        for (int pc = S.op_begin; pc < S.op_end; ++pc) {
            const ngh_op& o = sp->ops[pc];
            const int opc = o.opcode;
            auto reg_ok = [&](int r) { return r < sp->n_regs; };
            auto need = [&](int r) { return reg_ok(r) && defined[r]; };
            if (n_red_seen && !is_reduce(opc))
                return fail(NGH_E_INVALID, "stage %d: op %d follows a reduction inside the stage", s, pc);
            if (opc == NGH_OP_LOAD) {
                if (o.a >= sp->n_tensors || !reg_ok(o.dst)) return fail(NGH_E_INVALID, "op %d: bad LOAD", pc);
                defined[o.dst] = true;
                along0[o.dst] = sp->shape[0] > 1 && sp->tensors[o.a].strides[0] != 0;
            } else if (opc == NGH_OP_STORE || opc == NGH_OP_STORE_TRUNC) {
                if (o.dst >= sp->n_tensors || !need(o.a)) return fail(NGH_E_INVALID, "op %d: bad STORE", pc);
                const ngh_tensor& T = sp->tensors[o.dst];
                for (int a = 0; a < NGH_MAX_AXES; ++a) {
                    if (sp->shape[a] <= 1 || T.strides[a] != 0) continue;
                    // One value per row (axis 0 is the row, the axis reductions run along): allowed for a
                    // value that is the same all along the row -- computed from operands broadcast along
                    // it, such as the results of earlier stages' reductions.
                    if (a == 0 && opc == NGH_OP_STORE && !along0[o.a]) continue;
                    return fail(NGH_E_INVALID, "op %d: STORE to a tensor broadcast along axis %d", pc, a);
                }
            } else if (opc == NGH_OP_CONST) {
                if (o.a >= sp->n_consts || !reg_ok(o.dst)) return fail(NGH_E_INVALID, "op %d: bad CONST", pc);
                defined[o.dst] = true;
                along0[o.dst] = false;
            } else if (opc == NGH_OP_RNG_UNIFORM || opc == NGH_OP_RNG_NORMAL) {
                if (!reg_ok(o.dst)) return fail(NGH_E_INVALID, "op %d: bad RNG destination", pc);
                defined[o.dst] = true;
                along0[o.dst] = true;
            } else if (opc == NGH_OP_TAKE) {
                const int t = o.b & 15, axis = o.b >> 4;
                if (t >= sp->n_tensors || axis >= sp->rank || !need(o.a) || !reg_ok(o.dst))
                    return fail(NGH_E_INVALID, "op %d: bad TAKE", pc);
                if (sp->tensors[t].take_extent == 0)
                    return fail(NGH_E_INVALID, "op %d: TAKE from tensor %d without take_extent", pc, t);
                if (sp->tensors[t].take_extent > kExactIntegers)
                    return fail(NGH_E_UNSUPPORTED, "op %d: TAKE along an axis of %u entries: indices travel in fp32 "
                                "registers, exact up to 2^24", pc, sp->tensors[t].take_extent);
                defined[o.dst] = true;
                along0[o.dst] = true;
            } else if (opc == NGH_OP_IOTA) {
                if (o.a >= NGH_MAX_AXES || !reg_ok(o.dst)) return fail(NGH_E_INVALID, "op %d: bad IOTA", pc);
                if (sp->shape[o.a] > (long long)kExactIntegers)
                    return fail(NGH_E_UNSUPPORTED, "op %d: IOTA along an axis of %lld: index values travel in fp32 "
                                "registers, exact up to 2^24", pc, (long long)sp->shape[o.a]);
                defined[o.dst] = true;
                along0[o.dst] = true;
            } else if (is_unary(opc)) {
                if (!need(o.a) || !reg_ok(o.dst)) return fail(NGH_E_INVALID, "op %d: unary operand undefined", pc);
                defined[o.dst] = true;
                along0[o.dst] = along0[o.a];
            } else if (is_binary(opc)) {
                if (!need(o.a) || !need(o.b) || !reg_ok(o.dst))
                    return fail(NGH_E_INVALID, "op %d: binary operand undefined", pc);
                defined[o.dst] = true;
                along0[o.dst] = along0[o.a] || along0[o.b];
            } else if (is_reduce(opc)) {
                if (!need(o.a) || o.dst != n_red_seen || n_red_seen >= S.n_reductions)
                    return fail(NGH_E_INVALID, "op %d: reduction slot %d out of order", pc, o.dst);
                const int ot = S.red_out[n_red_seen];
                if (ot < 0 || ot >= sp->n_tensors) return fail(NGH_E_INVALID, "stage %d: red_out[%d]", s, n_red_seen);
                const ngh_tensor& T = sp->tensors[ot];
                // argmax / argmin store their index as an integer into integer storage; through any
                // other storage type it passes through fp32
                if ((opc == NGH_OP_RED_ARGMAX || opc == NGH_OP_RED_ARGMIN) && sp->shape[0] > (long long)kExactIntegers &&
                    T.dtype != NGH_I32 && T.dtype != NGH_U32)
                    return fail(NGH_E_UNSUPPORTED, "stage %d: argmax/argmin over %lld elements needs an int32 or "
                                "uint32 result (fp32 is exact up to 2^24)", s, (long long)sp->shape[0]);
                if (T.strides[0] != 0 && sp->shape[0] > 1)
                    return fail(NGH_E_INVALID, "stage %d: reduction output %d must have stride 0 on axis 0", s, ot);
                for (int a = 1; a < NGH_MAX_AXES; ++a)
                    if (sp->shape[a] > 1 && T.strides[a] == 0)
                        return fail(NGH_E_INVALID, "stage %d: reduction output broadcast along axis %d", s, a);
                ++n_red_seen;
            } else if (opc != NGH_OP_NOP) {
                return fail(NGH_E_INVALID, "op %d: unknown opcode %d", pc, opc);
            }
        }
        if (n_red_seen != S.n_reductions)
            return fail(NGH_E_INVALID, "stage %d: %d reduction ops for n_reductions %d", s, n_red_seen, S.n_reductions);
    }
    if (next != sp->n_ops) return fail(NGH_E_INVALID, "stages cover %d of %d ops", next, sp->n_ops);
    return NGH_OK;
}

// ---------------------------------------------------------------------------
// planner
// ---------------------------------------------------------------------------
enum Family { F_EW = 0, F_RED_ROW, F_RED_COL, F_EW_TILED };
constexpr int kRowWaveChunks = 1024;

struct Plan {
    Family   family = F_EW;
    int      V = 1;                               // elements per lane (pre-built kernels)
    int      Vi = 1;                              // elements per lane when the interpreter runs the stage
    KArgs    k;
    unsigned n_chunks = 0, chunks_per_row = 0;   // EW
    unsigned n_out = 0, n_seg = 1, seg_len = 0;  // reductions
    unsigned n_bx = 0;
    int      special = -1;                        // index into the specialised-kernel table
    long long tail = 0;                           // 1-D contiguous stage: elements left to a scalar launch
    int      perm[3] = {0, 1, 2};                 // kernel axis j holds spec axis perm[j]
    unsigned tx = 64;                                 // column reduction: column chunks per wavefront;
                                                      // short-row reduction: lanes per row
    bool     small_rows = false;                      // row reduction with several rows per workgroup
    unsigned tiles_a = 0, tiles_b = 0, n_tiles = 0;   // tiled elementwise
    int      tile = kTile;
    int      cache_policy = 0;
    unsigned load_mask = 0, store_mask = 0;           // tensors the stage loads / stores
};

// Which tensors does the stage touch (load or store or reduce into)?
void stage_tensors(const ngh_fused_spec& sp, const ngh_stage& S, bool* loads, bool* stores) {
    for (int t = 0; t < NGH_MAX_TENSORS; ++t) loads[t] = stores[t] = false;
    for (int pc = S.op_begin; pc < S.op_end; ++pc) {
        const ngh_op& o = sp.ops[pc];
        if (o.opcode == NGH_OP_LOAD) loads[o.a] = true;
        if (o.opcode == NGH_OP_STORE || o.opcode == NGH_OP_STORE_TRUNC) stores[o.dst] = true;
    }
}

void fill_kargs(const ngh_fused_spec& sp, const ngh_stage& S, const int perm[3], KArgs& k) {
    // kernel axis j holds spec axis perm[j]
    memset(&k, 0, sizeof(k));
    for (int j = 0; j < 3; ++j) {
        k.shape[j] = sp.shape[perm[j]];
        k.iota_map[perm[j]] = j;
    }
    k.n_tensors = sp.n_tensors;
    k.op_begin = S.op_begin;
    k.op_end = S.op_end;
    k.n_regs = sp.n_regs;
    k.n_red = S.n_reductions;
    k.red_axis = -1;
    k.probe = (sp.flags & NGH_SPEC_PROBE) ? 1 : 0;
    k.rng_seed = sp.rng_seed;
    k.rng_counter = sp.rng_counter;
    for (int r = 0; r < S.n_reductions; ++r) k.red_out[r] = S.red_out[r];
    if (S.n_reductions) k.red_axis = k.iota_map[0];
    bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS];
    stage_tensors(sp, S, loads, stores);
    for (int t = 0; t < sp.n_tensors; ++t) {
        const ngh_tensor& T = sp.tensors[t];
        KTensor& K = k.t[t];
        K.p = (char*)T.dev;
        for (int j = 0; j < 3; ++j) K.s[j] = T.strides[perm[j]];
        K.dtype = T.dtype;
        K.scale = T.scale;
        K.stats = T.dev_stats;
        K.dscale = T.dev_scale;
        K.stat_slot = -1;
        K.stage_slot = -1;
        K.take_extent = T.take_extent;
        if (stores[t] && T.dtype == NGH_FLEX16 && k.n_stat_slots < 4) {
            K.stat_slot = k.n_stat_slots;
            k.stat_ptr[k.n_stat_slots++] = T.dev_stats;
        } else if (stores[t] && T.dtype == NGH_FLEX16 && T.dev_stats != nullptr) {
            k.n_stat_slots = 5;      // more flex results with statistics than slots: plan_stage rejects
        }
    }
    // flex results of the stage's reductions take the statistics slots the stores left (their
    // max|mantissa| then travels through per-workgroup partial maxima like a store's, instead
    // of one atomic per result on the tensor's statistics word)
    k.n_store_stat_slots = std::min(k.n_stat_slots, 4);
    for (int r = 0; r < S.n_reductions && k.n_stat_slots < 4; ++r) {
        const int t = S.red_out[r];
        if (t < 0 || t >= sp.n_tensors) continue;
        KTensor& K = k.t[t];
        if (K.dtype == NGH_FLEX16 && K.stats != nullptr && K.stat_slot < 0) {
            K.stat_slot = k.n_stat_slots;
            k.stat_ptr[k.n_stat_slots++] = K.stats;
        }
    }
    memcpy(k.consts, sp.consts, sizeof(k.consts));
    memcpy(k.ops, sp.ops, sizeof(k.ops));
}

// Can the stage move V consecutive elements per lane along kernel axis 2?
bool vec_ok(const KArgs& k, const bool* used, int V, bool any_type = false) {
    if (k.shape[2] % V) return false;
    for (int t = 0; t < k.n_tensors; ++t) {
        if (!used[t]) continue;
        const KTensor& K = k.t[t];
        if (K.s[2] == 0) continue;
        if (K.s[2] != 1) return false;
        const int isz = itemsize_of(K.dtype);
        if (V >= 8 && isz != 2 && !any_type) return false;   // pre-built kernels: 8-wide only pays for 16-bit storage
        const int align = std::min(16, V * isz);
        if (((uintptr_t)K.p) % align) return false;
        for (int j = 0; j < 2; ++j)
            if (k.shape[j] > 1 && K.s[j] % V) return false;
    }
    return true;
}

bool vec4_ok(const KArgs& k, const bool* used) { return vec_ok(k, used, 4); }

// Can the stage move 4 elements per lane along kernel axis 2 although vec_ok says no -- rows whose
// length is not a multiple of 4, or that do not start on 16-byte boundaries?  The compiled
// programs can (program_ragged_ok has the conditions on the program), given unit strides.
// (chain: as a stage of a row chain, which also takes 16-bit operands whose every chunk of four
// lies on a 4-byte boundary: an aligned start, rows an even number of elements apart)
bool ragged_rows_ok(const KArgs& k, const bool* used, bool chain = false) {
    if (k.shape[2] < 8) return false;
    int dtypes[NGH_MAX_TENSORS];
    unsigned char bcast[NGH_MAX_TENSORS];
    for (int t = 0; t < NGH_MAX_TENSORS; ++t) {
        dtypes[t] = t < k.n_tensors ? k.t[t].dtype : NGH_F32;
        bcast[t] = (t < k.n_tensors && k.t[t].s[2] == 0) ? 1 : 0;
        if (t < k.n_tensors && used[t] && k.t[t].s[2] != 0 && k.t[t].s[2] != 1) return false;
        if (t < k.n_tensors && used[t] && k.t[t].s[2] == 1 && itemsize_of(k.t[t].dtype) == 2) {
            const KTensor& K = k.t[t];
            if (((uintptr_t)K.p) % 4) return false;
            for (int j = 0; j < 2; ++j)
                if (k.shape[j] > 1 && K.s[j] % 2) return false;
        }
    }
    return program_ragged_ok(4, k.ops + k.op_begin, k.op_end - k.op_begin, dtypes, bcast, chain);
}

constexpr size_t kInterpLdsPreferred = 64 * 1024;   // keeps >= 2 workgroups per CU
constexpr size_t kInterpLdsMax = 128 * 1024;
constexpr size_t kInterpLdsWide = 40 * 1024;        // budget when widening the interpreter's vectors

// registers (V elements each) + statistics slots + reduction accumulators (`na` per slot)
size_t interp_lds_bytes(const KArgs& k, int V, int na = 1) {
    return ((size_t)k.n_regs * V + k.n_stat_slots + 2 * k.n_red * na) * kBlock * sizeof(float);
}

size_t tiled_lds_bytes(const KArgs& k, int tile) {
    return interp_lds_bytes(k, tile * tile / kBlock) + (size_t)k.n_staged * tile_words(tile) * sizeof(float);
}

// Elements per lane of the gather kernel: 4 when every operand is contiguous (or broadcast)
// along the lanes and the register file still fits; 1 otherwise -- batching uncoalesced
// accesses only deepens the queue in front of the texture addresser (measured 1.4x slower).
int gather_width(const KArgs& k) {
    if (k.shape[0] * k.shape[1] * k.shape[2] < 256LL * kBlock * 4) return 1;   // too small to fill the chip 4-wide
    for (int t = 0; t < k.n_tensors; ++t)
        if (k.t[t].s[2] != 0 && k.t[t].s[2] != 1) return 1;
    return interp_lds_bytes(k, 4) <= kInterpLdsPreferred ? 4 : 1;
}

int plan_stage_impl(const ngh_context* ctx, const ngh_fused_spec& sp, int stage, Plan& P, bool allow_ragged);

int plan_stage(const ngh_context* ctx, const ngh_fused_spec& sp, int stage, Plan& P) {
    NGH_TRY(plan_stage_impl(ctx, sp, stage, P, !(ctx && (ctx->force_interp || ctx->no_ragged))));
    // Ragged rows are a mode of the compiled programs only: a stage without one (yet) is planned
    // again for the interpreter.  (Without a context the plan says what a program should be
    // compiled for.)
    if (P.k.ragged && ctx && (P.k.probe || match_special(P.family, P.V, P.k, 0) < 0)) {
        P = Plan();
        NGH_TRY(plan_stage_impl(ctx, sp, stage, P, false));
    }
    if (P.k.n_stat_slots > 4)
        return fail(NGH_E_UNSUPPORTED, "stage %d stores more than 4 flex16 tensors with statistics", stage);
    return NGH_OK;
}

int plan_stage_impl(const ngh_context* ctx, const ngh_fused_spec& sp, int stage, Plan& P, bool allow_ragged) {
    const ngh_stage& S = sp.stages[stage];
    bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS], used[NGH_MAX_TENSORS];
    stage_tensors(sp, S, loads, stores);
    for (int t = 0; t < NGH_MAX_TENSORS; ++t) used[t] = loads[t] || stores[t];
    long long total = sp.shape[0] * sp.shape[1] * sp.shape[2];
    if (total >= kMaxStageElems) return fail(NGH_E_UNSUPPORTED, "stage view of %lld elements exceeds 2^33", total);
    for (int pc = S.op_begin; pc < S.op_end; ++pc)
        if (sp.ops[pc].opcode == NGH_OP_STORE && sp.shape[0] > 1 && sp.tensors[sp.ops[pc].dst].strides[0] == 0)
            return fail(NGH_E_UNSUPPORTED, "stage %d stores one value per row: only a row chain runs it "
                        "(ngh_plan_chain tells whether the spec is one and has a compiled program)", stage);

    if (S.n_reductions == 0) {
        // fast axis = the one along which most memory traffic is contiguous: every
        // operand votes with the number of distinct elements it touches (stores twice)
        int best = -1;
        double best_score = -1.0;
        for (int a = NGH_MAX_AXES - 1; a >= 0; --a) {
            if (sp.shape[a] <= 1) continue;
            double score = 0.0;
            for (int t = 0; t < sp.n_tensors; ++t) {
                if (!used[t] || sp.tensors[t].strides[a] != 1) continue;
                double elems = 1.0;
                for (int b = 0; b < NGH_MAX_AXES; ++b)
                    if (sp.tensors[t].strides[b] != 0) elems *= (double)sp.shape[b];
                score += elems * itemsize_of(sp.tensors[t].dtype) * ((loads[t] ? 1 : 0) + (stores[t] ? 1 : 0));
            }
            if (score > best_score) { best_score = score; best = a; }
        }
        if (best < 0) best = 2;
        int perm[3], j = 0;
        for (int a = 0; a < 3; ++a) if (a != best) perm[j++] = a;
        perm[2] = best;
        fill_kargs(sp, S, perm, P.k);
        for (int a = 0; a < 3; ++a) P.perm[a] = perm[a];
        P.family = F_EW;
        P.V = vec_ok(P.k, used, 8) ? 8 : (vec_ok(P.k, used, 4) ? 4 : 1);
        P.tail = 0;
        if (P.V == 1 && P.k.shape[0] == 1 && P.k.shape[1] == 1 && P.k.shape[2] >= 16) {
            // contiguous 1-D view whose length is not a multiple of the vector width:
            // vector body + scalar tail
            const long long n = P.k.shape[2];
            for (int V : {8, 4}) {
                P.k.shape[2] = n - n % V;
                if (vec_ok(P.k, used, V)) { P.V = V; P.tail = n % V; break; }
                P.k.shape[2] = n;
            }
        }
        if (allow_ragged && P.V == 1 && P.tail == 0 && P.k.shape[0] * P.k.shape[1] > 1 && ragged_rows_ok(P.k, used)) {
            P.V = 4;
            P.k.ragged = 1;
        }
        bool plain_stores = true;     // a truncating store writes memory directly, never through a tile
        for (int pc = S.op_begin; pc < S.op_end; ++pc) plain_stores = plain_stores && sp.ops[pc].opcode != NGH_OP_STORE_TRUNC;
        if (P.V == 1 && P.tail == 0 && plain_stores && !(ctx && ctx->no_tiles)) {
            // Operands of mixed contiguity: if enough of the traffic is contiguous along a
            // second axis (transposed views), stage those operands through LDS tiles.
            double total = 0.0, along[NGH_MAX_AXES] = {0.0, 0.0, 0.0};
            for (int t = 0; t < sp.n_tensors; ++t) {
                if (!used[t]) continue;
                const ngh_tensor& T = sp.tensors[t];
                double elems = 1.0;
                for (int b = 0; b < NGH_MAX_AXES; ++b)
                    if (T.strides[b] != 0) elems *= (double)sp.shape[b];
                const double w = elems * itemsize_of(T.dtype) * ((loads[t] ? 1 : 0) + (stores[t] ? 1 : 0));
                total += w;
                if (T.strides[best] == 1 || T.strides[best] == 0) continue;
                for (int a = 0; a < NGH_MAX_AXES; ++a)
                    if (a != best && sp.shape[a] > 1 && T.strides[a] == 1) along[a] += w;
            }
            int second = -1;
            for (int a = 0; a < NGH_MAX_AXES; ++a)
                if (a != best && along[a] > 0.0 && (second < 0 || along[a] > along[second])) second = a;
            if (second >= 0 && along[second] >= 0.2 * total && sp.shape[second] >= 8 && sp.shape[best] >= 8) {
                int outer = 0;
                while (outer == best || outer == second) ++outer;
                const int tperm[3] = {outer, second, best};
                KArgs kt;
                fill_kargs(sp, S, tperm, kt);
                int n_staged = 0;
                for (int t = 0; t < sp.n_tensors; ++t) {
                    kt.t[t].stage_slot = -1;
                    if (used[t] && kt.t[t].s[1] == 1 && kt.t[t].s[2] != 0 && kt.t[t].s[2] != 1)
                        kt.t[t].stage_slot = n_staged++;
                }
                kt.n_staged = n_staged;
                kt.tile_diagonal = 1;
                for (int t = 0; t < sp.n_tensors; ++t) {
                    if (!used[t]) continue;
                    const long long strided = kt.t[t].stage_slot >= 0 ? kt.t[t].s[2] : kt.t[t].s[1];
                    if ((strided * itemsize_of(kt.t[t].dtype)) % 4096 != 0) kt.tile_diagonal = 0;
                }
                // small problems take 16 x 16 tiles: four times the workgroups, one element per lane
                int tile = kTile;
                if (kt.shape[0] * ((kt.shape[1] + 31) / 32) * ((kt.shape[2] + 31) / 32) < 4LL * (ctx ? ctx->cus : 256))
                    tile = 16;
                const long long ta = (kt.shape[1] + tile - 1) / tile, tb = (kt.shape[2] + tile - 1) / tile;
                const long long n_tiles = kt.shape[0] * ta * tb;
                if (n_staged > 0 && n_tiles < (1LL << 31) && tiled_lds_bytes(kt, tile) <= kInterpLdsPreferred - 1024) {
                    P.tile = tile;
                    P.k = kt;
                    for (int a = 0; a < 3; ++a) P.perm[a] = tperm[a];
                    P.family = F_EW_TILED;
                    P.tiles_a = (unsigned)ta;
                    P.tiles_b = (unsigned)tb;
                    P.n_tiles = (unsigned)n_tiles;
                    for (int t = 0; t < sp.n_tensors; ++t) {
                        if (loads[t]) P.load_mask |= 1u << t;
                        if (stores[t]) P.store_mask |= 1u << t;
                    }
                    return NGH_OK;
                }
            }
        }
        // The interpreter pays a fixed price per op whatever the width, so it takes 8 elements
        // per lane for every storage type when the register file still leaves several
        // workgroups per CU (16 per lane measured slower: the file crowds out occupancy).
        P.Vi = P.V;
        if (P.tail == 0 && P.V >= 4)
            if (P.V < 8 && vec_ok(P.k, used, 8, true) && interp_lds_bytes(P.k, 8) <= kInterpLdsWide) P.Vi = 8;
        const long long rows = P.k.shape[0] * P.k.shape[1];
        const long long cpr = (P.k.shape[2] + (P.k.ragged ? P.V - 1 : 0)) / P.V;
        if (rows * cpr >= (1LL << 32) || rows >= (1LL << 32))
            return fail(NGH_E_UNSUPPORTED, "stage has %lld chunks; split the launch", rows * cpr);
        P.chunks_per_row = (unsigned)cpr;
        P.n_chunks = (unsigned)(rows * cpr);
        return NGH_OK;
    }

    // ---- reduction stage: spec axis 0 is reduced, (1,2) index the outputs ----
    const long long R = sp.shape[0];
    bool r_contig = true, any_main = false;
    int out_contig_axis = -1;
    for (int t = 0; t < sp.n_tensors; ++t) {
        if (!loads[t]) continue;
        const ngh_tensor& T = sp.tensors[t];
        if (T.strides[0] == 0) continue;   // broadcast along the reduced axis
        any_main = true;
        if (T.strides[0] != 1) r_contig = false;
    }
    if (!any_main) r_contig = false;
    if (!r_contig) {
        for (int a = 2; a >= 1; --a) {
            if (sp.shape[a] <= 1) continue;
            bool ok = true, any = false;
            for (int t = 0; t < sp.n_tensors; ++t) {
                if (!loads[t] || sp.tensors[t].strides[0] == 0) continue;
                any = true;
                if (sp.tensors[t].strides[a] != 1) ok = false;
            }
            if (ok && any) { out_contig_axis = a; break; }
        }
    }
    const long long n_out = sp.shape[1] * sp.shape[2];
    if (n_out >= (1LL << 31) || R >= (1LL << 31)) return fail(NGH_E_UNSUPPORTED, "reduction extents exceed 2^31");
    const int target_wgs = (ctx ? ctx->cus * ctx->red_wgs_per_cu : 256 * 8);
    if (out_contig_axis >= 0) {
        const int other = (out_contig_axis == 2) ? 1 : 2;
        const int perm[3] = {0, other, out_contig_axis};
        fill_kargs(sp, S, perm, P.k);
        for (int a = 0; a < 3; ++a) P.perm[a] = perm[a];
        P.family = F_RED_COL;
        // 4 consecutive outputs per lane when every operand read allows 16-byte access
        P.V = (vec_ok(P.k, used, 4, true) && interp_lds_bytes(P.k, 4, 4) <= kInterpLdsPreferred) ? 4 : 1;
        // ... unless that leaves most of the chip without a workgroup
        if (P.V == 4 && ((P.k.shape[2] / 4 + 63) / 64) * P.k.shape[1] * std::max<long long>(1, R / 256) <
                            (ctx ? ctx->cus : 256))
            P.V = 1;
        P.n_out = (unsigned)n_out;
        const long long col_chunks = (P.k.shape[2] + P.V - 1) / P.V;
        P.tx = 1;
        while (P.tx < 64 && (long long)P.tx < col_chunks) P.tx <<= 1;
        // Column reductions run best on few, long-lived workgroups (measured with a cold cache on a
        // 268 MB matrix: one or two per compute unit reach 6.2-6.7 TB/s, eight 4.8), each walking
        // down its columns with several rows in flight.  With many columns the whole workgroup
        // lies along them: kBlock * V consecutive outputs per row step, every lane its own outputs.
        // (The interpreter is the opposite case: it hides its per-op cost behind many resident
        // wavefronts, so a stage without a compiled program keeps the large grid.)
        const bool compiled = !(ctx && ctx->force_interp) && !P.k.probe && match_special(F_RED_COL, P.V, P.k, 0) >= 0;
        const long long col_target = compiled ? (ctx ? ctx->cus * ctx->red_col_wgs_per_cu : 256 * 2) : target_wgs;
        // (... unless the last of those workgroups per row would be mostly idle lanes)
        const long long wide_blocks = (col_chunks + kBlock - 1) / kBlock;
        const bool wide = compiled && col_chunks >= kBlock && R * n_out > kSmallReduction && R >= (ctx ? ctx->wide_min_rows : 2) &&
                          col_chunks * 10 >= wide_blocks * kBlock * 9;
        if (wide) P.tx = kBlock;
        if (R * n_out <= kSmallReduction) {
            // A small problem is bound by latency: every row a lane walks down is a round trip
            // that depends on the one before.  Narrower column groups put more lanes on each
            // column (64 / TX rows per wavefront at once) while the workgroups still fit the chip.
            const long long cus = ctx ? ctx->cus : 256;
            while (P.tx > 4 && R > (long long)kWaves * (64 / P.tx) &&
                   ((col_chunks + P.tx / 2 - 1) / (P.tx / 2)) * P.k.shape[1] <= cus * 2)
                P.tx >>= 1;
        }
        P.n_bx = (unsigned)((col_chunks + P.tx - 1) / P.tx);
        const long long rows_per_pass = wide ? 1 : (long long)kWaves * (64 / P.tx);
        const long long base_wgs = (long long)P.n_bx * P.k.shape[1];
        long long seg = std::max<long long>(1, col_target / std::max<long long>(1, base_wgs));
        seg = std::min<long long>(seg, std::max<long long>(1, R / (rows_per_pass * 8)));
        seg = std::min<long long>(seg, 4096);
        // a small problem is bound by launches: a second one (the fold of the segments) costs more
        // than the parallelism the segments buy
        if (R * n_out <= kSmallReduction) seg = 1;
        P.seg_len = (unsigned)((R + seg - 1) / seg);
        P.n_seg = (unsigned)((R + P.seg_len - 1) / std::max(1u, P.seg_len));
        if (P.n_seg == 0) P.n_seg = 1;
    } else {
        const int perm[3] = {1, 2, 0};
        fill_kargs(sp, S, perm, P.k);
        for (int a = 0; a < 3; ++a) P.perm[a] = perm[a];
        P.family = F_RED_ROW;
        P.V = (r_contig && vec4_ok(P.k, used)) ? 4 : 1;
        if (allow_ragged && P.V == 1 && r_contig && ragged_rows_ok(P.k, used)) {
            P.V = 4;
            P.k.ragged = 1;
        }
        P.n_out = (unsigned)n_out;
        const long long chunks = (R + (P.k.ragged ? P.V - 1 : 0)) / P.V;
        if (chunks <= 64) {
            // short rows: TR lanes per row, several rows per workgroup, no segments
            P.small_rows = true;
            P.tx = 1;
            while ((long long)P.tx < chunks) P.tx <<= 1;
            // with rows enough to fill the chip several times over, a lane takes up to four chunks
            // of its row (all in flight at once) and a quarter of the wavefronts do the work
            const long long lanes_wanted = (ctx ? ctx->cus : 256) * 2048LL * 4;
            for (int shrink = 0; shrink < 2 && P.tx > 1 && (long long)n_out * (P.tx / 2) >= lanes_wanted; ++shrink)
                P.tx >>= 1;
            P.n_seg = 1;
            P.seg_len = (unsigned)chunks;
            return NGH_OK;
        }
        // rows of a few thousand elements, and enough of them to fill the chip that way: a
        // wavefront per row, every lane several chunks, the same butterfly -- a workgroup per
        // row would spend its time on the barrier and the launch of a workgroup per kilobyte
        const long long wave_chunks = ctx ? ctx->row_wave_chunks : kRowWaveChunks;
        const long long cus = ctx ? ctx->cus : 256;
        // (with one element per chunk the same row lengths qualify)
        if (chunks <= wave_chunks * (P.V == 1 ? 4 : 1) && (long long)n_out >= cus * 4 * kWaves) {
            P.small_rows = true;
            P.tx = 64;
            P.n_seg = 1;
            P.seg_len = (unsigned)chunks;
            return NGH_OK;
        }
        long long seg = std::max<long long>(1, target_wgs / std::max<long long>(1, n_out));
        seg = std::min<long long>(seg, std::max<long long>(1, chunks / (kBlock * 4)));
        seg = std::min<long long>(seg, 1024);
        if (R * n_out <= kSmallReduction && n_out >= 16) seg = 1;
        P.seg_len = (unsigned)((chunks + seg - 1) / seg);
        P.n_seg = (unsigned)((chunks + P.seg_len - 1) / std::max(1u, P.seg_len));
        if (P.n_seg == 0) P.n_seg = 1;
    }
    if ((long long)P.n_out * P.n_seg >= (1LL << 31)) return fail(NGH_E_UNSUPPORTED, "reduction grid too large");
    return NGH_OK;
}

// (While launches are being recorded into a graph, the context's buffers may not grow: growing
// synchronises the stream, and a recorded launch would keep the old buffer's address.)
static int no_growth_while_recording(const ngh_context* ctx, const char* what) {
    if (!ctx->capturing) return NGH_OK;
    return fail(NGH_E_INVALID, "%s would have to grow while a graph is being recorded: run the launches once "
                "before ngh_graph_begin", what);
}

int ensure_ws(ngh_context* ctx, size_t bytes) {
    if (bytes <= ctx->ws_bytes) return NGH_OK;
    NGH_TRY(no_growth_while_recording(ctx, "the workspace of split reductions"));
    if (ctx->ws) {
        HIP_TRY(hipStreamSynchronize(ctx->stream));
        HIP_TRY(hipFree(ctx->ws));
        ctx->ws = nullptr;
        ctx->ws_bytes = 0;
    }
    size_t want = std::max(bytes, (size_t)4 << 20);
    HIP_TRY(hipMalloc(&ctx->ws, want));
    ctx->ws_bytes = want;
    return NGH_OK;
}

// Arrival counters for kernels whose last workgroup finishes the job.  They are zero whenever
// no such kernel is running: allocated zeroed, and each kernel resets what it used.
// ---------------------------------------------------------------------------
// Deferred flex statistics: host side.  A record is "unsettled" while its current contents
// live in the shadow page or a fold of group words is outstanding; anything but the next
// deferred launch writing it needs it settled (one small kernel) first.
// ---------------------------------------------------------------------------
FlexTable* flex_table_of(ngh_context* ctx, const void* p, int32_t* id) {
    for (auto& T : ctx->flex_tables) {
        const char* b = (const char*)T.base;
        if ((const char*)p >= b && (const char*)p < b + (size_t)T.n * sizeof(ngh_flex_state)) {
            *id = (int32_t)(((const char*)p - b) / sizeof(ngh_flex_state));
            return &T;
        }
    }
    return nullptr;
}

int flex_settle_flush(ngh_context* ctx, FlexSettleArgs& a) {
    if (a.n == 0) return NGH_OK;
    hipLaunchKernelGGL(flex_settle_kernel, dim3((unsigned)a.n), dim3(64), 0, ctx->stream, a);
    HIP_TRY(hipGetLastError());
    a.n = 0;
    return NGH_OK;
}

// queue record `id` of T for settling (flushes when the batch is full)
int flex_settle_add(ngh_context* ctx, FlexTable& T, int32_t id, FlexSettleArgs& a) {
    FlexRecordHost& R = T.rec[(size_t)id];
    if (!R.unsettled()) return NGH_OK;
    for (int i = 0; i < a.n; ++i)
        if (a.slot[i].out == T.base + id) return NGH_OK;
    FlexLazySlot& sl = a.slot[a.n++];
    memset(&sl, 0, sizeof(sl));
    sl.in = T.page(id, R.page);
    sl.out = T.base + id;
    sl.words_in = R.pending ? T.set(id, R.seq) : nullptr;
    sl.tag_in = R.seq;
    sl.count_in = R.count;
    R.page = 0;
    R.pending = 0;
    ctx->flex_unsettled -= 1;
    if (a.n == kFlexMaxIds) return flex_settle_flush(ctx, a);
    return NGH_OK;
}

int flex_settle_range(ngh_context* ctx, const ngh_flex_state* dev, int32_t first, int32_t n) {
    if (ctx->flex_unsettled == 0) return NGH_OK;
    FlexSettleArgs a;
    a.n = 0;
    for (auto& T : ctx->flex_tables) {
        if (T.base != dev) continue;
        const int32_t end = std::min<int64_t>((int64_t)first + n, T.n);
        for (int32_t id = std::max(first, 0); id < end; ++id) NGH_TRY(flex_settle_add(ctx, T, id, a));
    }
    return flex_settle_flush(ctx, a);
}

int flex_settle_ids(ngh_context* ctx, const ngh_flex_state* dev, const int32_t* ids, int32_t n_ids) {
    if (ctx->flex_unsettled == 0) return NGH_OK;
    FlexSettleArgs a;
    a.n = 0;
    for (auto& T : ctx->flex_tables) {
        if (T.base != dev) continue;
        for (int i = 0; i < n_ids; ++i)
            if (ids[i] >= 0 && ids[i] < T.n) NGH_TRY(flex_settle_add(ctx, T, ids[i], a));
    }
    return flex_settle_flush(ctx, a);
}

// settle every record a spec's operands point into (scale or statistics word); with
// `writer` set, operands that carry one of that launch's statistics slots are left alone
// (the launch works on those records itself)
int flex_settle_spec(ngh_context* ctx, const ngh_fused_spec& sp, const KArgs* writer = nullptr) {
    if (ctx->flex_unsettled == 0) return NGH_OK;
    FlexSettleArgs a;
    a.n = 0;
    for (int t = 0; t < sp.n_tensors; ++t) {
        if (writer && writer->t[t].stat_slot >= 0) continue;
        const void* ptrs[2] = {sp.tensors[t].dev_scale, sp.tensors[t].dev_stats};
        for (const void* p : ptrs) {
            if (!p) continue;
            int32_t id = 0;
            FlexTable* T = flex_table_of(ctx, p, &id);
            if (T) NGH_TRY(flex_settle_add(ctx, *T, id, a));
        }
    }
    return flex_settle_flush(ctx, a);
}

int ensure_tickets(ngh_context* ctx, size_t n) {
    if (n <= ctx->n_tickets) return NGH_OK;
    NGH_TRY(no_growth_while_recording(ctx, "the arrival counters"));
    if (ctx->tickets) {
        HIP_TRY(hipStreamSynchronize(ctx->stream));
        HIP_TRY(hipFree(ctx->tickets));
        ctx->tickets = nullptr;
        ctx->n_tickets = 0;
    }
    const size_t want = std::max(n, (size_t)4096);
    HIP_TRY(hipMalloc((void**)&ctx->tickets, want * sizeof(unsigned)));
    HIP_TRY(hipMemsetAsync(ctx->tickets, 0, want * sizeof(unsigned), ctx->stream));
    ctx->n_tickets = want;
    return NGH_OK;
}

// The last (length % 4) elements of a contiguous 1-D stage, one element per lane.
// Point the stage's statistics slots at per-workgroup scratch for a launch of `blocks`
// workgroups, and, after the launch, fold the scratch into each tensor's statistics word.
int ensure_stat_ws(ngh_context* ctx, unsigned blocks) {
    if (blocks > ctx->stat_ws_blocks) {
        NGH_TRY(no_growth_while_recording(ctx, "the per-workgroup statistics buffer"));
        if (ctx->stat_ws) {
            HIP_TRY(hipStreamSynchronize(ctx->stream));
            HIP_TRY(hipFree(ctx->stat_ws));
            ctx->stat_ws = nullptr;
        }
        const unsigned cap = std::max(blocks, 65536u);
        HIP_TRY(hipMalloc((void**)&ctx->stat_ws, (size_t)cap * 4 * sizeof(int)));
        ctx->stat_ws_blocks = cap;
    }
    return NGH_OK;
}

int stat_scratch(ngh_context* ctx, KArgs& k, unsigned blocks) {
    if (k.n_stat_slots == 0) return NGH_OK;
    NGH_TRY(ensure_stat_ws(ctx, blocks));
    for (int s = 0; s < 4; ++s) k.stat_partial[s] = ctx->stat_ws + (size_t)s * ctx->stat_ws_blocks;
    return NGH_OK;
}

int stat_fold(ngh_context* ctx, const KArgs& k, unsigned blocks, int first = 0, int last = 4) {
    for (int s = first; s < k.n_stat_slots && s < last; ++s) {
        if (k.stat_ptr[s] == nullptr) continue;
        hipLaunchKernelGGL(stats_fold_kernel, dim3(1), dim3(256), 0, ctx->stream, k.stat_partial[s], blocks,
                           k.stat_ptr[s]);
        HIP_TRY(hipGetLastError());
    }
    return NGH_OK;
}

int launch_tail(ngh_context* ctx, const Plan& P) {
    // The same view as the body's, all of it, entered at element `body`: operand pointers stay
    // where they are, so index values, random-number counters and the table of a lookup (whose
    // stride on this axis is the table's own) see the coordinates of the whole view.
    KArgs kt = P.k;
    const long long body = P.k.shape[2];
    kt.shape[2] = body + P.tail;
    if (kt.shape[2] > 0xffffffffLL) return fail(NGH_E_UNSUPPORTED, "1-D stage of %lld elements with a scalar tail", kt.shape[2]);
    const size_t lds = interp_lds_bytes(kt, 1);
    if (lds > kInterpLdsMax) return fail(NGH_E_UNSUPPORTED, "program needs %zu bytes of LDS registers", lds);
    NGH_TRY(stat_scratch(ctx, kt, 1));
    hipLaunchKernelGGL(ew_gather_interp_kernel<1>, dim3(1), dim3(kBlock), lds, ctx->stream, kt,
                       (unsigned long long)P.tail, (unsigned long long)body);
    HIP_TRY(hipGetLastError());
    return stat_fold(ctx, kt, 1);
}

// Can the tiled stage move four elements per access on every operand (ew_tiled4_static_kernel)?
bool tile4_ok(const KArgs& k, unsigned used_mask) {
    if (k.shape[1] % 4 || k.shape[2] % 4) return false;
    for (int t = 0; t < k.n_tensors; ++t) {
        if (!(used_mask & (1u << t))) continue;
        const KTensor& T = k.t[t];
        if (T.stage_slot >= 0) {                       // contiguous along kernel axis 1
            if (((uintptr_t)T.p) % 16 || T.s[0] % 4 || T.s[2] % 4) return false;
        } else if (T.s[2] != 0) {                      // must be contiguous along kernel axis 2
            if (T.s[2] != 1 || ((uintptr_t)T.p) % 16 || T.s[0] % 4 || T.s[1] % 4) return false;
        }
    }
    return true;
}

// A compiled tiled stage takes 64 x 64 tiles when every operand allows 16-byte accesses and
// there are tiles of that size enough to fill the chip.
bool wants_tile4(const ngh_context* ctx, const Plan& P, long long& ta4, long long& tb4, long long& n4) {
    ta4 = (P.k.shape[1] + kTile4 - 1) / kTile4;
    tb4 = (P.k.shape[2] + kTile4 - 1) / kTile4;
    n4 = P.k.shape[0] * ta4 * tb4;
    return P.family == F_EW_TILED && P.special >= 0 && !P.k.probe && ctx->tile4 && P.tile == kTile &&
           n4 >= 4LL * ctx->cus && tile4_ok(P.k, P.load_mask | P.store_mask);
}

int launch_interp(ngh_context* ctx, Plan& P) {
    if (P.family == F_EW_TILED) {
        if (P.n_tiles == 0) return NGH_OK;
        const unsigned blocks = std::min<unsigned>(P.n_tiles, (unsigned)(ctx->cus * ctx->ew_blocks_per_cu));
        NGH_TRY(stat_scratch(ctx, P.k, blocks));
        if (P.special >= 0 && !P.k.probe) {
            // a compiled program takes 64 x 64 tiles with 16-byte accesses where every operand
            // allows them and there are tiles of that size enough to fill the chip
            long long ta4, tb4, n4;
            if (wants_tile4(ctx, P, ta4, tb4, n4)) {
                const unsigned blocks4 = (unsigned)std::min<long long>(n4, (long long)ctx->cus * ctx->ew_blocks_per_cu);
                NGH_TRY(stat_scratch(ctx, P.k, blocks4));
                HIP_TRY(launch_special_tiled(P.special, ctx->stream, blocks4, P.k, (unsigned)ta4, (unsigned)tb4,
                                             (unsigned)n4, kTile4));
                return stat_fold(ctx, P.k, blocks4);
            }
            HIP_TRY(launch_special_tiled(P.special, ctx->stream, blocks, P.k, P.tiles_a, P.tiles_b, P.n_tiles, P.tile));
            return stat_fold(ctx, P.k, blocks);
        }
        if (P.tile == 16)
            hipLaunchKernelGGL(ew_tiled_interp_kernel<16>, dim3(blocks), dim3(kBlock), tiled_lds_bytes(P.k, 16),
                               ctx->stream, P.k, P.tiles_a, P.tiles_b, P.n_tiles, P.load_mask, P.store_mask);
        else
            hipLaunchKernelGGL(ew_tiled_interp_kernel<32>, dim3(blocks), dim3(kBlock), tiled_lds_bytes(P.k, 32),
                               ctx->stream, P.k, P.tiles_a, P.tiles_b, P.n_tiles, P.load_mask, P.store_mask);
        HIP_TRY(hipGetLastError());
        return stat_fold(ctx, P.k, blocks);
    }
    if (P.k.ragged && P.special < 0) return fail(NGH_E_RUNTIME, "a stage planned for ragged rows has no compiled program");
    int V = (P.family == F_EW) ? P.Vi : P.V;
    size_t lds = interp_lds_bytes(P.k, V);
    while (lds > kInterpLdsPreferred && V > 1 && P.family == F_EW) {
        // too many live registers for a V-wide file: narrow the vector (the tail, if any, stays)
        const int narrower = (V > 4) ? V / 2 : 1;
        if (P.k.shape[0] * P.k.shape[1] * (P.k.shape[2] / narrower) >= (1LL << 32)) break;
        V = narrower;
        lds = interp_lds_bytes(P.k, V);
    }
    if (P.family == F_EW) {
        P.Vi = V;
        P.chunks_per_row = (unsigned)(P.k.shape[2] / V);
        P.n_chunks = (unsigned)(P.k.shape[0] * P.k.shape[1] * (P.k.shape[2] / V));
    }
    if (lds > kInterpLdsMax) return fail(NGH_E_UNSUPPORTED, "program needs %zu bytes of LDS registers", lds);
    KArgs& k = P.k;
    if (P.family == F_EW) {
        if (P.n_chunks == 0 && P.tail == 0) return NGH_OK;
        if (P.n_chunks && V == 1) {
            const int G = gather_width(k);
            const unsigned long long total = P.n_chunks;
            unsigned blocks = (unsigned)((total + (unsigned long long)kBlock * G - 1) / ((unsigned long long)kBlock * G));
            blocks = std::min<unsigned>(blocks, (unsigned)(ctx->cus * ctx->ew_blocks_per_cu));
            NGH_TRY(stat_scratch(ctx, k, blocks));
            if (G == 4)
                hipLaunchKernelGGL(ew_gather_interp_kernel<4>, dim3(blocks), dim3(kBlock), interp_lds_bytes(k, 4), ctx->stream, k, total, 0ull);
            else
                hipLaunchKernelGGL(ew_gather_interp_kernel<1>, dim3(blocks), dim3(kBlock), lds, ctx->stream, k, total, 0ull);
            HIP_TRY(hipGetLastError());
            NGH_TRY(stat_fold(ctx, k, blocks));
        } else if (P.n_chunks) {
            unsigned blocks = (P.n_chunks + kBlock - 1) / kBlock;
            blocks = std::min<unsigned>(blocks, (unsigned)(ctx->cus * ctx->ew_blocks_per_cu));
            NGH_TRY(stat_scratch(ctx, k, blocks));
            if (V == 8)
                hipLaunchKernelGGL(ew_interp_kernel<8>, dim3(blocks), dim3(kBlock), lds, ctx->stream, k, P.n_chunks, P.chunks_per_row);
            else
                hipLaunchKernelGGL(ew_interp_kernel<4>, dim3(blocks), dim3(kBlock), lds, ctx->stream, k, P.n_chunks, P.chunks_per_row);
            HIP_TRY(hipGetLastError());
            NGH_TRY(stat_fold(ctx, k, blocks));
        }
        if (P.tail) NGH_TRY(launch_tail(ctx, P));
        return NGH_OK;
    }
    if (P.n_out == 0) return NGH_OK;
    RedWs ws{nullptr, nullptr};
    if (P.n_seg > 1) {
        const size_t n = (size_t)k.n_red * P.n_seg * P.n_out;
        NGH_TRY(ensure_ws(ctx, n * 8));
        ws.val = (float*)ctx->ws;
        ws.idx = (int*)ctx->ws + n;
    }
    // the merge kernel of a split reduction: few outputs with many segments each take a wavefront
    // per output (with 256 segments or more also a thousand or two outputs: 64 of them a
    // workgroup would be a handful of workgroups walking a long chain of round trips); else 64
    // outputs a workgroup.  It emits the results, so the statistics of flex results come from
    // its workgroups (the partial arrays hold the larger of the two grids).
    // A handful of outputs with 256 segments or more each take a workgroup per output.
    const bool finish_by_block = P.n_seg >= 256 && P.n_out <= 64;
    const bool finish_by_wave = !finish_by_block && P.n_seg >= 32 && (P.n_out < 1024 || P.n_seg >= 256);
    // Else 64 outputs a workgroup, or 32 or 16 while that leaves compute units without a workgroup
    // and every group of lanes more than one batch of segments.
    unsigned finish_outs = 64;
    while (finish_outs > 16 && (P.n_out + finish_outs - 1) / finish_outs < (unsigned)ctx->cus &&
           P.n_seg / (kBlock / finish_outs) > 8)
        finish_outs >>= 1;
    const unsigned finish_blocks = P.n_seg <= 1 ? 0 : finish_by_block ? P.n_out
                                 : finish_by_wave ? (P.n_out + kWaves - 1) / kWaves
                                                  : (P.n_out + finish_outs - 1) / finish_outs;
    unsigned red_blocks = 0;
    if (P.special >= 0 && !k.probe) {
        // a pre-built reduction: same grid and workspace as the interpreter's kernel
        const bool small = P.family == F_RED_ROW && P.small_rows;
        const unsigned rows_per_wg = small ? kBlock / P.tx : 1;
        red_blocks = small ? (P.n_out + rows_per_wg - 1) / rows_per_wg
                   : P.family == F_RED_ROW ? P.n_out * P.n_seg
                                           : (unsigned)((unsigned long long)P.n_bx * (unsigned)k.shape[1] * P.n_seg);
        NGH_TRY(stat_scratch(ctx, k, std::max(red_blocks, finish_blocks)));
        // (a row reduction takes no TX unless its rows are short: TX lanes per row then)
        HIP_TRY(launch_special_red(P.special, ctx->stream, red_blocks, k, P.family == F_RED_ROW ? P.n_out : P.n_bx,
                                   P.n_seg, P.seg_len, P.family == F_RED_ROW && !small ? 0u : P.tx, ws, P.cache_policy));
    } else if (P.family == F_RED_ROW && P.small_rows) {
        const unsigned rows_per_wg = kBlock / P.tx;
        red_blocks = (P.n_out + rows_per_wg - 1) / rows_per_wg;
        NGH_TRY(stat_scratch(ctx, k, std::max(red_blocks, finish_blocks)));
        if (V == 4)
            hipLaunchKernelGGL(red_rows_small_interp_kernel<4>, dim3(red_blocks), dim3(kBlock), lds, ctx->stream, k, P.n_out, P.tx);
        else
            hipLaunchKernelGGL(red_rows_small_interp_kernel<1>, dim3(red_blocks), dim3(kBlock), lds, ctx->stream, k, P.n_out, P.tx);
    } else if (P.family == F_RED_ROW) {
        const unsigned blocks = red_blocks = P.n_out * P.n_seg;
        NGH_TRY(stat_scratch(ctx, k, std::max(blocks, finish_blocks)));
        if (V == 4)
            hipLaunchKernelGGL(red_row_interp_kernel<4>, dim3(blocks), dim3(kBlock), lds, ctx->stream, k, P.n_out, P.n_seg, P.seg_len, ws);
        else
            hipLaunchKernelGGL(red_row_interp_kernel<1>, dim3(blocks), dim3(kBlock), lds, ctx->stream, k, P.n_out, P.n_seg, P.seg_len, ws);
    } else {
        const unsigned long long blocks = (unsigned long long)P.n_bx * (unsigned)k.shape[1] * P.n_seg;
        if (blocks >= (1ULL << 31)) return fail(NGH_E_UNSUPPORTED, "reduction grid too large");
        red_blocks = (unsigned)blocks;
        NGH_TRY(stat_scratch(ctx, k, std::max(red_blocks, finish_blocks)));
        if (V == 4)
            hipLaunchKernelGGL(red_col_interp_kernel<4>, dim3(red_blocks), dim3(kBlock), interp_lds_bytes(k, 4, 4), ctx->stream, k, P.n_bx, P.n_seg, P.seg_len, P.tx, ws);
        else
            hipLaunchKernelGGL(red_col_interp_kernel<1>, dim3(red_blocks), dim3(kBlock), lds, ctx->stream, k, P.n_bx, P.n_seg, P.seg_len, P.tx, ws);
    }
    HIP_TRY(hipGetLastError());
    if (k.n_stat_slots) NGH_TRY(stat_fold(ctx, k, red_blocks, 0, P.n_seg > 1 ? k.n_store_stat_slots : 4));
    if (P.n_seg > 1) {
        if (finish_by_block)
            hipLaunchKernelGGL(red_finish_block_kernel, dim3(finish_blocks), dim3(kBlock), 0, ctx->stream,
                               k, P.n_out, P.n_seg, P.family == F_RED_ROW ? 1 : 0, ws);
        else if (finish_by_wave)
            hipLaunchKernelGGL(red_finish_wave_kernel, dim3(finish_blocks), dim3(kBlock), 0, ctx->stream,
                               k, P.n_out, P.n_seg, P.family == F_RED_ROW ? 1 : 0, ws);
        else
            hipLaunchKernelGGL(red_finish_kernel, dim3(finish_blocks), dim3(kBlock), 0, ctx->stream,
                               k, P.n_out, P.n_seg, P.family == F_RED_ROW ? 1 : 0, ws, finish_outs);
        HIP_TRY(hipGetLastError());
        if (k.n_stat_slots > k.n_store_stat_slots) NGH_TRY(stat_fold(ctx, k, finish_blocks, k.n_store_stat_slots, 4));
    }
    return NGH_OK;
}

void describe(const Plan& P, char* out, size_t n) {
    if (P.special >= 0) {
        snprintf(out, n, "special:%s", special_name(P.special));
        return;
    }
    switch (P.family) {
        case F_EW:
            if (P.Vi == 1) snprintf(out, n, "ew_gather_interp_g%d", gather_width(P.k));
            else snprintf(out, n, "ew_interp_v%d%s", P.Vi, P.tail ? "+tail" : "");
            break;
        case F_RED_ROW:
            if (P.small_rows) snprintf(out, n, "red_rows_small_interp_v%d_l%u", P.V, P.tx);
            else snprintf(out, n, "red_row_interp_v%d_s%u", P.V, P.n_seg);
            break;
        case F_RED_COL: snprintf(out, n, "red_col_interp_v%d_t%u_s%u", P.V, P.tx, P.n_seg); break;
        case F_EW_TILED: snprintf(out, n, "ew_tiled_interp_t%d_s%d", P.tile, P.k.n_staged); break;
    }
}

}  // namespace

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
extern "C" {

int ngh_abi_version(void) { return NGH_ABI_VERSION; }

const char* ngh_last_error(void) { return g_err; }

int ngh_device_count(int* count) {
    if (!count) return fail(NGH_E_INVALID, "count is NULL");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) { *count = 0; return fail(NGH_E_NODEVICE, "hipGetDeviceCount: %s", hipGetErrorString(e)); }
    *count = n;
    return NGH_OK;
}

int ngh_init(int device_id, ngh_context** out_ctx) {
    if (!out_ctx) return fail(NGH_E_INVALID, "out_ctx is NULL");
    *out_ctx = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return fail(NGH_E_NODEVICE, "no HIP device visible");
    if (device_id < 0 || device_id >= n) return fail(NGH_E_INVALID, "device %d not in 0..%d", device_id, n - 1);
    HIP_TRY(hipSetDevice(device_id));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device_id));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0 && !env_int("NGH_ALLOW_ANY_ARCH", 0))
        return fail(NGH_E_NODEVICE, "device %d is %s; this library is built for gfx950 only", device_id, prop.gcnArchName);
    if (device_id >= kMaxDevices) return fail(NGH_E_UNSUPPORTED, "device %d: at most %d devices", device_id, kMaxDevices);
    if (!g_scratch_of_device[device_id]) {
        void* p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(NGH_E_RUNTIME, "hipGetSymbolAddress returned no address for the scratch array");
        g_scratch_of_device[device_id] = p;
    }
    ngh_context* ctx = new ngh_context();
    ctx->noalloc_scratch = g_scratch_of_device[device_id];
    ctx->device = device_id;
    ctx->cus = prop.multiProcessorCount;
    ctx->total_bytes = prop.totalGlobalMem;
    snprintf(ctx->name, sizeof(ctx->name), "%s (%s)", prop.name, prop.gcnArchName);
    ctx->ew_blocks_per_cu = std::max(1, env_int("NGH_EW_BLOCKS_PER_CU", 64));
    ctx->force_interp = env_int("NGH_FORCE_INTERP", 0);
    ctx->flex_self_managed = env_int("NGH_FLEX_SELF_MANAGED", 2);
    ctx->flex_lazy_blocks_per_cu = env_int("NGH_FLEX_LAZY_BLOCKS_PER_CU", 6);
    if (ctx->flex_lazy_blocks_per_cu == 0) ctx->flex_lazy_blocks_per_cu = 1;
    ctx->no_tiles = env_int("NGH_NO_TILES", 0);
    ctx->no_ragged = env_int("NGH_NO_RAGGED", 0);
    ctx->no_chain = env_int("NGH_NO_CHAIN", 0);
    ctx->no_pairs = env_int("NGH_NO_PAIRS", 0);
    ctx->wide_min_rows = std::max(1, env_int("NGH_WIDE_MIN_ROWS", 2));
    ctx->red_wgs_per_cu = std::max(1, env_int("NGH_RED_WGS_PER_CU", 8));
    ctx->red_col_wgs_per_cu = std::max(1, env_int("NGH_RED_COL_WGS_PER_CU", 2));
    ctx->col_chain_wgs_per_cu = std::max(1, env_int("NGH_COL_CHAIN_WGS_PER_CU", 2));
    ctx->chain_wgs_per_cu = std::max(0, env_int("NGH_CHAIN_WGS_PER_CU", 0));
    ctx->row_wave_chunks = std::max(0, env_int("NGH_ROW_WAVE_CHUNKS", kRowWaveChunks));
    ctx->tile4 = env_int("NGH_TILE4", 1);
    ctx->cache_policy = env_int("NGH_CACHE_POLICY", -1);
    ctx->stream_bytes = (long long)env_int("NGH_STREAM_MIB", 192) << 20;
    ctx->moments_wgs_per_cu = std::max(1, env_int("NGH_MOMENTS_WGS_PER_CU", 8));
    ctx->copy_threads = std::max(0, std::min(64, env_int("NGH_COPY_THREADS", 8)));
    ctx->staging_slot_bytes = (size_t)std::max(1, env_int("NGH_STAGING_SLOT_MIB", 16)) << 20;
    ctx->ordered_arrival = env_int("NGH_ORDERED_ARRIVAL", 2);
    if (ctx->ordered_arrival < 0 || ctx->ordered_arrival > 2) ctx->ordered_arrival = 2;
    // the relaxed variant leans on what gfx950 does; on anything else it never runs
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0 && ctx->ordered_arrival == 0) ctx->ordered_arrival = 1;
    hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev0);
    if (e == hipSuccess) e = hipEventCreate(&ctx->ev1);
    if (e != hipSuccess) {
        delete ctx;
        return fail(NGH_E_RUNTIME, "stream/event creation: %s", hipGetErrorString(e));
    }
    // the interpreter's register file is dynamic LDS and may exceed the 64 KiB default
    const void* interp_kernels[] = {(const void*)ew_interp_kernel<8>, (const void*)ew_interp_kernel<4>,
                                    (const void*)ew_gather_interp_kernel<4>, (const void*)ew_gather_interp_kernel<1>,
                                    (const void*)red_row_interp_kernel<4>, (const void*)red_row_interp_kernel<1>,
                                    (const void*)red_col_interp_kernel<4>, (const void*)red_col_interp_kernel<1>,
                                    (const void*)red_rows_small_interp_kernel<4>, (const void*)red_rows_small_interp_kernel<1>,
                                    (const void*)ew_tiled_interp_kernel<16>,
                                    (const void*)ew_tiled_interp_kernel<32>};
    for (const void* fn : interp_kernels) {
        e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kInterpLdsMax);
        if (e != hipSuccess) {
            ngh_shutdown(ctx);
            return fail(NGH_E_RUNTIME, "hipFuncSetAttribute(max dynamic LDS): %s", hipGetErrorString(e));
        }
    }
    *out_ctx = ctx;
    return NGH_OK;
}

int ngh_shutdown(ngh_context* ctx) {
    if (!ctx) return NGH_OK;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    ctx->staging.release();
    if (ctx->io_tmp) (void)hipFree(ctx->io_tmp);
    if (ctx->ws) (void)hipFree(ctx->ws);
    if (ctx->stat_ws) (void)hipFree(ctx->stat_ws);
    if (ctx->tickets) (void)hipFree(ctx->tickets);
    for (auto& T : ctx->flex_tables) {
        if (T.shadow) (void)hipFree(T.shadow);
        if (T.words) (void)hipFree(T.words);
    }
    if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
    if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
    if (ctx->fork_ev) (void)hipEventDestroy(ctx->fork_ev);
    if (ctx->join_ev) (void)hipEventDestroy(ctx->join_ev);
    if (ctx->side_stream) (void)hipStreamDestroy(ctx->side_stream);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return NGH_OK;
}

int ngh_sync(ngh_context* ctx) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return NGH_OK;
}

int ngh_device_info(ngh_context* ctx, char* name256, int* compute_units, uint64_t* total_bytes) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    if (name256) { strncpy(name256, ctx->name, 255); name256[255] = 0; }
    if (compute_units) *compute_units = ctx->cus;
    if (total_bytes) *total_bytes = ctx->total_bytes;
    return NGH_OK;
}

int ngh_malloc(ngh_context* ctx, size_t bytes, void** out_dev) {
    if (!ctx || !out_dev) return fail(NGH_E_INVALID, "ngh_malloc: NULL argument");
    *out_dev = nullptr;
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipMalloc(out_dev, std::max<size_t>(bytes, 16)));
    return NGH_OK;
}

int ngh_free(ngh_context* ctx, void* dev) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    if (!dev) return NGH_OK;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    for (size_t i = 0; i < ctx->flex_tables.size(); ++i) {
        FlexTable& T = ctx->flex_tables[i];
        if ((void*)T.base != dev) continue;
        for (const auto& r : T.rec) ctx->flex_unsettled -= r.unsettled() ? 1 : 0;
        if (T.shadow) (void)hipFree(T.shadow);
        if (T.words) (void)hipFree(T.words);
        ctx->flex_tables.erase(ctx->flex_tables.begin() + i);
        break;
    }
    HIP_TRY(hipFree(dev));
    return NGH_OK;
}

// Large copies go through the context's pinned ring (ngh_hostio.h); small ones, and all of them
// with NGH_COPY_THREADS=0, are left to the runtime.
static bool staged(ngh_context* ctx, size_t bytes) {
    if (ctx->copy_threads <= 0 || bytes < ctx->staged_min_bytes) return false;
    if (ctx->staging.ensure(ctx->staging_slot_bytes, ctx->copy_threads) != hipSuccess) {
        (void)hipGetLastError();
        ctx->copy_threads = 0;          // no pinned memory to be had: never try again
        return false;
    }
    return true;
}

int ngh_memcpy_h2d(ngh_context* ctx, void* dev, const void* host, size_t bytes) {
    if (!ctx || (bytes && (!dev || !host))) return fail(NGH_E_INVALID, "ngh_memcpy_h2d: NULL argument");
    if (!bytes) return NGH_OK;
    if (staged(ctx, bytes)) {
        HIP_TRY(ctx->staging.to_device(dev, host, bytes, ctx->stream));
        return NGH_OK;
    }
    HIP_TRY(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return NGH_OK;
}

int ngh_memcpy_d2h(ngh_context* ctx, void* host, const void* dev, size_t bytes) {
    if (!ctx || (bytes && (!dev || !host))) return fail(NGH_E_INVALID, "ngh_memcpy_d2h: NULL argument");
    if (!bytes) return NGH_OK;
    if (staged(ctx, bytes)) {
        HIP_TRY(ctx->staging.to_host(host, dev, bytes, ctx->stream));
        return NGH_OK;
    }
    HIP_TRY(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return NGH_OK;
}

int ngh_io_scratch(ngh_context* ctx, size_t bytes, void** out_dev) {
    if (!ctx || !out_dev) return fail(NGH_E_INVALID, "ngh_io_scratch: NULL argument");
    if (bytes > ctx->io_tmp_bytes) {
        HIP_TRY(hipSetDevice(ctx->device));
        HIP_TRY(hipStreamSynchronize(ctx->stream));      // nothing may still be using the old one
        if (ctx->io_tmp) (void)hipFree(ctx->io_tmp);
        ctx->io_tmp = nullptr;
        ctx->io_tmp_bytes = 0;
        const size_t want = std::max<size_t>(bytes + bytes / 4, 1u << 20);
        HIP_TRY(hipMalloc(&ctx->io_tmp, want));
        ctx->io_tmp_bytes = want;
    }
    *out_dev = ctx->io_tmp;
    return NGH_OK;
}

int ngh_memcpy_d2d(ngh_context* ctx, void* dev_dst, const void* dev_src, size_t bytes) {
    if (!ctx || (bytes && (!dev_dst || !dev_src))) return fail(NGH_E_INVALID, "ngh_memcpy_d2d: NULL argument");
    if (!bytes) return NGH_OK;
    HIP_TRY(hipMemcpyAsync(dev_dst, dev_src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return NGH_OK;
}

int ngh_memset32(ngh_context* ctx, void* dev, uint32_t value, size_t count) {
    if (!ctx || (count && !dev)) return fail(NGH_E_INVALID, "ngh_memset32: NULL argument");
    if (!count) return NGH_OK;
    const unsigned blocks = (unsigned)std::min<size_t>((count + kBlock - 1) / kBlock, (size_t)ctx->cus * 16);
    hipLaunchKernelGGL(fill_kernel<uint32_t>, dim3(blocks), dim3(kBlock), 0, ctx->stream, (uint32_t*)dev, value, count);
    HIP_TRY(hipGetLastError());
    return NGH_OK;
}

int ngh_memset16(ngh_context* ctx, void* dev, uint16_t value, size_t count) {
    if (!ctx || (count && !dev)) return fail(NGH_E_INVALID, "ngh_memset16: NULL argument");
    if (!count) return NGH_OK;
    const unsigned blocks = (unsigned)std::min<size_t>((count + kBlock - 1) / kBlock, (size_t)ctx->cus * 16);
    hipLaunchKernelGGL(fill_kernel<uint16_t>, dim3(blocks), dim3(kBlock), 0, ctx->stream, (uint16_t*)dev, value, count);
    HIP_TRY(hipGetLastError());
    return NGH_OK;
}

int ngh_copy_strided(ngh_context* ctx, void* dev_dst, const void* dev_src, int32_t rank,
                     const int64_t* shape, const int64_t* dst_strides, const int64_t* src_strides,
                     int32_t itemsize) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    if (rank < 0 || rank > kCopyMaxRank) return fail(NGH_E_INVALID, "rank %d not in 0..%d", rank, kCopyMaxRank);
    if (itemsize != 1 && itemsize != 2 && itemsize != 4)
        return fail(NGH_E_INVALID, "itemsize %d (1, 2 or 4)", itemsize);
    if (rank && (!shape || !dst_strides || !src_strides)) return fail(NGH_E_INVALID, "NULL shape/strides");
    CopyArgs a;
    memset(&a, 0, sizeof(a));
    long long total = 1;
    bool empty = false;
    for (int i = 0; i < rank; ++i) {
        if (shape[i] < 0) return fail(NGH_E_INVALID, "negative shape");
        empty = empty || shape[i] == 0;
    }
    if (empty) return NGH_OK;
    // drop length-1 axes, merge axes that are contiguous in both views
    int r = 0;
    for (int i = 0; i < rank; ++i) {
        if (shape[i] >= (1LL << 31) || total > (1LL << 31) / shape[i])
            return fail(NGH_E_UNSUPPORTED, "copy of more than 2^31 elements; split it");
        total *= shape[i];
        if (shape[i] == 1) continue;
        if (r > 0 && a.ds[r - 1] == dst_strides[i] * shape[i] && a.ss[r - 1] == src_strides[i] * shape[i]) {
            a.shape[r - 1] *= shape[i];
            a.ds[r - 1] = dst_strides[i];
            a.ss[r - 1] = src_strides[i];
        } else {
            a.shape[r] = shape[i]; a.ds[r] = dst_strides[i]; a.ss[r] = src_strides[i];
            ++r;
        }
    }
    if (!dev_dst || !dev_src) return fail(NGH_E_INVALID, "NULL device pointer");
    // 32-bit element counters with grid-stride steps: stay well inside the range
    if (total >= (1LL << 31)) return fail(NGH_E_UNSUPPORTED, "copy of %lld elements; split it", total);
    a.rank = r;
    a.total = (unsigned)total;
    return launch_copy(ctx->stream, ctx->cus, dev_dst, dev_src, a, itemsize) == hipSuccess
               ? NGH_OK
               : fail(NGH_E_RUNTIME, "copy launch: %s", hipGetErrorString(hipGetLastError()));
}

int ngh_validate_fused(const ngh_fused_spec* spec) { return validate(spec); }

// Cache policy of a streaming stage (bit 0 non-temporal loads, bit 1 non-temporal stores).
// The hints only matter once the operands no longer fit the last-level cache (256 MiB on
// MI355X): below `stream_bytes` everything is left cacheable.  Above it, loads stream when
// every full-size operand read is marked as read by this kernel only, and stores stream
// when every operand written is marked as not read again soon.
// Bytes of the operands a stage touches (every operand once).
static long long stage_bytes(const ngh_fused_spec& sp, const ngh_stage& S) {
    bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS];
    stage_tensors(sp, S, loads, stores);
    long long bytes = 0;
    for (int t = 0; t < sp.n_tensors; ++t) {
        if (!loads[t] && !stores[t]) continue;
        long long n = 1;
        for (int a = 0; a < sp.rank; ++a)
            if (sp.tensors[t].strides[a] != 0) n *= sp.shape[a];
        bytes += n * itemsize_of(sp.tensors[t].dtype);
    }
    return bytes;
}

static int stage_cache_policy(const ngh_context* ctx, const ngh_fused_spec& sp, const ngh_stage& S) {
    if (ctx->cache_policy >= 0) return ctx->cache_policy & 3;
    bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS];
    stage_tensors(sp, S, loads, stores);
    long long bytes = 0;
    bool any_load = false, all_load = true, any_store = false, all_store = true;
    for (int t = 0; t < sp.n_tensors; ++t) {
        if (!loads[t] && !stores[t]) continue;
        long long n = 1;
        bool full = true;
        for (int a = 0; a < sp.rank; ++a) {
            if (sp.tensors[t].strides[a] != 0) n *= sp.shape[a];
            else if (sp.shape[a] > 1) full = false;
        }
        bytes += n * itemsize_of(sp.tensors[t].dtype);
        if (loads[t] && full) {
            any_load = true;
            all_load = all_load && (sp.tensors[t].cache_hint & NGH_CACHE_STREAM_LOAD);
        }
        if (stores[t]) {
            any_store = true;
            all_store = all_store && (sp.tensors[t].cache_hint & NGH_CACHE_STREAM_STORE);
        }
    }
    if (bytes < ctx->stream_bytes) return 0;
    return ((any_load && all_load) ? 1 : 0) | ((any_store && all_store) ? 2 : 0);
}

// ---------------------------------------------------------------------------
// Row chains: every stage of a spec in one kernel (row_chain_static_kernel).  Possible when the
// spec's rows -- spec axis 0, the axis its reduction stages reduce -- are short enough for a group
// of lanes of one wavefront each, and every stage can run over ragged rows (operands with unit
// stride along the row -- fp32, or flex16 / fp16 whose every chunk of four lies on a 4-byte
// boundary -- or broadcast along it).
// ---------------------------------------------------------------------------
constexpr int kChainManagedWgsPerCu = 8;    // grid of a chain launch that runs the exponent policy itself

struct ChainPlan {
    int      n = 0;                       // stages (the spec's non-empty ones)
    int      stage_of[NGH_MAX_STAGES];
    int      families[NGH_MAX_STAGES];
    KArgs    k[NGH_MAX_STAGES];
    unsigned n_out = 0, TR = 64;
    int      special = -1;
    KArgs    launch;                      // what the chain's kernel is launched with (row chains)
};

// Do the byte ranges two operands span in the spec's iteration space intersect?
static bool tensors_overlap(const ngh_fused_spec& sp, const ngh_tensor& A, const ngh_tensor& B) {
    auto range = [&](const ngh_tensor& T, unsigned long long& lo, unsigned long long& hi) {
        long long below = 0, above = 0;
        for (int a = 0; a < sp.rank; ++a) {
            const long long reach = (long long)T.strides[a] * (long long)(sp.shape[a] > 0 ? sp.shape[a] - 1 : 0);
            (reach < 0 ? below : above) += reach;
        }
        const long long item = itemsize_of(T.dtype);
        lo = (unsigned long long)T.dev + (unsigned long long)(below * item);
        hi = (unsigned long long)T.dev + (unsigned long long)((above + 1) * item);
    };
    unsigned long long alo, ahi, blo, bhi;
    range(A, alo, ahi);
    range(B, blo, bhi);
    return alo < bhi && blo < ahi;
}

// Could the spec run as a row chain (whether or not a compiled chain exists)?
bool plan_row_chain(const ngh_context* ctx, const ngh_fused_spec& sp, ChainPlan& C) {
    if (sp.flags & NGH_SPEC_PROBE) return false;
    const long long wave_chunks = ctx ? ctx->row_wave_chunks : kRowWaveChunks;
    const long long R = sp.shape[0], n_out = sp.shape[1] * sp.shape[2];
    const long long chunks = (R + 3) / 4;
    // (a group of lanes or a wavefront per row as far as the row reductions use them, beyond
    // that a workgroup per row while a lane's kChainAhead chunks cover the row)
    if (R < 8 || wave_chunks <= 0 || chunks > (long long)kBlock * kChainAhead || n_out < 1 || n_out >= (1LL << 31))
        return false;
    bool any_red = false;
    const int perm[3] = {1, 2, 0};
    for (int s = 0; s < sp.n_stages; ++s) {
        const ngh_stage& S = sp.stages[s];
        if (S.op_end == S.op_begin) continue;
        if (C.n == NGH_MAX_STAGES) return false;
        KArgs& k = C.k[C.n];
        fill_kargs(sp, S, perm, k);
        bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS], used[NGH_MAX_TENSORS];
        stage_tensors(sp, S, loads, stores);
        for (int t = 0; t < NGH_MAX_TENSORS; ++t) used[t] = loads[t] || stores[t];
        if (k.probe || !ragged_rows_ok(k, used, true) ||
            !program_loads_hoistable(k.ops + k.op_begin, k.op_end - k.op_begin))
            return false;
        for (int r = 0; r < S.n_reductions; ++r) {
            const ngh_tensor& T = sp.tensors[S.red_out[r]];
            if (T.strides[0] != 0 || (T.dtype != NGH_F32 && T.dtype != NGH_I32 && T.dtype != NGH_U32 &&
                                      T.dtype != NGH_FLEX16 && T.dtype != NGH_F16))
                return false;
        }
        any_red = any_red || S.n_reductions > 0;
        C.stage_of[C.n] = s;
        C.families[C.n] = S.n_reductions > 0 ? 1 : 0;
        ++C.n;
    }
    if (C.n < 2 || !any_red) return false;
    // The chain keeps operands in registers from stage to stage and hands reduction results
    // over without going through memory: two operand slots over the same memory, one of them
    // written by a stage, would see each other's writes when the stages are launched one by
    // one and not inside the chain.  Such a spec runs stage by stage.
    {
        bool written[NGH_MAX_TENSORS] = {}, used[NGH_MAX_TENSORS] = {};
        for (int i = 0; i < C.n; ++i) {
            bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS];
            const ngh_stage& S = sp.stages[C.stage_of[i]];
            stage_tensors(sp, S, loads, stores);
            for (int r = 0; r < S.n_reductions; ++r) stores[S.red_out[r]] = true;
            for (int t = 0; t < sp.n_tensors; ++t) {
                written[t] = written[t] || stores[t];
                used[t] = used[t] || loads[t] || stores[t];
            }
        }
        for (int t = 0; t < sp.n_tensors; ++t) {
            if (!written[t]) continue;
            for (int u = 0; u < sp.n_tensors; ++u)
                if (u != t && used[u] && tensors_overlap(sp, sp.tensors[t], sp.tensors[u])) return false;
        }
    }
    // The kernel's arguments: the last stage's, with the statistics slots of the whole chain --
    // one per flex16 tensor that a stage stores or reduces into, in operand order (the tables of
    // a chain's compiled stages number them the same way).
    C.launch = C.k[C.n - 1];
    {
        KArgs& L = C.launch;
        L.n_stat_slots = L.n_store_stat_slots = 0;
        for (int s = 0; s < 4; ++s) L.stat_ptr[s] = nullptr;
        for (int t = 0; t < sp.n_tensors; ++t) {
            L.t[t].stat_slot = -1;
            if (sp.tensors[t].dtype != NGH_FLEX16) continue;
            bool written = false;
            for (int i = 0; i < C.n; ++i) {
                bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS];
                const ngh_stage& S = sp.stages[C.stage_of[i]];
                stage_tensors(sp, S, loads, stores);
                written = written || stores[t];
                for (int r = 0; r < S.n_reductions; ++r) written = written || S.red_out[r] == t;
            }
            if (!written) continue;
            if (L.n_stat_slots == 4) return false;
            L.t[t].stat_slot = L.n_stat_slots;
            L.stat_ptr[L.n_stat_slots++] = sp.tensors[t].dev_stats;
        }
        L.n_store_stat_slots = L.n_stat_slots;
    }
    C.n_out = (unsigned)n_out;
    C.TR = 1;
    while ((long long)C.TR < chunks && C.TR < 64) C.TR <<= 1;
    if (chunks > 64 * kChainAhead || chunks > wave_chunks) C.TR = kBlock;
    // (rows enough to fill the chip several times over: a lane takes up to four chunks of its row)
    const long long lanes_wanted = (ctx ? ctx->cus : 256) * 2048LL * 4;
    for (int shrink = 0; shrink < 2 && chunks <= 64 && C.TR > 1 && n_out * (C.TR / 2) >= lanes_wanted; ++shrink)
        C.TR >>= 1;
    return true;
}

// Could the spec run as a column chain: the reduced axis (spec axis 0) strided, every operand
// contiguous (or broadcast) along spec axis 2 in whole aligned float4s, fp32 throughout (an
// argmax may keep its position in int32)?  Fills C like plan_row_chain; C.TR is the number of
// column chunks a workgroup is wide (TX), C.n_out the column blocks per index of spec axis 1.
bool plan_col_chain(const ngh_context* ctx, const ngh_fused_spec& sp, ChainPlan& C) {
    if (sp.flags & NGH_SPEC_PROBE) return false;
    // (the columns are the spec's last axis that has an extent: kernel axis 2; the other one is kernel axis 1)
    const int ca = sp.shape[2] > 1 ? 2 : 1, oa = 3 - ca;
    const long long R = sp.shape[0], n1 = sp.shape[oa], n2 = sp.shape[ca];
    if (R < 2 || n2 < 4 || n2 % 4 || n1 < 1 || R >= (1LL << 31) || n2 >= (1LL << 31)) return false;
    bool any_red = false;
    const int perm[3] = {0, oa, ca};
    C.n = 0;
    for (int s = 0; s < sp.n_stages; ++s) {
        const ngh_stage& S = sp.stages[s];
        if (S.op_end == S.op_begin) continue;
        if (C.n == NGH_MAX_STAGES) return false;
        KArgs& k = C.k[C.n];
        fill_kargs(sp, S, perm, k);
        if (k.n_stat_slots != 0 || k.probe) return false;
        bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS];
        stage_tensors(sp, S, loads, stores);
        for (int r = 0; r < S.n_reductions; ++r) {
            const ngh_tensor& T = sp.tensors[S.red_out[r]];
            if (T.strides[0] != 0 || T.strides[ca] != 1 ||
                (T.dtype != NGH_F32 && T.dtype != NGH_I32 && T.dtype != NGH_U32)) return false;
            if ((uintptr_t)T.dev % 16 || T.strides[oa] % 4) return false;
        }
        for (int t = 0; t < sp.n_tensors; ++t) {
            if (!loads[t] && !stores[t]) continue;
            const ngh_tensor& T = sp.tensors[t];
            // (integer results of an argmax are read back as they were written: one int per column)
            const bool int_result = T.dtype == NGH_I32 || T.dtype == NGH_U32;
            if (T.dtype != NGH_F32 && !(int_result && T.strides[0] == 0 && !stores[t])) return false;
            if (T.strides[ca] == 1) {
                if ((uintptr_t)T.dev % 16 || T.strides[0] % 4 || T.strides[oa] % 4) return false;
            } else if (T.strides[ca] != 0 || stores[t]) {
                return false;
            }
        }
        for (int pc = S.op_begin; pc < S.op_end; ++pc) {
            const int opc = sp.ops[pc].opcode;
            if (opc == NGH_OP_TAKE || opc == NGH_OP_IOTA || opc == NGH_OP_RNG_UNIFORM || opc == NGH_OP_RNG_NORMAL ||
                opc == NGH_OP_STORE_TRUNC)
                return false;
        }
        any_red = any_red || S.n_reductions > 0;
        C.stage_of[C.n] = s;
        C.families[C.n] = S.n_reductions > 0 ? 2 : 0;
        ++C.n;
    }
    if (C.n < 2 || !any_red) return false;
    {
        bool written[NGH_MAX_TENSORS] = {}, used[NGH_MAX_TENSORS] = {};
        for (int i = 0; i < C.n; ++i) {
            bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS];
            const ngh_stage& S = sp.stages[C.stage_of[i]];
            stage_tensors(sp, S, loads, stores);
            for (int r = 0; r < S.n_reductions; ++r) stores[S.red_out[r]] = true;
            for (int t = 0; t < sp.n_tensors; ++t) {
                written[t] = written[t] || stores[t];
                used[t] = used[t] || loads[t] || stores[t];
            }
        }
        for (int t = 0; t < sp.n_tensors; ++t) {
            if (!written[t]) continue;
            for (int u = 0; u < sp.n_tensors; ++u)
                if (u != t && used[u] && tensors_overlap(sp, sp.tensors[t], sp.tensors[u])) return false;
        }
    }
    // Workgroup shape: as many column chunks wide as leaves every compute unit a few workgroups;
    // the lanes that are not needed along the columns split the rows.
    const long long chunks = n2 / 4;
    const long long cus = ctx ? ctx->cus : 256;
    const long long wanted = cus * (ctx ? ctx->col_chain_wgs_per_cu : 2);
    unsigned TX = kBlock;
    auto workgroups = [&](unsigned tx) { return n1 * ((chunks + tx - 1) / tx); };
    if (workgroups(TX) < wanted) TX = 64;
    // (not below 128-byte runs along the columns: 64-byte ones fetch every cache line twice,
    // 137 against 81 us for a softmax over [1000, 32768])
    while (TX > 8 && workgroups(TX) < wanted && R / (kBlock / (TX / 2)) >= 4) TX >>= 1;
    // a lane that walks at most kColCached rows keeps them in registers and the operand is read
    // once: worth narrower workgroups, down to 256-byte runs along the columns
    auto rows_per_lane = [&](unsigned tx) { return tx == kBlock ? R : (R + kBlock / tx - 1) / (kBlock / tx); };
    if (rows_per_lane(TX) > (TX == kBlock ? kColCachedWide : kColCached)) {
        for (unsigned tx = (TX == kBlock ? 64u : TX / 2); tx >= 16; tx >>= 1)
            if (rows_per_lane(tx) <= kColCached) { TX = tx; break; }
    }
    C.TR = TX;
    C.n_out = (unsigned)((chunks + TX - 1) / TX);
    if (workgroups(TX) >= (1LL << 31)) return false;
    return true;
}

// the grid of a column chain
static unsigned col_chain_blocks(const ngh_fused_spec& sp, const ChainPlan& C) {
    return (unsigned)(sp.shape[sp.shape[2] > 1 ? 1 : 2] * (long long)C.n_out);
}

int ngh_launch_fused(ngh_context* ctx, const ngh_fused_spec* spec) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    NGH_TRY(validate(spec));
    NGH_TRY(flex_settle_spec(ctx, *spec));
    if (spec->n_stages > 1 && !ctx->force_interp && !ctx->no_chain) {
        ChainPlan C;
        if (plan_col_chain(ctx, *spec, C) && (C.special = match_chain(C.k, C.families, C.n, 5)) >= 0) {
            const int cp = stage_cache_policy(ctx, *spec, spec->stages[C.stage_of[C.n - 1]]) & kCpNtStore;
            HIP_TRY(launch_special_chain(C.special, ctx->stream, col_chain_blocks(*spec, C), C.k[C.n - 1], C.n_out, C.TR, cp));
            return NGH_OK;
        }
    }
    if (spec->n_stages > 1 && !ctx->force_interp && !ctx->no_chain && !ctx->no_ragged) {
        ChainPlan C;
        if (plan_row_chain(ctx, *spec, C) && (C.special = match_chain(C.k, C.families, C.n)) >= 0) {
            const unsigned rows_per_wg = kBlock / C.TR;
            unsigned blocks = (C.n_out + rows_per_wg - 1) / rows_per_wg;
            if (ctx->chain_wgs_per_cu > 0) blocks = std::min(blocks, (unsigned)(ctx->cus * ctx->chain_wgs_per_cu));
            const int cp = stage_cache_policy(ctx, *spec, spec->stages[C.stage_of[C.n - 1]]) & kCpNtStore;
            NGH_TRY(stat_scratch(ctx, C.launch, blocks));
            HIP_TRY(launch_special_chain(C.special, ctx->stream, blocks, C.launch, C.n_out, C.TR, cp));
            return stat_fold(ctx, C.launch, blocks);
        }
    }
    for (int s = 0; s < spec->n_stages; ++s) {
        if (spec->stages[s].op_end == spec->stages[s].op_begin) continue;
        Plan P;
        NGH_TRY(plan_stage(ctx, *spec, s, P));
        if (!ctx->force_interp && !P.k.probe && P.family == F_EW) {
            P.special = match_special(P.family, P.V, P.k, P.tail);
            if (P.special >= 0) {
                const unsigned blocks = streaming_blocks(ctx->cus, ctx->ew_blocks_per_cu, P.n_chunks);
                NGH_TRY(stat_scratch(ctx, P.k, blocks));
                hipError_t e = launch_special(P.special, ctx->stream, blocks, P.k, P.n_chunks, P.chunks_per_row,
                                              stage_cache_policy(ctx, *spec, spec->stages[s]));
                if (e != hipSuccess) return fail(NGH_E_RUNTIME, "special launch: %s", hipGetErrorString(e));
                if (P.n_chunks) NGH_TRY(stat_fold(ctx, P.k, blocks));
                if (P.tail) NGH_TRY(launch_tail(ctx, P));
                continue;
            }
        }
        if (!ctx->force_interp && !P.k.probe &&
            (P.family == F_RED_COL || P.family == F_EW_TILED || P.family == F_RED_ROW)) {
            P.special = match_special(P.family, P.V, P.k, 0);
            P.cache_policy = stage_cache_policy(ctx, *spec, spec->stages[s]);
        }
        NGH_TRY(launch_interp(ctx, P));
    }
    return NGH_OK;
}

// Two specs that do not depend on each other as ONE launch, when one of them is a single tiled
// elementwise stage and the other a single unsplit reduction across the contiguous axis and the
// library has their programs built as a pair (kPairTable); `dry` only says whether.
static int try_pair_launch(ngh_context* ctx, const ngh_fused_spec& A, const ngh_fused_spec& B, bool dry, bool* done) {
    *done = false;
    if (ctx->force_interp || ctx->no_pairs || ((A.flags | B.flags) & NGH_SPEC_PROBE)) return NGH_OK;
    auto only_stage = [](const ngh_fused_spec& sp) {
        int found = -1;
        for (int s = 0; s < sp.n_stages; ++s) {
            if (sp.stages[s].op_end == sp.stages[s].op_begin) continue;
            if (found >= 0) return -1;
            found = s;
        }
        return found;
    };
    const int sa = only_stage(A), sb = only_stage(B);
    if (sa < 0 || sb < 0) return NGH_OK;
    Plan PA, PB;
    NGH_TRY(plan_stage(ctx, A, sa, PA));
    NGH_TRY(plan_stage(ctx, B, sb, PB));
    if (PA.family != F_EW_TILED || PB.family != F_RED_COL) return NGH_OK;
    PA.special = match_special(PA.family, PA.V, PA.k, 0);
    PB.special = match_special(PB.family, PB.V, PB.k, 0);
    if (PA.special < 0 || PB.special < 0 || PA.special >= kStaticCount || PB.special >= kStaticCount) return NGH_OK;
    const PairEntry* pair = nullptr;
    for (int i = 0; i < kPairCount && !pair; ++i)
        if (!strcmp(kPairTable[i].first, special_name(PA.special)) && !strcmp(kPairTable[i].second, special_name(PB.special)))
            pair = &kPairTable[i];
    long long ta4, tb4, n4;
    if (!pair || PA.tile != 16 || wants_tile4(ctx, PA, ta4, tb4, n4) || PA.n_tiles == 0 || PB.n_out == 0 || PB.n_seg != 1 ||
        PA.k.n_stat_slots != 0 || PB.k.n_stat_slots != 0)
        return NGH_OK;
    const unsigned blocks_a = std::min<unsigned>(PA.n_tiles, (unsigned)(ctx->cus * ctx->ew_blocks_per_cu));
    const unsigned long long blocks_b = (unsigned long long)PB.n_bx * (unsigned)PB.k.shape[1] * PB.n_seg;
    if (blocks_b == 0 || blocks_a + blocks_b >= (1ULL << 31)) return NGH_OK;
    *done = true;
    if (dry) return NGH_OK;
    pair->launch(ctx->stream, blocks_a, PA.k, PA.tiles_a, PA.tiles_b, PA.n_tiles, (unsigned)blocks_b, PB.k, PB.n_bx, PB.n_seg,
                 PB.seg_len, PB.tx, RedWs{nullptr, nullptr});
    HIP_TRY(hipGetLastError());
    return NGH_OK;
}

int ngh_launch_fused_pair(ngh_context* ctx, const ngh_fused_spec* a, const ngh_fused_spec* b, int32_t* out_one_launch) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    NGH_TRY(validate(a));
    NGH_TRY(validate(b));
    NGH_TRY(flex_settle_spec(ctx, *a));
    NGH_TRY(flex_settle_spec(ctx, *b));
    bool done = false;
    NGH_TRY(try_pair_launch(ctx, *a, *b, false, &done));
    if (!done) NGH_TRY(try_pair_launch(ctx, *b, *a, false, &done));
    if (out_one_launch) *out_one_launch = done ? 1 : 0;
    if (done) return NGH_OK;
    NGH_TRY(ngh_launch_fused(ctx, a));
    return ngh_launch_fused(ctx, b);
}

int ngh_describe_fused(ngh_context* ctx, const ngh_fused_spec* spec, int32_t stage, char* name128) {
    if (!ctx || !name128) return fail(NGH_E_INVALID, "NULL argument");
    NGH_TRY(validate(spec));
    if (stage < 0 || stage >= spec->n_stages) return fail(NGH_E_INVALID, "stage %d", stage);
    if (spec->n_stages > 1 && !ctx->force_interp && !ctx->no_chain) {
        ChainPlan C;
        if (plan_col_chain(ctx, *spec, C) && (C.special = match_chain(C.k, C.families, C.n, 5)) >= 0) {
            const int cp = stage_cache_policy(ctx, *spec, spec->stages[C.stage_of[C.n - 1]]) & kCpNtStore;
            snprintf(name128, 128, "special:%s/column-chain-of-%d%s", special_name(C.special), C.n, cp ? "/nt-stores" : "");
            return NGH_OK;
        }
    }
    if (spec->n_stages > 1 && !ctx->force_interp && !ctx->no_chain && !ctx->no_ragged) {
        ChainPlan C;
        if (plan_row_chain(ctx, *spec, C) && (C.special = match_chain(C.k, C.families, C.n)) >= 0) {
            const int cp = stage_cache_policy(ctx, *spec, spec->stages[C.stage_of[C.n - 1]]) & kCpNtStore;
            snprintf(name128, 128, "special:%s/chain-of-%d%s", special_name(C.special), C.n, cp ? "/nt-stores" : "");
            return NGH_OK;
        }
    }
    Plan P;
    NGH_TRY(plan_stage(ctx, *spec, stage, P));
    if (!ctx->force_interp)
        P.special = match_special(P.family, P.V, P.k, P.tail);
    describe(P, name128, 128);
    long long ta4, tb4, n4;
    if (wants_tile4(ctx, P, ta4, tb4, n4)) strncat(name128, "/tiles64", 127 - strlen(name128));
    if (P.k.ragged) strncat(name128, "/ragged", 127 - strlen(name128));
    if (P.special >= 0 && P.family == F_EW) {
        static const char* const suffix[4] = {"", "/nt-loads", "/nt-stores", "/nt-loads-stores"};
        const int cp = stage_cache_policy(ctx, *spec, spec->stages[stage]);
        strncat(name128, suffix[cp], 127 - strlen(name128));
    }
    return NGH_OK;
}

int ngh_programs_load(ngh_context* ctx, const char* path, int32_t* out_added) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    if (!path || !*path) return fail(NGH_E_INVALID, "path is NULL or empty");
    HIP_TRY(hipSetDevice(ctx->device));
    void* handle = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    if (!handle) return fail(NGH_E_INVALID, "cannot load program library %s: %s", path, dlerror());
    typedef int (*table_fn)(int, unsigned, unsigned, const void**);
    table_fn table = (table_fn)dlsym(handle, "ngh_program_library");
    if (!table) {
        dlclose(handle);
        return fail(NGH_E_INVALID, "%s exports no ngh_program_library", path);
    }
    const void* entries = nullptr;
    const int n = table(NGH_ABI_VERSION, (unsigned)sizeof(StaticEntry), (unsigned)sizeof(KArgs), &entries);
    if (n < 0 || (n > 0 && !entries)) {
        dlclose(handle);
        return fail(NGH_E_INVALID, "%s was built from other sources than this library (ABI %d, entry %zu bytes, "
                    "argument block %zu bytes)", path, NGH_ABI_VERSION, sizeof(StaticEntry), sizeof(KArgs));
    }
    // the handle is kept for the life of the process: table entries point into the library
    const int added = add_loaded_programs((const StaticEntry*)entries, n);
    if (added < 0) return fail(NGH_E_UNSUPPORTED, "the program table is full (%d loaded programs)", kMaxLoadedPrograms);
    if (out_added) *out_added = added;
    return NGH_OK;
}

int ngh_program_kernels(const ngh_program_desc* descs, int32_t n, int32_t index, char* out, size_t out_bytes) {
    if (!descs || !out || n <= 0 || index < 0 || index >= n) return fail(NGH_E_INVALID, "descs / out / index");
    for (int i = 0; i < n;) {
        if (!desc_ok(descs[i]) || i + descs[i].n_stages >= n)
            return fail(NGH_E_INVALID, "program description %d is malformed", i);
        if (i == index) {
            std::string text;
            for (const std::string& name : rtc_kernel_names(descs[i], descs + i + 1)) text += name + "\n";
            if (text.size() + 1 > out_bytes) return fail(NGH_E_INVALID, "out holds %zu bytes, %zu needed", out_bytes, text.size() + 1);
            memcpy(out, text.c_str(), text.size() + 1);
            return NGH_OK;
        }
        if (index > i && index <= i + descs[i].n_stages) return fail(NGH_E_INVALID, "description %d is a stage of chain %d", index, i);
        i += 1 + descs[i].n_stages;
    }
    return fail(NGH_E_INVALID, "index %d", index);
}

int ngh_programs_load_code(ngh_context* ctx, const void* code, size_t code_bytes, const ngh_program_desc* descs,
                           int32_t n, const char* lowered, int32_t* out_added) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    if (!code || code_bytes < 64 || !descs || n <= 0 || !lowered) return fail(NGH_E_INVALID, "code / descs / lowered");
    // the lowered names, line by line
    std::vector<std::string> lines;
    for (const char* p = lowered; *p;) {
        const char* q = strchr(p, '\n');
        if (!q) return fail(NGH_E_INVALID, "lowered: a line without its newline");
        lines.emplace_back(p, q);
        p = q + 1;
    }
    int n_top = 0;
    for (int i = 0; i < n; i += 1 + descs[i].n_stages) {
        if (!desc_ok(descs[i]) || i + descs[i].n_stages >= n)
            return fail(NGH_E_INVALID, "program description %d is malformed", i);
        if ((descs[i].family >= 4) != (descs[i].n_stages > 0)) return fail(NGH_E_INVALID, "description %d: family %d with %d stages", i, descs[i].family, descs[i].n_stages);
        for (int j = 1; j <= descs[i].n_stages; ++j)
            if (!desc_ok(descs[i + j]) || descs[i + j].n_stages != 0 || descs[i + j].family > 2)
                return fail(NGH_E_INVALID, "stage description %d is malformed", i + j);
        ++n_top;
    }
    if ((int)lines.size() != n_top * kRtcMaxKernels)
        return fail(NGH_E_INVALID, "lowered holds %zu lines, %d programs x %d slots expected", lines.size(), n_top, kRtcMaxKernels);
    HIP_TRY(hipSetDevice(ctx->device));
    hipModule_t module = nullptr;
    hipError_t me = hipModuleLoadData(&module, code);
    if (me != hipSuccess) {
        (void)hipGetLastError();
        return fail(NGH_E_INVALID, "the code object does not load on this device: %s", hipGetErrorString(me));
    }
    // Everything is resolved before anything is published: a bundle that does not fit its
    // descriptions leaves no trace.
    std::vector<RtcProgram*> owned;
    std::vector<StaticEntry> entries;
    auto refuse = [&](int code) {
        for (RtcProgram* p : owned) delete p;
        (void)hipModuleUnload(module);
        (void)hipGetLastError();          // (a failed look-up must not surface in the next launch's check)
        return code;
    };
    int top = 0;
    for (int i = 0; i < n; i += 1 + descs[i].n_stages, ++top) {
        const ngh_program_desc& d = descs[i];
        // (kept for the life of the process, like a program library: the table points into it)
        RtcProgram* r = new RtcProgram();
        owned.push_back(r);
        r->module = module;
        r->ragged_ok = desc_ragged_ok(d);
        r->stores = desc_stores(d);
        r->quad_ok = program_quad_ok(d.ops, d.n_ops);
        r->stat_slots = d.n_stat_slots > 0;
        StaticEntry e;
        rtc_fill_entry(e, *r, d);
        for (int j = 0; j < d.n_stages; ++j) {
            RtcProgram* stage = new RtcProgram();
            owned.push_back(stage);
            rtc_fill_entry(r->stages[j], *stage, descs[i + 1 + j]);
        }
        e.chain_len = d.n_stages;
        e.chain = d.n_stages ? r->stages : nullptr;
        e.rtc = r;
        const std::vector<std::string> wanted = rtc_kernel_names(d, descs + i + 1);
        for (int s = 0; s < kRtcMaxKernels; ++s) {
            const std::string& name = lines[(size_t)top * kRtcMaxKernels + s];
            if (name.empty() != wanted[s].empty())
                return refuse(fail(NGH_E_INVALID, "program %s: kernel slot %d is %s in `lowered`", d.name, s, name.empty() ? "missing" : "not expected"));
            if (name.empty()) continue;
            hipError_t fe = hipModuleGetFunction(&r->fn[s], module, name.c_str());
            if (fe != hipSuccess) return refuse(fail(NGH_E_INVALID, "program %s: no kernel %s in the code object: %s", d.name, name.c_str(), hipGetErrorString(fe)));
        }
        entries.push_back(e);
    }
    const int added = add_loaded_programs(entries.data(), (int)entries.size());
    if (added < 0) return fail(NGH_E_UNSUPPORTED, "the program table is full (%d loaded programs)", kMaxLoadedPrograms);
    if (out_added) *out_added = added;
    return NGH_OK;
}

int ngh_programs_count(int32_t* built_in, int32_t* loaded) {
    if (built_in) *built_in = kStaticCount;
    if (loaded) *loaded = loaded_programs().count.load();
    return NGH_OK;
}

namespace {
// How ngh_moments_f32 splits rows into segments: enough workgroups to fill the chip, but at
// least 4 unrolled sweeps per segment.
struct MomentsPlan {
    unsigned R4, seg_chunks, n_seg;
    bool per_wave;       // many short rows: `lanes` lanes per row, no partial sums (moments_rows_kernel)
    unsigned lanes;
};

int plan_moments(const ngh_context* ctx, const float* dev_x, int64_t rows, int64_t R, int64_t row_stride,
                 const float* dev_mean, const float* dev_var, MomentsPlan& m) {
    if (rows < 0 || R <= 0) return fail(NGH_E_INVALID, "rows %lld, R %lld", (long long)rows, (long long)R);
    if (rows == 0) return NGH_OK;
    if (!dev_x || !dev_mean || !dev_var) return fail(NGH_E_INVALID, "NULL device pointer");
    if (((uintptr_t)dev_x) % 4) return fail(NGH_E_INVALID, "x is not aligned to its element size");
    if (rows >= (1LL << 24) || R >= (1LL << 32)) return fail(NGH_E_UNSUPPORTED, "extent too large");
    m.R4 = (unsigned)(R / 4);
    m.per_wave = (long long)m.R4 <= ctx->row_wave_chunks && rows >= (long long)ctx->cus * 4 * (kMomBlock / 64);
    // a lane per chunk of the row, up to a wavefront; with rows enough to fill the chip several
    // times over, a quarter of that (each lane then has four chunks in flight)
    m.lanes = 1;
    while (m.lanes < 64 && m.lanes < m.R4) m.lanes <<= 1;
    for (int shrink = 0; shrink < 2 && m.lanes > 1 && rows * (long long)(m.lanes / 2) >= (long long)ctx->cus * 2048 * 4; ++shrink)
        m.lanes >>= 1;
    long long seg = std::max<long long>(1, (long long)ctx->cus * ctx->moments_wgs_per_cu / rows);
    seg = std::min<long long>(seg, std::max<long long>(1, m.R4 / (kMomBlock * kMomUnroll * 2)));
    seg = std::min<long long>(seg, 4096);
    m.seg_chunks = std::max(1u, (unsigned)((m.R4 + seg - 1) / seg));
    m.n_seg = std::max(1u, (unsigned)((m.R4 + m.seg_chunks - 1) / m.seg_chunks));
    return NGH_OK;
}

int launch_moments(ngh_context* ctx, const MomentsPlan& m, const float* dev_x, int64_t rows, int64_t R,
                   int64_t row_stride, float2* partial, unsigned* tickets, float* dev_mean, float* dev_var,
                   float* dev_rstd, float eps, uint32_t x_cache_hint) {
    const bool stream_x = ctx->cache_policy >= 0
                              ? (ctx->cache_policy & 1)
                              : ((x_cache_hint & NGH_CACHE_STREAM_LOAD) && rows * R * 4 >= ctx->stream_bytes);
    if (m.per_wave) {
        const unsigned rows_per_wg = kMomBlock / m.lanes;
        const dim3 row_grid((unsigned)((rows + rows_per_wg - 1) / rows_per_wg));
        if (stream_x)
            hipLaunchKernelGGL(moments_rows_kernel<true>, row_grid, dim3(kMomBlock), 0, ctx->stream, dev_x,
                               (long long)row_stride, (unsigned)R, m.R4, (unsigned)rows, m.lanes, dev_mean, dev_var,
                               dev_rstd, eps);
        else
            hipLaunchKernelGGL(moments_rows_kernel<false>, row_grid, dim3(kMomBlock), 0, ctx->stream, dev_x,
                               (long long)row_stride, (unsigned)R, m.R4, (unsigned)rows, m.lanes, dev_mean, dev_var,
                               dev_rstd, eps);
        HIP_TRY(hipGetLastError());
        return NGH_OK;
    }
    const dim3 grid((unsigned)(rows * m.n_seg));
    if (stream_x)
        hipLaunchKernelGGL(moments_kernel<true>, grid, dim3(kMomBlock), 0, ctx->stream, dev_x, (long long)row_stride,
                           (unsigned)R, m.R4, m.n_seg, m.seg_chunks, partial, tickets, dev_mean, dev_var, dev_rstd, eps,
                           ctx->ordered_arrival);
    else
        hipLaunchKernelGGL(moments_kernel<false>, grid, dim3(kMomBlock), 0, ctx->stream, dev_x, (long long)row_stride,
                           (unsigned)R, m.R4, m.n_seg, m.seg_chunks, partial, tickets, dev_mean, dev_var, dev_rstd, eps,
                           ctx->ordered_arrival);
    HIP_TRY(hipGetLastError());
    if (ctx->ordered_arrival == 2) {
        const unsigned rows_per_wg = kMomBlock / 64;
        hipLaunchKernelGGL(moments_merge_kernel, dim3((unsigned)((rows + rows_per_wg - 1) / rows_per_wg)),
                           dim3(kMomBlock), 0, ctx->stream, dev_x, (long long)row_stride, (unsigned)R, m.R4,
                           (unsigned)rows, m.n_seg, partial, dev_mean, dev_var, dev_rstd, eps);
        HIP_TRY(hipGetLastError());
    }
    return NGH_OK;
}
}  // namespace

int ngh_moments_f32(ngh_context* ctx, const float* dev_x, int64_t rows, int64_t R, int64_t row_stride,
                    float* dev_mean, float* dev_var, float* dev_rstd, float eps, uint32_t x_cache_hint) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    MomentsPlan m;
    NGH_TRY(plan_moments(ctx, dev_x, rows, R, row_stride, dev_mean, dev_var, m));
    if (rows == 0) return NGH_OK;
    if (!m.per_wave) {
        NGH_TRY(ensure_ws(ctx, (size_t)rows * m.n_seg * sizeof(float2)));
        if (ctx->ordered_arrival != 2) NGH_TRY(ensure_tickets(ctx, (size_t)rows));
    }
    return launch_moments(ctx, m, dev_x, rows, R, row_stride, (float2*)ctx->ws, ctx->tickets, dev_mean, dev_var,
                          dev_rstd, eps, x_cache_hint);
}

int ngh_moments_f32_noalloc(ngh_context* ctx, const float* dev_x, int64_t rows, int64_t R, int64_t row_stride,
                            float* dev_mean, float* dev_var, float* dev_rstd, float eps, uint32_t x_cache_hint) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    MomentsPlan m;
    NGH_TRY(plan_moments(ctx, dev_x, rows, R, row_stride, dev_mean, dev_var, m));
    if (rows == 0) return NGH_OK;
    if (m.per_wave)            // a wavefront per row: no scratch at all
        return launch_moments(ctx, m, dev_x, rows, R, row_stride, nullptr, nullptr, dev_mean, dev_var, dev_rstd, eps,
                              x_cache_hint);
    if ((size_t)rows > kNoAllocRows || (size_t)rows * m.n_seg > kNoAllocPartials)
        return fail(NGH_E_UNSUPPORTED, "ngh_moments_f32_noalloc: %lld rows in %u segments each exceed the fixed scratch "
                    "(%zu rows, %zu partial sums); use ngh_moments_f32", (long long)rows, m.n_seg, kNoAllocRows,
                    kNoAllocPartials);
    unsigned char* base = (unsigned char*)ctx->noalloc_scratch;    // the device address, never the symbol
    float2* partial = (float2*)base;
    unsigned* tickets = (unsigned*)(base + kNoAllocPartials * sizeof(unsigned long long));
    // The array keeps what the last call left: the counters of the rows must start at zero (a fill
    // kernel rather than a memset, so that the call can be captured into a graph); the partial
    // sums need no clearing, every one that is read has been written by this launch.
    // (only the one-launch hand-overs count arrivals)
    if (ctx->ordered_arrival != 2) {
        const unsigned blocks = (unsigned)((rows + kBlock - 1) / kBlock);
        hipLaunchKernelGGL(fill_kernel<uint32_t>, dim3(blocks), dim3(kBlock), 0, ctx->stream, tickets, 0u, (size_t)rows);
        HIP_TRY(hipGetLastError());
    }
    return launch_moments(ctx, m, dev_x, rows, R, row_stride, partial, tickets, dev_mean, dev_var, dev_rstd, eps,
                          x_cache_hint);
}

int ngh_convert_to_flex16(ngh_context* ctx, int16_t* dev_out, const void* dev_in, int32_t in_dtype, int64_t n,
                          float scale, const float* dev_scale, int32_t* dev_stats) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    if (n < 0) return fail(NGH_E_INVALID, "n %lld", (long long)n);
    if (in_dtype != NGH_F32 && in_dtype != NGH_F16) return fail(NGH_E_INVALID, "source dtype %d (NGH_F32 or NGH_F16)", in_dtype);
    if (n == 0) return NGH_OK;
    if (!dev_out || !dev_in) return fail(NGH_E_INVALID, "NULL device pointer");
    if (((uintptr_t)dev_out) % 2 || ((uintptr_t)dev_in) % (in_dtype == NGH_F32 ? 4 : 2))
        return fail(NGH_E_INVALID, "misaligned pointer");
    if (dev_scale) {
        int32_t id = 0;
        FlexTable* T = flex_table_of(ctx, dev_scale, &id);
        if (T) {                                  // a scale inside a record: bring the record up to date first
            FlexSettleArgs a;
            a.n = 0;
            NGH_TRY(flex_settle_add(ctx, *T, id, a));
            NGH_TRY(flex_settle_flush(ctx, a));
        }
    }
    const bool vec = ((uintptr_t)dev_out) % 16 == 0 && ((uintptr_t)dev_in) % 16 == 0;
    const unsigned long long work = vec ? (unsigned long long)n / 8 + 8 : (unsigned long long)n;
    const unsigned blocks = (unsigned)std::max<unsigned long long>(
        1, std::min<unsigned long long>((work + kCvtBlock - 1) / kCvtBlock, (unsigned long long)ctx->cus * ctx->ew_blocks_per_cu));
    NGH_TRY(ensure_stat_ws(ctx, blocks));
    int* partial = ctx->stat_ws;
#define NGH_CVT_LAUNCH(SRC, VEC)                                                                                 \
    hipLaunchKernelGGL((convert_flex16_kernel<SRC, VEC>), dim3(blocks), dim3(kCvtBlock), 0, ctx->stream, dev_out, \
                       dev_in, (unsigned long long)n, scale, dev_scale, partial)
    if (in_dtype == NGH_F32) { if (vec) NGH_CVT_LAUNCH(NGH_F32, true); else NGH_CVT_LAUNCH(NGH_F32, false); }
    else                     { if (vec) NGH_CVT_LAUNCH(NGH_F16, true); else NGH_CVT_LAUNCH(NGH_F16, false); }
#undef NGH_CVT_LAUNCH
    HIP_TRY(hipGetLastError());
    if (dev_stats) {
        hipLaunchKernelGGL(stats_fold_kernel, dim3(1), dim3(256), 0, ctx->stream, partial, blocks, dev_stats);
        HIP_TRY(hipGetLastError());
    }
    return NGH_OK;
}

int ngh_plan_fused(const ngh_fused_spec* spec, int32_t stage, int32_t* out8) {
    if (!out8) return fail(NGH_E_INVALID, "out8 is NULL");
    NGH_TRY(validate(spec));
    if (stage < 0 || stage >= spec->n_stages) return fail(NGH_E_INVALID, "stage %d", stage);
    Plan P;
    NGH_TRY(plan_stage(nullptr, *spec, stage, P));
    if (P.k.ragged && env_int("NGH_NO_RAGGED", 0)) {
        // (no context here to carry the knob: the plan a program gets compiled for follows it too)
        P = Plan();
        NGH_TRY(plan_stage_impl(nullptr, *spec, stage, P, false));
    }
    out8[0] = (int)P.family; out8[1] = P.V;
    out8[2] = P.perm[0]; out8[3] = P.perm[1]; out8[4] = P.perm[2];
    out8[5] = (int)P.tail;
    out8[6] = match_special(P.family, P.V, P.k, P.tail);
    out8[7] = (int)P.n_seg;
    return NGH_OK;
}

int ngh_plan_chain(const ngh_fused_spec* spec, int32_t* out4) {
    if (!out4) return fail(NGH_E_INVALID, "out4 is NULL");
    NGH_TRY(validate(spec));
    // (no context here: the knobs a context would carry are read from the environment, as it does)
    const bool chains = spec->n_stages > 1 && !env_int("NGH_NO_CHAIN", 0) && !env_int("NGH_FORCE_INTERP", 0);
    {
        ChainPlan C;
        if (chains && plan_col_chain(nullptr, *spec, C)) {
            out4[0] = 2;
            out4[1] = match_chain(C.k, C.families, C.n, 5);
            out4[2] = (int)C.TR;
            out4[3] = C.n;
            return NGH_OK;
        }
    }
    ChainPlan C;
    const bool ok = chains && !env_int("NGH_NO_RAGGED", 0) && env_int("NGH_ROW_WAVE_CHUNKS", kRowWaveChunks) > 0 &&
                    plan_row_chain(nullptr, *spec, C);
    out4[0] = ok ? 1 : 0;
    out4[1] = ok ? match_chain(C.k, C.families, C.n) : -1;
    out4[2] = ok ? (int)C.TR : 0;
    out4[3] = ok ? C.n : 0;
    return NGH_OK;
}

int ngh_stats_alloc(ngh_context* ctx, int32_t n, int32_t** out_dev) {
    if (!ctx || !out_dev || n <= 0) return fail(NGH_E_INVALID, "ngh_stats_alloc: bad argument");
    void* p = nullptr;
    NGH_TRY(ngh_malloc(ctx, (size_t)n * 4, &p));
    *out_dev = (int32_t*)p;
    return ngh_memset32(ctx, p, 0, (size_t)n);
}

int ngh_stats_reset(ngh_context* ctx, int32_t* dev, int32_t n) {
    if (n <= 0) return NGH_OK;
    return ngh_memset32(ctx, dev, 0, (size_t)n);
}

int ngh_stats_read(ngh_context* ctx, const int32_t* dev, int32_t n, int32_t* host) {
    if (n <= 0) return NGH_OK;
    return ngh_memcpy_d2h(ctx, host, dev, (size_t)n * 4);
}

int ngh_flex_states_alloc(ngh_context* ctx, int32_t n, ngh_flex_state** out_dev) {
    if (!ctx || !out_dev || n <= 0) return fail(NGH_E_INVALID, "ngh_flex_states_alloc: bad argument");
    NGH_TRY(no_growth_while_recording(ctx, "ngh_flex_states_alloc: the table of flex records"));
    void* p = nullptr;
    NGH_TRY(ngh_malloc(ctx, (size_t)n * sizeof(ngh_flex_state), &p));
    std::vector<ngh_flex_state> init((size_t)n);
    for (auto& s : init) {
        memset(&s, 0, sizeof(s));
        s.dec = 8;
        s.next_dec = -1;
        s.scale = 1.0f / 256.0f;
    }
    *out_dev = (ngh_flex_state*)p;
    NGH_TRY(ngh_memcpy_h2d(ctx, p, init.data(), init.size() * sizeof(ngh_flex_state)));
    // second page and group words for deferred statistics (16 KiB a record; large tables go without
    // and their launches fold at the end of the kernel instead)
    FlexTable T;
    T.base = (ngh_flex_state*)p;
    T.n = n;
    T.rec.resize((size_t)n);
    if (n <= kFlexMaxLazyRecords) {
        const size_t wbytes = (size_t)n * kFlexWordsPerRecord * sizeof(unsigned long long);
        if (hipMalloc((void**)&T.shadow, (size_t)n * sizeof(ngh_flex_state)) != hipSuccess ||
            hipMalloc((void**)&T.words, wbytes) != hipSuccess) {
            (void)hipGetLastError();
            if (T.shadow) (void)hipFree(T.shadow);
            T.shadow = nullptr;
            T.words = nullptr;
        } else {
            HIP_TRY(hipMemsetAsync(T.words, 0, wbytes, ctx->stream));
            HIP_TRY(hipMemsetAsync(T.shadow, 0, (size_t)n * sizeof(ngh_flex_state), ctx->stream));
        }
    }
    ctx->flex_tables.push_back(std::move(T));
    return NGH_OK;
}

int ngh_flex_unsettled(ngh_context* ctx, int32_t* out_count) {
    if (!ctx || !out_count) return fail(NGH_E_INVALID, "ngh_flex_unsettled: NULL argument");
    *out_count = ctx->flex_unsettled;
    return NGH_OK;
}

int ngh_flex_states_write(ngh_context* ctx, ngh_flex_state* dev, int32_t first, int32_t n,
                          const ngh_flex_state* host) {
    if (n <= 0) return NGH_OK;
    if (!dev || !host || first < 0) return fail(NGH_E_INVALID, "ngh_flex_states_write: bad argument");
    NGH_TRY(flex_settle_range(ctx, dev, first, n));      // the copy must be the last writer
    return ngh_memcpy_h2d(ctx, dev + first, host, (size_t)n * sizeof(ngh_flex_state));
}

int ngh_flex_states_read(ngh_context* ctx, const ngh_flex_state* dev, int32_t first, int32_t n,
                         ngh_flex_state* host) {
    if (n <= 0) return NGH_OK;
    if (!dev || !host || first < 0) return fail(NGH_E_INVALID, "ngh_flex_states_read: bad argument");
    NGH_TRY(flex_settle_range(ctx, dev, first, n));
    return ngh_memcpy_d2h(ctx, host, dev + first, (size_t)n * sizeof(ngh_flex_state));
}

namespace {
int make_flex_ids(const int32_t* ids, const int32_t* in_place, int32_t n_ids, FlexIds& out) {
    if (n_ids < 0 || n_ids > kFlexMaxIds) return fail(NGH_E_INVALID, "n_ids %d not in 0..%d", n_ids, kFlexMaxIds);
    if (n_ids && !ids) return fail(NGH_E_INVALID, "ids is NULL");
    memset(&out, 0, sizeof(out));
    out.n = n_ids;
    for (int i = 0; i < n_ids; ++i) {
        if (ids[i] < 0) return fail(NGH_E_INVALID, "negative flex id");
        out.id[i] = ids[i];
        out.in_place[i] = in_place ? in_place[i] : 0;
    }
    return NGH_OK;
}
// ids are record numbers counted from `dev`: when `dev` lies in a table this context allocated,
// none may point past its end (the kernels index records without a bound of their own)
int check_flex_ids(ngh_context* ctx, const ngh_flex_state* dev, const int32_t* ids, int32_t n_ids) {
    int32_t first = 0;
    const FlexTable* T = flex_table_of(ctx, dev, &first);
    if (!T) return NGH_OK;
    for (int i = 0; i < n_ids; ++i)
        if (ids[i] < 0 || (int64_t)first + ids[i] >= T->n)
            return fail(NGH_E_INVALID, "flex id %d outside the table of %d records", ids[i], T->n);
    return NGH_OK;
}
}  // namespace

int ngh_flex_prepare(ngh_context* ctx, ngh_flex_state* dev, const int32_t* ids, const int32_t* in_place,
                     int32_t n_ids) {
    if (!ctx || !dev) return fail(NGH_E_INVALID, "ngh_flex_prepare: NULL argument");
    if (n_ids == 0) return NGH_OK;
    FlexIds f;
    NGH_TRY(make_flex_ids(ids, in_place, n_ids, f));
    NGH_TRY(check_flex_ids(ctx, dev, ids, n_ids));
    NGH_TRY(flex_settle_ids(ctx, dev, ids, n_ids));
    hipLaunchKernelGGL(flex_prepare_kernel, dim3(1), dim3(64), 0, ctx->stream, dev, f);
    HIP_TRY(hipGetLastError());
    return NGH_OK;
}

int ngh_flex_update(ngh_context* ctx, ngh_flex_state* dev, const int32_t* ids, int32_t n_ids, int32_t count) {
    if (!ctx || !dev) return fail(NGH_E_INVALID, "ngh_flex_update: NULL argument");
    if (n_ids == 0) return NGH_OK;
    FlexIds f;
    NGH_TRY(make_flex_ids(ids, nullptr, n_ids, f));
    NGH_TRY(check_flex_ids(ctx, dev, ids, n_ids));
    NGH_TRY(flex_settle_ids(ctx, dev, ids, n_ids));
    hipLaunchKernelGGL(flex_update_kernel, dim3((unsigned)n_ids), dim3(64), 0, ctx->stream, dev, f, (int)count);
    HIP_TRY(hipGetLastError());
    return NGH_OK;
}

// One launch instead of prepare + kernel + fold + update: possible when the spec is a single
// stage that a pre-built streaming kernel covers whole (no scalar tail) and every
// statistics slot belongs to one of the managed tensors.
static int try_self_managed_launch(ngh_context* ctx, const ngh_fused_spec* spec, ngh_flex_state* dev,
                                   const int32_t* ids, const int32_t* in_place, int32_t n_ids, int32_t count,
                                   bool* done) {
    *done = false;
    if (ctx->force_interp || !ctx->flex_self_managed || (spec->flags & NGH_SPEC_PROBE)) return NGH_OK;
    if (spec->n_stages > 1) {
        // A row chain whose every statistics slot belongs to one of the managed tensors: each
        // workgroup takes the write exponents from the records, the one that finishes last
        // applies the policy (the end-of-kernel mode of the streaming kernels).
        if (ctx->no_chain || ctx->no_ragged) return NGH_OK;
        ChainPlan C;
        if (!plan_row_chain(ctx, *spec, C) || (C.special = match_chain(C.k, C.families, C.n)) < 0) return NGH_OK;
        KArgs& L = C.launch;
        if (L.n_stat_slots != n_ids || n_ids < 1) return NGH_OK;
        int32_t slot_id[4] = {0, 0, 0, 0};
        for (int s = 0; s < L.n_stat_slots; ++s) {
            const ptrdiff_t off = (const char*)L.stat_ptr[s] - (const char*)dev;
            if (!L.stat_ptr[s] || off < 0 || off % (ptrdiff_t)sizeof(ngh_flex_state)) return NGH_OK;
            const int32_t id = (int32_t)(off / (ptrdiff_t)sizeof(ngh_flex_state));
            int j = 0;
            while (j < n_ids && ids[j] != id) ++j;
            if (j == n_ids) return NGH_OK;
            for (int q = 0; q < s; ++q)
                if (L.flex_state[q] == dev + id) return NGH_OK;      // two slots on one tensor
            L.flex_state[s] = dev + id;
            L.flex_in_place[s] = in_place ? in_place[j] : 0;
            slot_id[s] = id;
        }
        NGH_TRY(flex_settle_spec(ctx, *spec));
        NGH_TRY(flex_settle_ids(ctx, dev, slot_id, L.n_stat_slots));
        NGH_TRY(ensure_tickets(ctx, (size_t)kFlexTicketWords + kFlexGroupMaxWords));
        L.flex_count = count;
        L.ordered_arrival = ctx->ordered_arrival == 1;
        L.tickets = ctx->tickets;
        L.group_max = (int*)(ctx->tickets + kFlexTicketWords);
        // (every workgroup pays the hand-over at the end once: as many as keep the chip full, each
        // taking several turns, not one per group of rows)
        const unsigned rows_per_wg = kBlock / C.TR;
        const unsigned blocks = std::min((C.n_out + rows_per_wg - 1) / rows_per_wg,
                                         (unsigned)(ctx->cus * (ctx->chain_wgs_per_cu > 0 ? ctx->chain_wgs_per_cu : kChainManagedWgsPerCu)));
        const int cp = stage_cache_policy(ctx, *spec, spec->stages[C.stage_of[C.n - 1]]) & kCpNtStore;
        HIP_TRY(launch_special_chain(C.special, ctx->stream, blocks, L, C.n_out, C.TR, cp));
        *done = true;
        return NGH_OK;
    }
    if (spec->stages[0].op_end == spec->stages[0].op_begin) return NGH_OK;
    Plan P;
    NGH_TRY(plan_stage(ctx, *spec, 0, P));
    P.special = match_special(P.family, P.V, P.k, P.tail);
    if (P.special < 0 || P.tail || P.n_chunks == 0 || P.k.n_stat_slots != n_ids || n_ids < 1) return NGH_OK;
    // (the one-launch kernels work on vector-wide chunks; a one-element stage is the exception)
    if (P.V < 4 && P.k.shape[0] * P.k.shape[1] * P.k.shape[2] != 1) return NGH_OK;
    for (int s = 0; s < P.k.n_stat_slots; ++s) {
        const ptrdiff_t off = (const char*)P.k.stat_ptr[s] - (const char*)dev;
        if (!P.k.stat_ptr[s] || off < 0 || off % (ptrdiff_t)sizeof(ngh_flex_state)) return NGH_OK;
        const int32_t id = (int32_t)(off / (ptrdiff_t)sizeof(ngh_flex_state));
        int j = 0;
        while (j < n_ids && ids[j] != id) ++j;
        if (j == n_ids) return NGH_OK;
        for (int q = 0; q < s; ++q)
            if (P.k.flex_state[q] == dev + id) return NGH_OK;      // two slots on one tensor
        P.k.flex_state[s] = dev + id;
        P.k.flex_in_place[s] = in_place ? in_place[j] : 0;
    }
    // records the kernel writes: slot s <-> record slot_id[s]
    int32_t slot_id[4] = {0, 0, 0, 0};
    for (int s = 0; s < P.k.n_stat_slots; ++s) slot_id[s] = (int32_t)(P.k.flex_state[s] - dev);
    FlexTable* T = nullptr;
    if (ctx->flex_self_managed >= 2) {
        int32_t id0 = 0;
        T = flex_table_of(ctx, dev, &id0);
        if (T && (T->base != dev || !T->words)) T = nullptr;
        for (int s = 0; T && s < P.k.n_stat_slots; ++s)
            if (slot_id[s] >= T->n || T->rec[(size_t)slot_id[s]].seq >= 0xfffffff0u) T = nullptr;
        // a tensor that is read and then rewritten at a new scale needs its record settled
        // before the first load: not worth deferring
        bool loads[NGH_MAX_TENSORS], stores[NGH_MAX_TENSORS];
        stage_tensors(*spec, spec->stages[0], loads, stores);
        for (int t = 0; T && t < P.k.n_tensors; ++t)
            if (P.k.t[t].stat_slot >= 0 && loads[t] && !P.k.flex_in_place[P.k.t[t].stat_slot]) T = nullptr;
        // Deferring pays while the operands fit the last-level cache: the kernel then runs on few
        // long-lived workgroups (each pays the prologue), which streams operands of that size as
        // fast as a large grid does.  Beyond it the large grid is faster by more than the policy
        // step at the end of the kernel costs (x*y+x over flex16 tensors: 16 M elements 18.8 us
        // deferred / 22.1 us not, 32 M 37.3 / 38.4, 48 M 56.8 / 52.8, 64 M 75.3 / 69.2).
        if (T && ctx->flex_self_managed == 2 && stage_bytes(*spec, spec->stages[0]) > ctx->stream_bytes) T = nullptr;
    }
    if (T) {
        // deferred statistics: everything the kernel merely reads must be in its plain form
        NGH_TRY(flex_settle_spec(ctx, *spec, &P.k));
        for (int s = 0; s < P.k.n_stat_slots; ++s) {
            const int32_t id = slot_id[s];
            FlexRecordHost& R = T->rec[(size_t)id];
            FlexLazySlot& sl = P.k.lazy[s];
            sl.in = T->page(id, R.page);
            sl.out = T->page(id, R.page ^ 1);
            sl.words_in = R.pending ? T->set(id, R.seq) : nullptr;
            sl.tag_in = R.seq;
            sl.count_in = R.count;
            sl.in_place = P.k.flex_in_place[s];
            if (!R.unsettled()) ctx->flex_unsettled += 1;
            R.seq += 1;
            R.page ^= 1;
            R.pending = 1;
            R.count = count;
            sl.tag_out = R.seq;
            sl.words_out = T->set(id, R.seq);
            P.k.flex_state[s] = nullptr;
        }
        P.k.lazy_blocks_per_cu = ctx->flex_lazy_blocks_per_cu;
        P.k.flex_lazy = ctx->cus > 0 ? ctx->cus : 1;   // also the distance between workgroups of one CU
    } else {
        NGH_TRY(flex_settle_spec(ctx, *spec));
        NGH_TRY(flex_settle_ids(ctx, dev, slot_id, P.k.n_stat_slots));
        NGH_TRY(ensure_tickets(ctx, (size_t)kFlexTicketWords + kFlexGroupMaxWords));
        P.k.flex_count = count;
        P.k.ordered_arrival = ctx->ordered_arrival == 1;
        P.k.tickets = ctx->tickets;
        P.k.group_max = (int*)(ctx->tickets + kFlexTicketWords);
    }
    const unsigned blocks = streaming_blocks(ctx->cus, ctx->ew_blocks_per_cu, P.n_chunks);
    hipError_t e = launch_special(P.special, ctx->stream, blocks, P.k, P.n_chunks, P.chunks_per_row,
                                  stage_cache_policy(ctx, *spec, spec->stages[0]));
    if (e != hipSuccess) return fail(NGH_E_RUNTIME, "special launch: %s", hipGetErrorString(e));
    *done = true;
    return NGH_OK;
}

int ngh_launch_fused_flex(ngh_context* ctx, const ngh_fused_spec* spec, ngh_flex_state* dev,
                          const int32_t* ids, const int32_t* in_place, int32_t n_ids, int32_t count) {
    if (!ctx || !dev) return fail(NGH_E_INVALID, "ngh_launch_fused_flex: NULL argument");
    NGH_TRY(validate(spec));
    if (n_ids > 0 && !ids) return fail(NGH_E_INVALID, "ngh_launch_fused_flex: ids is NULL");
    if (n_ids < 0 || n_ids > kFlexMaxIds) return fail(NGH_E_INVALID, "n_ids %d not in 0..%d", n_ids, kFlexMaxIds);
    NGH_TRY(check_flex_ids(ctx, dev, ids, n_ids));
    bool done = false;
    NGH_TRY(try_self_managed_launch(ctx, spec, dev, ids, in_place, n_ids, count, &done));
    if (done) return NGH_OK;
    NGH_TRY(ngh_flex_prepare(ctx, dev, ids, in_place, n_ids));
    NGH_TRY(ngh_launch_fused(ctx, spec));
    return ngh_flex_update(ctx, dev, ids, n_ids, count);
}

// ---------------------------------------------------------------------------
// The launches of a computation as one HIP graph: what the caller launches between
// ngh_graph_begin and ngh_graph_end is recorded, not run; ngh_graph_launch replays it with one
// call.  Two launches that do not depend on each other may be recorded side by side
// (ngh_graph_fork / ngh_graph_side / ngh_graph_join), so that the device may run them
// together: worth it for computations of a few small kernels, whose time is launches, not work.
// ---------------------------------------------------------------------------
struct ngh_graph {
    hipGraph_t     graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int            nodes = 0;
};

static int graph_join(ngh_context* ctx) {
    if (ctx->side_open) {
        HIP_TRY(hipEventRecord(ctx->join_ev, ctx->side_stream));
        HIP_TRY(hipStreamWaitEvent(ctx->main_stream, ctx->join_ev, 0));
        ctx->side_open = false;
    }
    ctx->stream = ctx->main_stream;
    return NGH_OK;
}

int ngh_graph_begin(ngh_context* ctx) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    if (ctx->capturing) return fail(NGH_E_INVALID, "ngh_graph_begin: a capture is open already");
    if (!ctx->side_stream) {
        HIP_TRY(hipStreamCreateWithFlags(&ctx->side_stream, hipStreamNonBlocking));
        HIP_TRY(hipEventCreateWithFlags(&ctx->fork_ev, hipEventDisableTiming));
        HIP_TRY(hipEventCreateWithFlags(&ctx->join_ev, hipEventDisableTiming));
    }
    HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
    ctx->main_stream = ctx->stream;
    ctx->capturing = true;
    ctx->side_open = false;
    return NGH_OK;
}

int ngh_graph_fork(ngh_context* ctx) {
    if (!ctx || !ctx->capturing) return fail(NGH_E_INVALID, "ngh_graph_fork: no capture is open");
    NGH_TRY(graph_join(ctx));
    HIP_TRY(hipEventRecord(ctx->fork_ev, ctx->main_stream));
    HIP_TRY(hipStreamWaitEvent(ctx->side_stream, ctx->fork_ev, 0));
    ctx->side_open = true;
    return NGH_OK;
}

int ngh_graph_side(ngh_context* ctx, int32_t on) {
    if (!ctx || !ctx->capturing) return fail(NGH_E_INVALID, "ngh_graph_side: no capture is open");
    if (on && !ctx->side_open) return fail(NGH_E_INVALID, "ngh_graph_side: no fork is open");
    ctx->stream = on ? ctx->side_stream : ctx->main_stream;
    return NGH_OK;
}

int ngh_graph_join(ngh_context* ctx) {
    if (!ctx || !ctx->capturing) return fail(NGH_E_INVALID, "ngh_graph_join: no capture is open");
    return graph_join(ctx);
}

int ngh_graph_end(ngh_context* ctx, ngh_graph** out) {
    if (!ctx || !ctx->capturing) return fail(NGH_E_INVALID, "ngh_graph_end: no capture is open");
    const int joined = graph_join(ctx);
    ctx->stream = ctx->main_stream;
    ctx->capturing = false;
    ctx->side_open = false;
    hipGraph_t g = nullptr;
    const hipError_t e = hipStreamEndCapture(ctx->main_stream, &g);
    if (e != hipSuccess || !g || joined != NGH_OK || !out) {
        (void)hipGetLastError();
        if (g) (void)hipGraphDestroy(g);
        if (!out && e == hipSuccess) return NGH_OK;          // (the caller gave the capture up)
        return fail(NGH_E_RUNTIME, "ngh_graph_end: %s", e != hipSuccess ? hipGetErrorString(e) : "nothing was captured");
    }
    ngh_graph* G = new ngh_graph();
    G->graph = g;
    size_t n = 0;
    if (hipGraphGetNodes(g, nullptr, &n) == hipSuccess) G->nodes = (int)n;
    const hipError_t ei = hipGraphInstantiate(&G->exec, g, nullptr, nullptr, 0);
    if (ei != hipSuccess) {
        (void)hipGetLastError();
        (void)hipGraphDestroy(g);
        delete G;
        return fail(NGH_E_RUNTIME, "hipGraphInstantiate: %s", hipGetErrorString(ei));
    }
    *out = G;
    return NGH_OK;
}

int ngh_graph_launch(ngh_context* ctx, ngh_graph* graph) {
    if (!ctx || !graph || !graph->exec) return fail(NGH_E_INVALID, "ngh_graph_launch: NULL argument");
    if (ctx->capturing) return fail(NGH_E_INVALID, "ngh_graph_launch: a capture is open");
    HIP_TRY(hipGraphLaunch(graph->exec, ctx->stream));
    return NGH_OK;
}

int ngh_graph_nodes(const ngh_graph* graph, int32_t* out_nodes) {
    if (!graph || !out_nodes) return fail(NGH_E_INVALID, "ngh_graph_nodes: NULL argument");
    *out_nodes = graph->nodes;
    return NGH_OK;
}

int ngh_graph_free(ngh_context* ctx, ngh_graph* graph) {
    if (!graph) return NGH_OK;
    if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
    return NGH_OK;
}

int ngh_timer_begin(ngh_context* ctx) {
    if (!ctx) return fail(NGH_E_INVALID, "ctx is NULL");
    HIP_TRY(hipEventRecord(ctx->ev0, ctx->stream));
    return NGH_OK;
}

int ngh_timer_end(ngh_context* ctx, float* out_ms) {
    if (!ctx || !out_ms) return fail(NGH_E_INVALID, "NULL argument");
    HIP_TRY(hipEventRecord(ctx->ev1, ctx->stream));
    HIP_TRY(hipEventSynchronize(ctx->ev1));
    HIP_TRY(hipEventElapsedTime(out_ms, ctx->ev0, ctx->ev1));
    return NGH_OK;
}

}  // extern "C"
