// The generic fused kernels: an op-program interpreter running inside three
// memory-access skeletons (streaming elementwise, reduction along the
// contiguous axis, reduction across the contiguous axis).  They execute any
// spec the host lowers a fused op group to; the hand-specialised kernels in
// ngh_special.h cover the same programs faster for the common patterns.
//
// Reference behaviour reproduced: the stage loop, broadcast loads, last-write
// stores and reduction stores of ngraph/transformers/gpu/float_ew2.py:793-984
// and :1196-1409; launch shapes are chosen for gfx950 instead of following
// float_ew2.py:394-550.
#pragma once
#include "ngh_device.h"

namespace ngh {

constexpr int kBlock = 256;          // 4 wavefronts of 64
constexpr int kWaves = kBlock / 64;

// Extra LDS rows behind the register file: per-thread max|mantissa| of each
// statistics slot, then (value, index) of each reduction slot.
__device__ __forceinline__ int ex_stat(int slot) { return slot; }
// A reduction slot owns `na` accumulators per thread: one when the lane's V elements belong
// to the same output (reduction along the vector axis), V when each is an output of its own.
__device__ __forceinline__ int ex_accv(const KArgs& k, int slot, int na = 1, int v = 0) {
    return k.n_stat_slots + 2 * (slot * na + v);
}
__device__ __forceinline__ int ex_acci(const KArgs& k, int slot, int na = 1, int v = 0) {
    return k.n_stat_slots + 2 * (slot * na + v) + 1;
}

struct Extra {
    float* base;  // &extra[thread]
    int    nthr;
    __device__ __forceinline__ int   geti(int j) const { return __float_as_int(base[j * nthr]); }
    __device__ __forceinline__ float getf(int j) const { return base[j * nthr]; }
    __device__ __forceinline__ void  seti(int j, int x) { base[j * nthr] = __int_as_float(x); }
    __device__ __forceinline__ void  setf(int j, float x) { base[j * nthr] = x; }
};

// LDS tiles of the tiled skeleton: operand `stage_slot` owns tile number stage_slot; `at` is
// this thread's element inside every tile.
constexpr int kTile = 32;                       // 16 for problems too small to fill the chip
__host__ __device__ constexpr int tile_words(int tile) { return tile * (tile + 1); }
struct Tiles {
    float* base;
    int    at;      // this lane's element 0 inside every tile
    int    vstep;   // distance of the lane's next element
    int    words;   // floats per tile
};

// ---------------------------------------------------------------------------
// Where the V elements a lane works on live.  The interpreter pays a fixed price
// per op (decode, LDS register traffic) whatever V is, so every skeleton gives
// a lane several elements per op: consecutive ones where operands allow vector
// access (VecAt), otherwise V elements a fixed number of lanes apart (GatherAt),
// which keeps each wavefront access coalesced.
// ---------------------------------------------------------------------------
template <int V>
struct VecAt {   // (i0, i1, i2 .. i2 + V - 1)
    long long i0, i1, i2;
    __device__ __forceinline__ bool valid(int) const { return true; }
    __device__ __forceinline__ float iota(int ka, int v) const {
        return (float)(ka == 2 ? i2 + v : (ka == 1 ? i1 : i0));
    }
    __device__ __forceinline__ int red_index(int rmode, int v) const { return (int)(rmode == 1 ? i2 + v : i0); }
    __device__ __forceinline__ long long coord(int ka, int v) const { return ka == 2 ? i2 + v : (ka == 1 ? i1 : i0); }
    __device__ __forceinline__ void load(const KTensor& t, float (&x)[V]) const {
        const long long off = i0 * t.s[0] + i1 * t.s[1] + i2 * t.s[2];
        const float sc = (t.dtype == NGH_FLEX16) ? tensor_scale(t) : 1.0f;
        if (t.s[2] == 0) {
            const float b = load1(t, off, sc);
#pragma unroll
            for (int v = 0; v < V; ++v) x[v] = b;
        } else if (V >= 4 && t.s[2] == 1) {
            if constexpr (V >= 4) loadv<V>(t, off, sc, x);
        } else {
#pragma unroll
            for (int v = 0; v < V; ++v) x[v] = load1(t, off + v * t.s[2], sc);
        }
    }
    __device__ __forceinline__ void store(const KTensor& t, const float (&x)[V], int& fmax) const {
        const long long off = i0 * t.s[0] + i1 * t.s[1] + i2 * t.s[2];
        const float sc = (t.dtype == NGH_FLEX16) ? 1.0f / tensor_scale(t) : 1.0f;
        if (V >= 4 && t.s[2] == 1) {
            if constexpr (V >= 4) storev<V>(t, off, sc, x, fmax);
        } else {
#pragma unroll
            for (int v = 0; v < V; ++v) store1(t, off + v * t.s[2], x[v], sc, fmax);
        }
    }
};

template <int V>
struct GatherAt {   // element v at (i0[v], i1[v], i2[v]); only the first nv count -- the others must
                    // still name an element inside the view, because loads are not predicated
                    // (a branch per element would serialise the memory round trips)
    unsigned i0[V], i1[V], i2[V];
    int nv;
    __device__ __forceinline__ bool valid(int v) const { return v < nv; }
    // Picked with masks, not with `ka == 2 ? i2[v] : ...`: the compiler turns that into one load
    // at a run-time offset into this struct, which moves the whole struct to scratch memory.
    __device__ __forceinline__ unsigned pick(int ka, int v) const {
        const unsigned m1 = 0u - (unsigned)(ka == 1), m2 = 0u - (unsigned)(ka == 2);
        return (i0[v] & ~(m1 | m2)) | (i1[v] & m1) | (i2[v] & m2);
    }
    __device__ __forceinline__ float iota(int ka, int v) const { return (float)pick(ka, v); }
    __device__ __forceinline__ int red_index(int, int) const { return 0; }   // not used with reductions
    __device__ __forceinline__ long long coord(int ka, int v) const { return pick(ka, v); }
    __device__ __forceinline__ void load(const KTensor& t, float (&x)[V]) const {
        const float sc = (t.dtype == NGH_FLEX16) ? tensor_scale(t) : 1.0f;
#pragma unroll
        for (int v = 0; v < V; ++v)
            x[v] = load1(t, (long long)i0[v] * t.s[0] + (long long)i1[v] * t.s[1] + (long long)i2[v] * t.s[2], sc);
    }
    __device__ __forceinline__ void store(const KTensor& t, const float (&x)[V], int& fmax) const {
        const float sc = (t.dtype == NGH_FLEX16) ? 1.0f / tensor_scale(t) : 1.0f;
#pragma unroll
        for (int v = 0; v < V; ++v)
            if (v < nv)
                store1(t, (long long)i0[v] * t.s[0] + (long long)i1[v] * t.s[1] + (long long)i2[v] * t.s[2], x[v], sc, fmax);
    }
};

// RMODE: 0 = no reductions, 1 = reduction runs along kernel axis 2 (the vector
// axis), 2 = reduction runs along kernel axis 0.  TILED: operands with a stage slot are
// read from / written to their LDS tile instead of memory (element v at tiles.at + v * tiles.vstep).
template <int V, int RMODE, bool TILED = false, class At>
__device__ __forceinline__ void run_ops(const KArgs& k, LdsRegs<V>& rf, Extra& ex, const At& at,
                                        Tiles tiles = Tiles{nullptr, 0, 0, 0}) {
    for (int pc = k.op_begin; pc < k.op_end; ++pc) {
        const ngh_op o = k.ops[pc];
        const int opc = o.opcode;
        switch (opc) {
            case NGH_OP_LOAD: {
                const KTensor& t = k.t[o.a];
                if constexpr (TILED) {
                    if (t.stage_slot >= 0) {
                        const float* tl = tiles.base + t.stage_slot * tiles.words + tiles.at;
#pragma unroll
                        for (int v = 0; v < V; ++v) rf.set(o.dst, v, tl[v * tiles.vstep]);
                        break;
                    }
                }
                float x[V];
                at.load(t, x);
#pragma unroll
                for (int v = 0; v < V; ++v) rf.set(o.dst, v, x[v]);
            } break;
            case NGH_OP_STORE: {
                const KTensor& t = k.t[o.dst];
                if constexpr (TILED) {
                    if (t.stage_slot >= 0 && !k.probe) {
                        float* tl = tiles.base + t.stage_slot * tiles.words + tiles.at;
#pragma unroll
                        for (int v = 0; v < V; ++v) tl[v * tiles.vstep] = rf.get(o.a, v);
                        break;
                    }
                }
                int fmax = 0;
                float x[V];
#pragma unroll
                for (int v = 0; v < V; ++v) x[v] = rf.get(o.a, v);
                if (k.probe) {
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        if (at.valid(v)) fmax = max(fmax, probe_bits(x[v]));
                } else {
                    at.store(t, x, fmax);
                }
                if (t.stat_slot >= 0) ex.seti(ex_stat(t.stat_slot), max(ex.geti(ex_stat(t.stat_slot)), fmax));
            } break;
            case NGH_OP_STORE_TRUNC: {
                const KTensor& t = k.t[o.dst];
                int fmax = 0;
                if (t.dtype == NGH_FLEX16 && !k.probe) {
                    const float sc = 1.0f / tensor_scale(t);
#pragma unroll
                    for (int v = 0; v < V; ++v)
                        if (at.valid(v)) {
                            const int q = flex_quantize_trunc(sc * rf.get(o.a, v));
                            reinterpret_cast<short*>(t.p)[at.coord(0, v) * t.s[0] + at.coord(1, v) * t.s[1] +
                                                          at.coord(2, v) * t.s[2]] = (short)q;
                            fmax = max(fmax, iabs(q));
                        }
                } else {
                    float x[V];
#pragma unroll
                    for (int v = 0; v < V; ++v) x[v] = rf.get(o.a, v);
                    if (k.probe) {
#pragma unroll
                        for (int v = 0; v < V; ++v)
                            if (at.valid(v)) fmax = max(fmax, probe_bits(x[v]));
                    } else {
                        at.store(t, x, fmax);
                    }
                }
                if (t.stat_slot >= 0) ex.seti(ex_stat(t.stat_slot), max(ex.geti(ex_stat(t.stat_slot)), fmax));
            } break;
            case NGH_OP_RNG_UNIFORM: case NGH_OP_RNG_NORMAL: {
                // shape of the spec's axes, whatever order the kernel walks them in
                const unsigned long long n1 = (unsigned long long)k.shape[k.iota_map[1]];
                const unsigned long long n2 = (unsigned long long)k.shape[k.iota_map[2]];
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    const unsigned long long lin =
                        ((unsigned long long)at.coord(k.iota_map[0], v) * n1 + (unsigned long long)at.coord(k.iota_map[1], v)) * n2 +
                        (unsigned long long)at.coord(k.iota_map[2], v);
                    const Philox4 r = philox4x32_10((unsigned)lin, (unsigned)(lin >> 32), o.a, k.rng_counter,
                                                    k.rng_seed, 0x1BD11BDAu);
                    rf.set(o.dst, v, opc == NGH_OP_RNG_UNIFORM ? rng_uniform01(r.x[0]) : rng_normal(r.x[0], r.x[1]));
                }
            } break;
            case NGH_OP_TAKE: {
                // table lookup: the coordinate along one axis comes from a register
                const KTensor& t = k.t[o.b & 15];
                const int ka = k.iota_map[o.b >> 4];
                const float sc = (t.dtype == NGH_FLEX16) ? tensor_scale(t) : 1.0f;
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    long long idx = (long long)rf.get(o.a, v);            // astype(int): truncation
                    idx = idx < 0 ? 0 : (idx >= (long long)t.take_extent ? (long long)t.take_extent - 1 : idx);
                    long long off = idx * t.s[ka];
#pragma unroll
                    for (int a = 0; a < 3; ++a)
                        if (a != ka) off += at.coord(a, v) * t.s[a];
                    rf.set(o.dst, v, load1(t, off, sc));
                }
            } break;
            case NGH_OP_CONST: {
                const float c = k.consts[o.a];
#pragma unroll
                for (int v = 0; v < V; ++v) rf.set(o.dst, v, c);
            } break;
            case NGH_OP_IOTA: {
                const int ka = k.iota_map[o.a];
#pragma unroll
                for (int v = 0; v < V; ++v) rf.set(o.dst, v, at.iota(ka, v));
            } break;
#define NGH_UN(OPC)                                                                   \
    case OPC: {                                                                       \
        _Pragma("unroll") for (int v = 0; v < V; ++v)                                 \
            rf.set(o.dst, v, op_unary(OPC, rf.get(o.a, v)));                          \
    } break;
            NGH_UN(NGH_OP_ASSIGN) NGH_UN(NGH_OP_NEG) NGH_UN(NGH_OP_ABS) NGH_UN(NGH_OP_SQRT)
            NGH_UN(NGH_OP_SQR) NGH_UN(NGH_OP_EXP) NGH_UN(NGH_OP_LOG) NGH_UN(NGH_OP_RCP)
            NGH_UN(NGH_OP_EXP2) NGH_UN(NGH_OP_LOG2) NGH_UN(NGH_OP_SIG) NGH_UN(NGH_OP_TANH)
            NGH_UN(NGH_OP_SAFELOG) NGH_UN(NGH_OP_SGN) NGH_UN(NGH_OP_SIN) NGH_UN(NGH_OP_COS)
            NGH_UN(NGH_OP_I2F) NGH_UN(NGH_OP_U2F) NGH_UN(NGH_OP_INEG) NGH_UN(NGH_OP_IABS)
#undef NGH_UN
#define NGH_BIN(OPC)                                                                  \
    case OPC: {                                                                       \
        _Pragma("unroll") for (int v = 0; v < V; ++v)                                 \
            rf.set(o.dst, v, op_binary(OPC, rf.get(o.a, v), rf.get(o.b, v)));         \
    } break;
            NGH_BIN(NGH_OP_ADD) NGH_BIN(NGH_OP_SUB) NGH_BIN(NGH_OP_MUL) NGH_BIN(NGH_OP_DIV)
            NGH_BIN(NGH_OP_INT_DIV) NGH_BIN(NGH_OP_MOD) NGH_BIN(NGH_OP_EQ) NGH_BIN(NGH_OP_NE)
            NGH_BIN(NGH_OP_LT) NGH_BIN(NGH_OP_LE) NGH_BIN(NGH_OP_GT) NGH_BIN(NGH_OP_GE)
            NGH_BIN(NGH_OP_POW) NGH_BIN(NGH_OP_MINIMUM) NGH_BIN(NGH_OP_MAXIMUM)
            NGH_BIN(NGH_OP_IADD) NGH_BIN(NGH_OP_ISUB) NGH_BIN(NGH_OP_IMUL) NGH_BIN(NGH_OP_IMIN)
            NGH_BIN(NGH_OP_IMAX) NGH_BIN(NGH_OP_UMIN) NGH_BIN(NGH_OP_UMAX) NGH_BIN(NGH_OP_IEQ)
            NGH_BIN(NGH_OP_INE) NGH_BIN(NGH_OP_ILT) NGH_BIN(NGH_OP_ILE) NGH_BIN(NGH_OP_IGT)
            NGH_BIN(NGH_OP_IGE) NGH_BIN(NGH_OP_ULT) NGH_BIN(NGH_OP_ULE) NGH_BIN(NGH_OP_UGT)
            NGH_BIN(NGH_OP_UGE)
#undef NGH_BIN
            case NGH_OP_RED_SUM: case NGH_OP_RED_PROD: case NGH_OP_RED_MAX:
            case NGH_OP_RED_MIN: case NGH_OP_RED_ARGMAX: case NGH_OP_RED_ARGMIN: {
                // the index half of an accumulator only matters to argmax / argmin
                const bool with_index = opc >= NGH_OP_RED_ARGMAX;
                if constexpr (RMODE == 1) {
                    Acc a;
                    a.v = ex.getf(ex_accv(k, o.dst));
                    a.i = with_index ? ex.geti(ex_acci(k, o.dst)) : 0;
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        Acc b;
                        b.v = rf.get(o.a, v);
                        b.i = at.red_index(RMODE, v);
                        if (at.valid(v)) a = acc_merge(opc, a, b);
                    }
                    ex.setf(ex_accv(k, o.dst), a.v);
                    if (with_index) ex.seti(ex_acci(k, o.dst), a.i);
                } else if constexpr (RMODE == 2) {
                    // the lane's V elements are V different outputs
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        Acc a, b;
                        a.v = ex.getf(ex_accv(k, o.dst, V, v));
                        a.i = with_index ? ex.geti(ex_acci(k, o.dst, V, v)) : 0;
                        b.v = rf.get(o.a, v);
                        b.i = at.red_index(RMODE, v);
                        a = acc_merge(opc, a, b);
                        ex.setf(ex_accv(k, o.dst, V, v), a.v);
                        if (with_index) ex.seti(ex_acci(k, o.dst, V, v), a.i);
                    }
                }
            } break;
            default: break;
        }
    }
}

__device__ __forceinline__ void stats_epilogue(const KArgs& k, Extra& ex) {
    __shared__ int stat_lds[4][kWaves];
    for (int s = 0; s < k.n_stat_slots; ++s) block_stat_max(ex.geti(ex_stat(s)), k.stat_partial[s], stat_lds[s]);
}

// ---------------------------------------------------------------------------
// Streaming elementwise stage.  One chunk = V consecutive elements along
// kernel axis 2; chunks are dealt to threads in order so a wavefront touches
// 64*V consecutive elements of every contiguous operand.
// ---------------------------------------------------------------------------
template <int V>
__global__ __launch_bounds__(kBlock) void ew_interp_kernel(const KArgs k, unsigned n_chunks,
                                                           unsigned chunks_per_row) {
    extern __shared__ float lds[];
    LdsRegs<V> rf{lds + threadIdx.x, kBlock};
    Extra ex{lds + (size_t)k.n_regs * V * kBlock + threadIdx.x, kBlock};
    for (int s = 0; s < k.n_stat_slots; ++s) ex.seti(ex_stat(s), 0);

    const unsigned d1 = (unsigned)k.shape[1];
    const unsigned step = gridDim.x * kBlock;
    for (unsigned q = blockIdx.x * kBlock + threadIdx.x; q < n_chunks; q += step) {
        const unsigned row = q / chunks_per_row;
        const unsigned c2 = q - row * chunks_per_row;
        const unsigned i0 = row / d1;
        const unsigned i1 = row - i0 * d1;
        run_ops<V, 0>(k, rf, ex, VecAt<V>{i0, i1, (long long)c2 * V});
    }
    stats_epilogue(k, ex);
}

// ---------------------------------------------------------------------------
// Streaming elementwise stage without vector access (operands strided along
// kernel axis 2, or lengths that are not a multiple of the vector width).
// Elements are taken in the view's linear order; a lane works on G of them,
// 256 elements apart, so each of its accesses is as coalesced as the strides
// allow and every op is decoded once for G elements.
// ---------------------------------------------------------------------------
// `first` is the linear index of the launch's first element: the tail of a 1-D stage whose body
// a vector kernel has done starts there, with every coordinate (index values, random-number
// counters, table lookups) that of the whole view.
template <int G>
__global__ __launch_bounds__(kBlock) void ew_gather_interp_kernel(const KArgs k, unsigned long long total,
                                                                  unsigned long long first) {
    extern __shared__ float lds[];
    LdsRegs<G> rf{lds + threadIdx.x, kBlock};
    Extra ex{lds + (size_t)k.n_regs * G * kBlock + threadIdx.x, kBlock};
    for (int s = 0; s < k.n_stat_slots; ++s) ex.seti(ex_stat(s), 0);
    const unsigned d1 = (unsigned)k.shape[1], d2 = (unsigned)k.shape[2];
    const unsigned long long span = (unsigned long long)kBlock * G;
    for (unsigned long long base = blockIdx.x * span; base < total; base += gridDim.x * span) {
        GatherAt<G> at;
        at.nv = 0;
#pragma unroll
        for (int v = 0; v < G; ++v) {
            unsigned long long q = base + (unsigned)v * kBlock + threadIdx.x;
            at.i0[v] = at.i1[v] = at.i2[v] = 0;
            if (q < total) {
                at.nv = v + 1;
                q += first;
                unsigned row;
                if (first + total <= 0xffffffffull) {
                    row = (unsigned)q / d2;
                    at.i2[v] = (unsigned)q - row * d2;
                } else {
                    row = (unsigned)(q / d2);
                    at.i2[v] = (unsigned)(q - (unsigned long long)row * d2);
                }
                at.i0[v] = row / d1;
                at.i1[v] = row - at.i0[v] * d1;
            }
        }
        run_ops<G, 0>(k, rf, ex, at);
    }
    stats_epilogue(k, ex);
}

// ---------------------------------------------------------------------------
// Tiled elementwise stage for operands of mixed contiguity: some contiguous
// along kernel axis 2 (the axis lanes compute along), others -- transposed
// views -- contiguous along kernel axis 1.  A workgroup owns a 32 x 32 tile of
// axes (1, 2).  Operands of the second kind are staged through LDS: read with
// lanes along axis 1 (coalesced) into a padded tile, used by the program with
// lanes along axis 2 (pitch 33: conflict-free), and results bound for such
// operands travel the same way in reverse.  Every access to memory is
// coalesced whatever the orientation of the view (the reference's kernels
// index strided views directly, float_ew2.py:987-1132).
// ---------------------------------------------------------------------------
template <int TILE>
__global__ __launch_bounds__(kBlock) void ew_tiled_interp_kernel(const KArgs k, unsigned tiles_a,
                                                                 unsigned tiles_b, unsigned n_tiles,
                                                                 unsigned load_mask, unsigned store_mask) {
    constexpr int V = TILE * TILE / kBlock;        // elements per lane: 4 (32 x 32) or 1 (16 x 16)
    constexpr int kRowStep = kBlock / TILE;        // tile rows between a lane's elements
    extern __shared__ float lds[];
    LdsRegs<V> rf{lds + threadIdx.x, kBlock};
    Extra ex{lds + (size_t)k.n_regs * V * kBlock + threadIdx.x, kBlock};
    float* tile_base = lds + (size_t)(k.n_regs * V + k.n_stat_slots) * kBlock;
    for (int s = 0; s < k.n_stat_slots; ++s) ex.seti(ex_stat(s), 0);
    const unsigned A = (unsigned)k.shape[1], B = (unsigned)k.shape[2];
    constexpr int kTile = TILE, kTilePitch = TILE + 1, kTileWords = tile_words(TILE);
    const unsigned lx = threadIdx.x & (kTile - 1), ly = threadIdx.x / kTile;
    for (unsigned tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const unsigned tb = tile % tiles_b;
        const unsigned r = tile / tiles_b;
        // With strides that are multiples of 4 KiB, tiles are dealt along diagonals (consecutive
        // workgroups differ in both tile coordinates): the tiles of one tile row then start a
        // multiple of a large power of two apart on the transposed operand, on the same few memory
        // channels, and in row-major order all resident workgroups would go through those at once.
        const unsigned ta = k.tile_diagonal ? (r % tiles_a + tb) % tiles_a : r % tiles_a;
        const unsigned i0 = r / tiles_a;
        const unsigned a0 = ta * kTile, b0 = tb * kTile;
        // stage in: lanes along axis 1
        for (int t = 0; t < k.n_tensors; ++t) {
            const KTensor& T = k.t[t];
            if (T.stage_slot < 0 || !(load_mask >> t & 1u)) continue;
            const float sc = (T.dtype == NGH_FLEX16) ? tensor_scale(T) : 1.0f;
            float* tl = tile_base + T.stage_slot * kTileWords;
            if (a0 + lx < A)
                for (unsigned y = ly; y < kTile && b0 + y < B; y += kBlock / kTile)
                    tl[y * kTilePitch + lx] =
                        load1(T, (long long)i0 * T.s[0] + (long long)(a0 + lx) * T.s[1] + (long long)(b0 + y) * T.s[2], sc);
        }
        __syncthreads();
        // compute: lanes along axis 2
        if (b0 + lx < B && a0 + ly < A) {
            GatherAt<V> at;
            at.nv = 0;
#pragma unroll
            for (int v = 0; v < V; ++v) {
                at.i0[v] = i0;
                at.i1[v] = a0 + ly + v * kRowStep;
                at.i2[v] = b0 + lx;
                if (at.i1[v] < A) at.nv = v + 1;
                else at.i1[v] = a0 + ly;
            }
            run_ops<V, 0, true>(k, rf, ex, at, Tiles{tile_base, (int)(lx * kTilePitch + ly), kRowStep, kTileWords});
        }
        __syncthreads();
        // stage out: lanes along axis 1
        if (!k.probe) {
            for (int t = 0; t < k.n_tensors; ++t) {
                const KTensor& T = k.t[t];
                if (T.stage_slot < 0 || !(store_mask >> t & 1u)) continue;
                const float sc = (T.dtype == NGH_FLEX16) ? 1.0f / tensor_scale(T) : 1.0f;
                const float* tl = tile_base + T.stage_slot * kTileWords;
                int fmax = 0;
                if (a0 + lx < A)
                    for (unsigned y = ly; y < kTile && b0 + y < B; y += kBlock / kTile)
                        store1(T, (long long)i0 * T.s[0] + (long long)(a0 + lx) * T.s[1] + (long long)(b0 + y) * T.s[2],
                               tl[y * kTilePitch + lx], sc, fmax);
                if (T.stat_slot >= 0) ex.seti(ex_stat(T.stat_slot), max(ex.geti(ex_stat(T.stat_slot)), fmax));
            }
            __syncthreads();
        }
    }
    stats_epilogue(k, ex);
}

// Partial results of a reduction split over several workgroups.
struct RedWs {
    float* val;   // [slot][segment][output]
    int*   idx;
};

// max|mantissa| of the flex results a thread has emitted, by statistics slot
struct RedStats {
    int m[4] = {0, 0, 0, 0};
    __device__ __forceinline__ void note(int slot, int v) {
#pragma unroll
        for (int s = 0; s < 4; ++s) m[s] = (s == slot) ? max(m[s], v) : m[s];
    }
};

__device__ __forceinline__ void red_emit(const KArgs& k, int slot, Acc a, long long o0, long long o1,
                                         long long o2, unsigned out, unsigned n_out, unsigned seg,
                                         unsigned n_seg, RedWs ws, RedStats& stats) {
    if (n_seg == 1) {
        const KTensor& t = k.t[k.red_out[slot]];
        const long long off = o0 * t.s[0] + o1 * t.s[1] + o2 * t.s[2];
        const float sc = (t.dtype == NGH_FLEX16) ? 1.0f / tensor_scale(t) : 1.0f;
        const int opc = k.ops[k.op_end - k.n_red + slot].opcode;
        const float result = acc_result(opc, a);
        int fmax = 0;
        if (k.probe) {
            if (t.dtype == NGH_FLEX16) fmax = probe_bits(result);
        } else if (opc >= NGH_OP_RED_ARGMAX && (t.dtype == NGH_I32 || t.dtype == NGH_U32)) {
            reinterpret_cast<int*>(t.p)[off] = a.i;       // an index into integer storage: no trip through fp32
        } else {
            store1(t, off, result, sc, fmax);
        }
        // One statistics word per tensor and a result per workgroup or lane: thousands of
        // read-modify-writes on one address would run one after the other (8192 of them took
        // 250 us).  A result with a statistics slot is merged through the workgroup's partial
        // maximum like the results of STORE ops; without one (more flex results than slots),
        // a result that does not exceed what is there already (read at device scope) adds nothing.
        if (t.stat_slot >= 0) stats.note(t.stat_slot, fmax);
        else if (t.stats != nullptr && fmax > 0 &&
                 fmax > __hip_atomic_load(t.stats, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
            atomicMax(t.stats, fmax);
    } else {
        const size_t w = ((size_t)slot * n_seg + seg) * n_out + out;
        ws.val[w] = a.v;
        if (k.ops[k.op_end - k.n_red + slot].opcode >= NGH_OP_RED_ARGMAX) ws.idx[w] = a.i;   // only argmax / argmin carry one
    }
}

// The interpreter kernels keep statistics per thread in `ex`: add what the thread emitted.
__device__ __forceinline__ void red_stats_to_extra(const KArgs& k, Extra& ex, const RedStats& stats) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
        if (s >= k.n_store_stat_slots && s < k.n_stat_slots) ex.seti(ex_stat(s), max(ex.geti(ex_stat(s)), stats.m[s]));
}

// The reduction ops of a stage are its last n_red ops, slot k = k-th of them.
__device__ __forceinline__ int red_opcode(const KArgs& k, int slot) {
    return k.ops[k.op_end - k.n_red + slot].opcode;
}

// ---------------------------------------------------------------------------
// Reduction along kernel axis 2 (the axis lanes run along): workgroup =
// (output element, segment of the reduced axis).  Per-thread accumulate ->
// wavefront butterfly -> LDS across the 4 wavefronts.
// ---------------------------------------------------------------------------
template <int V>
__global__ __launch_bounds__(kBlock) void red_row_interp_kernel(const KArgs k, unsigned n_out,
                                                                unsigned n_seg, unsigned seg_chunks,
                                                                RedWs ws) {
    extern __shared__ float lds[];
    __shared__ Acc sh[NGH_MAX_REDUCTIONS][kWaves];
    LdsRegs<V> rf{lds + threadIdx.x, kBlock};
    Extra ex{lds + (size_t)k.n_regs * V * kBlock + threadIdx.x, kBlock};
    for (int s = 0; s < k.n_stat_slots; ++s) ex.seti(ex_stat(s), 0);
    for (int s = 0; s < k.n_red; ++s) {
        Acc a = acc_init(red_opcode(k, s));
        ex.setf(ex_accv(k, s), a.v);
        ex.seti(ex_acci(k, s), a.i);
    }
    const unsigned out = blockIdx.x / n_seg;
    const unsigned seg = blockIdx.x - out * n_seg;
    const unsigned d1 = (unsigned)k.shape[1];
    const unsigned i0 = out / d1;
    const unsigned i1 = out - i0 * d1;
    const unsigned total_chunks = (unsigned)(k.shape[2] / V);
    const unsigned c_begin = seg * seg_chunks;
    const unsigned c_end = min(total_chunks, c_begin + seg_chunks);
    for (unsigned c = c_begin + threadIdx.x; c < c_end; c += kBlock)
        run_ops<V, 1>(k, rf, ex, VecAt<V>{i0, i1, (long long)c * V});

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int s = 0; s < k.n_red; ++s) {
        const int opc = red_opcode(k, s);
        Acc a;
        a.v = ex.getf(ex_accv(k, s));
        a.i = ex.geti(ex_acci(k, s));
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) a = acc_merge(opc, a, acc_shfl_xor(a, m));
        if (lane == 0) sh[s][wave] = a;
    }
    __syncthreads();
    RedStats emitted;
    if (threadIdx.x == 0) {
        for (int s = 0; s < k.n_red; ++s) {
            const int opc = red_opcode(k, s);
            Acc a = sh[s][0];
            for (int w = 1; w < kWaves; ++w) a = acc_merge(opc, a, sh[s][w]);
            red_emit(k, s, a, i0, i1, 0, out, n_out, seg, n_seg, ws, emitted);
        }
    }
    red_stats_to_extra(k, ex, emitted);
    stats_epilogue(k, ex);
}

// ---------------------------------------------------------------------------
// Reduction along kernel axis 0 with outputs contiguous along kernel axis 2.
// Lanes run along axis 2 (V consecutive outputs each) so loads stay
// coalesced while every lane walks down axis 0.  A wavefront spans TX column
// chunks x 64/TX rows: with few outputs (TX < 64) the spare lanes take more
// rows instead of idling, and a butterfly over the row lanes folds them.
// The four wavefronts then meet in LDS.
// ---------------------------------------------------------------------------
template <int V>
__global__ __launch_bounds__(kBlock) void red_col_interp_kernel(const KArgs k, unsigned n_bx, unsigned n_seg,
                                                                unsigned seg_rows, unsigned TX, RedWs ws) {
    extern __shared__ float lds[];
    __shared__ Acc sh[kWaves][64][V];
    LdsRegs<V> rf{lds + threadIdx.x, kBlock};
    Extra ex{lds + (size_t)k.n_regs * V * kBlock + threadIdx.x, kBlock};
    for (int s = 0; s < k.n_stat_slots; ++s) ex.seti(ex_stat(s), 0);
    for (int s = 0; s < k.n_red; ++s) {
        const Acc a = acc_init(red_opcode(k, s));
#pragma unroll
        for (int v = 0; v < V; ++v) {
            ex.setf(ex_accv(k, s, V, v), a.v);
            ex.seti(ex_acci(k, s, V, v), a.i);
        }
    }
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // TX == kBlock: the whole workgroup lies along the columns (kBlock * V consecutive outputs per
    // row step: the longest contiguous runs this layout allows) and every lane owns its outputs
    const bool wide = TX == kBlock;
    const unsigned tx = wide ? threadIdx.x : (lane & (TX - 1)), ry = wide ? 0 : lane / TX;
    const unsigned rows_per_wave = wide ? 1 : 64 / TX;
    unsigned b = blockIdx.x;
    const unsigned seg = b % n_seg;  b /= n_seg;
    const unsigned bx = b % n_bx;    b /= n_bx;
    const unsigned i1 = b;
    const unsigned d2 = (unsigned)k.shape[2];
    const unsigned i2 = (bx * TX + tx) * V;
    const unsigned r_begin = seg * seg_rows;
    const unsigned r_end = min((unsigned)k.shape[0], r_begin + seg_rows);
    const unsigned n_out = (unsigned)k.shape[1] * d2;
    RedStats emitted;
    if (wide) {
        if (i2 < d2) {
            for (unsigned r = r_begin; r < r_end; ++r) run_ops<V, 2>(k, rf, ex, VecAt<V>{r, i1, i2});
            for (int s = 0; s < k.n_red; ++s) {
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    Acc a;
                    a.v = ex.getf(ex_accv(k, s, V, v));
                    a.i = ex.geti(ex_acci(k, s, V, v));
                    red_emit(k, s, a, 0, i1, i2 + v, i1 * d2 + i2 + v, n_out, seg, n_seg, ws, emitted);
                }
            }
        }
        red_stats_to_extra(k, ex, emitted);
        stats_epilogue(k, ex);
        return;
    }
    if (i2 < d2)
        for (unsigned r = r_begin + wave * rows_per_wave + ry; r < r_end; r += kWaves * rows_per_wave)
            run_ops<V, 2>(k, rf, ex, VecAt<V>{r, i1, i2});

    for (int s = 0; s < k.n_red; ++s) {
        const int opc = red_opcode(k, s);
#pragma unroll
        for (int v = 0; v < V; ++v) {
            Acc a;
            a.v = ex.getf(ex_accv(k, s, V, v));
            a.i = ex.geti(ex_acci(k, s, V, v));
            for (unsigned m = 32; m >= TX; m >>= 1) a = acc_merge(opc, a, acc_shfl_xor(a, (int)m));
            if (lane < TX) sh[wave][lane][v] = a;
        }
        __syncthreads();
        if (wave == 0 && lane < TX && i2 < d2) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                Acc a = sh[0][lane][v];
                for (int w = 1; w < kWaves; ++w) a = acc_merge(opc, a, sh[w][lane][v]);
                red_emit(k, s, a, 0, i1, i2 + v, i1 * d2 + i2 + v, n_out, seg, n_seg, ws, emitted);
            }
        }
        __syncthreads();
    }
    red_stats_to_extra(k, ex, emitted);
    stats_epilogue(k, ex);
}

// ---------------------------------------------------------------------------
// Reduction along kernel axis 2 for short rows: a row takes TR lanes (a power of
// two, at most a wavefront; a lane takes every TR-th chunk of V), a workgroup
// 256 / TR rows, and a butterfly inside the TR lanes finishes the row -- no LDS,
// no barrier, no idle wavefronts where one workgroup per row would leave most of
// its 256 threads without work.
// ---------------------------------------------------------------------------
template <int V>
__global__ __launch_bounds__(kBlock) void red_rows_small_interp_kernel(const KArgs k, unsigned n_out, unsigned TR) {
    extern __shared__ float lds[];
    LdsRegs<V> rf{lds + threadIdx.x, kBlock};
    Extra ex{lds + (size_t)k.n_regs * V * kBlock + threadIdx.x, kBlock};
    for (int s = 0; s < k.n_stat_slots; ++s) ex.seti(ex_stat(s), 0);
    for (int s = 0; s < k.n_red; ++s) {
        const Acc a = acc_init(red_opcode(k, s));
        ex.setf(ex_accv(k, s), a.v);
        ex.seti(ex_acci(k, s), a.i);
    }
    const unsigned pos = threadIdx.x & (TR - 1);
    const unsigned out = blockIdx.x * (kBlock / TR) + threadIdx.x / TR;
    const unsigned d1 = (unsigned)k.shape[1];
    const unsigned i0 = out / d1, i1 = out - i0 * d1;
    const unsigned chunks = (unsigned)(k.shape[2] / V);
    if (out < n_out)
        for (unsigned c = pos; c < chunks; c += TR) run_ops<V, 1>(k, rf, ex, VecAt<V>{i0, i1, (long long)c * V});
    RedWs none{nullptr, nullptr};
    RedStats emitted;
    for (int s = 0; s < k.n_red; ++s) {
        const int opc = red_opcode(k, s);
        Acc a;
        a.v = ex.getf(ex_accv(k, s));
        a.i = ex.geti(ex_acci(k, s));
        for (unsigned m = TR >> 1; m > 0; m >>= 1) a = acc_merge(opc, a, acc_shfl_xor(a, (int)m));
        if (pos == 0 && out < n_out) red_emit(k, s, a, i0, i1, 0, out, n_out, 0, 1, none, emitted);
    }
    red_stats_to_extra(k, ex, emitted);
    stats_epilogue(k, ex);
}

// The merge kernels of split reductions: the workgroup's maximum of what it emitted goes to the
// slot's per-workgroup partial (whole workgroup calls).
__device__ __forceinline__ void red_stats_flush(const KArgs& k, const RedStats& stats) {
    __shared__ int flush_lds[4][kWaves];
#pragma unroll
    for (int s = 0; s < 4; ++s)
        if (s >= k.n_store_stat_slots && s < k.n_stat_slots) block_stat_max(stats.m[s], k.stat_partial[s], flush_lds[s]);
}

// Second pass of a split reduction: merges an output's segments (in a fixed order) and
// stores through the output's storage type.  `row_mode` tells how an output number maps to
// kernel coordinates.  With few segments a thread takes an output; with many, a wavefront
// does: lanes stride over the segments and a butterfly folds them; a handful of outputs with
// hundreds of segments each take a workgroup per output.
__device__ __forceinline__ void red_finish_coords(const KArgs& k, unsigned out, int row_mode, long long& o0,
                                                  long long& o1, long long& o2) {
    if (row_mode) {
        const unsigned d1 = (unsigned)k.shape[1];
        o0 = out / d1; o1 = out - (unsigned)o0 * d1; o2 = 0;
    } else {
        const unsigned d2 = (unsigned)k.shape[2];
        o0 = 0; o1 = out / d2; o2 = out - (unsigned)o1 * d2;
    }
}

// A workgroup takes `outs` outputs (64, 32 or 16: partial results of consecutive outputs are
// consecutive in the workspace) and its 256 / outs groups of lanes an equal share of the segments
// each, in segment order; the shares meet in shared memory and are merged in group order.  Fewer
// outputs a workgroup are more workgroups with shorter chains of round trips, which is what a
// merge of a few thousand outputs consists of.
__global__ __launch_bounds__(kBlock) void red_finish_kernel(const KArgs k, unsigned n_out, unsigned n_seg,
                                                            int row_mode, RedWs ws, unsigned outs) {
    __shared__ Acc sh[kBlock];
    const unsigned mine = threadIdx.x & (outs - 1), group = threadIdx.x / outs, groups = kBlock / outs;
    const unsigned out = blockIdx.x * outs + mine;
    const unsigned per_group = (n_seg + groups - 1) / groups;
    const unsigned g_begin = min(n_seg, group * per_group), g_end = min(n_seg, g_begin + per_group);
    long long o0 = 0, o1 = 0, o2 = 0;
    if (out < n_out) red_finish_coords(k, out, row_mode, o0, o1, o2);
    RedStats emitted;
    for (int s = 0; s < k.n_red; ++s) {
        const int opc = red_opcode(k, s);
        const bool with_index = opc >= NGH_OP_RED_ARGMAX;
        Acc a = acc_init(opc);
        if (out < n_out) {
            // eight partial results are asked for before the first is merged: the loads are
            // independent, the merges are not, and one round trip per segment is what this
            // kernel's time would otherwise consist of
            constexpr int kBatch = 8;
            for (unsigned g0 = g_begin; g0 < g_end; g0 += kBatch) {
                Acc b[kBatch];
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const unsigned g = min(g0 + j, g_end - 1);          // (a repeated load, merged only once)
                    const size_t w = ((size_t)s * n_seg + g) * n_out + out;
                    b[j].v = ws.val[w];
                    b[j].i = with_index ? ws.idx[w] : 0;
                }
#pragma unroll
                for (int j = 0; j < kBatch; ++j)
                    if (g0 + j < g_end) a = acc_merge(opc, a, b[j]);
            }
        }
        sh[threadIdx.x] = a;
        __syncthreads();
        if (group == 0 && out < n_out) {
            // (a group that had no segments holds the reduction's identity)
            for (unsigned g = 1; g < groups; ++g) a = acc_merge(opc, a, sh[g * outs + mine]);
            RedWs none{nullptr, nullptr};
            red_emit(k, s, a, o0, o1, o2, out, n_out, 0, 1, none, emitted);
        }
        __syncthreads();
    }
    red_stats_flush(k, emitted);
}

// The partial results of output `out` that lanes first, first + step, ... of a group own, merged:
// four of them are asked for before the first is merged (independent loads, dependent merges).
__device__ __forceinline__ Acc red_finish_strided(const RedWs& ws, int opc, int s, unsigned n_seg, unsigned n_out,
                                                  unsigned out, unsigned first, unsigned step) {
    constexpr int kBatch = 4;
    const bool with_index = opc >= NGH_OP_RED_ARGMAX;
    Acc a = acc_init(opc);
    for (unsigned g0 = first; g0 < n_seg; g0 += step * kBatch) {
        Acc b[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const unsigned g = min(g0 + j * step, n_seg - 1);          // (a repeated load, merged only once)
            const size_t w = ((size_t)s * n_seg + g) * n_out + out;
            b[j].v = ws.val[w];
            b[j].i = with_index ? ws.idx[w] : 0;
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
            if (g0 + j * step < n_seg) a = acc_merge(opc, a, b[j]);
    }
    return a;
}

// A wavefront per output: for fewer outputs than would fill workgroups of 64, with many segments each.
__global__ __launch_bounds__(kBlock) void red_finish_wave_kernel(const KArgs k, unsigned n_out,
                                                                 unsigned n_seg, int row_mode, RedWs ws) {
    const unsigned lane = threadIdx.x & 63;
    const unsigned out = blockIdx.x * kWaves + (threadIdx.x >> 6);
    RedStats emitted;
    long long o0 = 0, o1 = 0, o2 = 0;
    if (out < n_out) red_finish_coords(k, out, row_mode, o0, o1, o2);
    for (int s = 0; s < k.n_red && out < n_out; ++s) {
        const int opc = red_opcode(k, s);
        Acc a = red_finish_strided(ws, opc, s, n_seg, n_out, out, lane, 64);
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) a = acc_merge(opc, a, acc_shfl_xor(a, m));
        if (lane == 0) {
            RedWs none{nullptr, nullptr};
            red_emit(k, s, a, o0, o1, o2, out, n_out, 0, 1, none, emitted);
        }
    }
    red_stats_flush(k, emitted);
}

// A workgroup per output: a handful of outputs with hundreds of segments each (a sum of a whole
// tensor into one number), where a wavefront per output would be one or two wavefronts walking a
// long chain of round trips.
__global__ __launch_bounds__(kBlock) void red_finish_block_kernel(const KArgs k, unsigned n_out,
                                                                  unsigned n_seg, int row_mode, RedWs ws) {
    __shared__ Acc sh[kWaves];
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned out = blockIdx.x;                 // (the grid has n_out workgroups)
    RedStats emitted;
    long long o0 = 0, o1 = 0, o2 = 0;
    red_finish_coords(k, out, row_mode, o0, o1, o2);
    for (int s = 0; s < k.n_red; ++s) {
        const int opc = red_opcode(k, s);
        Acc a = red_finish_strided(ws, opc, s, n_seg, n_out, out, threadIdx.x, kBlock);
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) a = acc_merge(opc, a, acc_shfl_xor(a, m));
        if (lane == 0) sh[wave] = a;
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < kWaves; ++w) a = acc_merge(opc, a, sh[w]);
            RedWs none{nullptr, nullptr};
            red_emit(k, s, a, o0, o1, o2, out, n_out, 0, 1, none, emitted);
        }
        __syncthreads();                             // (sh is written again for the next reduction)
    }
    red_stats_flush(k, emitted);
}

}  // namespace ngh
