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
__device__ __forceinline__ int ex_accv(const KArgs& k, int slot) { return k.n_stat_slots + 2 * slot; }
__device__ __forceinline__ int ex_acci(const KArgs& k, int slot) { return k.n_stat_slots + 2 * slot + 1; }

struct Extra {
    float* base;  // &extra[thread]
    int    nthr;
    __device__ __forceinline__ int   geti(int j) const { return __float_as_int(base[j * nthr]); }
    __device__ __forceinline__ float getf(int j) const { return base[j * nthr]; }
    __device__ __forceinline__ void  seti(int j, int x) { base[j * nthr] = __int_as_float(x); }
    __device__ __forceinline__ void  setf(int j, float x) { base[j * nthr] = x; }
};

// RMODE: 0 = no reductions, 1 = reduction runs along kernel axis 2 (the vector
// axis), 2 = reduction runs along kernel axis 0.
template <int V, int RMODE>
__device__ __forceinline__ void run_ops(const KArgs& k, LdsRegs<V>& rf, Extra& ex,
                                        long long i0, long long i1, long long i2) {
    for (int pc = k.op_begin; pc < k.op_end; ++pc) {
        const ngh_op o = k.ops[pc];
        const int opc = o.opcode;
        switch (opc) {
            case NGH_OP_LOAD: {
                const KTensor& t = k.t[o.a];
                const long long off = i0 * t.s[0] + i1 * t.s[1] + i2 * t.s[2];
                const float sc = (t.dtype == NGH_FLEX16) ? tensor_scale(t) : 1.0f;
                if (t.s[2] == 0) {
                    const float x = load1(t, off, sc);
#pragma unroll
                    for (int v = 0; v < V; ++v) rf.set(o.dst, v, x);
                } else if (V >= 4 && t.s[2] == 1) {
                    float x[V >= 4 ? V : 4];
                    if constexpr (V >= 4) loadv<V>(t, off, sc, x);
#pragma unroll
                    for (int v = 0; v < V; ++v) rf.set(o.dst, v, x[v]);
                } else {
#pragma unroll
                    for (int v = 0; v < V; ++v) rf.set(o.dst, v, load1(t, off + v * t.s[2], sc));
                }
            } break;
            case NGH_OP_STORE: {
                const KTensor& t = k.t[o.dst];
                const long long off = i0 * t.s[0] + i1 * t.s[1] + i2 * t.s[2];
                const float sc = (t.dtype == NGH_FLEX16) ? 1.0f / tensor_scale(t) : 1.0f;
                int fmax = 0;
                if (k.probe) {
#pragma unroll
                    for (int v = 0; v < V; ++v) fmax = max(fmax, probe_bits(rf.get(o.a, v)));
                } else if (V >= 4 && t.s[2] == 1) {
                    float x[V >= 4 ? V : 4];
#pragma unroll
                    for (int v = 0; v < V; ++v) x[v] = rf.get(o.a, v);
                    if constexpr (V >= 4) storev<V>(t, off, sc, x, fmax);
                } else {
#pragma unroll
                    for (int v = 0; v < V; ++v) store1(t, off + v * t.s[2], rf.get(o.a, v), sc, fmax);
                }
                if (t.stat_slot >= 0) ex.seti(ex_stat(t.stat_slot), max(ex.geti(ex_stat(t.stat_slot)), fmax));
            } break;
            case NGH_OP_CONST: {
                const float c = k.consts[o.a];
#pragma unroll
                for (int v = 0; v < V; ++v) rf.set(o.dst, v, c);
            } break;
            case NGH_OP_IOTA: {
                const int ka = k.iota_map[o.a];
#pragma unroll
                for (int v = 0; v < V; ++v)
                    rf.set(o.dst, v, (float)(ka == 2 ? i2 + v : (ka == 1 ? i1 : i0)));
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
#undef NGH_BIN
            case NGH_OP_RED_SUM: case NGH_OP_RED_PROD: case NGH_OP_RED_MAX:
            case NGH_OP_RED_MIN: case NGH_OP_RED_ARGMAX: case NGH_OP_RED_ARGMIN: {
                if (RMODE != 0) {
                    Acc a;
                    a.v = ex.getf(ex_accv(k, o.dst));
                    a.i = ex.geti(ex_acci(k, o.dst));
#pragma unroll
                    for (int v = 0; v < V; ++v) {
                        Acc b;
                        b.v = rf.get(o.a, v);
                        b.i = (int)(RMODE == 1 ? i2 + v : i0);
                        a = acc_merge(opc, a, b);
                    }
                    ex.setf(ex_accv(k, o.dst), a.v);
                    ex.seti(ex_acci(k, o.dst), a.i);
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
        run_ops<V, 0>(k, rf, ex, i0, i1, (long long)c2 * V);
    }
    stats_epilogue(k, ex);
}

// Partial results of a reduction split over several workgroups.
struct RedWs {
    float* val;   // [slot][segment][output]
    int*   idx;
};

__device__ __forceinline__ void red_emit(const KArgs& k, int slot, Acc a, long long o0, long long o1,
                                         long long o2, unsigned out, unsigned n_out, unsigned seg,
                                         unsigned n_seg, RedWs ws) {
    if (n_seg == 1) {
        const KTensor& t = k.t[k.red_out[slot]];
        const long long off = o0 * t.s[0] + o1 * t.s[1] + o2 * t.s[2];
        const float sc = (t.dtype == NGH_FLEX16) ? 1.0f / tensor_scale(t) : 1.0f;
        const float result = acc_result(k.ops[k.op_end - k.n_red + slot].opcode, a);
        int fmax = 0;
        if (k.probe) {
            if (t.dtype == NGH_FLEX16) fmax = probe_bits(result);
        } else {
            store1(t, off, result, sc, fmax);
        }
        if (t.stats != nullptr && fmax > 0) atomicMax(t.stats, fmax);
    } else {
        const size_t w = ((size_t)slot * n_seg + seg) * n_out + out;
        ws.val[w] = a.v;
        ws.idx[w] = a.i;
    }
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
        run_ops<V, 1>(k, rf, ex, i0, i1, (long long)c * V);

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
    if (threadIdx.x == 0) {
        for (int s = 0; s < k.n_red; ++s) {
            const int opc = red_opcode(k, s);
            Acc a = sh[s][0];
            for (int w = 1; w < kWaves; ++w) a = acc_merge(opc, a, sh[s][w]);
            red_emit(k, s, a, i0, i1, 0, out, n_out, seg, n_seg, ws);
        }
    }
    stats_epilogue(k, ex);
}

// ---------------------------------------------------------------------------
// Reduction along kernel axis 0 with outputs contiguous along kernel axis 2:
// workgroup = 64 consecutive outputs x 4 interleaved rows of the reduced
// axis; lanes stay coalesced along axis 2 while each walks down axis 0.
// ---------------------------------------------------------------------------
constexpr int kColTx = 64, kColTy = kBlock / kColTx;

__global__ __launch_bounds__(kBlock) void red_col_interp_kernel(const KArgs k, unsigned n_bx,
                                                                unsigned n_seg, unsigned seg_rows,
                                                                RedWs ws) {
    extern __shared__ float lds[];
    __shared__ Acc sh[NGH_MAX_REDUCTIONS][kColTy][kColTx];
    LdsRegs<1> rf{lds + threadIdx.x, kBlock};
    Extra ex{lds + (size_t)k.n_regs * kBlock + threadIdx.x, kBlock};
    for (int s = 0; s < k.n_stat_slots; ++s) ex.seti(ex_stat(s), 0);
    for (int s = 0; s < k.n_red; ++s) {
        Acc a = acc_init(red_opcode(k, s));
        ex.setf(ex_accv(k, s), a.v);
        ex.seti(ex_acci(k, s), a.i);
    }
    const unsigned tx = threadIdx.x & (kColTx - 1), ty = threadIdx.x / kColTx;
    unsigned b = blockIdx.x;
    const unsigned seg = b % n_seg;  b /= n_seg;
    const unsigned bx = b % n_bx;    b /= n_bx;
    const unsigned i1 = b;
    const unsigned d2 = (unsigned)k.shape[2];
    const unsigned i2 = bx * kColTx + tx;
    const unsigned r_begin = seg * seg_rows;
    const unsigned r_end = min((unsigned)k.shape[0], r_begin + seg_rows);
    if (i2 < d2)
        for (unsigned r = r_begin + ty; r < r_end; r += kColTy) run_ops<1, 2>(k, rf, ex, r, i1, i2);

    for (int s = 0; s < k.n_red; ++s) {
        Acc a;
        a.v = ex.getf(ex_accv(k, s));
        a.i = ex.geti(ex_acci(k, s));
        sh[s][ty][tx] = a;
    }
    __syncthreads();
    if (ty == 0 && i2 < d2) {
        const unsigned n_out = (unsigned)k.shape[1] * d2;
        const unsigned out = i1 * d2 + i2;
        for (int s = 0; s < k.n_red; ++s) {
            const int opc = red_opcode(k, s);
            Acc a = sh[s][0][tx];
            for (int y = 1; y < kColTy; ++y) a = acc_merge(opc, a, sh[s][y][tx]);
            red_emit(k, s, a, 0, i1, i2, out, n_out, seg, n_seg, ws);
        }
    }
    stats_epilogue(k, ex);
}

// Second pass of a split reduction: one thread per output merges the
// segments in order and stores through the output's storage type.
// `row_mode` tells how an output number maps to kernel coordinates.
__global__ __launch_bounds__(kBlock) void red_finish_kernel(const KArgs k, unsigned n_out,
                                                            unsigned n_seg, int row_mode, RedWs ws) {
    const unsigned out = blockIdx.x * kBlock + threadIdx.x;
    if (out >= n_out) return;
    long long o0, o1, o2;
    if (row_mode) {
        const unsigned d1 = (unsigned)k.shape[1];
        o0 = out / d1; o1 = out - (unsigned)o0 * d1; o2 = 0;
    } else {
        const unsigned d2 = (unsigned)k.shape[2];
        o0 = 0; o1 = out / d2; o2 = out - (unsigned)o1 * d2;
    }
    for (int s = 0; s < k.n_red; ++s) {
        const int opc = red_opcode(k, s);
        Acc a = acc_init(opc);
        for (unsigned g = 0; g < n_seg; ++g) {
            const size_t w = ((size_t)s * n_seg + g) * n_out + out;
            Acc b; b.v = ws.val[w]; b.i = ws.idx[w];
            a = acc_merge(opc, a, b);
        }
        RedWs none{nullptr, nullptr};
        red_emit(k, s, a, o0, o1, o2, out, n_out, 0, 1, none);
    }
}

}  // namespace ngh
