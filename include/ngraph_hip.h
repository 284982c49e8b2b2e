/*
 * ngraph_hip.h -- C ABI of libngraph_hip.so, the MI355X (gfx950) execution
 * library behind the `hipgpu` / `flexhip` transformers.
 *
 * The library replaces, for the fused elementwise / reduction / flex16 path,
 * what the reference GPU transformer obtains from pycuda + NVRTC:
 *   - device runtime        ngraph/transformers/gputransform.py:912-1000 (GPURuntime)
 *   - device memory         ngraph/transformers/gputransform.py:525-676  (drv.mem_alloc, views)
 *   - host <-> device I/O   ngraph/transformers/gputransform.py:710-909  (get / __setitem__)
 *   - compound kernels      ngraph/transformers/gpu/float_ew2.py:1135-1483
 *                           (_get_compound_kernel / prepared_async_call)
 *   - flex scale + maxabs   ngraph/transformers/gpu/float_ew2.py:93-98, 261-281, 1346-1404
 *                           ngraph/transformers/flexgputransform.py:56-61
 *   - strided copies        ngraph/transformers/gpu/kernels/cuda/copy_transpose.py:89-282
 *
 * Conventions: every entry point returns 0 on success and a negative
 * NGH_E_* code on failure; the text of the last failure on the calling
 * thread is available from ngh_last_error().  Nothing aborts.  Pointers
 * named `dev*` are device addresses obtained from ngh_malloc; all other
 * pointers are host memory.  All work is issued, in order, on one HIP
 * stream owned by the context; only ngh_sync, ngh_memcpy_d2h and
 * ngh_stats_read wait for it.
 */
#ifndef NGRAPH_HIP_H
#define NGRAPH_HIP_H

#if !defined(__HIPCC_RTC__)     /* (in-process compilation of kernels has these types built in) */
#include <stddef.h>
#include <stdint.h>
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define NGH_ABI_VERSION 7

/* ---- limits (float_ew2.py:285-286 MAX_AXES = 3) ------------------------ */
#define NGH_MAX_AXES      3
#define NGH_MAX_TENSORS   12
#define NGH_MAX_OPS       96
#define NGH_MAX_CONSTS    16
#define NGH_MAX_REGS      32
#define NGH_MAX_REDUCTIONS 4
#define NGH_MAX_STAGES    6

/* ---- error codes -------------------------------------------------------- */
#define NGH_OK             0
#define NGH_E_INVALID     -1   /* malformed argument or spec               */
#define NGH_E_RUNTIME     -2   /* a HIP runtime call failed                */
#define NGH_E_NOMEM       -3   /* device allocation failed                 */
#define NGH_E_UNSUPPORTED -4   /* valid but outside what the kernels cover */
#define NGH_E_NODEVICE    -5   /* no usable gfx950 device                  */

/* ---- storage types (float_ew2.py:615-641 _get_register_type) ------------ */
#define NGH_F32     0          /* float                                     */
#define NGH_FLEX16  1          /* int16 mantissa, shared per-tensor scale   */
#define NGH_I32     2          /* int32 (argmax / argmin results, indices)  */
#define NGH_F16     3          /* IEEE half in memory, float in registers   */
/* Integer storage: converted to float on load; a store converts toward zero and
 * saturates at the type's range (the device conversion the reference's generated
 * "(type)reg" assignment compiles to).  A value converted this way is exact up to 2^24; a caller
 * that wants the reference's integer registers (float_ew2.py:615-641) binds the int32 / uint32
 * tensor as NGH_F32, which moves its bits untouched, and uses the integer ops at the end of
 * the opcode list.  Where an index could exceed 2^24, the library keeps it an integer or refuses the spec with
 * NGH_E_UNSUPPORTED instead of losing bits: argmax / argmin into NGH_I32 / NGH_U32 storage
 * store the integer index itself (over more than 2^24 elements any other result type is
 * refused); NGH_OP_TAKE from a table of more than 2^24 entries along the looked-up axis and
 * NGH_OP_IOTA along an axis longer than 2^24 are refused.                              */
#define NGH_U32     4          /* uint32                                    */
#define NGH_I16     5          /* int16 (plain integers, no scale)          */
#define NGH_I8      6          /* int8                                      */
#define NGH_U8      7          /* uint8 (image bytes on the loader side)    */

/* ---- spec flags ---------------------------------------------------------
 * NGH_SPEC_PROBE: run the program but store NOTHING; instead every FLEX16
 * tensor the program would write gets, in its dev_stats word, the bit pattern
 * of max |fp32 value| it would have been asked to store (NaN ignored; compare
 * as int32).  A flex manager uses one probe launch to choose the first
 * exponent of a fresh output tensor from its true range, the state the
 * reference's known-answer vectors show after a tensor's first use
 * (tests/flex_tests/test_flexew/test_complex_math.py:31,47).                */
#define NGH_SPEC_PROBE  1

/* ---- opcodes ------------------------------------------------------------
 * One entry per template of float_ew2.py:31-68 (_op_templates) and
 * :70-77 (_redop_templates).  Arithmetic follows the NumPy float32 calls the
 * CPU transformer issues (cputransform.py:512-761) wherever the CUDA template
 * and NumPy disagree (floor_divide / mod on negative operands, sign of NaN).
 * Registers are fp32 unless an op says otherwise (the integer ops at the end). */
enum ngh_opcode {
    NGH_OP_NOP = 0,
    /* data movement: LOAD dst=reg a=tensor ; STORE dst=tensor a=reg ;
     * CONST dst=reg a=const slot ; IOTA dst=reg a=axis (index along axis) */
    NGH_OP_LOAD, NGH_OP_STORE, NGH_OP_CONST, NGH_OP_IOTA,
    /* unary: dst=reg a=reg */
    NGH_OP_ASSIGN, NGH_OP_NEG, NGH_OP_ABS, NGH_OP_SQRT, NGH_OP_SQR, NGH_OP_EXP,
    NGH_OP_LOG, NGH_OP_RCP, NGH_OP_EXP2, NGH_OP_LOG2, NGH_OP_SIG, NGH_OP_TANH,
    NGH_OP_SAFELOG, NGH_OP_SGN, NGH_OP_SIN, NGH_OP_COS,
    /* binary: dst=reg a=reg b=reg */
    NGH_OP_ADD, NGH_OP_SUB, NGH_OP_MUL, NGH_OP_DIV, NGH_OP_INT_DIV, NGH_OP_MOD,
    NGH_OP_EQ, NGH_OP_NE, NGH_OP_LT, NGH_OP_LE, NGH_OP_GT, NGH_OP_GE,
    NGH_OP_POW, NGH_OP_MINIMUM, NGH_OP_MAXIMUM,
    /* reductions over axis 0 of the stage's view: dst=reduction slot a=reg */
    NGH_OP_RED_SUM, NGH_OP_RED_PROD, NGH_OP_RED_MAX, NGH_OP_RED_MIN,
    NGH_OP_RED_ARGMAX, NGH_OP_RED_ARGMIN,
    /* lookup ("take", float_ew2.py:65, 122-125, 1242-1258; the fprop of LookupTableOp,
     * gputransform.py:197-199): dst=reg a=reg holding the index b=tensor | axis << 4.
     * Loads the tensor's element whose coordinate along `axis` is (int)index instead of the
     * loop coordinate; the tensor's stride on that axis is the table's stride along its
     * looked-up axis and take_extent its length there (indices are clamped to it).       */
    NGH_OP_TAKE,
    /* STORE whose conversion to a FLEX16 mantissa truncates toward zero instead of rounding
     * to nearest: the fill of a flex tensor, int(value / scale) clipped
     * (tensor_ops.py:690-707 FlexFillKernel).  Other storage types: same as STORE.        */
    NGH_OP_STORE_TRUNC,
    /* random fills (RngFillKernel, tensor_ops.py:621-661; RngOp, op_graph.py:2786-2870):
     * dst=reg a=stream number.  Each element draws from a counter-based generator
     * (Philox-4x32-10) keyed by the spec's rng_seed, with counter (linear index of the element
     * in the spec's axis order, stream, rng_counter): the value of an element does not depend
     * on how the launch is split over lanes, and a caller that bumps rng_counter per execution
     * gets fresh numbers every time.  UNIFORM is in [0, 1); NORMAL is standard normal
     * (Box-Muller).  The streams differ from the reference's (curand / numpy), as those two
     * differ from each other; only the distributions can be compared.                      */
    NGH_OP_RNG_UNIFORM, NGH_OP_RNG_NORMAL,
    /* 32-bit integer arithmetic.  The reference keeps int32 / uint32 operands in `int` /
     * `unsigned int` registers (float_ew2.py:615-641 _get_register_type) and NumPy computes
     * integer inputs with its integer loops before it casts to the output type
     * (cputransform.py:512-761 hands the arrays to the ufuncs as they are): where every
     * operand of an op is such an integer the arithmetic is integer arithmetic, exact over the
     * whole range and wrapping at 2^32.  A register holds 32 bits either way; these ops read
     * and write them as integers.  A tensor whose elements they produce or consume is bound as
     * NGH_F32, so that LOAD and STORE move its bits untouched.
     * unary: I2F / U2F = (float)int32 / (float)uint32, INEG, IABS (as int32)              */
    NGH_OP_I2F, NGH_OP_U2F, NGH_OP_INEG, NGH_OP_IABS,
    /* binary: IADD, ISUB, IMUL wrap (the same bits for int32 and uint32); IMIN / IMAX and
     * UMIN / UMAX compare as int32 / uint32; the comparisons give 1.0f / 0.0f              */
    NGH_OP_IADD, NGH_OP_ISUB, NGH_OP_IMUL, NGH_OP_IMIN, NGH_OP_IMAX, NGH_OP_UMIN, NGH_OP_UMAX,
    NGH_OP_IEQ, NGH_OP_INE, NGH_OP_ILT, NGH_OP_ILE, NGH_OP_IGT, NGH_OP_IGE,
    NGH_OP_ULT, NGH_OP_ULE, NGH_OP_UGT, NGH_OP_UGE,
    NGH_OP_COUNT_
};

/* ngh_tensor.cache_hint */
enum {
    NGH_CACHE_STREAM_LOAD  = 1u,  /* no other kernel of the computation reads the operand:
                                     load it non-temporally                                */
    NGH_CACHE_STREAM_STORE = 2u   /* nothing reads the result soon (not an in-place update,
                                     no later kernel of the computation reads it): store it
                                     non-temporally so it does not displace operands        */
};

typedef struct ngh_op {
    uint8_t opcode;            /* enum ngh_opcode                            */
    uint8_t dst;
    uint8_t a;
    uint8_t b;
} ngh_op;

/* One operand of a fused kernel: the strided view the reference passes as
 * (pointer, stride_a, stride_b, stride_c [, flex scale [, flex_stats]])
 * (float_ew2.py:987-1132).  Strides are in ELEMENTS; stride 0 broadcasts. */
typedef struct ngh_tensor {
    void*    dev;              /* device address of view element (0,0,0)     */
    int64_t  strides[NGH_MAX_AXES];
    int32_t  dtype;            /* one of the NGH_* storage types            */
    float    scale;            /* FLEX16 only: the tensor's scale 2**-dec.
                                  Loaded value = scale * int16; stored int16 =
                                  rni_sat(value * (1/scale)).  The reference
                                  binds entry.scale to inputs and 1/entry.scale
                                  to outputs (flexgputransform.py:56-61); one
                                  field serves both here because 1/scale is
                                  exact for a power of two, and a tensor
                                  updated in place needs both directions     */
    int32_t* dev_stats;        /* FLEX16 outputs: int32 max|mantissa| merged
                                  with atomic max (float_ew2.py:281,1404);
                                  NULL = no statistics                       */
    const float* dev_scale;    /* FLEX16 only, optional: when not NULL the
                                  kernel reads the scale from this device
                                  word instead of `scale` (lets an on-device
                                  exponent update feed the next launch
                                  without a host round trip)                 */
    uint32_t cache_hint;       /* NGH_CACHE_* bits: what the caller knows of
                                  this operand's reuse.  Hints only act in
                                  streaming kernels whose operands exceed the
                                  last-level cache; no counterpart in the
                                  reference (PTX loads there carry no hint)   */
    uint32_t take_extent;      /* operand of NGH_OP_TAKE: length of the looked-up
                                  axis; 0 otherwise                           */
} ngh_tensor;

/* One stage = a run of elementwise ops optionally ended by reductions
 * (float_ew2.py:553-612 _preprocess_ops).  Every stage iterates over the
 * spec's single view `shape`; reductions run over axis 0 of that view
 * (gputransform.py:117-122: reductions always pass axis 0), so the tensor
 * receiving a reduction has stride 0 on axis 0 (the "missing axis" of
 * float_ew2.py:307-309).  Stages run in order; a later stage reads an
 * earlier stage's reduction result as a broadcast load.                     */
typedef struct ngh_stage {
    int32_t  op_begin, op_end; /* half-open range into ngh_fused_spec.ops    */
    int32_t  n_reductions;     /* 0 = pure elementwise stage                 */
    int32_t  red_out[NGH_MAX_REDUCTIONS];  /* tensor index receiving slot k  */
} ngh_stage;

typedef struct ngh_fused_spec {
    int32_t     abi_version;   /* NGH_ABI_VERSION                            */
    int32_t     rank;          /* 1..3; axes beyond rank have length 1       */
    int64_t     shape[NGH_MAX_AXES];
    int32_t     n_tensors, n_ops, n_consts, n_stages, n_regs;
    int32_t     flags;         /* NGH_SPEC_* bits                            */
    ngh_tensor  tensors[NGH_MAX_TENSORS];
    float       consts[NGH_MAX_CONSTS];
    ngh_op      ops[NGH_MAX_OPS];
    ngh_stage   stages[NGH_MAX_STAGES];
    uint32_t    rng_seed;      /* NGH_OP_RNG_*: key of the generator            */
    uint32_t    rng_counter;   /* NGH_OP_RNG_*: execution number (caller bumps)  */
} ngh_fused_spec;

typedef struct ngh_context ngh_context;

/* ---- runtime: replaces GPURuntime / drv.init (gputransform.py:912-935) --- */
int  ngh_abi_version(void);
const char* ngh_last_error(void);
int  ngh_device_count(int* count);
int  ngh_init(int device_id, ngh_context** out_ctx);
int  ngh_shutdown(ngh_context* ctx);
int  ngh_sync(ngh_context* ctx);
/* name (<=255 chars + NUL), compute units, bytes of device memory */
int  ngh_device_info(ngh_context* ctx, char* name256, int* compute_units,
                     uint64_t* total_bytes);

/* ---- memory: replaces drv.mem_alloc / free / memcpy / GPUArray.fill
 *      (gputransform.py:547-569, 710-744, 807-871)                          */
int  ngh_malloc(ngh_context* ctx, size_t bytes, void** out_dev);
int  ngh_free(ngh_context* ctx, void* dev);
int  ngh_memcpy_h2d(ngh_context* ctx, void* dev, const void* host, size_t bytes);
int  ngh_memcpy_d2h(ngh_context* ctx, void* host, const void* dev, size_t bytes);
int  ngh_memcpy_d2d(ngh_context* ctx, void* dev_dst, const void* dev_src, size_t bytes);
/* The two host copies above block until the data has arrived, like GPUArray.set / .get.  From
 * 4 MiB on they go through pinned staging buffers owned by the context (4 x 16 MiB from
 * hipHostMalloc, allocated at the first such copy) with NGH_COPY_THREADS host threads (default
 * 8; 0 leaves the staging to the runtime) moving the data between the caller's pageable array
 * and the buffers while the copy engine works on the slot before.                            */
/* Device scratch of at least `bytes`, owned by the context and reused from call to call: the
 * contiguous intermediate of strided host reads and writes, which the reference allocates and
 * frees per access (gputransform.py:873-909 through copy_transpose).  Valid until the next call
 * that asks for more; the stream is drained before it is replaced.                           */
int  ngh_io_scratch(ngh_context* ctx, size_t bytes, void** out_dev);
int  ngh_memset32(ngh_context* ctx, void* dev, uint32_t value, size_t count);
int  ngh_memset16(ngh_context* ctx, void* dev, uint16_t value, size_t count);

/* ---- strided copy / dimshuffle: replaces _get_copy_transpose_kernel
 *      (copy_transpose.py:89-282) and DimShuffleKernel (tensor_ops.py:137-204).
 *      Copies an N-d view (rank <= 8) element by element; itemsize 1, 2 or 4. */
int  ngh_copy_strided(ngh_context* ctx, void* dev_dst, const void* dev_src,
                      int32_t rank, const int64_t* shape,
                      const int64_t* dst_strides, const int64_t* src_strides,
                      int32_t itemsize);

/* ---- compound kernels: replaces CudaSourceFile.add_kernel + compile +
 *      prepared_async_call (float_ew2.py:1553-1653, gputransform.py:343-345) */
int  ngh_validate_fused(const ngh_fused_spec* spec);
/* Stages run in order and each stage sees what the stages before it wrote, also when two
 * operand slots name overlapping memory (an in-place update through a second view): a spec
 * with such slots, one of them written, is never run as one row-chain kernel, whose stages
 * keep operands in registers; it is launched stage by stage.  Within ONE stage the reference's
 * rule holds (float_ew2.py:685-790: a buffer is one register per kernel): an element written
 * through one slot must not be read through another slot at a different position.          */
int  ngh_launch_fused(ngh_context* ctx, const ngh_fused_spec* spec);
/* Which pre-built kernel family ngh_launch_fused picks for stage `stage`
 * of `spec` (diagnostics and tests): writes a NUL-terminated name.          */
int  ngh_describe_fused(ngh_context* ctx, const ngh_fused_spec* spec,
                        int32_t stage, char* name128);

/* ---- run-time compiled programs: replaces the NVRTC step of the reference, which writes the
 *      CUDA C of a kernel and compiles it when the transformer is initialised
 *      (float_ew2.py:1553-1653 CudaSourceFile.add_kernel / compile).  Here the host side writes
 *      the op programs of a computation that the library has no compiled kernel for as C++
 *      tables, compiles them with hipcc into a program library, and hands its path over; from
 *      then on ngh_launch_fused finds those kernels the way it finds the built-in ones (a
 *      structural comparison, float_ew2.py:1486-1529 / :1560-1567 being the reference's hash
 *      lookup), in every context of the process.  The library stays loaded.  out_added, when
 *      not NULL, receives the number of programs that were new.  A library built from other
 *      sources than this one (NGH_ABI_VERSION, layout of the argument block) is rejected with
 *      NGH_E_INVALID.  A program library exports one function, named ngh_program_library,
 *      taking (int abi, unsigned entry_bytes, unsigned args_bytes, const void** out_entries)
 *      and returning the number of entries, or -1 when the three numbers are not its own.  */
int  ngh_programs_load(ngh_context* ctx, const char* path, int32_t* out_added);
/* number of compiled programs the process knows: built in, loaded */
int  ngh_programs_count(int32_t* built_in, int32_t* loaded);

/* ---- the same without a compiler on the machine: the reference compiles inside the process
 *      (NVRTC) and launches through the driver API (float_ew2.py:1626-1653
 *      CudaSourceFile.compile -> SourceModule.get_function -> prepared_async_call).  The host
 *      side compiles the generated source with hiprtc, device code only, into a code object and
 *      hands it over with a description of every program in it.  A description restates what the
 *      source's `struct <type_name>` holds, which is what ngh_launch_fused compares a stage
 *      with; for a chain (family 4: stages over the same rows, 5: over the same columns) the
 *      n_stages descriptions that follow it are its stages.                                   */
typedef struct ngh_program_desc {
    char     name[64];                        /* as shown by ngh_describe_fused            */
    char     type_name[64];                   /* the C++ struct of the source, in namespace ngh */
    int32_t  family, V, n_ops, n_tensors, n_red, n_stat_slots, n_stages;
    ngh_op   ops[NGH_MAX_OPS];
    int32_t  dtypes[NGH_MAX_TENSORS];
    uint8_t  bcast[NGH_MAX_TENSORS];          /* constant along the lanes' axis            */
    uint8_t  rowshared[NGH_MAX_TENSORS];      /* stages of a chain: the same for every row */
    int8_t   staged[NGH_MAX_TENSORS];         /* family 3: LDS tile number or -1           */
    int32_t  red_out[NGH_MAX_REDUCTIONS];
} ngh_program_desc;
#define NGH_PROGRAM_KERNEL_SLOTS 12
/* The C++ name expressions of the kernels that program `index` of descs[0..n) may launch
 * (cache-policy, ragged-row, deferred-statistics, tile-size and chunks-per-lane variants): what
 * the host gives hiprtcAddNameExpression.  Written to `out` as NGH_PROGRAM_KERNEL_SLOTS lines
 * ('\n'-terminated), an empty line for a slot the program has no kernel for.  `index` must be a
 * program of its own or a chain, not a chain's stage.  Needs no context and no device.        */
int  ngh_program_kernels(const ngh_program_desc* descs, int32_t n, int32_t index, char* out, size_t out_bytes);
/* Loads the code object (hipModuleLoadData on the context's device; it stays loaded) and
 * appends its programs to the table.  `lowered` holds, for every program of its own and every
 * chain of descs in order, NGH_PROGRAM_KERNEL_SLOTS lines: the lowered (mangled) names of the
 * kernels in the slots of ngh_program_kernels, empty where the slot is.  out_added as above.  */
int  ngh_programs_load_code(ngh_context* ctx, const void* code, size_t code_bytes,
                            const ngh_program_desc* descs, int32_t n, const char* lowered,
                            int32_t* out_added);

/* Per-row mean and (biased) variance of a [rows, R] fp32 matrix with contiguous rows in ONE
 * read of x (x_cache_hint: NGH_CACHE_* bits for x): fuses the reductions behind ng.mean + ng.variance
 * (op_graph.py:4007-4009, 4252-4266), the statistics of batch normalisation
 * (frontends/neon/layer.py:1242-1245).  row_stride in elements (any: rows need not start on
 * 16-byte boundaries).
 * dev_rstd, when not NULL, also receives 1/sqrt(var + eps), the factor of layer.py:1255.  */
int  ngh_moments_f32(ngh_context* ctx, const float* dev_x, int64_t rows, int64_t R, int64_t row_stride,
                     float* dev_mean, float* dev_var, float* dev_rstd, float eps, uint32_t x_cache_hint);

/* ngh_moments_f32 for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it).  No counterpart in the reference.  Same
 * arguments, same kernel and same results, but the per-segment partial sums and the per-row
 * arrival counters live in a fixed array inside the library (768 KiB per device, held until the
 * process ends) instead of context-owned allocations, and the call allocates and frees
 * nothing.  Limits: rows <= 65536 and rows x segments <= 65536 (segments = what it takes to
 * put 8 workgroups on every compute unit, at most 4096 a row); beyond them the call fails
 * with NGH_E_UNSUPPORTED and launches nothing.  Every call on a device shares that device's
 * array: calls that overlap there (two contexts, two host threads) race.                   */
int  ngh_moments_f32_noalloc(ngh_context* ctx, const float* dev_x, int64_t rows, int64_t R, int64_t row_stride,
                             float* dev_mean, float* dev_var, float* dev_rstd, float eps, uint32_t x_cache_hint);

/* ---- float -> flex16 converter: replaces `convert` (gpu/flex_conv.py:745-791,
 *      _prepare_convert_kernel :734-740), which turns the raw fp32 (or fp16) output of a dense
 *      kernel into a flex tensor.  dev_out[i] = (int16)trunc(dev_in[i] * scale), toward zero;
 *      values outside the int16 range (undefined in the reference's cast) saturate at
 *      -32768 / 32767, NaN gives 0.  in_dtype is NGH_F32 or NGH_F16.  max |mantissa| is merged
 *      into *dev_stats with an atomic max when dev_stats is not NULL (as int32: -32768 counts
 *      as 32768).  When dev_scale is not NULL the multiplier is 1 / *dev_scale instead of
 *      `scale`: the destination tensor's scale read on the device, for exponent management
 *      that lives there.                                                               */
int  ngh_convert_to_flex16(ngh_context* ctx, int16_t* dev_out, const void* dev_in, int32_t in_dtype, int64_t n,
                           float scale, const float* dev_scale, int32_t* dev_stats);

/* How stage `stage` would be launched, without a device (host-side tooling and
 * tests): out8 = {kernel family (0 streaming, 1 reduce along the contiguous axis,
 * 2 reduce across it, 3 streaming through LDS tiles for transposed operands), vector width, spec axis on kernel axes 0,1,2, tail length,
 * index of the matching pre-built specialisation or -1, reduction segments}.     */
int  ngh_plan_fused(const ngh_fused_spec* spec, int32_t stage, int32_t* out8);

/* Would ngh_launch_fused run every stage of the spec in ONE kernel -- the way the reference's
 * compound kernels run their stages one after the other inside one launch, a reduction's result
 * reaching the next stage without a trip through a second launch (float_ew2.py:1135-1483,
 * stage loop :1268-1321)?  Possible for a "row chain": rows (spec axis 0, the reduced one) of up
 * to 8192 elements, fp32 operands with unit stride along the row or broadcast along it (flex16
 * and fp16 operands too, when every row starts an even number of elements from a 4-byte-aligned
 * address; at most four flex16 tensors written), at least one reduction stage; and for a
 * "column chain": the reduced axis (spec axis 0) strided,
 * every operand contiguous along spec axis 2 in whole aligned groups of 4 floats (or broadcast
 * along it), fp32, any number of rows.  out4 = {1 for a row chain, 2 for a column chain, 0 for
 * neither; index of the compiled chain program or -1 (without one the stages are launched one
 * by one); lanes per row / column chunks per workgroup; stages}.
 * A stage of a row chain may also STORE one value per row: a value that does not vary along
 * axis 0 (computed from operands with stride 0 there, such as earlier stages' results) into a
 * tensor with stride 0 on axis 0; ngh_launch_fused refuses such a spec (NGH_E_UNSUPPORTED)
 * unless it runs as a chain.  No device needed (host-side tooling and tests).              */
int  ngh_plan_chain(const ngh_fused_spec* spec, int32_t* out4);

/* ---- flex statistics: the int32 device words FlexPtrDescription binds
 *      (float_ew2.py:363-374); replaces the manager's allocate/readback
 *      (flexgputransform.py:143-150, 361-366)                                */
int  ngh_stats_alloc(ngh_context* ctx, int32_t n, int32_t** out_dev);
int  ngh_stats_reset(ngh_context* ctx, int32_t* dev, int32_t n);
int  ngh_stats_read(ngh_context* ctx, const int32_t* dev, int32_t n, int32_t* host);

/* ---- device-resident flex exponent management -----------------------------
 * One record per flex tensor.  A fused kernel reads the tensor's scale through
 * ngh_tensor.dev_scale = &state.scale and merges max|mantissa| into
 * ngh_tensor.dev_stats = &state.stats; ngh_flex_prepare / ngh_flex_update run the
 * exponent policy on the device around a kernel, so no statistics travel to the host
 * between kernels (the reference reads them back after every kernel,
 * flexgputransform.py:361-366).  Policy: an overflow (max|mantissa| >= 32767) lowers
 * dec by 2; otherwise dec is the tightest fit of max(h) + 3 * stddev(h) over the last 16
 * recorded maxima h.  The host mirror is ngraph_hip/flex/hipflex.py.                */
#define NGH_FLEX_HISTORY 16
typedef struct ngh_flex_state {
    int32_t stats;          /* max |mantissa| merged by kernels since ngh_flex_prepare   */
    int32_t dec;            /* exponent of the data in memory: scale = 2**-dec           */
    int32_t next_dec;       /* exponent for the next full overwrite, -1 = none chosen    */
    int32_t initialized;
    float   scale;
    int32_t hist_len, hist_pos;
    int32_t last_maxabs, last_count, pad_;
    double  history[NGH_FLEX_HISTORY];   /* recent max |value|, ring buffer               */
} ngh_flex_state;

int  ngh_flex_states_alloc(ngh_context* ctx, int32_t n, ngh_flex_state** out_dev);
int  ngh_flex_states_write(ngh_context* ctx, ngh_flex_state* dev, int32_t first, int32_t n,
                           const ngh_flex_state* host);
int  ngh_flex_states_read(ngh_context* ctx, const ngh_flex_state* dev, int32_t first, int32_t n,
                          ngh_flex_state* host);     /* waits for the stream */
/* ids: up to 8 record indices; in_place[i] != 0 keeps record i's exponent (the kernel also
 * reads that tensor).  count is stored in last_count (the caller's autoflex_count).    */
int  ngh_flex_prepare(ngh_context* ctx, ngh_flex_state* dev, const int32_t* ids,
                      const int32_t* in_place, int32_t n_ids);
int  ngh_flex_update(ngh_context* ctx, ngh_flex_state* dev, const int32_t* ids, int32_t n_ids,
                     int32_t count);

/* ngh_flex_prepare + ngh_launch_fused + ngh_flex_update in one call (one host transition per
 * kernel instead of three; flexgputransform.py:347-366 is the loop it replaces).  When a
 * pre-built streaming kernel covers the spec, the library may go further and leave the
 * statistics of the launch unfolded: the next launch that writes the same tensors folds them
 * in its first instructions, and every other entry point that reads or writes a record, or
 * launches a kernel whose operands point into one, first brings it up to date.  A record read
 * through ngh_flex_states_read is therefore always current; device memory of a table must not
 * be copied out by other means while ngh_flex_unsettled reports a non-zero count.
 * A spec of several stages that runs as a row chain, every flex16 tensor it writes among `ids`,
 * is one launch as well: the chain takes the write exponents from the records and its last
 * workgroup applies the policy.                                                             */
int  ngh_launch_fused_flex(ngh_context* ctx, const ngh_fused_spec* spec, ngh_flex_state* dev,
                           const int32_t* ids, const int32_t* in_place, int32_t n_ids, int32_t count);
/* number of records whose statistics are still unfolded (no counterpart in the reference,
 * whose policy runs on the host after every kernel)                                        */
int  ngh_flex_unsettled(ngh_context* ctx, int32_t* out_count);

/* Two specs that do not depend on each other -- neither writes what the other touches; the
 * caller's knowledge -- in one call, and in ONE launch when the library has their programs built
 * as a pair: a single tiled elementwise stage and a single reduction across the contiguous axis,
 * the LSTM cell and the column sum for its bias gradient, which the reference's compound kernel
 * also has in one launch (layer.py:1630-1647, float_ew2.py:553-612).  The first workgroups of the
 * launch run one program, the rest the other.  Otherwise the same as ngh_launch_fused(a)
 * followed by ngh_launch_fused(b).  *out_one_launch (may be NULL) says which it was.         */
int  ngh_launch_fused_pair(ngh_context* ctx, const ngh_fused_spec* a, const ngh_fused_spec* b,
                           int32_t* out_one_launch);

/* ---- the launches of a computation as one HIP graph -----------------------
 * No counterpart in the reference, which launches kernel by kernel through pycuda
 * (gputransform.py:343-345, float_ew2.py:1553-1653): for computations of a few small kernels,
 * whose time is launches rather than work.  Between ngh_graph_begin and ngh_graph_end the
 * context's launches (ngh_launch_fused, ngh_copy_strided) are recorded instead of run;
 * ngh_graph_launch replays them, in the order of the context's other work.  Launches that do
 * not depend on each other may be recorded side by side so that the device may run them
 * together: ngh_graph_fork marks the point both sides start from, ngh_graph_side(1 / 0) says
 * which side the next launches belong to, ngh_graph_join (implied by fork and end) makes what
 * follows wait for both.  Whether two launches are independent is the caller's knowledge.
 * What a recorded launch was given -- addresses, constants, random-number counters -- is what
 * every replay uses: record only launches whose arguments do not change from call to call, and
 * none that allocates (a launch that ran once before with the same shapes allocates nothing; one
 * that would have to grow a buffer of the context while recording fails with NGH_E_INVALID and
 * records nothing) or waits for the device.  ngh_graph_end with out == NULL gives a capture up.
 * (Measured on an MI355X with ROCm 7.2: two 4 us kernels take 10.6 us as two launches, 18.3 us
 * as a graph of two nodes in a row, 31.4 us as two nodes side by side; the transformers record
 * graphs only when asked to.)                                                                  */
typedef struct ngh_graph ngh_graph;
int  ngh_graph_begin(ngh_context* ctx);
int  ngh_graph_fork(ngh_context* ctx);
int  ngh_graph_side(ngh_context* ctx, int32_t on);
int  ngh_graph_join(ngh_context* ctx);
int  ngh_graph_end(ngh_context* ctx, ngh_graph** out);
int  ngh_graph_launch(ngh_context* ctx, ngh_graph* graph);
int  ngh_graph_nodes(const ngh_graph* graph, int32_t* out_nodes);
int  ngh_graph_free(ngh_context* ctx, ngh_graph* graph);

/* ---- timing (HIP events on the context's stream; used by the bench) ----- */
int  ngh_timer_begin(ngh_context* ctx);
int  ngh_timer_end(ngh_context* ctx, float* out_ms);   /* waits for the stream */

#ifdef __cplusplus
}
#endif
#endif /* NGRAPH_HIP_H */
