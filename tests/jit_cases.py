"""Graphs whose kernels the tests of run-time compiled programs (test_jit.py) compile.

`precompile()` lowers every case without a device and compiles its program libraries into the
cache, so that a build on a machine without a GPU leaves nothing to compile for the GPU tests
(they compile on the spot if the cache lacks a library).
"""
import numpy as np

import ngraph_hip as ng
import ngraph_hip.transformers as ngt


def _ab(a=512, b=1024):
    return ng.make_axis(a, name="A"), ng.make_axis(b, name="B")


def case_elementwise():
    A, B = _ab()
    x, y, w = ng.placeholder([A, B]), ng.placeholder([A, B]), ng.placeholder([A, B])
    z = ng.tanh(x * y + 0.5) / (ng.absolute(y) + 1.0)
    return [z * w, ng.maximum(z, w) - x], [x, y, w]


def case_column_reduction_with_store():
    A, B = _ab()
    x, y = ng.placeholder([A, B]), ng.placeholder([A, B])
    z = ng.tanh(x * y + 0.5) / (ng.absolute(y) + 1.0)
    return [z, ng.max(z, out_axes=[B]), ng.argmax(z * x, out_axes=[B])], [x, y]


def case_row_reduction_with_store():
    A, B = _ab()
    x, y = ng.placeholder([A, B]), ng.placeholder([A, B])
    z = ng.sqrt(ng.absolute(x * y) + 0.25)
    return [z, ng.sum(z * z, out_axes=[A]), ng.min(z, out_axes=[A])], [x, y]


def case_transposed_operand():
    A, B = _ab()
    xs, x, y = ng.placeholder([B, A]), ng.placeholder([A, B]), ng.placeholder([A, B])
    return [ng.sigmoid(ng.axes_with_order(xs, [A, B]) * x) + y], [xs, x, y]


def case_transposed_operands_large():
    # enough 64 x 64 tiles for the compiled tiled program to take 16-byte accesses, with ragged
    # tiles at both edges (2052 = 32 * 64 + 4); a transposed fp32 operand, a transposed fp16
    # operand, and a result assigned through a transposed view of a variable
    A, B = ng.make_axis(2052, name="A"), ng.make_axis(2056, name="B")
    xs, hs = ng.placeholder([B, A]), ng.placeholder([B, A], dtype=np.float16)
    y = ng.placeholder([A, B])
    v = ng.variable([B, A], initial_value=0)
    z = ng.tanh(ng.axes_with_order(xs, [A, B]) * y) + ng.axes_with_order(hs, [A, B])
    return [ng.sequential([ng.assign(ng.axes_with_order(v, [A, B]), z * 0.5), z]), v * 1.0], [xs, hs, y]


def case_softmax():
    A, B = _ab()
    x = ng.placeholder([A, B])
    e = ng.exp(x - ng.max(x, out_axes=[A]))
    return [e / ng.sum(e, out_axes=[A])], [x]


def case_mixed_storage_types():
    A, B = _ab()
    x, h = ng.placeholder([A, B]), ng.placeholder([A, B], dtype=np.float16)
    i = ng.placeholder([A, B], dtype=np.int32)
    return [ng.minimum(x * h, 4.0) + i, ng.sum(h * x, out_axes=[B])], [x, h, i]


def case_integer_arithmetic():
    # int32 operands meeting each other: integer ops on the registers' bits, conversions as ops
    # of the program, the integer tensors bound so that loads and stores move bits
    A, B = _ab()
    i, j = ng.placeholder([A, B], dtype=np.int32), ng.placeholder([A, B], dtype=np.int32)
    x = ng.placeholder([A, B])
    k = ng.add(ng.multiply(i, j, dtype=np.int32), j, dtype=np.int32)
    return [k, ng.maximum(i, j) * x + ng.less(i, j), ng.sum(ng.subtract(i, j, dtype=np.int32), out_axes=[B])], [i, j, x]


def case_ragged():
    # extents that leave a tail after the vector-wide part and rows that are not a multiple of 4
    A, B = ng.make_axis(301, name="A"), ng.make_axis(77, name="B")
    x, y = ng.placeholder([A, B]), ng.placeholder([A, B])
    return [ng.exp(-ng.square(x)) * y + 1.0, ng.sum(x * y + 1.0, out_axes=[A])], [x, y]


def case_ragged_long_rows():
    # rows of 9001 elements (too long for a row chain): 4 elements per lane with a short last
    # chunk per row, a workgroup per row segment in the elementwise pass and per row in the reductions
    A, B = ng.make_axis(37, name="A"), ng.make_axis(9001, name="B")
    x, y = ng.placeholder([A, B]), ng.placeholder([A, B])
    return [ng.tanh(x * y) + x, ng.sum(x * y + 1.0, out_axes=[A]), ng.max(x - y, out_axes=[A]),
            ng.argmax(x + y, out_axes=[A])], [x, y]


def case_ragged_many_rows():
    # many rows of 1001: a wavefront per row
    C, N = ng.make_axis(1001, name="C"), ng.make_axis(4200, name="N")
    x = ng.placeholder([N, C])
    return [ng.sum(ng.exp(x) * 0.5, out_axes=[N])], [x]


def case_softmax_ragged_rows():
    # a softmax over many rows of 1001: its three kernels become the stages of one row chain
    C, N = ng.make_axis(1001, name="C"), ng.make_axis(4200, name="N")
    x = ng.placeholder([N, C])
    e = ng.exp(x - ng.max(x, out_axes=[N]))
    return [e / ng.sum(e, out_axes=[N])], [x]


def case_softmax_of_half_rows():
    # 16-bit storage in a row chain: fp16 operand and result, the row's maximum an fp16 tensor
    # too (rounded for its tensor and handed on in a register as a load would return it), the
    # sum fp32; rows of 1002 elements (a row starts on a 4-byte boundary, not on an 8-byte one)
    C, N = ng.make_axis(1002, name="C"), ng.make_axis(1200, name="N")
    x = ng.placeholder([N, C], dtype=np.float16)
    m = ng.max(x * 3.3, out_axes=[N], dtype=np.float16)
    e = ng.exp(x * 3.3 - m)
    return [ng.divide(e, ng.sum(e, out_axes=[N]), dtype=np.float16), m], [x]


def case_softmax_long_rows():
    # rows of 4099 and of 8192 elements: a workgroup per row in the chain kernel
    C, N, C2 = ng.make_axis(4099, name="C"), ng.make_axis(300, name="N"), ng.make_axis(8192, name="C2")
    x, x2 = ng.placeholder([N, C]), ng.placeholder([N, C2])
    e = ng.exp(x - ng.max(x, out_axes=[N]))
    e2 = ng.exp(x2 - ng.max(x2, out_axes=[N]))
    return [e / ng.sum(e, out_axes=[N]), e2 / ng.sum(e2, out_axes=[N]), ng.argmax(x2, out_axes=[N])], [x, x2]


def case_softmax_over_windows():
    # rows inside a window of a larger tensor: two kept axes that do not merge into one, rows that
    # start anywhere, a result written into a window as well
    A, B, C = ng.make_axis(37, name="A"), ng.make_axis(60, name="B"), ng.make_axis(310, name="C")
    x = ng.placeholder([A, B, C])
    xs = ng.tensor_slice(x, [slice(None), slice(5, 55), slice(3, 303)])
    e = ng.exp(xs - ng.max(xs, reduction_axes=xs.axes[2:]))
    return [e / ng.sum(e, reduction_axes=xs.axes[2:]), ng.argmax(xs, reduction_axes=xs.axes[2:])], [x]


def case_softmax_forward_and_backward():
    # a softmax and the derivative of a loss through it: five kernels over the same rows, one chain
    C, N = ng.make_axis(500, name="C"), ng.make_axis(3000, name="N")
    x, tgt = ng.placeholder([N, C]), ng.placeholder([N, C])
    e = ng.exp(x - ng.max(x, out_axes=[N]))
    y = e / ng.sum(e, out_axes=[N])
    return [y, ng.deriv(ng.sum(y * tgt, out_axes=()), x)], [x, tgt]


def case_row_chain_with_stored_intermediate():
    # log-softmax and the row norms of the same tensor: two results, reductions of different
    # kinds, an intermediate that is stored by one stage and read back by the next
    C, N = ng.make_axis(300, name="C"), ng.make_axis(5000, name="N")
    x = ng.placeholder([N, C])
    shifted = x - ng.max(x, out_axes=[N])
    logp = shifted - ng.log(ng.sum(ng.exp(shifted), out_axes=[N]))
    return [logp, ng.sqrt(ng.sum(logp * logp, out_axes=[N])), shifted], [x]


def case_misaligned_slices():
    # windows that start one element into rows of odd length: no vector access, so the
    # compiled program takes one element per lane with the operands' own strides
    A, B = ng.make_axis(300, name="A"), ng.make_axis(1025, name="B")
    x, y = ng.placeholder([A, B]), ng.placeholder([A, B])
    xs = ng.tensor_slice(x, [slice(None), slice(1, 1025)])
    ys = ng.cast_axes(ng.tensor_slice(y, [slice(None), slice(0, 1024)]), xs.axes)
    return [ng.tanh(xs * ys + 0.5) * ng.sigmoid(xs)], [x, y]


def case_short_rows():
    # softmax and its cross entropy over 100 classes: rows short enough that several share a
    # workgroup (the short-row reduction kernel)
    C, N = ng.make_axis(100, name="C"), ng.make_axis(2048, name="N")
    x, tgt = ng.placeholder([N, C]), ng.placeholder([N, C])
    e = ng.exp(x - ng.max(x, out_axes=[N]))
    sm = e / ng.sum(e, out_axes=[N])
    return [sm, ng.sum(-tgt * ng.log(sm), out_axes=[N]), ng.argmax(x, out_axes=[N])], [x, tgt]


def case_dropout():
    # a random mask made in the kernel (Philox keyed by seed, execution count and element
    # index): the compiled program must draw the very numbers the interpreter draws
    A, B = _ab()
    x = ng.placeholder([A, B])
    keep = ng.less_equal(ng.uniform(ng.temporary([A, B]), 0.0, 1.0), 0.75)
    return [x * keep * (1.0 / 0.75), ng.sum(keep, out_axes=[A])], [x]


def case_lookup_table():
    # rows of a table selected by an index tensor (LookupTableOp fprop), scaled afterwards
    V_, F, N = ng.make_axis(1000, name="V"), ng.make_axis(64, name="F"), ng.make_axis(256, name="N")
    lut, idx = ng.placeholder([V_, F]), ng.placeholder([N], dtype=np.int32)
    w = ng.placeholder([N, F])
    return [ng.lookuptable(lut, idx, ng.make_axes([N, F]), update=False) * w + 1.0], [lut, idx, w]


def case_softmax_over_classes():
    # classes x samples, the layout of the neon front end: the reduced axis is the strided one.
    # Its three kernels become the stages of one column chain; 300 rows: row lanes share a
    # column chunk and meet in LDS, and every stage streams x again
    A, B = ng.make_axis(300, name="A"), ng.make_axis(2048, name="B")
    x = ng.placeholder([A, B])
    e = ng.exp(x - ng.max(x, out_axes=[B]))
    return [e / ng.sum(e, out_axes=[B])], [x]


def case_softmax_over_few_classes():
    # 10 classes: a lane walks all rows of its four columns and keeps them in registers
    A, B = ng.make_axis(10, name="A"), ng.make_axis(65536, name="B")
    x = ng.placeholder([A, B])
    e = ng.exp(x - ng.max(x, out_axes=[B]))
    return [e / ng.sum(e, out_axes=[B]), ng.argmax(x, out_axes=[B])], [x]


def case_softmax_over_ten_classes_of_many_samples():
    # columns enough to fill the chip with workgroups 256 chunks wide: a lane owns its four
    # columns outright, all ten rows in registers, no folds between lanes
    A, B = ng.make_axis(10, name="A"), ng.make_axis(786432, name="B")
    x = ng.placeholder([A, B])
    e = ng.exp(x - ng.max(x, out_axes=[B]))
    return [e / ng.sum(e, out_axes=[B])], [x]


def case_column_statistics_chain():
    # batch statistics over the leading (strided) axis feeding a normalisation, with an outer axis
    N, C, F = ng.make_axis(64, name="N"), ng.make_axis(6, name="C"), ng.make_axis(1024, name="F")
    x, g = ng.placeholder([N, C, F]), ng.placeholder([C, F])
    mean = ng.sum(x, out_axes=[C, F]) * (1.0 / 64)
    d = x - mean
    var = ng.sum(d * d, out_axes=[C, F]) * (1.0 / 64)
    return [d * ng.reciprocal(ng.sqrt(var + 1e-3)) * g], [x, g]


def case_row_statistics_chain():
    # mean and variance of every row feeding a consumer: one moments kernel (one-pass variance)
    # plus a kernel for the consumer while interpreted, one row chain (sum, then the sum of
    # squared differences) once compiled -- two ways to the same statistics
    A, B = ng.make_axis(3000, name="A"), ng.make_axis(1000, name="B")
    x, g = ng.placeholder([A, B]), ng.placeholder([B])
    mean, var = ng.mean(x, out_axes=[A]), ng.variance(x, out_axes=[A])
    return [ng.tanh((x - mean) * ng.reciprocal(ng.sqrt(var + 1e-3))) * g + mean], [x, g]


FP32_CASES = [case_elementwise, case_column_reduction_with_store, case_row_reduction_with_store,
              case_transposed_operand, case_transposed_operands_large, case_softmax, case_mixed_storage_types,
              case_integer_arithmetic, case_ragged,
              case_ragged_long_rows, case_ragged_many_rows, case_softmax_ragged_rows, case_softmax_of_half_rows, case_softmax_long_rows, case_softmax_over_windows,
              case_softmax_forward_and_backward,
              case_row_chain_with_stored_intermediate, case_misaligned_slices, case_short_rows, case_dropout, case_lookup_table,
              case_row_statistics_chain, case_softmax_over_classes, case_softmax_over_few_classes,
              case_softmax_over_ten_classes_of_many_samples, case_column_statistics_chain]


def flex_case():
    P = ng.make_axis(1 << 16, name="P")
    x, w, b = ng.placeholder([P]), ng.placeholder([P]), ng.placeholder([P])
    return [ng.tanh(x * w) + b], [x, w, b]


# random graphs of tests/graph_generators.py: small shapes, so every stage counts as worth
# compiling (jit_min_elements=1); the odd programs a generator finds and a person would not write
RANDOM_SEEDS = list(range(8))


def random_case(seed, views):
    import graph_generators as T
    return (T.build_views if views else T.build)(seed)


def inputs_for(placeholders, seed):
    vals = []
    for i, p in enumerate(placeholders):
        rs = np.random.RandomState(seed + i)
        if p.dtype == np.int32:
            hi = 1000 if len(p.axes) == 1 else 6          # an index tensor / integer operands
            vals.append(rs.randint(0 if len(p.axes) == 1 else -5, hi, p.axes.lengths).astype(np.int32))
        else:
            vals.append(rs.uniform(-1, 1, p.axes.lengths).astype(p.dtype))
    return vals


def precompile(verbose=False):
    """Compile the program libraries of every case (no device needed); returns their paths."""
    from ngraph_hip.runtime import jit
    builders = [("hipgpu", case, {}) for case in FP32_CASES] + [("flexhip", flex_case, {})]
    for seed in RANDOM_SEEDS:
        for views in (False, True):
            builders.append(("hipgpu", lambda seed=seed, views=views: random_case(seed, views),
                             {"jit_min_elements": 1}))
    return jit.precompile_graphs(builders, verbose=verbose)
