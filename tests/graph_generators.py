"""Random graph generators shared by the parity tests: fixed seeds, shapes nobody wrote by hand
-- broadcasts over axis subsets, reordered and sliced views, reductions over several axes feeding
further elementwise ops, results shared by several consumers, sequences of assignments.  Pure
graph construction: nothing here runs a graph."""
import numpy as np

import ngraph_hip as ng

UNARY = [ng.tanh, ng.negative, ng.absolute, ng.square, ng.sigmoid, lambda x: ng.sqrt(ng.absolute(x) + 0.5),
         lambda x: ng.exp(x * 0.25), lambda x: ng.log(ng.absolute(x) + 1.0), ng.sign]


BINARY = [ng.add, ng.subtract, ng.multiply, ng.maximum, ng.minimum, lambda a, b: a / (ng.absolute(b) + 1.0),
          lambda a, b: ng.greater(a, b), lambda a, b: ng.less_equal(a, b)]


REDUCE = [ng.sum, ng.max, ng.min, ng.mean]


def build(seed):
    rs = np.random.RandomState(seed)
    n_axes = rs.randint(2, 5)
    lengths = [int(rs.choice([1, 2, 3, 5, 8, 16, 33])) for _ in range(n_axes)]
    all_axes = [ng.make_axis(n, name="ax%d_%d" % (seed, i)) for i, n in enumerate(lengths)]
    inputs, values = [], []
    for _ in range(rs.randint(2, 5)):
        k = rs.randint(1, n_axes + 1)
        idx = sorted(rs.choice(n_axes, size=k, replace=False))
        if rs.rand() < 0.4:
            idx = list(rs.permutation(idx))                       # stored in another axis order
        axes = [all_axes[i] for i in idx]
        inputs.append(ng.placeholder(axes))
        values.append(rs.uniform(-2, 2, [a.length for a in axes]).astype(np.float32))
    pool = list(inputs)
    for _ in range(rs.randint(4, 14)):
        kind = rs.rand()
        if kind < 0.35:
            x = pool[rs.randint(len(pool))]
            node = UNARY[rs.randint(len(UNARY))](x)
        elif kind < 0.8:
            a, b = pool[rs.randint(len(pool))], pool[rs.randint(len(pool))]
            node = BINARY[rs.randint(len(BINARY))](a, b)
        else:
            x = pool[rs.randint(len(pool))]
            if len(x.axes) == 0:
                continue
            k = rs.randint(1, len(x.axes) + 1)
            red = [x.axes[i] for i in sorted(rs.choice(len(x.axes), size=k, replace=False))]
            node = REDUCE[rs.randint(len(REDUCE))](x, reduction_axes=ng.make_axes(red))
        pool.append(node)
    results = [pool[-1]] + [pool[i] for i in rs.choice(np.arange(len(inputs), len(pool)), size=min(2, len(pool) - len(inputs)),
                                                       replace=False)]
    return results, inputs, values


# ------------------------------------------------------------------ second generator: larger shapes, views
def build_views(seed):
    """Larger tensors (vector, tiled and multi-segment kernels get chosen), up to five axes (the
    host loops over what does not fit three), sliced and reordered views as operands, argmax /
    prod reductions with explicit out_axes orders."""
    rs = np.random.RandomState(seed)
    n_axes = rs.randint(2, 6)
    lengths = [int(rs.choice([1, 2, 3, 4, 8, 16, 32, 64, 100])) for _ in range(n_axes)]
    while np.prod(lengths) > 400000:
        lengths[int(np.argmax(lengths))] //= 2
    all_axes = [ng.make_axis(n, name="bx%d_%d" % (seed, i)) for i, n in enumerate(lengths)]
    inputs, values, pool = [], [], []
    for _ in range(rs.randint(2, 4)):
        k = rs.randint(max(1, n_axes - 2), n_axes + 1)
        idx = list(rs.permutation(n_axes)[:k]) if rs.rand() < 0.5 else sorted(rs.choice(n_axes, size=k, replace=False))
        axes = [all_axes[i] for i in idx]
        p = ng.placeholder(axes)
        inputs.append(p)
        values.append(rs.uniform(-2, 2, [a.length for a in axes]).astype(np.float32))
        view = p
        if rs.rand() < 0.5 and len(axes) > 1:
            view = ng.axes_with_order(view, [axes[i] for i in rs.permutation(len(axes))])
        pool.append(view)
    # a sliced operand: a window of the first input along its first axis, renamed so it can
    # only meet operands through its other axes
    first = inputs[0]
    if first.axes[0].length >= 4:
        lo = int(rs.randint(0, first.axes[0].length // 2))
        hi = int(rs.randint(lo + 1, first.axes[0].length + 1))
        sl = ng.tensor_slice(first, [slice(lo, hi)] + [slice(None)] * (len(first.axes) - 1))
        pool.append(ng.sum(sl, reduction_axes=ng.make_axes([sl.axes[0]])) if len(sl.axes) > 1 else ng.sum(sl))
    for _ in range(rs.randint(5, 12)):
        kind = rs.rand()
        if kind < 0.3:
            node = UNARY[rs.randint(len(UNARY))](pool[rs.randint(len(pool))])
        elif kind < 0.75:
            node = BINARY[rs.randint(len(BINARY))](pool[rs.randint(len(pool))], pool[rs.randint(len(pool))])
        else:
            x = pool[rs.randint(len(pool))]
            if len(x.axes) == 0:
                continue
            which = rs.rand()
            if which < 0.25:
                node = ng.argmax(x, reduction_axes=ng.make_axes([x.axes[rs.randint(len(x.axes))]]))
            elif which < 0.4:
                node = ng.prod(x * 0.5, reduction_axes=ng.make_axes([x.axes[rs.randint(len(x.axes))]]))
            else:
                k = rs.randint(1, len(x.axes) + 1)
                red = [x.axes[i] for i in sorted(rs.choice(len(x.axes), size=k, replace=False))]
                kept = [a for a in x.axes if a not in red]
                out_axes = [kept[i] for i in rs.permutation(len(kept))]
                node = REDUCE[rs.randint(len(REDUCE))](x, out_axes=ng.make_axes(out_axes))
        pool.append(node)
    n_in = len(inputs)
    picks = rs.choice(np.arange(n_in, len(pool)), size=min(3, len(pool) - n_in), replace=False)
    return [pool[-1]] + [pool[i] for i in picks], inputs, values


# ------------------------------------------------------------------ third generator: state
def build_state(seed):
    """Sequences of assignments to a few variables (whole tensors and row windows), each value an
    expression of the variables' current contents and an input: in-place updates, reads after
    writes, writes after reads -- what the planner's hazard rules exist for."""
    rs = np.random.RandomState(seed)
    A = ng.make_axis(int(rs.choice([4, 16, 33])), name="sa%d" % seed)
    B = ng.make_axis(int(rs.choice([8, 64, 100])), name="sb%d" % seed)
    init = [rs.uniform(-1, 1, (A.length, B.length)).astype(np.float32) for _ in range(3)]
    variables = [ng.variable([A, B], initial_value=v) for v in init]
    x = ng.placeholder([A, B])
    xv = rs.uniform(-1, 1, (A.length, B.length)).astype(np.float32)

    def expr(depth=0):
        if depth > 2 or rs.rand() < 0.3:
            return variables[rs.randint(3)] if rs.rand() < 0.7 else x
        if rs.rand() < 0.4:
            return [ng.tanh, ng.negative, ng.absolute, lambda t: t * 0.5][rs.randint(4)](expr(depth + 1))
        return [ng.add, ng.subtract, ng.multiply, ng.maximum][rs.randint(4)](expr(depth + 1), expr(depth + 1))

    steps = []
    for _ in range(rs.randint(3, 9)):
        target = variables[rs.randint(3)]
        value = expr()
        if not hasattr(value, "axes") or len(value.axes) != 2:
            continue
        if rs.rand() < 0.3 and A.length >= 4:
            lo = int(rs.randint(0, A.length - 2))
            hi = int(rs.randint(lo + 1, A.length + 1))
            window = [slice(lo, hi), slice(None)]
            tgt = ng.tensor_slice(target, window)
            val = ng.cast_axes(ng.tensor_slice(value, window), tgt.axes)
            steps.append(ng.assign(tgt, val))
        else:
            steps.append(ng.assign(target, value))
    total = ng.sum(variables[0] + variables[1] * 2.0 + variables[2] * 3.0, out_axes=())
    return ng.sequential(steps + [total]), variables, x, xv
