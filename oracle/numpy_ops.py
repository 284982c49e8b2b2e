"""The NumPy call behind every op, as the reference CPU transformer emits it.

Oracle (test infrastructure).  One entry per `generate_op` overload of
ngraph/transformers/cputransform.py:512-761; the Add overload goes through
mkldnn.elementwise_add, whose fallback without MKL-DNN is np.add
(ngraph/transformers/cpu/cpuengine.py:353-360).  All buffers are float32
(cputransform.py:998-1007), so every call is made on float32 operands with a
float32 `out`.
"""
import numpy as np

f32 = np.float32


def _out(shape):
    return np.empty(shape, dtype=f32)


UNARY = {
    "abs": np.abs,                 # cputransform.py:512-514
    "neg": np.negative,            # :694-696
    "sqrt": np.sqrt,               # :735-737
    "sqr": np.square,              # :739-741
    "exp": np.exp,                 # :642-644
    "log": np.log,                 # :666-668
    "rcp": np.reciprocal,          # :719-721
    "tanh": np.tanh,               # :755-757
    "sgn": np.sign,                # :727-729
    "sin": np.sin,                 # :731-733
    "cos": np.cos,                 # :589-591
    "exp2": np.exp2,               # float_ew2.py:41 (no CPU overload; NumPy ufunc of the same name)
    "log2": np.log2,               # float_ew2.py:42
    "assign": lambda x, out: np.copyto(out, x),
}

BINARY = {
    "add": np.add,                 # :516-519 -> cpuengine.py:353-360
    "sub": np.subtract,            # :743-745
    "mul": np.multiply,            # :690-692
    "div": np.divide,              # :599-601
    "int_div": np.floor_divide,    # :603-605
    "mod": np.mod,                 # :607-609
    "pow": np.power,               # :706-708
    "minimum": np.minimum,         # :682-684
    "maximum": np.maximum,         # :674-676
    "eq": np.equal,                # :638-640
    "ne": np.not_equal,            # :698-700
    "lt": np.less,                 # :658-660
    "le": np.less_equal,           # :662-664
    "gt": np.greater,              # :650-652
    "ge": np.greater_equal,        # :654-656
}

REDUCE = {
    "sum": np.sum,                 # :747-749
    "prod": np.prod,               # :751-753
    "max": np.max,                 # :670-672
    "min": np.min,                 # :678-680
}


def unary(name, x):
    x = np.asarray(x, dtype=f32)
    out = _out(x.shape)
    if name == "sig":
        # SigmoidAtomicOp has no CPU overload; the graph-level sigmoid is the
        # composite reciprocal(exp(-x) + 1) (op_graph.py:4183-4197)
        t = _out(x.shape)
        np.negative(x, out=t)
        np.exp(t, out=t)
        np.add(t, f32(1), out=t)
        np.reciprocal(t, out=out)
        return out
    if name == "safelog":
        # the kernel template of float_ew2.py:48, (x > 0) ? logf(x) : -50.  The graph-level
        # ng.safelog is a composite of other ops, maximum(log(x + exp(limit)), limit)
        # (op_graph.py:3070-3072), and never reaches this template.
        with np.errstate(all="ignore"):
            np.log(x, out=out)
        out[~(x > 0)] = f32(-50.0)
        return out
    with np.errstate(all="ignore"):
        if name == "assign":
            np.copyto(out, x)
        else:
            UNARY[name](x, out=out)
    return out


def binary(name, x, y):
    x = np.asarray(x, dtype=f32)
    y = np.asarray(y, dtype=f32)
    out = _out(np.broadcast(x, y).shape)
    with np.errstate(all="ignore"):
        BINARY[name](x, y, out=out)   # comparisons write 0.0 / 1.0 into the float32 out
    return out


# Integer operands: the CPU transformer hands int32 / uint32 arrays to the same ufuncs
# (cputransform.py:512-761), and NumPy then runs its integer loop (exact, wrapping at 2^32)
# and casts the result to `out`'s type; the GPU transformer keeps such operands in `int` /
# `unsigned int` registers (float_ew2.py:615-641).  Names are the device library's: a
# leading "i" reads int32, "u" uint32.
INTEGER_UNARY = {
    "i2f": (np.int32, lambda x: x.astype(f32)),
    "u2f": (np.uint32, lambda x: x.astype(f32)),
    "ineg": (np.int32, np.negative),           # :694-696
    "iabs": (np.int32, np.abs),                # :512-514
}

INTEGER_BINARY = {
    "iadd": (np.int32, np.add), "isub": (np.int32, np.subtract), "imul": (np.int32, np.multiply),
    "imin": (np.int32, np.minimum), "imax": (np.int32, np.maximum),
    "umin": (np.uint32, np.minimum), "umax": (np.uint32, np.maximum),
    "ieq": (np.int32, np.equal), "ine": (np.int32, np.not_equal),
    "ilt": (np.int32, np.less), "ile": (np.int32, np.less_equal),
    "igt": (np.int32, np.greater), "ige": (np.int32, np.greater_equal),
    "ult": (np.uint32, np.less), "ule": (np.uint32, np.less_equal),
    "ugt": (np.uint32, np.greater), "uge": (np.uint32, np.greater_equal),
}


def integer_unary(name, x):
    """`x` holds 32-bit patterns (any 4-byte dtype); the result has the integer type of the op,
    float32 for the conversions."""
    kind, fn = INTEGER_UNARY[name]
    with np.errstate(all="ignore"):
        return fn(np.asarray(x).view(kind))


def integer_binary(name, x, y):
    """As `integer_unary`; comparisons return 0.0 / 1.0 in float32 like `binary`."""
    kind, fn = INTEGER_BINARY[name]
    with np.errstate(all="ignore"):
        r = fn(np.asarray(x).view(kind), np.asarray(y).view(kind))
    return r.astype(f32) if r.dtype == np.bool_ else r


def reduce(name, x, axis):
    x = np.asarray(x, dtype=f32)
    with np.errstate(all="ignore"):
        if name == "argmax":
            return np.ndarray.argmax(x, axis=axis)      # :521-523
        if name == "argmin":
            return np.ndarray.argmin(x, axis=axis)      # :525-527
        shape = tuple(s for i, s in enumerate(x.shape)
                      if i not in ((axis,) if isinstance(axis, int) else tuple(axis)))
        out = _out(shape)
        REDUCE[name](x, axis=axis, out=out)
        return out


def onehot(x, n_classes):
    # cputransform.py:702-704: o[:] = np.eye(o.shape[0])[:, x.astype(np.int32)]
    x = np.asarray(x)
    return np.eye(n_classes)[:, x.astype(np.int32)].astype(f32)
