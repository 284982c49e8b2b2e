"""The oracle's integer ops against arithmetic on Python integers.

NumPy's integer loops are what the CPU transformer runs on int32 / uint32 operands
(cputransform.py:512-761); that they are two's-complement arithmetic modulo 2^32 is pinned
here against unbounded Python integers reduced by hand, so that a wrong view, a swapped
signedness or a saturating variant would show.
"""
import operator

import numpy as np
import pytest

from oracle import numpy_ops

M = 1 << 32


def _signed(v):
    v %= M
    return v - M if v >= (1 << 31) else v


def _patterns(seed, n):
    rs = np.random.RandomState(seed)
    x = rs.randint(0, M, n, dtype=np.uint64).astype(np.uint32)
    x[:8] = [0, 1, 0x7fffffff, 0x80000000, 0xffffffff, 0x80000001, 1 << 24, (1 << 24) + 1]
    return x


_ARITH = {"add": operator.add, "sub": operator.sub, "mul": operator.mul, "min": min, "max": max}
_CMP = {"eq": operator.eq, "ne": operator.ne, "lt": operator.lt, "le": operator.le, "gt": operator.gt,
        "ge": operator.ge}


@pytest.mark.parametrize("name", sorted(numpy_ops.INTEGER_BINARY))
def test_integer_binary_is_arithmetic_modulo_two_to_the_32(name):
    x, y = _patterns(1, 600), _patterns(2, 600)[::-1].copy()
    y[::4] = x[::4]
    got = numpy_ops.integer_binary(name, x, y)
    read = _signed if name[0] == "i" else (lambda v: v % M)
    want = []
    for a, b in zip(x.tolist(), y.tolist()):
        a, b = read(a), read(b)
        if name[1:] in _ARITH:
            want.append(_ARITH[name[1:]](a, b) % M)
        else:
            want.append(1.0 if _CMP[name[1:]](a, b) else 0.0)
    if name[1:] in _ARITH:
        assert got.dtype.itemsize == 4 and got.dtype.kind in "iu"
        assert got.view(np.uint32).tolist() == want
    else:
        assert got.dtype == np.float32
        assert got.tolist() == want


@pytest.mark.parametrize("name", sorted(numpy_ops.INTEGER_UNARY))
def test_integer_unary_against_python_integers(name):
    x = _patterns(3, 600)
    got = numpy_ops.integer_unary(name, x)
    vals = x.tolist()
    if name == "ineg":
        assert got.view(np.uint32).tolist() == [(-_signed(v)) % M for v in vals]
    elif name == "iabs":
        assert got.view(np.uint32).tolist() == [abs(_signed(v)) % M for v in vals]      # |INT_MIN| wraps to itself
    else:
        read = _signed if name == "i2f" else (lambda v: v)
        assert got.dtype == np.float32
        # float(int) rounds to nearest even in float64 exactly (|v| < 2^53); float32 of that is one rounding
        assert got.tolist() == [float(np.float32(float(read(v)))) for v in vals]
