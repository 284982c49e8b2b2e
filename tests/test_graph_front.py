"""The slice of the `ngraph` graph front that drives the fused path: axes algebra, views, state
and execution protocol, checked the way the reference's own tests check them.

Sources of the behaviours and of the known-answer tables (data only, retyped as names and
numbers): tests/test_axes.py:24-130 and :273-327 (axes algebra, sliced axes),
tests/test_op_graph.py:84-117 (slices keep names, numpy-like slicing),
tests/transformer_dependent/test_ssa.py:23-83 (state), test_dimshuffle_op.py:28-153
(permutation vectors), test_constant.py:28-150 (constants),
test_op_graph_transformer_dependent.py:61-160, 201-250 (sequential, initial values, several
computations of one value), test_transformer.py:54-82 (argument checks),
test_axes_transformer_dependent.py:120-134 (scalar broadcast).
"""
import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.op_graph.axes import TensorDescription, slice_axis
from ngraph_hip.testing import executor
import oracle.cpu_transformer  # noqa: F401  registers "cpu"

BACKENDS = ["cpu", pytest.param("hipgpu", marks=pytest.mark.gpu),
            pytest.param("hipgpu-nofuse", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def backend(request):
    name = request.param
    factory = (ngt.make_transformer_factory("hipgpu", fusion=False) if name == "hipgpu-nofuse"
               else ngt.make_transformer_factory(name))
    ngt.set_transformer_factory(factory)
    yield name
    ngt.set_transformer_factory(None)


# ---- axes algebra --------------------------------------------------------------------------
_LEN = {"A": 2, "B": 3, "C": 4, "A_": 5, "B_": 6, "C_": 7}     # X_ has X's name, another length


def _axes(names):
    return ng.make_axes([ng.make_axis(_LEN[n], name=n.rstrip("_")) for n in names])


# (operation, left, right, expected): expected is a list of names, a truth value, or ValueError
AXES_OPS = [
    ("__add__", [], [], []), ("__add__", ["A"], [], ["A"]), ("__add__", ["A_"], [], ["A"]),
    ("__add__", ["A"], ["B"], ["A", "B"]), ("__add__", ["A_"], ["B_"], ["A", "B"]),
    ("__add__", ["A"], ["A"], ValueError), ("__add__", ["A"], ["A_"], ValueError),
    ("__add__", ["A"], ["A_", "B"], ValueError),
    ("__sub__", [], [], []), ("__sub__", [], ["A"], []), ("__sub__", ["A"], [], ["A"]),
    ("__sub__", ["A", "B"], ["B"], ["A"]), ("__sub__", ["A", "B"], ["B_"], ["A"]),
    ("__sub__", ["A", "B"], ["A"], ["B"]), ("__sub__", ["A", "B"], ["A_"], ["B"]),
    ("__sub__", ["A", "B"], ["B", "A"], []), ("__sub__", ["A", "B"], ["B_", "A_"], []),
    ("__or__", [], [], []), ("__or__", [], ["A"], ["A"]), ("__or__", ["A"], [], ["A"]),
    ("__or__", ["A"], ["B"], ["A", "B"]), ("__or__", ["A"], ["A_"], ["A"]),
    ("__and__", [], [], []), ("__and__", [], ["A"], []), ("__and__", ["A"], [], []),
    ("__and__", ["A"], ["B"], []), ("__and__", ["A", "B"], ["B", "C"], ["B"]),
    ("__and__", ["A", "B_"], ["B", "C"], ["B"]),
    ("__eq__", [], [], True), ("__eq__", ["A"], [], False), ("__eq__", ["A", "B"], ["B", "A"], False),
    ("__eq__", ["A", "B"], ["B_", "A_"], False), ("__eq__", ["A", "B"], ["A_", "B"], True),
    ("__eq__", ["A", "B"], ["A_", "B_"], True),
    ("__ne__", [], [], False), ("__ne__", ["A"], [], True), ("__ne__", ["A", "B"], ["B", "A"], True),
    ("__ne__", ["A", "B"], ["A_", "B_"], False),
    ("is_sub_set", [], [], True), ("is_sub_set", ["A"], [], False), ("is_sub_set", [], ["A"], True),
    ("is_sub_set", ["A_"], ["A"], True), ("is_sub_set", ["A", "B"], ["B", "A"], True),
    ("is_sub_set", ["A", "B"], ["B_", "A_"], True),
    ("is_super_set", [], [], True), ("is_super_set", ["A"], [], True), ("is_super_set", [], ["A"], False),
    ("is_super_set", ["A_"], ["A"], True), ("is_super_set", ["A", "B"], ["B", "A"], True),
    ("is_super_set", ["A"], ["B_", "A_"], False),
    ("is_equal_set", [], [], True), ("is_equal_set", ["A"], [], False), ("is_equal_set", ["A"], ["A"], True),
    ("is_equal_set", ["A"], ["A_"], True), ("is_equal_set", ["A", "B"], ["B_", "A_"], True),
    ("is_not_equal_set", [], [], False), ("is_not_equal_set", ["A"], [], True),
    ("is_not_equal_set", ["A"], ["A_"], False), ("is_not_equal_set", ["A", "B"], ["B_", "A_"], False),
]


@pytest.mark.parametrize("op,lhs,rhs,want", AXES_OPS)
def test_axes_ops(op, lhs, rhs, want):
    left, right = _axes(lhs), _axes(rhs)
    if want is ValueError:
        with pytest.raises(ValueError):
            getattr(left, op)(right)
        return
    got = getattr(left, op)(right)
    if isinstance(want, list):
        assert got == _axes(want), (op, lhs, rhs, got)
    else:
        assert bool(got) is want, (op, lhs, rhs, got)


def test_axis_equality_is_by_name_and_duplicates_are_refused():
    assert ng.make_axis(3, name="N") == ng.make_axis(5, name="N")
    assert ng.make_axis(3, name="N") != ng.make_axis(3, name="M")
    with pytest.raises(ValueError):
        ng.make_axes([ng.make_axis(name="X"), ng.make_axis(name="X")])
    with pytest.raises(ValueError) as e:
        ng.make_axes([ng.make_axis(1, name="N"), ng.make_axis(2, name="N")])
    assert "N" in str(e.value)
    a, b = ng.make_axis(2), ng.make_axis(2)              # unnamed axes get distinct names
    assert a != b and a.name != b.name


@pytest.mark.parametrize("s,length", [(slice(0, 5), 5), (slice(5, 0), 0), (slice(0, None), 10),
                                      (slice(5, 0, -1), 5), (slice(0, 5, -1), 0), (slice(None, None, -1), 10)])
def test_sliced_axis_lengths(s, length):
    assert slice_axis(ng.make_axis(10), s).length == length


def test_sliced_axis_roles_and_steps():
    with pytest.raises(ValueError):
        slice_axis(ng.make_axis(10), slice(0, 5, 2))
    assert slice_axis(ng.make_axis(10, name="N"), slice(0, 5)).is_batch is True
    assert slice_axis(ng.make_axis(10, name="REC"), slice(0, 5)).is_recurrent is True


def _np_view(td, buf):
    # this graph front counts a view's offset in elements; numpy wants bytes
    return np.ndarray(shape=td.shape, dtype=td.dtype, buffer=buf, offset=td.offset * np.dtype(td.dtype).itemsize,
                      strides=td.strides)


def test_broadcast_views_of_a_scalar_share_its_storage():
    A, B = ng.make_axis(2, name="A"), ng.make_axis(3, name="B")
    td = TensorDescription(())
    x = np.zeros(td.shape, dtype=td.dtype)
    one_d = _np_view(td.broadcast([A]), x)
    two_d = _np_view(td.broadcast([A, B]), x)
    x[()] = 3
    assert one_d.shape == (2,) and np.all(one_d == 3)
    assert two_d.shape == (2, 3) and np.all(two_d == 3)


def test_views_only_rewrite_the_description():
    A, B, C = ng.make_axis(10, name="A"), ng.make_axis(20, name="B"), ng.make_axis(5, name="C")
    x = ng.placeholder([A, B, C])
    assert x[:5].axes.full_lengths == (5, 20, 5)
    assert x[:, 2:7].axes.full_lengths == (10, 5, 5)
    assert x[:5, :, :-1].axes.full_lengths == (5, 20, 4)
    same = ng.tensor_slice(x, [slice(None), slice(None, None, 1), slice(None)])
    assert same.axes[0] == x.axes[0] and same.axes[1] == x.axes[1]
    base = np.arange(10 * 20 * 5, dtype=np.float32)
    for view, want in ((x[2:7, 3], base.reshape(10, 20, 5)[2:7, 3]),
                       (ng.axes_with_order(x, [C, A, B]), base.reshape(10, 20, 5).transpose(2, 0, 1)),
                       (ng.flatten(x), base)):
        td = view.tensor_description()
        assert not view.is_device_op
        np.testing.assert_array_equal(_np_view(td, base), want)


def test_reverse_slices_are_refused():
    # test_reshaping.py:174-186: a slice with a negative step would need a copy
    x = ng.placeholder([ng.make_axis(10), ng.make_axis(10)])
    with pytest.raises(ValueError):
        ng.tensor_slice(x, [slice(0, 10, -1), slice(0, 10)])
    with pytest.raises(ValueError):
        x[::-1]


# known answers of test_reshaping.py:100-141 and :190-222
@pytest.mark.parametrize("tensor,s,want", [
    ([[1, 3], [2, 5]], [0, 1], 3),
    ([[1, 3], [2, 5]], [slice(None), 0], [1, 2]),
    ([[1, 3], [2, 5]], [1, slice(None)], [2, 5]),
    ([[1, 4, 5], [2, 5, 6]], [1, slice(1, 3)], [5, 6])])
def test_slice_known_answers(backend, tensor, s, want):
    data = np.array(tensor, dtype=np.float32)
    x = ng.placeholder([ng.make_axis(n) for n in data.shape])
    with executor(ng.tensor_slice(x, s), x) as f:
        np.testing.assert_array_equal(f(data), np.array(want, dtype=np.float32))


def test_overlapping_slices(backend):
    x = ng.placeholder([ng.make_axis(2), ng.make_axis(3)])
    y1 = x[0, :] * 2 + x[1, :] * 3
    y2 = x[0, :] * 2 + x[1, :] * 3 + 4 * x[1, :]
    with executor([y1, y2], x) as f:
        a, b = f(np.array([[10, 20, 30], [1, 2, 3]], dtype=np.float32))
    np.testing.assert_allclose(a, [23, 46, 69])
    np.testing.assert_allclose(b, [27, 54, 81])


# ---- constants -----------------------------------------------------------------------------
def test_constants(backend):
    with executor(ng.constant(5)) as f:
        assert f() == 5
    with executor(ng.constant(np.arange(5))) as f:
        np.testing.assert_array_equal(f(), np.arange(5))
    with executor(ng.constant(1) + ng.constant(2)) as f:
        assert f() == 3
    with executor(ng.multiply(ng.constant(4), ng.constant(2))) as f:
        assert f() == 8
    M, N = ng.make_axis(1), ng.make_axis(3)
    a = ng.constant(np.array([[1, 2, 3]], dtype=np.float32), [M, N])
    b = ng.constant(np.array([[3, 2, 1]], dtype=np.float32), [M, N])
    with executor([ng.multiply(a, ng.constant(2)), ng.add(a, ng.constant(2)),
                   ng.multiply(b, ng.add(a, ng.constant(2))), a + a]) as f:
        twice, plus, fused, summed = f()
    np.testing.assert_array_equal(twice, [[2, 4, 6]])
    np.testing.assert_array_equal(plus, [[3, 4, 5]])
    np.testing.assert_array_equal(fused, [[9, 8, 5]])
    np.testing.assert_array_equal(summed, [[2, 4, 6]])


def test_scalar_broadcast(backend):
    x_axes = ng.make_axes([ng.make_axis(2), ng.make_axis(3)])
    with executor(ng.broadcast(ng.constant(1.0), x_axes)) as f:
        np.testing.assert_array_equal(f(), np.ones((2, 3), np.float32))


# ---- state ---------------------------------------------------------------------------------
def test_read_write_use_modify_fill_state(backend):
    N = ng.make_axis(3, name="N")
    four = np.ones(3, np.float32) * 4
    with executor(ng.variable([N], initial_value=four)) as f:
        np.testing.assert_array_equal(f(), four)
    p = ng.persistent_tensor([N])
    with executor(p, p) as f:
        np.testing.assert_array_equal(f(four), four)
    x = ng.variable([N], initial_value=four)
    with executor(x + x) as f:
        np.testing.assert_array_equal(f(), four + four)
    x = ng.variable([N], initial_value=four)
    with executor(ng.sequential([ng.assign(x, x + x), x])) as f:
        np.testing.assert_array_equal(f(), four + four)
    x = ng.variable([N], initial_value=four)
    with executor(ng.sequential([ng.fill(x, -1), x])) as f:
        np.testing.assert_array_equal(f(), -np.ones(3))


def test_sequential_orders_reads_and_writes(backend):
    N = ng.make_axis(1)
    x = ng.variable([N], initial_value=0)
    x0, x1 = x + x, x + x
    p = ng.sequential([x0, ng.assign(x, 2), x1, x0])
    with executor([x0, x1, p]) as f:
        x0_val, x1_val, p_val = f()
    assert x0_val == 0 and x1_val == 4 and p_val == 0


def test_sequential_with_reductions(backend):
    M = ng.make_axis(3)
    x = ng.variable([M], initial_value=1)
    x0 = x + x
    x1 = ng.sum(x0, out_axes=())
    x2 = ng.sum(x0, out_axes=()) + x0
    with executor([x0, x1, x2, ng.sequential([x0, x1, x2]), x]) as f:
        x0_val, x1_val, x2_val, p_val, x_val = f()
    np.testing.assert_allclose(x0_val, x_val + x_val)
    np.testing.assert_allclose(x1_val, np.sum(x0_val))
    np.testing.assert_allclose(x2_val, np.sum(x0_val) + x0_val)
    np.testing.assert_allclose(p_val, x2_val)


def test_sequential_side_effects_persist_between_calls(backend):
    M = ng.make_axis(3)
    x_np = np.array([1, 2, 3], dtype=np.float32)
    x = ng.variable([M], initial_value=x_np)
    x1 = ng.persistent_tensor(axes=(), initial_value=2)
    x2 = ng.persistent_tensor(axes=(), initial_value=3)
    b = ng.persistent_tensor(axes=(), initial_value=1)
    x1_before, x2_before = ng.value_of(x1), ng.value_of(x2)
    y = ng.sequential([x1_before, x2_before,
                       ng.assign(x1, ng.sum(x, out_axes=()) + x1 * b + (1 - b)),
                       ng.assign(x2, ng.mean(x, out_axes=()) + x2 * b + (1 - b)),
                       x * 2])
    t = ngt.make_transformer()
    try:
        main = t.computation((y, x1_before, x2_before, x1, x2))
        current = t.computation((x1, x2))
        want1, want2 = 2.0, 3.0
        for _ in range(2):
            y_val, before1, before2, after1, after2 = main()
            np.testing.assert_allclose(y_val, x_np * 2)
            np.testing.assert_allclose([before1, before2], [want1, want2])
            want1, want2 = x_np.sum() + want1, x_np.mean() + want2
            np.testing.assert_allclose([after1, after2], [want1, want2])
            np.testing.assert_allclose(current(), [want1, want2])
    finally:
        t.close()


def test_initial_values_and_several_computations_of_one_value(backend):
    C = ng.make_axis(4)
    w_init = np.random.RandomState(0).rand(4).astype(np.float32)
    with executor(ng.variable([C], initial_value=w_init)) as f:
        np.testing.assert_allclose(f(), w_init)
    w = [3, 4, 5]
    with executor(ng.variable([ng.make_axis(3)], initial_value=ng.constant(w))) as f:
        np.testing.assert_allclose(f(), np.asarray(w, np.float32))
    Cx, D = ng.make_axis(2), ng.make_axis(3)
    x = ng.placeholder([Cx, D])
    y1 = x[0, :] * 2 + x[1, :] * 3
    x_np = np.array([[10, 20, 30], [1, 2, 3]], dtype=np.float32)
    t = ngt.make_transformer()
    try:
        fs = [t.computation(y1, x) for _ in range(5)]
        for f in fs:
            np.testing.assert_allclose(f(x_np), x_np[0] * 2 + x_np[1] * 3)
    finally:
        t.close()


def test_argument_checks(backend):
    N = ng.make_axis(1)
    x, y = ng.placeholder([N]), ng.placeholder([N])
    with executor(x + y, x, y) as f:
        with pytest.raises(ValueError):
            f(1)
    tmp, var = ng.temporary([N]), ng.variable([N])
    with pytest.raises(ValueError):
        with executor(tmp + var, tmp, var):
            pass


def test_sign(backend):
    x_np = np.array([-1.2, 2.3, 0.0, 1.2], np.float32)
    x = ng.placeholder([ng.make_axis(4)])
    with executor(ng.sign(x), x) as f:
        np.testing.assert_array_equal(f(x_np), np.sign(x_np))


# ---- dimshuffle: known-answer permutations ---------------------------------------------------
def _dimshuffle_case(a_len):
    data = np.arange(1, a_len * 24 + 1, dtype=np.float32).reshape(a_len, 2, 3, 4)
    if a_len == 1:
        want = [[[[1, 5, 9]], [[2, 6, 10]], [[3, 7, 11]], [[4, 8, 12]]],
                [[[13, 17, 21]], [[14, 18, 22]], [[15, 19, 23]], [[16, 20, 24]]]]
    else:
        want = [[[[1, 5, 9], [25, 29, 33]], [[2, 6, 10], [26, 30, 34]],
                 [[3, 7, 11], [27, 31, 35]], [[4, 8, 12], [28, 32, 36]]],
                [[[13, 17, 21], [37, 41, 45]], [[14, 18, 22], [38, 42, 46]],
                 [[15, 19, 23], [39, 43, 47]], [[16, 20, 24], [40, 44, 48]]]]
    return data, np.array(want, dtype=np.float32)


@pytest.mark.parametrize("a_len", [1, 2])
def test_dimshuffle_known_answers(backend, a_len):
    data, want = _dimshuffle_case(a_len)
    A, B, C, D = (ng.make_axis(n, name=s) for n, s in zip((a_len, 2, 3, 4), "ABCD"))
    x = ng.placeholder([A, B, C, D])
    shuffled = ng.axes_with_order(ng.negative(x), [B, D, A, C])
    with executor([ng.negative(shuffled), ng.contiguous(ng.axes_with_order(x, [B, D, A, C]))], x) as f:
        through_ops, through_copy = f(data)
    np.testing.assert_array_equal(through_ops, want)
    np.testing.assert_array_equal(through_copy, want)
    assert through_copy.flags["C_CONTIGUOUS"]


def test_axes_with_order_argument_checks():
    A, B, C = ng.make_axis(2, name="A"), ng.make_axis(3, name="B"), ng.make_axis(4, name="C")
    x = ng.placeholder([A, B])
    for bad in ([B], [A, B, C], [A, C], [A, B, B]):
        with pytest.raises(ValueError):
            ng.axes_with_order(x, bad)


# ---- tensor_size, expand_dims, cast_axes (test_tensor_size.py:28-41, test_reshaping.py:31-98, 298-318)
def test_tensor_size(backend):
    x = ng.placeholder([ng.make_axis(3), ng.make_axis(4)])
    with executor(ng.tensor_size(x), x) as f:
        assert f(np.arange(12, dtype=np.float32).reshape(3, 4)) == 12
    # the default counts the sample axes only; the batch axis has its own count
    xb = ng.placeholder([ng.make_axis(3), ng.make_axis(4, name="N")])
    with executor([ng.tensor_size(xb), ng.batch_size(xb)], xb) as f:
        size, batch = f(np.arange(12, dtype=np.float32).reshape(3, 4))
    assert size == 3 and batch == 4


@pytest.mark.parametrize("tensor", [[[2, 5], [13, 5]], 2])
@pytest.mark.parametrize("new_length", [1, 2, 3, 4])
def test_expand_dims(backend, tensor, new_length):
    data = np.array(tensor, dtype=np.float32)
    for dim in range(data.ndim + 1):
        x = ng.placeholder([ng.make_axis(n) for n in data.shape])
        expanded = ng.expand_dims(x, ng.make_axis(new_length), dim)
        want = np.ndarray(buffer=data, dtype=data.dtype,
                          shape=data.shape[:dim] + (new_length,) + data.shape[dim:],
                          strides=data.strides[:dim] + (0,) + data.strides[dim:])
        with executor(expanded, x) as f:
            np.testing.assert_array_equal(f(data), want)


def test_cast_axes(backend):
    C, D = ng.make_axis(2), ng.make_axis(3)
    x = ng.placeholder([C, D])
    with pytest.raises(ValueError):
        ng.cast_axes(x, [D, C])
    y = x + ng.cast_axes(x[1, :], [D])          # the slice, named D again, broadcasts along C
    with executor(y, x) as f:
        np.testing.assert_allclose(f(np.array([[10, 20, 30], [1, 2, 3]], dtype=np.float32)),
                                   [[11, 22, 33], [2, 4, 6]])
