"""flex16 on the GPU.

* The reference's flex known-answer vectors (tests/golden/flex_vectors.json) run through
  the `flexhip` transformer with fusion off, i.e. one kernel and one rounding per op as the
  reference executes them, under the reference's acceptance rule (exact for one step, the
  flex tolerance for a sequence: tests/flex_known_answers.py).
* The fused relu(x*w+b) kernel over 8 iterations against the NumPy flex model: mantissas,
  exponents and max|mantissa| bit-exact every iteration.
"""
import json
import os

import numpy as np
import pytest
from conftest import default_kernel_choice

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.frontends import neon
from ngraph_hip.testing import executor
from flex_known_answers import run_vector, check_steps
from oracle import flex_model as fm
from oracle import configs

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
VECTORS = json.load(open(os.path.join(HERE, "golden", "flex_vectors.json")))

NG_OPS = {
    "neg": ng.negative, "sqrt": ng.sqrt, "abs": ng.absolute, "add": ng.add, "sub": ng.subtract,
    "mul": ng.multiply, "div": ng.divide, "mod": ng.mod, "pow": ng.power, "sum": ng.sum,
    "prod": ng.prod, "max": ng.max, "min": ng.min, "argmax": ng.argmax, "argmin": ng.argmin,
    "maximum": ng.maximum, "minimum": ng.minimum, "exp": ng.exp, "log": ng.log,
    "safelog": ng.safelog, "tanh": ng.tanh, "rcp": ng.reciprocal, "sqr": ng.square,
    "sigmoid": ng.sigmoid, "sig": ng.sigmoidAtomic, "eq": ng.equal, "ne": ng.not_equal,
    "lt": ng.less, "le": ng.less_equal, "gt": ng.greater, "ge": ng.greater_equal,
}


@pytest.fixture(params=[False, True], ids=["host-policy", "device-policy"])
def flex_unfused(request):
    """One kernel per op, as the vectors were recorded; under the reference's host-side exponent
    management and under the device-resident one (the default)."""
    ngt.set_transformer_factory(ngt.make_transformer_factory("flexhip", fusion=False, resident=request.param))
    yield
    ngt.set_transformer_factory(None)


def _as_operand(v):
    return np.array(v, dtype=np.float64) if isinstance(v, list) else v


@pytest.mark.parametrize("case", [c for c in VECTORS if not c.get("disabled")],
                         ids=lambda c: "%s@%s" % (c["op"], c["source"]))
def test_reference_flex_vector(flex_unfused, case):
    op = case["op"]
    operands = [tuple(_as_operand(v) for v in s["in"]) + (_as_operand(s["want"]),)
                for s in case["steps"]]
    if op == "assign":
        v, p = ng.variable(()), ng.placeholder(())
        vset = ng.sequential([ng.assign(v, p), v])
        with executor(vset, p) as ex:
            check_steps(ex, operands)
    else:
        run_vector(NG_OPS[op], operands)


def _c5_graph(t, n):
    P = ng.make_axis(n, name="P")
    x, w, b = ng.placeholder([P]), ng.placeholder([P]), ng.placeholder([P])
    y = neon.rectlin(x * w + b)
    return t.computation(y, x, w, b), (x, w, b), y


def _model_c5(xs, w, b):
    """NumPy flex model of the fused kernel over a sequence of x inputs."""
    tx, tw, tb, ty = (fm._SimTensor(w.shape) for _ in range(4))
    tw.host_write(w)
    tb.host_write(b)
    out = []
    for x in xs:
        tx.host_write(x)
        ty.kernel_write(lambda: configs.c5_cpu_float(tx.load(), tw.load(), tb.load()))
        out.append((ty.mantissa.copy(), ty.stored_dec, fm.maxabs(ty.mantissa), ty.policy.dec))
    return out


@pytest.mark.parametrize("resident", [False, True], ids=["host-policy", "device-policy"])
@pytest.mark.parametrize("n", [1 << 16, 100003, 1 << 21])
def test_c5_fused_flex_bit_exact_over_8_iterations(n, resident):
    x0, w, b = configs.c5_inputs(n, seed=4)
    # activations that grow, then collapse: exercises overflow (dec -= 2), the headroom
    # predictor and the slow return to finer exponents
    gains = [1.0, 1.0, 3.0, 40.0, 40.0, 0.5, 0.01, 1.0]
    xs = [(x0 * g).astype(np.float32) for g in gains]
    want = _model_c5(xs, w, b)

    t = ngt.make_transformer_factory("flexhip", resident=resident)()
    f, (x, wp, bp), y = _c5_graph(t, n)
    try:
        for i, xi in enumerate(xs):
            got = f(xi, w, b)
            kernel = t.kernel_groups[f].kernels[-1]
            y_view = t.get_op_tensor_view(f.computation_op.values[0])
            entry = y_view.flex_entry
            m_want, dec_want, maxabs_want, next_dec_want = want[i]
            mant = y_view._read_raw()
            assert entry.last_maxabs == maxabs_want, (i, entry.last_maxabs, maxabs_want)
            np.testing.assert_array_equal(mant, m_want, err_msg="iteration %d mantissas" % i)
            assert entry.dec == dec_want and entry.next_dec == next_dec_want, \
                (i, entry.dec, entry.next_dec, dec_want, next_dec_want)
            np.testing.assert_array_equal(got, fm.dequantize(m_want, dec_want))
        assert len(t.kernel_groups[f].kernels) == 1           # one fused kernel
        if default_kernel_choice():
            assert "special:flex_relu_fma" in kernel.describe()[0][0]
    finally:
        t.close()


def test_flex_host_io_truncates_and_dequantises():
    t = ngt.make_transformer_factory("flexhip")()
    A = ng.make_axis(4, name="A")
    x = ng.placeholder([A])
    f = t.computation(x * 1.0, x)
    try:
        got = f(np.array([1.2, 1.1, -1.3, 1.4]))
        # 1.4 -> dec 14; host write truncates (test_redop.py:117-120)
        np.testing.assert_array_equal(got, np.array([19660, 18022, -21299, 22937]) / 16384.0)
    finally:
        t.close()


def test_device_policy_follows_host_policy_state_for_state():
    """The exponent policy run by flex_update_kernel against the Python mirror, driven with the
    same max|mantissa| sequences through the C ABI (no fused kernel involved)."""
    from ngraph_hip.runtime import HipRuntime
    from ngraph_hip.flex.hipflex import HipFlexManager, STATE_DTYPE
    rt = HipRuntime(0)
    try:
        rs = np.random.RandomState(9)
        host = HipFlexManager()
        n = 8
        entries = [host.make_flex_entry("e%d" % i) for i in range(n)]
        for i, e in enumerate(entries):
            e.init_from_value(10.0 ** rs.uniform(-5, 4))
        dev = rt.flex_states_alloc(n)
        rt.flex_states_write(dev, 0, host.table[:n])
        ids = list(range(n))
        for step in range(60):
            maxima = rs.choice([0, 3, 900, 16384, 25000, 32766, 32767, 32768], size=n)
            # device: prepare (adopts next_dec, clears stats), plant the statistics, update
            rt.flex_prepare(dev, ids, [0] * n)
            table = np.zeros(n, dtype=STATE_DTYPE)
            rt.flex_states_read(dev, 0, table)
            table["stats"] = maxima
            rt.flex_states_write(dev, 0, table)
            rt.flex_update(dev, ids, step)
            rt.flex_states_read(dev, 0, table)
            for i, e in enumerate(entries):
                e.adjust_scale()
                e.manage_after_computation(int(maxima[i]), step)
            for field in ("dec", "next_dec", "scale", "hist_len", "hist_pos", "last_maxabs", "history"):
                np.testing.assert_array_equal(table[field], host.table[:n][field], err_msg=field)
    finally:
        rt.close()


@pytest.mark.parametrize("resident", [False, True], ids=["host-policy", "device-policy"])
@pytest.mark.parametrize("rule", ["adam", "sgd_momentum", "rmsprop"])
def test_flex_learning_rules_prebuilt_equals_interpreter(rule, resident, monkeypatch):
    """A flex learning-rule step is one fused kernel with up to four flex results.  The
    pre-built program and the interpreter must agree in every mantissa and exponent over
    several steps (same fp32 statements, same rounding); the parameters stay near the
    float64 rule."""
    from ngraph_hip.frontends import neon
    n = 1 << 18           # above the size below which the planner schedules ops differently
    rs = np.random.RandomState(3)
    p0 = rs.normal(0, 0.1, n).astype(np.float32)
    grads = [rs.normal(0, 0.01, n).astype(np.float32) for _ in range(4)]

    def run():
        t = ngt.make_transformer_factory("flexhip", resident=resident)()
        try:
            P = ng.make_axis(n, name="P")
            p, grad = ng.variable([P], initial_value=p0), ng.placeholder([P])
            if rule == "adam":
                opt = neon.Adam(learning_rate=0.01)
                opt()
                updates = opt.variable_update(p, grad)[0]
            elif rule == "sgd_momentum":
                updates = neon.GradientDescentMomentum(0.1, 0.9).variable_update(p, grad)[0]
            else:
                updates = neon.RMSProp(learning_rate=0.01).variable_update(p, grad)[0]
            f = t.computation(updates, grad)
            read = t.computation(p * 1.0)
            for g in grads:
                f(g)
            value = np.array(read())
            view = t.get_op_tensor_view(p)
            names = [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
            return value, view._read_raw().copy(), view.flex_entry.dec, names
        finally:
            t.close()

    monkeypatch.delenv("NGH_FORCE_INTERP", raising=False)
    v_static, m_static, dec_static, names = run()
    if default_kernel_choice():
        assert any(nm.startswith("special:flex_") for nm in names), names
    monkeypatch.setenv("NGH_FORCE_INTERP", "1")
    v_interp, m_interp, dec_interp, names = run()
    assert not any(nm.startswith("special:") for nm in names)
    assert dec_static == dec_interp
    np.testing.assert_array_equal(m_static, m_interp)
    # float64 rule (not for Adam: its second moment, ~1e-7 next to elements ~1e-3 under one
    # shared exponent, mostly quantises to zero, so flex16 Adam does not track the real rule)
    p, g64 = p0.astype(np.float64), [g.astype(np.float64) for g in grads]
    if rule == "adam":
        assert np.isfinite(v_static).all()
        return
    elif rule == "sgd_momentum":
        vel = np.zeros(n)
        for g in g64:
            vel = 0.9 * vel - 0.1 * g
            p = p + vel
    else:
        state, vel = np.ones(n), np.zeros(n)
        for g in g64:
            state = 0.95 * state + 0.05 * g * g
            p = p - 0.01 * g / np.sqrt(state + 1e-6)
    # state tensors start from zeros at the default exponent (resolution 2**-8) and only then
    # adapt, so the first steps are coarse: a sanity bound, not a precision claim
    assert np.abs(v_static - p).max() < 0.02, np.abs(v_static - p).max()


# ---- exponent management across launches with nobody looking in between --------------------
# The library can leave the statistics of a launch unfolded until the next launch that writes
# the tensor, or until something else needs the record.  Whatever it does, records, mantissas
# and consumers must see exactly what the launch-by-launch policy of the host gives.

# (name, NGH_FLEX_SELF_MANAGED, NGH_FLEX_LAZY_BLOCKS_PER_CU, NGH_ORDERED_ARRIVAL); the end-of-kernel
# policy hands over between workgroups with relaxed tickets (default) or release tickets and an acquire fence
# (name, NGH_FLEX_SELF_MANAGED, NGH_FLEX_LAZY_BLOCKS_PER_CU, NGH_ORDERED_ARRIVAL, NGH_STREAM_MIB); the last one
# lowers the size from which a stage takes the policy step at its end instead of deferring it, so
# that stages of both kinds follow each other on the same tensors
_AMBIENT_STREAM_MIB = os.environ.get("NGH_STREAM_MIB")
_POLICY_MODES = [("host", None, None, None, None), ("three-launches", "0", None, None, None),
                 ("end-of-kernel", "1", None, None, None),
                 ("end-of-kernel-release-acquire-tickets", "1", None, "1", None),
                 ("deferred", "2", None, None, None), ("deferred-small-grid", "2", "1", None, None),
                 ("mixed-by-size", "2", None, None, "1")]


def _entry_state(entry):
    return (entry.dec, entry.next_dec, entry.last_maxabs, tuple(entry.history))


def _with_policy_mode(monkeypatch, mode, grid, ordered=None, stream_mib=None):
    monkeypatch.delenv("NGH_FLEX_SELF_MANAGED", raising=False)
    if stream_mib is not None:
        monkeypatch.setenv("NGH_STREAM_MIB", stream_mib)
    elif _AMBIENT_STREAM_MIB is None:
        monkeypatch.delenv("NGH_STREAM_MIB", raising=False)
    else:
        monkeypatch.setenv("NGH_STREAM_MIB", _AMBIENT_STREAM_MIB)
    monkeypatch.delenv("NGH_FLEX_LAZY_BLOCKS_PER_CU", raising=False)
    monkeypatch.delenv("NGH_ORDERED_ARRIVAL", raising=False)
    if ordered is not None:
        monkeypatch.setenv("NGH_ORDERED_ARRIVAL", ordered)
    if mode is not None:
        monkeypatch.setenv("NGH_FLEX_SELF_MANAGED", mode)
    if grid is not None:
        monkeypatch.setenv("NGH_FLEX_LAZY_BLOCKS_PER_CU", grid)


@pytest.mark.parametrize("n", [1 << 18, 100003 * 8])
def test_device_only_iterations_agree_across_policy_modes(n, monkeypatch):
    x0, w, b = configs.c5_inputs(n, seed=11)
    x0 = (x0 * 30.0).astype(np.float32)           # saturates at the first exponent: the policy has to move
    seen = {}
    for name, mode, grid, ordered, stream_mib in _POLICY_MODES:
        _with_policy_mode(monkeypatch, mode, grid, ordered, stream_mib)
        t = ngt.make_transformer_factory("flexhip", resident=name != "host")()
        try:
            f, _, _ = _c5_graph(t, n)
            f(x0, w, b)
            group = t.kernel_groups[f]
            states = []
            for it in range(7):
                group()
                if name.startswith("deferred"):
                    if default_kernel_choice():
                        assert t.runtime.flex_unsettled() == 1    # y's record, and only that
                    else:           # a forced kernel choice may or may not take the one-launch path
                        assert t.runtime.flex_unsettled() in (0, 1)
                elif name == "mixed-by-size":
                    assert t.runtime.flex_unsettled() in (0, 1)
                elif name != "host":
                    assert t.runtime.flex_unsettled() == 0
                if it in (2, 6):                    # look twice: after a few launches, and at the end
                    view = t.get_op_tensor_view(f.computation_op.values[0])
                    states.append((_entry_state(view.flex_entry), view._read_raw().copy()))
            seen[name] = states
        finally:
            t.close()
    ref = seen["host"]
    assert ref[0][0] != ref[1][0]                   # the exponent state did evolve in between
    for name, states in seen.items():
        for (st, mant), (st_ref, mant_ref) in zip(states, ref):
            assert st == st_ref, (name, st, st_ref)
            np.testing.assert_array_equal(mant, mant_ref, err_msg=name)


def test_consumer_of_a_tensor_with_unfolded_statistics(monkeypatch):
    """A second computation reads, on the device, the scale of a tensor whose last writes left
    their statistics unfolded; a host fill of the same tensor in between must also win."""
    n = 1 << 18
    x0, w, b = configs.c5_inputs(n, seed=12)
    seen = {}
    for name, mode, grid, ordered, stream_mib in _POLICY_MODES:
        _with_policy_mode(monkeypatch, mode, grid, ordered, stream_mib)
        t = ngt.make_transformer_factory("flexhip", resident=name != "host")()
        try:
            P = ng.make_axis(n, name="P")
            x, wp, bp = ng.placeholder([P]), ng.placeholder([P]), ng.placeholder([P])
            v = ng.persistent_tensor([P], initial_value=0.0)
            write = t.computation(ng.assign(v, neon.rectlin(x * wp + bp)), x, wp, bp)
            read = t.computation(v * 0.5 + 1.0)
            write((x0 * 20.0).astype(np.float32), w, b)
            group = t.kernel_groups[write]
            for _ in range(3):
                group()
            first = np.array(read())
            for _ in range(2):
                group()
            view = t.get_op_tensor_view(v)
            second = (np.array(read()), _entry_state(view.flex_entry), view._read_raw().copy())
            seen[name] = (first, second)
        finally:
            t.close()
    ref_first, ref_second = seen["host"]
    for name, (first, second) in seen.items():
        np.testing.assert_array_equal(first, ref_first, err_msg=name)
        np.testing.assert_array_equal(second[0], ref_second[0], err_msg=name)
        assert second[1] == ref_second[1], (name, second[1], ref_second[1])
        np.testing.assert_array_equal(second[2], ref_second[2], err_msg=name)


def test_in_place_rule_iterated_on_the_device_agrees_across_policy_modes(monkeypatch):
    from ngraph_hip.frontends import neon as neon_front
    n = 1 << 18
    rs = np.random.RandomState(5)
    p0 = rs.normal(0, 0.1, n).astype(np.float32)
    g = rs.normal(0, 0.05, n).astype(np.float32)
    seen = {}
    for name, mode, grid, ordered, stream_mib in _POLICY_MODES:
        _with_policy_mode(monkeypatch, mode, grid, ordered, stream_mib)
        t = ngt.make_transformer_factory("flexhip", resident=name != "host")()
        try:
            P = ng.make_axis(n, name="P")
            p, grad = ng.variable([P], initial_value=p0), ng.placeholder([P])
            updates = neon_front.GradientDescentMomentum(0.1, 0.9).variable_update(p, grad)[0]
            f = t.computation(updates, grad)
            f(g)
            group = t.kernel_groups[f]
            for _ in range(5):
                group()
            if name.startswith("deferred") and default_kernel_choice():
                assert t.runtime.flex_unsettled() >= 1
            view = t.get_op_tensor_view(p)
            seen[name] = (_entry_state(view.flex_entry), view._read_raw().copy())
            assert name == "host" or t.runtime.flex_unsettled() == 0
        finally:
            t.close()
    for name, (st, mant) in seen.items():
        assert st == seen["host"][0], (name, st, seen["host"][0])
        np.testing.assert_array_equal(mant, seen["host"][1], err_msg=name)


@pytest.mark.gpu
def test_flex_statistics_file_holds_the_exponent_state_of_every_tensor(tmp_path):
    """set_output_statistics_file / save_output_statistics_file (base.py:407-417,
    flexgputransform.py:105-114, called by the neon callbacks at callbacks.py:126-135): with
    collect_flex_data the flex manager writes its per-tensor state."""
    path = str(tmp_path / "flex_stats.npz")
    t = ngt.make_transformer_factory("flexhip", collect_flex_data=True)()
    try:
        H = ng.make_axis(64, name="H")
        x = ng.placeholder([H])
        f = t.computation(x * 2.0 + 1.0, x)
        t.set_output_statistics_file(path)
        f(np.linspace(-3, 3, 64).astype(np.float32))
        t.save_output_statistics_file()
    finally:
        t.close()
    data = np.load(path)
    assert int(data["autoflex_count"]) >= 1
    decs = [k for k in data.files if k.endswith("/dec")]
    assert decs and all(0 <= int(data[k]) <= 31 for k in decs)
    # the result 2x + 1 reaches 7: 3 integer bits, so 15 - 3 - 1 fractional bits or fewer
    assert any(int(data[k]) <= 12 and int(data[k.replace("/dec", "/last_maxabs")]) > 0 for k in decs)
    # without collect_flex_data the calls are accepted and write nothing
    other = str(tmp_path / "none.npz")
    t = ngt.make_transformer_factory("flexhip")()
    try:
        t.set_output_statistics_file(other)
        t.save_output_statistics_file()
    finally:
        t.close()
    assert not os.path.exists(other)


# ---- row chains of flex kernels: one launch for the maximum, the sum of exponentials and the
# normalised result of a softmax, each a flex16 tensor with an exponent of its own -------------
def _rows_graph(t, rows, k, shift_only):
    R, K = ng.make_axis(rows, name="R"), ng.make_axis(k, name="K")
    x = ng.placeholder([R, K])
    m = ng.max(x, out_axes=[R])
    if shift_only:
        out = x - m
    else:
        e = ng.exp(x - m)
        out = e / ng.sum(e, out_axes=[R])
    return t.computation(out, x)


def _model_rows(xs, shift_only):
    """The fused kernels in the NumPy flex model: every stored tensor (the maximum, the sum, the
    result) rounds to its own exponent, what a later kernel loads is what was stored, and the
    values in between are float32 (op by op as the CPU transformer computes them)."""
    from oracle import numpy_ops as ops
    rows = xs[0].shape[0]
    tx, tm, ts, ty = fm._SimTensor(xs[0].shape), fm._SimTensor((rows,)), fm._SimTensor((rows,)), \
        fm._SimTensor(xs[0].shape)
    out = []
    for x in xs:
        tx.host_write(x)
        tm.kernel_write(lambda: ops.reduce("max", tx.load(), 1))
        shifted = lambda: ops.binary("sub", tx.load(), tm.load()[:, None])
        if shift_only:
            ty.kernel_write(shifted)
            sums = None
        else:
            ts.kernel_write(lambda: ops.reduce("sum", ops.unary("exp", shifted()), 1))
            ty.kernel_write(lambda: ops.binary("div", ops.unary("exp", shifted()), ts.load()[:, None]))
            sums = (ts.mantissa.copy(), ts.stored_dec, ts.policy.dec)
        out.append({"max": (tm.mantissa.copy(), tm.stored_dec, tm.policy.dec), "sum": sums,
                    "out": (ty.mantissa.copy(), ty.stored_dec, ty.policy.dec)})
    return out


def _run_rows(xs, shift_only, resident):
    """Per input: the result's mantissas, and (exponent in use, next exponent, last max
    |mantissa|) of every flex tensor the computation writes, in the order they are written."""
    rows, k = xs[0].shape
    t = ngt.make_transformer_factory("flexhip", resident=resident, jit=True)()
    try:
        f = _rows_graph(t, rows, k, shift_only)
        seen = []
        for x in xs:
            f(x)
            group = t.kernel_groups[f]
            view = t.get_op_tensor_view(f.computation_op.values[0])
            t.flex_manager.pull()
            entries = []
            for kernel in group.kernels:
                for e in kernel.output_flex_entries:
                    entries.append((e.dec, e.next_dec, e.last_maxabs))
            seen.append((view._read_raw().copy(), entries))
        names = [d for kernel in group.execution_units() for ds in kernel.describe() for d in ds]
        return seen, names
    finally:
        t.close()


@pytest.mark.parametrize("resident", [False, True], ids=["host-policy", "device-policy"])
@pytest.mark.parametrize("rows,k", [(512, 1024), (300, 1000), (64, 4098)])
def test_flex_row_chain_of_a_maximum_and_its_consumer_is_bit_exact(rows, k, resident, monkeypatch):
    """x - max(x) along rows: as one chain kernel, as two kernels, and in the NumPy flex model
    -- the same mantissas and exponents after every one of several inputs whose range moves."""
    rs = np.random.RandomState(21)
    x0 = rs.uniform(-2, 2, (rows, k)).astype(np.float32)
    xs = [(x0 * g).astype(np.float32) for g in (1.0, 1.0, 5.0, 40.0, 0.3, 0.01, 1.0)]
    want = _model_rows(xs, True)
    monkeypatch.delenv("NGH_NO_CHAIN", raising=False)
    chained, names = _run_rows(xs, True, resident)
    if default_kernel_choice():
        assert any("chain-of-2" in nm for nm in names), names
    monkeypatch.setenv("NGH_NO_CHAIN", "1")
    apart, names = _run_rows(xs, True, resident)
    assert not any("chain-of" in nm for nm in names), names
    for i, ((mant, entries), (mant2, entries2)) in enumerate(zip(chained, apart)):
        np.testing.assert_array_equal(mant, want[i]["out"][0], err_msg="input %d" % i)
        np.testing.assert_array_equal(mant2, want[i]["out"][0], err_msg="input %d, kernel by kernel" % i)
        assert entries == entries2, (i, entries, entries2)
        for (dec, next_dec, last), which in zip(entries, ("max", "out")):
            m_want, dec_want, next_want = want[i][which]
            assert (dec, next_dec, last) == (dec_want, next_want, fm.maxabs(m_want)), (i, which)


@pytest.mark.parametrize("resident", [False, True], ids=["host-policy", "device-policy"])
@pytest.mark.parametrize("rows,k", [(512, 1024), (300, 1000)])
def test_flex_softmax_of_rows_as_one_chain(rows, k, resident, monkeypatch):
    """A flex16 softmax of rows as one chain kernel against the same kernels launched one by one
    and against the NumPy flex model.  The sum of exponentials is added up in another order by
    each of the three and the device's exp differs from NumPy's in the last place, so a sum's
    mantissa may land on the neighbouring 16-bit value, which moves that row's results by the
    fraction 1 / (the sum's mantissa): the results agree to that plus one unit of rounding, most
    of them exactly, and the exponents are the same."""
    rs = np.random.RandomState(22)
    x0 = rs.uniform(-2, 2, (rows, k)).astype(np.float32)
    xs = [(x0 * g).astype(np.float32) for g in (1.0, 1.0, 4.0, 0.1, 1.0)]
    want = _model_rows(xs, False)
    monkeypatch.delenv("NGH_NO_CHAIN", raising=False)
    chained, names = _run_rows(xs, False, resident)
    if default_kernel_choice():
        assert any("chain-of-3" in nm for nm in names), names
    monkeypatch.setenv("NGH_NO_CHAIN", "1")
    apart, names = _run_rows(xs, False, resident)
    assert not any("chain-of" in nm for nm in names), names
    for i, ((mant, entries), (mant2, entries2)) in enumerate(zip(chained, apart)):
        for got, what in ((mant, "chain"), (mant2, "kernel by kernel")):
            m_out, m_sum = want[i]["out"][0].astype(np.float64), want[i]["sum"][0].astype(np.float64)
            diff = np.abs(got.astype(np.float64) - m_out)
            allowed = 1.0 + np.abs(m_out) / m_sum[:, None]
            assert (diff <= allowed).all(), (i, what, diff.max(), (diff - allowed).max())
            assert (diff != 0).mean() < 0.05, (i, what, (diff != 0).mean())
        for (dec, next_dec, last), (dec2, next2, last2), which in zip(entries, entries2, ("max", "sum", "out")):
            m_want, dec_want, next_want = want[i][which]
            assert (dec, next_dec) == (dec2, next2) == (dec_want, next_want), (i, which)
            assert abs(last - fm.maxabs(m_want)) <= 1 and abs(last2 - fm.maxabs(m_want)) <= 1, (i, which)


def test_flex_row_chain_agrees_across_policy_modes(monkeypatch):
    """The chain launched with nobody looking in between, under every way the library has of
    running the exponent policy (on the host, as three launches, at the end of the kernel):
    the same records and mantissas."""
    rows, k = 384, 1024
    rs = np.random.RandomState(23)
    x0 = rs.uniform(-2, 2, (rows, k)).astype(np.float32)
    seen = {}
    for name, mode, grid, ordered, stream_mib in _POLICY_MODES:
        _with_policy_mode(monkeypatch, mode, grid, ordered, stream_mib)
        t = ngt.make_transformer_factory("flexhip", resident=name != "host", jit=True)()
        try:
            f = _rows_graph(t, rows, k, True)
            states = []
            for gain in (1.0, 30.0, 30.0, 0.02):
                f((x0 * gain).astype(np.float32))
                group = t.kernel_groups[f]
                for it in range(3):
                    group()
                view = t.get_op_tensor_view(f.computation_op.values[0])
                t.flex_manager.pull()
                entries = [_entry_state(e) for kernel in group.kernels for e in kernel.output_flex_entries]
                states.append((entries, view._read_raw().copy()))
            seen[name] = states
        finally:
            t.close()
    ref = seen["host"]
    assert ref[0][0] != ref[1][0]
    for name, states in seen.items():
        for (st, mant), (st_ref, mant_ref) in zip(states, ref):
            assert st == st_ref, (name, st, st_ref)
            np.testing.assert_array_equal(mant, mant_ref, err_msg=name)
