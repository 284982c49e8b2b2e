"""The three large benchmark configurations at their full sizes, through the graph path with the
library's own kernel choice, against oracle/configs.py and oracle/flex_model.py.

  C2  batch-norm forward over x fp32 (256, 56, 56, 64), gamma, beta ~ U(0.5, 1.5)
      (frontends/neon/layer.py:1242-1257)
  C3  Adam over 25.6 M fp32 parameters, warm step then step 2 (frontends/neon/optimizer.py:457-468)
  C5  flex16 relu(x*w+b) over 16 M elements, 8 iterations, in both exponent-management modes
      (float_ew2.py:261-281 for the rounding and the statistics)

Tolerances are the ones the fp32 configurations are specified with, rtol 1e-5 / atol 1e-6, for
every output including the normalised y; flex results are compared bit for bit.  Each test also
checks that the kernels that ran are the ones the benchmark times at these sizes (the variants
with cache hints only exist above 192 MiB of operands).
"""
import numpy as np
import pytest
from conftest import default_kernel_choice

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.frontends import neon
from oracle import configs
from oracle import flex_model as fm

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-6


def _kernel_names(t, f):
    return [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]


def test_c2_batchnorm_at_full_size():
    dims = (256, 56, 56, 64)
    Cn, R = dims[0], dims[1] * dims[2] * dims[3]
    x_np, gamma_np, beta_np = configs.c2_inputs(Cn, R, seed=1)
    y_w, mean_w, var_w = configs.c2_cpu(x_np, gamma_np, beta_np)
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        C, H, W, N = (ng.make_axis(n, name=k) for k, n in zip("CHWN", dims))
        x = ng.placeholder([C, H, W, N])
        gamma = ng.variable([C], initial_value=gamma_np)
        beta = ng.variable([C], initial_value=beta_np)
        y, xmean, xvar = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
        f = t.computation([y, xmean, xvar], x)
        y_g, mean_g, var_g = f(x_np.reshape(dims))
        y_g = np.array(y_g).reshape(Cn, R)
        names = _kernel_names(t, f)
    finally:
        t.close()
    if default_kernel_choice():
        assert names == ["moments_f32", "special:batchnorm_k1/nt-stores"], names
    np.testing.assert_allclose(mean_g, mean_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(var_g, var_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(y_g, y_w, rtol=RTOL, atol=ATOL)
    # ... and against float64, which neither side computes in: the one-pass variance of the
    # device (pivot-shifted sums) and the two-pass one of the oracle both stay inside the bound
    x64 = x_np.astype(np.float64)
    mean64, var64 = x64.mean(axis=1), x64.var(axis=1)
    np.testing.assert_allclose(mean_g, mean64, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(var_g, var64, rtol=RTOL, atol=ATOL)
    for c in range(0, Cn, 17):
        y64 = gamma_np[c] * ((x64[c] - mean64[c]) / np.sqrt(var64[c] + 1e-5)) + beta_np[c]
        np.testing.assert_allclose(y_g[c], y64, rtol=RTOL, atol=ATOL)


def test_c3_adam_at_full_size():
    n = 25600000
    p_np, g_np, m_np, v_np = configs.c3_inputs(n, seed=2)
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        P = ng.make_axis(n, name="P")
        p = ng.variable([P], initial_value=p_np)
        grad = ng.placeholder([P])
        opt = neon.Adam()
        opt()
        updates, m, v = opt.variable_update(p, grad)
        f = t.computation(updates, grad)
        read = t.computation([p * 1.0, m * 1.0, v * 1.0])
        ws = configs.Workspace()
        for step in (1, 2):                      # the warm step (t = 1), then the step that is timed
            configs.c3_cpu(p_np, g_np, m_np, v_np, step, ws=ws)
            f(g_np)
        p_g, m_g, v_g = (np.array(a) for a in read())
        names = _kernel_names(t, f)
    finally:
        t.close()
    if default_kernel_choice():
        assert any(d.startswith("special:adam") and d.endswith("/nt-loads") for d in names), names
    np.testing.assert_allclose(m_g, m_np, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(v_g, v_np, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(p_g, p_np, rtol=RTOL, atol=ATOL)
    # the update is far below atol for these inputs (lr 1e-3): also compare it on its own scale
    p0 = configs.c3_inputs(n, seed=2)[0]
    np.testing.assert_allclose(p_g - p0, p_np - p0, rtol=1e-4, atol=1e-9)


@pytest.mark.parametrize("resident", [False, True], ids=["host-policy", "device-policy"])
def test_c5_flex_at_full_size_over_8_iterations(resident):
    n = 16 * 1024 * 1024
    x_np, w_np, b_np = configs.c5_inputs(n, seed=4)
    # the oracle: x, w, b written from the host, y written by the kernel, 8 times
    tx, tw, tb, ty = (fm._SimTensor((n,)) for _ in range(4))
    tw.host_write(w_np)
    tb.host_write(b_np)
    tx.host_write(x_np)
    assert tx.stored_dec == 12                     # x quantised at 2**-12, as the configuration says
    want = []
    ws = configs.Workspace()
    for _ in range(8):
        tx.host_write(x_np)
        ty.kernel_write(lambda: configs.c5_cpu_float(tx.load(), tw.load(), tb.load(), ws=ws))
        want.append((ty.mantissa.copy(), ty.stored_dec, fm.maxabs(ty.mantissa), ty.policy.dec))

    t = ngt.make_transformer_factory("flexhip", resident=resident)()
    try:
        P = ng.make_axis(n, name="P")
        x, w, b = ng.placeholder([P]), ng.placeholder([P]), ng.placeholder([P])
        f = t.computation(neon.rectlin(x * w + b), x, w, b)
        for i in range(8):
            got = f(x_np, w_np, b_np)
            y_view = t.get_op_tensor_view(f.computation_op.values[0])
            entry = y_view.flex_entry
            m_want, dec_want, maxabs_want, next_dec_want = want[i]
            assert entry.last_maxabs == maxabs_want, (i, entry.last_maxabs, maxabs_want)
            assert (entry.dec, entry.next_dec) == (dec_want, next_dec_want), \
                (i, entry.dec, entry.next_dec, dec_want, next_dec_want)
            np.testing.assert_array_equal(y_view._read_raw(), m_want, err_msg="iteration %d mantissas" % i)
            np.testing.assert_array_equal(got, fm.dequantize(m_want, dec_want))
        names = _kernel_names(t, f)
        # eight more iterations without the host in between (what the benchmark times): the
        # kernel group is launched back to back, nothing is read until the end
        group = t.kernel_groups[f]
        for _ in range(8):
            group()
            ty.kernel_write(lambda: configs.c5_cpu_float(tx.load(), tw.load(), tb.load(), ws=ws))
        y_view = t.get_op_tensor_view(f.computation_op.values[0])
        mant = y_view._read_raw()
        entry = y_view.flex_entry
        if resident:
            t.flex_manager.pull()
        assert (entry.dec, entry.next_dec, entry.last_maxabs) == \
            (ty.stored_dec, ty.policy.dec, fm.maxabs(ty.mantissa))
        np.testing.assert_array_equal(mant, ty.mantissa)
    finally:
        t.close()
    if default_kernel_choice():
        assert names == ["special:flex_relu_fma_k0"], names


@pytest.mark.parametrize("classes,samples,kept", [(10, 4194304, "12 rows in registers"), (1000, 32768, "streamed"),
                                                  (100, 327680, "8 rows in registers")])
def test_softmax_over_classes_at_full_size(classes, samples, kept):
    """ng.softmax in the neon layout -- classes x samples, the reduced axis the strided one
    (op_graph.py:3849, frontends/neon/activation.py:145-158) -- at the sizes the shape survey of
    bench.py times: the three kernels of the graph as ONE column chain, against the NumPy
    statements of the CPU transformer and against float64; every column sums to one."""
    rs = np.random.RandomState(11)
    x_np = rs.normal(0, 2, (classes, samples)).astype(np.float32)
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        A, B = ng.make_axis(classes, name="A"), ng.make_axis(samples, name="B")
        x = ng.placeholder([A, B])
        e = ng.exp(x - ng.max(x, out_axes=[B]))
        f = t.computation(e / ng.sum(e, out_axes=[B]), x)
        first = np.array(f(x_np)).copy()              # (may still run on the interpreter)
        assert t.kernel_groups[f].wait_for_programs(timeout=600) is None
        y = np.array(f(x_np)).copy()
        names = _kernel_names(t, f)
    finally:
        t.close()
    if default_kernel_choice():
        assert len(names) >= 1 and all("/column-chain-of-3" in n for n in names), names
    # the CPU transformer's statements, in float32
    m = x_np.max(axis=0)
    ew = np.exp(x_np - m)
    want = ew / ew.sum(axis=0, dtype=np.float32)
    np.testing.assert_allclose(y, want, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(first, want, rtol=RTOL, atol=ATOL)
    x64 = x_np.astype(np.float64)
    e64 = np.exp(x64 - x64.max(axis=0))
    np.testing.assert_allclose(y, e64 / e64.sum(axis=0), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(y.sum(axis=0, dtype=np.float64), 1.0, rtol=0, atol=1e-5)


@pytest.mark.parametrize("rows,k", [(32768, 1024), (32768, 1000)])
def test_flex16_softmax_of_rows_at_full_size(rows, k):
    """The flex16 softmax of rows that bench.py --shapes times, as ONE chain kernel with the
    exponent policy inside the launch, over three inputs whose range moves: against the NumPy flex
    model of the fused kernels (oracle/flex_model.py: every stored tensor rounds to its own
    exponent) within what the order of a row's sum can move a result -- one unit of the sum's
    mantissa, i.e. the fraction 1 / mantissa of a row's results, plus one unit of rounding -- with
    the same exponents chosen, and against float64 under the reference's flex acceptance rule
    (rtol 1e-2, atol 8 x scale: flexgputransform.py:80-103)."""
    from oracle import flex_model as fm
    from oracle import numpy_ops as ops
    rs = np.random.RandomState(31)
    x0 = rs.uniform(-2, 2, (rows, k)).astype(np.float32)
    xs = [x0, (x0 * 3).astype(np.float32), (x0 * 0.2).astype(np.float32)]
    compared = 0
    tx, tm, ts, ty = fm._SimTensor(x0.shape), fm._SimTensor((rows,)), fm._SimTensor((rows,)), fm._SimTensor(x0.shape)
    t = ngt.make_transformer_factory("flexhip")()
    try:
        R, K = ng.make_axis(rows, name="R"), ng.make_axis(k, name="K")
        x = ng.placeholder([R, K])
        e = ng.exp(x - ng.max(x, out_axes=[R]))
        f = t.computation(e / ng.sum(e, out_axes=[R]), x)
        f(xs[0])
        group = t.kernel_groups[f]
        assert group.wait_for_programs(timeout=600) is None
        f(xs[0])
        names = [d for kernel in group.execution_units() for ds in kernel.describe() for d in ds]
        if default_kernel_choice():
            assert len(names) == 3 and all("/chain-of-3" in n for n in names), names
        # the model: two calls with the first input (as above), then the others
        for step, xi in enumerate([xs[0], xs[0], xs[1], xs[2], xs[2]]):
            tx.host_write(xi)
            tm.kernel_write(lambda: ops.reduce("max", tx.load(), 1))
            shifted = lambda: ops.binary("sub", tx.load(), tm.load()[:, None])
            ts.kernel_write(lambda: ops.reduce("sum", ops.unary("exp", shifted()), 1))
            ty.kernel_write(lambda: ops.binary("div", ops.unary("exp", shifted()), ts.load()[:, None]))
            if step == 0:
                continue
            got = np.array(f(xi)).copy() if step > 1 else np.array(f(xs[0])).copy()
            view = t.get_op_tensor_view(f.computation_op.values[0])
            mant = view._read_raw().astype(np.float64)
            # (the next exponent is predicted from the recorded maxima, which may differ by the
            # unit the sum's order moves: next to a boundary the prediction can fall on either side)
            entries = [en for kernel in group.kernels for en in kernel.output_flex_entries]      # maximum, sum, result
            assert len(entries) == 3 and entries[2] is view.flex_entry
            for model, entry in zip((tm, ts, ty), entries):
                assert entry.dec == model.stored_dec and abs(entry.next_dec - model.policy.dec) <= 1, step
            m_out, m_sum = ty.mantissa.astype(np.float64), ts.mantissa.astype(np.float64)
            diff = np.abs(mant - m_out)
            assert (diff <= 1.0 + np.abs(m_out) / m_sum[:, None]).all(), (step, diff.max())
            for model, entry in zip((tm, ts, ty), entries):
                model.policy.dec = entry.next_dec             # (the model follows the device's choice from here)
            if max(fm.maxabs(tt.mantissa) for tt in (tm, ts, ty)) >= 32767:
                continue          # (a range that jumped saturates a tensor once, in the model as on the device; the policy then moves its exponent)
            x64 = fm.dequantize(tx.mantissa, tx.stored_dec).astype(np.float64)
            e64 = np.exp(x64 - x64.max(axis=1, keepdims=True))
            want = e64 / e64.sum(axis=1, keepdims=True)
            atol, rtol = t.get_default_tolerance(want)
            np.testing.assert_allclose(got, want, rtol=rtol, atol=atol)
            compared += 1
        assert compared >= 2
    finally:
        t.close()


def test_integer_arithmetic_over_the_whole_32_bit_range_at_full_size():
    """25.6 M int32 operands drawn from the whole range: sums, products and comparisons of integers
    are integer arithmetic (exact, wrapping at 2**32) as NumPy's integer loops and the reference's
    `int` registers compute them (float_ew2.py:615-641, cputransform.py:512-761); every element is
    compared for equality."""
    n = 25600000
    rs = np.random.RandomState(41)
    a = rs.randint(-2 ** 31, 2 ** 31, n, dtype=np.int64).astype(np.int32)
    b = rs.randint(-2 ** 31, 2 ** 31, n, dtype=np.int64).astype(np.int32)
    b[::7] = a[::7]
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        P = ng.make_axis(n, name="P")
        x, y = ng.placeholder([P], dtype=np.int32), ng.placeholder([P], dtype=np.int32)
        k = ng.add(ng.multiply(x, y, dtype=np.int32), y, dtype=np.int32)
        f = t.computation([k, ng.maximum(x, y), ng.equal(x, y), ng.less(x, y)], x, y)
        first = [np.array(r).copy() for r in f(a, b)]
        assert t.kernel_groups[f].wait_for_programs(timeout=600) is None
        got = [np.array(r).copy() for r in f(a, b)]
    finally:
        t.close()
    with np.errstate(over="ignore"):
        want = [a * b + b, np.maximum(a, b).astype(np.float32), (a == b).astype(np.float32), (a < b).astype(np.float32)]
    for i, (g0, g, w) in enumerate(zip(first, got, want)):
        assert g.dtype == w.dtype, (i, g.dtype, w.dtype)
        np.testing.assert_array_equal(g, w, err_msg="result %d" % i)
        np.testing.assert_array_equal(g0, w, err_msg="result %d, first call" % i)
