"""ngraph_hip/plugin.py: the adapters between the real package's tensor descriptions and the
lowering's, on hand-built inputs, and the binding of the backend to a foreign graph package
(tests/plugin_clone.py), without a device (the lowering is validated by the library) and on
the GPU against the oracle."""
import numpy as np
import pytest

from ngraph_hip import plugin
from oracle import configs
import plugin_clone


# ------------------------------------------------------------------ adapters, by hand
def test_flat_stride_takes_the_innermost_of_a_flattened_axis():
    # axes.py:1104-1150: an axis that flattens (H, W) of a c-contiguous fp32 [C, H, W] = [4, 5, 6]
    # holds (W * 4, 4) = (24, 4); flattening (C, H) holds (120, 24)
    assert plugin.flat_stride(24) == 24
    assert plugin.flat_stride((24, 4)) == 4
    assert plugin.flat_stride((120, 24)) == 24
    assert plugin.flat_stride(((480, 120), 24)) == 24          # nested twice
    assert plugin.flat_stride((0, 0)) == 0                      # a broadcast stays a broadcast
    with pytest.raises(ValueError):
        plugin.flat_stride(())
    assert plugin.flat_size((5, 6)) == 30 and plugin.flat_size(((4, 5), 6)) == 120 and plugin.flat_size(7) == 7


def test_element_strides_and_offsets_divide_by_the_item_size():
    assert plugin.element_strides((120, 24, 4), 4) == (30, 6, 1)
    assert plugin.element_strides(((120, 24), 4), 4) == (6, 1)
    assert plugin.element_strides((0, 2), 2) == (0, 1)          # int16 / flex16 storage
    assert plugin.element_strides((), 4) == ()
    assert plugin.element_offset(48, 4) == 12 and plugin.element_offset(0, 2) == 0
    with pytest.raises(ValueError):
        plugin.element_strides((6, 4), 4)                       # a view that splits an element
    with pytest.raises(ValueError):
        plugin.element_offset(3, 2)


class _FakeFlex(object):
    storage_bits = 16
    itemsize = 4           # what a careless caller would read: the register type's size


class _FakeDescription(object):
    """Only what ElementView reads, with the real package's conventions."""

    def __init__(self, shape, full_strides, offset, dtype):
        self.shape, self.full_strides, self.offset, self.dtype = shape, full_strides, offset, dtype
        self.base = self
        self.name = "t"


def test_element_view_of_a_description():
    f32 = np.dtype(np.float32)
    td = _FakeDescription((4, 30), (120 * 4, (6 * 4, 4)), 8, f32)
    v = plugin.adapt_tensor_description(td)
    assert (v.shape, v.full_strides, v.offset) == ((4, 30), (120, 1), 2)
    assert not v.c_contiguous                                    # rows of 30 in a pitch of 120
    assert plugin.adapt_tensor_description(v) is v               # idempotent
    assert v.base is td and v.name == "t"                        # everything else is the description's own
    # the device tensors are kept in dictionaries keyed by descriptions: a view finds them
    assert {td: "tensor"}[v] == "tensor" and v == td and not (v != td)
    assert plugin.adapt_tensor_description(_FakeDescription((4, 30), (120, 4), 0, f32)).c_contiguous
    # flex storage: 2 bytes per element whatever the dtype object calls its item size
    q = plugin.adapt_tensor_description(_FakeDescription((8,), (2,), 6, _FakeFlex()))
    assert (q.full_strides, q.offset) == ((1,), 3)
    # a scalar
    s = plugin.adapt_tensor_description(_FakeDescription((), (), 0, f32))
    assert s.c_contiguous and s.full_strides == ()


def test_register_needs_the_package():
    with pytest.raises(ImportError):
        plugin.register("no_such_graph_package")


# ------------------------------------------------------------------ binding to a foreign package
@pytest.fixture(scope="module")
def clone(tmp_path_factory):
    name = plugin_clone.make_clone(tmp_path_factory.mktemp("clone"))
    bound = plugin.bind(name, adapt=lambda td: plugin.adapt_tensor_description(plugin_clone.ByteDescription(td)))
    import importlib
    og = importlib.import_module(name + ".op_graph.op_graph")
    base = importlib.import_module(name + ".transformers.base")
    return bound, og, base


def test_bound_transformers_belong_to_the_package(clone):
    import ngraph_hip.transformers.base as own_base
    from ngraph_hip.transformers.hiptransform import HipTransformer as OwnHipTransformer
    bound, og, base = clone
    assert issubclass(bound.HipTransformer, base.ComputationGraphTransformer)
    assert not issubclass(bound.HipTransformer, own_base.ComputationGraphTransformer)
    assert bound.HipTransformer is not OwnHipTransformer
    assert issubclass(bound.FlexHipTransformer, bound.HipTransformer)
    # registered through the package's own metaclass, made by the package's own factory
    assert base.Transformer.transformers["hipgpu"] is bound.HipTransformer
    assert base.Transformer.transformers["flexhip"] is bound.FlexHipTransformer
    t = base.make_transformer_factory("hipgpu", dry_run=True)()
    assert type(t) is bound.HipTransformer
    t.close()
    assert plugin.bind(bound.package) is bound                   # one binding per package


def _bn_graph(og, dims, gamma_np, beta_np):
    C, H, W, N = (og.make_axis(n, name=k) for k, n in zip("CHWN", dims))
    x = og.placeholder([C, H, W, N])
    gamma = og.variable([C], initial_value=gamma_np)
    beta = og.variable([C], initial_value=beta_np)
    red = og.make_axes([H, W, N])
    flat = og.flatten(og.axes_with_order(x, [C, H, W, N]), og.make_axes([C]) | red.flatten(force=True))
    xmean = og.mean(flat, out_axes=[C])
    xvar = og.variance(flat, out_axes=[C])
    y = og.unflatten(gamma * ((flat - xmean) * og.reciprocal(og.sqrt(xvar + 1e-5))) + beta)
    return [y, xmean, xvar], x


def test_lowering_through_the_binding_matches_the_native_lowering(clone):
    """Batch norm over a flattened view (nested strides on the package's side) lowers, on the
    foreign package through byte-stride descriptions, to the very kernels and operand layouts
    the native front gives."""
    import ctypes
    import ngraph_hip.op_graph.op_graph as own_og
    import ngraph_hip.transformers as own_ngt
    bound, og, base = clone
    dims = (16, 7, 7, 8)
    _, gamma_np, beta_np = configs.c2_inputs(dims[0], 7 * 7 * 8)

    def lowered(graph_og, make_transformer):
        t = make_transformer()
        t.chain_kernels = False       # (kernel by kernel: rows this short would merge into a row chain)
        try:
            results, x = _bn_graph(graph_og, dims, gamma_np, beta_np)
            f = t.computation(results, x)
            t.initialize()
            group = t.kernel_groups[f]
            group.bind()
            out = []
            for k in group.kernels:
                if hasattr(k, "specs"):
                    for spec in k.specs:
                        tens = [(tuple(spec.tensors[i].strides), spec.tensors[i].dtype) for i in range(spec.n_tensors)]
                        ops = [(o.opcode, o.dst, o.a, o.b) for o in spec.ops[:spec.n_ops]]
                        out.append((tuple(spec.shape), tens, ops))
                else:
                    out.append((type(k).__name__, k.rows, k.R, k.row_stride))
            return out
        finally:
            t.close()

    native = lowered(own_og, own_ngt.make_transformer_factory("hipgpu", dry_run=True))
    foreign = lowered(og, base.make_transformer_factory("hipgpu", dry_run=True))
    assert foreign == native and len(native) >= 2


@pytest.mark.gpu
def test_foreign_package_runs_on_the_device(clone):
    """Elementwise chain, batch norm over a flattened view and the LSTM cell on transposed
    (strided) storage, built with the foreign package's ops and run through its own call
    protocol on the bound `hipgpu`, against the oracle."""
    bound, og, base = clone
    t = base.make_transformer_factory("hipgpu")()
    try:
        x_np, a, b = configs.c1_inputs((33, 65))
        H, W = og.make_axis(33, name="H"), og.make_axis(65, name="W")
        x, pa, pb = og.placeholder([H, W]), og.placeholder(()), og.placeholder(())
        f1 = t.computation(og.tanh(pa * x + pb) * og.sigmoid(x), x, pa, pb)
        dims = (16, 7, 7, 8)
        xb_np, gamma_np, beta_np = configs.c2_inputs(dims[0], 7 * 7 * 8)
        results, xb = _bn_graph(og, dims, gamma_np, beta_np)
        f2 = t.computation(results, xb)
        Hn, Nn = 48, 5
        gates_np, cprev_np = configs.c4_inputs(Hn, Nn)
        Hh, N, G = og.make_axis(Hn, name="Hh"), og.make_axis(Nn, name="N"), og.make_axis(4 * Hn, name="G")
        gates_st, cprev_st = og.placeholder([N, G]), og.placeholder([N, Hh])
        gates, c_prev = og.axes_with_order(gates_st, [G, N]), og.axes_with_order(cprev_st, [Hh, N])
        part = [og.cast_axes(og.tensor_slice(gates, [slice(j * Hn, (j + 1) * Hn), slice(None)]), [Hh, N])
                for j in range(4)]
        i_, f_, o_, g_ = og.sigmoid(part[0]), og.sigmoid(part[1]), og.sigmoid(part[2]), og.tanh(part[3])
        c = f_ * c_prev + i_ * g_
        f3 = t.computation([c, o_ * og.tanh(c), og.sum(gates, out_axes=[G])], gates_st, cprev_st)

        np.testing.assert_allclose(f1(x_np, a, b), configs.c1_cpu(x_np, a, b), rtol=1e-5, atol=1e-6)
        y_w, mean_w, var_w = configs.c2_cpu(xb_np, gamma_np, beta_np)
        y_g, mean_g, var_g = f2(xb_np.reshape(dims))
        np.testing.assert_allclose(mean_g, mean_w, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(var_g, var_w, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(np.array(y_g).reshape(dims[0], -1), y_w, rtol=1e-5, atol=1e-5)
        c_w, h_w, db_w = configs.c4_cpu(gates_np, cprev_np)
        c_g, h_g, db_g = f3(gates_np, cprev_np)
        np.testing.assert_allclose(c_g, c_w, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(h_g, h_w, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(db_g, db_w, rtol=1e-5, atol=1e-5)
    finally:
        t.close()
