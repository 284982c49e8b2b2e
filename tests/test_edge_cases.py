"""Edge cases the reference's tests cover for this path: empty / scalar / length-1 views, ragged
lengths around the vector widths, misaligned and broadcast operands, 16-bit storage, strided
copies (dimshuffle), strided host I/O, and the error paths of the boundary."""
import itertools

import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.runtime import FusedSpecBuilder, NGH_F32, NGH_FLEX16, NGH_F16, HipLibraryError
from ngraph_hip.transformers.base import UnsupportedTransformerException
from oracle import flex_model as fm

f32 = np.float32


# ------------------------------------------------------------------------------- no GPU needed
def test_backend_fails_loudly_without_a_gpu():
    """On a machine without an MI355X the transformers raise; nothing falls back to the CPU."""
    from ngraph_hip.runtime import hiplib
    import ctypes
    n = ctypes.c_int()
    hiplib.load_library().ngh_device_count(ctypes.byref(n))
    if n.value > 0:
        pytest.skip("a GPU is present")
    for name in ("hipgpu", "flexhip"):
        with pytest.raises(UnsupportedTransformerException):
            ngt.make_transformer_factory(name)()


def test_builder_limits_raise():
    # 40 values alive at once do not fit the 32 registers of a program ...
    sb = FusedSpecBuilder([8])
    t = sb.tensor(4096, [1])
    regs = [sb.load(t) for _ in range(40)]
    acc = regs[0]
    for r in regs[1:]:
        acc = sb.binary("add", acc, r)
    sb.store(t, acc)
    with pytest.raises(ValueError):
        sb.build()
    # ... but 40 values of which few are alive together do
    sb = FusedSpecBuilder([8])
    t = sb.tensor(4096, [1])
    acc = sb.load(t)
    for _ in range(40):
        acc = sb.unary("neg", acc)
    sb.store(t, acc)
    assert sb.build().n_regs <= 2
    with pytest.raises(ValueError):
        FusedSpecBuilder([2, 2, 2, 2])
    sb = FusedSpecBuilder([8])
    with pytest.raises(ValueError):
        for i in range(20):
            sb.tensor(4096 * (i + 1), [1])


# ------------------------------------------------------------------------------- GPU
gpu = pytest.mark.gpu


@gpu
@pytest.mark.parametrize("n", list(range(1, 20)) + [31, 32, 33, 63, 64, 65, 255, 257, 1023, 4097])
def test_ragged_lengths_fp32_and_flex(hip_runtime, n):
    """Vector body + scalar tail for every residue of the vector widths (4 for fp32, 8 for int16)."""
    rt = hip_runtime
    rs = np.random.RandomState(n)
    x, y = rs.normal(0, 1, n).astype(f32), rs.normal(0, 1, n).astype(f32)
    x_d, y_d, z_d = rt.array(x), rt.array(y), rt.empty((n,))
    sb = FusedSpecBuilder([n])
    tx, ty, tz = (sb.tensor(d.ptr, [1]) for d in (x_d, y_d, z_d))
    sb.store(tz, sb.binary("mul", sb.load(tx), sb.unary("tanh", sb.load(ty))))
    rt.launch_fused(sb.build())
    np.testing.assert_allclose(z_d.get(), x * np.tanh(y), rtol=1e-5, atol=1e-6)
    # the same on int16 mantissas: out = rni(a * 2) at the same scale, statistics = max|out|
    a = rs.randint(-16000, 16000, n).astype(np.int16)
    a_d, o_d = rt.array(a), rt.empty((n,), NGH_FLEX16)
    stats = rt.stats_alloc(1)
    sb = FusedSpecBuilder([n])
    ta = sb.tensor(a_d.ptr, [1], NGH_FLEX16, scale=2.0 ** -8)
    to = sb.tensor(o_d.ptr, [1], NGH_FLEX16, scale=2.0 ** -8, dev_stats=stats)
    sb.store(to, sb.binary("mul", sb.load(ta), sb.constant(2.0)))
    rt.launch_fused(sb.build())
    want = fm.quantize_rni(fm.dequantize(a, 8) * f32(2), 8)
    np.testing.assert_array_equal(o_d.get(), want)
    assert rt.stats_read(stats, 1)[0] == fm.maxabs(want)
    for d in (x_d, y_d, z_d, a_d, o_d):
        d.free()


@gpu
def test_flex_saturation_nan_and_statistics(hip_runtime):
    rt = hip_runtime
    vals = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 40000, -40000, np.nan, np.inf, -np.inf,
                     32767.49, 32767.5, -32768.5, 0.0, 1e-30], dtype=f32)
    x_d, o_d = rt.array(vals), rt.empty(vals.shape, NGH_FLEX16)
    stats = rt.stats_alloc(1)
    sb = FusedSpecBuilder([vals.size])
    tx = sb.tensor(x_d.ptr, [1])
    to = sb.tensor(o_d.ptr, [1], NGH_FLEX16, scale=1.0, dev_stats=stats)
    sb.store(to, sb.load(tx))
    rt.launch_fused(sb.build())
    want = fm.quantize_rni(vals, 0)
    assert want.tolist()[:11] == [0, 2, 2, 0, -2, -2, 32767, -32768, 0, 32767, -32768]
    np.testing.assert_array_equal(o_d.get(), want)
    assert rt.stats_read(stats, 1)[0] == 32768
    x_d.free()
    o_d.free()


@gpu
def test_fp16_storage(hip_runtime):
    rt = hip_runtime
    rs = np.random.RandomState(3)
    for n in (8, 24, 1000, 1003):
        x = rs.normal(0, 1, n).astype(np.float16)
        x_d, y_d = rt.array(x), rt.empty((n,), NGH_F16)
        sb = FusedSpecBuilder([n])
        tx, ty = sb.tensor(x_d.ptr, [1], NGH_F16), sb.tensor(y_d.ptr, [1], NGH_F16)
        sb.store(ty, sb.binary("add", sb.unary("sqr", sb.load(tx)), sb.constant(1.0)))
        rt.launch_fused(sb.build())
        want = (x.astype(f32) * x.astype(f32) + f32(1)).astype(np.float16)
        np.testing.assert_array_equal(y_d.get(), want)
        x_d.free()
        y_d.free()


@gpu
def test_misaligned_and_broadcast_operands(hip_runtime):
    rt = hip_runtime
    rs = np.random.RandomState(4)
    base = rs.normal(0, 1, (37, 67)).astype(f32)
    col, row = rs.normal(0, 1, 37).astype(f32), rs.normal(0, 1, 67).astype(f32)
    b_d, c_d, r_d = rt.array(base), rt.array(col), rt.array(row)
    sub = base[3:30, 5:66]                       # odd offset: no 16-byte alignment
    o_d = rt.empty(sub.shape)
    sb = FusedSpecBuilder(sub.shape)
    tb = sb.tensor(b_d.ptr + (3 * 67 + 5) * 4, [67, 1])
    tc = sb.tensor(c_d.ptr + 3 * 4, [1, 0])
    tr = sb.tensor(r_d.ptr + 5 * 4, [0, 1])
    to = sb.tensor(o_d.ptr, [sub.shape[1], 1])
    sb.store(to, sb.binary("add", sb.binary("mul", sb.load(tb), sb.load(tc)), sb.load(tr)))
    rt.launch_fused(sb.build())
    np.testing.assert_allclose(o_d.get(), sub * col[3:30, None] + row[None, 5:66], rtol=1e-6)
    for d in (b_d, c_d, r_d, o_d):
        d.free()


@gpu
@pytest.mark.parametrize("shape", [(5, 7, 11), (64, 64), (128, 70), (3, 130, 66), (2, 3, 4, 5), (256, 192),
                                   (4, 96, 200), (8, 1024)])
@pytest.mark.parametrize("itemsize", [4, 2, 1])
def test_strided_copy_all_permutations(hip_runtime, shape, itemsize):
    """Dimshuffle: every axis permutation against numpy.transpose (tensor_ops.py:137-204)."""
    from ngraph_hip.runtime import NGH_U8
    rt = hip_runtime
    dt = {4: np.float32, 2: np.int16, 1: np.uint8}[itemsize]
    code = {4: NGH_F32, 2: NGH_FLEX16, 1: NGH_U8}[itemsize]
    src = (np.arange(int(np.prod(shape))) % (251 if itemsize == 1 else 30011)).astype(dt).reshape(shape)
    s_d = rt.array(src, code)
    perms = list(itertools.permutations(range(len(shape))))
    for perm in perms[:: max(1, len(perms) // 8)] + [perms[-1]]:
        want = np.ascontiguousarray(src.transpose(perm))
        d_d = rt.empty(want.shape, code)
        src_strides = [src.strides[p] // itemsize for p in perm]
        dst_strides = [s // itemsize for s in want.strides]
        rt.copy_strided(d_d.ptr, s_d.ptr, want.shape, dst_strides, src_strides, itemsize)
        np.testing.assert_array_equal(d_d.get(), want)
        d_d.free()
    s_d.free()


@gpu
@pytest.mark.parametrize("rows,cols", [(8192, 4096), (8000, 4000), (4100, 2052)])
def test_transposes_whose_strides_are_multiples_of_4_kib(hip_runtime, rows, cols):
    """Transposes between buffers whose row pitch is a multiple of 4 KiB take the tiles along
    diagonals (and 128 x 128 tiles when there are enough of them); sub-views leave ragged tiles at
    the edges and must not touch what lies outside them."""
    rt = hip_runtime
    src = np.arange(8192 * 4096, dtype=np.float32).reshape(8192, 4096)
    s_d = rt.array(src)
    d_d = rt.empty((4096, 8192))
    rt.memset32(d_d.ptr, 0x7fc00000, 4096 * 8192)
    # dst[c, r] = src[r, c] for r < rows, c < cols
    rt.copy_strided(d_d.ptr, s_d.ptr, (cols, rows), (8192, 1), (1, 4096), 4)
    got = d_d.get()
    np.testing.assert_array_equal(got[:cols, :rows], src[:rows, :cols].T)
    assert np.isnan(got[cols:, :]).all() and np.isnan(got[:, rows:]).all()
    s_d.free()
    d_d.free()


@gpu
def test_strided_copy_argument_checks(hip_runtime):
    from ngraph_hip.runtime import HipLibraryError
    rt = hip_runtime
    a = rt.empty((16,))
    rt.copy_strided(a.ptr, a.ptr, (1 << 40, 0, 3), (0, 0, 1), (0, 0, 1), 4)       # empty: nothing to do
    for shape in [(1 << 62, 4), (1 << 31, 1), (1 << 16, 1 << 16), (-1, 4)]:
        with pytest.raises(HipLibraryError):
            rt.copy_strided(a.ptr, a.ptr, shape, (0, 1), (0, 1), 4)
    with pytest.raises(HipLibraryError):
        rt.copy_strided(a.ptr, a.ptr, (4,), (1,), (1,), 8)
    a.free()


@gpu
@pytest.mark.parametrize("offset", [0, 4, 3])
def test_strided_copy_of_row_slices(hip_runtime, offset):
    """Rows contiguous in both views (the 16-byte path when aligned, element-wise otherwise):
    a column window of a wider matrix, at aligned and unaligned starting columns."""
    rt = hip_runtime
    base = np.arange(70 * 200, dtype=np.float32).reshape(70, 200)
    s_d = rt.array(base)
    want = np.ascontiguousarray(base[5:65, offset:offset + 128])
    d_d = rt.empty(want.shape)
    rt.copy_strided(d_d.ptr, s_d.ptr + (5 * 200 + offset) * 4, want.shape, [128, 1], [200, 1], 4)
    np.testing.assert_array_equal(d_d.get(), want)
    # and scattered back into a wider destination
    w_d = rt.array(np.zeros((60, 200), np.float32))
    rt.copy_strided(w_d.ptr + offset * 4, d_d.ptr, want.shape, [200, 1], [128, 1], 4)
    back = w_d.get()
    np.testing.assert_array_equal(back[:, offset:offset + 128], want)
    assert not back[:, :offset].any() and not back[:, offset + 128:].any()
    for d in (s_d, d_d, w_d):
        d.free()


@gpu
def test_empty_scalar_and_unit_axes_graphs():
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        E, U, A = ng.make_axis(0, name="E"), ng.make_axis(1, name="U"), ng.make_axis(6, name="A")
        x0 = ng.placeholder([E, A])
        x1 = ng.placeholder([U, A])
        s = ng.placeholder(())
        f0 = t.computation(x0 * 2 + 1, x0)
        f1 = t.computation([ng.sum(x1, reduction_axes=[U]), ng.sum(x1, reduction_axes=[A]),
                            ng.sum(x1), ng.max(x1 * s, reduction_axes=[U, A])], x1, s)
        assert f0(np.zeros((0, 6), f32)).shape == (0, 6)
        v = np.arange(6, dtype=f32).reshape(1, 6)
        a, b, c, d = f1(v, 3.0)
        np.testing.assert_allclose(a, v[0])
        np.testing.assert_allclose(b, [15.0])
        np.testing.assert_allclose(c, 15.0)
        np.testing.assert_allclose(d, 15.0)
    finally:
        t.close()


@gpu
def test_strided_host_io_through_views():
    """Placeholders fed through transposed / sliced views (gputransform.py:873-909)."""
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        A, B = ng.make_axis(5, name="A"), ng.make_axis(9, name="B")
        x = ng.placeholder([A, B])
        xt = ng.axes_with_order(x, [B, A])
        f = t.computation([xt, ng.tensor_slice(x, [slice(1, 4), slice(2, 9)]), xt + 1], x)
        v = np.arange(45, dtype=f32).reshape(5, 9)
        r_t, r_s, r_p = f(v)
        np.testing.assert_array_equal(r_t, v.T)
        np.testing.assert_array_equal(r_s, v[1:4, 2:9])
        np.testing.assert_array_equal(r_p, v.T + 1)
        view = t.get_tensor_description_tensor_view(xt.tensor_description())
        view[...] = (v.T * 2)
        np.testing.assert_array_equal(t.get_op_tensor_view(x).get(None), v * 2)
    finally:
        t.close()


@gpu
@pytest.mark.parametrize("nbytes", [1, 4093, (4 << 20) - 4, 4 << 20, (16 << 20) + 1, (65 << 20) + 7, 136 << 20])
def test_host_copies_of_every_size_arrive_intact(hip_runtime, nbytes):
    """Copies below 4 MiB are left to the runtime; from there on they travel through the
    context's ring of four 16 MiB pinned buffers, filled and drained by host threads: sizes
    around the threshold, around a slot, ragged tails, and more chunks than the ring has
    slots, into a destination array whose pages have never been touched."""
    rt = hip_runtime
    src = np.random.RandomState(nbytes % 1000).randint(0, 256, nbytes).astype(np.uint8)
    dev = rt.malloc(nbytes)
    try:
        rt.memcpy_h2d(dev, src)
        back = np.empty(nbytes, dtype=np.uint8)
        rt.memcpy_d2h(back, dev)
        np.testing.assert_array_equal(back, src)
        # a second round through the same slots, other data, offset source and destination
        src2 = (src[::-1].copy() ^ 0x5a)[1:]
        rt.memcpy_h2d(dev + 1, src2) if nbytes > 1 else None
        back2 = np.empty(nbytes, dtype=np.uint8)
        rt.memcpy_d2h(back2, dev)
        assert back2[0] == src[0]
        np.testing.assert_array_equal(back2[1:], src2)
    finally:
        rt.free(dev)


@gpu
def test_keyed_host_writes_move_only_the_addressed_window():
    """tensor[key] = value for keys of integers and slices is a copy of the window alone (a
    contiguous copy in, a strided copy on the device); every other key reads the tensor back,
    patches it and writes it again.  Both must give what NumPy gives (gputransform.py:807-871)."""
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        A, B, C = ng.make_axis(6, name="A"), ng.make_axis(10, name="B"), ng.make_axis(7, name="C")
        x = ng.placeholder([A, B, C])
        f = t.computation(x * 1.0, x)
        rs = np.random.RandomState(3)
        want = rs.uniform(-1, 1, (6, 10, 7)).astype(f32)
        f(want)
        view = t.get_op_tensor_view(x)
        keys = [(slice(1, 4),), (2,), (-1, slice(None), 3), (slice(None), slice(2, 9, 3)), (Ellipsis, 5),
                (slice(0, 6, 2), Ellipsis, slice(1, 7, 2)), (1, 2, 3), (slice(4, 2),),
                (slice(None), [0, 3, 9]), (want[:, 0, 0] > 0,), (slice(5, None, -1),)]
        reads_before = []
        for i, key in enumerate(keys):
            value = rs.uniform(-1, 1, want[key].shape).astype(f32) if i % 2 else f32(i + 0.5)
            want[key] = value
            view[key] = value
            np.testing.assert_array_equal(view.get(None), want, err_msg=str(key))
        assert view._window_of((slice(None), [0, 3, 9])) is None            # fancy keys take the long way
        assert view._window_of((slice(1, 4),)) == (70, [3, 10, 7], [70, 7, 1])
        # through a transposed view of the same buffer
        xt = t.get_tensor_description_tensor_view(ng.axes_with_order(x, [C, A, B]).tensor_description())
        patch = rs.uniform(-1, 1, (2, 6, 4)).astype(f32)
        xt[1:3, :, 2:6] = patch
        want.transpose(2, 0, 1)[1:3, :, 2:6] = patch
        np.testing.assert_array_equal(view.get(None), want)
    finally:
        t.close()


@gpu
def test_library_rejects_bad_launches(hip_runtime):
    rt = hip_runtime
    x_d = rt.array(np.zeros(16, f32))
    sb = FusedSpecBuilder([16])
    t0 = sb.tensor(x_d.ptr, [1])
    sb.store(t0, sb.load(t0))
    spec = sb.build()
    spec.abi_version = 99
    with pytest.raises(HipLibraryError):
        rt.launch_fused(spec)
    spec.abi_version = 1
    spec.tensors[0].dtype = 17
    with pytest.raises(HipLibraryError):
        rt.launch_fused(spec)
    with pytest.raises(HipLibraryError):
        rt.copy_strided(x_d.ptr, x_d.ptr, [4, 4], [4, 1], [1, 4], 3)
    x_d.free()
