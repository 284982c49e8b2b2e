"""ngh_moments_f32_noalloc: the variant of ngh_moments_f32 that allocates nothing (its partial
sums and arrival counters live in a fixed device array inside the library) must give what
ngh_moments_f32 gives.  Both run the same kernel over the same segments and merge them in the
same order, so the comparison is exact; against float64 NumPy the tolerance is the fp32 one of
the moments tests.  Two calls in a row share the array, the second on a smaller input.
"""
import numpy as np
import pytest

from conftest import default_kernel_choice

from ngraph_hip.runtime.hiplib import HipLibraryError

pytestmark = pytest.mark.gpu

f32 = np.float32


def _both(rt, x, eps=1e-5):
    rows, R = x.shape
    stride = (R + 3) // 4 * 4                      # rows start on 16-byte boundaries
    padded = np.full((rows, stride), 1e30, f32)    # the padding must not be read
    padded[:, :R] = x
    x_d = rt.array(padded)
    outs = []
    for fn in (rt.moments_f32, rt.moments_f32_noalloc):
        o_d = rt.empty((3, rows))
        rt.memset32(o_d.ptr, 0x7fc00000, 3 * rows)             # NaN: every word must be written
        fn(x_d.ptr, rows, R, stride, o_d.ptr, o_d.ptr + 4 * rows, o_d.ptr + 8 * rows, eps)
        outs.append(o_d.get())
        o_d.free()
    x_d.free()
    return outs


def test_noalloc_moments_equal_the_allocating_entry_point(hip_runtime):
    rt = hip_runtime
    rs = np.random.RandomState(11)
    # first call: many segments per row; second: smaller, other segmenting, rows not a power of two;
    # third: more rows than compute units (one segment each), R not a multiple of 4
    # then many short rows, which a wavefront each reduces without any scratch (whole float4s
    # only, a ragged end, rows shorter than a float4, the longest rows that go this way)
    for rows, R in ((256, 100352), (37, 4100), (3000, 515), (8192, 64), (4500, 1027), (5000, 3), (4096, 4096)):
        x = rs.normal(0.5, 2.0, (rows, R)).astype(f32)
        want, got = _both(rt, x)
        assert not np.isnan(got).any()
        np.testing.assert_array_equal(got, want)
        x64 = x.astype(np.float64)
        np.testing.assert_allclose(got[0], x64.mean(axis=1), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(got[1], x64.var(axis=1), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(got[2], 1.0 / np.sqrt(x64.var(axis=1) + 1e-5), rtol=1e-5, atol=1e-6)


def test_noalloc_moments_reject_what_the_fixed_scratch_cannot_hold(hip_runtime):
    if not default_kernel_choice():
        pytest.skip("a kernel-choice knob of the library is set: rows of 8192 elements may then take "
                    "the wavefront-per-row kernel, which needs no scratch and has no such limit")
    rt = hip_runtime
    rows, R = 70000, 8192
    # (buffers of the sizes the call describes: a refusal must not be what keeps it in bounds)
    x_d, o_d = rt.empty((rows, R)), rt.empty((3, rows))
    with pytest.raises(HipLibraryError) as e:
        # 70000 rows of 8192 elements: more arrival counters than the array has; nothing is launched
        rt.moments_f32_noalloc(x_d.ptr, rows, R, 0, o_d.ptr, o_d.ptr + 4 * rows, o_d.ptr + 8 * rows, 0.0)
    assert e.value.code == -4 and "scratch" in str(e.value)
    x_d.free()
    o_d.free()
