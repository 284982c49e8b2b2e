"""Pins of the flex oracle (oracle/flex_model.py) and of the product's exponent policy.
No GPU needed.

* rounding / saturation / maxabs given a scale: brute force over every int16 mantissa and
  half-way point against an independent exact (fractions) implementation of
  round-half-even + clamp, the semantics of cvt.rni.s16.f32 (float_ew2.py:261-267);
* the whole model (arithmetic + exponent policy) against the reference's known-answer
  vectors, tests/golden/flex_vectors.json;
* the product's policy (ngraph_hip.flex.hipflex) against the oracle's on random histories.
"""
import fractions
import json
import os

import numpy as np
import pytest

from oracle import flex_model as fm
from ngraph_hip.flex import HipFlexManager, hipflex16

HERE = os.path.dirname(os.path.abspath(__file__))
VECTORS = json.load(open(os.path.join(HERE, "golden", "flex_vectors.json")))


def exact_rni_sat(value):
    fr = fractions.Fraction(float(value))
    lo = fr.numerator // fr.denominator
    rem = fr - lo
    if rem > fractions.Fraction(1, 2) or (rem == fractions.Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    return max(-32768, min(32767, lo))


def test_rni_saturation_brute_force():
    for dec in (0, 3, 8, 14):
        m = np.arange(-32768, 32768, dtype=np.int64)
        # every representable value round-trips exactly
        assert np.array_equal(fm.quantize_rni(fm.dequantize(m.astype(np.int16), dec), dec), m)
        # half-way points go to the even neighbour, out-of-range saturates
        for offs in (0.5, -0.5, 0.25, 0.75, 0.49999, 40000.0, -40000.0):
            vals = ((m + offs) * 2.0 ** -dec).astype(np.float32)
            got = fm.quantize_rni(vals, dec).astype(np.int64)
            step = 257 if abs(offs) < 1 else 4099
            for i in range(0, len(m), step):
                want = exact_rni_sat(np.float32(vals[i]) * np.float32(2.0 ** dec))
                assert got[i] == want, (dec, offs, vals[i], got[i], want)
    assert fm.quantize_rni(np.array([np.nan, np.inf, -np.inf], np.float32), 0).tolist() == [0, 32767, -32768]


def test_host_write_truncates_and_kernel_store_rounds():
    # test_redop.py:117-120: 1.2 -> 19660 * 2^-14 (nearest would be 19661)
    assert fm.quantize_host(1.2, 14) == 19660 and fm.quantize_host(1.4, 14) == 22937
    # test_complex_math.py:47: log(0.01) -> -18863 * 2^-12 (truncation would give -18862)
    assert fm.quantize_rni(np.float32(-18862.9 / 4096), 12) == -18863
    assert fm.maxabs(np.array([-32768, 5], np.int16)) == 32768


def _run_case(case):
    op, steps = case["op"], case["steps"]
    first = steps[0]["in"]
    shp = np.asarray(first[0]).shape
    if op == "assign":
        # FlexAssignKernel is a host round trip (tensor_ops.py:664-677)
        p, v, outs = fm._SimTensor(()), fm._SimTensor(()), []
        for s in steps:
            p.host_write(s["in"][0])
            v.host_write(p.host_read())
            outs.append(v.host_read())
        return outs
    if op == "sigmoid":
        shapes = {"x": shp, "one": (), "n": shp, "e": shp, "a": shp, "out": shp}
        sim = fm.FlexSim([("neg", "n", "x"), ("exp", "e", "n"), ("add", "a", "e", "one"),
                          ("rcp", "out", "a")], shapes)
        sim.tensors["one"].host_write(1.0)
        return [sim.run({"x": s["in"][0]}, "out") for s in steps]
    if op == "safelog":
        # ng.safelog is maximum(log(x + exp(-50)), -50) (op_graph.py:3070-3072): three kernels on
        # the unfused flex transformer, the two constants written from the host like any tensor
        shapes = {"x": shp, "off": (), "lim": (), "a": shp, "l": shp, "out": shp}
        sim = fm.FlexSim([("add", "a", "x", "off"), ("log", "l", "a"), ("maximum", "out", "l", "lim")], shapes)
        sim.tensors["off"].host_write(np.exp(-50.0))
        sim.tensors["lim"].host_write(-50.0)
        return [sim.run({"x": s["in"][0]}, "out") for s in steps]
    if len(first) == 1:
        red = op in ("sum", "prod", "max", "min", "argmax", "argmin")
        sim = fm.FlexSim([(op, "out", "x")], {"x": shp, "out": () if red else shp})
        return [sim.run({"x": s["in"][0]}, "out") for s in steps]
    shapes = {"x": np.asarray(first[0]).shape, "y": np.asarray(first[1]).shape,
              "out": np.broadcast(np.asarray(first[0]), np.asarray(first[1])).shape}
    sim = fm.FlexSim([(op, "out", "x", "y")], shapes)
    return [sim.run({"x": s["in"][0], "y": s["in"][1]}, "out") for s in steps]


def flex_close(got, want, single):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    if single:
        return np.array_equal(got, want)
    d = fm.fit_dec(np.max(np.abs(want)))
    atol = 8 * 2.0 ** -(fm.DEFAULT_DEC if d is None else d)        # flexgputransform.py:98-103
    return np.allclose(got, want, rtol=1e-2, atol=atol)


@pytest.mark.parametrize("case", [c for c in VECTORS if not c.get("disabled")],
                         ids=lambda c: "%s@%s" % (c["op"], c["source"]))
def test_model_reproduces_reference_vector(case):
    outs = _run_case(case)
    single = len(case["steps"]) == 1
    for step, got in zip(case["steps"], outs):
        assert flex_close(got, step["want"], single), (step, np.asarray(got).tolist())


def test_disabled_vectors_are_the_known_ones():
    """What the model does not reproduce, and why: cases the reference itself disables
    (bug_1064, bug_1227) and argmax/argmin ties, where the vectors record the reference GPU's
    butterfly order (issue #1424) while the CPU transformer, the oracle here, returns the
    first index (np.argmax)."""
    reasons = sorted(set(c["disabled"] for c in VECTORS if c.get("disabled")))
    assert reasons == ["bug_1064", "bug_1227", "issue_1424_thread_order"]
    assert sum(1 for c in VECTORS if c.get("disabled")) == 9


def test_product_policy_matches_oracle_policy():
    rs = np.random.RandomState(5)
    mgr = HipFlexManager()
    for trial in range(200):
        entry, pol = mgr.make_flex_entry("t%d" % trial), fm.FlexPolicy()
        first = float(10.0 ** rs.uniform(-6, 5))
        entry.manage_before_computation(np.array(first))
        pol.init_from_value(first)
        assert entry.dec == pol.dec
        for step in range(40):
            # a mantissa max that sometimes saturates, sometimes collapses
            m = int(rs.choice([0, 1, 7, 300, 5000, 16384, 20000, 32766, 32767, 32768]))
            entry.manage_after_computation(m, step)
            pol.record(m)
            assert entry.next_dec == pol.dec, (trial, step, m)
            entry.adjust_scale()             # the next write happens at the chosen exponent
            assert entry.dec == pol.dec
    assert hipflex16.fit_dec(0.0) is None and hipflex16.fit_dec(np.inf) == 0
    assert hipflex16.fit_dec(1.0) == 14 and hipflex16.fit_dec(32767) == 0 and hipflex16.fit_dec(2 ** -30) == 31
