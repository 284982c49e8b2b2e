"""Corrupted kernel specs against the library's validator and planner (host code, no GPU).

A spec that reaches a kernel indexes the tensor table, the constant table, the register
file and the reduction slots with the numbers it carries, so the validator has to refuse
every spec whose numbers point outside those tables.  The cases here start from specs the
builder makes, overwrite fields at random, and check that
  * validating and planning never crash, whatever the bytes are, and
  * whatever the validator accepts passes an independent statement of the table bounds
    written below (so "accepted" implies "indexes nothing out of range").
"""
import ctypes
import random

import numpy as np
import pytest

from ngraph_hip.runtime import FusedSpecBuilder, NGH_F32, NGH_FLEX16, NGH_I32, load_library
from ngraph_hip.runtime import hiplib
from ngraph_hip.runtime.hiplib import (OPCODES, UNARY_OPS, BINARY_OPS, REDUCTION_OPS, NGH_MAX_TENSORS,
                                       NGH_MAX_OPS, NGH_MAX_CONSTS, NGH_MAX_REGS, NGH_MAX_REDUCTIONS)

FAKE = 0x7f0000000000          # never dereferenced: nothing here launches


def _strides(shape):
    out, acc = [], 1
    for s in reversed(shape):
        out.insert(0, acc)
        acc *= s
    return out


def base_specs():
    specs = []
    # elementwise chain with a broadcast operand and a constant
    shape = (64, 96)
    sb = FusedSpecBuilder(shape)
    x = sb.load(sb.tensor(FAKE, _strides(shape)))
    b = sb.load(sb.tensor(FAKE + (1 << 24), [0, 1]))
    y = sb.binary("add", sb.unary("tanh", sb.binary("mul", x, sb.constant(0.5))), b)
    sb.store(sb.tensor(FAKE + (2 << 24), _strides(shape)), y)
    specs.append(sb.build())
    # two reductions over axis 0 followed by a second stage that uses them
    shape = (200, 48)
    sb = FusedSpecBuilder(shape)
    tx = sb.tensor(FAKE, _strides(shape))
    ts, tm = sb.tensor(FAKE + (1 << 24), [0, 1]), sb.tensor(FAKE + (2 << 24), [0, 1], NGH_I32)
    x = sb.load(tx)
    sb.reduce("sum", x, ts)
    sb.reduce("argmax", x, tm)
    sb.end_stage()
    y = sb.binary("sub", sb.load(tx), sb.load(ts))
    sb.store(sb.tensor(FAKE + (3 << 24), _strides(shape)), y)
    specs.append(sb.build())
    # flex operands, a gather, an iota and a random number
    shape = (8, 16, 32)
    sb = FusedSpecBuilder(shape)
    q = sb.load(sb.tensor(FAKE, _strides(shape), NGH_FLEX16, scale=2.0 ** -10))
    idx = sb.load(sb.tensor(FAKE + (1 << 24), [0, 32, 1], NGH_I32))
    table = sb.tensor(FAKE + (2 << 24), [50, 0, 1], take_extent=50)
    g = sb.take(table, idx, 0)
    r = sb.rng("uniform", 0)
    y = sb.binary("mul", sb.binary("add", q, g), sb.binary("add", r, sb.iota(2)))
    sb.store(sb.tensor(FAKE + (3 << 24), _strides(shape), NGH_FLEX16, scale=2.0 ** -8,
                       dev_stats=FAKE + (4 << 24)), y)
    specs.append(sb.build())
    return specs


def accepted_spec_is_in_bounds(sp):
    """The table bounds, restated: returns a reason string when a number in `sp` indexes
    outside a table, else None."""
    unary = set(OPCODES[n] for n in UNARY_OPS)
    binary = set(OPCODES[n] for n in BINARY_OPS)
    reduce_ = set(OPCODES[n] for n in REDUCTION_OPS)
    if not (1 <= sp.rank <= 3) or not (0 <= sp.n_tensors <= NGH_MAX_TENSORS):
        return "rank / n_tensors"
    if not (0 <= sp.n_ops <= NGH_MAX_OPS and 0 <= sp.n_consts <= NGH_MAX_CONSTS and 0 <= sp.n_regs <= NGH_MAX_REGS):
        return "table sizes"
    if any(s < 0 for s in sp.shape):
        return "negative shape"
    if sp.shape[0] * sp.shape[1] * sp.shape[2] > (1 << 33):         # Python integers: no wrap
        return "iteration space wraps 64-bit arithmetic or exceeds the kernels' counters"
    for t in range(sp.n_tensors):
        reach = sum((n - 1) * st for n, st in zip(sp.shape, sp.tensors[t].strides) if n > 1)
        if reach * 4 >= (1 << 63):
            return "element offsets wrap 64-bit arithmetic"
        if sp.tensors[t].dtype not in range(8):
            return "dtype"
        if any(s < 0 for s in sp.tensors[t].strides):
            return "negative stride"
    nxt = 0
    for s in range(sp.n_stages):
        st = sp.stages[s]
        if st.op_begin != nxt or not (st.op_begin <= st.op_end <= sp.n_ops):
            return "stage range"
        nxt = st.op_end
        if not (0 <= st.n_reductions <= NGH_MAX_REDUCTIONS):
            return "n_reductions"
        defined, slots = set(), 0
        for pc in range(st.op_begin, st.op_end):
            o = sp.ops[pc]
            name = hiplib._OPCODE_NAMES[o.opcode] if o.opcode < len(hiplib._OPCODE_NAMES) else None
            if name is None:
                return "opcode"
            reads, writes, tensors = [], None, []
            if name == "load":
                tensors, writes = [o.a], o.dst
            elif name in ("store", "store_trunc"):
                tensors, reads = [o.dst], [o.a]
            elif name == "const":
                if o.a >= sp.n_consts:
                    return "const index"
                writes = o.dst
            elif name in ("rng_uniform", "rng_normal"):
                writes = o.dst
            elif name == "iota":
                if o.a >= 3:
                    return "iota axis"
                writes = o.dst
            elif name == "take":
                tensors, reads, writes = [o.b & 15], [o.a], o.dst
                if (o.b >> 4) >= sp.rank:
                    return "take axis"
            elif o.opcode in unary:
                reads, writes = [o.a], o.dst
            elif o.opcode in binary:
                reads, writes = [o.a, o.b], o.dst
            elif o.opcode in reduce_:
                reads = [o.a]
                if o.dst != slots or slots >= st.n_reductions:
                    return "reduction slot"
                tensors = [st.red_out[slots]]
                slots += 1
            elif name != "nop":
                return "unclassified opcode %s" % name
            if any(t < 0 or t >= sp.n_tensors for t in tensors):
                return "tensor index"
            if any(r >= sp.n_regs or r not in defined for r in reads):
                return "register read before definition"
            if writes is not None:
                if writes >= sp.n_regs:
                    return "register index"
                defined.add(writes)
    if nxt != sp.n_ops:
        return "ops outside stages"
    return None


def clone(spec):
    out = hiplib.ngh_fused_spec()
    ctypes.memmove(ctypes.byref(out), ctypes.byref(spec), ctypes.sizeof(spec))
    return out


def mutate(sp, rnd):
    kind = rnd.randrange(12)
    n_ops = max(1, min(sp.n_ops, NGH_MAX_OPS))
    if kind == 0:
        o = sp.ops[rnd.randrange(n_ops)]
        setattr(o, rnd.choice(["opcode", "dst", "a", "b"]), rnd.randrange(256))
    elif kind == 1:
        o = sp.ops[rnd.randrange(n_ops)]
        o.opcode = rnd.randrange(len(hiplib._OPCODE_NAMES) + 3)
    elif kind == 2:
        setattr(sp, rnd.choice(["n_tensors", "n_ops", "n_consts", "n_regs", "n_stages", "rank"]),
                rnd.choice([-1, 0, 1, 2, 3, 5, 31, 32, 33, 96, 97, 255, 1 << 30]))
    elif kind == 3:
        st = sp.stages[rnd.randrange(4)]
        setattr(st, rnd.choice(["op_begin", "op_end", "n_reductions"]), rnd.choice([-5, 0, 1, 2, 4, 5, 7, 200]))
    elif kind == 4:
        sp.stages[rnd.randrange(4)].red_out[rnd.randrange(NGH_MAX_REDUCTIONS)] = rnd.choice([-1, 0, 3, 11, 12, 99])
    elif kind == 5:
        sp.shape[rnd.randrange(3)] = rnd.choice([-3, 0, 1, 2, 7, 64, 1 << 20, 1 << 40, (1 << 62)])
    elif kind == 6:
        sp.tensors[rnd.randrange(NGH_MAX_TENSORS)].strides[rnd.randrange(3)] = rnd.choice([-1, 0, 1, 3, 4, 1 << 33])
    elif kind == 7:
        sp.tensors[rnd.randrange(NGH_MAX_TENSORS)].dtype = rnd.choice([-1, 0, 1, 2, 3, 4, 5, 6, 7, 8, 100])
    elif kind == 8:
        sp.tensors[rnd.randrange(NGH_MAX_TENSORS)].dev = rnd.choice([0, FAKE + 1, FAKE + 2, FAKE + 6, FAKE + 64])
    elif kind == 9:
        sp.tensors[rnd.randrange(NGH_MAX_TENSORS)].take_extent = rnd.choice([0, 1, 1 << 31])
    elif kind == 10:
        sp.flags = rnd.randrange(1 << 8)
    else:
        raw = (ctypes.c_uint8 * ctypes.sizeof(sp)).from_address(ctypes.addressof(sp))
        raw[rnd.randrange(len(raw))] = rnd.randrange(256)


@pytest.mark.parametrize("seed", range(8))
def test_corrupted_specs_are_refused_or_in_bounds(seed):
    lib = load_library()
    rnd = random.Random(seed)
    bases = base_specs()
    for sp in bases:
        assert lib.ngh_validate_fused(ctypes.byref(sp)) == 0
        assert accepted_spec_is_in_bounds(sp) is None
    accepted = refused = 0
    out8 = (ctypes.c_int32 * 8)()
    for _ in range(1500):
        sp = clone(rnd.choice(bases))
        for _ in range(rnd.choice([1, 1, 1, 2, 3, 6])):
            mutate(sp, rnd)
        rc = lib.ngh_validate_fused(ctypes.byref(sp))
        for stage in (-1, 0, 1, 2, 3, 4, 9):
            prc = lib.ngh_plan_fused(ctypes.byref(sp), stage, out8)
            if rc != 0 or not (0 <= stage < sp.n_stages):
                assert prc != 0, "planned stage %d of a spec the validator refuses / does not hold" % stage
        if rc == 0:
            accepted += 1
            why = accepted_spec_is_in_bounds(sp)
            assert why is None, why
        else:
            refused += 1
            assert lib.ngh_last_error()
    assert accepted > 50 and refused > 200, (accepted, refused)


def test_plan_is_a_function_of_the_spec_only():
    """Planning twice gives the same answer, and does not write to the spec."""
    lib = load_library()
    out_a, out_b = (ctypes.c_int32 * 8)(), (ctypes.c_int32 * 8)()
    for sp in base_specs():
        before = bytes((ctypes.c_uint8 * ctypes.sizeof(sp)).from_address(ctypes.addressof(sp)))
        for stage in range(sp.n_stages):
            assert lib.ngh_plan_fused(ctypes.byref(sp), stage, out_a) == 0
            assert lib.ngh_plan_fused(ctypes.byref(sp), stage, out_b) == 0
            assert list(out_a) == list(out_b)
        after = bytes((ctypes.c_uint8 * ctypes.sizeof(sp)).from_address(ctypes.addressof(sp)))
        assert before == after
    assert np.dtype(np.float32).itemsize == 4 and NGH_F32 == 0


@pytest.mark.parametrize("shape", [(1 << 62, 4), (1 << 32, 1 << 32), (1 << 33, 2), (3, 1 << 62)])
def test_iteration_spaces_that_wrap_are_refused(shape):
    """2^62 x 4 is 0 in 64-bit arithmetic; such a spec must not pass for an empty one."""
    lib = load_library()
    sb = FusedSpecBuilder((4, 4))
    sb.store(sb.tensor(FAKE + (1 << 24), [4, 1]), sb.load(sb.tensor(FAKE, [4, 1])))
    sp = sb.build()
    assert lib.ngh_validate_fused(ctypes.byref(sp)) == 0
    sp.shape[0], sp.shape[1] = shape
    assert lib.ngh_validate_fused(ctypes.byref(sp)) != 0
    sp.shape[0], sp.shape[1] = 4, 4
    sp.tensors[0].strides[0] = 1 << 61
    assert lib.ngh_validate_fused(ctypes.byref(sp)) != 0


def test_indices_beyond_fp32_exactness_are_refused_not_rounded():
    """Registers are fp32 (integers exact to 2^24; the reference keeps int32 operands in integer
    registers, float_ew2.py:615-641).  Where an index could exceed that, the spec is refused:
    a lookup in a table longer than 2^24 along the looked-up axis, an index value along an axis
    longer than 2^24, an argmax over more than 2^24 elements into anything but int32 / uint32."""
    lib = load_library()
    big = (1 << 24) + 8

    def rc(sb):
        return lib.ngh_validate_fused(ctypes.byref(sb.build()))

    for extent, want in ((1 << 24, 0), (big, -4)):
        sb = FusedSpecBuilder([64, 8])
        idx = sb.load(sb.tensor(FAKE, [1, 0], NGH_I32))
        table = sb.tensor(FAKE + (1 << 30), [8, 1], take_extent=extent)
        sb.store(sb.tensor(FAKE + (2 << 30), [8, 1]), sb.take(table, idx, 0))
        assert rc(sb) == want, lib.ngh_last_error()
    for n, want in ((1 << 24, 0), (big, -4)):
        sb = FusedSpecBuilder([n])
        sb.store(sb.tensor(FAKE, [1]), sb.iota(0))
        assert rc(sb) == want, lib.ngh_last_error()
        assert want == 0 or b"2^24" in lib.ngh_last_error()
    for dtype, want in ((NGH_I32, 0), (hiplib.NGH_U32, 0), (NGH_F32, -4), (hiplib.NGH_I16, -4)):
        sb = FusedSpecBuilder([big, 4])
        x = sb.load(sb.tensor(FAKE, [4, 1]))
        sb.reduce("argmax", x, sb.tensor(FAKE + (1 << 32), [0, 1], dtype))
        assert rc(sb) == want, (dtype, lib.ngh_last_error())
    # a sum over as many elements is fine in any type
    sb = FusedSpecBuilder([big, 4])
    sb.reduce("sum", sb.load(sb.tensor(FAKE, [4, 1])), sb.tensor(FAKE + (1 << 32), [0, 1]))
    assert rc(sb) == 0
