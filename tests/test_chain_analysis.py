"""What the stages of a row chain pass each other is worked out at compile time (ChainInfo in
csrc/ngh_special.h): which operands stay in registers, which reduction results are handed on,
which computed values are kept, where a fence is needed.  These tests pin those decisions for two
chains with static_asserts that hipcc evaluates (no device needed)."""
import os
import subprocess

import pytest

from ngraph_hip.runtime import hiplib, jit

import test_jit as chains


def _check(spec, asserts, tmp_path):
    programs = jit.uncovered_programs([chains._SpecHolder(spec)], "chain", min_elements=1, include_covered=True)
    assert len(programs) == 1 and programs[0][8] == 4
    tag = "".join(c if c.isalnum() else "_" for c in programs[0][0])
    stages = ", ".join("LP_%s_0_%d" % (tag, j) for j in range(len(programs[0][1])))
    text = jit.source_text(programs)
    text += "\nnamespace ngh {\nusing Info = ChainInfo<%s>;\n%s\n}\n" % (
        stages, "\n".join('static_assert(%s, "%s");' % (a, a.replace('"', "'")) for a in asserts))
    src = os.path.join(str(tmp_path), "chain_analysis.hip")
    with open(src, "w") as fh:
        fh.write(text)
    flags, find_hipcc = jit._flags()
    cmd = [find_hipcc()] + [f for f in flags if f not in ("-shared", "-fPIC")] + \
        ["-fsyntax-only", "-I", jit.INCLUDE, "-I", jit.CSRC, src]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, universal_newlines=True)
    assert proc.returncode == 0, proc.stdout[-3000:]


def test_softmax_chain_keeps_the_row_the_results_and_the_exponentials_in_registers(tmp_path):
    # tensors: 0 x, 1 y, 2 row maximum, 3 row sum
    # stage 1: load x, load max, sub, exp, sum        stage 2: load x, load max, sub, exp, load sum, div, store
    spec = chains._softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1001, 300)
    _check(spec, [
        "Info::n == 3",
        "Info::cache_slot(0) == 0",                          # x: read from memory by the first stage only
        "Info::first_loader(0) == 0 && Info::last_loader(0) == 2",
        "!Info::from_memory(1, 0) && !Info::from_memory(2, 0)",
        "Info::forwarded(1, 2) >= 0 && Info::forwarded(2, 2) >= 0",   # the maximum, in a register
        "Info::forwarded(2, 3) >= 0",                                  # the sum
        "!Info::needs_fence(1) && !Info::needs_fence(2)",              # nothing goes through memory
        "Info::kept_value(0) >= 0",                                    # exp(x - max): computed once
        "Info::keep_slot(1, 3) == 0 && Info::reuse_slot(2, 3) == 0",
        "Info::keep_slot(1, 2) < 0 && Info::reuse_slot(2, 2) < 0",      # (x - max alone is not worth a slot)
    ], tmp_path)


def test_chain_results_that_cannot_stay_in_registers_wait_behind_a_fence(tmp_path):
    # tensors: 0 x, 1 position of the maximum (int32), 2 t (stored by stage 1, loaded by stage 2), 3 y, 4 sum of t*t
    spec = chains._fenced_chain_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 5 << 30, 777, 3000)
    _check(spec, [
        "Info::n == 3",
        "Info::forwarded(1, 1) < 0 && Info::needs_fence(1)",          # an int32 result is read back from memory
        "Info::stores(1, 2) && Info::loads(2, 2) && Info::cache_slot(2) < 0",
        "Info::from_memory(2, 2) && Info::needs_fence(2)",             # so is a tensor another stage stored
        "Info::forwarded(2, 4) >= 0",                                  # the fp32 sum is handed on
        "Info::cache_slot(0) == 0 && Info::last_loader(0) == 1",       # x: kept for the second stage, not needed by the third
    ], tmp_path)


def test_a_stage_that_overwrites_what_an_earlier_stage_read_waits_too(tmp_path):
    # tensors: 0 x, 1 a per-row factor b (one value per row), 2 the row sum, 3 y
    # stage 0: sum(x)      stage 1: y = x * b, b read from memory      stage 2: b = sum * 0.5, one store per row
    R, rows = 5000, 300
    sb = hiplib.FusedSpecBuilder([R, rows])
    tx, tb = sb.tensor(1 << 30, [1, R]), sb.tensor(2 << 30, [0, 1])
    ts, ty = sb.tensor(3 << 30, [0, 1]), sb.tensor(4 << 30, [1, R])
    sb.reduce("sum", sb.load(tx), ts)
    sb.end_stage()
    sb.store(ty, sb.binary("mul", sb.load(tx), sb.load(tb)))
    sb.end_stage()
    sb.store(tb, sb.binary("mul", sb.load(ts), sb.constant(0.5)))
    spec = sb.build()
    assert hiplib.plan_chain(spec)["eligible"]
    _check(spec, [
        "Info::n == 3",
        "Info::from_memory(1, 1) && !Info::needs_fence(1)",       # b: nobody wrote it before stage 1
        "Info::stores(2, 1) && Info::needs_fence(2)",              # lanes of other wavefronts may still be reading b
        "Info::forwarded(2, 2) >= 0",                              # the sum itself arrives in a register
    ], tmp_path)
