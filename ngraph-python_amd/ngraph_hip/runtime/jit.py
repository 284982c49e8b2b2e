"""Run-time compilation of the op programs of a computation.

The reference writes CUDA C for every compound kernel of a computation and compiles it with
NVRTC when the transformer is initialised (float_ew2.py:1135-1483 `_get_compound_kernel`,
:1553-1653 `CudaSourceFile`), keeping compiled kernels in a per-process cache keyed by a
structural hash (:1486-1529).  The library here carries compiled kernels for the programs that
dominate training graphs and an interpreter for everything else; this module closes the gap for
a user's own graphs: the stage programs that no compiled kernel covers are written out as the
same C++ tables the built-in ones are made from, compiled by hipcc into a *program library*
(one shared object per program, named by a hash of its table, the kernel headers and the
compiler flags) and handed to the library with `ngh_programs_load`.  The object files are
kept, so a program is compiled once per machine, not once per process.

Opt-in (`make_transformer_factory("hipgpu", jit=True)` or NGH_JIT=1): compiling takes seconds
per program, which pays for kernels that run many times over large tensors and not for a test
suite's thousands of one-shot graphs.
"""
from __future__ import print_function

import hashlib
import os
import subprocess

from ngraph_hip.runtime import hiplib
from ngraph_hip.runtime.programs import stage_programs, render

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))      # .../ngraph_hip
_ROOT = os.path.dirname(_PKG)
CSRC = os.path.join(_ROOT, "csrc")
INCLUDE = os.path.join(os.path.dirname(_ROOT), "include")
_KERNEL_HEADERS = ("ngh_device.h", "ngh_flex.h", "ngh_interp.h", "ngh_special.h")

_TRAILER = """
}  // namespace ngh

extern "C" int ngh_program_library(int abi, unsigned entry_bytes, unsigned args_bytes, const void** out_entries) {
    if (abi != NGH_ABI_VERSION || entry_bytes != sizeof(ngh::StaticEntry) || args_bytes != sizeof(ngh::KArgs))
        return -1;
    *out_entries = ngh::kLoadedTable;
    return ngh::kLoadedCount;
}
"""


def enabled_by_default():
    return os.environ.get("NGH_JIT", "0") not in ("", "0")


def cache_dir():
    """Where program libraries are kept: NGH_PROGRAM_CACHE, else next to libngraph_hip.so."""
    path = os.environ.get("NGH_PROGRAM_CACHE") or os.path.join(_PKG, "lib", "programs")
    os.makedirs(path, exist_ok=True)          # (several threads may get here at once)
    return path


def _flags():
    import build_ext
    return build_ext.HIPCC_FLAGS, build_ext.find_hipcc


def _sources_digest():
    h = hashlib.sha256()
    for name in _KERNEL_HEADERS:
        with open(os.path.join(CSRC, name), "rb") as fh:
            h.update(fh.read())
    with open(os.path.join(INCLUDE, "ngraph_hip.h"), "rb") as fh:
        h.update(fh.read())
    return h.hexdigest()


def source_text(programs):
    header = ["// Program library: op programs of a user's computation, compiled at run time.",
              '#include "ngh_special.h"', "", "namespace ngh {", ""]
    # the struct's name shows in the kernel's name (profilers group by it): make it the program's
    tag = "".join(c if c.isalnum() else "_" for c in programs[0][0]) if programs else "none"
    return render(programs, header, prefix="LP_%s_" % tag, table="kLoadedTable", count="kLoadedCount") + _TRAILER


def compile_programs(programs, verbose=False):
    """The path of a program library holding `programs` (records of programs.stage_programs),
    compiled now unless the cache has it."""
    flags, find_hipcc = _flags()
    text = source_text(programs)
    key = hashlib.sha256((text + _sources_digest() + " ".join(flags)).encode("utf-8")).hexdigest()[:20]
    base = os.path.join(cache_dir(), "ngh_programs_" + key)
    lib = base + ".so"
    if os.path.exists(lib):
        return lib
    src = base + ".hip"
    with open(src, "w") as fh:
        fh.write(text)
    tmp = "%s.%d.tmp" % (lib, os.getpid())
    try:
        hipcc = find_hipcc()
    except RuntimeError:
        raise RuntimeError("run-time compilation (jit=True / NGH_JIT=1) needs hipcc on this machine, or the "
                           "program library %s in the cache; without jit the same stages run on the "
                           "interpreter" % os.path.basename(lib))
    cmd = [hipcc] + list(flags) + ["-I", INCLUDE, "-I", CSRC, src, "-o", tmp]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, universal_newlines=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, proc.stdout))
    os.replace(tmp, lib)          # atomic: another process may be compiling the same programs
    return lib


def uncovered_programs(kernels, name, min_elements=4096, include_covered=False):
    """Records of the stage programs of `kernels` that run on the interpreter today and could run
    as compiled kernels (include_covered: also those that have a compiled kernel already)."""
    out = []
    for p in stage_programs(kernels, name, min_elements=min_elements):
        if p[-1] < 0 or include_covered:
            # named by content: the same program gets the same library in every process,
            # whatever the computation it comes from is called there
            digest = hashlib.sha256(repr(p[1:-1]).encode("utf-8")).hexdigest()[:10]
            out.append(("jit_" + digest,) + tuple(p[1:]))
    return out


def ensure_programs(runtime, kernels, name, min_elements=4096, verbose=False):
    """Compile (or find in the cache) and load kernels for the programs of `kernels` that have
    none; returns the number of programs added to the library's table."""
    programs = uncovered_programs(kernels, name, min_elements)
    if not programs:
        return 0
    # One library per program: what a library holds, and so its name in the cache, depends on the
    # program alone and not on which other programs this process happened to have loaded before.
    if len(programs) == 1:
        paths = [compile_programs(programs, verbose=verbose)]
    else:
        from multiprocessing.pool import ThreadPool          # the work is in hipcc subprocesses
        pool = ThreadPool(min(len(programs), max(1, min(8, (os.cpu_count() or 2) // 2))))
        try:
            paths = pool.map(lambda p: compile_programs([p], verbose=verbose), programs)
        finally:
            pool.close()
    return sum(runtime.programs_load(path) for path in paths)
