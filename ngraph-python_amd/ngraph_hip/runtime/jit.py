"""Run-time compilation of the op programs of a computation.

The reference writes CUDA C for every compound kernel of a computation and compiles it with
NVRTC when the transformer is initialised (float_ew2.py:1135-1483 `_get_compound_kernel`,
:1553-1653 `CudaSourceFile`), keeping compiled kernels in a per-process cache keyed by a
structural hash (:1486-1529).  The library here carries compiled kernels for the programs that
dominate training graphs and an interpreter for everything else; this module closes the gap for
a user's own graphs: the stage programs that no compiled kernel covers are written out as the
same C++ tables the built-in ones are made from, compiled into a *program library* (one per program, named by a hash of its table, the kernel
headers and the compiler flags) and handed to the library with `ngh_programs_load` or
`ngh_programs_load_code`.  The libraries are kept, so a program is compiled once per machine,
not once per process.  Two compilers (`compiler()`, NGH_JIT_COMPILER): hipcc, run as a
subprocess, makes a shared object with host launchers; hiprtc compiles the same source inside
this process, device code only, into a code object that the library launches through the module
API -- the reference's way (NVRTC), and the one that works on a machine without hipcc.

Three modes (`make_transformer_factory("hipgpu", jit=...)`, default from NGH_JIT, else "auto"):

  "auto"  stages over large tensors (at least `jit_auto_min_elements` elements) that no compiled
          kernel covers are handed to worker threads when the transformer is initialised
          (`jit_after_calls=0`, the default; with n > 0 only once the computation has run n
          times), while the computation starts on the interpreter; the kernel group loads the
          libraries when they are ready and the next launch finds them.  Program libraries
          already in the cache are loaded when the kernels are bound.  Without hipcc on the
          machine the computation simply stays on the interpreter.
  True    every stage of at least `jit_min_elements` elements is compiled before the first
          launch (the reference's behaviour: it compiles a computation's kernels when the
          transformer is initialised); a missing hipcc is an error.
  False   interpreter and built-in programs only.

Compiling takes seconds per program, which pays for kernels that run many times over large
tensors and not for a test suite's thousands of one-shot graphs: hence the size threshold of
the default mode.
"""
from __future__ import print_function

import hashlib
import os
import subprocess
import threading

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


def default_mode():
    """The transformer's jit mode when none is given: NGH_JIT=0 -> False, NGH_JIT=1 -> True,
    anything else (or unset) -> "auto"."""
    v = os.environ.get("NGH_JIT", "auto").strip().lower()
    if v in ("0", "false", "off", "no"):
        return False
    if v in ("1", "true", "on", "yes"):
        return True
    return "auto"


def normalize_mode(jit):
    if jit is None:
        return default_mode()
    if isinstance(jit, str):
        if jit.lower() == "auto":
            return "auto"
        raise ValueError("jit must be True, False or 'auto', not %r" % (jit,))
    return bool(jit)


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


def compiler():
    """Which compiler builds program libraries: NGH_JIT_COMPILER = "hiprtc" (device code compiled
    inside this process, launched through the module API: no hipcc needed, and about half the
    time per program), "hipcc" (a shared object with host launchers, built by a hipcc
    subprocess), or unset: hiprtc where the machine has libhiprtc, else hipcc."""
    choice = os.environ.get("NGH_JIT_COMPILER", "").strip().lower()
    if choice in ("hipcc", "hiprtc"):
        return choice
    from ngraph_hip.runtime import hiprtc
    return "hiprtc" if hiprtc.available() else "hipcc"


def _record_desc(record, type_name):
    """A program record as the dictionary hiplib.program_descs takes."""
    name, ops, dtypes, bcast, stat_slot, n_slots, n_regs, V, family, red_out, staged = record[:11]
    rowshared = record[14] if len(record) > 14 else [0] * len(dtypes)
    d = {"name": name, "type_name": type_name, "family": family, "V": V, "n_stat_slots": n_slots,
         "dtypes": list(dtypes), "bcast": list(bcast), "rowshared": list(rowshared), "red_out": list(red_out)}
    if family in (4, 5):
        d.update(ops=[], staged=[-1] * len(dtypes),
                 stages=[_record_desc(m, "%s_%d" % (type_name, j)) for j, m in enumerate(ops)])
    else:
        d.update(ops=[list(o) for o in ops], staged=list(staged) or [-1] * len(dtypes))
    return d


def device_source_text(programs):
    """The structs of `programs` alone: what hiprtc compiles (kernels are instantiated by name
    expression, there is no table and no host code)."""
    text = source_text(programs)
    lines, keep = [], True
    for line in text.split("\n"):
        if line.startswith("static const StaticEntry") or line.startswith("static const int kLoadedCount"):
            keep = False
        if line.startswith("}  // namespace ngh"):
            lines.append(line)
            break
        if keep:
            lines.append(line)
        elif line == "};":
            keep = True
    return "\n".join(lines) + "\n"


def _code_bundle(programs):
    """(path in the cache, source, descriptions, compiler options) of the code bundle of `programs`."""
    from ngraph_hip.runtime import hiprtc
    flags, _ = _flags()
    options = [f for f in flags if f not in ("-fPIC", "-shared")] + ["-I" + INCLUDE, "-I" + CSRC]
    text = device_source_text(programs)
    tag = "".join(c if c.isalnum() else "_" for c in programs[0][0])
    dicts = [_record_desc(p, "LP_%s_%d" % (tag, i)) for i, p in enumerate(programs)]
    key = hashlib.sha256((text + _sources_digest() + " ".join(flags) + "hiprtc " + hiprtc.version() +
                          repr(dicts)).encode("utf-8")).hexdigest()[:20]
    return os.path.join(cache_dir(), "ngh_programs_" + key + hiplib.CODE_BUNDLE_SUFFIX), text, dicts, options


def compile_programs_in_process(programs, verbose=False):
    """The path of a code bundle holding `programs`, compiled now with hiprtc unless the cache
    has it."""
    from ngraph_hip.runtime import hiprtc
    path, text, dicts, options = _code_bundle(programs)
    if os.path.exists(path):
        return path
    descs = hiplib.program_descs(dicts)
    index, expressions, slots = 0, [], []
    for d in dicts:
        names = hiplib.program_kernels(descs, index)
        slots.append(names)
        expressions.extend(n for n in names if n)
        index += 1 + len(d.get("stages", []))
    if verbose:
        print("hiprtc: %d kernels of %s" % (len(expressions), programs[0][0]))
    code, lowered = hiprtc.compile_source(text, expressions, options, name=os.path.basename(path) + ".hip")
    by_expression = dict(zip(expressions, lowered))
    lines = "".join(by_expression.get(n, "") + "\n" for names in slots for n in names)
    tmp = "%s.%d.%d.tmp" % (path, os.getpid(), threading.get_ident())
    hiplib.write_code_bundle(tmp, dicts, lines, code)
    os.replace(tmp, path)         # atomic: another process may be compiling the same programs
    return path


def compile_programs(programs, verbose=False):
    """The path of a program library holding `programs` (records of programs.stage_programs),
    compiled now unless the cache has it."""
    if compiler() == "hiprtc":
        return compile_programs_in_process(programs, verbose=verbose)
    flags, find_hipcc = _flags()
    text = source_text(programs)
    key = hashlib.sha256((text + _sources_digest() + " ".join(flags)).encode("utf-8")).hexdigest()[:20]
    base = os.path.join(cache_dir(), "ngh_programs_" + key)
    lib = base + ".so"
    if os.path.exists(lib):
        return lib
    src = base + ".hip"
    unique = "%d.%d.tmp" % (os.getpid(), threading.get_ident())
    # (the source goes into place whole as well: another thread or process compiling the same
    # programs may be reading it)
    with open(src + "." + unique, "w") as fh:
        fh.write(text)
    os.replace(src + "." + unique, src)
    tmp = "%s.%s" % (lib, unique)
    try:
        hipcc = find_hipcc()
    except RuntimeError:
        raise RuntimeError("run-time compilation (jit=True / NGH_JIT=1) with NGH_JIT_COMPILER=hipcc, or on a "
                           "machine without libhiprtc, needs hipcc, or the program library %s in the cache; "
                           "without jit the same stages run on the interpreter" % os.path.basename(lib))
    cmd = [hipcc] + list(flags) + ["-I", INCLUDE, "-I", CSRC, src, "-o", tmp]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, universal_newlines=True)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, proc.stdout))
    os.replace(tmp, lib)          # atomic: another process may be compiling the same programs
    return lib


def uncovered_programs(kernels, name, min_elements=4096, include_covered=False):
    """Records of the stage programs of `kernels` that run on the interpreter today and could run
    as compiled kernels (include_covered: also those that have a compiled kernel already)."""
    out = []
    for p in stage_programs(kernels, name, min_elements=min_elements):
        if p[-1] < 0 or include_covered:
            if p[8] in (4, 5):     # a chain: its stages are named by their place, not by the computation
                p = (p[0], [("stage%d" % j,) + tuple(m[1:]) for j, m in enumerate(p[1])]) + tuple(p[2:])
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


def library_path_of(programs):
    """Where the program library of `programs` lives in the cache (whether or not it exists)."""
    if compiler() == "hiprtc":
        return _code_bundle(programs)[0]
    flags, _ = _flags()
    text = source_text(programs)
    key = hashlib.sha256((text + _sources_digest() + " ".join(flags)).encode("utf-8")).hexdigest()[:20]
    return os.path.join(cache_dir(), "ngh_programs_" + key + ".so")


_executor = None
_executor_lock = threading.Lock()


def _compile_executor():
    """One small pool of compile workers for the whole process, however many computations ask:
    each job is a hipcc run (itself several processes), so a pool per computation would
    flood a machine that builds many graphs."""
    global _executor
    with _executor_lock:
        if _executor is None:
            from concurrent.futures import ThreadPoolExecutor
            workers = max(1, min(4, (os.cpu_count() or 2) // 2))
            _executor = ThreadPoolExecutor(max_workers=workers, thread_name_prefix="ngh-jit")
            _drop_pending_jobs_at_exit(_executor)
        return _executor


def _drop_pending_jobs_at_exit(executor):
    """Interpreter exit joins the workers, and a worker runs every job still queued before it
    ends: a process that built many graphs would sit through their compilations for nothing.
    The handler withdraws what has not started (a hipcc run in progress finishes, seconds).
    It has to run before the thread pool's own exit hook, which `atexit` handlers do not."""
    def drop():
        executor.shutdown(wait=False, cancel_futures=True)
    register = getattr(threading, "_register_atexit", None)
    if register is not None:
        try:
            register(drop)
            return
        except RuntimeError:            # the interpreter is already shutting down
            pass
    import atexit
    atexit.register(drop)


class BackgroundPrograms(object):
    """The uncovered programs of a kernel group, compiled off the launch path.

    Libraries the cache already holds are loaded at once.  The others are handed to the
    process-wide compile workers by `start`: at once with `after_calls` = 0, else once the
    computation has run `after_calls` times (a computation that runs fewer times never pays for
    a compiler run); the workers run hipcc and touch no device.  `poll`, called from the thread that owns the
    runtime, loads what has been compiled since the last call and returns True once nothing is
    outstanding.  A compiler that is missing or fails leaves the group on the interpreter; the
    message is kept in `error`.  `cancel` withdraws the jobs that have not started."""

    def __init__(self, runtime, programs, after_calls=2, verbose=False):
        self.runtime = runtime
        self.error = None
        self.loaded = 0
        self.verbose = verbose
        self.after_calls = int(after_calls)
        self.calls = 0
        self._futures = None               # None: compilation not started yet
        self._todo = []
        for p in programs:
            path = library_path_of([p])
            if os.path.exists(path):
                self.loaded += runtime.programs_load(path)
            else:
                self._todo.append(p)
        if self.after_calls <= 0 and self._todo:
            self.start()

    @property
    def started(self):
        return self._futures is not None

    def start(self):
        if self._futures is None:
            ex = _compile_executor()
            self._futures = [ex.submit(compile_programs, [p], self.verbose) for p in self._todo]
            self._todo = []

    def poll(self):
        """Called once per execution of the computation."""
        if self._futures is None:
            if not self._todo:
                return True
            self.calls += 1
            if self.calls >= self.after_calls:
                self.start()
            return False
        waiting = []
        for f in self._futures:
            if not f.done():
                waiting.append(f)
            elif not f.cancelled():
                try:
                    self.loaded += self.runtime.programs_load(f.result())
                except Exception as e:       # no hipcc, or it failed: stay on the interpreter
                    self.error = self.error or str(e)
        self._futures = waiting
        return not waiting

    def wait(self, timeout=None):
        from concurrent.futures import wait as wait_all
        self.start()
        wait_all(self._futures, timeout=timeout)
        return self.poll()

    def cancel(self):
        self._todo = []
        for f in self._futures or []:
            f.cancel()


def start_background(runtime, kernels, name, min_elements, after_calls=2, verbose=False, small_min_elements=None):
    """BackgroundPrograms for the stages of `kernels` (of at least min_elements elements) that run on
    the interpreter today, or None when there are none."""
    programs = uncovered_programs(kernels, name, min_elements)
    if not programs and small_min_elements is None:
        return None
    if small_min_elements is not None and (programs or _has_large_stage(kernels, min_elements)):
        # A computation over large tensors: its small stages (statistics combined between two
        # passes, per-channel factors) are launches on the same critical path, several
        # microseconds each on the interpreter, so they get programs too.
        programs = uncovered_programs(kernels, name, small_min_elements)
    if not programs:
        return None
    return BackgroundPrograms(runtime, programs, after_calls=after_calls, verbose=verbose)


def _has_large_stage(kernels, min_elements):
    for k in kernels:
        for spec in getattr(k, "specs", [])[:1]:
            if spec.shape[0] * spec.shape[1] * spec.shape[2] >= min_elements:
                return True
    return False


def precompile_graphs(builders, verbose=False):
    """Compile, without a device, the program libraries of the graphs in `builders` into the
    cache, so that a later process (on a machine with a GPU, perhaps without hipcc) finds them.
    builders: iterable of (backend name, build, transformer keyword arguments) with build()
    returning (results, inputs) of a computation.  Returns the libraries' paths."""
    from multiprocessing.pool import ThreadPool
    import ngraph_hip.transformers as ngt
    todo = {}
    for backend, build, kwargs in builders:
        if backend not in ngt.transformer_choices():
            continue
        t = ngt.make_transformer_factory(backend, dry_run=True, jit=False, **kwargs)()
        try:
            built = build()
            f = t.computation(built[0], *built[1])
            t.initialize()
            kernels = t.kernel_groups[f].kernels
            for k in kernels:
                k.bind_buffers()
            for p in uncovered_programs(kernels, "graph", min_elements=t.jit_min_elements):
                todo[p[0]] = p
        finally:
            t.close()
    if not todo:
        return []
    workers = max(1, min(8, os.cpu_count() or 2))
    if compiler() == "hiprtc":
        # hiprtc compiles one program at a time per process: processes, not threads (started
        # afresh, so that none inherits a device context)
        import multiprocessing
        from concurrent.futures import ProcessPoolExecutor
        with ProcessPoolExecutor(max_workers=workers, mp_context=multiprocessing.get_context("spawn")) as ex:
            return list(ex.map(_compile_one, list(todo.values())))
    pool = ThreadPool(workers)      # the work is in hipcc subprocesses
    try:
        return pool.map(lambda p: compile_programs([p], verbose=verbose), list(todo.values()))
    finally:
        pool.close()


def _compile_one(program):
    return compile_programs([program])
