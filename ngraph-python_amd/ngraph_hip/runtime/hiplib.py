"""ctypes binding of libngraph_hip.so (declared in include/ngraph_hip.h).

This is the layer that stands where pycuda stands in the reference GPU
transformer: device runtime, memory, and kernel launches
(ngraph/transformers/gputransform.py:912-1000, 525-676, 343-345).  It holds
no arithmetic of its own: every result comes from the HIP library, and a
missing library is an error, never a fallback.
"""
from __future__ import division
import ctypes
import os

import numpy as np

NGH_ABI_VERSION = 7
NGH_MAX_AXES = 3
NGH_MAX_TENSORS = 12
NGH_MAX_OPS = 96
NGH_MAX_CONSTS = 16
NGH_MAX_REGS = 32
NGH_MAX_REDUCTIONS = 4
NGH_MAX_STAGES = 6

NGH_F32, NGH_FLEX16, NGH_I32, NGH_F16 = 0, 1, 2, 3
NGH_U32, NGH_I16, NGH_I8, NGH_U8 = 4, 5, 6, 7
NGH_SPEC_PROBE = 1
NGH_CACHE_STREAM_LOAD, NGH_CACHE_STREAM_STORE = 1, 2

_OPCODE_NAMES = [
    "nop", "load", "store", "const", "iota",
    "assign", "neg", "abs", "sqrt", "sqr", "exp", "log", "rcp", "exp2", "log2", "sig", "tanh",
    "safelog", "sgn", "sin", "cos",
    "add", "sub", "mul", "div", "int_div", "mod", "eq", "ne", "lt", "le", "gt", "ge",
    "pow", "minimum", "maximum",
    "sum", "prod", "max", "min", "argmax", "argmin",
    "take", "store_trunc", "rng_uniform", "rng_normal",
    # 32-bit integer arithmetic on the registers' bits (include/ngraph_hip.h)
    "i2f", "u2f", "ineg", "iabs",
    "iadd", "isub", "imul", "imin", "imax", "umin", "umax",
    "ieq", "ine", "ilt", "ile", "igt", "ige", "ult", "ule", "ugt", "uge",
]
#: op name (the reference's template names, float_ew2.py:31-77) -> opcode
OPCODES = {name: i for i, name in enumerate(_OPCODE_NAMES)}
#: ops that read and write a register's 32 bits as an integer
INTEGER_UNARY_OPS = _OPCODE_NAMES[OPCODES["i2f"]:OPCODES["iabs"] + 1]
INTEGER_BINARY_OPS = _OPCODE_NAMES[OPCODES["iadd"]:OPCODES["uge"] + 1]
FLOAT_UNARY_OPS = _OPCODE_NAMES[OPCODES["assign"]:OPCODES["cos"] + 1]
FLOAT_BINARY_OPS = _OPCODE_NAMES[OPCODES["add"]:OPCODES["maximum"] + 1]
UNARY_OPS = FLOAT_UNARY_OPS + INTEGER_UNARY_OPS
BINARY_OPS = FLOAT_BINARY_OPS + INTEGER_BINARY_OPS
REDUCTION_OPS = _OPCODE_NAMES[OPCODES["sum"]:OPCODES["argmin"] + 1]


class ngh_op(ctypes.Structure):
    _fields_ = [("opcode", ctypes.c_uint8), ("dst", ctypes.c_uint8),
                ("a", ctypes.c_uint8), ("b", ctypes.c_uint8)]


class ngh_tensor(ctypes.Structure):
    _fields_ = [("dev", ctypes.c_void_p),
                ("strides", ctypes.c_int64 * NGH_MAX_AXES),
                ("dtype", ctypes.c_int32),
                ("scale", ctypes.c_float),
                ("dev_stats", ctypes.c_void_p),
                ("dev_scale", ctypes.c_void_p),
                ("cache_hint", ctypes.c_uint32),
                ("take_extent", ctypes.c_uint32)]


class ngh_stage(ctypes.Structure):
    _fields_ = [("op_begin", ctypes.c_int32), ("op_end", ctypes.c_int32),
                ("n_reductions", ctypes.c_int32),
                ("red_out", ctypes.c_int32 * NGH_MAX_REDUCTIONS)]


class ngh_fused_spec(ctypes.Structure):
    _fields_ = [("abi_version", ctypes.c_int32),
                ("rank", ctypes.c_int32),
                ("shape", ctypes.c_int64 * NGH_MAX_AXES),
                ("n_tensors", ctypes.c_int32), ("n_ops", ctypes.c_int32),
                ("n_consts", ctypes.c_int32), ("n_stages", ctypes.c_int32),
                ("n_regs", ctypes.c_int32),
                ("flags", ctypes.c_int32),
                ("tensors", ngh_tensor * NGH_MAX_TENSORS),
                ("consts", ctypes.c_float * NGH_MAX_CONSTS),
                ("ops", ngh_op * NGH_MAX_OPS),
                ("stages", ngh_stage * NGH_MAX_STAGES),
                ("rng_seed", ctypes.c_uint32), ("rng_counter", ctypes.c_uint32)]


class HipLibraryError(RuntimeError):
    """A call into libngraph_hip.so failed; carries the library's message."""

    def __init__(self, code, message):
        super(HipLibraryError, self).__init__("libngraph_hip error %d: %s" % (code, message))
        self.code = code


#: every symbol include/ngraph_hip.h declares: name -> (argtypes)
_vp, _i32, _i64p = ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64)
_SYMBOLS = {
    "ngh_abi_version": [],
    "ngh_last_error": [],
    "ngh_device_count": [ctypes.POINTER(ctypes.c_int)],
    "ngh_init": [ctypes.c_int, ctypes.POINTER(_vp)],
    "ngh_shutdown": [_vp],
    "ngh_sync": [_vp],
    "ngh_device_info": [_vp, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_uint64)],
    "ngh_malloc": [_vp, ctypes.c_size_t, ctypes.POINTER(_vp)],
    "ngh_free": [_vp, _vp],
    "ngh_memcpy_h2d": [_vp, _vp, _vp, ctypes.c_size_t],
    "ngh_memcpy_d2h": [_vp, _vp, _vp, ctypes.c_size_t],
    "ngh_memcpy_d2d": [_vp, _vp, _vp, ctypes.c_size_t],
    "ngh_io_scratch": [_vp, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)],
    "ngh_memset32": [_vp, _vp, ctypes.c_uint32, ctypes.c_size_t],
    "ngh_memset16": [_vp, _vp, ctypes.c_uint16, ctypes.c_size_t],
    "ngh_copy_strided": [_vp, _vp, _vp, _i32, _i64p, _i64p, _i64p, _i32],
    "ngh_validate_fused": [ctypes.POINTER(ngh_fused_spec)],
    "ngh_launch_fused": [_vp, ctypes.POINTER(ngh_fused_spec)],
    "ngh_describe_fused": [_vp, ctypes.POINTER(ngh_fused_spec), _i32, ctypes.c_char_p],
    "ngh_moments_f32": [_vp, _vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, _vp, _vp, _vp, ctypes.c_float,
                        ctypes.c_uint32],
    "ngh_moments_f32_noalloc": [_vp, _vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, _vp, _vp, _vp,
                                ctypes.c_float, ctypes.c_uint32],
    "ngh_convert_to_flex16": [_vp, _vp, _vp, _i32, ctypes.c_int64, ctypes.c_float, _vp, _vp],
    "ngh_plan_fused": [ctypes.POINTER(ngh_fused_spec), _i32, ctypes.POINTER(ctypes.c_int32)],
    "ngh_plan_chain": [ctypes.POINTER(ngh_fused_spec), ctypes.POINTER(ctypes.c_int32)],
    "ngh_stats_alloc": [_vp, _i32, ctypes.POINTER(_vp)],
    "ngh_stats_reset": [_vp, _vp, _i32],
    "ngh_stats_read": [_vp, _vp, _i32, _vp],
    "ngh_flex_states_alloc": [_vp, _i32, ctypes.POINTER(_vp)],
    "ngh_flex_states_write": [_vp, _vp, _i32, _i32, _vp],
    "ngh_flex_states_read": [_vp, _vp, _i32, _i32, _vp],
    "ngh_flex_prepare": [_vp, _vp, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32), _i32],
    "ngh_flex_update": [_vp, _vp, ctypes.POINTER(ctypes.c_int32), _i32, _i32],
    "ngh_launch_fused_flex": [_vp, ctypes.POINTER(ngh_fused_spec), _vp, ctypes.POINTER(ctypes.c_int32),
                              ctypes.POINTER(ctypes.c_int32), _i32, _i32],
    "ngh_flex_unsettled": [_vp, ctypes.POINTER(ctypes.c_int32)],
    "ngh_programs_load": [_vp, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int32)],
    "ngh_programs_count": [ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)],
    "ngh_program_kernels": [ctypes.c_void_p, _i32, _i32, ctypes.c_char_p, ctypes.c_size_t],
    "ngh_programs_load_code": [_vp, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, _i32, ctypes.c_char_p,
                               ctypes.POINTER(ctypes.c_int32)],
    "ngh_launch_fused_pair": [_vp, ctypes.POINTER(ngh_fused_spec), ctypes.POINTER(ngh_fused_spec),
                              ctypes.POINTER(ctypes.c_int32)],
    "ngh_graph_begin": [_vp],
    "ngh_graph_fork": [_vp],
    "ngh_graph_side": [_vp, _i32],
    "ngh_graph_join": [_vp],
    "ngh_graph_end": [_vp, ctypes.POINTER(_vp)],
    "ngh_graph_launch": [_vp, _vp],
    "ngh_graph_nodes": [_vp, ctypes.POINTER(ctypes.c_int32)],
    "ngh_graph_free": [_vp, _vp],
    "ngh_timer_begin": [_vp],
    "ngh_timer_end": [_vp, ctypes.POINTER(ctypes.c_float)],
}

NGH_PROGRAM_KERNEL_SLOTS = 12


class ngh_program_desc(ctypes.Structure):
    """What the library compares a stage with, restated for a program whose kernels arrive as a
    code object (include/ngraph_hip.h)."""
    _fields_ = [("name", ctypes.c_char * 64), ("type_name", ctypes.c_char * 64),
                ("family", ctypes.c_int32), ("V", ctypes.c_int32), ("n_ops", ctypes.c_int32),
                ("n_tensors", ctypes.c_int32), ("n_red", ctypes.c_int32), ("n_stat_slots", ctypes.c_int32),
                ("n_stages", ctypes.c_int32),
                ("ops", ngh_op * NGH_MAX_OPS),
                ("dtypes", ctypes.c_int32 * NGH_MAX_TENSORS),
                ("bcast", ctypes.c_uint8 * NGH_MAX_TENSORS),
                ("rowshared", ctypes.c_uint8 * NGH_MAX_TENSORS),
                ("staged", ctypes.c_int8 * NGH_MAX_TENSORS),
                ("red_out", ctypes.c_int32 * NGH_MAX_REDUCTIONS)]


_lib = None


def library_path():
    return os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "lib", "libngraph_hip.so")


def load_library():
    """Open libngraph_hip.so and type every entry point.  Raises if absent."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise HipLibraryError(-5, "%s is not built (run ngraph-python_amd/build_ext.py)" % path)
    lib = ctypes.CDLL(path)
    for name, argtypes in _SYMBOLS.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_char_p if name == "ngh_last_error" else ctypes.c_int
    if lib.ngh_abi_version() != NGH_ABI_VERSION:
        raise HipLibraryError(-1, "ABI version mismatch: library %d, binding %d"
                              % (lib.ngh_abi_version(), NGH_ABI_VERSION))
    _lib = lib
    return lib


def plan_fused(spec, stage=0):
    """(family, V, perm, tail, special index, segments) the library would use for a stage."""
    lib = load_library()
    out = (ctypes.c_int32 * 8)()
    _check(lib, lib.ngh_plan_fused(ctypes.byref(spec), int(stage), out))
    return {"family": out[0], "V": out[1], "perm": (out[2], out[3], out[4]), "tail": out[5],
            "special": out[6], "segments": out[7]}


def plan_chain(spec):
    """Would the library run every stage of `spec` in one kernel -- as a row chain (the reduced
    axis contiguous) or a column chain (the reduced axis strided, outputs along the contiguous
    one)?  lanes_per_row: lanes per row of a row chain, column chunks per workgroup of a column
    chain."""
    lib = load_library()
    out = (ctypes.c_int32 * 4)()
    _check(lib, lib.ngh_plan_chain(ctypes.byref(spec), out))
    return {"eligible": bool(out[0]), "kind": {0: None, 1: "row", 2: "column"}[out[0]], "special": out[1],
            "lanes_per_row": out[2], "stages": out[3]}


def program_descs(dicts):
    """An array of ngh_program_desc from plain dictionaries (a chain is followed by its stages)."""
    flat = []
    for d in dicts:
        flat.append(d)
        flat.extend(d.get("stages", []))
    arr = (ngh_program_desc * len(flat))()
    for rec, d in zip(arr, flat):
        rec.name = d["name"].encode("utf-8")
        rec.type_name = d["type_name"].encode("utf-8")
        rec.family, rec.V, rec.n_stat_slots = d["family"], d["V"], d["n_stat_slots"]
        rec.n_ops, rec.n_tensors, rec.n_red = len(d["ops"]), len(d["dtypes"]), len(d["red_out"])
        rec.n_stages = len(d.get("stages", []))
        for i, (opcode, dst, a, b) in enumerate(d["ops"]):
            rec.ops[i] = ngh_op(opcode, dst, a, b)
        for i in range(rec.n_tensors):
            rec.dtypes[i], rec.bcast[i] = d["dtypes"][i], d["bcast"][i]
            rec.rowshared[i], rec.staged[i] = d["rowshared"][i], d["staged"][i]
        for i, r in enumerate(d["red_out"]):
            rec.red_out[i] = r
    return arr


def program_kernels(descs, index):
    """The C++ name expressions of the kernels program `index` of `descs` may launch, one per
    slot ('' for an empty slot)."""
    lib = load_library()
    out = ctypes.create_string_buffer(NGH_PROGRAM_KERNEL_SLOTS * 1024)
    _check(lib, lib.ngh_program_kernels(ctypes.cast(descs, ctypes.c_void_p), len(descs), int(index), out, len(out)))
    names = out.value.decode("utf-8").split("\n")[:-1]
    assert len(names) == NGH_PROGRAM_KERNEL_SLOTS, names
    return names


def exported_symbols():
    return sorted(_SYMBOLS)


def _check(lib, rc):
    if rc != 0:
        msg = lib.ngh_last_error()
        raise HipLibraryError(rc, msg.decode("utf-8", "replace") if msg else "")


CODE_BUNDLE_SUFFIX = ".ngco"
_BUNDLE_MAGIC = b"NGHCODE1"


def write_code_bundle(path, dicts, lowered, code):
    """One file per program library compiled in process: the descriptions of its programs, the
    lowered names of their kernels (NGH_PROGRAM_KERNEL_SLOTS lines per program) and the code object."""
    import json
    import struct
    head = json.dumps({"abi": NGH_ABI_VERSION, "programs": dicts, "lowered": lowered}).encode("utf-8")
    with open(path, "wb") as fh:
        fh.write(_BUNDLE_MAGIC + struct.pack("<I", len(head)) + head + code)


def read_code_bundle(path):
    import json
    import struct
    with open(path, "rb") as fh:
        data = fh.read()
    if data[:8] != _BUNDLE_MAGIC:
        raise HipLibraryError(-1, "%s is not a code bundle of this library" % path)
    n = struct.unpack("<I", data[8:12])[0]
    head = json.loads(data[12:12 + n].decode("utf-8"))
    if head.get("abi") != NGH_ABI_VERSION:
        raise HipLibraryError(-1, "%s was made for ABI %s, this is %d" % (path, head.get("abi"), NGH_ABI_VERSION))
    return head["programs"], head["lowered"], data[12 + n:]


_NP_DTYPES = {NGH_F32: np.float32, NGH_FLEX16: np.int16, NGH_I32: np.int32, NGH_F16: np.float16,
              NGH_U32: np.uint32, NGH_I16: np.int16, NGH_I8: np.int8, NGH_U8: np.uint8}


class DeviceArray(object):
    """A contiguous device allocation with a shape and a storage type."""

    def __init__(self, runtime, shape, ngh_dtype=NGH_F32):
        self.runtime = runtime
        self.shape = tuple(int(s) for s in shape)
        self.ngh_dtype = ngh_dtype
        self.np_dtype = np.dtype(_NP_DTYPES[ngh_dtype])
        self.size = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        self.nbytes = self.size * self.np_dtype.itemsize
        self.ptr = runtime.malloc(self.nbytes)

    def set(self, host):
        host = np.ascontiguousarray(host, dtype=self.np_dtype)
        if host.size != self.size:
            raise ValueError("size mismatch: %d vs %d" % (host.size, self.size))
        self.runtime.memcpy_h2d(self.ptr, host)
        return self

    def get(self):
        out = np.empty(self.shape, dtype=self.np_dtype)
        self.runtime.memcpy_d2h(out, self.ptr)
        return out

    def free(self):
        if self.ptr:
            self.runtime.free(self.ptr)
            self.ptr = None


class HipRuntime(object):
    """One device context: stream, allocations, launches."""

    def __init__(self, device_id=0):
        self.lib = load_library()
        ctx = ctypes.c_void_p()
        _check(self.lib, self.lib.ngh_init(int(device_id), ctypes.byref(ctx)))
        self.ctx = ctx
        self._allocs = set()
        self.program_libraries = []        # what this context asked the library to load

    # -- lifetime --------------------------------------------------------
    def close(self):
        if getattr(self, "ctx", None):
            for ptr in list(self._allocs):
                self.lib.ngh_free(self.ctx, ctypes.c_void_p(ptr))
            self._allocs.clear()
            self.lib.ngh_shutdown(self.ctx)
            self.ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def device_info(self):
        name = ctypes.create_string_buffer(256)
        cus = ctypes.c_int()
        total = ctypes.c_uint64()
        _check(self.lib, self.lib.ngh_device_info(self.ctx, name, ctypes.byref(cus), ctypes.byref(total)))
        return name.value.decode(), cus.value, total.value

    def sync(self):
        _check(self.lib, self.lib.ngh_sync(self.ctx))

    # -- memory ----------------------------------------------------------
    def malloc(self, nbytes):
        ptr = ctypes.c_void_p()
        _check(self.lib, self.lib.ngh_malloc(self.ctx, int(nbytes), ctypes.byref(ptr)))
        self._allocs.add(ptr.value)
        return ptr.value

    def free(self, ptr):
        if ptr in self._allocs:
            self._allocs.discard(ptr)
            _check(self.lib, self.lib.ngh_free(self.ctx, ctypes.c_void_p(ptr)))

    def memcpy_h2d(self, dev, host):
        host = np.ascontiguousarray(host)
        _check(self.lib, self.lib.ngh_memcpy_h2d(self.ctx, ctypes.c_void_p(dev),
                                                 host.ctypes.data_as(ctypes.c_void_p), host.nbytes))

    def memcpy_d2h(self, host, dev):
        assert host.flags.c_contiguous
        _check(self.lib, self.lib.ngh_memcpy_d2h(self.ctx, host.ctypes.data_as(ctypes.c_void_p),
                                                 ctypes.c_void_p(dev), host.nbytes))

    def memcpy_d2d(self, dst, src, nbytes):
        _check(self.lib, self.lib.ngh_memcpy_d2d(self.ctx, ctypes.c_void_p(dst), ctypes.c_void_p(src), int(nbytes)))

    def io_scratch(self, nbytes):
        """Context-owned device scratch of at least nbytes (valid until the next, larger request)."""
        ptr = ctypes.c_void_p()
        _check(self.lib, self.lib.ngh_io_scratch(self.ctx, int(nbytes), ctypes.byref(ptr)))
        return ptr.value

    def memset32(self, dev, value, count):
        _check(self.lib, self.lib.ngh_memset32(self.ctx, ctypes.c_void_p(dev), int(value) & 0xffffffff, int(count)))

    def memset16(self, dev, value, count):
        _check(self.lib, self.lib.ngh_memset16(self.ctx, ctypes.c_void_p(dev), int(value) & 0xffff, int(count)))

    def fill_f32(self, dev, value, count):
        self.memset32(dev, int(np.float32(value).view(np.uint32)), count)

    def empty(self, shape, ngh_dtype=NGH_F32):
        return DeviceArray(self, shape, ngh_dtype)

    def array(self, host, ngh_dtype=None):
        host = np.asarray(host)
        if ngh_dtype is None:
            ngh_dtype = {np.dtype(np.float32): NGH_F32, np.dtype(np.int16): NGH_FLEX16,
                         np.dtype(np.int32): NGH_I32, np.dtype(np.float16): NGH_F16,
                         np.dtype(np.uint32): NGH_U32, np.dtype(np.int8): NGH_I8,
                         np.dtype(np.uint8): NGH_U8}[host.dtype]
        return DeviceArray(self, host.shape, ngh_dtype).set(host)

    def copy_strided(self, dst, src, shape, dst_strides, src_strides, itemsize):
        n = len(shape)
        arr = ctypes.c_int64 * max(n, 1)
        _check(self.lib, self.lib.ngh_copy_strided(
            self.ctx, ctypes.c_void_p(dst), ctypes.c_void_p(src), n,
            arr(*[int(s) for s in shape]), arr(*[int(s) for s in dst_strides]),
            arr(*[int(s) for s in src_strides]), int(itemsize)))

    # -- fused kernels ---------------------------------------------------
    def validate_fused(self, spec):
        _check(self.lib, self.lib.ngh_validate_fused(ctypes.byref(spec)))

    def launch_fused(self, spec):
        _check(self.lib, self.lib.ngh_launch_fused(self.ctx, ctypes.byref(spec)))

    def describe_fused(self, spec, stage=0):
        name = ctypes.create_string_buffer(128)
        _check(self.lib, self.lib.ngh_describe_fused(self.ctx, ctypes.byref(spec), int(stage), name))
        return name.value.decode()

    def moments_f32(self, x, rows, R, row_stride, mean, var, rstd=None, eps=0.0, x_cache_hint=0):
        _check(self.lib, self.lib.ngh_moments_f32(self.ctx, ctypes.c_void_p(x), int(rows), int(R),
                                                  int(row_stride), ctypes.c_void_p(mean),
                                                  ctypes.c_void_p(var), ctypes.c_void_p(rstd or None),
                                                  float(eps), int(x_cache_hint)))

    def moments_f32_noalloc(self, x, rows, R, row_stride, mean, var, rstd=None, eps=0.0, x_cache_hint=0):
        """moments_f32 on the library's fixed scratch: allocates nothing, limited in size."""
        _check(self.lib, self.lib.ngh_moments_f32_noalloc(self.ctx, ctypes.c_void_p(x), int(rows), int(R),
                                                          int(row_stride), ctypes.c_void_p(mean),
                                                          ctypes.c_void_p(var), ctypes.c_void_p(rstd or None),
                                                          float(eps), int(x_cache_hint)))

    def convert_to_flex16(self, out, src, src_dtype, n, scale=1.0, dev_scale=None, dev_stats=None):
        """out[i] = (int16)trunc(src[i] * scale), saturating; max|mantissa| merged into dev_stats
        (flex_conv.py:745-791).  With dev_scale the multiplier is 1 / *dev_scale."""
        _check(self.lib, self.lib.ngh_convert_to_flex16(self.ctx, ctypes.c_void_p(out), ctypes.c_void_p(src),
                                                        int(src_dtype), int(n), float(scale),
                                                        ctypes.c_void_p(dev_scale or None),
                                                        ctypes.c_void_p(dev_stats or None)))

    # -- flex statistics ---------------------------------------------------
    def stats_alloc(self, n):
        ptr = ctypes.c_void_p()
        _check(self.lib, self.lib.ngh_stats_alloc(self.ctx, int(n), ctypes.byref(ptr)))
        self._allocs.add(ptr.value)
        return ptr.value

    def stats_reset(self, dev, n=1):
        _check(self.lib, self.lib.ngh_stats_reset(self.ctx, ctypes.c_void_p(dev), int(n)))

    def stats_read(self, dev, n=1):
        out = np.zeros(n, dtype=np.int32)
        _check(self.lib, self.lib.ngh_stats_read(self.ctx, ctypes.c_void_p(dev), int(n),
                                                 out.ctypes.data_as(ctypes.c_void_p)))
        return out

    # -- device-resident flex state ------------------------------------------
    def flex_states_alloc(self, n):
        ptr = ctypes.c_void_p()
        _check(self.lib, self.lib.ngh_flex_states_alloc(self.ctx, int(n), ctypes.byref(ptr)))
        self._allocs.add(ptr.value)
        return ptr.value

    def flex_states_write(self, dev, first, records):
        records = np.ascontiguousarray(records)
        _check(self.lib, self.lib.ngh_flex_states_write(self.ctx, ctypes.c_void_p(dev), int(first),
                                                        len(records), records.ctypes.data_as(ctypes.c_void_p)))

    def flex_states_read(self, dev, first, records):
        assert records.flags.c_contiguous
        _check(self.lib, self.lib.ngh_flex_states_read(self.ctx, ctypes.c_void_p(dev), int(first),
                                                       len(records), records.ctypes.data_as(ctypes.c_void_p)))

    def flex_prepare(self, dev, ids, in_place):
        n = len(ids)
        arr = ctypes.c_int32 * max(n, 1)
        _check(self.lib, self.lib.ngh_flex_prepare(self.ctx, ctypes.c_void_p(dev), arr(*ids), arr(*in_place), n))

    def flex_update(self, dev, ids, count):
        n = len(ids)
        arr = ctypes.c_int32 * max(n, 1)
        _check(self.lib, self.lib.ngh_flex_update(self.ctx, ctypes.c_void_p(dev), arr(*ids), n, int(count)))

    def make_id_arrays(self, ids, in_place):
        arr = ctypes.c_int32 * max(len(ids), 1)
        return arr(*ids), arr(*in_place), len(ids)

    def launch_fused_flex(self, spec, dev, id_arrays, count):
        ids, in_place, n = id_arrays
        _check(self.lib, self.lib.ngh_launch_fused_flex(self.ctx, ctypes.byref(spec), ctypes.c_void_p(dev),
                                                        ids, in_place, n, int(count)))

    def flex_unsettled(self):
        """Records whose latest statistics the library has not folded in yet."""
        n = ctypes.c_int32()
        _check(self.lib, self.lib.ngh_flex_unsettled(self.ctx, ctypes.byref(n)))
        return n.value

    # -- compiled programs ---------------------------------------------------
    def programs_load(self, path):
        """Add the compiled programs of a program library (runtime/jit.py) to the library's
        table; returns how many were new."""
        n = ctypes.c_int32()
        self.program_libraries.append(path)
        if path.endswith(CODE_BUNDLE_SUFFIX):
            # kernels compiled in process: a code object with the descriptions of its programs
            dicts, lowered, code = read_code_bundle(path)
            descs = program_descs(dicts)
            buf = ctypes.create_string_buffer(code, len(code))
            _check(self.lib, self.lib.ngh_programs_load_code(self.ctx, ctypes.cast(buf, ctypes.c_void_p), len(code),
                                                             ctypes.cast(descs, ctypes.c_void_p), len(descs),
                                                             lowered.encode("utf-8"), ctypes.byref(n)))
            return n.value
        _check(self.lib, self.lib.ngh_programs_load(self.ctx, os.fsencode(path), ctypes.byref(n)))
        return n.value

    def launch_fused_pair(self, a, b):
        """Two specs that do not depend on each other; True when they ran as one launch."""
        one = ctypes.c_int32()
        _check(self.lib, self.lib.ngh_launch_fused_pair(self.ctx, ctypes.byref(a), ctypes.byref(b), ctypes.byref(one)))
        return bool(one.value)

    # -- launches recorded as one HIP graph ---------------------------------
    graphs = True

    def graph_begin(self):
        _check(self.lib, self.lib.ngh_graph_begin(self.ctx))

    def graph_fork(self):
        _check(self.lib, self.lib.ngh_graph_fork(self.ctx))

    def graph_side(self, on):
        _check(self.lib, self.lib.ngh_graph_side(self.ctx, 1 if on else 0))

    def graph_join(self):
        _check(self.lib, self.lib.ngh_graph_join(self.ctx))

    def graph_end(self):
        """The graph of what was launched since graph_begin (a handle for graph_launch)."""
        g = _vp()
        _check(self.lib, self.lib.ngh_graph_end(self.ctx, ctypes.byref(g)))
        return g

    def graph_abandon(self):
        self.lib.ngh_graph_end(self.ctx, None)

    def graph_launch(self, graph):
        _check(self.lib, self.lib.ngh_graph_launch(self.ctx, graph))

    def graph_nodes(self, graph):
        n = ctypes.c_int32()
        _check(self.lib, self.lib.ngh_graph_nodes(graph, ctypes.byref(n)))
        return n.value

    def graph_free(self, graph):
        _check(self.lib, self.lib.ngh_graph_free(self.ctx, graph))

    # -- timing ------------------------------------------------------------
    def timer_begin(self):
        _check(self.lib, self.lib.ngh_timer_begin(self.ctx))

    def timer_end(self):
        ms = ctypes.c_float()
        _check(self.lib, self.lib.ngh_timer_end(self.ctx, ctypes.byref(ms)))
        return ms.value


class DryRunRuntime(object):
    """Stands in for HipRuntime where no device exists: hands out fake, aligned device
    addresses and records launches.  It lets the host-side lowering (graph -> kernel specs)
    run and be validated by the library on a machine without a GPU; it computes nothing,
    and reading results through it raises."""

    def __init__(self):
        self.lib = load_library()
        self._next = 1 << 32
        self.launched = []
        self.program_libraries = []

    def close(self):
        pass

    def sync(self):
        pass

    def malloc(self, nbytes):
        ptr = self._next
        self._next += (int(nbytes) + 255) // 256 * 256 + 256
        return ptr

    def free(self, ptr):
        pass

    def memcpy_h2d(self, dev, host):
        pass

    def memcpy_d2h(self, host, dev):
        raise HipLibraryError(-5, "dry-run runtime holds no data")

    def io_scratch(self, nbytes):
        return self.malloc(nbytes)

    def copy_strided(self, *args):
        pass

    def validate_fused(self, spec):
        _check(self.lib, self.lib.ngh_validate_fused(ctypes.byref(spec)))

    def launch_fused(self, spec):
        self.validate_fused(spec)
        self.launched.append(spec)

    def describe_fused(self, spec, stage=0):
        return "dry-run"

    def moments_f32(self, *args):
        self.launched.append(("moments",) + args)

    def stats_alloc(self, n):
        return self.malloc(4 * n)

    def stats_reset(self, dev, n=1):
        pass

    def stats_read(self, dev, n=1):
        raise HipLibraryError(-5, "dry-run runtime holds no data")

    def flex_states_alloc(self, n):
        return self.malloc(168 * n)

    def flex_states_write(self, dev, first, records):
        pass

    def flex_states_read(self, dev, first, records):
        raise HipLibraryError(-5, "dry-run runtime holds no data")

    def flex_prepare(self, dev, ids, in_place):
        pass

    def flex_update(self, dev, ids, count):
        pass

    def make_id_arrays(self, ids, in_place):
        return (ids, in_place, len(ids))

    def launch_fused_flex(self, spec, dev, id_arrays, count):
        self.launch_fused(spec)

    def flex_unsettled(self):
        return 0

    def programs_load(self, path):
        self.program_libraries.append(path)      # compiled, not loaded: there is no device
        return 0


class FusedSpecBuilder(object):
    """Assembles an ngh_fused_spec: tensors, constants, ops, stages.

    The op vocabulary is the reference's (name, x, y, out, axis) tuples
    (gputransform.py:277-289) flattened into explicit load / compute /
    store steps on numbered registers.
    """

    def __init__(self, shape):
        shape = [int(s) for s in shape]
        if not 1 <= len(shape) <= NGH_MAX_AXES:
            raise ValueError("fused kernels take 1..3 axes, got %d" % len(shape))
        self.rank = len(shape)
        self.shape = shape + [1] * (NGH_MAX_AXES - len(shape))
        self.tensors = []
        self.consts = []
        self.ops = []
        self.stages = []
        self._stage_begin = 0
        self._stage_reds = []
        self.n_regs = 0

    def _pad_strides(self, strides):
        strides = [int(s) for s in strides]
        if len(strides) != self.rank:
            raise ValueError("strides %r do not match rank %d" % (strides, self.rank))
        return strides + [0] * (NGH_MAX_AXES - len(strides))

    def tensor(self, dev, strides, dtype=NGH_F32, scale=1.0, dev_stats=None, dev_scale=None,
               take_extent=0):
        """take_extent: for the table operand of `take`, the length of its looked-up axis (its
        stride on the take axis is then the table's stride along that axis)."""
        if len(self.tensors) >= NGH_MAX_TENSORS:
            raise ValueError("too many tensors in one fused kernel")
        self.tensors.append((int(dev), self._pad_strides(strides), int(dtype), float(scale),
                             dev_stats, dev_scale, int(take_extent)))
        return len(self.tensors) - 1

    def const(self, value):
        value = float(np.float32(value))
        for i, c in enumerate(self.consts):
            if c == value and (c != 0 or np.signbit(c) == np.signbit(value)):
                return i
        if len(self.consts) >= NGH_MAX_CONSTS:
            raise ValueError("too many constants in one fused kernel")
        self.consts.append(value)
        return len(self.consts) - 1

    def reg(self):
        """A fresh symbolic register; build() renumbers them by liveness, and it is the
        renumbered program that has to fit NGH_MAX_REGS."""
        self.n_regs += 1
        if self.n_regs > 255:
            raise ValueError("too many values in one fused kernel")
        return self.n_regs - 1

    def emit(self, name, dst=0, a=0, b=0):
        if len(self.ops) >= NGH_MAX_OPS:
            raise ValueError("too many ops in one fused kernel")
        self.ops.append((OPCODES[name], int(dst), int(a), int(b)))

    # convenience wrappers returning the destination register
    def load(self, t, dst=None):
        dst = self.reg() if dst is None else dst
        self.emit("load", dst, t)
        return dst

    def store(self, t, r, truncate=False):
        """truncate: a FLEX16 mantissa is cut toward zero (the fill rule) instead of rounded."""
        self.emit("store_trunc" if truncate else "store", t, r)

    def constant(self, value, dst=None):
        dst = self.reg() if dst is None else dst
        self.emit("const", dst, self.const(value))
        return dst

    def iota(self, axis, dst=None):
        dst = self.reg() if dst is None else dst
        self.emit("iota", dst, axis)
        return dst

    def unary(self, name, a, dst=None):
        dst = self.reg() if dst is None else dst
        self.emit(name, dst, a)
        return dst

    def binary(self, name, a, b, dst=None):
        dst = self.reg() if dst is None else dst
        self.emit(name, dst, a, b)
        return dst

    def rng(self, distribution, stream=0, dst=None):
        """dst = a fresh random number per element: "uniform" in [0, 1) or standard "normal"."""
        dst = self.reg() if dst is None else dst
        self.emit("rng_" + distribution, dst, int(stream))
        return dst

    def take(self, table, index_reg, axis, dst=None):
        """dst = table[.., (int)index_reg along `axis`, ..] (the other coordinates are the loop's)."""
        dst = self.reg() if dst is None else dst
        self.emit("take", dst, index_reg, int(table) | (int(axis) << 4))
        return dst

    def reduce(self, name, a, out_tensor):
        slot = len(self._stage_reds)
        if slot >= NGH_MAX_REDUCTIONS:
            raise ValueError("too many reductions in one stage")
        self.emit(name, slot, a)
        self._stage_reds.append(out_tensor)

    def end_stage(self):
        self.stages.append((self._stage_begin, len(self.ops), list(self._stage_reds)))
        self._stage_begin = len(self.ops)
        self._stage_reds = []

    def _compact_registers(self):
        """Renumber registers stage by stage so a register is reused once its
        value is dead; keeps the interpreter's LDS register file small."""
        src_fields = {}
        for name in UNARY_OPS:
            src_fields[OPCODES[name]] = (2,)
        for name in BINARY_OPS:
            src_fields[OPCODES[name]] = (2, 3)
        for name in REDUCTION_OPS:
            src_fields[OPCODES[name]] = (2,)
        src_fields[OPCODES["store"]] = (2,)
        src_fields[OPCODES["store_trunc"]] = (2,)
        src_fields[OPCODES["take"]] = (2,)
        writes = set(OPCODES[n] for n in UNARY_OPS + BINARY_OPS +
                     ["load", "const", "iota", "take", "rng_uniform", "rng_normal"])
        n_regs = 0
        for begin, end, _ in self.stages:
            last_use = {}
            for pc in range(begin, end):
                op = self.ops[pc]
                for f in src_fields.get(op[0], ()):
                    last_use[op[f]] = pc
            mapping, free, next_reg = {}, [], 0
            for pc in range(begin, end):
                op = list(self.ops[pc])
                srcs = [op[f] for f in src_fields.get(op[0], ())]
                for f in src_fields.get(op[0], ()):
                    op[f] = mapping[op[f]]
                # sources that die here may be reused by this op's destination
                for r in set(srcs):
                    if last_use.get(r) == pc and r in mapping:
                        free.append(mapping.pop(r))
                if op[0] in writes:
                    old = op[1]
                    if old in mapping:
                        new = mapping[old]
                    elif free:
                        new = free.pop()
                    else:
                        new = next_reg
                        next_reg += 1
                    if old not in last_use:      # never read: release straight away
                        free.append(new)
                    else:
                        mapping[old] = new
                    op[1] = new
                self.ops[pc] = tuple(op)
            n_regs = max(n_regs, next_reg)
        self.n_regs = max(n_regs, 1)

    def build(self, compact=True):
        if self._stage_begin != len(self.ops) or not self.stages:
            self.end_stage()
        if compact:
            self._compact_registers()
        if self.n_regs > NGH_MAX_REGS:
            raise ValueError("too many registers in one fused kernel (%d live values)" % self.n_regs)
        if len(self.stages) > NGH_MAX_STAGES:
            raise ValueError("too many stages in one fused kernel")
        spec = ngh_fused_spec()
        spec.abi_version = NGH_ABI_VERSION
        spec.rank = self.rank
        for i in range(NGH_MAX_AXES):
            spec.shape[i] = self.shape[i]
        spec.n_tensors = len(self.tensors)
        spec.n_ops = len(self.ops)
        spec.n_consts = len(self.consts)
        spec.n_stages = len(self.stages)
        spec.n_regs = self.n_regs
        for i, (dev, strides, dtype, scale, stats, dscale, take_extent) in enumerate(self.tensors):
            t = spec.tensors[i]
            t.dev = dev
            for j in range(NGH_MAX_AXES):
                t.strides[j] = strides[j]
            t.dtype = dtype
            t.scale = scale
            t.dev_stats = stats
            t.dev_scale = dscale
            t.take_extent = take_extent
        for i, c in enumerate(self.consts):
            spec.consts[i] = c
        for i, (opc, dst, a, b) in enumerate(self.ops):
            o = spec.ops[i]
            o.opcode, o.dst, o.a, o.b = opc, dst, a, b
        for i, (b, e, reds) in enumerate(self.stages):
            s = spec.stages[i]
            s.op_begin, s.op_end, s.n_reductions = b, e, len(reds)
            for j, t in enumerate(reds):
                s.red_out[j] = t
        return spec


def programs_count():
    """(built in, loaded) compiled programs the process knows."""
    lib = load_library()
    a, b = ctypes.c_int32(), ctypes.c_int32()
    _check(lib, lib.ngh_programs_count(ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value
