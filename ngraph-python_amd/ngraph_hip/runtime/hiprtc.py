"""In-process compilation of kernel source with hiprtc (the reference compiles with NVRTC inside
the process: float_ew2.py:1626-1653 `CudaSourceFile.compile`).  A thin ctypes binding: source
text and the C++ name expressions of the kernels to instantiate in, code object and the lowered
(mangled) names of those kernels out.  Needs libhiprtc, no hipcc and no device."""
import ctypes
import os

_rtc = None


class HiprtcError(RuntimeError):
    pass


def _candidates():
    yield os.environ.get("NGH_HIPRTC_LIBRARY") or ""
    for root in (os.environ.get("ROCM_PATH"), os.environ.get("HIP_PATH"), "/opt/rocm"):
        if root:
            yield os.path.join(root, "lib", "libhiprtc.so")
    yield "libhiprtc.so"


def library():
    """libhiprtc, loaded once; HiprtcError when the machine has none."""
    global _rtc
    if _rtc is None:
        errors = []
        for path in _candidates():
            if not path:
                continue
            try:
                _rtc = ctypes.CDLL(path)
                break
            except OSError as e:
                errors.append("%s: %s" % (path, e))
        else:
            raise HiprtcError("libhiprtc was not found (%s)" % "; ".join(errors))
        _rtc.hiprtcGetErrorString.restype = ctypes.c_char_p
    return _rtc


def available():
    try:
        library()
        return True
    except HiprtcError:
        return False


def version():
    rtc = library()
    major, minor = ctypes.c_int(), ctypes.c_int()
    rtc.hiprtcVersion(ctypes.byref(major), ctypes.byref(minor))
    return "%d.%d" % (major.value, minor.value)


def _check(rtc, rc, what, log=""):
    if rc != 0:
        raise HiprtcError("%s: %s%s" % (what, rtc.hiprtcGetErrorString(rc).decode("utf-8", "replace"),
                                        ("\n" + log) if log else ""))


def compile_source(source, name_expressions, options, name="ngh_programs.hip"):
    """(code object bytes, lowered names in the order of name_expressions)."""
    rtc = library()
    prog = ctypes.c_void_p()
    _check(rtc, rtc.hiprtcCreateProgram(ctypes.byref(prog), source.encode("utf-8"), name.encode("utf-8"),
                                        0, None, None), "hiprtcCreateProgram")
    try:
        expressions = [e.encode("utf-8") for e in name_expressions]
        for e in expressions:
            _check(rtc, rtc.hiprtcAddNameExpression(prog, e), "hiprtcAddNameExpression(%s)" % e.decode())
        opts = [o.encode("utf-8") for o in options]
        rc = rtc.hiprtcCompileProgram(prog, len(opts), (ctypes.c_char_p * len(opts))(*opts))
        n = ctypes.c_size_t()
        rtc.hiprtcGetProgramLogSize(prog, ctypes.byref(n))
        log = ctypes.create_string_buffer(n.value + 1)
        rtc.hiprtcGetProgramLog(prog, log)
        _check(rtc, rc, "hiprtcCompileProgram", log.value.decode("utf-8", "replace"))
        _check(rtc, rtc.hiprtcGetCodeSize(prog, ctypes.byref(n)), "hiprtcGetCodeSize")
        code = ctypes.create_string_buffer(n.value)
        _check(rtc, rtc.hiprtcGetCode(prog, code), "hiprtcGetCode")
        lowered = []
        for e in expressions:
            out = ctypes.c_char_p()
            _check(rtc, rtc.hiprtcGetLoweredName(prog, e, ctypes.byref(out)), "hiprtcGetLoweredName(%s)" % e.decode())
            lowered.append(out.value.decode("utf-8"))
        return code.raw, lowered
    finally:
        rtc.hiprtcDestroyProgram(ctypes.byref(prog))
