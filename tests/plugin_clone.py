"""A second graph package for the tests of ngraph_hip/plugin.py.

The real `ngraph` package cannot be imported in this environment, so the binding mechanism is
exercised against a package that is foreign in the sense that matters: separate modules and
classes under another name (`ngclone`), made from the graph front of this repository, and a
`ByteDescription` that presents its tensor descriptions the way the real package does -- strides
and offsets in bytes, nested stride tuples for flattened axes (ngraph/op_graph/axes.py:1104-1232).
"""
import os
import shutil
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FRONT = os.path.join(ROOT, "ngraph-python_amd", "ngraph_hip")
FILES = ["op_graph/__init__.py", "op_graph/axes.py", "op_graph/op_graph.py", "op_graph/autodiff.py",
         "transformers/base.py", "transformers/passes/__init__.py", "transformers/passes/passes.py"]


def make_clone(directory, name="ngclone"):
    """Write the package `name` under `directory` and put the directory on sys.path."""
    top = os.path.join(str(directory), name)
    for rel in FILES:
        dst = os.path.join(top, rel)
        os.makedirs(os.path.dirname(dst), exist_ok=True)
        with open(os.path.join(FRONT, rel)) as fh:
            text = fh.read().replace("ngraph_hip.", name + ".")
        with open(dst, "w") as fh:
            fh.write(text)
    for rel in ("__init__.py", "transformers/__init__.py"):
        with open(os.path.join(top, rel), "w") as fh:
            fh.write("")
    if str(directory) not in sys.path:
        sys.path.insert(0, str(directory))
    return name


class ByteDescription(object):
    """One of the clone's tensor descriptions as the real package would describe the view."""

    def __init__(self, td):
        self._td = td

    def _itemsize(self):
        bits = getattr(self._td.dtype, "storage_bits", None)
        return bits // 8 if bits is not None else self._td.dtype.itemsize

    @property
    def full_strides(self):
        out = []
        for axis, stride in zip(self._td.axes, self._td.full_strides):
            b = stride * self._itemsize()
            if getattr(axis, "is_flattened", False):
                # the strides of the axes it merges, innermost last; the innermost is the axis' own
                inner, nested = b, []
                for sub in reversed(list(axis.axes)):
                    nested.insert(0, inner)
                    inner *= sub.length
                out.append(tuple(nested))
            else:
                out.append(b)
        return tuple(out)

    @property
    def offset(self):
        return self._td.offset * self._itemsize()

    def __getattr__(self, name):
        return getattr(self._td, name)

    def __hash__(self):
        return hash(self._td)

    def __eq__(self, other):
        return self._td is (other._td if isinstance(other, ByteDescription) else other)
