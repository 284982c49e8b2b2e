"""`hipgpu` and `flexhip` as transformers of the real `ngraph` package.

What a maintainer of ngraph-python adds to `ngraph/transformers/__init__.py`, next to the
other optional backends (lines 34-52 there import them inside try/except):

    try:
        import ngraph_hip.plugin
        ngraph_hip.plugin.register()          # 'hipgpu' and 'flexhip' join Transformer.transformers
    except ImportError:
        pass

`register(package)` makes transformer classes that derive from THAT package's
`ComputationGraphTransformer` (ngraph/transformers/base.py:644-801), so they land in its
registry through its metaclass (base.py:265-279) and are made by its
`make_transformer_factory` / `allocate_transformer` (base.py:834-847).  Nothing of the
package is imported before `register` is called, so this module imports anywhere.

How: the lowering (`ngraph_hip/transformers/hiptransform.py` and the modules it is made of --
`hipdevice`, `hiplowering`, `hipmoments`, `hipchains`, `hipplanner` --, `flexhiptransform.py`,
`passes/hippasses.py`) reaches the graph package only through `import` statements naming
`ngraph_hip.op_graph...`, `ngraph_hip.transformers.base` and
`ngraph_hip.transformers.passes.passes` -- the modules this repository carries as stand-ins for
`ngraph.op_graph...`, `ngraph.transformers.base` and `ngraph.transformers.passes.passes`, with
the same names inside.  `bind(package)` executes those source files a second time as
modules of their own in which these imports resolve to the package's modules instead: the op
classes the lowering tests with isinstance, the base classes its own classes derive from and
the pass driver are then the package's.  The kernels, the C ABI binding, the flex manager and
the run-time compilation are independent of the graph package and shared.

The real package describes tensors differently from the stand-in in two ways, both handled
by `ElementView`, which the bound modules apply to every tensor description they look at:
strides and offsets are in bytes there (ngraph/op_graph/axes.py:1174-1232; elements here, as
in the kernels' arguments), and a flattened axis carries a nested tuple of the strides of the
axes it merges (axes.py:1104-1150 `_make_stride`), of which a kernel needs the innermost one
(axes.py:1090-1101 `_reduce_strides`).
"""
from __future__ import division
import importlib
import importlib.util
import sys
import types

# ------------------------------------------------------------------------------ pure adapters


def flat_stride(stride):
    """The stride of one axis from the package's (possibly nested) description: a flattened
    axis holds a tuple of the strides of the axes collapsed into it, itself possibly nested;
    the axis advances by the smallest of them (`_reduce_nested(elem, inf, min)`,
    ngraph/op_graph/axes.py:1076-1101)."""
    if isinstance(stride, (tuple, list)):
        inner = [flat_stride(s) for s in stride]
        if not inner:
            raise ValueError("a flattened axis without strides")
        return min(inner)
    return int(stride)


def flat_size(size):
    """The extent of one axis from a (possibly nested) size: the product of what it merges
    (`_reduce_nested(_, 1, operator.mul)`, axes.py:1640-1641)."""
    if isinstance(size, (tuple, list)):
        n = 1
        for s in size:
            n *= flat_size(s)
        return n
    return int(size)


def element_strides(full_strides, itemsize):
    """Byte strides, nested or not, -> one element stride per axis."""
    itemsize = int(itemsize)
    out = []
    for s in full_strides:
        b = flat_stride(s)
        if b % itemsize:
            raise ValueError("stride of %d bytes is not a multiple of the item size %d" % (b, itemsize))
        out.append(b // itemsize)
    return tuple(out)


def element_offset(offset, itemsize):
    offset, itemsize = int(offset), int(itemsize)
    if offset % itemsize:
        raise ValueError("offset of %d bytes is not a multiple of the item size %d" % (offset, itemsize))
    return offset // itemsize


def storage_itemsize(dtype):
    """Bytes per element in device memory: numpy dtypes say so; a flex dtype stores
    `storage_bits` (ngraph/flex/base.py:24-61)."""
    bits = getattr(dtype, "storage_bits", None)
    if bits is not None:
        return int(bits) // 8
    return int(dtype.itemsize)


class ElementView(object):
    """A tensor description of the package seen the way the lowering reads one: `shape`,
    `full_strides` (elements, flat), `offset` (elements), `c_contiguous`; everything else
    (`axes`, `base`, `dtype`, `parameter_key`, `name`, ...) is the description's own.  It
    hashes and compares as the description it wraps, so it finds the device tensors the
    transformer keeps in dictionaries keyed by descriptions (base.py:520-600)."""

    __slots__ = ("raw", "shape", "full_strides", "offset")

    def __init__(self, td):
        itemsize = storage_itemsize(td.dtype)
        self.raw = td
        self.shape = tuple(int(n) for n in td.shape)
        self.full_strides = element_strides(td.full_strides, itemsize)
        self.offset = element_offset(td.offset, itemsize)

    def __getattr__(self, name):              # only reached for what the slots do not hold
        return getattr(self.raw, name)

    def __hash__(self):
        return hash(self.raw)

    def __eq__(self, other):
        return self.raw == (other.raw if isinstance(other, ElementView) else other)

    def __ne__(self, other):
        return not self.__eq__(other)

    @property
    def c_contiguous(self):
        acc = 1
        for length, stride in zip(reversed(self.shape), reversed(self.full_strides)):
            if length != 1 and stride != acc:
                return False
            acc *= length
        return True


def adapt_tensor_description(td):
    """ElementView of a description of the package (idempotent)."""
    return td if isinstance(td, ElementView) else ElementView(td)


# ------------------------------------------------------------------------------ binding

#: stand-in module of this repository -> module of the package, relative to the package's name
SUBSTITUTED = {
    "ngraph_hip.op_graph.op_graph": "op_graph.op_graph",
    "ngraph_hip.op_graph.axes": "op_graph.axes",
    "ngraph_hip.op_graph": "op_graph",
    "ngraph_hip.transformers.base": "transformers.base",
    "ngraph_hip.transformers.passes.passes": "transformers.passes.passes",
}
#: modules executed again per package, in dependency order
REBOUND = ("ngraph_hip.transformers.passes.hippasses", "ngraph_hip.transformers.hipdevice",
           "ngraph_hip.transformers.hiplowering", "ngraph_hip.transformers.hipmoments",
           "ngraph_hip.transformers.hipchains", "ngraph_hip.transformers.hipplanner",
           "ngraph_hip.transformers.hiptransform", "ngraph_hip.transformers.flexhiptransform")

_bound = {}


class Bound(object):
    """The backend's modules bound to one graph package."""

    def __init__(self, package, modules):
        self.package, self.modules = package, modules
        self.hiptransform = modules["ngraph_hip.transformers.hiptransform"]
        self.flexhiptransform = modules["ngraph_hip.transformers.flexhiptransform"]
        self.HipTransformer = self.hiptransform.HipTransformer
        self.FlexHipTransformer = self.flexhiptransform.FlexHipTransformer


def _import_for(package, rebound):
    """An `__import__` for the re-executed sources: stand-in modules resolve to the package's,
    modules already re-executed to their bound instances, everything else as usual."""
    real_import = __import__

    def resolve(name):
        if name in rebound:
            return rebound[name]
        if name in SUBSTITUTED:
            return importlib.import_module(package + "." + SUBSTITUTED[name])
        return None

    def imp(name, globals=None, locals=None, fromlist=(), level=0):
        if level == 0:
            mod = resolve(name)
            if mod is not None:
                # `from a.b import c`: the module itself; `import a.b`: not used by these sources
                if fromlist:
                    for item in fromlist:        # `from ngraph_hip.op_graph import op_graph`
                        sub = resolve(name + "." + item)
                        if sub is not None and not hasattr(mod, item):
                            setattr(mod, item, sub)
                    return mod
                raise ImportError("plain `import %s` cannot be rebound; use `from ... import`" % name)
        return real_import(name, globals, locals, fromlist, level)
    return imp


def bind(package="ngraph", adapt=adapt_tensor_description):
    """Execute the lowering's modules against `package` (importable, with the layout of
    ngraph-python: `<package>.op_graph.op_graph`, `<package>.transformers.base`,
    `<package>.transformers.passes.passes`).  `adapt` turns the package's tensor descriptions
    into the element-stride view the lowering reads (None: they already are).  Creating the
    transformer classes registers them with the package.  Returns a `Bound`; repeated calls for
    one package return the same one."""
    if package in _bound:
        return _bound[package]
    importlib.import_module(package + ".transformers.base")          # fail early, with the real reason
    modules = {}
    builtins_mod = importlib.import_module("builtins")
    for name in REBOUND:
        spec = importlib.util.find_spec(name)
        source = spec.loader.get_source(name)
        mod = types.ModuleType("%s__on__%s" % (name, package.replace(".", "_")))
        mod.__file__ = spec.origin
        scope = dict(vars(builtins_mod))
        scope["__import__"] = _import_for(package, modules)
        mod.__dict__["__builtins__"] = scope
        sys.modules[mod.__name__] = mod
        try:
            exec(compile(source, spec.origin, "exec"), mod.__dict__)
        except Exception:
            del sys.modules[mod.__name__]
            raise
        if adapt is not None and hasattr(mod, "_adapt_td"):
            mod._adapt_td = adapt
        modules[name] = mod
    _bound[package] = Bound(package, modules)
    return _bound[package]


def register(package="ngraph"):
    """Make `hipgpu` and `flexhip` transformers of `package`; returns (HipTransformer,
    FlexHipTransformer).  Raises ImportError when the package is not importable, and the
    package's UnsupportedTransformerException only later, when a transformer is constructed
    on a machine without libngraph_hip.so or without an MI355X."""
    b = bind(package)
    return b.HipTransformer, b.FlexHipTransformer
