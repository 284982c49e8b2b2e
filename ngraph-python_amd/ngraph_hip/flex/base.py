"""The flex storage type, the per-tensor entry and the manager interface that the flex
transformer and its callers read (ngraph/flex/base.py:21-133): `Flex.{storage_bits, itemsize,
type, str, name, exp_bits}`, `FlexEntry.{flex_id, dtype, scale, dec}`,
`FlexManager.{default_dec, fixed_point_resolution, flex_entries, manage_before_computation,
manage_after_computation}`."""
from __future__ import division
import math


class Flex(object):
    """A storage type of `storage_bits`-bit integer mantissas that share one exponent of
    `exp_bits` bits per tensor.  It stands where a NumPy dtype does, so it answers the dtype
    attributes the transformers ask for."""

    type = "flex"
    name = "flex"

    def __init__(self, storage_bits, exp_bits=5):
        self.storage_bits, self.exp_bits = storage_bits, exp_bits

    @property
    def itemsize(self):
        return self.storage_bits // 8

    @property
    def str(self):
        # the NumPy type string of the mantissas: little-endian signed integers
        return "<i%d" % self.itemsize

    def _key(self):
        return (Flex.type, self.storage_bits)

    def __eq__(self, other):
        return isinstance(other, Flex) and self._key() == other._key()

    def __ne__(self, other):
        return not self.__eq__(other)

    def __hash__(self):
        return hash(self._key())

    def __repr__(self):
        return "flex%d" % self.storage_bits


flex16 = Flex(16)

# the name the flex transformer registers under (ngraph/flex/names.py)
flex_gpu_transformer_name = "flexhip"


class FlexEntry(object):
    """What is known about one flex tensor: which one it is, its storage type and the exponent
    its mantissas are stored with (value = mantissa * 2**-dec)."""

    def __init__(self, _id, dtype, init_dec):
        self._id, self.dtype = _id, dtype
        self._dec = int(init_dec)

    flex_id = property(lambda self: self._id)

    @property
    def dec(self):
        return self._dec

    @property
    def scale(self):
        return math.ldexp(1.0, -self._dec)

    @scale.setter
    def scale(self, value):
        mantissa, exponent = math.frexp(value)            # value = mantissa * 2**exponent, mantissa in [0.5, 1)
        if mantissa != 0.5:
            raise ValueError("a flex scale is a power of two, not %r" % (value,))
        self._dec = 1 - exponent


class FlexManager(object):
    """Keeps the entries of a transformer's flex tensors; a backend says what happens around
    each kernel."""

    default_dec = 8         # exponent of a tensor nothing is known about yet = the fixed-point resolution

    def __init__(self):
        self._num_flex_tensors = 0
        self.flex_entries = {}

    @staticmethod
    def fixed_point_resolution():
        return math.ldexp(1.0, -FlexManager.default_dec)

    def manage_before_computation(self, *args):
        raise NotImplementedError

    def manage_after_computation(self, *args):
        raise NotImplementedError
