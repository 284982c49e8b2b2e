"""Flex dtype, per-tensor entry and manager base (ngraph/flex/base.py:21-133)."""
from __future__ import division
import numpy as np


class Flex(object):
    """Flex dtype; supports the parts of the numpy dtype interface the transformers use.

    Arguments:
        storage_bits (int): bits used to store one number of this type
        exp_bits (int): bits of the shared exponent (DEC)
    """

    def __init__(self, storage_bits, exp_bits=5):
        self.storage_bits = storage_bits
        self.itemsize = int(storage_bits // 8)
        self.type = "flex"
        self.str = "<i2"
        self.name = "flex"
        self.exp_bits = exp_bits

    def __eq__(self, other):
        return (isinstance(other, Flex) and self.storage_bits == other.storage_bits and
                self.type is other.type)

    def __ne__(self, other):
        return not self == other

    def __hash__(self):
        return hash(("flex", self.storage_bits))

    def __repr__(self):
        return "flex%d" % self.storage_bits


flex16 = Flex(storage_bits=16)


class FlexEntry(object):
    """Associated with every flex tensor: its id, dtype and current scale = 2**-dec."""

    def __init__(self, _id, dtype, init_dec):
        self._id = _id
        self.dtype = dtype
        self.scale = 1.0 / 2 ** init_dec

    @property
    def flex_id(self):
        return self._id

    @property
    def dec(self):
        return int(np.log2(1.0 / self.scale))


class FlexManager(object):
    """Manages flex tensors.  Abstract base class."""

    default_dec = 8   # fixed point resolution and default initial dec

    @staticmethod
    def fixed_point_resolution():
        return 1.0 / 2 ** FlexManager.default_dec

    def __init__(self):
        self.flex_entries = {}
        self._num_flex_tensors = 0

    def manage_before_computation(self, *args):
        raise NotImplementedError

    def manage_after_computation(self, *args):
        raise NotImplementedError
