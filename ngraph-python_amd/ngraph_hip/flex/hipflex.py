"""The flex manager for the HIP backend.

Stands where `autoflex.gpu` stands for the reference (call sites:
ngraph/transformers/flexgputransform.py:58-217, gpu/float_ew2.py:371,
testing/execution.py:269-270): `HipFlexManager.{make_flex_entry, allocate,
manage_before_computation, manage_after_computation, autoflex_count,
fixed_point_resolution}`, `HipFlexEntry.{scale, dec, ptr, flex_id,
manage_before_computation(value), manage_after_computation(maxabs, count)}`,
`hipflex16.{storage_dtype, storage_bits, dtype_name, pclip, nclip, get_scale}`.

`autoflex` itself is not part of the reference tree, so the exponent policy
here is a re-derivation: the smallest rule set that reproduces the reference's
flex known-answer vectors (tests/flex_tests/test_flexew/*).
  first use    tightest fit: dec = 14 - floor(log2(max|value|)) within [0, 31];
               an all-zero first value gets default_dec
  overflow     stored max|mantissa| >= 32767: dec -= 2; the sample enters the
               history as twice the saturated magnitude
  otherwise    dec = tightest fit of max(h) + 3 * std(h) over the last 16
               recorded max|value|
With fixed_point=True every tensor keeps default_dec.
"""
from __future__ import division
import collections
import math

import numpy as np

from ngraph_hip.flex.base import Flex, FlexEntry, FlexManager


class HipFlex(Flex):
    dtype_name = "flex"

    def __init__(self, storage_bits, exp_bits=5):
        super(HipFlex, self).__init__(storage_bits, exp_bits)
        self.storage_dtype = np.dtype(np.int16)
        self.pclip = 2 ** (storage_bits - 1) - 1
        self.nclip = -2 ** (storage_bits - 1)
        self.min_dec = 0
        self.max_dec = 2 ** exp_bits - 1

    def fit_dec(self, maxabs):
        """Largest dec at which maxabs still fits storage_bits - 1 bits; None for 0 / NaN."""
        maxabs = abs(float(maxabs))
        if maxabs == 0.0 or math.isnan(maxabs):
            return None
        if math.isinf(maxabs):
            return self.min_dec
        dec = (self.storage_bits - 2) - int(math.floor(math.log2(maxabs)))
        return max(self.min_dec, min(self.max_dec, dec))

    def get_scale(self, maxabs):
        dec = self.fit_dec(maxabs)
        return 1.0 / 2 ** (FlexManager.default_dec if dec is None else dec)


hipflex16 = HipFlex(storage_bits=16)


class HipFlexEntry(FlexEntry):
    history_length = 16
    gamma = 3.0
    overflow_dec_step = 2

    def __init__(self, _id, dtype, init_dec, manager, name=None):
        super(HipFlexEntry, self).__init__(_id, dtype, init_dec)
        self.manager = manager
        self.name = name
        self.initialized = False
        self.history = collections.deque(maxlen=self.history_length)
        self.ptr = None                 # device int32 word receiving max|mantissa|
        self.last_maxabs = 0
        self.last_count = -1
        self.next_dec = None

    @property
    def dec(self):
        return int(round(-math.log2(self.scale)))

    def set_dec(self, dec):
        self.scale = 1.0 / 2 ** int(dec)

    # ---- policy -------------------------------------------------------------------------
    # `scale` always describes the mantissas currently in memory.  The policy's choice for
    # the NEXT write is kept in `next_dec` and only takes effect in adjust_scale(), which
    # runs immediately before something overwrites the whole tensor.
    def init_from_value(self, maxabs_value):
        if not self.manager.fixed_point:
            dec = self.dtype.fit_dec(maxabs_value)
            self.set_dec(FlexManager.default_dec if dec is None else dec)
        self.next_dec = self.dec
        self.initialized = True

    def adjust_scale(self):
        if self.initialized and self.next_dec is not None:
            self.set_dec(self.next_dec)

    def manage_before_computation(self, value=None):
        """Host write path: the first value a tensor receives fixes its initial scale; later
        writes use the scale the policy chose after the previous one."""
        if not self.initialized:
            if value is not None:
                value = np.asarray(value, dtype=np.float64)
                self.init_from_value(float(np.max(np.abs(value))) if value.size else 0.0)
        else:
            self.adjust_scale()

    def manage_after_computation(self, maxabs, autoflex_count):
        """Record max|mantissa| of what was just stored and choose the next scale."""
        maxabs = int(maxabs)
        self.last_maxabs, self.last_count = maxabs, autoflex_count
        self.initialized = True
        if self.manager.fixed_point:
            return
        value = maxabs * self.scale
        if maxabs >= self.dtype.pclip:
            self.history.append(2.0 * value)
            self.next_dec = max(self.dtype.min_dec, self.dec - self.overflow_dec_step)
            return
        self.history.append(value)
        h = np.asarray(self.history, dtype=np.float64)
        dec = self.dtype.fit_dec(float(h.max() + self.gamma * h.std()))
        self.next_dec = self.dec if dec is None else dec

    def reset_entry(self):
        self.history.clear()
        self.initialized = False
        self.next_dec = None
        self.set_dec(FlexManager.default_dec)


class HipFlexManager(FlexManager):
    """Creates entries, owns their device statistics words, runs the policy around kernels."""

    def __init__(self, fixed_point=False, verbose=False):
        super(HipFlexManager, self).__init__()
        self.fixed_point = fixed_point
        self.verbose = verbose
        self.autoflex_count = 0
        self.runtime = None
        self._stats_base = None
        self._allocated = 0

    def make_flex_entry(self, name=None, dtype=None):
        flex_id = self._num_flex_tensors
        entry = HipFlexEntry(flex_id, dtype or hipflex16, FlexManager.default_dec, self, name=name)
        self.flex_entries[flex_id] = entry
        self._num_flex_tensors += 1
        return entry

    def allocate(self, runtime=None):
        """Device words for every entry created so far (idempotent; grows when entries were added)."""
        if runtime is not None:
            self.runtime = runtime
        n = self._num_flex_tensors
        if n == 0 or n <= self._allocated:
            return
        base = self.runtime.stats_alloc(n)
        self._stats_base, self._allocated = base, n
        for flex_id, entry in self.flex_entries.items():
            entry.ptr = base + 4 * flex_id

    # ---- around kernels (flexgputransform.py:347-366) ------------------------------------
    def manage_before_computation(self, kernel):
        in_place = getattr(kernel, "in_place_flex_ids", ())
        for entry in kernel.output_flex_entries:
            if entry.flex_id not in in_place:
                # a tensor the kernel also reads keeps the scale its data was stored with
                entry.adjust_scale()
            self.runtime.stats_reset(entry.ptr, 1)

    def manage_after_computation(self, kernel):
        for entry in kernel.output_flex_entries:
            maxabs = int(self.runtime.stats_read(entry.ptr, 1)[0])
            entry.manage_after_computation(maxabs, self.autoflex_count)
            if self.verbose:
                print("flex %s: maxabs %d -> dec %d" % (entry.name, maxabs, entry.dec))

    def set_h5py_file(self, data_file):
        self.data_file = data_file

    def save_diagnostic_data(self):
        pass
