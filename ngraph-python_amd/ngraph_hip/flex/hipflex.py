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

from ngraph_hip.flex.base import Flex, FlexManager


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
        _, e = math.frexp(maxabs)            # maxabs = m * 2**e, 0.5 <= m < 1: floor(log2) = e - 1
        dec = (self.storage_bits - 2) - (e - 1)
        return max(self.min_dec, min(self.max_dec, dec))

    def get_scale(self, maxabs):
        dec = self.fit_dec(maxabs)
        return 1.0 / 2 ** (FlexManager.default_dec if dec is None else dec)


hipflex16 = HipFlex(storage_bits=16)

HISTORY = 16
#: host mirror of struct ngh_flex_state (include/ngraph_hip.h)
STATE_DTYPE = np.dtype([("stats", "<i4"), ("dec", "<i4"), ("next_dec", "<i4"), ("initialized", "<i4"),
                        ("scale", "<f4"), ("hist_len", "<i4"), ("hist_pos", "<i4"),
                        ("last_maxabs", "<i4"), ("last_count", "<i4"), ("pad_", "<i4"),
                        ("history", "<f8", (HISTORY,))])
assert STATE_DTYPE.itemsize == 168


def _policy_step(rec, maxabs, count, dtype):
    """Record max|mantissa| of what was just stored and choose the next exponent.

    Sequential double-precision steps; csrc/ngh_flex.h flex_update_kernel performs the same
    steps in the same order on the device, and the two must stay equivalent."""
    maxabs = int(maxabs)
    rec["last_maxabs"], rec["last_count"], rec["initialized"] = maxabs, count, 1
    value = float(maxabs) * float(rec["scale"])
    pos = int(rec["hist_pos"])
    hist = rec["history"]
    if maxabs >= dtype.pclip:
        hist[pos] = 2.0 * value
        rec["hist_pos"] = (pos + 1) % HISTORY
        rec["hist_len"] = min(HISTORY, int(rec["hist_len"]) + 1)
        rec["next_dec"] = max(dtype.min_dec, int(rec["dec"]) - 2)
        return
    hist[pos] = value
    rec["hist_pos"] = (pos + 1) % HISTORY
    rec["hist_len"] = min(HISTORY, int(rec["hist_len"]) + 1)
    n = int(rec["hist_len"])
    mx, total = float(hist[0]), 0.0
    for j in range(n):
        h = float(hist[j])
        mx = h if h > mx else mx
        total = total + h
    mean = total / float(n)
    ss = 0.0
    for j in range(n):
        d = float(hist[j]) - mean
        ss = ss + d * d
    sd = math.sqrt(ss / float(n))
    dec = dtype.fit_dec(mx + 3.0 * sd)
    rec["next_dec"] = int(rec["dec"]) if dec is None else dec


class HipFlexEntry(object):
    """Exponent state of one flex tensor: a view of one record of the manager's state table.

    `scale` always describes the mantissas currently in memory; the policy's choice for the
    next write is `next_dec`, applied by adjust_scale() right before the whole tensor is
    overwritten.
    """

    def __init__(self, _id, dtype, init_dec, manager, name=None):
        self._id = _id
        self.dtype = dtype
        self.manager = manager
        self.name = name
        rec = self._rec(sync=False)
        rec["dec"], rec["next_dec"], rec["scale"] = init_dec, -1, 1.0 / 2 ** init_dec

    def _rec(self, sync=True):
        if sync:
            self.manager.pull()
        return self.manager.table[self._id]

    def _touch(self):
        self.manager.host_dirty = True

    @property
    def flex_id(self):
        return self._id

    @property
    def scale(self):
        return float(self._rec()["scale"])

    @property
    def dec(self):
        return int(self._rec()["dec"])

    @property
    def next_dec(self):
        v = int(self._rec()["next_dec"])
        return None if v < 0 else v

    @property
    def initialized(self):
        return bool(self._rec()["initialized"])

    @property
    def last_maxabs(self):
        return int(self._rec()["last_maxabs"])

    @property
    def history(self):
        rec = self._rec()
        n, pos = int(rec["hist_len"]), int(rec["hist_pos"])
        h = [float(x) for x in rec["history"][:n]]
        return h if n < HISTORY else h[pos:] + h[:pos]

    @property
    def ptr(self):
        """Device address of this tensor's statistics word."""
        return self.manager.state_address(self._id, "stats")

    @property
    def scale_ptr(self):
        return self.manager.state_address(self._id, "scale")

    def set_dec(self, dec):
        rec = self._rec()
        rec["dec"], rec["scale"] = int(dec), 1.0 / 2 ** int(dec)
        self._touch()

    # ---- policy -------------------------------------------------------------------------
    def init_from_value(self, maxabs_value):
        rec = self._rec()
        if not self.manager.fixed_point:
            dec = self.dtype.fit_dec(maxabs_value)
            dec = FlexManager.default_dec if dec is None else dec
            rec["dec"], rec["scale"] = dec, 1.0 / 2 ** dec
        rec["next_dec"], rec["initialized"] = rec["dec"], 1
        self._touch()

    def adjust_scale(self):
        rec = self._rec()
        if rec["initialized"] and rec["next_dec"] >= 0:
            rec["dec"], rec["scale"] = rec["next_dec"], 1.0 / 2 ** int(rec["next_dec"])
            self._touch()

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
        rec = self._rec()
        if self.manager.fixed_point:
            rec["last_maxabs"], rec["last_count"], rec["initialized"] = int(maxabs), autoflex_count, 1
        else:
            _policy_step(rec, maxabs, autoflex_count, self.dtype)
        self._touch()

    def reset_entry(self):
        rec = self._rec()
        rec["hist_len"] = rec["hist_pos"] = rec["initialized"] = 0
        rec["next_dec"] = -1
        rec["dec"], rec["scale"] = FlexManager.default_dec, 1.0 / 2 ** FlexManager.default_dec
        self._touch()


class HipFlexManager(FlexManager):
    """Creates entries, owns the state table (host mirror + device copy), runs the policy.

    resident=False  statistics come back to the host after every kernel and the policy runs
                    in Python, as in the reference (flexgputransform.py:347-366).
    resident=True   kernels read scales from, and the policy runs on, the device copy of the
                    table; the host mirror is refreshed only when somebody looks at it.
    """

    def __init__(self, fixed_point=False, verbose=False, resident=False):
        super(HipFlexManager, self).__init__()
        self.fixed_point = fixed_point
        self.verbose = verbose
        self.resident = resident and not fixed_point
        self.autoflex_count = 0
        self.runtime = None
        self.table = np.zeros(64, dtype=STATE_DTYPE)
        self.dev_table = None          # device address of the table copy
        self._dev_capacity = 0
        self.host_dirty = False        # host mirror changed since the last push
        self.device_dirty = False      # device copy changed since the last pull

    def make_flex_entry(self, name=None, dtype=None):
        flex_id = self._num_flex_tensors
        if flex_id >= len(self.table):
            self.pull()
            grown = np.zeros(2 * len(self.table), dtype=STATE_DTYPE)
            grown[:len(self.table)] = self.table
            self.table = grown
        self._num_flex_tensors += 1
        entry = HipFlexEntry(flex_id, dtype or hipflex16, FlexManager.default_dec, self, name=name)
        self.flex_entries[flex_id] = entry
        self.host_dirty = True
        return entry

    # ---- device copy ---------------------------------------------------------------------
    def allocate(self, runtime=None):
        """(Re)create the device copy so it covers every entry made so far."""
        if runtime is not None:
            self.runtime = runtime
        n = self._num_flex_tensors
        if n == 0 or n <= self._dev_capacity:
            return
        self.pull()
        capacity = len(self.table)
        self.dev_table = self.runtime.flex_states_alloc(capacity)
        self._dev_capacity = capacity
        self.host_dirty = True
        self.push()

    def state_address(self, flex_id, field):
        if self.dev_table is None:
            return None
        return self.dev_table + flex_id * STATE_DTYPE.itemsize + STATE_DTYPE.fields[field][1]

    def push(self):
        if self.host_dirty and self.dev_table is not None:
            self.runtime.flex_states_write(self.dev_table, 0, self.table[:self._dev_capacity])
        self.host_dirty = False

    def pull(self):
        if self.device_dirty and self.dev_table is not None:
            self.device_dirty = False
            self.runtime.flex_states_read(self.dev_table, 0, self.table[:self._dev_capacity])

    # ---- around kernels (flexgputransform.py:347-366) ------------------------------------
    def manage_before_computation(self, kernel):
        entries = kernel.output_flex_entries
        if not entries:
            return
        in_place = getattr(kernel, "in_place_flex_ids", ())
        if self.resident:
            self.push()
            self.runtime.flex_prepare(self.dev_table, [e.flex_id for e in entries],
                                      [1 if e.flex_id in in_place else 0 for e in entries])
            self.device_dirty = True
            return
        for entry in entries:
            if entry.flex_id not in in_place:
                # a tensor the kernel also reads keeps the scale its data was stored with
                entry.adjust_scale()
        for entry in entries:
            self.runtime.stats_reset(entry.ptr, 1)

    def manage_after_computation(self, kernel):
        entries = kernel.output_flex_entries
        if not entries:
            return
        if self.resident:
            self.runtime.flex_update(self.dev_table, [e.flex_id for e in entries], self.autoflex_count)
            self.device_dirty = True
            return
        for entry in entries:
            maxabs = int(self.runtime.stats_read(entry.ptr, 1)[0])
            entry.manage_after_computation(maxabs, self.autoflex_count)
            if self.verbose:
                print("flex %s: maxabs %d -> next dec %s" % (entry.name, maxabs, entry.next_dec))

    def set_h5py_file(self, data_file):
        """Where save_diagnostic_data writes (flexgputransform.py:105-114 hands autoflex an h5py
        file for the same purpose): an object with h5py's `create_group` / `create_dataset`, or a
        path, which gets a NumPy .npz archive."""
        self.data_file = data_file

    def diagnostic_data(self):
        """Per flex tensor, by name: the exponent in use and the one chosen for the next write,
        the scale, the last max |mantissa|, whether it overflowed, and the recorded maxima."""
        out = {}
        for flex_id, entry in sorted(self.flex_entries.items()):
            name = "%04d_%s" % (flex_id, entry.name or "tensor")
            next_dec = entry.next_dec
            out[name] = {"dec": entry.dec, "next_dec": -1 if next_dec is None else next_dec, "scale": entry.scale,
                         "initialized": int(entry.initialized), "last_maxabs": entry.last_maxabs,
                         "overflow": int(entry.last_maxabs >= entry.dtype.pclip),
                         "history": np.asarray(entry.history, dtype=np.float64)}
        return out

    def save_diagnostic_data(self):
        target = getattr(self, "data_file", None)
        if target is None:
            return
        data = self.diagnostic_data()
        if hasattr(target, "create_group"):
            step = target.create_group("autoflex_count_%d" % self.autoflex_count)
            for name, fields in data.items():
                group = step.create_group(name)
                for key, value in fields.items():
                    group.create_dataset(key, data=value)
            return
        flat = {"%s/%s" % (name, key): np.asarray(value) for name, fields in data.items() for key, value in fields.items()}
        flat["autoflex_count"] = np.asarray(self.autoflex_count)
        np.savez(target, **flat)
