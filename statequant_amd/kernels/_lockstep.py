"""Shared machinery of the three lockstep state classes (``PackedGDNState``, ``PackedKDAState``,
``PackedMamba2State``): what a family stores per sequence is described once, as a table of fields, and everything
else -- allocation, the per-sequence strides the C ABI wants, reset, byte accounting -- is derived from that table.

A field is (name, rows per sequence, trailing shape, dtype, accounting class).  Rows per sequence are counted in
units of "one head's entry": value heads (hv) for everything a value head owns, key heads / groups (hk) for the
buffered keys that a grouped family shares.
"""
from __future__ import annotations

import torch

from . import _hip

_KINDS = ('state', 'buffer', 'decay')


def describe_format(fmt, bits, default_group):
    """(axis along the key dimension?, group length) of a packed format; the unquantized state has neither."""
    if fmt is None:
        return False, default_group
    return fmt.axis == 'k', fmt.group


def power_of_two(n):
    return n >= 1 and (n & (n - 1)) == 0


class LockstepState:
    """Tensors of B sequences that advance together, one contiguous tensor per field.

    Subclasses call ``_allocate`` with the packed state (codes, scales) and the family's decay shape, and implement
    ``step``.  Attribute access falls through to the field tensors (``st.KB``, ``st.GCUR``, ...), and ``st.T`` is the
    name -> tensor dict the launch helpers take."""

    def _allocate(self, codes, scales, decay_shape, out_shape, out_dtype):
        B, hv, hk, m = self.B, self.HV, self.HK, self.m
        dev = codes.device
        buf_dtype = torch.int8 if self.qbuf else torch.bfloat16
        spec = [
            # name, leading rows, trailing shape, dtype, accounting class
            ('KB', B * hk, (m, self.DK), buf_dtype, 'buffer'),
            ('KBS', B * hk, (m,), torch.float16, 'buffer-scale'),
            ('UB', B * hv, (m, self.DV), buf_dtype, 'buffer'),
            ('UBS', B * hv, (m,), torch.float16, 'buffer-scale'),
            ('GB', B * hv, (m,) + decay_shape, torch.float32, 'decay'),
            ('GCUR', B * hv, decay_shape, torch.float32, 'decay'),
        ]
        fields = {'S': codes.clone(), 'SC': scales.clone()}
        self._kind = {'S': 'state', 'SC': 'state-scale', 'NPTR': 'decay'}
        for name, rows, tail, dtype, kind in spec:
            fields[name] = torch.zeros((rows,) + tuple(tail), device=dev, dtype=dtype)
            self._kind[name] = kind
        fields['NPTR'] = torch.zeros(B, hv, device=dev, dtype=torch.int32)     # a counter copy per value head
        self.__dict__['T'] = fields
        self.O = torch.zeros(out_shape, device=dev, dtype=out_dtype)
        # elements between consecutive sequences, in the order the C ABI's state struct lists the fields
        per_seq = lambda name: fields[name].numel() // B                        # noqa: E731
        self._strides = tuple(per_seq(f) for f in ('S', 'SC', 'KB', 'KBS', 'UB', 'UBS', 'GB', 'GCUR'))
        self._lay = _hip.make_layout(self)

    def __getattr__(self, name):
        fields = self.__dict__.get('T')
        if fields is not None and name in fields:
            return fields[name]
        raise AttributeError(name)

    # the reference's names for the two state tensors
    codes = property(lambda self: self.T['S'])
    scales = property(lambda self: self.T['SC'])

    @property
    def n(self):
        """Buffered tokens (all sequences and heads move together)."""
        return int(self.T['NPTR'].flatten()[0])

    def _reset(self, codes, scales):
        for name, t in self.T.items():
            if name == 'S':
                t.copy_(codes)
            elif name == 'SC':
                t.copy_(scales)
            else:
                t.zero_()

    def stored_bytes(self):
        """Resident bytes by class: 'state' (codes, and scales where the state is quantized), 'buffer' (keys and
        values, and their scales where the buffer is int8), 'decay' (decays and counters), and 'total'."""
        counted = {'state': True, 'buffer': True, 'decay': True,
                   'state-scale': self.fmt is not None, 'buffer-scale': self.qbuf}
        out = dict.fromkeys(_KINDS, 0)
        for name, t in self.T.items():
            kind = self._kind[name]
            if counted[kind]:
                out[kind.split('-')[0]] += t.numel() * t.element_size()
        out['total'] = sum(out[k] for k in _KINDS)
        return out
