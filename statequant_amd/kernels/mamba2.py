"""Packed recurrent state for Mamba2 / SSD layers on HIP kernels: lockstep state and slot-addressed layout.

Mirrors the reference's ``statequant/kernels/mamba2.py`` (``/root/reference/src/statequant/kernels/mamba2.py``).
Per head h of H, group g = h // (H / G), one token:

    dt = softplus(dt_raw + dt_bias), clamped to dt_limit;    S = exp(A_h dt) S + (dt x) B^T;    y = S C + D_h x

This is the packed gated-delta decode with key B (per group), query C, buffered value u = dt x (no delta term, no
normalisation) and a scalar decay per head (mamba2.py:9-15).  States are [B, H, head_dim, d_state] = [B, H, d_v, d_k]
(value-major, vLLM's ssm state).
"""
from __future__ import annotations

import ctypes

import torch

from . import _hip
from ._lockstep import LockstepState, describe_format, power_of_two
from .fold import _bits, _require_kernel, pack_vk, packed_format, unpack_vk
from .slots import SlotLayout, field_table, slot_state, state_fields


def _activated_dt(dt, A, dt_bias, dt_softplus, dt_limit):
    """Raw dt [B, H] -> (dt after bias / softplus / clamp, log decay A dt), fp32 -- the kernel's gate in torch
    (mamba2.py:45-54).  softplus switches to the identity above 20, as the kernels do."""
    t = dt.float() if dt_bias is None else dt.float() + dt_bias.float()
    if dt_softplus:
        t = torch.where(t > 20.0, t, torch.log(torch.exp(t.clamp(max=20.0)) + 1.0))
    lo, hi = (0.0, float('inf')) if dt_limit is None else (float(dt_limit[0]), float(dt_limit[1]))
    if (lo, hi) != (0.0, float('inf')):
        t = torch.clamp(t, min=lo, max=hi)
    return t, t * A.float()


def mamba2_recurrence(S, x, dt, B, C, A, D=None, dt_bias=None, dt_softplus=False, dt_limit=None):
    """The unquantized recurrence, one token, on S [B, H, d_v, d_k] in place (mamba2.py:57-70):
    S <- exp(A dt) S + (dt x) B^T, y = S C + D x.  x [B, H, d_v], dt [B, H], B / C [B, G, d_k] (G groups, each shared
    by H / G heads), A / D / dt_bias [H].  Returns y [B, H, d_v] fp32."""
    heads, groups = dt.shape[1], B.shape[1]
    step, log_decay = _activated_dt(dt, A, dt_bias, dt_softplus, dt_limit)
    share = heads // groups
    key = torch.repeat_interleave(B.float(), share, dim=1)              # [B, H, d_k]
    query = torch.repeat_interleave(C.float(), share, dim=1)
    xf = x.float()
    S *= log_decay.exp()[:, :, None, None]
    S += torch.einsum('bhv,bhk->bhvk', step[..., None] * xf, key)
    y = (S * query[:, :, None, :]).sum(-1)
    return y if D is None else y + xf * D.float().view(1, heads, 1)


def _common(st, fmt, hv, hk, dk, dv, m, buffer_bits):
    """Geometry and format attributes of a Mamba2 state / layout (names as the launch helpers read them)."""
    st.fmt = packed_format(fmt)
    st.bits = _bits(st.fmt)
    st.axk, st.group = describe_format(st.fmt, st.bits, default_group=16)
    if hv % hk:
        raise AssertionError(f'{hv} heads do not split into {hk} groups')
    if not (power_of_two(m) and m <= 32):
        raise AssertionError('m must be a power of two <= 32')
    if buffer_bits not in (8, 16):
        raise AssertionError(f'buffer_bits {buffer_bits}: 8 (int8) or 16 (bf16)')
    assert dk >= 16 and dk % 2 == 0, dk
    if st.fmt is not None:
        axis_len = dk if st.axk else dv
        assert power_of_two(st.group), f'group {st.group} must be a power of two'
        assert axis_len % st.group == 0, f'group {st.group} must divide d_{st.fmt.axis} ({dk}, {dv})'
    st.HV, st.HK, st.gqa = hv, hk, hv // hk
    st.DK, st.DV, st.m = dk, dv, m
    st.buffer_bits, st.qbuf = buffer_bits, buffer_bits == 8


def _launch(st, lay, rows, x, dt, B, C, out, A, D, dt_bias, dt_softplus, dt_limit, idx, T, strides, nptr_stride,
            order=None):
    """One ``sq_mamba2_step`` call (replaces mamba2.py:223-241)."""
    assert x.stride(-1) == 1 and B.stride(-1) == 1 and C.stride(-1) == 1 and dt.stride(-1) == 1
    assert x.stride(-2) == st.DV and out.stride(-1) == 1 and out.stride(-2) == st.DV
    assert B.stride(-2) == st.DK and C.stride(-2) == st.DK
    assert A.is_contiguous() and (D is None or D.is_contiguous()) and (dt_bias is None or dt_bias.is_contiguous())
    _hip.same_device('Mamba2 step', T['S'], idx=idx, x=x, dt=dt, B=B, C=C, A=A, D=D, dt_bias=dt_bias, out=out)
    clamp = dt_limit is not None and tuple(dt_limit) != (0., float('inf'))
    lo, hi = (float(dt_limit[0]), float(dt_limit[1])) if clamp else (0., 0.)
    a = _hip.SqMamba2Args(
        st=_hip.make_state(T, strides, nptr_stride), lay=lay, rows=rows, idx=None if idx is None else idx.data_ptr(),
        x=x.data_ptr(), s_x=x.stride(0), x_dtype=_hip.dtype_code(x),
        dt=dt.data_ptr(), s_dt=dt.stride(0), dt_dtype=_hip.dtype_code(dt),
        B=B.data_ptr(), s_B=B.stride(0), B_dtype=_hip.dtype_code(B),
        C=C.data_ptr(), s_C=C.stride(0), C_dtype=_hip.dtype_code(C),
        A=A.data_ptr(), A_dtype=_hip.dtype_code(A),
        D=_hip.ptr(D), D_dtype=_hip.dtype_code(D) if D is not None else 0,
        dt_bias=_hip.ptr(dt_bias), dt_bias_dtype=_hip.dtype_code(dt_bias) if dt_bias is not None else 0,
        dt_softplus=int(bool(dt_softplus)), dt_clamp=int(clamp), dt_min=lo, dt_max=hi,
        out=out.data_ptr(), s_out=out.stride(0), out_dtype=_hip.dtype_code(out),
        order=_hip.check_order(order, rows, T['S']))
    _hip.check(_hip.lib().sq_mamba2_step(ctypes.byref(a), _hip.current_stream(out.device)))
    return out


class PackedMamba2State(LockstepState):
    """One Mamba2 layer's packed state and decode buffer for B sequences in lockstep (mamba2.py:259-335).

    S [B, H, d_v, d_k] (or [B*H, d_v, d_k]); fmt, m, hv (= H), hk (= G groups), buffer_bits as ``PackedGDNState``.
    ``step(x, dt, B, C, A, D, dt_bias, dt_softplus, dt_limit)`` returns the output buffer [B, H, d_v] (the same
    tensor every step).  One launch, no allocation."""

    def __init__(self, S, fmt, m=8, hv=None, hk=None, buffer_bits=8, out_dtype=torch.bfloat16, sbv=None, fbv=None,
                 warps=None):
        flat = S.float().flatten(0, -3) if S.dim() > 3 else S.float()           # [B * H, d_v, d_k]
        _hip.require_gpu(flat, 'PackedMamba2State')
        heads = hv if hv else flat.shape[0]
        groups = hk if hk else heads
        if flat.shape[0] % heads:
            raise AssertionError(f'{flat.shape[0]} state rows are not a multiple of {heads} heads')
        _common(self, fmt, heads, groups, flat.shape[2], flat.shape[1], m, buffer_bits)
        _require_kernel('mamba2', self)
        self.BH, self.B = flat.shape[0], flat.shape[0] // heads
        self._allocate(*pack_vk(flat, self.fmt), decay_shape=(), out_shape=(self.B, heads, self.DV),
                       out_dtype=out_dtype)

    @torch.no_grad()
    def load(self, S):
        """Replace the state (any shape that flattens to [B * H, d_v, d_k]) and empty the buffer."""
        self._reset(*pack_vk(S.float().reshape(self.BH, self.DV, self.DK), self.fmt))

    def dequantize(self):
        """The stored state (without the buffered tokens), fp32 [B * H, d_v, d_k]."""
        return unpack_vk(self.codes, self.scales, self.fmt, self.DK)

    def step(self, x, dt, B, C, A, D=None, dt_bias=None, dt_softplus=False, dt_limit=None):
        Bn, HV, HK = self.B, self.HV, self.HK
        x = x.reshape(Bn, HV, self.DV)
        dt = dt.reshape(Bn, HV)
        B = B.reshape(Bn, HK, self.DK)
        C = C.reshape(Bn, HK, self.DK)
        return _launch(self, self._lay, Bn, x, dt, B, C, self.O, A, D, dt_bias, dt_softplus, dt_limit, None, self.T,
                       self._strides, HV)


class Mamba2SlotLayout(SlotLayout):
    """The per-slot blob of one Mamba2 layer (``SlotLayout``'s fields: KB / KBS per group, UB / UBS, GB, GCUR per
    head; ``views``, ``alloc``, ``read``, ``write`` as there) and the Mamba2 decode step on a batch of slots
    (mamba2.py:341-396).

    fmt, hv (heads), hk (groups), dk (d_state), dv (head_dim), m, buffer_bits as ``PackedMamba2State``."""

    _family = 'mamba2'

    def __init__(self, fmt, hv, hk, dk, dv, m=8, buffer_bits=8, sbv=None, fbv=None, warps=None):
        _common(self, fmt, hv, hk, dk, dv, m, buffer_bits)
        self.fused = True
        self.state_dtype = torch.bfloat16
        self.fields, self.nbytes = field_table(state_fields(
            self.fmt, self.bits, self.axk, self.group, hv, hk, dk, dv, m, self.qbuf, (hv, m), (hv,), ragged=False))
        self._lay = None

    def __repr__(self):
        f = 'bf16' if self.fmt is None else f'int{self.bits}-{self.fmt.axis}-g{self.group}'
        return (f'Mamba2SlotLayout({f}, heads={self.HV}, groups={self.HK}, d_state={self.DK}, head_dim={self.DV}, '
                f'm={self.m}, buffer_bits={self.buffer_bits}, {self.nbytes} B/slot)')

    def step(self, views, idx, x, dt, B, C, out, A, D=None, dt_bias=None, dt_softplus=True,
             dt_limit=(0., float('inf')), order=None):
        """One decode token for every batch row b on slot ``idx[b]`` (int32 [rows]; <= 0 = padding: output zeroed,
        nothing read or written) (mamba2.py:377-396).

        x [rows, H, d_v], dt [rows, H] (raw: + dt_bias, softplus, clamp in the kernel), B / C [rows, G, d_k]: any row
        stride, contiguous rows; out [rows, H, d_v] (row stride free); A [H] (= -exp(A_log)), D, dt_bias [H] or None.
        ``order``: optional dispatch order of the rows (``fold_order``; not in the reference)."""
        rows = idx.shape[0]
        if rows == 0:
            return out
        assert idx.dtype == torch.int32 and idx.is_contiguous()
        T, strides, sN = slot_state(views)
        return _launch(self, self._layout_struct(), rows, x, dt, B, C, out, A, D, dt_bias, dt_softplus, dt_limit, idx,
                       T, strides, sN, order)


__all__ = ['PackedMamba2State', 'Mamba2SlotLayout', 'mamba2_recurrence']
