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
from .fold import _bits, _require_kernel, pack_vk, packed_format, unpack_vk
from .slots import SlotLayout, _order_ptr, field_table, slot_state, state_fields


def _gate(dt, A, dt_bias=None, dt_softplus=False, dt_limit=None):
    """dt (raw [B, H]) -> (dt, log decay g = A dt), fp32, as the kernel (mamba2.py:45-54)."""
    dt = dt.float()
    if dt_bias is not None:
        dt = dt + dt_bias.float()
    if dt_softplus:
        dt = torch.where(dt <= 20., torch.log(1. + torch.exp(dt)), dt)
    if dt_limit is not None and tuple(dt_limit) != (0., float('inf')):
        dt = dt.clamp(dt_limit[0], dt_limit[1])
    return dt, A.float() * dt


def mamba2_recurrence(S, x, dt, B, C, A, D=None, dt_bias=None, dt_softplus=False, dt_limit=None):
    """One plain fp32 Mamba2 step on S [B, H, d_v, d_k] (updated in place); x [B, H, d_v], dt [B, H], B / C
    [B, G, d_k], A / D / dt_bias [H].  Returns y [B, H, d_v] fp32 (mamba2.py:57-70)."""
    H, G = dt.shape[1], B.shape[1]
    dt, g = _gate(dt, A, dt_bias, dt_softplus, dt_limit)
    Bh = B.float().repeat_interleave(H // G, 1)
    Ch = C.float().repeat_interleave(H // G, 1)
    u = dt.unsqueeze(-1) * x.float()
    S.mul_(torch.exp(g)[..., None, None]).add_(u.unsqueeze(-1) * Bh.unsqueeze(-2))
    y = torch.einsum('bhvk,bhk->bhv', S, Ch)
    if D is not None:
        y = y + D.float()[:, None] * x.float()
    return y


def _check_dims(fmt, dk, dv):
    assert dk >= 16 and dk % 2 == 0, dk
    if fmt is not None:
        g = fmt.group
        assert g & (g - 1) == 0, f'group {g} must be a power of two'
        assert (dk if fmt.axis == 'k' else dv) % g == 0, f'group {g} must divide d_{fmt.axis} ({dk}, {dv})'


def _common(st, fmt, hv, hk, dk, dv, m, buffer_bits):
    st.fmt = packed_format(fmt)
    st.bits = _bits(st.fmt)
    st.HV, st.HK, st.DK, st.DV, st.m = hv, hk, dk, dv, m
    assert hv % hk == 0, (hv, hk)
    st.gqa = hv // hk
    assert m >= 1 and m & (m - 1) == 0 and m <= 32, 'm must be a power of two <= 32'
    _check_dims(st.fmt, dk, dv)
    assert buffer_bits in (8, 16)
    st.buffer_bits, st.qbuf = buffer_bits, buffer_bits == 8
    st.axk = st.fmt is not None and st.fmt.axis == 'k'
    st.group = st.fmt.group if st.fmt is not None else 16


def _launch(st, lay, rows, x, dt, B, C, out, A, D, dt_bias, dt_softplus, dt_limit, idx, T, strides, nptr_stride,
            order=None):
    """One ``sq_mamba2_step`` call (replaces mamba2.py:223-241)."""
    assert x.stride(-1) == 1 and B.stride(-1) == 1 and C.stride(-1) == 1 and dt.stride(-1) == 1
    assert x.stride(-2) == st.DV and out.stride(-1) == 1 and out.stride(-2) == st.DV
    assert B.stride(-2) == st.DK and C.stride(-2) == st.DK
    assert A.is_contiguous() and (D is None or D.is_contiguous()) and (dt_bias is None or dt_bias.is_contiguous())
    _hip.require_gpu(out, 'Mamba2 step')
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
        out=out.data_ptr(), s_out=out.stride(0), out_dtype=_hip.dtype_code(out), order=_order_ptr(order, rows))
    _hip.check(_hip.lib().sq_mamba2_step(ctypes.byref(a), _hip.current_stream(out.device)))
    return out


class PackedMamba2State:
    """One Mamba2 layer's packed state and decode buffer for B sequences in lockstep (mamba2.py:259-335).

    S [B, H, d_v, d_k] (or [B*H, d_v, d_k]); fmt, m, hv (= H), hk (= G groups), buffer_bits as ``PackedGDNState``.
    ``step(x, dt, B, C, A, D, dt_bias, dt_softplus, dt_limit)`` returns the output buffer [B, H, d_v] (the same
    tensor every step).  One launch, no allocation."""

    def __init__(self, S, fmt, m=8, hv=None, hk=None, buffer_bits=8, out_dtype=torch.bfloat16, sbv=None, fbv=None,
                 warps=None):
        S = S.float().reshape(-1, S.shape[-2], S.shape[-1])
        _hip.require_gpu(S, 'PackedMamba2State')
        BH, DV, DK = S.shape
        hv = hv or BH
        hk = hk or hv
        assert BH % hv == 0
        _common(self, fmt, hv, hk, DK, DV, m, buffer_bits)
        _require_kernel('mamba2', self)
        self.BH, self.B = BH, BH // hv
        dev = S.device
        c, s = pack_vk(S, self.fmt)
        bdt = torch.int8 if self.qbuf else torch.bfloat16
        self.T = dict(S=c.clone(), SC=s.clone(),
                      KB=torch.zeros(self.B * hk, m, DK, device=dev, dtype=bdt),
                      UB=torch.zeros(BH, m, DV, device=dev, dtype=bdt),
                      KBS=torch.zeros(self.B * hk, m, device=dev, dtype=torch.float16),
                      UBS=torch.zeros(BH, m, device=dev, dtype=torch.float16),
                      GB=torch.zeros(BH, m, device=dev), GCUR=torch.zeros(BH, device=dev),
                      NPTR=torch.zeros(self.B, hv, device=dev, dtype=torch.int32))
        self.O = torch.zeros(self.B, hv, DV, device=dev, dtype=out_dtype)
        T = self.T
        self._strides = (hv * T['S'][0].numel(), hv * T['SC'][0].numel(), hk * m * DK, hk * m, hv * m * DV, hv * m,
                         hv * m, hv)
        self._lay = _hip.make_layout(self)

    def __getattr__(self, name):
        T = self.__dict__.get('T')
        if T is not None and name in T:
            return T[name]
        raise AttributeError(name)

    @property
    def codes(self):
        return self.T['S']

    @property
    def scales(self):
        return self.T['SC']

    @property
    def n(self):
        return int(self.T['NPTR'].reshape(-1)[0])

    @torch.no_grad()
    def load(self, S):
        c, s = pack_vk(S.float().reshape(self.BH, self.DV, self.DK), self.fmt)
        self.T['S'].copy_(c)
        self.T['SC'].copy_(s)
        for k in ('KB', 'UB', 'KBS', 'UBS', 'GB', 'GCUR', 'NPTR'):
            self.T[k].zero_()

    def dequantize(self):
        return unpack_vk(self.T['S'], self.T['SC'], self.fmt, self.DK)

    def stored_bytes(self):
        nb = lambda t: t.numel() * t.element_size()          # noqa: E731
        T = self.T
        per = dict(state=nb(T['S']) + (nb(T['SC']) if self.fmt is not None else 0),          # bf16 state: no scales
                   buffer=nb(T['KB']) + nb(T['UB']) + ((nb(T['KBS']) + nb(T['UBS'])) if self.qbuf else 0),
                   decay=nb(T['GB']) + nb(T['GCUR']) + nb(T['NPTR']))
        per['total'] = sum(per.values())
        return per

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
        ``order``: optional dispatch order of the rows, as in ``SlotLayout.step``."""
        rows = idx.shape[0]
        if rows == 0:
            return out
        assert idx.dtype == torch.int32 and idx.is_contiguous()
        T, strides, sN = slot_state(views)
        return _launch(self, self._layout_struct(), rows, x, dt, B, C, out, A, D, dt_bias, dt_softplus, dt_limit, idx,
                       T, strides, sN, order)


__all__ = ['PackedMamba2State', 'Mamba2SlotLayout', 'mamba2_recurrence']
