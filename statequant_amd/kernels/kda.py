"""Packed recurrent state for KDA (Kimi Delta Attention) layers on HIP kernels: lockstep state and slot layout.

Mirrors the reference's ``statequant/kernels/kda.py`` (``/root/reference/src/statequant/kernels/kda.py``).  KDA is the
gated delta rule with a decay per KEY channel: per head, one token, a_t = exp(g_t) in R^{d_k},

    S_t = (I - beta_t k_t k_t^T) diag(a_t) S_{t-1} + beta_t k_t v_t^T,        o_t = S_t^T q_t

Packed decode (kda.py:10-19): the stored state S_0 is rounded and rewritten only every ``m`` tokens; the buffer keeps
(cumulative log decay G_i in R^{d_k}, normalised key k_i, delta value u_i).  States are value-major [B, H, d_v, d_k];
key heads = value heads.  Unlike the reference's Triton kernel, head dims need not be powers of two (multiples of 16
for d_k, of 32 for d_v); the slot layout and rounding are ``fold.pack_vk``'s for any such dims.
"""
from __future__ import annotations

import ctypes

import torch

from . import _hip
from .fold import _bits, _require_kernel, pack_vk, packed_format, unpack_vk
from .slots import SlotLayout, _order_ptr, field_table, slot_state, state_fields


def kda_recurrence(S, q, k, v, g, beta, scale=None):
    """One plain fp32 KDA step on S [BH, d_v, d_k] (value-major, updated in place); q, k raw [BH, d_k] (normalised
    here), v [BH, d_v], g [BH, d_k] log decay, beta [BH].  Returns o [BH, d_v] fp32 (kda.py:44-52)."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    nrm = lambda x: x.float() / torch.sqrt((x.float() ** 2).sum(-1, keepdim=True) + 1e-6)     # noqa: E731
    qn, kn = nrm(q) * scale, nrm(k)
    S.mul_(torch.exp(g.float()).unsqueeze(1))
    u = beta.float().unsqueeze(1) * (v.float() - torch.einsum('bvk,bk->bv', S, kn))
    S.add_(u.unsqueeze(2) * kn.unsqueeze(1))
    return torch.einsum('bvk,bk->bv', S, qn)


def _check(fmt, dk, dv, hv, hk, m, buffer_bits):
    """kda.py:55-64, with the power-of-two restriction on the head dims lifted."""
    assert dk >= 16 and dk % 2 == 0 and dv >= 16, (dk, dv)
    assert hk == hv, 'KDA: key heads must equal value heads'
    assert m >= 1 and m & (m - 1) == 0 and m <= 32, 'm must be a power of two <= 32'
    assert buffer_bits in (8, 16), buffer_bits
    if fmt is not None:
        g = fmt.group
        assert g >= 2 and g & (g - 1) == 0, f'group {g} must be a power of two'
        assert (dk if fmt.axis == 'k' else dv) % g == 0, f'group {g} must divide d_{fmt.axis} ({dk}, {dv})'
        assert fmt.axis == 'v' or dk // g <= 64, 'at most 64 key groups'


def _common(st, fmt, hv, hk, dk, dv, m, buffer_bits):
    st.fmt = packed_format(fmt)
    st.bits = _bits(st.fmt)
    st.HV, st.HK, st.DK, st.DV, st.m = hv, hk, dk, dv, m
    _check(st.fmt, dk, dv, hv, hk, m, buffer_bits)
    st.buffer_bits, st.qbuf = buffer_bits, buffer_bits == 8
    st.axk = st.fmt is not None and st.fmt.axis == 'k'
    st.group = st.fmt.group if st.fmt is not None else 16


def _launch(st, lay, rows, q, k, v, g, beta, out, scale, idx, T, strides, nptr_stride, order=None):
    """One ``sq_kda_step`` call (replaces kda.py:192-205)."""
    for t in (q, k, v, g):
        assert t.stride(-1) == 1, 'unit inner stride'
    assert q.stride(-2) == st.DK and k.stride(-2) == st.DK and v.stride(-2) == st.DV and g.stride(-2) == st.DK
    assert beta.stride(-1) == 1 and out.stride(-1) == 1 and out.stride(-2) == st.DV
    _hip.require_gpu(out, 'KDA step')
    a = _hip.SqKdaArgs(
        st=_hip.make_state(T, strides, nptr_stride), lay=lay, rows=rows, idx=None if idx is None else idx.data_ptr(),
        q=q.data_ptr(), s_q=q.stride(0), q_dtype=_hip.dtype_code(q),
        k=k.data_ptr(), s_k=k.stride(0), k_dtype=_hip.dtype_code(k),
        v=v.data_ptr(), s_v=v.stride(0), v_dtype=_hip.dtype_code(v),
        g=g.data_ptr(), s_g=g.stride(0), g_dtype=_hip.dtype_code(g),
        beta=beta.data_ptr(), s_beta=beta.stride(0), beta_dtype=_hip.dtype_code(beta),
        out=out.data_ptr(), s_out=out.stride(0), out_dtype=_hip.dtype_code(out), scale=float(scale),
        order=_order_ptr(order, rows))
    _hip.check(_hip.lib().sq_kda_step(ctypes.byref(a), _hip.current_stream(out.device)))
    return out


class PackedKDAState:
    """One KDA layer's packed state and decode buffer for B sequences in lockstep (kda.py:208-282).

    S [B, H, d_v, d_k] (or [B*H, d_v, d_k]); fmt, m, hv (= H), buffer_bits as ``PackedGDNState``.
    ``step(q, k, v, g, beta, scale)`` (q, k raw [B, H, d_k] or [BH, d_k]; v [.., d_v]; g [.., d_k] log decay;
    beta [B, H]) returns the output buffer [B, H, d_v] (the same tensor every step).  One launch, no allocation."""

    def __init__(self, S, fmt, m=8, hv=None, buffer_bits=8, out_dtype=torch.bfloat16, sbv=None, fbv=None,
                 warps=None):
        S = S.float().reshape(-1, S.shape[-2], S.shape[-1])
        _hip.require_gpu(S, 'PackedKDAState')
        BH, DV, DK = S.shape
        hv = hv or BH
        assert BH % hv == 0
        _common(self, fmt, hv, hv, DK, DV, m, buffer_bits)
        _require_kernel('kda', self)
        self.BH, self.B = BH, BH // hv
        dev = S.device
        c, s = pack_vk(S, self.fmt)
        bdt = torch.int8 if self.qbuf else torch.bfloat16
        self.T = dict(S=c.clone(), SC=s.clone(),
                      KB=torch.zeros(BH, m, DK, device=dev, dtype=bdt),
                      UB=torch.zeros(BH, m, DV, device=dev, dtype=bdt),
                      KBS=torch.zeros(BH, m, device=dev, dtype=torch.float16),
                      UBS=torch.zeros(BH, m, device=dev, dtype=torch.float16),
                      GB=torch.zeros(BH, m, DK, device=dev), GCUR=torch.zeros(BH, DK, device=dev),
                      NPTR=torch.zeros(self.B, hv, device=dev, dtype=torch.int32))
        self.O = torch.zeros(self.B, hv, DV, device=dev, dtype=out_dtype)
        T = self.T
        self._strides = (hv * T['S'][0].numel(), hv * T['SC'][0].numel(), hv * m * DK, hv * m, hv * m * DV, hv * m,
                         hv * m * DK, hv * DK)
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

    def step(self, q, k, v, g, beta, scale=None):
        Bn, HV, DK, DV = self.B, self.HV, self.DK, self.DV
        q, k = q.reshape(Bn, HV, DK), k.reshape(Bn, HV, DK)
        v, g, beta = v.reshape(Bn, HV, DV), g.reshape(Bn, HV, DK), beta.reshape(Bn, HV)
        return _launch(self, self._lay, Bn, q, k, v, g, beta, self.O, DK ** -0.5 if scale is None else scale, None,
                       self.T, self._strides, HV)


class KDASlotLayout(SlotLayout):
    """The per-slot blob of one KDA layer and the KDA decode step on a batch of slots (kda.py:288-386).

    Fields as ``SlotLayout`` except GB fp32 [H, m, d_k] (cumulative log decay per channel of each buffered token)
    and GCUR fp32 [H, d_k]; KBS / KB are per head (no grouped keys)."""

    _family = 'kda'

    def __init__(self, fmt, hv, dk, dv, m=8, buffer_bits=8, sbv=None, fbv=None, warps=None):
        _common(self, fmt, hv, hv, dk, dv, m, buffer_bits)
        self.gqa = 1
        self.fused = True
        self.state_dtype = torch.bfloat16
        self.fields, self.nbytes = field_table(state_fields(
            self.fmt, self.bits, self.axk, self.group, hv, hv, dk, dv, m, self.qbuf, (hv, m, dk), (hv, dk),
            ragged=False))
        self._lay = None

    def __repr__(self):
        f = 'bf16' if self.fmt is None else f'int{self.bits}-{self.fmt.axis}-g{self.group}'
        return (f'KDASlotLayout({f}, heads={self.HV}, d_k={self.DK}, d_v={self.DV}, m={self.m}, '
                f'buffer_bits={self.buffer_bits}, {self.nbytes} B/slot)')

    def step(self, views, idx, q, k, v, g, beta, out, scale=None, order=None):
        """One decode token for every batch row b on slot ``idx[b]`` (int32 [rows]; <= 0 = padding: output zeroed,
        nothing read or written) (kda.py:330-347).

        q, k [rows, H, d_k] raw, v [rows, H, d_v], g [rows, H, d_k] log decay, beta [rows, H] (after sigmoid): any
        row stride, contiguous rows; out [rows, H, d_v] (row stride free).  One launch, no host syncs.  ``order``:
        optional dispatch order of the rows, as in ``SlotLayout.step``."""
        rows = idx.shape[0]
        if rows == 0:
            return out
        assert idx.dtype == torch.int32 and idx.is_contiguous()
        T, strides, sN = slot_state(views)
        return _launch(self, self._layout_struct(), rows, q, k, v, g, beta, out,
                       self.DK ** -0.5 if scale is None else scale, idx, T, strides, sN, order)

    @torch.no_grad()
    def read(self, views, idx):
        """The current state of slots ``idx`` as fp32 [P, H, d_v, d_k]: diag(alpha_n) S_0 +
        sum_{i<n} diag(alpha_n / alpha_i) k_i u_i^T (value-major) (kda.py:351-372)."""
        out = self._read_hip(views, idx, kda=True)
        if out is not None:
            return out
        idx = idx.long()
        m = self.m
        S0 = self._stored(views, idx)
        Kb, Ub, n = self._buffer(views, idx)
        gcur = views['GCUR'][idx]                                                     # [P, H, DK]
        live = (torch.arange(m, device=idx.device)[None, :] < n[:, None])[:, None, :, None]   # [P, 1, m, 1]
        zero = torch.zeros((), device=idx.device)
        dec = torch.where(live, torch.exp(gcur[:, :, None, :] - torch.where(live, views['GB'][idx], zero)), zero)
        Ub = torch.where(live, Ub, zero)
        Kd = torch.where(live, Kb, zero) * dec
        return torch.exp(gcur)[:, :, None, :] * S0 + torch.einsum('phmv,phmk->phvk', Ub, Kd)


__all__ = ['PackedKDAState', 'KDASlotLayout', 'kda_recurrence']
