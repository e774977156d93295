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
from ._lockstep import LockstepState, describe_format, power_of_two
from .fold import _bits, _require_kernel, pack_vk, packed_format, unpack_vk
from .slots import SlotLayout, field_table, slot_state, state_fields


def _unit(x):
    """Rows of x scaled to unit length, the epsilon inside the square root (as the kernels normalise q and k)."""
    xf = x.float()
    return xf * torch.rsqrt(xf.square().sum(dim=-1, keepdim=True) + 1e-6)


def kda_recurrence(S, q, k, v, g, beta, scale=None):
    """The unquantized per-channel gated delta rule, one token, on S [BH, d_v, d_k] in place (kda.py:44-52): every key
    channel decays by exp(g), then the delta write beta (v - S k) k^T, then o = S q.  q, k raw [BH, d_k]; v [BH, d_v];
    g [BH, d_k] log decay; beta [BH].  Returns o [BH, d_v] fp32."""
    kn = _unit(k)
    qn = _unit(q) * (q.shape[-1] ** -0.5 if scale is None else scale)
    S *= g.float().exp()[:, None, :]
    err = v.float() - (S * kn[:, None, :]).sum(-1)
    S += (beta.float()[:, None] * err)[:, :, None] * kn[:, None, :]
    return (S * qn[:, None, :]).sum(-1)


def _common(st, fmt, hv, hk, dk, dv, m, buffer_bits):
    """Geometry and format attributes of a KDA state / layout (kda.py:55-64; head dims need not be powers of two)."""
    st.fmt = packed_format(fmt)
    st.bits = _bits(st.fmt)
    st.axk, st.group = describe_format(st.fmt, st.bits, default_group=16)
    if hk != hv:
        raise AssertionError('KDA: key heads must equal value heads')
    if not (power_of_two(m) and m <= 32):
        raise AssertionError('m must be a power of two <= 32')
    if buffer_bits not in (8, 16):
        raise AssertionError(f'buffer_bits {buffer_bits}: 8 (int8) or 16 (bf16)')
    assert dk >= 16 and dk % 2 == 0 and dv >= 16, (dk, dv)
    if st.fmt is not None:
        axis_len = dk if st.axk else dv
        assert st.group >= 2 and power_of_two(st.group), f'group {st.group} must be a power of two'
        assert axis_len % st.group == 0, f'group {st.group} must divide d_{st.fmt.axis} ({dk}, {dv})'
        assert not st.axk or dk // st.group <= 64, 'at most 64 key groups'
    st.HV, st.HK, st.DK, st.DV, st.m = hv, hk, dk, dv, m
    st.buffer_bits, st.qbuf = buffer_bits, buffer_bits == 8


def _launch(st, lay, rows, q, k, v, g, beta, out, scale, idx, T, strides, nptr_stride, order=None):
    """One ``sq_kda_step`` call (replaces kda.py:192-205)."""
    for t in (q, k, v, g):
        assert t.stride(-1) == 1, 'unit inner stride'
    assert q.stride(-2) == st.DK and k.stride(-2) == st.DK and v.stride(-2) == st.DV and g.stride(-2) == st.DK
    assert beta.stride(-1) == 1 and out.stride(-1) == 1 and out.stride(-2) == st.DV
    _hip.same_device('KDA step', T['S'], idx=idx, q=q, k=k, v=v, g=g, beta=beta, out=out)
    a = _hip.SqKdaArgs(
        st=_hip.make_state(T, strides, nptr_stride), lay=lay, rows=rows, idx=None if idx is None else idx.data_ptr(),
        q=q.data_ptr(), s_q=q.stride(0), q_dtype=_hip.dtype_code(q),
        k=k.data_ptr(), s_k=k.stride(0), k_dtype=_hip.dtype_code(k),
        v=v.data_ptr(), s_v=v.stride(0), v_dtype=_hip.dtype_code(v),
        g=g.data_ptr(), s_g=g.stride(0), g_dtype=_hip.dtype_code(g),
        beta=beta.data_ptr(), s_beta=beta.stride(0), beta_dtype=_hip.dtype_code(beta),
        out=out.data_ptr(), s_out=out.stride(0), out_dtype=_hip.dtype_code(out), scale=float(scale),
        order=_hip.check_order(order, rows, T['S']))
    _hip.check(_hip.lib().sq_kda_step(ctypes.byref(a), _hip.current_stream(out.device)))
    return out


class PackedKDAState(LockstepState):
    """One KDA layer's packed state and decode buffer for B sequences in lockstep (kda.py:208-282).

    S [B, H, d_v, d_k] (or [B*H, d_v, d_k]); fmt, m, hv (= H), buffer_bits as ``PackedGDNState``.
    ``step(q, k, v, g, beta, scale)`` (q, k raw [B, H, d_k] or [BH, d_k]; v [.., d_v]; g [.., d_k] log decay;
    beta [B, H]) returns the output buffer [B, H, d_v] (the same tensor every step).  One launch, no allocation."""

    def __init__(self, S, fmt, m=8, hv=None, buffer_bits=8, out_dtype=torch.bfloat16, sbv=None, fbv=None,
                 warps=None):
        flat = S.float().flatten(0, -3) if S.dim() > 3 else S.float()           # [B * H, d_v, d_k]
        _hip.require_gpu(flat, 'PackedKDAState')
        heads = hv if hv else flat.shape[0]
        if flat.shape[0] % heads:
            raise AssertionError(f'{flat.shape[0]} state rows are not a multiple of {heads} heads')
        _common(self, fmt, heads, heads, flat.shape[2], flat.shape[1], m, buffer_bits)
        _require_kernel('kda', self)
        self.BH, self.B = flat.shape[0], flat.shape[0] // heads
        self._allocate(*pack_vk(flat, self.fmt), decay_shape=(self.DK,), out_shape=(self.B, heads, self.DV),
                       out_dtype=out_dtype)                                     # one decay per key channel

    @torch.no_grad()
    def load(self, S):
        """Replace the state (any shape that flattens to [B * H, d_v, d_k]) and empty the buffer."""
        self._reset(*pack_vk(S.float().reshape(self.BH, self.DV, self.DK), self.fmt))

    def dequantize(self):
        """The stored state (without the buffered tokens), fp32 [B * H, d_v, d_k]."""
        return unpack_vk(self.codes, self.scales, self.fmt, self.DK)

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
        row stride, contiguous rows; out [rows, H, d_v] (row stride free).  ``order``: optional dispatch order of the
        rows (``fold_order``; not in the reference).  One launch, no host syncs."""
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
