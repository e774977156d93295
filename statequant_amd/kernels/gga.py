"""The packed GGA / STEP slot with the PW-S8 window on HIP kernels: per-head frozen widths (2, 4, 6, 8 bits, fp16
pivots), STEP's dual-axis fit re-done at every decoded token, the last m writes kept as FP8 vector pairs.

Mirrors ``GGAPacked`` of the reference (``/root/reference/src/statequant/integrations/vllm_gga.py:185-318``: same
constructor, ``views`` / ``alloc`` / ``step`` / ``stored`` / ``window`` / ``read`` / ``write``, same per-slot byte
layout, documented in ``/root/reference/src/statequant/kernels/_gga_triton.py:3-13``), with the reference's four
Triton launches replaced by ``sq_gga_step`` / ``sq_gga_store`` / ``sq_gga_load`` of ``libsqhip.so``.

``method`` is anything with the reference's plan attributes: ``plan`` {layer: (widths int [HV], impact factors
fp32 [HV, d_k])}, ``group`` (32) and ``name``; ``GGAPlan`` below holds one, and reads a file written by the
reference's ``StepQuant.save`` (``step_quant.py:248-252``).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _hip
from .slots import _ALIGN

WIDTHS = (2, 4, 6, 8, 16)


class GGAPlan:
    """A calibrated per-head plan: {layer: (widths [HV], impact factors [HV, d_k])}."""

    def __init__(self, plan, group=32, name='GGA'):
        self.plan = {k: (torch.as_tensor(b), torch.as_tensor(w).float()) for k, (b, w) in plan.items()}
        self.group, self.name = group, name

    @classmethod
    def load(cls, path):
        """From a file of the reference's ``StepQuant.save``: plain tensors and numbers only, so it is read with
        ``weights_only=True``."""
        d = torch.load(path, map_location='cpu', weights_only=True)
        return cls(d['plan'], group=d['group'], name=f"{d['class']}@{d['bits']}")


def head_bytes(b, dk, dv, group=32):
    """Stored bytes of one head at width b: codes + row factors (2 bit: group rows) + column factors; fp16 pivots
    (vllm_gga.py:174-180)."""
    if b == 16:
        return 2 * dk * dv
    if b == 2:
        return dk * dv // 4 + 2 * dk * (dv // group) + 2 * dv
    return dk * dv * b // 8 + 2 * dk + 2 * dv


def _al(n):
    return -(-n // _ALIGN) * _ALIGN


class GGAPacked:
    """The packed slot for every GDN layer of a plan: widths differ between layers, so each layer has its own offset
    table; one slot size serves all layers (``nbytes`` = the largest layer's + the windows)."""
    per_layer = True

    def __init__(self, method, hv, hk, dk, dv, pw=False, m=8):
        assert dk & (dk - 1) == 0 and dv & (dv - 1) == 0 and dv % 32 == 0, (dk, dv)
        assert method.group == 32, 'two-bit heads keep one row factor per 32 value columns'
        self.method, self.HV, self.HK, self.DK, self.DV = method, hv, hk, dk, dv
        self.pw, self.m, self.gqa = pw, m, hv // hk
        assert hv % hk == 0
        self.tables, self.bytes_per_layer = {}, {}
        for layer, (b, w) in method.plan.items():
            b = [int(x) for x in b]
            assert len(b) == hv and set(b) <= set(WIDTHS), b
            assert tuple(w.shape) == (hv, dk), (tuple(w.shape), hv, dk)
            offs, off = [], 16                                  # counters first
            for x in b:
                offs.append(off)
                off += _al(head_bytes(x, dk, dv, method.group))
            self.tables[layer] = (offs, b, w)
            self.bytes_per_layer[layer] = off
        self.QOFF = _al(max(self.bytes_per_layer.values()))
        self.QSZ = m * (dk + dv + 8)
        self.nbytes = self.QOFF + (hv * self.QSZ if pw else 0)
        self._dev = {}

    def __repr__(self):
        return (f'GGAPacked({self.method.name}{"+PW-S%d" % self.m if self.pw else ""}, hv={self.HV}, hk={self.HK}, '
                f'dk={self.DK}, dv={self.DV}, {self.nbytes} B/slot = max over layers; mean '
                f'{self.bits_per_value():.3f} b/value)')

    def bits_per_value(self):
        """Mean stored bits per state value over the layers (without the 16-byte counters), window included."""
        n = self.HV * self.DK * self.DV
        st = sum(sum(head_bytes(x, self.DK, self.DV, self.method.group) for x in t[1]) for t in self.tables.values())
        q = self.HV * self.QSZ * len(self.tables) if self.pw else 0
        return 8 * (st + q) / (n * len(self.tables))

    def supported(self):
        """Whether ``libsqhip.so`` has kernels for these head dims and window length."""
        return bool(_hip.lib().sq_gga_supported(self.DK, self.DV, self.m if self.pw else 1))

    def prepare(self, device):
        """Put every layer's tables on ``device`` now (before a graph capture: no copies inside it)."""
        for layer in self.tables:
            self._plan(layer, torch.device(device))
        return self

    def _plan(self, layer, dev):
        key = (layer, dev)
        if key not in self._dev:
            offs, b, w = self.tables[layer]
            self._dev[key] = (torch.tensor(offs, dtype=torch.int32, device=dev),
                              torch.tensor(b, dtype=torch.int32, device=dev),
                              w.to(dev, torch.float32).contiguous())
        return self._dev[key]

    def views(self, blob):
        assert blob.dtype == torch.uint8 and blob.dim() == 2 and blob.shape[1] >= self.nbytes
        assert blob.stride(1) == 1 and blob.stride(0) % _ALIGN == 0 and blob.data_ptr() % _ALIGN == 0
        return {'blob': blob}

    def alloc(self, num_slots, device='cuda'):
        """A zeroed blob; its slot stride is ``nbytes`` rounded up to 16 (``nbytes`` itself is not a multiple of 16 when
        the window length times the head count is odd)."""
        return torch.zeros(num_slots, _al(self.nbytes), dtype=torch.uint8, device=device)

    def _slots(self, blob, layer):
        _hip.require_gpu(blob, 'GGAPacked')
        offs, bits, w = self._plan(layer, blob.device)
        return _hip.SqGgaSlots(blob=blob.data_ptr(), slot_stride=blob.stride(0), offs=offs.data_ptr(),
                               bits=bits.data_ptr(), w=w.data_ptr(), hv=self.HV, hk=self.HK, dk=self.DK, dv=self.DV,
                               m=self.m, pw=int(self.pw), qoff=self.QOFF, qsz=self.QSZ)

    def step(self, views, idx, q, k, v, out, scale, *, g=None, beta=None, gate=None, layer=None, fused=None):
        """One decode token per row of ``idx`` (int32, <= 0: padding).  q, k [B, HK, d_k]; v [B, HV, d_v];
        ``gate=(a, b, A_log, dt_bias)`` as the reference takes it, or ``g`` (log decay) and ``beta`` [B, HV];
        ``out`` [B, HV, d_v] contiguous."""
        B = idx.shape[0]
        if B == 0:
            return out
        assert (gate is not None) != (g is not None and beta is not None), 'give gate=(a, b, A_log, dt_bias) or g and beta'
        assert q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1 and v.stride(1) == self.DV
        assert q.stride(1) == self.DK and k.stride(1) == self.DK
        assert out.is_contiguous() and idx.dtype == torch.int32 and idx.is_contiguous()
        assert out.shape[0] >= B and tuple(out.shape[1:]) == (self.HV, self.DV)
        blob = views['blob']
        a = _hip.SqGgaArgs(sl=self._slots(blob, layer), rows=B, idx=idx.data_ptr(),
                           q=q.data_ptr(), s_q=q.stride(0), q_dtype=_hip.dtype_code(q),
                           k=k.data_ptr(), s_k=k.stride(0), k_dtype=_hip.dtype_code(k),
                           v=v.data_ptr(), s_v=v.stride(0), v_dtype=_hip.dtype_code(v),
                           out=out.data_ptr(), out_dtype=_hip.dtype_code(out), scale=float(scale))
        if gate is not None:
            a_, b_, A_log, dt_bias = gate
            assert a_.stride(-1) == 1 and b_.stride(-1) == 1 and A_log.is_contiguous() and dt_bias.is_contiguous()
            a.gate = 1
            a.a, a.s_a, a.a_dtype = a_.data_ptr(), a_.stride(0), _hip.dtype_code(a_)
            a.b, a.s_b, a.b_dtype = b_.data_ptr(), b_.stride(0), _hip.dtype_code(b_)
            a.A_log, a.A_log_dtype = A_log.data_ptr(), _hip.dtype_code(A_log)
            a.dt_bias, a.dt_bias_dtype = dt_bias.data_ptr(), _hip.dtype_code(dt_bias)
        else:
            assert g.stride(-1) == 1 and beta.stride(-1) == 1
            a.gate = 0
            a.g, a.s_g, a.g_dtype = g.data_ptr(), g.stride(0), _hip.dtype_code(g)
            a.beta, a.s_beta, a.beta_dtype = beta.data_ptr(), beta.stride(0), _hip.dtype_code(beta)
        _hip.check(_hip.lib().sq_gga_step(C.byref(a), _hip.current_stream(blob.device)))
        return out

    @torch.no_grad()
    def stored(self, views, idx, layer):
        """The stored states of slots idx, canonical fp32 [P, HV, d_k, d_v] (without the window)."""
        idx32 = idx.to(torch.int32).contiguous()
        P = idx32.shape[0]
        Y = torch.empty(P, self.HV, self.DK, self.DV, device=idx.device)
        if P:
            blob = views['blob']
            sl = self._slots(blob, layer)
            _hip.check(_hip.lib().sq_gga_load(C.byref(sl), idx32.data_ptr(), P, Y.data_ptr(),
                                              _hip.current_stream(blob.device)))
        return Y

    @torch.no_grad()
    def window(self, views, idx):
        """The queued pairs of slots idx as reconstructed fp32 (P [n, m, HV, d_k], V [n, m, HV, d_v]) in ring order
        from the oldest, and the counts n [n]; dead entries zeroed."""
        li = idx.long()
        blob = views['blob'][li]
        m, HV, DK, DV = self.m, self.HV, self.DK, self.DV
        ct = blob[:, :16].view(torch.int32)
        n, hd = ct[:, 0], ct[:, 1]
        Qb = blob[:, self.QOFF:self.QOFF + HV * self.QSZ].reshape(-1, HV, self.QSZ)
        Pc = Qb[..., :m * DK].contiguous().view(torch.float8_e4m3fn).float().view(-1, HV, m, DK)
        Vc = Qb[..., m * DK:m * (DK + DV)].contiguous().view(torch.float8_e4m3fn).float().view(-1, HV, m, DV)
        sc = Qb[..., m * (DK + DV):].contiguous().view(torch.float32).view(-1, HV, 2, m)
        Pf = Pc * sc[:, :, 0, :, None]
        Vf = Vc * sc[:, :, 1, :, None]
        order = (hd[:, None] + torch.arange(m, device=li.device)[None, :]) % m          # oldest first
        Pf = torch.gather(Pf, 2, order[:, None, :, None].expand(-1, HV, -1, DK)).transpose(1, 2)
        Vf = torch.gather(Vf, 2, order[:, None, :, None].expand(-1, HV, -1, DV)).transpose(1, 2)
        live = (torch.arange(m, device=li.device)[None, :] < n[:, None])[:, :, None, None]
        return torch.where(live, Pf, 0.), torch.where(live, Vf, 0.), n

    @torch.no_grad()
    def read(self, views, idx, layer=None):
        """Logical state (stored + window), value-major fp32 [P, HV, d_v, d_k]."""
        S = self.stored(views, idx, layer)
        if self.pw and idx.shape[0]:
            P, V, _ = self.window(views, idx)
            _, bits, _ = self._plan(layer, idx.device)
            nonp = (bits != 16)[None, :, None, None].float()
            S = S + torch.einsum('bmhk,bmhv->bhkv', P, V) * nonp
        return S.transpose(-1, -2)

    @torch.no_grad()
    def write(self, views, idx, S, layer=None):
        """Fit + pack value-major states S [P, HV, d_v, d_k] into slots idx; empty the window."""
        idx32 = idx.to(torch.int32).contiguous()
        P = idx32.shape[0]
        if P == 0:
            return
        X = S.float().transpose(-1, -2).contiguous()
        blob = views['blob']
        sl = self._slots(blob, layer)
        _hip.check(_hip.lib().sq_gga_store(C.byref(sl), idx32.data_ptr(), P, X.data_ptr(),
                                           _hip.current_stream(blob.device)))
