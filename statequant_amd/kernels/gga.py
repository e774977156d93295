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
    """Bytes one head occupies at width b (vllm_gga.py:174-180): an fp16 pivot stores its dk x dv values; a coded head
    stores b-bit codes plus fp16 factors -- one row factor per row (2-bit heads: one per row and group of `group`
    value columns) and one column factor per column."""
    values = dk * dv
    if b == 16:
        return values * 2
    row_factors = dk * (dv // group) if b == 2 else dk
    return (values * b) // 8 + 2 * (row_factors + dv)


def _al(nbytes):
    """nbytes rounded up to the slot alignment."""
    return (nbytes + _ALIGN - 1) // _ALIGN * _ALIGN


class GGAPacked:
    """The packed slot for every GDN layer of a plan: widths differ between layers, so each layer has its own offset
    table; one slot size serves all layers (``nbytes`` = the largest layer's + the windows)."""
    per_layer = True

    def __init__(self, method, hv, hk, dk, dv, pw=False, m=8):
        for d in (dk, dv):
            if d & (d - 1):
                raise AssertionError((dk, dv))
        assert dv % 32 == 0, (dk, dv)
        assert hv % hk == 0, (hv, hk)
        self.method = method
        self.HV, self.HK, self.gqa = hv, hk, hv // hk
        self.DK, self.DV = dk, dv
        self.pw, self.m = pw, m
        # per layer: where each head starts inside the slot (after the 16 counter bytes), its width, the impact factors
        self.tables, self.bytes_per_layer = {}, {}
        for layer, (widths, impact) in method.plan.items():
            widths = [int(x) for x in widths]
            assert len(widths) == hv and all(x in WIDTHS for x in widths), (layer, widths)
            sizes = [_al(head_bytes(x, dk, dv, method.group)) for x in widths]
            starts = [16 + sum(sizes[:i]) for i in range(hv)]
            self.tables[layer] = (starts, widths, impact)
            self.bytes_per_layer[layer] = 16 + sum(sizes)
        # the windows follow the largest layer's heads: per head m left and m right FP8 vectors and their 2 m scales
        self.QOFF = _al(max(self.bytes_per_layer.values()))
        self.QSZ = m * (dk + dv) + 2 * m * 4
        self.nbytes = self.QOFF + hv * self.QSZ * int(bool(pw))
        self._dev = {}

    def __repr__(self):
        window = f'+PW-S{self.m}' if self.pw else ''
        return (f'GGAPacked({self.method.name}{window}, hv={self.HV}, hk={self.HK}, dk={self.DK}, dv={self.DV}, '
                f'{self.nbytes} B/slot = max over layers; mean {self.bits_per_value():.3f} b/value)')

    def bits_per_value(self):
        """Mean stored bits per state value over the layers (without the 16-byte counters), window included."""
        layers = len(self.tables)
        head_total = 0
        for _, widths, _ in self.tables.values():
            head_total += sum(head_bytes(x, self.DK, self.DV, self.method.group) for x in widths)
        window_total = layers * self.HV * self.QSZ if self.pw else 0
        return 8.0 * (head_total + window_total) / (layers * self.HV * self.DK * self.DV)

    def supported(self):
        """Whether ``libsqhip.so`` has kernels for these head dims and window length."""
        return bool(_hip.lib().sq_gga_supported(self.DK, self.DV, self.m if self.pw else 1))

    def prepare(self, device):
        """Put every layer's tables on ``device`` now (before a graph capture: no copies inside it)."""
        for layer in self.tables:
            self._plan(layer, torch.device(device))
        return self

    def _plan(self, layer, dev):
        """(head offsets int32 [HV], widths int32 [HV], impact factors fp32 [HV, d_k]) of a layer on device dev."""
        cached = self._dev.get((layer, dev))
        if cached is None:
            starts, widths, impact = self.tables[layer]
            as_i32 = lambda xs: torch.tensor(xs, dtype=torch.int32, device=dev)      # noqa: E731
            cached = (as_i32(starts), as_i32(widths), impact.to(device=dev, dtype=torch.float32).contiguous())
            self._dev[(layer, dev)] = cached
        return cached

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
        ga, gb, A_log, dt_bias = gate if gate is not None else (None,) * 4
        _hip.same_device('GGAPacked.step', blob, idx=idx, q=q, k=k, v=v, out=out, g=g, beta=beta, a=ga, b=gb,
                         A_log=A_log, dt_bias=dt_bias)
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
        blob = views['blob']
        idx32 = idx.to(device=blob.device, dtype=torch.int32).contiguous()
        P = idx32.shape[0]
        Y = torch.empty(P, self.HV, self.DK, self.DV, device=blob.device)
        if P:
            sl = self._slots(blob, layer)
            _hip.check(_hip.lib().sq_gga_load(C.byref(sl), idx32.data_ptr(), P, Y.data_ptr(),
                                              _hip.current_stream(blob.device)))
        return Y

    @torch.no_grad()
    def window(self, views, idx):
        """The queued pairs of slots idx as reconstructed fp32 (P [n, m, HV, d_k], V [n, m, HV, d_v]) in ring order
        from the oldest, and the counts n [n].  Dead entries are SELECTED away, never multiplied by zero: the store
        kernel resets the two counters only, so on a page that was not zero-filled a dead entry may decode to NaN
        (FP8 0x7F / 0xFF) or carry a non-finite scale."""
        m, HV, DK, DV = self.m, self.HV, self.DK, self.DV
        rows = views['blob'].index_select(0, idx.to(views['blob'].device).long())
        counters = rows[:, :8].contiguous().view(torch.int32)                  # n, ring position of the oldest
        count, oldest = counters[:, 0], counters[:, 1]
        win = rows[:, self.QOFF:self.QOFF + HV * self.QSZ].unflatten(1, (HV, self.QSZ))

        def fp8_block(lo, width):                                              # [n, HV, m, width] decoded codes
            raw = win[:, :, lo:lo + m * width].contiguous()
            return raw.view(torch.float8_e4m3fn).to(torch.float32).unflatten(2, (m, width))

        scales = win[:, :, m * (DK + DV):].contiguous().view(torch.float32).unflatten(2, (2, m))
        left = fp8_block(0, DK) * scales[:, :, 0].unsqueeze(-1)
        right = fp8_block(m * DK, DV) * scales[:, :, 1].unsqueeze(-1)
        # ring order -> age order, then entries beyond the count are dropped
        steps = torch.arange(m, device=rows.device)
        ring = torch.remainder(oldest.unsqueeze(1) + steps, m)                  # [n, m]
        alive = (steps.unsqueeze(0) < count.unsqueeze(1)).view(-1, m, 1, 1)

        def by_age(x):                                                          # [n, HV, m, d] -> [n, m, HV, d]
            picked = torch.stack([x[i, :, ring[i]] for i in range(x.shape[0])]) if x.shape[0] else x
            return torch.where(alive, picked.transpose(1, 2), torch.zeros((), device=x.device))

        return by_age(left), by_age(right), count

    @torch.no_grad()
    def read(self, views, idx, layer=None):
        """Logical state (stored + window), value-major fp32 [P, HV, d_v, d_k]."""
        state = self.stored(views, idx, layer)                                 # [P, HV, d_k, d_v]
        if self.pw and idx.numel():
            left, right, _ = self.window(views, idx)
            widths = self._plan(layer, state.device)[1]
            coded = (widths != 16).view(1, 1, -1, 1)                           # pivots keep no window: whatever
            left = torch.where(coded, left, torch.zeros((), device=left.device))      # their bytes hold is dropped
            right = torch.where(coded, right, torch.zeros((), device=right.device))
            state = state + torch.einsum('pmhk,pmhv->phkv', left, right)
        return state.mT

    @torch.no_grad()
    def write(self, views, idx, S, layer=None):
        """Fit + pack value-major states S [P, HV, d_v, d_k] into slots idx; empty the window."""
        blob = views['blob']
        idx32 = idx.to(device=blob.device, dtype=torch.int32).contiguous()
        P = idx32.shape[0]
        if P == 0:
            return
        X = S.to(device=blob.device, dtype=torch.float32).transpose(-1, -2).contiguous()
        sl = self._slots(blob, layer)
        _hip.check(_hip.lib().sq_gga_store(C.byref(sl), idx32.data_ptr(), P, X.data_ptr(),
                                           _hip.current_stream(blob.device)))
