"""Oracle (test infrastructure): the packed decode arithmetic of the three layer families in torch on the CPU, and the
textbook fp32 recurrences they must agree with when nothing is rounded.

Restates the reference's torch classes
    GDN     /root/reference/src/statequant/kernels/fold.py:197-274    (ReferenceGDNState)
    KDA     /root/reference/src/statequant/kernels/kda.py:95-186      (ReferenceKDAState), :44-52 (kda_recurrence)
    Mamba2  /root/reference/src/statequant/kernels/mamba2.py:116-217  (ReferenceMamba2State), :45-70
as one buffered-state machine with three ``step`` rules.  All states are VALUE-MAJOR here, [BH, d_v, d_k] (the stored
orientation; the reference's GDN class alone takes and keeps the transpose).

Common algebra: stored state S0 (rounded by the format), buffer of n < m tokens (K_i [d_k] per KEY head, U_i [d_v],
cumulative log decay G_i), running log decay gcur.  With dec_i = exp(gcur - G_i):

    state()  = exp(gcur) S0 + sum_{i<n} dec_i U_i (x) K_i                  (decays per head, or per key channel: KDA)
    fold()   : S = state() accumulated slot by slot in order, re-rounded by the format; gcur = 0, n = 0

``fmt`` = (bits, axis, group) | 'bf16' (or None: the bf16 state control) | IDENT for an UNROUNDED fp32 state (the
references' ``Identity()``); ``buffer_bits`` = 8 | 16 | 32 (32: unrounded).
"""
from __future__ import annotations

import torch

from .formats import as_fmt, l2norm, pack_vk, round_buf, unpack_vk

IDENT = 'ident'


class _Buffered:
    """State + buffer + fold, shared by the families.  ``per_channel``: decays are vectors over d_k (KDA)."""

    per_channel = False

    def __init__(self, S, fmt, m=8, hv=None, hk=None, buffer_bits=8, auto_fold=True):
        S = S.float().reshape(-1, S.shape[-2], S.shape[-1])
        self.BH, self.DV, self.DK = S.shape
        self.ident = isinstance(fmt, str) and fmt == IDENT
        self.fmt = None if self.ident else as_fmt(fmt)          # None: bf16 state (unless ident)
        self.m, self.buffer_bits, self.auto_fold = m, buffer_bits, auto_fold
        self.HV = hv or self.BH
        self.HK = hk or self.HV
        assert self.HV % self.HK == 0 and self.BH % self.HV == 0
        self.gqa, self.B = self.HV // self.HK, self.BH // self.HV
        self.load(S)

    # -- storage ----------------------------------------------------------------------------------------------
    def _store(self, S):
        if self.ident:
            self.codes, self.scales = S.clone(), None
            return S.clone()
        self.codes, self.scales = pack_vk(S, self.fmt)
        return unpack_vk(self.codes, self.scales, self.fmt, self.DK)

    def load(self, S):
        S = S.float().reshape(self.BH, self.DV, self.DK)
        self.S0 = self._store(S)
        self.K = torch.zeros(self.B * self.HK, self.m, self.DK)
        self.U = torch.zeros(self.BH, self.m, self.DV)
        gshape = (self.BH, self.m, self.DK) if self.per_channel else (self.BH, self.m)
        self.G = torch.zeros(*gshape)
        self.gcur = torch.zeros(self.BH, self.DK) if self.per_channel else torch.zeros(self.BH)
        self.n = 0

    def adopt(self, codes=None, scales=None):
        """Take over stored codes / scales produced elsewhere (tests re-sync the oracle to a kernel after a fold)."""
        self.codes, self.scales = codes.clone(), (None if scales is None else scales.clone())
        self.S0 = self.codes.clone() if self.ident else unpack_vk(self.codes, self.scales, self.fmt, self.DK)

    def dequantize(self):
        """The stored state S0 [BH, d_v, d_k] (without the buffered tokens)."""
        return self.S0.clone()

    def _round(self, x):
        return round_buf(x.float(), self.buffer_bits)

    def _heads(self, x):
        """[B * HK, ...] per key head / group -> [BH, ...] per value head."""
        return x.reshape(self.B, self.HK, 1, *x.shape[1:]).expand(-1, -1, self.gqa, *x.shape[1:]) \
                .reshape(self.BH, *x.shape[1:])

    def _first(self, x):
        """[BH, ...] -> the first value head of each group, [B * HK, ...] (the key that is buffered)."""
        return x.reshape(self.B, self.HK, self.gqa, *x.shape[1:])[:, :, 0].reshape(self.B * self.HK, *x.shape[1:])

    def _live(self):
        n = self.n
        return self._heads(self.K[:, :n]), self.U[:, :n], self.G[:, :n]

    def _decay(self, G):
        """dec_i of the given buffer entries: [BH, n] (or [BH, n, d_k] per channel)."""
        return torch.exp(self.gcur[:, None] - G)

    # -- state / fold -----------------------------------------------------------------------------------------
    def state(self):
        """The current state: S0 advanced across the pending buffer, [BH, d_v, d_k]."""
        if self.per_channel:
            S = torch.exp(self.gcur)[:, None, :] * self.S0
            if self.n:
                Kb, Ub, G = self._live()
                S = S + torch.einsum('biv,bik->bvk', Ub, Kb * self._decay(G))
            return S
        S = torch.exp(self.gcur)[:, None, None] * self.S0
        if self.n:
            Kb, Ub, G = self._live()
            S = S + torch.einsum('bi,biv,bik->bvk', self._decay(G), Ub, Kb)
        return S

    def fold(self):
        """Advance S0 across the full buffer, slot by slot in order, and re-round it (fold.py:263-274,
        kda.py:177-186, mamba2.py:207-217)."""
        assert self.n == self.m
        Kb, Ub, G = self._live()
        dec = self._decay(G)
        if self.per_channel:
            S = torch.exp(self.gcur)[:, None, :] * self.S0
            Kd = Kb * dec
            for i in range(self.m):
                S = S + Ub[:, i, :, None] * Kd[:, i, None, :]
        else:
            S = torch.exp(self.gcur)[:, None, None] * self.S0
            for i in range(self.m):
                S = S + (dec[:, i, None] * Ub[:, i])[:, :, None] * Kb[:, i, None, :]
        self.S_raw = S
        self.S0 = self._store(S)
        self.gcur = torch.zeros_like(self.gcur)
        self.n = 0

    def _append(self, u, kx, gnew):
        n = self.n
        self.U[:, n] = self._round(u)
        self.K[:, n] = self._round(kx)
        self.gcur = gnew
        self.G[:, n] = gnew
        self.n += 1
        if self.n == self.m and self.auto_fold:
            self.fold()

    def _buffer_term(self, x):
        """sum_{i<n} dec_i (K_i . x) U_i for a read-out x [BH, d_k] (scalar decays)."""
        Kb, Ub, G = self._live()
        return torch.einsum('bi,biv->bv', self._decay(G) * torch.einsum('bik,bk->bi', Kb, x), Ub)


class GDNOracle(_Buffered):
    """Gated DeltaNet (fold.py:233-261).  step(q, k, v, g, beta, scale): q, k raw [BH, d_k] or per key head
    [B * hk, d_k]; v [BH, d_v]; g log decay, beta (after sigmoid) [BH] -> o [BH, d_v] fp32."""

    @torch.no_grad()
    def step(self, q, k, v, g, beta, scale):
        BH = self.BH
        if q.shape[0] != BH:
            q, k = self._heads(q), self._heads(k)
        qn = l2norm(q) * scale
        kn = l2norm(k)
        alpha = torch.exp(self.gcur)[:, None]
        sq = alpha * torch.einsum('bvk,bk->bv', self.S0, qn)
        sk = alpha * torch.einsum('bvk,bk->bv', self.S0, kn)
        if self.n:
            sq = sq + self._buffer_term(qn)
            sk = sk + self._buffer_term(kn)
        a = torch.exp(g.float())[:, None]
        u = beta.float()[:, None] * (v.float() - a * sk)
        o = a * sq + (kn * qn).sum(-1, keepdim=True) * u
        self._append(u, self._first(kn), self.gcur + g.float())
        return o


def gdn_gate(a, b, A_log, dt_bias):
    """vLLM / fla's gating as the step forms it in-kernel (_fused_triton.py:96-100): g = -exp(A_log) softplus(a +
    dt_bias) with softplus passed through above 20, beta = sigmoid(b).  a, b [B, HV]; A_log, dt_bias [HV]."""
    x = a.float() + dt_bias.float()
    sp = torch.where(x <= 20.0, torch.log(1.0 + torch.exp(x)), x)
    return -torch.exp(A_log.float()) * sp, torch.sigmoid(b.float())


def gdn_recurrence(S, q, k, v, g, beta, scale):
    """One textbook gated-delta step on S [BH, d_v, d_k] in place: S <- a S; u = beta (v - S k); S += u k^T;
    o = S q (kda.py:44-52 with a scalar decay)."""
    qn, kn = l2norm(q) * scale, l2norm(k)
    S.mul_(torch.exp(g.float())[:, None, None])
    u = beta.float()[:, None] * (v.float() - torch.einsum('bvk,bk->bv', S, kn))
    S.add_(u[:, :, None] * kn[:, None, :])
    return torch.einsum('bvk,bk->bv', S, qn)


class KDAOracle(_Buffered):
    """KDA: decay per key channel (kda.py:152-175).  step(q, k, v, g, beta, scale=None): q, k raw [BH, d_k],
    v [BH, d_v], g [BH, d_k] log decay, beta [BH] -> o [BH, d_v] fp32.  No grouped keys."""

    per_channel = True

    @torch.no_grad()
    def step(self, q, k, v, g, beta, scale=None):
        BH, n = self.BH, self.n
        scale = self.DK ** -0.5 if scale is None else scale
        qn = l2norm(q.reshape(BH, self.DK)) * scale
        kn = l2norm(k.reshape(BH, self.DK))
        gnew = self.gcur + g.float().reshape(BH, self.DK)
        A = torch.exp(gnew)
        sq = torch.einsum('bvk,bk->bv', self.S0, A * qn)
        sk = torch.einsum('bvk,bk->bv', self.S0, A * kn)
        if n:
            Kd = self.K[:, :n] * torch.exp(gnew[:, None, :] - self.G[:, :n])
            sq = sq + torch.einsum('bi,biv->bv', torch.einsum('bik,bk->bi', Kd, qn), self.U[:, :n])
            sk = sk + torch.einsum('bi,biv->bv', torch.einsum('bik,bk->bi', Kd, kn), self.U[:, :n])
        u = beta.float().reshape(BH, 1) * (v.float().reshape(BH, self.DV) - sk)
        o = sq + (kn * qn).sum(-1, keepdim=True) * u
        self._append(u, kn, gnew)
        return o


def kda_recurrence(S, q, k, v, g, beta, scale=None):
    """One textbook KDA step on S [BH, d_v, d_k] in place (kda.py:44-52)."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    qn, kn = l2norm(q) * scale, l2norm(k)
    S.mul_(torch.exp(g.float())[:, None, :])
    u = beta.float()[:, None] * (v.float() - torch.einsum('bvk,bk->bv', S, kn))
    S.add_(u[:, :, None] * kn[:, None, :])
    return torch.einsum('bvk,bk->bv', S, qn)


def mamba2_gate(dt, A, dt_bias=None, dt_softplus=False, dt_limit=None):
    """dt (raw [B, H]) -> (dt, log decay A dt), fp32 (mamba2.py:45-54)."""
    dt = dt.float()
    if dt_bias is not None:
        dt = dt + dt_bias.float()
    if dt_softplus:
        dt = torch.where(dt <= 20.0, torch.log(1.0 + torch.exp(dt)), dt)
    if dt_limit is not None and tuple(dt_limit) != (0.0, float('inf')):
        dt = dt.clamp(dt_limit[0], dt_limit[1])
    return dt, A.float() * dt


class Mamba2Oracle(_Buffered):
    """Mamba2 / SSD (mamba2.py:176-205).  step(x, dt, B, C, A, D, dt_bias, dt_softplus, dt_limit): x [B, H, d_v],
    dt [B, H], B / C [B, G, d_k], A / D / dt_bias [H] -> y [BH, d_v] fp32.  hk = groups."""

    @torch.no_grad()
    def step(self, x, dt, B, C, A, D=None, dt_bias=None, dt_softplus=False, dt_limit=None):
        BH, n = self.BH, self.n
        dt, g = mamba2_gate(dt.reshape(self.B, self.HV), A, dt_bias, dt_softplus, dt_limit)
        dt, g = dt.reshape(BH), g.reshape(BH)
        x = x.float().reshape(BH, self.DV)
        Bg = B.float().reshape(self.B * self.HK, self.DK)
        Bh = self._heads(Bg)
        Ch = self._heads(C.float().reshape(self.B * self.HK, self.DK))
        u = dt[:, None] * x
        sq = torch.exp(self.gcur)[:, None] * torch.einsum('bvk,bk->bv', self.S0, Ch)
        if n:
            sq = sq + self._buffer_term(Ch)
        y = torch.exp(g)[:, None] * sq + (Bh * Ch).sum(-1, keepdim=True) * u
        if D is not None:
            y = y + D.float().repeat(self.B)[:, None] * x
        self._append(u, Bg, self.gcur + g)
        return y


def mamba2_recurrence(S, x, dt, B, C, A, D=None, dt_bias=None, dt_softplus=False, dt_limit=None):
    """One textbook Mamba2 step on S [B, H, d_v, d_k] in place (mamba2.py:57-70)."""
    H, G = dt.shape[1], B.shape[1]
    dt, g = mamba2_gate(dt, A, dt_bias, dt_softplus, dt_limit)
    Bh = B.float().repeat_interleave(H // G, 1)
    Ch = C.float().repeat_interleave(H // G, 1)
    u = dt[..., None] * x.float()
    S.mul_(torch.exp(g)[..., None, None]).add_(u[..., :, None] * Bh[..., None, :])
    y = torch.einsum('bhvk,bhk->bhv', S, Ch)
    if D is not None:
        y = y + D.float()[:, None] * x.float()
    return y
