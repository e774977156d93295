"""Oracle (test infrastructure): the mixed-width GGA / STEP slot with the PW window, in torch on the CPU.

Restates, from the reference's torch code (never its Triton kernels):
    half_clamp, step_fit      /root/reference/src/statequant/step_quant.py:35-36, 62-96  (STEP's dual-axis fit)
    fp8_vec, fp8_parts        /root/reference/src/statequant/methods_ext/gga.py:225-233  (R_FP8 per vector)
    GGAState.step/read/write  /root/reference/src/statequant/integrations/vllm_gga.py:86-168 (the fp32-valued slot
                              step of ``GGALayout``: Algorithm 1 with per-head frozen widths and fp16 pivots)
    head_bytes, slot_table    vllm_gga.py:174-217 (stored bytes per head, per-layer offset tables, window size)
    pack_head, unpack_head    the byte layout documented in /root/reference/src/statequant/kernels/_gga_triton.py:3-13
                              and its `_store_codes` / `_load_codes` (:40-95): a NumPy restatement used to check the
                              bytes the HIP kernels write

The state is canonical here: O [N, HV, d_k, d_v] (key-major, as the packed blob stores it), the window oldest first.

How it is pinned (tests/test_oracle_gga.py): ``step_fit`` and ``fp8_vec`` bit-for-bit against the reference's own
functions (tests/golden/gga.pt); the slot tables and bits-per-value figures against ``GGAPacked`` / ``GGA`` /
``pure_write`` of the reference (same file); ``GGAState.step`` step by step against the reference's ``PureWrite`` /
``StepQuant`` path driven as its tests/test_vllm_gga.py drives it (outputs, stored state, window entries), and, with
the roundings switched off, against the textbook gated delta rule; pack / unpack of every width against a
bit-twiddling brute force.
"""
from __future__ import annotations

import numpy as np
import torch

GROUP = 32
ALIGN = 16
WIDTHS = (2, 4, 6, 8, 16)


# ---------------------------------------------------------------------------------------------------------------
# STEP's dual-axis fit (step_quant.py:35-96)
# ---------------------------------------------------------------------------------------------------------------
def half_clamp(x):
    return x.clamp(2 ** -24, 65504).half().float()


def fit_parts(x, bits, w, group=GROUP):
    """x [B, H, K, V] fp32, bits [H] in {2, 4, 6, 8, 16}, w [H, K].  Returns (r_full [B,H,K,V], c [B,H,1,V],
    z [B,H,K,V], integer mask [1,H,1,1]); the fitted state is r_full * c * z on integer heads and fp16(x) on pivots."""
    x = x.float()
    b = bits.to(torch.int64)
    wb = w.float()[None, :, :, None]
    integer = (b != 16)[None, :, None, None]
    qmax = (2.0 ** (b.clamp_max(8).float() - 1) - 1)[None, :, None, None].expand(1, -1, x.shape[2], 1).clone()
    r = half_clamp((x.abs().mean(-1, keepdim=True).clamp_min(1e-20) / wb).sqrt())
    r_full = r.expand_as(x).clone()
    two = b == 2
    if two.any():
        assert x.shape[-1] % group == 0
        xg = x[:, two].reshape(*x[:, two].shape[:-1], -1, group)
        r2 = half_clamp((xg.abs().mean(-1).clamp_min(1e-20) / wb[:, two]).sqrt())
        r_full[:, two] = r2.repeat_interleave(group, -1)
        qmax[:, two] = 3
    y0 = x / r_full
    c = half_clamp(torch.where(integer, y0.abs() / qmax, torch.zeros(())).amax(-2, keepdim=True))

    def encode(cols):
        y = y0 / cols
        z = torch.round(y).maximum(-qmax).minimum(qmax)
        if two.any():
            y2 = y[:, two]
            z[:, two] = torch.where(y2 >= 0, 1., -1.) * torch.where(y2.abs() >= 2, 3., 1.)
        return z
    z = encode(c)
    vv = r_full * z
    ww = wb.square() * integer
    num = (ww * vv * x).sum(-2, keepdim=True)
    den = (ww * vv.square()).sum(-2, keepdim=True)
    c = half_clamp(torch.where(den > 0, num / den.clamp_min(1e-30), c))
    z = encode(c)
    return r_full, c, z, integer


def step_fit(x, bits, w, group=GROUP):
    """The fitted state (the reference's ``fit``)."""
    r_full, c, z, integer = fit_parts(x, bits, w, group)
    return torch.where(integer, r_full * c * z, x.float().half().float())


# ---------------------------------------------------------------------------------------------------------------
# FP8 vectors (methods_ext/gga.py:225-233)
# ---------------------------------------------------------------------------------------------------------------
def fp8_parts(x):
    """(e4m3 codes as uint8, scale fp32 [..., 1]) of R_FP8 per vector along the last axis."""
    amax = x.abs().amax(-1, keepdim=True)
    s = amax / torch.full_like(amax, 448.)
    safe = torch.where(s > 0, s, torch.ones_like(s))
    code = (x / safe).clamp(-448., 448.).to(torch.float8_e4m3fn)
    return code.view(torch.uint8), s


def fp8_vec(x):
    code, s = fp8_parts(x)
    safe = torch.where(s > 0, s, torch.ones_like(s))
    return torch.where(s > 0, code.view(torch.float8_e4m3fn).float() * safe, torch.zeros_like(x))


# ---------------------------------------------------------------------------------------------------------------
# the slot step (vllm_gga.py:86-168), on canonical tensors
# ---------------------------------------------------------------------------------------------------------------
class GGAState:
    """N slots of one layer: O [N, HV, d_k, d_v] fp32 values on each head's width, and with ``pw`` the window
    P [N, m, HV, d_k], V [N, m, HV, d_v] (reconstructed FP8 vectors, oldest first) with its fill count n [N].

    ``quant`` / ``enc`` replace the two roundings (tests switch them off to compare with the textbook rule)."""

    def __init__(self, bits, w, num_slots, hv, hk, dk, dv, pw=False, m=8, group=GROUP, quant=None, enc=None):
        self.bits, self.w = torch.as_tensor(bits), torch.as_tensor(w).float()
        self.HV, self.HK, self.DK, self.DV, self.pw, self.m, self.group = hv, hk, dk, dv, pw, (m if pw else 1), group
        self.gqa = hv // hk
        self.piv = self.bits == 16
        self.O = torch.zeros(num_slots, hv, dk, dv)
        self.P = torch.zeros(num_slots, self.m, hv, dk)
        self.V = torch.zeros(num_slots, self.m, hv, dv)
        self.n = torch.zeros(num_slots, dtype=torch.int64)
        self.quant = quant or (lambda S: step_fit(S, self.bits, self.w, self.group))
        self.enc = enc or fp8_vec

    @staticmethod
    def gate(a, b, A_log, dt_bias):
        g = -A_log.float().exp() * torch.nn.functional.softplus(a.float() + dt_bias.float())
        return g, b.float().sigmoid()

    def step(self, idx, q, k, v, scale, g, beta):
        """q, k [B, HK, d_k]; v [B, HV, d_v]; g (log decay), beta [B, HV]; idx [B] (<= 0: padding row).  Returns
        o [B, HV, d_v] fp32 (zero on padding rows)."""
        B = idx.shape[0]
        li = idx.long()
        valid = idx > 0
        qf, kf = q.float(), k.float()
        qf = qf * torch.rsqrt((qf * qf).sum(-1, keepdim=True) + 1e-6) * scale
        kf = kf * torch.rsqrt((kf * kf).sum(-1, keepdim=True) + 1e-6)
        qf, kf = qf.repeat_interleave(self.gqa, 1), kf.repeat_interleave(self.gqa, 1)
        a, bt, vf = g.float().exp(), beta.float(), v.float()
        O = self.O[li]
        AO = a[..., None, None] * (O - bt[..., None, None] * kf[..., None]
                                   * torch.einsum('bhk,bhkv->bhv', kf, O)[:, :, None])
        bk = bt[..., None] * kf
        new = bk[..., None] * vf[..., None, :]
        o = torch.einsum('bhkv,bhk->bhv', AO, qf) + (bk * qf).sum(-1, keepdim=True) * vf
        piv = self.piv
        if self.pw:
            m = self.m
            P, Vq = self.P[li], self.V[li]
            n = self.n[li].clamp(0, m)
            live = (torch.arange(m)[None, :] < n[:, None])[..., None, None]
            AP = a[:, None, :, None] * (P - bt[:, None, :, None] * kf[:, None]
                                        * (kf[:, None] * P).sum(-1, keepdim=True))
            P = torch.where(live, self.enc(AP), torch.zeros(()))
            o = o + torch.einsum('bmhk,bhk,bmhv->bhv', P, qf, Vq)
            full = (n == m)[:, None, None, None]
            Om = AO + torch.where(full, P[:, 0, :, :, None] * Vq[:, 0, :, None, :], torch.zeros(()))
            On = self.quant(Om)
            On = torch.where(piv[None, :, None, None], (AO + new).half().float(), On)
            nonp = (~piv)[None, :, None].float()
            pn, vn = self.enc(bk) * nonp, self.enc(vf) * nonp
            P_shift = torch.cat([P[:, 1:], pn[:, None]], 1)
            V_shift = torch.cat([Vq[:, 1:], vn[:, None]], 1)
            at = (torch.arange(m)[None, :] == n[:, None])[..., None, None]
            P_new = torch.where(full, P_shift, torch.where(at, pn[:, None], P))
            V_new = torch.where(full, V_shift, torch.where(at, vn[:, None], Vq))
            ok = valid[:, None, None, None]
            self.P[li] = torch.where(ok, P_new, self.P[li])
            self.V[li] = torch.where(ok, V_new, self.V[li])
            self.n[li] = torch.where(valid, (n + 1).clamp_max(m), self.n[li])
        else:
            On = self.quant(AO + new)                      # the fit itself keeps pivots in fp16
        self.O[li] = torch.where(valid[:, None, None, None], On, self.O[li])
        return torch.where(valid[:, None, None], o, torch.zeros(()))

    def read(self, idx):
        """Logical state O + sum of the queued pairs, canonical [P, HV, d_k, d_v]."""
        li = idx.long()
        S = self.O[li].clone()
        if self.pw:
            n = self.n[li].clamp(0, self.m)
            live = (torch.arange(self.m)[None, :] < n[:, None])[..., None, None]
            S = S + torch.einsum('bmhk,bmhv->bhkv', torch.where(live, self.P[li], torch.zeros(())),
                                 torch.where(live, self.V[li], torch.zeros(())))
        return S

    def write(self, idx, S):
        """Round canonical states S [P, HV, d_k, d_v] with the plan, store them, empty the window."""
        li = idx.long()
        self.O[li] = self.quant(S.float())
        self.n[li] = 0
        if self.pw:
            self.P[li] = 0.
            self.V[li] = 0.


def textbook_step(S, q, k, v, g, beta, scale, gqa):
    """One token of the gated delta rule on S [B, HV, d_k, d_v] (fla's normalisation); returns (o, S_new)."""
    qf, kf = q.float(), k.float()
    qf = qf * torch.rsqrt((qf * qf).sum(-1, keepdim=True) + 1e-6) * scale
    kf = kf * torch.rsqrt((kf * kf).sum(-1, keepdim=True) + 1e-6)
    qf, kf = qf.repeat_interleave(gqa, 1), kf.repeat_interleave(gqa, 1)
    Sa = g.float().exp()[..., None, None] * S
    u = beta.float()[..., None] * (v.float() - torch.einsum('bhkv,bhk->bhv', Sa, kf))
    Sn = Sa + kf[..., None] * u[:, :, None]
    return torch.einsum('bhkv,bhk->bhv', Sn, qf), Sn


# ---------------------------------------------------------------------------------------------------------------
# stored bytes (vllm_gga.py:174-217; _gga_triton.py:3-13, 40-95)
# ---------------------------------------------------------------------------------------------------------------
def _al(n):
    return -(-n // ALIGN) * ALIGN


def head_bytes(b, dk, dv, group=GROUP):
    if b == 16:
        return 2 * dk * dv
    if b == 2:
        return dk * dv // 4 + 2 * dk * (dv // group) + 2 * dv
    return dk * dv * b // 8 + 2 * dk + 2 * dv


def slot_table(widths, dk, dv, group=GROUP):
    """(byte offsets of the heads, bytes of the layer): 16 bytes of counters first, heads 16-byte aligned."""
    offs, off = [], 16
    for b in widths:
        offs.append(off)
        off += _al(head_bytes(int(b), dk, dv, group))
    return offs, off


def window_bytes(m, dk, dv):
    """Bytes of one head's window: P e4m3 [m, d_k], V e4m3 [m, d_v], PS fp32 [m], VS fp32 [m]."""
    return m * (dk + dv + 8)


def bits_per_value(tables, hv, dk, dv, pw, m, group=GROUP):
    """Mean stored bits per state value over the layers (without the counters), window included."""
    n = hv * dk * dv
    st = sum(sum(head_bytes(int(x), dk, dv, group) for x in widths) for widths in tables)
    q = hv * window_bytes(m, dk, dv) * len(tables) if pw else 0
    return 8 * (st + q) / (n * len(tables))


def pack_head(r, c, z, b, group=GROUP):
    """One head's stored bytes (numpy uint8) from its fit parts: r [d_k] (2 bit: [d_k, d_v / group]), c [d_v],
    z [d_k, d_v] signed levels (fp32 tensors); b = 16: ``z`` holds the values themselves."""
    z = np.asarray(z, dtype=np.float32)
    dk, dv = z.shape
    if b == 16:
        return z.astype(np.float16).view(np.uint8).reshape(-1)
    u = (((z + 3) / 2) if b == 2 else (z + (2 ** (b - 1) - 1))).astype(np.int64)
    assert u.min() >= 0 and u.max() < (1 << b)
    if b == 8:
        codes = u.astype(np.uint8)
    elif b == 4:
        codes = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    elif b == 2:
        codes = (u[:, 0::4] | (u[:, 1::4] << 2) | (u[:, 2::4] << 4) | (u[:, 3::4] << 6)).astype(np.uint8)
    else:
        wd = u[:, 0::4] | (u[:, 1::4] << 6) | (u[:, 2::4] << 12) | (u[:, 3::4] << 18)
        codes = np.stack([wd & 255, (wd >> 8) & 255, wd >> 16], -1).astype(np.uint8).reshape(dk, -1)
    rr = np.asarray(r, dtype=np.float32).astype(np.float16).view(np.uint8).reshape(-1)
    cc = np.asarray(c, dtype=np.float32).astype(np.float16).view(np.uint8).reshape(-1)
    return np.concatenate([codes.reshape(-1), rr, cc])


def unpack_head(raw, b, dk, dv, group=GROUP):
    """Inverse of ``pack_head``: the head's fp32 values [d_k, d_v] = (r * c) * z."""
    raw = np.asarray(raw, dtype=np.uint8)
    if b == 16:
        return raw[:2 * dk * dv].view(np.float16).astype(np.float32).reshape(dk, dv)
    nc = dk * dv * b // 8
    by = raw[:nc].astype(np.int64).reshape(dk, -1)
    u = np.zeros((dk, dv), dtype=np.int64)
    if b == 8:
        u = by
    elif b == 4:
        u[:, 0::2], u[:, 1::2] = by & 15, by >> 4
    elif b == 2:
        for t in range(4):
            u[:, t::4] = (by >> (2 * t)) & 3
    else:
        t3 = by.reshape(dk, dv // 4, 3)
        wd = t3[..., 0] | (t3[..., 1] << 8) | (t3[..., 2] << 16)
        for t in range(4):
            u[:, t::4] = (wd >> (6 * t)) & 63
    z = (u * 2 - 3 if b == 2 else u - (2 ** (b - 1) - 1)).astype(np.float32)
    nr = dk * (dv // group) if b == 2 else dk
    r = raw[nc:nc + 2 * nr].view(np.float16).astype(np.float32)
    c = raw[nc + 2 * nr:nc + 2 * nr + 2 * dv].view(np.float16).astype(np.float32)
    rf = np.repeat(r.reshape(dk, -1), group, 1) if b == 2 else np.repeat(r[:, None], dv, 1)
    return (rf * c[None, :]) * z
