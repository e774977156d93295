"""Oracle (test infrastructure): the per-slot byte layout of the serving cache and the prefill-side read / write, in
torch on the CPU.

Restates /root/reference/src/statequant/kernels/slots.py:76-95 (field order, 16-byte aligned offsets), :108-117
(typed views), :210-252 (read / write); the KDA variant kda.py:311-323, 351-386 (decays per key channel) and the
Mamba2 variant mamba2.py:359-370 (same fields as GDN, key buffer per group).
"""
from __future__ import annotations

import torch

from .formats import as_fmt, pack_vk, unpack_vk

ALIGN = 16
_SIZE = {torch.float32: 4, torch.int32: 4, torch.float16: 2, torch.bfloat16: 2, torch.int8: 1, torch.uint8: 1}


def layout(family, fmt, hv, hk, dk, dv, m=8, buffer_bits=8, state_dtype=torch.bfloat16):
    """{field: (offset, dtype, shape, nbytes)}, total bytes per slot.  family: 'gdn' | 'mamba2' | 'kda'."""
    fmt = as_fmt(fmt)
    per_channel = family == 'kda'
    if per_channel:
        assert hk == hv
    fields = [('GB', torch.float32, (hv, m, dk) if per_channel else (hv, m)),
              ('GCUR', torch.float32, (hv, dk) if per_channel else (hv,)),
              ('NPTR', torch.int32, (max(hv, 4),))]
    if fmt is not None:
        if fmt.axis == 'k':
            fields.append(('SC', torch.float16, (hv, dv, -(-dk // fmt.group))))
        else:
            fields.append(('SC', torch.float16, (hv, dv // fmt.group, dk)))
    if buffer_bits == 8:
        fields += [('KBS', torch.float16, (hk, m)), ('UBS', torch.float16, (hv, m))]
    if fmt is None:
        fields.append(('S', state_dtype, (hv, dv, dk)))
    else:
        fields.append(('S', torch.uint8, (hv, dv, dk // 2)) if fmt.bits == 4 else ('S', torch.int8, (hv, dv, dk)))
    bdt = torch.int8 if buffer_bits == 8 else torch.bfloat16
    fields += [('KB', bdt, (hk, m, dk)), ('UB', bdt, (hv, m, dv))]
    table, off = {}, 0
    for name, dt, shape in fields:
        nb = _SIZE[dt]
        for s in shape:
            nb *= s
        table[name] = (off, dt, shape, nb)
        off += (nb + ALIGN - 1) // ALIGN * ALIGN
    return table, off


def views(table, blob):
    """uint8 [num_slots, >= nbytes] -> {field: typed view [num_slots, *shape]}."""
    n = blob.shape[0]
    return {name: blob[:, off:off + nb].view(dt).view(n, *shape) for name, (off, dt, shape, nb) in table.items()}


def read(V, idx, fmt, hv, hk, dk, dv, m, per_channel=False):
    """The current state of slots idx as fp32 [P, hv, d_v, d_k]: the stored state advanced across the pending buffer
    (slots.py:210-233, kda.py:351-372).  Dead buffer entries are masked with where, never multiplied."""
    idx = idx.long()
    P = idx.shape[0]
    qbuf = 'KBS' in V
    codes = V['S'][idx].reshape(P * hv, *V['S'].shape[2:])
    sc = V['SC'][idx].reshape(P * hv, *V['SC'].shape[2:]) if 'SC' in V else None
    S0 = unpack_vk(codes, sc, fmt, dk).view(P, hv, dv, dk)
    Kb, Ub = V['KB'][idx].float(), V['UB'][idx].float()
    if qbuf:
        Kb = Kb * V['KBS'][idx].float()[..., None]
        Ub = Ub * V['UBS'][idx].float()[..., None]
    n = V['NPTR'][idx, 0] & (m - 1)
    gcur = V['GCUR'][idx]
    slot = torch.arange(m)[None, :] < n[:, None]                       # [P, m]
    if per_channel:
        live = slot[:, None, :, None]                                  # [P, 1, m, 1]
        dec = torch.where(live, torch.exp(gcur[:, :, None, :] - torch.where(live, V['GB'][idx], 0.)), 0.)
        Ub = torch.where(live, Ub, 0.)
        Kd = torch.where(live, Kb, 0.) * dec
        return torch.exp(gcur)[:, :, None, :] * S0 + torch.einsum('phmv,phmk->phvk', Ub, Kd)
    live = slot[:, None, :]                                            # [P, 1, m]
    dec = torch.where(live, torch.exp(gcur[..., None] - torch.where(live, V['GB'][idx], 0.)), 0.)
    Ub = torch.where(live[..., None], Ub, 0.)
    Kb = torch.where(live.expand(-1, hk, -1)[..., None], Kb, 0.)
    Kx = Kb.repeat_interleave(hv // hk, dim=1)
    return torch.exp(gcur)[..., None, None] * S0 + torch.einsum('phmv,phmk->phvk', Ub * dec[..., None], Kx)


def write(V, idx, S, fmt, hv, dk, dv):
    """Pack states S [P, hv, d_v, d_k] into slots idx and empty their buffers: NPTR = 0, GCUR = 0; buffer contents
    stay as they are (slots.py:236-252)."""
    idx = idx.long()
    P = idx.shape[0]
    if 'SC' not in V and V['S'].dtype == torch.float32:          # fp32 state: stored as is (slots.py:242-243)
        V['S'][idx] = S.reshape(P, *V['S'].shape[1:]).float()
        V['NPTR'][idx] = 0
        V['GCUR'][idx] = 0.
        return
    codes, sc = pack_vk(S.reshape(P * hv, dv, dk), fmt)
    V['S'][idx] = codes.view(P, *V['S'].shape[1:])
    if 'SC' in V:
        V['SC'][idx] = sc.view(P, *V['SC'].shape[1:])
    V['NPTR'][idx] = 0
    V['GCUR'][idx] = 0.
