"""Oracle (test infrastructure): the packed storage format and the rounding rules, in torch on the CPU.

Restates /root/reference/src/statequant/kernels/fold.py:123-191 (``pack_vk``, ``unpack_vk``, ``_nrm``, ``_round_buf``)
and /root/reference/src/statequant/quantizer.py:159-164 (``_cast_scale``).  A format is given as the plain tuple
(bits, axis, group) or None for the bf16 state control; Fmt below carries it.
"""
from __future__ import annotations

from typing import NamedTuple, Optional

import torch

FP16_TINY = 2.0 ** -24


class Fmt(NamedTuple):
    bits: int
    axis: str
    group: int

    @property
    def qmax(self):
        return 2 ** (self.bits - 1) - 1


def as_fmt(f) -> Optional[Fmt]:
    """(bits, axis, group) | object with those attributes | 'bf16' | None -> Fmt | None."""
    if f is None or f == 'bf16':
        return None
    if isinstance(f, Fmt):
        return f
    if isinstance(f, tuple):
        return Fmt(*f)
    return Fmt(f.bits, f.axis, f.group)


def fp16_scale(amax: torch.Tensor, qmax: float) -> torch.Tensor:
    """Stored scale of a group with absolute maximum ``amax``: max(amax, 1e-8) / qmax rounded to fp16 (nearest
    even, subnormals kept), read back as fp32 and floored at 2^-24 (quantizer.py:159-164, 177)."""
    return (amax.clamp_min(1e-8) / qmax).to(torch.float16).float().clamp_min(FP16_TINY)


def round_buf(x: torch.Tensor, bits: int) -> torch.Tensor:
    """A buffered vector after its store/load round trip (fold.py:186-191): bf16, or int8 with ONE fp16 absmax
    scale over the last axis; 32 = kept as is (the references' exact mode)."""
    if bits == 32:
        return x.float()
    if bits == 16:
        return x.to(torch.bfloat16).float()
    s = fp16_scale(x.abs().amax(-1, keepdim=True), 127)
    return torch.round(x / s).clamp(-127, 127) * s


def round_buf_parts(x: torch.Tensor):
    """The int8 codes and fp16 scale that ``round_buf(x, 8)`` stands for."""
    s = fp16_scale(x.abs().amax(-1, keepdim=True), 127)
    return torch.round(x / s).clamp(-127, 127).to(torch.int8), s.squeeze(-1).to(torch.float16)


def l2norm(x: torch.Tensor) -> torch.Tensor:
    """fla's normalisation, epsilon inside the square root (fold.py:181-183)."""
    x = x.float()
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def pack_vk(x: torch.Tensor, fmt):
    """Value-major state [N, d_v, d_k] -> (codes, scales) (fold.py:123-147).

    axis 'k': groups of ``group`` consecutive key entries within one value row; the last group may be shorter and is
    quantized with the absmax of its own entries.  axis 'v': groups of ``group`` consecutive value rows at one key
    column.  4-bit codes: two per byte, byte j = (c[2j] + 8) | (c[2j+1] + 8) << 4.  bf16: plain cast, scales = [1.]."""
    fmt = as_fmt(fmt)
    x = x.float().reshape(-1, x.shape[-2], x.shape[-1])
    N, DV, DK = x.shape
    if fmt is None:
        return x.to(torch.bfloat16).contiguous(), torch.ones(1, dtype=torch.float16)
    g, qmax = fmt.group, fmt.qmax
    if fmt.axis == 'k':
        ng = (DK + g - 1) // g
        codes = torch.empty(N, DV, DK, dtype=torch.int8)
        scales = torch.empty(N, DV, ng, dtype=torch.float32)
        for gi in range(ng):
            blk = x[:, :, gi * g:(gi + 1) * g]
            s = fp16_scale(blk.abs().amax(-1, keepdim=True), qmax)
            codes[:, :, gi * g:(gi + 1) * g] = torch.round(blk / s).clamp(-qmax, qmax).to(torch.int8)
            scales[:, :, gi] = s.squeeze(-1)
    else:
        assert DV % g == 0
        blk = x.reshape(N, DV // g, g, DK)
        s = fp16_scale(blk.abs().amax(2, keepdim=True), qmax)
        codes = torch.round(blk / s).clamp(-qmax, qmax).to(torch.int8).reshape(N, DV, DK)
        scales = s.reshape(N, DV // g, DK)
    if fmt.bits == 4:
        u = (codes + 8).to(torch.uint8)
        codes = u[..., 0::2] | (u[..., 1::2] << 4)
    return codes.contiguous(), scales.to(torch.float16).contiguous()


def unpack_vk(codes: torch.Tensor, scales, fmt, d_k: int) -> torch.Tensor:
    """Inverse of ``pack_vk``: fp32 [N, d_v, d_k] (fold.py:155-173)."""
    fmt = as_fmt(fmt)
    if fmt is None:
        return codes.float()
    N, DV = codes.shape[:2]
    if fmt.bits == 4:
        c = codes.to(torch.int32)
        x = torch.empty(N, DV, d_k, dtype=torch.float32)
        x[..., 0::2] = ((c & 15) - 8).float()
        x[..., 1::2] = (((c >> 4) & 15) - 8).float()
    else:
        x = codes.float()
    s = scales.float()
    g = fmt.group
    if fmt.axis == 'k':
        col_group = torch.arange(d_k) // g
        return x * s[:, :, col_group]
    row_group = torch.arange(DV) // g
    return x * s[:, row_group, :]


def fake(x: torch.Tensor, fmt) -> torch.Tensor:
    """Store/load round trip of a value-major state."""
    c, s = pack_vk(x, fmt)
    return unpack_vk(c, s, fmt, x.shape[-1])
