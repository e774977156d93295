"""Storage-format descriptors for a recurrent state (the interface of the reference's ``statequant/quantizer.py``).

The packed decode path only consumes the *description* of a format (bits, axis, group, ...) and, in tests, the
fake-quantization it implies.  This module keeps the reference's constructor signatures and attribute names
(``/root/reference/src/statequant/quantizer.py:44-121``) so that user code building ``Quantizer(4, 'k', 64)`` keeps
working, and implements ``fake`` for the formats the packed path can hold (symmetric absmax round-to-nearest-even with
fp32 or fp16 scales, axis 'k' / 'v' / 'head'; bf16 / fp16 casts; identity).  Affine grids, rotations and stochastic
rounding belong to the reference's evaluation path and raise ``NotImplementedError`` here.

States are [..., d_k, d_v] (the fla / transformers orientation), as in the reference.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

AXES = ('k', 'v', 'head')
FP16_TINY = 2.0 ** -24          # smallest fp16 subnormal: floor of a stored fp16 scale (quantizer.py:159-164)


class Format:
    """What every storage format offers: ``fake(S)`` -- S after one store / load round trip, same shape and dtype --
    and ``bits_per_value(d_k, d_v)``, payload and side information together.  Calling a format applies ``fake``."""

    def fake(self, S: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError(type(self).__name__)

    def bits_per_value(self, d_k: int, d_v: int) -> float:
        raise NotImplementedError(type(self).__name__)

    __call__ = lambda self, S: self.fake(S)                 # noqa: E731


@dataclass(frozen=True)
class Identity(Format):
    """Full precision: nothing is rounded (quantizer.py:44-53)."""
    bits: int = 32

    def fake(self, S):
        return S

    def bits_per_value(self, d_k, d_v):
        return float(self.bits)


@dataclass(frozen=True)
class FloatCast(Format):
    """Round trip through a float dtype, 'bf16' or 'fp16' (quantizer.py:56-78; fp8 and stochastic rounding are
    evaluation-only features and are not carried over)."""
    dtype: str = 'fp16'
    stochastic: bool = False

    def fake(self, S):
        if self.stochastic:
            raise NotImplementedError('stochastic FloatCast is not part of the packed decode path')
        dt = {'bf16': torch.bfloat16, 'fp16': torch.float16}[self.dtype]
        return S.float().to(dt).to(S.dtype)

    def bits_per_value(self, d_k, d_v):
        return 16.0


@dataclass(frozen=True)
class Quantizer(Format):
    """Integer grid with per-group scales (quantizer.py:81-121: same fields, same defaults).

    bits, axis ('k': groups of ``group`` key entries within one value column; 'v': groups of value entries within
    one key row; 'head': one scale per head), group, affine, zero_point, rotation, rounding, scale_bits,
    scale_dtype ('fp32': scale used as computed; 'fp16': rounded to fp16 and floored at 2^-24 before the payload is
    rounded against it, which is what a packed store holds).
    """
    bits: int = 4
    axis: str = 'k'
    group: int = 32
    affine: bool = False
    zero_point: str = 'int'
    rotation: str | None = None
    rounding: str = 'rtn'
    scale_bits: int = 16
    scale_dtype: str = 'fp32'

    def __post_init__(self):
        problems = []
        if self.axis not in AXES:
            problems.append(f'axis must be one of {AXES}, got {self.axis!r}')
        if not 2 <= self.bits <= 15:
            problems.append(f'bits must be in 2..15, got {self.bits}')
        if self.zero_point not in ('int', 'fp') or self.rounding not in ('rtn', 'sr'):
            problems.append(f'zero_point {self.zero_point!r} / rounding {self.rounding!r}')
        if self.rotation not in (None, 'hadamard'):
            problems.append(f'rotation {self.rotation!r}')
        if self.scale_bits not in (8, 16) or self.scale_dtype not in ('fp32', 'fp16'):
            problems.append(f'scale_bits {self.scale_bits} / scale_dtype {self.scale_dtype!r}')
        elif self.scale_dtype == 'fp16' and self.scale_bits != 16:
            problems.append('fp16 scales are 16-bit scales')
        assert not problems, '; '.join(problems)

    def _cast_scale(self, scale):
        """quantizer.py:159-164 (16-bit scales only)."""
        if self.scale_bits != 16:
            raise NotImplementedError('8-bit scales are not part of the packed decode path')
        if self.scale_dtype == 'fp16':
            return scale.to(torch.float16).float().clamp_min(FP16_TINY)
        return scale

    def fake(self, S):
        """Symmetric absmax round-to-nearest-even on the format's groups (quantizer.py:169-193, the non-affine,
        unrotated, 'rtn' branch).  A ragged last group is quantized on its own (its absmax is that of its own
        entries)."""
        if self.affine or self.rotation is not None or self.rounding != 'rtn':
            raise NotImplementedError('only symmetric round-to-nearest grids exist on the packed decode path')
        x = S.float()
        qmax = 2 ** (self.bits - 1) - 1
        if self.axis == 'head':
            amax = x.abs().amax((-1, -2), keepdim=True)
            sc = self._cast_scale(amax.clamp_min(1e-8) / qmax)
            return (torch.round(x / sc).clamp(-qmax, qmax) * sc).to(S.dtype)
        dim = -2 if self.axis == 'k' else -1
        out = torch.empty_like(x)
        n = x.shape[dim]
        for lo in range(0, n, self.group):
            sl = [slice(None)] * x.dim()
            sl[dim] = slice(lo, min(lo + self.group, n))
            blk = x[tuple(sl)]
            sc = self._cast_scale(blk.abs().amax(dim, keepdim=True).clamp_min(1e-8) / qmax)
            out[tuple(sl)] = torch.round(blk / sc).clamp(-qmax, qmax) * sc
        return out.to(S.dtype)

    def bits_per_value(self, d_k, d_v):
        """Payload bits plus the per-group side information (scale, and a zero point for affine grids) spread over the
        group's values; a ragged last group counts as a whole group."""
        per_group = self.scale_bits
        if self.affine:
            per_group += self.bits if self.zero_point == 'int' else self.scale_bits
        if self.axis == 'head':
            groups, values = 1, d_k * d_v
        else:
            values = d_k if self.axis == 'k' else d_v
            groups = (values + self.group - 1) // self.group
        return self.bits + per_group * groups / values
