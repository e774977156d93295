"""Packed recurrent-state storage for Gated DeltaNet and the lockstep decode step, on HIP kernels.

Mirrors the host API of the reference's ``statequant/kernels/fold.py`` (``/root/reference/src/statequant/kernels/
fold.py``): ``packed_format``, ``pack`` / ``unpack`` / ``pack_vk`` / ``unpack_vk``, ``check_dims``, ``use_fused`` and
``PackedGDNState`` keep their names, arguments and tensor layouts; the Triton launches (fold.py:400-424) are replaced
by one call into ``libsqhip.so`` (``sq_gdn_step``).

The decode algebra (fold.py:1-19): the stored state S_0 is kept rounded and rewritten only every ``m`` tokens; the
tokens in between sit in a buffer of (cumulative log decay G_i, normalised key k_i, delta value u_i); a step reads the
stored codes once and the buffer once; a full buffer is folded into the state, which is re-rounded on the device.

Layouts: states enter and leave as [BH, d_k, d_v]; they are stored value-major, [BH, d_v, d_k].
"""
from __future__ import annotations

import ctypes
import dataclasses

import torch

from ..quantizer import FloatCast, Quantizer
from . import _hip

_FP16_MIN = 2.0 ** -24


def pow2(n):
    """Smallest power of two >= n."""
    return 1 << max(0, (int(n) - 1).bit_length())


def packed_format(fmt):
    """The format a packed store holds: ``fmt`` with fp16 scales, or None for the bf16 control (fold.py:91-104).

    Accepts a symmetric round-to-nearest ``Quantizer`` (4 or 8 bits, axis 'k' or 'v', no rotation, 16-bit scales) or
    'bf16' / ``FloatCast('bf16')`` / None.  Any object with the Quantizer's attributes is taken (duck typing), so
    formats built with the reference's own class pass through."""
    if fmt is None or fmt == 'bf16':
        return None
    if isinstance(fmt, FloatCast) or type(fmt).__name__ == 'FloatCast':
        if fmt.dtype == 'bf16' and not fmt.stochastic:
            return None
    need = ('bits', 'axis', 'group', 'affine', 'rotation', 'rounding', 'scale_bits')
    assert all(hasattr(fmt, a) for a in need), f'packed storage needs a Quantizer or bf16, got {fmt!r}'
    assert fmt.bits in (4, 8) and fmt.axis in ('k', 'v'), (fmt.bits, fmt.axis)
    assert not fmt.affine and fmt.rotation is None and fmt.rounding == 'rtn' and fmt.scale_bits == 16, \
        'packed storage implements symmetric RTN with 16-bit scales and no rotation'
    assert fmt.group % 2 == 0
    if isinstance(fmt, Quantizer):
        return dataclasses.replace(fmt, scale_dtype='fp16')
    return Quantizer(fmt.bits, fmt.axis, fmt.group, scale_dtype='fp16')


def check_dims(fmt, dk, dv):
    """Head dims and groups a packed GDN store accepts (fold.py:63-76)."""
    assert dk >= 16 and dk % 2 == 0, f'd_k must be even and >= 16, got {dk}'
    assert dv % 32 == 0, f'd_v must be a multiple of 32, got {dv}'
    if fmt is not None:
        g = fmt.group
        assert g >= 2 and g & (g - 1) == 0, f'group {g} must be a power of two'
        if fmt.axis == 'k':
            assert g <= pow2(dk) and pow2(dk) // g <= 8, f'key group {g} on d_k {dk}: 1 .. 8 groups'
        else:
            assert dv % g == 0, f'value group {g} must divide d_v {dv}'


def use_fused(fused, bh, axis_v=False):
    """Kept for call compatibility (fold.py:79-85).  There is a single HIP step, always one launch."""
    return True


def _bits(fmt):
    return 16 if fmt is None else fmt.bits


def _scale_of(amax, qmax):
    """absmax -> stored scale: max(amax, 1e-8) / qmax, to fp16 and back, floored at 2^-24 (quantizer.py:159-164).
    The divisor is a device tensor: torch's GPU division by a Python scalar multiplies by the rounded reciprocal,
    which is not the IEEE quotient the kernels and the CPU path compute."""
    return (amax.clamp_min(1e-8) / torch.full((), qmax, device=amax.device)).to(torch.float16).float() \
        .clamp_min(_FP16_MIN)


# ---------------------------------------------------------------------------------------------------------------
# storage format (torch; the reference's pack / unpack are torch too, fold.py:111-173)
# ---------------------------------------------------------------------------------------------------------------
def pack_vk(x, fmt):
    """Value-major state [BH, d_v, d_k] (or [..., d_v, d_k]) -> (codes, scales) (fold.py:123-147).

    codes   int8 [BH, d_v, d_k]; 4 bit: uint8 [BH, d_v, d_k/2], byte j = (c[2j] + 8) | (c[2j+1] + 8) << 4;
            bf16 state: bf16 [BH, d_v, d_k]
    scales  fp16; axis 'k': [BH, d_v, ceil(d_k/group)] (a ragged last group has its own scale);
            axis 'v': [BH, d_v/group, d_k]; bf16 state: a [1] tensor of ones
    """
    fmt = packed_format(fmt)
    x = x.float().reshape(-1, x.shape[-2], x.shape[-1])
    n, dv, dk = x.shape
    if fmt is None:
        return x.to(torch.bfloat16).contiguous(), torch.ones(1, device=x.device, dtype=torch.float16)
    g = fmt.group
    qmax = float(2 ** (fmt.bits - 1) - 1)
    if x.is_cuda and n and (fmt.axis == 'k' or dv % g == 0):          # the HIP pack kernels (same arithmetic, one launch)
        codes = torch.empty(n, dv, dk if fmt.bits == 8 else dk // 2, device=x.device,
                            dtype=torch.int8 if fmt.bits == 8 else torch.uint8)
        sc = torch.empty((n, dv, -(-dk // g)) if fmt.axis == 'k' else (n, dv // g, dk), device=x.device,
                         dtype=torch.float16)
        lay = _hip.SqLayout(bits=fmt.bits, axis_k=int(fmt.axis == 'k'), group=g, buffer_bits=8, m=1, hv=1, hk=1,
                            dk=dk, dv=dv)
        _hip.pack_into(lay, x.contiguous().view(n, 1, dv, dk), codes, codes[0].numel(), sc, sc[0].numel())
        return codes, sc
    if fmt.axis == 'k':
        ng = -(-dk // g)
        xg = torch.nn.functional.pad(x, (0, ng * g - dk)).view(n, dv, ng, g)       # zero pad: same absmax
        sc = _scale_of(xg.abs().amax(3, keepdim=True), qmax)
        q = torch.round(xg / sc).clamp_(-qmax, qmax).view(n, dv, ng * g)[:, :, :dk]
        sc = sc.view(n, dv, ng)
    else:
        assert dv % g == 0, f'value group {g} must divide d_v {dv}'
        xg = x.view(n, dv // g, g, dk)
        sc = _scale_of(xg.abs().amax(2, keepdim=True), qmax)
        q = torch.round(xg / sc).clamp_(-qmax, qmax).view(n, dv, dk)
        sc = sc.view(n, dv // g, dk)
    q = q.to(torch.int8)
    if fmt.bits == 4:
        nib = (q + 8).to(torch.uint8)
        q = nib[:, :, 0::2] | (nib[:, :, 1::2] << 4)
    return q.contiguous(), sc.to(torch.float16).contiguous()


def unpack_vk(codes, scales, fmt, d_k):
    """Inverse of ``pack_vk``: -> fp32 [BH, d_v, d_k] (fold.py:155-173)."""
    fmt = packed_format(fmt)
    if fmt is None:
        return codes.float()
    n, dv = codes.shape[:2]
    if fmt.bits == 4:
        b = codes.to(torch.int16)
        x = torch.stack(((b & 15) - 8, ((b >> 4) & 15) - 8), dim=-1).view(n, dv, -1)[:, :, :d_k].float()
    else:
        x = codes.float()
    sc = scales.float()
    g = fmt.group
    if fmt.axis == 'k':
        return x * sc.repeat_interleave(g, dim=2)[:, :, :d_k]
    return (x.view(n, dv // g, g, d_k) * sc[:, :, None, :]).view(n, dv, d_k)


def pack(S, fmt):
    """[BH, d_k, d_v] (or [B, H, d_k, d_v]) float -> (codes, scales) of the value-major store (fold.py:111-120)."""
    x = S.float().reshape(-1, S.shape[-2], S.shape[-1]).transpose(1, 2).contiguous()
    return pack_vk(x, fmt)


def unpack(codes, scales, fmt, d_k):
    """Inverse of ``pack``: -> fp32 [BH, d_k, d_v] (fold.py:150-152)."""
    return unpack_vk(codes, scales, fmt, d_k).transpose(1, 2).contiguous()


def _flat(S):
    return S.float().reshape(-1, S.shape[-2], S.shape[-1]).contiguous()


def _require_kernel(family, st):
    """Fail at construction, with the reason, when no HIP kernel exists for a layout."""
    if not _hip.supported(family, st):
        what = 'an unquantized state' if st.fmt is None else \
            f'int{st.bits} {"key" if st.axk else "value"}-axis group {st.group}'
        raise NotImplementedError(
            f'no HIP kernel instance for {family}: {what}, d_k {st.DK}, d_v {st.DV}, '
            f'm {st.m}, buffer_bits {st.buffer_bits} (see statequant_amd/csrc/build.py: CASES)')


# ---------------------------------------------------------------------------------------------------------------
# lockstep state
# ---------------------------------------------------------------------------------------------------------------
from ._lockstep import LockstepState  # noqa: E402


class PackedGDNState(LockstepState):
    """One layer's packed recurrent state and decode buffer for B sequences stepped in lockstep (fold.py:280-424).

    S            [BH, d_k, d_v] (or [B, H, d_k, d_v]) float state to start from
    fmt          ``Quantizer(4 or 8, 'k', group)``; scales are stored fp16
    m            buffer length (power of two); the state is folded and re-rounded every m steps
    hv, hk       value / key heads per sequence (hv % hk == 0); BH = B * hv
    buffer_bits  8 (int8 + one fp16 absmax scale per vector) or 16 (bf16)
    out_dtype    dtype of the output
    The remaining keyword arguments of the reference (block sizes, warps, ``fused``) are accepted and ignored.

    ``step(q, k, v, g, beta, scale)``: q, k raw [BH, d_k] or per key head [B * hk, d_k]; v [BH, d_v]; g (log decay)
    and beta [BH].  Returns the output buffer [BH, d_v] (the same tensor every step).  Every tensor is allocated
    once and updated in place, and the step is one kernel launch on the current stream, so it can be graph-captured.
    """

    def __init__(self, S, fmt, m=8, hv=None, hk=None, buffer_bits=8, out_dtype=torch.bfloat16,
                 block_v=None, warps=None, fused=None, fused_warps=None):
        from ._lockstep import describe_format, power_of_two
        key_major = _flat(S)                                                     # [B * H, d_k, d_v]
        _hip.require_gpu(key_major, 'PackedGDNState')
        rows, dk, dv = key_major.shape
        heads = hv if hv else rows
        key_heads = hk if hk else heads
        if heads % key_heads or rows % heads:
            raise AssertionError(f'{rows} state rows, {heads} value heads, {key_heads} key heads do not divide')
        if not power_of_two(m):
            raise AssertionError('m must be a power of two')
        if buffer_bits not in (8, 16):
            raise AssertionError(f'buffer_bits {buffer_bits}: 8 (int8) or 16 (bf16)')
        self.fmt = packed_format(fmt)
        self.bits = _bits(self.fmt)
        check_dims(self.fmt, dk, dv)
        self.axk, self.group = describe_format(self.fmt, self.bits, default_group=32)
        self.BH, self.B, self.HV, self.HK, self.gqa = rows, rows // heads, heads, key_heads, heads // key_heads
        self.DK, self.DV, self.m = dk, dv, m
        self.buffer_bits, self.qbuf, self.fused = buffer_bits, buffer_bits == 8, True
        _require_kernel('gdn', self)
        self._allocate(*pack(key_major, self.fmt), decay_shape=(), out_shape=(rows, dv), out_dtype=out_dtype)
        self._T = self.T

    @torch.no_grad()
    def load(self, S):
        """Replace the state in place and empty the buffer."""
        self._reset(*pack(_flat(S), self.fmt))

    def dequantize(self):
        """The stored state S_0 (without the buffered tokens) as fp32 [BH, d_k, d_v]."""
        return unpack(self.codes, self.scales, self.fmt, self.DK)

    def step(self, q, k, v, g, beta, scale):
        BH, HV, HK = self.BH, self.HV, self.HK
        per_key = q.shape[0] != BH
        if per_key:
            assert q.shape[0] == self.B * HK and k.shape[0] == self.B * HK
        for t in (q, k, v, g, beta):
            assert t.is_contiguous()
        _hip.same_device('PackedGDNState.step', self.O, q=q, k=k, v=v, g=g, beta=beta)
        sqk = (HK if per_key else HV) * self.DK
        a = _hip.SqGdnArgs(
            st=_hip.make_state(self._T, self._strides, HV), lay=self._lay, rows=self.B, idx=None,
            q=q.data_ptr(), s_q=sqk, q_dtype=_hip.dtype_code(q), k=k.data_ptr(), s_k=sqk, k_dtype=_hip.dtype_code(k),
            v=v.data_ptr(), s_v=HV * self.DV, v_dtype=_hip.dtype_code(v), qk_per_key_head=int(per_key), gate=0,
            g=g.data_ptr(), s_g=HV, g_dtype=_hip.dtype_code(g),
            beta=beta.data_ptr(), s_beta=HV, beta_dtype=_hip.dtype_code(beta),
            out=self.O.data_ptr(), out_dtype=_hip.dtype_code(self.O), scale=float(scale))
        _hip.check(_hip.lib().sq_gdn_step(ctypes.byref(a), _hip.current_stream(self.O.device)))
        return self.O
