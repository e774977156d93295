"""Slot-addressed packed GDN states: one fixed-size byte blob per sequence slot, on HIP kernels.

Mirrors the reference's ``statequant/kernels/slots.py`` (``/root/reference/src/statequant/kernels/slots.py``).  A
serving engine keeps every running sequence's recurrent state in a slot of a preallocated cache and hands each step a
table of slot indices; ``SlotLayout`` defines the per-slot blob of one layer, runs the decode step on a batch of slots
(``sq_gdn_step`` with slot indirection), and provides the read (dequantize + apply the pending buffer) and write
(quantize, empty the buffer) used around prefill.

Per-slot blob (slots.py:9-22), every field offset rounded up to 16 bytes, in this order:

    GB    fp32  [HV, m]            cumulative log decay of each buffered token
    GCUR  fp32  [HV]               running log decay since the last fold
    NPTR  int32 [max(HV, 4)]       buffer fill counter n, one copy per value head (all equal between steps)
    SC    fp16  scales             axis 'k': [HV, d_v, ceil(d_k/g)]; axis 'v': [HV, d_v/g, d_k]; float state: absent
    KBS   fp16  [HK, m]            buffered key scales (int8 buffer only)
    UBS   fp16  [HV, m]            buffered delta-value scales (int8 buffer only)
    S     codes                    int4: uint8 [HV, d_v, d_k/2]; int8: int8 [HV, d_v, d_k]; float: [HV, d_v, d_k]
    KB    int8 / bf16 [HK, m, d_k] buffered normalised keys, per KEY head
    UB    int8 / bf16 [HV, m, d_v] buffered delta values

Slot index 0 and negative indices are padding rows for the step: nothing is read or written there and the output row
is zeroed.
"""
from __future__ import annotations

import ctypes
import math

import torch

from . import _hip
from .fold import _bits, _require_kernel, check_dims, pack_vk, packed_format, pow2, unpack_vk

_ALIGN = 16


def field_table(fields):
    """[(name, dtype, shape)] -> ({name: (offset, dtype, shape, nbytes)}, total bytes), offsets 16-byte aligned."""
    table, off = {}, 0
    for name, dt, shape in fields:
        nb = math.prod(shape) * torch.empty((), dtype=dt).element_size()
        table[name] = (off, dt, tuple(shape), nb)
        off += -(-nb // _ALIGN) * _ALIGN
    return table, off


def state_fields(fmt, bits, axk, group, hv, hk, dk, dv, m, qbuf, gb_shape, gcur_shape, state_dtype=torch.bfloat16,
                 ragged=True):
    """The field list shared by the three families; only the decay shapes differ (KDA keeps them per channel)."""
    bdt = torch.int8 if qbuf else torch.bfloat16
    fields = [('GB', torch.float32, gb_shape), ('GCUR', torch.float32, gcur_shape),
              ('NPTR', torch.int32, (max(hv, 4),))]
    if fmt is not None:
        ng = -(-dk // group) if ragged else dk // group
        fields.append(('SC', torch.float16, (hv, dv, ng) if axk else (hv, dv // group, dk)))
    if qbuf:
        fields += [('KBS', torch.float16, (hk, m)), ('UBS', torch.float16, (hv, m))]
    if fmt is None:
        fields.append(('S', state_dtype, (hv, dv, dk)))
    elif bits == 4:
        fields.append(('S', torch.uint8, (hv, dv, dk // 2)))
    else:
        fields.append(('S', torch.int8, (hv, dv, dk)))
    fields += [('KB', bdt, (hk, m, dk)), ('UB', bdt, (hv, m, dv))]
    return fields


def slot_state(views):
    """(tensor dict, per-sequence strides, counter stride) of a ``views`` dict, as the C ABI wants them."""
    V = views
    gb = V['GB']
    T = dict(S=V['S'], SC=V.get('SC', gb), KB=V['KB'], KBS=V.get('KBS', gb), UB=V['UB'], UBS=V.get('UBS', gb),
             GB=gb, GCUR=V['GCUR'], NPTR=V['NPTR'])
    st = lambda n: V[n].stride(0) if n in V else 0     # noqa: E731
    strides = (st('S'), st('SC'), st('KB'), st('KBS'), st('UB'), st('UBS'), st('GB'), st('GCUR'))
    return T, strides, st('NPTR')


class SlotLayout:
    """The packed per-slot layout of one GDN layer and the operations on a batch of slots (slots.py:40-121).

    fmt          ``Quantizer(4 or 8, 'k' or 'v', group)``, 'bf16' or 'fp32' (an unpacked float state)
    hv, hk       value / key heads of the layer; hv % hk == 0
    dk, dv       head dims
    m            buffer length (power of two)
    buffer_bits  8 (int8 + fp16 scale per vector) or 16 (bf16)
    fused        accepted for call compatibility; the HIP step is always one launch

    Every format has its byte layout, ``views``, ``read`` and ``write``; the decode ``step`` exists for the
    key-axis int4 / int8 formats.
    """

    def __init__(self, fmt, hv, hk, dk, dv, m=8, buffer_bits=8, fused=None):
        self.fused = fused
        self.state_dtype = torch.float32 if fmt == 'fp32' else torch.bfloat16
        fmt = 'bf16' if fmt == 'fp32' else fmt
        self.fmt = packed_format(fmt)
        self.bits = _bits(self.fmt)
        self.HV, self.HK, self.DK, self.DV, self.m = hv, hk, dk, dv, m
        assert hv % hk == 0
        self.gqa = hv // hk
        assert m >= 1 and m & (m - 1) == 0, 'm must be a power of two'
        check_dims(self.fmt, dk, dv)
        self.DKP, self.DVP = pow2(dk), pow2(dv)
        assert buffer_bits in (8, 16)
        self.buffer_bits, self.qbuf = buffer_bits, buffer_bits == 8
        self.axk = self.fmt is not None and self.fmt.axis == 'k'
        self.group = self.fmt.group if self.fmt is not None else 32
        self.fields, self.nbytes = field_table(state_fields(
            self.fmt, self.bits, self.axk, self.group, hv, hk, dk, dv, m, self.qbuf, (hv, m), (hv,),
            self.state_dtype))
        self._lay = None

    _family = 'gdn'

    def __repr__(self):
        f = ('bf16' if self.state_dtype == torch.bfloat16 else 'fp32') if self.fmt is None else \
            f'int{self.bits}-{self.fmt.axis}-g{self.group}'
        return (f'SlotLayout({f}, hv={self.HV}, hk={self.HK}, dk={self.DK}, dv={self.DV}, m={self.m}, '
                f'buffer_bits={self.buffer_bits}, {self.nbytes} B/slot)')

    def breakdown(self):
        """Bytes per slot by field (before alignment padding)."""
        return {n: f[3] for n, f in self.fields.items()}

    def _layout_struct(self):
        if self._lay is None:
            _require_kernel(self._family, self)
            self._lay = _hip.make_layout(self)
        return self._lay

    # -- views ------------------------------------------------------------------------------------------------
    def views(self, blob):
        """uint8 [num_slots, >= nbytes] (inner stride 1, slot stride and base 16-byte aligned) ->
        {field: typed view [num_slots, *shape]} (slots.py:108-117)."""
        assert blob.dtype == torch.uint8 and blob.dim() == 2 and blob.shape[1] >= self.nbytes, blob.shape
        assert blob.stride(1) == 1 and blob.stride(0) % _ALIGN == 0 and blob.data_ptr() % _ALIGN == 0
        n = blob.shape[0]
        return {name: blob[:, off:off + nb].view(dt).view(n, *shape)
                for name, (off, dt, shape, nb) in self.fields.items()}

    def alloc(self, num_slots, device='cuda'):
        """A standalone zeroed blob [num_slots, nbytes] uint8."""
        return torch.zeros(num_slots, self.nbytes, dtype=torch.uint8, device=device)

    # -- decode -----------------------------------------------------------------------------------------------
    def fold_order(self, views, idx, out=None):
        """A dispatch order for ``step(..., order=)`` (int32 [B] on the device; not in the reference): the rows whose
        buffer fills on the coming step spread evenly over the launch, the others in batch order.  For batches whose
        sequences are at different points of their fold period (a serving engine's): a folding row keeps its
        workgroups longer, and left where the batch order has them such rows end a launch late.  One small launch,
        no host synchronization; with ``out`` given no allocation either.  The counters of all layers of a model
        move together, so one list per decode step serves every layer."""
        assert idx.dtype == torch.int32 and idx.is_contiguous()
        return _hip.fold_order(views['NPTR'], slot_state(views)[2], self.m, idx, out)

    def step(self, views, idx, q, k, v, out, scale, *, g=None, beta=None, gate=None, fused='layout', order=None):
        """One decode token for every batch row b, on slot ``idx[b]`` (int32 [B]; <= 0 = padding row)
        (slots.py:124-187).

        q, k    [B, hk, d_k] per key head, raw (l2-normalised in the kernel); any row stride, unit inner stride
        v       [B, hv, d_v]
        out     [B, hv, d_v] contiguous; written (zeros on padding rows)
        g, beta [B, hv] log decay and (sigmoided) beta;  or ``gate=(a, b, A_log, dt_bias)``: formed in the kernel as
                g = -exp(A_log) softplus(a + dt_bias), beta = sigmoid(b)
        order   optional int32 [B] dispatch order (``fold_order``; not in the reference): which batch row each position
                of the launch works on.  Results do not depend on it
        One kernel launch on the current stream, no allocation, no host synchronization: graph-capturable.  Each
        row's buffer counter advances; rows whose buffer fills are folded and re-rounded in place.
        """
        B = idx.shape[0]
        if B == 0:
            return out
        HV, HK, DK, DV = self.HV, self.HK, self.DK, self.DV
        assert q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1
        assert q.stride(-2) == DK and k.stride(-2) == DK and v.stride(-2) == DV
        assert out.is_contiguous() and out.shape[0] >= B
        assert idx.dtype == torch.int32 and idx.is_contiguous()
        ga, gb, A_log, dt_bias = gate if gate is not None else (None,) * 4
        _hip.same_device('SlotLayout.step', views['S'], idx=idx, q=q, k=k, v=v, out=out, g=g, beta=beta, a=ga, b=gb,
                         A_log=A_log, dt_bias=dt_bias)
        lay = self._layout_struct()
        T, strides, sN = slot_state(views)
        a = _hip.SqGdnArgs(
            st=_hip.make_state(T, strides, sN), lay=lay, rows=B, idx=idx.data_ptr(),
            q=q.data_ptr(), s_q=q.stride(0), q_dtype=_hip.dtype_code(q),
            k=k.data_ptr(), s_k=k.stride(0), k_dtype=_hip.dtype_code(k),
            v=v.data_ptr(), s_v=v.stride(0), v_dtype=_hip.dtype_code(v), qk_per_key_head=1,
            out=out.data_ptr(), out_dtype=_hip.dtype_code(out), scale=float(scale),
            order=_hip.check_order(order, B, views['S']))
        if gate is not None:
            assert ga.stride(-1) == 1 and gb.stride(-1) == 1 and A_log.is_contiguous() and dt_bias.is_contiguous()
            a.gate = 1
            a.a, a.s_a, a.a_dtype = ga.data_ptr(), ga.stride(0), _hip.dtype_code(ga)
            a.b, a.s_b, a.b_dtype = gb.data_ptr(), gb.stride(0), _hip.dtype_code(gb)
            a.A_log, a.A_log_dtype = A_log.data_ptr(), _hip.dtype_code(A_log)
            a.dt_bias, a.dt_bias_dtype = dt_bias.data_ptr(), _hip.dtype_code(dt_bias)
        else:
            assert g.stride(-1) == 1 and beta.stride(-1) == 1
            a.gate = 0
            a.g, a.s_g, a.g_dtype = g.data_ptr(), g.stride(0), _hip.dtype_code(g)
            a.beta, a.s_beta, a.beta_dtype = beta.data_ptr(), beta.stride(0), _hip.dtype_code(beta)
        _hip.check(_hip.lib().sq_gdn_step(ctypes.byref(a), _hip.current_stream(out.device)))
        return out

    # -- prefill side: HIP kernels for blobs on the GPU, the reference's torch formulation for CPU blobs ----------
    def _buffer(self, views, idx):
        """Dequantized buffer of slots idx: keys [P, HK, m, DK], values [P, HV, m, DV], fill counts [P]."""
        V = views
        Kb, Ub = V['KB'][idx].float(), V['UB'][idx].float()
        if self.qbuf:
            Kb = Kb * V['KBS'][idx].float().unsqueeze(-1)
            Ub = Ub * V['UBS'][idx].float().unsqueeze(-1)
        n = V['NPTR'][idx, 0] & (self.m - 1)
        return Kb, Ub, n

    def _stored(self, views, idx):
        P = idx.shape[0]
        V = views
        codes = V['S'][idx].reshape(P * self.HV, *V['S'].shape[2:])
        sc = V['SC'][idx].reshape(P * self.HV, *V['SC'].shape[2:]) if 'SC' in V else None
        return unpack_vk(codes, sc, self.fmt, self.DK).view(P, self.HV, self.DV, self.DK)

    def _hip_format(self, views):
        """States on the GPU go through the HIP pack / read kernels and nothing else (a layout the library has no
        instance for raises, as in ``step``); the torch formulation below is for CPU tensors only."""
        return views['S'].is_cuda

    def _read_hip(self, views, idx, kda):
        """``sq_read`` for a blob on the GPU (``idx`` may live anywhere, as in the reference's indexing; rows with
        ``idx <= 0`` are padding and come back as zeros), None for a CPU blob."""
        if not self._hip_format(views) or idx.shape[0] == 0:
            return None
        dev = views['S'].device
        P = idx.shape[0]
        out = torch.empty(P, self.HV, self.DV, self.DK, device=dev, dtype=torch.float32)
        T, strides, sN = slot_state(views)
        _hip.read_state(_hip.make_layout(self), T, strides, sN, idx.to(device=dev, dtype=torch.int32).contiguous(),
                        out, kda)
        return out

    @torch.no_grad()
    def read(self, views, idx):
        """The current state of slots ``idx`` as fp32 [P, HV, d_v, d_k]: the stored state advanced across its
        pending buffer, S_n = a_n S_0 + sum_{i<n} (a_n/a_i) u_i k_i^T (slots.py:210-233).  Entries of dead buffer
        slots are discarded with ``where`` (they may hold anything)."""
        out = self._read_hip(views, idx, kda=False)
        if out is not None:
            return out
        idx = idx.long()
        m = self.m
        S0 = self._stored(views, idx)
        Kb, Ub, n = self._buffer(views, idx)
        gcur = views['GCUR'][idx]                                                     # [P, HV]
        live = (torch.arange(m, device=idx.device)[None, :] < n[:, None])[:, None, :]      # [P, 1, m]
        zero = torch.zeros((), device=idx.device)
        dec = torch.where(live, torch.exp(gcur[..., None] - torch.where(live, views['GB'][idx], zero)), zero)
        Ub = torch.where(live[..., None], Ub, zero)
        Kb = torch.where(live.expand(-1, self.HK, -1)[..., None], Kb, zero)
        Kx = Kb.repeat_interleave(self.gqa, dim=1)                                    # [P, HV, m, DK]
        return torch.exp(gcur)[..., None, None] * S0 + torch.einsum('phmv,phmk->phvk', Ub * dec[..., None], Kx)

    @torch.no_grad()
    def write(self, views, idx, S):
        """Store states S [P, HV, d_v, d_k] (value-major) packed into slots ``idx`` and empty their buffers
        (n = 0, running decay 0) (slots.py:236-252).  On the GPU rows with ``idx <= 0`` are padding and store nothing
        (slot 0 is the engine's null slot); the CPU formulation indexes like the reference."""
        P = idx.shape[0]
        V = views
        if self._hip_format(views):
            if P == 0:
                return
            dev = V['S'].device
            src = S.reshape(P, self.HV, self.DV, self.DK).to(device=dev, dtype=torch.float32).contiguous()
            gc = V['GCUR']
            sc = V.get('SC')
            _hip.pack_into(_hip.make_layout(self), src, V['S'], V['S'].stride(0), sc,
                           sc.stride(0) if sc is not None else 0,
                           idx=idx.to(device=dev, dtype=torch.int32).contiguous(), GCUR=gc, sGC=gc.stride(0),
                           gcur_per_head=gc[0].numel() // self.HV, NPTR=V['NPTR'], sN=V['NPTR'].stride(0))
            return
        idx = idx.long()
        if self.fmt is None and self.state_dtype == torch.float32:
            V['S'][idx] = S.reshape(P, *V['S'].shape[1:]).float()
        else:
            codes, sc = pack_vk(S.reshape(P * self.HV, self.DV, self.DK), self.fmt)
            V['S'][idx] = codes.view(P, *V['S'].shape[1:])
            if 'SC' in V:
                V['SC'][idx] = sc.view(P, *V['SC'].shape[1:])
        V['NPTR'][idx] = 0
        V['GCUR'][idx] = 0.

    def stored(self, views, idx):
        """(codes, scales) of slots ``idx`` (for tests)."""
        idx = idx.long()
        return views['S'][idx], (views['SC'][idx] if 'SC' in views else None)
