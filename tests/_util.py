"""Shared helpers of the GPU parity tests: seeded inputs in the distributions the benchmark configs name, and the
kernel <-> oracle hand-over used for per-step comparison.

Protocol (the reference's own, /root/reference/tests/test_kernels.py:83-110): the HIP kernel and the CPU oracle take
the same token; outputs are compared; the entries the kernel appended to its buffer are compared with the oracle's
and then ADOPTED by the oracle, and after a fold the kernel's codes and scales likewise, so a rounding flip is counted
once and never inherited by later steps.
"""
import torch

import statequant_amd as sq


def quantizer(fmt):
    """(bits, axis, group) -> Quantizer; 'bf16' / 'fp32' (the unquantized state controls) pass through."""
    return fmt if isinstance(fmt, str) else sq.Quantizer(*fmt)


def gdn_token(gen, B, HV, HK, DK, DV, dtype=torch.float32, v_scale=None):
    """q, k ~ N(0,1) per KEY head; v ~ N(0,1); beta = sigmoid(N(0,1)); g = -softplus(N(0,1)) (CPU tensors)."""
    r = lambda *s: torch.randn(*s, generator=gen)          # noqa: E731
    q, k, v = r(B, HK, DK), r(B, HK, DK), r(B, HV, DV)
    if v_scale is not None:
        v = v * v_scale[None, :, None]
    g = -torch.nn.functional.softplus(r(B, HV))
    beta = torch.sigmoid(r(B, HV))
    return q.to(dtype), k.to(dtype), v.to(dtype), g, beta


def buffer_entry(T, slot, qbuf):
    """Dequantized (K, U) of buffer slot ``slot`` from a kernel state's tensors (dict with KB, UB, KBS, UBS)."""
    kb, ub = T['KB'][:, slot].float(), T['UB'][:, slot].float()
    if qbuf:
        kb, ub = kb * T['KBS'][:, slot, None].float(), ub * T['UBS'][:, slot, None].float()
    return kb.cpu(), ub.cpu()


class Tally:
    """Running comparison figures of one kernel-vs-oracle run."""

    def __init__(self):
        self.worst_o = 0.0
        self.buf_flips = self.buf_entries = self.buf_scale_events = 0
        self.code_mism = self.code_n = self.scale_mism = 0
        self.code_far = 0                     # codes differing by more than one step
        self.worst_raw = 0.0
        self.worst_deq = 0.0
        self.folds = 0

    def out(self, o, ref, floor=1e-30):
        """Largest |o - ref| of the step relative to the largest |ref| -- or to ``floor``, the size the outputs
        have by construction, where a step's outputs happen to be much smaller than that (an empty state and a k
        nearly orthogonal to q leave o = (k.q) u with k.q the cancelled sum of d_k products: an absolute error of
        1e-9 is then 1e-4 of an output of 1e-5)."""
        self.worst_o = max(self.worst_o, ((o - ref).abs().max() / ref.abs().max().clamp_min(floor)).item())

    def entries(self, got, want):
        """Buffered vectors [..., d] as stored (dequantized).  A vector whose fp16 scale landed on the other side of a
        rounding boundary (its absmax differs in the last fp32 bit) has most of its entries differ, each by less than
        one code step; such a vector is counted once, as a scale event, not as d flipped entries."""
        diff = got != want
        per_vec = diff.sum(-1)
        step = want.abs().amax(-1) / 127.0 * 1.01 + 1e-30
        rescaled = (per_vec > 0.2 * want.shape[-1]) & ((got - want).abs().amax(-1) <= step)
        self.buf_scale_events += int(rescaled.sum())
        self.buf_flips += int(per_vec[~rescaled].sum())
        self.buf_entries += want.numel()

    def fold(self, codes, scales, ref, bits):
        """codes / scales of the kernel (CPU copies) vs the oracle that has just folded the same buffer."""
        self.folds += 1
        mism, far, n = code_diff(codes, ref.codes, bits)
        self.code_mism += mism
        self.code_far += far
        self.code_n += n
        self.scale_mism += (scales != ref.scales).sum().item()
        from oracle.formats import unpack_vk
        deq = unpack_vk(codes, scales, ref.fmt, ref.DK)
        den = ref.S_raw.abs().max().clamp_min(1e-30)
        self.worst_raw = max(self.worst_raw, ((deq - ref.S_raw).abs().max() / den).item())
        self.worst_deq = max(self.worst_deq, ((deq - ref.S0).abs().max() / den).item())

    def report(self, tag):
        return (f'[{tag}] max rel |o - o_oracle| {self.worst_o:.2e}; {self.folds} folds: codes differing '
                f'{self.code_mism} of {self.code_n} ({100 * self.code_mism / max(self.code_n, 1):.5f}%), by more than '
                f'1 LSB {self.code_far}, scales differing {self.scale_mism}; max rel |S - S_raw_oracle| '
                f'{self.worst_raw:.2e}; buffer entries flipped {self.buf_flips} of {self.buf_entries}, vectors with the scale one '
                f'fp16 step off {self.buf_scale_events}')


def code_diff(got, want, bits):
    """(codes differing, differing by more than one step, codes compared) of two stored states."""
    d = (unpack_nib(got, bits).int() - unpack_nib(want, bits).int()).abs()
    if bits == 16:          # bf16 numbers: "one step" is relative, and across zero it is an absolute matter
        fa, fb = got.float(), want.float()
        tol = torch.maximum(fa.abs(), fb.abs()) * 2.0 ** -7 + 1e-6 * fb.abs().max()
        far = ((fa - fb).abs() > tol).sum().item()
    else:
        far = (d > 1).sum().item()
    return (d != 0).sum().item(), far, d.numel()


def unpack_nib(codes, bits):
    """Stored codes -> one integer per code (int4 bytes split into their two nibbles).  A bf16 state (bits 16): an
    integer that orders like the value, so that neighbouring bf16 numbers differ by one."""
    if bits == 8:
        return codes.to(torch.int16)
    if bits == 16:
        raw = codes.view(torch.int16).int()
        return torch.where(raw < 0, -(raw & 0x7FFF), raw)
    c = codes.to(torch.int16)
    return torch.stack(((c & 15) - 8, ((c >> 4) & 15) - 8), -1).flatten(-2)


class SlotSync:
    """The re-sync protocol for a subset of the slots of a slot-addressed state: after every step the oracle's newest
    buffer entry is compared with the slots' and replaced by it, after every fold the oracle's codes and scales
    likewise, so that one rounding flip is counted once.  ``ref`` is an oracle over the slots ``sl`` (in that order,
    built with ``auto_fold=False``); ``views`` the typed views of the blob."""

    def __init__(self, views, sl, ref, bits, qbuf=True, exact_decay=True):
        """exact_decay=False (Mamba2): the log decay is A x softplus(dt + bias) formed in the kernel, whose logf / expf
        differ from torch's in the last bit, so the cumulative decays are compared to 5e-6 and taken over as well."""
        self.V, self.sl, self.ref, self.bits, self.qbuf = views, sl.long(), ref, bits, qbuf
        self.exact_decay = exact_decay
        self.tal = Tally()

    def _entry(self, i):
        V, sl = self.V, self.sl
        kb, ub = V['KB'][sl][:, :, i].float(), V['UB'][sl][:, :, i].float()
        if self.qbuf:
            kb, ub = kb * V['KBS'][sl][:, :, i, None].float(), ub * V['UBS'][sl][:, :, i, None].float()
        return kb.flatten(0, 1).cpu(), ub.flatten(0, 1).cpu()

    def after_step(self, got, want, i):
        """``got`` / ``want``: the outputs of the subset's rows; ``i``: the buffer index this step appended at."""
        ref, V, sl = self.ref, self.V, self.sl
        self.tal.out(got, want)
        kb, ub = self._entry(i)
        self.tal.entries(kb, ref.K[:, i])
        self.tal.entries(ub, ref.U[:, i])
        gb = V['GB'][sl][:, :, i].flatten(0, 1).cpu()
        if self.exact_decay:
            assert torch.equal(gb, ref.G[:, i]), 'cumulative decays must be bit-equal'
        else:
            assert torch.allclose(gb, ref.G[:, i], rtol=5e-6, atol=1e-7)
            ref.G[:, i] = gb
            ref.gcur = gb.clone()                          # (the fold below, if due, resets it)
        ref.K[:, i], ref.U[:, i] = kb, ub
        if ref.n == ref.m:
            ref.fold()
            codes = V['S'][sl].cpu().reshape(ref.codes.shape)
            scales = V['SC'][sl].cpu().reshape(ref.scales.shape)
            self.tal.fold(codes, scales, ref, self.bits)
            ref.adopt(codes, scales)
        n = V['NPTR'][sl][:, 0].cpu()
        assert (n == ref.n).all(), (n, ref.n)

    def verdict(self, tag, o_bound=2e-5):
        """The small tests' bounds: outputs 2e-5, codes at most 1e-4 off and never by more than one step."""
        t = self.tal
        print('\n' + t.report(tag))
        assert t.worst_o < o_bound, t.worst_o
        assert t.code_far == 0 and t.code_mism <= 1e-4 * max(t.code_n, 1), (t.code_mism, t.code_n)
        assert t.buf_flips <= 1e-3 * t.buf_entries, (t.buf_flips, t.buf_entries)
        assert t.folds >= 2
