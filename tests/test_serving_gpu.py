"""A serving engine's decode loop on the slot ops, the way the reference's vLLM plugin drives them
(/root/reference/src/statequant/integrations/vllm_plugin.py:386-430 there): a fixed-size padded batch whose rows point
at slots (padding rows at the null slot 0), q / k / v as views into one fused projection buffer (row stride = its full
width), the gate computed in the kernel from a, b, A_log, dt_bias, sequences that join and leave between steps, a
freed slot taken over by a new sequence (``write`` must empty the stale buffer), and a chunked-prefill continuation
(``read`` the state with its pending buffer, advance it outside, ``write`` it back).

Every sequence has its own CPU oracle; outputs are compared row by row.  After a fold the oracle adopts the slot's
codes (the reference's re-sync protocol), so a rounding tie is counted once.
"""
import pytest
import torch

import statequant_amd as sq
from oracle import states as ST
from statequant_amd.kernels import SlotLayout
from tests._util import unpack_nib

pytestmark = pytest.mark.gpu
DEV = 'cuda'
HV, HK, D, M = 4, 2, 64, 4
BATCH = 4                                                # the engine's padded decode batch


class Seq:
    """One sequence: its slot, its oracle, and how many tokens it still decodes."""

    def __init__(self, name, fmt, S0, left):
        self.name, self.left, self.slot = name, left, None
        self.ora = ST.GDNOracle(S0.reshape(HV, D, D), fmt, m=M, hv=HV, hk=HK, buffer_bits=8)


def prefill(gen, tokens, A_log, dt_bias, S=None):
    """A prompt (or a prompt chunk) through the textbook recurrence, from S (value-major [HV, d_v, d_k]) or zero."""
    S = torch.zeros(HV, D, D) if S is None else S.clone()
    for _ in range(tokens):
        q, k, v = torch.randn(HK, D, generator=gen), torch.randn(HK, D, generator=gen), torch.randn(HV, D, generator=gen)
        a, b = torch.randn(1, HV, generator=gen) * 0.5 - 1, torch.randn(1, HV, generator=gen)
        g, beta = ST.gdn_gate(a, b, A_log, dt_bias)
        ST.gdn_recurrence(S, q.repeat_interleave(HV // HK, 0), k.repeat_interleave(HV // HK, 0), v, g[0], beta[0], D ** -0.5)
    return S


@pytest.mark.parametrize('fmt', [(4, 'k', 64), (8, 'k', 32)])
def test_decode_loop_with_joins_leaves_and_chunked_prefill(fmt):
    gen = torch.Generator().manual_seed(17)
    lay = SlotLayout(sq.Quantizer(*fmt), HV, HK, D, D, m=M, buffer_bits=8)
    blob = lay.alloc(4, DEV)                               # slot 0 = the engine's null slot, 3 real slots
    views = lay.views(blob)
    A_log, dt_bias = torch.randn(HV, generator=gen) * 0.3, torch.randn(HV, generator=gen) * 0.3
    free, active, worst = [3, 2, 1], [], 0.0
    null_before = blob[0].clone()

    def admit(name, prompt, left):
        S = prefill(gen, prompt, A_log, dt_bias)
        s = Seq(name, fmt, S, left)
        s.slot = free.pop()
        lay.write(views, torch.tensor([s.slot], device=DEV), S[None].to(DEV))
        active.append(s)

    arrivals = {0: [('A', 5, 11), ('B', 3, 40)], 5: [('C', 9, 40)], 13: [('D', 2, 40)]}
    kd, width = HK * D, 2 * HK * D + HV * D
    for t in range(30):
        for name, prompt, left in arrivals.get(t, []):
            admit(name, prompt, left)
        if t == 18:                                        # chunked prefill: B's next prompt chunk arrives
            b_ = next(s for s in active if s.name == 'B')
            got = lay.read(views, torch.tensor([b_.slot], device=DEV)).cpu()[0]
            want = b_.ora.state().reshape(HV, D, D)
            assert ((got - want).abs().max() / want.abs().max()).item() < 1e-5
            S = prefill(gen, 3, A_log, dt_bias, S=got)
            lay.write(views, torch.tensor([b_.slot], device=DEV), S[None].to(DEV))
            b_.ora.load(S)
        # one decode step of the padded batch, rows in arrival order shuffled
        order = torch.randperm(len(active), generator=gen).tolist()
        rows = [active[i] for i in order]
        idx = torch.tensor([s.slot for s in rows] + [0] * (BATCH - len(rows)), dtype=torch.int32)
        x = torch.randn(BATCH, width, generator=gen)       # the fused projection output; padding rows hold junk too
        a, b = torch.randn(BATCH, HV, generator=gen) * 0.5 - 1, torch.randn(BATCH, HV, generator=gen)
        xd = x.to(DEV)
        q = xd[:, :kd].unflatten(1, (HK, D))
        k = xd[:, kd:2 * kd].unflatten(1, (HK, D))
        v = xd[:, 2 * kd:].unflatten(1, (HV, D))
        assert q.stride(0) == width and not q.is_contiguous()
        out = torch.full((BATCH, HV, D), 7.0, device=DEV)
        lay.step(views, idx.to(DEV), q, k, v, out, D ** -0.5, gate=(a.to(DEV), b.to(DEV), A_log.to(DEV), dt_bias.to(DEV)))
        out = out.cpu()
        g, beta = ST.gdn_gate(a, b, A_log, dt_bias)
        for r, s in enumerate(rows):
            want = s.ora.step(x[r, :kd].view(HK, D), x[r, kd:2 * kd].view(HK, D), x[r, 2 * kd:].view(HV, D), g[r], beta[r],
                              D ** -0.5)
            worst = max(worst, ((out[r] - want).abs().max() / want.abs().max()).item())
            n_slot = int(views['NPTR'][s.slot, 0])
            assert n_slot == s.ora.n, (t, s.name)
            if n_slot == 0:                                # folded on this step: adopt the slot's codes
                codes, scales = views['S'][s.slot].cpu(), views['SC'][s.slot].cpu()
                ref_codes = s.ora.codes.view(HV, D, -1)
                assert (unpack_nib(codes, fmt[0]).int() - unpack_nib(ref_codes, fmt[0]).int()).abs().max() <= 1
                s.ora.adopt(codes.view_as(s.ora.codes), scales.view_as(s.ora.scales))
            s.left -= 1
        assert float(out[len(rows):].abs().max()) == 0.0 if len(rows) < BATCH else True
        for s in [s for s in active if s.left == 0]:       # finished: the slot goes back to the pool as it is
            active.remove(s)
            free.append(s.slot)
    assert worst < 1e-2, worst                             # the task's bound on o
    assert torch.equal(blob[0], null_before)               # the null slot was never written
    assert {s.name for s in active} == {'B', 'C', 'D'} and len(free) == 0
