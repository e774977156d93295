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


@pytest.mark.parametrize('m,bb', [(4, 8), (2, 16)])
def test_external_function_on_the_unpacked_state(m, bb):
    """The plugin's ``external:`` mode (/root/reference/src/statequant/integrations/vllm_plugin.py:400-410 there): the
    state stays unpacked fp32 in the slot (``SlotLayout('fp32')``) and, right after a step, a user function is applied
    through the views to the rows whose buffer just folded -- the fixed-shape form used under graphs (function on
    every row, kept where folded).  The next step must read what the function left.  The function here is continuous
    (clamp and scale), so a last-bit difference between kernel and oracle does not grow."""
    fn = lambda S: S.clamp(-0.8, 0.8) * 0.9                 # noqa: E731
    lay = SlotLayout('fp32', HV, HK, D, D, m=m, buffer_bits=bb)
    gen = torch.Generator().manual_seed(23)
    views = lay.views(lay.alloc(5, DEV))
    slots = torch.tensor([4, 0, 2], dtype=torch.int32)       # the middle row is padding (null slot)
    live = [0, 2]
    S0 = torch.randn(2, HV, D, D, generator=gen) * 0.5
    lay.write(views, slots[live].to(DEV), S0.to(DEV))
    ref = ST.GDNOracle(S0.reshape(-1, D, D), ST.IDENT, m=m, hv=HV, hk=HK, buffer_bits=bb)
    idx = slots.to(DEV)
    null_before = views['S'][0].clone()
    applied = 0
    for t in range(3 * m + 1):
        q, k, v = torch.randn(3, HK, D, generator=gen), torch.randn(3, HK, D, generator=gen), torch.randn(3, HV, D, generator=gen)
        g, beta = -torch.rand(3, HV, generator=gen) * 0.2, torch.rand(3, HV, generator=gen)
        out = torch.empty(3, HV, D, device=DEV)
        lay.step(views, idx, q.to(DEV), k.to(DEV), v.to(DEV), out, D ** -0.5, g=g.to(DEV), beta=beta.to(DEV))
        folded = (views['NPTR'][idx.long(), 0] == 0) & (idx > 0)
        S = views['S'][idx.long()]
        views['S'][idx.long()] = torch.where(folded[:, None, None, None], fn(S), S)
        want = ref.step(q[live].reshape(-1, D), k[live].reshape(-1, D), v[live].reshape(-1, D), g[live].reshape(-1),
                        beta[live].reshape(-1), D ** -0.5).view(2, HV, D)
        if ref.n == 0:
            ref.S0 = fn(ref.S0)
            applied += 1
            assert folded.cpu().tolist() == [True, False, True]
        else:
            assert not folded.any()
        got = out.cpu()[live]
        assert ((got - want).abs().max() / want.abs().max()).item() < 1e-4, t
        assert float(out[1].abs().max()) == 0.0
    assert applied == 3
    got = views['S'][slots[live].long().to(DEV)].cpu().reshape(-1, D, D)
    assert ((got - ref.S0).abs().max() / ref.S0.abs().max()).item() < 1e-4
    assert float(got.abs().max()) <= 0.8 * 0.9 * 1.5         # the clamp took hold (steps after the fold add little)
    assert torch.equal(views['S'][0], null_before)
