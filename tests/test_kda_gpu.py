"""KDA HIP step (through the C ABI) against the CPU oracle and the reference's golden vectors.

Mirrors the reference's tests/test_kda_kernels.py: decode vs the torch reference with per-step re-sync, slot step vs
lockstep, read() predicting the next output; plus the benchmark's non-power-of-two variant (d = 96, about 60 % of
the batch rows occupied), which the reference's Triton kernel refuses (kda.py:56 there) and which is therefore
pinned by the oracle alone and by its equivalence to the same problem zero-padded to d_k = 128.
"""
import pytest
import torch

from oracle import states as ST
from statequant_amd.kernels import KDASlotLayout, PackedKDAState, kda_recurrence
from tests._util import Tally, buffer_entry, quantizer, unpack_nib

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def kda_token(gen, B, H, DK, DV, dtype=torch.float32):
    """q, k, v ~ N(0,1); per-channel log decay g = -softplus(N(0,1)); beta = sigmoid(N(0,1))."""
    r = lambda *s: torch.randn(*s, generator=gen)          # noqa: E731
    return (r(B, H, DK).to(dtype), r(B, H, DK).to(dtype), r(B, H, DV).to(dtype),
            -torch.nn.functional.softplus(r(B, H, DK)), torch.sigmoid(r(B, H)))


def run_decode(fmt, m, bb, B=2, H=4, DK=128, DV=128, T=24, seed=1, dtype=torch.float32, shape_token=None, S0_scale=0.5):
    gen = torch.Generator().manual_seed(seed)
    S0 = torch.randn(B * H, DV, DK, generator=gen) * S0_scale
    ker = PackedKDAState(S0.to(DEV), quantizer(fmt), m=m, hv=H, buffer_bits=bb, out_dtype=torch.float32)
    ref = ST.KDAOracle(S0, fmt, m=m, hv=H, buffer_bits=bb, auto_fold=False)
    assert torch.equal(ker.codes.cpu(), ref.codes) and torch.equal(ker.scales.cpu(), ref.scales)
    tal = Tally()
    for t in range(T):
        q, k, v, g, beta = kda_token(gen, B, H, DK, DV, dtype)
        if shape_token is not None:
            shape_token(q, k, v, g, beta)
        slot = ker.n
        o = ker.step(q.to(DEV), k.to(DEV), v.to(DEV), g.to(DEV), beta.to(DEV)).cpu().reshape(B * H, DV)
        r = ref.step(q.reshape(B * H, DK), k.reshape(B * H, DK), v.reshape(B * H, DV), g.reshape(B * H, DK),
                     beta.reshape(-1))
        tal.out(o, r)
        kb, ub = buffer_entry(ker.T, slot, bb == 8)
        tal.entries(kb, ref.K[:, slot])
        tal.entries(ub, ref.U[:, slot])
        assert torch.equal(ker.GB[:, slot].cpu(), ref.G[:, slot]), t            # decay vectors: bit-equal
        ref.K[:, slot], ref.U[:, slot] = kb, ub
        if ref.n == m:
            ref.fold()
        assert ker.n == ref.n
        if ref.n == 0:
            assert torch.equal(ker.GCUR.cpu(), torch.zeros(B * H, DK))
            codes, scales = ker.codes.cpu(), ker.scales.cpu()
            tal.fold(codes, scales, ref, 16 if fmt == 'bf16' else fmt[0])
            ref.adopt(codes, scales)
        else:
            assert torch.equal(ker.GCUR.cpu(), ref.gcur)
        assert torch.equal(ker.NPTR.cpu(), torch.full((B, H), ref.n, dtype=torch.int32))
    return tal


def check(tal, tag, T, m):
    print('\n' + tal.report(tag))
    assert tal.folds == T // m
    assert tal.worst_o < 2e-5, tal.worst_o
    assert tal.buf_flips <= max(1, 1e-4 * tal.buf_entries), tal.buf_flips
    assert tal.code_mism <= max(1, 1e-4 * tal.code_n) and tal.code_far == 0, (tal.code_mism, tal.code_far)
    assert tal.worst_raw < 0.2


@pytest.mark.parametrize('fmt,m,bb', [((4, 'v', 32), 8, 8), ((8, 'v', 32), 4, 16), ((4, 'v', 32), 1, 8), ((8, 'v', 64), 8, 8),
                                      ((4, 'v', 64), 4, 16), ((8, 'v', 32), 16, 16), ((4, 'v', 16), 8, 8),
                                      ((8, 'v', 16), 4, 16), ((4, 'v', 16), 1, 8), ((8, 'v', 16), 16, 8)])
def test_value_axis_groups(fmt, m, bb):
    """Scale groups of 32 value rows per key column, with KDA's per-channel decay on the stored state."""
    T = 4 if m == 1 else 34 if m == 16 else 24
    check(run_decode(fmt, m, bb, T=T), f'kda {fmt} m={m} buf{bb}', T, m)


@pytest.mark.parametrize('m,bb', [(8, 8), (4, 16), (1, 8), (16, 16)])
@pytest.mark.parametrize('D', [128, 96, 64])
def test_unquantized_state_control(m, bb, D):
    """The bf16 state (kda.py:304: the control for the packed formats) through the same step; the fold multiplies the
    stored state by the per-channel decay and rounds once to bf16."""
    T = 3 * m + 2 if m > 1 else 4
    check(run_decode('bf16', m, bb, DK=D, DV=D, T=T), f'kda bf16 state d={D} m={m} buf{bb}', T, m)


@pytest.mark.parametrize('fmt', [(4, 'k', 32), (4, 'k', 64), (8, 'k', 32), (8, 'k', 128)])
@pytest.mark.parametrize('m,bb', [(8, 8), (4, 16), (1, 8), (16, 8)])
def test_decode_vs_oracle(fmt, m, bb):
    T = 32 if m == 16 else 24
    check(run_decode(fmt, m, bb, T=T), f'kda {fmt} m={m} buf{bb}', T, m)


@pytest.mark.parametrize('D,fmt', [(96, (4, 'k', 32)), (96, (8, 'k', 32)), (64, (4, 'k', 32)), (64, (8, 'k', 64))])
def test_non_pow2_and_small_heads(D, fmt):
    check(run_decode(fmt, 4, 8, B=2, H=5, DK=D, DV=D, T=12), f'kda d={D} {fmt}', 12, 4)
    check(run_decode(fmt, 16, 16, B=1, H=3, DK=D, DV=D, T=33), f'kda d={D} {fmt} m=16', 33, 16)


@pytest.mark.parametrize('fmt,m,bb', [((4, 'k', 32), 8, 8), ((8, 'k', 32), 4, 16), ((4, 'k', 64), 1, 8), ((4, 'v', 32), 8, 8),
                                      ('bf16', 4, 8), ((8, 'k', 64), 16, 16), ((8, 'v', 16), 8, 8)])
def test_wide_value_heads(fmt, m, bb):
    """d_k 128, d_v 256: the 'wide' head of the reference's KDA tests (tests/test_kda_kernels.py:21 there)."""
    T = 4 if m == 1 else 34 if m == 16 else 20
    check(run_decode(fmt, m, bb, B=2, H=2, DK=128, DV=256, T=T), f'kda 128x256 {fmt} m={m} buf{bb}', T, m)


@pytest.mark.parametrize('fmt', [(4, 'k', 32), (4, 'v', 16), (8, 'k', 32), (8, 'v', 16), (8, 'k', 64), (4, 'v', 32), 'bf16'])
@pytest.mark.parametrize('m,bb', [(8, 8), (4, 16), (1, 8), (16, 16)])
def test_single_value_block_head(fmt, m, bb):
    """3 heads of d_k 64, d_v 32: the 'small' head of the reference's KDA tests (tests/test_kda_kernels.py:21 there) --
    one 32-row block per tile, so the pass, the fold and the re-read all run their first-and-last iteration at once."""
    T = 4 if m == 1 else 34 if m == 16 else 20
    check(run_decode(fmt, m, bb, B=2, H=3, DK=64, DV=32, T=T), f'kda 64x32 {fmt} m={m} buf{bb}', T, m)


@pytest.mark.parametrize('bb', [8, 16])
def test_bf16_control_tracks_the_fp32_recurrence(bb):
    """The bf16 state (the control arm) against the textbook fp32 recurrence over 64 tokens, to bf16 / int8-buffer
    accuracy -- the reference's own bounds for this comparison (tests/test_kda_kernels.py:151-172 there)."""
    H, DK, DV = 4, 128, 128
    gen = torch.Generator().manual_seed(5)
    S0 = torch.randn(2 * H, DV, DK, generator=gen)
    S = S0.to(torch.bfloat16).float()
    ker = PackedKDAState(S0.to(DEV), 'bf16', m=8, hv=H, buffer_bits=bb, out_dtype=torch.float32)
    rel2 = 0.0
    for t in range(64):
        q, k, v, g, beta = kda_token(gen, 2, H, DK, DV)
        want = ST.kda_recurrence(S, q.reshape(-1, DK), k.reshape(-1, DK), v.reshape(-1, DV), g.reshape(-1, DK),
                                 beta.reshape(-1))
        got = ker.step(q.to(DEV), k.to(DEV), v.to(DEV), g.to(DEV), beta.to(DEV)).cpu().reshape(-1, DV)
        rel2 = max(rel2, ((got - want).norm() / want.norm()).item())
    st = ((ker.dequantize().cpu().view_as(S) - S).norm() / S.norm()).item()
    print(f'\nkda bf16 state buf{bb} vs fp32 recurrence: rel l2 {rel2:.2e}, state {st:.2e}')
    assert rel2 < (1.5e-2 if bb == 8 else 5e-3) and st < 1e-2


@pytest.mark.parametrize('fmt,m,bb', [((4, 'k', 32), 8, 8), ((8, 'k', 64), 16, 16), ((4, 'v', 32), 16, 8), ('bf16', 16, 8)])
def test_strong_per_channel_decays(fmt, m, bb):
    """The reference's safe gate at its lower bound (tests/test_kda_kernels.py:33-41 there: g = -5 sigmoid(.)) on a
    quarter of the channels at every token: over a full buffer of 16 the cumulative log decay reaches -80, so
    exp(-G) of the buffered keys is near 5e34 and exp(G) near 2e-35 -- both still fp32 normal numbers -- and channels
    that do not decay at all (g = 0) sit next to them."""
    def shape_token(q, k, v, g, beta):                     # g [B, H, d_k]
        g[..., 0::4] = -5.0
        g[..., 1::4] = 0.0

    T = 2 * m + 3
    tal = run_decode(fmt, m, bb, T=T, shape_token=shape_token)
    check(tal, f'kda strong decays {fmt} m={m} buf{bb}', T, m)


def test_bf16_inputs():
    check(run_decode((4, 'k', 32), 8, 8, T=16, dtype=torch.bfloat16), 'kda bf16 inputs', 16, 8)


@pytest.mark.parametrize('name', ['kda_int4.pt', 'kda_int8_bf16buf.pt'])
def test_against_reference_golden_vectors(golden, name):
    rec = golden(name)
    B, H, DK, DV, m, bb = (rec[k] for k in ('B', 'HV', 'DK', 'DV', 'm', 'buffer_bits'))
    ker = PackedKDAState(rec['S0'].to(DEV), quantizer(rec['fmt']), m=m, hv=H, buffer_bits=bb, out_dtype=torch.float32)
    assert torch.equal(ker.codes.cpu(), rec['codes0']) and torch.equal(ker.scales.cpu(), rec['scales0'])
    from oracle.formats import round_buf_parts
    worst, flips, entries, mism, far, ncodes = 0.0, 0, 0, 0, 0, 0
    for st in rec['steps']:
        n = st['n']
        assert ker.n == n
        o = ker.step(*(st[k].to(DEV) for k in ('q', 'k', 'v', 'g', 'beta'))).cpu().reshape(B * H, DV)
        worst = max(worst, ((o - st['o']).abs().max() / st['o'].abs().max()).item())
        kb, ub = buffer_entry(ker.T, n, bb == 8)
        flips += (kb != st['K']).sum().item() + (ub != st['U']).sum().item()
        entries += kb.numel() + ub.numel()
        assert torch.equal(ker.GB[:, n].cpu(), st['G'])
        if 'codes' in st:
            d = (unpack_nib(ker.codes.cpu(), rec['fmt'][0]).int() - unpack_nib(st['codes'], rec['fmt'][0]).int()).abs()
            mism += (d != 0).sum().item()
            far += (d > 1).sum().item()
            ncodes += d.numel()
            ker.codes.copy_(st['codes'])
            ker.scales.copy_(st['scales'])
        elif bb == 8:
            kc, ks = round_buf_parts(st['K'])
            uc, us = round_buf_parts(st['U'])
            ker.KB[:, n].copy_(kc), ker.KBS[:, n].copy_(ks), ker.UB[:, n].copy_(uc), ker.UBS[:, n].copy_(us)
        else:
            ker.KB[:, n].copy_(st['K'].to(torch.bfloat16)), ker.UB[:, n].copy_(st['U'].to(torch.bfloat16))
    print(f'\n[{name}] max rel |o - o_ref| {worst:.2e}; buffer flips {flips}/{entries}; codes differing {mism}/{ncodes}')
    assert worst < 2e-5 and flips <= max(1, 1e-4 * entries) and mism <= max(1, 1e-4 * ncodes) and far == 0


def _setup(fmt, H, D, m, bb, n_slots=12, seed=0):
    gen = torch.Generator().manual_seed(seed)
    lay = KDASlotLayout(quantizer(fmt), H, D, D, m=m, buffer_bits=bb)
    raw = torch.randint(0, 256, (n_slots, lay.nbytes + 4096), dtype=torch.uint8, generator=gen).to(DEV)
    blob = raw[:, 2048:2048 + lay.nbytes]
    views = lay.views(blob)
    slots = [5, 2, 7, 9, 11]
    S0 = [torch.randn(H, D, D, generator=gen).to(DEV) * 0.5 for _ in slots]
    refs = [PackedKDAState(s, quantizer(fmt), m=m, hv=H, buffer_bits=bb, out_dtype=torch.float32) for s in S0]
    lay.write(views, torch.tensor(slots, device=DEV), torch.stack(S0))
    return lay, raw, blob, views, slots, refs


@pytest.mark.parametrize('H,D,fmt', [(4, 128, (4, 'k', 32)), (20, 96, (4, 'k', 32)), (4, 128, 'bf16')])
@pytest.mark.parametrize('m,bb', [(8, 8), (2, 16)])
def test_slot_step_with_occupancy_mask(H, D, fmt, m, bb):
    """Slot step == lockstep state per sequence, bit for bit, with about 40 % of the batch rows unoccupied
    (slot index 0 or -1): their output rows are zero and nothing outside the live slots' blobs is written."""
    lay, raw, blob, views, slots, refs = _setup(fmt, H, D, m, bb)
    outside = raw.clone()
    sched = torch.Generator().manual_seed(1)
    gens = [torch.Generator().manual_seed(10 + i) for i in range(len(slots))]
    steps = [0] * len(slots)
    n_pad = n_rows = 0
    for t in range(18):
        live = [i for i in torch.randperm(len(slots), generator=sched).tolist()
                if torch.rand(1, generator=sched).item() < 0.6]
        rows = live + ['pad0', 'padneg', 'pad0'][:max(1, round(len(live) * 2 / 3))]        # ~40 % unoccupied
        rows = [rows[j] for j in torch.randperm(len(rows), generator=sched).tolist()]
        idx = torch.tensor([slots[r] if isinstance(r, int) else (0 if r == 'pad0' else -1) for r in rows],
                           device=DEV, dtype=torch.int32)
        Bn = len(rows)
        q, k = torch.zeros(Bn, H, D, device=DEV), torch.zeros(Bn, H, D, device=DEV)
        v, g = torch.zeros(Bn, H, D, device=DEV), torch.zeros(Bn, H, D, device=DEV)
        beta = torch.zeros(Bn, H, device=DEV)
        want = {}
        for b, r in enumerate(rows):
            n_rows += 1
            if not isinstance(r, int):
                n_pad += 1
                continue
            tq, tk, tv, tg, tb = (z[0].to(DEV) for z in kda_token(gens[r], 1, H, D, D))
            q[b], k[b], v[b], g[b], beta[b] = tq, tk, tv, tg, tb
            want[b] = refs[r].step(tq, tk, tv, tg, tb).clone()
            steps[r] += 1
        out = torch.full((Bn, H, D), 7., device=DEV)
        lay.step(views, idx, q, k, v, g, beta, out)
        for b, r in enumerate(rows):
            if isinstance(r, int):
                assert torch.equal(out[b], want[b].view(H, D)), (t, b)
                assert views['NPTR'][slots[r], :H].tolist() == [steps[r] % m] * H
                assert torch.equal(views['S'][slots[r]], refs[r].codes.view(H, *refs[r].codes.shape[1:]))
                if 'SC' in views:
                    assert torch.equal(views['SC'][slots[r]], refs[r].scales.view(H, *refs[r].scales.shape[1:]))
                assert torch.equal(views['GCUR'][slots[r]], refs[r].GCUR.view(H, D))
            else:
                assert torch.equal(out[b], torch.zeros_like(out[b]))
    assert 0.3 < n_pad / n_rows < 0.5, n_pad / n_rows
    keep = torch.ones_like(raw, dtype=torch.bool)
    for s in slots:
        keep[s, 2048:2048 + lay.nbytes] = False
    assert torch.equal(raw[keep], outside[keep])


def test_d96_equals_zero_padded_d128():
    """A d_k = 96 head run == the same problem with keys, queries and state zero-padded to d_k = 128 (the reference
    pins its own padded tiles this way, tests/test_kernels_nonpow2.py:94-136): outputs bit for bit, stored codes and
    scales equal on the first 96 columns / 3 groups."""
    B, H, DV, m = 2, 3, 96, 4
    gen = torch.Generator().manual_seed(9)
    S0 = torch.randn(B * H, DV, 96, generator=gen) * 0.5
    S0p = torch.nn.functional.pad(S0, (0, 32))
    # d_v must be a compiled shape: 96 x 96 and 128 x 128 are, so pad the value dim too (zero rows stay zero)
    S0p = torch.nn.functional.pad(S0p, (0, 0, 0, 32))
    a = PackedKDAState(S0.to(DEV), quantizer((4, 'k', 32)), m=m, hv=H, out_dtype=torch.float32)
    b = PackedKDAState(S0p.to(DEV), quantizer((4, 'k', 32)), m=m, hv=H, out_dtype=torch.float32)
    for t in range(10):
        q, k, v, g, beta = kda_token(gen, B, H, 96, DV)
        pad = lambda x: torch.nn.functional.pad(x, (0, 32))          # noqa: E731
        oa = a.step(q.to(DEV), k.to(DEV), v.to(DEV), g.to(DEV), beta.to(DEV), scale=96 ** -0.5).clone()
        ob = b.step(pad(q).to(DEV), pad(k).to(DEV), pad(v).to(DEV), pad(g).to(DEV), beta.to(DEV), scale=96 ** -0.5)
        assert torch.allclose(oa, ob[..., :96], rtol=2e-6, atol=1e-7), (t, (oa - ob[..., :96]).abs().max())
    ca = unpack_nib(a.codes.cpu(), 4)
    cb = unpack_nib(b.codes.cpu(), 4)[:, :96, :96]
    assert (ca != cb).float().mean().item() < 1e-4
    assert (cb.abs() <= 7).all() and (unpack_nib(b.codes.cpu(), 4)[:, :, 96:] == 0).all()


def test_read_is_the_state_the_next_step_reads():
    H, D, m = 4, 128, 8
    lay, raw, blob, views, slots, refs = _setup((4, 'k', 32), H, D, m, 8)
    gens = [torch.Generator().manual_seed(10 + i) for i in range(len(slots))]
    idx = torch.tensor(slots, device=DEV, dtype=torch.int32)
    for t in range(13):
        toks = [kda_token(gn, 1, H, D, D) for gn in gens]
        q, k, v, g, beta = (torch.cat(z).to(DEV) for z in zip(*toks))
        out = torch.empty(len(slots), H, D, device=DEV)
        if t == 12:
            S = lay.read(views, idx).reshape(-1, D, D)
            o_pred = kda_recurrence(S, q.reshape(-1, D), k.reshape(-1, D), v.reshape(-1, D), g.reshape(-1, D),
                                    beta.reshape(-1)).view(len(slots), H, D)
        lay.step(views, idx, q, k, v, g, beta, out)
    rel = ((out - o_pred).norm() / o_pred.norm()).item()
    assert rel < 1e-5, rel


def _random_configs(n, seed=59, shapes=((128, 128), (96, 96), (64, 64), (128, 256))):
    import random
    rng = random.Random(seed)
    fmts = [(4, 'k', 32), (4, 'k', 64), (8, 'k', 32), (8, 'k', 128), (4, 'v', 32), (4, 'v', 16), (8, 'v', 64), 'bf16']
    out = []
    while len(out) < n:
        fmt = rng.choice(fmts)
        DK, DV = rng.choice(list(shapes))
        if fmt != 'bf16' and (DK if fmt[1] == 'k' else DV) % fmt[2]:      # KDA: a group divides its axis (kda.py:55-64)
            continue
        out.append(dict(fmt=fmt, DK=DK, DV=DV, m=rng.choice([1, 2, 4, 8, 16]), bb=rng.choice([8, 16]),
                        H=rng.choice([1, 3, 4, 5]), B=rng.choice([1, 3]), seed=rng.randrange(1000),
                        dtype=rng.choice([torch.float32, torch.bfloat16])))
    return out


@pytest.mark.parametrize('cfg', _random_configs(12) + _random_configs(6, seed=61, shapes=((64, 32), (128, 256)))
                         + _random_configs(12, seed=101),     # 101: holds a buffered vector whose scale sits on an fp16 boundary
                         ids=lambda c: f"{c['fmt']}-{c['DK']}x{c['DV']}-m{c['m']}-h{c['H']}")
def test_random_configurations(cfg):
    """Seeded random combinations of format, head shape, buffer, head count and input dtype; the task's bounds."""
    T = max(2 * cfg['m'] + 1, 5)
    tal = run_decode(cfg['fmt'], cfg['m'], cfg['bb'], B=cfg['B'], H=cfg['H'], DK=cfg['DK'], DV=cfg['DV'], T=T,
                     seed=cfg['seed'], dtype=cfg['dtype'])
    print('\n' + tal.report(str(cfg)))
    assert tal.folds == T // cfg['m']
    assert tal.worst_o < 1e-4, tal.worst_o
    assert tal.buf_flips <= max(1, 1e-3 * tal.buf_entries), (tal.buf_flips, tal.buf_entries)
    assert tal.code_mism <= max(1, 1e-3 * tal.code_n) and tal.code_far == 0, (tal.code_mism, tal.code_far)


@pytest.mark.parametrize('fmt', [(4, 'k', 32), (8, 'k', 64), (4, 'v', 32)])
@pytest.mark.parametrize('m', [1, 2])
def test_first_fold_from_an_empty_state(fmt, m):
    """The first fold after an empty state quantizes a sum of m products of low-precision numbers (bf16 buffer
    entries): its quotients by the new scale are exact half-integers by the thousand (with m = 1, wherever the key's
    largest entry has the significand 127/128), which rint(div_rn(.)) -- the reference's _rint_quot,
    _fused_triton.py:472-486 there -- sends to even.  The kernels take the IEEE quotient where the old state
    contributes nothing (an old scale at its floor); with the reciprocal shortcut of the other folds a third of a
    percent of such a fold's codes would be one step off.  One fold: no code may differ (two for the sums' order)."""
    worst = 0
    for seed in range(6):
        tal = run_decode(fmt, m, 16, B=2, H=4, T=m, seed=seed, S0_scale=0.0)
        assert tal.folds == 1 and tal.code_far == 0
        worst = max(worst, tal.code_mism)
    print(f'\nkda {fmt} m={m}: at most {worst} of {tal.code_n} codes differ after the first fold (6 seeds)')
    assert worst <= 2, worst


def test_fp16_tokens():
    """fp16 q / k / v (dtype 2 of the C ABI) through the KDA step."""
    check(run_decode((4, 'k', 32), 8, 8, dtype=torch.float16, T=17), 'kda fp16 tokens', 17, 8)


@pytest.mark.parametrize('gd,bd,od', [(torch.float32, torch.float32, torch.float32), (torch.bfloat16, torch.float16, torch.float16),
                                      (torch.float16, torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32, torch.float32)])
def test_operand_and_output_dtypes(gd, bd, od):
    """The per-channel log decay g, beta and the output in any of the three float dtypes (each has its own dtype code
    in the C ABI): the oracle on the same rounded operands, its output rounded to the output's dtype or the neighbour
    of that."""
    B, H, D, m = 2, 4, 128, 4
    ker = PackedKDAState(torch.zeros(B * H, D, D, device=DEV), quantizer((4, 'k', 32)), m=m, hv=H, buffer_bits=8, out_dtype=od)
    ref = ST.KDAOracle(torch.zeros(B * H, D, D), (4, 'k', 32), m=m, hv=H, buffer_bits=8)
    gen = torch.Generator().manual_seed(3)
    ulp = {torch.float32: 2e-5, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[od]
    for t in range(m):                                       # up to the first fold (later steps need the re-sync)
        q, k, v, g, beta = kda_token(gen, B, H, D, D, torch.float32)
        g, beta = g.to(gd), beta.to(bd)
        o = ker.step(q.to(DEV), k.to(DEV), v.to(DEV), g.to(DEV), beta.to(DEV)).float().cpu().reshape(B * H, D)
        r = ref.step(q, k, v, g.float(), beta.float())
        assert ((o - r).abs() <= r.abs() * ulp + 1e-5 * r.abs().max()).all(), t
