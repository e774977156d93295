"""Mamba2 / SSD HIP step (through the C ABI) against the CPU oracle and the reference's golden vectors.

Mirrors the reference's tests/test_mamba2.py: decode vs the torch reference with per-step re-sync, slot step vs
lockstep with padding rows, read() predicting the next output, dt options (bias, softplus, clamp, D).
"""
import pytest
import torch

from oracle import states as ST
from statequant_amd.kernels import Mamba2SlotLayout, PackedMamba2State, mamba2_recurrence, unpack_vk
from tests._util import Tally, buffer_entry, quantizer, unpack_nib

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def m2_token(gen, B, H, G, DK, DV, dtype=torch.float32):
    """x ~ N(0,1); B, C ~ N(0,1) per group; raw dt ~ N(-2, 0.5) (softplus in the kernel)."""
    r = lambda *s: torch.randn(*s, generator=gen)          # noqa: E731
    return r(B, H, DV).to(dtype), r(B, H) * 0.5 - 2, r(B, G, DK).to(dtype), r(B, G, DK).to(dtype)


def params(gen, H):
    A = -torch.exp(torch.rand(H, generator=gen) * 2)
    return A, torch.randn(H, generator=gen), torch.randn(H, generator=gen) * 0.1


def run_decode(fmt, m, bb, B=2, H=8, G=2, DK=128, DV=64, T=24, seed=1, dtype=torch.float32, use_D=True, use_bias=True,
               softplus=True, limit=(0., float('inf')), S0_scale=0.5):
    gen = torch.Generator().manual_seed(seed)
    S0 = torch.randn(B * H, DV, DK, generator=gen) * S0_scale
    A, D, dtb = params(gen, H)
    D = D if use_D else None
    dtb = dtb if use_bias else None
    ker = PackedMamba2State(S0.to(DEV), quantizer(fmt), m=m, hv=H, hk=G, buffer_bits=bb, out_dtype=torch.float32)
    ref = ST.Mamba2Oracle(S0, fmt, m=m, hv=H, hk=G, buffer_bits=bb, auto_fold=False)
    assert torch.equal(ker.codes.cpu(), ref.codes) and torch.equal(ker.scales.cpu(), ref.scales)
    tal = Tally()
    dv = lambda t: None if t is None else t.to(DEV)        # noqa: E731
    for t in range(T):
        x, dt, Bm, C = m2_token(gen, B, H, G, DK, DV, dtype)
        slot = ker.n
        y = ker.step(dv(x), dv(dt), dv(Bm), dv(C), dv(A), dv(D), dv(dtb), softplus, limit).cpu().reshape(B * H, DV)
        r = ref.step(x, dt, Bm, C, A, D, dtb, softplus, limit)
        tal.out(y, r)
        kb, ub = buffer_entry(ker.T, slot, bb == 8)
        tal.entries(kb, ref.K[:, slot])
        tal.entries(ub, ref.U[:, slot])
        # the decay goes through softplus (log (1 + exp)): the device's and the host's libm may differ in the last bit of
        # the exponential, which the logarithm of a sum near 1 magnifies -- compare to a few ulps of that and let the
        # oracle continue from the kernel's value
        gk = ker.GB[:, slot].cpu()
        assert torch.allclose(gk, ref.G[:, slot], rtol=5e-6, atol=1e-7), t
        ref.G[:, slot] = gk
        ref.gcur = gk.clone()
        ref.K[:, slot], ref.U[:, slot] = kb, ub
        if ref.n == m:
            ref.fold()
        assert ker.n == ref.n
        if ref.n == 0:
            codes, scales = ker.codes.cpu(), ker.scales.cpu()
            tal.fold(codes, scales, ref, 16 if fmt == 'bf16' else fmt[0])
            ref.adopt(codes, scales)
        assert torch.equal(ker.NPTR.cpu(), torch.full((B, H), ref.n, dtype=torch.int32))
    return tal


def check(tal, tag, T, m):
    print('\n' + tal.report(tag))
    assert tal.folds == T // m
    assert tal.worst_o < 2e-5, tal.worst_o
    assert tal.buf_flips <= max(1, 1e-4 * tal.buf_entries), tal.buf_flips
    assert tal.code_mism <= max(1, 1e-4 * tal.code_n) and tal.code_far == 0, (tal.code_mism, tal.code_far)
    assert tal.worst_raw < 0.2


@pytest.mark.parametrize('fmt,m,bb', [((8, 'v', 32), 8, 8), ((4, 'v', 32), 4, 16), ((8, 'v', 32), 1, 8), ((8, 'v', 64), 8, 8),
                                      ((4, 'v', 64), 4, 16), ((4, 'v', 32), 16, 8), ((4, 'v', 16), 8, 8),
                                      ((8, 'v', 16), 4, 16), ((8, 'v', 16), 1, 8), ((4, 'v', 16), 16, 16)])
def test_value_axis_groups(fmt, m, bb):
    T = 4 if m == 1 else 34 if m == 16 else 24
    check(run_decode(fmt, m, bb, T=T), f'mamba2 {fmt} m={m} buf{bb}', T, m)


@pytest.mark.parametrize('m,bb', [(8, 8), (4, 16), (1, 8), (16, 16)])
@pytest.mark.parametrize('DK,DV', [(128, 64), (128, 128), (64, 64)])
def test_unquantized_state_control(m, bb, DK, DV):
    """The bf16 state (mamba2.py:352: the control for the packed formats) through the same step."""
    T = 3 * m + 2 if m > 1 else 4
    check(run_decode('bf16', m, bb, DK=DK, DV=DV, T=T), f'mamba2 bf16 state {DK}x{DV} m={m} buf{bb}', T, m)


@pytest.mark.parametrize('fmt', [(8, 'k', 128), (8, 'k', 32), (4, 'k', 64), (4, 'k', 32)])
@pytest.mark.parametrize('m,bb', [(8, 8), (4, 16), (1, 8), (16, 8)])
def test_decode_vs_oracle(fmt, m, bb):
    T = 32 if m == 16 else 24
    check(run_decode(fmt, m, bb, T=T), f'mamba2 {fmt} m={m} buf{bb}', T, m)


# 14 / 2: seven heads per group, as in Nemotron-H (112 / 8); neither count is a power of two
@pytest.mark.parametrize('DK,DV,H,G', [(128, 128, 4, 1), (64, 64, 4, 4), (128, 64, 14, 2)])
def test_other_head_shapes(DK, DV, H, G):
    check(run_decode((8, 'k', 64), 4, 8, B=3, H=H, G=G, DK=DK, DV=DV, T=12), f'mamba2 {DK}x{DV}', 12, 4)
    check(run_decode((4, 'k', 32), 16, 16, B=2, H=H, G=G, DK=DK, DV=DV, T=33), f'mamba2 {DK}x{DV} m=16', 33, 16)


@pytest.mark.parametrize('DK,DV,H,G', [(128, 80, 6, 2), (96, 80, 6, 2)])
@pytest.mark.parametrize('fmt,m,bb', [((8, 'k', 32), 8, 8), ((4, 'k', 32), 4, 16), ((8, 'k', 128), 1, 8), ((4, 'k', 32), 16, 8),
                                      ((4, 'v', 16), 8, 8), ((8, 'v', 16), 4, 16), ((8, 'v', 16), 1, 8), ('bf16', 8, 8),
                                      ('bf16', 4, 16)])
def test_head_dim_80(DK, DV, H, G, fmt, m, bb):
    """head_dim 80 = two and a half row blocks: Nemotron-3-Nano's heads (96 x 80 x d_state 128, the model of the
    reference's end-to-end Mamba2 run, docs/vllm.md:108 there) and the odd head of its tests (d_state 96, head_dim 80,
    tests/test_mamba2.py:24).  The last block's empty half is neither read nor written."""
    if fmt != 'bf16' and fmt[1] == 'k' and DK % fmt[2]:
        pytest.skip('Mamba2: a key group divides d_state')
    T = 4 if m == 1 else 34 if m == 16 else 20
    check(run_decode(fmt, m, bb, B=2, H=H, G=G, DK=DK, DV=DV, T=T), f'mamba2 {DK}x{DV} {fmt} m={m} buf{bb}', T, m)


@pytest.mark.parametrize('fmt,m,bb', [((8, 'k', 128), 8, 8), ((4, 'k', 64), 4, 16), ((8, 'k', 32), 1, 8), ((4, 'k', 32), 16, 8),
                                      ('bf16', 8, 8), ('bf16', 4, 16)])
def test_d_state_256(fmt, m, bb):
    """d_state 256, head_dim 64 (Falcon-H1's larger models): four 64-column pieces per state row."""
    T = 4 if m == 1 else 34 if m == 16 else 20
    check(run_decode(fmt, m, bb, B=2, H=4, G=2, DK=256, DV=64, T=T), f'mamba2 256x64 {fmt} m={m} buf{bb}', T, m)


def test_large_gqa_one_group():
    """Mamba-2 / Falcon-H1 / Granite style: one B / C group shared by all 64 heads (tests/test_mamba2.py:115-132 there)."""
    check(run_decode((4, 'k', 64), 8, 8, B=2, H=64, G=1, DK=128, DV=64, T=12), 'mamba2 64 heads, 1 group', 12, 8)


@pytest.mark.parametrize('DK,DV,H,G', [(128, 64, 8, 2), (96, 80, 6, 2)])
@pytest.mark.parametrize('bb', [8, 16])
def test_bf16_control_tracks_the_fp32_recurrence(DK, DV, H, G, bb):
    """The bf16 state (the control arm) against the textbook fp32 recurrence over 64 tokens, to bf16 / int8-buffer
    accuracy -- the reference's own bounds for this comparison (tests/test_mamba2.py:156-174 there)."""
    gen = torch.Generator().manual_seed(5)
    S0 = torch.randn(2, H, DV, DK, generator=gen)
    S = S0.to(torch.bfloat16).float()
    ker = PackedMamba2State(S0.to(DEV), 'bf16', m=8, hv=H, hk=G, buffer_bits=bb, out_dtype=torch.float32)
    A, D, dtb = params(gen, H)
    rel2 = 0.0
    for t in range(64):
        x, dt, Bm, C = m2_token(gen, 2, H, G, DK, DV)
        want = ST.mamba2_recurrence(S, x, dt, Bm, C, A, D, dtb, True, None).reshape(2, H, DV)
        got = ker.step(x.to(DEV), dt.to(DEV), Bm.to(DEV), C.to(DEV), A.to(DEV), D.to(DEV), dtb.to(DEV), True).cpu()
        rel2 = max(rel2, ((got.view_as(want) - want).norm() / want.norm()).item())
    st = ((ker.dequantize().cpu().view_as(S) - S).norm() / S.norm()).item()
    print(f'\nmamba2 {DK}x{DV} bf16 state buf{bb} vs fp32 recurrence: rel l2 {rel2:.2e}, state {st:.2e}')
    assert rel2 < (1.5e-2 if bb == 8 else 5e-3) and st < 1e-2


def test_dt_options_and_bf16_inputs():
    """No D, no dt_bias, dt given pre-activated (dt_softplus=False), a dt clamp; bf16 x / B / C."""
    check(run_decode((8, 'k', 128), 4, 8, T=8, use_D=False, use_bias=False), 'no D, no bias', 8, 4)
    check(run_decode((8, 'k', 128), 4, 8, T=8, limit=(0.05, 0.2)), 'dt clamp', 8, 4)
    check(run_decode((4, 'k', 64), 4, 8, T=8, dtype=torch.bfloat16), 'bf16 inputs', 8, 4)
    # pre-activated dt: same result as activating in the kernel
    gen = torch.Generator().manual_seed(2)
    B, H, G, DK, DV = 2, 8, 2, 128, 64
    S0 = torch.randn(B * H, DV, DK, generator=gen).to(DEV)
    A, D, dtb = (t.to(DEV) for t in params(gen, H))
    a = PackedMamba2State(S0, quantizer((8, 'k', 128)), m=4, hv=H, hk=G, out_dtype=torch.float32)
    b = PackedMamba2State(S0, quantizer((8, 'k', 128)), m=4, hv=H, hk=G, out_dtype=torch.float32)
    for t in range(6):
        x, dt, Bm, C = (t_.to(DEV) for t_ in m2_token(gen, B, H, G, DK, DV))
        act, _ = ST.mamba2_gate(dt.cpu(), A.cpu(), dtb.cpu(), True, None)
        ya = a.step(x, dt, Bm, C, A, D, dtb, True, None).clone()
        yb = b.step(x, act.to(DEV), Bm, C, A, D, None, False, None)
        assert torch.allclose(ya, yb, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize('name', ['m2_int8.pt', 'm2_int4_bf16buf.pt'])
def test_against_reference_golden_vectors(golden, name):
    rec = golden(name)
    B, H, G, DK, DV, m, bb = (rec[k] for k in ('B', 'HV', 'HK', 'DK', 'DV', 'm', 'buffer_bits'))
    ker = PackedMamba2State(rec['S0'].to(DEV), quantizer(rec['fmt']), m=m, hv=H, hk=G, buffer_bits=bb,
                            out_dtype=torch.float32)
    assert torch.equal(ker.codes.cpu(), rec['codes0']) and torch.equal(ker.scales.cpu(), rec['scales0'])
    from oracle.formats import round_buf_parts
    A, D, dtb = (rec[k].to(DEV) for k in ('A', 'D', 'dt_bias'))
    worst, flips, entries, mism, far, ncodes = 0.0, 0, 0, 0, 0, 0
    for st in rec['steps']:
        n = st['n']
        assert ker.n == n
        y = ker.step(st['x'].to(DEV), st['dt'].to(DEV), st['B'].to(DEV), st['C'].to(DEV), A, D, dtb, True,
                     (0., float('inf'))).cpu().reshape(B * H, DV)
        worst = max(worst, ((y - st['o']).abs().max() / st['o'].abs().max()).item())
        kb, ub = buffer_entry(ker.T, n, bb == 8)
        flips += (kb != st['K']).sum().item() + (ub != st['U']).sum().item()
        entries += kb.numel() + ub.numel()
        assert torch.allclose(ker.GB[:, n].cpu(), st['G'], rtol=1e-6, atol=1e-7)     # softplus: see run_decode
        ker.GB[:, n].copy_(st['G'])
        if 'codes' not in st:
            ker.GCUR.copy_(st['G'])
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
    print(f'\n[{name}] max rel |y - y_ref| {worst:.2e}; buffer flips {flips}/{entries}; codes differing {mism}/{ncodes}')
    assert worst < 2e-5 and flips <= max(1, 1e-4 * entries) and mism <= max(1, 1e-4 * ncodes) and far == 0


# ---------------------------------------------------------------------------------------------------------------
SHAPE = H, G, DK, DV = 8, 2, 128, 64
NANO = 12, 2, 128, 80                                   # Nemotron-3-Nano's head shape, fewer heads
WIDE = 4, 2, 256, 64                                    # d_state 256


def _setup(fmt, m, bb, seed=0, shape=None):
    H, G, DK, DV = shape or SHAPE
    gen = torch.Generator().manual_seed(seed)
    lay = Mamba2SlotLayout(quantizer(fmt), H, G, DK, DV, m=m, buffer_bits=bb)
    raw = torch.randint(0, 256, (8, lay.nbytes + 4096), dtype=torch.uint8, generator=gen).to(DEV)
    blob = raw[:, 2048:2048 + lay.nbytes]
    views = lay.views(blob)
    slots = [5, 2, 7]
    S0 = [torch.randn(H, DV, DK, generator=gen).to(DEV) * 0.5 for _ in slots]
    refs = [PackedMamba2State(s, quantizer(fmt), m=m, hv=H, hk=G, buffer_bits=bb, out_dtype=torch.float32)
            for s in S0]
    lay.write(views, torch.tensor(slots, device=DEV), torch.stack(S0))
    A, D, dtb = (t.to(DEV) for t in params(gen, H))
    return lay, raw, blob, views, slots, refs, (A, D, dtb)


@pytest.mark.parametrize('fmt,shape', [((8, 'k', 128), SHAPE), ((4, 'k', 32), SHAPE), ('bf16', SHAPE),
                                       ((8, 'k', 128), NANO), ((4, 'k', 32), NANO), ((8, 'v', 16), NANO), ('bf16', NANO),
                                       ((8, 'k', 128), WIDE), ('bf16', WIDE)],
                         ids=lambda v: str(v).replace(' ', ''))
@pytest.mark.parametrize('m,bb', [(8, 8), (2, 16)])
def test_slot_step_matches_lockstep_per_sequence(fmt, shape, m, bb):
    H, G, DK, DV = shape
    lay, raw, blob, views, slots, refs, (A, D, dtb) = _setup(fmt, m, bb, shape=shape)
    outside = raw.clone()
    sched = torch.Generator().manual_seed(1)
    gens = [torch.Generator().manual_seed(10 + i) for i in range(len(slots))]
    steps = [0] * len(slots)
    for t in range(20):
        live = [i for i in torch.randperm(len(slots), generator=sched).tolist()
                if torch.rand(1, generator=sched).item() < 0.7]
        rows = live + ['pad0', 'padneg']
        rows = [rows[j] for j in torch.randperm(len(rows), generator=sched).tolist()]
        idx = torch.tensor([slots[r] if isinstance(r, int) else (0 if r == 'pad0' else -1) for r in rows],
                           device=DEV, dtype=torch.int32)
        Bn = len(rows)
        x, dt = torch.zeros(Bn, H, DV, device=DEV), torch.zeros(Bn, H, device=DEV)
        Bm, C = torch.zeros(Bn, G, DK, device=DEV), torch.zeros(Bn, G, DK, device=DEV)
        want = {}
        for b, r in enumerate(rows):
            if not isinstance(r, int):
                continue
            tx, tdt, tB, tC = (z[0].to(DEV) for z in m2_token(gens[r], 1, H, G, DK, DV))
            x[b], dt[b], Bm[b], C[b] = tx, tdt, tB, tC
            want[b] = refs[r].step(tx, tdt, tB, tC, A, D, dtb, True, (0., float('inf'))).clone()
            steps[r] += 1
        out = torch.full((Bn, H, DV), 7., device=DEV)
        lay.step(views, idx, x, dt, Bm, C, out, A, D, dtb)
        for b, r in enumerate(rows):
            if isinstance(r, int):
                assert torch.equal(out[b], want[b].view(H, DV)), (t, b)
                assert views['NPTR'][slots[r], :H].tolist() == [steps[r] % m] * H
                assert torch.equal(views['S'][slots[r]], refs[r].codes.view(H, *refs[r].codes.shape[1:]))
                if 'SC' in views:
                    assert torch.equal(views['SC'][slots[r]], refs[r].scales.view(H, *refs[r].scales.shape[1:]))
            else:
                assert torch.equal(out[b], torch.zeros_like(out[b]))
    keep = torch.ones_like(raw, dtype=torch.bool)
    for s in slots:
        keep[s, 2048:2048 + lay.nbytes] = False
    assert torch.equal(raw[keep], outside[keep])


@pytest.mark.parametrize('shape', [SHAPE, NANO, WIDE], ids=str)
def test_read_is_the_state_the_next_step_reads(shape):
    """read() + one textbook fp32 Mamba2 step == the kernel's next output (reference: tests/test_mamba2.py:273-300)."""
    m = 8
    H, G, DK, DV = shape
    lay, raw, blob, views, slots, refs, (A, D, dtb) = _setup((8, 'k', 32), m, 8, shape=shape)
    gens = [torch.Generator().manual_seed(10 + i) for i in range(len(slots))]
    idx = torch.tensor(slots, device=DEV, dtype=torch.int32)
    for t in range(13):
        toks = [m2_token(gn, 1, H, G, DK, DV) for gn in gens]
        x, dt, Bm, C = (torch.cat(z).to(DEV) for z in zip(*toks))
        out = torch.empty(len(slots), H, DV, device=DEV)
        if t == 12:
            S = lay.read(views, idx)
            y_pred = mamba2_recurrence(S, x, dt, Bm, C, A, D, dtb, True, None)
        lay.step(views, idx, x, dt, Bm, C, out, A, D, dtb)
    rel = ((out - y_pred).norm() / y_pred.norm()).item()
    assert rel < 1e-5, rel
    # write(read()) == pack(unpack())
    S = lay.read(views, idx)
    lay.write(views, idx, S)
    got = lay.read(views, idx)
    from statequant_amd.kernels import pack_vk
    c, s = pack_vk(S.reshape(-1, DV, DK), quantizer((8, 'k', 32)))
    assert torch.equal(got, unpack_vk(c, s, quantizer((8, 'k', 32)), DK).view_as(S))


def _random_configs(n, seed=31, shapes=((128, 64), (128, 128), (64, 64))):
    import random
    rng = random.Random(seed)
    fmts = [(4, 'k', 32), (4, 'k', 64), (8, 'k', 32), (8, 'k', 128), (4, 'v', 32), (8, 'v', 16), (8, 'v', 64), 'bf16']
    out = []
    while len(out) < n:
        fmt = rng.choice(fmts)
        DK, DV = rng.choice(list(shapes))
        if fmt != 'bf16' and ((fmt[1] == 'k' and DK % fmt[2]) or (fmt[1] == 'v' and DV % fmt[2])):
            continue                                         # Mamba2 groups must divide their axis (mamba2.py:73-78)
        G = rng.choice([1, 2, 3])
        out.append(dict(fmt=fmt, DK=DK, DV=DV, m=rng.choice([1, 2, 4, 8, 16]), bb=rng.choice([8, 16]), G=G,
                        H=G * rng.choice([1, 2, 7]), B=rng.choice([1, 3]), seed=rng.randrange(1000),
                        dtype=rng.choice([torch.float32, torch.bfloat16]), use_D=rng.random() < 0.7,
                        use_bias=rng.random() < 0.7))
    return out


@pytest.mark.parametrize('cfg', _random_configs(12) + _random_configs(6, seed=37, shapes=((128, 80), (96, 80))), ids=lambda c: f"{c['fmt']}-{c['DK']}x{c['DV']}-m{c['m']}-h{c['H']}g{c['G']}")
def test_random_configurations(cfg):
    """Seeded random combinations of format, head shape, buffer, head / group counts (also 7 heads per group), D /
    dt_bias present or not and input dtype; the task's bounds (99.9 % of entries and codes identical, none off by more than a step)."""
    T = max(2 * cfg['m'] + 1, 5)
    tal = run_decode(cfg['fmt'], cfg['m'], cfg['bb'], B=cfg['B'], H=cfg['H'], G=cfg['G'], DK=cfg['DK'], DV=cfg['DV'], T=T,
                     seed=cfg['seed'], dtype=cfg['dtype'], use_D=cfg['use_D'], use_bias=cfg['use_bias'])
    print('\n' + tal.report(str(cfg)))
    assert tal.folds == T // cfg['m']
    assert tal.worst_o < 1e-4, tal.worst_o
    assert tal.buf_flips <= max(1, 1e-3 * tal.buf_entries), (tal.buf_flips, tal.buf_entries)
    assert tal.code_mism <= max(1, 1e-3 * tal.code_n) and tal.code_far == 0, (tal.code_mism, tal.code_far)


@pytest.mark.parametrize('fmt', [(8, 'k', 128), (4, 'k', 64), (8, 'v', 32)])
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
        tal = run_decode(fmt, m, 16, B=2, H=8, G=2, T=m, seed=seed, S0_scale=0.0)
        assert tal.folds == 1 and tal.code_far == 0
        worst = max(worst, tal.code_mism)
    print(f'\nmamba2 {fmt} m={m}: at most {worst} of {tal.code_n} codes differ after the first fold (6 seeds)')
    assert worst <= 2, worst


def test_fp16_tokens():
    """fp16 x / B / C (dtype 2 of the C ABI) through both Mamba2 kernel kinds."""
    check(run_decode((8, 'k', 128), 8, 8, dtype=torch.float16, T=17), 'mamba2 fp16 tokens', 17, 8)
    check(run_decode((8, 'v', 32), 4, 16, dtype=torch.float16, T=9), 'mamba2 value-axis fp16 tokens', 9, 4)


@pytest.mark.parametrize('sd,od', [(torch.float32, torch.float32), (torch.bfloat16, torch.float16), (torch.float16, torch.bfloat16),
                                   (torch.float16, torch.float32)])
def test_operand_and_output_dtypes(sd, od):
    """dt, A, D, dt_bias in any of the three float dtypes and the output likewise (each has its own dtype code in the
    C ABI): the oracle on the same rounded operands, its output rounded to the output's dtype or the neighbour."""
    B, H, G, DK, DV, m = 2, 8, 2, 128, 64, 4
    gen = torch.Generator().manual_seed(5)
    A, Dp, dtb = (t.to(sd) for t in params(gen, H))
    ker = PackedMamba2State(torch.zeros(B * H, DV, DK, device=DEV), quantizer((8, 'k', 128)), m=m, hv=H, hk=G, buffer_bits=8,
                            out_dtype=od)
    ref = ST.Mamba2Oracle(torch.zeros(B * H, DV, DK), (8, 'k', 128), m=m, hv=H, hk=G, buffer_bits=8)
    ulp = {torch.float32: 2e-5, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[od]
    for t in range(m):                                       # up to the first fold (later steps need the re-sync)
        x, dt, Bm, C = m2_token(gen, B, H, G, DK, DV, torch.float32)
        dt = dt.to(sd)
        y = ker.step(x.to(DEV), dt.to(DEV), Bm.to(DEV), C.to(DEV), A.to(DEV), Dp.to(DEV), dtb.to(DEV), True,
                     (0., float('inf'))).float().cpu().reshape(B * H, DV)
        r = ref.step(x, dt.float(), Bm, C, A.float(), Dp.float(), dtb.float(), True, (0., float('inf')))
        assert ((y - r).abs() <= r.abs() * ulp + 1e-5 * r.abs().max()).all(), t
