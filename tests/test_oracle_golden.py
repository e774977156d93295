"""The CPU oracle against golden vectors recorded from the reference's own torch classes
(tests/golden/make_golden.py).  Every oracle function is replayed step by step from the reference's recorded state
("teacher forcing": after each comparison the oracle adopts the reference's buffer entries / codes, as the
reference's own kernel tests do, tests/test_kernels.py:88-109 there), so each step and each fold is checked on its
own and a last-bit difference in one step cannot hide or inflate a difference in the next."""
import pytest
import torch

from oracle import formats as F
from oracle import slots as SL
from oracle import states as ST

# fp32 sums may associate differently between the reference's orientation ([BH, d_k, d_v] einsums) and the oracle's;
# everything elementwise must be bit-identical.
O_TOL = 2e-6


def test_pack_unpack_bit_exact(golden):
    G = golden('pack.pt')
    Svm = G['S'].transpose(1, 2).contiguous()                      # the reference's pack takes [BH, d_k, d_v]
    for c in G['cases']:
        codes, scales = F.pack_vk(Svm, c['fmt'])
        assert codes.dtype == c['codes'].dtype and torch.equal(codes, c['codes']), c['fmt']
        assert scales.dtype == torch.float16 and torch.equal(scales, c['scales']), c['fmt']
        deq = F.unpack_vk(codes, scales, c['fmt'], Svm.shape[-1])
        assert torch.equal(deq.transpose(1, 2), c['deq']), c['fmt']
        assert torch.equal(deq.transpose(1, 2), c['fake']), c['fmt']            # == Quantizer(fp16 scales).fake
    for c in G['ragged']:
        codes, scales = F.pack_vk(G['ragged_X'], c['fmt'])
        assert torch.equal(codes, c['codes']) and torch.equal(scales, c['scales'])
        assert torch.equal(F.unpack_vk(codes, scales, c['fmt'], 96), c['deq'])
    cb, sb = F.pack_vk(Svm, 'bf16')
    assert torch.equal(cb, G['bf16_codes'])
    assert torch.equal(F.unpack_vk(cb, sb, 'bf16', Svm.shape[-1]).transpose(1, 2), G['bf16_deq'])


def test_round_buf_bit_exact(golden):
    G = golden('pack.pt')
    assert torch.equal(F.round_buf(G['rb_in'], 8), G['rb8'])
    assert torch.equal(F.round_buf(G['rb_in'], 16), G['rb16'])
    codes, s = F.round_buf_parts(G['rb_in'])
    assert torch.equal(codes.float() * s.float()[:, None], G['rb8'])


def _replay(rec, make, call):
    fam = rec['family']
    S0 = rec['S0'].transpose(1, 2).contiguous() if fam == 'gdn' else rec['S0']
    o = make(S0)
    assert torch.equal(o.codes, rec['codes0']) and torch.equal(o.scales, rec['scales0'])
    worst, flips, entries, code_mism, codes_n, folds = 0.0, 0, 0, 0, 0, 0
    for st in rec['steps']:
        n = o.n
        assert n == st['n']
        y = call(o, st)
        worst = max(worst, ((y - st['o']).abs().max() / st['o'].abs().max().clamp_min(1e-30)).item())
        assert torch.equal(o.G[:, n], st['G'])                       # decays: elementwise fp32 sums, exact
        flips += (o.U[:, n] != st['U']).sum().item() + (o.K[:, n] != st['K']).sum().item()
        entries += st['U'].numel() + st['K'].numel()
        o.U[:, n], o.K[:, n] = st['U'], st['K']                       # adopt the reference's entries
        if o.n == o.m:
            o.fold()
            raw = st['S_raw'].transpose(1, 2) if fam == 'gdn' else st['S_raw']
            assert torch.equal(o.S_raw, raw)                          # same entries in, elementwise fold: exact
            assert torch.equal(o.codes, st['codes']) and torch.equal(o.scales, st['scales'])
            code_mism += (o.codes != st['codes']).sum().item()
            codes_n += st['codes'].numel()
            folds += 1
        else:
            assert 'codes' not in st
    assert worst < O_TOL, worst
    assert flips <= max(1, 1e-4 * entries), (flips, entries)
    assert folds == len(rec['steps']) // rec['m']
    return worst, flips


@pytest.mark.parametrize('name', ['gdn_c1.pt', 'gdn_int4.pt', 'gdn_int8_m1.pt', 'gdn_int4v.pt', 'gdn_bf16.pt'])
def test_gdn_steps_and_folds(golden, name):
    rec = golden(name)
    mk = lambda S: ST.GDNOracle(S, rec['fmt'], m=rec['m'], hv=rec['HV'], hk=rec['HK'],      # noqa: E731
                                buffer_bits=rec['buffer_bits'], auto_fold=False)
    worst, flips = _replay(rec, mk, lambda o, s: o.step(s['q'], s['k'], s['v'], s['g'], s['beta'], rec['scale']))
    print(f'\n[{name}] max rel |o - o_ref| {worst:.2e}, buffer flips {flips}')


@pytest.mark.parametrize('name', ['kda_int4.pt', 'kda_int8_bf16buf.pt'])
def test_kda_steps_and_folds(golden, name):
    rec = golden(name)
    mk = lambda S: ST.KDAOracle(S, rec['fmt'], m=rec['m'], hv=rec['HV'], buffer_bits=rec['buffer_bits'],  # noqa: E731
                                auto_fold=False)
    worst, flips = _replay(rec, mk, lambda o, s: o.step(s['q'], s['k'], s['v'], s['g'], s['beta']))
    print(f'\n[{name}] max rel |o - o_ref| {worst:.2e}, buffer flips {flips}')


@pytest.mark.parametrize('name', ['m2_int8.pt', 'm2_int4_bf16buf.pt'])
def test_mamba2_steps_and_folds(golden, name):
    rec = golden(name)
    mk = lambda S: ST.Mamba2Oracle(S, rec['fmt'], m=rec['m'], hv=rec['HV'], hk=rec['HK'],   # noqa: E731
                                   buffer_bits=rec['buffer_bits'], auto_fold=False)
    call = lambda o, s: o.step(s['x'], s['dt'], s['B'], s['C'], rec['A'], rec['D'], rec['dt_bias'], True,  # noqa: E731
                               (0., float('inf')))
    worst, flips = _replay(rec, mk, call)
    print(f'\n[{name}] max rel |y - y_ref| {worst:.2e}, buffer flips {flips}')


_DT = {'torch.float32': torch.float32, 'torch.int32': torch.int32, 'torch.float16': torch.float16,
       'torch.bfloat16': torch.bfloat16, 'torch.int8': torch.int8, 'torch.uint8': torch.uint8}


def test_slot_layout_tables(golden):
    for t in golden('slots.pt')['tables']:
        a = dict(t['args'])
        fmt = a.pop('fmt')
        sd = torch.float32 if fmt == 'fp32' else torch.bfloat16
        fmt = 'bf16' if fmt == 'fp32' else fmt
        table, nbytes = SL.layout(t['family'], fmt, a['hv'], a.get('hk', a['hv']), a['dk'], a['dv'], a['m'],
                                  a['buffer_bits'], state_dtype=sd)
        assert nbytes == t['nbytes'], (t['args'], nbytes, t['nbytes'])
        assert list(table) == list(t['fields'])
        for name, (off, dt, shape, nb) in t['fields'].items():
            assert table[name] == (off, _DT[dt], tuple(shape), nb), (t['args'], name)


def test_slot_write_and_read(golden):
    for c in golden('slots.pt')['rw']:
        a = c['args']
        hk = a.get('hk', a['hv'])
        table, nbytes = SL.layout(c['family'], c['fmt'], a['hv'], hk, a['dk'], a['dv'], a['m'], a['buffer_bits'])
        # write: start from the same random blob the reference started from? only the written fields are compared
        blob = c['after_write'].clone()
        V = SL.views(table, blob)
        SL.write(V, c['idx'], c['S'], c['fmt'], a['hv'], a['dk'], a['dv'])
        assert torch.equal(blob, c['after_write'])                    # idempotent on the reference's own result
        got = SL.read(SL.views(table, c['blob'].clone()), c['idx'], c['fmt'], a['hv'], hk, a['dk'], a['dv'], a['m'],
                      per_channel=c['family'] == 'kda')
        rel = ((got - c['read']).abs().max() / c['read'].abs().max()).item()
        assert rel < 2e-6, (c['family'], rel)
