"""Writes the golden vectors under tests/golden/ by running the REFERENCE's own torch classes on seeded inputs.

Runs only where the reference checkout is mounted (default /root/reference; override with SQ_REFERENCE); the tests
never import the reference, they only load the .pt files written here (plain tensors, ``weights_only=True``).

    python tests/golden/make_golden.py

What is recorded (CPU, fp32, torch.manual_seed per case):
  pack_*.pt      pack / pack_vk / unpack on the reference tests' edge cases (all-zero groups, 1e-6-scaled states, a
                 ragged last key group), `_round_buf`, `Quantizer(..., scale_dtype='fp16').fake`
  gdn_*.pt       ReferenceGDNState: per step the inputs, the output, the entries appended to the buffer, and at
                 every fold the unrounded folded state, the codes and the scales
  kda_*.pt       ReferenceKDAState, likewise;   m2_*.pt  ReferenceMamba2State, likewise
  slots_*.pt     SlotLayout / KDASlotLayout / Mamba2SlotLayout: field tables, `write` then `read` on a blob with a
                 partly filled buffer
  gga.pt         the mixed-width GGA / STEP slot: `step_quant.fit` and `methods_ext.gga.fp8_vec` on seeded inputs (all
                 widths, zero and tiny vectors), the `GGAPacked` offset tables and bits-per-value figures, and decode
                 steps of the `PureWrite` / `StepQuant` reference path driven as the reference's tests/test_vllm_gga.py
                 drives it (per step: tokens, output, stored state, queued pairs), with and without the window
"""
import os
import sys

import torch

REF = os.environ.get('SQ_REFERENCE', '/root/reference')
HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(REF, 'src'))

import statequant as sq  # noqa: E402
from statequant.kernels import (KDASlotLayout, Mamba2SlotLayout, ReferenceGDNState, ReferenceKDAState,  # noqa: E402
                                ReferenceMamba2State, SlotLayout, pack, pack_vk, unpack, unpack_vk)
from statequant.kernels.fold import _round_buf  # noqa: E402

torch.set_num_threads(1)                 # one thread: reduction order independent of the host's core count


def save(name, obj):
    path = os.path.join(HERE, name)
    torch.save(obj, path)
    print(f'{name}: {os.path.getsize(path) / 1024:.0f} KiB')


def fmt_of(t):
    return sq.Quantizer(*t)


# ---------------------------------------------------------------------------------------------------------------
def golden_pack():
    torch.manual_seed(0)
    S = torch.randn(3, 64, 32) * torch.rand(3, 64, 1) * 3          # [BH, d_k, d_v]
    S[0, :32, :] = 0                                                # all-zero key groups
    S[1] *= 1e-6                                                    # scales in the fp16 subnormal range
    out = {'S': S, 'cases': []}
    for bits in (4, 8):
        for axis, group in (('k', 32), ('k', 64), ('v', 16), ('v', 32)):
            q = sq.Quantizer(bits, axis, group)
            c, s = pack(S, q)
            out['cases'].append(dict(fmt=(bits, axis, group), codes=c, scales=s, deq=unpack(c, s, q, 64),
                                     fake=sq.Quantizer(bits, axis, group, scale_dtype='fp16').fake(S)))
    # ragged last key group: d_k = 96, group 64 (value-major input)
    X = torch.randn(2, 32, 96)
    rag = []
    for bits in (4, 8):
        q = sq.Quantizer(bits, 'k', 64)
        c, s = pack_vk(X, q)
        rag.append(dict(fmt=(bits, 'k', 64), codes=c, scales=s, deq=unpack_vk(c, s, q, 96)))
    out['ragged_X'], out['ragged'] = X, rag
    cb, sb = pack(S, 'bf16')
    out['bf16_codes'], out['bf16_deq'] = cb, unpack(cb, sb, 'bf16', 64)
    v = torch.randn(5, 64) * torch.tensor([1., 1e-3, 50., 1e-7, 0.])[:, None]
    out['rb_in'], out['rb8'], out['rb16'] = v, _round_buf(v, 8), _round_buf(v, 16)
    save('pack.pt', out)


# ---------------------------------------------------------------------------------------------------------------
def run_gdn(name, fmt, B, HV, HK, DK, DV, m, bb, T, seed, S0_scale=0.5, per_key=True, v_head_scale=False):
    torch.manual_seed(seed)
    BH = B * HV
    S0 = torch.randn(BH, DK, DV) * S0_scale if S0_scale else torch.zeros(BH, DK, DV)
    ref = ReferenceGDNState(S0, fmt_of(fmt) if fmt != 'bf16' else 'bf16', m=m, hv=HV, hk=HK, buffer_bits=bb)
    rec = dict(family='gdn', fmt=fmt, B=B, HV=HV, HK=HK, DK=DK, DV=DV, m=m, buffer_bits=bb, scale=DK ** -0.5,
               S0=S0, codes0=ref.codes.clone(), scales0=ref.scales.clone(), steps=[])
    vs = torch.exp(torch.empty(HV).uniform_(-2.302585, 2.302585)) if v_head_scale else torch.ones(HV)
    for t in range(T):
        nq = B * HK if per_key else BH
        q, k = torch.randn(nq, DK), torch.randn(nq, DK)
        v = torch.randn(BH, DV) * vs.repeat(B)[:, None]
        g = -torch.nn.functional.softplus(torch.randn(BH))
        beta = torch.sigmoid(torch.randn(BH))
        n = ref.n
        o = ref.step(q, k, v, g, beta, DK ** -0.5)
        st = dict(q=q, k=k, v=v, g=g, beta=beta, o=o.clone(), n=n, U=ref.U[:, n].clone(), K=ref.K[:, n].clone(),
                  G=ref.G[:, n].clone())
        if ref.n == 0:                                              # folded in this step
            st.update(S_raw=ref.S_raw.clone(), codes=ref.codes.clone(), scales=ref.scales.clone())
        rec['steps'].append(st)
    save(name, rec)


def run_kda(name, fmt, B, H, DK, DV, m, bb, T, seed):
    torch.manual_seed(seed)
    BH = B * H
    S0 = torch.randn(BH, DV, DK) * 0.5
    ref = ReferenceKDAState(S0, fmt_of(fmt), m=m, hv=H, buffer_bits=bb)
    rec = dict(family='kda', fmt=fmt, B=B, HV=H, HK=H, DK=DK, DV=DV, m=m, buffer_bits=bb, S0=S0,
               codes0=ref.codes.clone(), scales0=ref.scales.clone(), steps=[])
    for t in range(T):
        q, k, v = torch.randn(BH, DK), torch.randn(BH, DK), torch.randn(BH, DV)
        g = -torch.nn.functional.softplus(torch.randn(BH, DK))
        beta = torch.sigmoid(torch.randn(BH))
        n = ref.n
        o = ref.step(q, k, v, g, beta)
        st = dict(q=q, k=k, v=v, g=g, beta=beta, o=o.clone(), n=n, U=ref.U[:, n].clone(), K=ref.K[:, n].clone(),
                  G=ref.G[:, n].clone())
        if ref.n == 0:
            st.update(S_raw=ref.S_raw.clone(), codes=ref.codes.clone(), scales=ref.scales.clone())
        rec['steps'].append(st)
    save(name, rec)


def run_m2(name, fmt, B, H, G, DK, DV, m, bb, T, seed):
    torch.manual_seed(seed)
    BH = B * H
    S0 = torch.randn(BH, DV, DK) * 0.5
    ref = ReferenceMamba2State(S0, fmt_of(fmt), m=m, hv=H, hk=G, buffer_bits=bb)
    A = -torch.exp(torch.rand(H) * 2)
    D = torch.randn(H)
    dt_bias = torch.randn(H) * 0.1
    rec = dict(family='mamba2', fmt=fmt, B=B, HV=H, HK=G, DK=DK, DV=DV, m=m, buffer_bits=bb, S0=S0, A=A, D=D,
               dt_bias=dt_bias, codes0=ref.codes.clone(), scales0=ref.scales.clone(), steps=[])
    for t in range(T):
        x = torch.randn(B, H, DV)
        dt = torch.randn(B, H) * 0.5 - 2
        Bm, C = torch.randn(B, G, DK), torch.randn(B, G, DK)
        n = ref.n
        y = ref.step(x, dt, Bm, C, A, D, dt_bias, True, (0., float('inf')))
        st = dict(x=x, dt=dt, B=Bm, C=C, o=y.clone(), n=n, U=ref.U[:, n].clone(), K=ref.K[:, n].clone(),
                  G=ref.G[:, n].clone())
        if ref.n == 0:
            st.update(S_raw=ref.S_raw.clone(), codes=ref.codes.clone(), scales=ref.scales.clone())
        rec['steps'].append(st)
    save(name, rec)


# ---------------------------------------------------------------------------------------------------------------
def golden_slots():
    out = {'tables': []}
    for fam, cls, args in (
            ('gdn', SlotLayout, dict(fmt=(4, 'k', 64), hv=32, hk=16, dk=128, dv=128, m=8, buffer_bits=8)),
            ('gdn', SlotLayout, dict(fmt=(8, 'k', 32), hv=32, hk=16, dk=128, dv=128, m=8, buffer_bits=8)),
            ('gdn', SlotLayout, dict(fmt=(8, 'k', 128), hv=32, hk=16, dk=128, dv=128, m=8, buffer_bits=16)),
            ('gdn', SlotLayout, dict(fmt=(4, 'k', 64), hv=30, hk=30, dk=96, dv=192, m=8, buffer_bits=8)),
            ('gdn', SlotLayout, dict(fmt='bf16', hv=4, hk=2, dk=64, dv=64, m=4, buffer_bits=16)),
            ('gdn', SlotLayout, dict(fmt='fp32', hv=4, hk=2, dk=64, dv=64, m=4, buffer_bits=8)),
            ('gdn', SlotLayout, dict(fmt=(4, 'v', 32), hv=4, hk=2, dk=128, dv=128, m=8, buffer_bits=8)),
            ('kda', KDASlotLayout, dict(fmt=(4, 'k', 32), hv=32, dk=128, dv=128, m=8, buffer_bits=8)),
            ('kda', KDASlotLayout, dict(fmt=(4, 'k', 64), hv=16, dk=128, dv=128, m=8, buffer_bits=8)),
            ('mamba2', Mamba2SlotLayout, dict(fmt=(8, 'k', 128), hv=128, hk=8, dk=128, dv=64, m=8, buffer_bits=8)),
            ('mamba2', Mamba2SlotLayout, dict(fmt=(8, 'k', 32), hv=112, hk=8, dk=128, dv=64, m=8, buffer_bits=8))):
        kw = dict(args)
        f = kw.pop('fmt')
        lay = cls(fmt_of(f) if isinstance(f, tuple) else f, **kw)
        out['tables'].append(dict(family=fam, args=args, nbytes=lay.nbytes,
                                  fields={n: (o, str(dt), tuple(sh), nb) for n, (o, dt, sh, nb) in lay.fields.items()}))
    # write -> partly filled buffer -> read, for the three families (small shapes)
    torch.manual_seed(7)
    rw = []
    for fam, cls, kw, f in (('gdn', SlotLayout, dict(hv=4, hk=2, dk=64, dv=32, m=4, buffer_bits=8), (4, 'k', 32)),
                            ('mamba2', Mamba2SlotLayout, dict(hv=4, hk=2, dk=32, dv=32, m=4, buffer_bits=16), (8, 'k', 32)),
                            ('kda', KDASlotLayout, dict(hv=2, dk=32, dv=32, m=4, buffer_bits=8), (8, 'k', 32))):
        lay = cls(fmt_of(f), **kw)
        blob = torch.randint(0, 256, (5, lay.nbytes), dtype=torch.uint8)
        V = lay.views(blob)
        idx = torch.tensor([3, 1])
        S = torch.randn(2, kw['hv'], kw['dv'], kw['dk'])
        lay.write(V, idx, S)
        after_write = blob.clone()
        # a buffer with n = 2 live entries: finite decays, finite scales; dead entries stay random bytes
        V['NPTR'][idx] = 2
        V['GCUR'][idx] = -torch.rand_like(V['GCUR'][idx])
        V['GB'][idx] = -torch.rand_like(V['GB'][idx]) * 0.5
        if 'KBS' in V:
            V['KBS'][idx] = (torch.rand_like(V['KBS'][idx].float()) * 0.01).half()
            V['UBS'][idx] = (torch.rand_like(V['UBS'][idx].float()) * 0.01).half()
        else:
            V['KB'][idx] = torch.randn(V['KB'][idx].shape).to(torch.bfloat16)
            V['UB'][idx] = torch.randn(V['UB'][idx].shape).to(torch.bfloat16)
        rw.append(dict(family=fam, fmt=f, args=kw, idx=idx, S=S, after_write=after_write, blob=blob.clone(),
                       read=lay.read(V, idx)))
    out['rw'] = rw
    save('slots.pt', out)


def golden_gga():
    from statequant.families import BY_NAME, Piece
    from statequant.integrations.vllm_gga import GGAPacked
    from statequant.methods_ext.gga import fp8_vec
    from statequant.step_quant import fit
    GDN = BY_NAME['gdn']
    out = {}
    # -- the fit: every width, columns spanning three decades, a zero row, a zero column, a zero head
    g = torch.Generator().manual_seed(0)
    bits = torch.tensor([2, 4, 6, 8, 16, 4])
    w = torch.rand(6, 64, generator=g) + 0.5
    x = torch.randn(2, 6, 64, 64, generator=g) * torch.logspace(-3, 0, 64)
    x[0, 1, 5, :] = 0
    x[0, 3, :, 7] = 0
    x[1, 5] = 0
    out['fit'] = dict(x=x, bits=bits, w=w, y=fit(x, bits, w))
    v = torch.randn(12, 64, generator=g)
    v[1] = 0
    v[2] *= 1e-40
    v[3] *= 1e-30
    v[4] *= 1e4
    v[5, 0] = 0
    out['fp8'] = dict(x=v, y=fp8_vec(v))
    # -- offset tables and storage accounting (the plan of the reference's tests/test_gga_packed.py)
    HV, D = 8, 128
    widths = [[2, 4, 6, 8, 16, 2, 4, 6], [8, 6, 4, 2, 2, 16, 8, 4]]
    q = sq.GGA(4, pivots=1)
    q.plan = {i: (torch.tensor(widths[i]), torch.rand(HV, D, generator=g) + 0.5) for i in range(2)}
    q.masks = {i: b == 16 for i, (b, _) in q.plan.items()}
    tab = dict(widths=widths, hv=HV, dk=D, dv=D, m=8, step_bits=q.bits_per_value(D, D),
               pw_bits=sq.pure_write(q).bits_per_value(D, D))
    for pw in (False, True):
        pk = GGAPacked(q, HV, 4, D, D, pw=pw)
        tab[pw] = dict(offs=[pk.tables[i][0] for i in range(2)], bytes_per_layer=[pk.bytes_per_layer[i] for i in range(2)],
                       QOFF=pk.QOFF, QSZ=pk.QSZ, nbytes=pk.nbytes, bits_per_value=pk.bits_per_value())
    out['tables'] = tab

    # -- decode steps of the reference path (PureWrite around the plan; without the window the plan's own rounding)
    def run(pw, m, T, seed):
        B, HV, HK, D = 2, 4, 2, 32
        gg = torch.Generator().manual_seed(seed)
        r = lambda *s: torch.randn(*s, generator=gg)      # noqa: E731
        qq = sq.GGA(4, pivots=1)
        qq.plan = {0: (torch.tensor([2, 4, 16, 8]), torch.rand(HV, D, generator=gg) + 0.5)}
        qq.masks = {0: qq.plan[0][0] == 16}
        S0 = r(B, HV, D, D) * 0.3
        O = qq.quantize(S0, 0)
        rec = dict(pw=pw, m=m, hv=HV, hk=HK, dk=D, dv=D, bits=qq.plan[0][0], w=qq.plan[0][1], S0=S0, O0=O,
                   scale=D ** -0.5, steps=[])
        ref = sq.pure_write(qq, m=m) if pw else qq
        if pw:
            ref.reset()
            ref.layers[0] = {'O': O, 'Q': [], 'R': []}
        for t in range(T):
            tq, tk, tv, ta, tb = r(B, HK, D), r(B, HK, D), r(B, HV, D), r(B, HV) * 0.5 - 2, r(B, HV)
            kw = {'q': tq[:, None], 'k': tk[:, None], 'v': tv[:, None], 'g': ta[:, None], 'beta': tb[:, None],
                  'A_log': torch.zeros(HV), 'dt_bias': torch.zeros(HV), 'use_gate_in_kernel': True,
                  'use_beta_sigmoid_in_kernel': True, 'use_qk_l2norm_in_kernel': True, 'scale': D ** -0.5}
            x = GDN.inputs(kw)

            def delta(S):
                Sa = x['log_decay'][:, 0].exp()[..., None, None] * S
                u = x['beta'][:, 0][..., None] * (x['v'][:, 0] - torch.einsum('bhkv,bhk->bhv', Sa, x['k'][:, 0]))
                Sn = Sa + x['k'][:, 0][..., None] * u[:, :, None]
                return torch.einsum('bhkv,bhk->bhv', Sn, x['q'][:, 0]), Sn
            pos = torch.full((B,), 3 + t)
            if pw:
                S = ref.prepare(ref._logical(ref.layers[0]), 0, Piece(kw, GDN, 0, None, pos))
                o, Sn = delta(S)
                d = ref.output_delta(0)
                o = o if d is None else o + d[:, 0]
                ref.piece(Sn, 0, Piece(kw, GDN, 0, S, pos, hit=torch.ones(B, dtype=torch.bool)))
                O = ref.layers[0]['O']
                Q = ref.layers[0]['Q']
                P = torch.stack([p for p, _ in Q], 1)                     # [B, n, HV, d_k], oldest first
                V = torch.stack([v_ for _, v_ in Q], 1)
            else:
                o, Sn = delta(O)
                O = qq.quantize(Sn, 0)
                P = V = None
            rec['steps'].append(dict(q=tq, k=tk, v=tv, a=ta, b=tb, o=o.clone(), O=O.clone(), P=P, V=V))
        return rec
    out['steps_pw'] = run(True, 4, 11, 5)
    out['steps_plain'] = run(False, 1, 4, 6)
    save('gga.pt', out)


CASES = {
    'pack.pt': golden_pack,
    # config 1 whole (B4 / HV4 / HK2 / d64, int8 per-row scale, bf16 buffer, zero start): 64 steps, eight folds
    'gdn_c1.pt': lambda: run_gdn('gdn_c1.pt', (8, 'k', 64), 4, 4, 2, 64, 64, 8, 16, 64, seed=1, S0_scale=0.0),
    'gdn_int4.pt': lambda: run_gdn('gdn_int4.pt', (4, 'k', 32), 2, 4, 2, 64, 64, 4, 8, 14, seed=2, v_head_scale=True),
    'gdn_int8_m1.pt': lambda: run_gdn('gdn_int8_m1.pt', (8, 'k', 32), 1, 2, 1, 64, 64, 1, 8, 4, seed=3, per_key=False),
    'gdn_int4v.pt': lambda: run_gdn('gdn_int4v.pt', (4, 'v', 32), 2, 4, 2, 64, 64, 4, 8, 10, seed=8),   # value-axis groups
    'gdn_bf16.pt': lambda: run_gdn('gdn_bf16.pt', 'bf16', 2, 4, 2, 64, 64, 4, 8, 10, seed=9),           # unquantized state
    'kda_int4.pt': lambda: run_kda('kda_int4.pt', (4, 'k', 32), 2, 3, 64, 64, 4, 8, 10, seed=4),
    'kda_int8_bf16buf.pt': lambda: run_kda('kda_int8_bf16buf.pt', (8, 'k', 64), 1, 2, 64, 64, 2, 16, 6, seed=5),
    'm2_int8.pt': lambda: run_m2('m2_int8.pt', (8, 'k', 64), 2, 4, 2, 64, 64, 4, 8, 10, seed=6),
    'm2_int4_bf16buf.pt': lambda: run_m2('m2_int4_bf16buf.pt', (4, 'k', 32), 1, 4, 1, 128, 64, 2, 16, 6, seed=7),
    'slots.pt': golden_slots,
    'gga.pt': golden_gga,
}

if __name__ == '__main__':
    for case in sys.argv[1:] or CASES:          # python tests/golden/make_golden.py [file.pt ...]: those, else all
        CASES[case]()
