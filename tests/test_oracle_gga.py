"""The CPU oracle of the mixed-width GGA / STEP slot (oracle/gga.py) against vectors recorded from the reference's own
torch code (tests/golden/gga.pt, written by tests/golden/make_golden.py) and against what the mathematics fixes."""
import numpy as np
import torch

from oracle import gga as G


def test_fit_bit_exact(golden):
    r = golden('gga.pt')['fit']
    assert torch.equal(G.step_fit(r['x'], r['bits'], r['w']), r['y'])
    # pivots are the fp16 cast; a zero head stays zero
    assert torch.equal(r['y'][:, 4], r['x'][:, 4].half().float())
    assert float(r['y'][1, 5].abs().max()) == 0.0


def test_fp8_vec_bit_exact(golden):
    r = golden('gga.pt')['fp8']
    y = G.fp8_vec(r['x'])
    assert torch.equal(y, r['y'])
    assert float(y[1].abs().max()) == 0.0                             # the zero vector
    code, s = G.fp8_parts(r['x'])
    safe = torch.where(s > 0, s, torch.ones_like(s))
    assert torch.equal(torch.where(s > 0, code.view(torch.float8_e4m3fn).float() * safe, torch.zeros(())), y)


def test_fit_properties():
    """What the fit's definition fixes, whatever the reduction order: codes on the grid, the error of an unclipped
    code within half a step of its row x column scale, two-bit levels in {-3, -1, 1, 3}."""
    g = torch.Generator().manual_seed(3)
    bits = torch.tensor([2, 4, 6, 8])
    w = torch.rand(4, 32, generator=g) + 0.5
    x = torch.randn(3, 4, 32, 64, generator=g)
    rf, c, z, _ = G.fit_parts(x, bits, w)
    qmax = torch.tensor([3., 7., 31., 127.])[None, :, None, None]
    assert bool((z.abs() <= qmax).all()) and bool((z == z.round()).all())
    assert set(z[:, 0].unique().tolist()) <= {-3., -1., 1., 3.}
    inner = (z.abs() < qmax) & (bits != 2)[None, :, None, None]
    err = (x - rf * c * z).abs()
    assert bool((err[inner] <= (0.5 * rf * c).expand_as(x)[inner] * (1 + 1e-5)).all())


def test_tables_and_accounting(golden):
    t = golden('gga.pt')['tables']
    hv, dk, dv, m = t['hv'], t['dk'], t['dv'], t['m']
    for pw in (False, True):
        ref = t[pw]
        tabs = [G.slot_table(wd, dk, dv) for wd in t['widths']]
        assert [o for o, _ in tabs] == ref['offs'] and [n for _, n in tabs] == ref['bytes_per_layer']
        qoff = G._al(max(n for _, n in tabs))
        assert qoff == ref['QOFF'] and G.window_bytes(m, dk, dv) == ref['QSZ']
        assert qoff + (hv * G.window_bytes(m, dk, dv) if pw else 0) == ref['nbytes']
        assert abs(G.bits_per_value(t['widths'], hv, dk, dv, pw, m) - ref['bits_per_value']) < 1e-12
    assert abs(G.bits_per_value(t['widths'], hv, dk, dv, False, m) - t['step_bits']) < 1e-6
    assert abs(G.bits_per_value(t['widths'], hv, dk, dv, True, m) - t['pw_bits']) < 1e-6
    # the widths' closed form: b bits per value + one fp16 per row and column (2 bit: per row group)
    assert G.head_bytes(4, 128, 128) == 128 * 128 // 2 + 2 * 128 + 2 * 128
    assert G.head_bytes(6, 128, 128) == 128 * 128 * 6 // 8 + 512
    assert G.head_bytes(2, 128, 128) == 128 * 128 // 4 + 2 * 128 * 4 + 256
    assert G.head_bytes(16, 128, 128) == 2 * 128 * 128


def _replay(rec):
    """Every step from the reference's own stored state and window; returns the worst output error and the fraction
    of stored values / window entries that differ."""
    B = rec['S0'].shape[0]
    st = G.GGAState(rec['bits'], rec['w'], B + 1, rec['hv'], rec['hk'], rec['dk'], rec['dv'], pw=rec['pw'], m=rec['m'])
    idx = torch.arange(1, B + 1, dtype=torch.int32)
    st.write(idx, rec['S0'])
    assert torch.equal(st.O[1:], rec['O0'])
    worst, flips, total, pflips, ptotal = 0.0, 0, 0, 0, 0
    zero = torch.zeros(rec['hv'])
    for t, s in enumerate(rec['steps']):
        g, beta = st.gate(s['a'], s['b'], zero, zero)
        o = st.step(idx, s['q'], s['k'], s['v'], rec['scale'], g, beta)
        worst = max(worst, ((o - s['o']).norm() / s['o'].norm()).item())
        flips += (st.O[1:] != s['O']).sum().item()
        total += s['O'].numel()
        if rec['pw']:
            n = s['P'].shape[1]
            assert st.n[1:].tolist() == [n] * B, t
            pflips += (st.P[1:, :n] != s['P']).sum().item() + (st.V[1:, :n] != s['V']).sum().item()
            ptotal += s['P'].numel() + s['V'].numel()
            st.P[1:, :n], st.V[1:, :n] = s['P'], s['V']
        st.O[1:] = s['O']                                               # adopt the reference's state
    return worst, flips / total, pflips / max(ptotal, 1)


def test_steps_follow_the_reference_path(golden):
    """The reference path sums in another association (it forms the logical state O + sum p v^T and applies the
    delta rule to it, the slot step keeps the parts apart), so outputs agree to float rounding and a stored code may
    flip where a value sits on a rounding threshold -- the tolerances of the reference's own comparison of the two
    (tests/test_vllm_gga.py:86-89 there: 2e-5 on outputs, < 1e-3 of the stored values off)."""
    for name in ('steps_plain', 'steps_pw'):
        worst, flips, pflips = _replay(golden('gga.pt')[name])
        assert worst < 2e-5, (name, worst)
        assert flips < 1e-3, (name, flips)
        assert pflips < 1e-3, (name, pflips)


def test_step_without_roundings_is_the_textbook_rule():
    """Identity roundings: the logical state (stored + window) follows the gated delta rule token by token, through
    fill, eviction and padding rows -- catches a wrong ring order, a dropped propagation, a transposed pair."""
    g = torch.Generator().manual_seed(11)
    B, HV, HK, D = 3, 4, 2, 16
    ident = lambda x: x.float()                                        # noqa: E731
    st = G.GGAState(torch.tensor([4, 4, 2, 8]), torch.ones(HV, D), 6, HV, HK, D, D, pw=True, m=3, quant=ident, enc=ident)
    idx = torch.tensor([4, 0, 2], dtype=torch.int32)
    S = torch.randn(B, HV, D, D, generator=g) * 0.3
    st.write(idx[[0, 2]], S[[0, 2]])
    keep = st.O[0].clone()
    for t in range(9):
        q, k = torch.randn(B, HK, D, generator=g), torch.randn(B, HK, D, generator=g)
        v = torch.randn(B, HV, D, generator=g)
        gl, beta = -torch.rand(B, HV, generator=g), torch.rand(B, HV, generator=g)
        o = st.step(idx, q, k, v, D ** -0.5, gl, beta)
        o_ref, S = G.textbook_step(S, q, k, v, gl, beta, D ** -0.5, HV // HK)
        assert torch.allclose(o[[0, 2]], o_ref[[0, 2]], atol=1e-5, rtol=1e-5), t
        assert float(o[1].abs().max()) == 0.0
        assert torch.allclose(st.read(idx[[0, 2]]), S[[0, 2]], atol=1e-5, rtol=1e-5), t
        assert st.n[[4, 2]].tolist() == [min(t + 1, 3)] * 2
    assert torch.equal(st.O[0], keep) and int(st.n[0]) == 0            # slot 0 (padding) untouched


def test_pack_unpack_every_width():
    g = torch.Generator().manual_seed(5)
    dk, dv = 32, 64
    for b in (2, 4, 6, 8):
        qmax = 3 if b == 2 else 2 ** (b - 1) - 1
        if b == 2:
            z = torch.randint(0, 4, (dk, dv), generator=g).float() * 2 - 3
            r = torch.rand(dk, dv // 32, generator=g).half().float()
        else:
            z = torch.randint(-qmax, qmax + 1, (dk, dv), generator=g).float()
            r = torch.rand(dk, generator=g).half().float()
        c = torch.rand(dv, generator=g).half().float()
        raw = G.pack_head(r, c, z, b)
        assert raw.size == G.head_bytes(b, dk, dv)
        rf = r.repeat_interleave(32, 1) if b == 2 else r[:, None]
        assert np.array_equal(G.unpack_head(raw, b, dk, dv), ((rf * c[None, :]) * z).numpy())
        # bit positions, by brute force on one row: value j of a row sits at bit j * b of the row's little-endian bits
        u = ((z + 3) / 2 if b == 2 else z + qmax).long()
        row = raw[:dv * b // 8]
        bitstr = int.from_bytes(row.tobytes(), 'little')
        if b == 6:                                                      # 4 values per 3 bytes, each group little-endian
            got = [(int.from_bytes(row[3 * (j // 4):3 * (j // 4) + 3].tobytes(), 'little') >> (6 * (j % 4))) & 63
                   for j in range(dv)]
        else:
            got = [(bitstr >> (j * b)) & ((1 << b) - 1) for j in range(dv)]
        assert got == u[0].tolist()
    x = torch.randn(dk, dv, generator=g)
    raw = G.pack_head(None, None, x, 16)
    assert np.array_equal(G.unpack_head(raw, 16, dk, dv), x.half().float().numpy())
