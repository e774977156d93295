"""The oracle's buffered algebra against the textbook recurrences, written out here in float64 numpy: with nothing
rounded (state kept as fp32 -- the references' ``Identity()`` -- and an fp32 buffer) m buffered tokens + a fold must
equal one rank-1 update per token.  A dropped decay, a wrong sign of the delta term, a transposed state or a buffer
slot read in the wrong order fails these (the reference checks its own torch classes the same way:
/root/reference/tests/test_kda_kernels.py:115-130, tests/test_mamba2.py:136-153 there)."""
import numpy as np
import pytest
import torch

from oracle import states as ST


def l2n(x):
    return x / np.sqrt((x * x).sum(-1, keepdims=True) + 1e-6)


def f64(t):
    return t.double().numpy()


@pytest.mark.parametrize('hv,hk,dk,dv,m', [(4, 2, 64, 64, 8), (6, 2, 96, 192, 4), (3, 3, 32, 64, 1)])
def test_gdn_identity_oracle_is_the_gated_delta_rule(hv, hk, dk, dv, m):
    gen = torch.Generator().manual_seed(1)
    B, T, scale = 2, 3 * m + 2, dk ** -0.5
    S0 = torch.randn(B * hv, dv, dk, generator=gen)
    ora = ST.GDNOracle(S0, ST.IDENT, m=m, hv=hv, hk=hk, buffer_bits=32)
    S = f64(S0)                                              # [BH, d_v, d_k]
    worst = 0.0
    for _ in range(T):
        q, k = torch.randn(B * hk, dk, generator=gen), torch.randn(B * hk, dk, generator=gen)
        v = torch.randn(B * hv, dv, generator=gen)
        g, beta = -torch.rand(B * hv, generator=gen), torch.rand(B * hv, generator=gen)
        o = ora.step(q, k, v, g, beta, scale)
        rep = lambda x: np.repeat(f64(x).reshape(B, hk, dk), hv // hk, axis=1).reshape(B * hv, dk)   # noqa: E731
        qn, kn = l2n(rep(q)) * scale, l2n(rep(k))
        S *= np.exp(f64(g))[:, None, None]
        u = f64(beta)[:, None] * (f64(v) - np.einsum('bvk,bk->bv', S, kn))
        S += u[:, :, None] * kn[:, None, :]
        want = np.einsum('bvk,bk->bv', S, qn)
        worst = max(worst, np.abs(f64(o) - want).max() / np.abs(want).max())
    assert worst < 1e-5, worst
    st = np.abs(f64(ora.state()) - S).max() / np.abs(S).max()
    assert st < 1e-5, st


@pytest.mark.parametrize('h,dk,dv,m', [(4, 64, 64, 8), (3, 64, 32, 4), (2, 128, 256, 2)])
def test_kda_identity_oracle_is_the_per_channel_delta_rule(h, dk, dv, m):
    gen = torch.Generator().manual_seed(2)
    B, T = 2, 3 * m + 2
    S0 = torch.randn(B * h, dv, dk, generator=gen)
    ora = ST.KDAOracle(S0, ST.IDENT, m=m, hv=h, buffer_bits=32)
    S = f64(S0)
    worst = 0.0
    for _ in range(T):
        q, k = torch.randn(B * h, dk, generator=gen), torch.randn(B * h, dk, generator=gen)
        v = torch.randn(B * h, dv, generator=gen)
        g = -torch.nn.functional.softplus(torch.randn(B * h, dk, generator=gen))
        beta = torch.rand(B * h, generator=gen)
        o = ora.step(q, k, v, g, beta)
        qn, kn = l2n(f64(q)) * dk ** -0.5, l2n(f64(k))
        S *= np.exp(f64(g))[:, None, :]                       # one decay per key channel
        u = f64(beta)[:, None] * (f64(v) - np.einsum('bvk,bk->bv', S, kn))
        S += u[:, :, None] * kn[:, None, :]
        want = np.einsum('bvk,bk->bv', S, qn)
        worst = max(worst, np.abs(f64(o) - want).max() / np.abs(want).max())
    assert worst < 1e-5, worst
    st = np.abs(f64(ora.state()) - S).max() / np.abs(S).max()
    assert st < 1e-5, st


@pytest.mark.parametrize('h,g_,dk,dv,m', [(8, 2, 128, 64, 8), (6, 2, 96, 80, 4), (64, 1, 32, 32, 2)])
def test_mamba2_identity_oracle_is_the_ssd_recurrence(h, g_, dk, dv, m):
    gen = torch.Generator().manual_seed(3)
    B, T = 2, 3 * m + 2
    S0 = torch.randn(B * h, dv, dk, generator=gen)
    ora = ST.Mamba2Oracle(S0, ST.IDENT, m=m, hv=h, hk=g_, buffer_bits=32)
    S = f64(S0)
    A, D, dtb = -torch.exp(torch.rand(h, generator=gen) * 2), torch.randn(h, generator=gen), torch.randn(h, generator=gen) * 0.3
    worst = 0.0
    for _ in range(T):
        x = torch.randn(B, h, dv, generator=gen)
        dt = torch.randn(B, h, generator=gen) * 0.5 - 2
        Bm, Cm = torch.randn(B, g_, dk, generator=gen), torch.randn(B, g_, dk, generator=gen)
        y = ora.step(x, dt, Bm, Cm, A, D, dtb, True, None)
        dt64 = np.log1p(np.exp(f64(dt) + f64(dtb)[None]))     # softplus(dt + dt_bias)
        rep = lambda z: np.repeat(f64(z), h // g_, axis=1).reshape(B * h, dk)      # noqa: E731
        Bh, Ch = rep(Bm), rep(Cm)
        dA = np.exp(dt64 * f64(A)[None]).reshape(B * h)
        S *= dA[:, None, None]
        S += (dt64.reshape(B * h, 1) * f64(x).reshape(B * h, dv))[:, :, None] * Bh[:, None, :]
        want = np.einsum('bvk,bk->bv', S, Ch) + np.tile(f64(D), B)[:, None] * f64(x).reshape(B * h, dv)
        worst = max(worst, np.abs(f64(y) - want).max() / np.abs(want).max())
    assert worst < 1e-5, worst
    st = np.abs(f64(ora.state()) - S).max() / np.abs(S).max()
    assert st < 1e-5, st


# ---------------------------------------------------------------------------------------------------------------
# The stand-alone helpers the GPU tests check against: the gates and the three one-line textbook recurrences.
# Each is compared with an independent formulation (torch's library softplus / sigmoid for the gates, float64 numpy
# for the recurrences), on inputs chosen so that a dropped term, a wrong sign or a wrong threshold fails.
# ---------------------------------------------------------------------------------------------------------------
def _gate_inputs():
    gen = torch.Generator().manual_seed(11)
    hv = 6
    # a + dt_bias on both sides of softplus' pass-through threshold (20), large negatives, and exactly 20
    a = torch.tensor([-30.0, -3.0, 0.0, 2.5, 19.0, 19.999, 20.0, 20.001, 21.0, 35.0])[:, None].repeat(1, hv)
    a = a + torch.randn(a.shape, generator=gen) * 1e-3
    a[6] = 20.0
    dt_bias = torch.tensor([0.0, 0.75, -1.5, 3.0, -0.25, 1.0])
    a[6] = a[6] - dt_bias                                      # row 6: a + dt_bias == 20 exactly (<= branch)
    b = torch.randn(a.shape, generator=gen) * 3
    A_log = torch.tensor([-2.0, -0.5, 0.0, 0.3, 1.0, 2.0])
    return a, b, A_log, dt_bias


def test_gdn_gate_is_minus_exp_A_softplus_and_sigmoid():
    """_fused_triton.py:96-100 / families.py:195-202 there: g = -exp(A_log) softplus(a + dt_bias) with softplus
    passed through above 20, beta = sigmoid(b)."""
    a, b, A_log, dt_bias = _gate_inputs()
    g, beta = ST.gdn_gate(a, b, A_log, dt_bias)
    sp = torch.nn.functional.softplus(a + dt_bias, beta=1.0, threshold=20.0)
    want = -torch.exp(A_log) * sp
    assert g.shape == a.shape and beta.shape == b.shape
    # the reference's device code forms log(1 + exp(x)) in fp32 as written: 1 + exp(x) is rounded to 2^-24, so the
    # comparison with the library softplus carries an absolute term of that size (times exp(A_log))
    assert ((g - want).abs() <= 2e-6 * want.abs() + 1.5e-7 * torch.exp(A_log)).all()
    assert torch.allclose(beta, torch.sigmoid(b), rtol=1e-6, atol=0)
    # float64, written out: the threshold matters (softplus(21) != 21 by 7.6e-10 -- invisible -- but the sign, the
    # exp(A_log) factor and dt_bias are not)
    x = f64(a) + f64(dt_bias)[None]
    want64 = -np.exp(f64(A_log))[None] * np.where(x <= 20.0, np.log1p(np.exp(x)), x)
    assert np.abs(f64(g) - want64).max() / np.abs(want64).max() < 1e-6
    assert (g <= 0).all() and (g[1:] < 0).all()
    row = f64(g)[6] / -np.exp(f64(A_log))                    # x = 20: both branches agree to 1e-10
    assert np.allclose(row, np.log1p(np.exp(20.0)), rtol=1e-6)
    # each ingredient is live: dropping dt_bias / A_log or flipping the sign moves the result far past the bound
    for wrong in (ST.gdn_gate(a, b, A_log, torch.zeros_like(dt_bias))[0],
                  ST.gdn_gate(a, b, torch.zeros_like(A_log), dt_bias)[0], -g):
        assert np.abs(f64(wrong) - want64).max() / np.abs(want64).max() > 1e-2


def test_gga_gate_with_nonzero_parameters():
    """vllm_gga.py's gate there (the same formula as the GDN one, with torch's default softplus threshold 20)."""
    from oracle import gga as G
    a, b, A_log, dt_bias = _gate_inputs()
    g, beta = G.GGAState.gate(a, b, A_log, dt_bias)
    x = f64(a) + f64(dt_bias)[None]
    want64 = -np.exp(f64(A_log))[None] * np.where(x <= 20.0, np.log1p(np.exp(x)), x)
    assert np.abs(f64(g) - want64).max() / np.abs(want64).max() < 1e-6
    assert np.abs(f64(beta) - 1.0 / (1.0 + np.exp(-f64(b)))).max() < 1e-6
    g2, beta2 = ST.gdn_gate(a, b, A_log, dt_bias)
    assert torch.allclose(g, g2, rtol=2e-6, atol=1e-6) and torch.allclose(beta, beta2, rtol=1e-6, atol=0)
    assert np.abs(f64(G.GGAState.gate(a, b, A_log, torch.zeros_like(dt_bias))[0]) - want64).max() > 1e-2


def test_gdn_recurrence_is_the_gated_delta_rule():
    """kda.py:44-52 there with a scalar decay, per head; q scaled, q / k l2-normalised with eps inside the root."""
    gen = torch.Generator().manual_seed(12)
    BH, dk, dv, scale = 6, 48, 80, 0.37
    S0 = torch.randn(BH, dv, dk, generator=gen)
    S_t, S = S0.clone(), f64(S0)
    for _ in range(5):
        q, k = torch.randn(BH, dk, generator=gen) * 3, torch.randn(BH, dk, generator=gen) * 0.2
        v = torch.randn(BH, dv, generator=gen)
        g, beta = -torch.rand(BH, generator=gen) * 2, torch.rand(BH, generator=gen)
        o = ST.gdn_recurrence(S_t, q, k, v, g, beta, scale)
        qn, kn = l2n(f64(q)) * scale, l2n(f64(k))
        S = S * np.exp(f64(g))[:, None, None]
        u = f64(beta)[:, None] * (f64(v) - np.einsum('bvk,bk->bv', S, kn))
        S = S + u[:, :, None] * kn[:, None, :]
        want = np.einsum('bvk,bk->bv', S, qn)
        assert np.abs(f64(o) - want).max() / np.abs(want).max() < 1e-5
        assert np.abs(f64(S_t) - S).max() / np.abs(S).max() < 1e-5


def test_kda_recurrence_is_the_per_channel_delta_rule():
    """kda.py:44-52 there: one decay per key channel, default scale d_k^-1/2."""
    gen = torch.Generator().manual_seed(13)
    BH, dk, dv = 5, 64, 32
    S0 = torch.randn(BH, dv, dk, generator=gen)
    for scale in (None, 0.61):
        S_t, S = S0.clone(), f64(S0)
        for _ in range(5):
            q, k = torch.randn(BH, dk, generator=gen) * 2, torch.randn(BH, dk, generator=gen)
            v = torch.randn(BH, dv, generator=gen)
            g = -torch.nn.functional.softplus(torch.randn(BH, dk, generator=gen) * 2)
            beta = torch.rand(BH, generator=gen)
            o = ST.kda_recurrence(S_t, q, k, v, g, beta, scale)
            qn, kn = l2n(f64(q)) * (dk ** -0.5 if scale is None else scale), l2n(f64(k))
            S = S * np.exp(f64(g))[:, None, :]
            u = f64(beta)[:, None] * (f64(v) - np.einsum('bvk,bk->bv', S, kn))
            S = S + u[:, :, None] * kn[:, None, :]
            want = np.einsum('bvk,bk->bv', S, qn)
            assert np.abs(f64(o) - want).max() / np.abs(want).max() < 1e-5
            assert np.abs(f64(S_t) - S).max() / np.abs(S).max() < 1e-5


@pytest.mark.parametrize('softplus,limit,with_D,with_bias', [(True, None, True, True), (False, None, False, False),
                                                             (True, (0.05, 0.2), True, False)])
def test_mamba2_recurrence_is_the_ssd_step(softplus, limit, with_D, with_bias):
    """mamba2.py:57-70 with the gate of mamba2.py:45-54 there: dt (+ bias) -> softplus above-20 pass-through ->
    clamp; S <- exp(A dt) S + (dt x) B^T; y = S C (+ D x); B / C shared by the heads of a group."""
    gen = torch.Generator().manual_seed(14)
    Bsz, H, G_, dk, dv = 2, 6, 2, 32, 24
    S0 = torch.randn(Bsz, H, dv, dk, generator=gen)
    S_t, S = S0.clone(), f64(S0)
    A = -torch.exp(torch.rand(H, generator=gen) * 2)
    D = torch.randn(H, generator=gen) if with_D else None
    dtb = torch.randn(H, generator=gen) * 0.5 if with_bias else None
    for t in range(5):
        x = torch.randn(Bsz, H, dv, generator=gen)
        dt = torch.randn(Bsz, H, generator=gen) * 0.5 - 2 if softplus else torch.rand(Bsz, H, generator=gen) * 0.3
        if softplus and t == 2:
            dt[0, 0] = 25.0                                   # above the softplus threshold
        Bm, Cm = torch.randn(Bsz, G_, dk, generator=gen), torch.randn(Bsz, G_, dk, generator=gen)
        y = ST.mamba2_recurrence(S_t, x, dt, Bm, Cm, A, D, dtb, softplus, limit)
        d = f64(dt) + (f64(dtb)[None] if with_bias else 0.0)
        if softplus:
            d = np.where(d <= 20.0, np.log1p(np.exp(d)), d)
        if limit is not None:
            d = np.clip(d, *limit)
        Bh, Ch = np.repeat(f64(Bm), H // G_, axis=1), np.repeat(f64(Cm), H // G_, axis=1)
        S = S * np.exp(d * f64(A)[None])[..., None, None]
        S = S + (d[..., None] * f64(x))[..., :, None] * Bh[..., None, :]
        want = np.einsum('bhvk,bhk->bhv', S, Ch)
        if with_D:
            want = want + f64(D)[None, :, None] * f64(x)
        assert np.abs(f64(y) - want).max() / np.abs(want).max() < 1e-5
        assert np.abs(f64(S_t) - S).max() / np.abs(S).max() < 1e-5
