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
