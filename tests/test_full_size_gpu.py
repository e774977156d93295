"""The Mamba2 and KDA steps at the benchmark configurations' full sizes, the ragged KDA variant with padding rows, and
the PACE-4 Gated DeltaNet configuration (d 128, int4 groups of 32, values scaled per head).

Full sizes are far beyond what the oracle steps in seconds, so -- as tests/test_scale_gpu.py does for the headline --
a run is checked through (i) a subset of its rows against the oracle, (ii) a size-independent property: batch rows r
and r + rows / 2 get the same state and the same inputs, so their slots must end byte-identical and their outputs equal
whichever tile, compute unit or XCD processed them, and (iii) the counters of every slot.  Mirrors the reference's
slot-step tests (tests/test_mamba2.py:273-300, tests/test_kda_kernels.py:238-265 there).
"""
import pytest
import torch

import statequant_amd as sq
from oracle import states as ST
from statequant_amd.kernels import KDASlotLayout, Mamba2SlotLayout
from tests._util import SlotSync
from tests.test_gdn_gpu import check as check_gdn, run_decode as run_gdn
from tests.test_kda_gpu import kda_token
from tests.test_mamba2_gpu import m2_token, params

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _twins_equal(views, idx, half, live=None, written=2):
    a_idx, b_idx = idx[:half].long(), idx[half:].long()
    if live is not None:
        a_idx, b_idx = a_idx[live], b_idx[live]
    for f in ('S', 'SC', 'GCUR', 'NPTR'):
        assert torch.equal(views[f][a_idx], views[f][b_idx]), f
    for f in ('UB', 'KB', 'GB', 'UBS', 'KBS'):                  # the buffer slots written since the fold
        assert torch.equal(views[f][a_idx][:, :, :written], views[f][b_idx][:, :, :written]), f


def test_mamba2_full_size_subset_and_twin_rows():
    """128 heads / 8 groups, head_dim 64, d_state 128, 128 slots, int8 state with one scale per (head, row)."""
    H, G, DK, DV, m, slots = 128, 8, 128, 64, 8, 128
    fmt = (8, 'k', 128)
    lay = Mamba2SlotLayout(sq.Quantizer(*fmt), H, G, DK, DV, m=m, buffer_bits=8)
    views = lay.views(lay.alloc(slots + 1, DEV))
    gen = torch.Generator().manual_seed(11)
    half = slots // 2
    idx = (torch.randperm(slots, generator=gen) + 1).to(torch.int32).to(DEV)
    S_half = torch.randn(half, H, DV, DK, generator=gen) * 0.5
    lay.write(views, idx[:half].long(), S_half.to(DEV))
    lay.write(views, idx[half:].long(), S_half.to(DEV))
    A, D, dtb = params(gen, H)
    rows = [0, 29, 63]
    ref = ST.Mamba2Oracle(S_half[rows].reshape(-1, DV, DK), fmt, m=m, hv=H, hk=G, buffer_bits=8, auto_fold=False)
    sync = SlotSync(views, idx[rows], ref, 8, exact_decay=False)
    two = lambda x: torch.cat([x, x]).to(DEV)              # noqa: E731
    steps = 2 * m + 2                                       # through two folds and two tokens beyond
    for t in range(steps):
        x, dt, Bm, C = m2_token(gen, half, H, G, DK, DV)
        out = torch.full((slots, H, DV), 7.0, device=DEV)
        lay.step(views, idx, two(x), two(dt), two(Bm), two(C), out, A.to(DEV), D.to(DEV), dtb.to(DEV))
        got = out.cpu()
        assert torch.equal(got[:half], got[half:]), f'twin rows differ at step {t}'
        i = ref.n
        want = ref.step(x[rows], dt[rows], Bm[rows], C[rows], A, D, dtb, True, (0., float('inf')))
        sync.after_step(got[rows].reshape(want.shape), want, i)
        assert torch.equal(views['NPTR'][idx.long(), :H].cpu(), torch.full((slots, H), (t + 1) % m, dtype=torch.int32))
    sync.verdict('mamba2 full size')
    _twins_equal(views, idx, half, written=steps % m)


def test_kda_full_size_subset_and_twin_rows():
    """32 heads, d_k = d_v = 128, 256 slots, int4 state in groups of 32."""
    H, D, m, slots = 32, 128, 8, 256
    fmt = (4, 'k', 32)
    lay = KDASlotLayout(sq.Quantizer(*fmt), H, D, D, m=m, buffer_bits=8)
    views = lay.views(lay.alloc(slots + 1, DEV))
    gen = torch.Generator().manual_seed(12)
    half = slots // 2
    idx = (torch.randperm(slots, generator=gen) + 1).to(torch.int32).to(DEV)
    S_half = torch.randn(half, H, D, D, generator=gen) * 0.5
    lay.write(views, idx[:half].long(), S_half.to(DEV))
    lay.write(views, idx[half:].long(), S_half.to(DEV))
    rows = [0, 57, 127]
    ref = ST.KDAOracle(S_half[rows].reshape(-1, D, D), fmt, m=m, hv=H, buffer_bits=8, auto_fold=False)
    sync = SlotSync(views, idx[rows], ref, 4)
    two = lambda x: torch.cat([x, x]).to(DEV)              # noqa: E731
    flat = lambda x: x[rows].reshape(len(rows) * H, *x.shape[2:])          # noqa: E731
    steps = 2 * m + 2
    for t in range(steps):
        q, k, v, g, beta = kda_token(gen, half, H, D, D)
        out = torch.full((slots, H, D), 7.0, device=DEV)
        lay.step(views, idx, two(q), two(k), two(v), two(g), two(beta), out)
        got = out.cpu()
        assert torch.equal(got[:half], got[half:]), f'twin rows differ at step {t}'
        i = ref.n
        want = ref.step(flat(q), flat(k), flat(v), flat(g), flat(beta))
        sync.after_step(got[rows].reshape(want.shape), want, i)
        assert torch.equal(views['NPTR'][idx.long(), :H].cpu(), torch.full((slots, H), (t + 1) % m, dtype=torch.int32))
    sync.verdict('kda full size')
    _twins_equal(views, idx, half, written=steps % m)


def test_kda_ragged_variant_with_padding_rows():
    """20 heads, d_k = d_v = 96 (neither a power of two), 256 batch rows of which about 40 % are padding (slot index
    0 or -1): padding rows give zeros and touch nothing, live rows behave as in the dense run."""
    H, D, m, nrows = 20, 96, 8, 256
    fmt = (4, 'k', 32)
    lay = KDASlotLayout(sq.Quantizer(*fmt), H, D, D, m=m, buffer_bits=8)
    blob = lay.alloc(nrows + 1, DEV)
    views = lay.views(blob)
    gen = torch.Generator().manual_seed(13)
    half = nrows // 2
    slot = torch.randperm(nrows, generator=gen) + 1
    dead = torch.rand(half, generator=gen) < 0.4                            # the same rows in both halves
    dead[[0, 57]] = False                                                   # rows checked against the oracle stay live
    pad = torch.where(torch.rand(half, generator=gen) < 0.5, 0, -1)
    slot[:half][dead], slot[half:][dead] = pad[dead], pad[dead]
    idx = slot.to(torch.int32).to(DEV)
    live = ~dead
    assert 0.3 < dead.float().mean().item() < 0.5
    S_half = torch.randn(half, H, D, D, generator=gen) * 0.5
    lay.write(views, idx[:half][live].long(), S_half[live].to(DEV))
    lay.write(views, idx[half:][live].long(), S_half[live].to(DEV))
    untouched = torch.ones(nrows + 1, dtype=torch.bool)
    untouched[slot[slot > 0]] = False                                       # slot 0 and the slots no row points at
    before = blob[untouched.to(DEV)].clone()
    rows = [0, 57]
    ref = ST.KDAOracle(S_half[rows].reshape(-1, D, D), fmt, m=m, hv=H, buffer_bits=8, auto_fold=False)
    sync = SlotSync(views, idx[rows], ref, 4)
    two = lambda x: torch.cat([x, x]).to(DEV)              # noqa: E731
    flat = lambda x: x[rows].reshape(len(rows) * H, *x.shape[2:])          # noqa: E731
    steps = 2 * m + 2
    for t in range(steps):
        q, k, v, g, beta = kda_token(gen, half, H, D, D)
        out = torch.full((nrows, H, D), 7.0, device=DEV)
        lay.step(views, idx, two(q), two(k), two(v), two(g), two(beta), out)
        got = out.cpu()
        assert torch.equal(got[:half], got[half:]), f'twin rows differ at step {t}'
        assert torch.equal(got[:half][dead], torch.zeros(int(dead.sum()), H, D)), 'padding rows must give zeros'
        i = ref.n
        want = ref.step(flat(q), flat(k), flat(v), flat(g), flat(beta))
        sync.after_step(got[rows].reshape(want.shape), want, i)
        n_live = views['NPTR'][idx[:half][live].long(), :H].cpu()
        assert torch.equal(n_live, torch.full((int(live.sum()), H), (t + 1) % m, dtype=torch.int32))
    sync.verdict('kda 20 heads, d 96, 40 % padding rows')
    assert torch.equal(blob[untouched.to(DEV)], before), 'a padding row wrote to a slot'
    _twins_equal(views, idx, half, live=live.to(DEV), written=steps % m)


@pytest.mark.parametrize('m,bb', [(8, 8), (8, 16)])
def test_gdn_pace4_d128_values_scaled_per_head(m, bb):
    """The PACE-4 configuration's numerics: d 128, int4 groups of 32, re-encode every 8 tokens, v scaled by a
    per-head log-uniform factor in [0.1, 10] (outlier channels), against the oracle step by step."""
    HV, T = 4, 5 * m
    vs = torch.exp(torch.empty(HV).uniform_(-2.302585, 2.302585, generator=torch.Generator().manual_seed(21)))
    assert vs.max() / vs.min() > 3

    tal = run_gdn((4, 'k', 32), m, bb, B=3, HV=HV, HK=2, D=128, T=T, seed=22, v_scale=vs)
    check_gdn(tal, f'gdn pace4 d128 per-head v scale, buf{bb}', T, m)


def _stepped_twice(step, blobs):
    """Run `step(views_index)` on blob 0 with the compiled-in serving case allowed and on blob 1 with it switched off
    (`select_instances(no_specialised=True)`: the general instance, which reads dtypes and options from the
    arguments)."""
    from statequant_amd.kernels import _hip
    a = step(0)
    _hip.select_instances(no_specialised=True)
    try:
        b = step(1)
    finally:
        _hip.select_instances()
    assert torch.equal(a, b)
    assert torch.equal(blobs[0], blobs[1])


@pytest.mark.parametrize('fmt', [(8, 'k', 128), (4, 'k', 32), (4, 'k', 64), (4, 'v', 32), 'bf16'])      # the last two: one wavefront per tile
@pytest.mark.parametrize('gated', [False, True])
def test_gdn_serving_case_instances_match_the_general_one(fmt, gated):
    """bf16 q / k / v / out with fp32 g, beta -- or the gate formed in the kernel from bf16 a, b and fp32 A_log, dt_bias
    -- take kernel instances with those choices compiled in; they must leave exactly the bytes and outputs of the
    general instance (two fold periods, a padding row, slots out of step)."""
    from statequant_amd.kernels import SlotLayout
    HV, HK, D, m, rows = 8, 4, 128, 8, 5
    lay = SlotLayout(fmt if fmt == 'bf16' else sq.Quantizer(*fmt), HV, HK, D, D, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(31)
    blobs = [lay.alloc(rows + 1, DEV) for _ in range(2)]
    views = [lay.views(b) for b in blobs]
    idx = torch.tensor([4, 0, 2, 5, 1], dtype=torch.int32, device=DEV)
    live = idx > 0
    S0 = (torch.randn(rows, HV, D, D, generator=gen) * 0.4).to(DEV)
    for v in views:
        lay.write(v, idx[live].long(), S0[live])
        v['NPTR'][idx[live].long()] = torch.tensor([0, 3, 6, 7], dtype=torch.int32, device=DEV)[:, None]
    A_log, dtb = (torch.randn(HV, generator=gen) * 0.3).to(DEV), (torch.randn(HV, generator=gen) * 0.3).to(DEV)
    r = lambda *s: torch.randn(*s, generator=gen).to(DEV)          # noqa: E731
    for t in range(2 * m + 1):
        q, k, v = r(rows, HK, D).bfloat16(), r(rows, HK, D).bfloat16(), r(rows, HV, D).bfloat16()
        if gated:
            kw = dict(gate=((r(rows, HV) * 0.5 - 2).bfloat16(), r(rows, HV).bfloat16(), A_log, dtb))
        else:
            kw = dict(g=-torch.nn.functional.softplus(r(rows, HV)), beta=torch.sigmoid(r(rows, HV)))

        def step(i):
            out = torch.full((rows, HV, D), 7.0, device=DEV, dtype=torch.bfloat16)
            return lay.step(views[i], idx, q, k, v, out, D ** -0.5, **kw).clone()
        _stepped_twice(step, blobs)


def test_mamba2_serving_case_instance_matches_the_general_one():
    H, G, DK, DV, m, rows = 16, 2, 128, 64, 8, 5
    lay = Mamba2SlotLayout(sq.Quantizer(8, 'k', 128), H, G, DK, DV, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(32)
    blobs = [lay.alloc(rows + 1, DEV) for _ in range(2)]
    views = [lay.views(b) for b in blobs]
    idx = torch.tensor([4, 0, 2, 5, 1], dtype=torch.int32, device=DEV)
    live = idx > 0
    S0 = (torch.randn(rows, H, DV, DK, generator=gen) * 0.4).to(DEV)
    for v in views:
        lay.write(v, idx[live].long(), S0[live])
        v['NPTR'][idx[live].long()] = torch.tensor([0, 3, 6, 7], dtype=torch.int32, device=DEV)[:, None]
    A, D_, dtb = (t.to(DEV) for t in params(gen, H))
    for t in range(2 * m + 1):
        x, dt, Bm, C = m2_token(gen, rows, H, G, DK, DV)
        x, Bm, C, dt = x.bfloat16().to(DEV), Bm.bfloat16().to(DEV), C.bfloat16().to(DEV), dt.to(DEV)

        def step(i):
            out = torch.full((rows, H, DV), 7.0, device=DEV, dtype=torch.bfloat16)
            return lay.step(views[i], idx, x, dt, Bm, C, out, A, D_, dtb).clone()
        _stepped_twice(step, blobs)


@pytest.mark.parametrize('fmt', [(4, 'k', 32), (8, 'v', 32)])
def test_kda_serving_case_instance_matches_the_general_one(fmt):
    H, D, m, rows = 4, 128, 8, 5
    lay = KDASlotLayout(sq.Quantizer(*fmt), H, D, D, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(33)
    blobs = [lay.alloc(rows + 1, DEV) for _ in range(2)]
    views = [lay.views(b) for b in blobs]
    idx = torch.tensor([4, 0, 2, 5, 1], dtype=torch.int32, device=DEV)
    live = idx > 0
    S0 = (torch.randn(rows, H, D, D, generator=gen) * 0.4).to(DEV)
    for v in views:
        lay.write(v, idx[live].long(), S0[live])
        v['NPTR'][idx[live].long()] = torch.tensor([0, 3, 6, 7], dtype=torch.int32, device=DEV)[:, None]
    for t in range(2 * m + 1):
        q, k, v, g, beta = kda_token(gen, rows, H, D, D)
        q, k, v, g, beta = q.bfloat16().to(DEV), k.bfloat16().to(DEV), v.bfloat16().to(DEV), g.to(DEV), beta.to(DEV)

        def step(i):
            out = torch.full((rows, H, D), 7.0, device=DEV, dtype=torch.bfloat16)
            return lay.step(views[i], idx, q, k, v, g, beta, out).clone()
        _stepped_twice(step, blobs)
