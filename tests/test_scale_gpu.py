"""The Gated DeltaNet step at the benchmark's full size and under HIP-graph replay.

Full size (32 value / 16 key heads, d = 128, 256 slots, the headline configuration): the oracle is far too slow for
8192 state tiles, so the run is checked through (i) a subset of slots against the oracle, (ii) a property that does
not depend on size -- batch rows r and r + 128 get the same initial state and the same inputs, so their slots must end
byte-identical and their outputs equal whichever tile, compute unit or XCD processed them -- and (iii) the counters of
every slot.  Graph replay: a captured fold period replayed several times, with eager work and synchronisation between
the replays, must leave exactly the bytes an eagerly stepped twin holds.
"""
import pytest
import torch

import statequant_amd as sq
from oracle import states as ST
from statequant_amd.kernels import SlotLayout
from tests._util import SlotSync, gdn_token

pytestmark = pytest.mark.gpu
DEV = 'cuda'


@pytest.mark.parametrize('fmt,warm', [((8, 'k', 128), 0), ((4, 'k', 32), 0), ((8, 'k', 128), 64)])
def test_full_size_subset_and_twin_rows(fmt, warm):
    """warm = 0: states written from fp32 (``write``).  warm = 64: the benchmark's situation -- every slot starts at
    zero and has been through 64 kernel steps (8 folds) before the comparison begins; the oracle then takes over the
    slots' codes and scales (the buffers are empty at a multiple of m) and follows for two more fold periods."""
    HV, HK, D, m, slots = 32, 16, 128, 8, 256
    lay = SlotLayout(sq.Quantizer(*fmt), HV, HK, D, D, m=m, buffer_bits=8)
    views = lay.views(lay.alloc(slots + 1, DEV))
    gen = torch.Generator().manual_seed(3)
    half = slots // 2
    perm = (torch.randperm(slots, generator=gen) + 1)
    idx = perm.to(torch.int32).to(DEV)                                    # row r works on slot perm[r]
    two = lambda x: torch.cat([x, x]).to(DEV)                             # noqa: E731
    check_rows = [0, 57, 127]                                             # rows checked against the oracle
    sl = idx[check_rows]
    if warm:
        for t in range(warm):
            q, k, v, g, beta = gdn_token(gen, half, HV, HK, D, D)
            out = torch.empty(slots, HV, D, device=DEV)
            lay.step(views, idx, two(q), two(k), two(v), out, D ** -0.5, g=two(g), beta=two(beta))
        assert int(views['NPTR'][idx.long(), :HV].abs().max()) == 0 and torch.isfinite(out).all()
        ref = ST.GDNOracle(torch.zeros(len(check_rows) * HV, D, D), fmt, m=m, hv=HV, hk=HK, buffer_bits=8, auto_fold=False)
        ref.adopt(views['S'][sl.long()].cpu().reshape(ref.codes.shape), views['SC'][sl.long()].cpu().reshape(ref.scales.shape))
        assert float(ref.S0.abs().max()) > 0.1                            # a state worth the name
    else:
        S_half = torch.randn(half, HV, D, D, generator=gen) * 0.3          # value-major; rows r, r + half share it
        lay.write(views, idx[:half].long(), S_half.to(DEV))
        lay.write(views, idx[half:].long(), S_half.to(DEV))
        ref = ST.GDNOracle(S_half[check_rows].reshape(-1, D, D), fmt, m=m, hv=HV, hk=HK, buffer_bits=8, auto_fold=False)
    sync = SlotSync(views, sl, ref, fmt[0])
    steps = 2 * m + 2                                                     # through two folds and two tokens beyond
    for t in range(steps):
        q, k, v, g, beta = gdn_token(gen, half, HV, HK, D, D)
        out = torch.full((slots, HV, D), 7.0, device=DEV)
        lay.step(views, idx, two(q), two(k), two(v), out, D ** -0.5, g=two(g), beta=two(beta))
        got = out.cpu()
        assert torch.equal(got[:half], got[half:]), f'twin rows differ at step {t}'
        i = ref.n
        want = ref.step(q[check_rows].reshape(-1, D), k[check_rows].reshape(-1, D), v[check_rows].reshape(-1, D),
                        g[check_rows].reshape(-1), beta[check_rows].reshape(-1), D ** -0.5)
        sync.after_step(got[check_rows].reshape(want.shape), want, i)
        n = (t + 1) % m
        assert torch.equal(views['NPTR'][idx.long(), :HV].cpu(), torch.full((slots, HV), n, dtype=torch.int32))
    sync.verdict(f'gdn {fmt} full size, {"after 64 kernel steps" if warm else "from written states"}')
    for f in ('S', 'SC', 'GCUR'):
        a, b = views[f][idx[:half].long()], views[f][idx[half:].long()]
        assert torch.equal(a, b), f
    w = steps % m                                                         # buffer slots written since the last fold
    for f in ('UB', 'KB', 'GB', 'UBS', 'KBS'):
        a, b = views[f][idx[:half].long()][:, :, :w], views[f][idx[half:].long()][:, :, :w]
        assert torch.equal(a, b), f


def test_graph_replay_matches_eager():
    HV, HK, D, m, slots = 8, 4, 128, 4, 6
    fmt = (8, 'k', 64)
    lay = SlotLayout(sq.Quantizer(*fmt), HV, HK, D, D, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(5)
    S0 = (torch.randn(slots, HV, D, D, generator=gen) * 0.4).to(DEV)
    idx = torch.arange(1, slots + 1, dtype=torch.int32, device=DEV)
    blobs = [lay.alloc(slots + 1, DEV) for _ in range(2)]                 # [0] graph, [1] eager twin
    views = [lay.views(b) for b in blobs]
    for v in views:
        lay.write(v, idx.long(), S0)
    toks = [[x.to(DEV) for x in gdn_token(gen, slots, HV, HK, D, D)] for _ in range(m)]
    outs = [[torch.zeros(slots, HV, D, device=DEV) for _ in range(m)] for _ in range(2)]

    def period(which):
        for s, (q, k, v, g, beta) in enumerate(toks):
            lay.step(views[which], idx, q, k, v, outs[which][s], D ** -0.5, g=g, beta=beta)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        period(0)                                                         # warm-up, eager, on the capture stream
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            period(0)
    torch.cuda.synchronize()
    period(1)                                                             # twin: the warm-up period
    for rep in range(3):
        graph.replay()
        period(1)
        torch.cuda.synchronize()
        scratch = torch.randn(1 << 20, device=DEV).sum().item()           # unrelated eager work between replays
        assert scratch == scratch
        assert torch.equal(blobs[0], blobs[1]), f'state differs after replay {rep}'
        for s in range(m):
            assert torch.equal(outs[0][s], outs[1][s]), (rep, s)


def _replay_with_changing_slot_tables(lay, call, feed, S0, tables, idx, rounds=5):
    """Capture ONE padded-batch step, replay it with the slot table and the inputs rewritten in place between replays
    (padding rows at the null slot and at -1, sequences whose counters diverge), next to an eager twin on a second
    blob; blobs and outputs must stay bit-identical (the reference's graph tests: tests/test_kda_kernels.py:313-345,
    tests/test_mamba2.py:350-385 there)."""
    blobs = [lay.alloc(8, DEV) for _ in range(2)]
    views = [lay.views(b) for b in blobs]
    live = torch.tensor(sorted({s for t in tables for s in t if s > 0}), device=DEV)
    for v in views:
        lay.write(v, live, S0[:len(live)])
    outs = [torch.zeros_like(feed(None)) for _ in range(2)]
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        call(views[0], outs[0])                              # warm-up on the capture stream: idx all padding
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            call(views[0], outs[0])
    torch.cuda.synchronize()
    gen = torch.Generator(device=DEV).manual_seed(5)
    for r, tab in enumerate(tables * rounds):
        idx.copy_(torch.tensor(tab, dtype=torch.int32))
        feed(gen)
        graph.replay()
        call(views[1], outs[1])
        torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]), (r, tab)
        assert torch.equal(blobs[0], blobs[1]), (r, tab)
    n = views[0]['NPTR'][live, 0].tolist()
    assert len(set(n)) > 1, n                                # the sequences really were out of step


TABLES = [[5, 2, 7, 0], [2, 0, -1, 0], [7, 5, 0, 0], [5, 7, 2, -1], [0, 0, 5, 0]]


@pytest.mark.parametrize('fmt', [(4, 'k', 64), (8, 'v', 32), 'bf16'])
def test_kda_graph_replay_with_changing_slot_tables(fmt):
    from statequant_amd.kernels import KDASlotLayout
    H, K, Vd, R = 4, 128, 128, 4
    lay = KDASlotLayout(fmt if fmt == 'bf16' else sq.Quantizer(*fmt), H, K, Vd, m=4, buffer_bits=8)
    idx = torch.zeros(R, device=DEV, dtype=torch.int32)
    proj = torch.zeros(R, 2 * H * K + H * Vd, device=DEV, dtype=torch.bfloat16)   # q / k / v: slices of one projection
    q, k, v = proj[:, :H * K].view(R, H, K), proj[:, H * K:2 * H * K].view(R, H, K), proj[:, 2 * H * K:].view(R, H, Vd)
    g, beta = torch.zeros(R, H, K, device=DEV), torch.zeros(R, H, device=DEV)

    def feed(gen):
        if gen is not None:
            proj.copy_(torch.randn(proj.shape, device=DEV, generator=gen))
            g.copy_(-5 * torch.sigmoid(torch.randn(g.shape, device=DEV, generator=gen) * 2 - 3))
            beta.copy_(torch.sigmoid(torch.randn(beta.shape, device=DEV, generator=gen)))
        return torch.zeros(R, H, Vd, device=DEV, dtype=torch.bfloat16)

    S0 = torch.randn(3, H, Vd, K, device=DEV) * 0.4
    _replay_with_changing_slot_tables(lay, lambda vw, o: lay.step(vw, idx, q, k, v, g, beta, o), feed, S0, TABLES, idx)


@pytest.mark.parametrize('fmt,P', [((8, 'k', 128), 64), ((4, 'k', 32), 80), ('bf16', 64)])
def test_mamba2_graph_replay_with_changing_slot_tables(fmt, P):
    from statequant_amd.kernels import Mamba2SlotLayout
    H, G, N, R = 8, 2, 128, 4
    lay = Mamba2SlotLayout(fmt if fmt == 'bf16' else sq.Quantizer(*fmt), H, G, N, P, m=4, buffer_bits=8)
    idx = torch.zeros(R, device=DEV, dtype=torch.int32)
    x = torch.zeros(R, H, P, device=DEV, dtype=torch.bfloat16)
    dt = torch.zeros(R, H, device=DEV)
    Bm, Cm = torch.zeros(R, G, N, device=DEV), torch.zeros(R, G, N, device=DEV)
    A = -torch.exp(torch.rand(H, device=DEV) * 2)
    D, dtb = torch.randn(H, device=DEV), torch.randn(H, device=DEV) * 0.3

    def feed(gen):
        if gen is not None:
            x.copy_(torch.randn(x.shape, device=DEV, generator=gen))
            dt.copy_(torch.randn(dt.shape, device=DEV, generator=gen) * 0.5 - 2)
            Bm.copy_(torch.randn(Bm.shape, device=DEV, generator=gen))
            Cm.copy_(torch.randn(Cm.shape, device=DEV, generator=gen))
        return torch.zeros(R, H, P, device=DEV)

    S0 = torch.randn(3, H, P, N, device=DEV) * 0.4
    _replay_with_changing_slot_tables(lay, lambda vw, o: lay.step(vw, idx, x, dt, Bm, Cm, o, A, D, dtb), feed, S0,
                                      TABLES, idx)
