"""The optional dispatch order of the step calls (``order``; ``fold_order``) -- an addition with no counterpart in the
reference, so its tests are properties: a step's results do not depend on the order it is dispatched in (bit for bit:
outputs, every byte of the blob), ``fold_order`` returns a permutation that follows its stated placement rule, and
both survive HIP-graph replay next to an eagerly stepped twin.
"""
import pytest
import torch

import statequant_amd as sq
from statequant_amd.kernels import KDASlotLayout, Mamba2SlotLayout, SlotLayout, _hip
from tests._util import gdn_token

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def expected_order(folds):
    """The placement rule of ``fold_order`` restated on the host: ``folds`` [rows] bool -> order [rows]."""
    rows = len(folds)
    F = int(sum(folds))
    R = rows // 8
    if rows % 8 or rows < 64 or F == 0 or 2 * ((F + 7) // 8) > R:
        return list(range(rows))
    per = [F // 8 + (c < F % 8) for c in range(8)]
    order = [None] * rows
    k = 0
    for r in range(rows):                                    # folding rows: dealt round-robin, one after s - 1 others
        if folds[r]:
            c, j = k % 8, k // 8
            s = max(2, R // (4 * per[c]))
            order[c * R + s * j + s - 1] = r
            k += 1
    free = [p for p in range(rows) if order[p] is None]      # the others keep their order
    for p, r in zip(free, [r for r in range(rows) if not folds[r]]):
        order[p] = r
    return order


@pytest.mark.parametrize('rows,m,pattern', [
    (256, 8, 'eighth'), (256, 8, 'random'), (64, 4, 'random'), (128, 8, 'none'), (128, 8, 'all'), (96, 8, 'half'),
    (72, 8, 'two'), (100, 8, 'random'), (48, 8, 'random'), (512, 16, 'random'), (256, 8, 'padding'), (1024, 2, 'third')])
def test_fold_order_follows_its_rule(rows, m, pattern):
    HV, HK, D = 4, 2, 64
    lay = SlotLayout(sq.Quantizer(8, 'k', 64), HV, HK, D, D, m=m, buffer_bits=8)
    views = lay.views(lay.alloc(rows + 1, DEV))
    gen = torch.Generator().manual_seed(rows + m)
    idx = (torch.randperm(rows, generator=gen) + 1).to(torch.int32)
    fill = torch.randint(0, m, (rows,), generator=gen)
    if pattern == 'eighth':
        fill = torch.arange(rows) % m
    elif pattern == 'none':
        fill = fill.clamp(max=m - 2)
    elif pattern == 'all':
        fill[:] = m - 1
    elif pattern == 'half':                                  # every second row folds: the limit of the rule
        fill = torch.where(torch.arange(rows) % 2 == 0, m - 1, 0)
    elif pattern == 'two':
        fill = fill.clamp(max=m - 2)
        fill[[5, 40]] = m - 1
    elif pattern == 'third':
        fill = torch.where(torch.arange(rows) % 3 == 0, m - 1, 0)
    elif pattern == 'padding':
        idx[torch.arange(0, rows, 5)] = 0                    # padding rows never fold, whatever slot 0 holds
        idx[torch.arange(3, rows, 17)] = -1
    views['NPTR'][idx.clamp(min=0).long().to(DEV)] = fill.to(torch.int32).to(DEV)[:, None]
    views['NPTR'][0] = m - 1
    got = lay.fold_order(views, idx.to(DEV)).cpu().tolist()
    folds = [(int(idx[r]) > 0 and int(fill[r]) == m - 1) for r in range(rows)]
    assert sorted(got) == list(range(rows)), 'not a permutation'
    assert got == expected_order(folds)
    if pattern in ('eighth', 'two', 'padding') or (pattern == 'random' and rows % 8 == 0 and rows >= 64):
        assert got != list(range(rows))                      # the rule applied
        R = rows // 8
        per = [sum(folds[r] for r in got[c * R:(c + 1) * R]) for c in range(8)]
        assert max(per) - min(per) <= 1, per                 # evenly over the eight ranges
        if 4 * max(per) <= R:                                # and, up to a quarter of a range, in its first half
            for c in range(8):
                assert not any(folds[r] for r in got[c * R + (R + 1) // 2:(c + 1) * R]), c
    # into a caller's buffer, without allocation
    buf = torch.full((rows + 3,), -7, dtype=torch.int32, device=DEV)
    assert lay.fold_order(views, idx.to(DEV), out=buf) is buf
    assert buf[:rows].cpu().tolist() == got and buf[rows:].eq(-7).all()


def _orders(lay, views, idx, rows, gen):
    yield torch.randperm(rows, generator=gen).to(torch.int32).to(DEV)
    yield lay.fold_order(views, idx)
    yield torch.arange(rows - 1, -1, -1, dtype=torch.int32, device=DEV)


def _mixed_fills(views, idx, m, gen):
    fill = torch.randint(0, m, (idx.shape[0],), generator=gen).to(torch.int32).to(DEV)
    live = idx > 0
    views['NPTR'][idx[live].long()] = fill[live][:, None]


@pytest.mark.parametrize('fmt,no_group', [((8, 'k', 128), False), ((4, 'k', 32), False), ((8, 'k', 128), True),
                                          ((4, 'v', 32), False), ('bf16', False)])
def test_gdn_results_do_not_depend_on_the_order(fmt, no_group):
    HV, HK, D, m, rows = 8, 4, 128, 4, 64
    lay = SlotLayout(fmt if fmt == 'bf16' else sq.Quantizer(*fmt), HV, HK, D, D, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(11)
    idx = (torch.randperm(rows, generator=gen) + 1).to(torch.int32)
    idx[[3, 20]] = 0
    idx[41] = -1
    idx = idx.to(DEV)
    blobs = [lay.alloc(rows + 1, DEV) for _ in range(2)]
    views = [lay.views(b) for b in blobs]
    S0 = (torch.randn(rows, HV, D, D, generator=gen) * 0.4).to(DEV)
    live = idx > 0
    for V in views:
        lay.write(V, idx[live].long(), S0[live])
        _mixed_fills(V, idx, m, torch.Generator().manual_seed(12))
    _hip.select_instances(no_group_kernel=no_group)
    try:
        orders = _orders(lay, views[1], idx, rows, gen)
        for t in range(2 * m + 1):
            q, k, v, g, beta = (x.to(DEV) for x in gdn_token(gen, rows, HV, HK, D, D, dtype=torch.bfloat16))
            outs = [torch.full((rows, HV, D), 3.0, device=DEV, dtype=torch.bfloat16) for _ in range(2)]
            lay.step(views[0], idx, q, k, v, outs[0], D ** -0.5, g=g, beta=beta)
            order = next(orders, None)
            if order is None:
                order = lay.fold_order(views[1], idx)
            lay.step(views[1], idx, q, k, v, outs[1], D ** -0.5, g=g, beta=beta, order=order)
            assert torch.equal(outs[0], outs[1]), t
            assert torch.equal(blobs[0], blobs[1]), t
    finally:
        _hip.select_instances()
    n = views[0]['NPTR'][idx[live].long(), 0].tolist()
    assert len(set(n)) > 1                                   # the sequences really were out of step


@pytest.mark.parametrize('fmt', [(4, 'k', 32), (8, 'v', 32)])
def test_kda_results_do_not_depend_on_the_order(fmt):
    H, K, Vd, m, rows = 4, 128, 128, 4, 64
    lay = KDASlotLayout(sq.Quantizer(*fmt), H, K, Vd, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(13)
    idx = (torch.randperm(rows, generator=gen) + 1).to(torch.int32)
    idx[[7, 30]] = 0
    idx = idx.to(DEV)
    blobs = [lay.alloc(rows + 1, DEV) for _ in range(2)]
    views = [lay.views(b) for b in blobs]
    S0 = (torch.randn(rows, H, Vd, K, generator=gen) * 0.4).to(DEV)
    live = idx > 0
    for V in views:
        lay.write(V, idx[live].long(), S0[live])
        _mixed_fills(V, idx, m, torch.Generator().manual_seed(14))
    r = lambda *s: torch.randn(*s, generator=gen)            # noqa: E731
    for t in range(2 * m + 1):
        q, k, v = r(rows, H, K).bfloat16().to(DEV), r(rows, H, K).bfloat16().to(DEV), r(rows, H, Vd).bfloat16().to(DEV)
        g = (-torch.nn.functional.softplus(r(rows, H, K))).to(DEV)
        beta = torch.sigmoid(r(rows, H)).to(DEV)
        outs = [torch.full((rows, H, Vd), 3.0, device=DEV, dtype=torch.bfloat16) for _ in range(2)]
        lay.step(views[0], idx, q, k, v, g, beta, outs[0])
        order = lay.fold_order(views[1], idx) if t % 2 else torch.randperm(rows, generator=gen).to(torch.int32).to(DEV)
        lay.step(views[1], idx, q, k, v, g, beta, outs[1], order=order)
        assert torch.equal(outs[0], outs[1]), t
        assert torch.equal(blobs[0], blobs[1]), t


@pytest.mark.parametrize('fmt,DV,H,G', [((8, 'k', 128), 64, 8, 2), ((4, 'k', 32), 80, 6, 2)])
def test_mamba2_results_do_not_depend_on_the_order(fmt, DV, H, G):
    DK, m, rows = 128, 4, 64
    lay = Mamba2SlotLayout(sq.Quantizer(*fmt), H, G, DK, DV, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(15)
    idx = (torch.randperm(rows, generator=gen) + 1).to(torch.int32)
    idx[[1, 50]] = 0
    idx = idx.to(DEV)
    blobs = [lay.alloc(rows + 1, DEV) for _ in range(2)]
    views = [lay.views(b) for b in blobs]
    S0 = (torch.randn(rows, H, DV, DK, generator=gen) * 0.4).to(DEV)
    live = idx > 0
    for V in views:
        lay.write(V, idx[live].long(), S0[live])
        _mixed_fills(V, idx, m, torch.Generator().manual_seed(16))
    r = lambda *s: torch.randn(*s, generator=gen)            # noqa: E731
    A = (-torch.exp(r(H) * 0.3)).to(DEV)
    D, bias = r(H).to(DEV), (r(H) * 0.1).to(DEV)
    for t in range(2 * m + 1):
        x, dt = r(rows, H, DV).bfloat16().to(DEV), (r(rows, H) * 0.5 - 2).to(DEV)
        B, C = r(rows, G, DK).bfloat16().to(DEV), r(rows, G, DK).bfloat16().to(DEV)
        outs = [torch.full((rows, H, DV), 3.0, device=DEV, dtype=torch.bfloat16) for _ in range(2)]
        lay.step(views[0], idx, x, dt, B, C, outs[0], A, D, bias)
        order = lay.fold_order(views[1], idx) if t % 2 else torch.randperm(rows, generator=gen).to(torch.int32).to(DEV)
        lay.step(views[1], idx, x, dt, B, C, outs[1], A, D, bias, order=order)
        assert torch.equal(outs[0], outs[1]), t
        assert torch.equal(blobs[0], blobs[1]), t


def test_order_under_graph_replay():
    """A captured decode step -- ``fold_order`` into a fixed buffer, then the layer steps with that order -- replayed
    while the sequences move through their fold periods out of step, next to an eager twin without an order."""
    HV, HK, D, m, rows, layers = 8, 4, 128, 4, 64, 2
    lay = SlotLayout(sq.Quantizer(8, 'k', 128), HV, HK, D, D, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(17)
    idx = (torch.randperm(rows, generator=gen) + 1).to(torch.int32).to(DEV)
    blobs = [[lay.alloc(rows + 1, DEV) for _ in range(layers)] for _ in range(2)]       # [0] graph, [1] eager twin
    views = [[lay.views(b) for b in bl] for bl in blobs]
    for vs in views:
        for L, V in enumerate(vs):
            lay.write(V, idx.long(), (torch.randn(rows, HV, D, D, generator=torch.Generator().manual_seed(L)) * 0.4).to(DEV))
            _mixed_fills(V, idx, m, torch.Generator().manual_seed(18))
    tok = [torch.zeros(s, device=DEV, dtype=torch.bfloat16) for s in ((rows, HK, D), (rows, HK, D), (rows, HV, D))]
    g, beta = torch.zeros(rows, HV, device=DEV), torch.zeros(rows, HV, device=DEV)
    outs = [[torch.zeros(rows, HV, D, device=DEV, dtype=torch.bfloat16) for _ in range(layers)] for _ in range(2)]
    order = torch.zeros(rows, dtype=torch.int32, device=DEV)

    def feed():
        q, k, v, g_, b_ = gdn_token(gen, rows, HV, HK, D, D, dtype=torch.bfloat16)
        tok[0].copy_(q); tok[1].copy_(k); tok[2].copy_(v); g.copy_(g_); beta.copy_(b_)

    def decode(which, ordered):
        if ordered:
            lay.fold_order(views[which][0], idx, out=order)
        for L in range(layers):
            lay.step(views[which][L], idx, *tok, outs[which][L], D ** -0.5, g=g, beta=beta,
                     order=order if ordered else None)

    stream = torch.cuda.Stream()
    feed()
    with torch.cuda.stream(stream):
        decode(0, True)                                      # warm-up on the capture stream
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            decode(0, True)
    torch.cuda.synchronize()
    decode(1, False)
    seen = set()
    for rep in range(2 * m + 1):
        feed()
        graph.replay()
        decode(1, False)
        torch.cuda.synchronize()
        seen.add(tuple(order.cpu().tolist()))
        for L in range(layers):
            assert torch.equal(outs[0][L], outs[1][L]), (rep, L)
            assert torch.equal(blobs[0][L], blobs[1][L]), (rep, L)
    assert len(seen) > 1                                     # the order followed the counters from replay to replay


@pytest.mark.parametrize('fmt', [(8, 'k', 128), (4, 'k', 64)])
def test_full_size_batch_out_of_step(fmt):
    """The benchmark's shape (256 sequences, 32 / 16 heads, d 128) with the fill levels dealt at random: stepped with
    ``fold_order``'s list and in batch order, the two blobs and the outputs stay equal bit for bit through two fold
    periods, and every sequence's counter advances by one per step."""
    HV, HK, D, m, rows = 32, 16, 128, 8, 256
    lay = SlotLayout(sq.Quantizer(*fmt), HV, HK, D, D, m=m, buffer_bits=8)
    gen = torch.Generator().manual_seed(19)
    idx = (torch.randperm(rows, generator=gen) + 1).to(torch.int32).to(DEV)
    blobs = [lay.alloc(rows + 1, DEV) for _ in range(2)]
    views = [lay.views(b) for b in blobs]
    S0 = (torch.randn(rows, HV, D, D, generator=gen) * 0.3).to(DEV)
    fill0 = torch.randint(0, m, (rows,), generator=gen).to(torch.int32).to(DEV)
    for V in views:
        lay.write(V, idx.long(), S0)
        V['NPTR'][idx.long()] = fill0[:, None]
    del S0
    order = torch.zeros(rows, dtype=torch.int32, device=DEV)
    moved = 0
    for t in range(2 * m + 1):
        q, k, v, g, beta = (x.to(DEV) for x in gdn_token(gen, rows, HV, HK, D, D, dtype=torch.bfloat16))
        outs = [torch.full((rows, HV, D), 3.0, device=DEV, dtype=torch.bfloat16) for _ in range(2)]
        lay.step(views[0], idx, q, k, v, outs[0], D ** -0.5, g=g, beta=beta)
        lay.fold_order(views[1], idx, out=order)
        moved += int((order != torch.arange(rows, device=DEV, dtype=torch.int32)).any())
        lay.step(views[1], idx, q, k, v, outs[1], D ** -0.5, g=g, beta=beta, order=order)
        assert torch.equal(outs[0], outs[1]), t
        assert torch.equal(blobs[0], blobs[1]), t
        want = (fill0 + t + 1) % m
        assert torch.equal(views[1]['NPTR'][idx.long(), 0], want), t
    assert moved == 2 * m + 1                                # every step had rows to place
