"""The serving-engine layer forwards (statequant_amd/integrations/: Qwen GDN ``_forward_core``, OLMo-Hybrid
``_forward_core``, KDA ``_forward``, Mamba2 ``conv_ssm_forward``) driven without an engine: layer and metadata objects
are plain namespaces with the attributes the forwards read, the engine's ops are the torch stand-ins of
tests/_engine_fakes.py (the reference's plugin tests do the same around a real vLLM,
/root/reference/tests/test_vllm_olmo_plugin.py:27-135, tests/test_vllm_plugin.py:48-63 there).

Every scenario is a prefill of several sequences, a mixed step (decode rows + a continued prompt + a new sequence in
a slot that still holds its previous owner's bytes), then decode-only steps through two folds in a batch padded with
null-slot rows.  Checked against the CPU oracle, per sequence:
  * decode rows: what the forward wrote into the output rows == the oracle's step on the conv output the forward
    computed (recorded), cut into q | k | v as the engine lays them out, with the engine's gate;
  * prefill rows: the initial state the chunk kernel was handed == the oracle's current state (stored state advanced
    over the pending buffer) for sequences with history, exactly zero for new ones; the chunk kernel's outputs land
    in the prefill rows; the slot then holds exactly the oracle's packing of the returned final state, buffer empty;
  * padding rows: output zero, the null slot's bytes untouched.
"""
from types import SimpleNamespace

import pytest
import torch

import statequant_amd as sq
from oracle import states as ST
from statequant_amd.integrations import vllm_kda, vllm_mamba2, vllm_olmo, vllm_plugin
from statequant_amd.kernels import KDASlotLayout, Mamba2SlotLayout, SlotLayout
from tests import _engine_fakes as F
from tests._util import unpack_nib

pytestmark = pytest.mark.gpu
DEV = 'cuda'
M, KC, NSLOT = 4, 4, 8                                    # buffer length, conv width, slots in the cache


def rel(a, b):
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


class Book:
    """One oracle per live slot; compares and re-syncs after folds (a rounding tie is then counted once)."""

    def __init__(self, make, bits):
        self.make, self.bits, self.ora, self.worst = make, bits, {}, 0.0

    def stored(self, slot, S, views):
        """The forward has just written S (fp32, value-major) into `slot`: the slot must hold the oracle's packing."""
        o = self.ora[slot] = self.make(S.cpu())
        got = views['S'][slot].cpu()
        assert torch.equal(got.reshape(o.codes.shape), o.codes), f'slot {slot}: codes after write'
        if o.scales is not None:
            assert torch.equal(views['SC'][slot].cpu().reshape(o.scales.shape), o.scales), f'slot {slot}: scales'
        assert int(views['NPTR'][slot].abs().max()) == 0 and float(views['GCUR'][slot].abs().max()) == 0.0

    def after_step(self, slot, got, want, views):
        self.worst = max(self.worst, rel(got, want))
        o = self.ora[slot]
        assert int(views['NPTR'][slot, 0]) == o.n, slot
        if o.n == 0:                                       # folded: adopt the slot's codes
            codes = views['S'][slot].cpu().reshape(o.codes.shape)
            assert (unpack_nib(codes, self.bits).int() - unpack_nib(o.codes, self.bits).int()).abs().max() <= 1
            o.adopt(codes, views['SC'][slot].cpu().reshape(o.scales.shape))


def gdn_layer(lay, gen, hk, hv, dk, dv, bias=True):
    C = 2 * hk * dk + hv * dv
    r = lambda *s: torch.randn(*s, generator=gen).to(DEV)          # noqa: E731
    layer = SimpleNamespace(
        prefix='model.layers.3.linear_attn', activation='silu', head_k_dim=dk, head_v_dim=dv,
        conv1d=SimpleNamespace(weight=r(C, 1, KC) * 0.5, bias=r(C) * 0.1 if bias else None),
        A_log=r(hv) * 0.3 - 1.0, dt_bias=r(hv) * 0.3,
        kv_cache=(torch.zeros(NSLOT, C, KC - 1, device=DEV), lay.alloc(NSLOT, DEV)),
        _sq_layout=lay, _sq_views=None, _sq_external=None, _sq_lk={})
    return layer, C


def scenario():
    """(decode slots, prefill slots, prefill lengths, prefill-has-history, padded rows) of each step."""
    steps = [([], [3, 1, 6], [3, 7, 5], [False, False, False], None),
             ([3, 1], [6, 2], [4, 2], [True, False], None)]
    steps += [([3, 1, 6, 2], [], [], [], 6)] * (2 * M + 1)
    return steps


@pytest.mark.parametrize('fmt', [(8, 'k', 32), (4, 'k', 64)])
@pytest.mark.parametrize('olmo', [False, True])
def test_gdn_forward_core(fmt, olmo):
    hk, hv, dk, dv = (3, 3, 96, 192) if olmo else (2, 4, 64, 64)
    gen = torch.Generator().manual_seed(41)
    lay = SlotLayout(sq.Quantizer(*fmt), hv, hk, dk, dv, m=M, buffer_bits=8)
    layer, C = gdn_layer(lay, gen, hk, hv, dk, dv, bias=not olmo)
    rec, ctx = F.Recorder(), {}
    ns = F.engine_module(rec, ctx)
    if olmo:
        vllm_olmo._state['O'] = ns
        layer.allow_neg_eigval = True
        kw = hk * dk
        layer.rearrange_mixed_qkv = lambda x: (x[:, :kw].reshape(1, -1, hk, dk), x[:, kw:2 * kw].reshape(1, -1, hk, dk),
                                               x[:, 2 * kw:].reshape(1, -1, hv, dv))
        forward = vllm_olmo._forward_core
    else:
        vllm_plugin._state['Q'] = ns
        layer.chunk_gated_delta_rule = ns.chunk_gated_delta_rule
        layer._warmup_prefill_kernels = lambda *a: pytest.fail('warm-up on a step with metadata')
        forward = vllm_plugin._forward_core
    views = lay.views(layer.kv_cache[1])
    layer.kv_cache[1][2].random_(0, 255)                   # slot 2 starts with a previous owner's bytes
    null_before = layer.kv_cache[1][0].clone()
    book = Book(lambda S: ST.GDNOracle(S.reshape(hv, dv, dk), fmt, m=M, hv=hv, hk=hk, buffer_bits=8), fmt[0])
    kw = hk * dk
    for dec, pre, lens, hist, pad in scenario():
        md = F.gdn_metadata(dec, pre, lens, hist, DEV, pad_to=pad)
        ctx['md'] = {layer.prefix: md}
        T = md.num_actual_tokens
        extra = 2                                          # the engine's buffers are longer than the step's tokens
        x_in = torch.randn(T + extra, C, generator=gen).to(DEV)
        a, b = (torch.randn(T + extra, hv, generator=gen) * 0.5 - 1).to(DEV), torch.randn(T + extra, hv, generator=gen).to(DEV)
        out = torch.full((T + extra, hv, dv), 7.0, device=DEV)
        before = {s: book.ora[s].state().clone() for s in pre if s in book.ora}
        rec.clear()
        forward(layer, x_in, b, a, out)
        x = (rec.last('conv_varlen').out.transpose(0, 1) if pre else rec.last('conv_update').out).cpu()
        nd = len(dec)
        if olmo:
            g, beta = (t[0].cpu() for t in rec.last('gating').out)
        else:
            g, beta = ST.gdn_gate(a[:T].cpu(), b[:T].cpu(), layer.A_log.cpu(), layer.dt_bias.cpu())
        for r, slot in enumerate(dec):
            want = book.ora[slot].step(x[r, :kw].view(hk, dk), x[r, kw:2 * kw].view(hk, dk), x[r, 2 * kw:].view(hv, dv),
                                       g[r], beta[r], dk ** -0.5)
            book.after_step(slot, out[r].cpu(), want.view(hv, dv), views)
        if pad:
            assert float(out[nd:T].abs().max()) == 0.0, 'padding rows'
        assert float((out[T:] - 7.0).abs().max()) == 0.0, 'rows beyond the step were touched'
        if pre:
            call = rec.last('chunk')
            init = call.kw['initial_state'].cpu()
            for p, slot in enumerate(pre):
                if hist[p]:
                    assert rel(init[p], before[slot].view(hv, dv, dk)) < 1e-5, f'initial state of slot {slot}'
                else:
                    assert float(init[p].abs().max()) == 0.0, f'slot {slot} starts from zero'
            o_chunk, last = call.out
            n_tok = sum(lens)
            assert torch.equal(out[nd:nd + n_tok], o_chunk[0].to(out.dtype))
            assert call.kw['cu_seqlens'].tolist() == [0] + torch.tensor(lens).cumsum(0).tolist()
            for p, slot in enumerate(pre):
                book.stored(slot, last[p], views)
    assert book.worst < 1e-2, book.worst                   # the task's bound on o; typical: 1e-6
    assert torch.equal(layer.kv_cache[1][0], null_before), 'the null slot was written'
    print(f'[{"olmo" if olmo else "qwen"} {fmt}] max rel |o - o_oracle| over decode rows {book.worst:.2e}')


def test_gdn_forward_core_without_metadata_warms_up_and_returns():
    lay = SlotLayout(sq.Quantizer(8, 'k', 32), 4, 2, 64, 64, m=M)
    layer, C = gdn_layer(lay, torch.Generator().manual_seed(1), 2, 4, 64, 64)
    vllm_plugin._state['Q'] = F.engine_module(F.Recorder(), {})
    warmed = []
    layer._warmup_prefill_kernels = lambda qkv, v_dim: warmed.append(v_dim)
    before = layer.kv_cache[1].clone()
    out = torch.full((3, 4, 64), 7.0, device=DEV)
    vllm_plugin._forward_core(layer, torch.zeros(3, C, device=DEV), torch.zeros(3, 4, device=DEV),
                              torch.zeros(3, 4, device=DEV), out)
    assert warmed == [0] and torch.equal(layer.kv_cache[1], before) and float((out - 7).abs().max()) == 0.0


@pytest.mark.parametrize('captured', [False, True])
def test_gdn_forward_core_external_quantizer(captured, tmp_path, monkeypatch):
    """``external:<file>:<fn>``: the slot keeps an unpacked fp32 state; fn(S, layer ordinal) replaces it at the end of
    a prefill chunk and on the rows whose buffer has just folded (under capture: called on every decode row, kept
    where folded).  fn sees key-major [rows, hv, d_k, d_v]."""
    hk, hv, dk, dv = 2, 4, 64, 64
    src = tmp_path / 'myquant.py'
    src.write_text('import torch\nSEEN = []\n'
                   'def fn(S, layer):\n'
                   '    SEEN.append((tuple(S.shape), layer))\n'
                   '    return S.clamp(-0.8, 0.8) * 0.9\n')
    monkeypatch.setenv('STATEQUANT_VLLM_EXTERNAL_GRAPHS', '1' if captured else '0')
    cfg = vllm_plugin.configure({'STATEQUANT_VLLM': f'external:{src}:fn', 'STATEQUANT_VLLM_M': str(M)})
    assert cfg[0] == 'fp32'
    gen = torch.Generator().manual_seed(43)
    lay = vllm_plugin.layout(hv, hk, dk, dv)
    layer, C = gdn_layer(lay, gen, hk, hv, dk, dv)
    layer.tp_size, layer.num_v_heads, layer.num_k_heads = 1, hv, hk
    config = SimpleNamespace(layer_types=['linear_attention', 'full_attention', 'linear_attention', 'linear_attention'])
    vcfg = SimpleNamespace(speculative_config=None, model_config=SimpleNamespace(enforce_eager=not captured),
                           cache_config=SimpleNamespace(enable_prefix_caching=False, mamba_cache_mode='none'))
    blob = layer.kv_cache[1]
    vllm_plugin.attach(layer, config, vcfg)
    assert layer._sq_layout is lay and layer._sq_external == (2, captured)      # layers.3 is the third GDN layer
    layer.kv_cache = (layer.kv_cache[0], blob)
    seen = vllm_plugin.external_fn().__globals__['SEEN']
    rec, ctx = F.Recorder(), {}
    ns = F.engine_module(rec, ctx)
    vllm_plugin._state['Q'] = ns
    layer.chunk_gated_delta_rule = ns.chunk_gated_delta_rule
    views = lay.views(blob)
    quant = lambda S: S.clamp(-0.8, 0.8) * 0.9                 # noqa: E731  (elementwise, continuous: layout-independent)
    ora = {}
    kw = hk * dk
    steps = [([], [5, 2], [4, 3], [False, False], None)] + [([5, 2], [], [], [], 3)] * (2 * M)
    for dec, pre, lens, hist, pad in steps:
        md = F.gdn_metadata(dec, pre, lens, hist, DEV, pad_to=pad)
        ctx['md'] = {layer.prefix: md}
        T = md.num_actual_tokens
        x_in = torch.randn(T, C, generator=gen).to(DEV)
        a, b = (torch.randn(T, hv, generator=gen) * 0.5 - 1).to(DEV), torch.randn(T, hv, generator=gen).to(DEV)
        out = torch.full((T, hv, dv), 7.0, device=DEV)
        rec.clear()
        n_seen = len(seen)
        vllm_plugin._forward_core(layer, x_in, b, a, out)
        if pre:
            last = rec.last('chunk').out[1].cpu()
            assert seen[n_seen:] == [((len(pre), hv, dk, dv), 2)]
            for p, slot in enumerate(pre):
                assert torch.equal(views['S'][slot].cpu(), quant(last[p]))
                ora[slot] = ST.GDNOracle(quant(last[p]), ST.IDENT, m=M, hv=hv, hk=hk, buffer_bits=8)
            continue
        x = rec.last('conv_update').out.cpu()
        g, beta = ST.gdn_gate(a.cpu(), b.cpu(), layer.A_log.cpu(), layer.dt_bias.cpu())
        folded = 0
        for r, slot in enumerate(dec):
            o = ora[slot]
            want = o.step(x[r, :kw].view(hk, dk), x[r, kw:2 * kw].view(hk, dk), x[r, 2 * kw:].view(hv, dv), g[r], beta[r],
                          dk ** -0.5)
            assert rel(out[r].cpu(), want.view(hv, dv)) < 1e-4
            if o.n == 0:                                   # folded on this step: fn was applied to the slot
                folded += 1
                got = views['S'][slot].cpu()
                assert rel(got, quant(o.S0).view(hv, dv, dk)) < 1e-5 and float(got.abs().max()) <= 0.72 + 1e-6
                o.S0 = got.reshape(o.S0.shape).clone()
        calls = seen[n_seen:]
        if captured:
            assert calls == [((pad, hv, dk, dv), 2)]
        else:
            assert calls == ([((folded, hv, dk, dv), 2)] if folded else [])
    vllm_plugin.configure({'STATEQUANT_VLLM': 'off'})


def test_kda_forward():
    H, D, fmt = 4, 64, (4, 'k', 32)
    gen = torch.Generator().manual_seed(47)
    r = lambda *s: torch.randn(*s, generator=gen).to(DEV)          # noqa: E731
    lay = KDASlotLayout(sq.Quantizer(*fmt), H, D, D, m=M, buffer_bits=8)
    C = H * D
    conv = lambda: SimpleNamespace(weight=r(C, 1, KC) * 0.5, bias=r(C) * 0.1)      # noqa: E731
    layer = SimpleNamespace(prefix='model.layers.0.attn', head_dim=D, safe_gate=False, lower_bound=None,
                            q_conv1d=conv(), k_conv1d=conv(), v_conv1d=conv(),
                            kv_cache=(torch.zeros(NSLOT, 3 * C, KC - 1, device=DEV), lay.alloc(NSLOT, DEV)),
                            _sq_layout=lay, _sq_views=None)
    rec, ctx = F.Recorder(), {}
    vllm_kda._state['M'] = F.engine_module(rec, ctx)
    views = lay.views(layer.kv_cache[1])
    layer.kv_cache[1][2].random_(0, 255)
    null_before = layer.kv_cache[1][0].clone()
    book = Book(lambda S: ST.KDAOracle(S.reshape(H, D, D), fmt, m=M, hv=H, buffer_bits=8), fmt[0])
    for dec, pre, lens, hist, pad in scenario():
        md = F.gdn_metadata(dec, pre, lens, hist, DEV, pad_to=pad)
        ctx['md'] = {layer.prefix: md}
        T = md.num_actual_tokens
        qs, ks, vs = r(T + 1, C), r(T + 1, C), r(T + 1, C)
        g1 = -torch.nn.functional.softplus(r(1, T + 1, H, D))
        beta = torch.sigmoid(r(1, T + 1, H))
        out = torch.full((1, T + 1, H, D), 7.0, device=DEV)
        before = {s: book.ora[s].state().clone() for s in pre if s in book.ora}
        rec.clear()
        vllm_kda._forward(layer, qs, ks, vs, g1, beta, out)
        name = 'conv_varlen' if pre else 'conv_update'
        q, k, v = [(c.out.transpose(0, 1) if pre else c.out).cpu() for c in rec.calls[name][-3:]]
        # the three convs ran on the three thirds of the conv state, in q, k, v order
        used = [c.kw.get('conv_states', c.args[1] if len(c.args) > 1 else None) for c in rec.calls[name][-3:]]
        thirds = layer.kv_cache[0].chunk(3, dim=-2)
        assert all(u.data_ptr() == t.data_ptr() for u, t in zip(used, thirds))
        nd = len(dec)
        for rr, slot in enumerate(dec):
            want = book.ora[slot].step(q[rr].view(H, D), k[rr].view(H, D), v[rr].view(H, D), g1[0, rr].cpu(),
                                       beta[0, rr].cpu(), D ** -0.5)
            book.after_step(slot, out[0, rr].cpu(), want.view(H, D), views)
        if pad:
            assert float(out[0, nd:T].abs().max()) == 0.0
        assert float((out[0, T:] - 7.0).abs().max()) == 0.0
        if pre:
            call = rec.last('chunk')
            init = call.kw['initial_state'].cpu()
            for p, slot in enumerate(pre):
                if hist[p]:
                    assert rel(init[p], before[slot].view(H, D, D)) < 1e-5
                else:
                    assert float(init[p].abs().max()) == 0.0
            o_chunk, last = call.out
            assert torch.equal(out[0, nd:T], o_chunk[0].to(out.dtype))
            assert torch.equal(call.kw['g'][0], g1[0, nd:T]) and torch.equal(call.kw['beta'][0], beta[0, nd:T])
            for p, slot in enumerate(pre):
                book.stored(slot, last[p], views)
    assert book.worst < 1e-2, book.worst
    assert torch.equal(layer.kv_cache[1][0], null_before)
    print(f'[kda {fmt}] max rel |o - o_oracle| over decode rows {book.worst:.2e}')


def test_mamba2_conv_ssm_forward():
    H, G, N, P_, fmt = 8, 2, 128, 64, (8, 'k', 128)
    gen = torch.Generator().manual_seed(53)
    r = lambda *s: torch.randn(*s, generator=gen).to(DEV)          # noqa: E731
    lay = Mamba2SlotLayout(sq.Quantizer(*fmt), H, G, N, P_, m=M, buffer_bits=8)
    inter, conv_dim = H * P_, H * P_ + 2 * G * N

    def split(xBC):
        return torch.split(xBC, [inter, G * N, G * N], dim=-1)
    layer = SimpleNamespace(prefix='backbone.layers.1.mixer', activation='silu', tped_intermediate_size=inter,
                            tped_conv_size=conv_dim, tped_dt_size=H, conv_weights=r(conv_dim, KC) * 0.5,
                            conv1d=SimpleNamespace(bias=r(conv_dim) * 0.1), split_hidden_states_B_C_fn=split,
                            A=-torch.exp(torch.rand(H, generator=gen) * 2).to(DEV), D=r(H), dt_bias=r(H) * 0.3,
                            kv_cache=(torch.zeros(NSLOT, conv_dim, KC - 1, device=DEV), lay.alloc(NSLOT, DEV)),
                            _sq_layout=lay, _sq_views=None)
    layer._warmup_ssd_kernels = lambda ps: pytest.fail('warm-up on a step with metadata')
    rec, ctx = F.Recorder(), {}
    vllm_mamba2._state['M'] = F.engine_module(rec, ctx)
    views = lay.views(layer.kv_cache[1])
    layer.kv_cache[1][2].random_(0, 255)
    null_before = layer.kv_cache[1][0].clone()
    book = Book(lambda S: ST.Mamba2Oracle(S.reshape(H, P_, N), fmt, m=M, hv=H, hk=G, buffer_bits=8), fmt[0])
    A, D_, dtb = layer.A.cpu(), layer.D.cpu(), layer.dt_bias.cpu()
    for dec, pre, lens, hist, pad in scenario():
        dec_rows = list(dec) + ([0] * (pad - len(dec)) if pad else [])           # padded rows are decode tokens here
        md = F.mamba2_metadata(dec_rows, pre, lens, hist, DEV)
        ctx['md'] = {layer.prefix: md}
        T = len(dec_rows) + sum(lens)
        proj = r(T + 1, inter + conv_dim + H)
        proj[:, -H:] = proj[:, -H:] * 0.5 - 2                                     # raw dt
        out = torch.full((T + 1, H * P_), 7.0, device=DEV)
        before = {s: book.ora[s].state().clone() for s in pre if s in book.ora}
        rec.clear()
        vllm_mamba2.conv_ssm_forward(layer, proj, out)
        nd = len(dec_rows)
        if dec_rows:
            x, Bm, Cm = (t.cpu() for t in split(rec.last('conv_update').out))
            dt = proj[:nd, -H:].cpu()
            for rr, slot in enumerate(dec):
                want = book.ora[slot].step(x[rr].view(1, H, P_), dt[rr].view(1, H), Bm[rr].view(1, G, N),
                                           Cm[rr].view(1, G, N), A, D_, dtb, True, None)
                book.after_step(slot, out[rr].view(H, P_).cpu(), want.view(H, P_), views)
            if pad:
                assert float(out[len(dec):nd].abs().max()) == 0.0
        assert float((out[T:] - 7.0).abs().max()) == 0.0
        if pre:
            call = rec.last('chunk')
            init = call.kw['initial_states']
            if any(hist):
                for p, slot in enumerate(pre):
                    if hist[p]:
                        assert rel(init[p].cpu(), before[slot].view(H, P_, N)) < 1e-5
                    else:
                        assert float(init[p].abs().max()) == 0.0
            else:
                assert init is None
            assert call.kw['out'].data_ptr() == out[nd:].data_ptr()               # the scan wrote the prefill rows
            for p, slot in enumerate(pre):
                book.stored(slot, call.out[p], views)
    assert book.worst < 1e-2, book.worst
    assert torch.equal(layer.kv_cache[1][0], null_before)
    print(f'[mamba2 {fmt}] max rel |y - y_oracle| over decode rows {book.worst:.2e}')


def test_dispatch_order_is_made_once_per_forward_pass(monkeypatch):
    """Two GDN layers of one model, 64 decode sequences out of step: the first layer of a pass makes the dispatch
    order from the counters, the second finds it on the forward context; a new pass makes a new one; and the layers'
    results are those of the same passes without any order, bit for bit."""
    from statequant_amd.integrations import _engine as E
    hk, hv, dk, dv, rows = 2, 4, 64, 64, 64
    gen = torch.Generator().manual_seed(47)
    lay = SlotLayout(sq.Quantizer(8, 'k', 64), hv, hk, dk, dv, m=M, buffer_bits=8)
    rec, ctx = F.Recorder(), {}
    ns = F.engine_module(rec, ctx)
    vllm_plugin._state['Q'] = ns
    C = 2 * hk * dk + hv * dv
    r = lambda *s: torch.randn(*s, generator=gen).to(DEV)          # noqa: E731

    def layers():
        out = []
        g2 = torch.Generator().manual_seed(48)
        for L in range(2):
            blob = lay.alloc(rows + 1, DEV)
            V = lay.views(blob)
            lay.write(V, torch.arange(1, rows + 1, device=DEV), (torch.randn(rows, hv, dv, dk, generator=g2) * 0.4).to(DEV))
            V['NPTR'][1:] = (torch.arange(rows, device=DEV, dtype=torch.int32) % M)[:, None]
            out.append(SimpleNamespace(
                prefix=f'model.layers.{L}.linear_attn', activation='silu', head_k_dim=dk, head_v_dim=dv,
                conv1d=SimpleNamespace(weight=torch.randn(C, 1, KC, generator=g2).to(DEV) * 0.5, bias=None),
                A_log=torch.randn(hv, generator=g2).to(DEV) * 0.3 - 1.0, dt_bias=torch.randn(hv, generator=g2).to(DEV) * 0.3,
                kv_cache=(torch.zeros(rows + 1, C, KC - 1, device=DEV), blob),
                _sq_layout=lay, _sq_views=None, _sq_external=None, _sq_lk={},
                chunk_gated_delta_rule=ns.chunk_gated_delta_rule,
                _warmup_prefill_kernels=lambda *a: pytest.fail('warm-up on a step with metadata')))
        return out

    ordered, plain = layers(), layers()
    calls, use = [], {'order': True}
    real_fold_order, real_dispatch_order = SlotLayout.fold_order, E.dispatch_order
    monkeypatch.setattr(SlotLayout, 'fold_order', lambda self, *a, **k: calls.append(1) or real_fold_order(self, *a, **k))
    monkeypatch.setattr(E, 'dispatch_order', lambda *a, **k: real_dispatch_order(*a, **k) if use['order'] else None)
    slots = list(range(1, rows + 1))
    for step in range(M + 2):
        md = F.gdn_metadata(slots, [], [], [], DEV)
        x_in, a, b = r(rows, C), r(rows, hv) * 0.5 - 1, r(rows, hv)
        outs = {}
        for name, group in (('ordered', ordered), ('plain', plain)):
            ctx.pop('fc', None)                              # a new forward pass
            ctx['md'] = {layer.prefix: md for layer in group}
            use['order'] = name == 'ordered'
            before = len(calls)
            outs[name] = []
            for layer in group:
                out = torch.full((rows, hv, dv), 7.0, device=DEV)
                vllm_plugin._forward_core(layer, x_in, b, a, out)
                outs[name].append(out)
            assert len(calls) - before == (1 if name == 'ordered' else 0), (name, step)
            assert hasattr(ctx['fc'], '_sq_dispatch_order') == (name == 'ordered')
        for o1, o2, l1, l2 in zip(outs['ordered'], outs['plain'], ordered, plain):
            assert torch.equal(o1, o2), step
            assert torch.equal(l1.kv_cache[1], l2.kv_cache[1]), step
    n = lay.views(ordered[0].kv_cache[1])['NPTR'][1:, 0].tolist()
    assert len(set(n)) == M                                  # the sequences were out of step throughout
