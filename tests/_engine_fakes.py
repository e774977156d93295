"""Stand-ins for the serving engine's side of the layer forwards (tests only): plain-torch versions of the ops the
patched forwards take from the engine module -- the causal convs, the gating helpers, the prefill chunk kernels --
with the engine's call signatures, plus recorders, so that a test sees what a forward fed to the engine and what it
got back.  The reference's own plugin tests build the same kind of objects around a real vLLM
(/root/reference/tests/test_vllm_olmo_plugin.py:27-57 there); these need no engine.

Nothing here is a faithful model of the engine's kernels' speed or chunking: a "chunk kernel" is the textbook
recurrence token by token.  What matters is that it is a deterministic function of its arguments, so the forward's
wiring (which rows, which slots, which columns, which state goes in and where the result goes) decides the outcome.
"""
from types import SimpleNamespace

import torch

from oracle import states as ST
from oracle.formats import l2norm


def silu(x):
    return x * torch.sigmoid(x)


def conv_update(x, conv_state, w, bias, activation=None, conv_state_indices=None, validate_data=False, **unused):
    """Single-token causal conv: x [rows, C], conv_state [slots, C, K-1] (updated in place), w [C, K]."""
    rows = x.shape[0]
    y = torch.zeros_like(x, dtype=torch.float32)
    for r in range(rows):
        s = int(conv_state_indices[r])
        if s < 0:
            continue
        win = torch.cat([conv_state[s].float(), x[r].float()[:, None]], -1)           # [C, K]
        acc = (win * w.float()).sum(-1)
        y[r] = acc if bias is None else acc + bias.float()
        conv_state[s] = win[:, 1:].to(conv_state.dtype)
    return (silu(y) if activation in ('silu', 'swish') else y).to(x.dtype)


def conv_varlen(xT, w, bias, activation=None, conv_states=None, has_initial_state=None, cache_indices=None,
                query_start_loc=None, metadata=None, **unused):
    """Variable-length causal conv: xT [C, tokens]; sequence i owns tokens [qsl[i], qsl[i+1]) and slot
    cache_indices[i]; its window starts from the slot's conv state where has_initial_state[i], else from zeros."""
    C, K = w.shape
    y = torch.zeros_like(xT, dtype=torch.float32)
    qsl = query_start_loc.tolist()
    for i in range(len(qsl) - 1):
        s = int(cache_indices[i])
        hist = conv_states[s].float() if bool(has_initial_state[i]) else torch.zeros(C, K - 1, device=xT.device)
        seq = torch.cat([hist, xT[:, qsl[i]:qsl[i + 1]].float()], -1)
        for t in range(qsl[i + 1] - qsl[i]):
            acc = (seq[:, t:t + K] * w.float()).sum(-1)
            y[:, qsl[i] + t] = acc if bias is None else acc + bias.float()
        conv_states[s] = seq[:, -(K - 1):].to(conv_states.dtype)
    return (silu(y) if activation in ('silu', 'swish') else y).to(xT.dtype)


def post_conv_prep(conv_output, a, b, A_log, dt_bias, num_k_heads, head_k_dim, head_v_dim, apply_l2norm=True,
                   output_g_exp=False):
    """The Qwen layer's prefill-side split + gate: q, k [T, hk, d_k] l2-normalised, v [T, hv, d_v], g, beta [T, hv]."""
    T = conv_output.shape[0]
    kw = num_k_heads * head_k_dim
    q = conv_output[:, :kw].float().view(T, num_k_heads, head_k_dim)
    k = conv_output[:, kw:2 * kw].float().view(T, num_k_heads, head_k_dim)
    v = conv_output[:, 2 * kw:].float().view(T, -1, head_v_dim)
    if apply_l2norm:
        q, k = l2norm(q), l2norm(k)
    g, beta = ST.gdn_gate(a.cpu(), b.cpu(), A_log.cpu(), dt_bias.cpu())
    return q, k, v, g.to(v.device), beta.to(v.device)


def olmo_gating(A_log, a, b, dt_bias, allow_neg_eigval):
    g, beta = ST.gdn_gate(a.cpu(), b.cpu(), A_log.cpu(), dt_bias.cpu())
    if allow_neg_eigval:
        beta = beta * 2.0
    return g.to(a.device)[None], beta.to(a.device)[None]


class Recorder:
    """Keeps the keyword arguments and the results of the last call of each recorded op."""

    def __init__(self):
        self.calls = {}

    def wrap(self, name, fn):
        def inner(*args, **kw):
            out = fn(*args, **kw)
            self.calls.setdefault(name, []).append(SimpleNamespace(args=args, kw=kw, out=out))
            return out
        return inner

    def last(self, name):
        return self.calls[name][-1]

    def clear(self):
        self.calls.clear()


def chunk_gdn(q, k, v, g, beta, initial_state, output_final_state=True, cu_seqlens=None, use_qk_l2norm_in_kernel=False,
              **unused):
    """Gated delta rule over packed sequences: q, k [1, T, hk, d_k], v [1, T, hv, d_v], g, beta [1, T, hv],
    initial_state [P, hv, d_v, d_k] value-major fp32 -> (o [1, T, hv, d_v], final states).  scale = d_k^-1/2.
    (Runs on the CPU whatever device the arguments are on; results go back to that device.)"""
    dev = v.device
    q, k, v, g, beta = (t[0].float().cpu() for t in (q, k, v, g, beta))
    S = initial_state.float().cpu().clone()
    hv, hk, dk = v.shape[1], q.shape[1], q.shape[2]
    o = torch.zeros_like(v)
    qsl = cu_seqlens.tolist()
    for p in range(len(qsl) - 1):
        for t in range(qsl[p], qsl[p + 1]):
            qq, kk = q[t].repeat_interleave(hv // hk, 0), k[t].repeat_interleave(hv // hk, 0)
            o[t] = ST.gdn_recurrence(S[p], qq, kk, v[t], g[t], beta[t], dk ** -0.5)
    return o[None].to(dev), S.to(dev)


def chunk_kda(q, k, v, g, beta, initial_state, output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=None,
              **unused):
    """Per-channel gated delta rule over packed sequences: q, k, v [1, T, H, d], g [1, T, H, d_k], beta [1, T, H]."""
    dev = v.device
    q, k, v, g, beta = (t[0].float().cpu() for t in (q, k, v, g, beta))
    S = initial_state.float().cpu().clone()
    o = torch.zeros_like(v)
    qsl = cu_seqlens.tolist()
    for p in range(len(qsl) - 1):
        for t in range(qsl[p], qsl[p + 1]):
            o[t] = ST.kda_recurrence(S[p], q[t], k[t], v[t], g[t], beta[t])
    return o[None].to(dev), S.to(dev)


def chunk_scan_mamba2(x, dt, A, B, C, chunk_size=None, D=None, z=None, dt_bias=None, seq_idx=None, cu_seqlens=None,
                      initial_states=None, dt_softplus=True, dt_limit=None, out=None, state_dtype=None, **unused):
    """SSD over packed sequences: x [T, H, P], dt [T, H], B, C [T, G, N]; writes ``out`` [T, H, P], returns the final
    states [seqs, H, P, N]."""
    dev = x.device
    qsl = cu_seqlens.tolist()
    n = len(qsl) - 1
    H, P_, N = x.shape[1], x.shape[2], B.shape[2]
    S = torch.zeros(n, H, P_, N) if initial_states is None else initial_states.float().cpu().clone()
    xc, dtc, Bc, Cc = x.float().cpu(), dt.float().cpu(), B.float().cpu(), C.float().cpu()
    y = torch.zeros(x.shape[0], H, P_)
    for p in range(n):
        for t in range(qsl[p], qsl[p + 1]):
            y[t] = ST.mamba2_recurrence(S[p:p + 1], xc[t:t + 1], dtc[t:t + 1], Bc[t:t + 1], Cc[t:t + 1], A.cpu(),
                                        None if D is None else D.cpu(), None if dt_bias is None else dt_bias.cpu(),
                                        dt_softplus, dt_limit)[0]
    out.copy_(y.to(dev).to(out.dtype))
    return S.to(dev)


def engine_module(rec, context, **extra):
    """A namespace with the engine-module attributes the forwards use; ``context['md']`` is the dict the forward
    context hands out as ``attn_metadata``."""
    def forward_context():                                   # one object per pass: a test starts a new pass by
        fc = context.setdefault('fc', SimpleNamespace())     # dropping context['fc']
        fc.attn_metadata = context.get('md')
        return fc

    ns = SimpleNamespace(
        get_forward_context=forward_context,
        is_conv_state_dim_first=lambda: True,
        causal_conv1d_fn=rec.wrap('conv_varlen', conv_varlen),
        causal_conv1d_update=rec.wrap('conv_update', conv_update),
        fused_post_conv_prep=rec.wrap('prep', post_conv_prep),
        fused_olmo_hybrid_gdn_gating=rec.wrap('gating', olmo_gating),
        chunk_gated_delta_rule=rec.wrap('chunk', chunk_gdn),
        chunk_kda=rec.wrap('chunk', chunk_kda),
        mamba_chunk_scan_combined_varlen=rec.wrap('chunk', chunk_scan_mamba2))
    for k, v in extra.items():
        setattr(ns, k, v)
    return ns


def gdn_metadata(dec_slots, pre_slots, pre_lens, pre_hist, device, pad_to=None):
    """The GDN attention metadata of one step: decode sequences first (one token each), then prefill sequences of
    ``pre_lens`` tokens; ``pad_to``: a decode-only step padded with null-slot rows to this many rows."""
    nd, npf = len(dec_slots), len(pre_slots)
    lens = [1] * nd + list(pre_lens)
    qsl = torch.tensor([0] + torch.tensor(lens, dtype=torch.int64).cumsum(0).tolist(), dtype=torch.int32)
    slots = list(dec_slots) + list(pre_slots)
    tokens = int(qsl[-1])
    if pad_to is not None:
        assert npf == 0 and pad_to >= nd
        slots += [0] * (pad_to - nd)
        tokens = pad_to
    md = SimpleNamespace(
        num_prefills=npf, num_prefill_tokens=sum(pre_lens), num_decodes=nd, num_decode_tokens=nd,
        num_actual_tokens=tokens, spec_sequence_masks=None, non_spec_query_start_loc=qsl.to(device),
        non_spec_state_indices_tensor=torch.tensor(slots, dtype=torch.int32, device=device),
        chunk_indices=None, chunk_offsets=None, aiter_prefill_metadata=None)
    if npf:
        hist = torch.tensor([True] * nd + list(pre_hist), device=device)
        md.has_initial_state = hist
        md.prefill_query_start_loc = (qsl[nd:] - nd).to(device)
        md.prefill_state_indices = torch.tensor(pre_slots, dtype=torch.int32, device=device)
        md.prefill_has_initial_state = hist[nd:]
    return md


def mamba2_metadata(dec_slots, pre_slots, pre_lens, pre_hist, device):
    nd, npf = len(dec_slots), len(pre_slots)
    md = SimpleNamespace(
        num_prefills=npf, num_prefill_tokens=sum(pre_lens), num_decodes=nd, num_decode_tokens=nd,
        checkpoint_chunk_idx=None, num_accepted_tokens=None, query_start_loc_d=None,
        state_indices_tensor_d=torch.tensor(dec_slots, dtype=torch.int32, device=device),
        chunk_size=8, seq_idx_p=None, cu_chunk_seqlen_p=None, last_chunk_indices_p=None)
    if npf:
        qsl = torch.tensor([0] + torch.tensor(list(pre_lens), dtype=torch.int64).cumsum(0).tolist(), dtype=torch.int32)
        md.query_start_loc_p = qsl.to(device)
        md.state_indices_tensor_p = torch.tensor(pre_slots, dtype=torch.int32, device=device)
        md.has_initial_states_p = torch.tensor(list(pre_hist), device=device)
        md.prep_initial_states = any(pre_hist)
    return md
