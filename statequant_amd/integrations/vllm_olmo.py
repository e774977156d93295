"""OLMo-Hybrid's Gated DeltaNet layer on the packed slot state
(/root/reference/src/statequant/integrations/vllm_olmo.py:33-150).

Differences from the Qwen layer that matter here: head dims 96 x 192 (the slot kernels pad key tiles internally and
store exactly d_k x d_v), one key head per value head, a conv without bias, and beta = 2 sigmoid(b) when the model
allows negative eigenvalues -- so the decode rows take g and beta from the engine's own gating op
(``fused_olmo_hybrid_gdn_gating``) instead of the step kernel's in-kernel gate, and the prefill chunk kernel
normalises q, k itself.  The state shape / dtype calculators are ``vllm_plugin``'s.
"""
from __future__ import annotations

from . import _engine as E

LAYER = ('vllm.model_executor.layers.mamba.gdn.olmo_gdn_linear_attn', 'OlmoHybridGatedDeltaNetAttention')
MODEL_MODULE = 'vllm.model_executor.models.olmo_hybrid'
_state = {}


def attach(layer, vllm_config, layout, log=None):
    """The patched ``__init__``'s additions: refusals, this rank's slot layout."""
    E.check_cache_settings(vllm_config, 'statequant vLLM plugin')
    tp = layer.tp_size
    layer._sq_layout = layout(layer.num_v_heads // tp, layer.num_k_heads // tp, layer.head_k_dim, layer.head_v_dim)
    layer._sq_views = None
    if log is not None and not _state.get('logged'):
        _state['logged'] = True
        lay = layer._sq_layout
        log.info('statequant: OLMo-Hybrid GDN recurrent state stored as %s, %d B/slot per layer (stock bf16 state %d '
                 'B); decode via the HIP slot kernels of libsqhip', lay, lay.nbytes, lay.HV * lay.DV * lay.DK * 2)


def patch(layout, O=None):
    """Patch ``OlmoHybridGatedDeltaNetAttention`` in the engine module ``O`` (imported from vLLM when None);
    ``layout(hv, hk, dk, dv)`` is ``vllm_plugin.layout``.  Idempotent."""
    if O is None:
        from vllm.model_executor.layers.mamba.gdn import olmo_gdn_linear_attn as O
    cls = O.OlmoHybridGatedDeltaNetAttention
    if getattr(cls, '_statequant_patched', False):
        return
    stock_init = cls.__init__
    _state['saved'] = (cls, {name: cls.__dict__.get(name) for name in ('__init__', '_forward_core')})

    def __init__(self, config, vllm_config, *args, **kw):
        stock_init(self, config, vllm_config, *args, **kw)
        import logging
        attach(self, vllm_config, layout, logging.getLogger('vllm'))

    cls.__init__ = __init__
    cls._forward_core = _forward_core
    cls._statequant_patched = True
    _state['O'] = O


def unpatch():
    """Undo ``patch`` (tests)."""
    saved = _state.get('saved')
    if saved is not None:
        cls, methods = saved
        for name, fn in methods.items():
            if fn is not None:
                setattr(cls, name, fn)
            elif name in cls.__dict__:
                delattr(cls, name)
        cls._statequant_patched = False
    _state.clear()


def _forward_core(self, mixed_qkv, b, a, core_attn_out):
    """``OlmoHybridGatedDeltaNetAttention._forward_core`` on the packed slot state (non-speculative path)."""
    O = _state['O']
    md = E.layer_metadata(O, self)
    if md is None:                                           # profiling / warm-up runs carry no metadata
        return
    assert md.spec_sequence_masks is None, 'statequant vLLM plugin: speculative decoding is not supported'
    lay, views = self._sq_layout, E.slot_views(self)
    tokens = md.num_actual_tokens
    n_dec, n_pre = md.num_decodes, md.num_prefills
    if n_dec == 0 and n_pre == 0:
        return
    mixed_qkv, b, a = mixed_qkv[:tokens], b[:tokens], a[:tokens]
    slots = md.non_spec_state_indices_tensor
    taps, cstate = E.conv_taps(self.conv1d), E.conv_state(O, self)
    if n_pre > 0:
        x = O.causal_conv1d_fn(mixed_qkv.transpose(0, 1), taps, None, activation=self.activation, conv_states=cstate,
                               has_initial_state=md.has_initial_state, cache_indices=slots,
                               query_start_loc=md.non_spec_query_start_loc, metadata=md).transpose(0, 1)
    else:
        x = O.causal_conv1d_update(mixed_qkv, cstate, taps, None, self.activation,
                                   conv_state_indices=slots[:tokens], validate_data=False)

    # the engine's gate for every token of the step: g, beta [1, tokens, hv]
    g, beta = O.fused_olmo_hybrid_gdn_gating(self.A_log, a, b, self.dt_bias, self.allow_neg_eigval)

    if n_dec > 0:
        rows = E.decode_row_count(tokens, n_dec, n_pre)
        xd, idx = E.unit_stride_rows(x, rows), E.slot_index(slots, rows)
        kw = lay.HK * lay.DK
        lay.step(views, idx, xd[:, :kw].unflatten(1, (lay.HK, lay.DK)), xd[:, kw:2 * kw].unflatten(1, (lay.HK, lay.DK)),
                 xd[:, 2 * kw:].unflatten(1, (lay.HV, lay.DV)), core_attn_out[:rows], self.head_k_dim ** -0.5,
                 g=g[0, :rows], beta=beta[0, :rows], order=E.dispatch_order(O, lay, views, slots, idx))

    if n_pre > 0:
        q, k, v = self.rearrange_mixed_qkv(x[n_dec:])
        pslots = md.prefill_state_indices
        init = E.prefill_initial_state(lay, views, pslots, md.prefill_has_initial_state)
        o, last = O.chunk_gated_delta_rule(
            q=q, k=k, v=v, g=g[:, n_dec:], beta=beta[:, n_dec:], initial_state=init, output_final_state=True,
            cu_seqlens=md.prefill_query_start_loc, chunk_indices=md.chunk_indices, chunk_offsets=md.chunk_offsets,
            use_qk_l2norm_in_kernel=True)
        lay.write(views, pslots, last)
        o = o.squeeze(0)
        core_attn_out[n_dec:n_dec + o.shape[0]] = o
