"""KDA layers (Ling-3.0's ``BailingMoeV3KimiDeltaAttention``) under STATEQUANT_VLLM: slot layouts, the allocator's
state shape, the calculator and layer patches and the layer forward
(/root/reference/src/statequant/integrations/vllm_kda.py:33-191).

The decay is a vector per key channel and token (``g1`` [1, tokens, H, d_k] fp32 from the engine's gating), there are
three separate convs (q, k, v) over one conv state split in three along its channel dim, and one key head per value
head.  Asserted: tensor parallel 1, no speculative decoding / MTP, no prefix caching.
"""
from __future__ import annotations

import sys

import torch

from . import _engine as E

# the state calculators answer packed only to callers from this engine module (its model hooks and the KDA layer)
_CALLERS = frozenset({'vllm.model_executor.models.bailing_moe_v3'})
_state = {}

_layouts = {}


def reset():
    _layouts.clear()


def layout(cfg, heads, head_dim):
    from ..kernels.kda import KDASlotLayout
    fmt, m, buffer_bits, _ = cfg
    if (heads, head_dim) not in _layouts:
        _layouts[(heads, head_dim)] = KDASlotLayout(fmt, heads, head_dim, head_dim, m=m, buffer_bits=buffer_bits)
    return _layouts[(heads, head_dim)]


def kda_state_shape(cfg, tp_world_size, num_heads, head_dim, num_k_heads=None, head_k_dim=None, num_spec=0):
    """The recurrent-state shape for the allocator: (bytes per slot,).  KDA here has one key head per value head and
    square heads; tensor parallelism and speculative decoding / MTP are refused, as in the reference."""
    assert tp_world_size == 1, 'statequant vLLM plugin (KDA): tensor parallel > 1 is not supported'
    assert num_spec == 0, 'statequant vLLM plugin (KDA): speculative decoding / MTP is not supported'
    assert num_k_heads in (None, num_heads) and head_k_dim in (None, head_dim), (num_k_heads, head_k_dim)
    return (layout(cfg, num_heads, head_dim).nbytes,)


def state_dtype():
    return torch.uint8


def _from_engine_model(depth=2):
    return sys._getframe(depth).f_globals.get('__name__') in _CALLERS


def _patch_calculators(cfg, mu=None, scoped=_from_engine_model):
    """Replace the engine's KDA state shape / dtype calculators (``mu``: its ``mamba_utils`` module); callers outside
    the KDA model's module keep the stock answer."""
    if mu is None:
        from vllm.model_executor.layers.mamba import mamba_utils as mu
    stock_shape = mu.MambaStateShapeCalculator.kda_state_shape
    stock_dtype = mu.MambaStateDtypeCalculator.kda_state_dtype
    _state['calculators'] = (mu, mu.MambaStateShapeCalculator.__dict__['kda_state_shape'],
                             mu.MambaStateDtypeCalculator.__dict__['kda_state_dtype'])

    def packed_shape(cls, tp_world_size, num_heads, head_dim, num_k_heads=None, head_k_dim=None, conv_kernel_size=4,
                     num_spec=0):
        conv_shape, rec_shape = stock_shape(tp_world_size, num_heads, head_dim, num_k_heads=num_k_heads,
                                            head_k_dim=head_k_dim, conv_kernel_size=conv_kernel_size,
                                            num_spec=num_spec)
        if not scoped():
            return conv_shape, rec_shape
        heads, dv, dk = rec_shape
        assert dv == dk == head_dim, rec_shape
        return conv_shape, kda_state_shape(cfg, tp_world_size, heads, head_dim, num_k_heads, head_k_dim, num_spec)

    def packed_dtype(cls, model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype='auto'):
        conv_dtype, rec_dtype = stock_dtype(model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype)
        return (conv_dtype, state_dtype()) if scoped() else (conv_dtype, rec_dtype)

    mu.MambaStateShapeCalculator.kda_state_shape = classmethod(packed_shape)
    mu.MambaStateDtypeCalculator.kda_state_dtype = classmethod(packed_dtype)


def attach(layer, cfg, vllm_config, log=None):
    """The patched ``__init__``'s additions: refusals, the slot layout."""
    assert layer.tp_size == 1, 'statequant vLLM plugin (KDA): tensor parallel > 1 is not supported'
    assert layer.num_speculative_tokens == 0 and vllm_config.speculative_config is None, \
        'statequant vLLM plugin (KDA): speculative decoding / MTP is not supported'
    E.check_cache_settings(vllm_config, 'statequant vLLM plugin (KDA)')
    layer._sq_layout = layout(cfg, layer.local_num_heads, layer.head_dim)
    layer._sq_views = None
    if log is not None and not _state.get('logged'):
        _state['logged'] = True
        lay = layer._sq_layout
        log.info('statequant: KDA recurrent state stored as %s; stock state %d B/slot per layer in fp32; decode via '
                 'the HIP slot kernel of libsqhip', lay, lay.HV * lay.DV * lay.DK * 4)


def _patch_layer(cfg, M=None):
    if M is None:
        from vllm.model_executor.models import bailing_moe_v3 as M
    cls = M.BailingMoeV3KimiDeltaAttention
    if getattr(cls, '_statequant_patched', False):
        return
    stock_init = cls.__init__
    _state['saved'] = (cls, stock_init, cls.__dict__.get('_forward'))

    def __init__(self, config, *args, **kw):
        stock_init(self, config, *args, **kw)
        log = None
        if hasattr(M, 'init_logger'):
            log = M.init_logger('vllm.statequant')
        attach(self, cfg, M.get_current_vllm_config(), log)

    cls.__init__ = __init__
    cls._forward = _forward
    cls._statequant_patched = True
    _state['M'] = M


def patch(cfg, M=None, mu=None):
    """Calculators + layer class (engine modules imported from vLLM when not given).  Idempotent."""
    if _state.get('patched'):
        return
    _state['cfg'] = cfg
    _patch_calculators(cfg, mu)
    _patch_layer(cfg, M)
    _state['patched'] = True


def unpatch():
    """Undo ``patch`` (tests)."""
    if 'calculators' in _state:
        mu, shape0, dtype0 = _state['calculators']
        mu.MambaStateShapeCalculator.kda_state_shape = shape0
        mu.MambaStateDtypeCalculator.kda_state_dtype = dtype0
    if 'saved' in _state:
        cls, init, fwd = _state['saved']
        cls.__init__ = init
        if fwd is None:
            del cls._forward
        else:
            cls._forward = fwd
        cls._statequant_patched = False
    _state.clear()


def _forward(self, q_proj_states, k_proj_states, v_proj_states, g1, beta, core_attn_out):
    """``BailingMoeV3KimiDeltaAttention._forward`` on the packed slot state (non-speculative path).

    q / k / v_proj_states [tokens, H d] before their convs, g1 [1, tokens, H, d_k] fp32 log decays, beta
    [1, tokens, H] fp32, core_attn_out [1, tokens, H, d_v] written in place."""
    M = _state['M']
    if M.get_forward_context().attn_metadata is None:
        return
    md = E.layer_metadata(M, self)
    if md is None:                                           # profile / warm-up runs
        return
    assert md.spec_sequence_masks is None, 'statequant vLLM plugin (KDA): speculative decoding is not supported'
    lay, views = self._sq_layout, E.slot_views(self)
    heads, d = lay.HV, lay.DK
    tokens = md.num_actual_tokens
    n_dec, n_pre = md.num_decodes, md.num_prefills
    if n_dec == 0 and n_pre == 0:
        return
    slots = md.non_spec_state_indices_tensor
    g1, beta = g1[0, :tokens], beta[0, :tokens]
    convs = (self.q_conv1d, self.k_conv1d, self.v_conv1d)
    streams = zip((q_proj_states[:tokens], k_proj_states[:tokens], v_proj_states[:tokens]), convs,
                  E.conv_state(M, self).chunk(3, dim=-2))
    if n_pre > 0:
        q, k, v = [M.causal_conv1d_fn(x.transpose(0, 1), E.conv_taps(c), c.bias, activation='silu', conv_states=cs,
                                      has_initial_state=md.has_initial_state, cache_indices=slots,
                                      query_start_loc=md.non_spec_query_start_loc, metadata=md).transpose(0, 1)
                   for x, c, cs in streams]
    else:
        q, k, v = [M.causal_conv1d_update(x, cs, E.conv_taps(c), c.bias, activation='silu',
                                          conv_state_indices=slots[:tokens], validate_data=False)
                   for x, c, cs in streams]

    if n_dec > 0:
        rows = E.decode_row_count(tokens, n_dec, n_pre)
        idx = E.slot_index(slots, rows)
        qd, kd, vd = (E.unit_stride_rows(x, rows).unflatten(1, (heads, d)) for x in (q, k, v))
        lay.step(views, idx, qd, kd, vd, g1[:rows], beta[:rows], core_attn_out[0, :rows], self.head_dim ** -0.5,
                 order=E.dispatch_order(M, lay, views, slots, idx))

    if n_pre > 0:
        span = tokens - n_dec
        qp, kp, vp = (x[n_dec:tokens].reshape(1, span, heads, d) for x in (q, k, v))
        pslots = md.prefill_state_indices
        init = E.prefill_initial_state(lay, views, pslots, md.prefill_has_initial_state)
        o, last = M.chunk_kda(q=qp, k=kp, v=vp, g=g1[n_dec:tokens].unsqueeze(0).contiguous(),
                              beta=beta[n_dec:tokens].unsqueeze(0).contiguous(), initial_state=init,
                              output_final_state=True, use_qk_l2norm_in_kernel=True, safe_gate=self.safe_gate,
                              lower_bound=self.lower_bound, cu_seqlens=md.prefill_query_start_loc)
        lay.write(views, pslots, last)
        core_attn_out[0, n_dec:tokens] = o[0]
