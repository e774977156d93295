"""Mamba2 / SSD layers (every model built on the engine's ``MambaMixer2``) under STATEQUANT_VLLM: format fitting,
slot layouts, the allocator's state shape, the calculator and layer patches and the layer's ``conv_ssm_forward``
(/root/reference/src/statequant/integrations/vllm_mamba2.py:32-209).

The ssm state (stock: [H, head_dim, d_state] fp32 or the model dtype) becomes one uint8 blob per slot; decode rows run
``Mamba2SlotLayout.step`` (dt bias + softplus in the kernel, D x added), prefill rows read their slot's state as fp32,
run the engine's chunk scan from it and store the final state packed.  Asserted: tensor parallel 1, no speculative
decoding, no prefix caching, no ReplaySSM, no prefill checkpoints.
"""
from __future__ import annotations

import dataclasses
import sys

import torch

from . import _engine as E

# the state calculators answer packed only to MambaMixer2 itself and to the model modules built on it
_CALLERS = frozenset('vllm.model_executor.' + name for name in (
    'layers.mamba.mamba_mixer2', 'models.nemotron_h', 'models.granitemoehybrid', 'models.zamba2',
    'models.falcon_h1', 'models.mamba2'))
_state = {}

_layouts = {}


def reset():
    _layouts.clear()


def _fmt_for(fmt, dk, dv):
    """The configured format with its group halved until it divides the axis it runs along -- a value-axis group of
    32 on head_dim 80 becomes 16 -- and never below 2 (vllm_mamba2.py:42-54)."""
    from ..kernels.fold import packed_format
    spec = packed_format(fmt)
    if spec is None:                                       # the unquantized control
        return fmt
    extent = dk if spec.axis == 'k' else dv
    group = spec.group
    while group > 2 and extent % group:
        group //= 2
    return fmt if group == spec.group else dataclasses.replace(fmt, group=group)


def layout(cfg, heads, groups, d_state, head_dim):
    from ..kernels.mamba2 import Mamba2SlotLayout
    fmt, m, buffer_bits, _ = cfg
    key = (heads, groups, d_state, head_dim)
    if key not in _layouts:
        _layouts[key] = Mamba2SlotLayout(_fmt_for(fmt, d_state, head_dim), heads, groups, d_state, head_dim, m=m,
                                         buffer_bits=buffer_bits)
    return _layouts[key]


def mamba2_state_shape(cfg, tp_world_size, n_groups, num_heads, head_dim, state_size, num_spec=0):
    """The ssm-state shape for the allocator: (bytes per slot,).  Asserted restrictions as in the reference."""
    assert tp_world_size == 1, 'statequant vLLM plugin (Mamba2): tensor parallel > 1 is not supported'
    assert num_spec == 0, 'statequant vLLM plugin (Mamba2): speculative decoding is not supported'
    return (layout(cfg, num_heads, n_groups, state_size, head_dim).nbytes,)


def state_dtype():
    return torch.uint8


def _from_mixer_or_model(depth=2):
    return sys._getframe(depth).f_globals.get('__name__') in _CALLERS


def _patch_calculators(cfg, mu=None, scoped=_from_mixer_or_model):
    """Replace the engine's Mamba2 state shape / dtype calculators (``mu``: its ``mamba_utils`` module); any caller
    outside ``_CALLERS`` keeps the stock answer."""
    if mu is None:
        from vllm.model_executor.layers.mamba import mamba_utils as mu
    stock_shape = mu.MambaStateShapeCalculator.mamba2_state_shape
    stock_dtype = mu.MambaStateDtypeCalculator.mamba2_state_dtype
    _state['calculators'] = (mu, mu.MambaStateShapeCalculator.__dict__['mamba2_state_shape'],
                             mu.MambaStateDtypeCalculator.__dict__['mamba2_state_dtype'])

    def packed_shape(cls, tp_world_size, intermediate_size, n_groups, num_heads, head_dim, state_size, conv_kernel,
                     num_spec=0):
        conv_shape, ssm_shape = stock_shape(tp_world_size=tp_world_size, intermediate_size=intermediate_size,
                                            n_groups=n_groups, num_heads=num_heads, head_dim=head_dim,
                                            state_size=state_size, conv_kernel=conv_kernel, num_spec=num_spec)
        if not scoped():
            return conv_shape, ssm_shape
        heads, hd, n = ssm_shape                              # this rank's heads
        return conv_shape, mamba2_state_shape(cfg, tp_world_size, n_groups, heads, hd, n, num_spec)

    def packed_dtype(cls, model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype):
        conv_dtype, ssm_dtype = stock_dtype(model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype)
        return (conv_dtype, state_dtype()) if scoped() else (conv_dtype, ssm_dtype)

    mu.MambaStateShapeCalculator.mamba2_state_shape = classmethod(packed_shape)
    mu.MambaStateDtypeCalculator.mamba2_state_dtype = classmethod(packed_dtype)


def attach(layer, cfg, vllm_config, log=None):
    """The patched ``__init__``'s additions: refusals, the slot layout."""
    assert layer.tp_size == 1, 'statequant vLLM plugin (Mamba2): tensor parallel > 1 is not supported'
    assert layer.num_spec == 0 and vllm_config.speculative_config is None, \
        'statequant vLLM plugin (Mamba2): speculative decoding is not supported'
    assert not layer.use_replayssm, 'statequant vLLM plugin (Mamba2): ReplaySSM (--use-replayssm) is not supported'
    E.check_cache_settings(vllm_config, 'statequant vLLM plugin (Mamba2)')
    layer._sq_layout = layout(cfg, layer.num_heads, layer.n_groups, layer.ssm_state_size, layer.head_dim)
    layer._sq_views = None
    if log is not None and not _state.get('logged'):
        _state['logged'] = True
        lay = layer._sq_layout
        log.info('statequant: Mamba2 ssm state stored as %s; stock state %d B/slot per layer in %s; decode via the '
                 'HIP slot kernel of libsqhip', lay, lay.HV * lay.DV * lay.DK * 4,
                 vllm_config.cache_config.mamba_ssm_cache_dtype)


def _patch_layer(cfg, M=None):
    if M is None:
        from vllm.model_executor.layers.mamba import mamba_mixer2 as M
    cls = M.MambaMixer2
    if getattr(cls, '_statequant_patched', False):
        return
    stock_init, stock_warmup = cls.__init__, cls._warmup_ssd_kernels
    _state['saved'] = (cls, stock_init, stock_warmup, cls.__dict__.get('conv_ssm_forward'))

    def __init__(self, *args, **kw):
        stock_init(self, *args, **kw)
        attach(self, cfg, M.get_current_vllm_config(), getattr(M, 'logger', None))

    def _warmup_ssd_kernels(self, projected_states):
        # the stock warm-up allocates a dummy ssm state in the state dtype: the chunk scan is warmed with fp32 states
        conv_dtype = type(self).get_state_dtype(self)[0]
        self.get_state_dtype = lambda: (conv_dtype, torch.float32)
        try:
            return stock_warmup(self, projected_states)
        finally:
            del self.get_state_dtype

    cls.__init__ = __init__
    cls._warmup_ssd_kernels = _warmup_ssd_kernels
    cls.conv_ssm_forward = conv_ssm_forward
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
        mu.MambaStateShapeCalculator.mamba2_state_shape = shape0
        mu.MambaStateDtypeCalculator.mamba2_state_dtype = dtype0
    if 'saved' in _state:
        cls, init, warmup, fwd = _state['saved']
        cls.__init__, cls._warmup_ssd_kernels = init, warmup
        if fwd is None:
            del cls.conv_ssm_forward
        else:
            cls.conv_ssm_forward = fwd
        cls._statequant_patched = False
    _state.clear()


def conv_ssm_forward(self, projected_states, output):
    """``MambaMixer2.conv_ssm_forward`` on the packed slot state.

    projected_states [tokens, intermediate | x B C | dt] (this rank's columns), output [tokens, H head_dim] written in
    place.  Here the engine orders a step's tokens decode-first and gives decode and prefill their own slot tensors
    (``state_indices_tensor_d`` / ``_p``)."""
    M = _state['M']
    xBC, dt = torch.split(projected_states[..., self.tped_intermediate_size:],
                          [self.tped_conv_size, self.tped_dt_size], dim=-1)
    md = E.layer_metadata(M, self)
    if md is None:                                           # the engine's profiling run, as stock
        self._warmup_ssd_kernels(projected_states)
        xBC = xBC.transpose(0, 1).clone().transpose(0, 1).contiguous()
        return self.split_hidden_states_B_C_fn(xBC)[0]
    assert md.checkpoint_chunk_idx is None, 'statequant vLLM plugin (Mamba2): prefill checkpoints are unsupported'
    lay, views = self._sq_layout, E.slot_views(self)
    cstate = E.conv_state(M, self)
    heads, groups, hd, n = lay.HV, lay.HK, lay.DV, lay.DK
    t_dec, t_pre = md.num_decode_tokens, md.num_prefill_tokens
    used = t_dec + t_pre
    xBC_d, xBC_p = torch.split(xBC[:used], [t_dec, t_pre], dim=0)
    dt_d, dt_p = torch.split(dt[:used], [t_dec, t_pre], dim=0)
    out_d, out_p = torch.split(output[:used], [t_dec, t_pre], dim=0)

    if md.num_prefills > 0:
        pslots = md.state_indices_tensor_p
        xBC_p = M.causal_conv1d_fn(xBC_p.transpose(0, 1), self.conv_weights, self.conv1d.bias,
                                   activation=self.activation, conv_states=cstate,
                                   has_initial_state=md.has_initial_states_p, cache_indices=pslots, metadata=md,
                                   query_start_loc=md.query_start_loc_p).transpose(0, 1)[:t_pre]
        x_p, B_p, C_p = self.split_hidden_states_B_C_fn(xBC_p)
        init = None
        if md.has_initial_states_p is not None and md.prep_initial_states:
            init = E.prefill_initial_state(lay, views, pslots, md.has_initial_states_p)
        final = M.mamba_chunk_scan_combined_varlen(
            x_p.view(t_pre, heads, hd), dt_p, self.A, B_p.view(t_pre, groups, -1), C_p.view(t_pre, groups, -1),
            chunk_size=md.chunk_size, D=self.D, z=None, dt_bias=self.dt_bias, seq_idx=md.seq_idx_p,
            cu_seqlens=md.query_start_loc_p, cu_chunk_seqlens=md.cu_chunk_seqlen_p,
            last_chunk_indices=md.last_chunk_indices_p, initial_states=init, return_intermediate_states=False,
            dt_softplus=True, dt_limit=(0.0, float('inf')), out=out_p.view(t_pre, -1, hd), state_dtype=torch.float32)
        lay.write(views, pslots, final)

    if md.num_decodes > 0:
        dslots = md.state_indices_tensor_d
        xBC_d = M.causal_conv1d_update(xBC_d, cstate, self.conv_weights, self.conv1d.bias, self.activation,
                                       conv_state_indices=dslots, num_accepted_tokens=md.num_accepted_tokens,
                                       query_start_loc=md.query_start_loc_d, max_query_len=dslots.size(-1))
        x_d, B_d, C_d = self.split_hidden_states_B_C_fn(xBC_d)
        idx = E.slot_index(dslots[:, 0] if dslots.dim() == 2 else dslots, t_dec)
        lay.step(views, idx, x_d.view(t_dec, heads, hd), dt_d, B_d.view(t_dec, groups, n), C_d.view(t_dec, groups, n),
                 out_d.view(t_dec, heads, hd), self.A, self.D, self.dt_bias, dt_softplus=True,
                 dt_limit=(0.0, float('inf')), order=E.dispatch_order(M, lay, views, dslots, idx))
