"""The serving-engine plugin for Gated DeltaNet layers: STATEQUANT_VLLM=<format> -> storage configuration ->
per-layer slot layouts -> the cache allocator's state shape -> the layer forward that decodes on the HIP slot ops.

Follows the reference's plugin (/root/reference/src/statequant/integrations/vllm_plugin.py): ``config`` (:76-120)
reads the environment, ``layout`` (:123-141) keeps one slot layout per head geometry, ``register`` (:144-166) is the
``vllm.general_plugins`` entry point, the patched state calculators (:252-279) answer "(nbytes,) of uint8" for the
recurrent state to the callers whose layers have a packed forward and refuse the others (:229-249), the layer patch
(:285-344) adds the construction-time checks, and ``_forward_core`` (:355-430) is the layer's core with the decode
rows on ``SlotLayout.step`` and the prefill rows on ``read`` -> the engine's chunk kernel -> ``write``.  The names,
the environment variables and the error texts' substance follow it, so that a deployment's settings carry over
unchanged.  Nothing here imports the engine at module level; ``register`` and the patch functions import it when they
run, or take the engine's modules as arguments (tests hand in stand-ins).

    STATEQUANT_VLLM              off | pace4 | int4k | int4v | int8k | int8v | bf16 | fp32 | int<4|8><k|v>g<group>
                                 | gga:<plan.pt>[:pw] | external:<file.py or module>:<function>
    STATEQUANT_VLLM_EXTERNAL_DTYPE   fp32 (default) | bf16: the unpacked slot state an external quantizer works on
    STATEQUANT_VLLM_EXTERNAL_GRAPHS  1: decode steps may be captured; the function then runs on every decode row
    STATEQUANT_VLLM_M            tokens per fold period (decode buffer length), default 8
    STATEQUANT_VLLM_BUFFER_BITS  8 (int8 buffer) or 16 (bf16), default 8
    STATEQUANT_VLLM_FUSED        0 | 1 | auto -- accepted and recorded; the HIP step is always one fused launch
    STATEQUANT_VLLM_LAYERS       comma-separated subset of gdn, mamba2, kda (default: all)
    STATEQUANT_VLLM_PW_M         window length of the gga:...:pw slot, default 8
"""
from __future__ import annotations

import os
import re

import torch

ENV = 'STATEQUANT_VLLM'
LAYER_KINDS = ('gdn', 'mamba2', 'kda')
OFF = ('', '0', 'off', 'none', 'stock')
# preset name -> (bits, axis, group)
PRESETS = {'pace4': (4, 'k', 64), 'int4k': (4, 'k', 64), 'int4v': (4, 'v', 32), 'int8k': (8, 'k', 32),
           'int8v': (8, 'v', 32)}
_SPELLED = re.compile(r'int(?P<bits>[48])(?P<axis>[kv])g(?P<group>\d+)')
_state = {}


def _env(environ, name, default=''):
    return (os.environ if environ is None else environ).get(name, default)


def parse_format(mode):
    """A format name -> Quantizer | 'bf16' | 'fp32'; AssertionError naming the accepted spellings otherwise."""
    from ..quantizer import Quantizer
    if mode in ('bf16', 'fp32'):
        return mode
    triple = PRESETS.get(mode)
    if triple is None:
        hit = _SPELLED.fullmatch(mode)
        assert hit, (f'{ENV}={mode!r}: use pace4, int4k, int4v, int8k, int8v, bf16, fp32, gga:<plan.pt>[:pw], external:<src>:<fn> or '
                     f'int<4|8><k|v>g<group>')
        triple = (int(hit['bits']), hit['axis'], int(hit['group']))
    return Quantizer(*triple)


def config(environ=None):
    """(fmt, m, buffer_bits, fused) from the environment (``environ``: a mapping to read instead of ``os.environ``),
    or None when the plugin is off.  fmt: Quantizer | 'bf16' | 'fp32' | 'gga' (then ``gga_settings()`` holds the plan
    file, the window flag and its length)."""
    raw = _env(environ, ENV).strip()
    mode = raw.lower()
    _state.pop('gga', None)
    _state.pop('external', None)
    _state.pop('external_fn', None)
    if mode in OFF:
        return None
    if mode.startswith('external:'):
        source, _, name = raw[len('external:'):].rpartition(':')
        assert source and name, f'{ENV}=external:<file.py or module>:<function>, got {raw[len("external:"):]!r}'
        kept_as = _env(environ, 'STATEQUANT_VLLM_EXTERNAL_DTYPE', 'fp32').strip().lower()
        assert kept_as in ('fp32', 'bf16'), f'STATEQUANT_VLLM_EXTERNAL_DTYPE={kept_as!r}: use fp32 or bf16'
        _state['external'] = (source, name)
        fmt = kept_as
    elif mode.startswith('gga:'):
        spec = raw[len('gga:'):]
        windowed = spec.endswith(':pw')
        path = spec[:-len(':pw')] if windowed else spec
        assert os.path.exists(path), f'{ENV}=gga:<plan.pt>[:pw]: no plan file {path!r}'
        _state['gga'] = (path, windowed, int(_env(environ, 'STATEQUANT_VLLM_PW_M', '8')))
        fmt = 'gga'
    else:
        fmt = parse_format(mode)
    m = int(_env(environ, 'STATEQUANT_VLLM_M', '8'))
    buffer_bits = int(_env(environ, 'STATEQUANT_VLLM_BUFFER_BITS', '8'))
    fz = _env(environ, 'STATEQUANT_VLLM_FUSED', 'auto').strip().lower()
    assert fz in ('auto', '', '0', '1'), f'STATEQUANT_VLLM_FUSED={fz!r}: use 0, 1 or auto'
    return fmt, m, buffer_bits, (None if fz in ('auto', '') else fz == '1')


def gga_settings():
    """(plan file, window kept, window length) of the last ``config()`` that read a gga: format."""
    return _state['gga']


def layer_kinds(environ=None):
    """The layer types to pack, from STATEQUANT_VLLM_LAYERS (default: all of LAYER_KINDS)."""
    listed = [k.strip() for k in _env(environ, 'STATEQUANT_VLLM_LAYERS').lower().split(',') if k.strip()]
    unknown = [k for k in listed if k not in LAYER_KINDS]
    assert not unknown, f'STATEQUANT_VLLM_LAYERS: unknown {unknown}; use a subset of {",".join(LAYER_KINDS)}'
    return tuple(listed) or LAYER_KINDS


def configure(environ=None):
    """Read the environment, drop every cached layout, and remember the configuration for ``layout``.  Returns the
    configuration (None: off).  fp32 and gga formats exist for Gated DeltaNet layers only."""
    from . import vllm_kda, vllm_mamba2
    cfg = config(environ)
    _state.pop('layouts', None)
    _state.pop('plan', None)
    vllm_mamba2.reset()
    vllm_kda.reset()
    _state['cfg'] = cfg
    if cfg is not None:
        kinds = layer_kinds(environ)
        if cfg[0] in ('fp32', 'gga') or 'external' in _state:
            assert kinds in (('gdn',), LAYER_KINDS), f'{ENV}={_env(environ, ENV)!r}: GDN layers only'
            kinds = ('gdn',)
        _state['kinds'] = kinds
    return cfg


def active_kinds():
    return _state.get('kinds', ())


def layout(hv, hk, dk, dv):
    """The slot layout of a Gated DeltaNet layer with this rank's head geometry; one object per geometry."""
    fmt, m, buffer_bits, fused = _state['cfg']
    cache = _state.setdefault('layouts', {})
    key = (hv, hk, dk, dv)
    if key not in cache:
        if fmt == 'gga':
            from ..kernels.gga import GGAPacked, GGAPlan
            path, windowed, window_len = _state['gga']
            if 'plan' not in _state:
                _state['plan'] = GGAPlan.load(path)
            cache[key] = GGAPacked(_state['plan'], hv, hk, dk, dv, pw=windowed, m=window_len)
        else:
            from ..kernels.slots import SlotLayout
            cache[key] = SlotLayout(fmt, hv, hk, dk, dv, m=m, buffer_bits=buffer_bits, fused=fused)
    return cache[key]


def gated_delta_net_state_shape(tp_world_size, num_k_heads, num_v_heads, head_k_dim, head_v_dim, num_spec=0):
    """The recurrent-state shape the engine's allocator gets for a GDN layer: one flat blob of the layout's bytes per
    slot.  Heads are split over tensor-parallel ranks (each rank packs its own heads); speculative decoding keeps
    several states per slot and is refused."""
    assert num_spec == 0, 'statequant vLLM plugin: speculative decoding is not supported'
    assert num_v_heads % tp_world_size == 0 and num_k_heads % tp_world_size == 0, (num_v_heads, num_k_heads, tp_world_size)
    return (layout(num_v_heads // tp_world_size, num_k_heads // tp_world_size, head_k_dim, head_v_dim).nbytes,)


def state_dtype():
    """The recurrent-state dtype under the plugin: raw bytes."""
    return torch.uint8


# ---------------------------------------------------------------------------------------------------------------
# external quantizer (vllm_plugin.py:86-96, 186-221 of the reference)
# ---------------------------------------------------------------------------------------------------------------
def external_fn():
    """The callable of ``STATEQUANT_VLLM=external:<src>:<fn>`` (imported once per configuration), or None.  ``src`` is
    a file path (ends in .py or holds a path separator) or an importable module name."""
    named = _state.get('external')
    if named is None:
        return None
    if 'external_fn' not in _state:
        import importlib
        import importlib.util
        source, name = named
        if source.endswith('.py') or os.path.sep in source:
            spec = importlib.util.spec_from_file_location(f'statequant_external_{abs(hash(source))}', source)
            module = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(module)
        else:
            module = importlib.import_module(source)
        fn = getattr(module, name)
        assert callable(fn), f'{source}:{name} is not callable'
        _state['external_fn'] = fn
    return _state['external_fn']


def gdn_ordinal(config, prefix):
    """Position of the layer named ``prefix`` ('...layers.<i>.linear_attn') among the model's linear-attention layers,
    counted from 0 in model order (``config.layer_types``)."""
    hit = re.search(r'layers\.(\d+)\.', prefix)
    assert hit, f'cannot read the layer index from {prefix!r}'
    i = int(hit.group(1))
    kinds = getattr(config, 'layer_types', None)
    assert kinds is not None, 'external quantizer: the config has no layer_types'
    assert kinds[i] == 'linear_attention', (i, kinds[i])
    return sum(k == 'linear_attention' for k in kinds[:i])


def apply_external(S_vk, layer):
    """The external function on value-major states [P, HV, d_v, d_k]: it sees fp32 key-major [P, HV, d_k, d_v] (the
    method's canonical layout) and the layer's ordinal; what it returns comes back value-major fp32."""
    P_, H_, dv, dk = S_vk.shape
    S_hat = external_fn()(S_vk.float().transpose(-1, -2).contiguous(), layer)
    assert tuple(S_hat.shape) == (P_, H_, dk, dv), (tuple(S_hat.shape), tuple(S_vk.shape))
    return S_hat.float().transpose(-1, -2)


# ---------------------------------------------------------------------------------------------------------------
# which callers get the packed state (vllm_plugin.py:178-249 of the reference)
# ---------------------------------------------------------------------------------------------------------------
PACKED_MODEL_MODULES = ('vllm.model_executor.models.qwen3_next', 'vllm.model_executor.models.qwen3_5',
                        'vllm.models.qwen4_exp', 'vllm.model_executor.models.olmo_hybrid')
PACKED_LAYER = ('vllm.model_executor.layers.mamba.gdn.qwen_gdn_linear_attn', 'QwenGatedDeltaNetAttention')
PACKED_LAYERS = (PACKED_LAYER, ('vllm.model_executor.layers.mamba.gdn.olmo_gdn_linear_attn',
                                'OlmoHybridGatedDeltaNetAttention'))


def _caller_supported(frame):
    """(does the caller of a GDN state calculator run a packed forward?, who it is).  A layer asking through its own
    ``get_state_shape`` / ``get_state_dtype`` is recognised by its class (anywhere in the MRO), a model-level hook by
    its module."""
    module = frame.f_globals.get('__name__', '?')
    obj, cls = frame.f_locals.get('self'), frame.f_locals.get('cls')
    owner = cls if obj is None else type(obj)
    who = module if owner is None else f'{getattr(owner, "__qualname__", "?")} ({module})'
    if obj is not None:
        return any((c.__module__, c.__name__) in PACKED_LAYERS for c in type(obj).__mro__), who
    return any(module == m or module.startswith(m + '.') for m in PACKED_MODEL_MODULES), who


def _refuse(who):
    raise NotImplementedError(
        f'statequant vLLM plugin ({ENV}={os.environ.get(ENV)!r}) stores packed GDN states only for Qwen3-Next / '
        f'Qwen3.5 / Qwen4-Exp (QwenGatedDeltaNetAttention) and OLMo-Hybrid (OlmoHybridGatedDeltaNetAttention), not '
        f'for {who}. Unset {ENV} to run this model with stock vLLM.')


def _patch_calculators(mu=None):
    """Replace the engine's GDN state shape / dtype calculators (``mu``: its ``mamba_utils`` module).  Supported
    callers get the conv state unchanged and ``(nbytes,)`` of uint8 for the recurrent state; any other caller raises
    NotImplementedError while the plugin is active, at model-configuration time."""
    import sys
    if mu is None:
        from vllm.model_executor.layers.mamba import mamba_utils as mu
    stock_shape = mu.MambaStateShapeCalculator.gated_delta_net_state_shape
    stock_dtype = mu.MambaStateDtypeCalculator.gated_delta_net_state_dtype
    _state['calculators'] = (mu, mu.MambaStateShapeCalculator.__dict__['gated_delta_net_state_shape'],
                             mu.MambaStateDtypeCalculator.__dict__['gated_delta_net_state_dtype'])

    def packed_shape(cls, tp_world_size, num_k_heads, num_v_heads, head_k_dim, head_v_dim, conv_kernel_size,
                     num_spec=0):
        ok, who = _caller_supported(sys._getframe(1))
        if not ok:
            _refuse(who)
        conv_shape, _ = stock_shape(tp_world_size, num_k_heads, num_v_heads, head_k_dim, head_v_dim,
                                    conv_kernel_size, num_spec)
        return conv_shape, gated_delta_net_state_shape(tp_world_size, num_k_heads, num_v_heads, head_k_dim,
                                                       head_v_dim, num_spec)

    def packed_dtype(cls, model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype='auto'):
        ok, who = _caller_supported(sys._getframe(1))
        if not ok:
            _refuse(who)
        conv_dtype, _ = stock_dtype(model_dtype, mamba_cache_dtype, mamba_ssm_cache_dtype)
        return conv_dtype, state_dtype()

    mu.MambaStateShapeCalculator.gated_delta_net_state_shape = classmethod(packed_shape)
    mu.MambaStateDtypeCalculator.gated_delta_net_state_dtype = classmethod(packed_dtype)


# ---------------------------------------------------------------------------------------------------------------
# the Qwen GDN layer (vllm_plugin.py:285-430 of the reference)
# ---------------------------------------------------------------------------------------------------------------
def attach(layer, config, vllm_config, log=None):
    """What the patched ``__init__`` adds to a freshly built Qwen GDN layer: the refusals (speculative decoding, prefix
    caching), this rank's slot layout, the layer ordinal for per-layer plans and the external quantizer."""
    from . import _engine
    _engine.check_cache_settings(vllm_config, 'statequant vLLM plugin')
    tp = layer.tp_size
    layer._sq_layout = layout(layer.num_v_heads // tp, layer.num_k_heads // tp, layer.head_k_dim, layer.head_v_dim)
    layer._sq_views = None
    layer._sq_external = None
    layer._sq_lk = {}
    if getattr(layer._sq_layout, 'per_layer', False):
        layer._sq_lk = {'layer': gdn_ordinal(config, layer.prefix)}
    if _state.get('external') is not None:
        assert tp == 1, 'statequant external quantizer: no tensor parallelism'
        captured = os.environ.get('STATEQUANT_VLLM_EXTERNAL_GRAPHS', '0').strip() == '1'
        assert captured or vllm_config.model_config.enforce_eager, \
            ('statequant external quantizer: run with enforce_eager=True (or STATEQUANT_VLLM_EXTERNAL_GRAPHS=1 '
             'for a capture-safe fn)')
        external_fn()                                        # import errors surface here, not on the first token
        layer._sq_external = (gdn_ordinal(config, layer.prefix), captured)
    if log is not None and not _state.get('logged'):
        _state['logged'] = True
        lay = layer._sq_layout
        log.info('statequant: GDN recurrent state stored as %s, %d B/slot per layer (stock bf16 state %d B); decode '
                 'via the HIP slot kernels of libsqhip', lay, lay.nbytes, lay.HV * lay.DV * lay.DK * 2)


def _patch_layer(Q=None, O=None, gdn_base=None):
    """Patch ``QwenGatedDeltaNetAttention`` (module ``Q``) and make the GDN base class refuse every subclass other
    than it and OLMo-Hybrid's (module ``O``) at construction, before any weights are loaded."""
    if Q is None:
        from vllm.model_executor.layers.mamba.gdn import base as gdn_base
        from vllm.model_executor.layers.mamba.gdn import olmo_gdn_linear_attn as O
        from vllm.model_executor.layers.mamba.gdn import qwen_gdn_linear_attn as Q
    cls = Q.QwenGatedDeltaNetAttention
    if getattr(cls, '_statequant_patched', False):
        return
    base = gdn_base.GatedDeltaNetAttention
    stock_base_init, stock_init, stock_warmup = base.__init__, cls.__init__, cls._warmup_prefill_kernels
    _state['saved'] = (base, stock_base_init, cls, stock_init, stock_warmup, cls.__dict__.get('_forward_core'))
    packed_classes = (cls, O.OlmoHybridGatedDeltaNetAttention)

    def base_init(self, *args, **kw):
        if not isinstance(self, packed_classes):
            _refuse(f'{type(self).__qualname__} ({type(self).__module__})')
        stock_base_init(self, *args, **kw)

    def __init__(self, config, vllm_config, *args, **kw):
        stock_init(self, config, vllm_config, *args, **kw)
        attach(self, config, vllm_config, getattr(Q, 'logger', None))

    def _warmup_prefill_kernels(self, qkv_or_qkvz, v_dim):
        # the stock warm-up builds a dummy state in the state dtype; the chunk kernels are warmed with fp32 states
        conv_dtype = type(self).get_state_dtype(self)[0]
        self.get_state_dtype = lambda: (conv_dtype, torch.float32)
        try:
            return stock_warmup(self, qkv_or_qkvz, v_dim)
        finally:
            del self.get_state_dtype

    base.__init__ = base_init
    cls.__init__ = __init__
    cls._warmup_prefill_kernels = _warmup_prefill_kernels
    cls._forward_core = _forward_core
    cls._statequant_patched = True
    _state['Q'] = Q


def unpatch():
    """Undo ``_patch_calculators`` / ``_patch_layer`` (tests)."""
    if 'calculators' in _state:
        mu, shape0, dtype0 = _state.pop('calculators')
        mu.MambaStateShapeCalculator.gated_delta_net_state_shape = shape0
        mu.MambaStateDtypeCalculator.gated_delta_net_state_dtype = dtype0
    if 'saved' in _state:
        base, base_init, cls, init, warmup, core = _state.pop('saved')
        base.__init__, cls.__init__, cls._warmup_prefill_kernels = base_init, init, warmup
        if core is None:
            del cls._forward_core
        else:
            cls._forward_core = core
        cls._statequant_patched = False
    for k in ('Q', 'registered', 'logged'):
        _state.pop(k, None)


def _forward_core(self, mixed_qkv, b, a, core_attn_out):
    """``QwenGatedDeltaNetAttention._forward_core`` on the packed slot state (non-speculative path).

    mixed_qkv [tokens, 2 hk d_k + hv d_v] (before the conv), b / a [tokens, hv] (the gate's raw inputs),
    core_attn_out [tokens, hv, d_v] written in place.  Decode rows: one ``step`` launch on their slots with the gate
    formed in the kernel.  Prefill rows: ``read`` -> the engine's gating + chunk kernel -> ``write``."""
    from . import _engine as E
    Q = _state['Q']
    md = E.layer_metadata(Q, self)
    if md is None:                                           # the engine's profiling run
        self._warmup_prefill_kernels(mixed_qkv, 0)
        return
    assert md.spec_sequence_masks is None, 'statequant vLLM plugin: speculative decoding is not supported'
    lay, views = self._sq_layout, E.slot_views(self)
    tokens = md.num_actual_tokens
    n_dec, n_pre = md.num_decodes, md.num_prefills
    if n_dec == 0 and n_pre == 0:
        return
    mixed_qkv, b, a = mixed_qkv[:tokens], b[:tokens], a[:tokens]
    slots = md.non_spec_state_indices_tensor
    taps, cstate = E.conv_taps(self.conv1d), E.conv_state(Q, self)

    # the causal conv is the engine's own: the varlen form when any row prefills, else the single-token update
    if n_pre > 0:
        x = Q.causal_conv1d_fn(mixed_qkv.transpose(0, 1), taps, self.conv1d.bias, activation=self.activation,
                               conv_states=cstate, has_initial_state=md.has_initial_state, cache_indices=slots,
                               query_start_loc=md.non_spec_query_start_loc, metadata=md).transpose(0, 1)
    else:
        x = Q.causal_conv1d_update(mixed_qkv, cstate, taps, self.conv1d.bias, self.activation,
                                   conv_state_indices=slots[:tokens], validate_data=False)

    if n_dec > 0:
        rows = E.decode_row_count(tokens, n_dec, n_pre)
        xd, idx = E.unit_stride_rows(x, rows), E.slot_index(slots, rows)
        kw = lay.HK * lay.DK                                 # q | k | v are column ranges of the conv output
        q = xd[:, :kw].unflatten(1, (lay.HK, lay.DK))
        k = xd[:, kw:2 * kw].unflatten(1, (lay.HK, lay.DK))
        v = xd[:, 2 * kw:].unflatten(1, (lay.HV, lay.DV))
        lay.step(views, idx, q, k, v, core_attn_out[:rows], self.head_k_dim ** -0.5,
                 gate=(a[:rows], b[:rows], self.A_log, self.dt_bias), **E.order_kw(Q, lay, views, slots, idx),
                 **self._sq_lk)
        if self._sq_external is not None:
            _external_after_decode(self, views, idx)

    if n_pre > 0:
        q, k, v, g, beta = Q.fused_post_conv_prep(
            conv_output=x[n_dec:], a=a[n_dec:], b=b[n_dec:], A_log=self.A_log, dt_bias=self.dt_bias,
            num_k_heads=lay.HK, head_k_dim=self.head_k_dim, head_v_dim=self.head_v_dim, apply_l2norm=True,
            output_g_exp=False)
        pslots = md.prefill_state_indices
        init = E.prefill_initial_state(lay, views, pslots, md.prefill_has_initial_state, **self._sq_lk)
        o, last = self.chunk_gated_delta_rule(
            q=q.unsqueeze(0), k=k.unsqueeze(0), v=v.unsqueeze(0), g=g.unsqueeze(0), beta=beta.unsqueeze(0),
            initial_state=init, output_final_state=True, cu_seqlens=md.prefill_query_start_loc,
            chunk_indices=md.chunk_indices, chunk_offsets=md.chunk_offsets, use_qk_l2norm_in_kernel=False,
            aiter_prefill_metadata=md.aiter_prefill_metadata)
        if self._sq_external is not None:                    # the end of a prefill chunk is a rounding point
            last = apply_external(last, self._sq_external[0])
        lay.write(views, pslots, last, **self._sq_lk)
        o = o.squeeze(0)
        core_attn_out[n_dec:n_dec + o.shape[0]] = o


def _external_after_decode(layer, views, idx):
    """Rows whose buffer has just been folded (their fill count is back at 0) get S <- fn(S) in the slot, cast to the
    slot's dtype.  Eagerly the function sees exactly those rows; under capture (fixed shapes) it sees every decode
    row and its result is kept where the row folded."""
    ordinal, captured = layer._sq_external
    S, where = views['S'], idx.long()
    folded = (views['NPTR'][where, 0] == 0) & (idx > 0)
    if captured:
        rows = S[where]
        S[where] = torch.where(folded[:, None, None, None], apply_external(rows, ordinal).to(S.dtype), rows)
    else:
        hit = where[folded]
        if hit.numel():
            S[hit] = apply_external(S[hit], ordinal).to(S.dtype)


def register():
    """The ``vllm.general_plugins`` entry point: a no-op unless STATEQUANT_VLLM is set, idempotent.  Patches the state
    calculators and the layer classes of the selected layer kinds (needs the engine importable)."""
    if _state.get('registered'):
        return
    cfg = configure()
    if cfg is None:
        return
    kinds = active_kinds()
    if 'gdn' in kinds:
        _patch_calculators()
        _patch_layer()
        if cfg[0] not in ('fp32', 'gga') and 'external' not in _state:
            from . import vllm_olmo
            vllm_olmo.patch(layout)
    if 'mamba2' in kinds:
        from . import vllm_mamba2
        vllm_mamba2.patch(cfg)
    if 'kda' in kinds:
        from . import vllm_kda
        vllm_kda.patch(cfg)
    _state['registered'] = True
