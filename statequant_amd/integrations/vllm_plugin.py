"""STATEQUANT_VLLM=<format> -> storage configuration -> per-layer slot layouts and the cache allocator's state shape.

What the reference's plugin does before it touches vLLM (/root/reference/src/statequant/integrations/vllm_plugin.py):
``config`` (:76-120) reads the environment, ``layout`` (:123-141) keeps one slot layout per head geometry, and the
patched state calculators (:252-279) answer "(nbytes,) of uint8" for the recurrent state.  The names, the environment
variables and the error texts' substance follow it, so that a deployment's settings carry over unchanged.

    STATEQUANT_VLLM              off | pace4 | int4k | int4v | int8k | int8v | bf16 | fp32 | int<4|8><k|v>g<group>
                                 | gga:<plan.pt>[:pw]
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
        assert hit, (f'{ENV}={mode!r}: use pace4, int4k, int4v, int8k, int8v, bf16, fp32, gga:<plan.pt>[:pw] or '
                     f'int<4|8><k|v>g<group>')
        triple = (int(hit['bits']), hit['axis'], int(hit['group']))
    return Quantizer(*triple)


def config(environ=None):
    """(fmt, m, buffer_bits, fused) from the environment (``environ``: a mapping to read instead of ``os.environ``),
    or None when the plugin is off.  fmt: Quantizer | 'bf16' | 'fp32' | 'gga' (then ``gga_settings()`` holds the plan
    file, the window flag and its length)."""
    raw = _env(environ, ENV).strip()
    mode = raw.lower()
    if mode in OFF:
        return None
    _state.pop('gga', None)
    if mode.startswith('gga:'):
        spec = raw[len('gga:'):]
        windowed = spec.endswith(':pw')
        path = spec[:-len(':pw')] if windowed else spec
        assert os.path.exists(path), f'{ENV}=gga:<plan.pt>[:pw]: no plan file {path!r}'
        _state['gga'] = (path, windowed, int(_env(environ, 'STATEQUANT_VLLM_PW_M', '8')))
        fmt = 'gga'
    else:
        assert not mode.startswith('external:'), \
            f'{ENV}={raw!r}: external quantizers (a Python callable per fold) have no HIP path in this build'
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
        if cfg[0] in ('fp32', 'gga'):
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
