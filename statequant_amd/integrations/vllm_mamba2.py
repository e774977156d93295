"""Mamba2 / SSD layers under STATEQUANT_VLLM: format fitting, slot layouts, the allocator's state shape
(/root/reference/src/statequant/integrations/vllm_mamba2.py:42-92)."""
from __future__ import annotations

import dataclasses

import torch

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
