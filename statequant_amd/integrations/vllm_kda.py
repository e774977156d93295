"""KDA layers under STATEQUANT_VLLM: slot layouts and the allocator's state shape
(/root/reference/src/statequant/integrations/vllm_kda.py:43-80)."""
from __future__ import annotations

import torch

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
