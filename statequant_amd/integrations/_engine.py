"""What the four patched layer forwards have in common.

A forward replaces one method of an engine layer class (vLLM's ``QwenGatedDeltaNetAttention._forward_core`` and its
siblings).  It never imports the engine: everything it needs from it -- the forward context, the causal-conv ops, the
prefill chunk kernels -- it takes from ``ns``, the engine module the layer class lives in (the patch functions store
that module; tests store a namespace of stand-ins with the same call signatures).  The layer object, the attention
metadata object and ``kv_cache`` are used through their attributes only.

Row conventions of the engine (``vllm_plugin.py:367-392`` of the reference): a step's tokens are the decode rows first
(one token each), then the prefill rows; ``non_spec_state_indices_tensor`` names the slot of every sequence in that
order.  A decode-only step may be padded to a captured batch size: the padding rows carry slot 0 (the null block) or
-1, which the step kernels skip.
"""
from __future__ import annotations

import torch


def layer_metadata(ns, layer):
    """The attention metadata of ``layer`` in the current forward context, or None on the engine's profiling and
    warm-up runs (no metadata at all, or none under this layer's prefix)."""
    md = ns.get_forward_context().attn_metadata
    if not isinstance(md, dict):
        return None
    return md.get(layer.prefix)


def slot_views(layer):
    """Typed views of the layer's state blob (``kv_cache[1]``), rebuilt only when the engine rebinds the cache."""
    blob = layer.kv_cache[1]
    tag = (blob.data_ptr(), tuple(blob.shape), tuple(blob.stride()))
    cached = layer._sq_views
    if cached is None or cached[0] != tag:
        cached = layer._sq_views = (tag, layer._sq_layout.views(blob))
    return cached[1]


def conv_state(ns, layer):
    """The conv state with the channel dim first, whichever way the engine stores it."""
    cs = layer.kv_cache[0]
    return cs if ns.is_conv_state_dim_first() else cs.transpose(-1, -2)


def conv_taps(conv):
    """[channels, 1, width] conv weight as the [channels, width] matrix the conv ops take."""
    w = conv.weight
    return w.view(w.size(0), w.size(2))


def decode_row_count(tokens, num_decodes, num_prefills):
    """How many leading rows of a step go through the decode kernel: all of them on a decode-only step (the engine's
    padded batch; padding rows point at slot <= 0), the decode sequences otherwise."""
    return tokens if num_prefills == 0 else num_decodes


def slot_index(idx_all, rows):
    """The first ``rows`` slot indices as the contiguous int32 vector the step kernels read."""
    idx = idx_all[:rows]
    if idx.dtype != torch.int32 or not idx.is_contiguous():
        idx = idx.to(torch.int32).contiguous()
    return idx


def dispatch_order(ns, lay, views, slots, idx):
    """The dispatch order of this forward pass's decode rows for ``step(..., order=)``, or None for the batch order.

    Not in the reference.  A serving batch's sequences are at different points of their fold period; the rows that
    fold on this token keep their workgroups longer, and ``fold_order`` places them where they do not decide when the
    launch ends (a quarter to a sixth off the step time at 256 sequences).  The counters of all layers move together,
    so the first patched layer of a pass computes the list (one small launch) and leaves it on the pass's forward
    context, where the other layers find it.  Below 64 rows, or a row count that is no multiple of 8, ``fold_order``
    would return the batch order: no launch then."""
    rows = idx.shape[0]
    if rows < 64 or rows % 8 or not hasattr(lay, 'fold_order'):           # (the mixed-width slot has no counters)
        return None
    ctx = ns.get_forward_context()
    key = (slots.data_ptr(), rows, lay.m)
    cached = getattr(ctx, '_sq_dispatch_order', None)
    if cached is not None and cached[0] == key:
        return cached[1]
    order = lay.fold_order(views, idx)
    try:
        ctx._sq_dispatch_order = (key, order)
    except AttributeError:                                   # a context that takes no attributes: one list per layer
        pass
    return order


def order_kw(ns, lay, views, slots, idx):
    """``dispatch_order`` as keyword arguments of a ``step`` that may not know ``order`` (the mixed-width slot's)."""
    order = dispatch_order(ns, lay, views, slots, idx)
    return {} if order is None else {'order': order}


def unit_stride_rows(x, rows):
    """The first ``rows`` rows of a 2-d activation with a unit inner stride (any row stride is fine for the kernels)."""
    x = x[:rows]
    return x if x.stride(-1) == 1 else x.contiguous()


def prefill_initial_state(lay, views, slots, has_history, **layer_kw):
    """fp32 value-major initial states for the prefill rows: the slot's stored state advanced across its pending
    buffer where the sequence has history, zeros where it starts (the slot may hold a previous owner's bytes)."""
    init = lay.read(views, slots, **layer_kw)
    keep = has_history[:, None, None, None]
    return torch.where(keep, init, torch.zeros((), dtype=init.dtype, device=init.device)).contiguous()


def check_cache_settings(vllm_config, what):
    """The cache features the packed state does not implement, refused when the layer is built."""
    assert vllm_config.speculative_config is None, f'{what}: speculative decoding unsupported'
    cc = vllm_config.cache_config
    assert not cc.enable_prefix_caching, f'{what}: prefix caching is unsupported (pass enable_prefix_caching=False)'
    assert cc.mamba_cache_mode == 'none', cc.mamba_cache_mode
