"""The serving-engine plugin of the packed state: how the engine's environment selects a storage format, which slot
layout a layer's head geometry maps to, what state shape / dtype the engine's cache allocator is told (one flat byte
blob per slot and layer), and the layer forwards that run decode rows on the HIP slot ops and prefill rows through
``read`` -> the engine's chunk kernel -> ``write``.

Mirrors the reference's vLLM plugin (/root/reference/src/statequant/integrations/vllm_plugin.py, vllm_olmo.py,
vllm_mamba2.py, vllm_kda.py): same environment variables, format names, asserted restrictions, slot sizes and call
sites.  No module here imports the engine when it is imported; ``vllm_plugin.register()`` (the
``vllm.general_plugins`` entry point) and the patch functions do, or are handed the engine's modules.
"""
from . import vllm_kda, vllm_mamba2, vllm_olmo, vllm_plugin  # noqa: F401
