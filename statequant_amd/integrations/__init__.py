"""The engine-facing glue of the packed state that needs no engine to run: how a serving engine's environment selects
a storage format, which slot layout a layer's head geometry maps to, and what state shape / dtype the engine's cache
allocator is told (one flat byte blob per slot and layer).

Mirrors the reference's vLLM plugin for these parts (/root/reference/src/statequant/integrations/vllm_plugin.py,
vllm_mamba2.py, vllm_kda.py): same environment variables, same format names, same asserted restrictions, same slot
sizes.  The monkey-patches of vLLM's layer classes themselves are not part of this package.
"""
from . import vllm_kda, vllm_mamba2, vllm_plugin  # noqa: F401
