"""Packed (real-storage) decode path on HIP kernels: int4 / int8 recurrent state with a delta-value decode buffer.

    from statequant_amd.kernels import PackedGDNState, SlotLayout, pack, unpack

Same names as the reference's ``statequant.kernels`` (``/root/reference/src/statequant/kernels/__init__.py:10-18``).
``pack`` / ``unpack`` are torch; ``PackedGDNState`` (sequences in lockstep), ``SlotLayout.step`` (slot-addressed
sequences: the serving layout), ``PackedMamba2State`` / ``Mamba2SlotLayout`` and ``PackedKDAState`` /
``KDASlotLayout`` call the HIP kernels in ``libsqhip.so`` and need an MI355X.  ``GGAPacked`` is the mixed-width
GGA / STEP slot with the FP8 write window (the reference keeps it in ``integrations/vllm_gga.py``).
"""
from .fold import PackedGDNState, check_dims, pack, pack_vk, packed_format, unpack, unpack_vk
from .kda import KDASlotLayout, PackedKDAState, kda_recurrence
from .mamba2 import Mamba2SlotLayout, PackedMamba2State, mamba2_recurrence
from .gga import GGAPacked, GGAPlan
from .slots import SlotLayout

__all__ = ['PackedGDNState', 'SlotLayout', 'pack', 'unpack', 'pack_vk', 'unpack_vk', 'packed_format', 'check_dims',
           'PackedMamba2State', 'Mamba2SlotLayout', 'mamba2_recurrence',
           'PackedKDAState', 'KDASlotLayout', 'kda_recurrence', 'GGAPacked', 'GGAPlan']
