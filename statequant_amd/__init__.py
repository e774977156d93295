"""statequant_amd: the packed recurrent-state decode step of statequant (Gated DeltaNet, KDA, Mamba2 / SSD) as
hand-written HIP kernels for MI355X (gfx950), behind the reference's Python op signatures and slot-blob layout.

    import statequant_amd as sq
    lay = sq.kernels.SlotLayout(sq.Quantizer(4, 'k', 64), hv=32, hk=16, dk=128, dv=128, m=8, buffer_bits=8)
    views = lay.views(blob)                      # blob: uint8 [num_slots, >= lay.nbytes], e.g. vLLM's state cache
    lay.step(views, idx, q, k, v, out, scale, g=g, beta=beta)
"""
from . import kernels
from .quantizer import FloatCast, Format, Identity, Quantizer

__version__ = '0.1.0'
__all__ = ['kernels', 'Quantizer', 'FloatCast', 'Identity', 'Format']
