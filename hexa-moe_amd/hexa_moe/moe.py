"""Public interface, same import path as the reference (hexa_moe_cuda/hexa_moe/moe.py:1-2)."""
from .impls.cascaded_moe import MoE_Buffer, MoE_Cascaded

__all__ = ["MoE_Cascaded", "MoE_Buffer"]
