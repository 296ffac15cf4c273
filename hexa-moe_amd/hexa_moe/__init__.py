"""hexa_moe for MI355X: the MoE_Cascaded / MoE_Buffer API of HEXA-MoE on hand-written gfx950 kernels.

    from hexa_moe import moe as hmoe
    layer = hmoe.MoE_Cascaded(gate_type={...}, model_dim_list=[...], ...)
"""
__version__ = "0.1.0"
