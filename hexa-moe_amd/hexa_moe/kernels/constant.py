"""Constants of the list format (reference: hexa_moe_triton/hexa_moe/kernels/basics.py:9-11)."""
MAX_TOKEN_CHUNK = 16
