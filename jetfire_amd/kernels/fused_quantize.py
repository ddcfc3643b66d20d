"""One-launch INT2 quantise + pack without the scatter (jetfire_vllm/kernels/fused_quantize.py:214-284)."""
from ..ops import quantize_and_pack, quantize_and_pack_asym


def fused_quantize_and_pack_int2(x, group_size: int):
    """fused_quantize.py:214-247"""
    return quantize_and_pack(x, group_size=group_size, nbits=2)


def fused_quantize_and_pack_int2_asym(x, group_size: int):
    """fused_quantize.py:250-284"""
    return quantize_and_pack_asym(x, group_size=group_size, nbits=2)


__all__ = ['fused_quantize_and_pack_int2', 'fused_quantize_and_pack_int2_asym']
