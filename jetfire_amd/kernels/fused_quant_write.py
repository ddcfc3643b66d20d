"""Quantise + pack + scatter writers (jetfire_vllm/kernels/fused_quant_write.py:242-781)."""
from ..ops import (fused_quant_write_int2_asym, fused_quant_write_int2_sym, fused_quant_write_int3_sym,
                   fused_quant_write_int4_sym, fused_quant_write_int4_sym_kv)

__all__ = ['fused_quant_write_int2_asym', 'fused_quant_write_int2_sym', 'fused_quant_write_int3_sym', 'fused_quant_write_int4_sym',
           'fused_quant_write_int4_sym_kv']
