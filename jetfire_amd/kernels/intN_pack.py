"""Quantise / pack / unpack of whole tensors (jetfire_vllm/kernels/intN_pack.py:35-311), on the GPU."""
from ..ops import packed_dim, quantize_and_pack, quantize_and_pack_asym, unpack

__all__ = ['packed_dim', 'quantize_and_pack', 'quantize_and_pack_asym', 'unpack']
