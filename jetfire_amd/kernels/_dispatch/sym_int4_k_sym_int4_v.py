"""KernelSet for SymInt4K_SymInt4V (jetfire_vllm/kernels/_dispatch/sym_int4_k_sym_int4_v.py): the stats-producing
Stage A of this pair starts at a correction width of 64."""
from ._sym import SymKernelSet

KERNELS = SymKernelSet(4, 4, min_top_k=64)
