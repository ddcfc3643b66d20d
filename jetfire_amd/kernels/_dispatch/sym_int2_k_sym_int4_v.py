"""KernelSet for SymInt2K_SymInt4V (jetfire_vllm/kernels/_dispatch/sym_int2_k_sym_int4_v.py)."""
from ._sym import SymKernelSet

KERNELS = SymKernelSet(2, 4)
