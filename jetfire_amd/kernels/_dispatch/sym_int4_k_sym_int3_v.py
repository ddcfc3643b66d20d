"""KernelSet for SymInt4K_SymInt3V (jetfire_vllm/kernels/_dispatch/sym_int4_k_sym_int3_v.py)."""
from ._sym import SymKernelSet

KERNELS = SymKernelSet(4, 3)
