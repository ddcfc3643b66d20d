"""KernelSet for SymInt3K_SymInt4V (jetfire_vllm/kernels/_dispatch/sym_int3_k_sym_int4_v.py)."""
from ._sym import SymKernelSet

KERNELS = SymKernelSet(3, 4)
