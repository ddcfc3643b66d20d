"""KernelSet for SymInt3K_SymInt2V (jetfire_vllm/kernels/_dispatch/sym_int3_k_sym_int2_v.py)."""
from ._sym import SymKernelSet

KERNELS = SymKernelSet(3, 2)
