"""KernelSet for AsymInt2K4Level_SymInt3V (jetfire_vllm/kernels/_dispatch/int2_asym_k_sym_int3_v.py)."""
from ._sym import AsymInt2KernelSet

KERNELS = AsymInt2KernelSet(3)
