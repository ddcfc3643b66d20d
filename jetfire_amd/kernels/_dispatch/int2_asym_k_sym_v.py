"""KernelSet for AsymInt2K4Level_SymInt2V (jetfire_vllm/kernels/_dispatch/int2_asym_k_sym_v.py)."""
from ._sym import AsymInt2KernelSet

KERNELS = AsymInt2KernelSet(2)
