"""KernelSet for SymInt3K_SymInt2V (jetfire_vllm/kernels/_dispatch/sym_int3_k_sym_int2_v.py:15-61)."""
from __future__ import annotations

from ... import _lib
from ...ops import SUPPORTED_TOP_K, fused_quant_write_int2_sym, fused_quant_write_int3_sym


class _SymInt3KSymInt2VKernels:
    nbits_k = 3
    nbits_v = 2
    asymmetric_k = False
    asymmetric_v = False
    head_dim = 128
    group_size = 128
    supported_top_k = SUPPORTED_TOP_K

    def load(self) -> None:
        _lib.load()

    def attn_with_scores(self, *args, **kwargs):
        raise NotImplementedError("SymInt3K_SymInt2V runs through the split / fused decode kernels")

    def fused_pre_correction_batched(self, *args, **kwargs):
        raise NotImplementedError("SymInt3K_SymInt2V has no GPU-only pre-correction: the CPU correction path is used")

    def fused_post_correction(self, *args, **kwargs):
        raise NotImplementedError("SymInt3K_SymInt2V has no GPU-only post-correction: the CPU correction path is used")

    def quant_write_k(self, key_tok, slot_idx, k_data, k_scales, k_zp, group_size):
        if k_zp is not None:
            raise ValueError("SymInt3K does not use a k_zp tensor.")
        fused_quant_write_int3_sym(key_tok, slot_idx, k_data, k_scales, int(group_size))

    def quant_write_v(self, value_tok, slot_idx, v_data, v_scales, v_zp, group_size):
        if v_zp is not None:
            raise ValueError("SymInt2V does not use a v_zp tensor.")
        fused_quant_write_int2_sym(value_tok, slot_idx, v_data, v_scales, int(group_size))


KERNELS = _SymInt3KSymInt2VKernels()
