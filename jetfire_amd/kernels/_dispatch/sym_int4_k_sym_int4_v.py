"""KernelSet for SymInt4K_SymInt4V (jetfire_vllm/kernels/_dispatch/sym_int4_k_sym_int4_v.py:24-91)."""
from __future__ import annotations

from ... import _lib
from ...ops import SUPPORTED_TOP_K, fused_quant_write_int4_sym, fused_quant_write_int4_sym_kv


class _SymInt4KSymInt4VKernels:
    nbits_k = 4
    nbits_v = 4
    asymmetric_k = False
    asymmetric_v = False
    head_dim = 128
    group_size = 128
    supported_top_k = tuple(k for k in SUPPORTED_TOP_K if k >= 64)

    def load(self) -> None:
        _lib.load()

    def attn_with_scores(self, *args, **kwargs):
        raise NotImplementedError("SymInt4K_SymInt4V runs through the split / fused decode kernels")

    def fused_pre_correction_batched(self, *args, **kwargs):
        raise NotImplementedError("SymInt4K_SymInt4V has no GPU-only pre-correction: the CPU correction path is used")

    def fused_post_correction(self, *args, **kwargs):
        raise NotImplementedError("SymInt4K_SymInt4V has no GPU-only post-correction: the CPU correction path is used")

    def quant_write_k(self, key_tok, slot_idx, k_data, k_scales, k_zp, group_size):
        if k_zp is not None:
            raise ValueError("SymInt4K does not use a k_zp tensor.")
        fused_quant_write_int4_sym(key_tok, slot_idx, k_data, k_scales, int(group_size))

    def quant_write_v(self, value_tok, slot_idx, v_data, v_scales, v_zp, group_size):
        if v_zp is not None:
            raise ValueError("SymInt4V does not use a v_zp tensor.")
        fused_quant_write_int4_sym(value_tok, slot_idx, v_data, v_scales, int(group_size))

    def quant_write_kv(self, key_tok, value_tok, slot_idx, k_data, k_scales, v_data, v_scales, group_size):
        fused_quant_write_int4_sym_kv(key_tok, value_tok, slot_idx, k_data, k_scales, v_data, v_scales, int(group_size))


KERNELS = _SymInt4KSymInt4VKernels()
