"""Kernel set of a symmetric K/V pair whose two sides are chosen independently by bit width, as the
reference's mixed-precision sets do (jetfire_vllm/kernels/_dispatch/sym_int4_k_sym_int2_v.py:15-61 and its
siblings): split-mode Stage A / Stage B plus the CPU correction, no GPU-only correction kernels."""
from __future__ import annotations

from ... import _lib, ops
from ...ops import SUPPORTED_TOP_K

_WRITERS = {2: ops.fused_quant_write_int2_sym, 3: ops.fused_quant_write_int3_sym, 4: ops.fused_quant_write_int4_sym}


class SymKernelSet:
    asymmetric_k = False
    asymmetric_v = False
    head_dim = 128
    group_size = 128
    supported_top_k = SUPPORTED_TOP_K

    def __init__(self, nbits_k: int, nbits_v: int) -> None:
        self.nbits_k, self.nbits_v = int(nbits_k), int(nbits_v)
        self.name = f"SymInt{self.nbits_k}K_SymInt{self.nbits_v}V"

    def load(self) -> None:
        _lib.load()

    def _split_only(self, what: str):
        raise NotImplementedError(f"{self.name} has no {what}: it runs through the split decode kernels and the "
                                  "CPU correction")

    def attn_with_scores(self, *args, **kwargs):
        self._split_only("fused WMMA decode kernel")

    def fused_pre_correction_batched(self, *args, **kwargs):
        self._split_only("GPU pre-correction kernel")

    def fused_post_correction(self, *args, **kwargs):
        self._split_only("GPU post-correction kernel")

    def quant_write_k(self, key_tok, slot_idx, k_data, k_scales, k_zp, group_size):
        if k_zp is not None:
            raise ValueError(f"SymInt{self.nbits_k}K does not use a k_zp tensor.")
        _WRITERS[self.nbits_k](key_tok, slot_idx, k_data, k_scales, int(group_size))

    def quant_write_v(self, value_tok, slot_idx, v_data, v_scales, v_zp, group_size):
        if v_zp is not None:
            raise ValueError(f"SymInt{self.nbits_v}V does not use a v_zp tensor.")
        _WRITERS[self.nbits_v](value_tok, slot_idx, v_data, v_scales, int(group_size))
