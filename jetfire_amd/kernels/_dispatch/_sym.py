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

    def __init__(self, nbits_k: int, nbits_v: int, *, min_top_k: int = 32) -> None:
        self.nbits_k, self.nbits_v = int(nbits_k), int(nbits_v)
        self.name = f"SymInt{self.nbits_k}K_SymInt{self.nbits_v}V"
        self.supported_top_k = tuple(k for k in SUPPORTED_TOP_K if k >= min_top_k)

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

    def quant_write_kv(self, key_tok, value_tok, slot_idx, k_data, k_scales, v_data, v_scales, group_size):
        """K and V in one launch where a single kernel takes both (INT4 / INT4), else two launches."""
        if (self.nbits_k, self.nbits_v) == (4, 4):
            ops.fused_quant_write_int4_sym_kv(key_tok, value_tok, slot_idx, k_data, k_scales, v_data, v_scales,
                                              int(group_size))
        else:
            self.quant_write_k(key_tok, slot_idx, k_data, k_scales, None, group_size)
            self.quant_write_v(value_tok, slot_idx, v_data, v_scales, None, group_size)


class AsymInt2KernelSet(SymKernelSet):
    """INT2 keys over the full four-level codebook with a zero-point per group, symmetric values
    (jetfire_vllm/kernels/_dispatch/int2_asym_k_sym_v.py and its INT3 / INT4 value siblings)."""
    asymmetric_k = True

    def __init__(self, nbits_v: int) -> None:
        super().__init__(2, nbits_v)
        self.name = f"AsymInt2K4Level_SymInt{self.nbits_v}V"

    def quant_write_k(self, key_tok, slot_idx, k_data, k_scales, k_zp, group_size):
        if k_zp is None:
            raise ValueError("AsymInt2K needs a k_zp tensor.")
        ops.fused_quant_write_int2_asym(key_tok, slot_idx, k_data, k_scales, k_zp, int(group_size))

    def quant_write_kv(self, *args, **kwargs):
        raise NotImplementedError(f"{self.name} writes keys (with zero-points) and values separately")
