"""Fused decode scan + top-k loader; the single-call contract of the reference's int2_fused_attn_topk
(jetfire_vllm/kernels/int2_fused_attn_topk.py:5-10) for the K3V2 and K4V4 schemes."""
from types import SimpleNamespace

from .. import _lib, ops


def load_fused_attn_topk_ext():
    _lib.load()
    return SimpleNamespace(fused_attn_topk=ops.fused_attn_topk)
