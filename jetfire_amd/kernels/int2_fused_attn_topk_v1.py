"""The reference's second fused INT2 kernel (jetfire_vllm/csrc/int2_fused_attn_topk_v1.cu:581-595: same
contract, tensor-core form, 1 / 2 / 4 query heads per kv-head, top_k a multiple of 32 up to 128).  Both names
run the same one-pass scan here, which takes 1..16 query heads per kv-head and top_k 32..8192 (powers of two)."""
from types import SimpleNamespace

from .. import _lib
from .int2_fused_attn_topk import int2_fused_attn_topk as int2_fused_attn_topk_v1


def load_int2_fused_attn_topk_v1_ext():
    _lib.load()
    return SimpleNamespace(int2_fused_attn_topk_v1=int2_fused_attn_topk_v1)
