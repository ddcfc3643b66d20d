"""Single-call INT2 attention + top-k with the reference's name and argument order
(jetfire_vllm/kernels/int2_fused_attn_topk.py:5-10, csrc/int2_fused_attn_topk.cu:403-417): asymmetric INT2
keys with zero-points, INT2 values, -> [o_hat, topk_slots, o_old_unnorm, W].  Runs the one-pass scan
(scheme "a2v2"); the scale tensors carry one (group 128) or two (group 64) groups per row."""
from types import SimpleNamespace

from .. import _lib, ops


def int2_fused_attn_topk(q, k_data, k_scales, k_zp, v_data, v_scales, block_table, seq_lens, max_S, H_q, H_kv,
                         block_size, top_k, attn_scale):
    out = ops.fused_attn_topk("a2v2", q, k_data, k_scales, v_data, v_scales, block_table, seq_lens, max_S, H_q,
                              H_kv, block_size, top_k, attn_scale, k_zp=k_zp)
    return list(out[:4])


def load_int2_fused_attn_topk_ext():
    _lib.load()
    return SimpleNamespace(int2_fused_attn_topk=int2_fused_attn_topk)
