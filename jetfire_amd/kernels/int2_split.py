"""INT2 split loaders: K Stage A for symmetric keys (jetfire_vllm/kernels/int2_split.py:28-47; module
jetfire_int2_qk_scores) and V Stage B (:49-60; module jetfire_int2_softmax_v)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_qk_scores_ext():
    _lib.load()
    return SimpleNamespace(int2_qk_scores=ops.int2_qk_scores, int2_qk_scores_topk=ops.int2_qk_scores_topk)


def load_softmax_v_ext():
    _lib.load()
    return SimpleNamespace(
        int2_softmax_v_with_pre_corr_wvs2=ops.int2_softmax_v_with_pre_corr_wvs2,
        int2_softmax_v_with_pre_corr_wvs2_inplace=ops.int2_softmax_v_with_pre_corr_wvs2_inplace,
        int2_softmax_v_with_pre_corr=ops.int2_softmax_v_with_pre_corr,
        int2_softmax_v=ops.int2_softmax_v)
