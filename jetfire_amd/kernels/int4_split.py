"""INT4 split loaders: K Stage A with the bf16 model (jetfire_vllm/kernels/int4_split.py:29-48; module
jetfire_int4_qk_scores) and V Stage B (:50-61; module jetfire_int4_softmax_v)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_qk_scores_ext():
    _lib.load()
    return SimpleNamespace(int4_qk_scores=ops.int4_qk_scores, int4_qk_scores_topk=ops.int4_qk_scores_topk,
                           int4_qk_scores_topk_stats=ops.int4_qk_scores_topk_stats)


def load_softmax_v_ext():
    _lib.load()
    return SimpleNamespace(
        int4_softmax_v_with_pre_corr_wvs2_scores=ops.int4_softmax_v_with_pre_corr_wvs2_scores,
        int4_softmax_v_with_pre_corr_wvs2=ops.int4_softmax_v_with_pre_corr_wvs2,
        int4_softmax_v_with_pre_corr_wvs2_inplace=ops.int4_softmax_v_with_pre_corr_wvs2_inplace)
