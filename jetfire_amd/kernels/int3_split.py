"""INT3 split loaders: K Stage A (jetfire_vllm/kernels/int3_split.py:29-48; module jetfire_int3_qk_scores) and
V Stage B (:50-68; module jetfire_int3_softmax_v)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_qk_scores_ext():
    _lib.load()
    return SimpleNamespace(int3_qk_scores=ops.int3_qk_scores, int3_qk_scores_topk=ops.int3_qk_scores_topk)


def load_softmax_v_ext():
    _lib.load()
    return SimpleNamespace(
        int3_softmax_v_with_pre_corr_wvs2=ops.int3_softmax_v_with_pre_corr_wvs2,
        int3_softmax_v_with_pre_corr_wvs2_inplace=ops.int3_softmax_v_with_pre_corr_wvs2_inplace,
        int3_softmax_v_with_pre_corr=ops.int3_softmax_v_with_pre_corr,
        int3_softmax_v=ops.int3_softmax_v)
