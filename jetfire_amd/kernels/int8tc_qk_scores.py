"""INT4 K int8-Q Stage A loader (jetfire_vllm/kernels/int8tc_qk_scores.py:39-40)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_int8tc_qk_scores_ext():
    _lib.load()
    return SimpleNamespace(int8tc_qk_scores=ops.int8tc_qk_scores, int8tc_qk_scores_topk=ops.int8tc_qk_scores_topk,
                           int8tc_qk_scores_topk_stats=ops.int8tc_qk_scores_topk_stats)
