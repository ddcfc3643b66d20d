"""INT3 K Stage A loader (jetfire_vllm/kernels/int3_split.py:29-68; module jetfire_int3_qk_scores)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_qk_scores_ext():
    _lib.load()
    return SimpleNamespace(int3_qk_scores=ops.int3_qk_scores, int3_qk_scores_topk=ops.int3_qk_scores_topk)
