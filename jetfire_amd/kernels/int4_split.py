"""INT4 V Stage B loader (jetfire_vllm/kernels/int4_split.py:60-61; module jetfire_int4_softmax_v)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_softmax_v_ext():
    _lib.load()
    return SimpleNamespace(
        int4_softmax_v_with_pre_corr_wvs2_scores=ops.int4_softmax_v_with_pre_corr_wvs2_scores,
        int4_softmax_v_with_pre_corr_wvs2=ops.int4_softmax_v_with_pre_corr_wvs2)
