"""INT2 V Stage B loader (jetfire_vllm/kernels/int2_split.py:59-60; module jetfire_int2_softmax_v)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_softmax_v_ext():
    _lib.load()
    return SimpleNamespace(
        int2_softmax_v_with_pre_corr_wvs2=ops.int2_softmax_v_with_pre_corr_wvs2,
        int2_softmax_v_with_pre_corr_wvs2_inplace=ops.int2_softmax_v_with_pre_corr_wvs2_inplace,
        int2_softmax_v_with_pre_corr=ops.int2_softmax_v_with_pre_corr,
        int2_softmax_v=ops.int2_softmax_v)
