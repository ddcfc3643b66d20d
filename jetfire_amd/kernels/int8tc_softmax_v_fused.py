"""INT4 V Stage B with Stage-A statistics (jetfire_vllm/kernels/int8tc_softmax_v_fused.py:45-46)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_ext():
    _lib.load()
    return SimpleNamespace(
        int8tc_softmax_v_with_pre_corr_reg_stats=ops.int8tc_softmax_v_with_pre_corr_reg_stats)
