"""CPU correction loader (jetfire_vllm/kernels/cpu_topk_attn.py:38-39; module jetfire_cpu_topk_attn)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_cpu_topk_attn_ext():
    _lib.load()
    return SimpleNamespace(cpu_topk_attn=ops.cpu_topk_attn, set_cpu_attn_threads=ops.set_cpu_attn_threads,
                           get_cpu_attn_threads=ops.get_cpu_attn_threads, CpuTopkHandoff=ops.CpuTopkHandoff)
