"""CPU correction loader (jetfire_vllm/kernels/cpu_topk_attn.py:38-39; module jetfire_cpu_topk_attn): the functions
the reference's extension module exports (jetfire_vllm/csrc/cpu_topk_attn.cpp:2509-2663), under its names."""
from types import SimpleNamespace

from .. import _lib, ops

_NAMES = (
    "cpu_topk_attn", "alloc_mapped_pinned_pair", "submit_cpu_topk_attn_async", "wait_for_flag", "persistent_worker_warmup",
    "set_cpu_attn_threads", "get_cpu_attn_threads", "stream_write_value64", "stream_wait_value64",
    "create_cpu_topk_submit_ctx", "stream_submit_cpu_topk_attn", "stream_wait_cpu_topk_attn", "graph_pool_warmup",
    "graph_pool_warmup_threads", "get_graph_submit_count", "get_cpu_topk_sanitize_count", "reset_graph_runtime_state",
    "clear_graph_contexts", "get_shadow_append_count", "reset_graph_submit_count", "get_graph_timing_stats",
)


def load_cpu_topk_attn_ext():
    _lib.load()
    ext = SimpleNamespace(**{n: getattr(ops, n) for n in _NAMES})
    # this library's own additions: the hand-off that also moves q / slots / o_new itself, status and ISA control
    ext.CpuTopkHandoff = ops.CpuTopkHandoff
    ext.check_cpu_topk_submit_ctx = ops.check_cpu_topk_submit_ctx
    ext.set_cpu_attn_isa = ops.set_cpu_attn_isa
    ext.get_cpu_attn_isa = ops.get_cpu_attn_isa
    ext.pool_wake = ops.pool_wake
    ext.pool_doorbell = ops.pool_doorbell
    return ext
