"""Decode entry of the adapter (`jetfire_vllm/adapter/decode_path.py:1156-1184,1667-1712,1712-3237`): one
layer's attention for a batch of single-token queries over the quantised cache,

    fused scan + top-k  ->  pinned hand-off + CPU correction over the bf16 shadow  ->  blend into `output`.

`try_jetfire_decode` returns `output` on success and None when a precondition fails (the caller then uses
its native attention); every miss is recorded with the reference's reason string.  The reference's trace
hooks, CUDA-graph capture mode, release policy and debug correction modes are not reproduced."""
from __future__ import annotations

import math
import os

import torch

from .. import ops
from .config import get_jetfire_config
from .kv_pool import get_global_kv_pool_manager

# correction widths the fused kernels take (the split entry points go up to 8192)
FUSED_SUPPORTED_TOP_K = (32, 64, 128, 256, 512, 1024)

_TOPK_CLAMP_LOGGED: set = set()
_HEAD_MAP_CACHE: dict = {}
_HANDOFFS: dict = {}
_O_NEW: dict = {}
_SEQ_LENS_CACHE: dict = {}


def _select_top_k(config_top_k: int, seq_len: int, supported: tuple) -> int | None:
    """Largest supported width <= the configured one that the context can fill; a context shorter than the
    smallest width still runs with that width (unused lanes are padded with -1).  None for an empty sequence
    or when no supported width is <= the configured one."""
    requested, length = int(config_top_k), int(seq_len)
    configured = [k for k in supported if 0 < k <= requested]
    if not configured or length <= 0:
        return None
    candidates = [k for k in configured if k <= length]
    selected = max(candidates) if candidates else min(configured)
    if selected != requested and (requested, selected) not in _TOPK_CLAMP_LOGGED:
        _TOPK_CLAMP_LOGGED.add((requested, selected))
        print(f"[jetfire] requested top_k={requested} clamped to kernel-supported top_k={selected}; "
              f"supported={tuple(supported)}.", flush=True)
    return selected


def _get_head_map_cpu(B: int, H_q: int, num_groups: int, K: int) -> torch.Tensor:
    """head_map[b, h, k] = h // num_groups: the kv-head every query head reads."""
    key = (B, H_q, num_groups, K)
    hm = _HEAD_MAP_CACHE.get(key)
    if hm is None:
        hm = (torch.arange(H_q, dtype=torch.int64) // num_groups).view(1, H_q, 1).expand(B, H_q, K).contiguous()
        _HEAD_MAP_CACHE[key] = hm
    return hm


def _decode_unsupported(*, impl, layer, query, attn_metadata) -> str | None:
    """Dispatcher gate: the reason string of a miss, or None."""
    pool = get_global_kv_pool_manager()
    if not pool.config.enabled:
        return "pool_disabled"
    if query.is_cuda and torch.cuda.is_current_stream_capturing():
        return "cuda_graph_capture"          # the hand-off blocks the host: not capturable
    if attn_metadata is None:
        return "profiling_run"
    attn_type = getattr(impl, "attn_type", None)
    if attn_type is not None and getattr(attn_type, "name", str(attn_type)) != "DECODER":
        return "attn_type"
    if getattr(attn_metadata, "use_cascade", False):
        return "cascade"
    if int(getattr(attn_metadata, "max_query_len", 1)) != 1:
        return "prefill_or_multi_query"
    n_seqs = int(attn_metadata.seq_lens.numel())
    if int(getattr(attn_metadata, "num_actual_tokens", n_seqs)) != n_seqs:
        return "batch_mismatch"
    if int(query.shape[0]) < n_seqs:
        return "empty_query"
    layer_name = getattr(layer, "layer_name", None)
    if layer_name is None:
        return "layer_name_missing"
    layer_cfg = pool.get_layer_config(layer_name)
    if layer_cfg is None:
        return "layer_config_missing"
    if int(query.shape[-1]) != layer_cfg.head_dim:
        return "head_dim_mismatch"
    if layer_cfg.head_dim % pool.config.group_size != 0:
        return "group_size_mismatch"
    return None


def _seq_lens_on_host(seq_lens: torch.Tensor) -> torch.Tensor:
    """Host copy of the step's sequence lengths.  Every layer of a step passes the same tensor: the copy (a
    device synchronisation) is made once per (storage, in-place version) and reused by the other layers."""
    key = (seq_lens.data_ptr(), int(seq_lens.numel()), seq_lens._version, str(seq_lens.device))
    hit = _SEQ_LENS_CACHE.get("k")
    if hit is not None and hit[0] == key:
        return hit[1]
    host = seq_lens.to("cpu", dtype=torch.long)
    _SEQ_LENS_CACHE["k"] = (key, host)
    return host


def _handoff_for(store, B: int, H_q: int, H_kv: int, K: int, scale: float):
    key = (id(store), B, H_q, K, float(scale))
    h = _HANDOFFS.get(key)
    if h is None:
        threads = get_jetfire_config().cpu_attn_threads
        if threads > 0:
            ops.set_cpu_attn_threads(threads)
        h = ops.CpuTopkHandoff(B, H_q, H_kv, K, store.k_shadow, store.v_shadow, scale)
        _HANDOFFS[key] = h
    return h


def reset_jetfire_decode_runtime_state() -> None:
    """Close the cached hand-off contexts and scratch tensors (call before the stores they point at go away)."""
    for h in _HANDOFFS.values():
        h.close()
    _HANDOFFS.clear()
    _O_NEW.clear()
    _HEAD_MAP_CACHE.clear()
    _SEQ_LENS_CACHE.clear()


def try_jetfire_decode(*, impl, layer, query, attn_metadata, output, key=None, value=None):
    """Production decode entry: `output` on success, None if a precondition fails."""
    return _decode_batched(impl=impl, layer=layer, query=query, attn_metadata=attn_metadata, output=output)


def _decode_batched(*, impl, layer, query, attn_metadata, output):
    pool = get_global_kv_pool_manager()
    pool.record_decode_attempt()
    layer_name = getattr(layer, "layer_name", "unknown_layer")
    pool.ensure_layer_config_from_layer(layer_name, layer)
    reason = _decode_unsupported(impl=impl, layer=layer, query=query, attn_metadata=attn_metadata)
    if reason is not None:
        pool.record_decode_fallback(reason)
        return None
    if not get_jetfire_config().cpu_correction:
        pool.record_decode_fallback("cpu_correction_disabled")
        return None
    layer_cfg = pool.get_layer_config(layer_name)
    store = pool.get_layer_store(layer_name)
    if store is None:
        pool.record_decode_fallback("store_missing")
        return None
    if store.scheme is None or store.block_size != 16 or layer_cfg.head_dim != 128 or not store.shadow_enabled:
        pool.record_decode_fallback("scheme_unsupported")
        return None
    store.flush_pending_writes()

    n_seqs = int(attn_metadata.seq_lens.numel())
    seq_lens_cpu = _seq_lens_on_host(attn_metadata.seq_lens)
    if os.environ.get("JETFIRE_FAST_STORE_COMPLETE_CHECK", "0") == "1":
        complete = store.fast_has_sequence(int(seq_lens_cpu.max().item()))      # host-side counter, no sync per sequence
    else:
        complete = all(n <= 0 or store.has_sequence(attn_metadata.block_table[i], int(n))
                       for i, n in enumerate(seq_lens_cpu.tolist()))
    if not complete:
        pool.record_decode_fallback("store_incomplete")
        return None

    H_q, H_kv, D = layer_cfg.num_query_heads, layer_cfg.num_kv_heads, layer_cfg.head_dim
    scale = float(getattr(impl, "scale", 1.0 / math.sqrt(D)))
    max_S = int(getattr(attn_metadata, "max_seq_len", int(seq_lens_cpu.max().item())))
    top_k = _select_top_k(pool.config.topk, max_S, FUSED_SUPPORTED_TOP_K)
    if top_k is None:
        pool.record_decode_fallback("seq_len_too_short")
        return None

    q_batch = query[:n_seqs].contiguous().view(n_seqs, H_q, D).to(torch.bfloat16)
    bt_batch = attn_metadata.block_table[:n_seqs].to(torch.int64).contiguous()
    seq_lens_batch = attn_metadata.seq_lens.to(device=query.device, dtype=torch.int32).contiguous()

    o_hat, topk_slots, o_old, W, _ = ops.fused_attn_topk(
        store.scheme, q_batch, store.k_data, store.k_scales, store.v_data, store.v_scales, bt_batch, seq_lens_batch,
        max_S, H_q, H_kv, store.block_size, top_k, scale)
    handoff = _handoff_for(store, n_seqs, H_q, H_kv, top_k, scale)
    handoff.submit(q_batch, topk_slots)
    o_new = _O_NEW.get((n_seqs, H_q, query.device))
    if o_new is None:
        o_new = _O_NEW[(n_seqs, H_q, query.device)] = torch.empty(n_seqs, H_q, D, dtype=torch.bfloat16, device=query.device)
    handoff.wait(o_new)

    out_view = output[:n_seqs].view(n_seqs, H_q, D)
    if out_view.dtype == torch.bfloat16 and out_view.is_contiguous():
        ops.blend_unnorm_into(o_hat, o_old, W, o_new, out_view)
    else:
        tmp = torch.empty(n_seqs, H_q, D, dtype=torch.bfloat16, device=query.device)
        ops.blend_unnorm_into(o_hat, o_old, W, o_new, tmp)
        out_view.copy_(tmp.to(out_view.dtype))
    pool.record_decode_hit()
    return output
