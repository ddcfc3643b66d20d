"""Decode entry of the adapter (`jetfire_vllm/adapter/decode_path.py:1156-1184,1667-1712,1712-3237`): one
layer's attention for a batch of single-token queries over the quantised cache,

    fused scan + top-k  ->  pinned hand-off + CPU correction over the bf16 shadow  ->  blend into `output`.

`try_jetfire_decode` returns `output` on success and None when a precondition fails (the caller then uses
its native attention); every miss is recorded with the reference's reason string.

Graph mode (`JETFIRE_DECODE_GRAPH=1`, `decode_path.py:634-646`): the hand-off uses the kernel-only submit /
wait pair, nothing in the entry synchronises with the device, and the whole layer can be captured into a HIP
graph and replayed; `warmup_graph_decode_submit_contexts` creates, before capture, whatever a capture may
not allocate.  A miss while a graph is being captured raises instead of baking the caller's fall-back into
the graph (`:698-706`).  With `JETFIRE_RELEASE_GRAPH_POLICY=1` the kernels of a step are the ones the release
policy names (`release_policy.py`).  Every stage runs inside a named profiler range (`_timer`, the reference's
`decode_path.py:60-85`: on ROCm `torch.cuda.nvtx` emits roctx ranges, which `rocprofv3 --marker-trace` shows on the
timeline); `JETFIRE_PROFILE_DECODE=1` additionally synchronises around each stage and accumulates its wall time for
`jetfire_get_profile()`.  The reference's step-trace files and debug correction modes are not reproduced."""
from __future__ import annotations

import bisect
import contextlib
import math
import os
import re
import struct
import time
import weakref

import torch

from .. import ops
from . import release_policy
from .config import get_jetfire_config
from .kv_pool import get_global_kv_pool_manager

# correction widths the fused kernels take (all the split entry points take)
FUSED_SUPPORTED_TOP_K = ops.FUSED_TOP_K
SPLIT_SUPPORTED_TOP_K = ops.SUPPORTED_TOP_K

_TOPK_CLAMP_LOGGED: set = set()
_HEAD_MAP_CACHE: dict = {}
_STORES_WITH_HANDOFFS: "weakref.WeakSet" = weakref.WeakSet()   # stores that carry hand-off contexts (`store._jf_handoffs`)
_O_NEW: dict = {}
_SEQ_LENS_CACHE: dict = {}
_PROFILE_ACCUM: dict = {}


@contextlib.contextmanager
def _timer(name: str):
    """Named profiler range around one stage of the decode entry (`decode_path.py:60-85`; the stage names are the
    reference's where the stage exists there).  The range is always emitted -- pushing one costs next to nothing when
    no profiler listens -- except while a graph is being captured, where it would mark the capture, not the replays.
    With JETFIRE_PROFILE_DECODE=1 (never in graph mode: it synchronises) the stage's wall time is accumulated."""
    capturing = _graph_capture_active()
    if not capturing:
        torch.cuda.nvtx.range_push(name)
    try:
        if capturing or os.environ.get("JETFIRE_PROFILE_DECODE", "0") != "1":
            yield
            return
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        try:
            yield
        finally:
            torch.cuda.synchronize()
            _PROFILE_ACCUM.setdefault(name, []).append((time.perf_counter() - t0) * 1e3)
    finally:
        if not capturing:
            torch.cuda.nvtx.range_pop()


def jetfire_get_profile() -> dict:
    """Milliseconds per stage accumulated since the last call (`decode_path.py:82-85`)."""
    out = {k: list(v) for k, v in _PROFILE_ACCUM.items()}
    _PROFILE_ACCUM.clear()
    return out


def _select_top_k(config_top_k: int, seq_len: int, supported: tuple) -> int | None:
    """Correction width for a step (contract of `decode_path.py:1156-1182`, table in
    `tests/test_runtime_edge_cases.py:13-35`): the widest supported width that neither exceeds the configured
    one nor the context length; a context shorter than every admissible width runs with the narrowest of them
    (the kernels pad unused lanes with -1).  None for an empty context or when no width is admissible."""
    want, have = int(config_top_k), int(seq_len)
    widths = sorted(w for w in supported if 0 < w <= want)
    if have <= 0 or not widths:
        return None
    fit = bisect.bisect_right(widths, have)          # widths[:fit] can be filled by the context
    chosen = widths[fit - 1] if fit else widths[0]
    note = (want, chosen, tuple(supported))
    if chosen != want and note not in _TOPK_CLAMP_LOGGED:
        _TOPK_CLAMP_LOGGED.add(note)
        print(f"[jetfire] requested top_k={want} clamped to kernel-supported top_k={chosen}; "
              f"supported={tuple(supported)}.", flush=True)
    return chosen


def _get_head_map_cpu(B: int, H_q: int, num_groups: int, K: int) -> torch.Tensor:
    """head_map[b, h, k] = h // num_groups: the kv-head every query head reads."""
    key = (B, H_q, num_groups, K)
    hm = _HEAD_MAP_CACHE.get(key)
    if hm is None:
        hm = (torch.arange(H_q, dtype=torch.int64) // num_groups).view(1, H_q, 1).expand(B, H_q, K).contiguous()
        _HEAD_MAP_CACHE[key] = hm
    return hm


def _graph_mode_enabled() -> bool:
    return os.environ.get("JETFIRE_DECODE_GRAPH", "0") == "1"


def _graph_capture_active() -> bool:
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


def _graph_context_batch_sizes(max_batch_size: int) -> list[int]:
    """Batch sizes that need a hand-off context before a capture (`decode_path.py:668-695`): every size up to
    the maximum, unless `JETFIRE_GRAPH_CAPTURE_SIZES` lists the captured sizes (comma or semicolon separated;
    sizes outside 1..max are ignored, the maximum is always included)."""
    top = int(max_batch_size)
    if top <= 0:
        return []
    spec = os.environ.get("JETFIRE_GRAPH_CAPTURE_SIZES", "").strip()
    if not spec:
        return list(range(1, top + 1))
    fields = [f for f in (piece.strip() for piece in re.split(r"[;,]", spec)) if f]
    if any(re.fullmatch(r"[+-]?\d+", f) is None for f in fields):
        raise RuntimeError(f"JETFIRE_GRAPH_CAPTURE_SIZES must be a comma-separated list of integers; got {spec!r}")
    return sorted({top} | {n for n in map(int, fields) if 1 <= n <= top})


def _raise_graph_decode_miss(reason: str, *, layer_name: str) -> None:
    """A miss during capture would record the caller's native attention into the graph: refuse instead
    (`decode_path.py:698-706`).  `reason=` and `layer=` are what callers parse."""
    raise RuntimeError(f"JetFire decode cannot miss while a HIP graph is being captured (the fall-back would be "
                       f"recorded into the graph): reason={reason} layer={layer_name}. Create the layer stores and "
                       f"call warmup_graph_decode_submit_contexts() before the capture, or unset JETFIRE_DECODE_GRAPH.")


def _decode_unsupported(*, impl, layer, query, attn_metadata) -> str | None:
    """Dispatcher gate (`decode_path.py:1667-1695`): the reference's reason string of the first failing
    precondition, or None.  The preconditions are evaluated lazily, in the reference's order."""
    pool = get_global_kv_pool_manager()
    md = attn_metadata
    state: dict = {}

    def attn_type_name():
        kind = getattr(impl, "attn_type", None)
        return "DECODER" if kind is None else getattr(kind, "name", str(kind))

    def n_seqs():
        return int(md.seq_lens.numel())

    def layer_cfg():
        if "cfg" not in state:
            state["cfg"] = pool.get_layer_config(getattr(layer, "layer_name", None))
        return state["cfg"]

    gate = (
        ("pool_disabled", lambda: not pool.config.enabled),
        # the host-blocking hand-off cannot be captured; graph mode uses the kernel-only pair
        ("cuda_graph_capture", lambda: query.is_cuda and torch.cuda.is_current_stream_capturing()
                                       and not _graph_mode_enabled()),
        ("profiling_run", lambda: md is None),
        ("attn_type", lambda: attn_type_name() != "DECODER"),
        ("cascade", lambda: bool(getattr(md, "use_cascade", False))),
        ("prefill_or_multi_query", lambda: int(getattr(md, "max_query_len", 1)) != 1),
        ("batch_mismatch", lambda: int(getattr(md, "num_actual_tokens", n_seqs())) != n_seqs()),
        ("empty_query", lambda: int(query.shape[0]) < n_seqs()),
        ("layer_name_missing", lambda: getattr(layer, "layer_name", None) is None),
        ("layer_config_missing", lambda: layer_cfg() is None),
        ("head_dim_mismatch", lambda: int(query.shape[-1]) != layer_cfg().head_dim),
        ("group_size_mismatch", lambda: layer_cfg().head_dim % pool.config.group_size != 0),
    )
    return next((reason for reason, fails in gate if fails()), None)


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


def _handoff_for(store, B: int, H_q: int, H_kv: int, K: int, scale: float, *, stream_mode: bool = False,
                 layer_name: str = "unknown_layer"):
    """Hand-off context of (store, shape, mode).  The contexts live ON the store object, so a store that goes
    away takes its contexts (pinned buffers, dispatcher thread, the pointers into its shadow) with it and a new
    store can never be served a context that reads another store's shadow."""
    cache = store.__dict__.setdefault("_jf_handoffs", {})
    # a context serves one of the two modes; the scale is keyed as the fp32 value the kernels receive, so that
    # 1 / sqrt(d) and d ** -0.5 (one ulp apart in double precision) name the same context
    key = (B, H_q, K, struct.unpack("f", struct.pack("f", float(scale)))[0], bool(stream_mode))
    h = cache.get(key)
    if h is None:
        if _graph_capture_active():        # pinned allocations and thread start-up are not capturable
            _raise_graph_decode_miss("submit_context_missing", layer_name=layer_name)
        threads = get_jetfire_config().cpu_attn_threads
        if threads > 0:
            ops.set_cpu_attn_threads(threads)
        h = ops.CpuTopkHandoff(B, H_q, H_kv, K, store.k_shadow, store.v_shadow, scale)
        if stream_mode and _sanitize_output_enabled():   # the graph-mode guard, inside the blending wait kernel
            h.set_output_sanitize(True)
        cache[key] = h
        _STORES_WITH_HANDOFFS.add(store)
    return h


def _sanitize_output_enabled() -> bool:
    """decode_path.py:1142: non-finite decode outputs become zero in graph mode unless JETFIRE_SANITIZE_DECODE_OUTPUT=0
    (a NaN that enters the next layer poisons q, k and v of every later step of a replayed graph)."""
    return os.environ.get("JETFIRE_SANITIZE_DECODE_OUTPUT", "1") != "0"


def _all_handoffs():
    return [h for store in list(_STORES_WITH_HANDOFFS) for h in store.__dict__.get("_jf_handoffs", {}).values()]


def check_decode_handoffs() -> None:
    """Raise if any hand-off context has failed: a CPU correction job that failed or timed out, or a
    device-side wait that ran into its limit (from then on a graph replay blends zeros instead of the
    correction, without any host call that could notice).  One load of a pinned status word per context, no
    synchronisation: call it after the step's synchronise.  The decode entry, `flush_pending_writes` of the pool
    and `reset_jetfire_decode_runtime_state` call it too."""
    for h in _all_handoffs():
        h.check_status()


def _o_new_for(n_seqs: int, H_q: int, D: int, device) -> torch.Tensor:
    key = (n_seqs, H_q, torch.device(device))
    o_new = _O_NEW.get(key)
    if o_new is None:
        o_new = _O_NEW[key] = torch.empty(n_seqs, H_q, D, dtype=torch.bfloat16, device=device)
    return o_new


def warmup_graph_decode_submit_contexts(*, max_batch_size: int, device=None, scale: float | None = None,
                                        max_seq_len: int | None = None) -> dict:
    """Create, before a decode step is captured, the graph-mode hand-off contexts (pinned buffers, poller
    registration happens on first submit) of every mirrored layer for every captured batch size and every
    correction width up to the configured one, the `o_new` buffers, and the stores' append state
    (`decode_path.py:851-1015`).  `scale` is the attention scale the layers use (default head_dim ** -0.5); with
    `max_seq_len` the fused scan's workspace is sized for the longest context too (call this on the stream the
    capture will use)."""
    if max_batch_size <= 0:
        raise RuntimeError("JETFIRE_DECODE_GRAPH=1 requires JETFIRE_MAX_BATCH_SIZE>0 so decode host buffers and "
                           "submit contexts have stable pointers before graph capture.")
    cfg = get_jetfire_config()
    if not cfg.cpu_correction:
        raise RuntimeError("JETFIRE_DECODE_GRAPH=1 currently requires JETFIRE_CPU_CORRECTION=1.")
    pool = get_global_kv_pool_manager()
    if not pool.layer_stores:
        raise RuntimeError("JETFIRE_DECODE_GRAPH=1 cannot warm submit contexts before JetFire layer stores exist.")
    sizes = _graph_context_batch_sizes(int(max_batch_size))
    created = 0
    widths = ()
    for name, store in pool.layer_stores.items():
        layer_cfg = pool.get_layer_config(name)
        if layer_cfg is None or not store.shadow_enabled:
            continue
        supported = SPLIT_SUPPORTED_TOP_K       # (widths beyond the fused form's run the stage-wise kernels)
        top_k = _select_top_k(cfg.topk, cfg.topk, supported)
        if top_k is None:
            raise RuntimeError(f"JETFIRE_TOPK={cfg.topk} is not supported by the active kernel set.")
        widths = tuple(k for k in supported if k <= top_k) or (top_k,)
        store.warmup_graph_append(int(max_batch_size))
        if (max_seq_len and store.scheme is not None and top_k in FUSED_SUPPORTED_TOP_K
                and store.device.type == "cuda"):
            # the scan's workspace of this stream, sized for the largest step, so that no capture has to grow it
            ops.reserve_fused_workspace(store.scheme, int(max_batch_size), layer_cfg.num_query_heads,
                                        layer_cfg.num_kv_heads, int(max_seq_len), top_k, store.device)
        sc = float(scale) if scale is not None else 1.0 / math.sqrt(layer_cfg.head_dim)
        for n in sizes:
            _o_new_for(n, layer_cfg.num_query_heads, layer_cfg.head_dim, device if device is not None else store.device)
            for k in widths:
                before = len(store.__dict__.get("_jf_handoffs", {}))
                _handoff_for(store, n, layer_cfg.num_query_heads, layer_cfg.num_kv_heads, k, sc, stream_mode=True,
                             layer_name=name)
                created += len(store._jf_handoffs) - before
    return {"layers": len(pool.layer_stores), "batch_sizes": sizes, "top_k": list(widths), "contexts_created": created}


def reset_jetfire_decode_runtime_state(*, check: bool = False) -> None:
    """Close every hand-off context and drop the scratch tensors (the pool manager calls this before it lets
    go of its stores).  `check=True` first raises if a context has failed."""
    if check:
        check_decode_handoffs()
    for store in list(_STORES_WITH_HANDOFFS):
        for h in store.__dict__.pop("_jf_handoffs", {}).values():
            h.close()
    _STORES_WITH_HANDOFFS.clear()
    _O_NEW.clear()
    _HEAD_MAP_CACHE.clear()
    _SEQ_LENS_CACHE.clear()


def _split_stages(store, q, bt, sl, max_S: int, H_q: int, H_kv: int, top_k: int, scale: float, plan=None):
    """Stage A and Stage B as separate kernels.  With a release plan (`release_policy.plan_release_graph`) the two
    operators are the ones the plan names; otherwise each side is chosen by its bit width as the reference does
    (`decode_path.py:2013-2131` Stage A, `:2695-2935` Stage B): the path of the schemes that have no fused kernel."""
    bs = store.block_size
    kd, ks, vd, vs = store.k_data, store.k_scales, store.v_data, store.v_scales
    if plan is not None:
        a_name, b_name = plan.operators()
        if a_name is None or b_name is None:
            raise RuntimeError(f"release plan {plan.stage_a} / {plan.stage_b} has no kernel in this library")
    else:
        if store.k_nbits == 4:
            int8tc = (ks.shape[-1] == 1 and top_k >= 64 and os.environ.get("JETFIRE_USE_INT8_TC", "1") == "1")
            a_name = "int8tc_qk_scores_topk_stats" if int8tc else "int4_qk_scores_topk_stats"
        else:
            a_name = f"int{store.k_nbits}_qk_scores_topk"
        if store.v_nbits == 4 and store.k_nbits == 4 and vs.shape[-1] == 1:
            b_name = "int8tc_softmax_v_with_pre_corr_reg_stats" if q.shape[0] > 1 else "int4_softmax_v_with_pre_corr_wvs2_scores"
        else:
            b_name = {2: "int2_softmax_v_with_pre_corr_wvs2", 3: "int3_softmax_v_with_pre_corr_wvs2",
                      4: "int4_softmax_v_with_pre_corr_wvs2_scores"}[store.v_nbits]
    stage_a, stage_b = getattr(ops, a_name), getattr(ops, b_name)
    m = iz = None
    if a_name == "int2_qk_scores_topk":
        scores, idx, slots = stage_a(q, kd, ks, store.k_zp, bt, sl, max_S, H_q, H_kv, bs, scale, top_k)
    else:
        res = stage_a(q, kd, ks, bt, sl, max_S, H_q, H_kv, bs, scale, top_k)
        scores, idx, slots = res[:3]
        if len(res) == 5:
            m, iz = res[3], res[4]
    if b_name == "int8tc_softmax_v_with_pre_corr_reg_stats":
        if m is None:
            raise RuntimeError("the int8-weight Stage B needs the statistics of the int8 Stage A")
        o_hat, o_old, W = stage_b(scores, m, iz, vd, vs, bt, sl, idx, max_S, H_q, H_kv, bs, top_k)
    else:
        o_hat, o_old, W = stage_b(scores, vd, vs, bt, sl, idx, max_S, H_q, H_kv, bs, top_k)
    return o_hat, slots, o_old, W


def try_jetfire_decode(*, impl, layer, query, attn_metadata, output, key=None, value=None):
    """Production decode entry: `output` on success, None if a precondition fails."""
    with _timer("D_total"):
        return _decode_batched(impl=impl, layer=layer, query=query, attn_metadata=attn_metadata, output=output)


def _decode_batched(*, impl, layer, query, attn_metadata, output):
    pool = get_global_kv_pool_manager()
    pool.record_decode_attempt()
    layer_name = getattr(layer, "layer_name", "unknown_layer")
    pool.ensure_layer_config_from_layer(layer_name, layer)
    graph_mode = _graph_mode_enabled()

    def miss(reason: str):
        pool.record_decode_fallback(reason)
        if graph_mode and _graph_capture_active():
            _raise_graph_decode_miss(reason, layer_name=layer_name)
        return None

    reason = _decode_unsupported(impl=impl, layer=layer, query=query, attn_metadata=attn_metadata)
    if reason is not None:
        return miss(reason)
    if not get_jetfire_config().cpu_correction:
        return miss("cpu_correction_disabled")
    layer_cfg = pool.get_layer_config(layer_name)
    store = pool.get_layer_store(layer_name)
    if store is None:
        return miss("store_missing")
    if store.block_size != 16 or layer_cfg.head_dim != 128 or not store.shadow_enabled or store.k_scales.shape[-1] > 2:
        return miss("scheme_unsupported")
    store.flush_pending_writes()
    for h in store.__dict__.get("_jf_handoffs", {}).values():
        h.check_status()                    # a failed context must not go on blending zeros silently

    n_seqs = int(attn_metadata.seq_lens.numel())
    H_q, H_kv, D = layer_cfg.num_query_heads, layer_cfg.num_kv_heads, layer_cfg.head_dim
    scale = float(getattr(impl, "scale", 1.0 / math.sqrt(D)))
    if graph_mode:
        # no device-to-host copy of the lengths and no completeness check: they would block a capture; the
        # caller guarantees that the stores hold the sequences (decode_path.py:1749-1755)
        max_S = int(getattr(attn_metadata, "max_seq_len", 0) or 0)
        if max_S <= 0:
            return miss("max_seq_len_missing")
    else:
        seq_lens_cpu = _seq_lens_on_host(attn_metadata.seq_lens)
        if os.environ.get("JETFIRE_FAST_STORE_COMPLETE_CHECK", "0") == "1":
            complete = store.fast_has_sequence(int(seq_lens_cpu.max().item()))      # host-side counter, no sync per sequence
        else:
            complete = all(n <= 0 or store.has_sequence(attn_metadata.block_table[i], int(n))
                           for i, n in enumerate(seq_lens_cpu.tolist()))
        if not complete:
            return miss("store_incomplete")
        max_S = int(getattr(attn_metadata, "max_seq_len", int(seq_lens_cpu.max().item())))
    # Under the release policy (JETFIRE_RELEASE_GRAPH_POLICY=1) the step runs the two kernels the policy names for
    # this cell, through the split operators; otherwise the fused scan where it covers the scheme.
    # (every store goes through the policy, as in the reference, `decode_path.py:1857-1868`: a mode outside the
    # release set raises there instead of falling through to another path silently)
    release = release_policy.release_policy_enabled()
    if release:
        release_policy.validate_release_environment()
    top_k = _select_top_k(pool.config.topk, max_S, SPLIT_SUPPORTED_TOP_K)
    if top_k is None:
        return miss("seq_len_too_short")
    # the fused scan where it covers the scheme and the width; wider corrections run the stage-wise kernels
    # The scoring model of INT4 keys with one scale per row depends on the width and on JETFIRE_USE_INT8_TC, as in
    # the reference (`decode_path.py:2012-2022`): the int8-quantised-query model from top_k 64 up, else the bf16 model.
    scheme = store.scheme
    if scheme is not None and scheme.startswith("k4") and (
            top_k < 64 or os.environ.get("JETFIRE_USE_INT8_TC", "1") != "1"):
        scheme = "b4" + scheme[2:]
    fused = (not release and scheme is not None and top_k in FUSED_SUPPORTED_TOP_K
             and int(store.k_data.shape[1]) <= ops.FUSED_MAX_SLOTS and os.environ.get("JETFIRE_USE_FUSED_ATTN_TOPK", "1") == "1")
    plan = None
    if release:
        mode = (f"AsymInt2K4Level_SymInt{store.v_nbits}V" if store.k_asymmetric
                else f"SymInt{store.k_nbits}K_SymInt{store.v_nbits}V")
        cfg_max_B = int(get_jetfire_config().max_batch_size or 0)
        plan = release_policy.plan_release_graph(
            mode=mode, group_size=store.group_size, top_k=top_k, head_dim=D,
            num_query_heads=H_q, num_kv_heads=H_kv,
            max_graph_batch=cfg_max_B if cfg_max_B > 0 else n_seqs,
            require_ready=release_policy.release_require_ready())

    with _timer("V2_00_prep"):
        q_batch = query[:n_seqs].contiguous().view(n_seqs, H_q, D).to(torch.bfloat16)
        bt_batch = attn_metadata.block_table[:n_seqs].to(torch.int64).contiguous()
        seq_lens_batch = attn_metadata.seq_lens.to(device=query.device, dtype=torch.int32).contiguous()

    with _timer("V2_01_attn"):          # Stage A + Stage B of the reference, one pass here where the scheme allows
        if fused:
            o_hat, topk_slots, o_old, W, _ = ops.fused_attn_topk(
                scheme, q_batch, store.k_data, store.k_scales, store.v_data, store.v_scales, bt_batch, seq_lens_batch,
                max_S, H_q, H_kv, store.block_size, top_k, scale, k_zp=store.k_zp if store.k_asymmetric else None)
        else:
            o_hat, topk_slots, o_old, W = _split_stages(store, q_batch, bt_batch, seq_lens_batch, max_S, H_q, H_kv, top_k,
                                                        scale, plan=plan)
    handoff = _handoff_for(store, n_seqs, H_q, H_kv, top_k, scale, stream_mode=graph_mode, layer_name=layer_name)
    o_new = _o_new_for(n_seqs, H_q, D, query.device)
    out_view = output[:n_seqs].view(n_seqs, H_q, D)
    direct = out_view.dtype == torch.bfloat16 and out_view.is_contiguous()
    if graph_mode:          # kernels only: nothing here waits for the CPU
        with _timer("V2_02c_tpe_submit"):
            handoff.stream_submit(q_batch, topk_slots)
        if direct:          # the device-side wait blends as the correction arrives
            with _timer("V2_04_05_fused"):
                handoff.stream_wait_blend(o_hat, o_old, W, out_view)
            pool.record_decode_hit()
            return output
        with _timer("V2_04_join"):
            handoff.stream_wait(o_new)
    else:
        with _timer("V2_02c_tpe_submit"):
            handoff.submit(q_batch, topk_slots)
        with _timer("V2_04_join"):
            handoff.wait(o_new)
    with _timer("V2_05_post_corr"):
        if direct:
            ops.blend_unnorm_into(o_hat, o_old, W, o_new, out_view)
        else:
            tmp = torch.empty(n_seqs, H_q, D, dtype=torch.bfloat16, device=query.device)
            ops.blend_unnorm_into(o_hat, o_old, W, o_new, tmp)
            out_view.copy_(tmp.to(out_view.dtype))
        if graph_mode and _sanitize_output_enabled():   # (decode_path.py:1133-1149)
            torch.nan_to_num(out_view, nan=0.0, posinf=0.0, neginf=0.0, out=out_view)
    pool.record_decode_hit()
    return output
