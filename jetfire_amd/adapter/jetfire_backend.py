"""Attention-backend shim (`jetfire_vllm/adapter/jetfire_backend.py:135-209`): the two methods a serving
engine's attention implementation calls per layer, `do_kv_cache_update` (append: quantise-on-write + shadow mirror)
and `forward` (decode through `try_jetfire_decode`, anything else through the engine's own implementation), with the
reference's optional deferral of a prefill chunk's append until the chunk's attention has been enqueued (`:32-63,196-209`).

The reference derives its class from vLLM's FlashAttentionImpl; here the engine's implementation class is a
parameter, so the shim does not import a serving engine: `make_jetfire_attention_impl(FlashAttentionImpl)` gives
the drop-in class.  Prefill attention is the engine's own (outside this library's decode path)."""
from __future__ import annotations

import os

import torch

from .config import get_jetfire_config
from .decode_path import try_jetfire_decode
from .kv_pool import get_global_kv_pool_manager

_FALLBACK_HELP = (
    "JetFire decode fell back to the native attention, but with JETFIRE_SKIP_NATIVE_KV=1 the engine keeps no KV "
    "cache of its own, so the fall-back would produce garbage.\nRecent decode_fallbacks: {fallbacks}\n"
    "Common causes:\n"
    "  - seq_len_too_short: empty sequence or unsupported JETFIRE_TOPK (use a positive supported correction width)\n"
    "  - cpu_correction_disabled: set JETFIRE_CPU_CORRECTION=1 (default) or JETFIRE_SKIP_NATIVE_KV=0\n"
    "  - store_missing: layer not mirrored. Check JETFIRE_MIRROR_LAYER_STRIDE (must be 1 when skip_native_kv=1)")


def _should_defer_prefill_kv_mirror(layer_name: str, key) -> bool:
    """Whether the append of a prefill chunk waits until the chunk's own attention has been enqueued
    (`jetfire_vllm/adapter/jetfire_backend.py:32-63`, JETFIRE_DEFER_PREFILL_KV_MIRROR = 1 | force): only for chunks of
    at least JETFIRE_DEFER_PREFILL_KV_MIRROR_MIN_TOKENS tokens on the GPU, outside graph capture, and - unless forced -
    only for a pure prefill step without earlier context, which is read from the serving engine's forward context;
    without such an engine nothing is deferred, as in the reference when that lookup fails."""
    mode = os.environ.get("JETFIRE_DEFER_PREFILL_KV_MIRROR", "0")
    if mode not in ("1", "force"):
        return False
    if key is None or not getattr(key, "is_cuda", False):
        return False
    if torch.cuda.is_current_stream_capturing():
        return False
    if int(key.shape[0]) < int(os.environ.get("JETFIRE_DEFER_PREFILL_KV_MIRROR_MIN_TOKENS", "64")):
        return False
    if mode == "force":
        return True
    try:
        from vllm.forward_context import get_forward_context  # (only inside the serving engine)
        md = get_forward_context().attn_metadata
        if isinstance(md, dict):
            md = md.get(layer_name)
        if md is None or int(getattr(md, "max_query_len", 0)) <= 1:
            return False
        nd = getattr(md, "num_decodes", None)
        if nd is not None and int(nd) != 0:
            return False
        return not bool(getattr(md, "jetfire_prefill_has_context", False))
    except Exception:
        return False


def _flush_deferred_kv_mirror(layer) -> None:
    """Run the append that `do_kv_cache_update` put off (`jetfire_vllm/adapter/decode_path.py:1322-1333`)."""
    pending = getattr(layer, "_jetfire_deferred_kv_mirror", None)
    if pending is None:
        return
    delattr(layer, "_jetfire_deferred_kv_mirror")
    name, key, value, slots = pending
    get_global_kv_pool_manager().mirror_kv(layer_name=name, key=key, value=value, slot_mapping=slots)


def make_jetfire_attention_impl(native_impl_cls):
    """Subclass of the engine's attention implementation with JetFire's append and decode."""

    class JetFireAttentionImpl(native_impl_cls):
        def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, output_scale=None,
                    output_block_scale=None):
            decode_like = attn_metadata is not None and int(getattr(attn_metadata, "max_query_len", 1)) == 1
            if decode_like:
                _flush_deferred_kv_mirror(layer)  # (a decode step reads what an earlier prefill appended)
            if output is not None:
                done = try_jetfire_decode(impl=self, layer=layer, query=query, key=key, value=value,
                                          attn_metadata=attn_metadata, output=output)
                if done is not None:
                    return done
            kind = getattr(getattr(self, "attn_type", None), "name", "DECODER")
            decode_step = attn_metadata is not None and int(getattr(attn_metadata, "max_query_len", 1)) == 1
            if get_jetfire_config().skip_native_kv and decode_step and kind == "DECODER":
                # (the profiling pass, attn_metadata None, may fall through: its output is discarded; so may
                # prefill, which attends over the tokens it is handed)
                raise RuntimeError(_FALLBACK_HELP.format(fallbacks=get_global_kv_pool_manager().decode_fallbacks))
            res = super().forward(layer, query, key, value, kv_cache, attn_metadata, output=output,
                                  output_scale=output_scale, output_block_scale=output_block_scale)
            _flush_deferred_kv_mirror(layer)  # the prefill's own attention is in the stream: now the append
            return res

        def do_kv_cache_update(self, layer, key, value, kv_cache, slot_mapping) -> None:
            pool = get_global_kv_pool_manager()
            name = getattr(layer, "layer_name", "unknown_layer")
            pool.ensure_layer_config_from_layer(name, layer)
            if _should_defer_prefill_kv_mirror(name, key):
                layer._jetfire_deferred_kv_mirror = (name, key, value, slot_mapping)
            else:
                pool.mirror_kv(layer_name=name, key=key, value=value, slot_mapping=slot_mapping)
            if not get_jetfire_config().skip_native_kv:
                super().do_kv_cache_update(layer, key, value, kv_cache, slot_mapping)

    JetFireAttentionImpl.__qualname__ = f"JetFireAttentionImpl[{native_impl_cls.__name__}]"
    return JetFireAttentionImpl
