"""Adapter-level glue around the decode kernels: the per-layer cache store, the pool manager that owns the
stores and the decode statistics, and the decode entry the attention backend calls.  Mirrors the names and
the behaviour of `jetfire_vllm/adapter/{cache_store,kv_pool,decode_path,config}.py` for the symmetric
INT3/INT2 and INT4/INT4 schemes, without any dependence on vLLM: the `impl`, `layer` and `attn_metadata`
arguments are read through the same attributes the reference reads."""
from .cache_store import JetFireInt4CacheStore, JetFireLayerView
from .config import JetFireConfig, get_jetfire_config, set_jetfire_config
from .decode_path import (check_decode_handoffs, jetfire_get_profile, reset_jetfire_decode_runtime_state,
                          try_jetfire_decode, warmup_graph_decode_submit_contexts)
from .kv_pool import (JetFireKVPoolConfig, JetFireKVPoolManager, JetFireLayerConfig, JetFireLayerLayout,
                      get_global_kv_pool_manager, reset_global_kv_pool_manager)

__all__ = [
    "JetFireInt4CacheStore", "JetFireLayerView", "JetFireConfig", "get_jetfire_config", "set_jetfire_config",
    "try_jetfire_decode", "warmup_graph_decode_submit_contexts", "check_decode_handoffs", "jetfire_get_profile",
    "reset_jetfire_decode_runtime_state", "JetFireKVPoolConfig", "JetFireKVPoolManager", "JetFireLayerConfig", "JetFireLayerLayout",
    "get_global_kv_pool_manager", "reset_global_kv_pool_manager",
]
