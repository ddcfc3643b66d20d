"""Pool manager: owns the per-layer cache stores, their shape registry and the decode statistics
(`jetfire_vllm/adapter/kv_pool.py:20-507`).  `mirror_kv` is what the attention layer calls with every new
K/V chunk; `get_layer_store` is what the decode entry reads."""
from __future__ import annotations

import re
from dataclasses import dataclass

import torch

from .cache_store import JetFireInt4CacheStore
from .config import get_jetfire_config


@dataclass(frozen=True)
class JetFireKVPoolConfig:
    enabled: bool
    group_size: int
    topk: int
    layer_stride: int
    k_nbits: int
    v_nbits: int
    k_asymmetric: bool
    v_asymmetric: bool


@dataclass(frozen=True)
class JetFireLayerConfig:
    num_query_heads: int
    num_kv_heads: int
    head_dim: int


@dataclass(frozen=True)
class JetFireLayerLayout:
    num_blocks: int
    block_size: int


class JetFireKVPoolManager:
    def __init__(self, config: JetFireKVPoolConfig):
        self.config = config
        self.token_counters: dict[str, int] = {}
        self.layer_stores: dict[str, JetFireInt4CacheStore] = {}
        self.layer_configs: dict[str, JetFireLayerConfig] = {}
        self.layer_layouts: dict[str, JetFireLayerLayout] = {}
        self.skipped_layers = 0
        self.written_slots = 0
        self.decode_attempts = 0
        self.decode_hits = 0
        self.decode_fallbacks: dict[str, int] = {}

    # ------------------------------------------------------------------ registry
    def register_layer_config(self, layer_name: str, *, num_query_heads: int, num_kv_heads: int, head_dim: int) -> None:
        self.layer_configs[layer_name] = JetFireLayerConfig(int(num_query_heads), int(num_kv_heads), int(head_dim))

    def register_layer_layout(self, layer_name: str, *, num_blocks: int, block_size: int) -> None:
        self.layer_layouts[layer_name] = JetFireLayerLayout(int(num_blocks), int(block_size))

    def get_layer_store(self, layer_name: str) -> JetFireInt4CacheStore | None:
        return self.layer_stores.get(layer_name)

    def get_layer_config(self, layer_name: str) -> JetFireLayerConfig | None:
        return self.layer_configs.get(layer_name)

    def ensure_layer_config_from_layer(self, layer_name: str, layer: object) -> JetFireLayerConfig | None:
        """Take the head counts from the attention layer object (or its `impl`) the first time it is seen."""
        config = self.layer_configs.get(layer_name)
        if config is not None:
            return config
        src = layer
        if getattr(src, "num_heads", None) is None and hasattr(layer, "impl"):
            src = layer.impl
        heads, kv_heads, size = (getattr(src, n, None) for n in ("num_heads", "num_kv_heads", "head_size"))
        if heads is None or kv_heads is None or size is None:
            return None
        self.register_layer_config(layer_name, num_query_heads=heads, num_kv_heads=kv_heads, head_dim=size)
        return self.layer_configs[layer_name]

    def _get_or_create_store(self, *, layer_name: str, device) -> JetFireInt4CacheStore:
        config, layout = self.layer_configs.get(layer_name), self.layer_layouts.get(layer_name)
        if config is None:
            raise RuntimeError(f"JetFire layer config missing for {layer_name}")
        if layout is None:
            raise RuntimeError(f"JetFire layer layout missing for {layer_name}")
        store = self.layer_stores.get(layer_name)
        if store is None or not store.compatible_with(num_kv_heads=config.num_kv_heads, head_dim=config.head_dim,
                                                      num_blocks=layout.num_blocks, block_size=layout.block_size):
            store = JetFireInt4CacheStore(
                num_kv_heads=config.num_kv_heads, head_dim=config.head_dim, group_size=self.config.group_size,
                num_blocks=layout.num_blocks, block_size=layout.block_size, device=device,
                k_nbits=self.config.k_nbits, v_nbits=self.config.v_nbits, k_asymmetric=self.config.k_asymmetric,
                v_asymmetric=self.config.v_asymmetric, shadow_enabled=get_jetfire_config().shadow_enabled)
            self.layer_stores[layer_name] = store
        return store

    def ensure_layer_store(self, layer_name: str, *, device) -> JetFireInt4CacheStore:
        return self._get_or_create_store(layer_name=layer_name, device=device)

    def ensure_all_layer_stores(self, *, device) -> int:
        n = 0
        for name in self.layer_configs:
            if name in self.layer_layouts and self._should_mirror_layer(name):
                self._get_or_create_store(layer_name=name, device=device)
                n += 1
        return n

    # ------------------------------------------------------------------ append
    def mirror_kv(self, layer_name: str, key: torch.Tensor, value: torch.Tensor,
                  slot_mapping: torch.Tensor | None = None) -> None:
        """Quantise the latest K/V chunk (T, Hkv, D) of a layer into its store."""
        if not self.config.enabled or key.numel() == 0 or value.numel() == 0:
            return
        if not self._should_mirror_layer(layer_name):
            self.skipped_layers += 1
            return
        config = self.layer_configs.get(layer_name)
        if config is None or self.layer_layouts.get(layer_name) is None:
            self.skipped_layers += 1      # shapes not registered yet (start-up profiling pass)
            return
        if int(key.shape[1]) != config.num_kv_heads or int(key.shape[2]) != config.head_dim:
            raise RuntimeError(f"JetFire layer config mismatch for {layer_name}: expected "
                               f"({config.num_kv_heads}, {config.head_dim}), got ({int(key.shape[1])}, {int(key.shape[2])})")
        store = self._get_or_create_store(layer_name=layer_name, device=key.device)
        if key.is_cuda and torch.cuda.is_current_stream_capturing():
            written = store.write_slots_graph(key=key, value=value, slot_mapping=slot_mapping,
                                              max_batch_size=get_jetfire_config().max_batch_size)
        else:
            written = store.write_slots(key=key, value=value, slot_mapping=slot_mapping)
        if written > 0:
            self.token_counters[layer_name] = self.token_counters.get(layer_name, 0) + written
            self.written_slots += written

    def flush_pending_writes(self) -> None:
        for store in self.layer_stores.values():
            store.flush_pending_writes()
            for h in store.__dict__.get("_jf_handoffs", {}).values():
                h.check_status()          # raises if a correction failed or a device-side wait hit its limit

    # ------------------------------------------------------------------ statistics
    def record_decode_attempt(self) -> None:
        self.decode_attempts += 1

    def record_decode_hit(self) -> None:
        self.decode_hits += 1

    def record_decode_fallback(self, reason: str) -> None:
        self.decode_fallbacks[reason] = self.decode_fallbacks.get(reason, 0) + 1

    def get_stats(self) -> dict[str, object]:
        return {
            "token_counters": dict(self.token_counters),
            "layer_configs": {k: vars(v) for k, v in self.layer_configs.items()},
            "layer_layouts": {k: vars(v) for k, v in self.layer_layouts.items()},
            "written_slots": self.written_slots,
            "decode_attempts": self.decode_attempts,
            "decode_hits": self.decode_hits,
            "decode_fallbacks": dict(self.decode_fallbacks),
            "skipped_layers": self.skipped_layers,
        }

    def reset_runtime_state(self, *, preserve_layouts: bool = True) -> None:
        from .decode_path import reset_jetfire_decode_runtime_state
        reset_jetfire_decode_runtime_state()      # the hand-off contexts point into the stores that go away now
        self.token_counters.clear()
        self.layer_stores.clear()
        if not preserve_layouts:
            self.layer_configs.clear()
            self.layer_layouts.clear()
        self.skipped_layers = self.written_slots = self.decode_attempts = self.decode_hits = 0
        self.decode_fallbacks.clear()

    def _should_mirror_layer(self, layer_name: str) -> bool:
        stride = max(1, int(self.config.layer_stride))
        if stride <= 1:
            return True
        m = re.search(r"\.(\d+)\.", layer_name)
        return True if m is None else int(m.group(1)) % stride == 0


_GLOBAL_MANAGER: JetFireKVPoolManager | None = None


def get_global_kv_pool_manager() -> JetFireKVPoolManager:
    global _GLOBAL_MANAGER
    if _GLOBAL_MANAGER is None:
        cfg = get_jetfire_config()
        _GLOBAL_MANAGER = JetFireKVPoolManager(JetFireKVPoolConfig(
            enabled=cfg.use_custom_backend, group_size=cfg.group_size, topk=cfg.topk, layer_stride=cfg.layer_stride,
            k_nbits=cfg.scheme.k_nbits, v_nbits=cfg.scheme.v_nbits, k_asymmetric=cfg.scheme.k_asymmetric,
            v_asymmetric=cfg.scheme.v_asymmetric))
    return _GLOBAL_MANAGER


def reset_global_kv_pool_manager() -> None:
    """Drop the global manager (and its stores); the next `get_global_kv_pool_manager` reads the configuration again."""
    global _GLOBAL_MANAGER
    from .decode_path import reset_jetfire_decode_runtime_state
    reset_jetfire_decode_runtime_state()
    _GLOBAL_MANAGER = None
