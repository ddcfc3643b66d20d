"""Runtime configuration of the adapter (the part of `jetfire_vllm/adapter/config.py:91-163` the decode path
reads): quantisation scheme, group size, correction width, switches.  Values come from the environment
variables the reference uses, and can be replaced programmatically with `set_jetfire_config`."""
from __future__ import annotations

import os
from dataclasses import dataclass, replace


@dataclass(frozen=True)
class QuantScheme:
    name: str
    k_nbits: int
    v_nbits: int
    k_asymmetric: bool = False
    v_asymmetric: bool = False
    default_group_size: int = 128


# the schemes of jetfire_vllm/adapter/config.py:91-163 that have kernels there: the nine symmetric pairs and the
# asymmetric INT2 keys; jetfire_vllm/artifact.py:59 gives the group sizes of the two release schemes
SCHEMES = {f"SymInt{k}K_SymInt{v}V": QuantScheme(f"SymInt{k}K_SymInt{v}V", k, v,
                                                 default_group_size=64 if (k, v) == (3, 2) else 128)
           for k in (2, 3, 4) for v in (2, 3, 4)}
# INT2 keys over the full four-level codebook with a zero-point per group, and their historical aliases
for _v in (2, 3, 4):
    SCHEMES[f"AsymInt2K4Level_SymInt{_v}V"] = QuantScheme(f"AsymInt2K4Level_SymInt{_v}V", 2, _v, k_asymmetric=True)
    SCHEMES[f"AsymInt2K_SymInt{_v}V"] = SCHEMES[f"AsymInt2K4Level_SymInt{_v}V"]


@dataclass(frozen=True)
class JetFireConfig:
    scheme: QuantScheme = SCHEMES["SymInt3K_SymInt2V"]
    group_size: int = 64
    topk: int = 256
    layer_stride: int = 1
    use_custom_backend: bool = True
    cpu_correction: bool = True
    shadow_enabled: bool = True
    skip_native_kv: bool = True         # the serving engine keeps no KV cache of its own (JETFIRE_SKIP_NATIVE_KV)
    max_batch_size: int = 0
    cpu_attn_threads: int = 0          # 0: the pool's default (all cores but two)
    debug_log: bool = False


_CONFIG: JetFireConfig | None = None


def _env(name: str, default, *aliases: str):
    """The reference's variable `name` (jetfire_vllm/adapter/config.py:306-388); `aliases` are names earlier versions
    of this adapter read, still honoured when the reference's own name is not set."""
    for n in (name, *aliases):
        if n in os.environ:
            return os.environ[n]
    return default


def _from_env() -> JetFireConfig:
    name = _env("JETFIRE_MODE", "SymInt3K_SymInt2V", "JETFIRE_QUANT_SCHEME")
    if name not in SCHEMES:
        raise ValueError(f"JETFIRE_MODE={name!r} is not a known quant scheme. Available: {sorted(SCHEMES)}")
    scheme = SCHEMES[name]
    use_custom = os.environ.get("JETFIRE_USE_CUSTOM_BACKEND", "1") == "1"
    cpu_corr = os.environ.get("JETFIRE_CPU_CORRECTION", "1") == "1"
    skip_native = os.environ.get("JETFIRE_SKIP_NATIVE_KV", "1") == "1"
    shadow = os.environ.get("JETFIRE_SHADOW", "1") == "1"
    stride = int(_env("JETFIRE_MIRROR_LAYER_STRIDE", 1, "JETFIRE_LAYER_STRIDE"))
    if use_custom:  # the reference's invariants (jetfire_vllm/adapter/config.py:337-358)
        if not cpu_corr and skip_native and shadow:
            raise ValueError("JETFIRE_CPU_CORRECTION=0 + JETFIRE_SKIP_NATIVE_KV=1 with shadow on is unsupported (decode "
                             "would have nowhere to go). Either enable CPU correction (default) or also set "
                             "JETFIRE_SHADOW=0 for a prefill-only configuration.")
        if stride > 1 and skip_native:
            raise ValueError(f"JETFIRE_MIRROR_LAYER_STRIDE={stride} skips some layers, which fall back to the native "
                             "attention, but JETFIRE_SKIP_NATIVE_KV=1 has freed the native KV cache. Set "
                             "JETFIRE_SKIP_NATIVE_KV=0 for this ablation.")
    return JetFireConfig(
        scheme=scheme,
        group_size=int(os.environ.get("JETFIRE_GROUP_SIZE", scheme.default_group_size)),
        topk=int(os.environ.get("JETFIRE_TOPK", 256)),
        layer_stride=stride,
        use_custom_backend=use_custom,
        cpu_correction=cpu_corr,
        shadow_enabled=shadow,
        skip_native_kv=skip_native,
        max_batch_size=int(os.environ.get("JETFIRE_MAX_BATCH_SIZE", 0)),
        cpu_attn_threads=int(os.environ.get("JETFIRE_CPU_ATTN_THREADS", 0)),
        debug_log=_env("JETFIRE_DEBUG_LOG", "0", "JETFIRE_DEBUG") == "1",
    )


def get_jetfire_config() -> JetFireConfig:
    global _CONFIG
    if _CONFIG is None:
        _CONFIG = _from_env()
    return _CONFIG


def set_jetfire_config(**changes) -> JetFireConfig:
    """Replace fields of the active configuration (`scheme` may be given by name).  Existing pool managers
    keep the configuration they were created with: reset the global manager afterwards."""
    global _CONFIG
    if isinstance(changes.get("scheme"), str):
        changes["scheme"] = SCHEMES[changes["scheme"]]
    _CONFIG = replace(get_jetfire_config(), **changes)
    return _CONFIG


def reset_jetfire_config() -> None:
    """Re-read the environment on the next `get_jetfire_config()` (jetfire_vllm/adapter/config.py:393-396)."""
    global _CONFIG
    _CONFIG = None
