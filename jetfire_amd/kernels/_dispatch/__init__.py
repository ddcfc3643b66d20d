"""Per-quant-scheme kernel sets (jetfire_vllm/kernels/_dispatch/__init__.py:24-127).

Only the two release schemes are provided: SymInt3K_SymInt2V and SymInt4K_SymInt4V."""
from __future__ import annotations

import importlib

_SCHEMES = {
    "SymInt3K_SymInt2V": "jetfire_amd.kernels._dispatch.sym_int3_k_sym_int2_v:KERNELS",
    "SymInt4K_SymInt4V": "jetfire_amd.kernels._dispatch.sym_int4_k_sym_int4_v:KERNELS",
}


def get_kernel_set(scheme_name: str):
    spec = _SCHEMES.get(scheme_name)
    if spec is None:
        raise ValueError(f"Unknown quant scheme {scheme_name!r}")
    module_path, _, attr = spec.partition(":")
    return getattr(importlib.import_module(module_path), attr)
