"""Per-quant-scheme kernel sets (jetfire_vllm/kernels/_dispatch/__init__.py:24-127).

The nine symmetric K/V pairs are provided; the asymmetric INT2-key schemes are not."""
from __future__ import annotations

import importlib

_SCHEMES = {f"SymInt{k}K_SymInt{v}V": f"jetfire_amd.kernels._dispatch.sym_int{k}_k_sym_int{v}_v:KERNELS"
            for k in (2, 3, 4) for v in (2, 3, 4)}


def get_kernel_set(scheme_name: str):
    spec = _SCHEMES.get(scheme_name)
    if spec is None:
        raise ValueError(f"Unknown quant scheme {scheme_name!r}")
    module_path, _, attr = spec.partition(":")
    return getattr(importlib.import_module(module_path), attr)
