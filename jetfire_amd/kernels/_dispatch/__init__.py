"""Per-quant-scheme kernel sets (jetfire_vllm/kernels/_dispatch/__init__.py:24-127).

The nine symmetric K/V pairs and the three asymmetric INT2-key schemes (with their historical aliases)."""
from __future__ import annotations

import importlib

_SCHEMES = {f"SymInt{k}K_SymInt{v}V": f"jetfire_amd.kernels._dispatch.sym_int{k}_k_sym_int{v}_v:KERNELS"
            for k in (2, 3, 4) for v in (2, 3, 4)}
for _v, _mod in ((2, "int2_asym_k_sym_v"), (3, "int2_asym_k_sym_int3_v"), (4, "int2_asym_k_sym_int4_v")):
    _SCHEMES[f"AsymInt2K4Level_SymInt{_v}V"] = f"jetfire_amd.kernels._dispatch.{_mod}:KERNELS"
    _SCHEMES[f"AsymInt2K_SymInt{_v}V"] = _SCHEMES[f"AsymInt2K4Level_SymInt{_v}V"]


def get_kernel_set(scheme_name: str):
    spec = _SCHEMES.get(scheme_name)
    if spec is None:
        raise ValueError(f"Unknown quant scheme {scheme_name!r}")
    module_path, _, attr = spec.partition(":")
    return getattr(importlib.import_module(module_path), attr)
