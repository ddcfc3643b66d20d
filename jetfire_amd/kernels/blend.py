"""Merge kernel loader (jetfire_vllm/kernels/blend.py:42-43; module jetfire_blend)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_blend_ext():
    _lib.load()
    return SimpleNamespace(blend_unnorm_into=ops.blend_unnorm_into, blend_unnorm=ops.blend_unnorm)
