"""Merge kernel loader (jetfire_vllm/kernels/blend.py:42-43; module jetfire_blend): blend, blend_into,
blend_unnorm_into, wait_and_blend_unnorm_into (jetfire_vllm/csrc/blend.cu:379-399)."""
from types import SimpleNamespace

from .. import _lib, ops


def load_blend_ext():
    _lib.load()
    return SimpleNamespace(blend=ops.blend, blend_into=ops.blend_into, blend_unnorm_into=ops.blend_unnorm_into,
                           wait_and_blend_unnorm_into=ops.wait_and_blend_unnorm_into, blend_unnorm=ops.blend_unnorm)
