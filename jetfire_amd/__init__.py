"""jetfire_amd — MI355X (gfx950) implementation of JetFire's GPU approximate-attention decode path.

The compute lives in libjetfire_amd.so (hand-written HIP + a C ABI, see include/jetfire_amd.h);
`jetfire_amd.kernels.*` mirror the reference's `jetfire_vllm.kernels.*` loader modules and
`jetfire_amd.ops` holds the torch-facing operators.
"""
from . import _lib  # noqa: F401

__version__ = "0.1.0"
