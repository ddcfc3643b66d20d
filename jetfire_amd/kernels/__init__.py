"""Loader modules with the reference's names (jetfire_vllm/kernels/*.py).  Each `load_*_ext()` returns an
object exposing the functions the reference's pybind module of that name exports."""
