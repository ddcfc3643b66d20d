"""The entry point that allocates nothing (`jf_fused_scan_topk_static`: workspace in a fixed device array)
against `jf_fused_scan_topk` with a caller-provided workspace, through the C ABI: bit-equal outputs on two
calls in a row, the second on a smaller input, and a clear error for a shape the array cannot hold."""
import ctypes as C

import numpy as np
import pytest
import torch

from tests.helpers import make_case, to_device

pytestmark = pytest.mark.gpu

SCALE = 128 ** -0.5
SCHEME_ID = {"k3v2": 32, "k4v4": 44}


def _outputs(B, Hq, K, S, dev):
    return dict(
        idx=torch.full((B, Hq, K), -7, dtype=torch.int64, device=dev),
        slots=torch.full((B, Hq, K), -7, dtype=torch.int64, device=dev),
        o_hat=torch.full((B, Hq, 128), float("nan"), dtype=torch.float32, device=dev),
        o_old=torch.full((B, Hq, 128), float("nan"), dtype=torch.float32, device=dev),
        W=torch.full((B, Hq), float("nan"), dtype=torch.float32, device=dev),
        m=torch.full((B, Hq), float("nan"), dtype=torch.float32, device=dev),
        iz=torch.full((B, Hq), float("nan"), dtype=torch.float32, device=dev),
        scores=torch.full((B, Hq, S), float("nan"), dtype=torch.float32, device=dev),
    )


def _call(lib, static, scheme, gs, c, d, S, K, out, workspace=None):
    stream = torch.cuda.current_stream().cuda_stream
    head = (SCHEME_ID[scheme], gs, d["q"].data_ptr(), d["kd"].data_ptr(), d["ks"].data_ptr(), d["vd"].data_ptr(),
            d["vs"].data_ptr(), d["bt"].data_ptr(), d["lens"].data_ptr(), c["B"], c["Hq"], c["Hkv"], S,
            d["bt"].size(1), d["kd"].size(1), 16, SCALE, K, out["idx"].data_ptr(), out["slots"].data_ptr(),
            out["o_hat"].data_ptr(), out["o_old"].data_ptr(), out["W"].data_ptr(), out["m"].data_ptr(),
            out["iz"].data_ptr(), out["scores"].data_ptr())
    if static:
        return lib.jf_fused_scan_topk_static(*head, stream)
    return lib.jf_fused_scan_topk(*head, workspace.data_ptr(), workspace.numel(), stream)


def _compare(scheme, seed, B, Hq, Hkv, S, K, lens=None):
    from jetfire_amd import _lib
    lib = _lib.load()
    kb, vb, gs = {"k3v2": (3, 2, 64), "k4v4": (4, 4, 128)}[scheme]
    c = make_case(seed, B, Hq, Hkv, S, kb, vb, gs, lens=lens)
    d = to_device(c)
    for t in ("ks", "vs"):
        if d[t].dim() == 2:
            d[t] = d[t].unsqueeze(-1)
        d[t] = d[t].contiguous()
    need = lib.jf_fused_workspace_bytes(SCHEME_ID[scheme], B, Hq, Hkv, S, K)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    ref, got = _outputs(B, Hq, K, S, "cuda"), _outputs(B, Hq, K, S, "cuda")
    _lib.check(_call(lib, False, scheme, gs, c, d, S, K, ref, ws))
    # a first call resolves the array's address and sizes the kernel's LDS; the call after it must leave both torch's
    # allocator and the device's free memory (hipMalloc / hipHostMalloc made behind torch's back) where they were
    _lib.check(_call(lib, True, scheme, gs, c, d, S, K, got))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _lib.check(_call(lib, True, scheme, gs, c, d, S, K, got))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point changed the device's free memory"
    for name in ref:
        a, b = ref[name].cpu().numpy(), got[name].cpu().numpy()
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), f"{scheme}: {name} differs"
    assert not torch.isnan(got["o_hat"]).any() and int(got["idx"].max()) < S


@pytest.mark.parametrize("scheme", ("k3v2", "k4v4"))
def test_static_scratch_entry_matches_the_workspace_entry_on_two_calls(scheme):
    # a multi-split shape first, then a smaller one that leaves stale bytes of the first call in the array
    _compare(scheme, 11, 2, 8, 2, 9000, 256, lens=[9000, 8191])
    _compare(scheme, 12, 1, 8, 2, 700, 64, lens=[683])


def test_static_scratch_entry_rejects_shapes_beyond_its_array():
    from jetfire_amd import _lib
    lib = _lib.load()
    B, Hq, Hkv, S, K = 64, 64, 8, 131072, 1024
    assert lib.jf_fused_workspace_bytes(32, B, Hq, Hkv, S, K) > (64 << 20)
    nul = C.c_void_p(0)
    rc = lib.jf_fused_scan_topk_static(32, 64, nul, nul, nul, nul, nul, nul, nul, B, Hq, Hkv, S, S // 16, 1 << 20, 16,
                                       SCALE, K, nul, nul, nul, nul, nul, nul, nul, nul, nul)
    assert rc != 0
    assert b"built-in scratch" in lib.jf_last_error()


def test_static_scratch_entry_names_the_entry_point_for_zero_point_schemes():
    from jetfire_amd import _lib
    lib = _lib.load()
    nul = C.c_void_p(0)
    rc = lib.jf_fused_scan_topk_static(12, 64, nul, nul, nul, nul, nul, nul, nul, 1, 8, 2, 256, 16, 1024, 16,
                                       SCALE, 32, nul, nul, nul, nul, nul, nul, nul, nul, nul)
    assert rc != 0
    assert b"jf_fused_scan_topk_asym" in lib.jf_last_error()
