"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares, the host
logic (CPU correction, worker pool, scheme tables) matches the oracle.  No GPU compute is called."""
import os
import re

import numpy as np
import pytest
import torch

from oracle import jetfire_oracle as O
from tests.helpers import bf16_tensor, bf16_to_f32, make_case

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "jetfire_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from jetfire_amd import _lib
    lib = _lib.load()
    names = header_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/jetfire_amd.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(names)
    assert b"gfx950" in lib.jf_version()


def test_every_declaration_cites_the_reference_interface_it_replaces():
    text = open(os.path.join(ROOT, "include", "jetfire_amd.h")).read()
    for cite in ("fused_quant_write.py", "int3_qk_scores.cu", "int8tc_qk_scores.cu", "int2_softmax_v.cu",
                 "int4_softmax_v.cu", "blend.cu", "cpu_topk_attn.cpp", "decode_path.py"):
        assert cite in text


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from jetfire_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_product_package_never_imports_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "jetfire_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.lower() or f == "build.py", f"{f} mentions the oracle"


@pytest.mark.parametrize("threads", (1, 3))
@pytest.mark.parametrize("B,Hq,Hkv,K", [(2, 8, 2, 32), (1, 32, 4, 256), (3, 4, 4, 7)])
def test_cpu_topk_attn_matches_oracle(threads, B, Hq, Hkv, K):
    from jetfire_amd import ops
    c = make_case(50 + K, B, Hq, Hkv, 256, 3, 2, 64, ragged=False)
    rng = np.random.default_rng(K)
    nslots = c["K"].shape[1]
    ts = rng.integers(0, nslots, size=(B, Hq, K)).astype(np.int64)
    ts[:, :, -1] = -1                                   # padding lane
    ts[0, 1, :] = -1                                    # a row with no valid slot -> zeros
    ts[0, 2, 0] = nslots + 5                            # out of range is masked
    hm = O.head_map(B, Hq, Hq // Hkv, K)
    ops.set_cpu_attn_threads(threads)
    assert ops.get_cpu_attn_threads() == threads
    out = torch.full((B, Hq, 128), 7.0, dtype=torch.bfloat16)
    done = torch.zeros(1, dtype=torch.int64)
    ops.cpu_topk_attn(bf16_tensor(c["q"]), bf16_tensor(c["K"]), bf16_tensor(c["V"]), torch.from_numpy(hm),
                      torch.from_numpy(ts), out, 128 ** -0.5, done)
    assert int(done[0]) == 1
    ref = O.cpu_topk_attn(c["q"], c["K"], c["V"], hm, ts, 128 ** -0.5)
    np.testing.assert_allclose(bf16_to_f32(out), ref, atol=2e-3, rtol=6e-3)    # scripts/validate_runtime.py:187-191
    assert (bf16_to_f32(out)[0, 1] == 0).all()


def test_cpu_topk_attn_single_slot_returns_the_value_row():
    from jetfire_amd import ops
    c = make_case(60, 1, 4, 2, 64, 3, 2, 64, ragged=False)
    ts = np.full((1, 4, 1), 9, dtype=np.int64)
    out = torch.empty((1, 4, 128), dtype=torch.bfloat16)
    ops.cpu_topk_attn(bf16_tensor(c["q"]), bf16_tensor(c["K"]), bf16_tensor(c["V"]),
                      torch.from_numpy(O.head_map(1, 4, 2, 1)), torch.from_numpy(ts), out, 0.1)
    for h in range(4):
        assert np.array_equal(bf16_to_f32(out)[0, h], c["V"][h // 2, 9])


def test_cpu_topk_attn_rejects_bad_tensors():
    from jetfire_amd import ops
    q = torch.zeros(1, 2, 128, dtype=torch.bfloat16)
    sh = torch.zeros(1, 16, 128, dtype=torch.bfloat16)
    idx = torch.zeros(1, 2, 4, dtype=torch.int64)
    with pytest.raises(RuntimeError):
        ops.cpu_topk_attn(q.float(), sh, sh, idx, idx, q.clone(), 0.1)
    with pytest.raises(RuntimeError):
        ops.cpu_topk_attn(q, sh, sh, idx.int(), idx, q.clone(), 0.1)


def test_kernel_sets_mirror_the_reference_dispatch_protocol():
    from jetfire_amd.kernels._dispatch import get_kernel_set
    k32 = get_kernel_set("SymInt3K_SymInt2V")
    assert (k32.nbits_k, k32.nbits_v, k32.asymmetric_k, k32.asymmetric_v, k32.head_dim) == (3, 2, False, False, 128)
    assert k32.supported_top_k == (32, 64, 128, 256, 512, 1024, 2048, 4096, 8192)
    k44 = get_kernel_set("SymInt4K_SymInt4V")
    assert (k44.nbits_k, k44.nbits_v) == (4, 4) and min(k44.supported_top_k) == 64
    with pytest.raises(NotImplementedError):
        k32.attn_with_scores()
    with pytest.raises(ValueError):
        k32.quant_write_k(None, None, None, None, object(), 64)
    with pytest.raises(ValueError):
        get_kernel_set("AsymInt2K4Level_SymInt2V")
