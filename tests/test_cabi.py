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


def header_symbols(name="jetfire_amd.h"):
    text = open(os.path.join(ROOT, "include", name)).read()
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


def test_debug_hooks_live_in_their_own_header_and_only_in_a_hooks_build():
    """The product header declares no measurement / test hook; a library exports the hooks of
    include/jetfire_amd_debug.h exactly when its version string says it was built with them."""
    from jetfire_amd import _lib
    lib = _lib.load()
    product, hooks = header_symbols(), header_symbols("jetfire_amd_debug.h")
    assert not [n for n in product if "debug" in n or "profile" in n or "calibrate" in n]
    assert set(hooks) == set(_lib.DEBUG_SIGNATURES) and not set(hooks) & set(product)
    built_with = lib.jf_version().decode().endswith("+debug-hooks")
    assert built_with == _lib.has_debug_hooks()
    for n in hooks:
        assert hasattr(lib, n) == built_with, f"{n}: exported={hasattr(lib, n)}, hooks build={built_with}"
    if not built_with:
        with pytest.raises(RuntimeError, match="--debug-hooks"):
            _lib.debug_hook("jf_debug_split_len")


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


def _host_isas():
    from jetfire_amd import ops
    ops.set_cpu_attn_isa(None)
    widest = ops.get_cpu_attn_isa()
    return ("scalar", "avx2", "avx512bf16")[:("scalar", "avx2", "avx512bf16").index(widest) + 1]


@pytest.fixture
def widest_isa_afterwards():
    yield
    from jetfire_amd import ops
    ops.set_cpu_attn_isa(None)


@pytest.mark.parametrize("isa", ("scalar", "avx2", "avx512bf16"))
@pytest.mark.parametrize("threads", (1, 3))
@pytest.mark.parametrize("B,Hq,Hkv,K", [(2, 8, 2, 32), (1, 32, 4, 256), (3, 4, 4, 7)])
def test_cpu_topk_attn_matches_oracle(threads, B, Hq, Hkv, K, isa, widest_isa_afterwards):
    from jetfire_amd import ops
    if isa not in _host_isas():
        pytest.skip(f"this host has no {isa}")
    ops.set_cpu_attn_isa(isa)
    assert ops.get_cpu_attn_isa() == isa
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


@pytest.mark.parametrize("isa", ("scalar", "avx2", "avx512bf16"))
def test_cpu_topk_attn_sanitises_non_finite_rows(isa, widest_isa_afterwards):
    """jetfire_vllm/csrc/cpu_topk_attn.cpp:809-826,839-846: a row whose output is not finite (here: an infinite V
    element among its slots) is recomputed by the scalar row and zeroed when it still is; such rows are counted
    and every other row is untouched."""
    from jetfire_amd import ops
    if isa not in _host_isas():
        pytest.skip(f"this host has no {isa}")
    ops.set_cpu_attn_isa(isa)
    B, Hq, Hkv, K = 2, 8, 2, 16
    c = make_case(77, B, Hq, Hkv, 128, 3, 2, 64, ragged=False)
    rng = np.random.default_rng(5)
    nslots = c["K"].shape[1]
    ts = rng.integers(0, nslots, size=(B, Hq, K)).astype(np.int64)
    hm = O.head_map(B, Hq, Hq // Hkv, K)
    V = c["V"].copy()
    bad_slot = int(ts[1, 5, 3])
    V[5 // (Hq // Hkv), bad_slot, 17] = np.inf
    poisoned = {(b, h) for b in range(B) for h in range(Hq) if h // (Hq // Hkv) == 5 // (Hq // Hkv) and bad_slot in ts[b, h]}
    assert (1, 5) in poisoned
    ops.reset_graph_runtime_state()
    out = torch.full((B, Hq, 128), 7.0, dtype=torch.bfloat16)
    ops.cpu_topk_attn(bf16_tensor(c["q"]), bf16_tensor(c["K"]), bf16_tensor(V), torch.from_numpy(hm), torch.from_numpy(ts), out,
                      128 ** -0.5)
    assert ops.get_cpu_topk_sanitize_count() == len(poisoned)
    got = bf16_to_f32(out)
    assert np.isfinite(got).all()
    ref = O.cpu_topk_attn(c["q"], c["K"], c["V"], hm, ts, 128 ** -0.5)
    for b in range(B):
        for h in range(Hq):
            if (b, h) in poisoned:
                assert (got[b, h] == 0).all()
            else:
                np.testing.assert_allclose(got[b, h], ref[b, h], atol=2e-3, rtol=6e-3)
    ops.reset_graph_runtime_state()
    assert ops.get_cpu_topk_sanitize_count() == 0


def test_async_submit_and_wait_for_flag_match_the_synchronous_call():
    """submit_cpu_topk_attn_async / wait_for_flag (jetfire_vllm/csrc/cpu_topk_attn.cpp:1184-1260)."""
    from jetfire_amd.kernels.cpu_topk_attn import load_cpu_topk_attn_ext
    ext = load_cpu_topk_attn_ext()
    for name in ("cpu_topk_attn", "alloc_mapped_pinned_pair", "submit_cpu_topk_attn_async", "wait_for_flag",
                 "create_cpu_topk_submit_ctx", "stream_submit_cpu_topk_attn", "stream_wait_cpu_topk_attn",
                 "stream_write_value64", "stream_wait_value64", "graph_pool_warmup", "graph_pool_warmup_threads",
                 "get_graph_submit_count", "get_cpu_topk_sanitize_count", "reset_graph_runtime_state",
                 "clear_graph_contexts", "set_cpu_attn_threads", "get_cpu_attn_threads"):
        assert callable(getattr(ext, name)), name
    from jetfire_amd.kernels.blend import load_blend_ext
    for name in ("blend", "blend_into", "blend_unnorm_into", "wait_and_blend_unnorm_into"):
        assert callable(getattr(load_blend_ext(), name)), name
    B, Hq, Hkv, K = 2, 8, 2, 32
    c = make_case(31, B, Hq, Hkv, 256, 3, 2, 64, ragged=False)
    rng = np.random.default_rng(9)
    ts = torch.from_numpy(rng.integers(-1, c["K"].shape[1], size=(B, Hq, K)).astype(np.int64))
    hm = torch.from_numpy(O.head_map(B, Hq, Hq // Hkv, K))
    q, ksh, vsh = bf16_tensor(c["q"]), bf16_tensor(c["K"]), bf16_tensor(c["V"])
    ext.graph_pool_warmup_threads(3)
    assert ext.get_cpu_attn_threads() == 3
    want = torch.zeros(B, Hq, 128, dtype=torch.bfloat16)
    ext.cpu_topk_attn(q, ksh, vsh, hm, ts, want, 0.09)
    for rep in range(3):
        got = torch.full((B, Hq, 128), 5.0, dtype=torch.bfloat16)
        flag = torch.zeros(1, dtype=torch.int64)
        ext.submit_cpu_topk_attn_async(q, ksh, vsh, hm, ts, got, 0.09, flag)
        ext.wait_for_flag(flag)
        assert int(flag[0]) == 1 and torch.equal(got.view(torch.int16), want.view(torch.int16))
    with pytest.raises(RuntimeError, match="flag must be"):
        ext.wait_for_flag(torch.zeros(2, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="unknown context handle"):
        ext.stream_submit_cpu_topk_attn(0, 12345)
    ext.set_cpu_attn_threads(2)


def test_cpu_pool_survives_oversubscription_and_resizing():
    """Many back-to-back jobs on far more workers than cores, with the pool resized in between: every job's
    output equals the single-thread result bit for bit (a late worker must never touch a newer job's rows)."""
    from jetfire_amd import ops
    B, Hq, Hkv, K = 4, 16, 4, 64
    c = make_case(91, B, Hq, Hkv, 512, 3, 2, 64, ragged=False)
    rng = np.random.default_rng(3)
    nslots = c["K"].shape[1]
    hm = torch.from_numpy(O.head_map(B, Hq, Hq // Hkv, K))
    ksh, vsh = bf16_tensor(c["K"]), bf16_tensor(c["V"])
    cases = []
    ops.set_cpu_attn_threads(1)
    for i in range(6):
        q = bf16_tensor(O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32)))
        ts = torch.from_numpy(rng.integers(-1, nslots, size=(B, Hq, K)).astype(np.int64))
        want = torch.zeros(B, Hq, 128, dtype=torch.bfloat16)
        ops.cpu_topk_attn(q, ksh, vsh, hm, ts, want, 0.09)
        cases.append((q, ts, want))
    out = torch.zeros(B, Hq, 128, dtype=torch.bfloat16)
    for threads in (33, 5, 64):
        ops.set_cpu_attn_threads(threads)
        for rep in range(60):
            q, ts, want = cases[rep % len(cases)]
            out.fill_(3.0)
            ops.cpu_topk_attn(q, ksh, vsh, hm, ts, out, 0.09)
            assert torch.equal(out.view(torch.int16), want.view(torch.int16)), (threads, rep)
    ops.set_cpu_attn_threads(2)


def test_cpu_pool_backs_up_a_row_whose_worker_has_stalled():
    """A worker that stalls inside a row (as if it had lost its core) must not hold the job: an idle worker recomputes
    the row after the grace period and commits it; what the stalled worker produces later is discarded, also when a
    newer job has reused the buffers by then."""
    import time
    from jetfire_amd import _lib, ops
    lib = _lib.load()
    B, Hq, Hkv, K = 2, 16, 4, 64
    c = make_case(92, B, Hq, Hkv, 512, 3, 2, 64, ragged=False)
    rng = np.random.default_rng(4)
    nslots = c["K"].shape[1]
    hm = torch.from_numpy(O.head_map(B, Hq, Hq // Hkv, K))
    ksh, vsh = bf16_tensor(c["K"]), bf16_tensor(c["V"])
    ops.set_cpu_attn_threads(4)

    def case():
        q = bf16_tensor(O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32)))
        ts = torch.from_numpy(rng.integers(-1, nslots, size=(B, Hq, K)).astype(np.int64))
        return q, ts
    q1, ts1 = case()
    q2, ts2 = case()
    want1, want2 = torch.zeros(B, Hq, 128, dtype=torch.bfloat16), torch.zeros(B, Hq, 128, dtype=torch.bfloat16)
    ops.cpu_topk_attn(q1, ksh, vsh, hm, ts1, want1, 0.09)
    ops.cpu_topk_attn(q2, ksh, vsh, hm, ts2, want2, 0.09)
    assert not torch.equal(want1, want2)
    q, ts, out = q1.clone(), ts1.clone(), torch.zeros(B, Hq, 128, dtype=torch.bfloat16)
    stall_s = 0.6
    _lib.check(_lib.debug_hook("jf_debug_pool_wait_stragglers")(0))
    try:
        _lib.check(_lib.debug_hook("jf_debug_pool_stall")(5, int(stall_s * 1e6)))
        t0 = time.perf_counter()
        ops.cpu_topk_attn(q, ksh, vsh, hm, ts, out, 0.09)
        took = time.perf_counter() - t0
        assert took < stall_s / 2, took                       # the job did not wait for the stalled worker
        assert torch.equal(out.view(torch.int16), want1.view(torch.int16))
        # a newer job over the same buffers while the stalled worker is still asleep on the old one
        q.copy_(q2)
        ts.copy_(ts2)
        ops.cpu_topk_attn(q, ksh, vsh, hm, ts, out, 0.09)
        assert torch.equal(out.view(torch.int16), want2.view(torch.int16))
        time.sleep(stall_s + 0.2)                             # the stalled worker wakes up, finishes, and must write nothing
        assert torch.equal(out.view(torch.int16), want2.view(torch.int16))
        ops.cpu_topk_attn(q, ksh, vsh, hm, ts, out, 0.09)     # and the pool is whole again
        assert torch.equal(out.view(torch.int16), want2.view(torch.int16))
    finally:
        _lib.check(_lib.debug_hook("jf_debug_pool_wait_stragglers")(1))
    # default behaviour of the synchronous call: it returns only when no worker is inside a row any more
    _lib.check(_lib.debug_hook("jf_debug_pool_stall")(3, 200000))
    t0 = time.perf_counter()
    ops.cpu_topk_attn(q, ksh, vsh, hm, ts, out, 0.09)
    assert time.perf_counter() - t0 >= 0.19
    assert torch.equal(out.view(torch.int16), want2.view(torch.int16))
    ops.set_cpu_attn_threads(2)


def test_cpu_pool_pins_its_workers_on_request():
    """JETFIRE_CPU_ATTN_PIN=1 (read once per process, so a child process): every worker ends up on one core of the
    set the process may use, each on a different one, and the rows come out as without the switch."""
    import os
    import subprocess
    import sys
    code = r"""
import os, sys, glob, numpy as np, torch
sys.path.insert(0, %r)
from jetfire_amd import ops
from oracle import jetfire_oracle as O
from tests.helpers import bf16_tensor, make_case
B, Hq, Hkv, K = 2, 8, 2, 32
c = make_case(5, B, Hq, Hkv, 256, 3, 2, 64, ragged=False)
rng = np.random.default_rng(1)
hm = torch.from_numpy(O.head_map(B, Hq, Hq // Hkv, K))
q = bf16_tensor(O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32)))
ts = torch.from_numpy(rng.integers(-1, c["K"].shape[1], size=(B, Hq, K)).astype(np.int64))
out = torch.zeros(B, Hq, 128, dtype=torch.bfloat16)
ops.set_cpu_attn_threads(3)
ops.cpu_topk_attn(q, bf16_tensor(c["K"]), bf16_tensor(c["V"]), hm, ts, out, 0.09)
import time
time.sleep(0.5)            # (a short job can end before the last worker thread has run its first instruction)
masks = []
for t in glob.glob("/proc/self/task/*/status"):
    txt = open(t).read()
    allowed = [l.split(":")[1].strip() for l in txt.splitlines() if l.startswith("Cpus_allowed_list")][0]
    masks.append(allowed)
print("MASKS", ";".join(sorted(masks)))
print("SUM", float(out.float().abs().sum()))
""" % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    runs = {}
    for pin in ("0", "1"):
        env = dict(os.environ, JETFIRE_CPU_ATTN_PIN=pin)
        res = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
        assert res.returncode == 0, res.stderr[-2000:]
        lines = dict(l.split(" ", 1) for l in res.stdout.splitlines() if l.startswith(("MASKS", "SUM")))
        runs[pin] = lines
    assert runs["0"]["SUM"] == runs["1"]["SUM"]
    allowed = sorted(os.sched_getaffinity(0))
    single = [m for m in runs["1"]["MASKS"].split(";") if m.isdigit()]       # threads bound to exactly one core
    if len(allowed) >= 3:
        assert sorted(int(m) for m in single) == allowed[:3], (single, allowed)
    assert not [m for m in runs["0"]["MASKS"].split(";") if m.isdigit()] or len(allowed) == 1


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
    for k in (2, 3, 4):
        for v in (2, 3, 4):
            ks = get_kernel_set(f"SymInt{k}K_SymInt{v}V")
            assert (ks.nbits_k, ks.nbits_v, ks.asymmetric_k) == (k, v, False)
    a2 = get_kernel_set("AsymInt2K_SymInt3V")                       # historical alias of the 4-level scheme
    assert a2 is get_kernel_set("AsymInt2K4Level_SymInt3V") and (a2.nbits_k, a2.nbits_v, a2.asymmetric_k) == (2, 3, True)
    with pytest.raises(ValueError):
        a2.quant_write_k(None, None, None, None, None, 64)          # zero-points are required
    with pytest.raises(ValueError):
        get_kernel_set("AsymInt3K_SymInt3V")                        # a placeholder in the reference too: no kernels


@pytest.mark.parametrize("scheme,gs,B,Hq,Hkv,S,K", [
    (32, 64, 4, 32, 8, 32768, 256),       # the headline shape
    (44, 128, 1, 32, 8, 131072, 512),     # long context, few rows: two-stage merge
    (32, 64, 2, 32, 4, 65536, 512),
    (32, 128, 1, 8, 8, 100, 32),
    (44, 128, 64, 32, 8, 2048, 1024),
    (44, 128, 1, 32, 8, 262144, 1024),
    (32, 64, 1, 16, 1, 0, 64),
])
def test_fused_plan_geometry_is_consistent(scheme, gs, B, Hq, Hkv, S, K):
    """Host logic of the fused launch (no GPU): the split grid covers max_S, stays inside the kernels' limits,
    the two-stage merge keeps its final pass register-resident, and the workspace grows with it."""
    import ctypes as C
    from jetfire_amd import _lib
    lib = _lib.load()
    out = [C.c_int() for _ in range(4)]
    _lib.check(lib.jf_fused_plan(scheme, gs, B, Hq, Hkv, S, K, *[C.byref(o) for o in out]))
    L, ns, cap, parts = [o.value for o in out]
    assert L % 256 == 0 and 256 <= L <= 4096
    assert ns >= 1 and ns * L >= S and (ns - 1) * L < max(S, 1)
    assert ns <= 256
    assert cap == min(L, K + 256)
    assert parts >= 1
    if ns * cap <= 8192:
        assert parts == 1
    if parts > 1:
        assert parts * K <= 8192 and parts * 2 <= ns
    need = lib.jf_fused_workspace_bytes(scheme, B, Hq, Hkv, S, K)
    rows = B * Hq
    floor = rows * ns * (8 + 128 * 4 + cap * 8 + 4) + (rows * parts * (K * 8 + 4) if parts > 1 else 0)
    assert need >= floor
    # forcing a split length is honoured (rounded up to 256, clamped) and switched off again by 0
    _lib.check(_lib.debug_hook("jf_debug_split_len")(300))
    try:
        _lib.check(lib.jf_fused_plan(scheme, gs, B, Hq, Hkv, S, K, C.byref(out[0]), None, None, None))
        assert out[0].value == 512 or (S > 512 * 256 and out[0].value > 512)
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))
    _lib.check(lib.jf_fused_plan(scheme, gs, B, Hq, Hkv, S, K, C.byref(out[0]), None, None, None))
    assert out[0].value == L


def test_fused_plan_rejects_bad_shapes():
    from jetfire_amd import _lib
    lib = _lib.load()
    assert lib.jf_fused_plan(7, 64, 1, 8, 2, 100, 32, None, None, None, None) != 0
    assert lib.jf_fused_plan(32, 64, 1, 8, 3, 100, 32, None, None, None, None) != 0
    assert lib.jf_fused_plan(32, 32, 1, 8, 2, 100, 32, None, None, None, None) != 0


def test_adapter_reads_the_reference_environment_names(monkeypatch):
    """`jetfire_vllm/adapter/config.py:306-388`: JETFIRE_MODE, JETFIRE_MIRROR_LAYER_STRIDE, JETFIRE_DEBUG_LOG (the names
    this adapter used before stay as aliases), and the two invariants that protect a freed native KV cache."""
    from jetfire_amd.adapter import config
    for n in list(os.environ):
        if n.startswith("JETFIRE_"):
            monkeypatch.delenv(n)
    config.reset_jetfire_config()
    try:
        monkeypatch.setenv("JETFIRE_MODE", "SymInt4K_SymInt4V")
        monkeypatch.setenv("JETFIRE_QUANT_SCHEME", "SymInt2K_SymInt2V")      # the reference's name wins
        monkeypatch.setenv("JETFIRE_DEBUG_LOG", "1")
        cfg = config.get_jetfire_config()
        assert cfg.scheme.name == "SymInt4K_SymInt4V" and cfg.debug_log and cfg.layer_stride == 1
        config.reset_jetfire_config()
        monkeypatch.delenv("JETFIRE_MODE")
        assert config.get_jetfire_config().scheme.name == "SymInt2K_SymInt2V"   # alias alone still works
        config.reset_jetfire_config()
        monkeypatch.setenv("JETFIRE_MIRROR_LAYER_STRIDE", "2")
        with pytest.raises(ValueError, match="JETFIRE_MIRROR_LAYER_STRIDE=2"):
            config.get_jetfire_config()
        monkeypatch.setenv("JETFIRE_SKIP_NATIVE_KV", "0")
        assert config.get_jetfire_config().layer_stride == 2
        config.reset_jetfire_config()
        monkeypatch.delenv("JETFIRE_MIRROR_LAYER_STRIDE")
        monkeypatch.setenv("JETFIRE_LAYER_STRIDE", "3")
        assert config.get_jetfire_config().layer_stride == 3
        config.reset_jetfire_config()
        monkeypatch.setenv("JETFIRE_SKIP_NATIVE_KV", "1")
        monkeypatch.delenv("JETFIRE_LAYER_STRIDE")
        monkeypatch.setenv("JETFIRE_CPU_CORRECTION", "0")
        with pytest.raises(ValueError, match="JETFIRE_CPU_CORRECTION=0"):
            config.get_jetfire_config()
        monkeypatch.setenv("JETFIRE_MODE", "NoSuchMode")
        with pytest.raises(ValueError, match="JETFIRE_MODE='NoSuchMode'"):
            config.get_jetfire_config()
    finally:
        config.reset_jetfire_config()


def test_pool_wake_needs_no_gpu():
    from jetfire_amd import ops
    ops.set_cpu_attn_threads(2)
    ops.pool_wake()
    ops.pool_wake()
    assert ops.get_cpu_attn_threads() == 2
    ops.set_cpu_attn_threads(0)


def test_bench_reports_counter_figures_only_for_the_loaded_build(monkeypatch, tmp_path):
    """bench.py takes `traffic` and the busy shares from the committed rocprofv3 summaries; a summary names the
    library build it was taken with, and one of another build is not reported."""
    import json
    import bench
    from jetfire_amd import _lib

    have = _lib.load().jf_version().decode()
    assert bench.lib_version() == have and "build" in have
    prof = tmp_path / "profiles"
    prof.mkdir()
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))

    def write(version):
        (prof / "fused_scan_k3v2_c2_traffic.json").write_text(json.dumps(
            {"traffic_bytes_per_launch": 123, "lib_version": version}))
        (prof / "decode_kernels_c2_sq_counters.json").write_text(json.dumps(
            {"fused_scan_kernel": {"mfma_busy_pct": 1.0, "valu_issue_pct": 2.0}, "lib_version": version}))

    write(have)
    out = bench.profile_counters("k3v2", "c2")
    assert out["traffic"] == 123 and out["mfma_busy_pct"] == 1.0 and "traffic_stale" not in out
    write("jetfire_amd 0.3 (gfx950) build 000000000000")
    out = bench.profile_counters("k3v2", "c2")
    assert out["traffic"] is None and "mfma_busy_pct" not in out
    assert "000000000000" in out["traffic_stale"] and "000000000000" in out["counters_stale"]
    # no summary at all: null, nothing claimed
    assert bench.profile_counters("k3v2", "nowhere") == {"traffic": None}


def test_committed_counter_summaries_belong_to_the_sources_in_the_tree():
    """The summaries under profiles/ name a build digest; it must be the digest of the sources, headers and flags the
    library is built from here, so that the default bench line can report them."""
    import glob
    import json
    from jetfire_amd import build

    want = build.build_id(["-DJF_DEBUG_HOOKS"])
    files = sorted(glob.glob(os.path.join(ROOT, "profiles", "*.json")))
    assert files
    for f in files:
        assert f"build {want}" in json.load(open(f)).get("lib_version", ""), f
