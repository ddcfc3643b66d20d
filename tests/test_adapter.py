"""Adapter glue: top-k width selection, dispatcher gate, pool registry (CPU), and a multi-step decode through
`mirror_kv` + `try_jetfire_decode` against the oracle (GPU)."""
import types

import numpy as np
import pytest
import torch

from oracle import jetfire_oracle as O
from tests.helpers import bf16_tensor, bf16_to_bits, bf16_to_f32


@pytest.fixture
def adapter():
    import jetfire_amd.adapter as A
    from jetfire_amd.adapter import decode_path
    A.reset_global_kv_pool_manager()
    yield A
    decode_path.reset_jetfire_decode_runtime_state()
    A.reset_global_kv_pool_manager()
    A.set_jetfire_config(scheme="SymInt3K_SymInt2V", group_size=64, topk=256, use_custom_backend=True,
                         cpu_correction=True, layer_stride=1, skip_native_kv=True)


def test_select_top_k_matches_the_reference_table(adapter):
    from jetfire_amd.adapter.decode_path import FUSED_SUPPORTED_TOP_K, _get_head_map_cpu, _select_top_k
    supported = (32, 64, 128, 256, 512, 1024)
    for req in (16, 32, 100, 256, 300, 1024, 5000):
        for n in (0, 1, 31, 32, 33, 255, 256, 257, 4096):
            assert _select_top_k(req, n, supported) == O.select_top_k(req, n, supported), (req, n)
    assert FUSED_SUPPORTED_TOP_K == supported + (2048, 4096, 8192)
    hm = _get_head_map_cpu(2, 8, 4, 5).numpy()
    assert np.array_equal(hm, O.head_map(2, 8, 4, 5))


def _meta(seq_lens, block_table, **kw):
    d = dict(seq_lens=seq_lens, block_table=block_table, use_cascade=False, max_query_len=1,
             num_actual_tokens=int(seq_lens.numel()), max_seq_len=int(seq_lens.max()) if seq_lens.numel() else 0)
    d.update(kw)
    return types.SimpleNamespace(**d)


def test_dispatcher_gate_reasons(adapter):
    from jetfire_amd.adapter.decode_path import _decode_unsupported
    pool = adapter.get_global_kv_pool_manager()
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=0.1)
    layer = types.SimpleNamespace(layer_name="model.layers.0.attn", num_heads=8, num_kv_heads=2, head_size=128)
    q = torch.zeros(2, 8 * 128)
    meta = _meta(torch.tensor([5, 7], dtype=torch.int32), torch.zeros(2, 1, dtype=torch.int64))
    gate = lambda **kw: _decode_unsupported(**{**dict(impl=impl, layer=layer, query=q.view(2, 8, 128), attn_metadata=meta), **kw})
    assert gate() == "layer_config_missing"
    pool.ensure_layer_config_from_layer(layer.layer_name, layer)
    assert pool.get_layer_config(layer.layer_name) == adapter.JetFireLayerConfig(8, 2, 128)
    assert gate() is None
    assert gate(attn_metadata=None) == "profiling_run"
    assert gate(impl=types.SimpleNamespace(attn_type=types.SimpleNamespace(name="ENCODER"))) == "attn_type"
    assert gate(attn_metadata=_meta(meta.seq_lens, meta.block_table, use_cascade=True)) == "cascade"
    assert gate(attn_metadata=_meta(meta.seq_lens, meta.block_table, max_query_len=4)) == "prefill_or_multi_query"
    assert gate(attn_metadata=_meta(meta.seq_lens, meta.block_table, num_actual_tokens=3)) == "batch_mismatch"
    assert gate(query=q.view(2, 8, 128)[:1]) == "empty_query"
    assert gate(layer=types.SimpleNamespace()) == "layer_name_missing"
    assert gate(query=torch.zeros(2, 8, 64)) == "head_dim_mismatch"
    # a miss is counted under its reason and the entry returns None
    out = torch.zeros(2, 8, 128)
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q.view(2, 8, 128), attn_metadata=meta, output=out) is None
    assert pool.get_stats()["decode_fallbacks"] == {"store_missing": 1} and pool.decode_attempts == 1


def test_graph_capture_batch_sizes_and_miss_message(adapter, monkeypatch):
    """`decode_path.py:668-706`: all sizes by default, the listed ones plus the maximum otherwise; a malformed
    list and a miss during capture raise with the fields callers parse."""
    from jetfire_amd.adapter.decode_path import _graph_context_batch_sizes, _raise_graph_decode_miss
    monkeypatch.delenv("JETFIRE_GRAPH_CAPTURE_SIZES", raising=False)
    assert _graph_context_batch_sizes(0) == [] and _graph_context_batch_sizes(-3) == []
    assert _graph_context_batch_sizes(4) == [1, 2, 3, 4]
    monkeypatch.setenv("JETFIRE_GRAPH_CAPTURE_SIZES", " 8; 2,2 ,, 64, 0 ,-1")
    assert _graph_context_batch_sizes(16) == [2, 8, 16]
    monkeypatch.setenv("JETFIRE_GRAPH_CAPTURE_SIZES", "1,two")
    with pytest.raises(RuntimeError, match="comma-separated list of integers"):
        _graph_context_batch_sizes(4)
    with pytest.raises(RuntimeError, match=r"reason=store_missing layer=model\.layers\.3"):
        _raise_graph_decode_miss("store_missing", layer_name="model.layers.3")


def test_handoff_contexts_belong_to_their_store(adapter, monkeypatch):
    """The cached hand-off contexts live on the store object: resetting the pool closes them, and a new store
    (even one that reuses the old one's id) gets contexts that read ITS shadow."""
    from jetfire_amd.adapter import decode_path
    made, closed = [], []

    class FakeHandoff:
        def __init__(self, B, H_q, H_kv, K, k_shadow, v_shadow, scale):
            self.k_ptr = k_shadow.data_ptr()
            self.failed = False
            made.append(self)

        def set_output_sanitize(self, on):
            self.sanitize = bool(on)

        def check_status(self):
            if self.failed:
                raise RuntimeError("handoff: the device-side wait for the CPU correction ran into its limit")

        def close(self):
            closed.append(self)

    monkeypatch.setattr(decode_path.ops, "CpuTopkHandoff", FakeHandoff)
    pool = adapter.get_global_kv_pool_manager()
    name = "model.layers.0.attn"
    pool.register_layer_config(name, num_query_heads=8, num_kv_heads=2, head_dim=128)
    pool.register_layer_layout(name, num_blocks=4, block_size=16)
    store = pool.ensure_layer_store(name, device="cpu")
    h1 = decode_path._handoff_for(store, 2, 8, 2, 32, 0.1, stream_mode=True)
    assert decode_path._handoff_for(store, 2, 8, 2, 32, 0.1, stream_mode=True) is h1
    assert decode_path._handoff_for(store, 2, 8, 2, 32, 0.1, stream_mode=False) is not h1
    assert h1.k_ptr == store.k_shadow.data_ptr() and len(made) == 2
    assert h1.sanitize and not hasattr(made[1], "sanitize")      # the graph-mode guard is set on stream-mode contexts only
    decode_path.check_decode_handoffs()
    h1.failed = True
    with pytest.raises(RuntimeError, match="ran into its limit"):
        decode_path.check_decode_handoffs()
    with pytest.raises(RuntimeError, match="ran into its limit"):
        pool.flush_pending_writes()
    h1.failed = False
    pool.reset_runtime_state()                       # drops the stores: their contexts are closed first
    assert len(closed) == 2 and not pool.layer_stores
    del store
    new_store = pool.ensure_layer_store(name, device="cpu")
    h2 = decode_path._handoff_for(new_store, 2, 8, 2, 32, 0.1, stream_mode=True)
    assert h2 is not h1 and h2.k_ptr == new_store.k_shadow.data_ptr()
    adapter.reset_global_kv_pool_manager()
    assert len(closed) == 3


def test_pool_registry_and_store_geometry(adapter):
    adapter.set_jetfire_config(scheme="SymInt4K_SymInt4V", group_size=128, layer_stride=2)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    assert (pool.config.k_nbits, pool.config.v_nbits, pool.config.group_size) == (4, 4, 128)
    for i in range(3):
        name = f"model.layers.{i}.attn"
        pool.register_layer_config(name, num_query_heads=8, num_kv_heads=2, head_dim=128)
        pool.register_layer_layout(name, num_blocks=6, block_size=16)
    assert pool.ensure_all_layer_stores(device="cpu") == 2          # layer_stride 2: layers 0 and 2
    store = pool.get_layer_store("model.layers.0.attn")
    assert pool.get_layer_store("model.layers.1.attn") is None
    assert store.k_data.shape == (2, 96, 64) and store.v_scales.shape == (2, 96, 1) and store.k_shadow.shape == (2, 96, 128)
    assert store.scheme == "k4v4" and store.num_slots == 96
    row = torch.tensor([4, 1, 3], dtype=torch.int64)
    slots = store.sequence_slots(row, 20)
    assert slots.tolist() == list(range(64, 80)) + [16, 17, 18, 19]
    assert torch.equal(store.sequence_slots_fast(row, 20), slots)
    assert not store.has_sequence(row, 20) and not store.fast_has_sequence(1)
    with pytest.raises(ValueError):
        store.sequence_slots(row, 0)
    with pytest.raises(ValueError):
        store.sequence_slots(torch.tensor([0, -1]), 20)
    asym = adapter.JetFireInt4CacheStore(num_kv_heads=2, head_dim=128, group_size=64, num_blocks=1, block_size=16,
                                         device="cpu", k_nbits=2, v_nbits=2, k_asymmetric=True, v_asymmetric=False)
    assert asym.k_zp.shape == asym.k_scales.shape == (2, 16, 2) and asym.scheme == "a2v2"    # INT2 keys with zero-points
    for kw in (dict(k_nbits=3, v_nbits=2, k_asymmetric=True), dict(k_nbits=2, v_nbits=2, v_asymmetric=True)):
        with pytest.raises(NotImplementedError):
            adapter.JetFireInt4CacheStore(num_kv_heads=2, head_dim=128, group_size=64, num_blocks=1, block_size=16,
                                          device="cpu", **kw)
    pool.mirror_kv("model.layers.1.attn", torch.zeros(1, 2, 128), torch.zeros(1, 2, 128), torch.tensor([0]))
    assert pool.skipped_layers == 1                                  # stride-skipped layer


@pytest.mark.gpu
@pytest.mark.parametrize("scheme_name,scheme,gs,kb,vb", [
    ("SymInt3K_SymInt2V", "k3v2", 64, 3, 2), ("SymInt4K_SymInt4V", "k4v4", 128, 4, 4),      # fused kernels
    # the other pairs: fused where the group size allows (an INT4 side needs group 128), else Stage A and Stage B as
    # separate kernels chosen by bit width
    ("SymInt2K_SymInt2V", "k2v2", 128, 2, 2), ("SymInt2K_SymInt3V", "k2v3", 128, 2, 3), ("SymInt2K_SymInt4V", "k2v4", 128, 2, 4),
    ("SymInt3K_SymInt3V", "k3v3", 64, 3, 3), ("SymInt3K_SymInt4V", "k3v4", 128, 3, 4),
    ("SymInt4K_SymInt2V", "k4v2", 128, 4, 2), ("SymInt4K_SymInt3V", "k4v3", 64, 4, 3),
    # asymmetric INT2 keys (zero-point per group)
    ("AsymInt2K4Level_SymInt2V", "k2v2", 128, 2, 2), ("AsymInt2K_SymInt4V", "k2v4", 64, 2, 4),
    ("AsymInt2K4Level_SymInt3V", "k2v3", 64, 2, 3), ("AsymInt2K4Level_SymInt4V", "k2v4", 128, 2, 4)])
def test_prefill_then_decode_steps_match_the_oracle(adapter, scheme_name, scheme, gs, kb, vb):
    B, Hq, Hkv, D, bs = 3, 8, 2, 128, 16
    lens0 = [300, 37, 512]
    steps = 3
    adapter.set_jetfire_config(scheme=scheme_name, group_size=gs, topk=64, layer_stride=1, cpu_attn_threads=4)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    name = "model.layers.0.self_attn.attn"
    layer = types.SimpleNamespace(layer_name=name, num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=D ** -0.5)
    rng = np.random.default_rng(5)
    per_seq = (max(lens0) + steps + bs - 1) // bs
    nblk = B * per_seq + 2
    bt = rng.permutation(nblk)[:B * per_seq].reshape(B, per_seq).astype(np.int64)
    pool.ensure_layer_config_from_layer(name, layer)
    pool.register_layer_layout(name, num_blocks=nblk, block_size=bs)
    bt_dev = torch.from_numpy(bt).cuda()

    def slot_of(b, pos):
        return int(bt[b, pos // bs]) * bs + pos % bs

    def new_kv(n):
        k = O.bf16_round(rng.standard_normal((n, Hkv, D)).astype(np.float32))
        k[..., [3, 40, 77, 101]] *= 8
        return O.bf16_round(k), O.bf16_round(rng.standard_normal((n, Hkv, D)).astype(np.float32))

    # prefill: every sequence's tokens in one call, plus two padding tokens (slot -1) that must be ignored
    toks = [(b, p) for b in range(B) for p in range(lens0[b])]
    k_np, v_np = new_kv(len(toks) + 2)
    slot_map = np.array([slot_of(b, p) for b, p in toks] + [-1, -1], dtype=np.int64)
    pool.mirror_kv(name, bf16_tensor(k_np).cuda(), bf16_tensor(v_np).cuda(), torch.from_numpy(slot_map).cuda())
    store = pool.get_layer_store(name)
    Kfull = np.zeros((Hkv, nblk * bs, D), np.float32)
    Vfull = np.zeros_like(Kfull)
    Kfull[:, slot_map[:-2]] = k_np[:-2].transpose(1, 0, 2)
    Vfull[:, slot_map[:-2]] = v_np[:-2].transpose(1, 0, 2)
    lens = list(lens0)
    for step in range(steps):
        # append one token per sequence, then decode
        k_np, v_np = new_kv(B)
        slot_map = np.array([slot_of(b, lens[b]) for b in range(B)], dtype=np.int64)
        pool.mirror_kv(name, bf16_tensor(k_np).cuda(), bf16_tensor(v_np).cuda(), torch.from_numpy(slot_map).cuda())
        Kfull[:, slot_map] = k_np.transpose(1, 0, 2)
        Vfull[:, slot_map] = v_np.transpose(1, 0, 2)
        lens = [n + 1 for n in lens]
        q_np = O.bf16_round((rng.standard_normal((B, Hq, D)) / np.sqrt(D)).astype(np.float32))
        seq_lens = torch.tensor(lens, dtype=torch.int32, device="cuda")
        meta = _meta(seq_lens, bt_dev)
        out = torch.zeros(B + 1, Hq * D, dtype=torch.bfloat16, device="cuda")          # one spare row, as vLLM pads
        got = adapter.try_jetfire_decode(impl=impl, layer=layer, query=bf16_tensor(q_np).cuda(), attn_metadata=meta, output=out)
        assert got is out
        torch.cuda.synchronize()
        # the cache holds exactly what the oracle quantiser packs, the shadow the bf16 rows
        filled = store.slot_filled.cpu().numpy()
        asym = scheme_name.startswith("Asym")
        if asym:
            ref_kd, ref_ks, ref_kz = O.quantize_and_pack_asym(Kfull, gs, kb)
            assert np.array_equal(bf16_to_bits(store.k_zp)[:, filled], ref_kz[:, filled])
        else:
            ref_kd, ref_ks = O.quantize_and_pack(Kfull, gs, kb)
            ref_kz = None
        ref_vd, ref_vs = O.quantize_and_pack(Vfull, gs, vb)
        assert np.array_equal(store.k_data.cpu().numpy()[:, filled], ref_kd[:, filled])
        assert np.array_equal(bf16_to_bits(store.k_scales)[:, filled], ref_ks[:, filled])
        assert np.array_equal(store.v_data.cpu().numpy()[:, filled], ref_vd[:, filled])
        assert np.array_equal(bf16_to_f32(store.k_shadow)[:, filled], Kfull[:, filled])
        r = O.decode_reference(q_np, ref_kd, ref_ks, ref_vd, ref_vs, bt, np.array(lens, np.int32), max(lens), Hq, Hkv, bs,
                               D ** -0.5, 64, scheme, Kfull, Vfull, group_size=gs, k_zp_bits=ref_kz)
        res = bf16_to_f32(out[:B]).reshape(B, Hq, D)
        np.testing.assert_allclose(res, r["out"], atol=6e-3, rtol=1.5e-2)                # validate_runtime.py:195
        err = np.abs(res - r["out"])
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        assert float(out[B].float().abs().sum()) == 0.0
    stats = pool.get_stats()
    assert stats["decode_hits"] == steps and stats["decode_fallbacks"] == {}
    assert stats["written_slots"] == sum(lens0) + 2 + steps * B
    # a sequence whose rows were never written is reported, not computed
    bad = _meta(torch.tensor([lens[0] + 5, lens[1], lens[2]], dtype=torch.int32, device="cuda"), bt_dev)
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=torch.zeros(B, Hq, D, dtype=torch.bfloat16, device="cuda"),
                                      attn_metadata=bad, output=out) is None
    assert pool.get_stats()["decode_fallbacks"] == {"store_incomplete": 1}


# ----------------------------------------------------------------------------- shadow mirror (GPU)
def _bits(t):
    return t.contiguous().view(torch.int16)


@pytest.mark.gpu
@pytest.mark.parametrize("misalign", [0, 2])
def test_shadow_write_matches_a_host_scatter(misalign):
    """`ops.shadow_write` against the reference's serial mirror (permute + `index_copy_`, cache_store.py:744-759)
    on strided token views (slices of one fused qkv activation), padding slots and a slot outside the shadow."""
    from jetfire_amd import ops
    T, Hq, Hkv, D, num_slots = 1000, 8, 4, 128, 2048
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn(T, (Hq + 2 * Hkv) * D + 8, generator=g).to(torch.bfloat16)
    qkv_dev = qkv.cuda()
    lo = Hq * D + misalign                                  # misalign = 2 elements: rows only 4-byte aligned
    key = qkv_dev[:, lo:lo + Hkv * D].view(T, Hkv, D)
    value = qkv_dev[:, lo + Hkv * D:lo + 2 * Hkv * D].view(T, Hkv, D)
    slots = torch.randperm(num_slots, generator=g)[:T].to(torch.int64)
    slots[::37] = -1
    slots[5] = num_slots + 3                                # never stored
    k_shadow = torch.zeros(Hkv, num_slots, D, dtype=torch.bfloat16, pin_memory=True)
    v_shadow = torch.zeros(Hkv, num_slots, D, dtype=torch.bfloat16, pin_memory=True)
    ops.shadow_write(key, value, slots.cuda(), k_shadow, v_shadow)
    torch.cuda.synchronize()
    keep = (slots >= 0) & (slots < num_slots)
    want_k = torch.zeros(Hkv, num_slots, D, dtype=torch.bfloat16)
    want_v = torch.zeros_like(want_k)
    want_k.index_copy_(1, slots[keep], qkv[:, lo:lo + Hkv * D].reshape(T, Hkv, D).permute(1, 0, 2)[:, keep].contiguous())
    want_v.index_copy_(1, slots[keep], qkv[:, lo + Hkv * D:lo + 2 * Hkv * D].reshape(T, Hkv, D).permute(1, 0, 2)[:, keep].contiguous())
    assert torch.equal(_bits(k_shadow), _bits(want_k))
    assert torch.equal(_bits(v_shadow), _bits(want_v))


@pytest.mark.gpu
def test_shadow_write_rejects_pageable_memory_and_bad_shapes():
    from jetfire_amd import ops
    key = torch.zeros(4, 2, 128, dtype=torch.bfloat16, device="cuda")
    slots = torch.arange(4, device="cuda")
    pageable = torch.zeros(2, 64, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="pinned|not known"):
        ops.shadow_write(key, key, slots, pageable, pageable)
    pinned = torch.zeros(3, 64, 128, dtype=torch.bfloat16, pin_memory=True)
    with pytest.raises(RuntimeError, match="shadow must be"):
        ops.shadow_write(key, key, slots, pinned, pinned)          # kv-head count differs
    ok = torch.zeros(2, 64, 128, dtype=torch.bfloat16, pin_memory=True)
    with pytest.raises(RuntimeError, match="slots"):
        ops.shadow_write(key, key, slots[:3], ok, ok)
    ops.shadow_write(key[:0], key[:0], slots[:0], ok, ok)          # empty append is a no-op
    torch.cuda.synchronize()
    assert float(ok.float().abs().sum()) == 0.0


@pytest.mark.gpu
def test_prefill_chunks_mirror_off_stream_until_flush():
    """Chunks of >= JETFIRE_PIPELINE_MIN_TOKENS tokens go to the side stream and stay pending until
    `flush_pending_writes`; afterwards the shadow holds every chunk, the later write of a slot winning."""
    from jetfire_amd.adapter.cache_store import JetFireInt4CacheStore
    Hkv, D, nblk, bs = 4, 128, 512, 16
    store = JetFireInt4CacheStore(num_kv_heads=Hkv, head_dim=D, group_size=64, num_blocks=nblk, block_size=bs,
                                  device="cuda", k_nbits=3, v_nbits=2)
    g = torch.Generator().manual_seed(3)
    want_k = torch.zeros(Hkv, nblk * bs, D, dtype=torch.bfloat16)
    want_v = torch.zeros_like(want_k)
    perm = torch.randperm(nblk * bs, generator=g)
    chunks = [(0, 4096), (4096, 6144), (6144, 6200), (100, 300)]            # the last one rewrites slots of the first
    for i, (a, b) in enumerate(chunks):
        k = torch.randn(b - a, Hkv, D, generator=g).to(torch.bfloat16)
        v = torch.randn(b - a, Hkv, D, generator=g).to(torch.bfloat16)
        slots = perm[a:b].clone()
        assert store.write_slots(key=k.cuda(), value=v.cuda(), slot_mapping=slots.cuda()) == b - a
        want_k.index_copy_(1, slots, k.permute(1, 0, 2).contiguous())
        want_v.index_copy_(1, slots, v.permute(1, 0, 2).contiguous())
    assert len(store._pending_mirrors) == 3                                  # the 56-token chunk stayed on the stream
    store.flush_pending_writes()
    torch.cuda.current_stream().synchronize()                                # the small chunk ran on this stream
    assert store._pending_mirrors == []
    assert torch.equal(_bits(store.k_shadow), _bits(want_k))
    assert torch.equal(_bits(store.v_shadow), _bits(want_v))
    filled = torch.zeros(nblk * bs, dtype=torch.bool)
    filled[perm[:6200]] = True
    assert torch.equal(store.slot_filled.cpu(), filled)
    assert store.written_count == sum(b - a for a, b in chunks)


@pytest.mark.gpu
def test_decode_append_replays_from_a_hip_graph():
    """`write_slots_graph` (cache_store.py:531-642) captured once and replayed with new tokens and slots in the
    same static buffers: every replay lands in the INT cache and in the shadow; eager work in between."""
    from jetfire_amd.adapter.cache_store import JetFireInt4CacheStore
    Hkv, D, nblk, bs, Bmax = 2, 128, 8, 16, 4
    store = JetFireInt4CacheStore(num_kv_heads=Hkv, head_dim=D, group_size=128, num_blocks=nblk, block_size=bs,
                                  device="cuda", k_nbits=4, v_nbits=4)
    eager = JetFireInt4CacheStore(num_kv_heads=Hkv, head_dim=D, group_size=128, num_blocks=nblk, block_size=bs,
                                  device="cuda", k_nbits=4, v_nbits=4)
    key = torch.zeros(Bmax, Hkv, D, dtype=torch.bfloat16, device="cuda")
    value = torch.zeros_like(key)
    slots = torch.full((Bmax,), -1, dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="max_batch_size"):
        store.write_slots_graph(key=key, value=value, slot_mapping=slots, max_batch_size=2)
    store.warmup_graph_append(Bmax)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        store.write_slots_graph(key=key, value=value, slot_mapping=slots, max_batch_size=Bmax)   # warm-up, all padding
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        store.write_slots_graph(key=key, value=value, slot_mapping=slots, max_batch_size=Bmax)
    g = torch.Generator().manual_seed(9)
    for step in range(4):
        k = torch.randn(Bmax, Hkv, D, generator=g).to(torch.bfloat16)
        v = torch.randn(Bmax, Hkv, D, generator=g).to(torch.bfloat16)
        s = torch.tensor([step, 16 + step, -1 if step % 2 else 40 + step, 100 + step], dtype=torch.int64)
        key.copy_(k.cuda()); value.copy_(v.cuda()); slots.copy_(s.cuda())
        graph.replay()
        eager.write_slots(key=k.cuda(), value=v.cuda(), slot_mapping=s.cuda())
        torch.cuda.synchronize()
        for name in ("k_data", "k_scales", "v_data", "v_scales"):
            a, b = getattr(store, name), getattr(eager, name)
            assert torch.equal(a.view(torch.uint8) if a.dtype == torch.uint8 else _bits(a),
                               b.view(torch.uint8) if b.dtype == torch.uint8 else _bits(b)), (step, name)
        assert torch.equal(_bits(store.k_shadow), _bits(eager.k_shadow)), step
        assert torch.equal(_bits(store.v_shadow), _bits(eager.v_shadow)), step
        keep = s >= 0
        assert torch.equal(_bits(store.k_shadow[:, s[keep]]), _bits(k.permute(1, 0, 2)[:, keep].contiguous())), step


@pytest.mark.gpu
def test_graph_mode_decode_step_replays_against_the_oracle(adapter, monkeypatch):
    """JETFIRE_DECODE_GRAPH=1: two layers' append + decode captured once into a HIP graph (quantise-on-write,
    shadow mirror kernel, fused scan, merge, publish, device-side wait, blend) and replayed for three decode
    steps with new tokens, slots, lengths and queries in the same buffers; every step is checked against the
    oracle, and a miss during capture raises."""
    monkeypatch.setenv("JETFIRE_DECODE_GRAPH", "1")
    B, Hq, Hkv, D, bs, K, max_S = 2, 8, 2, 128, 16, 32, 160
    gs, kb, vb, scheme = 64, 3, 2, "k3v2"
    lens0 = [100, 70]
    adapter.set_jetfire_config(scheme="SymInt3K_SymInt2V", group_size=gs, topk=K, layer_stride=1, cpu_attn_threads=2,
                               max_batch_size=B)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    names = [f"model.layers.{i}.self_attn.attn" for i in range(2)]
    layers = [types.SimpleNamespace(layer_name=n, num_heads=Hq, num_kv_heads=Hkv, head_size=D) for n in names]
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=D ** -0.5)
    rng = np.random.default_rng(21)
    per_seq = max_S // bs
    nblk = B * per_seq + 1
    bt = rng.permutation(nblk)[:B * per_seq].reshape(B, per_seq).astype(np.int64)
    bt_dev = torch.from_numpy(bt).cuda()

    def slot_of(b, pos):
        return int(bt[b, pos // bs]) * bs + pos % bs

    def new_kv(n):
        k = O.bf16_round(rng.standard_normal((n, Hkv, D)).astype(np.float32))
        k[..., [3, 40, 77, 101]] *= 8
        return O.bf16_round(k), O.bf16_round(rng.standard_normal((n, Hkv, D)).astype(np.float32))

    Kfull = [np.zeros((Hkv, nblk * bs, D), np.float32) for _ in names]
    Vfull = [np.zeros((Hkv, nblk * bs, D), np.float32) for _ in names]
    toks = [(b, p) for b in range(B) for p in range(lens0[b])]
    slot_map = np.array([slot_of(b, p) for b, p in toks], dtype=np.int64)
    for li, (name, layer) in enumerate(zip(names, layers)):
        pool.ensure_layer_config_from_layer(name, layer)
        pool.register_layer_layout(name, num_blocks=nblk, block_size=bs)
        k_np, v_np = new_kv(len(toks))
        pool.mirror_kv(name, bf16_tensor(k_np).cuda(), bf16_tensor(v_np).cuda(), torch.from_numpy(slot_map).cuda())
        Kfull[li][:, slot_map] = k_np.transpose(1, 0, 2)
        Vfull[li][:, slot_map] = v_np.transpose(1, 0, 2)
    pool.flush_pending_writes()

    # static buffers of the captured step
    key_buf = [torch.zeros(B, Hkv, D, dtype=torch.bfloat16, device="cuda") for _ in names]
    val_buf = [torch.zeros(B, Hkv, D, dtype=torch.bfloat16, device="cuda") for _ in names]
    q_buf = [torch.zeros(B, Hq, D, dtype=torch.bfloat16, device="cuda") for _ in names]
    out_buf = [torch.zeros(B, Hq * D, dtype=torch.bfloat16, device="cuda") for _ in names]
    slot_buf = torch.full((B,), -1, dtype=torch.int64, device="cuda")
    seq_lens = torch.tensor(lens0, dtype=torch.int32, device="cuda")
    meta = _meta(seq_lens, bt_dev, max_seq_len=max_S)

    def step():
        for li, (name, layer) in enumerate(zip(names, layers)):
            pool.mirror_kv(name, key_buf[li], val_buf[li], slot_buf)
            got = adapter.try_jetfire_decode(impl=impl, layer=layer, query=q_buf[li], attn_metadata=meta, output=out_buf[li])
            assert got is out_buf[li]

    # a capture without the pre-created contexts must raise, not record a fall-back
    probe = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="submit_context_missing"):
        with torch.cuda.graph(probe):
            step()
    del probe
    info = adapter.warmup_graph_decode_submit_contexts(max_batch_size=B)
    assert info["contexts_created"] == 2 * B and info["top_k"] == [32]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                     # warm-up: all-padding append, decode of the prefill
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()

    lens = list(lens0)
    for it in range(3):
        sm = np.array([slot_of(b, lens[b]) for b in range(B)], dtype=np.int64)
        slot_buf.copy_(torch.from_numpy(sm).cuda())
        lens = [n + 1 for n in lens]
        seq_lens.copy_(torch.tensor(lens, dtype=torch.int32).cuda())
        q_np = []
        for li in range(len(names)):
            k_np, v_np = new_kv(B)
            key_buf[li].copy_(bf16_tensor(k_np).cuda()); val_buf[li].copy_(bf16_tensor(v_np).cuda())
            Kfull[li][:, sm] = k_np.transpose(1, 0, 2)
            Vfull[li][:, sm] = v_np.transpose(1, 0, 2)
            q_np.append(O.bf16_round((rng.standard_normal((B, Hq, D)) / np.sqrt(D)).astype(np.float32)))
            q_buf[li].copy_(bf16_tensor(q_np[li]).cuda())
        graph.replay()
        torch.cuda.synchronize()
        for li, name in enumerate(names):
            store = pool.get_layer_store(name)
            assert np.array_equal(bf16_to_f32(store.k_shadow)[:, sm], Kfull[li][:, sm])
            ref_kd, ref_ks = O.quantize_and_pack(Kfull[li], gs, kb)
            ref_vd, ref_vs = O.quantize_and_pack(Vfull[li], gs, vb)
            assert np.array_equal(store.k_data.cpu().numpy()[:, sm], ref_kd[:, sm])
            r = O.decode_reference(q_np[li], ref_kd, ref_ks, ref_vd, ref_vs, bt, np.array(lens, np.int32), max(lens), Hq, Hkv,
                                   bs, D ** -0.5, K, scheme, Kfull[li], Vfull[li])
            res = bf16_to_f32(out_buf[li]).reshape(B, Hq, D)
            np.testing.assert_allclose(res, r["out"], atol=6e-3, rtol=1.5e-2, err_msg=f"step {it} layer {li}")
            err = np.abs(res - r["out"])
            assert err.max() <= 2e-2 and err.mean() <= 1e-3
    del graph


@pytest.mark.gpu
def test_graph_mode_reports_a_correction_that_never_arrives(adapter, monkeypatch):
    """Graph mode makes no host call per step, so a device-side wait that runs into its limit (here: the
    dispatcher is told to ignore the flag, limit 20 ms; every kernel ends normally) would blend zeros from then
    on without anyone noticing: `check_decode_handoffs`, the pool's flush and the next decode call all raise."""
    from jetfire_amd.adapter import decode_path
    monkeypatch.setenv("JETFIRE_DECODE_GRAPH", "1")
    B, Hq, Hkv, D, bs, K, max_S = 1, 8, 2, 128, 16, 32, 64
    adapter.set_jetfire_config(scheme="SymInt3K_SymInt2V", group_size=64, topk=K, layer_stride=1, cpu_attn_threads=2,
                               max_batch_size=B)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    name = "model.layers.0.self_attn.attn"
    layer = types.SimpleNamespace(layer_name=name, num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=D ** -0.5)
    pool.ensure_layer_config_from_layer(name, layer)
    pool.register_layer_layout(name, num_blocks=max_S // bs, block_size=bs)
    g = torch.Generator().manual_seed(5)
    n = 40
    k = torch.randn(n, Hkv, D, generator=g).to(torch.bfloat16).cuda()
    v = torch.randn(n, Hkv, D, generator=g).to(torch.bfloat16).cuda()
    pool.mirror_kv(name, k, v, torch.arange(n, dtype=torch.int64, device="cuda"))
    pool.flush_pending_writes()
    adapter.warmup_graph_decode_submit_contexts(max_batch_size=B)
    store = pool.get_layer_store(name)
    (h,) = store._jf_handoffs.values()
    meta = _meta(torch.tensor([n], dtype=torch.int32, device="cuda"),
                 torch.arange(max_S // bs, dtype=torch.int64, device="cuda").view(1, -1), max_seq_len=max_S)
    q = (torch.randn(B, Hq, D, generator=g) / D ** 0.5).to(torch.bfloat16).cuda()
    out = torch.zeros(B, Hq * D, dtype=torch.bfloat16, device="cuda")
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out) is out
    torch.cuda.synchronize()
    decode_path.check_decode_handoffs()                       # a healthy step: nothing to report
    good = out.clone()
    h.debug_pause(True)
    h.set_device_wait_limit_us(20000)
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out) is out
    torch.cuda.synchronize()
    assert not torch.equal(out, good)                         # the correction is missing from this step's output
    with pytest.raises(RuntimeError, match="limit"):
        decode_path.check_decode_handoffs()
    with pytest.raises(RuntimeError, match="limit"):
        pool.flush_pending_writes()
    with pytest.raises(RuntimeError, match="limit"):
        adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out)
    h.debug_pause(False)


@pytest.mark.gpu
@pytest.mark.parametrize("scheme_name,gs", [("SymInt3K_SymInt2V", 64), ("SymInt4K_SymInt4V", 128)])
def test_release_policy_selects_the_named_split_kernels(adapter, monkeypatch, scheme_name, gs):
    """JETFIRE_RELEASE_GRAPH_POLICY=1: the step runs the Stage A / Stage B operators the plan names (recorded by
    wrapping them), gives the fused path's result within the stage tolerances, and an experimental switch raises."""
    from jetfire_amd import ops as jops
    from jetfire_amd.adapter import release_policy
    for name in list(__import__("os").environ):
        if name.startswith("JETFIRE_"):
            monkeypatch.delenv(name)
    B, Hq, Hkv, D, bs, K, max_S = 2, 8, 2, 128, 16, 64, 256
    adapter.set_jetfire_config(scheme=scheme_name, group_size=gs, topk=K, layer_stride=1, cpu_attn_threads=2, max_batch_size=B)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    name = "model.layers.0.self_attn.attn"
    layer = types.SimpleNamespace(layer_name=name, num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=D ** -0.5)
    pool.ensure_layer_config_from_layer(name, layer)
    per_seq = max_S // bs
    pool.register_layer_layout(name, num_blocks=B * per_seq, block_size=bs)
    g = torch.Generator().manual_seed(11)
    lens = [200, 131]
    bt = torch.arange(B * per_seq, dtype=torch.int64).view(B, per_seq).cuda()
    slots = torch.cat([bt[b, p // bs].cpu() * bs + p % bs for b in range(B) for p in [torch.arange(lens[b])]]).cuda()
    n = int(slots.numel())
    pool.mirror_kv(name, torch.randn(n, Hkv, D, generator=g).to(torch.bfloat16).cuda(),
                   torch.randn(n, Hkv, D, generator=g).to(torch.bfloat16).cuda(), slots)
    pool.flush_pending_writes()
    meta = _meta(torch.tensor(lens, dtype=torch.int32, device="cuda"), bt, max_seq_len=max(lens))
    q = (torch.randn(B, Hq, D, generator=g) / D ** 0.5).to(torch.bfloat16).cuda()
    fused_out = torch.zeros(B, Hq * D, dtype=torch.bfloat16, device="cuda")
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=fused_out) is fused_out
    torch.cuda.synchronize()
    store = pool.get_layer_store(name)
    plan = release_policy.plan_release_graph(mode=scheme_name, group_size=gs, top_k=K, max_graph_batch=B)
    called = []
    for op_name in plan.operators():
        real = getattr(jops, op_name)
        monkeypatch.setattr(jops, op_name, (lambda f, nm: (lambda *a, **k: (called.append(nm), f(*a, **k))[1]))(real, op_name))
    monkeypatch.setenv("JETFIRE_RELEASE_GRAPH_POLICY", "1")
    monkeypatch.setenv("JETFIRE_RELEASE_REQUIRE_READY", "1")
    out = torch.zeros_like(fused_out)
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out) is out
    torch.cuda.synchronize()
    assert called == list(plan.operators())
    err = (out.float() - fused_out.float()).abs()
    assert float(err.max()) <= 2e-2 and float(err.mean()) <= 1e-3
    monkeypatch.setenv("JETFIRE_USE_FUSED_ATTN_TOPK", "1")
    with pytest.raises(release_policy.ReleasePolicyError, match="JETFIRE_USE_FUSED_ATTN_TOPK"):
        adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out)
    assert store.scheme is not None


@pytest.mark.gpu
def test_a_wide_correction_keeps_its_width(adapter, monkeypatch):
    """JETFIRE_TOPK=4096: the width reaches the fused step unclamped; with nearly every position corrected the output
    is the exact attention over the bf16 shadow."""
    from jetfire_amd import ops as jops
    for name in list(__import__("os").environ):
        if name.startswith("JETFIRE_"):
            monkeypatch.delenv(name)
    B, Hq, Hkv, D, bs, K = 1, 8, 2, 128, 16, 4096
    S = 4100                                       # (the four uncorrected positions keep their INT2 values)
    adapter.set_jetfire_config(scheme="SymInt3K_SymInt2V", group_size=64, topk=K, layer_stride=1, cpu_attn_threads=4)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    name = "model.layers.0.self_attn.attn"
    layer = types.SimpleNamespace(layer_name=name, num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=D ** -0.5)
    pool.ensure_layer_config_from_layer(name, layer)
    per_seq = (S + bs - 1) // bs
    pool.register_layer_layout(name, num_blocks=per_seq, block_size=bs)
    g = torch.Generator().manual_seed(3)
    bt = torch.arange(per_seq, dtype=torch.int64).view(1, per_seq).cuda()
    k = torch.randn(S, Hkv, D, generator=g).to(torch.bfloat16).cuda()
    v = torch.randn(S, Hkv, D, generator=g).to(torch.bfloat16).cuda()
    pool.mirror_kv(name, k, v, torch.arange(S, dtype=torch.int64).cuda())
    pool.flush_pending_writes()
    meta = _meta(torch.tensor([S], dtype=torch.int32, device="cuda"), bt, max_seq_len=S)
    q = (torch.randn(B, Hq, D, generator=g) / D ** 0.5).to(torch.bfloat16).cuda()
    called = []
    for op_name in ("fused_attn_topk", "int3_qk_scores_topk", "int2_softmax_v_with_pre_corr_wvs2"):
        real = getattr(jops, op_name)
        monkeypatch.setattr(jops, op_name, (lambda f, nm: (lambda *a, **kw: (called.append((nm, a, kw)), f(*a, **kw))[1]))(real, op_name))
    out = torch.zeros(B, Hq * D, dtype=torch.bfloat16, device="cuda")
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out) is out
    torch.cuda.synchronize()
    names = [c[0] for c in called]
    assert names == ["fused_attn_topk"]
    assert int(called[0][1][12]) == K                                 # the configured width reaches the fused step
    G = Hq // Hkv
    att = torch.softmax(torch.einsum("hd,shd->hs", q[0].float(), k.float().repeat_interleave(G, dim=1)) * D ** -0.5, dim=-1)
    ref = torch.einsum("hs,shd->hd", att, v.float().repeat_interleave(G, dim=1))
    err = (out.view(Hq, D).float() - ref).abs()
    assert float(err.max()) <= 2e-2 and float(err.mean()) <= 1e-3


class _NativeImpl:
    """Stand-in for the serving engine's attention implementation: records what reaches it."""

    def __init__(self):
        self.attn_type = types.SimpleNamespace(name="DECODER")
        self.scale = 128 ** -0.5
        self.native_forward = 0
        self.native_updates = 0

    def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, output_scale=None,
                output_block_scale=None):
        self.native_forward += 1
        return "native"

    def do_kv_cache_update(self, layer, key, value, kv_cache, slot_mapping):
        self.native_updates += 1


def test_backend_shim_routes_appends_and_fallbacks(adapter):
    """`jetfire_backend.py:135-209`: appends always reach the pool (and the engine's own cache only when it keeps
    one); a decode miss with no native cache raises with the recorded reasons; the profiling pass and prefill
    fall through to the engine's implementation."""
    from jetfire_amd.adapter.jetfire_backend import make_jetfire_attention_impl
    Impl = make_jetfire_attention_impl(_NativeImpl)
    impl = Impl()
    layer = types.SimpleNamespace(layer_name="model.layers.0.attn", num_heads=8, num_kv_heads=2, head_size=128)
    pool = adapter.get_global_kv_pool_manager()
    pool.register_layer_layout(layer.layer_name, num_blocks=2, block_size=16)
    k = torch.zeros(3, 2, 128, dtype=torch.bfloat16)
    seen = []
    pool.mirror_kv = lambda **kw: seen.append(sorted(kw))
    adapter.set_jetfire_config(skip_native_kv=True)
    impl.do_kv_cache_update(layer, k, k, None, torch.arange(3))
    assert seen == [["key", "layer_name", "slot_mapping", "value"]] and impl.native_updates == 0
    assert pool.get_layer_config(layer.layer_name) == adapter.JetFireLayerConfig(8, 2, 128)
    adapter.set_jetfire_config(skip_native_kv=False)
    impl.do_kv_cache_update(layer, k, k, None, torch.arange(3))
    assert len(seen) == 2 and impl.native_updates == 1
    q = torch.zeros(2, 8, 128, dtype=torch.bfloat16)
    out = torch.zeros(2, 8 * 128, dtype=torch.bfloat16)
    meta = _meta(torch.tensor([5, 7], dtype=torch.int32), torch.zeros(2, 1, dtype=torch.int64))
    assert impl.forward(layer, q, None, None, None, meta, output=out) == "native"        # store missing, native cache kept
    assert pool.decode_fallbacks.get("store_missing") == 1
    adapter.set_jetfire_config(skip_native_kv=True)
    with pytest.raises(RuntimeError, match="store_missing"):
        impl.forward(layer, q, None, None, None, meta, output=out)
    assert impl.forward(layer, q, None, None, None, None, output=out) == "native"        # profiling pass
    prefill = _meta(meta.seq_lens, meta.block_table, max_query_len=4)
    assert impl.forward(layer, q, None, None, None, prefill, output=out) == "native"     # prefill is the engine's
    assert impl.native_forward == 3


@pytest.mark.gpu
def test_backend_shim_appends_and_decodes_on_the_gpu(adapter):
    from jetfire_amd.adapter.jetfire_backend import make_jetfire_attention_impl
    B, Hq, Hkv, D, bs, K, max_S = 2, 8, 2, 128, 16, 32, 128
    adapter.set_jetfire_config(scheme="SymInt3K_SymInt2V", group_size=64, topk=K, layer_stride=1, cpu_attn_threads=2,
                               skip_native_kv=True)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    impl = make_jetfire_attention_impl(_NativeImpl)()
    layer = types.SimpleNamespace(layer_name="model.layers.0.self_attn.attn", num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    per_seq = max_S // bs
    pool.register_layer_layout(layer.layer_name, num_blocks=B * per_seq, block_size=bs)
    rng = np.random.default_rng(13)
    lens = [90, 47]
    bt = np.arange(B * per_seq, dtype=np.int64).reshape(B, per_seq)
    slots = np.concatenate([bt[b, np.arange(lens[b]) // bs] * bs + np.arange(lens[b]) % bs for b in range(B)])
    n = len(slots)
    k_np = O.bf16_round(rng.standard_normal((n, Hkv, D)).astype(np.float32))
    v_np = O.bf16_round(rng.standard_normal((n, Hkv, D)).astype(np.float32))
    impl.do_kv_cache_update(layer, bf16_tensor(k_np).cuda(), bf16_tensor(v_np).cuda(), None, torch.from_numpy(slots).cuda())
    q_np = O.bf16_round((rng.standard_normal((B, Hq, D)) / np.sqrt(D)).astype(np.float32))
    out = torch.zeros(B, Hq * D, dtype=torch.bfloat16, device="cuda")
    meta = _meta(torch.tensor(lens, dtype=torch.int32, device="cuda"), torch.from_numpy(bt).cuda(), max_seq_len=max(lens))
    got = impl.forward(layer, bf16_tensor(q_np).cuda(), None, None, None, meta, output=out)
    torch.cuda.synchronize()
    assert got is out and impl.native_forward == 0 and pool.decode_hits == 1
    Kfull = np.zeros((Hkv, B * max_S, D), np.float32)
    Vfull = np.zeros((Hkv, B * max_S, D), np.float32)
    Kfull[:, slots] = k_np.transpose(1, 0, 2)
    Vfull[:, slots] = v_np.transpose(1, 0, 2)
    kd, ks = O.quantize_and_pack(Kfull, 64, 3)
    vd, vs = O.quantize_and_pack(Vfull, 64, 2)
    r = O.decode_reference(q_np, kd, ks, vd, vs, bt, np.array(lens, np.int32), max(lens), Hq, Hkv, bs, D ** -0.5, K, "k3v2",
                           Kfull, Vfull)
    res = bf16_to_f32(out).reshape(B, Hq, D)
    np.testing.assert_allclose(res, r["out"], atol=6e-3, rtol=1.5e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("top_k,int8_tc,k_model", [(32, "1", "bf16"), (64, "0", "bf16"), (64, "1", "int8")])
def test_int4_keys_take_the_reference_scoring_model_for_the_width(adapter, monkeypatch, top_k, int8_tc, k_model):
    """INT4 keys with one scale per row are scored with the int8-quantised-query model only from top_k 64 up and
    with JETFIRE_USE_INT8_TC=1 (`jetfire_vllm/adapter/decode_path.py:2012-2022`); otherwise with the bf16 model of
    `int4_qk_scores`.  The fused path must follow: the winners equal the oracle's under that model."""
    monkeypatch.setenv("JETFIRE_USE_INT8_TC", int8_tc)
    B, Hq, Hkv, D, bs, max_S = 2, 8, 2, 128, 16, 256
    adapter.set_jetfire_config(scheme="SymInt4K_SymInt4V", group_size=128, topk=top_k, layer_stride=1, cpu_attn_threads=2)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    name = "model.layers.0.self_attn.attn"
    layer = types.SimpleNamespace(layer_name=name, num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=D ** -0.5)
    pool.ensure_layer_config_from_layer(name, layer)
    per_seq = max_S // bs
    pool.register_layer_layout(name, num_blocks=B * per_seq, block_size=bs)
    rng = np.random.default_rng(29)
    lens = [230, 117]
    bt = np.arange(B * per_seq, dtype=np.int64).reshape(B, per_seq)
    slots = np.concatenate([bt[b, np.arange(lens[b]) // bs] * bs + np.arange(lens[b]) % bs for b in range(B)])
    n = len(slots)
    k_np = O.bf16_round(rng.standard_normal((n, Hkv, D)).astype(np.float32))
    v_np = O.bf16_round(rng.standard_normal((n, Hkv, D)).astype(np.float32))
    pool.mirror_kv(name, bf16_tensor(k_np).cuda(), bf16_tensor(v_np).cuda(), torch.from_numpy(slots).cuda())
    pool.flush_pending_writes()
    q_np = O.bf16_round((rng.standard_normal((B, Hq, D)) / np.sqrt(D)).astype(np.float32))
    out = torch.zeros(B, Hq * D, dtype=torch.bfloat16, device="cuda")
    meta = _meta(torch.tensor(lens, dtype=torch.int32, device="cuda"), torch.from_numpy(bt).cuda(), max_seq_len=max(lens))
    from jetfire_amd import ops as jops
    seen = []
    real = jops.fused_attn_topk
    monkeypatch.setattr(jops, "fused_attn_topk", lambda scheme, *a, **k: (seen.append(scheme), real(scheme, *a, **k))[1])
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=bf16_tensor(q_np).cuda(), attn_metadata=meta,
                                      output=out) is out
    torch.cuda.synchronize()
    assert seen == [("b4v4" if k_model == "bf16" else "k4v4")]
    Kfull = np.zeros((Hkv, B * max_S, D), np.float32)
    Vfull = np.zeros((Hkv, B * max_S, D), np.float32)
    Kfull[:, slots] = k_np.transpose(1, 0, 2)
    Vfull[:, slots] = v_np.transpose(1, 0, 2)
    kd, ks = O.quantize_and_pack(Kfull, 128, 4)
    vd, vs = O.quantize_and_pack(Vfull, 128, 4)
    r = O.decode_reference(q_np, kd, ks, vd, vs, bt, np.array(lens, np.int32), max(lens), Hq, Hkv, bs, D ** -0.5, top_k,
                           "k4v4", Kfull, Vfull, group_size=128, k_model=k_model)
    res = bf16_to_f32(out).reshape(B, Hq, D)
    np.testing.assert_allclose(res, r["out"], atol=6e-3, rtol=1.5e-2)
    err = np.abs(res - r["out"])
    assert err.max() <= 2e-2 and err.mean() <= 1e-3


@pytest.mark.gpu
def test_release_policy_refuses_a_store_outside_the_release_modes(adapter, monkeypatch):
    """Under JETFIRE_RELEASE_GRAPH_POLICY=1 every store is planned (`decode_path.py:1857-1868`): asymmetric INT2 keys
    are outside the release modes and raise instead of running another path silently."""
    from jetfire_amd.adapter import release_policy
    for name in list(__import__("os").environ):
        if name.startswith("JETFIRE_"):
            monkeypatch.delenv(name)
    B, Hq, Hkv, D, bs, K, max_S = 1, 8, 2, 128, 16, 64, 128
    adapter.set_jetfire_config(scheme="AsymInt2K4Level_SymInt2V", group_size=64, topk=K, layer_stride=1,
                               cpu_attn_threads=2, max_batch_size=0)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    name = "model.layers.0.self_attn.attn"
    layer = types.SimpleNamespace(layer_name=name, num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=D ** -0.5)
    pool.ensure_layer_config_from_layer(name, layer)
    pool.register_layer_layout(name, num_blocks=max_S // bs, block_size=bs)
    g = torch.Generator().manual_seed(3)
    n = 100
    pool.mirror_kv(name, torch.randn(n, Hkv, D, generator=g).to(torch.bfloat16).cuda(),
                   torch.randn(n, Hkv, D, generator=g).to(torch.bfloat16).cuda(), torch.arange(n).cuda())
    pool.flush_pending_writes()
    meta = _meta(torch.tensor([n], dtype=torch.int32, device="cuda"), torch.arange(max_S // bs).view(1, -1).cuda(),
                 max_seq_len=n)
    q = torch.zeros(B, Hq, D, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(B, Hq * D, dtype=torch.bfloat16, device="cuda")
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out) is out
    monkeypatch.setenv("JETFIRE_RELEASE_GRAPH_POLICY", "1")
    with pytest.raises(release_policy.ReleasePolicyError, match="mode"):
        adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out)


@pytest.mark.gpu
def test_backend_shim_defers_a_prefill_append_until_its_attention_is_enqueued(adapter, monkeypatch):
    """JETFIRE_DEFER_PREFILL_KV_MIRROR=force (`jetfire_backend.py:32-63,196-209`): `do_kv_cache_update` parks a large
    chunk on the layer, the engine's prefill `forward` runs, then the append happens; small chunks are never parked."""
    from jetfire_amd.adapter.jetfire_backend import make_jetfire_attention_impl
    monkeypatch.setenv("JETFIRE_DEFER_PREFILL_KV_MIRROR", "force")
    B, Hq, Hkv, D, bs = 1, 8, 2, 128, 16
    adapter.set_jetfire_config(scheme="SymInt3K_SymInt2V", group_size=64, topk=32, layer_stride=1, cpu_attn_threads=2,
                               skip_native_kv=True)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    impl = make_jetfire_attention_impl(_NativeImpl)()
    layer = types.SimpleNamespace(layer_name="model.layers.0.self_attn.attn", num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    pool.register_layer_layout(layer.layer_name, num_blocks=16, block_size=bs)
    k = torch.randn(96, Hkv, D).to(torch.bfloat16).cuda()
    slots = torch.arange(96).cuda()
    impl.do_kv_cache_update(layer, k, k, None, slots)
    assert hasattr(layer, "_jetfire_deferred_kv_mirror")
    store = pool.get_layer_store(layer.layer_name)
    assert store is None or int(store.slot_filled.sum()) == 0
    prefill = _meta(torch.tensor([96], dtype=torch.int32, device="cuda"), torch.arange(16).view(1, -1).cuda(),
                    max_query_len=96)
    out = torch.zeros(96, Hq * D, dtype=torch.bfloat16, device="cuda")
    assert impl.forward(layer, torch.zeros(96, Hq, D, dtype=torch.bfloat16, device="cuda"), k, k, None, prefill,
                        output=out) == "native"
    assert not hasattr(layer, "_jetfire_deferred_kv_mirror")
    pool.flush_pending_writes()
    torch.cuda.synchronize()
    store = pool.get_layer_store(layer.layer_name)
    assert int(store.slot_filled.sum()) == 96
    small = torch.randn(4, Hkv, D).to(torch.bfloat16).cuda()
    impl.do_kv_cache_update(layer, small, small, None, torch.arange(96, 100).cuda())
    assert not hasattr(layer, "_jetfire_deferred_kv_mirror")


@pytest.mark.gpu
def test_decode_entry_reports_its_stages_under_profile_decode(adapter, monkeypatch):
    """JETFIRE_PROFILE_DECODE=1 (`decode_path.py:60-85`): every stage of the decode entry is a named profiler range
    and its wall time is accumulated under the reference's stage names; without the switch nothing is accumulated."""
    B, Hq, Hkv, D, bs, K, max_S = 1, 8, 2, 128, 16, 32, 128
    adapter.set_jetfire_config(scheme="SymInt3K_SymInt2V", group_size=64, topk=K, layer_stride=1, cpu_attn_threads=2)
    adapter.reset_global_kv_pool_manager()
    pool = adapter.get_global_kv_pool_manager()
    name = "model.layers.0.self_attn.attn"
    layer = types.SimpleNamespace(layer_name=name, num_heads=Hq, num_kv_heads=Hkv, head_size=D)
    impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=D ** -0.5)
    pool.ensure_layer_config_from_layer(name, layer)
    pool.register_layer_layout(name, num_blocks=max_S // bs, block_size=bs)
    g = torch.Generator().manual_seed(5)
    n = 100
    pool.mirror_kv(name, torch.randn(n, Hkv, D, generator=g).to(torch.bfloat16).cuda(),
                   torch.randn(n, Hkv, D, generator=g).to(torch.bfloat16).cuda(), torch.arange(n).cuda())
    pool.flush_pending_writes()
    meta = _meta(torch.tensor([n], dtype=torch.int32, device="cuda"), torch.arange(max_S // bs).view(1, -1).cuda(),
                 max_seq_len=n)
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16).cuda()
    out = torch.zeros(B, Hq * D, dtype=torch.bfloat16, device="cuda")
    adapter.jetfire_get_profile()
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out) is out
    assert adapter.jetfire_get_profile() == {}
    plain = out.clone()
    monkeypatch.setenv("JETFIRE_PROFILE_DECODE", "1")
    assert adapter.try_jetfire_decode(impl=impl, layer=layer, query=q, attn_metadata=meta, output=out) is out
    prof = adapter.jetfire_get_profile()
    assert {"D_total", "V2_00_prep", "V2_01_attn", "V2_02c_tpe_submit", "V2_04_join", "V2_05_post_corr"} <= set(prof)
    assert all(len(v) == 1 and v[0] > 0.0 for v in prof.values())
    assert prof["D_total"][0] >= prof["V2_01_attn"][0]
    assert adapter.jetfire_get_profile() == {}          # reading clears
    assert torch.equal(out, plain)                      # the ranges change nothing
