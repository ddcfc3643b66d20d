#!/usr/bin/env python3
"""Benchmark of the fused decode scan + top-k on one MI355X.

A step is one decode step of the attention path over all layers of the workload: per layer the fused
scan (packed K and V streamed once from HBM), the top-k merge kernel and the GPU-side blend, on distinct
per-layer caches that are resident in HBM before the timed region (together far larger than the caches,
so no layer is served from L2 / Infinity Cache left by the previous step).

Prints ONE JSON line (see --help for the workload choices).  `value` is packed KV bytes per second over
the whole step; `roofline` is for the dominant kernel (fused_scan_kernel), its device time measured with
HIP events recorded around every launch inside the timed region; `cpu_baseline` is the reference's
PyTorch CPU path (unpack + dequant + attention + top-k) restated in oracle/torch_cpu_path.py, timed on
this box's host cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def cpu_baseline(w, target_s: float = 10.0, budget_s: float = 25.0):
    """Time the torch CPU path on sequence 0 / layer 0 of the workload (all kv heads, full context): repeated for
    about `target_s` seconds of CPU work (at least five runs, at most `budget_s`), median per run."""
    import torch
    from oracle import torch_cpu_path as T
    S, Hkv, gs = w.S, w.H_kv, w.group
    from jetfire_amd import workloads
    kb, vb, _ = workloads.scheme_bits(w.scheme)
    lay = w.layers[0]
    # sequence 0 occupies slots [0, S) with the identity block table
    kd = lay.k_data[:, :S].cpu().unsqueeze(0)
    ks = lay.k_scales[:, :S].cpu().unsqueeze(0)
    vd = lay.v_data[:, :S].cpu().unsqueeze(0)
    vs = lay.v_scales[:, :S].cpu().unsqueeze(0)
    q = w.q[:1].cpu()
    threads = torch.get_num_threads()
    T.decode_path(q, kd, ks, vd, vs, gs, kb, vb, w.top_k)                 # warm-up
    times = []
    t_start = time.perf_counter()
    while (len(times) < 5 or time.perf_counter() - t_start < target_s) and time.perf_counter() - t_start < budget_s:
        t0 = time.perf_counter()
        T.decode_path(q, kd, ks, vd, vs, gs, kb, vb, w.top_k)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    sample_bytes = Hkv * S * (w.packed_bytes_per_layer // (w.B * w.H_kv * w.S))
    return {
        "value": round(sample_bytes / med / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"1 of {w.B} sequences x {Hkv} kv-heads x {S} positions of one layer ({sample_bytes / 1e6:.1f} MB packed), "
                  f"median of {len(times)} runs ({sum(times):.1f} s of CPU work), {med * 1e3:.1f} ms per run",
        "ms_per_layer_equiv": round(med * w.B * 1e3, 2),
    }


def cpu_baseline_c1(target_s: float = 4.0):
    """The whole of configuration C1 (B1, 32 query / 8 kv heads, 4096 positions, K4V4, top-k 64: the reference's own
    CPU-runnable case) through the torch CPU path: median seconds per layer pass."""
    import torch
    from jetfire_amd import workloads
    from oracle import torch_cpu_path as T
    w = workloads.build("c1")
    lay = w.layers[0]
    kd, ks = lay.k_data.cpu().unsqueeze(0), lay.k_scales.cpu().unsqueeze(0)
    vd, vs = lay.v_data.cpu().unsqueeze(0), lay.v_scales.cpu().unsqueeze(0)
    q = w.q.cpu()
    T.decode_path(q, kd, ks, vd, vs, w.group, 4, 4, w.top_k)
    times = []
    t_start = time.perf_counter()
    while len(times) < 5 or time.perf_counter() - t_start < target_s:
        t0 = time.perf_counter()
        T.decode_path(q, kd, ks, vd, vs, w.group, 4, 4, w.top_k)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"workload": "c1: B1 Hq32 Hkv8 S4096 k4v4 g128 top_k64, one layer, whole configuration",
            "value": round(w.packed_bytes_per_layer / med / 1e9, 4), "unit": "GB/s", "ms_per_layer": round(med * 1e3, 3),
            "runs": len(times), "cores": torch.get_num_threads()}


def _median_ms(fn, sync, n=10, warm=2):
    import time
    ts = []
    for i in range(warm + n):
        sync()
        t0 = time.perf_counter()
        fn()
        sync()
        if i >= warm:
            ts.append((time.perf_counter() - t0) * 1e3)
    ts.sort()
    return ts[len(ts) // 2]


def component_append(args):
    """A prefill chunk of --tokens tokens appended to one layer's store at the workload's geometry: the
    quantise-on-write kernels, the mirror kernel that stores the bf16 rows into the pinned host shadow, the
    store's whole `write_slots` + `flush_pending_writes`, and beside it the serial host mirror the reference
    falls back to (device-to-host copy of the permuted chunk + `index_copy_`, cache_store.py:744-759)."""
    import torch
    from jetfire_amd import ops, workloads
    from jetfire_amd.adapter.cache_store import JetFireInt4CacheStore
    _, _, Hkv, _, scheme, gs, _, _ = workloads.CONFIGS[args.workload]
    T = int(args.tokens)
    kb, vb = (3, 2) if scheme == "k3v2" else (4, 4)
    nblk = 2 * ((T + 15) // 16)
    store = JetFireInt4CacheStore(num_kv_heads=Hkv, head_dim=128, group_size=gs, num_blocks=nblk, block_size=16,
                                  device="cuda", k_nbits=kb, v_nbits=vb)
    g = torch.Generator().manual_seed(0)
    key = torch.randn(T, Hkv, 128, generator=g).to(torch.bfloat16).cuda()
    value = torch.randn(T, Hkv, 128, generator=g).to(torch.bfloat16).cuda()
    blocks = torch.randperm(nblk, generator=g)[:(T + 15) // 16]
    slots = (blocks[:, None] * 16 + torch.arange(16)[None, :]).reshape(-1)[:T].cuda()     # paged: runs of 16 slots
    sync = torch.cuda.synchronize
    quant_ms = _median_ms(lambda: store._quantise(key, value, slots), sync)
    mirror_ms = _median_ms(lambda: store._mirror(key, value, slots), sync)

    def whole():
        store.write_slots(key=key, value=value, slot_mapping=slots)
        store.flush_pending_writes()
    whole_ms = _median_ms(whole, sync)
    import time
    sync()
    t0 = time.perf_counter()
    store.write_slots(key=key, value=value, slot_mapping=slots)
    torch.cuda.current_stream().synchronize()            # what the model's stream waits for
    main_ms = (time.perf_counter() - t0) * 1e3
    store.flush_pending_writes()
    slots_cpu = slots.cpu()

    def serial_host():
        k_host = key.permute(1, 0, 2).to("cpu")
        v_host = value.permute(1, 0, 2).to("cpu")
        store.k_shadow.index_copy_(1, slots_cpu, k_host)
        store.v_shadow.index_copy_(1, slots_cpu, v_host)
    serial_ms = _median_ms(serial_host, sync, n=5, warm=1)
    bf16_bytes = 2 * T * Hkv * 256
    return {"component": "append", "workload": args.workload, "tokens": T, "H_kv": Hkv, "scheme": scheme,
            "quantise_write_ms": round(quant_ms, 4), "shadow_mirror_kernel_ms": round(mirror_ms, 3),
            "shadow_mirror_GBps_over_pcie": round(bf16_bytes / mirror_ms / 1e6, 1),
            "write_slots_plus_flush_ms": round(whole_ms, 3), "model_stream_busy_ms": round(main_ms, 3),
            "serial_host_mirror_ms": round(serial_ms, 3), "bf16_bytes_mirrored": bf16_bytes}


def component_cpu_correction(args):
    """The CPU correction alone (cpu_topk_attn.cpp:854-956) at the workload's (B, Hq, K): slots redrawn for every
    call over a shadow much larger than the last-level cache, so the gather comes from DRAM
    (the method of the reference's bench/cpu_correction_microbench.py:150-158)."""
    import time
    import torch
    from jetfire_amd import ops, workloads
    B, Hq, Hkv, S, _, _, K, _ = workloads.CONFIGS[args.workload]
    num_slots = B * S
    g = torch.Generator().manual_seed(0)
    k_shadow = torch.randn(Hkv, num_slots, 128, generator=g).to(torch.bfloat16)
    v_shadow = torch.randn(Hkv, num_slots, 128, generator=g).to(torch.bfloat16)
    q = (torch.randn(B, Hq, 128, generator=g) / 128 ** 0.5).to(torch.bfloat16)
    head_map = (torch.arange(Hq) // (Hq // Hkv))[None, :, None].expand(B, Hq, K).contiguous()
    o_new = torch.zeros(B, Hq, 128, dtype=torch.bfloat16)
    threads = args.cpu_threads
    ops.set_cpu_attn_threads(threads)
    ts = []
    for i in range(23):
        base = (torch.arange(B) * S)[:, None, None]
        slots = (torch.randint(0, S, (B, Hq, K), generator=g) + base).contiguous()
        t0 = time.perf_counter()
        ops.cpu_topk_attn(q, k_shadow, v_shadow, head_map, slots, o_new, 128 ** -0.5)
        if i >= 3:
            ts.append(time.perf_counter() - t0)
    ts.sort()
    med = ts[len(ts) // 2]
    return {"component": "cpu-correction", "workload": args.workload, "B": B, "H_q": Hq, "top_k": K, "threads": threads,
            "us_per_call": round(med * 1e6, 1), "min_us": round(ts[0] * 1e6, 1),
            "gathered_GBps": round(B * Hq * K * 512 / med / 1e9, 1), "rows_gathered": B * Hq * K * 2}


def component_pcie(args):
    """Pinned host <-> device copy latency by size (the reference's bench/pcie_transfer_microbench.py:20-42), and
    the hand-off's own transfer of the workload: one publish kernel down, one fetch kernel up."""
    import torch
    out = {"component": "pcie", "sizes": {}}
    sync = torch.cuda.synchronize
    for nbytes in (4 << 10, 32 << 10, 256 << 10, 2 << 20, 16 << 20, 128 << 20):
        host = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
        dev = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        d2h = _median_ms(lambda: host.copy_(dev, non_blocking=True), sync, n=20, warm=3)
        h2d = _median_ms(lambda: dev.copy_(host, non_blocking=True), sync, n=20, warm=3)
        out["sizes"][str(nbytes)] = {"d2h_us": round(d2h * 1e3, 1), "h2d_us": round(h2d * 1e3, 1),
                                     "d2h_GBps": round(nbytes / d2h / 1e6, 2), "h2d_GBps": round(nbytes / h2d / 1e6, 2)}
    return out


def component_split(args):
    """The split-form operators (one per reference kernel: Stage A scores + top-k, Stage B) at the workload's
    shape, a few layers, eagerly: wall time per layer, and a launch sequence for a kernel trace."""
    import torch
    from jetfire_amd import ops, workloads
    w = workloads.build(args.workload, n_layers=args.layers or 4)
    sync = torch.cuda.synchronize

    def layer(lay):
        if w.scheme == "k3v2":
            scores, idx, slots = ops.int3_qk_scores_topk(w.q, lay.k_data, lay.k_scales, w.block_table, w.seq_lens, w.S, w.H_q,
                                                         w.H_kv, 16, w.attn_scale, w.top_k)
            return ops.int2_softmax_v_with_pre_corr_wvs2(scores, lay.v_data, lay.v_scales, w.block_table, w.seq_lens, idx,
                                                         w.S, w.H_q, w.H_kv, 16, w.top_k)
        scores, idx, slots, m, iz = ops.int8tc_qk_scores_topk_stats(w.q, lay.k_data, lay.k_scales, w.block_table, w.seq_lens,
                                                                    w.S, w.H_q, w.H_kv, 16, w.attn_scale, w.top_k)
        fn = ops.int8tc_softmax_v_with_pre_corr_reg_stats if w.B > 1 else None
        if fn is not None:
            return fn(scores, m, iz, lay.v_data, lay.v_scales, w.block_table, w.seq_lens, idx, w.S, w.H_q, w.H_kv, 16, w.top_k)
        return ops.int4_softmax_v_with_pre_corr_wvs2_scores(scores, lay.v_data, lay.v_scales, w.block_table, w.seq_lens, idx,
                                                            w.S, w.H_q, w.H_kv, 16, w.top_k)

    def step():
        for lay in w.layers:
            layer(lay)
    ms = _median_ms(step, sync, n=5, warm=2)
    return {"component": "split", "workload": args.workload, "layers": len(w.layers),
            "us_per_layer": round(ms * 1e3 / len(w.layers), 1),
            "packed_GBps": round(w.packed_bytes_per_layer * len(w.layers) / ms / 1e6, 1)}


def measure_gpu_path(name: str, steps: int, warmup: int, lib):
    """One more workload inside the same run: the GPU path (scan + merge + blend per layer, replayed from a HIP
    graph) timed like the main one, the scan kernel timed with HIP events in a separate eager pass."""
    import torch
    from jetfire_amd import _lib, ops, workloads
    w = workloads.build(name)
    n_layers = len(w.layers)
    o_new = torch.zeros(w.B, w.H_q, 128, dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(o_new)

    def step():
        for lay in w.layers:
            ops.fused_attn_topk(w.scheme, w.q, lay.k_data, lay.k_scales, lay.v_data, lay.v_scales, w.block_table,
                                w.seq_lens, w.S, w.H_q, w.H_kv, 16, w.top_k, w.attn_scale, blend=(o_new, out), k_zp=lay.k_zp)
    for _ in range(max(1, warmup)):
        step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
    torch.cuda.current_stream().wait_stream(s)
    with torch.cuda.graph(graph, stream=s):
        step()
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    total_ms, launches = ctypes.c_double(0.0), ctypes.c_int(0)
    _lib.check(_lib.debug_hook("jf_profile_scan_begin")(n_layers * 3))
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    _lib.check(_lib.debug_hook("jf_profile_scan_end")(ctypes.byref(total_ms), ctypes.byref(launches)))
    scan_us = total_ms.value / max(1, launches.value) * 1e3
    achieved = w.packed_bytes_per_layer / (scan_us * 1e-6) / 1e9
    rec = {"workload": f"{name}: B{w.B} Hq{w.H_q} Hkv{w.H_kv} D128 S{w.S} {w.scheme} g{w.group} top_k{w.top_k} x{n_layers} layers",
           "packed_bytes_per_layer": w.packed_bytes_per_layer, "steps": steps, "ms_per_step": round(ms_per_step, 4),
           "us_per_layer": round(ms_per_step * 1e3 / n_layers, 2),
           "value": round(w.packed_bytes_per_layer * n_layers / (ms_per_step * 1e-3) / 1e9, 2), "unit": "GB/s",
           "roofline": {"bound": "hbm", "kernel": "fused_scan_kernel", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS,
                        "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "kernel_us": round(scan_us, 2),
                        "launches_timed": launches.value, **profile_counters(w.scheme, name)}}
    del graph, w
    torch.cuda.empty_cache()
    return rec


def measure_e2e(name: str, steps: int, cpu_threads: int):
    """Configuration C4 / C5 end to end inside the default run: per layer the fused scan + merge, the publish kernel
    (slots + q to pinned memory), the CPU correction on the host's worker pool and the device-side wait that fetches
    o_new and blends, the whole step replayed from ONE HIP graph whose first node is the pool's doorbell.  Wall time
    per layer, and what the device-side waits themselves measured (their waiting time, 100 MHz clock)."""
    import torch
    from jetfire_amd import _lib, ops, workloads
    w = workloads.build(name, keep_shadow=4)
    n_layers = len(w.layers)
    ops.set_cpu_attn_threads(cpu_threads)
    ctxs = [ops.CpuTopkHandoff(w.B, w.H_q, w.H_kv, w.top_k, ksh, vsh, w.attn_scale) for ksh, vsh in w.shadows]
    out = torch.empty(w.B, w.H_q, 128, dtype=torch.bfloat16, device="cuda")
    cap = 4096
    log = torch.zeros(cap + 1, dtype=torch.int64, device="cuda")
    _lib.check(_lib.debug_hook("jf_debug_wait_log")(log.data_ptr(), cap))

    def step():
        ops.pool_doorbell()
        for li, lay in enumerate(w.layers):
            o_hat, slots, o_old, W, _ = ops.fused_attn_topk(w.scheme, w.q, lay.k_data, lay.k_scales, lay.v_data, lay.v_scales,
                                                            w.block_table, w.seq_lens, w.S, w.H_q, w.H_kv, 16, w.top_k,
                                                            w.attn_scale)
            h = ctxs[li % len(ctxs)]
            h.stream_submit(w.q, slots)
            h.stream_wait_blend(o_hat, o_old, W, out)
    try:
        step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            step()
        torch.cuda.current_stream().wait_stream(s)
        with torch.cuda.graph(graph, stream=s):
            step()
        graph.replay()
        torch.cuda.synchronize()
        time.sleep(0.02)                      # the pool goes to sleep, as between two decode steps of a served model
        log.zero_()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        for h in ctxs:
            h.check_status()
        rec_n = int(log[0].item())
        waits = (log[1:1 + min(rec_n, cap)].cpu().numpy() / 100.0)      # microseconds
        waits.sort()
        us_layer = elapsed / steps / n_layers * 1e6
        return {"workload": f"{name}: B{w.B} Hq{w.H_q} Hkv{w.H_kv} D128 S{w.S} {w.scheme} g{w.group} top_k{w.top_k} x{n_layers} "
                            "layers, scan + merge + pinned hand-off + CPU correction + device-side wait and blend, one HIP "
                            "graph per step with the pool's doorbell at its head",
                "steps": steps, "us_per_layer": round(us_layer, 2), "ms_per_step": round(elapsed / steps * 1e3, 3),
                "cpu_threads": ops.get_cpu_attn_threads(),
                "value": round(w.packed_bytes_per_layer / us_layer / 1e3, 2), "unit": "GB/s",
                "wait_kernel_us": {"launches": rec_n, "median": round(float(waits[len(waits) // 2]), 1) if len(waits) else None,
                                   "p99": round(float(waits[int(len(waits) * 0.99)]), 1) if len(waits) else None,
                                   "max": round(float(waits[-1]), 1) if len(waits) else None,
                                   "clock": "device-side, 100 MHz"}}
    finally:
        _lib.check(_lib.debug_hook("jf_debug_wait_log")(None, 0))
        torch.cuda.synchronize()
        for h in ctxs:
            h.close()


def lib_version() -> str:
    """jf_version() of the loaded library: it carries a digest of the sources, headers and flags it was built from."""
    from jetfire_amd import _lib
    return _lib.load().jf_version().decode()


def profile_counters(scheme: str, workload: str):
    """Counter-derived figures of the scan kernel for this workload, from the committed rocprofv3 summaries (they
    cannot be collected from inside a benchmark process): HBM traffic per launch, MFMA and VALU busy shares.  A summary
    names the library build it was taken with; figures of another build than the loaded one are not reported
    (`traffic` stays null and `*_stale` says which build the summary belongs to)."""
    out = {"traffic": None}
    have = lib_version()
    tpath = os.path.join(ROOT, "profiles", f"fused_scan_{scheme}_{workload}_traffic.json")
    cpath = os.path.join(ROOT, "profiles", f"decode_kernels_{workload}_sq_counters.json")
    try:
        t = json.load(open(tpath))
        if t.get("lib_version") == have:
            out["traffic"] = t.get("traffic_bytes_per_launch")
            out["traffic_source"] = os.path.relpath(tpath, ROOT)
        else:
            out["traffic_stale"] = f"{os.path.relpath(tpath, ROOT)} was taken with {t.get('lib_version', 'an unnamed build')}"
    except Exception:
        pass
    try:
        cj = json.load(open(cpath))
        if cj.get("lib_version") == have:
            c = cj["fused_scan_kernel"]
            out["mfma_busy_pct"] = c.get("mfma_busy_pct")
            out["valu_issue_pct"] = c.get("valu_issue_pct")
            out["counters_source"] = os.path.relpath(cpath, ROOT)
        else:
            out["counters_stale"] = f"{os.path.relpath(cpath, ROOT)} was taken with {cj.get('lib_version', 'an unnamed build')}"
    except Exception:
        pass
    return out


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c2k4", "c3", "c4", "c5"],
                    help="c1: B1 S4096 K4V4 k64, one layer (the reference's CPU-runnable case); "
                         "c2: Llama-3.1-8B B4 S32768 K3V2 k256 x32 layers (the headline); c2k4: the c2 shape with K4V4; "
                         "c3: B1 S131072 K4V4 k512; "
                         "c4: Qwen3-30B-A3B B4 GQA8 K3V2 x48; c5: Llama-3.3-70B TP2 shard B2 S65536 K3V2 x80")
    ap.add_argument("--scheme", default=None,
                    help="run the workload's shape with another quantisation scheme: k{2,3,4}v{2,3,4}, or a2v{2,3,4} for "
                         "the asymmetric INT2 keys (GPU path only; no CPU baseline, no extra workloads)")
    ap.add_argument("--group", type=int, default=None, choices=[64, 128], help="with --scheme: the quantisation group size")
    ap.add_argument("--layers", type=int, default=None, help="override the number of distinct layer caches")
    ap.add_argument("--paged", action="store_true", help="random block table instead of the identity mapping")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", dest="graph", action="store_true", default=None,
                    help="replay the step from a HIP graph (default; with the hand-off the graph holds the publish kernel "
                         "and the device-side wait of every layer; the roofline kernel timing comes from a separate "
                         "eager pass)")
    ap.add_argument("--eager", dest="graph", action="store_false", help="launch every kernel eagerly in the timed region (with the hand-off: the host-blocking wait)")
    ap.add_argument("--handoff", dest="handoff", action="store_true", default=None,
                    help="include the pinned hand-off and the CPU correction per layer (default for c4 and c5, "
                         "whose definition is end to end)")
    ap.add_argument("--no-handoff", dest="handoff", action="store_false")
    ap.add_argument("--cpu-threads", type=int, default=14,
                    help="CPU correction worker threads (hand-off mode); the box gives 16 cores, two stay free for "
                         "the launching thread and the hand-off's dispatcher / poller")
    ap.add_argument("--via-adapter", action="store_true",
                    help="hand-off mode only: run every layer through jetfire_amd.adapter.try_jetfire_decode (pool "
                         "manager, cache stores, dispatcher gate) instead of calling the operators directly")
    ap.add_argument("--split-len", type=int, default=0,
                    help="measurement aid: force the fused scan's split length (0 = the library's planner)")
    ap.add_argument("--separate-blend", action="store_true",
                    help="GPU-only path: launch the blend as its own kernel instead of the merge kernel's epilogue")
    ap.add_argument("--no-extras", action="store_true",
                    help="default run only: skip the K4V4 records (c2k4 and c3, a few layers fewer would not change them) "
                         "that the c2 line carries besides its own figures")
    ap.add_argument("--calibrate-read", action="store_true",
                    help="stream 1 GiB with a kernel that only reads (10 times) and exit: the read-stream ceiling")
    ap.add_argument("--component", default=None, choices=["append", "cpu-correction", "pcie", "split"],
                    help="time one component of the path at the workload's geometry, print its own JSON line and exit: "
                         "append = quantise-on-write + shadow mirror of a prefill chunk (--tokens); cpu-correction = the "
                         "CPU pool alone on freshly drawn random slots; pcie = pinned copy latency by size")
    ap.add_argument("--tokens", type=int, default=32768, help="--component append: tokens in the prefill chunk")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a plain 1 GiB device copy 10 times and exit (reference for the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU (no sharding, no collectives); --gpus must be 1", file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    from jetfire_amd import _lib, ops, workloads

    lib = _lib.load()
    torch.cuda.set_device(0)
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 100.0       # per copy
        print(json.dumps({"calibrate_copy_bytes_read": 1 << 30, "calibrate_copy_bytes_written": 1 << 30, "launches": 11,
                          "us_per_copy": round(us, 1), "copy_read_plus_write_GBps": round(2 * (1 << 30) / us / 1e3, 1)}))
        return 0
    if args.calibrate_read:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
        sink = torch.zeros(4, dtype=torch.uint8, device="cuda")
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(_lib.debug_hook("jf_calibrate_stream_read")(src.data_ptr(), src.numel(), sink.data_ptr(), st))
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            _lib.check(_lib.debug_hook("jf_calibrate_stream_read")(src.data_ptr(), src.numel(), sink.data_ptr(), st))
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 100.0
        print(json.dumps({"calibrate_read_bytes": 1 << 30, "launches": 11, "us_per_pass": round(us, 1),
                          "read_GBps": round((1 << 30) / us / 1e3, 1), "frac_of_8TBps": round((1 << 30) / us / 1e3 / HBM_PEAK_GBPS, 4)}))
        return 0
    if args.component is not None:
        print(json.dumps({"append": component_append, "cpu-correction": component_cpu_correction,
                          "pcie": component_pcie, "split": component_split}[args.component](args)))
        return 0
    if args.scheme or args.group:
        if args.via_adapter or args.scheme not in (None, *ops.FUSED_SCHEMES):
            print("bench.py: --scheme takes one of " + ", ".join(sorted(ops.FUSED_SCHEMES)) + " and excludes --via-adapter",
                  file=sys.stderr)
            return 2
        B_, Hq_, Hkv_, S_, sch_, gs_, K_, L_ = workloads.CONFIGS[args.workload]
        workloads.CONFIGS[args.workload] = (B_, Hq_, Hkv_, S_, args.scheme or sch_, args.group or gs_, K_, L_)
        args.no_cpu_baseline = args.no_extras = True
    if args.split_len:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(args.split_len))
    handoff = args.handoff if args.handoff is not None else args.workload in ("c4", "c5")
    if args.graph is None:
        args.graph = not args.via_adapter
    if handoff and args.graph and args.via_adapter:
        print("bench.py: --graph with the hand-off goes through the operators, not the adapter", file=sys.stderr)
        return 2
    n_shadow = 4 if handoff else 0   # distinct host shadows, cycled over the layers (a layer's shadow is 2*H_kv*slots*256 B)
    w = workloads.build(args.workload, n_layers=args.layers, keep_shadow=n_shadow)
    n_layers = len(w.layers)
    o_new = torch.zeros(w.B, w.H_q, 128, dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(o_new)
    ctxs = []
    if args.via_adapter and not handoff:
        print("bench.py: --via-adapter needs the hand-off mode", file=sys.stderr)
        return 2
    if handoff and not args.via_adapter:
        ops.set_cpu_attn_threads(args.cpu_threads)
        ctxs = [ops.CpuTopkHandoff(w.B, w.H_q, w.H_kv, w.top_k, ksh, vsh, w.attn_scale) for ksh, vsh in w.shadows]
    adapter_layers = []
    if args.via_adapter:
        # Four cache stores (one per distinct host shadow) own the packed tensors of the first four layers; the
        # layers of the step cycle over them.  The stores are filled from the workload's tensors (quantised by
        # the same append kernels) instead of being re-appended token by token.
        import types
        import jetfire_amd.adapter as adapter
        os.environ["JETFIRE_FAST_STORE_COMPLETE_CHECK"] = "1"
        adapter.set_jetfire_config(scheme={"k3v2": "SymInt3K_SymInt2V", "k4v4": "SymInt4K_SymInt4V"}[w.scheme],
                                   group_size=w.group, topk=w.top_k, cpu_attn_threads=args.cpu_threads)
        adapter.reset_global_kv_pool_manager()
        pool = adapter.get_global_kv_pool_manager()
        impl = types.SimpleNamespace(attn_type=types.SimpleNamespace(name="DECODER"), scale=w.attn_scale)
        meta = types.SimpleNamespace(seq_lens=w.seq_lens, block_table=w.block_table, use_cascade=False, max_query_len=1,
                                     num_actual_tokens=w.B, max_seq_len=w.S)
        num_blocks = w.layers[0].k_data.size(1) // 16
        for i, (ksh, vsh) in enumerate(w.shadows):
            name = f"model.layers.{i}.self_attn.attn"
            pool.register_layer_config(name, num_query_heads=w.H_q, num_kv_heads=w.H_kv, head_dim=128)
            pool.register_layer_layout(name, num_blocks=num_blocks, block_size=16)
            st = pool.ensure_layer_store(name, device=torch.device("cuda"))
            lay = w.layers[i]
            st.k_data, st.k_scales, st.v_data, st.v_scales = lay.k_data, lay.k_scales.view_as(st.k_scales), lay.v_data, lay.v_scales.view_as(st.v_scales)
            st.k_shadow, st.v_shadow = ksh, vsh
            st.slot_filled.fill_(True)
            st.written_count = w.S
            adapter_layers.append(types.SimpleNamespace(layer_name=name, num_heads=w.H_q, num_kv_heads=w.H_kv, head_size=128))
        n_layers_adapter = n_layers

    def step():
        if adapter_layers:
            for li in range(n_layers_adapter):
                got = adapter.try_jetfire_decode(impl=impl, layer=adapter_layers[li % len(adapter_layers)], query=w.q,
                                                 attn_metadata=meta, output=out)
                assert got is not None, pool.get_stats()["decode_fallbacks"]
            return
        if ctxs:
            ops.pool_doorbell() if args.graph else ops.pool_wake()   # the pool spins when the first layer's job arrives
        for li, lay in enumerate(w.layers):
            o_hat, slots, o_old, W, idx = ops.fused_attn_topk(
                w.scheme, w.q, lay.k_data, lay.k_scales, lay.v_data, lay.v_scales, w.block_table, w.seq_lens,
                w.S, w.H_q, w.H_kv, 16, w.top_k, w.attn_scale, blend=None if (ctxs or args.separate_blend) else (o_new, out),
                k_zp=lay.k_zp)
            if not ctxs and not args.separate_blend:
                continue            # the merge kernel has written `out` (o_new is known up front without a hand-off)
            if ctxs:
                h = ctxs[li % len(ctxs)]
                if args.graph:      # kernels only: the publish kernel, then a device-side wait that also blends
                    h.stream_submit(w.q, slots)
                    h.stream_wait_blend(o_hat, o_old, W, out)
                    continue
                h.submit(w.q, slots)
                h.wait(o_new)
            ops.blend_unnorm_into(o_hat, o_old, W, o_new, out)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    graph = None
    if args.graph:
        graph = torch.cuda.CUDAGraph()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            step()
        torch.cuda.current_stream().wait_stream(s)
        with torch.cuda.graph(graph, stream=s):
            step()
        graph.replay()
        torch.cuda.synchronize()

    # ---- timed region (whole-job throughput), with HIP events around every scan-kernel launch when eager
    total_ms = ctypes.c_double(0.0)
    launches = ctypes.c_int(0)
    if graph is None:
        _lib.check(_lib.debug_hook("jf_profile_scan_begin")(args.steps * n_layers))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        if graph is not None:
            graph.replay()
        else:
            step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    for h in ctxs:
        if args.graph:
            h.check_status()
    if graph is None:
        _lib.check(_lib.debug_hook("jf_profile_scan_end")(ctypes.byref(total_ms), ctypes.byref(launches)))
    else:   # kernel time from a separate eager pass
        _lib.check(_lib.debug_hook("jf_profile_scan_begin")(n_layers * 3))
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        _lib.check(_lib.debug_hook("jf_profile_scan_end")(ctypes.byref(total_ms), ctypes.byref(launches)))

    ms_per_step = elapsed / args.steps * 1e3
    bytes_layer = w.packed_bytes_per_layer
    value = bytes_layer * n_layers / (ms_per_step * 1e-3) / 1e9
    scan_us = total_ms.value / max(1, launches.value) * 1e3
    achieved = bytes_layer / (scan_us * 1e-6) / 1e9 if scan_us > 0 else 0.0
    counters = profile_counters(w.scheme, args.workload)

    res = {
        "metric": "decode-scan HBM GB/s on packed KV (fused scan + top-k + merge, all layers of one decode step)",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "us_per_layer": round(ms_per_step * 1e3 / n_layers, 2),
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8 codes; int8/bf16 MFMA, fp32 softmax", "data": "synthetic", "lib_version": lib_version(),
        "config": {"workload": f"{args.workload}: B{w.B} Hq{w.H_q} Hkv{w.H_kv} D128 S{w.S} {w.scheme} g{w.group} "
                               f"top_k{w.top_k} x{n_layers} layers, {'paged (random)' if args.paged else 'identity'} block table",
                   "packed_bytes_per_layer": bytes_layer, "launch": "hip-graph" if graph is not None else "eager",
                   **({"split_len_forced": args.split_len} if args.split_len else {}),
                   **({"via": "jetfire_amd.adapter.try_jetfire_decode (4 cache stores cycled over the layers)"} if args.via_adapter else {}),
                   "handoff": (f"slots + q to pinned memory, CPU correction on {ops.get_cpu_attn_threads()} threads, o_new back, every layer"
                               + (" (device-side wait, whole step in one graph)" if args.graph else " (host-blocking wait)")
                               if handoff else "not in the timed region (GPU path only)")},
        "roofline": {"bound": "hbm", "kernel": "fused_scan_kernel", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "kernel_us": round(scan_us, 2),
                     "launches_timed": launches.value, **counters},
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(w)
        res["cpu_baseline"]["c1"] = cpu_baseline_c1()
    for h in ctxs:
        h.close()
    default_run = (args.workload == "c2" and not handoff and not args.no_extras and args.layers is None
                   and not args.paged and not args.split_len and graph is not None)
    if default_run:
        # the metric is quoted for K3V2 and K4V4: the K4V4 figures of the same run
        del graph
        w.layers.clear()
        torch.cuda.empty_cache()
        res["k4v4"] = [measure_gpu_path(name, max(3, args.steps // 2), 1, lib) for name in ("c2k4", "c3")]
        # C4 is defined end to end (hand-off + CPU correction + merge): its figure of the same run
        res["e2e"] = measure_e2e("c4", min(10, max(3, args.steps // 2)), args.cpu_threads)
    print(json.dumps(res))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
