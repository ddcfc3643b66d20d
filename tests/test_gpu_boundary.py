"""The reference's own operator sequence for the CPU hand-off and the merge, driven through the names its
extension modules export (jetfire_vllm/csrc/cpu_topk_attn.cpp:2509-2663, jetfire_vllm/csrc/blend.cu:379-399) in
the order its adapter calls them (jetfire_vllm/adapter/decode_path.py:2243-2267 pinned copies, :2473-2477
cpu_topk_attn, :2526-2527 stream_write_value64 + stream_submit_cpu_topk_attn, :3070 stream_wait_cpu_topk_attn,
:3161-3163 blend_unnorm_into), eagerly and from a HIP graph, against the oracle."""
import numpy as np
import pytest
import torch

from oracle import jetfire_oracle as O
from tests.helpers import bf16_tensor, bf16_to_f32, make_case, to_device

pytestmark = pytest.mark.gpu

SCALE = 128 ** -0.5


def _exts():
    from jetfire_amd.kernels.blend import load_blend_ext
    from jetfire_amd.kernels.cpu_topk_attn import load_cpu_topk_attn_ext
    from jetfire_amd.kernels.int2_split import load_softmax_v_ext
    from jetfire_amd.kernels.int3_split import load_qk_scores_ext
    return load_cpu_topk_attn_ext(), load_blend_ext(), load_qk_scores_ext(), load_softmax_v_ext()


def test_mapped_pinned_pair_is_one_buffer():
    cpu, _, _, _ = _exts()
    host, dev = cpu.alloc_mapped_pinned_pair((2, 3, 128), torch.bfloat16)
    assert host.is_pinned() and dev.is_cuda and host.shape == dev.shape == (2, 3, 128) and dev.dtype == torch.bfloat16
    host.copy_(torch.arange(768, dtype=torch.float32).view(2, 3, 128).to(torch.bfloat16))
    torch.cuda.synchronize()
    assert torch.equal(dev.cpu().view(torch.int16), host.view(torch.int16))          # the GPU reads what the CPU wrote
    dev.mul_(2)
    torch.cuda.synchronize()
    assert float(host[1, 2, 5].float()) == 2 * float(torch.tensor(645.0).to(torch.bfloat16))   # and the other way
    fh, fd = cpu.alloc_mapped_pinned_pair((1,), torch.int64)
    stream = torch.cuda.current_stream().cuda_stream
    cpu.stream_write_value64(stream, fd, 41)
    torch.cuda.synchronize()
    assert int(fh[0]) == 41
    fh[0] = 7
    cpu.stream_wait_value64(stream, fd, 7)                                          # already satisfied: returns at once
    torch.cuda.synchronize()


@pytest.mark.parametrize("graph", (False, True))
def test_reference_call_sequence_for_one_decode_layer(graph):
    cpu, blend, stage_a, stage_b = _exts()
    B, Hq, Hkv, S, K = 2, 8, 2, 512, 64
    c = make_case(123, B, Hq, Hkv, S, 3, 2, 64)
    d = to_device(c)
    ksh, vsh = bf16_tensor(c["K"]), bf16_tensor(c["V"])
    cpu.graph_pool_warmup_threads(4)
    cpu.reset_graph_runtime_state()
    # the adapter's stable buffers (decode_path.py:411-417, 454-470)
    q_buf = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, pin_memory=True)
    ts_buf = torch.zeros(B, Hq, K, dtype=torch.int64, pin_memory=True)
    o_new_pin = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, pin_memory=True)
    head_map = torch.from_numpy(O.head_map(B, Hq, Hq // Hkv, K))
    flag_host, flag_dev = cpu.alloc_mapped_pinned_pair((1,), torch.int64)
    ctx = cpu.create_cpu_topk_submit_ctx(q_buf, ksh, vsh, head_map, ts_buf, o_new_pin, SCALE, flag_host)
    assert isinstance(ctx, int) and ctx > 0
    q_dev = d["q"].clone()
    o_new_gpu = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    # Stage B output buffers of the in-place entry (decode_path.py:2875-2919)
    weights = torch.empty(B, Hq, S, dtype=torch.float32, device="cuda")
    o_hat = torch.empty(B, Hq, 128, dtype=torch.float32, device="cuda")
    o_old = torch.empty_like(o_hat)
    W = torch.empty(B, Hq, dtype=torch.float32, device="cuda")

    def layer():
        stream_id = torch.cuda.current_stream().cuda_stream
        scores, idx, slots = stage_a.int3_qk_scores_topk(q_dev, d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, SCALE, K)
        q_buf.copy_(q_dev, non_blocking=True)
        ts_buf.copy_(slots, non_blocking=True)
        cpu.stream_write_value64(stream_id, flag_dev, 0)
        cpu.stream_submit_cpu_topk_attn(stream_id, ctx)
        stage_b.int2_softmax_v_with_pre_corr_wvs2_inplace(scores, d["vd"], d["vs"], d["bt"], d["lens"], idx, weights, o_hat,
                                                          o_old, W, S, Hq, Hkv, 16, K)
        cpu.stream_wait_cpu_topk_attn(stream_id, ctx)
        o_new_gpu.copy_(o_new_pin, non_blocking=True)
        blend.blend_unnorm_into(o_hat, o_old, W, o_new_gpu, out)

    def check(q_np, n_done):
        torch.cuda.synchronize()
        cpu.check_cpu_topk_submit_ctx(ctx)
        assert int(flag_host[0]) == 1 and cpu.get_graph_submit_count() == n_done
        r = O.decode_reference(q_np, c["kd"], c["ks"], c["vd"], c["vs"], c["bt"], c["lens"], S, Hq, Hkv, 16, SCALE, K,
                               "k3v2", c["K"], c["V"])
        np.testing.assert_allclose(bf16_to_f32(o_new_gpu), r["o_new"], atol=2e-3, rtol=6e-3)
        got = bf16_to_f32(out)
        np.testing.assert_allclose(got, r["out"], atol=6e-3, rtol=1.5e-2)
        err = np.abs(got - r["out"])
        assert err.max() <= 2e-2 and err.mean() <= 1e-3

    rng = np.random.default_rng(8)
    if not graph:
        layer()
        check(c["q"], 1)
        q2 = O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32))
        q_dev.copy_(bf16_tensor(q2).cuda())
        layer()
        check(q2, 2)
    else:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            layer()                                        # warm-up outside the capture (allocations, poller start)
        torch.cuda.current_stream().wait_stream(side)
        check(c["q"], 1)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            layer()
        for rep in range(3):
            qn = O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32))
            q_dev.copy_(bf16_tensor(qn).cuda())
            out.zero_()
            g.replay()
            check(qn, 2 + rep)
            torch.cuda.synchronize()
        del g
    # the mapped o_new form with the host-side join (blend.cu:292-377): no H2D copy at all
    o_map_host, o_map_dev = cpu.alloc_mapped_pinned_pair((B, Hq, 128), torch.bfloat16)
    done = torch.zeros(1, dtype=torch.int64)
    scores, idx, slots = stage_a.int3_qk_scores_topk(q_dev, d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, SCALE, K)
    q_host, ts_host = q_dev.cpu(), slots.cpu()
    cpu.submit_cpu_topk_attn_async(q_host, ksh, vsh, head_map, ts_host, o_map_host, SCALE, done)
    o_hat2, o_old2, W2 = stage_b.int2_softmax_v_with_pre_corr_wvs2(scores, d["vd"], d["vs"], d["bt"], d["lens"], idx, S, Hq,
                                                                   Hkv, 16, K)
    out2 = torch.zeros_like(out)
    blend.wait_and_blend_unnorm_into(done, o_hat2, o_old2, W2, o_map_dev, out2)
    torch.cuda.synchronize()
    assert torch.equal(out2.view(torch.int16), out.view(torch.int16))
    cpu.clear_graph_contexts()
    with pytest.raises(RuntimeError, match="unknown context handle"):
        cpu.stream_submit_cpu_topk_attn(torch.cuda.current_stream().cuda_stream, ctx)
    cpu.set_cpu_attn_threads(2)


def test_blend_forms_agree():
    """blend / blend_into take a normalised o_old: with o_old = o_old_unnorm / W they give what blend_unnorm_into
    gives (jetfire_vllm/adapter/decode_path.py:3219-3222), and bit-equal values to the formula evaluated in fp32."""
    _, blend, _, _ = _exts()
    g = torch.Generator().manual_seed(3)
    B, Hq = 3, 8
    o_hat = torch.randn(B, Hq, 128, generator=g).cuda()
    o_old = torch.randn(B, Hq, 128, generator=g).cuda()
    W = torch.rand(B, Hq, generator=g).cuda()
    o_new = torch.randn(B, Hq, 128, generator=g).to(torch.bfloat16).cuda()
    got = blend.blend(o_hat, o_old, W, o_new)
    into = torch.zeros_like(got)
    blend.blend_into(o_hat, o_old, W, o_new, into)
    assert torch.equal(got.view(torch.int16), into.view(torch.int16))
    want = torch.addcmul(o_hat.double(), W.double().unsqueeze(-1), o_new.double() - o_old.double())
    ref = torch.empty_like(got)
    ref.copy_(want.float())          # fp64 fma then one rounding to fp32 equals the fp32 fma except at double-rounding ties
    assert (got.float() - ref.float()).abs().max() <= 2 ** -7 * want.abs().max()
    unnorm = torch.zeros_like(got)
    blend.blend_unnorm_into(o_hat, o_old * W.unsqueeze(-1), W, o_new, unnorm)
    assert (got.float() - unnorm.float()).abs().max() <= 0.02 * (1 + want.abs().max())
    with pytest.raises(RuntimeError, match="o_old shape mismatch"):
        blend.blend(o_hat, o_old[:, :4], W, o_new)


def test_graph_statistics_carry_the_reference_names():
    """What `jetfire_get_graph_stats` / `reset_jetfire_graph_stats` call on the extension module
    (`jetfire_vllm/adapter/decode_path.py:1017-1045`): get_shadow_append_count, get_graph_timing_stats,
    reset_graph_submit_count, next to the counters that were already there."""
    from jetfire_amd import ops
    cpu, _, _, _ = _exts()
    cpu.reset_graph_submit_count()
    assert cpu.get_shadow_append_count() == 0 and cpu.get_graph_submit_count() == 0
    Hkv, n = 2, 40
    k = torch.randn(n, Hkv, 128).to(torch.bfloat16).cuda()
    ksh = torch.zeros(Hkv, 64, 128, dtype=torch.bfloat16, pin_memory=True)
    vsh = torch.zeros_like(ksh).pin_memory()
    for _ in range(3):
        ops.shadow_write(k, k, torch.arange(n).cuda(), ksh, vsh)
    torch.cuda.synchronize()
    assert cpu.get_shadow_append_count() == 3
    assert torch.equal(ksh[:, :n].view(torch.int16), k.cpu().transpose(0, 1).contiguous().view(torch.int16))
    st = cpu.get_graph_timing_stats()
    for key in ("topk_jobs", "topk_done_avg_us", "topk_done_max_us", "shadow_append_jobs", "join_jobs",
                "join_wait_avg_us", "join_wait_max_us", "pool_workers", "pool_done_count", "pool_initialized"):
        assert key in st
    assert st["shadow_append_jobs"] == 3 and isinstance(st["topk_done_avg_us"], float)
    cpu.reset_graph_submit_count()
    assert cpu.get_shadow_append_count() == 0 and cpu.get_graph_timing_stats()["topk_jobs"] == 0


def test_handoff_jobs_show_up_in_the_timing_statistics_and_the_doorbell_wakes_the_pool():
    from jetfire_amd import ops
    cpu, _, _, _ = _exts()
    B, Hq, Hkv, S, K = 1, 8, 2, 256, 32
    c = make_case(5, B, Hq, Hkv, S, 3, 2, 64)
    d = to_device(c)
    cpu.graph_pool_warmup_threads(2)
    cpu.reset_graph_submit_count()
    h = ops.CpuTopkHandoff(B, Hq, Hkv, K, bf16_tensor(c["K"]), bf16_tensor(c["V"]), SCALE)
    slots = torch.arange(K, dtype=torch.int64).repeat(B, Hq, 1).cuda()
    o_new = torch.empty(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    cpu.pool_doorbell()                       # head of a step: a kernel, then the poller wakes the workers
    h.stream_submit(d["q"], slots)
    h.stream_wait(o_new)
    torch.cuda.synchronize()
    h.check_status()
    st = cpu.get_graph_timing_stats()
    assert st["topk_jobs"] == 1 and st["topk_done_max_us"] > 0 and st["pool_done_count"] >= 1 and st["pool_workers"] == 2
    h.close()
    cpu.pool_wake()                           # the host-side form: no error with or without sleeping workers


def test_int4_stage_b_writes_caller_owned_buffers():
    """`int4_softmax_v_with_pre_corr_wvs2_inplace`, the name graph mode looks up
    (`jetfire_vllm/adapter/decode_path.py:2872-2919`): same numbers as the allocating form."""
    from jetfire_amd.kernels.int4_split import load_softmax_v_ext
    from jetfire_amd.kernels.int8tc_qk_scores import load_int8tc_qk_scores_ext
    B, Hq, Hkv, S, K = 2, 8, 2, 384, 64
    c = make_case(31, B, Hq, Hkv, S, 4, 4, 128)
    d = to_device(c)
    sa, sb = load_int8tc_qk_scores_ext(), load_softmax_v_ext()
    scores, idx, _ = sa.int8tc_qk_scores_topk(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, SCALE, K)[:3]
    ref = sb.int4_softmax_v_with_pre_corr_wvs2_scores(scores, d["vd"], d["vs"], d["bt"], d["lens"], idx, S, Hq, Hkv, 16, K)
    o_hat = torch.full((B, Hq, 128), float("nan"), device="cuda")
    o_old = torch.full((B, Hq, 128), float("nan"), device="cuda")
    W = torch.full((B, Hq), float("nan"), device="cuda")
    weights = torch.empty(B, Hq, S, device="cuda")
    assert sb.int4_softmax_v_with_pre_corr_wvs2_inplace(scores, d["vd"], d["vs"], d["bt"], d["lens"], idx, weights, o_hat,
                                                        o_old, W, S, Hq, Hkv, 16, K) is None
    torch.cuda.synchronize()
    for a, b in zip(ref, (o_hat, o_old, W)):
        assert torch.equal(a, b)
