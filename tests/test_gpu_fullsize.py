"""Parity of the fused decode step at the benchmark's full shapes (one layer), through properties that do
not need the slow CPU oracle: the reference's own validation formulas evaluated with torch on the GPU
(dequantised cache via the torch restatement of `unpack`, dense fp32 attention; for INT4 keys the int8-quantised
query model restated with torch, bit for bit), exact top-k on the kernel's own scores, the clear-margin winners of
the reference scores, softmax statistics, and run-to-run determinism."""
import pytest
import torch

from oracle import torch_cpu_path as T

pytestmark = pytest.mark.gpu


def _run(w, lay, **kw):
    from jetfire_amd import ops
    return ops.fused_attn_topk(w.scheme, w.q, lay.k_data, lay.k_scales, lay.v_data, lay.v_scales, w.block_table,
                               w.seq_lens, w.S, w.H_q, w.H_kv, 16, w.top_k, w.attn_scale, k_zp=lay.k_zp, **kw)


def _check_layer_properties(w):
    from jetfire_amd import workloads
    lay = w.layers[0]
    B, Hq, Hkv, S, K = w.B, w.H_q, w.H_kv, w.S, w.top_k
    G = Hq // Hkv
    kb, vb, asym = workloads.scheme_bits(w.scheme)
    o_hat, slots, o_old, W, idx, m, iz, scores = _run(w, lay, return_scores=True, return_stats=True)
    again = _run(w, lay, return_scores=True, return_stats=True)
    for a, b in zip((o_hat, slots, o_old, W, idx, m, iz, scores), again):
        assert torch.equal(a, b)                                   # deterministic

    # --- top-k: exact on the kernel's own scores, ascending positions, slots through the block table
    tv, _ = scores.topk(K, dim=-1)
    got = scores.gather(-1, idx)
    assert torch.equal(got.sort(dim=-1, descending=True).values, tv)
    assert (idx[..., 1:] > idx[..., :-1]).all()
    pos_slots = torch.gather(w.block_table, 1, (idx // 16).reshape(B, -1)).reshape(B, Hq, K) * 16 + idx % 16
    assert torch.equal(slots, pos_slots)

    # --- softmax statistics of those scores
    assert torch.equal(m, scores.max(dim=-1).values)
    z = (scores - m[..., None]).exp().sum(-1)
    torch.testing.assert_close(iz, 1.0 / z, rtol=2e-5, atol=0)

    # --- dense reference from the dequantised cache (per sequence, one kv-head at a time to bound memory)
    pos = torch.arange(S, device="cuda")
    max_sc = 0.0
    for b in range(B):
        sl = w.block_table[b, pos // 16] * 16 + pos % 16
        for h in range(Hkv):
            if asym:    # khat = bf16(fma(code - 2, scale, zp)); (code - 2) * scale is exact in fp32, so mul + add is the fma
                codes = T.unpack(lay.k_data[h, sl], torch.ones_like(lay.k_scales[h, sl]), w.group, kb).float()
                kf = (codes.reshape(S, -1, w.group) * lay.k_scales[h, sl].float()[..., None]
                      + lay.k_zp[h, sl].float()[..., None])
                khat = kf.to(torch.bfloat16).float().reshape(S, 128)
            else:
                khat = T.unpack(lay.k_data[h, sl], lay.k_scales[h, sl], w.group, kb).float()      # (S, 128)
            # Stage B multiplies by the unrounded fp32 scale: redo the dequant without the bf16 rounding
            vq = T.unpack(lay.v_data[h, sl], torch.ones_like(lay.v_scales[h, sl]), w.group, vb).float()
            vexact = (vq.reshape(S, -1, w.group) * lay.v_scales[h, sl].float()[..., None]).reshape(S, 128)
            qh = w.q[b, h * G:(h + 1) * G].float()
            ref = (qh @ khat.T) * w.attn_scale                                                  # (G, S)
            mine = scores[b, h * G:(h + 1) * G]
            if kb != 4 or w.scheme[0] == "b":   # same scoring model: bf16-rounded dequantised keys
                torch.testing.assert_close(mine, ref, atol=3e-5, rtol=3e-5)
                # every winner of the reference scores that is clear of the cut by more than the score tolerance
                # must be among the kernel's winners (near-ties at the cut may differ legitimately)
                top = ref.topk(K, dim=-1)
                clear = top.values > top.values[:, -1:] + 1e-4
                chosen = torch.zeros(G, S, dtype=torch.bool, device="cuda")
                chosen.scatter_(1, idx[b, h * G:(h + 1) * G], True)
                assert bool(chosen.gather(1, top.indices)[clear].all())
                assert int(clear.sum()) >= G * (K - 8)
            else:                       # int8-quantised query model, restated with torch: bit-equal
                model = T.int8_q_scores(w.q[b, h * G:(h + 1) * G], lay.k_data[h, sl], lay.k_scales[h, sl], w.attn_scale)
                assert torch.equal(mine.view(torch.int32), model.view(torch.int32))
                assert (mine - ref).abs().max() < 0.05 * ref.abs().max()    # and near the dense bf16 model
            max_sc = max(max_sc, float(mine.abs().max()))
            p = torch.softmax(mine, dim=-1)
            torch.testing.assert_close(o_hat[b, h * G:(h + 1) * G], p @ vexact, atol=4e-6, rtol=1e-4)
            sel = idx[b, h * G:(h + 1) * G]
            pw = p.gather(-1, sel)
            torch.testing.assert_close(W[b, h * G:(h + 1) * G], pw.sum(-1), atol=4e-6, rtol=1e-4)
            old = torch.einsum("gk,gkd->gd", pw, vexact[sel])
            torch.testing.assert_close(o_old[b, h * G:(h + 1) * G], old, atol=4e-6, rtol=1e-4)
            del khat, vq, vexact
    assert max_sc > 0


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_full_size_layer_properties(name):
    from jetfire_amd import workloads
    _check_layer_properties(workloads.build(name, n_layers=1, paged=True))


@pytest.mark.parametrize("scheme,gs,Hq,Hkv", [
    ("k3v3", 64, 8, 2), ("k2v3", 128, 8, 2), ("k4v3", 128, 16, 2), ("k2v2", 64, 8, 2), ("k3v4", 64, 8, 2), ("k2v4", 128, 4, 2),
    ("a2v2", 64, 8, 2), ("a2v3", 128, 8, 2), ("a2v4", 64, 16, 2), ("b4v4", 64, 8, 2), ("b4v3", 128, 16, 2),
    ("k4v2", 128, 14, 2), ("k3v2", 64, 6, 2)])
def test_full_length_splits_of_the_other_schemes(scheme, gs, Hq, Hkv):
    """The same properties for the schemes the benchmark shapes do not use, at the longest split a workgroup takes
    (4096 positions: the full LDS layout, four chunks per wavefront), on a paged cache; the last two rows have 7 and
    3 query heads per kv-head."""
    from jetfire_amd import _lib, workloads
    lib = _lib.load()
    workloads.CONFIGS["other"] = (2, Hq, Hkv, 16384, scheme, gs, 256, 1)
    try:
        w = workloads.build("other", n_layers=1, paged=True)
    finally:
        del workloads.CONFIGS["other"]
    _lib.check(_lib.debug_hook("jf_debug_split_len")(4096))
    try:
        _check_layer_properties(w)
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))


def test_c1_gpu_split_path_agrees_with_the_cpu_torch_path():
    """C1 is the configuration the reference itself runs on a CPU (unpack -> einsum -> topk in torch, fp32 q times
    bf16-rounded keys).  The split-form INT4 kernels with the same scoring model (int4_qk_scores, exact top-k,
    int4_softmax_v) against the torch restatement of that CPU path on the full C1 shape: the same winners
    wherever the margin exceeds accumulation noise, and the same attention output up to the bf16 rounding the
    CPU path applies to the dequantised values."""
    from jetfire_amd import ops, workloads
    w = workloads.build("c1", n_layers=1, paged=False)
    lay = w.layers[0]
    S, K, Hq, Hkv = w.S, w.top_k, w.H_q, w.H_kv
    scores, idx, slots, m, iz = ops.int4_qk_scores_topk_stats(w.q, lay.k_data, lay.k_scales, w.block_table, w.seq_lens, S,
                                                             Hq, Hkv, 16, w.attn_scale, K)
    o_hat, o_old, W = ops.int4_softmax_v_with_pre_corr_wvs2_scores(scores, lay.v_data, lay.v_scales, w.block_table,
                                                                   w.seq_lens, idx, S, Hq, Hkv, 16, K)
    def cpu(t):                                       # the sequence occupies slots [0, S) of the identity block table
        t = t[:, :S].cpu()
        return (t.unsqueeze(-1) if t.dim() == 2 else t).unsqueeze(0)
    ref_o, ref_idx = T.decode_path(w.q.cpu(), cpu(lay.k_data), cpu(lay.k_scales), cpu(lay.v_data), cpu(lay.v_scales),
                                   w.group, 4, 4, K)
    sc = scores[0].cpu()
    for h in range(Hq):
        cut = sc[h].topk(K).values[-1]
        clear = {int(i) for i in ref_idx[0, h].tolist() if sc[h, int(i)] > cut + 1e-4}
        assert clear <= set(idx[0, h].cpu().tolist())
        assert len(clear) >= K - 4                                        # almost every winner is clear of the cut
    torch.testing.assert_close(o_hat.cpu(), ref_o.float(), atol=2e-3, rtol=2e-2)
    assert float((o_hat.cpu() - ref_o.float()).abs().mean()) < 2e-4


@pytest.mark.parametrize("name", ["c2", "c3", "c4"])
def test_two_call_form_equals_the_one_pass_form_at_full_size(name):
    """The reference-named Stage A and Stage B operators run on the same kernels as the one-pass form (without the
    other stage): scores, winners, slots and statistics come out bit-equal, and so do o_hat, o_old_unnorm and W
    (exact integer accumulation, the same split geometry)."""
    from jetfire_amd import ops, workloads
    w = workloads.build(name, n_layers=1, paged=True)
    lay = w.layers[0]
    S, K, Hq, Hkv = w.S, w.top_k, w.H_q, w.H_kv
    assert ops.get_split_impl() == "fast"
    o_hat, slots, o_old, W, idx, m, iz, scores = _run(w, lay, return_scores=True, return_stats=True)
    if w.scheme == "k3v2":
        sc2, idx2, slots2 = ops.int3_qk_scores_topk(w.q, lay.k_data, lay.k_scales, w.block_table, w.seq_lens, S, Hq, Hkv, 16,
                                                    w.attn_scale, K)
        stage_b = ops.int2_softmax_v_with_pre_corr_wvs2
    else:
        sc2, idx2, slots2, m2, iz2 = ops.int8tc_qk_scores_topk_stats(w.q, lay.k_data, lay.k_scales, w.block_table,
                                                                     w.seq_lens, S, Hq, Hkv, 16, w.attn_scale, K)
        assert torch.equal(m2, m) and torch.equal(iz2, iz)
        stage_b = ops.int4_softmax_v_with_pre_corr_wvs2_scores
    assert torch.equal(sc2.view(torch.int32), scores.view(torch.int32))
    assert torch.equal(idx2, idx) and torch.equal(slots2, slots)
    o_hat2, o_old2, W2 = stage_b(sc2, lay.v_data, lay.v_scales, w.block_table, w.seq_lens, idx2, S, Hq, Hkv, 16, K)
    assert torch.equal(o_hat2, o_hat) and torch.equal(o_old2, o_old) and torch.equal(W2, W)


@pytest.mark.parametrize("name,units", [("c4", ((0, 1), (3, 2))), ("c5", ((0, 1), (1, 2)))])
def test_end_to_end_with_handoff_matches_the_oracle_on_sampled_units(name, units):
    """Configurations C4 (B4, 32 query / 4 kv heads, 32768 positions, top-k 256) and C5 (B2, 65536 positions, top-k
    512) at their full shapes, K3V2, paged, one layer, the whole step: fused scan + merge, pinned hand-off, CPU
    correction from the bf16 host shadow, device-side wait and blend.  The oracle's `decode_reference` (numpy) is run
    on two sampled (sequence, kv-head) units - all eight query heads of each over the full context - and the blended
    output must match it within the acceptance bounds (2e-2 max-abs, 1e-3 mean-abs in bf16) and the reference's own
    blend tolerance."""
    import numpy as np
    from jetfire_amd import ops, workloads
    from oracle import jetfire_oracle as O
    from tests.helpers import bf16_to_bits, bf16_to_f32
    w = workloads.build(name, n_layers=1, paged=True, keep_shadow=1)
    lay = w.layers[0]
    ksh, vsh = w.shadows[0]
    B, Hq, Hkv, S, K = w.B, w.H_q, w.H_kv, w.S, w.top_k
    G = Hq // Hkv
    ops.set_cpu_attn_threads(8)
    h = ops.CpuTopkHandoff(B, Hq, Hkv, K, ksh, vsh, w.attn_scale)
    try:
        o_hat, slots, o_old, W, idx = ops.fused_attn_topk(w.scheme, w.q, lay.k_data, lay.k_scales, lay.v_data, lay.v_scales,
                                                          w.block_table, w.seq_lens, S, Hq, Hkv, 16, K, w.attn_scale)
        out = torch.empty(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
        h.stream_submit(w.q, slots)
        h.stream_wait_blend(o_hat, o_old, W, out)
        torch.cuda.synchronize()
        h.check_status()
    finally:
        h.close()
    res = bf16_to_f32(out)
    bt = w.block_table.cpu().numpy()
    for b, kvh in units:
        hs = slice(kvh * G, (kvh + 1) * G)
        r = O.decode_reference(
            bf16_to_f32(w.q[b:b + 1, hs]), lay.k_data[kvh:kvh + 1].cpu().numpy(), bf16_to_bits(lay.k_scales[kvh:kvh + 1]),
            lay.v_data[kvh:kvh + 1].cpu().numpy(), bf16_to_bits(lay.v_scales[kvh:kvh + 1]), bt[b:b + 1],
            np.array([S], np.int32), S, G, 1, 16, w.attn_scale, K, "k3v2", bf16_to_f32(ksh[kvh:kvh + 1]),
            bf16_to_f32(vsh[kvh:kvh + 1]), group_size=w.group)
        got = res[b, hs]
        np.testing.assert_allclose(got, r["out"][0], atol=6e-3, rtol=1.5e-2)
        err = np.abs(got - r["out"][0])
        assert err.max() <= 2e-2 and err.mean() <= 1e-3
        # the kernel's winners against the oracle's: identical up to near-ties at the cut
        mine = idx[b, hs].cpu().numpy()
        for g in range(G):
            assert len(set(mine[g].tolist()) & set(r["topk_idx"][0, g].tolist())) >= K - 4
