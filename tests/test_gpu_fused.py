"""GPU parity of the fused decode scan + top-k (and of the whole fused decode step with the CPU
correction hand-off and the merge) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import jetfire_oracle as O
from tests.helpers import bf16_tensor, bf16_to_f32, make_case, to_device

pytestmark = pytest.mark.gpu

SCALE = 128 ** -0.5


def ops():
    from jetfire_amd import ops as _ops
    return _ops


def run_fused(scheme, c, d, S, K):
    o = ops()
    return o.fused_attn_topk(scheme.split("_")[0], d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"], d["lens"], S,
                             c["Hq"], c["Hkv"], 16, K, SCALE, return_scores=True, return_stats=True, k_zp=d.get("kz"))


def check_against_oracle(scheme, c, S, K, out, atol_out=3e-6):
    o_hat, slots, o_old, W, idx, m, iz, scores = [t.cpu().numpy() for t in out]
    kb, vb, gs = c["kbits"], c["vbits"], c["gs"]
    Hq, Hkv = c["Hq"], c["Hkv"]
    if kb in (2, 3) or scheme.startswith("b"):
        ref_sc = O.scores_bf16_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, SCALE, kb, gs,
                                     k_zp_bits=c.get("kzp"))
        valid = np.isfinite(ref_sc)
        assert np.array_equal(np.isneginf(scores), ~valid)
        np.testing.assert_allclose(scores[valid], ref_sc[valid], atol=2e-5, rtol=2e-5)
    else:
        ref_sc = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, SCALE)
        assert np.array_equal(scores.view(np.uint32), ref_sc.view(np.uint32))
    # top-k: exact on the kernel's own scores (and therefore on the oracle's when those are bit-equal)
    ridx, rslots = O.topk_select(scores, c["lens"], c["bt"], S, K)
    assert np.array_equal(idx, ridx)
    assert np.array_equal(slots, rslots)
    # every oracle winner whose margin to the cut exceeds the score tolerance must be selected
    oidx, _ = O.topk_select(ref_sc, c["lens"], c["bt"], S, K)
    for b in range(c["B"]):
        n = min(S, int(c["lens"][b]))
        if n <= K:
            continue
        for h in range(Hq):
            cut = np.sort(ref_sc[b, h, :n])[-K]
            clear = [i for i in oidx[b, h] if ref_sc[b, h, i] > cut + 5e-5]
            assert set(clear) <= set(idx[b, h].tolist())
    rm, riz = O.softmax_stats(scores, c["lens"], S)
    np.testing.assert_allclose(m, rm, atol=1e-7)
    np.testing.assert_allclose(iz, riz, rtol=2e-5)
    r_hat, r_old, r_W = O.softmax_v(scores, c["vd"], c["vs"], c["bt"], c["lens"], idx, S, Hq, Hkv, 16, vb, gs)
    np.testing.assert_allclose(o_hat, r_hat, atol=atol_out, rtol=2e-5)
    np.testing.assert_allclose(o_old, r_old, atol=atol_out, rtol=2e-5)
    np.testing.assert_allclose(W, r_W, atol=atol_out, rtol=2e-5)
    return ref_sc


CASES = [
    # scheme, B, Hq, Hkv, S, lens, K
    ("k3v2", 2, 8, 2, 512, None, 64),
    ("k4v4", 2, 8, 2, 512, None, 64),
    ("k3v2", 3, 32, 4, 512, [17, 257, 512], 256),          # G=8, short rows (reference edge geometry)
    ("k4v4", 3, 32, 4, 512, [17, 257, 512], 256),
    ("k3v2", 4, 8, 2, 32, [0, 1, 9, 17], 32),             # S < K, zero-length row
    ("k4v4", 4, 8, 2, 32, [0, 1, 9, 17], 64),
    ("k3v2", 1, 8, 2, 5000, [4987], 256),                 # many splits, ragged tail
    ("k4v4", 1, 8, 2, 5000, [4987], 512),
    ("k3v2_g128", 2, 8, 2, 700, None, 128),               # INT3/INT2 with one scale group
    ("k3v2", 1, 4, 4, 300, None, 32),                     # G=1
    ("k4v4", 1, 4, 2, 300, None, 64),                     # G=2
    ("k3v2", 1, 16, 1, 600, None, 64),                    # G=16
    ("k4v4", 1, 16, 1, 600, None, 64),
    # the mixed pairs: the key side of one scheme with the value side of the other (group 128)
    ("k3v4", 2, 8, 2, 512, None, 64), ("k4v2", 2, 8, 2, 512, None, 64),
    ("k3v4", 3, 32, 4, 512, [17, 257, 512], 256), ("k4v2", 3, 32, 4, 512, [17, 257, 512], 256),
    ("k3v4", 4, 8, 2, 32, [0, 1, 9, 17], 32), ("k4v2", 4, 8, 2, 32, [0, 1, 9, 17], 64),
    ("k3v4", 1, 8, 2, 5000, [4987], 256), ("k4v2", 1, 8, 2, 5000, [4987], 512),
    ("k3v4", 1, 4, 4, 300, None, 32), ("k4v2", 1, 4, 2, 300, None, 64),
    ("k3v4", 1, 16, 1, 600, None, 64), ("k4v2", 1, 16, 1, 600, None, 64),
    # symmetric INT2 keys (bf16 model, exact for every code)
    ("k2v2", 2, 8, 2, 512, None, 64), ("k2v2_g128", 2, 8, 2, 700, None, 128), ("k2v4", 2, 8, 2, 512, None, 64),
    ("k2v2", 3, 32, 4, 512, [17, 257, 512], 256), ("k2v4", 3, 32, 4, 512, [17, 257, 512], 256),
    ("k2v2", 4, 8, 2, 32, [0, 1, 9, 17], 32), ("k2v2", 1, 8, 2, 5000, [4987], 256), ("k2v4", 1, 8, 2, 5000, [4987], 512),
    ("k2v2", 1, 4, 4, 300, None, 32), ("k2v4", 1, 4, 2, 300, None, 64), ("k2v2", 1, 16, 1, 600, None, 64),
    # planar INT3 values with every key format
    ("k3v3", 2, 8, 2, 512, None, 64), ("k3v3_g128", 2, 8, 2, 700, None, 128), ("k2v3", 2, 8, 2, 512, None, 64),
    ("k2v3_g128", 2, 8, 2, 700, None, 128), ("k4v3", 2, 8, 2, 512, None, 64),
    ("k3v3", 3, 32, 4, 512, [17, 257, 512], 256), ("k4v3", 3, 32, 4, 512, [17, 257, 512], 256),
    ("k2v3", 3, 32, 4, 512, [17, 257, 512], 256),
    ("k3v3", 4, 8, 2, 32, [0, 1, 9, 17], 32), ("k4v3", 4, 8, 2, 32, [0, 1, 9, 17], 64),
    ("k3v3", 1, 8, 2, 5000, [4987], 256), ("k4v3", 1, 8, 2, 5000, [4987], 512), ("k2v3", 1, 8, 2, 5000, [4987], 1024),
    ("k3v3", 1, 4, 4, 300, None, 32), ("k4v3", 1, 4, 2, 300, None, 64), ("k3v3_g128", 1, 16, 1, 600, None, 64),
    ("k2v3", 1, 16, 1, 600, None, 64),
    # wide corrections: the merge kernels keep the winners in dynamic LDS beyond 2048
    ("k3v2", 1, 8, 2, 9000, [8987], 4096), ("k4v4", 2, 4, 2, 9000, [5000, 9000], 8192), ("k3v3", 1, 8, 1, 4200, None, 4096),
    ("a2v2", 1, 4, 4, 8192, None, 8192), ("k2v4", 1, 28, 4, 6000, None, 4096),
    ("k3v2", 1, 8, 2, 5000, [4987], 2048), ("k4v4", 2, 8, 2, 3000, [1000, 3000], 2048),
    ("k3v3", 1, 32, 4, 6000, None, 2048), ("k2v4", 2, 4, 4, 2048, [2048, 2047], 2048),
    # asymmetric INT2 keys (a zero-point per group) with every value format
    ("a2v2", 2, 8, 2, 512, None, 64), ("a2v2_g128", 2, 8, 2, 700, None, 128), ("a2v3", 2, 8, 2, 512, None, 64),
    ("a2v3_g128", 2, 8, 2, 700, None, 128), ("a2v4", 2, 8, 2, 512, None, 64),
    ("a2v2", 3, 32, 4, 512, [17, 257, 512], 256), ("a2v4", 3, 32, 4, 512, [17, 257, 512], 256),
    ("a2v2", 4, 8, 2, 32, [0, 1, 9, 17], 32), ("a2v3", 1, 8, 2, 5000, [4987], 256), ("a2v4", 1, 8, 2, 5000, [4987], 1024),
    ("a2v2", 1, 4, 4, 300, None, 32), ("a2v4", 1, 4, 2, 300, None, 64), ("a2v2_g128", 1, 16, 1, 600, None, 64),
    ("a2v3", 1, 16, 1, 600, None, 64),
    # INT4 values with 64-channel groups (keys other than INT4)
    ("k3v4_g64", 2, 8, 2, 512, None, 64), ("k2v4_g64", 3, 32, 4, 512, [17, 257, 512], 256), ("a2v4_g64", 1, 8, 2, 5000, [4987], 256),
    ("k3v4_g64", 1, 16, 1, 600, None, 64), ("k2v4_g64", 1, 4, 4, 300, None, 32), ("a2v4_g64", 1, 4, 2, 300, None, 64),
    # INT4 keys scored with the bf16 model (any group size)
    ("b4v4", 2, 8, 2, 512, None, 64), ("b4v4_g128", 2, 8, 2, 700, None, 128), ("b4v2", 2, 8, 2, 512, None, 64),
    ("b4v2_g128", 3, 32, 4, 512, [17, 257, 512], 256), ("b4v3", 3, 32, 4, 512, [17, 257, 512], 256),
    ("b4v4", 4, 8, 2, 32, [0, 1, 9, 17], 32), ("b4v3", 1, 8, 2, 5000, [4987], 256), ("b4v4", 1, 8, 2, 5000, [4987], 1024),
    ("b4v2", 1, 4, 4, 300, None, 32), ("b4v4_g128", 1, 4, 2, 300, None, 64), ("b4v4", 1, 16, 1, 600, None, 64),
    ("b4v4", 2, 28, 4, 700, [700, 650], 64),
    # query heads per kv-head that are not a power of two (28/4, 24/8, 40/8, 48/8, 12/1 ...): the next larger kernel
    ("k3v2", 2, 28, 4, 700, [700, 650], 64), ("k4v4", 2, 24, 8, 512, None, 64), ("k3v3", 1, 40, 8, 900, None, 128),
    ("a2v2", 2, 12, 2, 512, [17, 512], 32), ("k2v4", 1, 12, 1, 600, None, 64), ("k4v2", 1, 9, 1, 300, None, 32),
    ("k3v2", 3, 21, 3, 32, [0, 9, 17], 32), ("k4v4", 1, 7, 1, 5000, [4987], 256),
]
SCHEME_GEOMETRY = {f"k{kb}v{vb}": (kb, vb, 128 if 4 in (kb, vb) else 64) for kb in (2, 3, 4) for vb in (2, 3, 4)}
SCHEME_GEOMETRY.update({f"k{kb}v{vb}_g128": (kb, vb, 128) for kb in (2, 3) for vb in (2, 3)})
# INT4 keys with the bf16 scoring model
SCHEME_GEOMETRY.update({"b4v2": (4, 2, 64), "b4v2_g128": (4, 2, 128), "b4v3": (4, 3, 64), "b4v4": (4, 4, 64), "b4v4_g128": (4, 4, 128)})
# asymmetric INT2 keys
SCHEME_GEOMETRY.update({"k3v4_g64": (3, 4, 64), "k2v4_g64": (2, 4, 64), "a2v4_g64": (2, 4, 64)})   # INT4 values, two scale groups
SCHEME_GEOMETRY.update({"a2v2": (2, 2, 64), "a2v2_g128": (2, 2, 128), "a2v3": (2, 3, 64), "a2v3_g128": (2, 3, 128),
                        "a2v4": (2, 4, 128)})


@pytest.mark.parametrize("scheme,B,Hq,Hkv,S,lens,K", CASES)
def test_fused_scan_matches_oracle(scheme, B, Hq, Hkv, S, lens, K):
    kb, vb, gs = SCHEME_GEOMETRY[scheme]
    c = make_case(70 + S + Hq, B, Hq, Hkv, S, kb, vb, gs, lens=lens, extra_blocks=3, k_asym=scheme.startswith("a"))
    d = to_device(c)
    out = run_fused(scheme, c, d, S, K)
    check_against_oracle(scheme, c, S, K, out)


@pytest.mark.parametrize("scheme,S,lens,K,split_len", [
    ("k3v2", 5000, [4987], 256, 256),      # 20 short splits: single-stage merge over many lists
    ("k3v2", 10000, [9989], 256, 512),     # 20 lists of 512 candidates: two-stage merge
    ("k4v4", 10000, [9000], 512, 768),     # two-stage, lists of top_k + 256 entries, empty tail splits
    ("k4v4", 10000, [10000], 1024, 1280),  # widest top-k: parts limited to 8192 / top_k
    ("k3v2", 3000, [3000], 64, 1024),      # longer than the planner would pick for this size
    ("k3v4", 10000, [9989], 256, 512), ("k4v2", 10000, [9000], 512, 768),      # two-stage merges of the mixed pairs
    ("k3v2", 20000, [19989], 2048, 512),   # every position a candidate, 40 lists: two-stage merge at the widest correction
    ("k4v4", 40000, [39000], 2048, 0),     # the planner's own split: lists of 2304 entries, first stage beyond the registers
    ("k3v2", 40000, [39990], 4096, 0),     # every position a candidate; two-stage merge whose parts exceed the registers
    ("k4v4", 20000, [19000], 8192, 1024),  # single stage over every position, most candidates re-read from global memory
])
def test_fused_scan_with_forced_split_length(scheme, S, lens, K, split_len):
    from jetfire_amd import _lib
    lib = _lib.load()
    kb, vb, gs = {"k3v2": (3, 2, 64), "k4v4": (4, 4, 128), "k3v4": (3, 4, 128), "k4v2": (4, 2, 128)}[scheme]
    c = make_case(11 + S + K, 1, 8, 2, S, kb, vb, gs, lens=lens, extra_blocks=3)
    d = to_device(c)
    _lib.check(_lib.debug_hook("jf_debug_split_len")(split_len))
    try:
        out = run_fused(scheme, c, d, S, K)
        forced = [t.clone() for t in out]
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))
    check_against_oracle(scheme, c, S, K, forced)
    # the planner's own split length selects the same positions
    again = run_fused(scheme, c, d, S, K)
    assert torch.equal(forced[4], again[4]) and torch.equal(forced[1], again[1])


@pytest.mark.parametrize("mode", ("zero_query", "few_values", "one_huge_many_tiny"))
@pytest.mark.parametrize("scheme,G,Hkv,S,K,split_len", [
    ("k3v2", 4, 2, 3000, 256, 0), ("k3v2", 8, 1, 2100, 2048, 512), ("k3v2", 16, 1, 2100, 2048, 512),
    ("k4v4", 4, 2, 5000, 64, 1024), ("k2v2", 8, 1, 9000, 512, 0), ("a2v2", 4, 2, 3000, 256, 0),
])
def test_fused_scan_on_degenerate_queries(scheme, G, Hkv, S, K, split_len, mode):
    """Queries that stress the fixed-point arithmetic and the selection: all zero (every score equal: the exact
    selection and its ties), a few distinct values (massive ties at the cut), and one huge element among many tiny ones
    per 64-channel group (the tiny ones keep few bits of the group's shared exponent; the softmax is peaked, so the
    23-bit weights are coarse against the sum of the weights).  Scores stay within 2e-5 and the top-k exact; o_hat,
    o_old and W within 6e-6 (on random queries: 3e-6; the measured worst case here is 4.4e-6 on isolated elements)."""
    from jetfire_amd import _lib
    lib = _lib.load()
    kb, vb, gs = {"k3v2": (3, 2, 64), "k4v4": (4, 4, 128), "k2v2": (2, 2, 64), "a2v2": (2, 2, 64)}[scheme]
    c = make_case(4242, 2, G * Hkv, Hkv, S, kb, vb, gs, lens=[S, S - 37], extra_blocks=1, k_asym=scheme.startswith("a"))
    q = c["q"]
    if mode == "zero_query":
        q[...] = 0
    elif mode == "few_values":
        q[...] = np.sign(q) * 0.5 * (np.abs(q) > 1.0)
    else:
        q[...] = torch.tensor(q * 0.01).to(torch.bfloat16).float().numpy()
        q[:, :, 5] = 8.0
        q[:, :, 70] = -8.0
    d = to_device(c)
    _lib.check(_lib.debug_hook("jf_debug_split_len")(split_len))
    try:
        out = [t.clone() for t in run_fused(scheme, c, d, S, K)]
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))
    check_against_oracle(scheme, c, S, K, out, atol_out=6e-6)


@pytest.mark.parametrize("gs", (128, 64))
def test_int2_single_call_names_of_the_reference(gs):
    """int2_fused_attn_topk and int2_fused_attn_topk_v1 (jetfire_vllm/csrc/int2_fused_attn_topk.cu:403-417,
    int2_fused_attn_topk_v1.cu:581-595): the reference's argument order with the zero-points fourth, four
    tensors back; scale tensors without the trailing group axis, as the reference passes them at group 128."""
    from jetfire_amd.kernels.int2_fused_attn_topk import load_int2_fused_attn_topk_ext
    from jetfire_amd.kernels.int2_fused_attn_topk_v1 import load_int2_fused_attn_topk_v1_ext
    scheme = "a2v2_g128" if gs == 128 else "a2v2"
    S, K = 700, 128
    c = make_case(91 + gs, 2, 8, 2, S, 2, 2, gs, lens=[333, 700], extra_blocks=3, k_asym=True)
    d = to_device(c)
    full = run_fused(scheme, c, d, S, K)
    check_against_oracle(scheme, c, S, K, full)
    sq = (lambda t: t.squeeze(-1)) if gs == 128 else (lambda t: t)
    for fn in (load_int2_fused_attn_topk_ext().int2_fused_attn_topk,
               load_int2_fused_attn_topk_v1_ext().int2_fused_attn_topk_v1):
        got = fn(d["q"], d["kd"], sq(d["ks"]), sq(d["kz"]), d["vd"], sq(d["vs"]), d["bt"], d["lens"], S, c["Hq"], c["Hkv"],
                 16, K, SCALE)
        assert len(got) == 4
        for a, b in zip(got, full[:4]):
            assert torch.equal(a, b)
    with pytest.raises(RuntimeError, match="top_k"):
        fn(d["q"], d["kd"], d["ks"], d["kz"], d["vd"], d["vs"], d["bt"], d["lens"], S, c["Hq"], c["Hkv"], 16, 96, SCALE)


@pytest.mark.parametrize("S,K,split_len", [(600, 64, 0), (10000, 256, 512)])
def test_fused_scan_ties_go_to_the_lower_position(S, K, split_len):
    # identical keys in every slot -> every score of a head is equal: winners are positions 0..K-1
    # (the second case goes through the two-stage merge)
    from jetfire_amd import _lib
    lib = _lib.load()
    c = make_case(5, 1, 8, 2, S, 3, 2, 64, ragged=False, shuffle=True)
    c["kd"][:] = c["kd"][:, :1]
    c["ks"][:] = c["ks"][:, :1]
    d = to_device(c)
    _lib.check(_lib.debug_hook("jf_debug_split_len")(split_len))
    try:
        out = run_fused("k3v2", c, d, S, K)
        idx = out[4].cpu().numpy()
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))
    assert (idx == np.arange(K)[None, None, :]).all()


def test_fused_scan_is_deterministic_and_matches_split_path():
    c = make_case(6, 2, 32, 8, 2048, 3, 2, 64)
    d = to_device(c)
    o = ops()
    a = run_fused("k3v2", c, d, 2048, 256)
    b2 = run_fused("k3v2", c, d, 2048, 256)
    for x, y in zip(a, b2):
        assert torch.equal(x, y)
    scores, idx, slots = o.int3_qk_scores_topk(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], 2048, 32, 8, 16, SCALE, 256)
    o_hat, o_old, W = o.int2_softmax_v_with_pre_corr_wvs2(scores, d["vd"], d["vs"], d["bt"], d["lens"], idx, 2048, 32, 8, 16, 256)
    np.testing.assert_allclose(a[7].cpu().numpy(), scores.cpu().numpy(), atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(a[0].cpu().numpy(), o_hat.cpu().numpy(), atol=3e-6, rtol=2e-5)


@pytest.mark.parametrize("scheme,B,Hq,Hkv,S,lens,K,split_len", [
    ("k3v2", 2, 32, 8, 2048, None, 256, 0),
    ("k4v4", 3, 32, 4, 512, [0, 257, 512], 256, 0),       # a zero-length row: out = bf16(0 + 0 * o_new - 0)
    ("k4v4", 1, 8, 2, 10000, [9000], 512, 768),           # two-stage merge: the epilogue runs in the final stage only
])
def test_fused_blend_epilogue_equals_the_separate_blend(scheme, B, Hq, Hkv, S, lens, K, split_len):
    """jf_fused_scan_topk_blend: the merge kernel's `out` is bit-equal to jf_blend_unnorm on its other outputs,
    and those are what jf_fused_scan_topk writes."""
    from jetfire_amd import _lib
    kb, vb, gs = {"k3v2": (3, 2, 64), "k4v4": (4, 4, 128)}[scheme]
    c = make_case(91 + S, B, Hq, Hkv, S, kb, vb, gs, lens=lens, extra_blocks=2)
    d = to_device(c)
    o = ops()
    g = torch.Generator(device="cuda").manual_seed(5)
    o_new = torch.randn(B, Hq, 128, generator=g, device="cuda").to(torch.bfloat16)
    out = torch.full_like(o_new, 7.0)
    lib = _lib.load()
    _lib.check(_lib.debug_hook("jf_debug_split_len")(split_len))
    try:
        plain = o.fused_attn_topk(scheme, d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"], d["lens"], S, Hq, Hkv, 16, K, SCALE)
        fused = o.fused_attn_topk(scheme, d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"], d["lens"], S, Hq, Hkv, 16, K, SCALE,
                                  blend=(o_new, out))
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))
    for x, y in zip(plain, fused):
        assert torch.equal(x, y)
    ref = o.blend_unnorm(fused[0], fused[2], fused[3], o_new)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    with pytest.raises(RuntimeError, match="bf16"):
        o.fused_attn_topk(scheme, d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"], d["lens"], S, Hq, Hkv, 16, K, SCALE,
                          blend=(o_new.float(), out))


@pytest.mark.parametrize("scheme,B,Hq,Hkv,S,lens,K", [
    ("k3v2", 2, 32, 8, 1024, None, 256),
    ("k4v4", 2, 32, 8, 1024, None, 256),
    ("k3v2", 2, 32, 4, 768, [700, 768], 256),             # the TP2 70B local-head geometry
    ("k4v4", 4, 8, 2, 32, [0, 1, 9, 17], 64),
    ("k3v4", 2, 32, 8, 1024, None, 256), ("k4v2", 2, 32, 4, 768, [700, 768], 256),
])
def test_fused_decode_step_end_to_end(scheme, B, Hq, Hkv, S, lens, K):
    """scan+top-k -> pinned hand-off -> CPU correction -> merge, checked against the oracle's whole step and the
    acceptance bar for attention outputs (max-abs 2e-2, mean-abs 1e-3 in bf16)."""
    kb, vb, gs = {"k3v2": (3, 2, 64), "k4v4": (4, 4, 128), "k3v4": (3, 4, 128), "k4v2": (4, 2, 128)}[scheme]
    c = make_case(80 + B + Hq, B, Hq, Hkv, S, kb, vb, gs, lens=lens)
    d = to_device(c)
    o = ops()
    o.set_cpu_attn_threads(4)
    h = o.CpuTopkHandoff(B, Hq, Hkv, K, bf16_tensor(c["K"]), bf16_tensor(c["V"]), SCALE)
    out = torch.empty(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    o_new = torch.empty_like(out)
    o_hat, slots, o_old, W, idx = o.fused_attn_topk(scheme, d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"],
                                                    d["lens"], S, Hq, Hkv, 16, K, SCALE)
    h.submit(d["q"], slots)
    h.wait(o_new)
    o.blend_unnorm_into(o_hat, o_old, W, o_new, out)
    torch.cuda.synchronize()
    r = O.decode_reference(c["q"], c["kd"], c["ks"], c["vd"], c["vs"], c["bt"], c["lens"], S, Hq, Hkv, 16, SCALE, K,
                           scheme, c["K"], c["V"])
    got = bf16_to_f32(out)
    np.testing.assert_allclose(got, r["out"], atol=6e-3, rtol=1.5e-2)
    err = np.abs(got - r["out"])
    assert err.max() <= 2e-2 and err.mean() <= 1e-3
    h.close()


def test_fused_step_replays_from_a_hip_graph():
    """scan + merge + blend captured once and replayed: every replay, with eager work and synchronisations in
    between, reproduces the eager result bit for bit (nothing in the path allocates or memsets per call)."""
    c = make_case(31, 2, 32, 8, 2048, 3, 2, 64)
    d = to_device(c)
    o = ops()
    o_new = torch.randn(2, 32, 128, device="cuda").to(torch.bfloat16)

    def step():
        o_hat, slots, o_old, W, idx = o.fused_attn_topk("k3v2", d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"],
                                                        d["lens"], 2048, 32, 8, 16, 256, SCALE)
        out = torch.empty(2, 32, 128, dtype=torch.bfloat16, device="cuda")
        o.blend_unnorm_into(o_hat, o_old, W, o_new, out)
        return o_hat, slots, idx, out

    ref = [t.clone() for t in step()]
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
    torch.cuda.current_stream().wait_stream(s)
    with torch.cuda.graph(g, stream=s):
        outs = step()
    for _ in range(3):
        for t in outs:
            t.fill_(0) if t.dtype != torch.int64 else t.fill_(-7)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, ref):
            assert torch.equal(got, want)
        eager = step()                      # eager work between the replays
        torch.cuda.synchronize()
        for got, want in zip(eager, ref):
            assert torch.equal(got, want)


@pytest.mark.parametrize("scheme,S,K,split_len", [("k3v2", 300, 64, 256), ("k4v4", 1500, 256, 512), ("k3v3", 700, 512, 256),
                                                  ("k2v4", 5000, 128, 1024)])
def test_many_rows_take_the_light_merge_with_identical_results(scheme, S, K, split_len):
    """More than two rows per CU with few candidates each run the merge with four wavefronts per row; its sums are
    arranged like the sixteen-wavefront shape's, so a batch gives bit for bit what its halves give alone (those are
    small enough for the regular shape), and the oracle's values.  (The split length is pinned: the planner's own
    choice depends on the batch size.)"""
    from jetfire_amd import _lib
    lib = _lib.load()
    kb, vb, gs = SCHEME_GEOMETRY[scheme]
    B, Hq, Hkv = 20, 32, 8                                    # 640 rows
    lens = [S - 7 * b for b in range(B)]
    c = make_case(300 + S, B, Hq, Hkv, S, kb, vb, gs, lens=lens)
    d = to_device(c)
    _lib.check(_lib.debug_hook("jf_debug_split_len")(split_len))
    try:
        whole = [t.clone() for t in run_fused(scheme, c, d, S, K)]
        for lo, hi in ((0, 10), (10, 20)):
            part = ops().fused_attn_topk(scheme, d["q"][lo:hi].contiguous(), d["kd"], d["ks"], d["vd"], d["vs"],
                                         d["bt"][lo:hi].contiguous(), d["lens"][lo:hi].contiguous(), S, Hq, Hkv, 16, K,
                                         SCALE, return_scores=True, return_stats=True)
            for a, b in zip(whole, part):
                assert torch.equal(a[lo:hi], b)
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))
    if S <= 1500:
        check_against_oracle(scheme, c, S, K, whole)


@pytest.mark.parametrize("scheme,kb,vb,gs", [("k4v4", 4, 4, 128), ("k3v2", 3, 2, 64)])
def test_fused_scan_addresses_the_top_of_a_4gb_pool(scheme, kb, vb, gs):
    """The largest pool the fused form addresses: 2^26 slots per kv-head (4 GB of 64-byte rows).  A small case whose
    pages sit in the last blocks of such a pool gives the outputs of the same case in a small pool, bit for bit,
    with the slots shifted; one slot more is rejected."""
    o = ops()
    S, K, Hq, Hkv = 700, 64, 4, 1
    c = make_case(77, 2, Hq, Hkv, S, kb, vb, gs, extra_blocks=2)
    d = to_device(c)
    small = o.fused_attn_topk(scheme, d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"], d["lens"], S, Hq, Hkv, 16, K,
                              SCALE, return_scores=True, return_stats=True)
    n_small = d["kd"].size(1)
    n_big = 1 << 26
    shift = n_big - n_small                                   # (a multiple of 16: whole blocks)
    big = {}
    for name in ("kd", "ks", "vd", "vs"):
        t = torch.zeros((Hkv, n_big) + tuple(d[name].shape[2:]), dtype=d[name].dtype, device="cuda")
        t[:, shift:] = d[name]
        big[name] = t
    bt_big = d["bt"] + shift // 16
    out = o.fused_attn_topk(scheme, d["q"], big["kd"], big["ks"], big["vd"], big["vs"], bt_big, d["lens"], S, Hq, Hkv, 16,
                            K, SCALE, return_scores=True, return_stats=True)
    for i, (a, b) in enumerate(zip(out, small)):
        if i == 1:                                            # topk_slots
            assert torch.equal(a, torch.where(b >= 0, b + shift, b))
        else:
            assert torch.equal(a, b)
    # one block more is refused before anything is launched (the argument check alone sees the slot count)
    from jetfire_amd import _lib
    lib = _lib.load()
    idx, slots, o_hat, o_old, W = out[4], out[1], out[0], out[2], out[3]
    ws = torch.empty(lib.jf_fused_workspace_bytes(10 * kb + vb, 2, Hq, Hkv, S, K), dtype=torch.uint8, device="cuda")
    rc = lib.jf_fused_scan_topk(10 * kb + vb, gs, d["q"].data_ptr(), big["kd"].data_ptr(), big["ks"].data_ptr(),
                                big["vd"].data_ptr(), big["vs"].data_ptr(), bt_big.data_ptr(), d["lens"].data_ptr(), 2, Hq,
                                Hkv, S, bt_big.size(1), n_big + 16, 16, SCALE, K, idx.data_ptr(), slots.data_ptr(),
                                o_hat.data_ptr(), o_old.data_ptr(), W.data_ptr(), None, None, None, ws.data_ptr(),
                                ws.numel(), None)
    assert rc != 0 and "num_slots" in lib.jf_last_error().decode()


def test_fused_scan_rejects_unsupported_arguments():
    c = make_case(9, 1, 8, 2, 64, 3, 2, 64)
    d = to_device(c)
    o = ops()
    with pytest.raises(RuntimeError):
        o.fused_attn_topk("k3v2", d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"], d["lens"], 64, 8, 2, 16, 48, SCALE)
    with pytest.raises(RuntimeError):
        o.fused_attn_topk("k3v2", d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"], d["lens"], 64, 8, 2, 32, 64, SCALE)
    with pytest.raises(RuntimeError):
        o.fused_attn_topk("k9", d["q"], d["kd"], d["ks"], d["vd"], d["vs"], d["bt"], d["lens"], 64, 8, 2, 16, 64, SCALE)
