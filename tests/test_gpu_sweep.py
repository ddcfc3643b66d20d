"""Seeded sweep of the fused scan over randomly drawn geometries (GQA group, batch, ragged lengths, correction
width, forced split lengths, block-table permutations) for the fused schemes, each case checked against
the oracle exactly as the hand-picked cases are."""
import numpy as np
import pytest

from tests.helpers import make_case, to_device
from tests.test_gpu_fused import check_against_oracle, run_fused

pytestmark = pytest.mark.gpu

SCHEMES = {"k3v2": (3, 2, 64), "k3v2_g128": (3, 2, 128), "k4v4": (4, 4, 128), "k3v4": (3, 4, 128), "k4v2": (4, 2, 128),
           "k2v2": (2, 2, 64), "k2v2_g128": (2, 2, 128), "k2v4": (2, 4, 128),
           "k3v3": (3, 3, 64), "k3v3_g128": (3, 3, 128), "k2v3": (2, 3, 64), "k4v3": (4, 3, 128),
           "a2v2": (2, 2, 64), "a2v2_g128": (2, 2, 128), "a2v3": (2, 3, 64), "a2v4": (2, 4, 128),
           "k3v4_g64": (3, 4, 64), "a2v4_g64": (2, 4, 64), "b4v4": (4, 4, 64), "b4v2_g128": (4, 2, 128)}


def _draw(seed):
    rng = np.random.default_rng(1000 + seed)
    scheme = list(SCHEMES)[seed % len(SCHEMES)]
    G = int(rng.choice([1, 2, 4, 8, 16, 3, 5, 6, 7, 12]))
    Hkv = int(rng.choice([1, 2, 4])) if G < 12 else 1
    B = int(rng.integers(1, 4))
    S = int(rng.choice([48, 200, 777, 1500, 2600, 4100]))
    lens = [int(x) for x in rng.integers(0, S + 1, size=B)]
    lens[int(rng.integers(0, B))] = S                       # at least one full-length row
    K = int(rng.choice([32, 64, 128, 256, 512, 1024, 2048, 4096]))
    split = int(rng.choice([0, 0, 256, 512, 1024]))
    return scheme, B, G * Hkv, Hkv, S, lens, K, split


@pytest.mark.parametrize("seed", range(160))
def test_fused_scan_random_geometry(seed):
    from jetfire_amd import _lib
    scheme, B, Hq, Hkv, S, lens, K, split = _draw(seed)
    kb, vb, gs = SCHEMES[scheme]
    c = make_case(500 + seed, B, Hq, Hkv, S, kb, vb, gs, lens=lens, extra_blocks=int(seed % 4),
                  k_asym=scheme.startswith("a"))
    d = to_device(c)
    lib = _lib.load()
    print(f"case: {scheme} B={B} Hq={Hq} Hkv={Hkv} S={S} lens={lens} K={K} split={split}", flush=True)
    _lib.check(_lib.debug_hook("jf_debug_split_len")(split))
    try:
        out = [t.clone() for t in run_fused(scheme, c, d, S, K)]
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))
    check_against_oracle(scheme, c, S, K, out)


@pytest.mark.parametrize("seed", range(0, 64, 2))
def test_two_call_form_random_geometry(seed):
    """The same draw through the reference-named Stage A and Stage B operators (run on the kernels of the one-pass
    form without the other stage): every output bit-equal to the one-pass form's, which the test above pins to the
    oracle."""
    import torch
    from jetfire_amd import _lib, ops
    scheme, B, Hq, Hkv, S, lens, K, split = _draw(seed)
    if scheme not in ("k3v2", "k3v2_g128", "k4v4", "k3v3", "k3v3_g128"):   # the operator pairs below: K3V2, K3V3, K4V4
        scheme = "k3v2" if seed % 4 == 0 else "k4v4"
    if scheme == "k4v4" and K < 64:
        K = 64                                              # int8tc_qk_scores_topk_stats starts at 64
    kb, vb, gs = SCHEMES[scheme]
    c = make_case(500 + seed, B, Hq, Hkv, S, kb, vb, gs, lens=lens, extra_blocks=int(seed % 4))
    d = to_device(c)
    lib = _lib.load()
    print(f"case: {scheme} B={B} Hq={Hq} Hkv={Hkv} S={S} lens={lens} K={K} split={split}", flush=True)
    assert ops.get_split_impl() == "fast"
    _lib.check(_lib.debug_hook("jf_debug_split_len")(split))
    try:
        o_hat, slots, o_old, W, idx, m, iz, scores = [t.clone() for t in run_fused(scheme, c, d, S, K)]
        args = (d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, 128 ** -0.5, K)
        if kb == 3:
            sc2, idx2, slots2 = ops.int3_qk_scores_topk(*args)
            stage_b = ops.int2_softmax_v_with_pre_corr_wvs2 if vb == 2 else ops.int3_softmax_v_with_pre_corr_wvs2
        else:
            sc2, idx2, slots2, m2, iz2 = ops.int8tc_qk_scores_topk_stats(*args)
            assert torch.equal(m2, m) and torch.equal(iz2, iz)
            stage_b = ops.int4_softmax_v_with_pre_corr_wvs2_scores
        assert torch.equal(sc2.view(torch.int32), scores.view(torch.int32))
        assert torch.equal(idx2, idx) and torch.equal(slots2, slots)
        o_hat2, o_old2, W2 = stage_b(sc2, d["vd"], d["vs"], d["bt"], d["lens"], idx2, S, Hq, Hkv, 16, K)
    finally:
        _lib.check(_lib.debug_hook("jf_debug_split_len")(0))
    assert torch.equal(o_hat2, o_hat) and torch.equal(o_old2, o_old) and torch.equal(W2, W)
