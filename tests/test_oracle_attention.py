"""Pins the oracle's scoring, top-k, softmax-V, CPU correction and merge restatements
with closed forms, invariants, special cases and brute force (no formula retyping)."""
import json
import os

import numpy as np
import pytest

from oracle import jetfire_oracle as O

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_wire_vectors.json")))


def make_case(seed, B, Hq, Hkv, S, kbits, vbits, gs, ragged=True, shuffle=True):
    rng = np.random.default_rng(seed)
    nblk = B * ((S + 15) // 16)
    slots_total = nblk * 16
    K = O.bf16_round(rng.standard_normal((slots_total, Hkv, 128)).astype(np.float32))
    K[..., rng.permutation(128)[:4]] *= 8
    K = O.bf16_round(K)
    V = O.bf16_round(rng.standard_normal((slots_total, Hkv, 128)).astype(np.float32))
    q = O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32))
    kd, ks = O.quantize_and_pack(K.transpose(1, 0, 2), gs, kbits)
    vd, vs = O.quantize_and_pack(V.transpose(1, 0, 2), gs, vbits)
    bt = (rng.permutation(nblk) if shuffle else np.arange(nblk)).reshape(B, -1).astype(np.int64)
    lens = np.array([S - 13 * b if ragged else S for b in range(B)], dtype=np.int32)
    return dict(q=q, kd=kd, ks=ks, vd=vd, vs=vs, bt=bt, lens=lens, K=K.transpose(1, 0, 2).copy(),
                V=V.transpose(1, 0, 2).copy(), S=S, B=B, Hq=Hq, Hkv=Hkv)


@pytest.mark.parametrize("kbits,gs", [(3, 64), (2, 64), (2, 128), (4, 64), (4, 128)])
def test_bf16_score_model_one_hot_query_reads_one_dequantised_channel(kbits, gs):
    c = make_case(1, 2, 8, 2, 64, kbits, 2, gs)
    q = np.zeros_like(c["q"])
    q[:, :, 37] = 1.0
    sc = O.scores_bf16_model(q, c["kd"], c["ks"], c["bt"], c["lens"], 64, 8, 2, 16, 0.5, kbits, gs)
    khat = O.unpack(c["kd"], c["ks"], gs, kbits)
    slots = O.slots_from_block_table(c["bt"], 64)
    for b in range(2):
        S = c["lens"][b]
        for h in range(8):
            assert np.array_equal(sc[b, h, :S], khat[h // 4, slots[b, :S], 37] * np.float32(0.5))
            assert np.isneginf(sc[b, h, S:]).all()


def test_int8_score_model_agrees_with_validator_restatement_and_closed_form():
    c = make_case(2, 2, 8, 2, 128, 4, 4, 128)
    a = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], 128, 8, 2, 16, 128 ** -0.5)
    d = O.scores_int8_model_dense(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], 128, 8, 2, 16, 128 ** -0.5)
    valid = np.isfinite(d)
    assert np.array_equal(valid, np.isfinite(a))
    np.testing.assert_allclose(a[valid], d[valid], rtol=2e-6, atol=2e-7)
    # closed form: q = 127 * e_5 -> qi = 127 in group 0, qs = 1; score = 127*(nib-8)*ks*scale exactly
    q = np.zeros_like(c["q"])
    q[:, :, 5] = 127.0
    sc = O.scores_int8_model(q, c["kd"], c["ks"], c["bt"], c["lens"], 128, 8, 2, 16, 0.25)
    codes = O.decode_codes(c["kd"], 4).astype(np.float32) - 8
    ks = O.bf16_bits_to_f32(c["ks"])[..., 0]
    slots = O.slots_from_block_table(c["bt"], 128)
    S = c["lens"][1]
    exp = (np.float32(127.0) * codes[1, slots[1, :S], 5]) * ks[1, slots[1, :S]] * np.float32(0.25)
    assert np.array_equal(sc[1, 5, :S], exp.astype(np.float32))


def test_query_quantiser_matches_reference_rule():
    rng = np.random.default_rng(3)
    q = O.bf16_round((rng.standard_normal((3, 4, 128)) * 0.1).astype(np.float32))
    qi, qs = O.quantize_query_int8(q)
    assert qi.min() >= -128 and qi.max() <= 127
    assert (np.abs(qi).max(-1) == 127).all()                      # amax element maps to +-127
    deq = qi * qs[..., None]
    assert (np.abs(deq - q.reshape(3, 4, 4, 32)) <= qs[..., None] * 0.501).all()   # half a step, plus the reciprocal rounding
    z = np.zeros((1, 1, 128), dtype=np.float32)
    qi, qs = O.quantize_query_int8(z)
    assert (qs == np.float32(1e-12)).all() and (qi == 0).all()


def test_topk_matches_bruteforce_with_lower_index_tie_break():
    rng = np.random.default_rng(4)
    B, Hq, S, K = 2, 3, 50, 8
    sc = rng.integers(-3, 4, size=(B, Hq, S)).astype(np.float32)      # many exact ties
    sc[0, 0, 7] = -0.0
    sc[0, 0, 9] = 0.0
    lens = np.array([50, 37], dtype=np.int32)
    bt = rng.permutation(8).reshape(2, 4).astype(np.int64)
    idx, slots = O.topk_select(sc, lens, bt, S, K)
    for b in range(B):
        for h in range(Hq):
            n = lens[b]
            # python sort is stable: sort by descending key keeps ascending position inside ties
            cand = sorted(range(n), key=lambda i: -int(O.radix_key(sc[b, h, i:i + 1])[0]))[:K]
            assert sorted(cand) == list(idx[b, h])
            for j, p in enumerate(idx[b, h]):
                assert slots[b, h, j] == bt[b, p // 16] * 16 + p % 16


def test_topk_short_rows_emit_each_position_once_then_minus_one():
    # validate_runtime_edges.py:124-142
    sc = np.random.default_rng(5).standard_normal((1, 2, 32)).astype(np.float32)
    bt = np.array([[3, 1]], dtype=np.int64)
    for S in (0, 1, 9, 17):
        idx, slots = O.topk_select(sc, np.array([S], dtype=np.int32), bt, 32, 32)
        for h in range(2):
            assert list(idx[0, h, :S]) == list(range(S))
            assert (idx[0, h, S:] == -1).all() and (slots[0, h, S:] == -1).all()


def test_radix_key_is_order_preserving():
    v = np.array([-np.inf, -3.5, -1e-30, -0.0, 0.0, 1e-30, 2.0, np.inf], dtype=np.float32)
    k = O.radix_key(v).astype(np.int64)
    assert (np.diff(k) > 0).all()


@pytest.mark.parametrize("vbits,vg", [(2, 64), (3, 64), (3, 128), (4, 64)])
def test_softmax_v_invariants(vbits, vg):
    c = make_case(6, 2, 8, 2, 96, 3, vbits, vg)
    sc = O.scores_bf16_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], 96, 8, 2, 16, 128 ** -0.5, 3, vg)
    # K >= S: all positions selected -> W == 1, o_old == o_hat
    idx, _ = O.topk_select(sc, c["lens"], c["bt"], 96, 128)
    o_hat, o_old, W = O.softmax_v(sc, c["vd"], c["vs"], c["bt"], c["lens"], idx, 96, 8, 2, 16, vbits, vg)
    np.testing.assert_allclose(W, 1.0, atol=1e-6)
    np.testing.assert_allclose(o_old, o_hat, atol=1e-6)
    # uniform scores: o_hat is the plain mean of the dequantised V rows
    flat = np.where(np.isfinite(sc), np.float32(0.25), sc)
    o_hat, o_old, W = O.softmax_v(flat, c["vd"], c["vs"], c["bt"], c["lens"], None, 96, 8, 2, 16, vbits, vg)
    v0 = O.dequant(c["vd"], c["vs"], vbits, vg, bf16=False)
    slots = O.slots_from_block_table(c["bt"], 96)
    for b in range(2):
        S = c["lens"][b]
        np.testing.assert_allclose(o_hat[b, 5], v0[1, slots[b, :S]].mean(0), atol=2e-6)
    # partial top-k: 0 <= W <= 1 and W equals the softmax mass of the winners
    idx, _ = O.topk_select(sc, c["lens"], c["bt"], 96, 32)
    _, _, W = O.softmax_v(sc, c["vd"], c["vs"], c["bt"], c["lens"], idx, 96, 8, 2, 16, vbits, vg)
    assert (W > 0).all() and (W < 1).all()
    p = np.exp(sc[0, 0, :96].astype(np.float64))
    p /= p.sum()
    np.testing.assert_allclose(W[0, 0], p[idx[0, 0]].sum(), rtol=1e-6)


def test_softmax_v_zero_length_row_is_zero():
    c = make_case(7, 2, 4, 2, 32, 4, 4, 128, ragged=False)
    lens = np.array([0, 32], dtype=np.int32)
    sc = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], lens, 32, 4, 2, 16, 0.1)
    assert np.isneginf(sc[0]).all()
    m, iz = O.softmax_stats(sc, lens, 32)
    assert (m[0] == 0).all() and (iz[0] == 0).all()
    o_hat, o_old, W = O.softmax_v(sc, c["vd"], c["vs"], c["bt"], lens, None, 32, 4, 2, 16, 4, 128)
    assert (o_hat[0] == 0).all()


def test_int8_tile_model_tracks_dense_model():
    c = make_case(8, 1, 4, 1, 256, 4, 4, 128, ragged=False)
    sc = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], 256, 4, 1, 16, 128 ** -0.5)
    idx, _ = O.topk_select(sc, c["lens"], c["bt"], 256, 64)
    m, iz = O.softmax_stats(sc, c["lens"], 256)
    d = O.softmax_v(sc, c["vd"], c["vs"], c["bt"], c["lens"], idx, 256, 4, 1, 16, 4, 128)
    t = O.softmax_v_int8_tiles(sc, m, iz, c["vd"], c["vs"], c["bt"], c["lens"], idx, 256, 4, 1, 16)
    np.testing.assert_allclose(t[0], d[0], atol=3e-3)            # validate_runtime.py:173-176
    np.testing.assert_allclose(t[1], d[1], atol=3e-6, rtol=3e-6)
    np.testing.assert_allclose(t[2], d[2], atol=3e-6, rtol=3e-6)


def test_int8_tile_model_equals_the_validators_restatement_on_aligned_contexts():
    """scripts/validate_runtime_edges.py:146-164 models the tile arithmetic for contexts that are multiples of 256
    (eight ranges aligned to the 32-position tiles) as: reshape(P * v_scale) to (..., 32), scale = amax / 127,
    round(weighted / scale).clamp(+-127) * scale, then a dense contraction with the V codes.  Restated here with
    numpy and compared with the oracle's tile walk."""
    B, Hq, Hkv, S = 2, 4, 2, 512
    c = make_case(18, B, Hq, Hkv, S, 4, 4, 128, ragged=False)
    sc = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, 128 ** -0.5)
    m, iz = O.softmax_stats(sc, c["lens"], S)
    got, _, _ = O.softmax_v_int8_tiles(sc, m, iz, c["vd"], c["vs"], c["bt"], c["lens"], None, S, Hq, Hkv, 16)
    slots = O.slots_from_block_table(c["bt"], S, 16)
    codes = O.decode_codes(c["vd"], 4).astype(np.float64) - 8
    vs = O.bf16_bits_to_f32(c["vs"]).reshape(Hkv, -1)
    for b in range(B):
        for h in range(Hq):
            hk = h // (Hq // Hkv)
            p = (np.exp((sc[b, h] - m[b, h]).astype(np.float64)) * float(iz[b, h])).astype(np.float32)
            weighted = (p * vs[hk, slots[b]]).astype(np.float32).reshape(-1, 32)
            amax = np.abs(weighted).max(-1, keepdims=True)
            tile_scale = (amax / np.float32(127)).astype(np.float32)
            inverse = np.where(tile_scale > 0, np.float32(1) / np.where(tile_scale > 0, tile_scale, 1), 0).astype(np.float32)
            qw = (np.clip(np.rint((weighted * inverse).astype(np.float32)), -127, 127) * tile_scale).reshape(-1)
            want = qw.astype(np.float64) @ codes[hk, slots[b]]
            np.testing.assert_allclose(got[b, h], want, atol=3e-6, rtol=3e-6)


def test_int8_tile_model_tile_origin_on_unaligned_ranges():
    """Brute force where ceil(S / 8) = 25 is not a page multiple: every range's tiles are page pairs counted from
    the page of its first position (int8tc_softmax_v_fused.cu:1052,1178), restricted to the range (:1218).  The
    range [25, 50) is therefore TWO tiles, [25, 48) and [48, 50), not the single tile a walk in steps of 32 from
    position 25 would make; the two give different sums because each tile has its own scale."""
    S, Hq, Hkv = 200, 1, 1
    c = make_case(19, 1, Hq, Hkv, S, 4, 4, 128, ragged=False)
    rng = np.random.default_rng(4)
    sc = rng.standard_normal((1, 1, S)).astype(np.float32) * 2
    m, iz = O.softmax_stats(sc, c["lens"], S)
    got, _, _ = O.softmax_v_int8_tiles(sc, m, iz, c["vd"], c["vs"], c["bt"], c["lens"], None, S, Hq, Hkv, 16)
    slots = O.slots_from_block_table(c["bt"], S, 16)[0]
    codes = O.decode_codes(c["vd"], 4).astype(np.float64)[0] - 8
    vs = O.bf16_bits_to_f32(c["vs"]).reshape(Hkv, -1)[0]
    p = (np.exp((sc[0, 0] - m[0, 0]).astype(np.float64)) * float(iz[0, 0])).astype(np.float32)

    def walk(origin_of):
        total = np.zeros(128)
        for r in range(8):
            s0, s1 = 25 * r, min(25 * r + 25, S)
            for tile0 in range(origin_of(s0), s1, 32):
                pos = [t for t in range(tile0, tile0 + 32) if s0 <= t < s1]
                if not pos:
                    continue
                pv = (p[pos] * vs[slots[pos]]).astype(np.float32)
                rs = np.float32(np.abs(pv).max() / np.float32(127))
                if rs > 0:
                    pq = np.clip(np.rint(pv * (np.float32(1) / rs)), -127, 127)
                    total += (pq @ codes[slots[pos]]) * float(rs)
        return total

    np.testing.assert_allclose(got[0, 0], walk(lambda s0: (s0 // 16) * 16), atol=1e-6)
    assert np.abs(got[0, 0] - walk(lambda s0: s0)).max() > 1e-5     # the other tiling is a different function


def test_cpu_correction_special_cases():
    c = make_case(9, 2, 8, 2, 64, 3, 2, 64, ragged=False)
    hm = O.head_map(2, 8, 4, 1)
    ts = np.full((2, 8, 1), 5, dtype=np.int64)
    out = O.cpu_topk_attn(c["q"], c["K"], c["V"], hm, ts, 0.1)
    for h in range(8):                                            # K=1 -> the bf16 V row itself
        assert np.array_equal(out[0, h], c["V"][h // 4, 5])
    ts = np.full((2, 8, 4), -1, dtype=np.int64)                   # all invalid -> zeros
    assert (O.cpu_topk_attn(c["q"], c["K"], c["V"], O.head_map(2, 8, 4, 4), ts, 0.1) == 0).all()
    ts[:, :, 2] = 7
    ts[:, :, 3] = 10 ** 9                                         # out of range is masked too
    out = O.cpu_topk_attn(c["q"], c["K"], c["V"], O.head_map(2, 8, 4, 4), ts, 0.1)
    assert np.array_equal(out[1, 3], c["V"][0, 7])


def test_blend_special_cases_and_end_to_end_identity():
    rng = np.random.default_rng(10)
    hat = rng.standard_normal((2, 4, 128)).astype(np.float32)
    z = np.zeros_like(hat)
    assert np.array_equal(O.blend_unnorm(hat, z, np.zeros((2, 4), np.float32), z), O.bf16_round(hat))
    # shadow == dequantised cache and K >= S  =>  corrected output == o_new (up to fp32/bf16 rounding)
    c = make_case(11, 1, 4, 1, 48, 3, 2, 64, ragged=False)
    kshadow = O.unpack(c["kd"], c["ks"], 64, 3)
    vshadow = O.dequant(c["vd"], c["vs"], 2, 64, bf16=False)      # V2 codes*bf16 scale are bf16-exact
    assert np.array_equal(vshadow, O.bf16_round(vshadow))
    r = O.decode_reference(c["q"], c["kd"], c["ks"], c["vd"], c["vs"], c["bt"], c["lens"], 48, 4, 1, 16,
                           128 ** -0.5, 64, "k3v2", kshadow, vshadow)
    np.testing.assert_allclose(r["W"], 1.0, atol=1e-6)
    np.testing.assert_allclose(r["out"], r["o_new"], atol=2e-2 * np.abs(r["o_new"]).max())
    assert np.abs(r["out"] - r["o_new"]).max() <= 2 ** -7 * np.abs(r["o_new"]).max() + 1e-6


def test_reference_select_top_k_table_and_head_map():
    g = GOLD["select_top_k"]
    for length, expected in g["cases"]:
        assert O.select_top_k(g["requested"], length, tuple(g["supported"])) == expected
    for req, length, sup in g["rejected"]:
        assert O.select_top_k(req, length, tuple(sup)) is None
    hm = O.head_map(2, 32, 8, 256)                                # tests/test_runtime_edge_cases.py:29-35
    assert hm.shape == (2, 32, 256) and hm.flags["C_CONTIGUOUS"]
    for h in range(32):
        assert (hm[:, h] == h // 8).all()


@pytest.mark.parametrize("kbits,vbits,gs", [(3, 2, 64), (4, 4, 128)])
def test_torch_cpu_path_agrees_with_the_numpy_oracle(kbits, vbits, gs):
    """The torch restatement timed as the CPU baseline: its unpack is bit-equal to the oracle's bf16
    dequant, and its dense attention + top-k agree with the oracle's bf16-dequant model."""
    import torch
    from oracle import torch_cpu_path as T
    from tests.helpers import bf16_tensor, bits_to_bf16, bf16_to_bits
    B, Hq, Hkv, S, K = 1, 8, 2, 160, 32
    c = make_case(21, B, Hq, Hkv, S, kbits, vbits, gs, ragged=False, shuffle=False)
    kd, vd = torch.from_numpy(c["kd"]), torch.from_numpy(c["vd"])
    ks, vs = bits_to_bf16(c["ks"]), bits_to_bf16(c["vs"])
    for data, sc, nb, npd, nps in ((kd, ks, kbits, c["kd"], c["ks"]), (vd, vs, vbits, c["vd"], c["vs"])):
        got = bf16_to_bits(T.unpack(data, sc, gs, nb))
        want = O.f32_to_bf16_bits(O.dequant(npd, nps, nb, gs, bf16=True))
        assert np.array_equal(got, want)
    o_hat, idx = T.decode_path(bf16_tensor(c["q"]), kd[None, :, :S], ks[None, :, :S], vd[None, :, :S], vs[None, :, :S],
                               gs, kbits, vbits, K)
    ref_sc = O.scores_bf16_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, 128 ** -0.5, kbits, gs)
    ridx, _ = O.topk_select(ref_sc, c["lens"], c["bt"], S, K)
    # same winners unless a margin is inside fp32 accumulation noise
    for h in range(Hq):
        cut = np.sort(ref_sc[0, h])[-K]
        clear = [i for i in ridx[0, h] if ref_sc[0, h, i] > cut + 1e-5]
        assert set(clear) <= set(idx[0, h].tolist())
    # o_hat: the oracle's Stage B dequantises V without the bf16 rounding; compare against the bf16-rounded V
    vhat = O.dequant(c["vd"], c["vs"], vbits, gs, bf16=True)
    p = np.exp(ref_sc[0].astype(np.float64) - ref_sc[0].max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("hs,hsd->hd", p, vhat[np.arange(Hq) // (Hq // Hkv)][:, :S].astype(np.float64))
    np.testing.assert_allclose(o_hat[0].numpy(), want, atol=2e-5, rtol=1e-4)


def test_torch_int8_q_restatement_is_bit_equal_to_the_oracle():
    """oracle/torch_cpu_path.int8_q_scores (used on the GPU at full context lengths) against scores_int8_model."""
    import torch
    from oracle import torch_cpu_path as T
    from tests.helpers import bf16_tensor, bits_to_bf16
    B, Hq, Hkv, S = 2, 8, 2, 300
    c = make_case(23, B, Hq, Hkv, S, 4, 4, 128, ragged=True)
    ref = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, 128 ** -0.5)
    slots = O.slots_from_block_table(c["bt"], S, 16)
    G = Hq // Hkv
    for b in range(B):
        n = int(c["lens"][b])
        for h in range(Hkv):
            sl = torch.from_numpy(slots[b, :n])
            got = T.int8_q_scores(bf16_tensor(c["q"][b, h * G:(h + 1) * G]), torch.from_numpy(c["kd"][h])[sl],
                                  bits_to_bf16(c["ks"][h])[sl], 128 ** -0.5).numpy()
            assert np.array_equal(got.view(np.uint32), ref[b, h * G:(h + 1) * G, :n].view(np.uint32))
