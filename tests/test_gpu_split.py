"""GPU parity of the split-form operators (pack, Stage A, top-k, Stage B, merge, hand-off) against the
CPU oracle.  Bit-exact for packed bytes, scale bits, INT4-key scores, top-k indices/slots and the merge;
fp32 accumulation-order tolerances (the reference's own, scripts/validate_runtime.py:147-195) elsewhere."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import jetfire_oracle as O
from tests.helpers import bf16_tensor, bf16_to_bits, bf16_to_f32, bits_to_bf16, make_case, to_device

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_wire_vectors.json")))


def ops():
    from jetfire_amd import ops as _ops
    return _ops


# ------------------------------------------------------------------ pack


@pytest.mark.parametrize("gs", GOLD["group_sizes"])
@pytest.mark.parametrize("vec", GOLD["vectors"], ids=lambda v: f"int{v['bits']}")
def test_pack_reference_wire_vectors(vec, gs):
    bits, values, planes = vec["bits"], vec["values"], vec["planes"]
    x = torch.tensor(values, dtype=torch.bfloat16).repeat(128 // len(values)).view(1, 1, 128).cuda()
    P = 128 * bits // 8
    data = torch.zeros(1, 4, P, dtype=torch.uint8, device="cuda")
    scales = torch.zeros(1, 4, 128 // gs, dtype=torch.bfloat16, device="cuda")
    getattr(ops(), f"fused_quant_write_int{bits}_sym")(x, torch.tensor([2], device="cuda"), data, scales, gs)
    repeats = 128 // (8 if bits == 3 else 8 // bits)
    expected = torch.tensor([b for b in planes for _ in range(repeats)], dtype=torch.uint8)
    assert torch.equal(data[0, 2].cpu(), expected)
    assert torch.equal(scales[0, 2].cpu(), torch.ones(128 // gs, dtype=torch.bfloat16))
    assert int(data[0, [0, 1, 3]].abs().sum()) == 0


@pytest.mark.parametrize("bits", (2, 3, 4))
@pytest.mark.parametrize("gs", (32, 64, 128))
def test_pack_bit_exact_scatter_masked_and_strided(bits, gs):
    rng = np.random.default_rng(100 * bits + gs)
    T, H = 257, 3
    xn = O.bf16_round((rng.standard_normal((T, H, 128)) * 10 ** rng.uniform(-3, 2, (T, H, 1))).astype(np.float32))
    xn[..., rng.permutation(128)[:4]] *= 8
    xn[5] = 0.0                                                   # all-zero rows: scale clamps at 1e-8
    xn[7, 0, :64] = np.array([0.5, 1.5, 2.5, -0.5] * 16)          # exact ties
    xn = O.bf16_round(xn)
    big = torch.zeros(T + 1, H + 1, 256, dtype=torch.bfloat16)
    big[:T, :H, :128] = bf16_tensor(xn)
    big[T, :H, :128] = bf16_tensor(xn[0])
    x = big.cuda()[:, :H, :128]                                   # strided view, last dim contiguous
    slots_np = np.concatenate([rng.permutation(T), [-1]]).astype(np.int64)
    P = 128 * bits // 8
    data = torch.full((H, T + 1, P), 0xA5, dtype=torch.uint8, device="cuda")
    scales = torch.zeros(H, T + 1, 128 // gs, dtype=torch.bfloat16, device="cuda")
    getattr(ops(), f"fused_quant_write_int{bits}_sym")(x, torch.from_numpy(slots_np).cuda(), data, scales, gs)
    ref_d, ref_s = O.quantize_and_pack(xn, gs, bits)              # (T, H, ...)
    got_d = data.cpu().numpy()[:, slots_np[:T]].transpose(1, 0, 2)
    got_s = bf16_to_bits(scales)[:, slots_np[:T]].transpose(1, 0, 2)
    assert np.array_equal(got_s, ref_s)
    assert np.array_equal(got_d, ref_d)
    assert bool((data[:, T] == 0xA5).all())                       # the masked token wrote nothing


@pytest.mark.parametrize("bits", (2, 3, 4))
def test_pack_rounding_is_exact_for_every_mantissa_pair(bits):
    """The pack kernel replaces the division by the scale with a reciprocal and one residual correction; this
    sweeps every (group maximum, element) mantissa pair over the binades where the quotient can reach a code
    boundary (ties included), at several magnitudes, and compares the bytes with the oracle's true division."""
    gs = 64
    qm = (1 << (bits - 1)) - 1
    # elements: every bf16 value in [2^-5, 2), both signs, plus zero
    mags = (np.arange(1 << 7, dtype=np.uint32)[None, :] | ((np.arange(122, 128, dtype=np.uint32)[:, None]) << 7)).reshape(-1)
    elems = np.concatenate([mags, mags | 0x8000, [0]]).astype(np.uint16)
    elems_f = O.bf16_bits_to_f32(elems)                                          # 1537 values, |x| < 2
    rows = []
    for e_a in (127, 128):                                                       # group maxima in [1, 4): scales in [1/qm, 4/qm)
        for m_a in range(128):
            a = O.bf16_bits_to_f32(np.array([(e_a << 7) | m_a], dtype=np.uint16))[0]
            vals = elems_f[np.abs(elems_f) <= a]
            pad = (-len(vals)) % (gs - 1)
            vals = np.concatenate([vals, np.zeros(pad, np.float32)]).reshape(-1, gs - 1)
            grp = np.concatenate([np.full((len(vals), 1), a, np.float32), vals], axis=1)   # (n, 64): maximum first
            if len(grp) % 2:
                grp = np.concatenate([grp, grp[:1]])
            rows.append(grp.reshape(-1, 128))
    base = np.concatenate(rows)                                                  # (T0, 128)
    xs = [base * np.float32(sc) for sc in (1.0, 2.0 ** -9, 2.0 ** 11, 3.0)]      # x3: other scale mantissas after bf16 rounding
    xn = O.bf16_round(np.concatenate(xs)).astype(np.float32)[:, None, :]         # (T, 1, 128)
    T = xn.shape[0]
    P = 128 * bits // 8
    data = torch.zeros(1, T, P, dtype=torch.uint8, device="cuda")
    scales = torch.zeros(1, T, 128 // gs, dtype=torch.bfloat16, device="cuda")
    slots = torch.arange(T, dtype=torch.int64, device="cuda")
    getattr(ops(), f"fused_quant_write_int{bits}_sym")(bf16_tensor(xn).cuda(), slots, data, scales, gs)
    ref_d, ref_s = O.quantize_and_pack(xn, gs, bits)
    assert np.array_equal(bf16_to_bits(scales)[0], ref_s[:, 0])
    assert np.array_equal(data.cpu().numpy()[0], ref_d[:, 0])
    codes = O.decode_codes(ref_d[:, 0], bits)
    assert codes.min() == 1 and codes.max() == 2 * qm + 1                        # both ends of the code range occur


@pytest.mark.parametrize("gs", (32, 64, 128))
def test_asymmetric_int2_pack_and_scores(gs):
    """fused_quant_write_int2_asym bit-exact against the oracle's quantize_and_pack_asym (codes, scale and
    zero-point bits; scattered, masked, strided), then int2_qk_scores with those zero-points against the
    oracle's bf16(fma(code - 2, scale, zp)) model."""
    rng = np.random.default_rng(40 + gs)
    T, H, nslots = 203, 4, 256
    wide = O.bf16_round((rng.standard_normal((T, H, 136)) * 1.3 + rng.standard_normal((T, H, 1))).astype(np.float32))
    wide[3, 1, :128] = 0.25                                              # a constant row: the 1e-8 floor
    x = wide[..., :128]
    slots = rng.permutation(nslots)[:T].astype(np.int64)
    slots[::29] = -1
    keep = slots >= 0
    data = torch.zeros(H, nslots, 32, dtype=torch.uint8, device="cuda")
    sc = torch.zeros(H, nslots, 128 // gs, dtype=torch.bfloat16, device="cuda")
    zp = torch.zeros_like(sc)
    o = ops()
    o.fused_quant_write_int2_asym(bf16_tensor(wide).cuda()[..., :128], torch.from_numpy(slots).cuda(), data, sc, zp, gs)
    rd, rs, rz = O.quantize_and_pack_asym(x, gs, 2)
    got_d, got_s, got_z = data.cpu().numpy(), bf16_to_bits(sc), bf16_to_bits(zp)
    assert np.array_equal(got_d[:, slots[keep]].transpose(1, 0, 2), rd[keep])
    assert np.array_equal(got_s[:, slots[keep]].transpose(1, 0, 2), rs[keep])
    assert np.array_equal(got_z[:, slots[keep]].transpose(1, 0, 2), rz[keep])
    untouched = np.setdiff1d(np.arange(nslots), slots[keep])
    assert not got_d[:, untouched].any() and not got_s[:, untouched].any()
    if gs == 32:
        return                                                           # Stage A takes one or two scale groups per row
    # scores over the rows just written: one sequence whose positions are the kept slots in order
    order = np.sort(slots[keep])
    S = (len(order) // 16) * 16
    blocks = np.arange(nslots // 16, dtype=np.int64)[None, :]
    lens = np.array([S - 5], np.int32)
    Hq = 8
    q = O.bf16_round((rng.standard_normal((1, Hq, 128)) / np.sqrt(128)).astype(np.float32))
    scores = o.int2_qk_scores(bf16_tensor(q).cuda(), data, sc, zp, torch.from_numpy(blocks).cuda(),
                              torch.from_numpy(lens).cuda(), S, Hq, H, 16, 0.11)
    ref = O.scores_bf16_model(q, got_d, got_s, blocks, lens, S, Hq, H, 16, 0.11, 2, gs, k_zp_bits=got_z)
    got = scores.cpu().numpy()
    valid = np.isfinite(ref)
    assert np.array_equal(np.isneginf(got), ~valid)
    np.testing.assert_allclose(got[valid], ref[valid], atol=2e-5, rtol=2e-5)
    # an unaligned token view is refused, not mis-read
    with pytest.raises(RuntimeError, match="16-byte"):
        o.fused_quant_write_int2_asym(bf16_tensor(wide).cuda()[..., 2:130], torch.from_numpy(slots).cuda(), data, sc, zp, gs)


@pytest.mark.parametrize("gs", (32, 64, 128))
@pytest.mark.parametrize("bits", (2, 3, 4))
def test_whole_tensor_quantise_and_unpack_match_the_oracle(bits, gs):
    """The reference's tensor-level API (kernels/intN_pack.py:60-107,227-311) through the loader module of its
    name: packed bytes, scale bits and the dequantised bf16 values bit-exact against the oracle, for a
    tensor with several leading dimensions, an odd row count and rows that hit the clamp."""
    from jetfire_amd.kernels import intN_pack as P
    rng = np.random.default_rng(100 * bits + gs)
    x = O.bf16_round((rng.standard_normal((3, 5, 7, 128)) * np.exp(rng.standard_normal((3, 5, 7, 1)))).astype(np.float32))
    x[0, 0, 0] = 0.0
    x[1, 2, 3, ::2] = 0.5                                   # exact halves of the scale: round-half-even ties
    xd = bf16_tensor(x).cuda()
    data, scales = P.quantize_and_pack(xd, group_size=gs, nbits=bits)
    rd, rs = O.quantize_and_pack(x, gs, bits)
    assert data.shape == (3, 5, 7, P.packed_dim(128, bits)) and scales.shape == (3, 5, 7, 128 // gs)
    assert np.array_equal(data.cpu().numpy(), rd) and np.array_equal(bf16_to_bits(scales), rs)
    back = P.unpack(data, scales, group_size=gs, nbits=bits)
    assert back.shape == x.shape and back.dtype == torch.bfloat16
    assert np.array_equal(bf16_to_bits(back), O.f32_to_bf16_bits(O.unpack(rd, rs, gs, bits)))
    # rows that are a slice of a wider tensor (part of one kv-head of a cache)
    cache = torch.zeros(4, 40, P.packed_dim(128, bits), dtype=torch.uint8, device="cuda")
    cache[2, :35] = data.view(-1, data.shape[-1])[:35]
    sc = torch.ones(4, 40, 128 // gs, dtype=torch.bfloat16, device="cuda")
    sc[2, :35] = scales.view(-1, scales.shape[-1])[:35]
    part = P.unpack(cache[2, 3:35], sc[2, 3:35], group_size=gs, nbits=bits)
    assert torch.equal(part, back.view(-1, 128)[3:35])
    # nothing to do
    e_d, e_s = P.quantize_and_pack(xd[:0], group_size=gs, nbits=bits)
    assert e_d.shape == (0, 5, 7, P.packed_dim(128, bits)) and P.unpack(e_d, e_s, gs, bits).shape == (0, 5, 7, 128)


@pytest.mark.parametrize("gs", (32, 64, 128))
def test_whole_tensor_asymmetric_int2_and_unpack_with_zero_points(gs):
    from jetfire_amd.kernels import fused_quantize as FQ, intN_pack as P
    rng = np.random.default_rng(300 + gs)
    x = O.bf16_round((rng.standard_normal((11, 3, 128)) * 0.7 + rng.standard_normal((11, 3, 1))).astype(np.float32))
    xd = bf16_tensor(x).cuda()
    data, scales, zps = P.quantize_and_pack_asym(xd, group_size=gs, nbits=2)
    rd, rs, rz = O.quantize_and_pack_asym(x, gs, 2)
    assert np.array_equal(data.cpu().numpy(), rd)
    assert np.array_equal(bf16_to_bits(scales), rs) and np.array_equal(bf16_to_bits(zps), rz)
    back = P.unpack(data, scales, group_size=gs, nbits=2, zps=zps)
    assert np.array_equal(bf16_to_bits(back), O.f32_to_bf16_bits(O.unpack(rd, rs, gs, 2, zp_bits=rz)))
    # the one-launch names of the reference (kernels/fused_quantize.py:214-284) are the same functions
    d2, s2, z2 = FQ.fused_quantize_and_pack_int2_asym(xd, gs)
    assert torch.equal(d2, data) and torch.equal(s2, scales) and torch.equal(z2, zps)
    d3, s3 = FQ.fused_quantize_and_pack_int2(xd, gs)
    rd3, rs3 = O.quantize_and_pack(x, gs, 2)
    assert np.array_equal(d3.cpu().numpy(), rd3) and np.array_equal(bf16_to_bits(s3), rs3)
    with pytest.raises(NotImplementedError):
        P.quantize_and_pack_asym(xd, group_size=gs, nbits=4)


@pytest.mark.parametrize("bits", (3, 4))
def test_unpack_with_zero_points_of_wider_codes_rounds_twice(bits):
    """Zero-points over INT3 / INT4 codes have no writer here, but unpack takes them as the reference does;
    with 3- and 4-bit codes the product needs more than bf16's 8 bits, so the two roundings show."""
    from jetfire_amd.kernels import intN_pack as P
    rng = np.random.default_rng(50 + bits)
    codes = rng.integers(0, 1 << bits, size=(97, 128)).astype(np.uint8)
    data = O.pack_codes(codes, bits)
    sb = O.f32_to_bf16_bits((np.exp(rng.standard_normal((97, 2))) * (1 + 2.0 ** -7)).astype(np.float32))
    zb = O.f32_to_bf16_bits(rng.standard_normal((97, 2)).astype(np.float32))
    got = P.unpack(torch.from_numpy(data).cuda(), bits_to_bf16(sb).cuda(), 64, bits, zps=bits_to_bf16(zb).cuda())
    assert np.array_equal(bf16_to_bits(got), O.f32_to_bf16_bits(O.unpack(data, sb, 64, bits, zp_bits=zb)))


def test_unpack_refuses_what_it_cannot_read():
    from jetfire_amd.kernels import intN_pack as P
    d = torch.zeros(4, 64, dtype=torch.uint8, device="cuda")
    s = torch.ones(4, 1, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="data must be"):
        P.unpack(d, s, 128, 3)
    with pytest.raises(RuntimeError, match="scales must be"):
        P.unpack(d, s, 64, 4)
    with pytest.raises(RuntimeError, match="Unsupported nbits"):
        P.unpack(d, s, 128, 8)
    with pytest.raises(RuntimeError, match="bf16"):
        P.quantize_and_pack(torch.zeros(2, 128, device="cuda"), 128, 4)


def test_pack_int4_kv_single_launch_matches_two_launches():
    rng = np.random.default_rng(7)
    T, H = 70, 8
    k = bf16_tensor(O.bf16_round(rng.standard_normal((T, H, 128)).astype(np.float32))).cuda()
    v = bf16_tensor(O.bf16_round(rng.standard_normal((T, H, 128)).astype(np.float32))).cuda()
    slots = torch.from_numpy(rng.permutation(T + 9)[:T].astype(np.int64)).cuda()
    mk = lambda: (torch.zeros(H, T + 9, 64, dtype=torch.uint8, device="cuda"),
                  torch.zeros(H, T + 9, 1, dtype=torch.bfloat16, device="cuda"))
    kd, ks = mk(); vd, vs = mk(); kd2, ks2 = mk(); vd2, vs2 = mk()
    ops().fused_quant_write_int4_sym_kv(k, v, slots, kd, ks, vd, vs, 128)
    ops().fused_quant_write_int4_sym(k, slots, kd2, ks2, 128)
    ops().fused_quant_write_int4_sym(v, slots, vd2, vs2, 128)
    assert torch.equal(kd, kd2) and torch.equal(vd, vd2) and torch.equal(ks, ks2) and torch.equal(vs, vs2)
    ref_d, ref_s = O.quantize_and_pack(bf16_to_f32(v), 128, 4)
    assert np.array_equal(vd.cpu().numpy()[:, slots.cpu().numpy()].transpose(1, 0, 2), ref_d)


def test_pack_rejects_bad_arguments():
    x = torch.zeros(2, 2, 128, dtype=torch.float16, device="cuda")
    d = torch.zeros(2, 4, 48, dtype=torch.uint8, device="cuda")
    s = torch.zeros(2, 4, 2, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError):
        ops().fused_quant_write_int3_sym(x, torch.zeros(2, dtype=torch.int64, device="cuda"), d, s, 64)
    with pytest.raises(RuntimeError):
        ops().fused_quant_write_int3_sym(x.bfloat16(), torch.zeros(2, dtype=torch.int64, device="cuda"), d, s, 48)


# ------------------------------------------------------------------ Stage A + top-k


@pytest.fixture(params=["fast", "simple"])
def impl(request):
    """Both implementations of the Stage A / Stage B operators: on the kernels of the fused step, and one plain
    kernel per reference kernel."""
    prev = ops().set_split_impl(request.param)
    yield request.param
    ops().set_split_impl(prev)


CASES_A = [  # (B, Hq, Hkv, S)
    (2, 8, 2, 512), (3, 32, 8, 300), (2, 32, 4, 272), (1, 8, 2, 17),
    (2, 28, 4, 300), (1, 24, 8, 272), (2, 12, 1, 200),          # 7, 3 and 12 query heads per kv-head
]


@pytest.mark.parametrize("B,Hq,Hkv,S", CASES_A)
@pytest.mark.parametrize("gs", (64, 128))
def test_int3_scores_and_topk(B, Hq, Hkv, S, gs, impl):
    c = make_case(11 + S + gs, B, Hq, Hkv, S, 3, 2, gs)
    d = to_device(c)
    scale = 128 ** -0.5
    K = 32 if S < 64 else 64
    scores, idx, slots = ops().int3_qk_scores_topk(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, scale, K)
    ref = O.scores_bf16_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, scale, 3, gs)
    got = scores.cpu().numpy()
    valid = np.isfinite(ref)
    assert np.array_equal(np.isneginf(got), ~valid)               # -inf exactly on the padding
    np.testing.assert_allclose(got[valid], ref[valid], atol=2e-5, rtol=2e-5)   # validate_runtime.py:147-148
    # top-k is exact on the scores the GPU itself produced, ties to the lower position, ascending order
    ridx, rslots = O.topk_select(got, c["lens"], c["bt"], S, K)
    assert np.array_equal(idx.cpu().numpy(), ridx)
    assert np.array_equal(slots.cpu().numpy(), rslots)
    alone = ops().int3_qk_scores(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, scale)
    assert torch.equal(alone, scores)                            # the scores-only operator: the same kernel arithmetic


@pytest.mark.parametrize("B,Hq,Hkv,S", CASES_A)
@pytest.mark.parametrize("kb,gs", [(2, 64), (2, 128), (4, 64), (4, 128)])
def test_int2_and_int4_scores_with_the_bf16_model(B, Hq, Hkv, S, kb, gs, impl):
    """int2_qk_scores (symmetric keys, empty k_zp) and int4_qk_scores: bf16 q times bf16-rounded keys."""
    c = make_case(13 + S + gs + kb, B, Hq, Hkv, S, kb, 2, gs)
    d = to_device(c)
    scale = 128 ** -0.5
    K = 32 if S < 64 else 64
    o = ops()
    if kb == 2:
        scores, idx, slots = o.int2_qk_scores_topk(d["q"], d["kd"], d["ks"], None, d["bt"], d["lens"], S, Hq, Hkv, 16, scale, K)
    else:
        scores, idx, slots, m, iz = o.int4_qk_scores_topk_stats(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv,
                                                                16, scale, K)
    ref = O.scores_bf16_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, scale, kb, gs)
    got = scores.cpu().numpy()
    valid = np.isfinite(ref)
    assert np.array_equal(np.isneginf(got), ~valid)
    np.testing.assert_allclose(got[valid], ref[valid], atol=2e-5, rtol=2e-5)   # validate_runtime.py:147-148
    ridx, rslots = O.topk_select(got, c["lens"], c["bt"], S, K)
    assert np.array_equal(idx.cpu().numpy(), ridx)
    assert np.array_equal(slots.cpu().numpy(), rslots)
    if kb == 4:
        rm, riz = O.softmax_stats(got, c["lens"], S)
        np.testing.assert_allclose(m.cpu().numpy(), rm, rtol=0, atol=0)
        np.testing.assert_allclose(iz.cpu().numpy(), riz, rtol=2e-5)


@pytest.mark.parametrize("B,Hq,Hkv,S", CASES_A)
def test_int8tc_scores_bit_exact_topk_and_stats(B, Hq, Hkv, S, impl):
    c = make_case(21 + S, B, Hq, Hkv, S, 4, 4, 128)
    d = to_device(c)
    scale = 128 ** -0.5
    K = 64
    scores, idx, slots, m, iz = ops().int8tc_qk_scores_topk_stats(
        d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, scale, K)
    ref = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, scale)
    got = scores.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))          # integer model: bit-exact
    ridx, rslots = O.topk_select(ref, c["lens"], c["bt"], S, K)
    assert np.array_equal(idx.cpu().numpy(), ridx)
    assert np.array_equal(slots.cpu().numpy(), rslots)
    rm, riz = O.softmax_stats(ref, c["lens"], S)
    np.testing.assert_allclose(m.cpu().numpy(), rm, atol=0, rtol=0)
    np.testing.assert_allclose(iz.cpu().numpy(), riz, rtol=1e-5)
    alone = ops().int8tc_qk_scores(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, scale)
    assert torch.equal(alone, scores)
    three = ops().int8tc_qk_scores_topk(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, scale, K)
    assert torch.equal(three[1], idx) and torch.equal(three[2], slots)


def test_topk_ties_short_rows_and_zero_length(impl):
    rng = np.random.default_rng(3)
    B, Hq, S, K = 4, 4, 96, 32
    sc = rng.integers(-2, 3, size=(B, Hq, S)).astype(np.float32)            # heavy ties
    sc[0, 0, 5], sc[0, 0, 6] = -0.0, 0.0
    lens = np.array([96, 0, 1, 31], dtype=np.int32)
    bt = rng.permutation(B * 6).reshape(B, 6).astype(np.int64)
    from jetfire_amd import _lib
    lib = _lib.load()
    t, lens_t, bt_t = torch.from_numpy(sc).cuda(), torch.from_numpy(lens).cuda(), torch.from_numpy(bt).cuda()
    idx = torch.empty(B, Hq, K, dtype=torch.int64, device="cuda")
    slots = torch.empty_like(idx)
    torch.cuda.synchronize()
    _lib.check(lib.jf_topk_slots(t.data_ptr(), lens_t.data_ptr(), bt_t.data_ptr(), B, Hq, S, 6, 16, K,
                                 idx.data_ptr(), slots.data_ptr(), None, None, None))   # raw C ABI, default stream
    torch.cuda.synchronize()
    ridx, rslots = O.topk_select(sc, lens, bt, S, K)
    assert np.array_equal(idx.cpu().numpy(), ridx)
    assert np.array_equal(slots.cpu().numpy(), rslots)
    # the operator-level selection (either implementation), with the statistics
    idx2, slots2, m2, iz2 = ops()._topk(t, bt_t, lens_t, S, Hq, 16, K, True, "t")
    assert np.array_equal(idx2.cpu().numpy(), ridx) and np.array_equal(slots2.cpu().numpy(), rslots)
    rm, riz = O.softmax_stats(sc, lens, S)
    np.testing.assert_allclose(m2.cpu().numpy(), rm, rtol=0, atol=0)
    np.testing.assert_allclose(iz2.cpu().numpy(), riz, rtol=2e-5)


def test_topk_large_row_and_k(impl):
    rng = np.random.default_rng(4)
    B, Hq, S, K = 1, 2, 40000, 512
    sc = (rng.standard_normal((B, Hq, S)) * 0.15).astype(np.float32)
    sc[0, 1, ::3] = np.float32(0.25)                                          # a tie class straddling the cut
    lens = np.array([39990], dtype=np.int32)
    bt = rng.permutation(2500).reshape(1, 2500).astype(np.int64)
    o = ops()
    idx, slots, _, _ = o._topk(torch.from_numpy(sc).cuda(), torch.from_numpy(bt).cuda(), torch.from_numpy(lens).cuda(),
                               S, Hq, 16, K, False, "t")
    ridx, rslots = O.topk_select(sc, lens, bt, S, K)
    assert np.array_equal(idx.cpu().numpy(), ridx)
    assert np.array_equal(slots.cpu().numpy(), rslots)


def test_unsupported_top_k_raises():
    c = make_case(1, 1, 8, 2, 64, 3, 2, 64)
    d = to_device(c)
    with pytest.raises(RuntimeError, match="unsupported radix-select top_k"):
        ops().int3_qk_scores_topk(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], 64, 8, 2, 16, 0.1, 48)
    with pytest.raises(RuntimeError):
        ops().int3_qk_scores(d["q"].float(), d["kd"], d["ks"], d["bt"], d["lens"], 64, 8, 2, 16, 0.1)


# ------------------------------------------------------------------ Stage B + merge


@pytest.mark.parametrize("scheme", ("k3v2", "k4v4", "k3v2_g128", "k3v3", "k3v3_g128", "k3v4_g64"))
@pytest.mark.parametrize("B,Hq,Hkv,lens", [(2, 8, 2, None), (3, 32, 4, [17, 257, 512]), (4, 8, 2, [0, 1, 9, 17]),
                                           (2, 28, 4, [400, 512]), (2, 10, 2, None)])      # 7 and 5 heads per kv-head
def test_stage_b_outputs(scheme, B, Hq, Hkv, lens, impl):
    kb, vb, gs = {"k3v2": (3, 2, 64), "k4v4": (4, 4, 128), "k3v2_g128": (3, 2, 128), "k3v3": (3, 3, 64),
                  "k3v3_g128": (3, 3, 128), "k3v4_g64": (3, 4, 64)}[scheme]
    S = 512 if lens is None or max(lens) > 32 else 32
    c = make_case(31 + B, B, Hq, Hkv, S, kb, vb, gs, lens=lens)
    d = to_device(c)
    scale = 128 ** -0.5
    K = 64
    o = ops()
    if kb == 3:
        ref_sc = O.scores_bf16_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, scale, 3, gs)
    else:
        ref_sc = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, scale)
    ridx, _ = O.topk_select(ref_sc, c["lens"], c["bt"], S, K)
    sc_t, idx_t = torch.from_numpy(ref_sc).cuda(), torch.from_numpy(ridx).cuda()
    fn = {2: o.int2_softmax_v_with_pre_corr_wvs2, 3: o.int3_softmax_v_with_pre_corr_wvs2,
          4: o.int4_softmax_v_with_pre_corr_wvs2_scores}[vb]
    o_hat, o_old, W = fn(sc_t, d["vd"], d["vs"], d["bt"], d["lens"], idx_t, S, Hq, Hkv, 16, K)
    r_hat, r_old, r_W = O.softmax_v(ref_sc, c["vd"], c["vs"], c["bt"], c["lens"], ridx, S, Hq, Hkv, 16, vb, gs)
    np.testing.assert_allclose(o_hat.cpu().numpy(), r_hat, atol=3e-6, rtol=3e-6)     # validate_runtime.py:173-177
    np.testing.assert_allclose(o_old.cpu().numpy(), r_old, atol=3e-6, rtol=3e-6)
    np.testing.assert_allclose(W.cpu().numpy(), r_W, atol=3e-6, rtol=3e-6)
    if vb != 3:                                                   # without winners: o_hat alone
        plain = {2: o.int2_softmax_v, 4: None}[vb]
        if plain is not None:
            only = plain(sc_t, d["vd"], d["vs"], d["bt"], d["lens"], S, Hq, Hkv, 16)
            np.testing.assert_allclose(only.cpu().numpy(), r_hat, atol=3e-6, rtol=3e-6)
        padded = idx_t.clone()
        padded[:, :, K // 2:] = -1                                # half of the winners dropped: -1 entries carry no weight
        h_idx = ridx.copy()
        h_idx[:, :, K // 2:] = -1
        _, p_old, p_W = fn(sc_t, d["vd"], d["vs"], d["bt"], d["lens"], padded, S, Hq, Hkv, 16, K)
        _, q_old, q_W = O.softmax_v(ref_sc, c["vd"], c["vs"], c["bt"], c["lens"], h_idx, S, Hq, Hkv, 16, vb, gs)
        np.testing.assert_allclose(p_old.cpu().numpy(), q_old, atol=3e-6, rtol=3e-6)
        np.testing.assert_allclose(p_W.cpu().numpy(), q_W, atol=3e-6, rtol=3e-6)
    if vb == 4 and gs == 128:                                     # the int8-weight variant, handed Stage-A statistics
        m, iz = O.softmax_stats(ref_sc, c["lens"], S)
        o2 = o.int8tc_softmax_v_with_pre_corr_reg_stats(sc_t, torch.from_numpy(m).cuda(), torch.from_numpy(iz).cuda(),
                                                        d["vd"], d["vs"], d["bt"], d["lens"], idx_t, S, Hq, Hkv, 16, K)
        # the reference's own tile arithmetic, at the tolerance its validator uses for it
        # (scripts/validate_runtime_edges.py:146-171); the pre-correction terms use exact fp32 weights
        t_hat, t_old, t_W = O.softmax_v_int8_tiles(ref_sc, m, iz, c["vd"], c["vs"], c["bt"], c["lens"], ridx, S, Hq, Hkv, 16)
        np.testing.assert_allclose(o2[0].cpu().numpy(), t_hat, atol=3e-6, rtol=3e-6)
        np.testing.assert_allclose(o2[1].cpu().numpy(), t_old, atol=3e-6, rtol=3e-6)
        np.testing.assert_allclose(o2[2].cpu().numpy(), t_W, atol=3e-6, rtol=3e-6)
        if lens is None:   # long rows: the approximation stays within the reference's int8-P tolerance of the dense
            # result (validate_runtime.py:173-176); on short peaked rows it strays further (validate_runtime_edges.py:146-152)
            np.testing.assert_allclose(o2[0].cpu().numpy(), r_hat, atol=3e-3)


@pytest.mark.parametrize("S,lens", [(1000, [1000, 333]), (72, [72, 5]), (256, [256, 0])])
def test_int8_tile_stage_b_on_ranges_that_do_not_start_on_a_page(S, lens):
    """ceil(S / 8) is not a multiple of 16 here: tiles start at the page holding a range's first position and the
    positions of that page before the range carry no weight (int8tc_softmax_v_fused.cu:1052,1178,1218)."""
    B, Hq, Hkv, K = 2, 8, 2, 64
    c = make_case(5 + S, B, Hq, Hkv, S, 4, 4, 128, lens=lens)
    d = to_device(c)
    o = ops()
    ref_sc = O.scores_int8_model(c["q"], c["kd"], c["ks"], c["bt"], c["lens"], S, Hq, Hkv, 16, 128 ** -0.5)
    ridx, _ = O.topk_select(ref_sc, c["lens"], c["bt"], S, K)
    m, iz = O.softmax_stats(ref_sc, c["lens"], S)
    got = o.int8tc_softmax_v_with_pre_corr_reg_stats(torch.from_numpy(ref_sc).cuda(), torch.from_numpy(m).cuda(),
                                                     torch.from_numpy(iz).cuda(), d["vd"], d["vs"], d["bt"], d["lens"],
                                                     torch.from_numpy(ridx).cuda(), S, Hq, Hkv, 16, K)
    want = O.softmax_v_int8_tiles(ref_sc, m, iz, c["vd"], c["vs"], c["bt"], c["lens"], ridx, S, Hq, Hkv, 16)
    for g, w in zip(got, want):
        np.testing.assert_allclose(g.cpu().numpy(), w, atol=3e-6, rtol=3e-6)


def test_blend_bit_exact():
    rng = np.random.default_rng(8)
    hat = rng.standard_normal((3, 8, 128)).astype(np.float32)
    old = (rng.standard_normal((3, 8, 128)) * 0.3).astype(np.float32)
    W = rng.uniform(0, 1, (3, 8)).astype(np.float32)
    new = O.bf16_round(rng.standard_normal((3, 8, 128)).astype(np.float32))
    out = torch.empty(3, 8, 128, dtype=torch.bfloat16, device="cuda")
    ops().blend_unnorm_into(torch.from_numpy(hat).cuda(), torch.from_numpy(old).cuda(), torch.from_numpy(W).cuda(),
                            bf16_tensor(new).cuda(), out)
    ref = O.blend_unnorm(hat, old, W, new)
    assert np.array_equal(bf16_to_bits(out), O.f32_to_bf16_bits(ref))


# ------------------------------------------------------------------ end-to-end split pipeline with the pinned hand-off


@pytest.mark.parametrize("scheme,B,Hq,Hkv,lens,K", [
    ("k3v2", 2, 8, 2, None, 256), ("k4v4", 2, 8, 2, None, 256),
    ("k3v2", 3, 32, 4, [17, 257, 512], 256), ("k4v4", 4, 8, 2, [0, 1, 9, 17], 64),
])
def test_split_pipeline_with_handoff(scheme, B, Hq, Hkv, lens, K):
    kb, vb, gs = (3, 2, 64) if scheme == "k3v2" else (4, 4, 128)
    S = 512 if lens is None or max(lens) > 32 else 32
    c = make_case(41 + B, B, Hq, Hkv, S, kb, vb, gs, lens=lens)
    d = to_device(c)
    o = ops()
    scale = 128 ** -0.5
    ksh, vsh = bf16_tensor(c["K"]), bf16_tensor(c["V"])
    o.set_cpu_attn_threads(4)
    h = o.CpuTopkHandoff(B, Hq, Hkv, K, ksh, vsh, scale)
    out = torch.empty(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    o_new = torch.empty_like(out)
    for rep in range(2):                                          # the context is reusable
        if scheme == "k3v2":
            scores, idx, slots = o.int3_qk_scores_topk(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, scale, K)
        else:
            scores, idx, slots, m, iz = o.int8tc_qk_scores_topk_stats(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S,
                                                                      Hq, Hkv, 16, scale, K)
        h.submit(d["q"], slots)
        if scheme == "k3v2":
            o_hat, o_old, W = o.int2_softmax_v_with_pre_corr_wvs2(scores, d["vd"], d["vs"], d["bt"], d["lens"], idx, S,
                                                                  Hq, Hkv, 16, K)
        else:
            o_hat, o_old, W = o.int4_softmax_v_with_pre_corr_wvs2_scores(scores, d["vd"], d["vs"], d["bt"], d["lens"],
                                                                         idx, S, Hq, Hkv, 16, K)
        h.wait(o_new)
        o.blend_unnorm_into(o_hat, o_old, W, o_new, out)
        torch.cuda.synchronize()
    assert h.submit_count == 2
    r = O.decode_reference(c["q"], c["kd"], c["ks"], c["vd"], c["vs"], c["bt"], c["lens"], S, Hq, Hkv, 16, scale, K,
                           scheme, c["K"], c["V"])
    np.testing.assert_allclose(bf16_to_f32(o_new), r["o_new"], atol=2e-3, rtol=6e-3)          # validate_runtime.py:191
    got = bf16_to_f32(out)
    np.testing.assert_allclose(got, r["out"], atol=6e-3, rtol=1.5e-2)                         # validate_runtime.py:195
    err = np.abs(got - r["out"])
    assert err.max() <= 2e-2 and err.mean() <= 1e-3               # the acceptance bar for attention outputs
    h.close()


def test_handoff_protocol_edges():
    """wait without a submit returns at once; closing a context with a submit that was never waited for lets
    the job finish first."""
    B, Hq, Hkv, K, S = 1, 8, 2, 32, 64
    c = make_case(77, B, Hq, Hkv, S, 3, 2, 64)
    d = to_device(c)
    o = ops()
    ksh, vsh = bf16_tensor(c["K"]), bf16_tensor(c["V"])
    o.set_cpu_attn_threads(2)
    scale = 128 ** -0.5
    _, idx, slots = o.int3_qk_scores_topk(d["q"], d["kd"], d["ks"], d["bt"], d["lens"], S, Hq, Hkv, 16, scale, K)
    o_new = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    h = o.CpuTopkHandoff(B, Hq, Hkv, K, ksh, vsh, scale)
    h.wait(o_new)                                                 # nothing outstanding
    h.submit(d["q"], slots)
    h.wait(o_new)
    torch.cuda.synchronize()
    ref = O.cpu_topk_attn(c["q"], c["K"], c["V"], O.head_map(B, Hq, Hq // Hkv, K), slots.cpu().numpy(), scale)
    np.testing.assert_allclose(bf16_to_f32(o_new), ref, atol=2e-3, rtol=6e-3)
    assert h.submit_count == 1
    h.submit(d["q"], slots)                                       # left outstanding on purpose
    h.close()                                                     # must wait for the job, then free
    torch.cuda.synchronize()


def test_handoff_stream_mode_replays_from_a_hip_graph():
    """The kernel-only submit / wait pair: eager calls, then a captured graph (publish, device-side wait + blend)
    replayed with new queries and slots in the same buffers, eager work and synchronisations in between; every
    result equals the host-blocking pair's on the same inputs."""
    B, Hq, Hkv, K, S = 2, 8, 2, 32, 256
    c = make_case(78, B, Hq, Hkv, S, 3, 2, 64, ragged=False)
    o = ops()
    ksh, vsh = bf16_tensor(c["K"]), bf16_tensor(c["V"])
    o.set_cpu_attn_threads(2)
    scale = 128 ** -0.5
    rng = np.random.default_rng(1)
    num_slots = ksh.shape[1]

    def draw():
        q = bf16_tensor(O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32))).cuda()
        s = torch.from_numpy(np.stack([rng.choice(num_slots, K, replace=False) for _ in range(B * Hq)]).reshape(B, Hq, K)).cuda()
        s[0, 0, :3] = -1                                          # padding entries are masked on the CPU side
        return q, s

    def host_pair(q, s):
        h = o.CpuTopkHandoff(B, Hq, Hkv, K, ksh, vsh, scale)
        out = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
        h.submit(q, s)
        h.wait(out)
        torch.cuda.synchronize()
        h.close()
        return out

    h = o.CpuTopkHandoff(B, Hq, Hkv, K, ksh, vsh, scale)
    q_buf, s_buf = draw()
    o_new = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="stream_submit"):
        h.stream_wait(o_new)                                      # nothing was submitted in this mode
    for _ in range(2):                                            # eager
        q, s = draw()
        h.stream_submit(q, s)
        h.stream_wait(o_new)
        torch.cuda.synchronize()
        h.check_status()
        assert torch.equal(o_new.view(torch.int16), host_pair(q, s).view(torch.int16))
    with pytest.raises(RuntimeError, match="stream mode"):
        h.submit(q_buf, s_buf)                                    # one mode per context
    o_hat = torch.randn(B, Hq, 128, device="cuda")
    o_old = torch.randn(B, Hq, 128, device="cuda") * 0.1
    W = torch.rand(B, Hq, device="cuda")
    out = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        h.stream_submit(q_buf, s_buf)
        h.stream_wait_blend(o_hat, o_old, W, out, o_new)          # wait + fetch + blend in one kernel
    for step in range(4):
        q, s = draw()
        q_buf.copy_(q); s_buf.copy_(s)
        graph.replay()
        torch.cuda.synchronize()
        h.check_status()
        want_new = host_pair(q, s)
        assert torch.equal(o_new.view(torch.int16), want_new.view(torch.int16)), step
        want = torch.zeros_like(out)
        o.blend_unnorm_into(o_hat, o_old, W, want_new, want)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), step
    assert h.submit_count == 6
    h.close()


def test_handoff_stream_wait_blend_more_rows_than_one_pass():
    """288 rows: the wait + blend kernel (one workgroup, 4096 eight-element items per pass) takes a second pass."""
    B, Hq, Hkv, K = 9, 32, 4, 32
    o = ops()
    rng = np.random.default_rng(5)
    num_slots = 512
    ksh = bf16_tensor(O.bf16_round(rng.standard_normal((Hkv, num_slots, 128)).astype(np.float32)))
    vsh = bf16_tensor(O.bf16_round(rng.standard_normal((Hkv, num_slots, 128)).astype(np.float32)))
    q = bf16_tensor(O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32))).cuda()
    s = torch.from_numpy(rng.integers(0, num_slots, size=(B, Hq, K)).astype(np.int64)).cuda()
    o.set_cpu_attn_threads(3)
    o_hat = torch.randn(B, Hq, 128, device="cuda")
    o_old = torch.randn(B, Hq, 128, device="cuda") * 0.1
    W = torch.rand(B, Hq, device="cuda")
    h = o.CpuTopkHandoff(B, Hq, Hkv, K, ksh, vsh, 0.1)
    out = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    o_new = torch.zeros_like(out)
    h.stream_submit(q, s)
    h.stream_wait_blend(o_hat, o_old, W, out, o_new)
    torch.cuda.synchronize()
    h.check_status()
    h.close()
    want_new = torch.zeros(B, Hq, 128, dtype=torch.bfloat16)
    o.cpu_topk_attn(q.cpu(), ksh, vsh, torch.from_numpy(O.head_map(B, Hq, Hq // Hkv, K)), s.cpu(), want_new, 0.1)
    assert torch.equal(o_new.cpu().view(torch.int16), want_new.view(torch.int16))
    want = torch.zeros_like(out)
    o.blend_unnorm_into(o_hat, o_old, W, o_new, want)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


def test_handoff_stream_wait_blend_can_zero_non_finite_outputs():
    """The graph-mode guard of the reference (decode_path.py:1133-1149) inside the blending wait kernel: with the option
    set, non-finite outputs come out as zero and every other element is the plain blend; without it they pass."""
    B, Hq, Hkv, K = 2, 8, 2, 32
    o = ops()
    rng = np.random.default_rng(6)
    num_slots = 256
    ksh = bf16_tensor(O.bf16_round(rng.standard_normal((Hkv, num_slots, 128)).astype(np.float32)))
    vsh = bf16_tensor(O.bf16_round(rng.standard_normal((Hkv, num_slots, 128)).astype(np.float32)))
    q = bf16_tensor(O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32))).cuda()
    s = torch.from_numpy(rng.integers(0, num_slots, size=(B, Hq, K)).astype(np.int64)).cuda()
    o.set_cpu_attn_threads(2)
    o_hat = torch.randn(B, Hq, 128, device="cuda")
    o_old = torch.randn(B, Hq, 128, device="cuda") * 0.1
    W = torch.rand(B, Hq, device="cuda")
    o_hat[0, 1, 5] = float("nan")
    o_hat[1, 7, 127] = float("inf")
    o_old[1, 0, 0] = float("inf")
    outs = []
    for on in (False, True):
        h = o.CpuTopkHandoff(B, Hq, Hkv, K, ksh, vsh, 0.1)
        h.set_output_sanitize(on)
        out = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
        o_new = torch.zeros_like(out)
        h.stream_submit(q, s)
        h.stream_wait_blend(o_hat, o_old, W, out, o_new)
        torch.cuda.synchronize()
        h.check_status()
        h.close()
        outs.append((out, o_new))
    plain = o.blend_unnorm(o_hat, o_old, W, outs[0][1])
    assert torch.equal(outs[0][0].view(torch.int16), plain.view(torch.int16))
    assert not torch.isfinite(outs[0][0].float()).all()
    clean = torch.nan_to_num(plain.float(), nan=0.0, posinf=0.0, neginf=0.0).to(torch.bfloat16)
    assert torch.equal(outs[1][0].view(torch.int16), clean.view(torch.int16))
    assert torch.isfinite(outs[1][0].float()).all()


def test_handoff_stream_wait_is_bounded():
    """A correction that never finishes (the dispatcher is told to ignore the flag): the device-side wait runs
    into its limit, the kernel ends, o_new is zero, the status reports it, and later waits fall through."""
    import time
    B, Hq, Hkv, K = 1, 4, 2, 32
    o = ops()
    ksh = torch.zeros(Hkv, 64, 128, dtype=torch.bfloat16)
    h = o.CpuTopkHandoff(B, Hq, Hkv, K, ksh, ksh, 0.1)
    h.debug_pause(True)
    h.set_device_wait_limit_us(20000)
    q = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    s = torch.zeros(B, Hq, K, dtype=torch.int64, device="cuda")
    o_new = torch.ones(B, Hq, 128, dtype=torch.bfloat16, device="cuda")
    h.stream_submit(q, s)
    h.stream_wait(o_new)
    t0 = time.perf_counter()
    torch.cuda.synchronize()
    assert time.perf_counter() - t0 < 5.0
    with pytest.raises(RuntimeError, match="limit"):
        h.check_status()
    assert float(o_new.float().abs().sum()) == 0.0
    o_new.fill_(1)
    h.stream_wait(o_new)                                          # falls through: no second 20 ms wait needed
    torch.cuda.synchronize()
    assert float(o_new.float().abs().sum()) == 0.0
    with pytest.raises(RuntimeError, match="failed or timed out"):
        h.stream_submit(q, s)
    h.debug_pause(False)
    h.close()
