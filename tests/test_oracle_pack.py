"""Pins the oracle's wire format and quantiser.

Golden vectors are the ones the reference's own test holds
(tests/test_int_pack.py:10-35 in the reference tree); the rest are closed
forms, invariants and brute force that a dropped term or wrong index fails.
"""
import numpy as np
import pytest

from oracle import jetfire_oracle as O

WIRE = (
    (2, (-1, 0, 1, 0), (0x6E,)),
    (3, (-3, -2, -1, 0, 1, 2, 3, 0), (0x29, 0xCB, 0xBC)),
    (4, (-7, 7), (0x1F,)),
)


@pytest.mark.parametrize("group_size", (64, 128))
@pytest.mark.parametrize("bits,values,planes", WIRE)
def test_reference_wire_bytes_round_trip(bits, values, planes, group_size):
    x = np.tile(np.array(values, dtype=np.float32), 128 // len(values)).reshape(1, 128)
    data, sbits = O.quantize_and_pack(x, group_size, bits)
    assert (O.bf16_bits_to_f32(sbits) == 1.0).all()
    repeats = 128 // (8 if bits == 3 else 8 // bits)
    expected = np.array([b for b in planes for _ in range(repeats)], dtype=np.uint8)
    assert np.array_equal(data[0], expected)
    assert np.array_equal(O.unpack(data, sbits, group_size, bits), x)


@pytest.mark.parametrize("bits", (2, 3, 4))
def test_reference_zero_groups_remain_finite(bits):
    x = np.zeros((2, 128), dtype=np.float32)
    data, sbits = O.quantize_and_pack(x, 64, bits)
    s = O.bf16_bits_to_f32(sbits)
    assert np.isfinite(s).all() and (s > 0).all()
    assert np.array_equal(O.unpack(data, sbits, 64, bits), x)
    assert (O.decode_codes(data, bits) == O.offset(bits)).all()


def _bf16_randn(rng, *shape, scale=1.0):
    return O.bf16_round((rng.standard_normal(shape) * scale).astype(np.float32))


@pytest.mark.parametrize("bits", (2, 3, 4))
def test_pack_decode_is_a_bijection_on_the_full_code_range(bits):
    rng = np.random.default_rng(bits)
    codes = rng.integers(0, 1 << bits, size=(5, 7, 128), dtype=np.uint8)
    data = O.pack_codes(codes, bits)
    assert data.shape[-1] == O.packed_dim(128, bits)
    assert np.array_equal(O.decode_codes(data, bits), codes)


def test_int3_planes_follow_the_closed_form():
    # intN_pack.py:6-29: w = sum code[i] << (21-3i); planes hold w>>16, (w>>8)&255, w&255
    rng = np.random.default_rng(3)
    codes = rng.integers(0, 8, size=(128,), dtype=np.uint8)
    data = O.pack_codes(codes[None], 3)[0]
    for g in range(16):
        w = 0
        for i in range(8):
            w |= int(codes[8 * g + i]) << (21 - 3 * i)
        assert data[g] == (w >> 16) & 255 and data[16 + g] == (w >> 8) & 255 and data[32 + g] == w & 255


@pytest.mark.parametrize("bits", (2, 3, 4))
@pytest.mark.parametrize("gs", (64, 128))
def test_quantiser_invariants(bits, gs):
    rng = np.random.default_rng(10 * bits + gs)
    x = _bf16_randn(rng, 64, 8, 128, scale=3.0)
    x[..., :4] *= 8
    x = O.bf16_round(x)
    codes, sbits = O.quantize_codes(x, gs, bits)
    qm = O.qmax(bits)
    assert codes.min() >= 1 and codes.max() <= 2 * qm + 1          # symmetric codes never use 0
    s = O.bf16_bits_to_f32(sbits)
    xg = x.reshape(64, 8, 128 // gs, gs)
    ratio = np.abs(xg) / s[..., None]
    xhat = (codes.astype(np.float32) - O.offset(bits)).reshape(xg.shape) * s[..., None]
    inside = ratio <= qm
    assert (np.abs(xhat - xg)[inside] <= s[..., None].repeat(gs, -1)[inside] * 0.5 * (1 + 1e-6)).all()
    # every group reaches |q| == qmax at its amax element (scale is amax/qmax up to bf16 rounding)
    assert (np.abs(codes.astype(np.int32) - O.offset(bits)).reshape(xg.shape).max(-1) == qm).all()


def test_quantiser_ties_round_half_to_even_and_clamp():
    # scale == 1 (amax 7 -> 7/7), elements at exact .5 ties
    x = np.zeros((1, 128), dtype=np.float32)
    x[0, 0] = 7.0
    x[0, 1:7] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    codes, sbits = O.quantize_codes(x, 128, 4)
    assert O.bf16_bits_to_f32(sbits)[0, 0] == 1.0
    assert list(codes[0, :7].astype(int) - 8) == [7, 0, 2, 2, 0, -2, -2]
    # amax/qmax not representable in bf16 and rounding DOWN => |x/scale| > qmax => clamp to qmax
    x = np.zeros((1, 128), dtype=np.float32)
    x[0, 0] = 3.03125  # bf16 value; 3.03125/3 = 1.0104... rounds DOWN to bf16 1.0078125
    codes, sbits = O.quantize_codes(x, 128, 3)
    s = float(O.bf16_bits_to_f32(sbits)[0, 0])
    assert s == 1.0078125 and 3.03125 / s > 3
    assert int(codes[0, 0]) - 4 == 3


def test_quantiser_matches_bruteforce_scalar_ieee():
    """Independent scalar restatement with Python floats rounded through float32 at each step."""
    rng = np.random.default_rng(99)
    x = _bf16_randn(rng, 16, 128, scale=2.0)
    for bits, gs in ((2, 64), (3, 64), (4, 128)):
        codes, sbits = O.quantize_codes(x, gs, bits)
        qm = O.qmax(bits)
        for r in range(16):
            for g in range(128 // gs):
                grp = x[r, g * gs:(g + 1) * gs]
                amax = np.float32(max(abs(float(v)) for v in grp))
                sc = np.float32(amax / np.float32(qm))
                sc = sc if sc > np.float32(1e-8) else np.float32(1e-8)
                sb = O.f32_to_bf16_bits(np.array([sc]))[0]
                assert sb == sbits[r, g]
                sf = O.bf16_bits_to_f32(np.array([sb]))[0]
                for i, v in enumerate(grp):
                    qv = float(np.float32(v) / sf)
                    fl = np.floor(qv)
                    d = qv - fl
                    rn = fl + (1 if d > 0.5 or (d == 0.5 and fl % 2 == 1) else 0)
                    rn = max(-qm, min(qm, rn))
                    assert int(codes[r, g * gs + i]) == int(rn) + O.offset(bits)


def test_bf16_rounding_is_rne():
    v = np.array([1.0, 1.00390625, 1.01171875, -1.00390625, 3.0e38, 1e-40], dtype=np.float32)
    # 1 + 2^-8 is a tie -> even (1.0); 1 + 3*2^-8 is a tie -> even (1.015625)
    got = O.bf16_round(v)
    assert got[0] == 1.0 and got[1] == 1.0 and got[2] == 1.015625 and got[3] == -1.0
    assert np.isfinite(got[4]) or np.isinf(got[4])


def test_write_cache_scatter_and_masked_slot():
    # validate_runtime.py:61-99: permuted slots, one masked (-1) row, canary byte untouched
    rng = np.random.default_rng(5)
    T, H = 33, 2
    x = _bf16_randn(rng, T, H, 128)
    slots = rng.permutation(T).astype(np.int64)
    data = np.full((H, T + 1, 48), 0xA5, dtype=np.uint8)
    sc = np.zeros((H, T + 1, 2), dtype=np.uint16)
    O.write_cache(np.concatenate([x, x[:1]]), np.concatenate([slots, [-1]]), data, sc, 64, 3)
    ref_d, ref_s = O.quantize_and_pack(x, 64, 3)
    assert np.array_equal(data[:, slots].transpose(1, 0, 2), ref_d)
    assert np.array_equal(sc[:, slots].transpose(1, 0, 2), ref_s)
    assert (data[:, -1] == 0xA5).all()


def test_fmaf_is_correctly_rounded():
    from fractions import Fraction
    rng = np.random.default_rng(0)
    a = rng.integers(-60000, 60000, 2000).astype(np.float32)
    b = (rng.standard_normal(2000) * 1e-3).astype(np.float32)
    c = (rng.standard_normal(2000) * 10 ** rng.uniform(-6, 3, 2000)).astype(np.float32)
    got = O.fmaf(a, b, c)
    for i in range(2000):
        exact = Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(c[i]))
        g = Fraction(float(got[i]))
        up = Fraction(float(np.nextafter(got[i], np.float32(np.inf))))
        dn = Fraction(float(np.nextafter(got[i], np.float32(-np.inf))))
        assert abs(g - exact) <= abs(up - exact) and abs(g - exact) <= abs(dn - exact)


@pytest.mark.parametrize("gs", (32, 64, 128))
def test_asymmetric_int2_quantiser_is_pinned_by_its_closed_form(gs):
    """quantize_and_pack_asym (intN_pack.py:110-169) has no vector in the reference's tests; what the formulas
    fix: scale = (max - min) / 3 and zp = min + 2 * scale on exactly representable inputs, the group minimum
    maps to code 0 and the maximum to code 3, a point of the grid maps to itself, the error inside the range is
    at most scale / 2 (+ the bf16 rounding of zp), a constant group takes the 1e-8 floor, and the reference's own
    self-test (:375-403): the asymmetric grid is not worse than the symmetric one by more than 5 % MSE."""
    # closed form: a group spanning [-1, 2] exactly: scale 1, zp 1, grid {-1, 0, 1, 2}
    x = np.zeros((1, 128), np.float32)
    x[0, ::4], x[0, 1::4], x[0, 2::4], x[0, 3::4] = -1.0, 0.0, 1.0, 2.0
    codes, sb, zb = O.quantize_codes_asym(x, gs, 2)
    assert (O.bf16_bits_to_f32(sb) == 1.0).all() and (O.bf16_bits_to_f32(zb) == 1.0).all()
    assert np.array_equal(codes[0, :4], [0, 1, 2, 3])
    # ties at .5 round to even: -0.5 -> q = rint(-1.5) = -2 -> code 0 ; 0.5 -> rint(-0.5) = -0 -> code 2
    y = x.copy(); y[0, 5], y[0, 6] = -0.5, 0.5
    cy, _, _ = O.quantize_codes_asym(y, gs, 2)
    assert cy[0, 5] == 0 and cy[0, 6] == 2
    rng = np.random.default_rng(gs)
    x = O.bf16_round((rng.standard_normal((64, 128)) * 1.7 + rng.standard_normal((64, 1))).astype(np.float32))
    codes, sb, zb = O.quantize_codes_asym(x, gs, 2)
    xg, cg = x.reshape(64, -1, gs), codes.reshape(64, -1, gs)
    assert codes.min() == 0 and codes.max() == 3
    assert (cg[np.arange(64)[:, None], np.arange(128 // gs)[None, :], xg.argmin(-1)] == 0).all()
    assert (cg[np.arange(64)[:, None], np.arange(128 // gs)[None, :], xg.argmax(-1)] == 3).all()
    data, sb2, zb2 = O.quantize_and_pack_asym(x, gs, 2)
    assert np.array_equal(sb, sb2) and np.array_equal(O.decode_codes(data, 2), codes)
    sf, zf = O.bf16_bits_to_f32(sb)[..., None], O.bf16_bits_to_f32(zb)[..., None]
    xhat = (cg.astype(np.float32) - 2) * sf + zf
    inside = (xg >= zf - 2 * sf) & (xg <= zf + sf)
    assert (np.abs(xhat - xg)[inside] <= sf.repeat(gs, -1)[inside] * 0.5 + 1e-6).all()
    # the kernel's dequant (one fma, then bf16) stays within bf16 rounding of that grid
    kd = O.dequant_asym_bf16(data, sb, zb, 2, gs).reshape(64, -1, gs)
    assert (np.abs(kd - xhat) <= np.abs(xhat) * 2.0 ** -8 + 1e-30).all()
    # a constant group: scale takes the floor, every element lands on one code
    c = np.full((2, 128), 0.375, np.float32)
    cc, cs, cz = O.quantize_codes_asym(c, gs, 2)
    assert (O.bf16_bits_to_f32(cs) == O.bf16_round(np.float32(1e-8))).all() and len(np.unique(cc)) == 1
    # the reference's self-test criterion
    sd, ss = O.quantize_and_pack(x, gs, 2)
    sym_mse = ((O.dequant(sd, ss, 2, gs, bf16=False) - x) ** 2).mean()
    asym_mse = ((xhat.reshape(64, 128) - x) ** 2).mean()
    assert asym_mse <= sym_mse * 1.05


def test_unpack_with_zero_points_rounds_twice():
    """intN_pack.py:251-256 rounds the product to bf16 before the zero-point is added.  Hand-worked case
    that a single rounding (or a fused multiply-add) fails: code 3 at scale 1 + 2^-7 is 3.0234375, a tie
    between the bf16 neighbours 3.015625 and 3.03125 that goes to the even one, 3.03125; adding the
    zero-point -2^-7 gives 3.0234375 again -> 3.03125.  One rounding of 3.0234375 - 0.0078125 = 3.015625
    would give 3.015625."""
    codes = np.full((1, 128), 3 + 8, dtype=np.uint8)
    data = O.pack_codes(codes, 4)
    sbits = O.f32_to_bf16_bits(np.array([[1.0 + 2.0 ** -7]], dtype=np.float32))
    zbits = O.f32_to_bf16_bits(np.array([[-(2.0 ** -7)]], dtype=np.float32))
    assert O.bf16_bits_to_f32(sbits)[0, 0] == 1.0 + 2.0 ** -7      # representable: the case is what it says
    out = O.unpack(data, sbits, 128, 4, zp_bits=zbits)
    assert (out == np.float32(3.03125)).all()
    # plain codebook check: scale 1, zero-point 0.5 shifts the INT2 grid -2..1 to -1.5..1.5
    c2 = np.tile(np.arange(4, dtype=np.uint8), 32).reshape(1, 128)
    out = O.unpack(O.pack_codes(c2, 2), O.f32_to_bf16_bits(np.ones((1, 2), np.float32)), 64, 2,
                   zp_bits=O.f32_to_bf16_bits(np.array([[0.5, -0.5]], np.float32)))
    assert np.array_equal(out[0, :4], np.array([-1.5, -0.5, 0.5, 1.5], np.float32))
    assert np.array_equal(out[0, 64:68], np.array([-2.5, -1.5, -0.5, 0.5], np.float32))
