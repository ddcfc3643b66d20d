"""CPU oracle for the JetFire approximate-attention decode path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests, the smoke check and
the CPU-baseline leg of the benchmark may import it.  It restates, in plain
numpy, the arithmetic the reference defines for

  * INT2/3/4 symmetric quantise + pack + unpack   (jetfire_vllm/kernels/intN_pack.py:60-107,172-222,227-311)
  * the independent wire decoder                  (scripts/validate_runtime.py:22-43)
  * Stage-A scores, bf16-dequant model (INT3 K)   (jetfire_vllm/csrc/int3_qk_scores.cu:90-99,268-311)
  * Stage-A scores, int8-Q model (INT4 K)         (jetfire_vllm/csrc/int8tc_qk_scores.cu:250-290,435-488;
                                                   scripts/validate_runtime.py:46-58)
  * radix-select top-k + slot translation         (jetfire_vllm/csrc/int3_qk_scores.cu:393-554)
  * softmax statistics                            (jetfire_vllm/csrc/int8tc_qk_scores.cu:1790-1799,
                                                   jetfire_vllm/csrc/int4_softmax_v.cu:124-160)
  * Stage-B  o_hat / o_old_unnorm / W, fp32 model (jetfire_vllm/csrc/int2_softmax_v.cu:601-789,
                                                   jetfire_vllm/csrc/int4_softmax_v.cu:599-817)
  * Stage-B int8 tile-quantised P model           (jetfire_vllm/csrc/int8tc_softmax_v_fused.cu:1203-1311;
                                                   scripts/validate_runtime_edges.py:146-164)
  * CPU top-k correction                          (jetfire_vllm/csrc/cpu_topk_attn.cpp:602-690)
  * merge                                         (jetfire_vllm/csrc/blend.cu:202-226)
  * width selection / head map                    (jetfire_vllm/adapter/decode_path.py:400-408,1156-1182)

Pinning status (what fixes each function besides its own formula) is listed in
``PINNED_BY`` at the bottom; tests/test_oracle_*.py execute those checks.

bf16 tensors are carried as float32 arrays whose values are bf16-representable,
or as uint16 bit patterns (``*_bits``).
"""
from __future__ import annotations

import numpy as np

HEAD_DIM = 128
BLOCK = 16

# --------------------------------------------------------------------------- bf16


def f32_to_bf16_bits(x) -> np.ndarray:
    """IEEE round-to-nearest-even float32 -> bfloat16 bit pattern (uint16)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    nan = np.isnan(x)
    r = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)
    r = r.astype(np.uint16)
    r[nan] = ((u[nan] >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16)
    return r


def bf16_bits_to_f32(b) -> np.ndarray:
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def bf16_round(x) -> np.ndarray:
    """float32 -> nearest bf16 value, returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


def fmaf(a, b, c) -> np.ndarray:
    """Exact float32 fused multiply-add for float32 inputs.

    The product of two float32 is exact in float64.  The float64 sum is exact
    whenever Knuth's TwoSum error term is zero; elements where it is not are
    recomputed with rational arithmetic, so the result is always the correctly
    rounded float32 of a*b+c.
    """
    a64 = np.asarray(a, dtype=np.float32).astype(np.float64)
    b64 = np.asarray(b, dtype=np.float32).astype(np.float64)
    c64 = np.asarray(c, dtype=np.float32).astype(np.float64)
    a64, b64, c64 = np.broadcast_arrays(a64, b64, c64)
    p = a64 * b64
    s = p + c64
    bb = s - p
    err = (p - (s - bb)) + (c64 - bb)
    out = s.astype(np.float32)
    bad = np.flatnonzero((err != 0) & np.isfinite(s))
    if bad.size:
        from fractions import Fraction
        of, pf, cf = out.reshape(-1), p.reshape(-1), c64.reshape(-1)
        of = of.copy()
        for i in bad:
            exact = Fraction(float(pf[i])) + Fraction(float(cf[i]))
            lo = np.float32(float(exact))  # float(Fraction) is correctly rounded to f64; refine below
            cand = [lo, np.nextafter(lo, np.float32(np.inf)), np.nextafter(lo, np.float32(-np.inf))]
            best = min(cand, key=lambda v: (abs(Fraction(float(v)) - exact), int(np.float32(v).view(np.uint32)) & 1))
            of[i] = best
        out = of.reshape(out.shape)
    return out


# --------------------------------------------------------------------------- wire format


def packed_dim(head_dim: int, nbits: int) -> int:
    """intN_pack.py:35-44"""
    if nbits == 2:
        return head_dim // 4
    if nbits == 3:
        return head_dim * 3 // 8
    if nbits == 4:
        return head_dim // 2
    raise ValueError(f"Unsupported nbits={nbits}, must be 2, 3, or 4")


def qmax(nbits: int) -> int:
    return (1 << (nbits - 1)) - 1


def offset(nbits: int) -> int:
    return 1 << (nbits - 1)


def pack_codes(codes: np.ndarray, nbits: int) -> np.ndarray:
    """Unsigned codes (..., D) -> packed bytes (intN_pack.py:172-222)."""
    c = np.asarray(codes).astype(np.uint32)
    lead, D = c.shape[:-1], c.shape[-1]
    if nbits == 4:
        return ((c[..., 0::2] << 4) | c[..., 1::2]).astype(np.uint8)
    if nbits == 2:
        return ((c[..., 0::4] << 6) | (c[..., 1::4] << 4) | (c[..., 2::4] << 2) | c[..., 3::4]).astype(np.uint8)
    if nbits == 3:
        g = c.reshape(*lead, D // 8, 8)
        w = np.zeros(g.shape[:-1], dtype=np.uint32)
        for i in range(8):
            w |= g[..., i] << np.uint32(21 - 3 * i)
        planes = [(w >> 16) & 0xFF, (w >> 8) & 0xFF, w & 0xFF]
        return np.concatenate(planes, axis=-1).astype(np.uint8)
    raise ValueError(f"Unsupported nbits={nbits}")


def decode_codes(data: np.ndarray, nbits: int) -> np.ndarray:
    """Packed bytes -> unsigned codes, full code range (validate_runtime.py:22-32)."""
    d = np.asarray(data).astype(np.int32)
    lead = d.shape[:-1]
    if nbits == 3:
        n = d.shape[-1] // 3
        w = (d[..., :n] << 16) | (d[..., n:2 * n] << 8) | d[..., 2 * n:3 * n]
        return np.stack([(w >> (21 - 3 * i)) & 7 for i in range(8)], axis=-1).reshape(*lead, n * 8)
    per = 8 // nbits
    mask = (1 << nbits) - 1
    return np.stack([(d >> (8 - nbits * (i + 1))) & mask for i in range(per)], axis=-1).reshape(*lead, d.shape[-1] * per)


def quantize_codes(x: np.ndarray, group_size: int, nbits: int):
    """Golden symmetric quantiser (intN_pack.py:60-107).

    x: float32 array of bf16-representable values, (..., D).
    Returns (unsigned codes uint8 (..., D), scale bits uint16 (..., D/gs)).
    All arithmetic is IEEE float32: amax/qmax (true division), clamp 1e-8,
    round to bf16, divide by the bf16 scale, round-half-even, clamp.
    """
    x = np.asarray(x, dtype=np.float32)
    lead, D = x.shape[:-1], x.shape[-1]
    assert D % group_size == 0
    ng = D // group_size
    xg = x.reshape(*lead, ng, group_size)
    amax = np.abs(xg).max(axis=-1)
    scales = np.maximum(amax / np.float32(qmax(nbits)), np.float32(1e-8)).astype(np.float32)
    sbits = f32_to_bf16_bits(scales)
    sf = bf16_bits_to_f32(sbits)[..., None]
    with np.errstate(over="ignore", invalid="ignore"):
        q = np.rint(xg / sf)  # np.rint is round-half-even, like torch.round
    q = np.clip(q, -qmax(nbits), qmax(nbits)).astype(np.int32) + offset(nbits)
    return q.reshape(*lead, D).astype(np.uint8), sbits


def quantize_and_pack(x: np.ndarray, group_size: int = 128, nbits: int = 4):
    """(data uint8 (..., packed_dim), scale bits uint16 (..., D/gs))."""
    codes, sbits = quantize_codes(x, group_size, nbits)
    return pack_codes(codes, nbits), sbits


def quantize_codes_asym(x: np.ndarray, group_size: int, nbits: int = 2):
    """Golden asymmetric quantiser over the full codebook (intN_pack.py:110-169; the fused writer
    fused_quant_write.py:85-133 uses the same formulas): per group
        scale = bf16(max((xmax - xmin) / (2^n - 1), 1e-8)),  zp = bf16(xmin + 2^(n-1) * scale_f32),
        q = clamp(rint((x - f32(zp)) / f32(scale)), -2^(n-1), 2^(n-1) - 1),  code = q + 2^(n-1).
    All arithmetic is IEEE float32.  Returns (codes uint8 (..., D), scale bits, zp bits uint16 (..., D/gs))."""
    x = np.asarray(x, dtype=np.float32)
    lead, D = x.shape[:-1], x.shape[-1]
    assert D % group_size == 0
    ng = D // group_size
    off = offset(nbits)
    xg = x.reshape(*lead, ng, group_size)
    xmax, xmin = xg.max(axis=-1), xg.min(axis=-1)
    scale = np.maximum((xmax - xmin).astype(np.float32) / np.float32(2 * off - 1), np.float32(1e-8)).astype(np.float32)
    zp = (xmin + (np.float32(off) * scale).astype(np.float32)).astype(np.float32)
    sbits, zbits = f32_to_bf16_bits(scale), f32_to_bf16_bits(zp)
    sf, zf = bf16_bits_to_f32(sbits)[..., None], bf16_bits_to_f32(zbits)[..., None]
    with np.errstate(over="ignore", invalid="ignore"):
        q = np.rint(((xg - zf).astype(np.float32) / sf).astype(np.float32))
    q = np.clip(q, -off, off - 1).astype(np.int32) + off
    return q.reshape(*lead, D).astype(np.uint8), sbits, zbits


def quantize_and_pack_asym(x: np.ndarray, group_size: int = 128, nbits: int = 2):
    """(data uint8 (..., packed_dim), scale bits, zp bits uint16 (..., D/gs))."""
    codes, sbits, zbits = quantize_codes_asym(x, group_size, nbits)
    return pack_codes(codes, nbits), sbits, zbits


def dequant_asym_bf16(data, scale_bits, zp_bits, nbits: int, group_size: int) -> np.ndarray:
    """bf16(fma(code - offset, f32(scale), f32(zp))): what the Stage A kernel feeds its matrix unit
    (int2_qk_scores.cu:66-79: `float(q) * scale + zp` is one fused multiply-add under nvcc's default
    contraction, then __float2bfloat16)."""
    codes = decode_codes(data, nbits).astype(np.float32) - np.float32(offset(nbits))
    shape = codes.shape
    s = bf16_bits_to_f32(scale_bits).reshape(*shape[:-1], -1)[..., None]
    z = bf16_bits_to_f32(zp_bits).reshape(*shape[:-1], -1)[..., None]
    c = codes.reshape(*shape[:-1], -1, group_size)
    return bf16_round(fmaf(c, np.broadcast_to(s, c.shape), np.broadcast_to(z, c.shape))).reshape(shape)


def dequant(data, scale_bits, nbits: int, group_size: int, *, bf16: bool = True) -> np.ndarray:
    """(code - offset) * f32(scale); optionally rounded to bf16 (validate_runtime.py:35-43)."""
    codes = decode_codes(data, nbits).astype(np.float32) - np.float32(offset(nbits))
    shape = codes.shape
    s = bf16_bits_to_f32(scale_bits).reshape(*shape[:-1], -1)
    out = (codes.reshape(*shape[:-1], -1, group_size) * s[..., None]).reshape(shape)
    return bf16_round(out) if bf16 else out


def unpack(data, scale_bits, group_size: int = 128, nbits: int = 4, zp_bits=None) -> np.ndarray:
    """intN_pack.py:227-311: dequantised values rounded to the scale dtype (bf16).  With zero-points the
    rounded product is widened, the zero-point added in fp32 and the sum rounded again (:251-256): two
    roundings, unlike the fused multiply-add of the Stage A kernel (dequant_asym_bf16)."""
    out = dequant(data, scale_bits, nbits, group_size, bf16=True)
    if zp_bits is None:
        return out
    z = bf16_bits_to_f32(zp_bits).reshape(*out.shape[:-1], -1)
    z = np.repeat(z, group_size, axis=-1).astype(np.float32)
    return bf16_round((out.astype(np.float32) + z).astype(np.float32))


def write_cache(x, slots, data, scale_bits, group_size: int, nbits: int) -> None:
    """Quantise + pack + scatter (fused_quant_write.py:135-194,633-743).

    x (T, Hkv, D) float32/bf16-valued; slots (T,) int64, negative = skip;
    data (Hkv, num_slots, P) uint8; scale_bits (Hkv, num_slots, NG) uint16.  In place.
    """
    d, s = quantize_and_pack(x, group_size, nbits)
    for t, slot in enumerate(np.asarray(slots).tolist()):
        if slot < 0:
            continue
        data[:, slot, :] = d[t]
        scale_bits[:, slot, :] = s[t]


# --------------------------------------------------------------------------- paging


def slots_from_block_table(block_table: np.ndarray, max_S: int, block_size: int = BLOCK) -> np.ndarray:
    """slot[b, pos] = bt[b, pos // bs] * bs + pos % bs  (validate_runtime.py:118-121)."""
    pos = np.arange(max_S)
    bt = np.asarray(block_table).astype(np.int64)
    return bt[:, pos // block_size] * block_size + pos % block_size


# --------------------------------------------------------------------------- Stage A


def scores_bf16_model(q, k_data, k_scale_bits, block_table, seq_lens, max_S, H_q, H_kv,
                      block_size, attn_scale, nbits: int, group_size: int, k_zp_bits=None) -> np.ndarray:
    """scores[b,h,s] = f32(sum_d q_d * bf16(code_d*scale_g)) * attn_scale; -inf for s >= seq_len.

    int3_qk_scores.cu:90-99 (bf16 rounding of every dequantised K element),
    :268-311 (fp32 accumulate, multiply by attn_scale on emit, -inf padding).
    The dot product is accumulated in float64 and rounded once to float32; the
    reference's fp32 accumulation order is hardware-defined, so kernels are
    compared with a tolerance (validate_runtime.py:147-148 uses 2e-5).
    """
    q = np.asarray(q, dtype=np.float32)
    B = q.shape[0]
    G = H_q // H_kv
    if k_zp_bits is None:
        khat = dequant(k_data, k_scale_bits, nbits, group_size, bf16=True).astype(np.float64)
    else:   # asymmetric keys (int2_qk_scores.cu:66-79)
        khat = dequant_asym_bf16(k_data, k_scale_bits, k_zp_bits, nbits, group_size).astype(np.float64)
    slots = slots_from_block_table(block_table, max_S, block_size)
    out = np.full((B, H_q, max_S), -np.inf, dtype=np.float32)
    for b in range(B):
        S = int(min(max_S, seq_lens[b]))
        if S <= 0:
            continue
        for hk in range(H_kv):
            kk = khat[hk, slots[b, :S]]                              # (S, D)
            qq = q[b, hk * G:(hk + 1) * G].astype(np.float64)         # (G, D)
            acc = (qq @ kk.T).astype(np.float32)
            out[b, hk * G:(hk + 1) * G, :S] = acc * np.float32(attn_scale)
    return out


def quantize_query_int8(q):
    """Per (row, 32 channels): qs = max(amax/127, 1e-12); qi = clamp(rint(q * (1/qs)), -128, 127).

    int8tc_qk_scores.cu:250-290 (fp32 division, fp32 reciprocal, __float2int_rn).
    Returns (qi int32 (..., 4, 32), qs float32 (..., 4)).
    """
    q = np.asarray(q, dtype=np.float32)
    g = q.reshape(*q.shape[:-1], -1, 32)
    amax = np.abs(g).max(axis=-1)
    qs = np.maximum(amax / np.float32(127.0), np.float32(1e-12)).astype(np.float32)
    inv = (np.float32(1.0) / qs).astype(np.float32)
    qi = np.clip(np.rint((g * inv[..., None]).astype(np.float32)), -128, 127).astype(np.int32)
    return qi, qs


def scores_int8_model(q, k_data, k_scale_bits, block_table, seq_lens, max_S, H_q, H_kv,
                      block_size, attn_scale) -> np.ndarray:
    """INT4 K, g128, int8-quantised Q (int8tc_qk_scores.cu:435-488).

    acc_kk = sum_{d in 32-channel group kk} qi_d * (nibble_d - 8)      exact int32
    s      = fma(acc_3,qs_3, fma(acc_2,qs_2, fma(acc_1,qs_1, acc_0*qs_0)))   fp32, in this order
    score  = (s * f32(k_scale)) * attn_scale                           two fp32 multiplies
    The reference source writes `s += (float)acc * qs` for kk = 0..3 starting from 0;
    contracted to fused multiply-adds that is the chain above.  Every step is exactly
    reproducible, so kernels are compared bit-for-bit.
    """
    q = np.asarray(q, dtype=np.float32)
    B = q.shape[0]
    G = H_q // H_kv
    qi, qs = quantize_query_int8(q)                                  # (B,Hq,4,32), (B,Hq,4)
    codes = decode_codes(k_data, 4).astype(np.int64) - 8             # (Hkv, slots, 128)
    ks = bf16_bits_to_f32(k_scale_bits).reshape(k_data.shape[0], k_data.shape[1], -1)[..., 0]
    slots = slots_from_block_table(block_table, max_S, block_size)
    out = np.full((B, H_q, max_S), -np.inf, dtype=np.float32)
    for b in range(B):
        S = int(min(max_S, seq_lens[b]))
        if S <= 0:
            continue
        for hk in range(H_kv):
            kc = codes[hk, slots[b, :S]].reshape(S, 4, 32)
            ksc = ks[hk, slots[b, :S]]
            for g in range(G):
                h = hk * G + g
                acc = np.einsum("skd,kd->sk", kc, qi[b, h].astype(np.int64)).astype(np.float32)  # exact ints
                s = (acc[:, 0] * qs[b, h, 0]).astype(np.float32)
                for kk in range(1, 4):
                    s = fmaf(acc[:, kk], qs[b, h, kk], s)
                out[b, h, :S] = ((s * ksc).astype(np.float32) * np.float32(attn_scale)).astype(np.float32)
    return out


def scores_int8_model_dense(q, k_data, k_scale_bits, block_table, seq_lens, max_S, H_q, H_kv,
                            block_size, attn_scale) -> np.ndarray:
    """The validator's restatement of the same model: einsum(dequantised Q codes, exact K dequant) * scale
    (validate_runtime.py:46-58,127-145).  Agrees with scores_int8_model to fp32 rounding; used as a pin."""
    q = np.asarray(q, dtype=np.float32)
    qi, qs = quantize_query_int8(q)
    qref = (qi.astype(np.float32) * qs[..., None]).reshape(q.shape).astype(np.float64)
    k0 = dequant(k_data, k_scale_bits, 4, 128, bf16=False).astype(np.float64)
    B = q.shape[0]
    G = H_q // H_kv
    slots = slots_from_block_table(block_table, max_S, block_size)
    out = np.full((B, H_q, max_S), -np.inf, dtype=np.float32)
    for b in range(B):
        S = int(min(max_S, seq_lens[b]))
        for hk in range(H_kv):
            if S > 0:
                out[b, hk * G:(hk + 1) * G, :S] = ((qref[b, hk * G:(hk + 1) * G] @ k0[hk, slots[b, :S]].T)
                                                    * attn_scale).astype(np.float32)
    return out


# --------------------------------------------------------------------------- top-k


def radix_key(scores: np.ndarray) -> np.ndarray:
    """Order-preserving uint32 of an fp32 score (int3_qk_scores.cu:421-424)."""
    u = np.ascontiguousarray(scores, dtype=np.float32).view(np.uint32)
    neg = (u & np.uint32(0x80000000)) != 0
    return np.where(neg, ~u, u | np.uint32(0x80000000)).astype(np.uint32)


def topk_select(scores, seq_lens, block_table, max_S, top_k, block_size: int = BLOCK):
    """Exact top-k per (b, query head) over positions < min(max_S, seq_len)
    (int3_qk_scores.cu:426-554).  The reference emits winners in atomic order and breaks
    threshold ties arbitrarily; this restatement fixes the total order (key descending,
    position ascending) and emits winners in ascending position, then -1 padding.
    Returns (topk_idx, topk_slots) int64 (B, Hq, K).
    """
    scores = np.asarray(scores, dtype=np.float32)
    B, Hq, _ = scores.shape
    idx = np.full((B, Hq, top_k), -1, dtype=np.int64)
    slots = np.full((B, Hq, top_k), -1, dtype=np.int64)
    bt = np.asarray(block_table).astype(np.int64)
    max_blocks = bt.shape[1]
    for b in range(B):
        S = int(min(max_S, seq_lens[b]))
        if S <= 0:
            continue
        for h in range(Hq):
            key = radix_key(scores[b, h, :S]).astype(np.int64)
            order = np.lexsort((np.arange(S), -key))       # key desc, then position asc
            win = np.sort(order[:min(top_k, S)])
            n = win.size
            idx[b, h, :n] = win
            blk = win // block_size
            ok = blk < max_blocks
            sl = np.where(ok, bt[b, np.minimum(blk, max_blocks - 1)] * block_size + win % block_size, -1)
            slots[b, h, :n] = sl
    return idx, slots


def softmax_stats(scores, seq_lens, max_S):
    """m = row max over valid positions (0 if not finite); inv_z = 1/sum exp(s-m) (0 if sum <= 0).
    int8tc_qk_scores.cu:1790-1799, int4_softmax_v.cu:124-160."""
    scores = np.asarray(scores, dtype=np.float32)
    B, Hq, _ = scores.shape
    m = np.zeros((B, Hq), dtype=np.float32)
    iz = np.zeros((B, Hq), dtype=np.float32)
    for b in range(B):
        S = int(min(max_S, seq_lens[b]))
        if S <= 0:
            continue
        row = scores[b, :, :S].astype(np.float64)
        mm = row.max(axis=-1)
        mm = np.where(np.isfinite(mm), mm, 0.0)
        with np.errstate(over="ignore", invalid="ignore"):
            z = np.exp(row - mm[:, None]).sum(axis=-1)
        m[b] = mm.astype(np.float32)
        iz[b] = np.where(z > 0, 1.0 / z, 0.0).astype(np.float32)
    return m, iz


# --------------------------------------------------------------------------- Stage B


def softmax_v(scores, v_data, v_scale_bits, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
              block_size, nbits: int, group_size: int):
    """o_hat = sum_s p_s * Vhat_s ; o_old_unnorm = sum_{s in topk} p_s * Vhat_s ; W = sum_{s in topk} p_s
    with p = softmax(scores[:seq_len]) and Vhat = (code - offset) * f32(scale) WITHOUT bf16 rounding
    (int2_softmax_v.cu:101-144,681-706,738-788; int4_softmax_v.cu:162-176,709-735;
     validate_runtime.py:164-172).  top-k entries < 0 or >= seq_len are skipped.
    Accumulated in float64, returned as float32.
    """
    scores = np.asarray(scores, dtype=np.float32)
    B = scores.shape[0]
    G = H_q // H_kv
    D = HEAD_DIM
    v0 = dequant(v_data, v_scale_bits, nbits, group_size, bf16=False).astype(np.float64)
    slots = slots_from_block_table(block_table, max_S, block_size)
    o_hat = np.zeros((B, H_q, D), dtype=np.float32)
    o_old = np.zeros((B, H_q, D), dtype=np.float32)
    W = np.zeros((B, H_q), dtype=np.float32)
    m, iz = softmax_stats(scores, seq_lens, max_S)
    for b in range(B):
        S = int(min(max_S, seq_lens[b]))
        if S <= 0:
            continue
        for h in range(H_q):
            hk = h // G
            with np.errstate(over="ignore", invalid="ignore"):
                p = np.exp(scores[b, h, :S].astype(np.float64) - float(m[b, h])) * float(iz[b, h])
            p = np.nan_to_num(p, nan=0.0, posinf=0.0, neginf=0.0)
            vv = v0[hk, slots[b, :S]]
            o_hat[b, h] = (p @ vv).astype(np.float32)
            if topk_idx is not None:
                t = np.asarray(topk_idx[b, h]).astype(np.int64)
                t = t[(t >= 0) & (t < S)]
                o_old[b, h] = (p[t] @ vv[t]).astype(np.float32)
                W[b, h] = np.float32(p[t].sum())
    return o_hat, o_old, W


def softmax_v_int8_tiles(scores, softmax_m, softmax_inv_z, v_data, v_scale_bits, block_table, seq_lens,
                         topk_idx, max_S, H_q, H_kv, block_size, splits: int = 8):
    """INT4 V with int8-quantised P (int8tc_softmax_v_fused.cu:1203-1236,1298-1311;
    validate_runtime_edges.py:146-164).  The sequence is cut into `splits` ranges of
    ceil(max_S/splits) positions (:1049-1052); a range is walked in tiles of two pages starting at the page of
    its first position (:1178); per tile and per row:
      pv = p * f32(v_scale); rs = amax|pv| / 127; pq = clamp(rint(pv / rs), -127, 127) (0 if rs == 0)
      o_hat += f32(sum_t pq_t * (nibble - 8)) * rs
    o_old_unnorm and W use the exact fp32 weights.
    """
    scores = np.asarray(scores, dtype=np.float32)
    B = scores.shape[0]
    G = H_q // H_kv
    D = HEAD_DIM
    codes = decode_codes(v_data, 4).astype(np.int64) - 8
    vs_all = bf16_bits_to_f32(v_scale_bits).reshape(v_data.shape[0], v_data.shape[1], -1)[..., 0]
    slots = slots_from_block_table(block_table, max_S, block_size)
    o_hat = np.zeros((B, H_q, D), dtype=np.float32)
    o_old = np.zeros((B, H_q, D), dtype=np.float32)
    W = np.zeros((B, H_q), dtype=np.float32)
    chunk = (max_S + splits - 1) // splits
    for b in range(B):
        S = int(min(max_S, seq_lens[b]))
        if S <= 0:
            continue
        for h in range(H_q):
            hk = h // G
            with np.errstate(over="ignore", invalid="ignore"):
                p = (np.exp((scores[b, h, :S] - softmax_m[b, h]).astype(np.float32).astype(np.float64))
                     * float(softmax_inv_z[b, h])).astype(np.float32)
            p = np.nan_to_num(p, nan=0.0, posinf=0.0, neginf=0.0)
            vs = vs_all[hk, slots[b, :S]]
            vc = codes[hk, slots[b, :S]]
            acc = np.zeros(D, dtype=np.float64)
            for s0 in range(0, S, chunk):
                s1 = min(s0 + chunk, S)
                # tiles are pairs of pages counted from the page that holds s0 (int8tc_softmax_v_fused.cu:1052,1178);
                # positions of a tile outside [s0, s1) carry zero weight (:1218)
                origin = (s0 // block_size) * block_size
                for tile0 in range(origin, s1, 2 * block_size):
                    t0, t1 = max(tile0, s0), min(tile0 + 2 * block_size, s1)
                    pv = (p[t0:t1] * vs[t0:t1]).astype(np.float32)
                    amax = np.abs(pv).max() if t1 > t0 else np.float32(0)
                    rs = np.float32(amax) / np.float32(127.0)
                    if rs > 0:
                        inv = np.float32(1.0) / rs
                        pq = np.clip(np.rint((pv * inv).astype(np.float32)), -127, 127).astype(np.int64)
                        acc += (pq @ vc[t0:t1]).astype(np.float64) * float(rs)
            o_hat[b, h] = acc.astype(np.float32)
            if topk_idx is not None:
                t = np.asarray(topk_idx[b, h]).astype(np.int64)
                t = t[(t >= 0) & (t < S)]
                pvx = p[t].astype(np.float64) * vs[t].astype(np.float64)
                o_old[b, h] = (pvx @ vc[t].astype(np.float64)).astype(np.float32)
                W[b, h] = np.float32(p[t].astype(np.float64).sum())
    return o_hat, o_old, W


# --------------------------------------------------------------------------- CPU correction + merge


def cpu_topk_attn(q, k_shadow, v_shadow, head_map, ts_buf, scale):
    """Exact softmax attention over the top-k slots from the bf16 shadow (cpu_topk_attn.cpp:602-690).

    q (B,Hq,D), k_shadow/v_shadow (Hkv, num_slots, D): bf16-valued float32; head_map, ts_buf (B,Hq,K) int64.
    Invalid slots (<0 or >= num_slots) score -inf; a row with no valid slot, or a non-positive /
    non-finite denominator, yields zeros.  Output is rounded to bf16 (returned as float32).
    """
    q = np.asarray(q, dtype=np.float32)
    B, Hq, D = q.shape
    num_slots = k_shadow.shape[1]
    out = np.zeros((B, Hq, D), dtype=np.float32)
    for b in range(B):
        for h in range(Hq):
            sl = np.asarray(ts_buf[b, h]).astype(np.int64)
            hm = np.asarray(head_map[b, h]).astype(np.int64)
            ok = (sl >= 0) & (sl < num_slots)
            if not ok.any():
                continue
            kk = k_shadow[hm[ok], sl[ok]].astype(np.float64)
            vv = v_shadow[hm[ok], sl[ok]].astype(np.float64)
            s = ((kk @ q[b, h].astype(np.float64)).astype(np.float32) * np.float32(scale)).astype(np.float64)
            with np.errstate(over="ignore", invalid="ignore"):
                e = np.exp(s - s.max())
            den = e.sum()
            if not (den > 0) or not np.isfinite(den):
                continue
            out[b, h] = bf16_round(((e / den) @ vv).astype(np.float32))
    return out


def blend_unnorm(o_hat, o_old_unnorm, W, o_new):
    """out = bf16_rne(fma(W, f32(o_new), o_hat) - o_old_unnorm)  (blend.cu:221-224:
    `hat + w*n - old` evaluated left to right, the multiply-add contracted)."""
    o_hat = np.asarray(o_hat, dtype=np.float32)
    w = np.asarray(W, dtype=np.float32)[..., None]
    v = (fmaf(np.broadcast_to(w, o_hat.shape), np.asarray(o_new, dtype=np.float32), o_hat)
         - np.asarray(o_old_unnorm, dtype=np.float32)).astype(np.float32)
    return bf16_round(v)


def select_top_k(config_top_k: int, seq_len: int, supported):
    """decode_path.py:1156-1182."""
    requested, length = int(config_top_k), int(seq_len)
    configured = [k for k in supported if 0 < k <= requested]
    if not configured or length <= 0:
        return None
    candidates = [k for k in configured if k <= length]
    return max(candidates) if candidates else min(configured)


def head_map(B: int, H_q: int, num_groups: int, K: int) -> np.ndarray:
    """decode_path.py:400-408: head_map[b,h,k] = h // num_groups."""
    hm = (np.arange(H_q, dtype=np.int64) // num_groups)[None, :, None]
    return np.ascontiguousarray(np.broadcast_to(hm, (B, H_q, K)))


# --------------------------------------------------------------------------- end-to-end reference


def decode_reference(q, k_data, k_scale_bits, v_data, v_scale_bits, block_table, seq_lens, max_S,
                     H_q, H_kv, block_size, attn_scale, top_k, scheme: str, k_shadow=None, v_shadow=None,
                     group_size: int | None = None, k_model: str | None = None, k_zp_bits=None):
    """Whole per-layer decode step in the reference's order (decode_path.py:2081-2131,2785-2935,3126-3226).
    scheme: "k<kb>v<vb>" with kb, vb in {2, 3, 4}; group_size defaults to 64 for "k3v2" and 128 otherwise
    (jetfire_vllm/artifact.py:59).  k_model: "bf16" (bf16 q times bf16-rounded keys: the INT2 / INT3 / native
    INT4 Stage A) or "int8" (INT4 keys with one scale per slot through the int8 tensor-core Stage A,
    decode_path.py:2013-2024); default "int8" for 4-bit keys at group 128, else "bf16".
    Returns a dict of every intermediate."""
    kb, vb = int(scheme[1]), int(scheme[3])
    if group_size is None:
        group_size = 64 if scheme == "k3v2" else 128
    if k_model is None:
        k_model = "int8" if (kb == 4 and group_size == 128) else "bf16"
    if k_model == "int8":
        assert kb == 4 and group_size == 128
        sc = scores_int8_model(q, k_data, k_scale_bits, block_table, seq_lens, max_S, H_q, H_kv,
                               block_size, attn_scale)
    else:
        sc = scores_bf16_model(q, k_data, k_scale_bits, block_table, seq_lens, max_S, H_q, H_kv,
                               block_size, attn_scale, kb, group_size, k_zp_bits)
    vg = group_size
    idx, slots = topk_select(sc, seq_lens, block_table, max_S, top_k, block_size)
    m, iz = softmax_stats(sc, seq_lens, max_S)
    o_hat, o_old, W = softmax_v(sc, v_data, v_scale_bits, block_table, seq_lens, idx, max_S, H_q, H_kv,
                                block_size, vb, vg)
    res = dict(scores=sc, topk_idx=idx, topk_slots=slots, softmax_m=m, softmax_inv_z=iz,
               o_hat=o_hat, o_old_unnorm=o_old, W=W)
    if k_shadow is not None:
        B = np.asarray(q).shape[0]
        hm = head_map(B, H_q, H_q // H_kv, top_k)
        o_new = cpu_topk_attn(q, k_shadow, v_shadow, hm, slots, attn_scale)
        res["o_new"] = o_new
        res["out"] = blend_unnorm(o_hat, o_old, W, o_new)
    return res


PINNED_BY = {
    "pack_codes/decode_codes": "reference wire vectors tests/test_int_pack.py:14-18 (0x6E; 0x29,0xCB,0xBC planar; 0x1F), "
                               "round trip, closed form intN_pack.py:6-29",
    "quantize_codes": "scale==1 vectors and zero-group case (tests/test_int_pack.py:10-35); invariants codes in "
                      "[1, 2^n-1], |xhat-x| <= scale/2 unless clamped; brute-force ties (.5 -> even); "
                      "amax not bf16-representable -> clamp",
    "scores_bf16_model": "one-hot q gives the dequantised channel; agreement with dense float64 einsum",
    "quantize_codes_asym": "no vector in the reference's tests; pinned by what the formulas fix: the group minimum maps "
                           "to code 0 and the maximum to code 2^n-1, scale and zp reproduce intN_pack.py:121's closed "
                           "form on exactly representable inputs, |xhat - x| <= scale/2 + rounding of zp inside the "
                           "range, a constant group gives scale 1e-8 clamped, and the asymmetric grid is never worse "
                           "than the symmetric one by more than 5 % MSE (the reference's own self-test, intN_pack.py:375-403)",
    "scores_int8_model": "agreement with validator restatement scores_int8_model_dense (validate_runtime.py:46-58) "
                         "within fp32 rounding; one-hot q closed form",
    "topk_select": "brute-force sort on tiny inputs; S<K: every valid position once then -1 "
                   "(validate_runtime_edges.py:124-142); value multiset equals a plain descending sort",
    "softmax_v": "K>=S => W=1 and o_old==o_hat; uniform scores => mean of Vhat; 0<=W<=1",
    "softmax_v_int8_tiles": "converges to softmax_v within 3e-3 (validate_runtime.py:173-176); exact when P*vs is "
                            "constant inside a tile",
    "cpu_topk_attn": "K=1 => bf16(V row); invalid slots masked (validate_runtime_edges.py:172-177)",
    "blend_unnorm": "W=0, old=0 => bf16(o_hat); shadow==dequant and K>=S => out==o_new",
    "select_top_k/head_map": "reference tables tests/test_runtime_edge_cases.py:13-35",
}
