"""The reference's PyTorch CPU decode path, restated: unpack + dequant + attention + top-k.

TEST / BENCHMARK INFRASTRUCTURE ONLY (the CPU-baseline leg of bench.py and the tests import it).
It follows the torch arithmetic of jetfire_vllm/kernels/intN_pack.py:227-311 (`unpack`: decode the
codes, multiply by the fp32 scale, round to bf16) and the dense math of
jetfire_vllm/bench/topk_quality_probe.py:154-174 (scores = q . K-hat^T * D^-1/2, softmax,
P . V-hat, topk) on an unpaged (H_kv, S, P) cache.  Pinned by tests/test_oracle_attention.py
(agreement with the numpy oracle on seeded inputs).
"""
from __future__ import annotations

import torch


def unpack(data: torch.Tensor, scales: torch.Tensor, group_size: int, nbits: int) -> torch.Tensor:
    """(..., P) uint8 + (..., D/gs) bf16 -> (..., D) bf16 (intN_pack.py:227-311)."""
    lead = data.shape[:-1]
    d = data.to(torch.int32)
    if nbits == 4:
        xq = torch.stack([(d >> 4) & 0xF, d & 0xF], dim=-1).reshape(*lead, -1) - 8
    elif nbits == 2:
        xq = torch.stack([(d >> 6) & 3, (d >> 4) & 3, (d >> 2) & 3, d & 3], dim=-1).reshape(*lead, -1) - 2
    elif nbits == 3:
        n = d.shape[-1] // 3
        w = (d[..., :n] << 16) | (d[..., n:2 * n] << 8) | d[..., 2 * n:]
        xq = torch.stack([(w >> (21 - 3 * i)) & 7 for i in range(8)], dim=-1).reshape(*lead, -1) - 4
    else:
        raise ValueError(f"Unsupported nbits={nbits}")
    D = xq.shape[-1]
    xg = xq.float().reshape(*lead, D // group_size, group_size)
    return (xg * scales.float().unsqueeze(-1)).reshape(*lead, D).to(scales.dtype)


def decode_path(q, k_data, k_scales, v_data, v_scales, group_size: int, k_nbits: int, v_nbits: int, top_k: int):
    """q (B,Hq,D) bf16; caches (B, H_kv, S, P) uint8 / (B, H_kv, S, NG) bf16 (one contiguous cache per sequence).
    Returns (o_hat (B,Hq,D) fp32, topk_idx (B,Hq,K) int64)."""
    B, Hq, D = q.shape
    Hkv = k_data.shape[1]
    G = Hq // Hkv
    khat = unpack(k_data, k_scales, group_size, k_nbits).float()          # (B, Hkv, S, D)
    vhat = unpack(v_data, v_scales, group_size, v_nbits).float()
    qg = q.float().reshape(B, Hkv, G, D)
    scores = torch.einsum("bhgd,bhsd->bhgs", qg, khat) * (D ** -0.5)
    probs = torch.softmax(scores, dim=-1)
    o_hat = torch.einsum("bhgs,bhsd->bhgd", probs, vhat).reshape(B, Hq, D)
    idx = scores.topk(min(top_k, scores.shape[-1]), dim=-1).indices.reshape(B, Hq, -1)
    return o_hat, idx


def int8_q_scores(q: torch.Tensor, k_data: torch.Tensor, k_scales: torch.Tensor, attn_scale: float) -> torch.Tensor:
    """The int8-quantised-query scoring model of the reference's INT4 Stage A
    (jetfire_vllm/csrc/int8tc_qk_scores.cu:250-290 query quantisation, :435-469 rescale order), restated with torch
    so that it can run on the GPU at full context lengths:
        qs_kk = max(amax_{32 channels}|q| / 127, 1e-12), qi = clamp(rint(q * (1 / qs_kk)), -128, 127)
        acc_kk = sum_{32} qi * (nibble - 8)                      exact integers
        s = fma(acc_3, qs_3, fma(acc_2, qs_2, fma(acc_1, qs_1, acc_0 * qs_0)));  score = (s * k_scale) * attn_scale
    q (G, 128) bf16 (the query heads of one kv-head), k_data (S, 64) uint8, k_scales (S,) or (S, 1) bf16 -> (G, S) fp32.
    The query is quantised on the host (IEEE division); every fused multiply-add is evaluated in float64, where the
    product is exact, and rounded once to fp32."""
    dev = k_data.device
    qf = q.detach().float().cpu().reshape(-1, 4, 32)
    qs = torch.clamp(qf.abs().amax(-1) / 127.0, min=1e-12)                       # (G, 4) fp32
    inv = 1.0 / qs
    qi = torch.clamp(torch.round(qf * inv[..., None]), -128, 127)                # (G, 4, 32), round half to even
    d = k_data.to(torch.int32)
    codes = (torch.stack([(d >> 4) & 0xF, d & 0xF], dim=-1).reshape(d.shape[0], 4, 32) - 8).float()   # (S, 4, 32)
    acc = torch.einsum("skd,gkd->gsk", codes, qi.to(dev))                        # integers below 2^24: exact in fp32
    qs64 = qs.to(dev).double()
    s = (acc[..., 0].double() * qs64[:, None, 0]).float()
    for kk in range(1, 4):
        s = (acc[..., kk].double() * qs64[:, None, kk] + s.double()).float()
    ks = k_scales.reshape(-1).float()
    return (s * ks[None, :]) * torch.tensor(attn_scale, dtype=torch.float32, device=dev)
