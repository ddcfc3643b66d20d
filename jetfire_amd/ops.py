"""Torch-facing operators over the C ABI.

Function names, positional argument order, dtypes, return values and error behaviour follow the
reference's extension modules (jetfire_vllm/csrc/*.cu pybind blocks and
jetfire_vllm/kernels/fused_quant_write.py), so an adapter written for those calls these unchanged.
Tensors are only used for device memory and the current stream; all arithmetic is in the HIP library.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional

import torch

from . import _lib

HEAD_DIM = 128
SUPPORTED_TOP_K = (32, 64, 128, 256, 512, 1024, 2048, 4096, 8192)
FUSED_TOP_K = SUPPORTED_TOP_K                           # widths of the one-pass form and of the fast stage-wise forms
FUSED_MAX_SLOTS = 1 << 26                               # slots per kv-head tensor those forms address (4 GB of 64-byte rows)

_workspaces: dict = {}
_retired_workspaces: list = []   # superseded buffers, kept because captured graphs may still point at them


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _workspace(device: torch.device, nbytes: int, tag: str) -> torch.Tensor:
    """Per-(device, stream, tag) scratch buffer that only grows; safe under stream ordering.  A buffer that is
    replaced by a larger one is kept alive: a HIP graph captured earlier on the stream has its address baked into
    its kernels, and the allocator must not hand that memory to anyone else while the graph can be replayed."""
    key = (device, torch.cuda.current_stream(device).cuda_stream, tag)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _retired_workspaces.append(buf)
        buf = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


# the nine symmetric (key bits, value bits) pairs of the fused step: name -> 10 * key bits + value bits
FUSED_SCHEMES = {f"k{kb}v{vb}": 10 * kb + vb for kb in (2, 3, 4) for vb in (2, 3, 4)}
# and the asymmetric INT2 keys (four levels, zero-points in k_zp): key digit 1
FUSED_SCHEMES.update({f"a2v{vb}": 10 + vb for vb in (2, 3, 4)})
# and INT4 keys scored with the bf16 model (what the reference runs for INT4 keys with 64-channel groups): key digit 5
FUSED_SCHEMES.update({f"b4v{vb}": 50 + vb for vb in (2, 3, 4)})


def reserve_fused_workspace(scheme: str, B: int, H_q: int, H_kv: int, max_S: int, top_k: int, device) -> int:
    """Size the current stream's fused-scan workspace for a shape ahead of time (before a graph capture, so that
    no capture or later eager call has to grow it).  Returns the size in bytes."""
    scheme_id = FUSED_SCHEMES[scheme]
    need = int(_lib.load().jf_fused_workspace_bytes(scheme_id, int(B), int(H_q), int(H_kv), int(max_S), int(top_k)))
    return int(_workspace(torch.device(device), need, "fused").numel())


def _gpu(*ts: torch.Tensor) -> None:
    for t in ts:
        _check(t.is_cuda, "all inputs must be on the GPU")


# --------------------------------------------------------------------------- quantise-on-append


def _quant_write(x, slots, out_data, out_scale, group_size: int, nbits: int) -> None:
    lib = _lib.load()
    _check(x.is_cuda and x.dtype == torch.bfloat16, "key/value tokens must be bf16 on the GPU")
    _check(x.dim() == 3 and x.shape[2] == HEAD_DIM, "tokens must be (T, H_kv, 128)")
    _check(x.stride(2) == 1, "tokens must be contiguous in the last dimension")
    _check(slots.is_cuda and slots.dtype == torch.int64 and slots.dim() == 1 and slots.shape[0] == x.shape[0],
           "slots must be (T,) int64 on the token device")
    T, H_kv, D = x.shape
    _check(D % group_size == 0, f"D={D} not divisible by gs={group_size}")
    if out_scale.dim() == 2:
        out_scale = out_scale.unsqueeze(-1)
    _check(out_data.dtype == torch.uint8 and out_scale.dtype == torch.bfloat16, "cache must be uint8 data + bf16 scales")
    _check(out_data.shape[0] == H_kv and out_data.shape[2] == D * nbits // 8 and out_data.stride(2) == 1,
           f"cache data must be (H_kv, num_slots, {D * nbits // 8})")
    _check(out_scale.shape[0] == H_kv and out_scale.shape[2] == D // group_size and out_scale.stride(2) == 1,
           "cache scales must be (H_kv, num_slots, D/group_size)")
    slots = slots.contiguous()
    _lib.check(lib.jf_quant_write_sym(
        x.data_ptr(), x.stride(0), x.stride(1), slots.data_ptr(), T, H_kv,
        out_data.data_ptr(), out_data.stride(0), out_data.stride(1),
        out_scale.data_ptr(), out_scale.stride(0), out_scale.stride(1),
        out_data.shape[1], int(group_size), nbits, _stream(x)))


def fused_quant_write_int2_sym(val_tok, slots, out_data, out_scale, group_size: int) -> None:
    """fused_quant_write.py:242-270"""
    _quant_write(val_tok, slots, out_data, out_scale, group_size, 2)


def fused_quant_write_int3_sym(value_tok, slot_idx, v_data, v_scales, group_size: int) -> None:
    """fused_quant_write.py:746-781"""
    _quant_write(value_tok, slot_idx, v_data, v_scales, group_size, 3)


def fused_quant_write_int4_sym(value_tok, slot_idx, v_data, v_scales, group_size: int) -> None:
    """fused_quant_write.py:337-369"""
    _quant_write(value_tok, slot_idx, v_data, v_scales, group_size, 4)


def fused_quant_write_int2_asym(key_tok, slots, out_data, out_scale, out_zp, group_size: int) -> None:
    """fused_quant_write.py:204-239: asymmetric INT2 keys over the full codebook, in place."""
    lib = _lib.load()
    _check(key_tok.is_cuda and key_tok.dtype == torch.bfloat16 and key_tok.dim() == 3 and key_tok.shape[2] == HEAD_DIM,
           "key_tok must be (T, H_kv, 128) bf16 on the GPU")
    _check(key_tok.stride(2) == 1, "tokens must be contiguous in the last dimension")
    T, H_kv, D = key_tok.shape
    _check(D % group_size == 0, f"D={D} not divisible by gs={group_size}")
    if out_scale.dim() == 2:
        out_scale = out_scale.unsqueeze(-1)
    if out_zp.dim() == 2:
        out_zp = out_zp.unsqueeze(-1)
    _check(out_data.dtype == torch.uint8 and out_data.shape[0] == H_kv and out_data.shape[2] == D // 4
           and out_data.stride(2) == 1, "cache data must be (H_kv, num_slots, 32) uint8")
    for t in (out_scale, out_zp):
        _check(t.dtype == torch.bfloat16 and t.shape[0] == H_kv and t.shape[2] == D // group_size and t.stride(2) == 1,
               "scales / zero-points must be (H_kv, num_slots, D / group_size) bf16")
    _check(slots.is_cuda and slots.dtype == torch.int64 and slots.shape == (T,), "slots must be (T,) int64")
    slots = slots.contiguous()
    _lib.check(lib.jf_quant_write_int2_asym(
        key_tok.data_ptr(), key_tok.stride(0), key_tok.stride(1), slots.data_ptr(), T, H_kv,
        out_data.data_ptr(), out_data.stride(0), out_data.stride(1), out_scale.data_ptr(), out_scale.stride(0),
        out_scale.stride(1), out_zp.data_ptr(), out_zp.stride(0), out_zp.stride(1), out_data.shape[1], int(group_size),
        _stream(key_tok)))


def fused_quant_write_int4_sym_kv(key_tok, value_tok, slot_idx, k_data, k_scales, v_data, v_scales,
                                  group_size: int) -> None:
    """fused_quant_write.py:552-617 (K and V in one launch)."""
    lib = _lib.load()
    _check(key_tok.is_cuda and value_tok.is_cuda, "tokens must be on the GPU")
    _check(key_tok.dtype == torch.bfloat16 and value_tok.dtype == torch.bfloat16, "tokens must be bf16")
    _check(value_tok.shape == key_tok.shape and key_tok.dim() == 3 and key_tok.shape[2] == HEAD_DIM,
           "key/value tokens must both be (T, H_kv, 128)")
    _check(key_tok.stride(2) == 1 and value_tok.stride(2) == 1, "tokens must be contiguous in the last dimension")
    T, H_kv, D = key_tok.shape
    _check(D % group_size == 0, f"D={D} not divisible by gs={group_size}")
    if k_scales.dim() == 2:
        k_scales = k_scales.unsqueeze(-1)
    if v_scales.dim() == 2:
        v_scales = v_scales.unsqueeze(-1)
    for d, s in ((k_data, k_scales), (v_data, v_scales)):
        _check(d.dtype == torch.uint8 and s.dtype == torch.bfloat16, "cache must be uint8 data + bf16 scales")
        _check(d.shape[0] == H_kv and d.shape[2] == D // 2 and d.stride(2) == 1, "cache data must be (H_kv, num_slots, 64)")
        _check(s.shape[0] == H_kv and s.shape[2] == D // group_size and s.stride(2) == 1, "bad cache scales shape")
    _check(slot_idx.is_cuda and slot_idx.dtype == torch.int64 and slot_idx.shape == (T,), "slots must be (T,) int64")
    slot_idx = slot_idx.contiguous()
    _lib.check(lib.jf_quant_write_int4_sym_kv(
        key_tok.data_ptr(), key_tok.stride(0), key_tok.stride(1),
        value_tok.data_ptr(), value_tok.stride(0), value_tok.stride(1),
        slot_idx.data_ptr(), T, H_kv,
        k_data.data_ptr(), k_data.stride(0), k_data.stride(1), k_scales.data_ptr(), k_scales.stride(0), k_scales.stride(1),
        v_data.data_ptr(), v_data.stride(0), v_data.stride(1), v_scales.data_ptr(), v_scales.stride(0), v_scales.stride(1),
        k_data.shape[1], int(group_size), _stream(key_tok)))


def packed_dim(head_dim: int, nbits: int) -> int:
    """intN_pack.py:35-44: bytes of one packed row."""
    _check(nbits in (2, 3, 4), f"Unsupported nbits={nbits}")
    _check(head_dim % 8 == 0, f"head_dim={head_dim} must be a multiple of 8")
    return head_dim * nbits // 8


def _rows_for_pack(x, name: str):
    _check(x.is_cuda and x.dtype == torch.bfloat16, f"{name}: x must be bf16 on the GPU")
    _check(x.dim() >= 1 and x.shape[-1] == HEAD_DIM, f"{name}: the last dimension must be {HEAD_DIM}")
    return x.reshape(-1, 1, HEAD_DIM), tuple(x.shape[:-1])


def quantize_and_pack(x, group_size: int = 128, nbits: int = 4):
    """intN_pack.py:60-107 on the GPU: (..., 128) bf16 -> data (..., 128 * nbits / 8) uint8, scales
    (..., 128 / group_size) bf16.  The rows go through the cache writer with the identity slot mapping."""
    _check(nbits in (2, 3, 4), f"Unsupported nbits={nbits}")
    rows, lead = _rows_for_pack(x, "quantize_and_pack")
    n = rows.shape[0]
    data = torch.empty(1, n, HEAD_DIM * nbits // 8, dtype=torch.uint8, device=x.device)
    scales = torch.empty(1, n, HEAD_DIM // group_size, dtype=torch.bfloat16, device=x.device)
    if n:
        _quant_write(rows, torch.arange(n, dtype=torch.int64, device=x.device), data, scales, group_size, nbits)
    return data.view(*lead, data.shape[-1]), scales.view(*lead, scales.shape[-1])


def quantize_and_pack_asym(x, group_size: int = 128, nbits: int = 2):
    """intN_pack.py:110-169 on the GPU, for the one width whose zero-point form has kernels (INT2):
    returns data, scales, zps."""
    if nbits != 2:
        raise NotImplementedError("only INT2 has an asymmetric (zero-point) form in this library")
    rows, lead = _rows_for_pack(x, "quantize_and_pack_asym")
    n = rows.shape[0]
    data = torch.empty(1, n, HEAD_DIM // 4, dtype=torch.uint8, device=x.device)
    scales = torch.empty(1, n, HEAD_DIM // group_size, dtype=torch.bfloat16, device=x.device)
    zps = torch.empty_like(scales)
    if n:
        fused_quant_write_int2_asym(rows, torch.arange(n, dtype=torch.int64, device=x.device), data, scales, zps,
                                    group_size)
    return data.view(*lead, data.shape[-1]), scales.view(*lead, scales.shape[-1]), zps.view(*lead, zps.shape[-1])


def unpack(data, scales, group_size: int = 128, nbits: int = 4, zps=None):
    """intN_pack.py:227-256 on the GPU: packed rows -> dequantised (..., 128) bf16."""
    lib = _lib.load()
    _check(nbits in (2, 3, 4), f"Unsupported nbits={nbits}")
    _check(data.is_cuda and data.dtype == torch.uint8 and data.shape[-1] == HEAD_DIM * nbits // 8,
           f"unpack: data must be (..., {HEAD_DIM * nbits // 8}) uint8 on the GPU")
    ng = HEAD_DIM // group_size
    lead = tuple(data.shape[:-1])
    for t, name in ((scales, "scales"), (zps, "zps")):
        if t is not None:
            _check(t.is_cuda and t.dtype == torch.bfloat16 and tuple(t.shape) == lead + (ng,),
                   f"unpack: {name} must be {lead + (ng,)} bf16 on the GPU")
    d2 = data.reshape(-1, data.shape[-1]).contiguous()
    s2 = scales.reshape(-1, ng).contiguous()
    z2 = zps.reshape(-1, ng).contiguous() if zps is not None else None
    out = torch.empty(d2.shape[0], HEAD_DIM, dtype=torch.bfloat16, device=data.device)
    _lib.check(lib.jf_unpack(d2.data_ptr(), d2.stride(0), s2.data_ptr(), s2.stride(0), _ptr(z2),
                             z2.stride(0) if z2 is not None else 0, d2.shape[0], int(group_size), nbits,
                             out.data_ptr(), out.stride(0), _stream(data)))
    return out.view(*lead, HEAD_DIM)


def host_buffer_device_pointer(t: torch.Tensor) -> int:
    """Address under which the GPU reaches the pinned host tensor `t`; raises for pageable memory."""
    import ctypes
    lib = _lib.load()
    _check(not t.is_cuda, "expected a host tensor")
    out = ctypes.c_void_p()
    _lib.check(lib.jf_host_buffer_device_pointer(t.data_ptr(), ctypes.byref(out)))
    return int(out.value)


def shadow_write(key_tok, value_tok, slot_idx, k_shadow, v_shadow, *, k_shadow_dev: int | None = None,
                 v_shadow_dev: int | None = None) -> None:
    """Mirror the appended rows into the pinned bf16 host shadows `(H_kv, num_slots, 128)`:
    `k_shadow[h, slot_idx[t]] = key_tok[t, h]` (cache_store.py:686-759,1224-1338 in one kernel launch on the
    current stream; asynchronous).  `*_dev` are the shadows' device-visible addresses when the caller has
    looked them up already."""
    lib = _lib.load()
    _check(key_tok.is_cuda and value_tok.is_cuda, "tokens must be on the GPU")
    _check(key_tok.dtype == torch.bfloat16 and value_tok.dtype == torch.bfloat16, "tokens must be bf16")
    _check(value_tok.shape == key_tok.shape and key_tok.dim() == 3 and key_tok.shape[2] == HEAD_DIM,
           "key/value tokens must both be (T, H_kv, 128)")
    _check(key_tok.stride(2) == 1 and value_tok.stride(2) == 1, "tokens must be contiguous in the last dimension")
    T, H_kv, D = key_tok.shape
    for s in (k_shadow, v_shadow):
        _check(not s.is_cuda and s.dtype == torch.bfloat16 and s.dim() == 3 and s.shape[0] == H_kv and s.shape[2] == D
               and s.stride(2) == 1, "shadow must be a (H_kv, num_slots, 128) bf16 host tensor")
    _check(k_shadow.shape == v_shadow.shape and k_shadow.stride() == v_shadow.stride(), "K and V shadows must match")
    _check(slot_idx.is_cuda and slot_idx.dtype == torch.int64 and slot_idx.shape == (T,), "slots must be (T,) int64")
    slot_idx = slot_idx.contiguous()
    kd = host_buffer_device_pointer(k_shadow) if k_shadow_dev is None else int(k_shadow_dev)
    vd = host_buffer_device_pointer(v_shadow) if v_shadow_dev is None else int(v_shadow_dev)
    _lib.check(lib.jf_shadow_write(
        key_tok.data_ptr(), key_tok.stride(0), key_tok.stride(1),
        value_tok.data_ptr(), value_tok.stride(0), value_tok.stride(1),
        slot_idx.data_ptr(), T, H_kv, kd, vd, k_shadow.stride(0), k_shadow.stride(1), k_shadow.shape[1],
        _stream(key_tok)))


# --------------------------------------------------------------------------- Stage A
#
# The reference's Stage A and Stage B operators come in two implementations here: "fast" (default) runs them on the
# kernels of the fused step wherever its shape limits allow (jf_stage_a_topk / jf_stage_b_softmax_v), "simple" is one
# plain kernel per reference kernel (every width, group layout and top_k up to 8192; also the second implementation
# the parity tests compare against).  JETFIRE_SPLIT_IMPL=simple or set_split_impl("simple") forces the latter.

_split_impl = os.environ.get("JETFIRE_SPLIT_IMPL", "fast").strip().lower() or "fast"


def set_split_impl(name: str) -> str:
    """Select the implementation of the Stage A / Stage B operators ("fast" or "simple"); returns the previous one."""
    global _split_impl
    _check(name in ("fast", "simple"), "split implementation must be 'fast' or 'simple'")
    prev, _split_impl = _split_impl, name
    return prev


def get_split_impl() -> str:
    return _split_impl


def _fast_shape(H_q, H_kv, block_size, max_S, num_slots, top_k=None) -> bool:
    return (_split_impl == "fast" and H_kv > 0 and H_q % H_kv == 0 and 1 <= H_q // H_kv <= 16
            and int(block_size) == 16 and 0 < int(max_S) <= 262144 and 0 < int(num_slots) <= FUSED_MAX_SLOTS
            and (top_k is None or int(top_k) in FUSED_TOP_K))


def _stage_a_fast(fmt: int, q, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, top_k, stats: bool, k_zp=None):
    """jf_stage_a_topk: -> (scores, idx, slots, m, iz); top_k None: scores alone."""
    lib = _lib.load()
    B, dev = q.size(0), q.device
    scores = torch.empty((B, H_q, max_S), dtype=torch.float32, device=dev)
    idx = slots = m = iz = ws = None
    if top_k is not None:
        idx = torch.empty((B, H_q, top_k), dtype=torch.int64, device=dev)
        slots = torch.empty((B, H_q, top_k), dtype=torch.int64, device=dev)
        if stats:
            m = torch.empty((B, H_q), dtype=torch.float32, device=dev)
            iz = torch.empty((B, H_q), dtype=torch.float32, device=dev)
        ws = _workspace(dev, lib.jf_fused_workspace_bytes(fmt, B, H_q, H_kv, int(max_S), int(top_k)), "fused")
    tail = (bt.data_ptr(), sl.data_ptr(), B, H_q, H_kv, int(max_S), bt.size(1), kd.size(1), 16, float(attn_scale),
            0 if top_k is None else int(top_k), scores.data_ptr(), _ptr(idx), _ptr(slots), _ptr(m), _ptr(iz), _ptr(ws),
            0 if ws is None else ws.numel(), _stream(q))
    if k_zp is None:
        _lib.check(lib.jf_stage_a_topk(fmt, HEAD_DIM // ks.size(2), q.data_ptr(), kd.data_ptr(), ks.data_ptr(), *tail))
    else:       # asymmetric INT2 keys (fmt 12)
        _lib.check(lib.jf_stage_a_topk_asym(HEAD_DIM // ks.size(2), q.data_ptr(), kd.data_ptr(), ks.data_ptr(),
                                            k_zp.data_ptr(), *tail))
    return scores, idx, slots, m, iz


def _check_top_k(top_k, name: str, minimum: int = 32) -> None:
    _check(int(top_k) in SUPPORTED_TOP_K and int(top_k) >= minimum,
           f"{name}: unsupported radix-select top_k={top_k} (supported: "
           f"{','.join(str(k) for k in SUPPORTED_TOP_K if k >= minimum)})")


def _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, packed):
    _gpu(q, k_data, k_scales, block_table, seq_lens)
    _check(q.dtype == torch.bfloat16, "q must be bf16")
    _check(k_data.dtype == torch.uint8, "k_data must be uint8")
    _check(k_scales.dtype == torch.bfloat16, "k_scales must be bf16")
    _check(block_table.dtype == torch.int64, "block_table must be int64")
    _check(seq_lens.dtype == torch.int32, "seq_lens must be int32")
    _check(q.dim() == 3 and q.size(2) == HEAD_DIM, "q must be (B, H_q, 128)")
    _check(q.size(1) == H_q, "q.size(1) must equal H_q")
    _check(H_q % H_kv == 0, "H_q must be divisible by H_kv")
    _check(k_data.dim() == 3 and k_data.size(-1) == packed, f"k_data last dim must be {packed}")
    _check(k_data.size(0) == H_kv, "k_data.size(0) must equal H_kv")
    _check(block_table.dim() == 2 and block_table.size(0) == q.size(0), "block_table must be (B, max_blocks)")
    _check(seq_lens.numel() == q.size(0), "seq_lens must be (B,)")
    ks = k_scales.unsqueeze(-1) if k_scales.dim() == 2 else k_scales
    return q.contiguous(), k_data.contiguous(), ks.contiguous(), block_table.contiguous(), seq_lens.contiguous()


def int3_qk_scores(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale):
    """int3_qk_scores.cu:318-390 -> scores (B, H_q, max_S) fp32."""
    lib = _lib.load()
    q, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, 48)
    ng = ks.size(2)
    _check(ng in (1, 2), f"int3_qk_scores currently supports K quant groups 1 or 2, got {ng}")
    B = q.size(0)
    if _fast_shape(H_q, H_kv, block_size, max_S, kd.size(1)):
        return _stage_a_fast(32, q, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, None, False)[0]
    scores = torch.empty((B, H_q, max_S), dtype=torch.float32, device=q.device)
    _lib.check(lib.jf_int3_qk_scores(q.data_ptr(), kd.data_ptr(), ks.data_ptr(), bt.data_ptr(), sl.data_ptr(),
                                     B, H_q, H_kv, int(max_S), bt.size(1), kd.size(1), ng, int(block_size),
                                     float(attn_scale), scores.data_ptr(), _stream(q)))
    return scores


def _intn_qk_scores(nbits: int, name: str, q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size,
                    attn_scale, k_zp=None):
    lib = _lib.load()
    q, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, HEAD_DIM * nbits // 8)
    ng = ks.size(2)
    _check(ng in (1, 2), f"{name} currently supports K quant groups 1 or 2, got {ng}")
    if k_zp is not None:
        k_zp = (k_zp.unsqueeze(-1) if k_zp.dim() == 2 else k_zp).contiguous()
        _check(k_zp.is_cuda and k_zp.dtype == torch.bfloat16 and k_zp.shape == ks.shape,
               "k_zp must be bf16 with the shape of k_scales")
    if _fast_shape(H_q, H_kv, block_size, max_S, kd.size(1)):       # (INT4 keys: the bf16 model, tag 52)
        fmt = 52 if nbits == 4 else (22 if k_zp is None else 12)
        return _stage_a_fast(fmt, q, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, None, False, k_zp=k_zp)[0]
    B = q.size(0)
    scores = torch.empty((B, H_q, max_S), dtype=torch.float32, device=q.device)
    _lib.check(lib.jf_intn_qk_scores(nbits, q.data_ptr(), kd.data_ptr(), ks.data_ptr(), _ptr(k_zp), bt.data_ptr(), sl.data_ptr(),
                                     B, H_q, H_kv, int(max_S), bt.size(1), kd.size(1), ng, int(block_size),
                                     float(attn_scale), scores.data_ptr(), _stream(q)))
    return scores


def int2_qk_scores(q, k_data, k_scales, k_zp, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale):
    """int2_qk_scores.cu:279-420 -> scores (B, H_q, max_S) fp32.  `k_zp` empty or None: symmetric keys; else the
    zero-points of the asymmetric INT2 keys, shaped like `k_scales`."""
    if k_zp is not None and k_zp.numel() == 0:
        k_zp = None
    return _intn_qk_scores(2, "int2_qk_scores", q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size,
                           attn_scale, k_zp)


def int2_qk_scores_topk(q, k_data, k_scales, k_zp, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale,
                        top_k) -> List[torch.Tensor]:
    """int2_qk_scores.cu:583-660 -> [scores, topk_idx, topk_slots]."""
    if k_zp is not None and k_zp.numel() == 0:
        k_zp = None
    if _fast_shape(H_q, H_kv, block_size, max_S, k_data.size(1) if k_data.dim() == 3 else 0, top_k):
        q_, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, 32)
        _check(ks.size(2) in (1, 2), f"int2_qk_scores currently supports K quant groups 1 or 2, got {ks.size(2)}")
        if k_zp is not None:
            k_zp = (k_zp.unsqueeze(-1) if k_zp.dim() == 2 else k_zp).contiguous()
            _check(k_zp.is_cuda and k_zp.dtype == torch.bfloat16 and k_zp.shape == ks.shape,
                   "k_zp must be bf16 with the shape of k_scales")
        return list(_stage_a_fast(22 if k_zp is None else 12, q_, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, int(top_k),
                                  False, k_zp=k_zp)[:3])
    scores = int2_qk_scores(q, k_data, k_scales, k_zp, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale)
    idx, slots, _, _ = _topk(scores, block_table, seq_lens, max_S, H_q, block_size, top_k, False, "int2_qk_scores_topk")
    return [scores, idx, slots]


def int4_qk_scores(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale):
    """int4_qk_scores.cu:280-420 (bf16 q times bf16-rounded INT4 keys) -> scores (B, H_q, max_S) fp32."""
    return _intn_qk_scores(4, "int4_qk_scores", q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size,
                           attn_scale)


def int4_qk_scores_topk(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale,
                        top_k) -> List[torch.Tensor]:
    """int4_qk_scores.cu:714-786 -> [scores, topk_idx, topk_slots]."""
    if _fast_shape(H_q, H_kv, block_size, max_S, k_data.size(1) if k_data.dim() == 3 else 0, top_k):
        q_, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, 64)
        _check(ks.size(2) in (1, 2), f"int4_qk_scores currently supports K quant groups 1 or 2, got {ks.size(2)}")
        return list(_stage_a_fast(52, q_, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, int(top_k), False)[:3])
    scores = int4_qk_scores(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale)
    idx, slots, _, _ = _topk(scores, block_table, seq_lens, max_S, H_q, block_size, top_k, False, "int4_qk_scores_topk")
    return [scores, idx, slots]


def int4_qk_scores_topk_stats(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale,
                              top_k) -> List[torch.Tensor]:
    """int4_qk_scores.cu:788-848 -> [scores, topk_idx, topk_slots, softmax_m, softmax_inv_z]."""
    if _fast_shape(H_q, H_kv, block_size, max_S, k_data.size(1) if k_data.dim() == 3 else 0, top_k):
        q_, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, 64)
        _check(ks.size(2) in (1, 2), f"int4_qk_scores currently supports K quant groups 1 or 2, got {ks.size(2)}")
        return list(_stage_a_fast(52, q_, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, int(top_k), True))
    scores = int4_qk_scores(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale)
    idx, slots, m, iz = _topk(scores, block_table, seq_lens, max_S, H_q, block_size, top_k, True,
                              "int4_qk_scores_topk_stats")
    return [scores, idx, slots, m, iz]


def int8tc_qk_scores(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale):
    """int8tc_qk_scores.cu:1263-1331 -> scores (B, H_q, max_S) fp32."""
    lib = _lib.load()
    if k_scales.dim() == 3:
        _check(k_scales.size(2) == 1, "int8tc_qk_scores needs one K scale per token (group 128)")
    q, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, 64)
    B = q.size(0)
    if _fast_shape(H_q, H_kv, block_size, max_S, kd.size(1)):
        return _stage_a_fast(44, q, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, None, False)[0]
    scores = torch.empty((B, H_q, max_S), dtype=torch.float32, device=q.device)
    _lib.check(lib.jf_int8tc_qk_scores(q.data_ptr(), kd.data_ptr(), ks.data_ptr(), bt.data_ptr(), sl.data_ptr(),
                                       B, H_q, H_kv, int(max_S), bt.size(1), kd.size(1), int(block_size),
                                       float(attn_scale), scores.data_ptr(), _stream(q)))
    return scores


def _topk(scores, block_table, seq_lens, max_S, H_q, block_size, top_k, stats: bool, name: str, minimum: int = 32):
    lib = _lib.load()
    _check_top_k(top_k, name, minimum)
    _check(max_S <= 262144, f"{name}: max_S={max_S} exceeds supported limit (262144).")
    B = scores.size(0)
    bt, sl = block_table.contiguous(), seq_lens.contiguous()
    idx = torch.empty((B, H_q, top_k), dtype=torch.int64, device=scores.device)
    slots = torch.empty((B, H_q, top_k), dtype=torch.int64, device=scores.device)
    m = iz = None
    if stats:
        m = torch.empty((B, H_q), dtype=torch.float32, device=scores.device)
        iz = torch.empty((B, H_q), dtype=torch.float32, device=scores.device)
    if _split_impl == "fast" and int(top_k) <= FUSED_TOP_K[-1] and int(block_size) == 16 and max_S > 0 and B > 0:
        sc = scores.contiguous()
        ws = _workspace(scores.device, lib.jf_topk_slots_fast_workspace_bytes(B, H_q, int(max_S), int(top_k)), "fused")
        _lib.check(lib.jf_topk_slots_fast(sc.data_ptr(), sl.data_ptr(), bt.data_ptr(), B, H_q, int(max_S), bt.size(1), 16,
                                          int(top_k), idx.data_ptr(), slots.data_ptr(), _ptr(m), _ptr(iz), ws.data_ptr(),
                                          ws.numel(), _stream(scores)))
        return idx, slots, m, iz
    _lib.check(lib.jf_topk_slots(scores.data_ptr(), sl.data_ptr(), bt.data_ptr(), B, H_q, int(max_S), bt.size(1),
                                 int(block_size), int(top_k), idx.data_ptr(), slots.data_ptr(), _ptr(m), _ptr(iz),
                                 _stream(scores)))
    return idx, slots, m, iz


def int3_qk_scores_topk(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale,
                        top_k) -> List[torch.Tensor]:
    """int3_qk_scores.cu:562-633 -> [scores, topk_idx, topk_slots]."""
    if _fast_shape(H_q, H_kv, block_size, max_S, k_data.size(1) if k_data.dim() == 3 else 0, top_k):
        q_, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, 48)
        _check(ks.size(2) in (1, 2), f"int3_qk_scores currently supports K quant groups 1 or 2, got {ks.size(2)}")
        return list(_stage_a_fast(32, q_, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, int(top_k), False)[:3])
    scores = int3_qk_scores(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale)
    idx, slots, _, _ = _topk(scores, block_table, seq_lens, max_S, H_q, block_size, top_k, False, "int3_qk_scores_topk")
    return [scores, idx, slots]


def int8tc_qk_scores_topk(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale,
                          top_k) -> List[torch.Tensor]:
    """int8tc_qk_scores.cu:2345-2424 -> [scores, topk_idx, topk_slots]."""
    if _fast_shape(H_q, H_kv, block_size, max_S, k_data.size(1) if k_data.dim() == 3 else 0, top_k):
        _check(k_scales.dim() == 2 or k_scales.size(2) == 1, "int8tc_qk_scores needs one K scale per token (group 128)")
        q_, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, 64)
        return list(_stage_a_fast(44, q_, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, int(top_k), False)[:3])
    scores = int8tc_qk_scores(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale)
    idx, slots, _, _ = _topk(scores, block_table, seq_lens, max_S, H_q, block_size, top_k, False, "int8tc_qk_scores_topk")
    return [scores, idx, slots]


def int8tc_qk_scores_topk_stats(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale,
                                top_k) -> List[torch.Tensor]:
    """int8tc_qk_scores.cu:2426-2482 -> [scores, topk_idx, topk_slots, softmax_m, softmax_inv_z]."""
    _check_top_k(top_k, "int8tc_qk_scores_topk_stats", 64)
    if _fast_shape(H_q, H_kv, block_size, max_S, k_data.size(1) if k_data.dim() == 3 else 0, top_k):
        _check(k_scales.dim() == 2 or k_scales.size(2) == 1, "int8tc_qk_scores needs one K scale per token (group 128)")
        q_, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, 64)
        return list(_stage_a_fast(44, q_, kd, ks, bt, sl, max_S, H_q, H_kv, attn_scale, int(top_k), True))
    scores = int8tc_qk_scores(q, k_data, k_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size, attn_scale)
    idx, slots, m, iz = _topk(scores, block_table, seq_lens, max_S, H_q, block_size, top_k, True,
                              "int8tc_qk_scores_topk_stats", minimum=64)
    return [scores, idx, slots, m, iz]


# --------------------------------------------------------------------------- Stage B


def _softmax_v(scores, m, iz, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv, block_size, top_k,
               nbits: int, outs=None, int8_tiles: bool = False):
    lib = _lib.load()
    _gpu(scores, v_data, v_scales, block_table, seq_lens)
    _check(scores.dtype == torch.float32 and scores.dim() == 3, "scores must be (B, H_q, max_S) fp32")
    _check(v_data.dtype == torch.uint8 and v_scales.dtype == torch.bfloat16, "v_data uint8 / v_scales bf16")
    _check(block_table.dtype == torch.int64 and seq_lens.dtype == torch.int32, "block_table int64 / seq_lens int32")
    _check(v_data.dim() == 3 and v_data.size(2) == HEAD_DIM * nbits // 8, f"v_data last dim must be {HEAD_DIM * nbits // 8}")
    _check(H_q % H_kv == 0, "H_q must be divisible by H_kv")
    _check(int(block_size) == 16, "wvs2 only supports block_size=16")
    _check(scores.size(2) == max_S and scores.size(1) == H_q, "scores must be (B, H_q, max_S)")
    if topk_idx is not None:
        _check(topk_idx.is_cuda and topk_idx.dtype == torch.int64 and topk_idx.dim() == 3 and topk_idx.size(2) == top_k,
               "topk_idx must be (B, H_q, top_k) int64")
        topk_idx = topk_idx.contiguous()
    vs = v_scales.unsqueeze(-1) if v_scales.dim() == 2 else v_scales
    ng = vs.size(2)
    _check(ng in (1, 2), f"wvs2 requires num_groups=1 or 2 (got {ng})")
    sc, vd, vs = scores.contiguous(), v_data.contiguous(), vs.contiguous()
    bt, sl = block_table.contiguous(), seq_lens.contiguous()
    B = sc.size(0)
    dev = sc.device
    if outs is None:
        o_hat = torch.empty((B, H_q, HEAD_DIM), dtype=torch.float32, device=dev)
        o_old = torch.zeros((B, H_q, HEAD_DIM), dtype=torch.float32, device=dev)
        W = torch.zeros((B, H_q), dtype=torch.float32, device=dev)
    else:
        o_hat, o_old, W = outs
        for t in outs:
            _check(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous(), "output buffers must be contiguous fp32")
    if (not int8_tiles and m is None and nbits in (2, 3, 4) and vd.size(0) == H_kv
            and _fast_shape(H_q, H_kv, block_size, max_S, vd.size(1), top_k if topk_idx is not None else None)):
        fmt = {2: 32, 3: 33, 4: 44 if ng == 1 else 34}[nbits]      # (value side of the tag; 34: INT4 values, two groups)
        k_eff = int(top_k) if topk_idx is not None else 32
        ws = _workspace(dev, lib.jf_fused_workspace_bytes(fmt, B, H_q, H_kv, int(max_S), k_eff), "fused")
        _lib.check(lib.jf_stage_b_softmax_v(
            fmt, HEAD_DIM // ng, sc.data_ptr(), vd.data_ptr(), vs.data_ptr(), bt.data_ptr(), sl.data_ptr(), _ptr(topk_idx),
            B, H_q, H_kv, int(max_S), bt.size(1), vd.size(1), 16, k_eff, o_hat.data_ptr(), o_old.data_ptr(), W.data_ptr(),
            ws.data_ptr(), ws.numel(), _stream(sc)))
        return [o_hat, o_old, W]
    need = lib.jf_softmax_v_workspace_bytes(B, H_q, int(max_S))
    ws = _workspace(dev, need, "softmax_v")
    if m is not None:
        m, iz = m.contiguous(), iz.contiguous()
    if int8_tiles:
        _lib.check(lib.jf_softmax_v_int8_tiles(
            sc.data_ptr(), _ptr(m), _ptr(iz), vd.data_ptr(), vs.data_ptr(), bt.data_ptr(), sl.data_ptr(), _ptr(topk_idx),
            B, H_q, H_kv, int(max_S), bt.size(1), vd.size(1), int(block_size), int(top_k),
            o_hat.data_ptr(), o_old.data_ptr(), W.data_ptr(), ws.data_ptr(), ws.numel(), _stream(sc)))
        return [o_hat, o_old, W]
    _lib.check(lib.jf_softmax_v_pre_corr(
        sc.data_ptr(), _ptr(m), _ptr(iz), vd.data_ptr(), vs.data_ptr(), bt.data_ptr(), sl.data_ptr(), _ptr(topk_idx),
        B, H_q, H_kv, int(max_S), bt.size(1), vd.size(1), int(block_size), int(top_k), nbits, ng,
        o_hat.data_ptr(), o_old.data_ptr(), W.data_ptr(), ws.data_ptr(), ws.numel(), _stream(sc)))
    return [o_hat, o_old, W]


def int2_softmax_v_with_pre_corr_wvs2(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
                                      block_size, top_k) -> List[torch.Tensor]:
    """int2_softmax_v.cu:792-901 -> [o_hat, o_old_unnorm, W]."""
    return _softmax_v(scores, None, None, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
                      block_size, top_k, 2)


def int2_softmax_v_with_pre_corr_wvs2_inplace(scores, v_data, v_scales, block_table, seq_lens, topk_idx, weights,
                                              o_hat, o_old_unnorm, W_out, max_S, H_q, H_kv, block_size, top_k) -> None:
    """int2_softmax_v.cu:903-1010: caller-owned outputs (graph capture). `weights` is accepted and unused:
    this implementation never materialises the softmax weights."""
    _softmax_v(scores, None, None, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv, block_size,
               top_k, 2, outs=(o_hat, o_old_unnorm, W_out))


def int2_softmax_v_with_pre_corr(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
                                 block_size, top_k) -> List[torch.Tensor]:
    return int2_softmax_v_with_pre_corr_wvs2(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q,
                                             H_kv, block_size, top_k)


def int2_softmax_v(scores, v_data, v_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size) -> torch.Tensor:
    return _softmax_v(scores, None, None, v_data, v_scales, block_table, seq_lens, None, max_S, H_q, H_kv, block_size,
                      32, 2)[0]


def int3_softmax_v_with_pre_corr_wvs2(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
                                      block_size, top_k) -> List[torch.Tensor]:
    """int3_softmax_v.cu:752-860 (planar INT3 values) -> [o_hat, o_old_unnorm, W]."""
    return _softmax_v(scores, None, None, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
                      block_size, top_k, 3)


def int3_softmax_v_with_pre_corr_wvs2_inplace(scores, v_data, v_scales, block_table, seq_lens, topk_idx, weights,
                                              o_hat, o_old_unnorm, W_out, max_S, H_q, H_kv, block_size, top_k) -> None:
    """int3_softmax_v.cu:862-985: caller-owned outputs; `weights` is accepted and unused."""
    _softmax_v(scores, None, None, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv, block_size,
               top_k, 3, outs=(o_hat, o_old_unnorm, W_out))


def int3_softmax_v_with_pre_corr(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
                                 block_size, top_k) -> List[torch.Tensor]:
    return int3_softmax_v_with_pre_corr_wvs2(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q,
                                             H_kv, block_size, top_k)


def int3_softmax_v(scores, v_data, v_scales, block_table, seq_lens, max_S, H_q, H_kv, block_size) -> torch.Tensor:
    return _softmax_v(scores, None, None, v_data, v_scales, block_table, seq_lens, None, max_S, H_q, H_kv, block_size,
                      32, 3)[0]


def int4_softmax_v_with_pre_corr_wvs2_scores(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q,
                                             H_kv, block_size, top_k) -> List[torch.Tensor]:
    """int4_softmax_v.cu:2203-2235 -> [o_hat, o_old_unnorm, W]."""
    return _softmax_v(scores, None, None, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
                      block_size, top_k, 4)


def int4_softmax_v_with_pre_corr_wvs2(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv,
                                      block_size, top_k) -> List[torch.Tensor]:
    return int4_softmax_v_with_pre_corr_wvs2_scores(scores, v_data, v_scales, block_table, seq_lens, topk_idx, max_S,
                                                    H_q, H_kv, block_size, top_k)


def int4_softmax_v_with_pre_corr_wvs2_inplace(scores, v_data, v_scales, block_table, seq_lens, topk_idx, weights,
                                              o_hat, o_old_unnorm, W_out, max_S, H_q, H_kv, block_size, top_k) -> None:
    """int4_softmax_v.cu:927-1040 (what graph mode looks up under JETFIRE_GRAPH_STAGEB_INPLACE,
    jetfire_vllm/adapter/decode_path.py:2872-2919): caller-owned outputs; `weights` is accepted and unused."""
    _softmax_v(scores, None, None, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q, H_kv, block_size,
               top_k, 4, outs=(o_hat, o_old_unnorm, W_out))


def int8tc_softmax_v_with_pre_corr_reg_stats(scores, softmax_m, softmax_inv_z, v_data, v_scales, block_table, seq_lens,
                                             topk_idx, max_S, H_q, H_kv, block_size, top_k) -> List[torch.Tensor]:
    """int8tc_softmax_v_fused.cu:1591-1734 -> [o_hat, o_old_unnorm, W], with the reference's arithmetic: P * v_scale
    quantised to int8 per 32-position tile and row (:1203-1236), int32 tile sums scaled back in fp32 (:1298-1311),
    exact fp32 weights for o_old_unnorm and W (:1340-1400).  Uses the Stage-A statistics it is handed."""
    _check(softmax_m is not None and softmax_inv_z is not None, "int8tc_softmax_v requires the Stage-A statistics")
    _check(softmax_m.dtype == torch.float32 and softmax_inv_z.dtype == torch.float32, "softmax stats must be fp32")
    vs = v_scales.unsqueeze(-1) if v_scales.dim() == 2 else v_scales
    _check(vs.size(2) == 1, "int8tc_softmax_v requires one V scale per token (group 128)")
    _check(H_q // H_kv <= 16, "int8tc_softmax_v requires H_q/H_kv <= 16")
    return _softmax_v(scores, softmax_m, softmax_inv_z, v_data, v_scales, block_table, seq_lens, topk_idx, max_S, H_q,
                      H_kv, block_size, top_k, 4, int8_tiles=True)


# --------------------------------------------------------------------------- fused scan


def fused_attn_topk(scheme: str, q, k_data, k_scales, v_data, v_scales, block_table, seq_lens, max_S, H_q, H_kv,
                    block_size, top_k, attn_scale, group_size: Optional[int] = None, return_scores: bool = False,
                    return_stats: bool = False, blend=None, k_zp=None):
    """One fused pass: -> (o_hat, topk_slots, o_old_unnorm, W, topk_idx[, softmax_m, softmax_inv_z][, scores]).

    blend=(o_new, out), both (B, H_q, 128) bf16 on the GPU: the merge kernel also writes
    out = bf16(fma(W, o_new, o_hat) - o_old_unnorm), bit-equal to blend_unnorm_into (for callers that hold o_new
    when the step is enqueued).

    The single-call contract is the one of the reference's int2_fused_attn_topk
    (jetfire_vllm/kernels/int2_fused_attn_topk.py:5-10) extended to INT3 / INT4 keys (INT4: the int8-Q scoring
    model), symmetric INT2 keys, and INT2 / INT3 / INT4 values: "k{2,3,4}v{2,3,4}"; pairs with INT4 keys take
    group 128, the others group 64 or 128.  "a2v{2,3,4}": asymmetric INT2 keys, whose zero-points come in `k_zp`
    (shaped like k_scales), the reference's int2_asym_k_* kernel sets.  "b4v{2,3,4}": INT4 keys scored with the bf16 model
    of int4_qk_scores (group 64 or 128), what the reference runs for INT4 keys with 64-channel groups."""
    lib = _lib.load()
    scheme_id = FUSED_SCHEMES.get(scheme)
    _check(scheme_id is not None, f"unknown scheme {scheme!r} ({', '.join(sorted(FUSED_SCHEMES))})")
    asym = scheme_id // 10 == 1
    kp, vp = {1: 32, 5: 64}.get(scheme_id // 10, 16 * (scheme_id // 10)), 16 * (scheme_id % 10)
    q, kd, ks, bt, sl = _stage_a_args(q, k_data, k_scales, block_table, seq_lens, H_q, H_kv, kp)
    _check(asym == (k_zp is not None), "k_zp goes with the a2v* schemes, and only with them")
    if asym:
        k_zp = (k_zp.unsqueeze(-1) if k_zp.dim() == 2 else k_zp).contiguous()
        _check(k_zp.is_cuda and k_zp.dtype == torch.bfloat16 and k_zp.shape == ks.shape,
               "k_zp must be bf16 with the shape of k_scales")
    _gpu(v_data, v_scales)
    _check(v_data.dtype == torch.uint8 and v_data.dim() == 3 and v_data.size(2) == vp, f"v_data last dim must be {vp}")
    _check(v_scales.dtype == torch.bfloat16, "v_scales must be bf16")
    vs = (v_scales.unsqueeze(-1) if v_scales.dim() == 2 else v_scales).contiguous()
    vd = v_data.contiguous()
    _check(ks.size(2) == vs.size(2), "K and V must use the same group size")
    gs = HEAD_DIM // ks.size(2)
    if group_size is not None:
        _check(int(group_size) == gs, f"group_size={group_size} does not match the scale tensors ({gs})")
    _check(int(top_k) in SUPPORTED_TOP_K, f"unsupported top_k={top_k}")
    _check(kd.size(1) == vd.size(1), "K and V caches must have the same number of slots")
    B = q.size(0)
    dev = q.device
    idx = torch.empty((B, H_q, top_k), dtype=torch.int64, device=dev)
    slots = torch.empty((B, H_q, top_k), dtype=torch.int64, device=dev)
    o_hat = torch.empty((B, H_q, HEAD_DIM), dtype=torch.float32, device=dev)
    o_old = torch.empty((B, H_q, HEAD_DIM), dtype=torch.float32, device=dev)
    W = torch.empty((B, H_q), dtype=torch.float32, device=dev)
    m = torch.empty((B, H_q), dtype=torch.float32, device=dev) if return_stats else None
    iz = torch.empty((B, H_q), dtype=torch.float32, device=dev) if return_stats else None
    scores = torch.empty((B, H_q, max_S), dtype=torch.float32, device=dev) if return_scores else None
    need = lib.jf_fused_workspace_bytes(scheme_id, B, H_q, H_kv, int(max_S), int(top_k))
    ws = _workspace(dev, need, "fused")
    head = (scheme_id, gs, q.data_ptr(), kd.data_ptr(), ks.data_ptr(), *((k_zp.data_ptr(),) if asym else ()),
            vd.data_ptr(), vs.data_ptr(), bt.data_ptr(),
            sl.data_ptr(), B, H_q, H_kv, int(max_S), bt.size(1), kd.size(1), int(block_size), float(attn_scale), int(top_k),
            idx.data_ptr(), slots.data_ptr(), o_hat.data_ptr(), o_old.data_ptr(), W.data_ptr(), _ptr(m), _ptr(iz),
            _ptr(scores))
    if blend is None and not asym:
        _lib.check(lib.jf_fused_scan_topk(*head, ws.data_ptr(), ws.numel(), _stream(q)))
    elif blend is None:
        _lib.check(lib.jf_fused_scan_topk_asym(*head, None, None, ws.data_ptr(), ws.numel(), _stream(q)))
    else:
        o_new, out = blend
        _gpu(o_new, out)
        _check(o_new.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "o_new / out must be bf16")
        _check(tuple(o_new.shape) == (B, H_q, HEAD_DIM) and tuple(out.shape) == (B, H_q, HEAD_DIM),
               "o_new / out must be (B, H_q, 128)")
        _check(o_new.is_contiguous() and out.is_contiguous(), "o_new / out must be contiguous")
        entry = lib.jf_fused_scan_topk_asym if asym else lib.jf_fused_scan_topk_blend
        _lib.check(entry(*head, o_new.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(), _stream(q)))
    out = [o_hat, slots, o_old, W, idx]
    if return_stats:
        out += [m, iz]
    if return_scores:
        out.append(scores)
    return tuple(out)


# --------------------------------------------------------------------------- merge


def blend_unnorm_into(o_hat, o_old_unnorm, W, o_new, out) -> None:
    """blend.cu:229-290"""
    lib = _lib.load()
    _check(o_hat.is_cuda and o_old_unnorm.is_cuda and W.is_cuda and o_new.is_cuda and out.is_cuda,
           "blend_unnorm_into: all tensors must be on the GPU")
    _check(o_hat.dtype == torch.float32 and o_old_unnorm.dtype == torch.float32 and W.dtype == torch.float32,
           "o_hat / o_old_unnorm / W must be fp32")
    _check(o_new.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "o_new / out must be bf16")
    _check(o_hat.dim() == 3 and o_old_unnorm.dim() == 3 and o_new.dim() == 3 and out.dim() == 3, "tensors must be 3D")
    _check(W.dim() == 2, "W must be 2D")
    _check(out.is_contiguous(), "out must be contiguous")
    hc, oc, wc, nc = o_hat.contiguous(), o_old_unnorm.contiguous(), W.contiguous(), o_new.contiguous()
    _check(oc.shape == hc.shape and nc.shape == hc.shape and out.shape == hc.shape, "shape mismatch")
    _check(wc.shape == hc.shape[:2], "W must be (B, H_q)")
    B, H_q, D = hc.shape
    _lib.check(lib.jf_blend_unnorm(hc.data_ptr(), oc.data_ptr(), wc.data_ptr(), nc.data_ptr(), out.data_ptr(), B, H_q, D,
                                   _stream(out)))


def blend_unnorm(o_hat, o_old_unnorm, W, o_new) -> torch.Tensor:
    out = torch.empty_like(o_new)
    blend_unnorm_into(o_hat, o_old_unnorm, W, o_new, out)
    return out


def _blend_args(name, o_hat, o_old, W, o_new, out):
    _check(o_hat.is_cuda and o_old.is_cuda and W.is_cuda and o_new.is_cuda and (out is None or out.is_cuda),
           f"{name}: all tensors must be on the GPU")
    _check(o_hat.dtype == torch.float32 and o_old.dtype == torch.float32 and W.dtype == torch.float32,
           "o_hat / o_old / W must be fp32")
    _check(o_new.dtype == torch.bfloat16 and (out is None or out.dtype == torch.bfloat16), "o_new / out must be bf16")
    _check(o_hat.dim() == 3 and o_old.dim() == 3 and o_new.dim() == 3, "o_hat/o_old/o_new must be 3D (B, H_q, D)")
    _check(W.dim() == 2, "W must be 2D (B, H_q)")
    hc, oc, wc, nc = o_hat.contiguous(), o_old.contiguous(), W.contiguous(), o_new.contiguous()
    _check(oc.shape == hc.shape, "o_old shape mismatch")
    _check(nc.shape == hc.shape, "o_new shape mismatch")
    _check(wc.shape == hc.shape[:2], "W shape mismatch")
    if out is not None:
        _check(out.is_contiguous(), "out must be contiguous")
        _check(out.shape == hc.shape, "out shape mismatch")
    return hc, oc, wc, nc


def blend_into(o_hat, o_old, W, o_new, out) -> None:
    """blend.cu:130-190: out = bf16(o_hat + W * (o_new - o_old)) with a normalised o_old, into `out`."""
    hc, oc, wc, nc = _blend_args("blend_into", o_hat, o_old, W, o_new, out)
    B, H_q, D = hc.shape
    _lib.check(_lib.load().jf_blend(hc.data_ptr(), oc.data_ptr(), wc.data_ptr(), nc.data_ptr(), out.data_ptr(), B, H_q, D,
                                    _stream(out)))


def blend(o_hat, o_old, W, o_new) -> torch.Tensor:
    """blend.cu:68-128: as blend_into, returning a new (B, H_q, D) bf16 tensor."""
    hc, oc, wc, nc = _blend_args("blend", o_hat, o_old, W, o_new, None)
    out = torch.empty(hc.shape, dtype=torch.bfloat16, device=hc.device)
    B, H_q, D = hc.shape
    _lib.check(_lib.load().jf_blend(hc.data_ptr(), oc.data_ptr(), wc.data_ptr(), nc.data_ptr(), out.data_ptr(), B, H_q, D,
                                    _stream(out)))
    return out


def _flag_ptr(flag, name: str) -> int:
    _check(isinstance(flag, torch.Tensor) and not flag.is_cuda and flag.numel() == 1 and flag.dtype == torch.int64,
           f"{name} must be a 1-element int64 CPU tensor")
    return flag.data_ptr()


def wait_and_blend_unnorm_into(done_flag, o_hat, o_old_unnorm, W, o_new, out) -> None:
    """blend.cu:292-377: the calling thread waits until the CPU correction has stored 1 to `done_flag`, then
    launches blend_unnorm_into on the current stream (o_new is the device view of the mapped pinned buffer the
    correction wrote)."""
    ptr = _flag_ptr(done_flag, "done_flag")
    _check(o_hat.is_cuda and o_old_unnorm.is_cuda and W.is_cuda and o_new.is_cuda and out.is_cuda,
           "wait_and_blend_unnorm_into: all device tensors must be on the GPU")
    _lib.check(_lib.load().jf_wait_for_flag(ptr, 0.0))
    blend_unnorm_into(o_hat, o_old_unnorm, W, o_new, out)


# --------------------------------------------------------------------------- CPU correction


def cpu_topk_attn(q, k_shadow, v_shadow, head_map, ts_buf, o_new, scale, done_flag=None) -> None:
    """cpu_topk_attn.cpp:854-956: all CPU tensors; synchronous on the calling thread."""
    lib = _lib.load()
    for t in (q, k_shadow, v_shadow, head_map, ts_buf, o_new):
        _check(not t.is_cuda, "cpu_topk_attn: all tensors must be CPU")
    _check(q.dtype == torch.bfloat16 and k_shadow.dtype == torch.bfloat16 and v_shadow.dtype == torch.bfloat16
           and o_new.dtype == torch.bfloat16, "q / shadows / o_new must be bf16")
    _check(head_map.dtype == torch.int64 and ts_buf.dtype == torch.int64, "head_map / ts_buf must be int64")
    _check(q.dim() == 3 and q.size(2) == HEAD_DIM and k_shadow.dim() == 3 and k_shadow.size(2) == HEAD_DIM,
           "q must be (B, H_q, 128) and shadows (H_kv, num_slots, 128)")
    _check(v_shadow.shape == k_shadow.shape, "k_shadow / v_shadow shape mismatch")
    _check(head_map.shape == ts_buf.shape and ts_buf.dim() == 3 and ts_buf.shape[:2] == q.shape[:2],
           "head_map / ts_buf must be (B, H_q, K)")
    _check(o_new.shape == q.shape and o_new.is_contiguous(), "o_new must be contiguous (B, H_q, 128)")
    for t in (q, k_shadow, v_shadow, head_map, ts_buf):
        _check(t.is_contiguous(), "cpu_topk_attn: inputs must be contiguous")
    if done_flag is not None:
        _check(done_flag.dtype == torch.int64 and done_flag.numel() == 1 and not done_flag.is_cuda,
               "done_flag must be a 1-element int64 CPU tensor")
    B, H_q, _ = q.shape
    _lib.check(lib.jf_cpu_topk_attn(q.data_ptr(), k_shadow.data_ptr(), v_shadow.data_ptr(), head_map.data_ptr(),
                                    ts_buf.data_ptr(), o_new.data_ptr(), B, H_q, ts_buf.size(2), k_shadow.size(0),
                                    k_shadow.size(1), float(scale), _ptr(done_flag)))


def set_cpu_attn_threads(n: int) -> None:
    _lib.check(_lib.load().jf_set_cpu_attn_threads(int(n)))


def get_cpu_attn_threads() -> int:
    return int(_lib.load().jf_get_cpu_attn_threads())


class _DeviceView:
    """Zero-copy device tensor over pinned host memory (the GPU addresses it across PCIe)."""

    def __init__(self, ptr: int, shape, dtype: torch.dtype, owner):
        typestr = {torch.bfloat16: "<u2", torch.float16: "<f2", torch.float32: "<f4", torch.int64: "<i8",
                   torch.int32: "<i4", torch.uint8: "|u1", torch.int16: "<i2"}[dtype]
        self.__cuda_array_interface__ = {"shape": tuple(int(x) for x in shape), "typestr": typestr, "data": (int(ptr), False),
                                         "version": 2, "strides": None}
        self._owner = owner


def alloc_mapped_pinned_pair(shape, dtype):
    """cpu_topk_attn.cpp:972-1023 -> (host_tensor, device_tensor) over the same pinned host memory: what the CPU
    stores through the host tensor the GPU reads through the device tensor, with no copy."""
    shape = tuple(int(x) for x in shape)
    _check(len(shape) > 0 and all(x > 0 for x in shape), "alloc_mapped_pinned_pair: empty shape")
    host = torch.zeros(shape, dtype=dtype, pin_memory=True)
    dev_ptr = host_buffer_device_pointer(host)
    if dtype == torch.bfloat16:      # the array interface has no bf16: view 16-bit words, then reinterpret
        dev = torch.as_tensor(_DeviceView(dev_ptr, shape, torch.int16, host), device="cuda").view(torch.bfloat16)
    else:
        dev = torch.as_tensor(_DeviceView(dev_ptr, shape, dtype, host), device="cuda")
    _check(dev.data_ptr() == dev_ptr, "alloc_mapped_pinned_pair: the device view does not alias the host buffer")
    dev._jf_host = host              # the view borrows: keep the owner alive with it
    return host, dev


def _cpu_job_args(name, q, k_shadow, v_shadow, head_map, ts_buf, o_new):
    for t in (q, k_shadow, v_shadow, head_map, ts_buf, o_new):
        _check(not t.is_cuda, f"{name}: all tensors must be CPU")
    _check(q.dtype == torch.bfloat16 and k_shadow.dtype == torch.bfloat16 and v_shadow.dtype == torch.bfloat16
           and o_new.dtype == torch.bfloat16, "q / shadows / o_new must be bf16")
    _check(head_map.dtype == torch.int64 and ts_buf.dtype == torch.int64, "head_map / ts_buf must be int64")
    _check(q.dim() == 3 and q.size(2) == HEAD_DIM and k_shadow.dim() == 3 and k_shadow.size(2) == HEAD_DIM,
           "q must be (B, H_q, 128) and shadows (H_kv, num_slots, 128)")
    _check(v_shadow.shape == k_shadow.shape, "k_shadow / v_shadow shape mismatch")
    _check(head_map.shape == ts_buf.shape and ts_buf.dim() == 3 and ts_buf.shape[:2] == q.shape[:2],
           "head_map / ts_buf must be (B, H_q, K)")
    _check(o_new.shape == q.shape, "o_new must be (B, H_q, 128)")
    for t in (q, k_shadow, v_shadow, head_map, ts_buf, o_new):
        _check(t.is_contiguous(), f"{name}: tensors must be contiguous")


_ASYNC_KEEP: list = []      # tensors of asynchronous jobs in flight (released by wait_for_flag)
_CTX_KEEP: dict = {}        # context handle -> the tensors it points at


def submit_cpu_topk_attn_async(q, k_shadow, v_shadow, head_map, ts_buf, o_new, scale, flag) -> None:
    """cpu_topk_attn.cpp:1184-1205: cpu_topk_attn on the library's executor thread; returns at once, 1 is stored to
    `flag` (1-element int64 CPU tensor) when o_new is complete."""
    _cpu_job_args("submit_cpu_topk_attn_async", q, k_shadow, v_shadow, head_map, ts_buf, o_new)
    fp = _flag_ptr(flag, "flag")
    B, H_q, _ = q.shape
    _ASYNC_KEEP.append((flag, q, k_shadow, v_shadow, head_map, ts_buf, o_new))
    _lib.check(_lib.load().jf_cpu_topk_attn_async(q.data_ptr(), k_shadow.data_ptr(), v_shadow.data_ptr(), head_map.data_ptr(),
                                                  ts_buf.data_ptr(), o_new.data_ptr(), B, H_q, ts_buf.size(2),
                                                  k_shadow.size(0), k_shadow.size(1), float(scale), fp))


def wait_for_flag(flag) -> None:
    """cpu_topk_attn.cpp:1217-1260: block until `flag` reads non-zero."""
    fp = _flag_ptr(flag, "flag")
    _lib.check(_lib.load().jf_wait_for_flag(fp, 0.0))
    _ASYNC_KEEP[:] = [k for k in _ASYNC_KEEP if k[0].data_ptr() != fp]


def persistent_worker_warmup() -> None:
    _lib.check(_lib.load().jf_graph_pool_warmup(0))


def create_cpu_topk_submit_ctx(q, k_shadow, v_shadow, head_map, ts_buf, o_new, scale, flag_host) -> int:
    """cpu_topk_attn.cpp:2054-2163 -> opaque int handle for stream_submit_cpu_topk_attn / stream_wait_cpu_topk_attn.
    All tensors are CPU (pinned q / ts_buf / o_new that the caller fills and reads with its own stream-ordered
    copies); `flag_host` is the host half of an alloc_mapped_pinned_pair and receives 1 when a correction is done."""
    _cpu_job_args("create_cpu_topk_submit_ctx", q, k_shadow, v_shadow, head_map, ts_buf, o_new)
    fp = _flag_ptr(flag_host, "flag_host")
    B, H_q, _ = q.shape
    lib = _lib.load()
    h = int(lib.jf_submit_ctx_create(q.data_ptr(), k_shadow.data_ptr(), v_shadow.data_ptr(), head_map.data_ptr(),
                                     ts_buf.data_ptr(), o_new.data_ptr(), B, H_q, ts_buf.size(2), k_shadow.size(0),
                                     k_shadow.size(1), float(scale), fp))
    if h <= 0:
        raise RuntimeError(lib.jf_last_error().decode())
    _CTX_KEEP[h] = (q, k_shadow, v_shadow, head_map, ts_buf, o_new, flag_host)
    return h


def stream_submit_cpu_topk_attn(stream_id: int, ctx_handle: int) -> None:
    """cpu_topk_attn.cpp:2239: start the context's CPU correction in stream order (graph-capturable: a kernel)."""
    _lib.check(_lib.load().jf_submit_ctx_stream_submit(int(ctx_handle), int(stream_id)))


def stream_wait_cpu_topk_attn(stream_id: int, ctx_handle: int) -> None:
    """cpu_topk_attn.cpp:2302: make the stream wait for the context's correction (graph-capturable: a kernel with a
    bounded device-side wait; check_cpu_topk_submit_ctx reports a wait that ran into its limit)."""
    _lib.check(_lib.load().jf_submit_ctx_stream_wait(int(ctx_handle), int(stream_id)))


def check_cpu_topk_submit_ctx(ctx_handle: int) -> None:
    _lib.check(_lib.load().jf_submit_ctx_status(int(ctx_handle)))


def _flag_dev_ptr(flag_device) -> int:
    _check(isinstance(flag_device, torch.Tensor) and flag_device.is_cuda and flag_device.dtype == torch.int64
           and flag_device.numel() >= 1, "flag_device must be the int64 device tensor of an alloc_mapped_pinned_pair")
    return flag_device.data_ptr()


def stream_write_value64(stream_id: int, flag_device, value: int) -> None:
    """cpu_topk_attn.cpp:1293-1318"""
    _lib.check(_lib.load().jf_stream_write_value64(int(stream_id), _flag_dev_ptr(flag_device), int(value)))


def stream_wait_value64(stream_id: int, flag_device, value: int) -> None:
    """cpu_topk_attn.cpp:1320-1344 (EQ)"""
    _lib.check(_lib.load().jf_stream_wait_value64(int(stream_id), _flag_dev_ptr(flag_device), int(value)))


def graph_pool_warmup() -> None:
    _lib.check(_lib.load().jf_graph_pool_warmup(0))


def graph_pool_warmup_threads(n_threads: int) -> None:
    _check(int(n_threads) > 0, "graph_pool_warmup_threads: n_threads must be positive")
    _lib.check(_lib.load().jf_graph_pool_warmup(int(n_threads)))


def get_graph_submit_count() -> int:
    return int(_lib.load().jf_graph_submit_count())


def get_cpu_topk_sanitize_count() -> int:
    return int(_lib.load().jf_cpu_topk_sanitize_count())


def get_shadow_append_count() -> int:
    """Mirror-kernel launches that have run on the current device, graph replays included
    (jetfire_vllm/csrc/cpu_topk_attn.cpp:2353-2355)."""
    n = ctypes.c_int64(0)
    _lib.check(_lib.load().jf_shadow_append_count(ctypes.byref(n), 0))
    return int(n.value)


def reset_graph_submit_count() -> None:
    """Zero the submit / shadow-append / sanitise counters and the timing statistics
    (jetfire_vllm/csrc/cpu_topk_attn.cpp:2436-2470)."""
    _lib.check(_lib.load().jf_reset_graph_submit_count())


_TIMING_FIELDS = ("topk_jobs", "topk_done_avg_us", "topk_done_max_us", "shadow_append_jobs", "join_jobs",
                  "join_wait_avg_us", "join_wait_max_us", "pool_workers", "pool_done_count")


def get_graph_timing_stats() -> dict:
    """The counters this library keeps under the reference's key names
    (jetfire_vllm/csrc/cpu_topk_attn.cpp:2361-2434): counts are ints, times floats in microseconds."""
    buf = (ctypes.c_double * len(_TIMING_FIELDS))()
    _lib.check(_lib.load().jf_graph_timing_stats(buf, len(_TIMING_FIELDS)))
    out = {k: (float(v) if k.endswith("_us") else int(v)) for k, v in zip(_TIMING_FIELDS, buf)}
    out["pool_initialized"] = out["pool_workers"] > 0
    return out


def pool_wake() -> None:
    """Sleeping workers of the correction pool go back to spinning for the next job (call at the start of a decode
    step issued from the host)."""
    _lib.check(_lib.load().jf_pool_wake())


def pool_doorbell(stream_id: Optional[int] = None) -> None:
    """The same from the GPU's side: a one-lane kernel on the stream (capturable; put it at the head of a decode
    step's graph) that has the poller thread wake the pool when the GPU reaches it."""
    st = torch.cuda.current_stream().cuda_stream if stream_id is None else int(stream_id)
    _lib.check(_lib.load().jf_pool_doorbell(st))


def reset_graph_runtime_state() -> None:
    _lib.check(_lib.load().jf_reset_graph_runtime_state())


def clear_graph_contexts() -> None:
    _lib.check(_lib.load().jf_clear_graph_contexts())
    _CTX_KEEP.clear()


def set_cpu_attn_isa(name) -> None:
    """Row implementation of the CPU correction: None / "widest", "scalar", "avx2", "avx512bf16"."""
    code = {None: -1, "widest": -1, "scalar": 0, "avx2": 1, "avx512bf16": 2}[name]
    _lib.check(_lib.load().jf_set_cpu_attn_isa(code))


def get_cpu_attn_isa() -> str:
    return ("scalar", "avx2", "avx512bf16")[int(_lib.load().jf_get_cpu_attn_isa())]


class CpuTopkHandoff:
    """Pinned hand-off context (create_cpu_topk_submit_ctx / stream_submit_cpu_topk_attn /
    stream_wait_cpu_topk_attn in cpu_topk_attn.cpp:2054-2163,2239,2302).  The shadows must stay alive
    and unmoved for the life of the context."""

    def __init__(self, B, H_q, H_kv, K, k_shadow, v_shadow, scale):
        lib = _lib.load()
        _check(not k_shadow.is_cuda and not v_shadow.is_cuda and k_shadow.is_contiguous() and v_shadow.is_contiguous(),
               "shadows must be contiguous CPU tensors")
        _check(k_shadow.dtype == torch.bfloat16 and v_shadow.dtype == torch.bfloat16, "shadows must be bf16")
        _check(k_shadow.shape == v_shadow.shape and k_shadow.size(0) == H_kv and k_shadow.size(2) == HEAD_DIM,
               "shadows must be (H_kv, num_slots, 128)")
        self._keep = (k_shadow, v_shadow)
        self.shape = (B, H_q, K)
        self._h = lib.jf_handoff_create(B, H_q, H_kv, K, k_shadow.size(1), k_shadow.data_ptr(), v_shadow.data_ptr(),
                                        float(scale))
        if not self._h:
            raise RuntimeError(lib.jf_last_error().decode())

    def submit(self, q, topk_slots) -> None:
        B, H_q, K = self.shape
        _check(q.is_cuda and q.dtype == torch.bfloat16 and q.is_contiguous() and q.shape == (B, H_q, HEAD_DIM),
               "q must be contiguous (B, H_q, 128) bf16 on the GPU")
        _check(topk_slots.is_cuda and topk_slots.dtype == torch.int64 and topk_slots.is_contiguous()
               and topk_slots.shape == (B, H_q, K), "topk_slots must be contiguous (B, H_q, K) int64 on the GPU")
        _lib.check(_lib.load().jf_handoff_submit(self._h, q.data_ptr(), topk_slots.data_ptr(), _stream(q)))

    def wait(self, o_new) -> None:
        B, H_q, _ = self.shape
        _check(o_new.is_cuda and o_new.dtype == torch.bfloat16 and o_new.is_contiguous()
               and o_new.shape == (B, H_q, HEAD_DIM), "o_new must be contiguous (B, H_q, 128) bf16 on the GPU")
        _lib.check(_lib.load().jf_handoff_wait(self._h, o_new.data_ptr(), _stream(o_new)))

    def stream_submit(self, q, topk_slots) -> None:
        """Graph-capturable submit (cpu_topk_attn.cpp:1805-1900 without the host callback): kernels only."""
        B, H_q, K = self.shape
        _check(q.is_cuda and q.dtype == torch.bfloat16 and q.is_contiguous() and q.shape == (B, H_q, HEAD_DIM),
               "q must be contiguous (B, H_q, 128) bf16 on the GPU")
        _check(topk_slots.is_cuda and topk_slots.dtype == torch.int64 and topk_slots.is_contiguous()
               and topk_slots.shape == (B, H_q, K), "topk_slots must be contiguous (B, H_q, K) int64 on the GPU")
        _lib.check(_lib.load().jf_handoff_stream_submit(self._h, q.data_ptr(), topk_slots.data_ptr(), _stream(q)))

    def stream_wait(self, o_new) -> None:
        """Graph-capturable join: a kernel waits (bounded) for the correction and brings o_new to the device."""
        B, H_q, _ = self.shape
        _check(o_new.is_cuda and o_new.dtype == torch.bfloat16 and o_new.is_contiguous()
               and o_new.shape == (B, H_q, HEAD_DIM), "o_new must be contiguous (B, H_q, 128) bf16 on the GPU")
        _lib.check(_lib.load().jf_handoff_stream_wait(self._h, o_new.data_ptr(), _stream(o_new)))

    def stream_wait_blend(self, o_hat, o_old_unnorm, W, out, o_new=None) -> None:
        """`stream_wait` and `blend_unnorm_into` in one kernel: `out = bf16(fma(W, o_new, o_hat) - o_old_unnorm)`."""
        B, H_q, _ = self.shape
        for t in (o_hat, o_old_unnorm):
            _check(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.shape == (B, H_q, HEAD_DIM),
                   "o_hat / o_old_unnorm must be contiguous (B, H_q, 128) fp32 on the GPU")
        _check(W.is_cuda and W.dtype == torch.float32 and W.is_contiguous() and W.shape == (B, H_q), "W must be (B, H_q) fp32")
        for t in (out,) + ((o_new,) if o_new is not None else ()):
            _check(t.is_cuda and t.dtype == torch.bfloat16 and t.is_contiguous() and t.shape == (B, H_q, HEAD_DIM),
                   "out / o_new must be contiguous (B, H_q, 128) bf16 on the GPU")
        _lib.check(_lib.load().jf_handoff_stream_wait_blend(self._h, o_hat.data_ptr(), o_old_unnorm.data_ptr(), W.data_ptr(),
                                                            out.data_ptr(), _ptr(o_new), _stream(out)))

    def set_output_sanitize(self, on: bool) -> None:
        """stream_wait_blend writes zero for non-finite outputs (decode_path.py:1133-1149)."""
        _lib.check(_lib.load().jf_handoff_set_output_sanitize(self._h, 1 if on else 0))

    def check_status(self) -> None:
        """Raises if a correction failed or a device-side wait ran into its limit (call after a synchronise)."""
        _lib.check(_lib.load().jf_handoff_status(self._h))

    def set_device_wait_limit_us(self, us: int) -> None:
        _lib.check(_lib.load().jf_handoff_set_device_wait_limit_us(self._h, int(us)))

    def debug_pause(self, on: bool) -> None:
        _lib.check(_lib.debug_hook("jf_handoff_debug_pause")(self._h, 1 if on else 0))

    @property
    def submit_count(self) -> int:
        return int(_lib.load().jf_handoff_submit_count(self._h))

    def close(self) -> None:
        if self._h:
            _lib.load().jf_handoff_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
