"""Slot-addressable quantised KV cache of one layer plus its bf16 host shadow
(`jetfire_vllm/adapter/cache_store.py:183-759,1340-1445`), for the symmetric INT2/3/4 schemes.

Layout (kept byte for byte): `k_data (Hkv, num_slots, Pk) u8`, `k_scales (Hkv, num_slots, D/group) bf16`,
the same for V, `slot = block * block_size + offset`; shadow `(Hkv, num_slots, D)` bf16 in host memory.
Appends go through the library's quantise-on-write kernels; the shadow rows are copied to the host in the
same call (the reference's serial path, `:686-759`).  The reference's prefill side-stream pipeline and its
graph-mode append are not part of this path: `flush_pending_writes` has nothing to wait for."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import ops

_SEQ_SLOTS_CACHE: dict = {}


def packed_dim(head_dim: int, nbits: int) -> int:
    return head_dim * nbits // 8


@dataclass
class JetFireLayerView:
    k_data: torch.Tensor
    k_scales: torch.Tensor
    v_data: torch.Tensor
    v_scales: torch.Tensor
    seq_len: int
    k_zp: torch.Tensor | None = None
    v_zp: torch.Tensor | None = None


class JetFireInt4CacheStore:
    """Quantised KV cache of one layer.  Independent K and V bit widths (2, 3 or 4), symmetric only."""

    def __init__(self, *, num_kv_heads: int, head_dim: int, group_size: int, num_blocks: int, block_size: int,
                 device, k_nbits: int, v_nbits: int, k_asymmetric: bool = False, v_asymmetric: bool = False,
                 shadow_enabled: bool = True) -> None:
        if head_dim % group_size != 0:
            raise ValueError(f"head_dim={head_dim} must be divisible by group_size={group_size}")
        if k_asymmetric or v_asymmetric:
            raise NotImplementedError("asymmetric (zero-point) schemes are outside this library's decode path")
        if int(k_nbits) not in (2, 3, 4) or int(v_nbits) not in (2, 3, 4):
            raise ValueError(f"unsupported bit widths k={k_nbits} v={v_nbits}")
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.group_size = int(group_size)
        self.num_blocks = int(num_blocks)
        self.block_size = int(block_size)
        self.num_slots = self.num_blocks * self.block_size
        self.device = torch.device(device)
        self.k_nbits, self.v_nbits = int(k_nbits), int(v_nbits)
        self.k_asymmetric = self.v_asymmetric = False
        ng = self.head_dim // self.group_size
        dev = self.device
        # zero-initialised: positions past a sequence's end are never scored, but they are read
        self.k_data = torch.zeros(self.num_kv_heads, self.num_slots, packed_dim(self.head_dim, self.k_nbits), dtype=torch.uint8, device=dev)
        self.k_scales = torch.zeros(self.num_kv_heads, self.num_slots, ng, dtype=torch.bfloat16, device=dev)
        self.v_data = torch.zeros(self.num_kv_heads, self.num_slots, packed_dim(self.head_dim, self.v_nbits), dtype=torch.uint8, device=dev)
        self.v_scales = torch.zeros(self.num_kv_heads, self.num_slots, ng, dtype=torch.bfloat16, device=dev)
        self.k_zp = self.v_zp = None
        self.slot_filled = torch.zeros(self.num_slots, dtype=torch.bool, device=dev)
        self.written_count = 0
        self.shadow_enabled = bool(shadow_enabled)
        if self.shadow_enabled:
            pin = dev.type == "cuda"
            self.k_shadow = torch.zeros(self.num_kv_heads, self.num_slots, self.head_dim, dtype=torch.bfloat16, pin_memory=pin)
            self.v_shadow = torch.zeros(self.num_kv_heads, self.num_slots, self.head_dim, dtype=torch.bfloat16, pin_memory=pin)
        else:
            self.k_shadow = self.v_shadow = None
        self.k_full_cpu, self.v_full_cpu = self.k_shadow, self.v_shadow   # the reference's legacy aliases

    # ------------------------------------------------------------------ geometry
    def compatible_with(self, *, num_kv_heads: int, head_dim: int, num_blocks: int | None = None,
                        block_size: int | None = None) -> bool:
        return (self.num_kv_heads == int(num_kv_heads) and self.head_dim == int(head_dim)
                and (num_blocks is None or self.num_blocks == int(num_blocks))
                and (block_size is None or self.block_size == int(block_size)))

    @property
    def scheme(self) -> str | None:
        """Name the fused decode kernels know this store by, or None (split kernels / unsupported)."""
        if (self.k_nbits, self.v_nbits) == (3, 2) and self.group_size in (64, 128):
            return "k3v2"
        if (self.k_nbits, self.v_nbits) == (4, 4) and self.group_size == 128:
            return "k4v4"
        return None

    # ------------------------------------------------------------------ append
    def write_slots(self, *, key: torch.Tensor, value: torch.Tensor, slot_mapping: torch.Tensor | None) -> int:
        """Quantise `key` / `value` (T, Hkv, D) into the rows named by `slot_mapping` (T,); negative slots are
        padding and are skipped.  Returns the number of rows offered (as the reference does)."""
        if slot_mapping is None or slot_mapping.numel() == 0:
            return 0
        n = min(int(slot_mapping.numel()), int(key.shape[0]), int(value.shape[0]))
        slots = slot_mapping[:n].to(device=self.device, dtype=torch.long).contiguous()
        key_tok, value_tok = key[:n], value[:n]
        if key_tok.shape[1:] != (self.num_kv_heads, self.head_dim) or value_tok.shape[1:] != key_tok.shape[1:]:
            raise ValueError(f"key/value must be (T, {self.num_kv_heads}, {self.head_dim}); got {tuple(key.shape)}, {tuple(value.shape)}")
        key_tok = key_tok.to(device=self.device, dtype=torch.bfloat16)
        value_tok = value_tok.to(device=self.device, dtype=torch.bfloat16)
        if self.k_nbits == 4 and self.v_nbits == 4:
            ops.fused_quant_write_int4_sym_kv(key_tok, value_tok, slots, self.k_data, self.k_scales, self.v_data,
                                              self.v_scales, self.group_size)
        else:
            sym = {2: ops.fused_quant_write_int2_sym, 3: ops.fused_quant_write_int3_sym, 4: ops.fused_quant_write_int4_sym}
            sym[self.k_nbits](key_tok, slots, self.k_data, self.k_scales, self.group_size)
            sym[self.v_nbits](value_tok, slots, self.v_data, self.v_scales, self.group_size)
        valid = slots >= 0
        self.slot_filled[slots[valid]] = True
        if self.shadow_enabled:
            # the host copy synchronises with the stream, as the reference's serial path does
            slots_cpu = slots.to("cpu")
            keep = slots_cpu >= 0
            k_host = key_tok.permute(1, 0, 2).to("cpu")
            v_host = value_tok.permute(1, 0, 2).to("cpu")
            if not bool(keep.all()):
                slots_cpu, k_host, v_host = slots_cpu[keep], k_host[:, keep], v_host[:, keep]
            self.k_shadow.index_copy_(1, slots_cpu, k_host)
            self.v_shadow.index_copy_(1, slots_cpu, v_host)
        self.written_count += n
        return n

    def flush_pending_writes(self) -> None:
        """Appends are complete when `write_slots` returns: nothing is pending."""
        return None

    # ------------------------------------------------------------------ lookups
    def sequence_slots(self, block_table_row: torch.Tensor, seq_len: int) -> torch.Tensor:
        if seq_len <= 0:
            raise ValueError(f"seq_len must be positive, got {seq_len}")
        nb = (int(seq_len) + self.block_size - 1) // self.block_size
        blocks = block_table_row[:nb].to(device=self.device, dtype=torch.long).flatten()
        if blocks.numel() != nb:
            raise ValueError("block_table row is too short for requested seq_len")
        if bool(torch.any(blocks < 0)):
            raise ValueError("block_table contains invalid negative block ids")
        off = torch.arange(self.block_size, device=self.device, dtype=torch.long)
        return (blocks[:, None] * self.block_size + off[None, :]).reshape(-1)[:seq_len]

    def sequence_slots_fast(self, block_table_row: torch.Tensor, seq_len: int) -> torch.Tensor:
        """`sequence_slots` without validation (no device-to-host sync), cached for the last row asked for."""
        key = (int(block_table_row.data_ptr()), int(seq_len), id(self))
        hit = _SEQ_SLOTS_CACHE.get(key)
        if hit is not None:
            return hit
        nb = (int(seq_len) + self.block_size - 1) // self.block_size
        blocks = block_table_row[:nb].to(device=self.device, dtype=torch.long).flatten()
        off = torch.arange(self.block_size, device=self.device, dtype=torch.long)
        slots = (blocks[:, None] * self.block_size + off[None, :]).reshape(-1)[:seq_len]
        _SEQ_SLOTS_CACHE.clear()
        _SEQ_SLOTS_CACHE[key] = slots
        return slots

    def fast_has_sequence(self, seq_len: int) -> bool:
        return self.written_count >= seq_len

    def has_sequence(self, block_table_row: torch.Tensor, seq_len: int) -> bool:
        return bool(torch.all(self.slot_filled[self.sequence_slots(block_table_row, seq_len)]).item())

    def gather_sequence(self, block_table_row: torch.Tensor, seq_len: int) -> JetFireLayerView:
        slots = self.sequence_slots(block_table_row, seq_len)
        return JetFireLayerView(k_data=self.k_data.index_select(1, slots), k_scales=self.k_scales.index_select(1, slots),
                                v_data=self.v_data.index_select(1, slots), v_scales=self.v_scales.index_select(1, slots),
                                seq_len=int(seq_len))
