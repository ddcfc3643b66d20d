"""Slot-addressable quantised KV cache of one layer plus its bf16 host shadow
(`jetfire_vllm/adapter/cache_store.py:183-759,1340-1445`), for the symmetric INT2/3/4 schemes.

Layout (kept byte for byte): `k_data (Hkv, num_slots, Pk) u8`, `k_scales (Hkv, num_slots, D/group) bf16`,
the same for V, `slot = block * block_size + offset`; shadow `(Hkv, num_slots, D)` bf16 in pinned host memory.

Appends never synchronise with the host.  The quantise-on-write kernels run on the caller's stream.  The
shadow mirror is ONE kernel that stores the bf16 rows straight into the pinned shadow across PCIe
(`ops.shadow_write`); it takes the place of the reference's three mirror paths: the serial host copy +
`index_copy_` (`:686-759`), the prefill pipeline of D2H copies into pinned staging buffers and a worker
thread's scatter (`:1075-1338`), and the graph-mode decode append with its host callback (`:531-642`).
Chunks of at least `JETFIRE_PIPELINE_MIN_TOKENS` tokens (prefill) are mirrored on a side stream so that
the model's stream does not wait for PCIe; `flush_pending_writes` waits for those, as in the reference.
Smaller appends (decode tokens) stay on the caller's stream, ahead of the hand-off kernel that publishes
the step's slots to the CPU, and can be captured in a HIP graph (`write_slots_graph`)."""
from __future__ import annotations

import os
from dataclasses import dataclass

import torch

from .. import ops

_SEQ_SLOTS_CACHE: dict = {}


def _prefill_pipeline_enabled() -> bool:
    return os.environ.get("JETFIRE_PREFILL_PIPELINE", "1") == "1"


def _pipeline_min_tokens() -> int:
    return int(os.environ.get("JETFIRE_PIPELINE_MIN_TOKENS", "64"))


def _shadow_needed() -> bool:
    """The shadow is only read by the CPU correction; `JETFIRE_SHADOW=0` skips its writes
    (`jetfire_vllm/adapter/cache_store.py:172-180`)."""
    return os.environ.get("JETFIRE_SHADOW", "1") != "0"


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
    """Quantised KV cache of one layer.  Independent K and V bit widths (2, 3 or 4), symmetric, plus the
    asymmetric INT2 keys (full four-level codebook with a zero-point per group, `k_zp`)."""

    def __init__(self, *, num_kv_heads: int, head_dim: int, group_size: int, num_blocks: int, block_size: int,
                 device, k_nbits: int, v_nbits: int, k_asymmetric: bool = False, v_asymmetric: bool = False,
                 shadow_enabled: bool = True) -> None:
        if head_dim % group_size != 0:
            raise ValueError(f"head_dim={head_dim} must be divisible by group_size={group_size}")
        if v_asymmetric or (k_asymmetric and int(k_nbits) != 2):
            raise NotImplementedError("only INT2 keys have an asymmetric (zero-point) form in this library")
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
        self.k_asymmetric, self.v_asymmetric = bool(k_asymmetric), False
        ng = self.head_dim // self.group_size
        dev = self.device
        # zero-initialised: positions past a sequence's end are never scored, but they are read
        self.k_data = torch.zeros(self.num_kv_heads, self.num_slots, packed_dim(self.head_dim, self.k_nbits), dtype=torch.uint8, device=dev)
        self.k_scales = torch.zeros(self.num_kv_heads, self.num_slots, ng, dtype=torch.bfloat16, device=dev)
        self.v_data = torch.zeros(self.num_kv_heads, self.num_slots, packed_dim(self.head_dim, self.v_nbits), dtype=torch.uint8, device=dev)
        self.v_scales = torch.zeros(self.num_kv_heads, self.num_slots, ng, dtype=torch.bfloat16, device=dev)
        self.v_zp = None
        self.k_zp = torch.zeros(self.num_kv_heads, self.num_slots, ng, dtype=torch.bfloat16, device=dev) if self.k_asymmetric else None
        # one spare entry at the end takes the marks of padding tokens (slot < 0), so that marking needs no mask
        self._slot_filled_buf = torch.zeros(self.num_slots + 1, dtype=torch.bool, device=dev)
        self.slot_filled = self._slot_filled_buf[:self.num_slots]
        self.written_count = 0
        self.shadow_enabled = bool(shadow_enabled)
        if self.shadow_enabled:
            pin = dev.type == "cuda"
            self.k_shadow = torch.zeros(self.num_kv_heads, self.num_slots, self.head_dim, dtype=torch.bfloat16, pin_memory=pin)
            self.v_shadow = torch.zeros(self.num_kv_heads, self.num_slots, self.head_dim, dtype=torch.bfloat16, pin_memory=pin)
        else:
            self.k_shadow = self.v_shadow = None
        self.k_full_cpu, self.v_full_cpu = self.k_shadow, self.v_shadow   # the reference's legacy aliases
        self._shadow_dev: tuple[int, int] | None = None      # device-visible addresses of the two shadows
        self._mirror_stream: torch.cuda.Stream | None = None
        self._pending_mirrors: list = []                     # (event, tensors kept alive until the event)

    # ------------------------------------------------------------------ geometry
    def compatible_with(self, *, num_kv_heads: int, head_dim: int, num_blocks: int | None = None,
                        block_size: int | None = None) -> bool:
        return (self.num_kv_heads == int(num_kv_heads) and self.head_dim == int(head_dim)
                and (num_blocks is None or self.num_blocks == int(num_blocks))
                and (block_size is None or self.block_size == int(block_size)))

    @property
    def scheme(self) -> str | None:
        """Name the fused decode kernels know this store by, or None (split kernels / unsupported)."""
        if self.k_nbits not in (2, 3, 4) or self.v_nbits not in (2, 3, 4) or (self.k_asymmetric and self.k_nbits != 2):
            return None
        if self.group_size not in (64, 128):
            return None
        if self.k_asymmetric:
            return f"a2v{self.v_nbits}"
        if self.k_nbits == 4 and self.group_size == 64:      # two key scales per row: the bf16 model, as the reference
            return f"b4v{self.v_nbits}"                       # (jetfire_vllm/adapter/decode_path.py:2016-2022)
        return f"k{self.k_nbits}v{self.v_nbits}"

    # ------------------------------------------------------------------ append
    def _prepare(self, key, value, slot_mapping):
        n = min(int(slot_mapping.numel()), int(key.shape[0]), int(value.shape[0]))
        slots = slot_mapping[:n].to(device=self.device, dtype=torch.long).contiguous()
        key_tok, value_tok = key[:n], value[:n]
        if key_tok.shape[1:] != (self.num_kv_heads, self.head_dim) or value_tok.shape[1:] != key_tok.shape[1:]:
            raise ValueError(f"key/value must be (T, {self.num_kv_heads}, {self.head_dim}); got {tuple(key.shape)}, {tuple(value.shape)}")
        key_tok = key_tok.to(device=self.device, dtype=torch.bfloat16)
        value_tok = value_tok.to(device=self.device, dtype=torch.bfloat16)
        return n, slots, key_tok, value_tok

    def _quantise(self, key_tok, value_tok, slots) -> None:
        sym = {2: ops.fused_quant_write_int2_sym, 3: ops.fused_quant_write_int3_sym, 4: ops.fused_quant_write_int4_sym}
        if self.k_asymmetric:
            ops.fused_quant_write_int2_asym(key_tok, slots, self.k_data, self.k_scales, self.k_zp, self.group_size)
            sym[self.v_nbits](value_tok, slots, self.v_data, self.v_scales, self.group_size)
        elif self.k_nbits == 4 and self.v_nbits == 4:
            ops.fused_quant_write_int4_sym_kv(key_tok, value_tok, slots, self.k_data, self.k_scales, self.v_data,
                                              self.v_scales, self.group_size)
        else:
            sym[self.k_nbits](key_tok, slots, self.k_data, self.k_scales, self.group_size)
            sym[self.v_nbits](value_tok, slots, self.v_data, self.v_scales, self.group_size)

    def _mirror(self, key_tok, value_tok, slots) -> None:
        if self._shadow_dev is None:
            self._shadow_dev = (ops.host_buffer_device_pointer(self.k_shadow), ops.host_buffer_device_pointer(self.v_shadow))
        ops.shadow_write(key_tok, value_tok, slots, self.k_shadow, self.v_shadow,
                         k_shadow_dev=self._shadow_dev[0], v_shadow_dev=self._shadow_dev[1])

    def write_slots(self, *, key: torch.Tensor, value: torch.Tensor, slot_mapping: torch.Tensor | None) -> int:
        """Quantise `key` / `value` (T, Hkv, D) into the rows named by `slot_mapping` (T,) and mirror them into
        the shadow; negative slots are padding and are skipped.  Asynchronous: nothing here waits for the GPU.
        Returns the number of rows offered (as the reference does)."""
        if slot_mapping is None or slot_mapping.numel() == 0:
            return 0
        n, slots, key_tok, value_tok = self._prepare(key, value, slot_mapping)
        if n <= 0:
            return 0
        self._quantise(key_tok, value_tok, slots)
        self._slot_filled_buf.index_fill_(0, torch.where(slots >= 0, slots, self.num_slots), True)
        if self.shadow_enabled and _shadow_needed():
            side = (_prefill_pipeline_enabled() and n >= _pipeline_min_tokens()
                    and not torch.cuda.is_current_stream_capturing())
            if side:
                # prefill chunk: PCIe-bound, so off the model's stream (cache_store.py:1075-1110)
                if self._mirror_stream is None:
                    self._mirror_stream = torch.cuda.Stream(device=self.device)
                main = torch.cuda.current_stream(self.device)
                produced = torch.cuda.Event()
                produced.record(main)
                with torch.cuda.stream(self._mirror_stream):
                    self._mirror_stream.wait_event(produced)
                    self._mirror(key_tok, value_tok, slots)
                    done = torch.cuda.Event()
                    done.record(self._mirror_stream)
                self._pending_mirrors.append((done, key_tok, value_tok, slots))
            else:
                self._mirror(key_tok, value_tok, slots)
        self.written_count += n
        return n

    def write_slots_graph(self, *, key: torch.Tensor, value: torch.Tensor, slot_mapping: torch.Tensor | None,
                          max_batch_size: int) -> int:
        """Capture-safe decode append (`cache_store.py:531-642`): the quantise kernels and the mirror kernel on
        the capturing stream, nothing else.  The bookkeeping of filled slots is skipped, as in the reference."""
        if slot_mapping is None or slot_mapping.numel() == 0:
            return 0
        if not key.is_cuda or not value.is_cuda:
            raise RuntimeError("JetFire graph KV append requires GPU K/V tensors.")
        n = min(int(slot_mapping.numel()), int(key.shape[0]), int(value.shape[0]))
        if n <= 0:
            return 0
        if int(max_batch_size) <= 0 or n > int(max_batch_size):
            raise RuntimeError("JetFire graph KV append needs JETFIRE_MAX_BATCH_SIZE >= decode tokens. "
                               f"Got max_batch_size={int(max_batch_size)}, tokens={n}.")
        slots = slot_mapping[:n]
        if slots.device != key.device or slots.dtype != torch.long or not slots.is_contiguous():
            raise RuntimeError("JetFire graph KV append requires contiguous int64 slot_mapping on the same "
                               "device as K/V.")
        if key.dtype != torch.bfloat16 or value.dtype != torch.bfloat16:
            raise RuntimeError("JetFire graph KV append requires BF16 K/V.")
        key_tok, value_tok = key[:n], value[:n]
        self._quantise(key_tok, value_tok, slots)
        if self.shadow_enabled and _shadow_needed():
            if self._shadow_dev is None and torch.cuda.is_current_stream_capturing():
                raise RuntimeError("JetFire graph KV append context was not pre-created before graph capture "
                                   "(call warmup_graph_append first).")
            self._mirror(key_tok, value_tok, slots)
        return n

    def warmup_graph_append(self, max_batch_size: int) -> None:
        """Everything `write_slots_graph` may not do while a graph is being captured
        (`cache_store.py:411-419`): here only the look-up of the shadows' device-visible addresses."""
        if max_batch_size > 0 and self.shadow_enabled and self._shadow_dev is None:
            self._shadow_dev = (ops.host_buffer_device_pointer(self.k_shadow), ops.host_buffer_device_pointer(self.v_shadow))

    def flush_pending_writes(self) -> None:
        """Wait until every mirror launched on the side stream has landed in the shadow, so that the host may
        read `k_shadow` / `v_shadow` (`cache_store.py:1340-1374`).  Appends made on the caller's own stream
        are ordered ahead of whatever that stream does next and are not waited for here."""
        for done, *_ in self._pending_mirrors:
            done.synchronize()
        self._pending_mirrors.clear()

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
                                seq_len=int(seq_len),
                                k_zp=self.k_zp.index_select(1, slots) if self.k_zp is not None else None)
