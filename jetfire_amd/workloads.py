"""Synthetic decode workloads at the benchmark shapes: seeded K/V (bf16 N(0,1), four key channels
scaled x8 as outliers), q ~ N(0,1)/sqrt(128), quantised on the GPU with the library's own
quantise-on-append kernels into the reference cache layout, one cache per layer."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List

import torch

from . import ops

HEAD_DIM = 128
BLOCK = 16

# name: (B, H_q, H_kv, S, scheme, group, top_k, layers)
CONFIGS = {
    "c1": (1, 32, 8, 4096, "k4v4", 128, 64, 1),
    "c2": (4, 32, 8, 32768, "k3v2", 64, 256, 32),
    "c2k4": (4, 32, 8, 32768, "k4v4", 128, 256, 32),     # the c2 shape with INT4 keys and values (the metric's "K4V4 at 32k")
    "c3": (1, 32, 8, 131072, "k4v4", 128, 512, 32),
    "c4": (4, 32, 4, 32768, "k3v2", 64, 256, 48),
    "c5": (2, 32, 4, 65536, "k3v2", 64, 512, 80),
}


def scheme_bits(scheme: str):
    """"k3v2" -> (3, 2, False); "a2v4" (asymmetric INT2 keys with zero-points) -> (2, 4, True); "b4v4" (INT4 keys
    scored with the bf16 model: the same cache as "k4v4") -> (4, 4, False)."""
    return int(scheme[1]), int(scheme[3]), scheme[0] == "a"


def bytes_per_token_head(scheme: str, group: int) -> int:
    """Packed codes plus bf16 scales (and zero-points) of one token of one kv-head, K and V together."""
    kb, vb, asym = scheme_bits(scheme)
    ng = HEAD_DIM // group
    return 16 * kb + 16 * vb + 2 * ng * (3 if asym else 2)



@dataclass
class LayerCache:
    k_data: torch.Tensor
    k_scales: torch.Tensor
    v_data: torch.Tensor
    v_scales: torch.Tensor
    k_zp: torch.Tensor | None = None        # asymmetric INT2 keys only


@dataclass
class Workload:
    name: str
    B: int
    H_q: int
    H_kv: int
    S: int
    scheme: str
    group: int
    top_k: int
    layers: List[LayerCache]
    q: torch.Tensor
    block_table: torch.Tensor
    seq_lens: torch.Tensor
    attn_scale: float

    @property
    def packed_bytes_per_layer(self) -> int:
        return self.B * self.H_kv * self.S * bytes_per_token_head(self.scheme, self.group)


def build(name: str, n_layers: int | None = None, seed: int = 0, paged: bool = False, device: str = "cuda",
          keep_shadow: int = 0) -> Workload:
    """keep_shadow: number of layers (the first ones) whose bf16 K/V are also kept on the host in the cache's
    slot order, as the CPU correction's shadow."""
    B, Hq, Hkv, S, scheme, gs, top_k, layers = CONFIGS[name]
    if n_layers is not None:
        layers = n_layers
    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    cpu_gen = torch.Generator().manual_seed(seed)
    outliers = torch.randperm(HEAD_DIM, generator=cpu_gen)[:4].to(dev)
    T = B * S
    nblk = T // BLOCK
    if paged:
        perm = torch.randperm(nblk, generator=cpu_gen)
    else:
        perm = torch.arange(nblk)
    block_table = perm.reshape(B, S // BLOCK).to(torch.int64).to(dev)
    pos = torch.arange(S, device=dev)
    slots = (block_table[:, pos // BLOCK] * BLOCK + pos % BLOCK).reshape(-1)      # token t = b*S + pos
    kb, vb, asym = scheme_bits(scheme)
    sym_writer = {2: ops.fused_quant_write_int2_sym, 3: ops.fused_quant_write_int3_sym, 4: ops.fused_quant_write_int4_sym}
    caches = []
    shadows = []
    for _ in range(layers):
        k = torch.randn(T, Hkv, HEAD_DIM, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
        k[..., outliers] *= 8
        v = torch.randn(T, Hkv, HEAD_DIM, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
        kd = torch.empty(Hkv, T, HEAD_DIM * kb // 8, dtype=torch.uint8, device=dev)
        ks = torch.empty(Hkv, T, HEAD_DIM // gs, dtype=torch.bfloat16, device=dev)
        vd = torch.empty(Hkv, T, HEAD_DIM * vb // 8, dtype=torch.uint8, device=dev)
        vs = torch.empty(Hkv, T, HEAD_DIM // gs, dtype=torch.bfloat16, device=dev)
        kz = None
        if scheme == "k4v4":
            ops.fused_quant_write_int4_sym_kv(k, v, slots, kd, ks, vd, vs, gs)
        else:
            if asym:
                kz = torch.empty_like(ks)
                ops.fused_quant_write_int2_asym(k, slots, kd, ks, kz, gs)
            else:
                sym_writer[kb](k, slots, kd, ks, gs)
            sym_writer[vb](v, slots, vd, vs, gs)
        caches.append(LayerCache(kd, ks, vd, vs, kz))
        if len(shadows) < int(keep_shadow):
            ksh = torch.empty(Hkv, T, HEAD_DIM, dtype=torch.bfloat16)
            vsh = torch.empty(Hkv, T, HEAD_DIM, dtype=torch.bfloat16)
            ksh[:, slots.cpu()] = k.permute(1, 0, 2).cpu()
            vsh[:, slots.cpu()] = v.permute(1, 0, 2).cpu()
            shadows.append((ksh, vsh))
        del k, v
    q = (torch.randn(B, Hq, HEAD_DIM, generator=gen, device=dev, dtype=torch.float32) / HEAD_DIM ** 0.5).to(torch.bfloat16)
    seq_lens = torch.full((B,), S, dtype=torch.int32, device=dev)
    w = Workload(name, B, Hq, Hkv, S, scheme, gs, top_k, caches, q, block_table, seq_lens, HEAD_DIM ** -0.5)
    w.shadows = shadows
    return w
