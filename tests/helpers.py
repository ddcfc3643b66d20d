"""Shared test plumbing: seeded cases built with the oracle, numpy <-> torch conversions."""
import numpy as np
import torch

from oracle import jetfire_oracle as O


def bf16_tensor(a: np.ndarray) -> torch.Tensor:
    """float32 array of bf16-representable values -> torch bf16 (exact)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16)


def bits_to_bf16(b: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(b, dtype=np.uint16).view(np.int16)).view(torch.bfloat16)


def bf16_to_bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_to_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().float().numpy()


SCHEMES = {"k3v2": (3, 2, 64), "k4v4": (4, 4, 128), "k3v2_g128": (3, 2, 128)}


def make_case(seed, B, Hq, Hkv, S, kbits, vbits, gs, ragged=True, shuffle=True, lens=None, extra_blocks=0, k_asym=False):
    """Seeded decode-step inputs: K/V ~ N(0,1) with 4 outlier key channels x8, q ~ N(0,1)/sqrt(128),
    quantised with the oracle quantiser into a paged cache with a (optionally shuffled) block table.
    k_asym: the keys take the asymmetric quantiser (zero-points in `kzp`); kbits must be 2."""
    rng = np.random.default_rng(seed)
    per_seq = (S + 15) // 16
    nblk = B * per_seq + extra_blocks
    slots_total = nblk * 16
    K = O.bf16_round(rng.standard_normal((slots_total, Hkv, 128)).astype(np.float32))
    K[..., rng.permutation(128)[:4]] *= 8
    K = O.bf16_round(K)
    V = O.bf16_round(rng.standard_normal((slots_total, Hkv, 128)).astype(np.float32))
    q = O.bf16_round((rng.standard_normal((B, Hq, 128)) / np.sqrt(128)).astype(np.float32))
    Kh, Vh = np.ascontiguousarray(K.transpose(1, 0, 2)), np.ascontiguousarray(V.transpose(1, 0, 2))
    kzp = None
    if k_asym:
        kd, ks, kzp = O.quantize_and_pack_asym(Kh, gs, kbits)
    else:
        kd, ks = O.quantize_and_pack(Kh, gs, kbits)
    vd, vs = O.quantize_and_pack(Vh, gs, vbits)
    perm = rng.permutation(nblk) if shuffle else np.arange(nblk)
    bt = perm[:B * per_seq].reshape(B, per_seq).astype(np.int64)
    if lens is None:
        lens = [max(0, S - 13 * b) if ragged else S for b in range(B)]
    lens = np.array(lens, dtype=np.int32)
    return dict(q=q, kd=kd, ks=ks, vd=vd, vs=vs, bt=bt, lens=lens, K=Kh, V=Vh, S=S, B=B, Hq=Hq, Hkv=Hkv,
                kbits=kbits, vbits=vbits, gs=gs, kzp=kzp)


def to_device(c, device="cuda"):
    """Torch views of a case on `device`."""
    return dict(
        kz=None if c.get("kzp") is None else bits_to_bf16(c["kzp"]).to(device),
        q=bf16_tensor(c["q"]).to(device),
        kd=torch.from_numpy(c["kd"]).to(device), ks=bits_to_bf16(c["ks"]).to(device),
        vd=torch.from_numpy(c["vd"]).to(device), vs=bits_to_bf16(c["vs"]).to(device),
        bt=torch.from_numpy(c["bt"]).to(device), lens=torch.from_numpy(c["lens"]).to(device),
    )
