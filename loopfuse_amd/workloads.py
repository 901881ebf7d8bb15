"""Seeded synthetic inputs for the five benchmark configurations.

Generated on the CPU generator in fp32 and cast, so a CPU checker and the GPU
kernel see identical bits whatever the device.  Shapes follow the reference's
benchmark harness (``tests/benchmark.py:68-76, 207-217, 380-398, 510-520``) with
the sizes of the five benchmark configurations.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

import torch


@dataclasses.dataclass
class Workload:
    name: str
    q: torch.Tensor
    k: torch.Tensor                    # dense [B,Hkv,Sk,D] or page pool [N,P,Hkv,D]
    v: torch.Tensor
    mask: Optional[str] = None
    window: int = 0
    softcap: Optional[float] = None
    k_table: Optional[torch.Tensor] = None
    v_table: Optional[torch.Tensor] = None
    score_bias: Optional[torch.Tensor] = None      # a mask given as a tensor of 0 / -inf
    counts_as: Optional[str] = None                # mask whose work formula applies when the mask is a tensor
    visible_keys: Optional[int] = None             # decode with a mask tensor: keys with a finite bias, summed over the batch

    @property
    def scale(self) -> float:
        return self.q.shape[-1] ** -0.5

    def to(self, device) -> "Workload":
        mv = lambda t: None if t is None else t.to(device)
        return dataclasses.replace(self, q=mv(self.q), k=mv(self.k), v=mv(self.v),
                                   k_table=mv(self.k_table), v_table=mv(self.v_table), score_bias=mv(self.score_bias))

    # work counts, conventions of the reference's benchmark (tests/benchmark.py:110,
    # 280-284, 369, 452): Q, O and table traffic are not counted
    def flops(self) -> int:
        B, Hq, Sq, D = self.q.shape
        if self.mask == "sliding":
            w = self.window
            return 2 * B * Hq * (2 * Sq * w - w * w) * D
        if self.mask == "causal" or self.counts_as == "causal":
            return 2 * B * Hq * Sq * Sq * D
        Sk = self.kv_len()
        return 4 * B * Hq * Sq * Sk * D

    def kv_len(self) -> int:
        if self.k_table is not None:
            return self.k_table.shape[1] * (self.k.shape[1] if self.k.dim() == 4 else 1)
        return self.k.shape[2]

    def kv_heads(self) -> int:
        return self.k.shape[-2] if self.k_table is not None else self.k.shape[1]

    def kv_bytes(self) -> int:
        B, D = self.q.shape[0], self.q.shape[-1]
        if self.visible_keys is not None:      # only the keys a sequence can see have to be read
            return 2 * self.k.element_size() * self.kv_heads() * self.visible_keys * D
        return 2 * self.k.element_size() * B * self.kv_heads() * self.kv_len() * D


def _randn(gen, shape, dtype):
    return torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype)


def make(name: str, seed: int = 0, dtype: torch.dtype = torch.bfloat16, *, B=None, S=None) -> Workload:
    """name in {"c1","c2","c2_softcap","c3","c4","c5"}; B / S override the size (tests).
    Variants whose mask is a tensor: "c2_mask" (config 2 with its causal mask as a [1,1,S,S]
    tensor of 0 / -inf), "c5_padded" (config 5 with a left padding of up to 512 keys per
    sequence), "cache4096" (decode B64 Hq32/Hkv8 over a contiguous cache of 4096 slots of
    which 300-600 per sequence are filled)."""
    g = torch.Generator().manual_seed(seed)
    if name == "c1":      # fp32 CPU-runnable case
        B, S = B or 2, S or 512
        q, k, v = (_randn(g, (B, 8, S, 64), torch.float32) for _ in range(3))
        return Workload(name, q, k, v, mask="causal")
    if name in ("c2", "c2_softcap"):
        B, S = B or 8, S or 2048
        q, k, v = (_randn(g, (B, 32, S, 128), dtype) for _ in range(3))
        return Workload(name, q, k, v, mask="causal", softcap=30.0 if name == "c2_softcap" else None)
    if name == "c2_mask":
        w = make("c2", seed, dtype, B=B, S=S)
        S = w.q.shape[2]
        i = torch.arange(S)
        bias = torch.zeros(S, S).masked_fill(i[None, :] > i[:, None], float("-inf")).to(dtype)[None, None]
        return dataclasses.replace(w, name=name, mask=None, score_bias=bias, counts_as="causal")
    if name == "c5_padded":
        w = make("c5", seed, dtype, B=B, S=S)
        Bn, Sk = w.q.shape[0], w.kv_len()
        pad = torch.randint(0, min(512, Sk // 2) + 1, (Bn,), generator=g)
        bias = torch.zeros(Bn, 1, 1, Sk).masked_fill(torch.arange(Sk)[None, None, None, :] < pad[:, None, None, None],
                                                     float("-inf")).to(dtype)
        return dataclasses.replace(w, name=name, score_bias=bias, visible_keys=int(Bn * Sk - pad.sum()))
    if name == "cache4096":
        B, S = B or 64, S or 4096
        q = _randn(g, (B, 32, 1, 128), dtype)
        k = _randn(g, (B, 8, S, 128), dtype)
        v = _randn(g, (B, 8, S, 128), dtype)
        fill = torch.randint(min(300, S // 2), min(600, S) + 1, (B,), generator=g)
        bias = torch.zeros(B, 1, 1, S).masked_fill(torch.arange(S)[None, None, None, :] >= fill[:, None, None, None],
                                                   float("-inf")).to(dtype)
        return Workload(name, q, k, v, score_bias=bias, visible_keys=int(fill.sum()))
    if name == "c3":
        B, S = B or 8, S or 2048
        q = _randn(g, (B, 32, S, 128), dtype)
        k = _randn(g, (B, 8, S, 128), dtype)
        v = _randn(g, (B, 8, S, 128), dtype)
        return Workload(name, q, k, v, mask="sliding", window=256, softcap=30.0)
    if name == "c4":
        B, S = B or 64, S or 2048
        q = _randn(g, (B, 32, 1, 128), dtype)
        k = _randn(g, (B, 32, S, 128), dtype)
        v = _randn(g, (B, 32, S, 128), dtype)
        return Workload(name, q, k, v)
    if name == "c5":
        B, S = B or 64, S or 2048
        P = 16
        pages = S // P
        n = B * pages
        q = _randn(g, (B, 32, 1, 128), dtype)
        kp = _randn(g, (n, P, 8, 128), dtype)
        vp = _randn(g, (n, P, 8, 128), dtype)
        table = torch.randperm(n, generator=g).view(B, pages).to(torch.int32)
        return Workload(name, q, kp, vp, k_table=table, v_table=table.clone())
    raise ValueError(name)


def run(w: Workload, **kw) -> torch.Tensor:
    """One pass of the hot path over a workload (tensors must be on the GPU)."""
    from . import lowering

    plan = lowering.AttnPlan(mask=w.mask, window=w.window, scale=w.scale, softcap=w.softcap,
                             k_paged=w.k_table is not None, v_paged=w.v_table is not None)
    if w.score_bias is not None:
        kw = {"score_bias": w.score_bias, **kw}
    return lowering.attention(w.q, w.k, w.v, plan, w.k_table, w.v_table, **kw)
