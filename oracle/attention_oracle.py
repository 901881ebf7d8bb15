"""Eager fp32 restatement of the attention path.  TEST INFRASTRUCTURE ONLY
(see ``oracle/__init__.py``): never imported by the product.

It follows the un-compiled side of the reference -- the graph the user writes
and the reference's own accuracy tests evaluate eagerly
(``/root/reference/tests/test_accuracy.py:13-14, 130-134``):

    scores = Q @ K^T * scale                 reference README.md:75-79
    scores = cap * tanh(scores / cap)        tests/benchmark.py:144      (optional)
    scores = mask(scores)                    torch_backend/__init__.py:4-8 (causal),
                                             torch_backend/ops.py:733-741 (causal window)
    P      = softmax(scores, dim=-1)
    O      = P @ V

with K/V heads repeated for GQA (``repeat_interleave``, tests/test_accuracy.py:
153-156) and K/V optionally gathered through a page table
(``out[*s,*t] = buffer[block_table[*s],*t]``, torch_backend/__init__.py:46-56).
Inputs are upcast to fp32 first; the result stays fp32.

Pinning (tests/test_oracle.py): the reference ships no golden vectors for this
path (no seeds, no stored tensors anywhere in its tests), so every function here
is pinned by what the mathematics fixes instead:
  * attention_reference  -- against a float64 pure-Python triple loop on tiny
    inputs (a dropped scale, wrong mask orientation, transposed operand or
    missing softcap each fail it), rows of P summing to 1, the uniform-V
    invariance O == V[0] and closed forms for 1-key and constant-score cases;
  * dense_mask           -- against the closed forms i>=j / 0<=i-j<w and torch.tril;
  * gather_paged         -- identity table == contiguous; permutation round trip;
  * online_tiled_reference -- the tiled rescaling recurrence of the reference's
    optimiser (compiler/passes/factor_acc.py:23-109, README.md:85-99) against
    attention_reference, for any tile size and for the block-skip ranges;
  * visited_tiles_dense  -- brute force over the dense mask (this *is* the spec).
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def dense_mask(kind: Optional[str], Sq: int, Sk: int, window: int = 0) -> torch.Tensor:
    """[Sq, Sk] bool, True = keep.  Top-left aligned (reference ops.py:696, 733-741)."""
    i = torch.arange(Sq).unsqueeze(1)
    j = torch.arange(Sk).unsqueeze(0)
    if kind in (None, "none"):
        return torch.ones(Sq, Sk, dtype=torch.bool)
    if kind == "causal":
        return j <= i
    if kind == "sliding":
        return (j <= i) & (i - j < window)
    raise ValueError(kind)


def gather_paged(pool: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """pool [N, Hkv, D] or [N, P, Hkv, D], table [B, pages] -> dense [B, Hkv, Sk, D]."""
    g = pool[table.long()]                      # [B, pages, (P,) Hkv, D]
    if pool.dim() == 4:
        B, pages, P, H, D = g.shape
        g = g.reshape(B, pages * P, H, D)
    return g.transpose(1, 2)


def attention_reference(q, k, v, *, mask: Optional[str] = None, window: int = 0,
                        scale: Optional[float] = None, softcap: Optional[float] = None,
                        k_table=None, v_table=None, score_bias=None, out_bias=None,
                        denom_add: float = 0.0, q2=None, k2=None) -> torch.Tensor:
    """fp32 eager attention.  q [B,Hq,Sq,D]; k, v [B,Hkv,Sk,D] or page pools + tables.
    ``score_bias`` (broadcastable to [B,Hq,Sq,Sk]) is added to the scaled / capped scores
    before the mask and ``out_bias`` ([B,Hq,Sq,D]) to the result, as in the reference's
    modified-attention graph (tests/test_accuracy.py:172-196).  ``denom_add`` = c gives the
    probabilities e^(s - m) / (sum_j e^(s_j - m) + c) with m the row maximum, the explicit
    softmax of the reference's tests/test_attention.py:95-125 (c = 1 there).  ``q2``
    [B,Hq,Sq,D2] and ``k2`` [B,H2,Sk,D2] (heads repeated like K's) add a second product to
    the raw scores, (Q K^T + Q2 K2^T) * scale, the two-part scores of the reference's
    tests/test_attention.py:126-151 (``scale`` must then be given: that graph uses
    (D + D2)^-0.5)."""
    q = q.float()
    k = gather_paged(k.float(), k_table) if k_table is not None else k.float()
    v = gather_paged(v.float(), v_table) if v_table is not None else v.float()
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    if scale is None:
        scale = D ** -0.5
    if Hq != Hkv:
        k = k.repeat_interleave(Hq // Hkv, dim=1)
        v = v.repeat_interleave(Hq // Hkv, dim=1)
    s = torch.matmul(q, k.transpose(-2, -1))
    if q2 is not None:
        k2 = k2.float()
        if k2.shape[1] != Hq:
            k2 = k2.repeat_interleave(Hq // k2.shape[1], dim=1)
        s = s + torch.matmul(q2.float(), k2.transpose(-2, -1))
    s = s * scale
    if softcap is not None:
        s = torch.tanh(s / softcap) * softcap
    if score_bias is not None:
        s = s + score_bias.float()
    keep = dense_mask(mask, Sq, Sk, window).to(s.device)
    s = s.masked_fill(~keep, float("-inf"))
    if denom_add:
        e = torch.exp(s - s.max(dim=-1, keepdim=True).values)
        p = e / (e.sum(dim=-1, keepdim=True) + denom_add)
    else:
        p = torch.softmax(s, dim=-1)
    out = torch.matmul(p, v)
    if out_bias is not None:
        out = out + out_bias.float()
    return out


def online_tiled_reference(q, k, v, *, mask=None, window=0, scale=None, softcap=None,
                           bm: int = 128, bn: int = 64, tile_ranges=None) -> torch.Tensor:
    """The fused loop nest the reference's optimiser produces (FlashAttention-2
    forward): per Q tile, walk KV tiles keeping (m, l, acc) and rescaling by
    2^(m_prev - m_new).  ``tile_ranges[qt] = (begin, end)`` restricts the walk
    (block skip).  fp32 throughout; only for checking the recurrence."""
    q, k, v = q.float(), k.float(), v.float()
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    if scale is None:
        scale = D ** -0.5
    if Hq != Hkv:
        k = k.repeat_interleave(Hq // Hkv, dim=1)
        v = v.repeat_interleave(Hq // Hkv, dim=1)
    keep_all = dense_mask(mask, Sq, Sk, window)
    out = torch.empty(B, Hq, Sq, D)
    log2e = 1.0 / math.log(2.0)
    for qt in range((Sq + bm - 1) // bm):
        r0, r1 = qt * bm, min((qt + 1) * bm, Sq)
        m = torch.full((B, Hq, r1 - r0, 1), float("-inf"))
        l = torch.zeros(B, Hq, r1 - r0, 1)
        acc = torch.zeros(B, Hq, r1 - r0, D)
        nkt = (Sk + bn - 1) // bn
        begin, end = (0, nkt) if tile_ranges is None else tile_ranges[qt]
        for kt in range(begin, end):
            c0, c1 = kt * bn, min((kt + 1) * bn, Sk)
            s = torch.matmul(q[:, :, r0:r1], k[:, :, c0:c1].transpose(-2, -1)) * scale
            if softcap is not None:
                s = torch.tanh(s / softcap) * softcap
            s = s.masked_fill(~keep_all[r0:r1, c0:c1], float("-inf")) * log2e
            m_new = torch.maximum(m, s.max(dim=-1, keepdim=True).values)
            m_sub = torch.where(torch.isinf(m_new), torch.zeros_like(m_new), m_new)
            p = torch.exp2(s - m_sub)
            r = torch.exp2(m - m_sub)
            l = l * r + p.sum(dim=-1, keepdim=True)
            acc = acc * r + torch.matmul(p, v[:, :, c0:c1])
            m = m_new
        out[:, :, r0:r1] = acc / l
    return out


def visited_tiles_dense(mask: Optional[str], Sq: int, Sk: int, window: int, bm: int, bn: int) -> torch.Tensor:
    """[nqt, nkt] bool: tile (qt, kt) holds at least one unmasked score.  The
    specification of the block-skip set (reference skip_loop_iterations.py:
    318-341: a step is skipped iff every carried variable keeps its value)."""
    keep = dense_mask(mask, Sq, Sk, window)
    nqt, nkt = (Sq + bm - 1) // bm, (Sk + bn - 1) // bn
    out = torch.zeros(nqt, nkt, dtype=torch.bool)
    for qt in range(nqt):
        for kt in range(nkt):
            out[qt, kt] = bool(keep[qt * bm:(qt + 1) * bm, kt * bn:(kt + 1) * bn].any())
    return out


def eager_reference_graph(q, k, v):
    """The reference's CPU-runnable path for config 1, op for op: plain ATen on
    the host (reference README.md:75-79; the mask is the eager body of
    ``loopfuse::causal_mask``, torch_backend/__init__.py:4-8).  Timed by
    bench.py's cpu_baseline leg."""
    s = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
    n = s.shape[-1]
    keep = torch.tril(torch.ones(n, n, dtype=torch.bool, device=s.device))
    s = s.masked_fill(~keep, float("-inf"))
    return torch.softmax(s, dim=-1) @ v
