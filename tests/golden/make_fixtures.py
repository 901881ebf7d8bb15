#!/usr/bin/env python3
"""Writes the small known-answer fixtures under tests/golden/ (run from the repo root:
``python tests/golden/make_fixtures.py``).

The reference holds no golden vectors for this path (no seeds, no stored tensors in
its tests), and it was not executed to make these: inputs come from a seeded CPU
generator, expected outputs from this repository's fp32 oracle
(oracle/attention_oracle.py), which tests/test_oracle.py pins independently against
float64 loops and closed forms.  The fixtures freeze those results so that a later
change to the oracle OR to the kernels shows up as a diff against stored numbers.

Format: one .npz per case (numpy, no pickle): bf16/fp16 inputs stored as uint16 bit
patterns, expected output as float32, parameters as 0-dim arrays.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attention_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    # name: (dtype, B, Hq, Hkv, Sq, Sk, D, mask, window, softcap, paged page size or 0)
    "causal_bf16_s72_d64": (torch.bfloat16, 1, 1, 1, 72, 72, 64, "causal", 0, None, 0),
    "causal_fp16_s40_d128": (torch.float16, 1, 1, 1, 40, 40, 128, "causal", 0, None, 0),
    "sliding24_softcap30_gqa_bf16": (torch.bfloat16, 1, 2, 1, 70, 70, 64, "sliding", 24, 30.0, 0),
    "decode_gqa_bf16_s100": (torch.bfloat16, 1, 4, 2, 1, 100, 64, None, 0, None, 0),
    "paged16_decode_gqa_bf16": (torch.bfloat16, 2, 4, 2, 1, 48, 64, None, 0, None, 16),
    "paged1_prefill_causal_bf16": (torch.bfloat16, 1, 2, 2, 40, 40, 64, "causal", 0, None, 1),
}


# extras per case: additive biases, softmax denominator sum + c, a second score product of depth d2
# with h2 key heads (scores (Q K^T + Q2 K2^T) (D + d2)^-0.5)
EXTRAS = {
    "biased_causal_bf16_s48": dict(case=(torch.bfloat16, 1, 2, 2, 48, 48, 64, "causal", 0, None, 0), score_bias=True, out_bias=True),
    "denom1_sliding16_fp16_s56": dict(case=(torch.float16, 1, 2, 1, 56, 56, 64, "sliding", 16, None, 0), denom_add=1.0),
    "two_part_d128_16_causal_bf16_s40": dict(case=(torch.bfloat16, 1, 2, 2, 40, 40, 128, "causal", 0, None, 0), d2=16, h2=1),
}
for _n, _e in EXTRAS.items():
    CASES[_n] = _e["case"]


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def build(name):
    dtype, B, Hq, Hkv, Sq, Sk, D, mask, window, softcap, page = CASES[name]
    g = torch.Generator().manual_seed(sum(name.encode()))
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32).to(dtype)
    q = rnd(B, Hq, Sq, D)
    out = {"q": bits(q), "dtype": np.array(0 if dtype == torch.bfloat16 else 1), "page": np.array(page),
           "mask": np.array({None: 0, "causal": 1, "sliding": 2}[mask]), "window": np.array(window),
           "softcap": np.array(softcap or 0.0, dtype=np.float32)}
    ex = EXTRAS.get(name, {})
    kw = {}
    if ex.get("score_bias"):
        kw["score_bias"] = rnd(B, Hq, Sq, Sk)
        out["score_bias"] = bits(kw["score_bias"])
    if ex.get("out_bias"):
        kw["out_bias"] = rnd(B, Hq, Sq, D)
        out["out_bias"] = bits(kw["out_bias"])
    if ex.get("denom_add"):
        kw["denom_add"] = ex["denom_add"]
        out["denom_add"] = np.array(ex["denom_add"], dtype=np.float32)
    if ex.get("d2"):
        kw["q2"], kw["k2"] = rnd(B, Hq, Sq, ex["d2"]), rnd(B, ex["h2"], Sk, ex["d2"])
        kw["scale"] = (D + ex["d2"]) ** -0.5
        out["q2"], out["k2"] = bits(kw["q2"]), bits(kw["k2"])
        out["scale"] = np.array(kw["scale"], dtype=np.float32)
    if page:
        n = B * Sk // page
        shape = (n, page, Hkv, D) if page > 1 else (n, Hkv, D)
        k, v = rnd(*shape), rnd(*shape)
        table = torch.randperm(n, generator=g).view(B, Sk // page).to(torch.int32)
        want = O.attention_reference(q, k, v, mask=mask, window=window, softcap=softcap, k_table=table, v_table=table)
        out["table"] = table.numpy()
    else:
        k, v = rnd(B, Hkv, Sk, D), rnd(B, Hkv, Sk, D)
        want = O.attention_reference(q, k, v, mask=mask, window=window, softcap=softcap, **kw)
    out.update({"k": bits(k), "v": bits(v), "expected": want.numpy().astype(np.float32)})
    return out


if __name__ == "__main__":
    # with arguments: only the named cases (stored archives carry a time stamp, so rewriting
    # an unchanged case would change its bytes)
    for name in (sys.argv[1:] or CASES):
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **build(name))
        print("wrote", name)
