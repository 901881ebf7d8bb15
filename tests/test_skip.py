"""Block-skip set: closed-form tile ranges == brute force over the dense mask, bit-exact."""
import dataclasses

import pytest
import torch

from loopfuse_amd import skip
from oracle import attention_oracle as O


@pytest.mark.parametrize("mask,window", [(None, 0), ("causal", 0), ("sliding", 1), ("sliding", 2), ("sliding", 63),
                                         ("sliding", 64), ("sliding", 65), ("sliding", 128), ("sliding", 129),
                                         ("sliding", 256), ("sliding", 1000), ("sliding", 5000)])
@pytest.mark.parametrize("Sq,Sk", [(1, 1), (64, 64), (127, 127), (128, 128), (129, 129), (593, 593), (2048, 2048),
                                   (300, 1000), (1000, 300), (2048, 2049)])
def test_tile_ranges_match_dense_mask(mask, window, Sq, Sk):
    bm, bn = skip.PREFILL_BM, skip.PREFILL_BN
    dense = O.visited_tiles_dense(mask, Sq, Sk, window, bm, bn)
    got = torch.zeros_like(dense)
    for qt, (b, e) in enumerate(skip.visited_tiles(mask, Sq, Sk, window)):
        got[qt, b:e] = True
    assert torch.equal(got, dense)


@pytest.mark.parametrize("bm,bn", [(32, 16), (16, 48), (7, 5)])
def test_other_tile_shapes(bm, bn):
    for mask, w in (("causal", 0), ("sliding", 9), ("sliding", 33)):
        dense = O.visited_tiles_dense(mask, 101, 97, w, bm, bn)
        got = torch.zeros_like(dense)
        for qt, (b, e) in enumerate(skip.visited_tiles(mask, 101, 97, w, bm, bn)):
            got[qt, b:e] = True
        assert torch.equal(got, dense)


def test_baseline_counts():
    # C2 (causal, S=2048): tiles of 128x64 -> sum_{qt} 2(qt+1) = 272 of 512
    assert sum(e - b for b, e in skip.visited_tiles("causal", 2048, 2048)) == 272
    # executed vs algorithmic flops for C2 = 272/256
    assert skip.executed_flops("causal", 8, 32, 2048, 2048, 128) * 256 == 2 * 8 * 32 * 2048 * 2048 * 128 * 272


def test_tuning_key_buckets_sizes():
    import torch
    from loopfuse_amd import lowering

    plan = lowering.AttnPlan(mask="causal", scale=0.1)
    mk = lambda B, H, S: torch.empty(B, H, S, 64, dtype=torch.bfloat16, device="meta")
    a = lowering._tune_key(mk(2, 4, 1000), mk(2, 4, 1000), plan, None, 0)
    b = lowering._tune_key(mk(2, 4, 1024), mk(2, 4, 1024), plan, None, 0)
    c = lowering._tune_key(mk(2, 4, 1025), mk(2, 4, 1025), plan, None, 0)
    assert a == b != c
    assert lowering._tune_key(mk(2, 8, 1000), mk(2, 4, 1000), plan, None, 0) != a       # GQA group differs


def test_mask_tensor_workloads_are_consistent():
    """Host side of the bench's mask-tensor workloads: the bias is 0 / -inf, every sequence keeps
    a visible key, and the byte count covers exactly the visible keys."""
    from loopfuse_amd import workloads
    w = workloads.make("c2_mask", seed=1, B=1, S=128)
    i = torch.arange(128)
    assert torch.equal(torch.isfinite(w.score_bias.float())[0, 0], i[None, :] <= i[:, None])
    assert w.mask is None and w.flops() == workloads.make("c2", seed=1, B=1, S=128).flops()
    for name in ("c5_padded", "cache4096"):
        w = workloads.make(name, seed=1, B=3, S=256)
        live = torch.isfinite(w.score_bias.float())
        assert w.score_bias.shape == (3, 1, 1, 256) and set(w.score_bias.float().unique().tolist()) <= {0.0, float("-inf")}
        assert live.any(dim=-1).all()
        assert w.visible_keys == int(live.sum())
        assert w.kv_bytes() == 2 * w.k.element_size() * w.kv_heads() * w.visible_keys * w.q.shape[-1]
        assert w.kv_bytes() < dataclasses.replace(w, visible_keys=None).kv_bytes()
