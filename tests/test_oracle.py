"""Pins the CPU oracle (oracle/attention_oracle.py) by what the mathematics fixes.

The reference holds no golden vectors for this path, so the checks are: a float64
pure-Python triple loop on tiny inputs, closed forms, invariants, and agreement of
the tiled online-softmax recurrence with the direct formula.
"""
import math

import pytest
import torch

from oracle import attention_oracle as O


def brute_force(q, k, v, mask, window, scale, softcap, score_bias=None, out_bias=None, denom_add=0.0):
    """float64 loops straight from the definition; no shared code with the oracle."""
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    g = Hq // Hkv
    out = [[[[0.0] * D for _ in range(Sq)] for _ in range(Hq)] for _ in range(B)]
    for b in range(B):
        for h in range(Hq):
            hk = h // g
            for i in range(Sq):
                sc = []
                for j in range(Sk):
                    keep = True
                    if mask == "causal":
                        keep = j <= i
                    elif mask == "sliding":
                        keep = (j <= i) and (i - j < window)
                    if not keep:
                        sc.append(None)
                        continue
                    dot = sum(float(q[b, h, i, d]) * float(k[b, hk, j, d]) for d in range(D)) * scale
                    if softcap is not None:
                        dot = softcap * math.tanh(dot / softcap)
                    if score_bias is not None:
                        dot += float(score_bias[b, h, i, j])
                    sc.append(dot)
                mx = max(x for x in sc if x is not None)
                w = [0.0 if x is None else math.exp(x - mx) for x in sc]
                tot = sum(w) + denom_add
                for d in range(D):
                    out[b][h][i][d] = sum(w[j] * float(v[b, hk, j, d]) for j in range(Sk)) / tot
                    if out_bias is not None:
                        out[b][h][i][d] += float(out_bias[b, h, i, d])
    return torch.tensor(out, dtype=torch.float64)


@pytest.mark.parametrize("mask,window", [(None, 0), ("causal", 0), ("sliding", 3)])
@pytest.mark.parametrize("softcap", [None, 2.5])
@pytest.mark.parametrize("hq,hkv", [(2, 2), (4, 2)])
def test_reference_matches_float64_loops(mask, window, softcap, hq, hkv):
    g = torch.Generator().manual_seed(7)
    B, S, D = 2, 9, 5
    q = torch.randn(B, hq, S, D, generator=g)
    k = torch.randn(B, hkv, S, D, generator=g)
    v = torch.randn(B, hkv, S, D, generator=g)
    scale = 0.7
    got = O.attention_reference(q, k, v, mask=mask, window=window, scale=scale, softcap=softcap)
    want = brute_force(q, k, v, mask, window, scale, softcap)
    assert torch.allclose(got.double(), want, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("mask", [None, "causal"])
@pytest.mark.parametrize("softcap", [None, 2.5])
def test_biases_match_float64_loops(mask, softcap):
    g = torch.Generator().manual_seed(11)
    B, H, S, D = 2, 2, 7, 4
    q, k, v = (torch.randn(B, H, S, D, generator=g) for _ in range(3))
    sb = torch.randn(B, H, S, S, generator=g)
    ob = torch.randn(B, H, S, D, generator=g)
    got = O.attention_reference(q, k, v, mask=mask, scale=0.6, softcap=softcap, score_bias=sb, out_bias=ob)
    want = brute_force(q, k, v, mask, 0, 0.6, softcap, sb, ob)
    assert torch.allclose(got.double(), want, atol=2e-6, rtol=1e-5)


def test_denominator_offset():
    g = torch.Generator().manual_seed(13)
    q, k, v = (torch.randn(1, 2, 6, 4, generator=g) for _ in range(3))
    got = O.attention_reference(q, k, v, mask="causal", scale=0.5, denom_add=1.0)
    want = brute_force(q, k, v, "causal", 0, 0.5, None, denom_add=1.0)
    assert torch.allclose(got.double(), want, atol=2e-6, rtol=1e-5)
    # row 0 sees one key: its probability is 1 / (1 + c)
    assert torch.allclose(got[:, :, 0], v[:, :, 0] / 2.0, atol=1e-6)
    # the offset is relative to the row maximum: shifting all scores of a row changes nothing
    shift = torch.randn(1, 2, 6, 1, generator=g).expand(1, 2, 6, 6)
    assert torch.allclose(O.attention_reference(q, k, v, mask="causal", scale=0.5, denom_add=1.0, score_bias=shift),
                          got, atol=1e-6)
    # c = 0 is the plain softmax; the output shrinks monotonically with c
    assert torch.equal(O.attention_reference(q, k, v, denom_add=0.0), O.attention_reference(q, k, v))
    plain = O.attention_reference(q, k, v, mask="causal", scale=0.5)
    l = torch.exp((q @ k.transpose(-2, -1) * 0.5).masked_fill(~O.dense_mask("causal", 6, 6), float("-inf")))
    l = (l / l.max(-1, keepdim=True).values).sum(-1, keepdim=True)
    assert torch.allclose(got, plain * l / (l + 1.0), atol=1e-6)


def test_two_part_scores():
    """(Q K^T + Q2 K2^T) * scale: float64 loops, the concatenation identity, shared K2 heads."""
    g = torch.Generator().manual_seed(17)
    B, H, S, D, D2 = 2, 4, 6, 4, 3
    q, k, v = (torch.randn(B, H, S, D, generator=g) for _ in range(3))
    q2 = torch.randn(B, H, S, D2, generator=g)
    k2 = torch.randn(B, 2, S, D2, generator=g)          # one K2 head per two query heads
    scale = (D + D2) ** -0.5
    got = O.attention_reference(q, k, v, mask="causal", scale=scale, q2=q2, k2=k2)
    want = [[[[0.0] * D for _ in range(S)] for _ in range(H)] for _ in range(B)]
    for b in range(B):
        for h in range(H):
            for i in range(S):
                sc = [(sum(float(q[b, h, i, d]) * float(k[b, h, j, d]) for d in range(D))
                       + sum(float(q2[b, h, i, d]) * float(k2[b, h // 2, j, d]) for d in range(D2))) * scale
                      for j in range(i + 1)]
                mx = max(sc)
                w = [math.exp(x - mx) for x in sc]
                for d in range(D):
                    want[b][h][i][d] = sum(w[j] * float(v[b, h, j, d]) for j in range(i + 1)) / sum(w)
    assert torch.allclose(got.double(), torch.tensor(want, dtype=torch.float64), atol=2e-6, rtol=1e-5)
    # [Q | Q2] [K | K2]^T = Q K^T + Q2 K2^T: one product over the concatenated depth
    k2r = k2.repeat_interleave(2, dim=1)
    s_cat = torch.cat([q, q2], -1) @ torch.cat([k, k2r], -1).transpose(-2, -1) * scale
    p = torch.softmax(s_cat.masked_fill(~O.dense_mask("causal", S, S), float("-inf")), -1)
    assert torch.allclose(got, p @ v, atol=1e-6)
    # a zero second part changes nothing; swapping the two parts' roles in the scores neither
    assert torch.equal(O.attention_reference(q, k, v, mask="causal", scale=scale, q2=torch.zeros_like(q2), k2=k2),
                       O.attention_reference(q, k, v, mask="causal", scale=scale))
    vv = torch.randn(B, H, S, D2, generator=g)
    a = O.attention_reference(q, k, vv, scale=scale, q2=q2, k2=k2r)
    b_ = O.attention_reference(q2, k2r, vv, scale=scale, q2=q, k2=k)
    assert torch.allclose(a, b_, atol=1e-6)


def test_bias_closed_forms():
    g = torch.Generator().manual_seed(12)
    q, k, v = (torch.randn(1, 2, 6, 8, generator=g) for _ in range(3))
    base = O.attention_reference(q, k, v, mask="causal")
    # a bias constant along the key axis cancels in the softmax
    row_const = torch.randn(1, 2, 6, 1, generator=g).expand(1, 2, 6, 6)
    assert torch.allclose(O.attention_reference(q, k, v, mask="causal", score_bias=row_const), base, atol=1e-6)
    # a -inf-like bias on every key but one selects that key's V row (the bias comes before the mask:
    # a masked key stays masked whatever its bias)
    pick = torch.full((1, 2, 6, 6), -1e4)
    pick[..., 0] = 0.0
    sel = O.attention_reference(q, k, v, mask="causal", score_bias=pick)
    assert torch.allclose(sel, v[:, :, :1].expand(1, 2, 6, 8), atol=1e-5)
    unmask = torch.zeros(1, 2, 6, 6)
    unmask[..., 5] = 1e4           # key 5 is masked for rows 0..4 under the causal mask
    got = O.attention_reference(q, k, v, mask="causal", score_bias=unmask)
    assert torch.allclose(got[:, :, :5], base[:, :, :5], atol=1e-6)
    # the output bias is a plain shift
    ob = torch.randn(1, 2, 6, 8, generator=g)
    assert torch.allclose(O.attention_reference(q, k, v, mask="causal", out_bias=ob), base + ob, atol=1e-6)


def test_default_scale_is_rsqrt_head_dim():
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(1, 1, 4, 16, generator=g) for _ in range(3))
    a = O.attention_reference(q, k, v)
    b = O.attention_reference(q, k, v, scale=0.25)
    assert torch.equal(a, b)


def test_closed_forms():
    g = torch.Generator().manual_seed(2)
    q = torch.randn(2, 3, 6, 8, generator=g)
    k = torch.randn(2, 3, 6, 8, generator=g)
    v = torch.randn(2, 3, 6, 8, generator=g)
    # causal row 0 sees only key 0 -> O[0] == V[0]
    o = O.attention_reference(q, k, v, mask="causal")
    assert torch.allclose(o[:, :, 0], v[:, :, 0], atol=1e-6)
    # window 1 keeps only the diagonal -> O == V
    o = O.attention_reference(q, k, v, mask="sliding", window=1)
    assert torch.allclose(o, v, atol=1e-6)
    # identical value rows -> output is that row whatever the scores
    vv = v[:, :, :1].expand(-1, -1, 6, -1)
    o = O.attention_reference(q, k, vv, mask="causal", softcap=3.0)
    assert torch.allclose(o, vv, atol=1e-6)
    # zero queries -> uniform weights -> causal running mean of V
    o = O.attention_reference(torch.zeros_like(q), k, v, mask="causal")
    want = torch.cumsum(v, dim=2) / torch.arange(1, 7).view(1, 1, 6, 1)
    assert torch.allclose(o, want, atol=1e-6)
    # very large cap == no cap; tiny cap bounds the logits so weights approach uniform
    a = O.attention_reference(q, k, v, softcap=1e6)
    b = O.attention_reference(q, k, v)
    assert torch.allclose(a, b, atol=1e-4)
    c = O.attention_reference(q, k, v, softcap=1e-4)
    assert torch.allclose(c, v.mean(dim=2, keepdim=True).expand_as(c), atol=1e-3)


def test_dense_mask_closed_forms():
    assert torch.equal(O.dense_mask("causal", 7, 7), torch.tril(torch.ones(7, 7, dtype=torch.bool)))
    m = O.dense_mask("sliding", 9, 9, 3)
    for i in range(9):
        for j in range(9):
            assert bool(m[i, j]) == (0 <= i - j <= 2)
    # window >= S degenerates to causal; non-square masks are top-left aligned
    assert torch.equal(O.dense_mask("sliding", 6, 6, 6), O.dense_mask("causal", 6, 6))
    assert torch.equal(O.dense_mask("causal", 3, 5), torch.tril(torch.ones(5, 5, dtype=torch.bool))[:3])
    assert O.dense_mask(None, 2, 3).all()


def test_paged_gather():
    g = torch.Generator().manual_seed(3)
    B, Hkv, S, D, P = 2, 3, 8, 4, 2
    dense = torch.randn(B, Hkv, S, D, generator=g)
    # identity table over a pool laid out from the dense tensor reproduces it
    pool = dense.transpose(1, 2).reshape(B * S // P, P, Hkv, D).contiguous()
    table = torch.arange(B * S // P).view(B, S // P)
    assert torch.equal(O.gather_paged(pool, table), dense)
    # a permuted pool with the matching table reproduces it too
    perm = torch.randperm(pool.shape[0], generator=g)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel())
    assert torch.equal(O.gather_paged(pool[perm], inv[table]), dense)
    # one-token pages (the reference's only format)
    pool1 = dense.transpose(1, 2).reshape(B * S, Hkv, D)
    assert torch.equal(O.gather_paged(pool1, torch.arange(B * S).view(B, S)), dense)
    q = torch.randn(B, 6, 1, D, generator=g)
    a = O.attention_reference(q, pool[perm], pool[perm], k_table=inv[table], v_table=inv[table])
    b = O.attention_reference(q, dense, dense)
    assert torch.allclose(a, b, atol=1e-6)


@pytest.mark.parametrize("mask,window", [(None, 0), ("causal", 0), ("sliding", 5), ("sliding", 40)])
@pytest.mark.parametrize("bm,bn", [(8, 4), (16, 16), (5, 7)])
def test_online_tiled_recurrence(mask, window, bm, bn):
    g = torch.Generator().manual_seed(4)
    q = torch.randn(1, 4, 37, 8, generator=g) * 2
    k = torch.randn(1, 2, 37, 8, generator=g) * 2
    v = torch.randn(1, 2, 37, 8, generator=g)
    want = O.attention_reference(q, k, v, mask=mask, window=window, softcap=4.0)
    got = O.online_tiled_reference(q, k, v, mask=mask, window=window, softcap=4.0, bm=bm, bn=bn)
    assert torch.allclose(got, want, atol=2e-6, rtol=1e-5)
    # restricting the walk to tiles with any unmasked score changes nothing
    vis = O.visited_tiles_dense(mask, 37, 37, window, bm, bn)
    ranges = []
    for row in vis:
        idx = row.nonzero().flatten()
        assert idx.numel() > 0 and int(idx[-1]) - int(idx[0]) + 1 == idx.numel()  # contiguous band
        ranges.append((int(idx[0]), int(idx[-1]) + 1))
    got2 = O.online_tiled_reference(q, k, v, mask=mask, window=window, softcap=4.0, bm=bm, bn=bn,
                                    tile_ranges=ranges)
    assert torch.allclose(got2, want, atol=2e-6, rtol=1e-5)


def test_decode_is_last_row_of_unmasked_prefill():
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, 4, 7, 8, generator=g)
    k = torch.randn(2, 4, 7, 8, generator=g)
    v = torch.randn(2, 4, 7, 8, generator=g)
    full = O.attention_reference(q, k, v, mask="causal")
    last = O.attention_reference(q[:, :, -1:], k, v)
    assert torch.allclose(full[:, :, -1:], last, atol=1e-6)


def test_eager_reference_graph_is_causal_attention():
    g = torch.Generator().manual_seed(6)
    q, k, v = (torch.randn(2, 2, 12, 8, generator=g) for _ in range(3))
    assert torch.allclose(O.eager_reference_graph(q, k, v), O.attention_reference(q, k, v, mask="causal"), atol=1e-6)
