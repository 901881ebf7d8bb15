"""GPU parity: HIP kernels (through the C-ABI shim) vs the CPU fp32 oracle on the
same seeded inputs.  Tolerances: max-abs <= 2e-2 for bf16,
<= 5e-3 for fp16.  Mirrors the reference's tests/test_accuracy.py cases (causal
S in {256, 593}, GQA, sliding window 256, paged K, paged GQA) plus the benchmark
configs.
"""
import pytest
import torch

from loopfuse_amd import lowering, skip, workloads
from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}


def dev():
    return torch.device("cuda:0")


def rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def check(q, k, v, *, mask=None, window=0, softcap=None, k_table=None, v_table=None, scale=None,
          score_bias=None, out_bias=None, denom_add=0.0, q2=None, k2=None, **kw):
    dtype = q.dtype
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    plan = lowering.AttnPlan(mask=mask, window=window, scale=scale, softcap=softcap,
                             k_paged=k_table is not None, v_paged=v_table is not None, denom_add=denom_add)
    mv = lambda t: None if t is None else t.to(dev())
    got = lowering.attention(mv(q), mv(k), mv(v), plan, mv(k_table), mv(v_table),
                             score_bias=mv(score_bias), out_bias=mv(out_bias), q2=mv(q2), k2=mv(k2), **kw)
    if isinstance(got, tuple):
        got = got[0]
    torch.cuda.synchronize()
    want = O.attention_reference(q, k, v, mask=mask, window=window, softcap=softcap, scale=scale,
                                 k_table=k_table, v_table=v_table, score_bias=score_bias, out_bias=out_bias,
                                 denom_add=denom_add, q2=q2, k2=k2)
    got = got.float().cpu()
    assert torch.isfinite(got).all()
    if out_bias is not None:
        # the bias moves the result away from O(1): add the storage format's half-ulp
        # (2^-8 relative for bf16, 2^-11 for fp16) of the expected value to the budget
        rel = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        excess = ((got - want).abs() - rel * want.abs()).max().item()
        assert excess <= TOL[dtype], f"max abs err beyond output rounding {excess} > {TOL[dtype]}"
        return excess
    err = (got - want).abs().max().item()
    assert err <= TOL[dtype], f"max abs err {err} > {TOL[dtype]}"
    return err


# ---------------------------------------------------------------- prefill
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("S", [256, 593])
@pytest.mark.parametrize("D", [64, 128])
def test_causal_prefill(dtype, S, D):
    q, k, v = (rand((2, 4, S, D), dtype, s) for s in (1, 2, 3))
    check(q, k, v, mask="causal")


@pytest.mark.parametrize("bn", [32, 64])
@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 128), (torch.float16, 128), (torch.bfloat16, 64)])
def test_prefill_tile_shapes(bn, dtype, D):
    """Both tile shapes of lf_attn_prefill_swp (32 keys per tile with three workgroups per CU, 64 with two)
    on every mask, with and without a cap, grouped heads packed and unpacked, page pools, ragged lengths."""
    c = {"bn": bn}
    for S in (65, 593):
        q, k, v = (rand((1, 4, S, D), dtype, s) for s in (1, 2, 3))
        for mask, window in ((None, 0), ("causal", 0), ("sliding", 100)):
            for cap in (None, 30.0):
                check(q, k, v, mask=mask, window=window, softcap=cap, choice=c, force_family="prefill")
                assert lowering.attention.last_launch["kv_tile_rows"] == bn
                assert lowering.attention.last_launch["kernels"] == ["lf_attn_prefill_swp"]
    q = rand((2, 8, 300, D), dtype, 4)
    k, v = (rand((2, 2, 450, D), dtype, s) for s in (5, 6))
    for pack in (True, False):
        check(q, k, v, mask="sliding", window=256, softcap=30.0, choice={**c, "pack": pack})
        assert lowering.attention.last_launch["kv_tile_rows"] == bn
    n, P = 2 * 29, 16                                      # page pool [N, P, Hkv, D], 464 tokens per sequence
    pool_k, pool_v = (rand((n, P, 2, D), dtype, s) for s in (7, 8))
    table = torch.randperm(n, generator=torch.Generator().manual_seed(9)).view(2, 29).to(torch.int32)
    check(q, pool_k, pool_v, mask="causal", k_table=table, v_table=table, choice=c)
    assert lowering.attention.last_launch["kv_tile_rows"] == bn


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("q_scale", [1.0, 4.0, 8.0, 20.0])
def test_softcap_forms(dtype, q_scale):
    """The cap is a fused polynomial while a tile's scores are small (|score * scale / cap| <= 0.15), a polynomial
    in place up to 0.4 and on tiles under a mask, and 1 - 2 / (e^2x + 1) beyond: larger queries move tiles from one
    form to the next, and rows mix them.  V is scaled down so that the peaked softmax of large scores stays
    within the storage format's rounding."""
    for mask, window, S in (("causal", 0, 700), ("sliding", 256, 700), (None, 0, 200)):
        q = (rand((1, 4, S, 128), torch.float32, 11) * q_scale).to(dtype)
        k = rand((1, 2, S, 128), dtype, 12)
        v = (rand((1, 2, S, 128), torch.float32, 13) * 0.25).to(dtype)
        for cap in (30.0, 5.0):
            for bn in (32, 64):
                check(q, k, v, mask=mask, window=window, softcap=cap, choice={"bn": bn}, force_family="prefill")


@pytest.mark.parametrize("D", [40, 80, 96, 120])
def test_other_head_dims_run_zero_padded(D):
    """Head dims other than 64 / 128 (up to 128, dense operands): the rows are zero-padded to the next kernel
    width, which changes neither Q K^T nor the kept columns of P V."""
    q = rand((2, 4, 300, D), torch.bfloat16, 1)
    k, v = (rand((2, 2, 300, D), torch.bfloat16, s) for s in (2, 3))
    check(q, k, v, mask="causal")
    check(q, k, v, mask="sliding", window=64, softcap=20.0)
    check(rand((2, 4, 1, D), torch.float16, 4), k.half(), v.half())          # decode shape
    out = torch.full((2, 4, 300, D), 7.0, dtype=torch.bfloat16, device=dev())
    got = lowering.attention(q.to(dev()), k.to(dev()), v.to(dev()), lowering.AttnPlan(mask="causal", scale=D ** -0.5), out=out)
    assert got is out and (out.float().cpu() - O.attention_reference(q, k, v, mask="causal")).abs().max().item() <= 2e-2
    pool = rand((40, 16, 2, D), torch.bfloat16, 5)
    table = torch.arange(40, dtype=torch.int32).view(2, 20)
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention(q.to(dev()), pool.to(dev()), pool.to(dev()), lowering.AttnPlan(scale=0.1, k_paged=True, v_paged=True),
                           table.to(dev()), table.to(dev()))


@pytest.mark.parametrize("v_tr", [True, False])
def test_causal_prefill_v_read_paths(v_tr):
    q, k, v = (rand((1, 2, 320, 128), torch.bfloat16, s) for s in (1, 2, 3))
    check(q, k, v, mask="causal", v_tr=v_tr)


@pytest.mark.parametrize("S", [1, 17, 64, 65, 128, 129])
def test_causal_prefill_edge_lengths(S):
    q, k, v = (rand((1, 3, S, 128), torch.bfloat16, s) for s in (4, 5, 6))
    check(q, k, v, mask="causal")


def test_unmasked_prefill_rectangular():
    q = rand((2, 4, 200, 128), torch.bfloat16, 1)
    k = rand((2, 4, 333, 128), torch.bfloat16, 2)
    v = rand((2, 4, 333, 128), torch.bfloat16, 3)
    check(q, k, v, force_family="prefill")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gqa_causal(dtype):
    q = rand((2, 8, 1024, 64), dtype, 1)
    k = rand((2, 4, 1024, 64), dtype, 2)
    v = rand((2, 4, 1024, 64), dtype, 3)
    check(q, k, v, mask="causal")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("window", [1, 100, 256, 4096])
def test_sliding_window(dtype, window):
    q, k, v = (rand((2, 4, 1024, 64), dtype, s) for s in (1, 2, 3))
    check(q, k, v, mask="sliding", window=window)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_softcap_causal(dtype):
    q, k, v = (rand((2, 4, 512, 128), dtype, s) for s in (1, 2, 3))
    check(q, k, v, mask="causal", softcap=30.0)
    check(q * 4, k * 4, v, mask="causal", softcap=5.0)


def test_c3_shape_small():
    w = workloads.make("c3", seed=3, B=1, S=1024)
    check(w.q, w.k, w.v, mask=w.mask, window=w.window, softcap=w.softcap)


def test_noncontiguous_inputs():
    # [B, S, H, D] storage viewed as [B, H, S, D]
    q, k, v = (rand((2, 300, 4, 128), torch.bfloat16, s).transpose(1, 2) for s in (1, 2, 3))
    check(q, k, v, mask="causal")


def test_paged_k_prefill():
    # reference tests/test_accuracy.py:253-278: K gathered token by token, V dense
    B, H, S, D = 2, 4, 512, 64
    pool = rand((B * S * 2, H, D), torch.bfloat16, 1)
    g = torch.Generator().manual_seed(9)
    table = torch.randint(0, B * S * 2, (B, S), generator=g, dtype=torch.int32)
    q = rand((B, H, S, D), torch.bfloat16, 2)
    v = rand((B, H, S, D), torch.bfloat16, 3)
    check(q, pool, v, mask="causal", k_table=table)


def test_paged_kv_prefill_page16_int64():
    B, H, S, D, P = 2, 2, 256, 128, 16
    n = B * S // P
    kp = rand((n, P, H, D), torch.bfloat16, 1)
    vp = rand((n, P, H, D), torch.bfloat16, 2)
    g = torch.Generator().manual_seed(9)
    table = torch.randperm(n, generator=g).view(B, S // P)
    q = rand((B, 2 * H, S, D), torch.bfloat16, 3)
    check(q, kp, vp, mask="causal", k_table=table, v_table=table)


# ---------------------------------------------------------------- additive biases
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("which", ["score", "out", "both"])
@pytest.mark.parametrize("S", [333, 336])
def test_biased_attention(dtype, which, S):
    # reference tests/test_accuracy.py:172-196 (scores * 3.5 + bias, causal, + output bias);
    # S = 333: bias rows start at odd offsets (element loads), S = 336: 8-byte loads
    B, H, D = 2, 4, 64
    q, k, v = (rand((B, H, S, D), dtype, s) for s in (1, 2, 3))
    sb = rand((B, H, S, S), dtype, 4) if which != "out" else None
    ob = rand((B, H, S, D), dtype, 5) if which != "score" else None
    check(q, k, v, mask="causal", scale=3.5 * D ** -0.5, score_bias=sb, out_bias=ob)


def test_biased_attention_broadcast_and_softcap_gqa():
    B, Hq, Hkv, S, D = 2, 8, 2, 200, 128
    q = rand((B, Hq, S, D), torch.bfloat16, 1)
    k, v = (rand((B, Hkv, S, D), torch.bfloat16, s) for s in (2, 3))
    sb = rand((1, 1, S, S), torch.bfloat16, 4)            # one bias shared by batch and heads
    ob = rand((1, Hq, 1, D), torch.bfloat16, 5)
    check(q, k, v, mask="sliding", window=64, softcap=20.0, score_bias=sb, out_bias=ob)
    check(q[:, :, :1], k, v, score_bias=sb[:, :, :1], out_bias=ob)      # a single query row, no mask


def test_biased_attention_paged_kv():
    B, H, S, D, P = 2, 2, 256, 128, 16
    n = B * S // P
    kp, vp = rand((n, P, H, D), torch.bfloat16, 1), rand((n, P, H, D), torch.bfloat16, 2)
    table = torch.randperm(n, generator=torch.Generator().manual_seed(9)).view(B, S // P).to(torch.int32)
    q = rand((B, H, S, D), torch.bfloat16, 3)
    sb = rand((B, H, S, S), torch.bfloat16, 4)
    check(q, kp, vp, mask="causal", k_table=table, v_table=table, score_bias=sb)


@pytest.mark.parametrize("copy", ["1", "0"])
def test_unaligned_bias_rows(copy, monkeypatch):
    # contiguous [.., 333, 333] bias: rows start at odd element offsets -> a copy with padded
    # rows (small tensors, the default) or element loads in the kernel
    monkeypatch.setenv("LOOPFUSE_BIAS_COPY", copy)
    B, H, S, D = 1, 2, 333, 64
    q, k, v = (rand((B, H, S, D), torch.bfloat16, s) for s in (1, 2, 3))
    sb = rand((B, H, S, S), torch.bfloat16, 4)
    ob = rand((B, H, S, D + 2), torch.bfloat16, 5)[..., 1:D + 1]
    check(q, k, v, mask="causal", score_bias=sb, out_bias=ob)


def test_bias_with_wrong_dtype_is_refused():
    q, k, v = (rand((1, 1, 64, 64), torch.bfloat16, s).to(dev()) for s in (1, 2, 3))
    sb = rand((1, 1, 64, 64), torch.float16, 4).to(dev())
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention(q, k, v, lowering.AttnPlan(mask="causal", scale=0.125), score_bias=sb)


# ---------------------------------------------------------------- shifted softmax denominator
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mask,S,c", [("causal", 593, 1.0), ("sliding", 300, 0.25), (None, 129, 3.0)])
def test_shifted_denominator(dtype, mask, S, c):
    # probabilities e^(s-m) / (sum e^(s-m) + c), reference tests/test_attention.py:95-125
    q, k, v = (rand((2, 4, S, 128), dtype, s) for s in (1, 2, 3))
    check(q, k, v, mask=mask, window=77, denom_add=c)
    check(q * 6, k, v, mask=mask, window=77, denom_add=c)          # sharp rows: the max dominates the sum


def test_shifted_denominator_single_row_and_gqa_paged():
    B, Hq, Hkv, S, D, P = 2, 8, 2, 256, 64, 16
    n = B * S // P
    kp, vp = rand((n, P, Hkv, D), torch.bfloat16, 1), rand((n, P, Hkv, D), torch.bfloat16, 2)
    table = torch.randperm(n, generator=torch.Generator().manual_seed(9)).view(B, S // P).to(torch.int32)
    check(rand((B, Hq, 1, D), torch.bfloat16, 3), kp, vp, k_table=table, v_table=table, denom_add=1.0)
    check(rand((B, Hq, S, D), torch.bfloat16, 3), kp, vp, mask="causal", k_table=table, v_table=table, denom_add=1.0)


# ---------------------------------------------------------------- paged prefill, direct-to-LDS loads
@pytest.mark.parametrize("D,P,S,i64,which", [(128, 16, 336, False, 3), (128, 32, 352, True, 3), (64, 16, 336, False, 3),
                                             (64, 8, 200, True, 3), (128, 16, 1040, False, 1), (128, 64, 448, False, 2)])
@pytest.mark.parametrize("mask,window", [("causal", 0), ("sliding", 90), (None, 0)])
def test_paged_prefill_direct_loads(D, P, S, i64, which, mask, window):
    """lf_attn_prefill_swp on page pools: page sizes 8..64, lengths that end inside a KV tile,
    int32 / int64 tables, K only / V only / both paged, GQA (packed heads) and not."""
    B, Hq, Hkv = 2, 8, 2
    n = B * S // P
    gen = torch.Generator().manual_seed(S + P)
    q = rand((B, Hq, S, D), torch.bfloat16, 1)
    table = torch.randperm(n, generator=gen).view(B, S // P).to(torch.int64 if i64 else torch.int32)
    pool = lambda seed: rand((n, P, Hkv, D), torch.bfloat16, seed)
    dense = lambda seed: O.gather_paged(pool(seed), table).contiguous()
    k, kt = (pool(2), table) if which & 1 else (dense(2), None)
    v, vt = (pool(3), table) if which & 2 else (dense(3), None)
    check(q, k, v, mask=mask, window=window, k_table=kt, v_table=vt)
    assert lowering.attention.last_launch["kernels"] == ["lf_attn_prefill_swp"]


def test_paged_prefill_falls_back_where_direct_loads_cannot_serve(monkeypatch):
    B, Hq, Hkv, S, D = 2, 4, 4, 256, 128
    q = rand((B, Hq, S, D), torch.bfloat16, 1)
    for P in (1, 4):                       # pages smaller than the rows of one wave-level load
        n = B * S // P
        table = torch.randperm(n, generator=torch.Generator().manual_seed(P)).view(B, S // P).to(torch.int32)
        shape = (n, P, Hkv, D) if P > 1 else (n, Hkv, D)
        check(q, rand(shape, torch.bfloat16, 2), rand(shape, torch.bfloat16, 3), mask="causal", k_table=table, v_table=table)
        assert lowering.attention.last_launch["kernels"] == ["lf_attn_prefill"]
    monkeypatch.setenv("LOOPFUSE_PAGED_SWP", "0")
    n = B * S // 16
    table = torch.randperm(n, generator=torch.Generator().manual_seed(3)).view(B, S // 16).to(torch.int32)
    check(q, rand((n, 16, Hkv, D), torch.bfloat16, 2), rand((n, 16, Hkv, D), torch.bfloat16, 3), mask="causal",
          k_table=table, v_table=table)
    assert lowering.attention.last_launch["kernels"] == ["lf_attn_prefill"]


# ---------------------------------------------------------------- empty inputs
def test_empty_inputs():
    dt, d = torch.bfloat16, dev()
    k, v = rand((2, 4, 64, 128), dt, 1).to(d), rand((2, 4, 64, 128), dt, 2).to(d)
    plan = lowering.AttnPlan(mask="causal", scale=0.1)
    # no query rows / no batch: an empty result and no launch
    o = lowering.attention(torch.empty((2, 4, 0, 128), dtype=dt, device=d), k, v, plan)
    assert o.shape == (2, 4, 0, 128) and lowering.attention.last_launch["kernels"] == []
    e = torch.empty((0, 4, 64, 128), dtype=dt, device=d)
    assert lowering.attention(e, e, e, plan).shape == (0, 4, 64, 128)
    # no keys: softmax over nothing is undefined, the lowering refuses (torch.compile then runs the graph as it is)
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention(rand((2, 4, 8, 128), dt, 3).to(d), k[:, :, :0], v[:, :, :0], lowering.AttnPlan(scale=0.1))


# ---------------------------------------------------------------- two-part scores
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D,D2,S", [(128, 16, 593), (128, 64, 300), (64, 32, 129), (64, 16, 1024)])
def test_two_part_scores(dtype, D, D2, S):
    # scores (Q K^T + Q2 K2^T) (D + D2)^-0.5, reference tests/test_attention.py:126-151
    q, k, v = (rand((2, 4, S, D), dtype, s) for s in (1, 2, 3))
    q2, k2 = rand((2, 4, S, D2), dtype, 4), rand((2, 4, S, D2), dtype, 5)
    check(q, k, v, mask="causal", scale=(D + D2) ** -0.5, q2=q2, k2=k2)
    # the second part alone decides: zero Q makes the first product vanish
    check(torch.zeros_like(q), k, v, mask="causal", scale=D2 ** -0.5, q2=q2, k2=k2)


def test_two_part_scores_shared_key_gqa_window_softcap_bias():
    B, Hq, Hkv, S, D, D2 = 2, 8, 2, 700, 128, 64
    q, k, v = rand((B, Hq, S, D), torch.bfloat16, 1), rand((B, Hkv, S, D), torch.bfloat16, 2), rand((B, Hkv, S, D), torch.bfloat16, 3)
    q2 = rand((B, Hq, S, D2), torch.bfloat16, 4)
    k2 = rand((B, 1, S, D2), torch.bfloat16, 5)             # one positional key shared by all heads
    sc = (D + D2) ** -0.5
    check(q, k, v, mask="sliding", window=200, softcap=20.0, scale=sc, q2=q2, k2=k2)
    check(q, k, v, scale=sc, q2=q2, k2=k2)                  # unmasked
    check(q, k, v, mask="causal", scale=sc, q2=q2, k2=k2, score_bias=rand((B, Hq, S, S), torch.bfloat16, 6),
          denom_add=1.0)
    # strided operands: Q2 / K2 as slices of wider tensors
    wide_q, wide_k = rand((B, Hq, S, D + D2), torch.bfloat16, 7), rand((B, Hkv, S, D + D2), torch.bfloat16, 8)
    got = lowering.attention(wide_q.to(dev())[..., :D], wide_k.to(dev())[..., :D], v.to(dev()),
                             lowering.AttnPlan(mask="causal", scale=sc),
                             q2=wide_q.to(dev())[..., D:], k2=wide_k.to(dev())[..., D:])
    want = O.attention_reference(wide_q[..., :D], wide_k[..., :D], v, mask="causal", scale=sc,
                                 q2=wide_q[..., D:], k2=wide_k[..., D:])
    assert (got.float().cpu() - want).abs().max().item() <= TOL[torch.bfloat16]


def test_two_part_scores_few_rows_and_paged_kv():
    B, Hq, Hkv, S, D, D2, P = 2, 4, 4, 256, 128, 64, 16
    n = B * S // P
    kp, vp = rand((n, P, Hkv, D), torch.bfloat16, 1), rand((n, P, Hkv, D), torch.bfloat16, 2)
    table = torch.randperm(n, generator=torch.Generator().manual_seed(9)).view(B, S // P).to(torch.int32)
    k2 = rand((B, Hkv, S, D2), torch.bfloat16, 5)
    sc = (D + D2) ** -0.5
    check(rand((B, Hq, S, D), torch.bfloat16, 3), kp, vp, mask="causal", k_table=table, v_table=table, scale=sc,
          q2=rand((B, Hq, S, D2), torch.bfloat16, 4), k2=k2)
    # a single query row without mask (decode shape) takes the same kernel
    k, v = rand((B, Hkv, S, D), torch.bfloat16, 6), rand((B, Hkv, S, D), torch.bfloat16, 7)
    check(rand((B, Hq, 1, D), torch.bfloat16, 3), k, v, scale=sc, q2=rand((B, Hq, 1, D2), torch.bfloat16, 4), k2=k2)


def test_two_part_scores_rejects_what_it_cannot_serve():
    q, k, v = (rand((1, 2, 64, 128), torch.bfloat16, s).to(dev()) for s in (1, 2, 3))
    plan = lowering.AttnPlan(mask="causal", scale=0.1)
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention(q, k, v, plan, q2=q[..., :24].contiguous(), k2=k[..., :24].contiguous())   # depth 24
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention(q, k, v, plan, q2=q[..., :16].contiguous())                                 # no k2
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention(q, k, v, plan, q2=q[..., :16].contiguous(), k2=k[:, :, :32, :16].contiguous())


# ---------------------------------------------------------------- block skip
@pytest.mark.parametrize("variant", ["w32", "swp"])
@pytest.mark.parametrize("mask,window,S", [("causal", 0, 593), ("sliding", 256, 2048), ("sliding", 100, 700),
                                           (None, 0, 300)])
def test_visited_tiles_bit_exact(mask, window, S, variant, monkeypatch):
    """The KV tiles each workgroup actually walks == tiles with any unmasked score."""
    monkeypatch.setenv("LOOPFUSE_PREFILL", variant)
    bm, bn = skip.TILE_SHAPES[lowering.prefill_variant(S)]
    q, k, v = (rand((1, 2, S, 128), torch.bfloat16, s).to(dev()) for s in (1, 2, 3))
    plan = lowering.AttnPlan(mask=mask, window=window, scale=128 ** -0.5)
    _, visits = lowering.attention(q, k, v, plan, record_visits=True, force_family="prefill")
    torch.cuda.synchronize()
    bn = lowering.attention.last_launch["kv_tile_rows"]      # 32 or 64 keys per tile, the launch's choice
    assert lowering.attention.last_launch["q_tile_rows"] == bm
    nqt = skip.cdiv(S, bm)
    visits = visits.cpu().view(2, nqt, -1).bool()
    dense = O.visited_tiles_dense(mask, S, S, window, bm, bn)
    for h in range(2):
        assert torch.equal(visits[h], dense)
    # and the host-side closed form agrees with both
    host = torch.zeros_like(dense)
    for qt, (b, e) in enumerate(skip.visited_tiles(mask, S, S, window, bm, bn)):
        host[qt, b:e] = True
    assert torch.equal(host, dense)


@pytest.mark.parametrize("g", [4, 2])
@pytest.mark.parametrize("mask,window,S", [("causal", 0, 593), ("sliding", 256, 2048), ("sliding", 100, 700), (None, 0, 300)])
def test_visited_tiles_bit_exact_with_packed_query_heads(mask, window, S, g):
    """Grouped-query attention: a workgroup takes 32 rows of 4 query heads (or 64 rows of 2) of
    one group; its walked KV tiles == tiles with any unmasked score for those rows."""
    bm, bn = skip.TILE_SHAPES["prefill_swp_pack" if g == 4 else "prefill_swp_pack2"]
    q = rand((2, 8, S, 128), torch.bfloat16, 1).to(dev())
    k, v = (rand((2, 8 // g, S, 128), torch.bfloat16, s).to(dev()) for s in (2, 3))
    plan = lowering.AttnPlan(mask=mask, window=window, scale=128 ** -0.5)
    out, visits = lowering.attention(q, k, v, plan, record_visits=True)
    torch.cuda.synchronize()
    assert lowering.attention.last_launch["heads_per_workgroup"] == g and lowering.attention.last_launch["q_tile_rows"] == bm
    bn = lowering.attention.last_launch["kv_tile_rows"]
    nqt = skip.cdiv(S, bm)
    visits = visits.cpu().view(2 * (8 // g), nqt, -1).bool()   # (batch x packs of g heads, q tile, kv tile)
    dense = O.visited_tiles_dense(mask, S, S, window, bm, bn)
    for u in range(2 * (8 // g)):
        assert torch.equal(visits[u], dense)
    want = O.attention_reference(q.cpu(), k.cpu(), v.cpu(), mask=mask, window=window)
    assert (out.float().cpu() - want).abs().max().item() <= TOL[torch.bfloat16]
    # and the unpacked walk gives the same numbers up to rounding
    ref = lowering.attention(q, k, v, plan, choice={"pack": False})
    assert (out.float() - ref.float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("variant", ["w32", "swp"])
@pytest.mark.parametrize("case", ["causal593", "sliding", "softcap_gqa", "rect", "tiny"])
def test_prefill_variants(variant, case, monkeypatch):
    """Both prefill kernels serve every shape class (the default picks by size)."""
    monkeypatch.setenv("LOOPFUSE_PREFILL", variant)
    dt = torch.bfloat16
    if case == "causal593":
        q, k, v = (rand((2, 4, 593, 128), dt, s) for s in (1, 2, 3))
        check(q, k, v, mask="causal")
    elif case == "sliding":
        q, k, v = (rand((1, 4, 1100, 64), torch.float16, s) for s in (1, 2, 3))
        check(q, k, v, mask="sliding", window=77)
    elif case == "softcap_gqa":
        q = rand((2, 8, 700, 128), dt, 1)
        k, v = (rand((2, 2, 700, 128), dt, s) for s in (2, 3))
        check(q, k, v, mask="causal", softcap=20.0)
    elif case == "rect":
        q = rand((1, 2, 300, 128), dt, 1)
        k, v = (rand((1, 2, 1000, 128), dt, s) for s in (2, 3))
        check(q, k, v, force_family="prefill")
    else:
        q, k, v = (rand((1, 1, 5, 64), dt, s) for s in (1, 2, 3))
        check(q, k, v, mask="causal")


# ---------------------------------------------------------------- decode
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Sk", [16, 100, 2048, 2049])
def test_decode_contiguous(dtype, Sk):
    q = rand((3, 8, 1, 128), dtype, 1)
    k = rand((3, 8, Sk, 128), dtype, 2)
    v = rand((3, 8, Sk, 128), dtype, 3)
    check(q, k, v)


@pytest.mark.parametrize("group", [2, 4, 8])
@pytest.mark.parametrize("D", [64, 128])
def test_decode_gqa(group, D):
    q = rand((2, 2 * group, 1, D), torch.bfloat16, 1)
    k = rand((2, 2, 777, D), torch.bfloat16, 2)
    v = rand((2, 2, 777, D), torch.bfloat16, 3)
    check(q, k, v)


def test_decode_rows_view():
    # the reference's GQA decode passes Q as [B, Hkv, group, D] (tests/benchmark.py:439-443)
    q = rand((2, 4, 4, 128), torch.bfloat16, 1)
    k = rand((2, 4, 1000, 128), torch.bfloat16, 2)
    v = rand((2, 4, 1000, 128), torch.bfloat16, 3)
    check(q, k, v)


@pytest.mark.parametrize("splits", [1, 2, 3, 8])
def test_decode_split_invariance(splits):
    q = rand((2, 8, 1, 128), torch.bfloat16, 1)
    k = rand((2, 2, 1500, 128), torch.bfloat16, 2)
    v = rand((2, 2, 1500, 128), torch.bfloat16, 3)
    check(q, k, v, num_splits=splits)


def test_decode_softcap():
    q = rand((2, 8, 1, 128), torch.bfloat16, 1) * 3
    k = rand((2, 2, 600, 128), torch.bfloat16, 2) * 3
    v = rand((2, 2, 600, 128), torch.bfloat16, 3)
    check(q, k, v, softcap=10.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_decode_paged_page16(dtype):
    w = workloads.make("c5", seed=1, dtype=dtype, B=4, S=512)
    check(w.q, w.k, w.v, k_table=w.k_table, v_table=w.v_table)


@pytest.mark.parametrize("pk,pv", [(16, 64), (32, 16), (1, 16), (16, 4)])
def test_mixed_page_sizes(pk, pv):
    """K and V pools with different page sizes and their own tables (decode and prefill)."""
    B, Hq, Hkv, S, D = 3, 8, 2, 320, 128
    gen = torch.Generator().manual_seed(pk * 100 + pv)
    nk, nv = B * S // pk, B * S // pv
    kp = rand((nk, pk, Hkv, D), torch.bfloat16, 1) if pk > 1 else rand((nk, Hkv, D), torch.bfloat16, 1)
    vp = rand((nv, pv, Hkv, D), torch.bfloat16, 2)
    kt = torch.randperm(nk, generator=gen).view(B, S // pk).to(torch.int32)
    vt = torch.randperm(nv, generator=gen).view(B, S // pv).to(torch.int32)
    check(rand((B, Hq, 1, D), torch.bfloat16, 3), kp, vp, k_table=kt, v_table=vt)
    check(rand((B, Hq, S, D), torch.bfloat16, 4), kp, vp, mask="causal", k_table=kt, v_table=vt)


def test_decode_head_major_pool_keeps_per_wave_loads():
    """A page pool whose storage is [pages, Hkv, page, D] (viewed as [pages, page, Hkv, D]): the cooperative
    block loads assume the heads of a token side by side, so even when one head per wave is asked for the
    launch must fall to the per-wave loads, which follow the head stride."""
    w = workloads.make("c5", seed=3, B=2, S=256)
    kp = w.k.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    vp = w.v.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    assert kp.stride(2) != kp.shape[3] and torch.equal(kp, w.k)
    check(w.q, kp, vp, k_table=w.k_table, v_table=w.v_table, choice={"head_per_wave": True, "splits": 2})
    assert lowering.attention.last_launch["head_per_wave"] and not lowering.attention.last_launch["cooperative_loads"]
    check(w.q, w.k, w.v, k_table=w.k_table, v_table=w.v_table, choice={"head_per_wave": True, "splits": 2})
    assert lowering.attention.last_launch["cooperative_loads"]


def test_decode_paged_identity_table_equals_contiguous(monkeypatch):
    w = workloads.make("c5", seed=2, B=2, S=256)
    n = w.k.shape[0]
    ident = torch.arange(n, dtype=torch.int32).view(2, -1)
    dense_k = O.gather_paged(w.k, ident).contiguous()
    dense_v = O.gather_paged(w.v, ident).contiguous()
    plan = lowering.AttnPlan(scale=w.scale, k_paged=True, v_paged=True)
    b = lowering.attention(w.q.to(dev()), dense_k.to(dev()), dense_v.to(dev()), lowering.AttnPlan(scale=w.scale))
    # same work split (4 waves share a head): the page table changes addresses only, so bit-equal
    monkeypatch.setenv("LOOPFUSE_DECODE_HEADWAVE", "0")
    a = lowering.attention(w.q.to(dev()), w.k.to(dev()), w.v.to(dev()), plan, ident.to(dev()), ident.to(dev()))
    torch.cuda.synchronize()
    assert torch.equal(a.cpu(), b.cpu())
    # one head per wave (the default for this pool layout) sums in another order
    monkeypatch.delenv("LOOPFUSE_DECODE_HEADWAVE")
    a2 = lowering.attention(w.q.to(dev()), w.k.to(dev()), w.v.to(dev()), plan, ident.to(dev()), ident.to(dev()))
    torch.cuda.synchronize()
    assert (a2.float() - b.float()).abs().max().item() <= 4e-3


def test_decode_paged_one_token_pages_int64():
    B, Hkv, S, D = 3, 2, 300, 64
    kp = rand((B * S * 2, Hkv, D), torch.bfloat16, 1)
    vp = rand((B * S * 2, Hkv, D), torch.bfloat16, 2)
    g = torch.Generator().manual_seed(9)
    kt = torch.randint(0, B * S * 2, (B, S), generator=g)
    vt = torch.randint(0, B * S * 2, (B, S), generator=g)
    q = rand((B, Hkv, 1, D), torch.bfloat16, 3)
    check(q, kp, vp, k_table=kt, v_table=vt)


@pytest.mark.parametrize("paged", [False, True])
def test_decode_long_context(paged):
    """K_len = 65536 with few (batch, head) units: the KV range is split 64 ways."""
    B, Hq, Hkv, S, D, P = 2, 8, 2, 65536, 128, 16
    q = rand((B, Hq, 1, D), torch.bfloat16, 1)
    if paged:
        n = B * S // P
        kp, vp = rand((n, P, Hkv, D), torch.bfloat16, 2), rand((n, P, Hkv, D), torch.bfloat16, 3)
        table = torch.randperm(n, generator=torch.Generator().manual_seed(4)).view(B, S // P).to(torch.int32)
        check(q, kp, vp, k_table=table, v_table=table)
    else:
        check(q, rand((B, Hkv, S, D), torch.bfloat16, 2), rand((B, Hkv, S, D), torch.bfloat16, 3))
    assert lowering.attention.last_launch["grid"][1] == 64


def test_decode_equals_last_prefill_row():
    q = rand((2, 4, 256, 128), torch.bfloat16, 1)
    k = rand((2, 4, 256, 128), torch.bfloat16, 2)
    v = rand((2, 4, 256, 128), torch.bfloat16, 3)
    plan_c = lowering.AttnPlan(mask="causal", scale=128 ** -0.5)
    plan_n = lowering.AttnPlan(scale=128 ** -0.5)
    full = lowering.attention(q.to(dev()), k.to(dev()), v.to(dev()), plan_c)
    last = lowering.attention(q[:, :, -1:].contiguous().to(dev()), k.to(dev()), v.to(dev()), plan_n)
    torch.cuda.synchronize()
    assert (full[:, :, -1:].float() - last.float()).abs().max().item() <= 1e-2


# ---------------------------------------------------------------- benchmark configs at full size
def _full_size_check(w):
    """Full-size run, EVERY output element against the oracle: ``O.attention_reference`` is plain
    torch, so it is evaluated here on the GPU in fp32, one (batch, kv head) unit at a time
    (scores of a unit: group x Sq x Sk floats), on the same tensors the kernel read."""
    wd = w.to(dev())
    got = workloads.run(wd)
    torch.cuda.synchronize()
    assert torch.isfinite(got.float()).all()
    B, Hq = w.q.shape[:2]
    Hkv = w.kv_heads()
    g = Hq // Hkv
    worst, where = 0.0, None
    for b in range(B):
        if w.k_table is not None:
            kb = O.gather_paged(wd.k, wd.k_table[b:b + 1])
            vb = O.gather_paged(wd.v, wd.v_table[b:b + 1])
        else:
            kb, vb = wd.k[b:b + 1], wd.v[b:b + 1]
        for hk in range(Hkv):
            want = O.attention_reference(wd.q[b:b + 1, hk * g:(hk + 1) * g], kb[:, hk:hk + 1], vb[:, hk:hk + 1],
                                         mask=w.mask, window=w.window, softcap=w.softcap)
            err = (got[b:b + 1, hk * g:(hk + 1) * g].float() - want).abs().max().item()
            if not err <= worst:        # also catches NaN
                worst, where = err, (b, hk)
    assert worst <= TOL[w.q.dtype], (worst, where)
    return got


@pytest.mark.parametrize("name", ["c2", "c2_softcap", "c3", "c4", "c5"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_baseline_config_full_size(name, dtype):
    w = workloads.make(name, seed=0, dtype=dtype)
    got = _full_size_check(w)
    # size-independent property: softmax weights are a convex combination, so every
    # output lies within the per-(batch, kv head) range of V
    if w.k_table is None:
        g = w.q.shape[1] // w.k.shape[1]
        vmax = w.v.float().amax(dim=2, keepdim=True).repeat_interleave(g, dim=1)
        vmin = w.v.float().amin(dim=2, keepdim=True).repeat_interleave(g, dim=1)
        o = got.float().cpu()
        assert (o <= vmax + 1e-2).all() and (o >= vmin - 1e-2).all()


@pytest.mark.parametrize("name", ["c2", "c3", "c5"])
def test_full_size_linearity_and_scaling_in_v(name):
    """Size-independent properties at the baseline sizes: the output is linear in V.
    att(2 V) == 2 att(V) bit for bit (a power of two commutes with every rounding), and
    att(V1) + att(V2) == att(V1 + V2) up to the bf16 rounding of the summed operand."""
    w = workloads.make(name, seed=3).to(dev())
    v1 = w.v
    v2 = torch.randn(v1.shape, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).to(dev())
    o1 = workloads.run(w).clone()
    w.v = v1 * 2
    assert torch.equal(workloads.run(w), o1 * 2)
    w.v = v2
    o2 = workloads.run(w).clone()
    w.v = (v1.float() + v2.float()).to(torch.bfloat16)
    o12 = workloads.run(w)
    torch.cuda.synchronize()
    want = o1.float() + o2.float()
    # three bf16 roundings are involved (o1, o2, o12): allow an ulp of the result's magnitude
    assert ((o12.float() - want).abs() - 2.0 ** -7 * want.abs()).max().item() <= 2e-2


@pytest.mark.parametrize("bn", [32, 64])
def test_full_size_causal_prefix_is_bit_equal(bn):
    """Causal attention over a prefix equals the first rows of causal attention over the
    whole sequence, bit for bit: a q tile walks the same KV tiles either way (for one tile
    shape: the default picks it by the size of the launch, so it is fixed here)."""
    w = workloads.make("c2", seed=5).to(dev())
    plan = lowering.AttnPlan(mask="causal", scale=w.scale)
    whole = lowering.attention(w.q, w.k, w.v, plan, choice={"bn": bn})
    for n in (1024, 593, 128):
        part = lowering.attention(w.q[:, :, :n], w.k[:, :, :n], w.v[:, :, :n], plan, choice={"bn": bn})
        torch.cuda.synchronize()
        assert torch.equal(part, whole[:, :, :n]), n


@pytest.mark.parametrize("variant", ["swp", "w32"])
def test_long_sequence_rows(variant, monkeypatch):
    """S = 32768 (byte offsets up to 2^23 rows x 256 B): sampled rows of the causal result
    against the oracle, row i being plain attention over keys 0..i."""
    monkeypatch.setenv("LOOPFUSE_PREFILL", variant)
    S, D = 32768, 128
    q, k, v = (rand((1, 2, S, D), torch.bfloat16, s) for s in (1, 2, 3))
    got = lowering.attention(q.to(dev()), k.to(dev()), v.to(dev()), lowering.AttnPlan(mask="causal", scale=D ** -0.5))
    torch.cuda.synchronize()
    got = got.float().cpu()
    for i in (0, 1, 127, 128, 12345, 20000, S - 1):
        want = O.attention_reference(q[:, :, i:i + 1], k[:, :, :i + 1], v[:, :, :i + 1])
        assert (got[:, :, i:i + 1] - want).abs().max().item() <= TOL[torch.bfloat16], i
    # window variant at the same length: only the last 300 keys of each row count
    got = lowering.attention(q.to(dev()), k.to(dev()), v.to(dev()),
                             lowering.AttnPlan(mask="sliding", window=300, scale=D ** -0.5)).float().cpu()
    for i in (5, 299, 300, 25000, S - 1):
        lo = max(0, i - 299)
        want = O.attention_reference(q[:, :, i:i + 1], k[:, :, lo:i + 1], v[:, :, lo:i + 1])
        assert (got[:, :, i:i + 1] - want).abs().max().item() <= TOL[torch.bfloat16], i


def test_c1_on_gpu_vs_cpu_eager():
    # config 1 (fp32, CPU-runnable): same tensors through the CPU eager graph and,
    # cast to bf16, through the GPU kernel
    w = workloads.make("c1", seed=0)
    want = O.eager_reference_graph(w.q, w.k, w.v)
    q, k, v = (t.to(torch.bfloat16) for t in (w.q, w.k, w.v))
    plan = lowering.AttnPlan(mask="causal", scale=w.scale)
    got = lowering.attention(q.to(dev()), k.to(dev()), v.to(dev()), plan)
    torch.cuda.synchronize()
    # inputs are rounded to bf16 for the kernel: compare against the oracle on the rounded inputs
    want_r = O.attention_reference(q, k, v, mask="causal")
    assert (got.float().cpu() - want_r).abs().max().item() <= 2e-2
    assert (got.float().cpu() - want).abs().max().item() <= 6e-2


# ---------------------------------------------------------------- seeded sweep
def _sweep_case(i):
    """Case i of a seeded sweep over shapes, masks, head groupings, paging and biases."""
    g = torch.Generator().manual_seed(1000 + i)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    pick = lambda xs: xs[ri(0, len(xs) - 1)]
    dtype = pick([torch.bfloat16, torch.float16])
    D = pick([64, 128])
    B = ri(1, 3)
    Hkv = pick([1, 2, 3, 8])
    group = pick([1, 1, 2, 4])
    kind = pick(["prefill", "prefill", "decode", "rect"])
    if kind == "prefill":
        Sq = Sk = ri(1, 700)
        mask = pick([None, "causal", "causal", "sliding"])
    elif kind == "rect":
        Sq, Sk = ri(1, 300), ri(1, 900)
        mask = pick([None, "causal", "sliding"])
    else:
        Sq, Sk = 1, ri(16, 3000)
        mask = None
    window = ri(1, 400) if mask == "sliding" else 0
    softcap = pick([None, None, 15.0, 50.0])
    paged = pick([0, 0, 1, 3]) if kind != "rect" else 0
    page = pick([1, 16, 32]) if paged else 1
    bias = pick([0, 0, 0, 1, 2, 3]) if kind != "decode" else 0
    return dict(dtype=dtype, D=D, B=B, Hkv=Hkv, group=group, Sq=Sq, Sk=Sk, mask=mask, window=window,
                softcap=softcap, paged=paged, page=page, bias=bias, seed=2000 + i)


@pytest.mark.parametrize("i", range(40))
def test_seeded_sweep(i):
    c = _sweep_case(i)
    dt, D, B, Hkv, Sq, Sk = c["dtype"], c["D"], c["B"], c["Hkv"], c["Sq"], c["Sk"]
    Hq = Hkv * c["group"]
    if c["mask"] is not None and Sq > Sk:
        Sq = Sk             # keep every query row with at least one visible key
    q = rand((B, Hq, Sq, D), dt, c["seed"])
    kt = vt = None
    if c["paged"]:
        P = c["page"]
        Skp = (Sk + P - 1) // P * P
        Sk = Skp
        if c["mask"] is not None:
            Sq = min(Sq, Sk)
            q = q[:, :, :Sq].contiguous()
        n = B * Skp // P * 2
        pool_shape = (n, Hkv, D) if P == 1 else (n, P, Hkv, D)
        gen = torch.Generator().manual_seed(c["seed"] + 7)
        k = rand(pool_shape, dt, c["seed"] + 1)
        kt = torch.randint(0, n, (B, Skp // P), generator=gen, dtype=torch.int32 if c["seed"] % 2 else torch.int64)
        if c["paged"] & 2:
            v = rand(pool_shape, dt, c["seed"] + 2)
            vt = torch.randint(0, n, (B, Skp // P), generator=gen, dtype=kt.dtype)
        else:
            v = rand((B, Hkv, Sk, D), dt, c["seed"] + 2)
    else:
        k = rand((B, Hkv, Sk, D), dt, c["seed"] + 1)
        v = rand((B, Hkv, Sk, D), dt, c["seed"] + 2)
    sb = rand((B, Hq, Sq, Sk), dt, c["seed"] + 3) if c["bias"] & 1 else None
    ob = rand((B, Hq, Sq, D), dt, c["seed"] + 4) if c["bias"] & 2 else None
    print("sweep case", i, {**c, "Sq": Sq, "Sk": Sk}, flush=True)
    check(q, k, v, mask=c["mask"], window=c["window"], softcap=c["softcap"], k_table=kt, v_table=vt,
          score_bias=sb, out_bias=ob)


# ---------------------------------------------------------------- measured launch heuristics
@pytest.mark.parametrize("name", ["c2", "c5"])
def test_tuned_attention_matches_and_remembers(name, monkeypatch, tmp_path):
    monkeypatch.setattr(lowering, "_TUNE_FILE", str(tmp_path / "autotune.json"))
    monkeypatch.setattr(lowering, "_tuned", {})
    w = workloads.make(name, seed=5, B=2, S=512)
    plan = lowering.AttnPlan(mask=w.mask, window=w.window, scale=w.scale, softcap=w.softcap,
                             k_paged=w.k_table is not None, v_paged=w.v_table is not None)
    mv = lambda t: None if t is None else t.to(dev())
    args = (mv(w.q), mv(w.k), mv(w.v), plan, mv(w.k_table), mv(w.v_table))
    got = lowering.tuned_attention(*args)
    assert len(lowering._tuned) == 1
    key, choice = next(iter(lowering._tuned.items()))
    again = lowering.tuned_attention(*args)            # no second search
    assert len(lowering._tuned) == 1 and torch.equal(got, again)
    import json
    assert json.load(open(lowering._TUNE_FILE)) == {key: choice}
    want = O.attention_reference(w.q, w.k, w.v, mask=w.mask, k_table=w.k_table, v_table=w.v_table)
    assert (got.float().cpu() - want).abs().max().item() <= TOL[torch.bfloat16]


# ---------------------------------------------------------------- HIP graph capture
@pytest.mark.parametrize("name", ["c5", "c2"])
def test_launches_can_be_captured_in_a_hip_graph(name):
    """A serving loop captures the decode step once and replays it: the launches go to
    the capturing stream, allocate nothing during capture (output and split scratch
    exist beforehand) and read their inputs by address, so refreshed inputs are seen.
    Every replay is checked against the eager launch, with eager work in between."""
    w = workloads.make(name, seed=11, B=2, S=512).to(dev())
    plan = lowering.AttnPlan(mask=w.mask, window=w.window, scale=w.scale, softcap=w.softcap,
                             k_paged=w.k_table is not None, v_paged=w.v_table is not None)
    q = w.q.clone()
    out = lowering.attention(q, w.k, w.v, plan, w.k_table, w.v_table)      # warm: code objects, scratch
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        lowering.attention(q, w.k, w.v, plan, w.k_table, w.v_table, out=out)
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            lowering.attention(q, w.k, w.v, plan, w.k_table, w.v_table, out=out)
    for rep in range(3):
        q.copy_(rand(tuple(q.shape), torch.bfloat16, 100 + rep).to(dev()))
        want = lowering.attention(q, w.k, w.v, plan, w.k_table, w.v_table).clone()    # eager, other buffer
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {rep} differs from the eager launch"


def test_page_ids_outside_the_pool_are_reported_when_asked(monkeypatch):
    """LOOPFUSE_CHECK_TABLES=1 validates page ids on the host before anything is launched."""
    monkeypatch.setenv("LOOPFUSE_CHECK_TABLES", "1")
    w = workloads.make("c5", seed=0, B=2, S=256).to(dev())
    plan = lowering.AttnPlan(scale=w.scale, k_paged=True, v_paged=True)
    good = lowering.attention(w.q, w.k, w.v, plan, w.k_table, w.v_table)
    bad = w.k_table.clone()
    bad[1, 3] = w.k.shape[0]
    with pytest.raises(ValueError, match="page table holds ids"):
        lowering.attention(w.q, w.k, w.v, plan, bad, w.v_table)
    bad[1, 3] = -1
    with pytest.raises(ValueError, match="page table holds ids"):
        lowering.attention(w.q, w.k, w.v, plan, w.k_table, bad)
    assert torch.equal(good, lowering.attention(w.q, w.k, w.v, plan, w.k_table, w.v_table))


def test_operands_on_another_device_are_refused():
    """Every operand must live where Q lives; nothing is launched otherwise."""
    w = workloads.make("c5", seed=0, B=2, S=256).to(dev())
    plan = lowering.AttnPlan(scale=w.scale, k_paged=True, v_paged=True)
    with pytest.raises(RuntimeError, match="K page table is on cpu"):
        lowering.attention(w.q, w.k, w.v, plan, w.k_table.cpu(), w.v_table)
    q, k, v = (rand((1, 2, 64, 64), torch.bfloat16, s).to(dev()) for s in (1, 2, 3))
    with pytest.raises(RuntimeError, match="score bias is on cpu"):
        lowering.attention(q, k, v, lowering.AttnPlan(scale=0.125), score_bias=rand((1, 2, 64, 64), torch.bfloat16, 4))
    with pytest.raises(RuntimeError, match="not on the GPU"):
        lowering.attention(q, k.cpu(), v, lowering.AttnPlan(scale=0.125))


def _mask_bias(kind, Sq, Sk, dtype, seed=0):
    """Additive masks as a caller would pass them: 0 where a key is visible, -inf elsewhere."""
    i = torch.arange(Sq)[:, None]
    j = torch.arange(Sk)[None, :]
    if kind == "causal":
        keep = j <= i
    elif kind == "window":
        keep = (j <= i) & (i - j < 100)
    elif kind == "documents":            # block-diagonal: three documents packed into one sequence
        edges = torch.tensor([0, Sk // 3, Sk // 2, Sk])
        doc = lambda t: torch.bucketize(t, edges[1:-1], right=True)
        keep = (doc(i) == doc(j)) & (j <= i)
    elif kind == "padding":              # the last keys are padding; a finite bias elsewhere
        keep = (j < Sk - 200).expand(Sq, Sk)
    else:
        raise ValueError(kind)
    m = torch.zeros(Sq, Sk).masked_fill(~keep, float("-inf"))
    if kind == "padding":
        m = m + torch.randn(Sq, Sk, generator=torch.Generator().manual_seed(seed)) * keep
    return m.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ["causal", "window", "documents", "padding"])
@pytest.mark.parametrize("S,D", [(593, 64), (1300, 128)])
def test_mask_tensors_skip_dead_tiles_without_changing_the_result(dtype, kind, S, D, monkeypatch):
    """Mask tensors are biases of 0 / -inf; KV tiles that are -inf for a whole q tile are left
    out of the loop.  Both kernels that serve them -- the direct-to-LDS kernel on classified tiles
    (default) and the register-staged one with its list of live tiles -- must equal the oracle, and
    the latter, bit for bit, the result of the same kernel walking every tile."""
    q, k, v = (rand((2, 3, S, D), dtype, s) for s in (1, 2, 3))
    bias = _mask_bias(kind, S, S, dtype)[None, None].expand(2, 1, S, S).contiguous()
    plan = lowering.AttnPlan(scale=D ** -0.5)
    on = [t.to(dev()) for t in (q, k, v, bias)]
    want = O.attention_reference(q, k, v, score_bias=bias.float())
    got = lowering.attention(*on[:3], plan, score_bias=on[3])
    assert lowering.attention.last_launch["kernels"] == ["lf_bias_classify", "lf_attn_prefill_swp"]
    assert (got.float().cpu() - want).abs().max().item() <= TOL[dtype]
    monkeypatch.setenv("LOOPFUSE_BIAS_TILES", "0")
    staged = lowering.attention(*on[:3], plan, score_bias=on[3])
    assert lowering.attention.last_launch["kernels"] == ["lf_attn_prefill"]
    assert (staged.float().cpu() - want).abs().max().item() <= TOL[dtype]
    monkeypatch.setenv("LOOPFUSE_KOPTS", "-DLF_LIVE_LIST=0")
    every_tile = lowering.attention(*on[:3], plan, score_bias=on[3])
    assert torch.equal(staged, every_tile)


def test_mask_tensor_with_rows_that_see_nothing():
    """Rows whose keys are all masked come out as NaN, as softmax of all -inf does; the
    other rows are unaffected (a q tile may have no live KV tile at all)."""
    S, D = 400, 64
    q, k, v = (rand((1, 2, S, D), torch.bfloat16, s) for s in (1, 2, 3))
    bias = _mask_bias("causal", S, S, torch.bfloat16).clone()
    bias[128:256] = float("-inf")          # one whole q tile
    bias[300] = float("-inf")              # one row of another
    bias = bias[None, None]
    got = lowering.attention(*[t.to(dev()) for t in (q, k, v)], lowering.AttnPlan(scale=D ** -0.5),
                             score_bias=bias.to(dev())).float().cpu()
    want = O.attention_reference(q, k, v, score_bias=bias.float())
    blind = torch.zeros(S, dtype=torch.bool)
    blind[128:256] = True
    blind[300] = True
    assert torch.isnan(want[:, :, blind]).all() and torch.isnan(got[:, :, blind]).all()
    assert (got[:, :, ~blind] - want[:, :, ~blind]).abs().max().item() <= TOL[torch.bfloat16]


@pytest.mark.parametrize("Sk", [200_000, 270_000])
def test_mask_tensor_over_a_long_key_range(Sk):
    """Dead-tile list over many 64-bit words (3125 KV tiles) and, past 4096 tiles, the
    walk over every tile: live keys are scattered islands, the rest is masked."""
    Sq, D = 128, 64
    q, k, v = rand((1, 2, Sq, D), torch.bfloat16, 1), rand((1, 1, Sk, D), torch.bfloat16, 2), rand((1, 1, Sk, D), torch.bfloat16, 3)
    bias = torch.full((Sq, Sk), float("-inf"))
    for start in (0, 4096 + 17, 64 * 1000, 64 * 2047 + 5, Sk - 300):      # islands, some across tile and word borders
        bias[:, start:start + 150] = 0.0
    bias[5, 64 * 3000:64 * 3000 + 3] = 0.5                                # one row keeps a far tile alive
    bias = bias.to(torch.bfloat16)[None, None]
    got = lowering.attention(*[t.to(dev()) for t in (q, k, v)], lowering.AttnPlan(scale=D ** -0.5),
                             score_bias=bias.to(dev())).float().cpu()
    want = O.attention_reference(q, k, v, score_bias=bias.float())
    assert (got - want).abs().max().item() <= TOL[torch.bfloat16]


def test_mask_tensor_over_an_odd_number_of_keys():
    """Rows of a [.., 593, 593] mask do not start on 8-byte borders: the launcher pads them
    in a copy, and the dead-tile list applies as for aligned masks."""
    S, D = 593, 128
    q, k, v = (rand((2, 2, S, D), torch.bfloat16, s) for s in (1, 2, 3))
    bias = _mask_bias("window", S, S, torch.bfloat16)[None, None]
    on = [t.to(dev()) for t in (q, k, v, bias)]
    got = lowering.attention(*on[:3], lowering.AttnPlan(scale=D ** -0.5), score_bias=on[3])
    want = O.attention_reference(q, k, v, score_bias=bias.float())
    assert (got.float().cpu() - want).abs().max().item() <= TOL[torch.bfloat16]
    flagged = lowering.attention(*on[:3], lowering.AttnPlan(mask="sliding", window=100, scale=D ** -0.5))
    assert (got.float() - flagged.float()).abs().max().item() <= 2 ** -6


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", ["gqa_left_padding", "per_head_bias_softcap", "rows_view", "paged_page16", "paged_one_token",
                                  "paged_head_per_wave"])
def test_decode_with_score_bias(dtype, case):
    """Decode shapes with an additive score bias (mask tensors of batched generation: left
    padding; per-head biases) stay on the streaming decode kernel."""
    g = torch.Generator().manual_seed(11)
    B, Hkv, group, D, Sk, Sq = 3, 2, 4, 128, 1000, 1
    softcap = None
    kw = {}
    if case == "rows_view":
        group, Sq, Sk, D = 1, 5, 333, 64
    if case == "paged_head_per_wave":
        Hkv, B = 8, 2
        kw["choice"] = {"head_per_wave": True, "splits": 2}
    Hq = Hkv * group
    q = rand((B, Hq, Sq, D), dtype, 1)
    k, v = rand((B, Hkv, Sk, D), dtype, 2), rand((B, Hkv, Sk, D), dtype, 3)
    if case == "gqa_left_padding":
        pad = torch.tensor([0, 700, 37])            # batch 1 has its first splits fully masked
        bias = torch.zeros(B, 1, 1, Sk).masked_fill(torch.arange(Sk)[None, None, None, :] < pad[:, None, None, None], float("-inf"))
        kw["num_splits"] = 4
    elif case == "per_head_bias_softcap":
        bias, softcap = torch.randn(1, Hq, 1, Sk, generator=g), 20.0
    elif case == "rows_view":
        bias = torch.randn(B, Hq, Sq, Sk + 3, generator=g)[..., :Sk]       # row stride Sk + 3 = 336: aligned rows
    else:
        bias = torch.randn(B, 1, 1, Sk, generator=g).masked_fill(torch.rand(B, 1, 1, Sk, generator=g) < 0.2, float("-inf"))
    bias = bias.to(dtype)
    k_in, v_in, kt, vt = k, v, None, None
    if case.startswith("paged"):
        P = 1 if case == "paged_one_token" else 16
        Skp = (Sk + P - 1) // P * P
        n = B * Skp // P
        perm = torch.randperm(n, generator=g)
        table = perm.view(B, Skp // P).to(torch.int32)
        pool_k = torch.zeros(n, P, Hkv, D, dtype=dtype)
        pool_v = torch.zeros(n, P, Hkv, D, dtype=dtype)
        kp = torch.nn.functional.pad(k, (0, 0, 0, Skp - Sk)).transpose(1, 2).reshape(B, Skp // P, P, Hkv, D)
        vp = torch.nn.functional.pad(v, (0, 0, 0, Skp - Sk)).transpose(1, 2).reshape(B, Skp // P, P, Hkv, D)
        pool_k[table.long()] = kp
        pool_v[table.long()] = vp
        if P == 1:
            pool_k, pool_v = pool_k[:, 0], pool_v[:, 0]
        k_in, v_in, kt, vt = pool_k, pool_v, table, table.clone()
        if Skp != Sk:      # the padded keys exist in the pool: mask them
            bias = torch.nn.functional.pad(bias, (0, Skp - Sk), value=float("-inf"))
            k = torch.nn.functional.pad(k, (0, 0, 0, Skp - Sk))
            v = torch.nn.functional.pad(v, (0, 0, 0, Skp - Sk))
    plan = lowering.AttnPlan(scale=D ** -0.5, softcap=softcap, k_paged=kt is not None, v_paged=vt is not None)
    on = lambda t: None if t is None else t.to(dev())
    got = lowering.attention(on(q), on(k_in), on(v_in), plan, on(kt), on(vt), score_bias=on(bias), **kw)
    assert lowering.attention.last_launch["kernels"][0] == "lf_attn_decode"
    assert lowering.attention.last_launch["head_per_wave"] == (case == "paged_head_per_wave")
    want = O.attention_reference(q, k, v, softcap=softcap, score_bias=bias.float())
    assert (got.float().cpu() - want).abs().max().item() <= TOL[dtype]
    if case == "gqa_left_padding":
        one = lowering.attention(on(q), on(k_in), on(v_in), plan, score_bias=on(bias), num_splits=1)
        assert (got.float() - one.float()).abs().max().item() <= 2 ** -7


@pytest.mark.parametrize("shape", ["prefill", "decode", "decode_split"])
def test_rows_that_see_nothing_give_zeros_when_asked(shape):
    """AttnPlan.zero_blind_rows (what torch's fused attention ops do, and what the front end
    sets for them): zeros instead of NaN for rows whose keys are all masked; other rows unchanged."""
    D = 64
    if shape == "prefill":
        B, H, Sq, Sk = 1, 2, 400, 400
        bias = _mask_bias("causal", Sq, Sk, torch.bfloat16).clone()
        bias[128:256] = float("-inf")
        bias[300] = float("-inf")
        bias = bias[None, None]
        blind = torch.isinf(bias[0, 0]).all(-1)[None, None].expand(B, H, Sq)
        kw = {}
    else:
        B, H, Sq, Sk = 3, 4, 1, 1200
        bias = torch.zeros(B, 1, 1, Sk)
        bias[1] = float("-inf")                     # one sequence of the batch sees nothing
        bias[2, ..., :900] = float("-inf")
        bias = bias.to(torch.bfloat16)
        blind = torch.zeros(B, H, Sq, dtype=torch.bool)
        blind[1] = True
        kw = {"num_splits": 4 if shape == "decode_split" else 1}
    q, k, v = rand((B, H, Sq, D), torch.bfloat16, 1), rand((B, H, Sk, D), torch.bfloat16, 2), rand((B, H, Sk, D), torch.bfloat16, 3)
    on = [t.to(dev()) for t in (q, k, v, bias)]
    want = O.attention_reference(q, k, v, score_bias=bias.float())
    assert torch.isnan(want[blind]).all()
    for zero in (False, True):
        got = lowering.attention(*on[:3], lowering.AttnPlan(scale=D ** -0.5, zero_blind_rows=zero), score_bias=on[3], **kw).float().cpu()
        assert lowering.attention.last_launch["kernels"] == (["lf_bias_classify", "lf_attn_prefill_swp"] if shape == "prefill"
                                                            else ["lf_attn_decode"] + ["lf_attn_decode_combine"] * (shape == "decode_split"))
        assert (got[blind] == 0).all() if zero else torch.isnan(got[blind]).all()
        assert (got[~blind] - want[~blind]).abs().max().item() <= TOL[torch.bfloat16]


@pytest.mark.parametrize("i", range(14))
def test_bias_tile_classes(i, monkeypatch):
    """The direct-to-LDS kernel with the bias classified tile by tile (lf_bias_classify): the tiles
    it walks are each q tile's first .. last block that is not all -inf (brute force over the bias),
    and its output equals the oracle's and the register-staged bias kernel's.  Leading, trailing and
    interior dead blocks, zero blocks, blocks of real values, lengths that are no multiple of 4, 64 or
    128, every broadcast form, rows that see nothing."""
    g = torch.Generator().manual_seed(7000 + i)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    pick = lambda xs: xs[ri(0, len(xs) - 1)]
    dt, D = pick([torch.bfloat16, torch.float16]), pick([64, 128])
    B, H = ri(1, 2), pick([1, 3])
    Sq, Sk = pick([17, 100, 128, 129, 300, 515]), pick([4, 63, 64, 65, 130, 333, 700, 1101])    # (up to 16 rows: decode kernels)
    bshape = [pick([1, B]), pick([1, H]), pick([1, Sq, Sq]), Sk]
    bias = torch.randn(bshape, generator=g) * 0.5 if pick([False, True]) else torch.zeros(bshape)
    bias[..., :ri(0, Sk // 2)] = float("-inf")                       # leading dead keys
    bias[..., Sk - ri(0, Sk // 3):] = float("-inf")                  # trailing dead keys
    for _ in range(ri(0, 4)):                                        # holes, some wider than a tile
        c0 = ri(0, Sk - 1)
        r0 = ri(0, bshape[2] - 1)
        bias[..., r0:r0 + ri(1, 300), c0:c0 + ri(1, 300)] = float("-inf")
    if pick([False, True]) and Sk > 200:
        bias[..., 100:164] = 0.0                                      # a whole zero tile
    bias = bias.to(dt)
    q, k, v = rand((B, H, Sq, D), dt, 7100 + i), rand((B, H, Sk, D), dt, 7200 + i), rand((B, H, Sk, D), dt, 7300 + i)
    cap = pick([None, None, 5.0, 30.0])
    print("bias tile case", i, dict(dt=dt, D=D, B=B, H=H, Sq=Sq, Sk=Sk, bshape=bshape, softcap=cap), flush=True)
    on = [t.to(dev()) for t in (q, k, v, bias)]
    plan = lowering.AttnPlan(scale=D ** -0.5, softcap=cap)
    got, visits = lowering.attention(*on[:3], plan, score_bias=on[3], record_visits=True)
    assert lowering.attention.last_launch["kernels"] == ["lf_bias_classify", "lf_attn_prefill_swp"]
    # walked tiles against brute force
    nqt, nkt = (Sq + 127) // 128, (Sk + 63) // 64
    full = bias.float().expand(B, H, Sq, Sk)
    want_vis = torch.zeros(B * H * nqt, nkt, dtype=torch.uint8)
    for bh in range(B * H):
        for qt in range(nqt):
            blk = full[bh // H, bh % H, 128 * qt:128 * qt + 128]
            live = [kt for kt in range(nkt) if not torch.isinf(blk[:, 64 * kt:64 * kt + 64]).all()]
            if live:
                want_vis[bh * nqt + qt, live[0]:live[-1] + 1] = 1
    assert torch.equal(visits.cpu(), want_vis)
    # values against the oracle and the other kernel
    want = O.attention_reference(q, k, v, score_bias=bias.float(), softcap=cap)
    blind = torch.isnan(want).any(-1)
    gotc = got.float().cpu()
    assert torch.isnan(gotc[blind]).all()
    assert (gotc[~blind] - want[~blind]).abs().max().item() <= TOL[dt] if (~blind).any() else True
    monkeypatch.setenv("LOOPFUSE_BIAS_TILES", "0")
    other = lowering.attention(*on[:3], plan, score_bias=on[3]).float().cpu()
    assert lowering.attention.last_launch["kernels"] == ["lf_attn_prefill"]
    assert torch.equal(torch.isnan(other), torch.isnan(gotc))
    assert (other[~blind] - gotc[~blind]).abs().max().item() <= TOL[dt] if (~blind).any() else True


@pytest.mark.parametrize("per_head", [False, True])
@pytest.mark.parametrize("group", [2, 4])
def test_bias_tiles_with_grouped_query_heads(group, per_head):
    """A mask shared by all heads keeps the packing of query heads (q tiles of 32 or 64 rows, classes at
    that granularity); a bias that differs per head runs one head per workgroup.  Both equal the oracle."""
    B, Hkv, Sq, Sk, D = 2, 2, 300, 333, 128
    Hq = Hkv * group
    q, k, v = rand((B, Hq, Sq, D), torch.bfloat16, 1), rand((B, Hkv, Sk, D), torch.bfloat16, 2), rand((B, Hkv, Sk, D), torch.bfloat16, 3)
    i, j = torch.arange(Sq)[:, None], torch.arange(Sk)[None, :]
    keep = (j <= i + 33) & (i + 33 - j < 100)
    bias = torch.zeros(B, Hq if per_head else 1, Sq, Sk).masked_fill(~keep, float("-inf"))
    bias[1, :, :, 150:170] = float("-inf")                       # a hole in the second sequence
    if per_head:
        bias = bias + (torch.arange(Hq).float()[None, :, None, None] * 0.01 * (j - i)).masked_fill(~keep, 0.0)
    bias = bias.to(torch.bfloat16)
    on = [t.to(dev()) for t in (q, k, v, bias)]
    got = lowering.attention(*on[:3], lowering.AttnPlan(scale=D ** -0.5), score_bias=on[3]).float().cpu()
    assert lowering.attention.last_launch["kernels"] == ["lf_bias_classify", "lf_attn_prefill_swp"]
    assert lowering.attention.last_launch["heads_per_workgroup"] == (1 if per_head else group)
    want = O.attention_reference(q, k, v, score_bias=bias.float())
    assert (got - want).abs().max().item() <= TOL[torch.bfloat16]


def _mask_sweep_case(i):
    """Case i of a seeded sweep over score biases that hold -inf regions (mask tensors)."""
    g = torch.Generator().manual_seed(5000 + i)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    pick = lambda xs: xs[ri(0, len(xs) - 1)]
    kind = pick(["prefill", "prefill", "rect", "decode", "decode"])
    c = dict(dtype=pick([torch.bfloat16, torch.float16]), D=pick([64, 128]), B=ri(1, 3), Hkv=pick([1, 2, 8]),
             group=pick([1, 2, 4]), kind=kind, softcap=pick([None, None, 30.0]),
             bcast=pick(["none", "batch", "head", "both", "row"]), noise=pick([False, True]),
             blocks=ri(1, 6), flag=pick([None, None, "causal"]) if kind == "prefill" else None, seed=6000 + i)
    if kind == "prefill":
        c["Sq"] = c["Sk"] = ri(1, 900)
    elif kind == "rect":
        c["Sq"], c["Sk"] = ri(1, 300), ri(1, 1500)
    else:
        c["Sq"], c["Sk"] = 1, ri(16, 4000)
        c["splits"] = pick([None, None, 1, 3])
    return c


@pytest.mark.parametrize("i", range(24))
def test_seeded_mask_sweep(i):
    c = _mask_sweep_case(i)
    dt, D, B, Hkv, Sq, Sk = c["dtype"], c["D"], c["B"], c["Hkv"], c["Sq"], c["Sk"]
    Hq = Hkv * c["group"]
    g = torch.Generator().manual_seed(c["seed"])
    bshape = [B, Hq, Sq, Sk]
    if c["bcast"] in ("batch", "both"):
        bshape[0] = 1
    if c["bcast"] in ("head", "both"):
        bshape[1] = 1
    if c["bcast"] == "row":
        bshape[2] = 1
    bias = torch.randn(bshape, generator=g) if c["noise"] else torch.zeros(bshape)
    for _ in range(c["blocks"]):              # rectangles of -inf, some larger than a 128 x 64 tile
        r0, c0 = int(torch.randint(0, bshape[2], (1,), generator=g)), int(torch.randint(0, Sk, (1,), generator=g))
        h, w = int(torch.randint(1, 400, (1,), generator=g)), int(torch.randint(1, 900, (1,), generator=g))
        bias[..., r0:r0 + h, c0:c0 + w] = float("-inf")
    # every row keeps a visible key: the first one, or any one for decode shapes (spans that
    # start and end anywhere)
    bias[..., int(torch.randint(0, Sk, (1,), generator=g)) if c["kind"] == "decode" else 0] = 0.0
    bias = bias.to(dt)
    q, k, v = rand((B, Hq, Sq, D), dt, c["seed"] + 1), rand((B, Hkv, Sk, D), dt, c["seed"] + 2), rand((B, Hkv, Sk, D), dt, c["seed"] + 3)
    print("mask sweep case", i, {**c, "bias_shape": bshape}, flush=True)
    kw = {"num_splits": c["splits"]} if c.get("splits") else {}
    check(q, k, v, mask=c["flag"], softcap=c["softcap"], score_bias=bias, **kw)


@pytest.mark.parametrize("paged", [False, True])
def test_decode_reads_only_the_live_span_of_a_fixed_size_cache(paged):
    """A cache allocated for 4096 keys with 37..700 of them filled, left padding in front: the
    mask leaves a short live span per sequence; results equal attention over exactly those keys."""
    B, Hkv, group, D, Sk = 4, 8, 4, 128, 4096
    Hq = Hkv * group
    lo = torch.tensor([0, 100, 33, 512])
    hi = torch.tensor([37, 700, 34, 4096])           # one sequence with a single live key, one filled to the end
    j = torch.arange(Sk)[None, :]
    keep = (j >= lo[:, None]) & (j < hi[:, None])
    bias = torch.zeros(B, 1, 1, Sk).masked_fill(~keep[:, None, None, :], float("-inf")).to(torch.bfloat16)
    q, k, v = rand((B, Hq, 1, D), torch.bfloat16, 1), rand((B, Hkv, Sk, D), torch.bfloat16, 2), rand((B, Hkv, Sk, D), torch.bfloat16, 3)
    want = torch.stack([O.attention_reference(q[b:b + 1], k[b:b + 1, :, lo[b]:hi[b]], v[b:b + 1, :, lo[b]:hi[b]])[0] for b in range(B)])
    k_in, v_in, kt, vt = k, v, None, None
    if paged:
        P = 16
        n = B * Sk // P
        table = torch.randperm(n, generator=torch.Generator().manual_seed(4)).view(B, Sk // P).to(torch.int32)
        pool_k = torch.empty(n, P, Hkv, D, dtype=torch.bfloat16)
        pool_v = torch.empty(n, P, Hkv, D, dtype=torch.bfloat16)
        pool_k[table.long()] = k.transpose(1, 2).reshape(B, Sk // P, P, Hkv, D)
        pool_v[table.long()] = v.transpose(1, 2).reshape(B, Sk // P, P, Hkv, D)
        k_in, v_in, kt, vt = pool_k, pool_v, table, table.clone()
    on = lambda t: None if t is None else t.to(dev())
    plan = lowering.AttnPlan(scale=D ** -0.5, k_paged=paged, v_paged=paged)
    got = lowering.attention(on(q), on(k_in), on(v_in), plan, on(kt), on(vt), score_bias=on(bias)).float().cpu()
    assert lowering.attention.last_launch["kernels"][0] == "lf_attn_decode"
    assert (got - want).abs().max().item() <= TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", ["prefill", "decode"])
def test_masks_filled_with_the_most_negative_finite_value(dtype, shape):
    """Masks are often filled with torch.finfo(dtype).min instead of -inf.  With
    zero_blind_rows (attentions taken over from torch's fused op) such keys are left out like
    -inf ones: bit-equal to the -inf mask, equal to the oracle on rows that see a key, finite
    on rows that see none."""
    D = 64
    if shape == "prefill":
        B, H, Sq, Sk = 2, 2, 700, 700
        keep = (torch.arange(Sk)[None, :] <= torch.arange(Sq)[:, None]) & (torch.arange(Sk)[None, :] >= 200)
        keep = keep[None, None].expand(B, 1, Sq, Sk)
    else:
        B, H, Sq, Sk = 4, 4, 1, 3000          # the last sequence sees no key at all
        keep = ((torch.arange(Sk)[None, :] >= torch.tensor([0, 2100, 64, 7])[:, None]) &
                (torch.arange(Sk)[None, :] < torch.tensor([500, 2600, 65, 7])[:, None]))[:, None, None, :]
    lowest = torch.zeros(keep.shape).masked_fill(~keep, torch.finfo(dtype).min).to(dtype)
    ninf = torch.zeros(keep.shape).masked_fill(~keep, float("-inf")).to(dtype)
    q, k, v = rand((B, H, Sq, D), dtype, 1), rand((B, H, Sk, D), dtype, 2), rand((B, H, Sk, D), dtype, 3)
    on = [t.to(dev()) for t in (q, k, v)]
    plan = lowering.AttnPlan(scale=D ** -0.5, zero_blind_rows=True)
    a = lowering.attention(*on, plan, score_bias=lowest.to(dev()))
    b = lowering.attention(*on, plan, score_bias=ninf.to(dev()))
    sees = keep.any(-1).expand(B, H, Sq)
    assert torch.isfinite(a).all() and torch.equal(a[sees.to(dev())], b[sees.to(dev())])
    # rows that see no key give zeros with either fill, also where they share a walked tile / span
    # with rows that do see keys (fp16: the finite fill times log2(e) stays finite, so it has to be
    # mapped to -inf where it is added, not only where tiles are left out)
    assert (~sees).any() and (a[(~sees).to(dev())] == 0).all() and (b[(~sees).to(dev())] == 0).all()
    want = O.attention_reference(q, k, v, score_bias=ninf.float())
    assert (a.float().cpu()[sees] - want[sees]).abs().max().item() <= TOL[dtype]


@pytest.mark.parametrize("name,B,S", [("c2_mask", 2, 512), ("c5_padded", 4, 1024), ("cache4096", 4, 1024)])
def test_mask_tensor_workloads_of_the_bench(name, B, S):
    """The bench's workloads whose mask is a tensor of 0 / -inf (causal mask as [1,1,S,S], left
    padding, partly filled cache), at sizes the oracle finishes in seconds: same result as the
    oracle given the same tensor, and as the kernel's own flag path where one exists."""
    w = workloads.make(name, seed=7, B=B, S=S)
    got = workloads.run(w.to(dev())).float().cpu()
    want = O.attention_reference(w.q, w.k, w.v, mask=w.mask, k_table=w.k_table, v_table=w.v_table,
                                 score_bias=w.score_bias)
    assert (got - want).abs().max().item() <= TOL[w.q.dtype]
    if name == "c2_mask":
        flag = workloads.make("c2", seed=7, B=B, S=S)
        assert torch.equal(flag.q, w.q) and w.flops() == flag.flops()
        by_flag = workloads.run(flag.to(dev())).float().cpu()
        assert (got - by_flag).abs().max().item() <= TOL[w.q.dtype]
    else:
        # only the keys a sequence can see count as traffic
        seen = int(torch.isfinite(w.score_bias.float()).sum())
        assert w.visible_keys == seen
        assert w.kv_bytes() == 2 * 2 * w.kv_heads() * seen * w.q.shape[-1]
