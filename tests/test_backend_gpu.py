"""torch.compile(backend=loopfuse_backend) on the GPU: the graphs of the reference's
own accuracy tests (tests/test_accuracy.py:125-311) and of its benchmark
(tests/benchmark.py:78-84, 141-147, 216-226, 400-406) must take the fused HIP
path (checked through interface.stats, so an eager fallback cannot pass) and match
the CPU fp32 oracle within the bf16 tolerance.  Graphs the backend does not lower
(the reference's add / matmul+add / biased attention cases) must still be right.
"""
import pytest
import torch

import loopfuse_amd
from loopfuse_amd import loopfuse_backend
from loopfuse_amd.torch_backend import interface
from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 2e-2


def rand(shape, dtype=torch.bfloat16, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def run_fused(fn, inputs, mode=None, derived=None):
    """``derived``: True / False = the loop-nest front end must / cannot have produced the plan."""
    torch._dynamo.reset()
    before = dict(interface.stats)
    out = torch.compile(fn, backend=loopfuse_backend, dynamic=True, mode=mode)(*[t.to(DEV) for t in inputs])
    torch.cuda.synchronize()
    assert interface.stats["fused"] == before["fused"] + 1, "the fused HIP path was not taken"
    if derived is not None:
        assert interface.stats["derived_graphs"] == before["derived_graphs"] + int(derived)
    assert interface.stats["eager_graph"] == before["eager_graph"]
    assert interface.stats["eager_runtime"] == before["eager_runtime"]
    return out.float().cpu()


@pytest.mark.parametrize("S", [256, 593])
def test_standard_attn(S):
    def fn(Q, K, V):
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    Q, K, V = (rand((4, 8, S, 64), seed=s) for s in (1, 2, 3))
    torch._dynamo.mark_static(Q, 3)
    torch._dynamo.mark_dynamic(Q, 2)
    got = run_fused(fn, (Q, K, V), derived=True)
    assert (got - O.attention_reference(Q, K, V, mask="causal")).abs().max() <= TOL


def test_gqa_attn():
    def fn(Q, K, V):
        g = Q.shape[1] // K.shape[1]
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    Q = rand((4, 8, 1024, 64), seed=1)
    K, V = (rand((4, 4, 1024, 64), seed=s) for s in (2, 3))
    got = run_fused(fn, (Q, K, V), derived=True)
    assert (got - O.attention_reference(Q, K, V, mask="causal")).abs().max() <= TOL


def test_sliding_mask_softcap_gqa():
    def fn(Q, K, V):
        g = Q.shape[1] // K.shape[1]
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        QK = torch.tanh(QK / 30) * 30
        return torch.softmax(torch.ops.loopfuse.sliding_mask(QK, 256), dim=-1) @ V

    Q = rand((2, 32, 1024, 128), seed=1)
    K, V = (rand((2, 8, 1024, 128), seed=s) for s in (2, 3))
    got = run_fused(fn, (Q, K, V), mode="max-autotune", derived=True)
    want = O.attention_reference(Q, K, V, mask="sliding", window=256, softcap=30.0)
    assert (got - want).abs().max() <= TOL


def test_paged_attention_k_only():
    def fn(Q, K_cache, K_block_table, V):
        K = torch.ops.loopfuse.paged_load(K_cache, K_block_table).transpose(1, 2)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    B, H, S, D = 4, 8, 1024, 64
    n = B * S * 2
    Kc = rand((n, H, D), seed=1)
    tab = torch.randint(0, n, (B, S), generator=torch.Generator().manual_seed(5), dtype=torch.int32)
    Q, V = rand((B, H, S, D), seed=2), rand((B, H, S, D), seed=3)
    got = run_fused(fn, (Q, Kc, tab, V), derived=True)
    want = O.attention_reference(Q, Kc, V, mask="causal", k_table=tab)
    assert (got - want).abs().max() <= TOL


def test_paged_attention_gqa():
    # reference tests/test_accuracy.py:281-311: paged K (one-token pages) + GQA, causal prefill
    def fn(Q, K_cache, K_block_table, V):
        K = torch.ops.loopfuse.paged_load(K_cache, K_block_table).transpose(1, 2)
        g = Q.shape[1] // K.shape[1]
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    B, Hq, Hk, S, D = 4, 8, 4, 256, 64
    n = B * S * 2
    Kc = rand((n, Hk, D), seed=1)
    tab = torch.randint(0, n, (B, S), generator=torch.Generator().manual_seed(5), dtype=torch.int32)
    Q, V = rand((B, Hq, S, D), seed=2), rand((B, Hk, S, D), seed=3)
    torch._dynamo.mark_static(Q, 3)
    torch._dynamo.mark_dynamic(Q, 2)
    got = run_fused(fn, (Q, Kc, tab, V), derived=True)
    want = O.attention_reference(Q, Kc, V, mask="causal", k_table=tab)
    assert (got - want).abs().max() <= TOL


def test_modified_attn():
    # reference tests/test_accuracy.py:172-196: query bias, score scale and bias, output bias
    def fn(Q, K, V, q_bias, scores_bias, out_bias):
        QK = (Q + q_bias) @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        QK = QK * 3.5 + scores_bias
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V + out_bias

    B, H, S, D = 4, 8, 1024, 64
    Q, K, V, qb = (rand((B, H, S, D), seed=s) for s in (1, 2, 3, 4))
    sb, ob = rand((B, H, S, S), seed=5), rand((B, H, S, D), seed=6)
    torch._dynamo.mark_static(Q, 3)
    torch._dynamo.mark_dynamic(Q, 2)
    got = run_fused(fn, (Q, K, V, qb, sb, ob), derived=True)
    # the graph adds the query bias in bf16 before the first product; so does the oracle input
    want = O.attention_reference(Q + qb, K, V, mask="causal", scale=3.5 * D ** -0.5, score_bias=sb, out_bias=ob)
    excess = ((got - want).abs() - 2.0 ** -8 * want.abs()).max()     # bf16 rounding of the shifted output
    assert excess <= TOL


def test_broadcast_score_bias_gqa():
    # an ALiBi-like bias shared by the batch, one slope per head, with grouped K/V
    def fn(Q, K, V, bias):
        g = Q.shape[1] // K.shape[1]
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5) + bias
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    B, Hq, Hkv, S, D = 2, 8, 2, 512, 128
    Q = rand((B, Hq, S, D), seed=1)
    K, V = (rand((B, Hkv, S, D), seed=s) for s in (2, 3))
    pos = torch.arange(S)
    slopes = 2.0 ** -(torch.arange(1, Hq + 1).float())
    bias = (-(pos[:, None] - pos[None, :]).abs().float() * slopes[:, None, None]).to(torch.bfloat16)[None]
    got = run_fused(fn, (Q, K, V, bias), derived=True)
    want = O.attention_reference(Q, K, V, mask="causal", score_bias=bias)
    assert (got - want).abs().max() <= TOL


def test_explicit_softmax_shifted_denominator():
    # reference tests/test_attention.py:95-125: online-softmax hint with scan_max, out = e / (S + 1)
    import math

    def _softmax(X):
        Xf = X.to(torch.float32)
        Xf_scaled = Xf * 1 / math.log(2)
        X_mik, X_mi = torch.ops.loopfuse.scan_max(Xf_scaled)
        expX = torch.exp2(Xf_scaled - X_mik) * torch.exp2(X_mik - X_mi)
        return expX / (torch.sum(expX, dim=-1, keepdim=True) + 1)

    def fn(Q, K, V):
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return _softmax(torch.ops.loopfuse.causal_mask(QK)).to(Q.dtype) @ V

    Q, K, V = (rand((2, 8, 700, 128), seed=s) for s in (1, 2, 3))
    torch._dynamo.mark_static(Q, 3)
    torch._dynamo.mark_dynamic(Q, 2)
    got = run_fused(fn, (Q, K, V), derived=True)
    assert (got - O.attention_reference(Q, K, V, mask="causal", denom_add=1.0)).abs().max() <= TOL


def test_prefix_attention_two_fused_calls():
    # reference tests/test_attention.py:339-362: a shared prefix (batch 1, broadcast) attended without
    # a mask plus the causal suffix, each with its own softmax, summed
    def fn(Q, Kp, Vp, Ks, Vs):
        QKp = Q @ Kp.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        QKs = Q @ Ks.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(QKp, dim=-1) @ Vp + torch.softmax(torch.ops.loopfuse.causal_mask(QKs), dim=-1) @ Vs

    B, H, Sq, Sp, D = 3, 4, 320, 512, 128
    Q, Ks, Vs = (rand((B, H, Sq, D), seed=s) for s in (1, 2, 3))
    Kp, Vp = (rand((B, H, Sp, D), seed=s) for s in (4, 5))
    got = run_fused(fn, (Q, Kp, Vp, Ks, Vs), derived=False)       # two attentions in one graph: the matcher's
    assert len(interface.last_matches) == 2
    want = O.attention_reference(Q, Kp, Vp) + O.attention_reference(Q, Ks, Vs, mask="causal")
    assert (got - want).abs().max() <= 2 * TOL      # two bf16 results added in bf16


@pytest.mark.parametrize("shared_rope", [False, True])
def test_mla_two_part_scores(shared_rope):
    # reference tests/test_attention.py:126-151 (D_pe = D / 8); the second variant shares the
    # positional key across heads, as latent-attention models do
    def fn(Q_nope, Q_pe, K_nope, K_pe, V):
        qk_nope = Q_nope @ K_nope.transpose(-2, -1)
        qk_pe = Q_pe @ K_pe.expand(-1, Q_pe.shape[1], -1, -1).transpose(-2, -1)
        qk = qk_nope + qk_pe
        qk *= (Q_nope.shape[-1] + Q_pe.shape[-1]) ** (-0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(qk), dim=-1) @ V

    B, H, S, D = 2, 8, 1024, 128
    Dp = D // 8
    Qn, Kn, V = (rand((B, H, S, D), seed=s) for s in (1, 2, 3))
    Qp, Kp = rand((B, H, S, Dp), seed=4), rand((B, 1 if shared_rope else H, S, Dp), seed=5)
    torch._dynamo.mark_static(Qn, 3)
    torch._dynamo.mark_static(Qp, 3)
    torch._dynamo.mark_dynamic(Qn, 2)
    got = run_fused(fn, (Qn, Qp, Kn, Kp, V), derived=True)
    want = O.attention_reference(Qn, Kn, V, mask="causal", scale=(D + Dp) ** -0.5, q2=Qp, k2=Kp)
    assert (got - want).abs().max() <= TOL


def test_key_given_transposed():
    # reference tests/test_attention.py:265-282: K arrives as [B, H, D, S] and the graph has no transpose
    def fn(Q, K, V):
        QK = Q @ K * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    Q, V = rand((2, 4, 593, 128), seed=1), rand((2, 4, 593, 128), seed=3)
    Kt = rand((2, 4, 128, 593), seed=2)
    got = run_fused(fn, (Q, Kt, V))
    assert (got - O.attention_reference(Q, Kt.transpose(-2, -1), V, mask="causal")).abs().max() <= TOL


def test_query_reshaped_from_merged_batch_and_heads():
    # reference tests/test_attention.py:285-302 (marked broken there): Q arrives as [B*H, S, D]
    def fn(Q, K, V):
        Q = Q.reshape(*V.shape)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    B, H, S, D = 2, 4, 384, 128
    Q = rand((B * H, S, D), seed=1)
    K, V = rand((B, H, S, D), seed=2), rand((B, H, S, D), seed=3)
    got = run_fused(fn, (Q, K, V))
    assert (got - O.attention_reference(Q.view(B, H, S, D), K, V, mask="causal")).abs().max() <= TOL


@pytest.mark.parametrize("which", ["einsum", "rank3", "bshd"])
@pytest.mark.parametrize("dynamic", [True, None])
def test_other_spellings_of_attention(which, dynamic):
    """einsum-written products, [B*H, S, D] inputs, [B, S, H, D] storage; dynamic and static tracing."""
    def fn(Q, K, V):
        if which == "einsum":
            sc = torch.einsum("bhqd,bhkd->bhqk", Q, K) * (Q.shape[-1] ** -0.5)
            return torch.einsum("bhqk,bhkd->bhqd", torch.softmax(torch.ops.loopfuse.causal_mask(sc), dim=-1), V)
        if which == "bshd":
            Q, K, V = (t.transpose(1, 2) for t in (Q, K, V))
        o = torch.softmax(torch.ops.loopfuse.causal_mask(Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)), dim=-1) @ V
        return o.transpose(1, 2) if which == "bshd" else o

    B, H, S, D = 4, 8, 1100, 128
    shape = {"einsum": (B, H, S, D), "rank3": (B * H, S, D), "bshd": (B, S, H, D)}[which]
    Q, K, V = (rand(shape, seed=s) for s in (1, 2, 3))
    torch._dynamo.reset()
    before = dict(interface.stats)
    got = torch.compile(fn, backend=loopfuse_backend, dynamic=dynamic)(*[t.to(DEV) for t in (Q, K, V)]).float().cpu()
    torch.cuda.synchronize()
    assert interface.stats["fused"] == before["fused"] + 1, "the fused HIP path was not taken"
    to4 = {"einsum": lambda t: t, "rank3": lambda t: t.view(B, H, S, D), "bshd": lambda t: t.transpose(1, 2)}[which]
    want = O.attention_reference(to4(Q), to4(K), to4(V), mask="causal")
    assert (to4(got) - want).abs().max() <= TOL


def test_operands_computed_in_the_graph():
    # reference tests/test_attention.py:465-481: elementwise functions of Q, K, V feed the attention
    def fn(Q, K, V):
        QK = torch.sin(Q) @ torch.cos(K).transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ torch.exp(V)

    Q, K, V = (rand((2, 4, 320, 128), seed=s) for s in (1, 2, 3))
    got = run_fused(fn, (Q, K, V))
    sin, cos, ex = (f(t.float()).to(torch.bfloat16) for f, t in ((torch.sin, Q), (torch.cos, K), (torch.exp, V)))
    assert (got - O.attention_reference(sin, cos, ex, mask="causal")).abs().max() <= 4 * TOL   # exp(V) reaches ~30


def test_sliding_mask_with_one_query_row():
    # reference tests/test_attention.py:365-381: top-left alignment leaves row 0 its first key only
    def fn(Q, K, V):
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.sliding_mask(QK, 256), dim=-1) @ V

    Q = rand((2, 4, 1, 128), seed=1)
    K, V = rand((2, 4, 512, 128), seed=2), rand((2, 4, 512, 128), seed=3)
    torch._dynamo.mark_static(Q, 3)
    got = run_fused(fn, (Q, K, V))
    assert (got - O.attention_reference(Q, K, V, mask="sliding", window=256)).abs().max() <= TOL
    assert (got - V[:, :, :1].float()).abs().max() <= TOL


def test_gqa_decoding_with_repeat_interleave():
    # reference tests/test_attention.py:172-189
    def fn(Q, K, V):
        g = Q.shape[1] // K.shape[1]
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(QK, dim=-1) @ V

    Q = rand((4, 32, 1, 128), seed=1)
    K, V = rand((4, 4, 1024, 128), seed=2), rand((4, 4, 1024, 128), seed=3)
    torch._dynamo.mark_static(Q, 3)
    got = run_fused(fn, (Q, K, V))
    assert (got - O.attention_reference(Q, K, V)).abs().max() <= TOL


def test_attention_inside_a_transformer_block():
    # the attention is found inside projections and a residual; everything else runs as it is
    def fn(x, wq, wk, wv, wo):
        B, S, E = x.shape
        H = 8
        q = (x @ wq).view(B, S, H, E // H).transpose(1, 2)
        k = (x @ wk).view(B, S, H, E // H).transpose(1, 2)
        v = (x @ wv).view(B, S, H, E // H).transpose(1, 2)
        a = torch.softmax(torch.ops.loopfuse.causal_mask(q @ k.transpose(-2, -1) * (E // H) ** -0.5), dim=-1) @ v
        return a.transpose(1, 2).reshape(B, S, E) @ wo + x

    x = rand((2, 384, 1024), seed=1)
    ws = [rand((1024, 1024), seed=s) * 0.03 for s in (2, 3, 4, 5)]
    ws = [w.to(torch.bfloat16) for w in ws]
    got = run_fused(fn, (x, *ws))
    want = fn(*[t.to(DEV) for t in (x, *ws)]).float().cpu()       # the same graph, eager, on the GPU
    assert (got - want).abs().max() <= 4 * TOL and (got - want).abs().mean() <= 4e-3


@pytest.mark.parametrize("which", ["on_zeros", "alibi"])
def test_scores_spelled_with_baddbmm(which):
    """The decoders that merge batch and heads and take the scores from ``torch.baddbmm``: on a tensor of
    zeros (GPT-NeoX) -- read as zeros from the graph, no bias at all -- or on an ALiBi term of shape
    [B*H, 1, S] (BLOOM, Falcon), which becomes the kernels' score bias with batch and heads sharing a dim."""
    B, H, S, D = 2, 8, 333, 64

    def fn(q, k, v, alibi):
        bs, nh, ql, hd = q.shape
        qq, kk = q.reshape(bs * nh, ql, hd), k.reshape(bs * nh, ql, hd)
        base = torch.zeros(bs * nh, ql, ql, dtype=q.dtype, device=q.device) if which == "on_zeros" else alibi
        scores = torch.baddbmm(base, qq, kk.transpose(1, 2), beta=1.0, alpha=hd ** -0.5).view(bs, nh, ql, ql)
        w = torch.softmax(torch.ops.loopfuse.causal_mask(scores), dim=-1, dtype=torch.float32).to(q.dtype)
        return torch.matmul(w, v)

    q, k, v = (rand((B, H, S, D), seed=s) for s in (1, 2, 3))
    slopes = 2.0 ** -torch.arange(1, H + 1).float()
    alibi = (slopes[:, None, None] * torch.arange(S).float()[None, None, :]).repeat(B, 1, 1).to(torch.bfloat16)   # [B*H, 1, S]
    got = run_fused(fn, (q, k, v, alibi))
    (m,) = interface.last_matches
    assert m.mask == "causal" and (m.bias is not None) == (which == "alibi")
    bias = None if which == "on_zeros" else alibi.float().view(B, H, 1, S).expand(B, H, S, S)
    assert (got - O.attention_reference(q, k, v, mask="causal", score_bias=bias)).abs().max() <= TOL


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_softmax_asked_for_in_float32(dtype):
    """``F.softmax(scores, dim=-1, dtype=torch.float32).to(q.dtype)``, the decoder layers' spelling: for
    fp16 scores on the GPU it traces to ``_softmax(..., half_to_float=True)``, for bf16 to a cast and a
    plain softmax; both are the fused attention."""
    import torch.nn.functional as F

    def fn(q, k, v):
        s = torch.ops.loopfuse.causal_mask(q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5)
        return F.softmax(s, dim=-1, dtype=torch.float32).to(q.dtype) @ v

    Q, K, V = (rand((2, 4, 300, 64), dtype=dtype, seed=s) for s in (1, 2, 3))
    got = run_fused(fn, (Q, K, V))
    assert (got - O.attention_reference(Q, K, V, mask="causal")).abs().max() <= (TOL if dtype == torch.bfloat16 else 5e-3)


@pytest.mark.parametrize("which", ["buffer_eq_zero", "arange_where", "key_padding_decode", "band"])
def test_boolean_masks_written_by_hand(which):
    """``masked_fill`` / ``where`` with a boolean tensor and -inf (a causal buffer cut to the sequence as in
    the common GPT module, index comparisons built in the graph, a key-padding mask on a decode step, a
    symmetric band): fused, the mask travelling as a 0 / -inf score term."""
    import math
    ninf = float("-inf")
    if which == "buffer_eq_zero":
        def fn(x, wqkv, wo, buf):
            B, T, E = x.shape
            q, k, v = ((x @ w).view(B, T, 8, E // 8).transpose(1, 2) for w in wqkv.unbind(0))
            att = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(k.size(-1)))
            att = att.masked_fill(buf[:, :, :T, :T] == 0, ninf)
            y = torch.softmax(att, dim=-1) @ v
            return y.transpose(1, 2).contiguous().view(B, T, E) @ wo
        ins = (rand((2, 593, 512), seed=1), rand((3, 512, 512), seed=2) * 0.04, rand((512, 512), seed=3) * 0.04,
               torch.tril(torch.ones(1024, 1024)).view(1, 1, 1024, 1024))
        ins = tuple(t.to(torch.bfloat16) if i < 3 else t for i, t in enumerate(ins))
    elif which == "arange_where":
        def fn(q, k, v):
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            i = torch.arange(q.shape[-2], device=q.device)[:, None]
            j = torch.arange(k.shape[-2], device=q.device)[None, :]
            return torch.softmax(torch.where((j <= i) & (i - j < 100), s, ninf), -1) @ v
        ins = tuple(rand((2, 4, 700, 128), seed=s) for s in (1, 2, 3))
    elif which == "key_padding_decode":
        def fn(q, k, v, pad):
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            return torch.softmax(s.masked_fill(pad[:, None, None, :], ninf), -1) @ v
        pad = torch.zeros(8, 1024, dtype=torch.bool)
        for b in range(8):
            pad[b, 200 + 100 * b:] = True
        ins = (rand((8, 8, 1, 128), seed=1), rand((8, 8, 1024, 128), seed=2), rand((8, 8, 1024, 128), seed=3), pad)
    else:
        def fn(q, k, v):
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            i = torch.arange(q.shape[-2], device=q.device)[:, None]
            j = torch.arange(k.shape[-2], device=q.device)[None, :]
            return torch.softmax(s.masked_fill((i - j).abs() >= 64, ninf), -1) @ v
        ins = (rand((1, 4, 300, 64), seed=1), rand((1, 4, 420, 64), seed=2), rand((1, 4, 420, 64), seed=3))
    got = run_fused(fn, ins)
    (m,) = interface.last_matches
    if which == "arange_where":        # built from indices alone: recognised as a causal window, no mask tensor at all
        assert m.mask == "sliding" and m.window == 100 and m.bias is None
    else:
        assert m.mask is None and m.bias is not None and m.bias.keep in (1, -1)
    want = fn(*[t.to(DEV).float() if t.dtype == torch.bfloat16 else t.to(DEV) for t in ins]).float().cpu()   # eager, fp32
    assert torch.isfinite(got).all()
    assert (got - want).abs().max() <= (4 * TOL if which == "buffer_eq_zero" else TOL)


@pytest.mark.parametrize("which", ["causal", "gqa_decode", "scale_rect", "module", "bool_mask", "float_mask"])
@pytest.mark.parametrize("dynamic", [True, False])
def test_torch_fused_attention_calls_are_taken_over(which, dynamic):
    """F.scaled_dot_product_attention arrives as one aten._scaled_dot_product_* node;
    without a mask tensor or dropout it is the same attention and runs on the HIP kernels
    (the output keeps the memory order the traced op gives, which later views rely on)."""
    import torch.nn.functional as F
    if which == "causal":
        fn = lambda q, k, v: F.scaled_dot_product_attention(q, k, v, is_causal=True)
        ins = (rand((2, 8, 333, 128), seed=1), rand((2, 8, 333, 128), seed=2), rand((2, 8, 333, 128), seed=3))
        want = O.attention_reference(*ins, mask="causal")
    elif which == "gqa_decode":
        fn = lambda q, k, v: F.scaled_dot_product_attention(q, k, v, enable_gqa=True)
        ins = (rand((4, 32, 1, 128), seed=1), rand((4, 8, 1000, 128), seed=2), rand((4, 8, 1000, 128), seed=3))
        want = O.attention_reference(*ins)
    elif which == "scale_rect":
        fn = lambda q, k, v: F.scaled_dot_product_attention(q, k, v, scale=0.05) * 2
        ins = (rand((2, 4, 100, 64), seed=1), rand((2, 4, 260, 64), seed=2), rand((2, 4, 260, 64), seed=3))
        want = O.attention_reference(*ins, scale=0.05) * 2
    elif which in ("bool_mask", "float_mask"):
        fn = lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m)
        if which == "bool_mask":
            m = torch.rand(2, 1, 200, 264, generator=torch.Generator().manual_seed(5)) > 0.3
            m[..., 0] = True
            bias = torch.zeros(m.shape).masked_fill(~m, float("-inf"))
        else:
            m = rand((1, 4, 200, 264), seed=5)
            bias = m.float()
        ins = (rand((2, 4, 200, 64), seed=1), rand((2, 4, 264, 64), seed=2), rand((2, 4, 264, 64), seed=3), m)
        want = O.attention_reference(*ins[:3], score_bias=bias)
    else:
        def fn(x, wqkv, wo):
            B, S, E = x.shape
            q, k, v = ((x @ w).view(B, S, 8, E // 8).transpose(1, 2) for w in wqkv.unbind(0))
            a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
            return a.transpose(1, 2).reshape(B, S, E) @ wo
        ins = (rand((2, 200, 512), seed=1), rand((3, 512, 512), seed=2) * 0.04, rand((512, 512), seed=3) * 0.04)
        want = None
    torch._dynamo.reset()
    before = dict(interface.stats)
    dev_ins = [t.to(DEV) for t in ins]
    with torch.no_grad():
        got = torch.compile(fn, backend=loopfuse_backend, dynamic=dynamic, mode=None)(*dev_ins)
        if want is None:
            want = fn(*dev_ins).float().cpu()
    torch.cuda.synchronize()
    assert interface.stats["fused"] == before["fused"] + 1, "the fused HIP path was not taken"
    err = (got.float().cpu() - want).abs().max().item()
    assert err <= (4 * TOL if which == "module" else 2 * TOL if which == "scale_rect" else TOL), err


@pytest.mark.parametrize("S,P,use_mask", [(300, 0, False), (1, 700, False), (64, 700, True)])
def test_decoder_layer_with_cache_and_repeated_kv_heads(S, P, use_mask):
    """The decoder-layer attention block of tests/test_capture.py (rotary embedding, cache
    concatenation, kv heads repeated by expand + reshape, F.scaled_dot_product_attention)
    in bf16 with D = 128: prefill, one-token decode and a masked chunk all run on the HIP
    kernels with the un-repeated cache as K and V."""
    from test_capture import DecoderLayerAttention, decoder_layer_inputs
    torch.manual_seed(0)
    m = DecoderLayerAttention(E=1024, H=8, Hkv=2).eval().to(DEV).to(torch.bfloat16)
    ins = [None if t is None else t.to(DEV) for t in decoder_layer_inputs(1024, 8, 2, S, P, use_mask, torch.bfloat16)]
    torch._dynamo.reset()
    before = dict(interface.stats)
    with torch.no_grad():
        got = torch.compile(m, backend=loopfuse_backend, dynamic=True, mode=None)(*ins)
        want = m(*ins)
    torch.cuda.synchronize()
    assert interface.stats["fused"] == before["fused"] + 1, "the fused HIP path was not taken"
    match = interface.last_matches[-1]
    assert match.k.group == 4 and match.inputs[match.k.index].name.startswith("cat")
    assert (got[0].float() - want[0].float()).abs().max().item() <= 4 * TOL
    assert torch.equal(got[1], want[1]) and torch.equal(got[2], want[2])


def test_batched_decode_with_a_padding_mask_stays_on_the_decode_kernel():
    """One-token decode of a left-padded batch: F.scaled_dot_product_attention with a boolean
    [B, 1, 1, Sk] mask and grouped kv heads runs on the streaming decode kernel."""
    import torch.nn.functional as F
    from loopfuse_amd import lowering
    B, Hq, Hkv, Sk, D = 4, 32, 8, 1500, 128
    q, k, v = rand((B, Hq, 1, D), seed=1), rand((B, Hkv, Sk, D), seed=2), rand((B, Hkv, Sk, D), seed=3)
    pad = torch.tensor([0, 1200, 64, 333])
    keep = (torch.arange(Sk)[None, :] >= pad[:, None])[:, None, None, :]
    def repeat_kv(h, n):
        b, hk, s, d = h.shape
        return h[:, :, None, :, :].expand(b, hk, n, s, d).reshape(b, hk * n, s, d)

    fn = lambda q, k, v, m: F.scaled_dot_product_attention(q, repeat_kv(k, Hq // Hkv), repeat_kv(v, Hq // Hkv), attn_mask=m)
    got = run_fused(fn, (q, k, v, keep))
    assert lowering.attention.last_launch["kernels"][0] == "lf_attn_decode"
    want = O.attention_reference(q, k, v, score_bias=torch.zeros(keep.shape).masked_fill(~keep, float("-inf")))
    assert (got - want).abs().max().item() <= TOL


def test_rows_without_a_visible_key_give_zeros_like_the_stock_op():
    """Left-padded prefill: the padded query rows see no key.  torch's fused attention returns
    zeros for them (NaN there would leak into later layers through K and V); so does the take-over."""
    import torch.nn.functional as F
    B, H, S, D = 2, 4, 300, 64
    q, k, v = (rand((B, H, S, D), seed=s) for s in (1, 2, 3))
    pad = torch.tensor([0, 130])
    i, j = torch.arange(S)[:, None], torch.arange(S)[None, :]
    keep = ((j <= i)[None] & (j[None] >= pad[:, None, None]))[:, None]            # causal and not padding
    fn = lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m)
    got = run_fused(fn, (q, k, v, keep))
    stock = fn(*[t.to(DEV) for t in (q, k, v, keep)]).float().cpu()
    assert (got[1, :, :130] == 0).all() and (stock[1, :, :130] == 0).all()
    assert (got - stock).abs().max().item() <= TOL


def test_module_with_parameters_outside_and_inside_no_grad():
    """A module's parameters require grad: called outside torch.no_grad() the graph is
    traced for training and runs unfused (and can be differentiated); inside it the
    attention takes the HIP kernels."""
    class Attn(torch.nn.Module):
        def __init__(self):
            super().__init__()
            torch.manual_seed(0)
            self.qkv = torch.nn.Linear(512, 3 * 512, bias=False)
            self.out = torch.nn.Linear(512, 512, bias=False)

        def forward(self, x):
            B, S, E = x.shape
            q, k, v = (t.view(B, S, 8, 64).transpose(1, 2) for t in self.qkv(x).chunk(3, dim=-1))
            a = torch.softmax(torch.ops.loopfuse.causal_mask(q @ k.transpose(-2, -1) * 0.125), dim=-1) @ v
            return self.out(a.transpose(1, 2).reshape(B, S, E))

    m = Attn().to(DEV).to(torch.bfloat16)
    x = rand((2, 200, 512), seed=3).to(DEV)
    torch._dynamo.reset()
    before = dict(interface.stats)
    cm = torch.compile(m, backend=loopfuse_backend, dynamic=True, mode=None)
    y = cm(x)
    y.float().square().mean().backward()
    g_compiled = m.qkv.weight.grad.float().clone()
    m.zero_grad()
    y_eager = m(x)
    y_eager.float().square().mean().backward()
    assert interface.stats["fused"] == before["fused"] and interface.stats["eager_training"] >= before["eager_training"] + 2
    assert (y.float() - y_eager.float()).abs().max() <= 1e-2
    assert (g_compiled - m.qkv.weight.grad.float()).abs().max() <= 1e-3 * m.qkv.weight.grad.float().abs().max() + 1e-6
    torch._dynamo.reset()
    with torch.no_grad():
        y2 = torch.compile(m, backend=loopfuse_backend, dynamic=True, mode=None)(x)
    torch.cuda.synchronize()
    assert interface.stats["fused"] == before["fused"] + 1
    assert (y2.float() - y_eager.float()).abs().max() <= 4 * TOL


def test_paged_decode_gqa_reference_format():
    # tests/benchmark.py:400-443: one-token pages, Q viewed [B, Hkv, group, D]
    def fn(Q, Kc, kt, Vc, vt):
        K = torch.ops.loopfuse.paged_load(Kc, kt).transpose(-3, -2)
        V = torch.ops.loopfuse.paged_load(Vc, vt).transpose(-3, -2)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(QK, dim=-1) @ V

    B, Hkv, grp, S, D = 8, 4, 8, 2048, 128
    n = B * S * 2
    Kc, Vc = rand((n, Hkv, D), seed=1), rand((n, Hkv, D), seed=2)
    g = torch.Generator().manual_seed(5)
    kt = torch.randint(0, n, (B, S), generator=g, dtype=torch.int32)
    vt = torch.randint(0, n, (B, S), generator=g, dtype=torch.int32)
    Q = rand((B, Hkv, grp, D), seed=3)
    got = run_fused(fn, (Q, Kc, kt, Vc, vt))
    want = O.attention_reference(Q, Kc, Vc, k_table=kt, v_table=vt)
    assert (got - want).abs().max() <= TOL


def test_paged_decode_page16_config5_shape():
    def fn(Q, Kc, kt, Vc, vt):
        B, pages = kt.shape
        P, H, D = Kc.shape[1:]
        K = torch.ops.loopfuse.paged_load(Kc, kt).reshape(B, pages * P, H, D).transpose(1, 2)
        V = torch.ops.loopfuse.paged_load(Vc, vt).reshape(B, pages * P, H, D).transpose(1, 2)
        g = Q.shape[1] // H
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(QK, dim=-1) @ V

    from loopfuse_amd import workloads
    w = workloads.make("c5", seed=4, B=8, S=1024)
    got = run_fused(fn, (w.q, w.k, w.k_table, w.v, w.v_table))
    want = O.attention_reference(w.q, w.k, w.v, k_table=w.k_table, v_table=w.v_table)
    assert (got - want).abs().max() <= TOL


@pytest.mark.parametrize("pv,kernel", [(4, "lf_attn_prefill"), (64, "lf_attn_prefill_swp")])
def test_paged_pools_with_different_page_sizes(pv, kernel):
    # K pool in pages of 16 tokens, V pool in pages of 4 (register-staged kernel) or 64
    # (direct-to-LDS kernel), each with its own table
    def fn(Q, Kc, kt, Vc, vt):
        B = kt.shape[0]
        H, D = Kc.shape[2:]
        K = torch.ops.loopfuse.paged_load(Kc, kt).reshape(B, -1, H, D).transpose(1, 2)
        V = torch.ops.loopfuse.paged_load(Vc, vt).reshape(B, -1, H, D).transpose(1, 2)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    B, H, S, D = 2, 4, 512, 128
    g = torch.Generator().manual_seed(5)
    Kc, Vc = rand((B * S // 16, 16, H, D), seed=1), rand((B * S // pv, pv, H, D), seed=2)
    kt = torch.randperm(B * S // 16, generator=g).view(B, -1).to(torch.int32)
    vt = torch.randperm(B * S // pv, generator=g).view(B, -1).to(torch.int32)
    Q = rand((B, H, S, D), seed=3)
    got = run_fused(fn, (Q, Kc, kt, Vc, vt))
    want = O.attention_reference(Q, Kc, Vc, mask="causal", k_table=kt, v_table=vt)
    assert (got - want).abs().max() <= TOL
    from loopfuse_amd import lowering
    assert lowering.attention.last_launch["kernels"] == [kernel]


def test_static_shapes_at_baseline_sizes():
    """torch.compile WITHOUT dynamic=True (static shapes) on configs 2 and 5 at full size."""
    from loopfuse_amd import workloads

    def prefill(Q, K, V):
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    def decode(Q, Kc, kt, Vc, vt):
        B, pages = kt.shape
        P, H, D = Kc.shape[1:]
        K = torch.ops.loopfuse.paged_load(Kc, kt).reshape(B, pages * P, H, D).transpose(1, 2)
        V = torch.ops.loopfuse.paged_load(Vc, vt).reshape(B, pages * P, H, D).transpose(1, 2)
        g = Q.shape[1] // H
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        return torch.softmax(Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5), dim=-1) @ V

    for fn, w in ((prefill, workloads.make("c2", seed=1)), (decode, workloads.make("c5", seed=1))):
        ins = (w.q, w.k, w.v) if w.k_table is None else (w.q, w.k, w.k_table, w.v, w.v_table)
        torch._dynamo.reset()
        before = dict(interface.stats)
        got = torch.compile(fn, backend=loopfuse_backend)(*[t.to(DEV) for t in ins]).float().cpu()
        torch.cuda.synchronize()
        assert interface.stats["fused"] == before["fused"] + 1, "the static graph was not fused"
        b, h = 3, 17                                   # one (batch, head) against the oracle
        hk = h // (w.q.shape[1] // (w.k.shape[-2] if w.k_table is not None else w.k.shape[1]))
        if w.k_table is None:
            want = O.attention_reference(w.q[b:b + 1, h:h + 1], w.k[b:b + 1, hk:hk + 1], w.v[b:b + 1, hk:hk + 1], mask="causal")
        else:
            kk = O.gather_paged(w.k, w.k_table[b:b + 1])[:, hk:hk + 1]
            vv = O.gather_paged(w.v, w.v_table[b:b + 1])[:, hk:hk + 1]
            want = O.attention_reference(w.q[b:b + 1, h:h + 1], kk, vv)
        assert (got[b:b + 1, h:h + 1] - want).abs().max() <= TOL


def test_decode_contiguous():
    def fn(Q, K, V):
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(QK, dim=-1) @ V

    Q = rand((8, 32, 1, 128), seed=1)
    K, V = (rand((8, 32, 2048, 128), seed=s) for s in (2, 3))
    got = run_fused(fn, (Q, K, V))
    assert (got - O.attention_reference(Q, K, V)).abs().max() <= TOL


def test_recompile_free_new_sequence_length():
    """Sequence length is a kernel argument: a second length reuses the code object."""
    from loopfuse_amd import lowering

    def fn(Q, K, V):
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    torch._dynamo.reset()
    cf = torch.compile(fn, backend=loopfuse_backend, dynamic=True)
    outs = []
    for S in (384, 640):
        Q, K, V = (rand((2, 4, S, 128), seed=s) for s in (1, 2, 3))
        torch._dynamo.mark_dynamic(Q, 2)
        n_before = len(lowering._compiled)
        o = cf(Q.to(DEV), K.to(DEV), V.to(DEV)).float().cpu()
        assert (o - O.attention_reference(Q, K, V, mask="causal")).abs().max() <= TOL
        outs.append(len(lowering._compiled) - n_before)
    assert outs[1] == 0


def _softmax64(x):
    e = (x - x.amax(dim=-1, keepdim=True)).exp()
    return e / e.sum(dim=-1, keepdim=True)


@pytest.mark.parametrize("which", ["add", "add_2dim", "matmul_add", "matmul_add_3dim", "modified_attn", "softmax_matmul",
                                   "paged_add", "simplified_attn"])
def test_graphs_without_attention_run_as_generated_kernels(which):
    """Reference tests/test_accuracy.py:29-82, 172-211, 233-250, 314-333: graphs with no attention
    in them (lowered nest by nest to plain generated HIP kernels), plus the modified-attention
    graph in fp32 (the MFMA kernels take bf16 / fp16 only and refuse it; its generated kernels
    serve the call).  Each result is checked against an independent
    float64 computation on the CPU, spelled differently from the compiled function (einsum /
    explicit exponentials / index loops), not against the same graph run eagerly."""
    f64 = lambda ts: [t.double() if t.is_floating_point() else t for t in ts]
    if which == "add":
        fn = lambda a, b: a + b
        ins = (rand((4, 1024, 128), torch.float32, 1), rand((4, 1024, 128), torch.float32, 2))
        ref = lambda a, b: torch.stack([a, b]).sum(dim=0)
    elif which == "add_2dim":          # reference tests/test_accuracy.py:40-50
        fn = lambda a, b: a + b
        ins = (rand((512, 1024), torch.float32, 1), rand((512, 1024), torch.float32, 2))
        ref = lambda a, b: torch.stack([a, b]).sum(dim=0)
    elif which == "matmul_add_3dim":   # reference tests/test_accuracy.py:66-82
        fn = lambda a, b, c: a @ b + c
        ins = (rand((4, 256, 64), torch.float32, 1) * 0.1, rand((4, 64, 128), torch.float32, 2) * 0.1,
               rand((4, 256, 128), torch.float32, 3))
        ref = lambda a, b, c: torch.einsum("bik,bkj->bij", a, b) + c
    elif which == "simplified_attn":   # reference tests/test_accuracy.py:314-332: no exponential, not a softmax
        def fn(Q, K, V):
            QK = Q @ K.transpose(-2, -1)
            m = torch.max(QK, dim=-1, keepdim=True)[0] + torch.sum(QK, dim=-1, keepdim=True)
            return (QK / (m + 1e-3)) @ V
        ins = tuple(rand((2, 4, 256, 64), torch.float32, s) * 0.2 for s in (1, 2, 3))

        def ref(Q, K, V):
            s = torch.einsum("bhid,bhjd->bhij", Q, K)
            den = s.amax(dim=-1) + torch.einsum("bhij->bhi", s) + 1e-3
            return torch.einsum("bhij,bhjd->bhid", s, V) / den[..., None]
    elif which == "matmul_add":
        fn = lambda a, b, c: a @ b + c
        ins = (rand((256, 128), torch.float32, 1), rand((128, 128), torch.float32, 2), rand((256, 128), torch.float32, 3))
        ref = lambda a, b, c: torch.einsum("ik,kj->ij", a, b) + c
    elif which == "modified_attn":
        def fn(Q, K, V, qb, sb, ob):
            QK = (Q + qb) @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
            QK = QK * 3.5 + sb
            return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V + ob
        ins = tuple(rand((2, 2, 128, 64), torch.float32, s) for s in (1, 2, 3, 4)) + \
            (rand((2, 2, 128, 128), torch.float32, 5), rand((2, 2, 128, 64), torch.float32, 6))

        def ref(Q, K, V, qb, sb, ob):
            s = torch.einsum("bhid,bhjd->bhij", Q + qb, K) * (3.5 / 8.0) + sb
            i = torch.arange(s.shape[-2])[:, None]
            j = torch.arange(s.shape[-1])[None, :]
            s = torch.where(j <= i, s, torch.full_like(s, float("-inf")))
            return torch.einsum("bhij,bhjd->bhid", _softmax64(s), V) + ob
    elif which == "paged_add":       # reference tests/test_accuracy.py:233-250
        fn = lambda buf, tab: torch.ops.loopfuse.paged_load(buf, tab) + 1
        ins = (rand((64, 4, 32), torch.float32, 1),
               torch.randint(0, 64, (3, 20), generator=torch.Generator().manual_seed(2), dtype=torch.int32))
        ref = lambda buf, tab: torch.stack([torch.stack([buf[int(tab[b, s])] for s in range(tab.shape[1])])
                                            for b in range(tab.shape[0])]) + 1
    else:
        fn = lambda x, y: torch.softmax(x, dim=-1) @ y
        ins = (rand((2, 4, 128, 64), torch.float32, 1), rand((2, 4, 64, 128), torch.float32, 2))
        ref = lambda x, y: torch.einsum("bhij,bhjd->bhid", _softmax64(x), y)
    torch._dynamo.reset()
    dev_ins = [t.to(DEV) for t in ins]
    want = ref(*f64(ins))
    before = dict(interface.stats)
    got = torch.compile(fn, backend=loopfuse_backend, dynamic=True)(*dev_ins)
    tol = 1e-2 if which == "simplified_attn" else 1e-4      # the reference checks that case at rtol 1e-2 too
    torch.testing.assert_close(got.double().cpu(), want, rtol=tol, atol=tol)
    ran = {k: interface.stats[k] - before[k] for k in ("fused", "fused_generic", "eager_graph", "eager_runtime")}
    assert ran == {"fused": 0, "fused_generic": 1, "eager_graph": 0, "eager_runtime": 0}, ran


def test_generated_kernels_read_bf16_and_follow_new_shapes():
    """The generated kernels convert on load / store (bf16 in and out, fp32 arithmetic) and take
    every extent and stride as a run-time argument: one compiled graph serves a second shape and
    a transposed operand."""
    fn = lambda a, b, c: a @ b + c
    torch._dynamo.reset()
    compiled = torch.compile(fn, backend=loopfuse_backend, dynamic=True)
    before = dict(interface.stats)
    for seed, (m, k, n), t in ((1, (64, 32, 48), False), (2, (80, 40, 24), False), (3, (80, 40, 24), True)):
        a = rand((m, k), torch.bfloat16, seed).to(DEV)
        b = (rand((n, k), torch.bfloat16, seed + 10).to(DEV).t() if t else rand((k, n), torch.bfloat16, seed + 10).to(DEV))
        c = rand((m, n), torch.bfloat16, seed + 20).to(DEV)
        got = compiled(a, b, c)
        assert got.dtype == torch.bfloat16
        want = torch.einsum("ik,kj->ij", a.double().cpu(), b.double().cpu()) + c.double().cpu()
        torch.testing.assert_close(got.double().cpu(), want, rtol=2e-2, atol=2e-2)
    assert interface.stats["fused_generic"] == before["fused_generic"] + 3
    assert interface.stats["eager_runtime"] == before["eager_runtime"]


@pytest.mark.parametrize("name", ["c2", "c2_softcap", "c3", "c4", "c5"])
def test_loop_nest_front_end_on_the_gpu(name, monkeypatch):
    """LOOPFUSE_FRONTEND=ir: the benchmark configurations' graphs go through the loop-nest front
    end (per-op nests -> fuse -> online softmax -> block skip -> derived plan) to the HIP kernels
    and match the oracle."""
    from loopfuse_amd import workloads

    monkeypatch.setenv("LOOPFUSE_FRONTEND", "ir")

    def mods(s, cap):
        return s if cap is None else torch.tanh(s / cap) * cap

    def dense(cap, mask, window):
        def fn(q, k, v):
            g = q.shape[1] // k.shape[1]
            if g > 1:
                k, v = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
            s = mods(q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5), cap)
            if mask == "causal":
                s = torch.ops.loopfuse.causal_mask(s)
            elif mask == "sliding":
                s = torch.ops.loopfuse.sliding_mask(s, window)
            return torch.softmax(s, dim=-1) @ v
        return fn

    def paged(Q, Kc, kt, Vc, vt):
        B, pages = kt.shape
        P, H, D = Kc.shape[1:]
        K = torch.ops.loopfuse.paged_load(Kc, kt).reshape(B, pages * P, H, D).transpose(-3, -2)
        V = torch.ops.loopfuse.paged_load(Vc, vt).reshape(B, pages * P, H, D).transpose(-3, -2)
        return torch.softmax(Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5), dim=-1) @ V

    w = workloads.make(name, seed=11, B=2, S=640 if name in ("c2", "c2_softcap", "c3") else 1024)
    before = interface.stats["derived_graphs"]
    if name == "c5":
        B, Hq, _, D = w.q.shape
        Hkv = w.k.shape[2]
        got = run_fused(paged, (w.q.view(B, Hkv, Hq // Hkv, D), w.k, w.k_table, w.v, w.v_table)).view(B, Hq, 1, D)
    else:
        got = run_fused(dense(w.softcap, w.mask, w.window), (w.q, w.k, w.v))
    assert interface.stats["derived_graphs"] == before + 1, "the loop-nest front end did not derive this graph"
    want = O.attention_reference(w.q, w.k, w.v, mask=w.mask, window=w.window, softcap=w.softcap,
                                 k_table=w.k_table, v_table=w.v_table)
    assert (got - want).abs().max() <= TOL
