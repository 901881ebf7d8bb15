"""Backward of the fused attention (lf_attn_bwd.hip) against torch autograd on an fp32 eager
graph of the same attention (float64 accumulation of the reference values), through
``lowering.attention(..., lse=...)`` and ``lowering.attention_backward``.

The reference has no backward (its README lists it as future work), so there is no reference
test to mirror; the cases follow its forward matrix: masks none / causal / sliding, grouped
query heads, ragged lengths, both dtypes and head dims."""
import math

import pytest
import torch

from loopfuse_amd import lowering

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ref(q, k, v, dout, mask, window, scale, softcap=None):
    """O and the gradients from autograd on the eager graph, in float64."""
    q, k, v = (t.double().detach().requires_grad_(True) for t in (q, k, v))
    g = q.shape[1] // k.shape[1]
    kk, vv = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    s = q @ kk.transpose(-2, -1) * scale
    if softcap is not None:
        s = softcap * torch.tanh(s / softcap)
    Sq, Sk = s.shape[-2:]
    i = torch.arange(Sq, device=s.device)[:, None]
    j = torch.arange(Sk, device=s.device)[None, :]
    keep = torch.ones(Sq, Sk, dtype=torch.bool, device=s.device)
    if mask in ("causal", "sliding"):
        keep &= j <= i
    if mask == "sliding":
        keep &= (i - j) < window
    s = s.masked_fill(~keep, float("-inf"))
    lse2 = torch.logsumexp(s, dim=-1) / math.log(2.0)
    o = torch.softmax(s, dim=-1) @ vv
    o.backward(dout.double())
    return o.detach(), lse2.detach(), q.grad, k.grad, v.grad


CASES = [
    # B, Hq, Hkv, Sq, Sk, D, mask, window, dtype
    (2, 4, 4, 256, 256, 128, "causal", 0, torch.bfloat16),
    (2, 4, 4, 256, 256, 128, None, 0, torch.bfloat16),
    (1, 8, 2, 320, 320, 128, "causal", 0, torch.bfloat16),          # grouped query heads
    (1, 4, 4, 200, 200, 64, "causal", 0, torch.float16),            # ragged, D 64
    (1, 4, 2, 384, 384, 128, "sliding", 100, torch.bfloat16),
    (1, 2, 2, 192, 333, 64, None, 0, torch.bfloat16),               # Sq != Sk
    (1, 2, 1, 130, 130, 128, "sliding", 7, torch.float16),
    (3, 6, 3, 593, 593, 128, "causal", 0, torch.bfloat16),          # odd length; 9 (batch, kv head) pairs: padded slot groups
    (1, 3, 3, 1000, 1500, 64, None, 0, torch.float16),              # many tiles, Sq != Sk, neither a tile multiple
    (2, 4, 1, 700, 700, 128, "sliding", 4096, torch.bfloat16),      # window wider than the sequence; four query heads per kv head
]


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,mask,window,dtype", CASES)
def test_backward_matches_autograd(B, Hq, Hkv, Sq, Sk, D, mask, window, dtype):
    g = torch.Generator().manual_seed(Sq * 7 + Sk + D)
    q, k, v = (torch.randn(shape, generator=g).to(dtype).to(DEV)
               for shape in ((B, Hq, Sq, D), (B, Hkv, Sk, D), (B, Hkv, Sk, D)))
    dout = torch.randn((B, Hq, Sq, D), generator=g).to(dtype).to(DEV)
    scale = D ** -0.5
    plan = lowering.AttnPlan(mask=mask, window=window, scale=scale)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=DEV)
    o = lowering.attention(q, k, v, plan, lse=lse)
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = _ref(q, k, v, dout, mask, window, scale)
    tol = 2e-2 if dtype == torch.bfloat16 else 5e-3
    assert (o.double() - o_ref).abs().max().item() <= tol
    torch.testing.assert_close(lse.double(), lse_ref, rtol=1e-3, atol=2e-3)
    dq, dk, dv = lowering.attention_backward(q, k, v, o, lse, dout, plan)
    assert dq.dtype == dtype and dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    # gradients are sums of up to Sq (dK, dV: times the group) rounded products: tolerance relative to their size
    for name, got, want in (("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
        err = (got.double() - want).abs().max().item()
        bound = (4e-2 if dtype == torch.bfloat16 else 1e-2) * max(1.0, want.abs().max().item())
        assert err <= bound, f"{name}: max abs err {err} > {bound}"
        rel = ((got.double() - want).norm() / want.norm()).item()
        assert rel <= (2e-2 if dtype == torch.bfloat16 else 4e-3), f"{name}: relative error {rel}"


def _ref_head_fp32(q, k, v, dout, mask, window, scale):
    """Reference for one (batch, kv head): q, dout [G, Sq, D] (the G query heads of the group), k, v
    [Sk, D], all on the GPU; fp32 autograd on the dense graph.  Returns dq [G, Sq, D], dk, dv [Sk, D]."""
    q, k, v = (t.float().detach().requires_grad_(True) for t in (q, k, v))
    s = q @ k.t() * scale
    Sq, Sk = s.shape[-2:]
    i = torch.arange(Sq, device=s.device)[:, None]
    j = torch.arange(Sk, device=s.device)[None, :]
    keep = torch.ones(Sq, Sk, dtype=torch.bool, device=s.device)
    if mask in ("causal", "sliding"):
        keep &= j <= i
    if mask == "sliding":
        keep &= (i - j) < window
    o = torch.softmax(s.masked_fill(~keep, float("-inf")), dim=-1) @ v
    o.backward(dout.float())
    return q.grad, k.grad, v.grad


@pytest.mark.parametrize("name,Hkv,mask,window", [("config 2", 32, "causal", 0), ("config 3 without its softcap", 8, "sliding", 256)])
def test_backward_full_size_every_head(name, Hkv, mask, window):
    """The benchmark shapes (B8 Hq32 S2048 D128 bf16) at full size: every gradient element of every
    (batch, head) against fp32 autograd on the dense graph, evaluated on the GPU one kv head at a time."""
    B, Hq, S, D = 8, 32, 2048, 128
    G = Hq // Hkv
    g = torch.Generator().manual_seed(17)
    q = torch.randn((B, Hq, S, D), generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn((B, Hkv, S, D), generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn((B, Hkv, S, D), generator=g).to(torch.bfloat16).to(DEV)
    dout = torch.randn((B, Hq, S, D), generator=g).to(torch.bfloat16).to(DEV)
    scale = D ** -0.5
    plan = lowering.AttnPlan(mask=mask, window=window, scale=scale)
    lse = torch.empty((B, Hq, S), dtype=torch.float32, device=DEV)
    o = lowering.attention(q, k, v, plan, lse=lse)
    dq, dk, dv = lowering.attention_backward(q, k, v, o, lse, dout, plan)
    worst = {"dq": 0.0, "dk": 0.0, "dv": 0.0}
    for b in range(B):
        for hk in range(Hkv):
            hs = slice(hk * G, (hk + 1) * G)
            rq, rk, rv = _ref_head_fp32(q[b, hs], k[b, hk], v[b, hk], dout[b, hs], mask, window, scale)
            for nm, got, want in (("dq", dq[b, hs], rq), ("dk", dk[b, hk], rk), ("dv", dv[b, hk], rv)):
                rel = ((got.float() - want).norm() / want.norm()).item()
                err = (got.float() - want).abs().max().item() / max(1.0, want.abs().max().item())
                worst[nm] = max(worst[nm], rel)
                assert rel <= 2e-2 and err <= 4e-2, f"{name} {nm} batch {b} kv head {hk}: relative {rel}, max abs {err}"
    assert all(w > 0.0 for w in worst.values())       # the comparison saw data


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,D,mask,window,dtype,cap,qscale", [
    (1, 4, 4, 256, 256, 128, "causal", 0, torch.bfloat16, 30.0, 1.0),
    (1, 8, 2, 320, 320, 128, "sliding", 96, torch.bfloat16, 30.0, 1.0),
    (1, 2, 2, 200, 333, 64, None, 0, torch.float16, 2.0, 3.0),          # a cap that bites: |scores| reach several caps
    (1, 2, 1, 130, 130, 64, "causal", 0, torch.float16, -5.0, 2.0),      # cap given with a minus sign
])
def test_backward_with_softcap_matches_autograd(B, Hq, Hkv, Sq, Sk, D, mask, window, dtype, cap, qscale):
    g = torch.Generator().manual_seed(Sq * 5 + Sk + D)
    q = (torch.randn((B, Hq, Sq, D), generator=g) * qscale).to(dtype).to(DEV)
    k, v = (torch.randn((B, Hkv, Sk, D), generator=g).to(dtype).to(DEV) for _ in range(2))
    dout = torch.randn((B, Hq, Sq, D), generator=g).to(dtype).to(DEV)
    scale = D ** -0.5
    plan = lowering.AttnPlan(mask=mask, window=window, scale=scale, softcap=cap)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=DEV)
    o = lowering.attention(q, k, v, plan, lse=lse)
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = _ref(q, k, v, dout, mask, window, scale, cap)
    tol = 2e-2 if dtype == torch.bfloat16 else 5e-3
    assert (o.double() - o_ref).abs().max().item() <= tol
    torch.testing.assert_close(lse.double(), lse_ref, rtol=1e-3, atol=4e-3)
    dq, dk, dv = lowering.attention_backward(q, k, v, o, lse, dout, plan)
    for name, got, want in (("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
        rel = ((got.double() - want).norm() / want.norm()).item()
        assert rel <= (2e-2 if dtype == torch.bfloat16 else 5e-3), f"{name}: relative error {rel}"
        err = (got.double() - want).abs().max().item()
        assert err <= (4e-2 if dtype == torch.bfloat16 else 1e-2) * max(1.0, want.abs().max().item()), f"{name}: max abs err {err}"


def test_backward_is_reproducible_and_refuses_what_it_does_not_serve():
    g = torch.Generator().manual_seed(5)
    q, k, v, dout = (torch.randn((1, 2, 256, 128), generator=g).to(torch.bfloat16).to(DEV) for _ in range(4))
    plan = lowering.AttnPlan(mask="causal", scale=128 ** -0.5)
    lse = torch.empty((1, 2, 256), dtype=torch.float32, device=DEV)
    o = lowering.attention(q, k, v, plan, lse=lse)
    a = lowering.attention_backward(q, k, v, o, lse, dout, plan)
    b = lowering.attention_backward(q, k, v, o, lse, dout, plan)
    assert all(torch.equal(x, y) for x, y in zip(a, b))          # no atomics: bit for bit
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention_backward(q, k, v, o, lse, dout, lowering.AttnPlan(mask="causal", scale=0.1, denom_add=1.0))
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention_backward(q, k, v, o, lse, dout, lowering.AttnPlan(mask="causal", scale=0.1, softcap=0.0))


def test_training_ops_repack_views_beyond_the_direct_loads_reach():
    """K rows 4 MiB apart (a view into a 4 GiB tensor) lie beyond the 32-bit offsets of the direct-to-LDS loads:
    the operator refuses them, and the custom ops of a training graph go through packed copies instead of
    aborting -- same values as on packed operands."""
    from loopfuse_amd.torch_backend import training

    S, D, R = 1025, 128, 1 << 21
    g = torch.Generator().manual_seed(9)
    q, k, v, dout = (torch.randn((1, 1, S, D), generator=g).to(torch.bfloat16).to(DEV) for _ in range(4))
    wide = torch.empty((1, 1, S, R), dtype=torch.bfloat16, device=DEV)
    wide[..., :D] = k
    k_view = wide[..., :D]
    plan = lowering.AttnPlan(mask="causal", scale=D ** -0.5)
    lse = torch.empty((1, 1, S), dtype=torch.float32, device=DEV)
    with pytest.raises(lowering.UnsupportedPlan):
        lowering.attention(q, k_view, v, plan, lse=lse, choice={"prefill": "swp"})
    before = training.counters["repacked"]
    o1, lse1 = torch.ops.loopfuse_amd.attention_fwd(q, k_view, v, 1, 0, D ** -0.5, 0.0)
    o2, lse2 = torch.ops.loopfuse_amd.attention_fwd(q, k, v, 1, 0, D ** -0.5, 0.0)
    assert torch.equal(o1, o2) and torch.equal(lse1, lse2)
    g1 = torch.ops.loopfuse_amd.attention_bwd(q, k_view, v, o1, lse1, dout, 1, 0, D ** -0.5, 0.0)
    g2 = torch.ops.loopfuse_amd.attention_bwd(q, k, v, o2, lse2, dout, 1, 0, D ** -0.5, 0.0)
    assert all(torch.equal(a, b) for a, b in zip(g1, g2))
    assert training.counters["repacked"] == before + 2
    del wide


# ---- through torch.compile(backend=loopfuse_backend): graphs traced for training
def _train_case(name):
    from loopfuse_amd import workloads  # noqa: F401

    def causal(q, k, v):
        s = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(s), dim=-1) @ v

    def sliding_gqa(q, k, v):
        g = q.shape[1] // k.shape[1]
        kk, vv = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
        s = q @ kk.transpose(-2, -1) / math.sqrt(q.shape[-1])
        return torch.softmax(torch.ops.loopfuse.sliding_mask(s, 96), dim=-1) @ vv

    def plain_bshd(q, k, v):            # [B, S, H, D] storage viewed transposed, no mask
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))
        return (torch.softmax(q @ k.transpose(-2, -1) * 0.125, dim=-1) @ v).transpose(1, 2)

    def capped(q, k, v):                # config 2 + softcap as the reference spells it (tests/benchmark.py:142-147)
        s = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
        s = 30.0 * torch.tanh(s / 30.0)
        return torch.softmax(torch.ops.loopfuse.causal_mask(s), dim=-1) @ v

    def tril_by_hand(q, k, v):          # the common GPT module: the triangle built in the graph, filled with -inf
        T = q.shape[-2]
        att = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(k.size(-1)))
        att = att.masked_fill(torch.tril(torch.ones(T, T, device=q.device)).view(1, 1, T, T) == 0, float("-inf"))
        return torch.softmax(att, dim=-1) @ v

    if name == "tril_by_hand":
        return tril_by_hand, [(2, 4, 300, 64)] * 3, "causal", 0
    if name == "capped":
        return capped, [(1, 4, 256, 128)] * 3, "causal", 0
    if name == "causal":
        return causal, [(2, 4, 256, 128)] * 3, "causal", 0
    if name == "sliding_gqa":
        return sliding_gqa, [(1, 8, 320, 64), (1, 2, 320, 64), (1, 2, 320, 64)], "sliding", 96
    return plain_bshd, [(2, 192, 4, 64)] * 3, None, 0


@pytest.mark.parametrize("name", ["causal", "sliding_gqa", "plain_bshd", "capped", "tril_by_hand"])
def test_training_graph_runs_the_fused_forward_and_backward(name):
    """``torch.compile(backend=loopfuse_backend)`` on a function whose inputs require grad: the
    forward and the backward graph both run the HIP kernels (counted), and the gradients match
    float64 autograd on the eager graph."""
    from loopfuse_amd import loopfuse_backend
    from loopfuse_amd.torch_backend import interface, training

    fn, shapes, mask, window = _train_case(name)
    g = torch.Generator().manual_seed(11)
    leaves = [torch.randn(s, generator=g).to(torch.bfloat16).to(DEV).requires_grad_(True) for s in shapes]
    refs = [t.detach().double().requires_grad_(True) for t in leaves]
    torch._dynamo.reset()
    before, ops_before = dict(interface.stats), dict(training.counters)
    out = torch.compile(fn, backend=loopfuse_backend)(*leaves)
    dout = torch.randn(out.shape, generator=g).to(torch.bfloat16).to(DEV)
    out.backward(dout)
    want = fn(*refs)
    want.backward(dout.double())
    assert interface.stats["training_graphs"] == before["training_graphs"] + 1
    assert interface.stats["eager_training"] == before["eager_training"]
    assert training.counters["fwd"] == ops_before["fwd"] + 1 and training.counters["bwd"] == ops_before["bwd"] + 1
    assert (out.double() - want).abs().max().item() <= 2e-2
    for got, ref in zip(leaves, refs):
        rel = ((got.grad.double() - ref.grad).norm() / ref.grad.norm()).item()
        assert rel <= 2e-2, rel


def test_training_graph_with_an_unserved_attention_stays_unfused():
    from loopfuse_amd import loopfuse_backend
    from loopfuse_amd.torch_backend import interface

    def biased(q, k, v, bias):          # an additive score bias: fused for inference, no backward kernel
        s = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5) + bias
        return torch.softmax(torch.ops.loopfuse.causal_mask(s), dim=-1) @ v

    leaves = [torch.randn((1, 2, 128, 64), generator=torch.Generator().manual_seed(s)).to(torch.bfloat16).to(DEV).requires_grad_(True)
              for s in range(3)]
    bias = torch.randn((1, 2, 128, 128), generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).to(DEV)
    torch._dynamo.reset()
    before = dict(interface.stats)
    out = torch.compile(biased, backend=loopfuse_backend)(*leaves, bias)
    out.sum().backward()
    assert interface.stats["training_graphs"] == before["training_graphs"]
    assert interface.stats["eager_training"] > before["eager_training"]
    assert leaves[0].grad is not None and torch.isfinite(leaves[0].grad.float()).all()


@pytest.mark.parametrize("spelling", ["mask_op", "sdpa_view", "sdpa_gqa"])
def test_module_with_projections_trains_with_the_fused_attention(spelling):
    """A block with parameters (qkv projection, attention, output projection) compiled with
    static shapes and called outside ``torch.no_grad()``: the attention in the middle runs the
    fused forward and backward, the projections around it stay ATen ops, and the parameter
    gradients match the uncompiled module.  The attention spelled with the reference's mask op, or
    as ``F.scaled_dot_product_attention(is_causal=True)`` whose output is viewed without a copy
    (the view relies on the op's [B, S, H, D] memory order), also with grouped kv heads."""
    import torch.nn.functional as F

    from loopfuse_amd import loopfuse_backend
    from loopfuse_amd.torch_backend import interface, training

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            torch.manual_seed(0)
            self.kvh = 2 if spelling == "sdpa_gqa" else 4
            self.qkv = torch.nn.Linear(256, 256 + 2 * 64 * self.kvh, bias=False)
            self.out = torch.nn.Linear(256, 256, bias=False)

        def forward(self, x):
            B, S, E = x.shape
            q, k, v = self.qkv(x).split([256, 64 * self.kvh, 64 * self.kvh], dim=-1)
            q = q.view(B, S, 4, 64).transpose(1, 2)
            k, v = (t.view(B, S, self.kvh, 64).transpose(1, 2) for t in (k, v))
            if spelling == "mask_op":
                a = torch.softmax(torch.ops.loopfuse.causal_mask(q @ k.transpose(-2, -1) * 0.125), dim=-1) @ v
                return self.out(a.transpose(1, 2).reshape(B, S, E))
            a = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=spelling == "sdpa_gqa")
            return self.out(a.transpose(1, 2).view(B, S, E))

    m = Block().to(DEV).to(torch.bfloat16)
    x = (torch.randn((2, 192, 256), generator=torch.Generator().manual_seed(3)) * 0.5).to(torch.bfloat16).to(DEV)
    torch._dynamo.reset()
    before, ops_before = dict(interface.stats), dict(training.counters)
    y = torch.compile(m, backend=loopfuse_backend)(x)
    y.float().square().mean().backward()
    got = {n: p.grad.float().clone() for n, p in m.named_parameters()}
    m.zero_grad()
    y_ref = m(x)
    y_ref.float().square().mean().backward()
    assert interface.stats["training_graphs"] == before["training_graphs"] + 1
    assert training.counters["fwd"] == ops_before["fwd"] + 1 and training.counters["bwd"] == ops_before["bwd"] + 1
    assert (y.float() - y_ref.float()).abs().max() <= 2e-2
    for n, p in m.named_parameters():
        ref = p.grad.float()
        assert ((got[n] - ref).norm() / ref.norm()).item() <= 3e-2, n
