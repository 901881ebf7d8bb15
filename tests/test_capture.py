"""Front end on the CPU: custom-op semantics, graph capture -> plan, CODEGEN_ONLY-style
compilation of the matched kernels, and eager fallback for everything else."""
import math

import pytest
import torch

import loopfuse_amd  # noqa: F401  (registers torch.ops.loopfuse.*)
from loopfuse_amd import lowering
from loopfuse_amd.torch_backend import capture, interface
from oracle import attention_oracle as O
from torch._functorch.aot_autograd import aot_module_simplified


def test_custom_op_semantics():
    g = torch.Generator().manual_seed(0)
    a = torch.randn(2, 3, 6, 6, generator=g)
    assert torch.equal(torch.ops.loopfuse.causal_mask(a), a.masked_fill(~O.dense_mask("causal", 6, 6), float("-inf")))
    assert torch.equal(torch.ops.loopfuse.sliding_mask(a, 3),
                       a.masked_fill(~O.dense_mask("sliding", 6, 6, 3), float("-inf")))
    run, fin = torch.ops.loopfuse.scan_max(a)
    assert torch.equal(run, torch.cummax(a, -1).values) and torch.equal(fin, a.max(-1, keepdim=True).values)
    buf = torch.randn(10, 4, 5, generator=g)
    tab = torch.randint(0, 10, (2, 3), generator=g, dtype=torch.int32)
    assert torch.equal(torch.ops.loopfuse.paged_load(buf, tab), buf[tab.long()])


def test_custom_op_gradients():
    """The operators' autograd formulas against the same functions spelled with
    differentiable torch ops (double precision), and against finite differences."""
    g = torch.Generator().manual_seed(1)
    a = torch.randn(2, 5, 5, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(2, 5, 5, generator=g, dtype=torch.float64)
    for op, keep in ((torch.ops.loopfuse.causal_mask, O.dense_mask("causal", 5, 5)),
                     (lambda x: torch.ops.loopfuse.sliding_mask(x, 2), O.dense_mask("sliding", 5, 5, 2))):
        (got,) = torch.autograd.grad((torch.softmax(op(a), -1) * w).sum(), a)
        (want,) = torch.autograd.grad((torch.softmax(a.masked_fill(~keep, float("-inf")), -1) * w).sum(), a)
        assert torch.allclose(got, want, atol=1e-12) and got[:, ~keep].abs().max() == 0
    run, fin = torch.ops.loopfuse.scan_max(a)
    (got,) = torch.autograd.grad((run * w).sum() + (fin * w[..., :1]).sum(), a)
    cm = torch.cummax(a, -1).values
    (want,) = torch.autograd.grad((cm * w).sum() + (cm[..., -1:] * w[..., :1]).sum(), a)
    assert torch.allclose(got, want, atol=1e-12)
    buf = torch.randn(7, 2, 3, generator=g, dtype=torch.float64, requires_grad=True)
    tab = torch.tensor([[1, 4, 1], [6, 1, 0]], dtype=torch.int32)          # page 1 is gathered three times
    wl = torch.randn(2, 3, 2, 3, generator=g, dtype=torch.float64)
    (got,) = torch.autograd.grad((torch.ops.loopfuse.paged_load(buf, tab) * wl).sum(), buf)
    (want,) = torch.autograd.grad((buf[tab.long()] * wl).sum(), buf)
    assert torch.allclose(got, want, atol=1e-12) and got[[2, 3, 5]].abs().max() == 0
    assert torch.autograd.gradcheck(lambda x: torch.ops.loopfuse.paged_load(x, tab), (buf,))
    assert torch.autograd.gradcheck(lambda x: torch.softmax(torch.ops.loopfuse.sliding_mask(x, 3), -1), (a,))


def test_graph_traced_for_training_runs_unfused_and_differentiates():
    """Inputs that require grad (a module's parameters outside torch.no_grad()): the
    reference fails while tracing (its operators have no autograd formula); here the
    graph runs as captured and gradients equal those of the uncompiled function."""
    def fn(q, k, v):
        s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
        return torch.softmax(torch.ops.loopfuse.causal_mask(s), dim=-1) @ v

    g = torch.Generator().manual_seed(2)
    ins = [torch.randn(1, 2, 24, 16, generator=g, requires_grad=True) for _ in range(3)]
    ref = [t.detach().clone().requires_grad_() for t in ins]
    torch._dynamo.reset()
    before = dict(interface.stats)
    out = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
    out.square().sum().backward()
    fn(*ref).square().sum().backward()
    for a, b in zip(ins, ref):
        assert torch.allclose(a.grad, b.grad, atol=1e-5, rtol=1e-5)
    assert interface.stats["eager_training"] - before["eager_training"] == 2      # forward and backward graph
    assert interface.stats["fused"] == before["fused"] and interface.stats["matched_graphs"] == before["matched_graphs"]
    # the same function under no_grad takes the matching route
    torch._dynamo.reset()
    with torch.no_grad():
        torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
    assert interface.stats["matched_graphs"] == before["matched_graphs"] + 1


def test_strict_mode_refuses_training_graphs(monkeypatch):
    monkeypatch.setenv("LOOPFUSE_STRICT", "1")
    torch._dynamo.reset()
    x = torch.randn(1, 1, 8, 16, requires_grad=True)
    fn = lambda q: torch.softmax(torch.ops.loopfuse.causal_mask(q @ q.transpose(-2, -1)), -1) @ q
    with pytest.raises(Exception, match="forward-only"):
        torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(x)
    torch._dynamo.reset()


def capture_graph(fn, inputs, marks=()):
    """Trace fn with dynamic shapes and return the AttentionMatch (or the NoMatch)."""
    box = {}

    def backend(gm, sample):
        def fw(g, _):
            try:
                box["matches"] = capture.match_attention(g)
                box["match"] = box["matches"][0]
            except capture.NoMatch as e:
                box["nomatch"] = e
            box["gm"] = g
            return g.forward

        return aot_module_simplified(gm, sample, fw_compiler=fw)

    torch._dynamo.reset()
    for t, dim, kind in marks:
        (torch._dynamo.mark_static if kind == "static" else torch._dynamo.mark_dynamic)(t, dim)
    with torch.inference_mode():
        torch.compile(fn, backend=backend, dynamic=True)(*inputs)
    return box


def bf(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16)


def _flat_args(box, tensors):
    """The flat placeholder list of a call: ints for SymInt placeholders, tensors (in
    order of first use) otherwise."""
    it = iter(tensors)
    return [next(it) if isinstance(p.meta["val"], torch.Tensor) else int(p.meta["val"].node.hint)
            for p in box["gm"].graph.nodes if p.op == "placeholder"]


def _vals(box, m, tensors):
    """Run-time values of the fused call's inputs for a call with these tensors."""
    return m.input_values(box["gm"], _flat_args(box, tensors))


def test_capture_causal_static_head_dim():
    def fn(q, k, v):
        s = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(s), dim=-1) @ v

    q, k, v = bf(2, 4, 96, 64), bf(2, 4, 96, 64, seed=1), bf(2, 4, 96, 64, seed=2)
    m = capture_graph(fn, (q, k, v), [(q, 3, "static"), (q, 2, "dynamic")])["match"]
    assert m.mask == "causal" and not m.has_tanh and not m.k.paged
    assert (m.q.perm, m.k.perm, m.v.perm) == ((0, 1, 2, 3),) * 3


def test_capture_gqa_softcap_sliding_and_plan_values():
    def fn(Q, K, V):
        g = Q.shape[1] // K.shape[1]
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        s = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        s = torch.tanh(s / 30) * 30
        return torch.softmax(torch.ops.loopfuse.sliding_mask(s, 256), dim=-1) @ V

    q, k, v = bf(2, 8, 80, 64), bf(2, 2, 80, 64, seed=1), bf(2, 2, 80, 64, seed=2)
    box = capture_graph(fn, (q, k, v))
    m = box["match"]
    assert m.mask == "sliding" and m.has_tanh
    plan = m.plan_for(_vals(box, m, (q, k, v)))
    assert plan.mask == "sliding" and plan.window == 256
    assert plan.softcap == pytest.approx(30.0) and plan.scale == pytest.approx(64 ** -0.5, rel=1e-6)


def test_capture_modified_attention_biases():
    # reference tests/test_accuracy.py:172-196
    def fn(Q, qb, K, sb, V, ob):       # parameters in order of first use = placeholder order
        QK = (Q + qb) @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        QK = QK * 3.5 + sb
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V + ob

    q, k, v, qb = (bf(2, 4, 48, 64, seed=s) for s in range(4))
    sb, ob = bf(2, 4, 48, 48, seed=5), bf(2, 4, 48, 64, seed=6)
    box = capture_graph(fn, (q, qb, k, sb, v, ob))
    m = box["match"]
    assert m.mask == "causal" and m.inputs[m.q.index].op == "call_function"   # Q is the node Q + q_bias
    assert m.bias is not None and m.bias.dims == (0, 1, 2, 3) and m.inputs[m.bias.index].op == "placeholder"
    assert m.out_bias is not None and m.out_bias.dims == (0, 1, 2, 3)
    vals = _vals(box, m, (q, qb, k, sb, v, ob))
    plan = m.plan_for(vals)
    assert plan.scale == pytest.approx(3.5 * 64 ** -0.5, rel=1e-6)
    # views handed to the kernels: the inputs themselves, Q replaced by the eager sum
    assert torch.equal(m._operand(m.q, vals)[0], q + qb)
    assert m._bias_view(m.bias, vals, (2, 4, 48, 48)).data_ptr() == sb.data_ptr()


def test_capture_broadcast_and_transposed_bias():
    def fn(Q, K, bias, V):
        s = Q @ K.transpose(-2, -1) * 0.125 + bias.transpose(0, 1)      # stored [H, 1, Sq, Sk]
        return torch.softmax(s, dim=-1) @ V

    q, k, v = (bf(3, 4, 40, 64, seed=s) for s in range(3))
    bias = bf(4, 1, 40, 40, seed=4)
    box = capture_graph(fn, (q, k, bias, v))
    m = box["match"]
    assert m.bias.dims == (None, 0, 2, 3)                # batch broadcast, heads walk source dim 0
    view = m._bias_view(m.bias, _vals(box, m, (q, k, bias, v)), (3, 4, 40, 40))
    assert torch.equal(view, bias.transpose(0, 1).expand(3, 4, 40, 40))


def test_bias_after_mask_or_scaled_afterwards_is_not_matched():
    def scaled_after(Q, K, V, bias):
        s = (Q @ K.transpose(-2, -1) + bias) * 0.125
        return torch.softmax(s, dim=-1) @ V

    q, k, v = (bf(2, 2, 40, 64, seed=s) for s in range(3))
    box = capture_graph(scaled_after, (q, k, v, bf(2, 2, 40, 40, seed=4)))
    assert "match" not in box and "nomatch" in box


def test_capture_paged_decode():
    def fn(Q, Kc, kt, Vc, vt):
        K = torch.ops.loopfuse.paged_load(Kc, kt).transpose(-3, -2)
        V = torch.ops.loopfuse.paged_load(Vc, vt).transpose(-3, -2)
        s = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(s, dim=-1) @ V

    B, Hkv, grp, D, S = 3, 2, 4, 64, 32
    Kc, Vc = bf(B * S * 2, Hkv, D), bf(B * S * 2, Hkv, D, seed=1)
    g = torch.Generator().manual_seed(3)
    kt = torch.randint(0, B * S * 2, (B, S), generator=g, dtype=torch.int32)
    vt = torch.randint(0, B * S * 2, (B, S), generator=g, dtype=torch.int32)
    Q = bf(B, Hkv, grp, D, seed=2)
    m = capture_graph(fn, (Q, Kc, kt, Vc, vt))["match"]
    assert m.k.paged and m.v.paged and m.mask is None
    assert m.k.table_index != m.v.table_index


def test_capture_paged_page16_reshape():
    def fn(Q, Kc, kt, Vc, vt):
        B, pages = kt.shape
        P, H, D = Kc.shape[1:]
        K = torch.ops.loopfuse.paged_load(Kc, kt).reshape(B, pages * P, H, D).transpose(1, 2)
        V = torch.ops.loopfuse.paged_load(Vc, vt).reshape(B, pages * P, H, D).transpose(1, 2)
        g = Q.shape[1] // H
        K = K.repeat_interleave(g, dim=1)
        V = V.repeat_interleave(g, dim=1)
        s = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(s, dim=-1) @ V

    B, Hkv, grp, D, S, P = 3, 2, 4, 64, 64, 16
    n = B * S // P
    Kc, Vc = bf(n, P, Hkv, D), bf(n, P, Hkv, D, seed=1)
    tab = torch.randperm(n, generator=torch.Generator().manual_seed(3)).view(B, S // P).to(torch.int32)
    Q = bf(B, Hkv * grp, 1, D, seed=2)
    box = capture_graph(fn, (Q, Kc, tab, Vc, tab.clone()))
    assert "match" in box, box.get("nomatch")
    assert box["match"].k.paged and box["match"].v.paged


@pytest.mark.parametrize("which", ["gated_probs", "add", "softmax_matmul"])
def test_unrecognised_graphs_do_not_match(which):
    if which == "gated_probs":
        def fn(q, k, v, b):
            s = q @ k.transpose(-2, -1) * 0.125
            return (torch.softmax(torch.ops.loopfuse.causal_mask(s), dim=-1) * b) @ v
        ins = (bf(1, 2, 32, 64), bf(1, 2, 32, 64, seed=1), bf(1, 2, 32, 64, seed=2), bf(1, 2, 32, 32, seed=3))
    elif which == "add":
        def fn(a, b):
            return a + b
        ins = (bf(4, 8), bf(4, 8, seed=1))
    else:
        def fn(x, y):
            return torch.softmax(x, dim=-1) @ y
        ins = (bf(2, 2, 16, 8), bf(2, 2, 8, 16, seed=1))
    box = capture_graph(fn, ins)
    assert "match" not in box and "nomatch" in box


def _oracle_run(self, vals):
    """Stand-in for AttentionMatch.run on the CPU: same operand plumbing, oracle arithmetic."""
    q, _ = self._operand(self.q, vals)
    k, kt = self._operand(self.k, vals)
    v, vt = self._operand(self.v, vals)
    B, Hq, Sq, Sk, D = self._shapes(vals)
    plan = self.plan_for(vals)
    out = O.attention_reference(q, k, v, mask=plan.mask, window=plan.window, scale=plan.scale, softcap=plan.softcap,
                                k_table=kt, v_table=vt, denom_add=plan.denom_add,
                                score_bias=self._bias_view(self.bias, vals, (B, Hq, Sq, Sk)),
                                out_bias=self._bias_view(self.out_bias, vals, (B, Hq, Sq, D)),
                                **self._second_product(vals)).to(q.dtype)
    if plan.zero_blind_rows:
        out = out.nan_to_num(nan=0.0)
    return self.empty_out(vals, out.dtype, out.device).copy_(out.reshape(self.out_shape(vals)))


def _explicit_softmax(X, base2=True, c=1.0):
    """The reference's hand-written online-softmax hint (tests/test_attention.py:95-107)."""
    Xf = X.to(torch.float32)
    if base2:
        Xf = Xf * 1 / math.log(2)
    run, fin = torch.ops.loopfuse.scan_max(Xf)
    ex = torch.exp2 if base2 else torch.exp
    e = ex(Xf - run) * ex(run - fin)
    return e / (torch.sum(e, dim=-1, keepdim=True) + c)


def test_capture_explicit_softmax_with_shifted_denominator():
    def fn(Q, K, V):
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return _explicit_softmax(torch.ops.loopfuse.causal_mask(QK)).to(Q.dtype) @ V

    q, k, v = (bf(2, 4, 48, 64, seed=s) for s in range(3))
    box = capture_graph(fn, (q, k, v), [(q, 3, "static"), (q, 2, "dynamic")])
    m = box["match"]
    assert m.mask == "causal" and m.denom_add == (1.0,) and m.base2
    plan = m.plan_for(_vals(box, m, (q, k, v)))
    assert plan.denom_add == 1.0 and plan.scale == pytest.approx(64 ** -0.5, rel=1e-6)   # 1/ln2 and ln2 cancel


@pytest.mark.parametrize("which", ["two_outputs", "prefix", "inside_block", "modified", "softmax1", "softmax_e",
                                   "mla", "mla_shared_rope", "double_k", "einsum", "rank3", "bshd",
                                   "sdpa_causal_gqa", "sdpa_scale_expand", "sdpa_bshd_block", "sdpa_bool_mask",
                                   "sdpa_float_mask"])
def test_rewritten_graphs_compute_the_same(which, monkeypatch):
    """Sub-graph fusion: the attention(s) inside a larger graph are replaced by fused
    calls and the rest keeps running.  Here the fused call is the oracle (no GPU), so
    the test pins the rewrite and the operand plumbing (reference graphs:
    tests/test_attention.py:72-92, 339-362)."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)
    f32 = lambda *shape, seed=0: torch.randn(*shape, generator=torch.Generator().manual_seed(seed))
    if which == "two_outputs":
        def fn(q, k, v):
            p = torch.softmax(q @ k.transpose(-2, -1), dim=-1)
            return p @ v, p
        ins, n_attn = (f32(1, 2, 32, 64), f32(1, 2, 32, 64, seed=1), f32(1, 2, 32, 64, seed=2)), 1
    elif which == "prefix":
        def fn(Q, Kp, Vp, Ks, Vs):
            QKp = Q @ Kp.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
            QKs = Q @ Ks.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
            return torch.softmax(QKp, dim=-1) @ Vp + torch.softmax(torch.ops.loopfuse.causal_mask(QKs), dim=-1) @ Vs
        ins = (f32(3, 2, 24, 64), f32(3, 2, 40, 64, seed=1), f32(3, 2, 40, 64, seed=2),
               f32(3, 2, 24, 64, seed=3), f32(3, 2, 24, 64, seed=4))
        n_attn = 2
    elif which == "inside_block":
        def fn(x, wq, wk, wv, wo):
            B, S, E = x.shape
            H = 4
            q = (x @ wq).view(B, S, H, E // H).transpose(1, 2)
            k = (x @ wk).view(B, S, H, E // H).transpose(1, 2)
            v = (x @ wv).view(B, S, H, E // H).transpose(1, 2)
            a = torch.softmax(torch.ops.loopfuse.causal_mask(q @ k.transpose(-2, -1) * 0.125), dim=-1) @ v
            return a.transpose(1, 2).reshape(B, S, E) @ wo + x
        ins = (f32(2, 24, 256),) + tuple(f32(256, 256, seed=s) * 0.06 for s in (1, 2, 3, 4))
        n_attn = 1
    elif which in ("mla", "mla_shared_rope"):
        # two-part scores (reference tests/test_attention.py:126-151); the second variant
        # writes the small product first and shares its key across heads
        shared = which == "mla_shared_rope"

        def fn(Q_nope, Q_pe, K_nope, K_pe, V):
            if shared:
                qk = Q_pe @ K_pe.expand(-1, Q_pe.shape[1], -1, -1).transpose(-2, -1) + Q_nope @ K_nope.transpose(-2, -1)
            else:
                qk = Q_nope @ K_nope.transpose(-2, -1) + Q_pe @ K_pe.transpose(-2, -1)
            qk = qk * (Q_nope.shape[-1] + Q_pe.shape[-1]) ** (-0.5)
            return torch.softmax(torch.ops.loopfuse.causal_mask(qk), dim=-1) @ V
        ins = (f32(2, 3, 40, 64), f32(2, 3, 40, 16, seed=1), f32(2, 3, 40, 64, seed=2),
               f32(2, 1 if shared else 3, 40, 16, seed=3), f32(2, 3, 40, 64, seed=4))
        n_attn = 1
    elif which in ("einsum", "rank3", "bshd"):
        # other spellings of the same attention: einsum (lowers to view -> permute -> view
        # chains around both products), inputs without a batch dim, [B, S, H, D] storage
        def fn(Q, K, V):
            if which == "einsum":
                sc = torch.einsum("bhqd,bhkd->bhqk", Q, K) * (Q.shape[-1] ** -0.5)
                return torch.einsum("bhqk,bhkd->bhqd", torch.softmax(torch.ops.loopfuse.causal_mask(sc), dim=-1), V)
            if which == "bshd":
                Q, K, V = (t.transpose(1, 2) for t in (Q, K, V))
            o = torch.softmax(torch.ops.loopfuse.causal_mask(Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)), dim=-1) @ V
            return o.transpose(1, 2) if which == "bshd" else o
        shape = {"einsum": (2, 3, 40, 64), "rank3": (6, 40, 64), "bshd": (2, 40, 3, 64)}[which]
        ins, n_attn = (f32(*shape), f32(*shape, seed=1), f32(*shape, seed=2)), 1
    elif which.startswith("sdpa"):
        # torch's own fused attention call: one aten._scaled_dot_product_* node in the graph
        import torch.nn.functional as F
        if which == "sdpa_causal_gqa":          # default scale, kv heads grouped by the op itself
            fn = lambda Q, K, V: F.scaled_dot_product_attention(Q, K, V, is_causal=True, enable_gqa=True)
            ins = (f32(2, 8, 40, 64), f32(2, 2, 40, 64, seed=1), f32(2, 2, 40, 64, seed=2))
        elif which == "sdpa_scale_expand":      # explicit scale, one kv head expanded, rectangular, something after it
            fn = lambda Q, K, V: F.scaled_dot_product_attention(Q, K.expand(-1, 4, -1, -1), V.expand(-1, 4, -1, -1),
                                                                scale=0.3) + 1
            ins = (f32(2, 4, 24, 64), f32(2, 1, 56, 64, seed=1), f32(2, 1, 56, 64, seed=2))
        elif which in ("sdpa_bool_mask", "sdpa_float_mask"):
            # a mask tensor: torch hands it to the op as an additive term (0 / -inf for booleans)
            fn = lambda Q, K, V, M: F.scaled_dot_product_attention(Q, K, V, attn_mask=M)
            if which == "sdpa_bool_mask":
                m = torch.rand(2, 1, 24, 40, generator=torch.Generator().manual_seed(5)) > 0.3
                m[..., 0] = True                # no row without a visible key
            else:
                m = f32(1, 4, 24, 40, seed=5)
            ins = (f32(2, 4, 24, 64), f32(2, 4, 40, 64, seed=1), f32(2, 4, 40, 64, seed=2), m)
        else:                                   # the usual module spelling: [B, S, H*D] -> heads -> attention -> back
            def fn(x, wqkv, wo):
                B, S, E = x.shape
                q, k, v = ((x @ w).view(B, S, 4, E // 4).transpose(1, 2) for w in wqkv.unbind(0))
                a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
                return a.transpose(1, 2).reshape(B, S, E) @ wo
            ins = (f32(2, 24, 256), f32(3, 256, 256, seed=1) * 0.06, f32(256, 256, seed=2) * 0.06)
        n_attn = 1
    elif which == "double_k":
        # reference tests/test_attention.py:441-462 with its commented-out tail restored
        def fn(Q, K, K2, V):
            QK1 = Q[..., :64] @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
            QK2 = Q[..., 64:] @ K2.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
            return torch.softmax(torch.ops.loopfuse.causal_mask(QK1 + QK2), dim=-1) @ V
        ins = (f32(2, 3, 24, 96), f32(2, 3, 24, 64, seed=1), f32(2, 3, 24, 32, seed=2), f32(2, 3, 24, 64, seed=3))
        n_attn = 1
    elif which in ("softmax1", "softmax_e"):
        base2, c = (True, 1.0) if which == "softmax1" else (False, 0.25)

        def fn(Q, K, V):
            QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
            return _explicit_softmax(torch.ops.loopfuse.causal_mask(QK), base2, c).to(Q.dtype) @ V
        ins, n_attn = (f32(2, 3, 40, 64), f32(2, 3, 40, 64, seed=1), f32(2, 3, 40, 64, seed=2)), 1
    else:
        def fn(Q, qb, K, sb, V, ob):
            QK = (Q + qb) @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
            return torch.softmax(torch.ops.loopfuse.causal_mask(QK * 3.5 + sb), dim=-1) @ V + ob
        ins = (f32(2, 3, 24, 64), f32(2, 3, 24, 64, seed=1), f32(2, 3, 24, 64, seed=2), f32(2, 3, 24, 24, seed=3),
               f32(2, 3, 24, 64, seed=4), f32(2, 3, 24, 64, seed=5))
        n_attn = 1
    torch._dynamo.reset()
    before = dict(interface.stats)
    got = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
    assert interface.stats["fused"] == before["fused"] + 1
    assert len(interface.last_matches) == n_attn
    want = fn(*ins)
    for g, w in zip(got if isinstance(got, tuple) else (got,), want if isinstance(want, tuple) else (want,)):
        torch.testing.assert_close(g, w, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("which", ["buffer_eq_zero", "tril_in_graph", "arange_where", "where_full_like",
                                   "where_masked_first", "key_padding", "band_not_causal"])
def test_boolean_masks_written_by_hand_are_fused(which, monkeypatch):
    """Masks spelled with ``masked_fill`` / ``where`` on a boolean tensor (a registered buffer cut to
    the sequence, ``ones().tril()``, ``arange`` comparisons, a key-padding mask), filled with -inf:
    the attention is fused with the mask as a 0 / -inf score term, whatever shape the mask has."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)
    f32 = lambda *shape, seed=0: torch.randn(*shape, generator=torch.Generator().manual_seed(seed))
    S, Sk, D = 24, 40, 64
    ninf = float("-inf")
    q, k, v = f32(2, 3, S, D), f32(2, 3, S, D, seed=1), f32(2, 3, S, D, seed=2)
    kr, vr = f32(2, 3, Sk, D, seed=3), f32(2, 3, Sk, D, seed=4)
    if which == "buffer_eq_zero":
        def fn(q, k, v, buf):                  # the mask of a 64-token context cut to the sequence at hand
            T = q.shape[-2]
            att = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(k.size(-1)))
            return torch.softmax(att.masked_fill(buf[:, :, :T, :T] == 0, ninf), dim=-1) @ v
        ins = (q, k, v, torch.tril(torch.ones(64, 64)).view(1, 1, 64, 64))
    elif which == "tril_in_graph":
        def fn(q, k, v):                       # bottom-right aligned on a rectangular problem
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            m = torch.ones(q.shape[-2], k.shape[-2], dtype=torch.bool).tril(diagonal=k.shape[-2] - q.shape[-2])
            return torch.softmax(s.masked_fill(~m, ninf), -1) @ v
        ins = (q, kr, vr)
    elif which == "arange_where":
        def fn(q, k, v):
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            i, j = torch.arange(q.shape[-2])[:, None], torch.arange(k.shape[-2])[None, :]
            return torch.softmax(torch.where(j <= i, s, ninf), -1) @ v
        ins = (q, k, v)
    elif which == "where_full_like":
        def fn(q, k, v, m):
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            return torch.softmax(torch.where(m, s, torch.full_like(s, ninf)), -1) @ v
        ins = (q, k, v, torch.ones(S, S, dtype=torch.bool).tril())
    elif which == "where_masked_first":
        def fn(q, k, v, m):
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            return torch.softmax(torch.where(m, ninf, s), -1) @ v
        ins = (q, k, v, torch.ones(S, S, dtype=torch.bool).triu(diagonal=1))
    elif which == "key_padding":
        def fn(q, k, v, pad):                  # [B, Sk] True = padding
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            return torch.softmax(s.masked_fill(pad[:, None, None, :], ninf), -1) @ v
        pad = torch.zeros(2, Sk, dtype=torch.bool)
        pad[0, 30:] = True
        pad[1, 17:] = True
        ins = (q, kr, vr, pad)
    else:
        def fn(q, k, v):                       # a symmetric band: neither of the two mask flags
            s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
            i, j = torch.arange(q.shape[-2])[:, None], torch.arange(k.shape[-2])[None, :]
            return torch.softmax(s.masked_fill((i - j).abs() >= 5, ninf), -1) @ v
        ins = (q, k, v)
    torch._dynamo.reset()
    before = dict(interface.stats)
    with torch.no_grad():
        got = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
    assert interface.stats["fused"] == before["fused"] + 1
    (m,) = interface.last_matches
    if which == "arange_where":            # a mask built from indices alone that is the causal triangle: a flag
        assert m.mask == "causal" and m.bias is None
    else:
        assert m.mask is None and m.bias is not None and m.bias.keep in (1, -1)
    torch.testing.assert_close(got, fn(*ins), rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("fill", [-1e9, 0.0, torch.finfo(torch.float32).min])
def test_finite_fill_values_are_not_taken_for_masks(fill):
    """A finite fill value replaces the score; only -inf can be read as an additive term (a row whose
    keys are all filled differs otherwise), so these graphs run as captured."""
    def fn(q, k, v, m):
        s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
        return torch.softmax(s.masked_fill(~m, fill), -1) @ v
    f32 = lambda *shape, seed=0: torch.randn(*shape, generator=torch.Generator().manual_seed(seed))
    ins = (f32(1, 2, 24, 64), f32(1, 2, 24, 64, seed=1), f32(1, 2, 24, 64, seed=2), torch.ones(24, 24, dtype=torch.bool).tril())
    box = capture_graph(fn, ins)
    assert "match" not in box


@pytest.mark.parametrize("which", ["on_zeros", "on_a_bias", "beta_zero", "scaled_bias"])
def test_scores_spelled_with_baddbmm(which, monkeypatch):
    """``torch.baddbmm(zeros, q, k^T, beta=1, alpha=scale)`` on operands merged to [B*H, S, D] (the
    GPT-NeoX / Falcon spelling): the zeros are read as such from the graph and dropped, a real tensor
    becomes the score bias, a bias scaled by beta stays unfused."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)
    f32 = lambda *shape, seed=0: torch.randn(*shape, generator=torch.Generator().manual_seed(seed))
    B, H, S, D = 2, 3, 24, 64

    def fn(q, k, v, bias):
        bs, nh, ql, hd = q.shape
        qq, kk = q.view(bs * nh, ql, hd), k.view(bs * nh, k.size(-2), hd)
        base = torch.zeros(bs * nh, ql, k.size(-2), dtype=q.dtype) if which in ("on_zeros", "beta_zero") else bias
        beta = {"on_zeros": 1.0, "on_a_bias": 1.0, "beta_zero": 0.0, "scaled_bias": 0.5}[which]
        scores = torch.baddbmm(base, qq, kk.transpose(1, 2), beta=beta, alpha=hd ** -0.5).view(bs, nh, ql, -1)
        w = torch.softmax(torch.ops.loopfuse.causal_mask(scores), dim=-1)
        return torch.matmul(w, v)

    ins = (f32(B, H, S, D), f32(B, H, S, D, seed=1), f32(B, H, S, D, seed=2), f32(B * H, S, S, seed=3))
    torch._dynamo.reset()
    before = dict(interface.stats)
    with torch.no_grad():
        got = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
    fused = interface.stats["fused"] - before["fused"]
    assert fused == (0 if which == "scaled_bias" else 1)
    if fused:
        (m,) = interface.last_matches
        assert m.mask == "causal" and (m.bias is not None) == (which == "on_a_bias")
    torch.testing.assert_close(got, fn(*ins), rtol=2e-4, atol=2e-4)


def test_dynamic_width_split_into_heads(monkeypatch):
    """``qkv.chunk(3, -1)`` of a tensor whose width is a symbol: head dim (s + 2) // 12.  The stand-in
    sizes must divide as the traced ones do (an arbitrary stand-in once gave a head dim of 0)."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)
    B, N, H, D = 2, 24, 4, 64

    def fn(qkv):
        q, k, v = qkv.chunk(3, dim=-1)
        sh = lambda t: t.view(B, N, H, D).transpose(1, 2)
        return F.scaled_dot_product_attention(sh(q), sh(k), sh(v), is_causal=True).transpose(1, 2).reshape(B, N, H * D)

    import torch.nn.functional as F
    x = torch.randn(B, N, 3 * H * D, generator=torch.Generator().manual_seed(0))
    torch._dynamo.reset()
    before = dict(interface.stats)
    with torch.no_grad():
        got = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(x)
    assert interface.stats["fused"] == before["fused"] + 1 and interface.stats["match_errors"] == before["match_errors"]
    torch.testing.assert_close(got, fn(x), rtol=2e-4, atol=2e-4)


def test_constant_tensors_in_the_graph_do_not_stop_the_fusion(monkeypatch):
    """``torch.tensor([...])`` inside the traced function becomes an attribute of the graph; the
    attention beside it is fused all the same, and a constant can be one of its operands (a bias)."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)
    outer = torch.linspace(-1.0, 1.0, 24)              # one value per key

    def fn(q, k, v):
        s = q @ k.transpose(-2, -1) * 0.125 + outer[None, None, None, :]
        out = torch.softmax(torch.ops.loopfuse.causal_mask(s), -1) @ v
        return out * torch.tensor([1.0, 2.0, 3.0])[None, :, None, None]

    ins = [torch.randn(2, 3, 24, 64, generator=torch.Generator().manual_seed(s)) for s in range(3)]
    torch._dynamo.reset()
    before = dict(interface.stats)
    with torch.no_grad():
        got = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
    assert interface.stats["fused"] == before["fused"] + 1
    torch.testing.assert_close(got, fn(*ins), rtol=2e-4, atol=2e-4)


def test_an_error_inside_the_matcher_leaves_the_graph_running(monkeypatch):
    """The backend never fails a compilation because its own pattern matching broke: the graph runs
    as captured and the event is counted."""
    def boom(gm, *a, **kw):
        raise ZeroDivisionError("0.0 cannot be raised to a negative power")
    monkeypatch.setattr(capture, "match_attention", boom)
    from loopfuse_amd import compiler
    monkeypatch.setattr(compiler, "compile_graph", boom)          # the loop-nest front end (tried first) as well

    def fn(q, k, v):
        return torch.softmax(torch.ops.loopfuse.causal_mask(q @ k.transpose(-2, -1) * 0.125), -1) @ v
    ins = [torch.randn(1, 2, 16, 64, generator=torch.Generator().manual_seed(s)) for s in range(3)]
    torch._dynamo.reset()
    before = dict(interface.stats)
    with torch.no_grad():
        got = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
    assert interface.stats["match_errors"] == before["match_errors"] + 2 and interface.stats["fused"] == before["fused"]
    torch.testing.assert_close(got, fn(*ins))


def test_backend_on_cpu_tensors_runs_graph_unfused():
    """CPU tensors have no HIP path: the compiled function must still be correct (it
    runs the captured graph) and must say so in the stats."""
    def fn(q, k, v):
        s = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(s), dim=-1) @ v

    q, k, v = (torch.randn(1, 2, 48, 64, generator=torch.Generator().manual_seed(s)) for s in (0, 1, 2))
    torch._dynamo.reset()
    before = dict(interface.stats)
    out = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(q, k, v)
    assert torch.allclose(out, O.attention_reference(q, k, v, mask="causal"), atol=1e-5)
    assert interface.stats["matched_graphs"] == before["matched_graphs"] + 1
    assert interface.stats["eager_runtime"] == before["eager_runtime"] + 1
    assert interface.stats["fused"] == before["fused"]


def test_repeated_refusals_stop_the_attempts(monkeypatch):
    """A call the kernels cannot serve latches its argument layout: later calls with the same
    layout go straight to the captured graph (the part of the rewritten graph before the fused
    call is not run for nothing), a call with another layout is tried again."""
    attempts = []

    def refuse(self, vals):
        attempts.append(1)
        raise lowering.UnsupportedPlan("not served")

    monkeypatch.setattr(capture.AttentionMatch, "run", refuse)
    fn = lambda q, k, v: torch.softmax(q @ k.transpose(-2, -1), dim=-1) @ v
    q, k, v = (torch.randn(1, 2, 16, 64, generator=torch.Generator().manual_seed(s)) for s in (0, 1, 2))
    torch._dynamo.reset()
    before = dict(interface.stats)
    compiled = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)
    for _ in range(5):
        assert torch.allclose(compiled(q, k, v), fn(q, k, v), atol=1e-6)
    assert len(attempts) == 1 and interface.stats["eager_runtime"] == before["eager_runtime"] + 5
    assert interface.stats["refused_signatures"] == before["refused_signatures"] + 1
    # another layout of the same graph (a strided view of K) is a new signature: tried once more
    k2 = torch.randn(1, 2, 16, 128, generator=torch.Generator().manual_seed(3))[..., :64]
    graphs = interface.stats["compiled_graphs"]
    for _ in range(3):
        assert torch.allclose(compiled(q, k2, v), fn(q, k2, v), atol=1e-6)
    if interface.stats["compiled_graphs"] == graphs:      # same compiled graph served the new layout
        assert len(attempts) == 2


def test_unfused_graph_still_correct():
    def fn(a, b):
        return torch.relu(a) + b

    a, b = torch.randn(4, 8), torch.randn(4, 8)
    torch._dynamo.reset()
    out = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(a, b)
    assert torch.equal(out, torch.relu(a) + b)


def test_requested_specialisations_are_recorded_and_read_back(shim_built, monkeypatch, tmp_path):
    """LOOPFUSE_RECORD_SPECS: one line per specialisation asked for, first request only;
    specs_from_file gives the same KernelSpec objects back (extra options included)."""
    path = tmp_path / "specs.jsonl"
    monkeypatch.setenv("LOOPFUSE_RECORD_SPECS", str(path))
    monkeypatch.setattr(lowering, "_compiled", {})
    a = lowering.KernelSpec("decode", 0, 128, paged=3, page_size=16, rows=16, waves=8, headwave=True)
    b = lowering.KernelSpec("prefill", 1, 64, lowering.MASK_SLIDING, True, bias=5, extra=("-DLF_DMA=1",))
    for spec in (a, b, a):
        lowering.compile_spec(spec)
    assert len(path.read_text().splitlines()) == 2
    assert lowering.specs_from_file(str(path)) == [a, b]
    import __graft_entry__
    listed = __graft_entry__.standard_specs()
    assert len(listed) == len(set(listed)) and a in listed


def test_kernel_specs_compile_without_gpu(shim_built):
    spec = lowering.KernelSpec("prefill", 0, 128, lowering.MASK_CAUSAL)
    ck = lowering.compile_spec(spec)
    assert ck.code_object[:4] == b"\x7fELF"
    assert "lf_attn_prefill" in ck.code and "-DLF_MASK=1" in ck.code


def test_cpu_tensors_fail_loudly_on_direct_call():
    q = torch.randn(1, 1, 16, 64).to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        lowering.attention(q, q, q, lowering.AttnPlan(scale=0.125))


def test_codegen_only_returns_kernel_objects_without_a_gpu(shim_built, monkeypatch):
    """CODEGEN_ONLY=1 (reference interface.py:615-622, used as ``prg.code`` in
    tests/test_attention.py:28-29): the compiled callable returns what would be launched."""
    monkeypatch.setattr(interface, "CODEGEN_ONLY", True)

    def fn(Q, K, V):
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V

    q, k, v = (bf(2, 4, 256, 128, seed=s) for s in range(3))
    torch._dynamo.reset()
    prg = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(q, k, v)
    assert len(prg) == 1 and prg[0].code_object[:4] == b"\x7fELF"
    assert "-DLF_MASK=1" in prg.code and "lf_attn_prefill" in prg.code and "-DLF_HEAD_DIM=128" in prg.code

    def two(Q, Kp, Vp, Ks, Vs):      # two fused calls in one graph
        a = torch.softmax(Q @ Kp.transpose(-2, -1) * 0.1, dim=-1) @ Vp
        return a + torch.softmax(torch.ops.loopfuse.sliding_mask(Q @ Ks.transpose(-2, -1) * 0.1, 64), dim=-1) @ Vs

    torch._dynamo.reset()
    prg = torch.compile(two, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(q, k, v, k, v)
    assert len(prg) == 2 and "-DLF_MASK=0" in prg[0].code and "-DLF_MASK=2" in prg[1].code

    def decode(Q, K, V, M):          # one query row per head, grouped kv heads, a padding mask: the streaming kernel
        S = (Q @ K.repeat_interleave(4, dim=1).transpose(-2, -1)) * 0.125 + M
        return torch.softmax(S, dim=-1) @ V.repeat_interleave(4, dim=1)

    torch._dynamo.reset()
    prg = torch.compile(decode, backend=loopfuse_amd.loopfuse_backend, dynamic=True)(
        bf(2, 8, 1, 64), bf(2, 2, 320, 64, seed=1), bf(2, 2, 320, 64, seed=2), bf(2, 1, 1, 320, seed=3))
    assert len(prg) == 1 and "lf_attn_decode" in prg.code and "-DLF_BIAS=1" in prg.code


@pytest.mark.parametrize("which", ["causal", "gqa_window_softcap", "paged_decode", "block"])
def test_static_shapes_at_real_sizes_are_matched(which, monkeypatch):
    """torch.compile without dynamic=True traces static shapes: the literal sizes in the
    graph are then the real ones, too large for id tensors, and the front end has to shrink
    static dims and re-derive the literal view shapes.  The fused call is the oracle here."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)
    r = lambda *shape, seed=0: torch.randn(*shape, generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16)
    if which == "causal":
        def fn(Q, K, V):
            QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
            return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V
        ins = (r(4, 8, 1024, 128), r(4, 8, 1024, 128, seed=1), r(4, 8, 1024, 128, seed=2))
    elif which == "gqa_window_softcap":
        def fn(Q, K, V):
            g = Q.shape[1] // K.shape[1]
            K = K.repeat_interleave(g, dim=1)
            V = V.repeat_interleave(g, dim=1)
            QK = torch.tanh(Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5) / 30) * 30
            return torch.softmax(torch.ops.loopfuse.sliding_mask(QK, 100), dim=-1) @ V
        ins = (r(2, 16, 1024, 128), r(2, 4, 1024, 128, seed=1), r(2, 4, 1024, 128, seed=2))
    elif which == "paged_decode":
        def fn(Q, Kc, kt, Vc, vt):
            B, pages = kt.shape
            P, H, D = Kc.shape[1:]
            K = torch.ops.loopfuse.paged_load(Kc, kt).reshape(B, pages * P, H, D).transpose(1, 2)
            V = torch.ops.loopfuse.paged_load(Vc, vt).reshape(B, pages * P, H, D).transpose(1, 2)
            g = Q.shape[1] // H
            K = K.repeat_interleave(g, dim=1)
            V = V.repeat_interleave(g, dim=1)
            return torch.softmax(Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5), dim=-1) @ V
        n = 16 * 64
        gen = torch.Generator().manual_seed(3)
        ins = (r(16, 32, 1, 128), r(n, 16, 8, 128, seed=1), torch.randperm(n, generator=gen).view(16, 64).int(),
               r(n, 16, 8, 128, seed=2), torch.randperm(n, generator=gen).view(16, 64).int())
    else:
        def fn(x, wq, wk, wv, wo):
            B, S, E = x.shape
            H = 8
            q = (x @ wq).view(B, S, H, E // H).transpose(1, 2)
            k = (x @ wk).view(B, S, H, E // H).transpose(1, 2)
            v = (x @ wv).view(B, S, H, E // H).transpose(1, 2)
            a = torch.softmax(torch.ops.loopfuse.causal_mask(q @ k.transpose(-2, -1) * 0.125), dim=-1) @ v
            return a.transpose(1, 2).reshape(B, S, E) @ wo + x
        ins = (r(8, 1024, 1024),) + tuple((r(1024, 1024, seed=s).float() * 0.03).to(torch.bfloat16) for s in (1, 2, 3, 4))
    torch._dynamo.reset()
    before = dict(interface.stats)
    got = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend)(*ins)        # static shapes
    assert interface.stats["fused"] == before["fused"] + 1, "static graph at real size was not matched"
    want = fn(*ins)
    assert (got.float() - want.float()).abs().max().item() <= 6e-2


def test_factor_after_the_mask(monkeypatch):
    """x * f commutes with the mask only for f > 0.  A literal positive factor is folded at
    trace time; one that is only known per call is checked per call, and a non-positive
    value sends that call down the unfused graph."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)

    def fn(Q, K, V, alpha):
        s = torch.ops.loopfuse.causal_mask(Q @ K.transpose(-2, -1)) * alpha
        return torch.softmax(s, dim=-1) @ V

    q, k, v = (torch.randn(2, 3, 24, 64, generator=torch.Generator().manual_seed(s)) for s in (0, 1, 2))
    torch._dynamo.reset()
    cf = torch.compile(fn, backend=loopfuse_amd.loopfuse_backend, dynamic=True)
    before = dict(interface.stats)
    pos = cf(q, k, v, torch.tensor(0.125))
    assert interface.stats["fused"] == before["fused"] + 1
    torch.testing.assert_close(pos, O.attention_reference(q, k, v, mask="causal", scale=0.125), rtol=2e-4, atol=2e-4)
    neg = cf(q, k, v, torch.tensor(-0.125))      # -inf * negative = +inf: not a masked softmax any more
    assert interface.stats["eager_runtime"] == before["eager_runtime"] + 1
    torch.testing.assert_close(neg, fn(q, k, v, torch.tensor(-0.125)), equal_nan=True)


def test_fused_attention_op_with_dropout_is_left_alone():
    """Dropout inside F.scaled_dot_product_attention (torch then traces its unfused
    decomposition, with a dropout step on the probabilities) is not taken over."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, 2, 16, 32, generator=g) for _ in range(3))
    box = capture_graph(lambda q, k, v: F.scaled_dot_product_attention(q, k, v, dropout_p=0.5), (q, k, v))
    assert "match" not in box and "nomatch" in box


def _rotate_half(x):
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def _repeat_kv(h, n):
    b, hk, s, d = h.shape
    return h[:, :, None, :, :].expand(b, hk, n, s, d).reshape(b, hk * n, s, d)


class DecoderLayerAttention(torch.nn.Module):
    """Attention block as decoder models commonly write it: projections, rotary embedding,
    key/value cache appended by concatenation, kv heads repeated with expand + reshape,
    F.scaled_dot_product_attention, output projection, residual."""

    def __init__(self, E=256, H=8, Hkv=2):
        super().__init__()
        self.H, self.Hkv, self.D = H, Hkv, E // H
        self.q = torch.nn.Linear(E, H * self.D, bias=False)
        self.k = torch.nn.Linear(E, Hkv * self.D, bias=False)
        self.v = torch.nn.Linear(E, Hkv * self.D, bias=False)
        self.o = torch.nn.Linear(E, E, bias=False)
        self.norm = torch.nn.LayerNorm(E)

    def forward(self, x, cos, sin, past_k, past_v, mask=None):
        import torch.nn.functional as F
        B, S, E = x.shape
        h = self.norm(x)
        q = self.q(h).view(B, S, self.H, self.D).transpose(1, 2)
        k = self.k(h).view(B, S, self.Hkv, self.D).transpose(1, 2)
        v = self.v(h).view(B, S, self.Hkv, self.D).transpose(1, 2)
        q = q * cos + _rotate_half(q) * sin
        k = k * cos + _rotate_half(k) * sin
        k = torch.cat([past_k, k], dim=2)
        v = torch.cat([past_v, v], dim=2)
        g = self.H // self.Hkv
        a = F.scaled_dot_product_attention(q, _repeat_kv(k, g), _repeat_kv(v, g), attn_mask=mask,
                                           is_causal=mask is None and S > 1 and past_k.shape[2] == 0)
        return x + self.o(a.transpose(1, 2).contiguous().view(B, S, E)), k, v


def decoder_layer_inputs(E, H, Hkv, S, P, use_mask, dtype=torch.float32):
    g = torch.Generator().manual_seed(S + P)
    D = E // H
    r = lambda *shape: torch.randn(*shape, generator=g).to(dtype)
    mask = None
    if use_mask:      # causal mask of a chunk of S rows appended to P cached positions
        mask = torch.zeros(2, 1, S, P + S).masked_fill(torch.ones(S, P + S).triu(P + 1).bool(), float("-inf")).to(dtype)
    return r(2, S, E), r(1, 1, S, D), r(1, 1, S, D), r(2, Hkv, P, D), r(2, Hkv, P, D), mask


@pytest.mark.parametrize("S,P,use_mask", [(24, 0, False), (1, 40, False), (8, 40, True)])
@pytest.mark.parametrize("dynamic", [True, False])
def test_decoder_layer_with_cache_and_repeated_kv_heads(S, P, use_mask, dynamic, monkeypatch):
    """Prefill, one-token decode and a masked chunk of a decoder layer: the attention is
    taken over, K and V are the un-repeated cache tensors (grouped heads are not copied)."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)
    torch.manual_seed(0)
    m = DecoderLayerAttention().eval()
    ins = decoder_layer_inputs(256, 8, 2, S, P, use_mask)
    torch._dynamo.reset()
    before = dict(interface.stats)
    with torch.no_grad():
        got = torch.compile(m, backend=loopfuse_amd.loopfuse_backend, dynamic=dynamic)(*ins)
        want = m(*ins)
    assert interface.stats["fused"] == before["fused"] + 1
    match = interface.last_matches[-1]
    assert match.k.group == 4 and match.v.group == 4
    assert match.inputs[match.k.index].name.startswith("cat") and (match.bias is not None) == use_mask
    for a, b in zip(got, want):
        torch.testing.assert_close(a, b, rtol=2e-4, atol=2e-4)


def test_reference_import_path_is_a_drop_in():
    # reference loopfuse/__init__.py:1-3 and its tests import `from loopfuse import loopfuse_backend`
    import loopfuse
    from loopfuse import loopfuse_backend as ref_path_backend
    from loopfuse_amd import loopfuse_backend as own_backend

    assert ref_path_backend is own_backend and loopfuse.__all__ == ["loopfuse_backend"]
    for op in ("causal_mask", "sliding_mask", "scan_max", "paged_load"):
        assert hasattr(torch.ops.loopfuse, op)
    x = torch.randn(2, 3, 5, 5)
    fn = torch.compile(lambda a: torch.ops.loopfuse.causal_mask(a) + 1, backend=ref_path_backend, dynamic=True)
    assert torch.equal(fn(x), torch.ops.loopfuse.causal_mask(x) + 1)
