"""The loop-nest front end (loopfuse_amd/compiler): per-op nests, fusion, online-softmax and
block-skip passes, and the attention parameters read off the fused nest -- for the graphs of
the five benchmark configurations as the reference spells them (tests/benchmark.py:78-84,
142-147, 216-247, 400-406).  CPU only.

What pins it: the interpreter evaluates the nests before and after the passes and both must
equal the traced graph itself run by torch; the derived kv-tile ranges must equal, bit for
bit, the brute-force set over the dense mask (oracle.visited_tiles_dense); the derived plan
must equal the one the sub-graph matcher extracts independently."""
import pytest
import torch
from torch._functorch.aot_autograd import aot_module_simplified

import loopfuse_amd  # noqa: F401  (registers the ops)
from loopfuse_amd import compiler, lowering
from loopfuse_amd.compiler import interp, ir, passes
from loopfuse_amd.torch_backend import capture, interface
from oracle import attention_oracle as O


def c2(q, k, v):
    qk = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
    return torch.softmax(torch.ops.loopfuse.causal_mask(qk), dim=-1) @ v


def c2_softcap(q, k, v):
    qk = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
    qk = torch.tanh(qk / 30.0) * 30.0
    return torch.softmax(torch.ops.loopfuse.causal_mask(qk), dim=-1) @ v


def c3(q, k, v):
    g = q.shape[1] // k.shape[1]
    k, v = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    qk = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
    qk = torch.tanh(qk / 30.0) * 30.0
    return torch.softmax(torch.ops.loopfuse.sliding_mask(qk, 24), dim=-1) @ v


def c4(q, k, v):
    return torch.softmax(q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5), dim=-1) @ v


def c5(Q, Kc, kt, Vc, vt):
    B, pages = kt.shape
    P, H, D = Kc.shape[1:]
    K = torch.ops.loopfuse.paged_load(Kc, kt).reshape(B, pages * P, H, D).transpose(-3, -2)
    V = torch.ops.loopfuse.paged_load(Vc, vt).reshape(B, pages * P, H, D).transpose(-3, -2)
    return torch.softmax(Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5), dim=-1) @ V


def _r(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def _inputs(name):
    if name in ("c2", "c2_softcap"):
        return tuple(_r(2, 3, 40, 16, seed=s) for s in (1, 2, 3))
    if name == "c3":
        return _r(2, 8, 40, 16, seed=1), _r(2, 2, 40, 16, seed=2), _r(2, 2, 40, 16, seed=3)
    if name == "c4":
        return _r(3, 4, 1, 16, seed=1), _r(3, 4, 48, 16, seed=2), _r(3, 4, 48, 16, seed=3)
    n = 3 * 6
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(5)).view(3, 6).int()
    return _r(3, 2, 4, 16, seed=1), _r(n, 8, 2, 16, seed=2), perm, _r(n, 8, 2, 16, seed=3), perm.clone()


GRAPHS = {"c2": c2, "c2_softcap": c2_softcap, "c3": c3, "c4": c4, "c5": c5}


def _aten_graph(fn, ins):
    """The ATen graph and flat arguments the backend's fw_compiler sees (dynamic shapes)."""
    got = {}

    def backend(gm, sample):
        def fw(g, flat):
            got["gm"] = g
            def run(*args):
                got["args"] = args
                return g(*args)
            return run
        return aot_module_simplified(gm, sample, fw_compiler=fw)

    torch._dynamo.reset()
    with torch.no_grad():
        got["out"] = torch.compile(fn, backend=backend, dynamic=True)(*ins)
    return got["gm"], got["args"], got["out"]


@pytest.mark.parametrize("name", list(GRAPHS))
def test_passes_keep_the_meaning_of_the_nests(name):
    gm, args, out = _aten_graph(GRAPHS[name], _inputs(name))
    p = compiler.build.parse(gm)
    feeds = {b.name: args[b.placeholder] for b in p.inputs}
    before = interp.Interpreter(feeds).run(p.nests, args)[p.out.buf.name]
    n_ops = len(p.nests)
    nests = passes.fuse(p.nests, p.out.buf)
    assert len(nests) == 3 and n_ops >= 7          # max, sum and the second contraction are what fusion leaves
    fused = interp.Interpreter(feeds).run(nests, args)[p.out.buf.name]
    nests = passes.online_softmax(nests, p.out.buf)
    assert len(nests) == 1 and isinstance(nests[0].stmt, ir.Rescaled)
    online = interp.Interpreter(feeds).run(nests, args)[p.out.buf.name]
    want = out.double().reshape(before.shape)
    for got in (before, fused, online):
        assert (got - want).abs().max().item() <= 1e-5


@pytest.mark.parametrize("name", list(GRAPHS))
def test_derived_plan_equals_the_matchers(name):
    gm, args, _ = _aten_graph(GRAPHS[name], _inputs(name))
    comp = compiler.compile_graph(gm)
    derived = interface.match_from_nests(gm, comp)
    matched = capture.match_attention(gm)
    assert len(matched) == 1
    m = matched[0]
    vals_m = m.input_values(gm, args)
    a, b = derived.plan_for(list(args)), m.plan_for(vals_m)
    assert (a.mask, a.window, a.k_paged, a.v_paged) == (b.mask, b.window, b.k_paged, b.v_paged)
    assert a.scale == pytest.approx(b.scale, rel=1e-6) and (a.softcap is None) == (b.softcap is None)
    if a.softcap is not None:
        assert a.softcap == pytest.approx(b.softcap)
    # the same tensors in the same roles and layouts
    for od, om in ((derived.q, m.q), (derived.k, m.k), (derived.v, m.v)):
        td, tm = derived._operand(od, list(args)), m._operand(om, vals_m)
        assert td[0].shape == tm[0].shape and td[0].data_ptr() == tm[0].data_ptr() and td[0].stride() == tm[0].stride()
        assert (td[1] is None) == (tm[1] is None) and (td[1] is None or td[1].data_ptr() == tm[1].data_ptr())
    assert comp.attention.k.group == {"c3": 4}.get(name, 1)


@pytest.mark.parametrize("mask,window", [("causal", 0), ("sliding", 1), ("sliding", 24), ("sliding", 64), ("sliding", 200),
                                         (None, 0)])
@pytest.mark.parametrize("bm,bn", [(128, 64), (32, 64), (256, 64), (64, 32)])
def test_derived_tile_ranges_are_bit_exact(mask, window, bm, bn):
    def fn(q, k, v):
        s = q @ k.transpose(-2, -1) * 0.25
        if mask == "causal":
            s = torch.ops.loopfuse.causal_mask(s)
        elif mask == "sliding":
            s = torch.ops.loopfuse.sliding_mask(s, window)
        return torch.softmax(s, dim=-1) @ v

    gm, _, _ = _aten_graph(fn, tuple(_r(1, 2, 24, 16, seed=s) for s in (1, 2, 3)))
    bounds = compiler.compile_graph(gm, bm, bn).attention.bounds
    for S in (1, 17, 63, 64, 65, 129, 300, 593, 1024):
        dense = O.visited_tiles_dense(mask, S, S, window, bm, bn)
        for qt in range(dense.shape[0]):
            b, e = bounds.range(qt, S, S)
            got = torch.zeros(dense.shape[1], dtype=torch.bool)
            got[b:e] = True
            assert torch.equal(got, dense[qt]), (S, qt, b, e)
    # rectangular: more queries than keys and the other way round
    for Sq, Sk in ((300, 100), (100, 300), (129, 64)):
        dense = O.visited_tiles_dense(mask, Sq, Sk, window, bm, bn)
        for qt in range(dense.shape[0]):
            b, e = bounds.range(qt, Sq, Sk)
            got = torch.zeros(dense.shape[1], dtype=torch.bool)
            got[b:min(e, dense.shape[1])] = True
            assert torch.equal(got, dense[qt]), (Sq, Sk, qt, b, e)


# ---- the graphs the reference modifies its attention into (tests/test_accuracy.py:172-196,
# tests/test_attention.py:95-151): added tensors, an operand computed in the graph, the explicit
# exp2 softmax with its scan_max hint and a shifted denominator, two-part scores
def _modified(Q, K, V, q_bias, scores_bias, out_bias):
    QK = (Q + q_bias) @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
    QK = QK * 3.5 + scores_bias
    return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V + out_bias


def _explicit(Q, K, V):
    import math

    def _softmax(X):
        Xf = X.to(torch.float32)
        Xf_scaled = Xf * 1 / math.log(2)
        X_mik, X_mi = torch.ops.loopfuse.scan_max(Xf_scaled)
        expX = torch.exp2(Xf_scaled - X_mik) * torch.exp2(X_mik - X_mi)
        return expX / (torch.sum(expX, dim=-1, keepdim=True) + 1)
    QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
    return _softmax(torch.ops.loopfuse.causal_mask(QK)).to(Q.dtype) @ V


def _mla(Q_nope, Q_pe, K_nope, K_pe, V):
    qk = Q_nope @ K_nope.transpose(-2, -1) + Q_pe @ K_pe.expand(-1, Q_pe.shape[1], -1, -1).transpose(-2, -1)
    qk *= (Q_nope.shape[-1] + Q_pe.shape[-1]) ** (-0.5)
    return torch.softmax(torch.ops.loopfuse.causal_mask(qk), dim=-1) @ V


def _bias_gqa(Q, K, V, bias):
    g = Q.shape[1] // K.shape[1]
    K, V = K.repeat_interleave(g, dim=1), V.repeat_interleave(g, dim=1)
    QK = torch.tanh((Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)) / 20.0) * 20.0 + bias
    return torch.softmax(torch.ops.loopfuse.sliding_mask(QK, 17), dim=-1) @ V


WIDER = {
    "modified": (_modified, lambda: tuple(_r(2, 3, 40, 16, seed=s) for s in (1, 2, 3, 4)) + (_r(2, 3, 40, 40, seed=5), _r(2, 3, 40, 16, seed=6))),
    "explicit": (_explicit, lambda: tuple(_r(2, 3, 40, 16, seed=s) for s in (1, 2, 3))),
    "mla": (_mla, lambda: (_r(2, 4, 40, 16, seed=1), _r(2, 4, 40, 8, seed=2), _r(2, 4, 40, 16, seed=3), _r(2, 1, 40, 8, seed=4), _r(2, 4, 40, 16, seed=5))),
    "bias_gqa": (_bias_gqa, lambda: (_r(2, 8, 40, 16, seed=1), _r(2, 2, 40, 16, seed=2), _r(2, 2, 40, 16, seed=3), _r(1, 8, 40, 40, seed=4))),
}


@pytest.mark.parametrize("name", list(WIDER))
def test_modified_attentions_fall_out_of_the_same_passes(name):
    """fuse -> simplify -> online softmax leave one rescaled nest (plus the nest of an operand the graph
    computes from its inputs), which evaluates to what torch computes for the traced graph; the derived
    plan and operands equal what the sub-graph matcher extracts independently."""
    fn, make = WIDER[name]
    gm, args, out = _aten_graph(fn, make())
    comp = compiler.compile_graph(gm)
    p = compiler.build.parse(gm)                                     # the pipeline's steps, once more, for the interpreter
    nests = passes.fuse(p.nests, p.out.buf, keep_operands=True)
    nests = passes.online_softmax(passes.simplify(nests), p.out.buf)
    assert sum(isinstance(n.stmt, ir.Rescaled) for n in nests) == 1
    assert len(nests) == (2 if name == "modified" else 1)
    feeds = {b.name: args[b.placeholder] for b in p.inputs}
    got = interp.Interpreter(feeds).run(nests, args)[p.out.buf.name]
    assert (got - out.double().reshape(got.shape)).abs().max().item() <= 1e-5
    att = comp.attention
    assert (att.bias is not None) == (name in ("modified", "bias_gqa")) and (att.out_bias is not None) == (name == "modified")
    assert (att.q2 is not None) == (name == "mla") and att.base2 == (name == "explicit") and len(att.denom_add) == (name == "explicit")
    assert (att.q.node is not None) == (name == "modified")
    # against the matcher
    derived = interface.match_from_nests(gm, comp)
    matched = capture.match_attention(gm)
    assert len(matched) == 1
    m = matched[0]
    vals_d, vals_m = derived.input_values(gm, args), m.input_values(gm, args)
    a, b = derived.plan_for(vals_d), m.plan_for(vals_m)
    assert (a.mask, a.window, a.denom_add) == (b.mask, b.window, b.denom_add)
    assert a.scale == pytest.approx(b.scale, rel=1e-6) and a.softcap == (pytest.approx(b.softcap) if b.softcap else None)
    pairs = [(derived.q, m.q), (derived.k, m.k), (derived.v, m.v)]
    if name == "mla":
        pairs += [(derived.q2, m.q2), (derived.k2, m.k2)]
    for od, om in pairs:
        td, tm = derived._operand(od, vals_d)[0], m._operand(om, vals_m)[0]
        assert td.shape == tm.shape and td.stride() == tm.stride() and torch.equal(td, tm)
    B, Hq, Sq, Sk, D = derived._shapes(vals_d)
    for bd, bm_, shape in ((derived.bias, m.bias, (B, Hq, Sq, Sk)), (derived.out_bias, m.out_bias, (B, Hq, Sq, D))):
        assert (bd is None) == (bm_ is None)
        if bd is not None:
            assert torch.equal(derived._bias_view(bd, vals_d, shape), m._bias_view(bm_, vals_m, shape))


def test_a_running_maximum_that_does_not_cancel_is_refused():
    def fn(Q, K, V):
        x = Q @ K.transpose(-2, -1)
        run, mx = torch.ops.loopfuse.scan_max(x)
        e = torch.exp2(x - run)                       # not the hint: the running maximum stays in the value
        return (e / torch.sum(e, dim=-1, keepdim=True)) @ V
    gm, _, _ = _aten_graph(fn, tuple(_r(1, 2, 8, 8, seed=s) for s in (1, 2, 3)))
    with pytest.raises(compiler.NotDerivable, match="running maximum"):
        compiler.compile_graph(gm)


def test_graphs_that_are_not_one_attention_are_refused():
    for fn, ins in ((lambda a, b: a + b, (_r(4, 8), _r(4, 8))),
                    (lambda x, y: torch.softmax(x, dim=-1) @ y, (_r(2, 4, 8, 8), _r(2, 4, 8, 16))),
                    (lambda q, k, v: torch.softmax(q @ k.transpose(-2, -1), dim=-2) @ v, tuple(_r(1, 2, 8, 8) for _ in range(3))),
                    (lambda q, k, v: torch.sigmoid(q @ k.transpose(-2, -1)) @ v, tuple(_r(1, 2, 8, 8) for _ in range(3)))):
        gm, _, _ = _aten_graph(fn, ins)
        with pytest.raises(compiler.NotDerivable):
            compiler.compile_graph(gm)


@pytest.mark.parametrize("name", ["c2", "c3", "c5"])
def test_loop_nest_front_end_feeds_the_lowering(name, monkeypatch, shim_built):
    """LOOPFUSE_FRONTEND=ir under CODEGEN_ONLY: the kernels the derived plan asks for are the ones
    the matcher's plan asks for."""
    monkeypatch.setattr(interface, "CODEGEN_ONLY", True)
    if name == "c5":
        perm = torch.randperm(18, generator=torch.Generator().manual_seed(5)).view(3, 6).int()
        ins = [_r(3, 2, 4, 64).bfloat16(), _r(18, 16, 2, 64).bfloat16(), perm, _r(18, 16, 2, 64).bfloat16(), perm.clone()]
    else:
        ins = [torch.randn(2, h, 40, 64).to(torch.bfloat16) for h in ((8, 2, 2) if name == "c3" else (3, 3, 3))]
    specs = {}
    for fe in ("ir", "match"):
        monkeypatch.setenv("LOOPFUSE_FRONTEND", fe)
        torch._dynamo.reset()
        before = interface.stats["derived_graphs"]
        with torch.no_grad():
            res = torch.compile(GRAPHS[name], backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
        assert (interface.stats["derived_graphs"] == before + 1) == (fe == "ir")
        specs[fe] = [k.spec for k in res]
        assert "__global__" in res.code
    assert specs["ir"] == specs["match"] and len(specs["ir"]) == 1
