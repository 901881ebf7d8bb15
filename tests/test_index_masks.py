"""Masks built from indices alone (loopfuse_amd/torch_backend/index_masks.py): the symbolic value
of every node the tracker claims to understand is compared, element by element, with the tensor
the node really produces; and the front end turns such masks into the kernels' causal / window flag
exactly when the visible set is ``0 <= i - j [<= w - 1]``."""

import pytest
import torch
from torch.fx.experimental.proxy_tensor import make_fx

import loopfuse_amd  # noqa: F401
from loopfuse_amd.torch_backend import capture, index_masks, interface

from test_capture import _oracle_run

NINF = float("-inf")


def _ar(n):
    return torch.arange(n)


BUILDERS = {
    "tril_bool": lambda a, b: torch.ones(a, b, dtype=torch.bool).tril(),
    "not_tril": lambda a, b: ~torch.ones(a, b, dtype=torch.bool).tril(),
    "tril_float_eq0": lambda a, b: torch.tril(torch.ones(a, b)) == 0,
    "tril_view_ne0": lambda a, b: torch.tril(torch.ones(a, b)).view(1, 1, a, b) != 0,
    "tril_diag": lambda a, b: torch.ones(a, b, dtype=torch.bool).tril(diagonal=3),
    "triu_diag": lambda a, b: torch.ones(a, b, dtype=torch.bool).triu(diagonal=-2),
    "band": lambda a, b: torch.ones(a, b, dtype=torch.bool).tril() & torch.ones(a, b, dtype=torch.bool).triu(diagonal=-4),
    "ge": lambda a, b: _ar(a)[:, None] >= _ar(b)[None, :],
    "lt_unsqueeze": lambda a, b: _ar(b).unsqueeze(0) < _ar(a).unsqueeze(-1),
    "window": lambda a, b: (_ar(b)[None, :] <= _ar(a)[:, None]) & (_ar(a)[:, None] - _ar(b)[None, :] < 7),
    "or_masked": lambda a, b: ((_ar(a)[:, None] - _ar(b)[None, :]) < 0) | ((_ar(a)[:, None] - _ar(b)[None, :]) >= 9),
    "diff_plus_const": lambda a, b: (_ar(a)[:, None] - _ar(b)[None, :] + 2) > 1,
    "rsub": lambda a, b: (5 - _ar(b))[None, :] <= _ar(a)[:, None],
    "eq_diag": lambda a, b: _ar(a)[:, None] == _ar(b)[None, :],
    "ne_diag": lambda a, b: _ar(a)[:, None] != _ar(b)[None, :],
    "rows_only": lambda a, b: (_ar(a)[:, None] >= 3).expand(a, b),
    "prefix_slice": lambda a, b: torch.ones(a + 5, b + 5, dtype=torch.bool).tril()[:a, :b],
    "batched": lambda a, b: (_ar(a)[None, None, :, None] >= _ar(b)[None, None, None, :]),
    "times_tril": lambda a, b: torch.ones(a, b).tril() * torch.ones(a, b).triu(diagonal=-1),
}


def _eval_aff(aff, shape):
    out = torch.full(shape, aff.const, dtype=torch.int64)
    for pos, c in aff.coef:
        n = shape[pos]
        view = [1] * len(shape)
        view[pos] = n
        out = out + c * torch.arange(n).view(view)
    return out


def _eval_pred(p, shape):
    out = torch.ones(shape, dtype=torch.bool)
    for cl in p.clauses:
        out &= _eval_aff(cl, shape) >= 0
    return ~out if p.negated else out


@pytest.mark.parametrize("name", sorted(BUILDERS))
@pytest.mark.parametrize("sizes", [(9, 9), (7, 12), (13, 6), (1, 5)])
def test_symbolic_value_equals_the_tensor(name, sizes):
    gm = make_fx(lambda: BUILDERS[name](*sizes))()
    sym, actual = {}, {}

    class Rec(torch.fx.Interpreter):
        def run_node(self, n):
            r = super().run_node(n)
            actual[n] = r
            return r

    Rec(gm).run()
    understood = 0
    for n in gm.graph.nodes:
        if n.op != "call_function":
            continue
        sym[n] = index_masks.step(n, sym)
        got = sym[n]
        if got is None:
            continue
        understood += 1
        t = actual[n]
        if isinstance(got, index_masks.Aff):
            assert torch.equal(t.to(torch.int64), _eval_aff(got, tuple(t.shape))), n.name
        else:
            assert torch.equal(t != 0, _eval_pred(got, tuple(t.shape))), n.name
    out = list(gm.graph.nodes)[-1].args[0]
    out = out[0] if isinstance(out, (tuple, list)) else out
    assert sym.get(out) is not None, "the builder's result was not understood"
    assert understood >= 2


@pytest.mark.parametrize("name,keep,want", [
    ("tril_bool", +1, (0, None)), ("not_tril", -1, (0, None)), ("tril_float_eq0", -1, (0, None)),
    ("tril_view_ne0", +1, (0, None)), ("ge", +1, (0, None)), ("lt_unsqueeze", +1, (1, None)),
    ("window", +1, (0, 6)), ("or_masked", -1, (0, 8)), ("band", +1, (0, 4)), ("tril_diag", +1, (-3, None)),
    ("triu_diag", +1, (None, 2)), ("diff_plus_const", +1, (0, None)), ("eq_diag", +1, (0, 0)),
    ("ne_diag", +1, "no band"), ("rows_only", +1, "no band"), ("rsub", +1, "no band"), ("prefix_slice", +1, (0, None)),
    ("batched", +1, (0, None)), ("times_tril", +1, (0, 1)),
])
def test_band_of_a_mask(name, keep, want):
    gm = make_fx(lambda: BUILDERS[name](11, 11))()
    sym = {}
    for n in gm.graph.nodes:
        if n.op == "call_function":
            sym[n] = index_masks.step(n, sym)
    out = list(gm.graph.nodes)[-1].args[0]
    out = out[0] if isinstance(out, (tuple, list)) else out
    got = index_masks.band(sym[out], keep)
    if want == "no band":
        assert got is None
    else:
        lo, hi = got
        assert (None if lo == float("-inf") else lo, None if hi == float("inf") else hi) == want


@pytest.mark.parametrize("which,mask,window", [
    ("tril_bool", "causal", 0), ("tril_float_eq0", "causal", 0), ("arange_ge", "causal", 0),
    ("arange_window", "sliding", 7), ("band", "sliding", 5), ("tril_diag1", None, 0), ("bottom_right", None, 0),
])
def test_front_end_turns_index_masks_into_flags(which, mask, window, monkeypatch):
    """Fused either way; as a flag (no bias operand, the mask's nodes leave the graph) exactly for the
    causal triangle and causal windows, as a 0 / -inf term otherwise.  Result against eager."""
    monkeypatch.setattr(capture.AttentionMatch, "run", _oracle_run)
    f32 = lambda *shape, seed=0: torch.randn(*shape, generator=torch.Generator().manual_seed(seed))
    sc = lambda q, k: q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
    ones = lambda q, k: torch.ones(q.shape[-2], k.shape[-2], dtype=torch.bool)
    rows = lambda q: torch.arange(q.shape[-2])[:, None]
    cols = lambda k: torch.arange(k.shape[-2])[None, :]
    fns = {
        "tril_bool": lambda q, k, v: torch.softmax(sc(q, k).masked_fill(~ones(q, k).tril(), NINF), -1) @ v,
        "tril_float_eq0": lambda q, k, v: torch.softmax(sc(q, k).masked_fill(
            torch.tril(torch.ones(q.shape[-2], k.shape[-2])).view(1, 1, q.shape[-2], k.shape[-2]) == 0, NINF), -1) @ v,
        "arange_ge": lambda q, k, v: torch.softmax(torch.where(rows(q) >= cols(k), sc(q, k), NINF), -1) @ v,
        "arange_window": lambda q, k, v: torch.softmax(torch.where(
            (cols(k) <= rows(q)) & (rows(q) - cols(k) < 7), sc(q, k), NINF), -1) @ v,
        "band": lambda q, k, v: torch.softmax(sc(q, k).masked_fill(
            ~(ones(q, k).tril() & ones(q, k).triu(diagonal=-4)), NINF), -1) @ v,
        "tril_diag1": lambda q, k, v: torch.softmax(sc(q, k).masked_fill(~ones(q, k).tril(diagonal=1), NINF), -1) @ v,
        "bottom_right": lambda q, k, v: torch.softmax(sc(q, k).masked_fill(
            ~ones(q, k).tril(diagonal=k.shape[-2] - q.shape[-2]), NINF), -1) @ v,
    }
    rect = which in ("arange_ge", "bottom_right", "tril_float_eq0")
    ins = (f32(2, 3, 24, 64), f32(2, 3, 40 if rect else 24, 64, seed=1), f32(2, 3, 40 if rect else 24, 64, seed=2))
    torch._dynamo.reset()
    before = dict(interface.stats)
    with torch.no_grad():
        got = torch.compile(fns[which], backend=loopfuse_amd.loopfuse_backend, dynamic=True)(*ins)
    assert interface.stats["fused"] == before["fused"] + 1
    (m,) = interface.last_matches
    assert m.mask == mask and (m.window if mask == "sliding" else 0) == window
    assert (m.bias is None) == (mask is not None)
    torch.testing.assert_close(got, fns[which](*ins), rtol=2e-4, atol=2e-4)
