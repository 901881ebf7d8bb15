"""Graph capture: find ``softmax(mask(mods(Q K^T) [+ bias])) V [+ bias]`` sub-graphs in an ATen graph.

The reference turns every ATen node into a tiled loop nest and lets its
optimiser discover the fused form (``loopfuse/torch_backend/interface.py:
357-527`` ``GraphParser``, ``torch_backend/ops.py:344-751``).  This front end
goes the other way: it abstract-interprets the graph once, at compile time,
with three kinds of abstract values

  * ``Ids``     a tensor that is only a *view* of a graph input (or of a
                ``loopfuse.paged_load`` result): carried as an int64 tensor of
                element ids, so that transpose / expand / view / clone /
                unsqueeze chains (GQA ``repeat_interleave``, batch flattening
                for ``bmm``; reference ``interface.py:212-280``) are simply
                executed and their net effect read off afterwards;
  * ``Scalar``  a 0-dim value computed from shapes (``D ** -0.5`` with a
                dynamic D), re-evaluated on every call;
  * ``Stage``   scores / probabilities / output of the attention pipeline,
                with the score-modification chain seen so far.

Every other node is left to run as it is: its result is an ``Ids`` over a fresh
"computed" source, so an attention whose operands are produced by other ops
(``Q + q_bias``, projections, a second attention ...) is still recognised, and a graph
may hold several attentions.  The caller (``interface.py``) replaces each matched
output node by one fused call and lets dead-code elimination drop the unfused chain.

Shapes are symbolic under ``dynamic=True``; the interpretation runs on small
concrete stand-in sizes that keep the divisibility relations of the traced
example, so it costs microseconds and is immune to duck-sized symbols
(``S == D`` traced as one symbol).
"""
from __future__ import annotations

import dataclasses
import itertools
import math
import operator
from typing import Any, Optional

import torch

from .. import lowering
from . import index_masks

aten = torch.ops.aten
prims = torch.ops.prims


class NoMatch(Exception):
    """The graph is not a fused-attention pattern this backend lowers."""


# ----------------------------------------------------------------------------
# abstract values
# ----------------------------------------------------------------------------

@dataclasses.dataclass
class Source:
    """Where an ``Ids`` tensor's elements come from."""

    kind: str                      # "node" (a placeholder or any eagerly computed node) | "paged"
    node: Any                      # fx node holding the tensor (the pool, for paged)
    table_node: Any = None         # paged: fx node holding the page table
    shape: tuple[int, ...] = ()    # stand-in shape the ids enumerate (row-major)
    table_rank: int = 0            # paged: leading dims that come from the table


@dataclasses.dataclass
class Ids:
    src: Source
    t: torch.Tensor                # int64 element ids into src (row-major over src.shape)


@dataclasses.dataclass
class Scalar:
    node: torch.fx.Node            # re-evaluated at call time
    value: float                   # value for the stand-in sizes (unused beyond sanity)
    # how to compute it in plain Python at call time, if every step is understood:
    # ("lit", x) | ("arg", fx node holding a number) | ("dim", fx node holding a tensor, axis) |
    # ("op", name, operand, ...); None = run the node
    expr: Any = None


@dataclasses.dataclass
class Stage:
    kind: str                      # "scores" | "probs" | "out"
    shape: tuple[int, ...]         # stand-in logical shape
    q: Ids
    kt: Ids                        # K^T operand [.., D, Sk]
    v: Optional[Ids] = None
    q2: Optional[Ids] = None       # second score product (scores = Q K^T + Q2 K2^T), reference
    kt2: Optional[Ids] = None      # tests/test_attention.py:126-151
    factors: list = dataclasses.field(default_factory=list)       # multipliers before tanh
    post_factors: list = dataclasses.field(default_factory=list)  # multipliers after tanh
    has_tanh: bool = False
    mask: Optional[str] = None
    window: Any = 0                # int or fx.Node (SymInt)
    bias: Optional[tuple] = None       # (Ids, stage shape when added): additive score bias, before the mask
    bias_keep: int = 0                 # the "bias" is a boolean tensor: +1 True = visible, -1 True = masked (filled with -inf)
    out_bias: Optional[tuple] = None   # (Ids, stage shape when added): additive output bias
    # explicit softmax written with loopfuse.scan_max (reference tests/test_attention.py:95-125):
    uid: int = 0                       # set when scan_max is applied to this value
    sm: str = ""                       # "" | "minus_run" (x - running max) | "exp_run" | "num" (b^(x - max))
    base2: bool = False                # the exponentials are exp2
    denom_add: tuple = ()              # probabilities = num / (sum num + these terms)
    # scores / probabilities that currently sit in a permuted or regrouped layout (einsum lowers
    # to view -> permute -> view chains): ids of the canonical [batch..., Sq, Sk] elements in the
    # current shape; None while the value is a plain reshape of the canonical layout
    lay: Any = None
    mat: tuple = ()                    # (Sq, Sk) stand-ins
    late_factors: list = dataclasses.field(default_factory=list)   # run-time factors applied after the mask: must be > 0
    zero_blind_rows: bool = False      # torch's fused attention ops: a row with every key masked gives zeros


@dataclasses.dataclass
class Aux:
    """By-products of an explicit softmax on the scores with id ``uid``."""

    kind: str                          # "run" | "fin" (scan_max results) | "gap" (run - fin) | "expgap" | "den"
    uid: int
    c: tuple = ()                      # den: terms (numbers or Scalar nodes) added to the sum so far
    base2: bool = False


_VIEW_OPS = {
    aten.view.default, aten._unsafe_view.default, aten.reshape.default, aten.expand.default,
    aten.transpose.int, aten.permute.default, aten.unsqueeze.default, aten.squeeze.dim,
    aten.clone.default, aten.alias.default, aten.t.default, aten.contiguous.default,
    aten.detach.default,
}
_SHAPE_ONLY_VIEW_OPS = {aten.view.default, aten._unsafe_view.default, aten.reshape.default,
                        aten.expand.default, aten.clone.default, aten.alias.default,
                        aten.detach.default, aten.contiguous.default}
# F.scaled_dot_product_attention in an ATen graph (which one depends on the device and dtype)
_SDPA_OPS = {getattr(aten, name).default for name in (
    "_scaled_dot_product_flash_attention", "_scaled_dot_product_efficient_attention",
    "_scaled_dot_product_flash_attention_for_cpu") if hasattr(aten, name)}
_CAST_OPS = {prims.convert_element_type.default, aten._to_copy.default}


def _hint(sym) -> int:
    try:
        return int(sym.node.hint)
    except Exception:
        return 8


def _stand_in_sizes(hints: dict) -> dict:
    """Small concrete value per traced size, keeping small-ratio divisibility."""
    distinct = sorted(set(hints.values()))
    fresh = iter([5, 7, 3, 11, 13, 17, 19, 23, 29, 31, 37, 41])
    small: dict[int, int] = {}
    for h in distinct:
        if h <= 4:
            small[h] = h
            continue
        base = None
        for h2 in sorted(small, reverse=True):
            if 2 <= h2 < h and h % h2 == 0 and h // h2 <= 64 and small[h2] * (h // h2) <= 64:
                base = h2
                break
        small[h] = small[base] * (h // base) if base is not None else next(fresh)
    return {s: small[h] for s, h in hints.items()}


# ----------------------------------------------------------------------------
# result of a successful match
# ----------------------------------------------------------------------------

@dataclasses.dataclass
class Operand:
    """How to obtain a [B, H, S, D] strided view of Q/K/V from the fused call's inputs."""

    index: int                     # position in AttentionMatch.inputs (the pool when paged)
    perm: tuple[int, ...] = ()     # dense: permutation giving [B, H, S, D]
    paged: bool = False
    table_index: int = -1
    group: int = 1                 # head repeat factor seen in the graph (stand-in value)


@dataclasses.dataclass
class BiasOperand:
    """An additive bias as a strided [B, Hq, Sq, X] view of one of the fused call's inputs."""

    index: int
    dims: tuple                    # per logical dim (b, h, row, col): source dim it walks, or None (broadcast)
    keep: int = 0                  # a boolean mask instead of an additive term: +1 True = visible, -1 True = masked


@dataclasses.dataclass
class AttentionMatch:
    """One attention sub-graph.  ``inputs`` are the graph nodes (placeholders or nodes
    that keep running unfused) whose run-time values the fused call receives, in
    order; operands, factors and the window refer to them by position."""

    out_node: torch.fx.Node        # node whose value the fused call replaces
    inputs: list
    q: Operand
    k: Operand
    v: Operand
    factors: list                  # float | ("arg", i) | ("recip", x), multiplied together
    post_factors: list
    has_tanh: bool
    mask: Optional[str]
    window: Any                    # int | ("arg", i)
    out_rank: int
    bias: Optional[BiasOperand] = None
    out_bias: Optional[BiasOperand] = None
    tune: bool = False             # mode="max-autotune": measure the launch heuristics per shape class
    denom_add: tuple = ()          # explicit softmax with denominator (sum + these terms): floats | ("arg", i)
    base2: bool = False            # explicit softmax written with exp2: scores are in log2 units
    q2: Optional[Operand] = None   # second score product: scores = Q K^T + Q2 K2^T
    k2: Optional[Operand] = None
    late_factors: tuple = ()       # factors (also listed above) that the graph applies after the mask
    # memory order of the traced output when it is not row-major (torch's fused attention ops
    # return [B, H, S, D] views of [B, S, H, D] storage, and the graph after them may rely on
    # it): dims from outermost to innermost; () = row-major
    out_order: tuple = ()
    zero_blind_rows: bool = False  # rows whose keys are all masked give zeros (torch's fused attention ops), not NaN

    def empty_out(self, vals, dtype, device) -> torch.Tensor:
        """Uninitialised output in the traced shape and memory order."""
        shape = self.out_shape(vals)
        if not self.out_order:
            return torch.empty(shape, dtype=dtype, device=device)
        inverse = [self.out_order.index(i) for i in range(len(shape))]
        return torch.empty([shape[i] for i in self.out_order], dtype=dtype, device=device).permute(inverse)

    def describe(self) -> str:
        nm = lambda i: self.inputs[i].name
        return (f"attention -> {self.out_node.name}: Q={nm(self.q.index)}{self.q.perm} K={nm(self.k.index)}"
                f"{'[paged by %s]' % nm(self.k.table_index) if self.k.paged else self.k.perm} "
                f"V={nm(self.v.index)}{'[paged by %s]' % nm(self.v.table_index) if self.v.paged else self.v.perm} "
                f"mask={self.mask} window={self.window} tanh={self.has_tanh} "
                f"factors={self.factors} post={self.post_factors}"
                f"{' denom+%s' % (self.denom_add,) if self.denom_add else ''}{' exp2' if self.base2 else ''}"
                f"{' +Q2=%s K2=%s' % (nm(self.q2.index), nm(self.k2.index)) if self.q2 else ''}"
                f"{' +score_bias(%s)' % nm(self.bias.index) if self.bias else ''}"
                f"{' +out_bias(%s)' % nm(self.out_bias.index) if self.out_bias else ''}")

    # -- call-time evaluation of shape-derived scalars
    @staticmethod
    def _number(x, vals) -> float:
        if isinstance(x, tuple) and x[0] == "recip":
            return 1.0 / AttentionMatch._number(x[1], vals)
        if isinstance(x, tuple) and x[0] == "expr":
            return _eval_scalar(x[1], lambda i: vals[i])
        if isinstance(x, tuple) and x[0] == "fn":        # a scalar the loop-nest front end derived: callable over the inputs
            return float(x[1](vals))
        if isinstance(x, tuple) and x[0] == "arg":
            x = vals[x[1]]
        return float(x.item() if isinstance(x, torch.Tensor) else x)

    def _product(self, items, vals) -> float:
        r = 1.0
        for f in items:
            r *= self._number(f, vals)
        return r

    def plan_for(self, vals) -> lowering.AttnPlan:
        for f in self.late_factors:
            # x * f commutes with the mask only for f > 0 (-inf must stay -inf)
            if not self._number(f, vals) > 0.0:
                raise lowering.UnsupportedPlan("a non-positive factor is applied to masked scores")
        pre = self._product(self.factors, vals)
        if self.has_tanh:
            cap = self._product(self.post_factors, vals)
            scale, softcap = pre * cap, cap
        else:
            scale, softcap = pre, None
        window = self._number(self.window, vals) if self.mask == "sliding" else 0
        if self.base2:              # 2^x = e^(x ln 2): the kernels take natural-exponent scores
            if softcap is not None:
                raise lowering.UnsupportedPlan("softcap inside an exp2-based explicit softmax")
            scale *= math.log(2.0)
        return lowering.AttnPlan(mask=self.mask, window=int(window), scale=scale, softcap=softcap,
                                 k_paged=self.k.paged, v_paged=self.v.paged,
                                 denom_add=sum(self._number(t, vals) for t in self.denom_add),
                                 zero_blind_rows=self.zero_blind_rows)

    def _operand(self, op: Operand, vals):
        t = vals[op.index]
        if op.paged:
            return t, vals[op.table_index]
        if t.dim() == 3:
            t = t.unsqueeze(0)         # [B*H, S, D] given without a batch dim
        t = t.permute(op.perm)
        # the kernels read rows of D contiguous elements with 16-byte loads: a view that
        # walks D with a stride (K given as [B, H, D, S], reference tests/test_attention.py:265-282)
        # or sits on odd strides is copied once, O(S D) beside the O(S^2 D) attention
        if t.is_cuda and (t.stride(-1) != 1 or t.data_ptr() % 16
                          or any(n > 1 and st % 8 for n, st in zip(t.shape[:-1], t.stride()[:-1]))):
            t = t.clone(memory_format=torch.contiguous_format)
        return t, None

    def _bias_view(self, bo: Optional[BiasOperand], vals, shape, dtype=None):
        if bo is None:
            return None
        t = vals[bo.index]
        if bo.keep:
            # a boolean mask written with masked_fill / where: the kernels take it as the additive
            # term 0 / -inf (of the mask's own, possibly broadcast, shape; tiles that are all -inf
            # are never walked)
            if t.dtype != torch.bool:
                raise lowering.UnsupportedPlan("the mask is not the boolean tensor seen at trace time")
            t = torch.zeros(t.shape, dtype=dtype or torch.float32, device=t.device).masked_fill_(
                t if bo.keep < 0 else ~t, float("-inf"))
        # ("merged", k) / ("inner", k): batch and heads share source dim k ([B*H, ..], what baddbmm takes)
        def stride_of(d):
            if d is None:
                return 0
            if isinstance(d, tuple):
                return t.stride(d[1]) * (shape[1] if d[0] == "merged" else 1)
            return t.stride(d)

        strides = tuple(stride_of(d) for d in bo.dims)
        for i, (size, d) in enumerate(zip(shape, bo.dims)):
            if isinstance(d, tuple):
                want = shape[0] * shape[1] if bo.dims[0] is not None else shape[1]
                ok = t.shape[d[1]] == want
            else:
                ok = d is None or t.shape[d] == size
            if not ok:
                raise lowering.UnsupportedPlan("bias does not have the shape seen at trace time")
        return torch.as_strided(t, tuple(shape), strides, t.storage_offset())

    def _second_product(self, vals) -> dict:
        if self.q2 is None:
            return {}
        return {"q2": self._operand(self.q2, vals)[0], "k2": self._operand(self.k2, vals)[0]}

    def _shapes(self, vals):
        q, _ = self._operand(self.q, vals)
        k, kt = self._operand(self.k, vals)
        B, Hq, Sq, D = q.shape
        Sk = kt.shape[1] * (k.shape[1] if k.dim() == 4 else 1) if kt is not None else k.shape[2]
        return B, Hq, Sq, Sk, D

    def out_shape(self, vals) -> tuple:
        B, Hq, Sq, _, D = self._shapes(vals)
        return (B * Hq, Sq, D) if self.out_rank == 3 else (B, Hq, Sq, D)

    def input_values(self, gm: torch.fx.GraphModule, flat_args) -> list:
        """Run-time values of ``inputs`` for a call of the ORIGINAL graph with
        ``flat_args`` (runs the graph node by node; for tests and debugging)."""
        class Rec(torch.fx.Interpreter):
            def run_node(inner, n):
                r = super().run_node(n)
                if n in self.inputs:
                    got[n] = r
                return r

        got: dict = {}
        Rec(gm).run(*flat_args)
        return [got[n] for n in self.inputs]

    def run(self, vals) -> torch.Tensor:
        """``vals``: run-time values of ``inputs``."""
        q, _ = self._operand(self.q, vals)
        if not q.is_cuda:
            raise lowering.UnsupportedPlan("tensors are not on the GPU")
        k, kt = self._operand(self.k, vals)
        v, vt = self._operand(self.v, vals)
        B, Hq, Sq, Sk, D = self._shapes(vals)
        run = lowering.tuned_attention if self.tune else lowering.attention
        given = {"out": self.empty_out(vals, q.dtype, q.device)} if self.out_order else {}
        out = run(q, k, v, self.plan_for(vals), kt, vt, **given,
                                 score_bias=self._bias_view(self.bias, vals, (B, Hq, Sq, Sk), q.dtype),
                                 out_bias=self._bias_view(self.out_bias, vals, (B, Hq, Sq, D)),
                                 **self._second_product(vals))
        if self.out_rank == 3:
            out = out.view(out.shape[0] * out.shape[1], out.shape[2], out.shape[3])
        return out

    def kernel_specs_for(self, vals):
        """Specialisations the call would use (for CODEGEN_ONLY; no GPU needed)."""
        q, _ = self._operand(self.q, vals)
        plan = self.plan_for(vals)
        k = vals[self.k.index]
        D = q.shape[-1]
        dt = lowering._DTYPE_CODE.get(q.dtype)
        if dt is None or D > 128 or (D not in (64, 128) and (self.k.paged or self.v.paged or self.q2 is not None)):
            raise lowering.UnsupportedPlan("dtype/head dim not served by the HIP kernels")
        if D not in (64, 128):
            D = 64 if D < 64 else 128          # dense operands of other head dims run zero-padded
        paged = (1 if self.k.paged else 0) | (2 if self.v.paged else 0)
        ps = 1
        i64 = False
        if self.k.paged:
            ps = k.shape[1] if k.dim() == 4 else 1
            i64 = vals[self.k.table_index].dtype == torch.int64
        psv = 0
        if self.v.paged:
            vp = vals[self.v.index]
            pv = vp.shape[1] if vp.dim() == 4 else 1
            if self.k.paged and pv != ps:
                psv = pv
            elif not self.k.paged:
                ps, i64 = pv, vals[self.v.table_index].dtype == torch.int64
        mask = lowering._MASK_NAMES[plan.mask]
        bias = (1 if self.bias else 0) | (2 if self.out_bias else 0)
        d2 = self._operand(self.q2, vals)[0].shape[-1] if self.q2 is not None else 0
        if d2 not in (0, 16, 32, 64):
            raise lowering.UnsupportedPlan("depth of the second score product not served by the HIP kernels")
        kd, _ = self._operand(self.k, vals)
        B, Hq, Sq, Sk, _ = self._shapes(vals)
        hkv = kd.shape[-2] if self.k.paged else kd.shape[1]
        grp = Hq // max(hkv, 1)
        if plan.mask is None and bias in (0, 1) and not d2 and plan.denom_add == 0.0 and Sk >= 16 and \
                ((Sq == 1 and grp <= 64) or (grp == 1 and Sq <= 16)):
            # decode shapes stream K/V once (which of the two work splits serves them depends on the
            # device; the four-wave one is reported)
            return [lowering.KernelSpec("decode", dt, D, lowering.MASK_NONE, plan.softcap is not None, paged, ps, i64,
                                        rows=lowering.DECODE_QROWS, waves=4, page_size_v=psv, bias=bias,
                                        safe=plan.zero_blind_rows and bool(bias))]
        family = "prefill" if (paged or bias or d2) else lowering.prefill_variant(q.shape[-2])
        extra = ("-DLF_DMA=1",) if ((bias or d2) and not paged) else ()
        pack = 0
        if family == "prefill_swp":
            kd, _ = self._operand(self.k, vals)
            grp = q.shape[1] // max(kd.shape[1], 1)
            if q.shape[1] % max(kd.shape[1], 1) == 0 and grp % 2 == 0:
                pack = 4 if grp % 4 == 0 else 2
        bn = 0
        if family == "prefill_swp":       # the tile shape the launch would take for a grid of this size
            bn = lowering.prefill_kv_tile(D, bias, None, B * (Hq // (pack or 1)) * (-(-Sq // (128 // (pack or 1)))))
        return [lowering.KernelSpec(family, dt, D, mask, plan.softcap is not None, paged, ps, i64, bias=bias, d2=d2,
                                    page_size_v=psv, pack=pack, extra=extra, bn=bn,
                                    safe=plan.zero_blind_rows and bool(bias & 1) and family == "prefill")]


# ----------------------------------------------------------------------------
# the interpreter
# ----------------------------------------------------------------------------

def _fit_operand(x: torch.Tensor, src: Source, rows_are_d: bool) -> tuple[tuple[int, ...], int]:
    """Find (perm, group) with  x[b*H + h, r, c] == base.permute(perm)[b, h // group, r, c]."""
    if x.dim() == 4:
        x = x.reshape(x.shape[0] * x.shape[1], x.shape[2], x.shape[3])
    if x.dim() != 3:
        raise NoMatch("matmul operand is not a batched matrix")
    shape = list(src.shape)
    merged = None
    if src.kind == "paged" and len(shape) == 5:
        # [B, pages, P, Hkv, D]: tokens = (page, slot) merged
        merged = shape[2]
        shape = [shape[0], shape[1] * shape[2], shape[3], shape[4]]
    if len(shape) == 3 and src.kind == "node":
        shape = [1] + shape            # [B*H, S, D] inputs: one batch of B*H heads
    if len(shape) != 4:
        raise NoMatch(f"attention operand has rank {len(shape)} (need [B, H, S, D])")
    strides = [0] * 4
    acc = 1
    for i in range(3, -1, -1):
        strides[i] = acc
        acc *= shape[i]
    bflat, R, C = x.shape
    for perm in itertools.permutations(range(4)):
        db, dh, dr, dc = perm
        if shape[dr] != R or shape[dc] != C:
            continue
        Bn, Hn = shape[db], shape[dh]
        if Bn * Hn == 0 or bflat % (Bn * Hn):
            continue
        g = bflat // (Bn * Hn)
        ar = torch.arange
        ids = (ar(Bn) * strides[db]).view(Bn, 1, 1, 1) + ((ar(Hn * g) // g) * strides[dh]).view(1, Hn * g, 1, 1) \
            + (ar(R) * strides[dr]).view(1, 1, R, 1) + (ar(C) * strides[dc]).view(1, 1, 1, C)
        if torch.equal(ids.reshape(bflat, R, C), x):
            # perm that yields [B, H, S, D]
            out = (db, dh, dc, dr) if rows_are_d else (db, dh, dr, dc)
            return out, g
    raise NoMatch("operand is not a (head-repeated) permuted view of one input")


def _fit_bias(entry: tuple, logical: tuple):
    """Express a bias (ids broadcast against the stage it was added to) as a strided
    [B, Hq, Sq, X] view of its source: per logical dim, the source dim it walks.
    Returns (source node, dims)."""
    ids, stage_shape = entry
    src = ids.src
    if src.kind != "node":
        raise NoMatch("bias must be a plain tensor")
    try:
        x = torch.broadcast_to(ids.t, stage_shape).reshape(logical)
    except RuntimeError as e:
        raise NoMatch(f"bias does not broadcast to the scores/output: {e}")
    shape = list(src.shape)
    cstride = [math.prod(shape[i + 1:]) for i in range(len(shape))]
    zero = (0,) * len(logical)
    if int(x[zero]) != 0:
        raise NoMatch("bias view does not start at the first element of its source")
    dims = []
    recon = torch.zeros(logical, dtype=torch.int64)
    for d, n in enumerate(logical):
        if n == 1:
            dims.append(None)
            continue
        idx = list(zero)
        idx[d] = 1
        step = int(x[tuple(idx)])
        if step == 0:
            dims.append(None)
            continue
        cand = [k for k in range(len(shape)) if cstride[k] == step and shape[k] == n]
        if not cand and d == 0:
            # batch and heads merged into one source dim ([B*H, Sq, Sk], what baddbmm takes): the batch walks
            # that dim in steps of the head count
            merged = [k for k in range(len(shape)) if cstride[k] * logical[1] == step and shape[k] == n * logical[1]]
            if merged:
                dims.append(("merged", merged[0]))
                recon = recon + (torch.arange(n) * step).view([n, 1, 1, 1])
                continue
        if not cand and d == 1:
            inner = [k for k in range(len(shape)) if cstride[k] == step and shape[k] == n * logical[0]]
            if inner and dims and dims[0] in (None, ("merged", inner[0])):
                cand = [("inner", inner[0])]        # the heads' share of a merged [B*H] dim
        if not cand:
            raise NoMatch("bias is not a permuted / broadcast view of one tensor")
        dims.append(cand[0])
        view = [1] * len(logical)
        view[d] = n
        recon = recon + (torch.arange(n) * step).view(view)
    if not torch.equal(recon, x):
        raise NoMatch("bias is not an affine view of its source")
    if dims[3] is None and logical[3] > 1:
        raise NoMatch("bias is broadcast along its last dim")
    return src.node, tuple(dims)


def _regroup(real_in, real_out, stand_in, stand_out_hint):
    """Stand-in shape of a view/reshape: ``real_in -> real_out`` regroups contiguous dims;
    the same regrouping is applied to ``stand_in``.  A target dim that merges source dims
    is their stand-in product; where a source dim is split, the targets take
    ``stand_out_hint`` (per target dim, may be None) and must multiply back to it.
    Returns None when the stand-ins cannot follow the regrouping."""
    out = []
    i = j = 0
    ni, nj = len(real_in), len(real_out)
    while i < ni or j < nj:
        gi, gj = [], []
        pi = pj = 1
        # smallest groups of source / target dims with equal products
        while True:
            if (pi == pj and gi and gj) or (i >= ni and j >= nj):
                break
            take_in = (pi < pj) or (pi == pj and not gi)
            if (take_in and i < ni) or j >= nj:
                pi *= real_in[i]
                gi.append(i)
                i += 1
            else:
                pj *= real_out[j]
                gj.append(j)
                j += 1
        if pi != pj:
            return None
        prod_in = math.prod(stand_in[k] for k in gi)
        if len(gj) == 1:
            out.append(prod_in)
            continue
        if not gj:
            if prod_in != 1:
                return None
            continue
        vals = []
        for k in gj:
            if real_out[k] == 1:
                vals.append(1)
            elif stand_out_hint[k] is None:
                return None
            else:
                vals.append(stand_out_hint[k])
        if math.prod(vals) != prod_in:
            return None
        out.extend(vals)
    return out


_SCALAR_BINARY = {aten.mul.Tensor: "mul", aten.div.Tensor: "div", aten.add.Tensor: "add", aten.sub.Tensor: "sub",
                  aten.pow.Tensor_Tensor: "pow", aten.pow.Tensor_Scalar: "pow"}
_SCALAR_UNARY = {aten.reciprocal.default: "recip", aten.sqrt.default: "sqrt", aten.rsqrt.default: "rsqrt",
                 aten.neg.default: "neg"}


def _scalar_expr(node: torch.fx.Node, tgt, a, kw):
    """Python-evaluable form of a 0-dim computation on shape-derived values, or None."""
    def operand(i):
        x = a[i]
        if isinstance(x, Scalar):
            return x.expr
        raw = node.args[i]
        if isinstance(raw, torch.fx.Node):
            return ("arg", raw)
        return ("lit", float(x)) if isinstance(x, (int, float)) and not isinstance(x, bool) else None

    if tgt in _CAST_OPS or tgt in (aten.clone.default, aten.alias.default, aten.detach.default):
        return operand(0)
    if tgt in _SCALAR_BINARY and len(a) >= 2 and kw.get("alpha", 1) == 1:
        x, y = operand(0), operand(1)
        return None if x is None or y is None else ("op", _SCALAR_BINARY[tgt], x, y)
    if tgt in _SCALAR_UNARY:
        x = operand(0)
        return None if x is None else ("op", _SCALAR_UNARY[tgt], x)
    return None


def _eval_scalar(e, leaf) -> float:
    kind = e[0]
    if kind == "lit":
        return float(e[1])
    if kind == "arg":
        x = leaf(e[1])
        return float(x.item() if isinstance(x, torch.Tensor) else x)
    if kind == "dim":
        return float(leaf(e[1]).shape[e[2]])
    name, xs = e[1], [_eval_scalar(x, leaf) for x in e[2:]]
    if name == "mul":
        return xs[0] * xs[1]
    if name == "div":
        return xs[0] / xs[1]
    if name == "add":
        return xs[0] + xs[1]
    if name == "sub":
        return xs[0] - xs[1]
    if name == "pow":
        return xs[0] ** xs[1]
    if name == "recip":
        return 1.0 / xs[0]
    if name == "sqrt":
        return math.sqrt(xs[0])
    if name == "rsqrt":
        return 1.0 / math.sqrt(xs[0])
    if name == "neg":
        return -xs[0]
    raise ValueError(name)


def _same_expr(x, y) -> bool:
    if x is None or y is None or x[0] != y[0]:
        return False
    if x[0] == "lit":
        return x[1] == y[1]
    if x[0] == "arg":
        return x[1] is y[1]
    if x[0] == "dim":
        return x[1] is y[1] and x[2] == y[2]
    return x[1] == y[1] and len(x) == len(y) and all(_same_expr(p, q) for p, q in zip(x[2:], y[2:]))


def _same_scalar(x, y) -> bool:
    """Two score factors (numbers, graph nodes, ("recip", f)) that are the same value by
    construction: identical, or the same pure computation on the same inputs."""
    if x is y:
        return True
    if isinstance(x, Scalar) and isinstance(y, Scalar):
        return _same_expr(x.expr, y.expr) or _same_scalar(x.node, y.node)
    if isinstance(x, tuple) and isinstance(y, tuple):
        return len(x) == len(y) and all(_same_scalar(a, b) for a, b in zip(x, y))
    if isinstance(x, torch.fx.Node) and isinstance(y, torch.fx.Node):
        return (x.op == y.op == "call_function" and x.target is y.target and len(x.args) == len(y.args)
                and not x.kwargs and not y.kwargs and all(_same_scalar(a, b) for a, b in zip(x.args, y.args)))
    if isinstance(x, (int, float, str)) and isinstance(y, (int, float, str)):
        return type(x) is type(y) and x == y
    return False


def match_attention(gm: torch.fx.GraphModule) -> list:
    """Interpret ``gm`` abstractly; return its attention sub-graphs (``AttentionMatch``
    list, possibly several) or raise ``NoMatch`` with the reason none was found.

    The fw_compiler runs under AOTAutograd's fake-tensor mode; the stand-in id
    tensors must be real, so dispatch modes are switched off for the duration.
    """
    from torch.utils._python_dispatch import _disable_current_modes

    with _disable_current_modes():
        return _match_attention(gm)


class _Skip(Exception):
    """This node does not continue an attention pattern: treat it as an ordinary op."""


def _match_attention(gm: torch.fx.GraphModule) -> list:
    graph = gm.graph
    placeholders = [n for n in graph.nodes if n.op == "placeholder"]
    outputs = [n for n in graph.nodes if n.op == "output"]
    if len(outputs) != 1:
        raise NoMatch("no single output node")

    # ---- stand-in sizes for every free symbol
    import sympy

    hints: dict = {}

    def collect(val):
        if isinstance(val, torch.SymInt):
            for s in val.node.expr.free_symbols:
                hints.setdefault(s, None)

    for p in placeholders:
        val = p.meta.get("val")
        if isinstance(val, torch.Tensor):
            for d in val.shape:
                collect(d)
        else:
            collect(val)
    for p in placeholders:
        val = p.meta.get("val")
        if isinstance(val, torch.SymInt) and isinstance(val.node.expr, sympy.Symbol):
            hints[val.node.expr] = _hint(val)
    for p in placeholders:
        val = p.meta.get("val")
        if isinstance(val, torch.Tensor):
            for d in val.shape:
                if isinstance(d, torch.SymInt) and isinstance(d.node.expr, sympy.Symbol) and hints.get(d.node.expr) is None:
                    hints[d.node.expr] = _hint(d)
    for s, h in list(hints.items()):
        if h is None:
            hints[s] = 8
    sizes = _stand_in_sizes(hints)
    # a symbol that some shape divides (x.chunk(3, -1) of a dynamic width: (s + 2) // 3) keeps its traced
    # value: an arbitrary stand-in would not divide the same way (down to a dim of 0)
    for n in graph.nodes:
        val = n.meta.get("val")
        for t in (val if isinstance(val, (tuple, list)) else (val,)):
            for d in (t.shape if isinstance(t, torch.Tensor) else (t,)):
                if isinstance(d, torch.SymInt) and any(
                        type(e).__name__ in ("FloorDiv", "CleanDiv", "CeilDiv", "Mod", "PythonMod", "ModularIndexing", "floor")
                        for e in sympy.preorder_traversal(d.node.expr)):
                    for sym_ in d.node.expr.free_symbols:
                        sizes[sym_] = hints[sym_]

    # Static dims normally keep their values (a head dim of 128 marked static).  A graph
    # traced with static shapes at real sizes would need id tensors of the real size: then
    # the static dims of the inputs get stand-ins too (one per distinct value, chosen
    # together with the symbols' so that small ratios such as Hq = g * Hkv survive), and the
    # literal shapes in view / expand nodes are re-derived from the nodes' real shapes.
    CAP = 1 << 22
    real = lambda d: _hint(d) if isinstance(d, torch.SymInt) else int(d)
    fmap: dict = {}

    def _numel_as_is(val) -> int:
        return math.prod(int(d.node.expr.subs(sizes)) if isinstance(d, torch.SymInt) else int(d) for d in val.shape)

    if any(isinstance(p.meta.get("val"), torch.Tensor) and _numel_as_is(p.meta["val"]) > CAP for p in placeholders):
        statics = sorted({int(d) for p in placeholders if isinstance(p.meta.get("val"), torch.Tensor)
                          for d in p.meta["val"].shape if not isinstance(d, torch.SymInt) and int(d) > 4})
        joint = dict(hints)
        joint.update({("static", v): v for v in statics})
        both = _stand_in_sizes(joint)
        sizes = {k: v for k, v in both.items() if not isinstance(k, tuple)}
        fmap = {k[1]: v for k, v in both.items() if isinstance(k, tuple)}
    shrink_static = bool(fmap)

    # Equalities the trace relies on without having solved them for one symbol (two page
    # pools with pages_k * page_k == pages_v * page_v tokens): where the stand-ins break a
    # matmul's contraction or batch dims, the symbols involved keep their traced values,
    # which satisfy every such equality by construction.
    def _expr(d):
        return d.node.expr if isinstance(d, torch.SymInt) else sympy.Integer(int(d))

    pairs = []
    for n in graph.nodes:
        if n.op == "call_function" and n.target in (aten.bmm.default, aten.mm.default, aten.matmul.default):
            va, vb = (x.meta.get("val") if isinstance(x, torch.fx.Node) else None for x in n.args[:2])
            if isinstance(va, torch.Tensor) and isinstance(vb, torch.Tensor) and va.dim() >= 2 and vb.dim() >= 2:
                pairs.append((_expr(va.shape[-1]), _expr(vb.shape[-2])))
                if va.dim() == vb.dim():
                    pairs += [(_expr(x), _expr(y)) for x, y in zip(va.shape[:-2], vb.shape[:-2])
                              if _expr(x) != 1 and _expr(y) != 1]          # 1 broadcasts
    for _ in range(len(hints) + 1):
        broken = [(x, y) for x, y in pairs if x.subs(sizes) != y.subs(sizes)]
        if not broken:
            break
        for x, y in broken:
            for sym in (x.free_symbols | y.free_symbols):
                sizes[sym] = hints[sym]

    def concrete(d) -> int:
        if isinstance(d, torch.SymInt):
            v = int(d.node.expr.subs(sizes))
            if v < 0 or (v == 0 and _hint(d) != 0):
                raise NoMatch("stand-in sizes do not reproduce the traced shapes")
            return v
        d = int(d)
        if d in fmap:
            return fmap[d]
        if shrink_static and d > 4:
            # a literal product of two input dims (batch * heads, tokens * width)
            for a_, fa in fmap.items():
                if d % a_ == 0 and (d // a_) in fmap:
                    return fa * fmap[d // a_]
        return d

    def stand_in_view_shape(node, in_shape):
        """Target shape of a view / reshape / expand node for an input of stand-in shape
        ``in_shape``, derived from the node's real shapes instead of its literal arguments."""
        src = node.args[0]
        rin = [real(d) for d in src.meta["val"].shape]
        rout = [real(d) for d in node.meta["val"].shape]
        hint = [concrete(d) for d in node.meta["val"].shape]
        if node.target is aten.expand.default:
            pad = len(rout) - len(rin)
            return [in_shape[j - pad] if j >= pad and rin[j - pad] == rout[j] else hint[j] for j in range(len(rout))]
        got = _regroup(rin, rout, list(in_shape), hint)
        if got is None:
            raise _Skip("view not reproducible on stand-in sizes")
        return got

    def fresh_ids(node: torch.fx.Node, val) -> Any:
        """A tensor-valued node that simply runs: ids over its own (stand-in) shape."""
        if val.dim() == 0:
            return Scalar(node, 1.0, ("arg", node))    # e.g. a Python float that dynamo passes as a 0-dim tensor
        shape = tuple(concrete(d) for d in val.shape)
        n = math.prod(shape)
        if n > CAP:
            raise NoMatch("stand-in tensor too large")
        return Ids(Source("node", node, shape=shape), torch.arange(n, dtype=torch.int64).reshape(shape))

    env: dict[torch.fx.Node, Any] = {}
    for p in placeholders:
        val = p.meta.get("val")
        if isinstance(val, torch.Tensor):
            env[p] = fresh_ids(p, val)
        elif isinstance(val, (torch.SymInt, int)):
            env[p] = concrete(val)
        elif isinstance(val, (torch.SymFloat, float)):
            env[p] = Scalar(p, float(val) if isinstance(val, float) else 1.0, ("arg", p))
        else:
            raise NoMatch(f"unsupported placeholder {p.name}")

    def arg(a):
        return torch.fx.node.map_arg(a, lambda n: env[n])

    def is_number(x) -> bool:
        return isinstance(x, (int, float)) and not isinstance(x, bool)

    def is_neg_inf(x) -> bool:
        return (is_number(x) and x == float("-inf")) or (isinstance(x, Scalar) and x.expr == ("lit", float("-inf")))

    def is_bool(ids) -> bool:
        val = ids.src.node.meta.get("val") if isinstance(ids, Ids) and ids.src.kind == "node" else None
        return isinstance(val, torch.Tensor) and val.dtype == torch.bool

    def bool_mask(st, ids, keep, mask_node):
        """Scores whose masked elements are filled with -inf according to a boolean tensor.  A mask the
        graph builds from indices alone (tril of ones, arange comparisons) that comes out as the causal
        triangle or a causal window becomes the kernels' mask flag; any other boolean tensor is taken as
        an additive 0 / -inf term (only -inf commutes with that reading: a finite fill value replaces
        the score, it does not add to it)."""
        if not (isinstance(st, Stage) and st.kind == "scores" and st.mask is None and st.bias is None and st.uid == 0
                and st.sm == "" and st.lay is None):
            raise _Skip("boolean mask on scores that already carry a mask or a bias")
        pred = sym.get(mask_node) if isinstance(mask_node, torch.fx.Node) else None
        if isinstance(pred, index_masks.Pred):
            lo_hi = index_masks.band(pred, keep)
            if lo_hi is not None and lo_hi[0] == 0:
                if lo_hi[1] == math.inf:
                    return dataclasses.replace(st, mask="causal")
                if lo_hi[1] >= 0:
                    return dataclasses.replace(st, mask="sliding", window=int(lo_hi[1]) + 1)
        return dataclasses.replace(st, bias=(ids, st.shape), bias_keep=keep)

    def meta_view(target, shape, args, kwargs):
        m = torch.empty(shape, device="meta")
        return tuple(target(m, *args, **kwargs).shape)

    matches: list = []
    reasons: list = []
    sym: dict = {}
    finalised: dict = {}
    uid_box = [0]

    def finalise(node: torch.fx.Node) -> None:
        """``node`` holds a finished attention that something outside the pattern reads."""
        if node in finalised:
            return
        finalised[node] = None
        try:
            finalised[node] = _build_match(node, env[node])
            matches.append(finalised[node])
        except NoMatch as e:
            reasons.append(str(e))

    def consume(values) -> None:
        for x in values:
            if isinstance(x, torch.fx.Node) and isinstance(env.get(x), Stage) and env[x].kind == "out":
                finalise(x)

    def sdpa_stage(node, tgt, a, kw) -> Stage:
        """torch's fused attention ops (what F.scaled_dot_product_attention becomes in an
        ATen graph) as a finished attention: softmax(causal?(Q K^T * scale)) V."""
        names = [arg_.name for arg_ in tgt._schema.arguments]
        given = dict(zip(names, a))
        given.update(kw)
        qi, ki, vi = given["query"], given["key"], given["value"]
        if not all(isinstance(x, Ids) and x.t.dim() == 4 for x in (qi, ki, vi)):
            raise _Skip("fused attention op on operands that are not rank-4 tensors")
        bias = given.get("attn_mask") if given.get("attn_mask") is not None else given.get("attn_bias")
        if bias is not None and not isinstance(bias, Ids):
            raise _Skip("fused attention op with a mask that is not a tensor")
        if bias is not None and given.get("is_causal", False):
            raise _Skip("fused attention op with a mask tensor and is_causal")
        if given.get("dropout_p", 0.0) != 0.0:
            raise _Skip("fused attention op with dropout")
        if qi.t.shape[0] != ki.t.shape[0] or qi.t.shape[-1] != ki.t.shape[-1] or vi.t.shape[:3] != ki.t.shape[:3] \
                or ki.t.shape[1] < 1 or qi.t.shape[1] % ki.t.shape[1]:
            raise _Skip("fused attention op: Q, K, V shapes disagree")
        if qi.t.shape[1] != ki.t.shape[1]:
            # enable_gqa: query head h reads kv head h // group, as repeat_interleave would give
            group = qi.t.shape[1] // ki.t.shape[1]
            ki = Ids(ki.src, ki.t.repeat_interleave(group, dim=1))
            vi = Ids(vi.src, vi.t.repeat_interleave(group, dim=1))
        scale = given.get("scale")
        if scale is None:
            d = node.args[0].meta["val"].shape[-1]
            if isinstance(d, int):
                scale = float(d) ** -0.5
            else:
                # fully dynamic graph: the head dim is read off the query tensor at call time
                scale = Scalar(node, float(qi.t.shape[-1]) ** -0.5, ("op", "rsqrt", ("dim", node.args[0], -1)))
        elif isinstance(scale, (int, float)):
            raw = node.kwargs.get("scale")
            scale = raw if isinstance(raw, torch.fx.Node) else float(scale)
        elif not isinstance(scale, Scalar):
            raise _Skip("fused attention op: scale not understood")
        sq, sk = qi.t.shape[-2], ki.t.shape[-2]
        # a mask tensor reaches the op as an additive term in the query's dtype (torch turns
        # boolean masks into 0 / -inf before it dispatches): the kernels' score bias
        return Stage("out", tuple(qi.t.shape[:-1]) + (vi.t.shape[-1],), qi, Ids(ki.src, ki.t.transpose(-1, -2)), vi,
                     factors=[scale], mask="causal" if given.get("is_causal", False) else None, mat=(sq, sk),
                     bias=None if bias is None else (bias, tuple(qi.t.shape[:-1]) + (sk,)), zero_blind_rows=True)

    def pattern_step(node, tgt, a, kw, first):
        """The abstract value of ``node`` if it continues a pattern; raises _Skip otherwise."""
        # -- integer / float arithmetic on sizes
        if all(is_number(x) for x in a) and tgt in (
                operator.mul, operator.floordiv, operator.add, operator.sub, operator.truediv,
                operator.pow, operator.neg, operator.mod):
            return tgt(*a)
        if tgt is aten.sym_size.int:
            # size of an intermediate (duck-sized batch == heads makes dynamo re-read it)
            if isinstance(first, Stage):
                return int(first.shape[a[1]])
            if isinstance(first, Ids):
                return int(first.t.shape[a[1]])
            raise _Skip("sym_size on an unsupported value")

        # -- scalars derived from sizes
        if tgt is aten.scalar_tensor.default and is_number(a[0]):
            raw0 = node.args[0]
            return Scalar(node, float(a[0]), ("arg", raw0) if isinstance(raw0, torch.fx.Node) else ("lit", float(a[0])))
        val = node.meta.get("val")
        if isinstance(first, Scalar) and isinstance(val, torch.Tensor) and val.dim() == 0 and all(
                isinstance(x, (Scalar, int, float, bool, str, torch.dtype, type(None)))
                for x in list(a) + list(kw.values())):
            return Scalar(node, 1.0, _scalar_expr(node, tgt, a, kw))   # any arithmetic among shape-derived 0-dim values

        # -- explicit softmax by-products (running / final max, their gap, the denominator)
        if tgt is operator.getitem and isinstance(first, list) and isinstance(a[1], int):
            return first[a[1]]
        if isinstance(first, Aux):
            x = first
            if tgt is aten.sub.Tensor and x.kind == "run" and isinstance(a[1], Aux) and a[1].kind == "fin" \
                    and a[1].uid == x.uid and kw.get("alpha", 1) == 1:
                return Aux("gap", x.uid)
            if tgt in (aten.exp2.default, aten.exp.default) and x.kind == "gap":
                return Aux("expgap", x.uid, base2=tgt is aten.exp2.default)
            if tgt is aten.add.Tensor and x.kind == "den" and kw.get("alpha", 1) == 1 and (
                    (is_number(a[1]) and a[1] >= 0) or isinstance(a[1], Scalar)):
                raw = node.args[1]
                term = a[1] if isinstance(a[1], Scalar) else (raw if isinstance(raw, torch.fx.Node) else float(a[1]))
                return Aux("den", x.uid, c=x.c + (term,))
            if tgt is aten.mul.Tensor and x.kind == "expgap" and isinstance(a[1], Stage):
                a = (a[1], a[0])            # handled below with the stage first
                first = a[0]
            else:
                raise _Skip(f"op on a softmax by-product: {tgt}")

        # -- tensor + scores / tensor + output with the tensor written first
        if tgt is aten.add.Tensor and isinstance(first, Ids) and len(a) > 1 and isinstance(a[1], Stage) \
                and kw.get("alpha", 1) == 1:
            a = (a[1], a[0]) + tuple(a[2:])
            first = a[0]

        # -- views of tensors
        if isinstance(first, Ids):
            if tgt is aten.slice.Tensor:
                # x[:, :, None] style indexing leaves one whole-range slice per dim in a dynamic graph
                rest = list(a[1:]) + [None] * 4
                start, end, step = rest[1], rest[2], rest[3]
                if start in (0, None) and step in (1, None) and (end is None or (is_number(end) and end >= 1 << 62)) \
                        and not kw:
                    return first
                raise _Skip("a slice that is not the whole range")
            if tgt in _VIEW_OPS:
                if shrink_static and tgt in (aten.view.default, aten._unsafe_view.default, aten.reshape.default,
                                             aten.expand.default):
                    a = (a[0], stand_in_view_shape(node, first.t.shape)) + tuple(a[2:])
                try:
                    out = Ids(first.src, tgt(first.t, *a[1:], **kw))
                except Exception as e:  # invalid for the stand-in sizes
                    raise _Skip(f"view chain not reproducible on stand-in sizes: {e}")
                if first.src.kind == "node" and len(first.src.shape) != 4 and out.t.dim() == 4:
                    # a projection output [B*S, E] viewed as [B, S, H, D]: operands are described
                    # as permutations of a rank-4 tensor, so this view becomes the source
                    raise _Skip("rank-4 view of a tensor of another rank: taken as a source of its own")
                return out
            if tgt is torch.ops.loopfuse.paged_load.default:
                pool, table = a[0], a[1]
                if not (isinstance(table, Ids) and pool.src.kind == "node" and table.src.kind == "node"):
                    raise _Skip("paged_load operands must be plain tensors")
                if pool.t.shape != pool.src.shape or table.t.shape != table.src.shape or \
                        not torch.equal(pool.t.reshape(-1), torch.arange(pool.t.numel())) or \
                        not torch.equal(table.t.reshape(-1), torch.arange(table.t.numel())):
                    raise _Skip("paged_load operands must be whole tensors, not views")
                shape = tuple(table.src.shape) + tuple(pool.src.shape[1:])
                src = Source("paged", pool.src.node, table.src.node, shape, len(table.src.shape))
                return Ids(src, torch.arange(math.prod(shape), dtype=torch.int64).reshape(shape))
            if tgt in _SDPA_OPS:
                return [sdpa_stage(node, tgt, a, kw)] + [None] * 8      # (output, log-sum-exp, ...)
            if tgt in (aten.bmm.default, aten.mm.default, aten.matmul.default) and isinstance(a[1], Ids):
                qi, ki = a[0], a[1]
                if qi.t.dim() < 3 or ki.t.dim() != qi.t.dim():
                    raise _Skip("QK^T is not a batched matmul")
                if qi.t.shape[:-2] != ki.t.shape[:-2] or qi.t.shape[-1] != ki.t.shape[-2]:
                    raise _Skip("QK^T shapes disagree")
                shape = tuple(qi.t.shape[:-1]) + (ki.t.shape[-1],)
                return Stage("scores", shape, qi, ki, mat=(shape[-2], shape[-1]))
            if tgt is aten.baddbmm.default and len(a) == 3 and isinstance(a[1], Ids) and isinstance(a[2], Ids):
                # beta * bias + alpha * (Q K^T): the score product of the decoders that spell it with baddbmm on a
                # tensor of zeros (or on a bias); alpha is the scale
                qi, ki = a[1], a[2]
                beta, alpha = kw.get("beta", 1), kw.get("alpha", 1)
                if qi.t.dim() != 3 or ki.t.dim() != 3 or qi.t.shape[0] != ki.t.shape[0] or qi.t.shape[-1] != ki.t.shape[-2]:
                    raise _Skip("baddbmm operands are not a batched Q K^T")
                if not is_number(beta) or not (is_number(alpha) or isinstance(alpha, Scalar)):
                    raise _Skip("baddbmm factors not understood")
                shape = tuple(qi.t.shape[:-1]) + (ki.t.shape[-1],)
                st = Stage("scores", shape, qi, ki, mat=(shape[-2], shape[-1]))
                raw = node.kwargs.get("alpha", 1)
                if isinstance(alpha, Scalar) or isinstance(raw, torch.fx.Node) or float(alpha) != 1.0:
                    st.factors = [alpha if isinstance(alpha, Scalar) else (raw if isinstance(raw, torch.fx.Node) else float(alpha))]
                if sym.get(node.args[0]) is index_masks.ZERO or beta == 0:
                    return st
                if beta != 1:
                    raise _Skip("baddbmm with a scaled bias")
                return dataclasses.replace(st, bias=(first, shape))
            if tgt is aten.where.self and len(a) == 3 and is_bool(first):
                # where(keep, scores, -inf) / where(masked, -inf, scores): a mask given as a boolean tensor
                pos = 1 if isinstance(a[1], Stage) else (2 if isinstance(a[2], Stage) else 0)
                if pos and is_neg_inf(a[3 - pos]):
                    return bool_mask(a[pos], first, +1 if pos == 1 else -1, node.args[0])
            raise _Skip(f"op on a tensor view: {tgt}")

        # -- the attention pipeline
        if isinstance(first, Stage):
            st = first
            if tgt in _VIEW_OPS and st.kind in ("scores", "probs"):
                # executed on ids of the canonical layout, like the views of operands
                kw2 = {k: v for k, v in kw.items() if k != "memory_format"}
                if shrink_static and tgt in (aten.view.default, aten._unsafe_view.default, aten.reshape.default,
                                             aten.expand.default):
                    a = (a[0], stand_in_view_shape(node, st.shape)) + tuple(a[2:])
                n = math.prod(st.shape)
                lay = st.lay if st.lay is not None else torch.arange(n, dtype=torch.int64).reshape(st.shape)
                try:
                    new = tgt(lay, *a[1:], **kw2)
                except Exception as e:
                    raise _Skip(f"view of the scores not reproducible: {e}")
                if new.numel() != n:
                    raise _Skip("view changes the number of scores")
                plain = tuple(new.shape[-2:]) == tuple(st.mat) and torch.equal(new.reshape(-1), torch.arange(n))
                return dataclasses.replace(st, shape=tuple(new.shape), lay=None if plain else new)
            if st.lay is not None and not (tgt in _CAST_OPS or tgt is aten.tanh.default or (
                    tgt in (aten.mul.Tensor, aten.div.Tensor) and not isinstance(a[1], (Stage, Ids, Aux)))):
                raise _Skip("scores are used in a permuted layout")
            if tgt in _SHAPE_ONLY_VIEW_OPS:
                kw2 = {k: v for k, v in kw.items() if k != "memory_format"}
                if shrink_static and tgt in (aten.view.default, aten._unsafe_view.default, aten.reshape.default,
                                             aten.expand.default):
                    a = (a[0], stand_in_view_shape(node, st.shape)) + tuple(a[2:])
                try:
                    new_shape = meta_view(tgt, st.shape, a[1:], kw2)
                except Exception as e:
                    raise _Skip(f"reshape of scores not reproducible: {e}")
                if new_shape[-2:] != st.shape[-2:] or math.prod(new_shape) != math.prod(st.shape):
                    raise _Skip("reshape changes the matrix dims of the scores")
                return dataclasses.replace(st, shape=new_shape)
            if tgt in _CAST_OPS:
                return st
            if st.kind == "scores":
                # the explicit softmax: x - run_max, exp, * exp(run_max - max), / (sum + c)
                if tgt is torch.ops.loopfuse.scan_max.default and st.sm == "" and st.uid == 0:
                    uid_box[0] += 1
                    st.uid = uid_box[0]
                    return [Aux("run", st.uid), Aux("fin", st.uid)]
                if tgt is aten.sub.Tensor and st.sm == "" and st.uid and isinstance(a[1], Aux) and a[1].kind == "run" \
                        and a[1].uid == st.uid and kw.get("alpha", 1) == 1:
                    return dataclasses.replace(st, sm="minus_run")
                if tgt in (aten.exp2.default, aten.exp.default) and st.sm == "minus_run":
                    return dataclasses.replace(st, sm="exp_run", base2=tgt is aten.exp2.default)
                if tgt is aten.mul.Tensor and st.sm == "exp_run" and isinstance(a[1], Aux) and a[1].kind == "expgap" \
                        and a[1].uid == st.uid and a[1].base2 == st.base2:
                    return dataclasses.replace(st, sm="num")
                if tgt is aten.sum.dim_IntList and st.sm == "num" and list(a[1]) in ([-1], [len(st.shape) - 1]) \
                        and len(a) > 2 and a[2] is True:
                    return Aux("den", st.uid)
                if tgt is aten.div.Tensor and st.sm == "num" and isinstance(a[1], Aux) and a[1].kind == "den" \
                        and a[1].uid == st.uid:
                    return dataclasses.replace(st, kind="probs", sm="", denom_add=a[1].c)
                if st.sm != "":
                    raise _Skip(f"op inside an explicit softmax: {tgt}")
                # a positive constant factor commutes with the mask (-inf stays -inf)
                if tgt in (aten.mul.Tensor, aten.div.Tensor) and st.mask is not None and st.bias is None and st.uid == 0 \
                        and (isinstance(a[1], Scalar) or (is_number(a[1]) and (a[1] > 0 or isinstance(node.args[1], torch.fx.Node)))):
                    raw = node.args[1]
                    if isinstance(a[1], Scalar):
                        f = a[1]
                    else:
                        f = raw if isinstance(raw, torch.fx.Node) else float(a[1])
                    if tgt is aten.div.Tensor:
                        f = ("recip", f)
                    new = dataclasses.replace(st)
                    if st.has_tanh:
                        new.post_factors = st.post_factors + [f]
                    else:
                        new.factors = st.factors + [f]
                    if not is_number(f):
                        # a factor only known per call (D ** -0.5 of a dynamic D): its sign is checked then
                        new.late_factors = st.late_factors + [f]
                    return new
            if st.kind == "scores" and tgt is aten.add.Tensor and isinstance(a[1], Stage):
                # Q K^T + Q2 K2^T: two bare products (or two products with the same factors)
                o = a[1]
                plain = lambda x: (x.kind == "scores" and x.q2 is None and not x.has_tanh and x.mask is None
                                   and x.bias is None and x.uid == 0 and x.sm == "" and not x.post_factors)
                if not (plain(st) and plain(o)) or kw.get("alpha", 1) != 1 or tuple(st.shape) != tuple(o.shape):
                    raise _Skip("sum of two score tensors that are not bare products of one shape")
                same = len(st.factors) == len(o.factors) and all(_same_scalar(x, y) for x, y in zip(st.factors, o.factors))
                if not same:
                    raise _Skip("the two score products carry different factors")
                return dataclasses.replace(st, q2=o.q, kt2=o.kt)
            if st.kind == "scores" and tgt is aten.add.Tensor and isinstance(a[1], Ids) and st.mask is None \
                    and st.bias is None and kw.get("alpha", 1) == 1:
                return dataclasses.replace(st, bias=(a[1], st.shape))
            if st.kind == "out" and tgt is aten.add.Tensor and isinstance(a[1], Ids) and st.out_bias is None \
                    and kw.get("alpha", 1) == 1:
                return dataclasses.replace(st, out_bias=(a[1], st.shape))
            if st.kind == "scores" and st.bias is not None and tgt in (aten.mul.Tensor, aten.div.Tensor, aten.tanh.default):
                raise _Skip("score modification after the additive bias")
            if st.kind == "scores":
                if tgt in (aten.mul.Tensor, aten.div.Tensor) and st.mask is None:
                    other = a[1]
                    raw = node.args[1]
                    if isinstance(other, Scalar):
                        f = other
                    elif is_number(other):
                        f = raw if isinstance(raw, torch.fx.Node) else float(other)
                    else:
                        raise _Skip("scores multiplied by a tensor")
                    if tgt is aten.div.Tensor:
                        f = ("recip", f)
                    new = dataclasses.replace(st)
                    if st.has_tanh:
                        new.post_factors = st.post_factors + [f]
                    else:
                        new.factors = st.factors + [f]
                    return new
                if tgt is aten.tanh.default and not st.has_tanh and st.mask is None:
                    return dataclasses.replace(st, has_tanh=True)
                if tgt is torch.ops.loopfuse.causal_mask.default and st.mask is None:
                    return dataclasses.replace(st, mask="causal")
                if tgt in (aten.masked_fill.Scalar, aten.masked_fill.Tensor) and len(a) == 3 and isinstance(a[1], Ids) \
                        and is_bool(a[1]) and is_neg_inf(a[2]):
                    return bool_mask(st, a[1], -1, node.args[1])          # scores.masked_fill(masked, -inf)
                if tgt is aten.full_like.default and len(a) > 1 and is_neg_inf(a[1]):
                    return Scalar(node, float("-inf"), ("lit", float("-inf")))     # the other branch of a where()
                if tgt is torch.ops.loopfuse.sliding_mask.default and st.mask is None:
                    w = node.args[1]
                    return dataclasses.replace(st, mask="sliding", window=w if isinstance(w, torch.fx.Node) else int(a[1]))
                if tgt is aten._softmax.default:
                    dim = a[1]
                    # (a[2], half_to_float: the probabilities of fp16 scores come out in fp32 -- what
                    # softmax(..., dtype=torch.float32) traces to; a cast like any other to the matcher)
                    if dim not in (-1, len(st.shape) - 1):
                        raise _Skip("softmax not over the key dimension")
                    return dataclasses.replace(st, kind="probs")
                raise _Skip(f"unsupported score modification: {tgt}")
            if st.kind == "probs":
                if tgt in (aten.bmm.default, aten.mm.default, aten.matmul.default) and isinstance(a[1], Ids):
                    vi = a[1]
                    if vi.t.dim() != len(st.shape) or vi.t.shape[:-2] != st.shape[:-2] or vi.t.shape[-2] != st.shape[-1]:
                        raise _Skip("PV shapes disagree")
                    return dataclasses.replace(st, kind="out", v=vi, shape=tuple(st.shape[:-1]) + (vi.t.shape[-1],))
                raise _Skip(f"unsupported op on probabilities: {tgt}")
            raise _Skip(f"op on the attention output: {tgt}")

        raise _Skip(f"ordinary node {node.name}")

    for node in graph.nodes:
        if node.op == "placeholder":
            continue
        if node.op == "output":
            consume(node.all_input_nodes)
            continue
        if node.op == "get_attr":
            # a constant tensor of the graph (torch.tensor([...]) in the traced function): a value that is
            # simply there, like the result of an ordinary op
            val = node.meta.get("val")
            if not isinstance(val, torch.Tensor):
                try:
                    val = getattr(gm, node.target)
                except AttributeError:
                    val = None
            env[node] = fresh_ids(node, val) if isinstance(val, torch.Tensor) else None
            continue
        if node.op != "call_function":
            raise NoMatch(f"unsupported node kind {node.op}")
        sym[node] = index_masks.step(node, sym)       # masks built from indices alone, as predicates
        a = arg(node.args)
        kw = arg(node.kwargs)
        first = a[0] if a else None
        try:
            env[node] = pattern_step(node, node.target, a, kw, first)
            continue
        except _Skip as e:
            if node.target in _SDPA_OPS or any(isinstance(x, Stage) for x in list(a) + list(kw.values())):
                reasons.append(str(e))
        # an ordinary op: it keeps running as it is; finished attentions it reads are fused
        consume(node.all_input_nodes)
        val = node.meta.get("val")
        if isinstance(val, torch.Tensor):
            env[node] = fresh_ids(node, val)
        elif isinstance(val, (tuple, list)):
            env[node] = None      # its elements are reached through getitem nodes, each a source of its own
        elif isinstance(val, (torch.SymInt, int)) and not isinstance(val, bool):
            env[node] = concrete(val)
        elif isinstance(val, (torch.SymFloat, float)):
            env[node] = Scalar(node, 1.0, ("arg", node))
        else:
            env[node] = None

    if not matches:
        raise NoMatch(reasons[0] if reasons else "no attention pattern in the graph")
    return matches


def _build_match(out_node: torch.fx.Node, st: Stage) -> AttentionMatch:
    """Operands, factors and biases of a finished attention in terms of graph nodes."""
    inputs: list = []

    def slot(n: torch.fx.Node) -> int:
        if n not in inputs:
            inputs.append(n)
        return inputs.index(n)

    if st.q2 is not None and st.q.t.shape[-1] != st.v.t.shape[-1] and st.q2.t.shape[-1] == st.v.t.shape[-1]:
        # the product whose depth is V's head dim is the kernel's main one
        st = dataclasses.replace(st, q=st.q2, kt=st.kt2, q2=st.q, kt2=st.kt)
    qperm, qg = _fit_operand(st.q.t, st.q.src, rows_are_d=False)
    kperm, kg = _fit_operand(st.kt.t, st.kt.src, rows_are_d=True)
    vperm, vg = _fit_operand(st.v.t, st.v.src, rows_are_d=False)
    if st.q.src.kind != "node" or qg != 1:
        raise NoMatch("Q must be a plain tensor")
    if kg != vg:
        raise NoMatch("K and V head repeat factors differ")

    def operand(ids: Ids, perm, g) -> Operand:
        if ids.src.kind == "paged":
            if perm != (0, 2, 1, 3) or ids.src.table_rank != 2:
                raise NoMatch("paged operand must be pool[N,(P,)H,D] gathered by table[B,pages]")
            return Operand(slot(ids.src.node), (), True, slot(ids.src.table_node), g)
        return Operand(slot(ids.src.node), perm, False, -1, g)

    q_op = operand(st.q, qperm, qg)
    k_op = operand(st.kt, kperm, kg)
    v_op = operand(st.v, vperm, vg)

    q2_op = k2_op = None
    if st.q2 is not None:
        q2perm, q2g = _fit_operand(st.q2.t, st.q2.src, rows_are_d=False)
        k2perm, k2g = _fit_operand(st.kt2.t, st.kt2.src, rows_are_d=True)
        if st.q2.src.kind != "node" or q2g != 1 or st.kt2.src.kind != "node":
            raise NoMatch("the second score product needs plain (unpaged) tensors")
        q2_op = operand(st.q2, q2perm, q2g)
        k2_op = operand(st.kt2, k2perm, k2g)

    q_src_shape = tuple(st.q.src.shape) if len(st.q.src.shape) == 4 else (1,) + tuple(st.q.src.shape)
    qshape = tuple(q_src_shape[i] for i in qperm)          # stand-in [B, Hq, Sq, D]
    if len(st.shape) == 4:
        if tuple(st.shape) != qshape:
            raise NoMatch("output is not shaped [B, Hq, Sq, D]")
        out_rank = 4
    elif len(st.shape) == 3:
        if tuple(st.shape) != (qshape[0] * qshape[1], qshape[2], qshape[3]):
            raise NoMatch("output is not shaped [B*Hq, Sq, D]")
        out_rank = 3
    else:
        raise NoMatch("unsupported output rank")

    def scalar(f):
        if isinstance(f, tuple) and f[0] == "recip":
            return ("recip", scalar(f[1]))
        if isinstance(f, Scalar):
            if f.expr is None:
                return ("arg", slot(f.node))        # not understood: the graph computes it, the call reads it

            def conv(e):
                if e[0] == "arg":
                    return ("arg", slot(e[1]))
                if e[0] == "dim":
                    return ("dim", slot(e[1]), e[2])
                return e if e[0] == "lit" else e[:2] + tuple(conv(x) for x in e[2:])
            return ("expr", conv(f.expr))
        if isinstance(f, torch.fx.Node):
            return ("arg", slot(f))
        return f

    sk = st.kt.t.shape[-1]
    bias_op = obias_op = None
    if st.bias is not None:
        n, dims = _fit_bias(st.bias, (qshape[0], qshape[1], qshape[2], sk))
        bias_op = BiasOperand(slot(n), dims, st.bias_keep)
    if st.out_bias is not None:
        n, dims = _fit_bias(st.out_bias, qshape)
        obias_op = BiasOperand(slot(n), dims)
    window = scalar(st.window) if st.mask == "sliding" else 0
    out_order = ()
    val = out_node.meta.get("val")
    if out_rank == 4 and isinstance(val, torch.Tensor) and val.dim() == 4:
        strides = [s_ if isinstance(s_, int) else _hint(s_) for s_ in val.stride()]
        order = tuple(sorted(range(4), key=lambda i: (-strides[i], i)))
        if order[3] != 3:
            raise NoMatch("traced output does not keep the head dim innermost")
        if order != (0, 1, 2, 3):
            out_order = order
    return AttentionMatch(out_node, inputs, q_op, k_op, v_op, [scalar(f) for f in st.factors],
                          [scalar(f) for f in st.post_factors], st.has_tanh, st.mask, window, out_rank,
                          bias_op, obias_op, denom_add=tuple(scalar(t) for t in st.denom_add), base2=st.base2,
                          q2=q2_op, k2=k2_op, late_factors=tuple(scalar(f) for f in st.late_factors),
                          out_order=out_order, zero_blind_rows=st.zero_blind_rows)
