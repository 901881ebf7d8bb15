"""Graph capture: recognise ``softmax(mask(mods(Q K^T))) V`` in an ATen graph.

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

    kind: str                      # "input" | "paged" | "computed"
    index: int                     # placeholder position (pool, for paged; -1 for computed)
    table_index: int = -1          # placeholder position of the page table
    shape: tuple[int, ...] = ()    # stand-in shape the ids enumerate (row-major)
    table_rank: int = 0            # paged: leading dims that come from the table
    node: Any = None               # computed: the fx node whose value (an elementwise combination of
                                   # inputs, e.g. Q + q_bias) is evaluated eagerly at call time


@dataclasses.dataclass
class Ids:
    src: Source
    t: torch.Tensor                # int64 element ids into src (row-major over src.shape)


@dataclasses.dataclass
class Scalar:
    node: torch.fx.Node            # re-evaluated at call time
    value: float                   # value for the stand-in sizes (unused beyond sanity)


@dataclasses.dataclass
class Stage:
    kind: str                      # "scores" | "probs" | "out"
    shape: tuple[int, ...]         # stand-in logical shape
    q: Ids
    kt: Ids                        # K^T operand [.., D, Sk]
    v: Optional[Ids] = None
    factors: list = dataclasses.field(default_factory=list)       # multipliers before tanh
    post_factors: list = dataclasses.field(default_factory=list)  # multipliers after tanh
    has_tanh: bool = False
    mask: Optional[str] = None
    window: Any = 0                # int or fx.Node (SymInt)
    bias: Optional[tuple] = None       # (Ids, stage shape when added): additive score bias, before the mask
    out_bias: Optional[tuple] = None   # (Ids, stage shape when added): additive output bias


_VIEW_OPS = {
    aten.view.default, aten._unsafe_view.default, aten.reshape.default, aten.expand.default,
    aten.transpose.int, aten.permute.default, aten.unsqueeze.default, aten.squeeze.dim,
    aten.clone.default, aten.alias.default, aten.t.default, aten.contiguous.default,
    aten.detach.default,
}
_SHAPE_ONLY_VIEW_OPS = {aten.view.default, aten._unsafe_view.default, aten.reshape.default,
                        aten.expand.default, aten.clone.default, aten.alias.default,
                        aten.detach.default, aten.contiguous.default}
_CAST_OPS = {prims.convert_element_type.default, aten._to_copy.default}
_ELEMENTWISE_OPS = {aten.add.Tensor, aten.sub.Tensor, aten.mul.Tensor, aten.div.Tensor}
_SCALAR_OPS = {aten.scalar_tensor.default, aten.pow.Tensor_Tensor, aten.pow.Tensor_Scalar,
               aten.pow.Scalar, aten.mul.Tensor, aten.div.Tensor, aten.reciprocal.default,
               aten.sqrt.default, aten.rsqrt.default, aten.neg.default,
               prims.convert_element_type.default, aten._to_copy.default}


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
    """How to obtain a [B, H, S, D] strided view of Q/K/V from the call's arguments."""

    index: int                     # placeholder position of the tensor (pool when paged)
    perm: tuple[int, ...] = ()     # dense: permutation giving [B, H, S, D]
    paged: bool = False
    table_index: int = -1
    group: int = 1                 # head repeat factor seen in the graph (stand-in value)
    node: Any = None               # computed operand: fx node evaluated eagerly at call time


@dataclasses.dataclass
class BiasOperand:
    """An additive bias as a strided [B, Hq, Sq, X] view of a graph input (or computed value)."""

    index: int
    node: Any
    dims: tuple                    # per logical dim (b, h, row, col): source dim it walks, or None (broadcast)


@dataclasses.dataclass
class AttentionMatch:
    gm: torch.fx.GraphModule
    placeholders: list[torch.fx.Node]
    q: Operand
    k: Operand
    v: Operand
    factors: list                  # floats / fx.Nodes, multiplied together
    post_factors: list
    has_tanh: bool
    mask: Optional[str]
    window: Any
    out_rank: int
    bias: Optional[BiasOperand] = None
    out_bias: Optional[BiasOperand] = None

    def describe(self) -> str:
        return (f"attention: Q=arg{self.q.index}{self.q.perm} K=arg{self.k.index}"
                f"{'[paged by arg%d]' % self.k.table_index if self.k.paged else self.k.perm} "
                f"V=arg{self.v.index}{'[paged by arg%d]' % self.v.table_index if self.v.paged else self.v.perm} "
                f"mask={self.mask} window={self.window} tanh={self.has_tanh} "
                f"factors={self.factors} post={self.post_factors}"
                f"{' +score_bias' if self.bias else ''}{' +out_bias' if self.out_bias else ''}")

    # -- call-time evaluation of shape-derived scalars
    def _eval(self, x, env: dict) -> Any:
        if isinstance(x, tuple) and len(x) == 2 and x[0] == "recip":   # from aten.div
            val = self._eval(x[1], env)
            return 1.0 / float(val.item() if isinstance(val, torch.Tensor) else val)
        if isinstance(x, torch.fx.Node):
            if x in env:
                return env[x]
            args = torch.fx.node.map_arg(x.args, lambda n: self._eval(n, env))
            kwargs = torch.fx.node.map_arg(x.kwargs, lambda n: self._eval(n, env))
            kwargs = {k: v for k, v in kwargs.items() if k != "device"}
            val = x.target(*args, **kwargs)
            env[x] = val
            return val
        return x

    def _product(self, items, env) -> float:
        r = 1.0
        for f in items:
            val = self._eval(f, env)
            r *= float(val.item() if isinstance(val, torch.Tensor) else val)
        return r

    def plan_for(self, args) -> lowering.AttnPlan:
        env = {p: a for p, a in zip(self.placeholders, args)}
        pre = self._product(self.factors, env)
        if self.has_tanh:
            cap = self._product(self.post_factors, env)
            scale, softcap = pre * cap, cap
        else:
            scale, softcap = pre, None
        window = self._eval(self.window, env) if self.mask == "sliding" else 0
        return lowering.AttnPlan(mask=self.mask, window=int(window), scale=scale, softcap=softcap,
                                 k_paged=self.k.paged, v_paged=self.v.paged)

    def _source(self, index: int, node, args):
        if node is None:
            return args[index]
        env = {p: a for p, a in zip(self.placeholders, args)}
        return self._eval(node, env)      # e.g. Q + q_bias: run those graph nodes as they are

    def _operand(self, op: Operand, args):
        t = self._source(op.index, op.node, args)
        if op.paged:
            return t, args[op.table_index]
        return t.permute(op.perm), None

    def _bias_view(self, bo: Optional[BiasOperand], args, shape):
        if bo is None:
            return None
        t = self._source(bo.index, bo.node, args)
        strides = tuple(0 if d is None else t.stride(d) for d in bo.dims)
        for size, d in zip(shape, bo.dims):
            if d is not None and t.shape[d] != size:
                raise lowering.UnsupportedPlan("bias does not have the shape seen at trace time")
        return torch.as_strided(t, tuple(shape), strides, t.storage_offset())

    def run(self, args) -> torch.Tensor:
        q, _ = self._operand(self.q, args)
        if not q.is_cuda:
            raise lowering.UnsupportedPlan("tensors are not on the GPU")
        k, kt = self._operand(self.k, args)
        v, vt = self._operand(self.v, args)
        B, Hq, Sq, D = q.shape
        Sk = kt.shape[1] * (k.shape[1] if k.dim() == 4 else 1) if kt is not None else k.shape[2]
        out = lowering.attention(q, k, v, self.plan_for(args), kt, vt,
                                 score_bias=self._bias_view(self.bias, args, (B, Hq, Sq, Sk)),
                                 out_bias=self._bias_view(self.out_bias, args, (B, Hq, Sq, D)))
        if self.out_rank == 3:
            out = out.view(out.shape[0] * out.shape[1], out.shape[2], out.shape[3])
        return out

    def kernel_specs_for(self, args):
        """Specialisations the call would use (for CODEGEN_ONLY; no GPU needed)."""
        q, _ = self._operand(self.q, args)
        plan = self.plan_for(args)
        k = args[self.k.index]
        D = q.shape[-1]
        dt = lowering._DTYPE_CODE.get(q.dtype)
        if dt is None or D not in (64, 128):
            raise lowering.UnsupportedPlan("dtype/head dim not served by the HIP kernels")
        paged = (1 if self.k.paged else 0) | (2 if self.v.paged else 0)
        ps = 1
        i64 = False
        if self.k.paged:
            ps = k.shape[1] if k.dim() == 4 else 1
            i64 = args[self.k.table_index].dtype == torch.int64
        mask = lowering._MASK_NAMES[plan.mask]
        bias = (1 if self.bias else 0) | (2 if self.out_bias else 0)
        family = "prefill" if (paged or bias) else lowering.prefill_variant(q.shape[-2])
        extra = ("-DLF_DMA=1",) if (bias and not paged) else ()
        return [lowering.KernelSpec(family, dt, D, mask, plan.softcap is not None, paged, ps, i64, bias=bias, extra=extra)]


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


def _fit_bias(entry: tuple, logical: tuple) -> BiasOperand:
    """Express a bias (ids broadcast against the stage it was added to) as a strided
    [B, Hq, Sq, X] view of its source: per logical dim, the source dim it walks."""
    ids, stage_shape = entry
    src = ids.src
    if src.kind not in ("input", "computed"):
        raise NoMatch("bias must be a graph input or an elementwise combination of inputs")
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
    return BiasOperand(src.index, src.node, tuple(dims))


def match_attention(gm: torch.fx.GraphModule) -> AttentionMatch:
    """Interpret ``gm`` abstractly; return the match or raise ``NoMatch``.

    The fw_compiler runs under AOTAutograd's fake-tensor mode; the stand-in id
    tensors must be real, so dispatch modes are switched off for the duration.
    """
    from torch.utils._python_dispatch import _disable_current_modes

    with _disable_current_modes():
        return _match_attention(gm)


def _match_attention(gm: torch.fx.GraphModule) -> AttentionMatch:
    graph = gm.graph
    placeholders = [n for n in graph.nodes if n.op == "placeholder"]
    outputs = [n for n in graph.nodes if n.op == "output"]
    if len(outputs) != 1:
        raise NoMatch("no single output node")
    out_args = outputs[0].args[0]
    if not isinstance(out_args, (tuple, list)) or len(out_args) != 1 or not isinstance(out_args[0], torch.fx.Node):
        raise NoMatch("graph does not return exactly one tensor")

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

    def concrete(d) -> int:
        if isinstance(d, torch.SymInt):
            return int(d.node.expr.subs(sizes))
        return int(d)

    env: dict[torch.fx.Node, Any] = {}
    for i, p in enumerate(placeholders):
        val = p.meta.get("val")
        if isinstance(val, torch.Tensor):
            shape = tuple(concrete(d) for d in val.shape)
            n = math.prod(shape)
            if n > (1 << 22):
                raise NoMatch("stand-in tensor too large")
            env[p] = Ids(Source("input", i, shape=shape), torch.arange(n, dtype=torch.int64).reshape(shape))
        elif isinstance(val, (torch.SymInt, int)):
            env[p] = concrete(val)
        elif isinstance(val, (torch.SymFloat, float)):
            env[p] = Scalar(p, float(val) if isinstance(val, float) else 1.0)
        else:
            raise NoMatch(f"unsupported placeholder {p.name}")

    def arg(a):
        return torch.fx.node.map_arg(a, lambda n: env[n])

    def is_number(x) -> bool:
        return isinstance(x, (int, float)) and not isinstance(x, bool)

    def meta_view(target, shape, args, kwargs):
        m = torch.empty(shape, device="meta")
        return tuple(target(m, *args, **kwargs).shape)

    for node in graph.nodes:
        if node.op in ("placeholder", "output"):
            continue
        if node.op == "get_attr":
            raise NoMatch("graph has constant tensors")
        if node.op != "call_function":
            raise NoMatch(f"unsupported node kind {node.op}")
        tgt = node.target
        a = arg(node.args)
        kw = arg(node.kwargs)
        first = a[0] if a else None

        # -- integer / float arithmetic on sizes
        if all(is_number(x) for x in a) and tgt in (
                operator.mul, operator.floordiv, operator.add, operator.sub, operator.truediv,
                operator.pow, operator.neg, operator.mod):
            env[node] = tgt(*a)
            continue
        if tgt in (aten.sym_size.int,):
            # size of an intermediate (duck-sized batch == heads makes dynamo re-read it)
            if isinstance(first, Stage):
                env[node] = int(first.shape[a[1]])
            elif isinstance(first, Ids):
                env[node] = int(first.t.shape[a[1]])
            else:
                raise NoMatch("sym_size on an unsupported value")
            continue

        # -- scalars derived from sizes
        if tgt is aten.scalar_tensor.default:
            env[node] = Scalar(node, float(a[0]))
            continue
        if isinstance(first, Scalar) and tgt in _SCALAR_OPS and all(
                isinstance(x, (Scalar, int, float, torch.dtype)) for x in a):
            env[node] = Scalar(node, 1.0)
            continue

        # -- tensor + scores / tensor + output with the tensor written first
        if tgt is aten.add.Tensor and isinstance(first, Ids) and len(a) > 1 and isinstance(a[1], Stage) \
                and not kw.get("alpha", 1) != 1:
            a = (a[1], a[0]) + tuple(a[2:])
            first = a[0]

        # -- views of inputs
        if isinstance(first, Ids):
            if tgt in _ELEMENTWISE_OPS and len(a) == 2 and isinstance(a[1], (Ids, int, float)) \
                    and not isinstance(a[1], bool) and not kw:
                # an elementwise combination of inputs (the reference's Q + q_bias,
                # tests/test_accuracy.py:176): a new source, computed eagerly per call
                other_shape = tuple(a[1].t.shape) if isinstance(a[1], Ids) else ()
                try:
                    shape = tuple(torch.broadcast_shapes(tuple(first.t.shape), other_shape))
                except RuntimeError as e:
                    raise NoMatch(f"elementwise operands do not broadcast: {e}")
                n = math.prod(shape)
                src = Source("computed", -1, shape=shape, node=node)
                env[node] = Ids(src, torch.arange(n, dtype=torch.int64).reshape(shape))
                continue
            if tgt in _VIEW_OPS:
                try:
                    env[node] = Ids(first.src, tgt(first.t, *a[1:], **kw))
                except Exception as e:  # invalid for the stand-in sizes
                    raise NoMatch(f"view chain not reproducible on stand-in sizes: {e}")
                continue
            if tgt is torch.ops.loopfuse.paged_load.default:
                pool, table = a[0], a[1]
                if not (isinstance(table, Ids) and pool.src.kind == "input" and table.src.kind == "input"):
                    raise NoMatch("paged_load operands must be graph inputs")
                if pool.t.shape != pool.src.shape or table.t.shape != table.src.shape or \
                        not torch.equal(pool.t.reshape(-1), torch.arange(pool.t.numel())) or \
                        not torch.equal(table.t.reshape(-1), torch.arange(table.t.numel())):
                    raise NoMatch("paged_load operands must be untouched graph inputs")
                shape = tuple(table.src.shape) + tuple(pool.src.shape[1:])
                src = Source("paged", pool.src.index, table.src.index, shape, len(table.src.shape))
                env[node] = Ids(src, torch.arange(math.prod(shape), dtype=torch.int64).reshape(shape))
                continue
            if tgt in (aten.bmm.default, aten.mm.default, aten.matmul.default) and isinstance(a[1], Ids):
                qi, ki = a[0], a[1]
                if qi.t.dim() < 3 or ki.t.dim() != qi.t.dim():
                    raise NoMatch("QK^T is not a batched matmul")
                if qi.t.shape[:-2] != ki.t.shape[:-2] or qi.t.shape[-1] != ki.t.shape[-2]:
                    raise NoMatch("QK^T shapes disagree")
                shape = tuple(qi.t.shape[:-1]) + (ki.t.shape[-1],)
                env[node] = Stage("scores", shape, qi, ki)
                continue
            raise NoMatch(f"unsupported op on an input view: {tgt}")

        # -- the attention pipeline
        if isinstance(first, Stage):
            st = first
            if tgt in _SHAPE_ONLY_VIEW_OPS:
                kw2 = {k: v for k, v in kw.items() if k != "memory_format"}
                try:
                    new_shape = meta_view(tgt, st.shape, a[1:], kw2)
                except Exception as e:
                    raise NoMatch(f"reshape of scores not reproducible: {e}")
                if new_shape[-2:] != st.shape[-2:] or math.prod(new_shape) != math.prod(st.shape):
                    raise NoMatch("reshape changes the matrix dims of the scores")
                env[node] = dataclasses.replace(st, shape=new_shape)
                continue
            if tgt in _CAST_OPS:
                env[node] = st
                continue
            if st.kind == "scores" and tgt is aten.add.Tensor and isinstance(a[1], Ids) and st.mask is None \
                    and st.bias is None and kw.get("alpha", 1) == 1:
                env[node] = dataclasses.replace(st, bias=(a[1], st.shape))
                continue
            if st.kind == "out" and tgt is aten.add.Tensor and isinstance(a[1], Ids) and st.out_bias is None \
                    and kw.get("alpha", 1) == 1:
                env[node] = dataclasses.replace(st, out_bias=(a[1], st.shape))
                continue
            if st.kind == "scores" and st.bias is not None and tgt in (aten.mul.Tensor, aten.div.Tensor, aten.tanh.default):
                raise NoMatch("score modification after the additive bias")
            if st.kind == "scores":
                if tgt in (aten.mul.Tensor, aten.div.Tensor) and st.mask is None:
                    other = a[1]
                    raw = node.args[1]
                    if isinstance(other, Scalar):
                        f = other.node
                    elif is_number(other):
                        f = raw if isinstance(raw, torch.fx.Node) else float(other)
                    else:
                        raise NoMatch("scores multiplied by a tensor (bias/modified attention)")
                    if tgt is aten.div.Tensor:
                        f = ("recip", f)
                    new = dataclasses.replace(st)
                    if st.has_tanh:
                        new.post_factors = st.post_factors + [f]
                    else:
                        new.factors = st.factors + [f]
                    env[node] = new
                    continue
                if tgt is aten.tanh.default and not st.has_tanh and st.mask is None:
                    env[node] = dataclasses.replace(st, has_tanh=True)
                    continue
                if tgt is torch.ops.loopfuse.causal_mask.default and st.mask is None:
                    env[node] = dataclasses.replace(st, mask="causal")
                    continue
                if tgt is torch.ops.loopfuse.sliding_mask.default and st.mask is None:
                    w = node.args[1]
                    env[node] = dataclasses.replace(st, mask="sliding", window=w if isinstance(w, torch.fx.Node) else int(a[1]))
                    continue
                if tgt is aten._softmax.default:
                    dim = a[1]
                    if dim not in (-1, len(st.shape) - 1) or a[2]:
                        raise NoMatch("softmax not over the key dimension")
                    env[node] = dataclasses.replace(st, kind="probs")
                    continue
                raise NoMatch(f"unsupported score modification: {tgt}")
            if st.kind == "probs":
                if tgt in (aten.bmm.default, aten.mm.default, aten.matmul.default) and isinstance(a[1], Ids):
                    vi = a[1]
                    if vi.t.dim() != len(st.shape) or vi.t.shape[:-2] != st.shape[:-2] or vi.t.shape[-2] != st.shape[-1]:
                        raise NoMatch("PV shapes disagree")
                    env[node] = dataclasses.replace(st, kind="out", v=vi, shape=tuple(st.shape[:-1]) + (vi.t.shape[-1],))
                    continue
                raise NoMatch(f"unsupported op on probabilities: {tgt}")
            raise NoMatch(f"unsupported op on the attention output: {tgt}")

        raise NoMatch(f"unsupported node {node.format_node()}")

    result = env.get(out_args[0])
    if not isinstance(result, Stage) or result.kind != "out":
        raise NoMatch("output is not an attention result")
    st = result
    qperm, qg = _fit_operand(st.q.t, st.q.src, rows_are_d=False)
    kperm, kg = _fit_operand(st.kt.t, st.kt.src, rows_are_d=True)
    vperm, vg = _fit_operand(st.v.t, st.v.src, rows_are_d=False)
    if st.q.src.kind not in ("input", "computed") or qg != 1:
        raise NoMatch("Q must be a graph input or an elementwise combination of inputs")
    if kg != vg:
        raise NoMatch("K and V head repeat factors differ")

    def operand(ids: Ids, perm, g) -> Operand:
        if ids.src.kind == "paged":
            if perm != (0, 2, 1, 3) or ids.src.table_rank != 2:
                raise NoMatch("paged operand must be pool[N,(P,)H,D] gathered by table[B,pages]")
            return Operand(ids.src.index, (), True, ids.src.table_index, g)
        return Operand(ids.src.index, perm, False, -1, g, node=ids.src.node)

    q_op = operand(st.q, qperm, qg)
    k_op = operand(st.kt, kperm, kg)
    v_op = operand(st.v, vperm, vg)

    qshape = tuple(st.q.src.shape[i] for i in qperm)       # stand-in [B, Hq, Sq, D]
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

    sk = st.kt.t.shape[-1]
    bias_op = _fit_bias(st.bias, (qshape[0], qshape[1], qshape[2], sk)) if st.bias is not None else None
    obias_op = _fit_bias(st.out_bias, qshape) if st.out_bias is not None else None
    m = AttentionMatch(gm, placeholders, q_op, k_op, v_op, list(st.factors), list(st.post_factors),
                       st.has_tanh, st.mask, st.window, out_rank, bias_op, obias_op)
    return m
