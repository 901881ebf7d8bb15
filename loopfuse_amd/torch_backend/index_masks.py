"""Masks that a graph builds from indices alone, read as predicates on (row, column).

``torch.ones(S, S).tril()``, ``arange(S)[:, None] >= arange(S)[None, :]``, ``(i - j) < w`` and their
conjunctions do not depend on any data: they are boolean functions of the element's position.
This module follows such values through an ATen graph symbolically -- an integer tensor is an affine
form in the indices of its last dims, a boolean tensor a conjunction of ``form >= 0`` clauses (or the
negation of one) -- so that the front end can tell a causal or a sliding-window mask from its
definition and hand it to the kernels as a flag (tiles outside the band are never visited,
``loopfuse/compiler/passes/skip_loop_iterations.py:267-378`` derives the same from the predicate of
its mask ops) instead of as a tensor.  Whatever is not understood simply has no symbolic value; the
caller then treats the mask as data.

Positions are counted from the right (-1 = last dim = key index j, -2 = query index i), which is how
broadcasting aligns a mask with the scores.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Optional

import torch

aten = torch.ops.aten


@dataclasses.dataclass(frozen=True)
class Aff:
    """Integer tensor whose element at index (.., x_-2, x_-1) is sum(coef[p] * x_p) + const."""

    coef: tuple                    # ((position from the right, coefficient), ...) sorted, no zeros
    const: int = 0

    @staticmethod
    def make(coef: dict, const: int = 0) -> "Aff":
        return Aff(tuple(sorted((p, c) for p, c in coef.items() if c != 0)), int(const))

    def d(self) -> dict:
        return dict(self.coef)

    def __add__(self, o):
        if isinstance(o, int):
            return Aff(self.coef, self.const + o)
        c = self.d()
        for p, k in o.coef:
            c[p] = c.get(p, 0) + k
        return Aff.make(c, self.const + o.const)

    def __neg__(self):
        return Aff(tuple((p, -k) for p, k in self.coef), -self.const)

    def __sub__(self, o):
        return self + (-o if isinstance(o, Aff) else -int(o))


@dataclasses.dataclass(frozen=True)
class Pred:
    """Boolean (or 0 / 1 valued) tensor: every clause >= 0, or the negation of that."""

    clauses: tuple = ()            # of Aff
    negated: bool = False

    def __invert__(self):
        if len(self.clauses) == 1 and not self.negated:
            # not (e >= 0)  <=>  -e - 1 >= 0 for integers: stays a plain conjunction
            return Pred(((-self.clauses[0]) + (-1),), False)
        return Pred(self.clauses, not self.negated)

    def plain(self) -> Optional["Pred"]:
        if not self.negated:
            return self
        if len(self.clauses) == 1:
            return ~Pred(self.clauses, False)
        return None

    def __and__(self, o):
        a, b = self.plain(), o.plain()
        if a is None or b is None:
            return None
        return Pred(a.clauses + b.clauses, False)


class _Zero:
    """A tensor of zeros (``torch.zeros(...)`` and views of it): as an additive term it is nothing."""

    def __repr__(self):
        return "ZERO"


ZERO = _Zero()


def _is_int(x) -> bool:
    return isinstance(x, int) and not isinstance(x, bool)


def _shift(v, rank: int, dim: int):
    """Positions after ``unsqueeze(dim)`` of a rank-``rank`` value."""
    if dim < 0:
        dim += rank + 1

    def mv(p):
        return p if rank + p >= dim else p - 1
    if isinstance(v, Aff):
        return Aff.make({mv(p): c for p, c in v.coef}, v.const)
    return Pred(tuple(Aff.make({mv(p): c for p, c in cl.coef}, cl.const) for cl in v.clauses), v.negated)


def _cmp(kind: str, a, b):
    """Pred of ``a <kind> b`` for affine forms / Python ints."""
    if not isinstance(a, Aff):
        if not _is_int(a):
            return None
        a = Aff((), a)
    if not isinstance(b, Aff):
        if not _is_int(b):
            return None
        b = Aff((), b)
    if kind == "ge":
        return Pred((a - b,))
    if kind == "gt":
        return Pred((a - b + (-1),))
    if kind == "le":
        return Pred((b - a,))
    if kind == "lt":
        return Pred((b - a + (-1),))
    if kind == "eq":
        return Pred((a - b, b - a))
    if kind == "ne":
        return ~Pred((a - b, b - a))
    return None


_CMP = {aten.ge.Tensor: "ge", aten.ge.Scalar: "ge", aten.gt.Tensor: "gt", aten.gt.Scalar: "gt",
        aten.le.Tensor: "le", aten.le.Scalar: "le", aten.lt.Tensor: "lt", aten.lt.Scalar: "lt",
        aten.eq.Tensor: "eq", aten.eq.Scalar: "eq", aten.ne.Tensor: "ne", aten.ne.Scalar: "ne"}
_IDENTITY = {aten.expand.default, aten.clone.default, aten.alias.default, aten.contiguous.default,
             aten.detach.default, aten._to_copy.default, torch.ops.prims.convert_element_type.default,
             aten.to.dtype, aten.lift_fresh_copy.default}


def step(node: torch.fx.Node, sym: dict):
    """Symbolic value of ``node`` given those of its inputs (``sym``), or None."""
    t = node.target
    args = node.args
    kw = node.kwargs

    def val(x):
        return sym.get(x) if isinstance(x, torch.fx.Node) else x

    def rank(x) -> int:
        m = x.meta.get("val") if isinstance(x, torch.fx.Node) else None
        return m.dim() if isinstance(m, torch.Tensor) else -1

    if t is aten.arange.default and len(args) == 1:
        return Aff.make({-1: 1})
    if t is aten.arange.start and len(args) >= 2 and args[0] == 0 and (len(args) < 3 or args[2] == 1):
        return Aff.make({-1: 1})
    if t is aten.arange.start_step and args[0] == 0 and args[2] == 1:
        return Aff.make({-1: 1})
    if t in (aten.ones.default, aten.ones_like.default) or \
            (t in (aten.full.default, aten.full_like.default) and len(args) > 1 and args[1] in (1, 1.0, True)):
        return Pred(())                                       # true everywhere
    if t in (aten.zeros.default, aten.zeros_like.default) or \
            (t in (aten.full.default, aten.full_like.default) and len(args) > 1 and args[1] in (0, 0.0) and args[1] is not False):
        return ZERO
    if not args:
        return None
    x = val(args[0])
    if x is ZERO:
        views = _IDENTITY | {aten.unsqueeze.default, aten.slice.Tensor, aten.view.default, aten.reshape.default,
                             aten._unsafe_view.default, aten.transpose.int, aten.permute.default, aten.squeeze.dim}
        return ZERO if t in views else None
    if t in _CMP:
        a, b = x, val(args[1])
        if isinstance(a, Pred) and b in (0, 0.0, False) and _CMP[t] in ("eq", "ne"):
            return ~a if _CMP[t] == "eq" else a               # mask == 0, mask != 0
        return _cmp(_CMP[t], a, b)
    if t in (aten.add.Tensor, aten.sub.Tensor, aten.rsub.Scalar, aten.add.Scalar, aten.sub.Scalar) \
            and kw.get("alpha", 1) == 1 and len(args) == 2:
        a, b = x, val(args[1])
        if t is aten.rsub.Scalar:
            a, b = b, a
        if not (isinstance(a, Aff) or isinstance(b, Aff)) or not all(isinstance(v, Aff) or _is_int(v) for v in (a, b)):
            return None
        a = a if isinstance(a, Aff) else Aff((), a)
        return a + b if t in (aten.add.Tensor, aten.add.Scalar) else a - b
    if t is aten.neg.default and isinstance(x, Aff):
        return -x
    if x is None or not isinstance(x, (Aff, Pred)):
        return None
    if t in _IDENTITY:
        return x
    if t is aten.unsqueeze.default:
        return _shift(x, rank(args[0]), args[1])
    if t in (aten.view.default, aten.reshape.default, aten._unsafe_view.default):
        # leading dims of size 1 added (mask.view(1, 1, S, S)): positions from the right stay
        old, new = args[0].meta.get("val"), node.meta.get("val")
        if isinstance(old, torch.Tensor) and isinstance(new, torch.Tensor) and new.dim() >= old.dim() and \
                all(str(d) == "1" for d in new.shape[:new.dim() - old.dim()]) and \
                all(str(a) == str(b) for a, b in zip(new.shape[new.dim() - old.dim():], old.shape)):
            return x
        return None
    if t is aten.slice.Tensor:
        # a prefix x[..., :n] keeps every element's index
        rest = list(args[1:]) + [None] * 4
        if rest[1] in (0, None) and rest[3] in (1, None):
            return x
        return None
    if isinstance(x, Pred):
        if t in (aten.bitwise_not.default, aten.logical_not.default):
            return ~x
        if t in (aten.bitwise_and.Tensor, aten.logical_and.default, aten.mul.Tensor):
            y = val(args[1])
            return (x & y) if isinstance(y, Pred) else None
        if t in (aten.bitwise_or.Tensor, aten.logical_or.default):
            y = val(args[1])
            both = ((~x) & (~y)) if isinstance(y, Pred) else None       # a or b = not (not a and not b)
            return None if both is None else ~both
        if t in (aten.tril.default, aten.triu.default) and rank(args[0]) >= 2:
            k = args[1] if len(args) > 1 else kw.get("diagonal", 0)
            if not _is_int(k):
                return None
            band = Aff.make({-2: 1, -1: -1}, k) if t is aten.tril.default else Aff.make({-2: -1, -1: 1}, -k)
            return x & Pred((band,))
    return None


def band(p: Pred, keep: int):
    """The visible set ``lo <= i - j <= hi`` of a mask (``keep`` = +1: the predicate marks visible
    elements, -1: masked ones), or None when the predicate is anything else."""
    p = (p if keep > 0 else ~p).plain()
    if p is None or not p.clauses:
        return None
    lo, hi = -math.inf, math.inf
    for cl in p.clauses:
        c = cl.d()
        if set(c) != {-2, -1} or c[-2] != -c[-1] or abs(c[-2]) != 1:
            return None
        if c[-2] == 1:             # (i - j) + const >= 0
            lo = max(lo, -cl.const)
        else:                      # -(i - j) + const >= 0
            hi = min(hi, cl.const)
    return lo, hi
