"""Passes over the loop nests (reference ``loopfuse/optimize.py:34-60``).

  fuse             pointwise producer -> consumer inlining (reference compiler/passes/fuse.py
                   + store/load forwarding of cleanup_passes.py:183-208, as one step: a
                   temporary written by an ``Assign`` nest is substituted where it is read)
  online_softmax   the three reductions over the key atoms -- row maximum, sum of exponentials,
                   probabilities @ V -- become one pass with rescaled accumulators
                   (reference compiler/passes/factor_acc.py:23-109)
  block_skip       the mask clauses, evaluated over whole (q tile, kv tile) boxes, give the
                   range of kv tiles a q tile has to visit
                   (reference compiler/passes/skip_loop_iterations.py:26-81, 267-378)
"""
from __future__ import annotations

import dataclasses
import math
from typing import Callable, Optional, Sequence

from . import ir
from .ir import Atom, Nest


class PassError(Exception):
    pass


# ---------------------------------------------------------------- atom renaming
def _refinement(prod: Sequence[Atom], cons: Sequence[Atom]) -> dict:
    """Map each leaf of ``prod`` to the consumer leaves that index the same range (the consumer
    may have split an atom the producer iterates whole)."""
    ps = [a for a in ir.leaves(prod)]
    cs = [a for a in ir.leaves(cons)]
    out: dict = {}
    ci = 0
    for p in ps:
        if p.hint == 1:
            out[p.id] = []
            continue
        got, have = [], 1
        while have < p.hint:
            while ci < len(cs) and cs[ci].hint == 1:
                ci += 1
            if ci >= len(cs):
                raise PassError("consumer indexes a smaller range than the producer writes")
            got.append(cs[ci])
            have *= cs[ci].hint
            ci += 1
        if have != p.hint:
            raise PassError("consumer atoms do not refine the producer's")
        out[p.id] = got
    return out


def _rename_atoms(atoms: Sequence[Atom], m: dict) -> list[Atom]:
    out = []
    for a in ir.leaves(atoms):
        out.extend(m.get(a.id, [a]))
    return out


def rename(e: ir.Expr, m: dict) -> ir.Expr:
    """``e`` with every atom replaced through ``m`` (atom id -> list of atoms)."""
    def fn(x):
        if isinstance(x, ir.Read):
            g = None
            if x.gather is not None:
                g = (x.gather[0], x.gather[1], [_rename_atoms(t, m) for t in x.gather[2]])
            return ir.Read(x.buf, [_rename_atoms(d, m) for d in x.idx], g)
        if isinstance(x, ir.Select):
            cl = [ir.Clause(c.ci, c.cj, c.c0, _rename_atoms(c.row, m), _rename_atoms(c.col, m), c.c0_fn) for c in x.clauses]
            return ir.Select(cl, rename(x.a, m), x.other)
        if isinstance(x, ir.Dot):
            return ir.Dot(rename(x.a, m), rename(x.b, m), _rename_atoms(x.over, m))
        return None
    return ir.substitute(e, fn)


# ---------------------------------------------------------------- fuse
def _under_dot(e: ir.Expr, buf: ir.Buffer, inside: bool = False) -> bool:
    """Whether ``buf`` is read inside a contraction of ``e``."""
    if isinstance(e, ir.Read):
        return inside and e.buf is buf
    return any(_under_dot(c, buf, inside or isinstance(e, ir.Dot)) for c in e.children())


def is_operand_prep(nest: Nest) -> bool:
    """An element-wise nest over graph inputs alone (``Q + q_bias``): when a contraction reads its result,
    the kernels take that result as an operand, so the nest keeps running as the graph node it came from."""
    return (isinstance(nest.stmt, ir.Assign) and not nest.red and nest.stmt.buf.node is not None
            and not any(isinstance(x, (ir.Dot, ir.Select)) for x in ir.walk(nest.stmt.value))
            and all(r.buf.kind == "input" and r.gather is None for r in ir.reads(nest.stmt.value)))


def fuse(nests: list[Nest], keep: ir.Buffer, keep_contractions: bool = False, keep_operands: bool = False,
         operand_pred=None) -> list[Nest]:
    """Inline every temporary written by a pointwise (``Assign``) nest into its readers and drop
    its nest; reductions (``Accum``) and the result buffer stay.  Runs to a fixed point.

    ``keep_contractions``: a producer that holds a contraction is inlined only into a single
    pointwise reader (the epilogue of a matmul); where it would be recomputed per element of
    another contraction or reduction, or by several readers, it stays a temporary.  The
    attention pipeline inlines everything (its kernels keep the score tile on chip); the plain
    one-thread-per-element kernels would repeat the contraction instead.

    ``keep_operands``: a pointwise producer that is read only as a direct operand of contractions stays a tensor
    of its own when ``operand_pred(producer)`` holds (default: ``is_operand_prep``)."""
    nests = list(nests)
    changed = True
    while changed:
        changed = False
        for prod in nests:
            if not isinstance(prod.stmt, ir.Assign) or prod.stmt.buf is keep or prod.red:
                continue
            buf = prod.stmt.buf
            users = [n for n in nests if n is not prod and any(r.buf is buf for r in _stmt_reads(n.stmt))]
            if not users:
                continue
            if keep_contractions and any(isinstance(x, ir.Dot) for x in ir.walk(prod.stmt.value)):
                u = users[0]
                if len(users) > 1 or not isinstance(u.stmt, ir.Assign) or _under_dot(u.stmt.value, buf):
                    continue
            if keep_operands and (operand_pred or is_operand_prep)(prod) and \
                    all(_only_under_dot(u.stmt.score if isinstance(u.stmt, ir.Rescaled) else u.stmt.value, buf) for u in users):
                continue                      # an operand of the products: stays a tensor of its own

            def inline(x, buf=buf, prod=prod):
                if isinstance(x, ir.Read) and x.buf is buf:
                    m: dict = {}
                    for pd, cd in zip(buf.dims, x.idx):
                        m.update(_refinement(pd, cd))
                    return rename(prod.stmt.value, m)
                return None

            for u in users:
                u.stmt.value = ir.substitute(u.stmt.value, inline)
            nests.remove(prod)
            changed = True
            break
    return nests


def _only_under_dot(e: ir.Expr, buf: ir.Buffer, inside: bool = False) -> bool:
    """Whether every read of ``buf`` in ``e`` is a direct operand of a contraction."""
    if isinstance(e, ir.Read):
        return e.buf is not buf or inside
    if isinstance(e, ir.Dot):
        return all(_only_under_dot(c, buf, isinstance(c, ir.Read)) for c in e.children())
    return all(_only_under_dot(c, buf, False) for c in e.children())


def _stmt_reads(stmt) -> list[ir.Read]:
    if isinstance(stmt, ir.Rescaled):
        return ir.reads(stmt.score) + [stmt.weights] + ([stmt.epilogue] if stmt.epilogue is not None else [])
    return ir.reads(stmt.value)


# ---------------------------------------------------------------- simplify
def _same(a: ir.Expr, b: ir.Expr) -> bool:
    """Structural equality over the very same atoms."""
    m: dict = {}
    if not _struct_eq(a, b, m):
        return False
    return True


def _terms(e: ir.Expr, sign: int, out: list) -> None:
    if isinstance(e, ir.Bin) and e.op in ("add", "sub"):
        _terms(e.a, sign, out)
        _terms(e.b, sign if e.op == "add" else -sign, out)
    else:
        out.append((sign, e))


def _cancel(e: ir.Expr) -> ir.Expr:
    """A sum / difference tree with the terms that occur with both signs removed."""
    ts: list = []
    _terms(e, 1, ts)
    live = [True] * len(ts)
    for i, (si, ti) in enumerate(ts):
        if not live[i]:
            continue
        for j in range(i + 1, len(ts)):
            if live[j] and ts[j][0] == -si and _same(ti, ts[j][1]) and _identity_atoms(ti, ts[j][1]):
                live[i] = live[j] = False
                break
    rest = [(sg, t) for (sg, t), ok in zip(ts, live) if ok]
    if len(rest) == len(ts):
        return e
    if not rest:
        return ir.Const(0.0)
    pos = [t for sg, t in rest if sg > 0]
    neg = [t for sg, t in rest if sg < 0]
    acc = pos[0] if pos else ir.Un("neg", neg.pop(0))
    for t in pos[1:]:
        acc = ir.Bin("add", acc, t)
    for t in neg:
        acc = ir.Bin("sub", acc, t)
    return acc


def _identity_atoms(a: ir.Expr, b: ir.Expr) -> bool:
    m: dict = {}
    _struct_eq(a, b, m)
    return all(k == v.id for k, v in m.items())


def simplify(nests: list[Nest]) -> list[Nest]:
    """Algebra that makes the graph's own online-softmax hints disappear (reference
    compiler/passes/cleanup_passes.py + factor_acc.py:140-211 do this with sympy):
    exp(a) * exp(b) -> exp(a + b) (same for exp2), sums with a term and its negative cancelled,
    x * 1, x / 1, x + 0.  The running maximum of ``scan_max`` has no nest of its own: it has to
    cancel, as in exp2(x - run) * exp2(run - max)."""
    def step(x):
        if isinstance(x, ir.Bin) and x.op == "mul":
            a, b = ir.substitute(x.a, step), ir.substitute(x.b, step)
            if isinstance(a, ir.Un) and isinstance(b, ir.Un) and a.op == b.op and a.op in ("exp", "exp2"):
                return ir.Un(a.op, _cancel(ir.Bin("add", a.a, b.a)))
            for u, w in ((a, b), (b, a)):
                if isinstance(w, ir.Const) and w.value == 1.0:
                    return u
            return ir.Bin("mul", a, b)
        if isinstance(x, ir.Bin) and x.op == "div":
            a, b = ir.substitute(x.a, step), ir.substitute(x.b, step)
            if isinstance(b, ir.Const) and b.value == 1.0:
                return a
            return ir.Bin("div", a, b)
        return None

    for n in nests:
        if isinstance(n.stmt, (ir.Assign, ir.Accum)):
            n.stmt.value = ir.substitute(n.stmt.value, step)
    for n in nests:
        for r in _stmt_reads(n.stmt):
            if r.buf.kind == "scan":
                raise PassError("a running maximum (scan_max) is used outside a cancelling online-softmax hint")
    return nests


# ---------------------------------------------------------------- online softmax
def _same_atoms(a: Sequence[Atom], b: Sequence[Atom]) -> bool:
    la, lb = [x for x in ir.leaves(a) if x.hint != 1], [x for x in ir.leaves(b) if x.hint != 1]
    return len(la) == len(lb) and all(x is y for x, y in zip(la, lb))


def _struct_eq(a: ir.Expr, b: ir.Expr, m: dict) -> bool:
    """Structural equality of two expressions up to the atom renaming ``m`` (ids of a's atoms ->
    atoms of b), which is extended on the way."""
    if type(a) is not type(b):
        return False
    def atoms_eq(x, y):
        lx, ly = [t for t in ir.leaves(x) if t.hint != 1], [t for t in ir.leaves(y) if t.hint != 1]
        if len(lx) != len(ly):
            return False
        for s, t in zip(lx, ly):
            if m.setdefault(s.id, t) is not t:
                return False
        return True
    if isinstance(a, ir.Const):
        return a.value == b.value
    if isinstance(a, ir.Scalar):
        return a.text == b.text
    if isinstance(a, ir.Read):
        if a.buf is not b.buf or (a.gather is None) != (b.gather is None):
            return False
        if a.gather is not None and (a.gather[0] != b.gather[0] or a.gather[1] is not b.gather[1] or
                                     not all(atoms_eq(x, y) for x, y in zip(a.gather[2], b.gather[2]))):
            return False
        return all(atoms_eq(x, y) for x, y in zip(a.idx, b.idx))
    if isinstance(a, ir.Bin):
        return a.op == b.op and _struct_eq(a.a, b.a, m) and _struct_eq(a.b, b.b, m)
    if isinstance(a, ir.Un):
        return a.op == b.op and _struct_eq(a.a, b.a, m)
    if isinstance(a, ir.Dot):
        return atoms_eq(a.over, b.over) and _struct_eq(a.a, b.a, m) and _struct_eq(a.b, b.b, m)
    if isinstance(a, ir.Select):
        return (a.other == b.other and len(a.clauses) == len(b.clauses) and
                all((c.ci, c.cj, c.c0) == (d.ci, d.cj, d.c0) and atoms_eq(c.row, d.row) and atoms_eq(c.col, d.col)
                    for c, d in zip(a.clauses, b.clauses)) and _struct_eq(a.a, b.a, m))
    return False


def online_softmax(nests: list[Nest], keep: ir.Buffer) -> list[Nest]:
    """After ``fuse`` an attention graph is three nests over the same rows:

        m[r]    = max_j  x[r, j]                                        (Accum max)
        l[r]    = sum_j  e(x[r, j] - m[r])                              (Accum add; e = exp or exp2)
        o[r, d] = dot_j( e(x[r, j] - m[r]) / (l[r] + c),  v[j, d] ) + b[r, d]

    (c and b optional).  The divisor does not depend on j, so it moves out of the contraction, and
    so does b; what remains of the second and third nest are sums over j of terms that carry the
    same factor e(-m[r]).  With a running maximum in place of m, growing it from m_old to m_new
    multiplies every term already summed by e(m_old - m_new) -- a factor free of j -- so one pass
    that rescales both accumulators whenever the maximum grows computes the same values (the
    "online hoist" of the reference, factor_acc.py:23-109, 140-211).  x is whatever the graph makes
    of its score products -- scales, a cap, added tensors, a second product, masks -- and is carried
    over as it is.  The pass checks that the nests have this form, with the same x, and replaces
    them by one ``Rescaled`` nest."""
    out_nest = next((n for n in nests if n.writes() is keep), None)
    if out_nest is None or not isinstance(out_nest.stmt, ir.Assign):
        raise PassError("the result is not written by an element-wise nest")
    val, epilogue = out_nest.stmt.value, None
    if isinstance(val, ir.Bin) and val.op == "add":
        # result = contraction + tensor: the tensor is added once per element after the normalisation
        for d, t in ((val.a, val.b), (val.b, val.a)):
            if isinstance(d, ir.Dot) and isinstance(t, ir.Read):
                val, epilogue = d, t
                break
    if not isinstance(val, ir.Dot):
        raise PassError("the result is not a contraction")
    dot = val
    p, v = dot.a, dot.b
    # p = e(x - m[r]) / (l[r] + c...)
    if not (isinstance(p, ir.Bin) and p.op == "div"):
        raise PassError("left operand of the contraction is not a normalised value")
    e, den = p.a, p.b
    den_terms: list = []
    _terms(den, 1, den_terms)
    l_reads = [t for sg, t in den_terms if isinstance(t, ir.Read)]
    extra = [t for sg, t in den_terms if not isinstance(t, ir.Read)]
    if len(l_reads) != 1 or any(sg < 0 for sg, _ in den_terms) or not all(isinstance(t, (ir.Const, ir.Scalar)) for t in extra):
        raise PassError("the normaliser is not the row sum plus constants")
    l_read = l_reads[0]
    if not (isinstance(e, ir.Un) and e.op in ("exp", "exp2") and isinstance(e.a, ir.Bin) and e.a.op == "sub"
            and isinstance(e.a.b, ir.Read)):
        raise PassError("numerator is not exp(x - m)")
    x, m_read = e.a.a, e.a.b
    if not isinstance(v, ir.Read):
        raise PassError("right operand of the contraction is not a tensor read")
    l_nest = next((n for n in nests if n.writes() is l_read.buf), None)
    m_nest = next((n for n in nests if n.writes() is m_read.buf), None)
    if l_nest is None or m_nest is None or not isinstance(l_nest.stmt, ir.Accum) or not isinstance(m_nest.stmt, ir.Accum):
        raise PassError("row statistics are not reductions")
    if l_nest.stmt.op != "add" or m_nest.stmt.op != "max":
        raise PassError("row statistics are not a sum and a maximum")
    # l's summand is the numerator, m's operand is x -- over the contraction's own atoms
    ren: dict = {}
    if not _struct_eq(l_nest.stmt.value, e, ren) or not _struct_eq(m_nest.stmt.value, x, ren):
        raise PassError("sum / maximum are not taken of the contraction's own scores")
    for a, b in ((l_nest.red, dot.over), (m_nest.red, dot.over)):
        la = [ren.get(t.id, t) for t in ir.leaves(a) if t.hint != 1]
        if not _same_atoms(la, dot.over):
            raise PassError("reductions run over different key ranges")
    # x may not depend on the statistics themselves
    if any(r.buf in (l_read.buf, m_read.buf) for r in ir.reads(x)):
        raise PassError("scores depend on their own statistics")
    if epilogue is not None and any(r.buf in (l_read.buf, m_read.buf) for r in [epilogue]):
        raise PassError("the added tensor is a row statistic")
    new = Nest(out_nest.name, out_nest.par, list(dot.over),
               ir.Rescaled(keep, x, v, base2=(e.op == "exp2"), denom_add=tuple(extra), epilogue=epilogue))
    return [n for n in nests if n not in (out_nest, l_nest, m_nest)] + [new]


# ---------------------------------------------------------------- block skip
@dataclasses.dataclass
class TileBounds:
    """[start, end) of kv tiles for q tile ``qt``: callables over (qt, Sq, Sk) and their text."""

    start: Callable
    end: Callable
    text: str

    def range(self, qt: int, Sq: int, Sk: int, args=None) -> tuple[int, int]:
        """``args``: the call's flat arguments, for clauses whose constant is a run-time integer of
        the graph (a window passed as a variable); without them the traced value is used."""
        b, e = self.start(qt, Sq, Sk, args), self.end(qt, Sq, Sk, args)
        return b, max(b, e)


def _floordiv(a: int, b: int) -> int:
    return a // b


def block_skip(nests: list[Nest], bm: int, bn: int) -> list[Nest]:
    """Tighten the kv-tile loop of the ``Rescaled`` nest.  A kv tile whose every score is masked
    leaves the running maximum, the sum and the accumulator unchanged (the masked value is
    -inf: exp gives 0, max ignores it), so it can be left out (reference
    skip_loop_iterations.py:318-341).  Whether a clause ci*i + cj*j + c0 <= 0 can hold anywhere
    in the box i in [i_lo, i_hi], j in [j_lo, j_hi] follows from its minimum over the box
    (interval arithmetic, reference :26-81); solved for the kv tile index this bounds the loop
    from above (cj > 0) or from below (cj < 0) (reference :343-376).  Clauses over the same
    difference i - j, which is all the two mask ops produce, make the conjunction exact."""
    nest = next((n for n in nests if isinstance(n.stmt, ir.Rescaled)), None)
    if nest is None:
        raise PassError("no online-softmax nest to tile")
    clauses: list[ir.Clause] = []
    for x in ir.walk(nest.stmt.score):
        if isinstance(x, ir.Select):
            if x.other != float("-inf"):
                raise PassError("masked value is not -inf: skipping would change the result")
            clauses.extend(x.clauses)
    uppers, lowers, texts = [], [], []
    for c in clauses:
        if c.cj == 0:
            continue                                     # does not bound the key loop
        # the row extreme that makes the clause easiest to satisfy
        def i_ext(qt, Sq, c=c):
            lo, hi = qt * bm, min(qt * bm + bm, Sq) - 1
            return lo if c.ci > 0 else hi
        if c.cj > 0:
            # min over the box = ci*i_ext + cj*j_lo + c0 <= 0  <=>  kt*bn <= (-c0 - ci*i_ext) / cj
            uppers.append(lambda qt, Sq, Sk, args, c=c, f=i_ext: _floordiv(_floordiv(-c.const(args) - c.ci * f(qt, Sq), c.cj), bn) + 1)
            texts.append(f"kt*{bn} <= ({-c.c0} - {c.ci}*i_{'lo' if c.ci > 0 else 'hi'}) // {c.cj}")
        else:
            # min = ci*i_ext + cj*j_hi + c0 <= 0  <=>  j_hi >= ceil((ci*i_ext + c0) / -cj) =: L, j_hi = min(kt*bn + bn, Sk) - 1
            def lower(qt, Sq, Sk, args, c=c, f=i_ext):
                L = -_floordiv(-(c.ci * f(qt, Sq) + c.const(args)), -c.cj)
                if L > Sk - 1:
                    return 1 << 30                        # no key satisfies it: empty range
                return max(0, _floordiv(L, bn)) if L > 0 else 0
            lowers.append(lower)
            texts.append(f"min(kt*{bn}+{bn}, Sk)-1 >= ceil(({c.ci}*i_{'lo' if c.ci > 0 else 'hi'} + {c.c0}) / {-c.cj})")

    def start(qt, Sq, Sk, args=None):
        return max([0] + [f(qt, Sq, Sk, args) for f in lowers])

    def end(qt, Sq, Sk, args=None):
        nkt = -(-Sk // bn)
        if min(qt * bm + bm, Sq) - 1 < qt * bm:
            return 0
        return min([nkt] + [f(qt, Sq, Sk, args) for f in uppers])

    nest.stmt.tile = (bm, bn, TileBounds(start, end, " and ".join(texts) or "all"))
    return nests
