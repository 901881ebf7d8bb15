"""Loop IR of the front end.

Tensors are indexed through *atoms*.  An atom is one radix of a mixed-radix index: a
dimension of size ``B*H`` that came from merging ``[B, H]`` is the atom list ``[B, H]``, a
dimension ``Hq`` that a later reshape splits into ``[Hkv, g]`` becomes two child atoms.
Every loop of a nest runs over one (leaf) atom, and the index a buffer dimension is read
at is the mixed-radix composition of that dimension's atoms -- so views (transpose, expand,
reshape, repeat_interleave) never leave div/mod arithmetic behind: they only regroup atoms
(the reference folds views into pointer arithmetic per load instead,
``loopfuse/torch_backend/ops.py:131-341``).

Statements of a nest are in static single assignment over *buffers*: ``Assign`` writes a
buffer element once, ``Accum`` folds a value into it with an associative op over the nest's
reduction atoms.  Expressions are pointwise over buffer reads.
"""
from __future__ import annotations

import dataclasses
import itertools
from typing import Callable, Optional, Sequence

_ids = itertools.count()


class Atom:
    """One radix of an index.  ``size`` is symbolic (a string such as ``"s37"`` or ``"s25//s85"``),
    ``hint`` its value for the traced example.  ``children`` is set when a reshape splits it."""

    def __init__(self, size: str, hint: int, name: str = ""):
        self.size, self.hint = str(size), int(hint)
        self.id = next(_ids)
        self.name = name or f"a{self.id}"
        self.children: Optional[list["Atom"]] = None
        self.broadcast = False          # an expanded size-1 dimension: reads ignore its index
        self.alias: Optional["Atom"] = None   # set when unified with another atom: that one stands for both

    def rep(self) -> "Atom":
        a = self
        while a.alias is not None:
            a = a.alias
        return a

    def leaves(self) -> list["Atom"]:
        a = self.rep()
        if a.children is None:
            return [a]
        return [l for c in a.children for l in c.leaves()]

    def split(self, outer_hint: int, outer_size: str, inner_size: str) -> None:
        """Replace this atom by [outer, inner] (index = outer * inner.size + inner)."""
        assert self.alias is None and self.children is None and self.hint % outer_hint == 0
        a, b = Atom(outer_size, outer_hint, self.name + "o"), Atom(inner_size, self.hint // outer_hint, self.name + "i")
        a.broadcast = b.broadcast = self.broadcast
        self.children = [a, b]

    def __repr__(self) -> str:
        return f"{self.name}[{self.size}]"


def leaves(atoms: Sequence[Atom]) -> list[Atom]:
    return [l for a in atoms for l in a.leaves()]


def unify(xs: Sequence[Atom], ys: Sequence[Atom]) -> None:
    """Make two atom lists that index the same range the same atoms: equal radices are merged,
    a larger radix is split to fit the other side (``Hq`` against ``[Hkv, g]``).  Size-1 atoms
    index nothing and are skipped."""
    xs = [a for a in leaves(xs) if a.hint != 1]
    ys = [a for a in leaves(ys) if a.hint != 1]
    while xs and ys:
        x, y = xs[0], ys[0]
        if x is y:
            xs.pop(0), ys.pop(0)
        elif x.hint == y.hint:
            if x.broadcast and not y.broadcast:
                x.alias = y
            else:
                y.alias = x
            xs.pop(0), ys.pop(0)
        elif x.hint > y.hint and x.hint % y.hint == 0:
            x.split(y.hint, y.size, f"({x.size})//({y.size})")
            xs[0:1] = x.children
        elif y.hint > x.hint and y.hint % x.hint == 0:
            y.split(x.hint, x.size, f"({y.size})//({x.size})")
            ys[0:1] = y.children
        else:
            raise ValueError(f"index ranges do not line up: {x} vs {y}")
    if xs or ys:
        raise ValueError(f"index ranges of different extent: left over {xs or ys}")


@dataclasses.dataclass(eq=False)
class Buffer:
    """A tensor in memory.  ``dims`` lists, per dimension, its atoms from outer to inner.
    kind: "input" (graph placeholder), "temp" (intermediate), "output"."""

    name: str
    dims: list[list[Atom]]
    kind: str = "temp"
    dtype: str = "f32"
    placeholder: int = -1            # index among the graph's placeholders (inputs)
    node: object = None              # temporaries: the graph node whose value this is
    scan_of: Optional["Buffer"] = None   # kind "scan": the running form of this reduction's result (scan_max)

    def __repr__(self) -> str:
        return self.name


# ---------------------------------------------------------------- expressions (pointwise values)
class Expr:
    def children(self) -> tuple:
        return ()


@dataclasses.dataclass(eq=False)
class Const(Expr):
    value: float


@dataclasses.dataclass(eq=False)
class Scalar(Expr):
    """A 0-dim value the graph computes from sizes (``D ** -0.5``): a callable over the size
    environment, evaluated per call."""

    fn: Callable[[dict], float]
    text: str


@dataclasses.dataclass(eq=False)
class Read(Expr):
    """``buf[idx]``: per buffer dimension the atoms whose composition is the index.  A dimension
    indexed through a table (page gather) carries ``gather`` = (table buffer, its atom lists)."""

    buf: Buffer
    idx: list[list[Atom]]
    gather: Optional[tuple] = None   # (dim, table Buffer, table idx) : buf dim `dim` is table[idx]


@dataclasses.dataclass(eq=False)
class Bin(Expr):
    op: str                          # add sub mul div max
    a: Expr
    b: Expr

    def children(self):
        return (self.a, self.b)


@dataclasses.dataclass(eq=False)
class Un(Expr):
    op: str                          # exp exp2 tanh neg recip relu sigmoid silu gelu gelu_tanh sqrt rsqrt abs
    a: Expr

    def children(self):
        return (self.a,)


@dataclasses.dataclass(eq=False)
class Clause:
    """ci * i + cj * j + c0 <= 0 over a row index i and a column index j, each the composition
    of an atom list.  Masks are conjunctions of clauses (reference ops.py:696, 733-741)."""

    ci: int
    cj: int
    c0: int                          # at the traced sizes
    row: list[Atom]
    col: list[Atom]
    c0_fn: Optional[Callable] = None  # set when the constant is a run-time integer of the graph: args -> int

    def const(self, args=None) -> int:
        return int(self.c0_fn(args)) if (self.c0_fn is not None and args is not None) else self.c0


@dataclasses.dataclass(eq=False)
class Select(Expr):
    """value where every clause holds, else ``other`` (-inf for the masks)."""

    clauses: list[Clause]
    a: Expr
    other: float

    def children(self):
        return (self.a,)


# ---------------------------------------------------------------- statements and nests
@dataclasses.dataclass(eq=False)
class Assign:
    buf: Buffer
    value: Expr


@dataclasses.dataclass(eq=False)
class Accum:
    buf: Buffer
    op: str                          # add | max
    value: Expr
    init: float = 0.0


@dataclasses.dataclass(eq=False)
class Rescaled:
    """What the online-softmax pass leaves behind: a single pass over ``red`` that keeps a
    running maximum of ``score`` and, rescaled by 2^(m_old - m_new) whenever it grows, the sum
    of exponentials and the accumulation ``weights``; ``out = acc / sum`` after the loop
    (reference factor_acc.py:23-109, README.md:85-99)."""

    out: Buffer
    score: Expr                      # per (row, key) value whose softmax is taken
    weights: Read                    # per (key, d) operand of the second product
    tile: Optional[tuple] = None     # (BM, BN, bounds): set by the block-skip pass
    base2: bool = False              # the graph's exponentials are 2^x: the score is in log2 units
    denom_add: tuple = ()            # out = acc / (sum + these): Const / Scalar terms, in units where the
                                     # row maximum contributes 1 (reference tests/test_attention.py:95-125)
    epilogue: Optional[Read] = None  # added to acc / sum element by element (an output bias)


@dataclasses.dataclass(eq=False)
class Nest:
    """``for par... : for red... : stmt`` -- one statement per nest (the reference appends one
    loop nest per op too, interface.py:288-311)."""

    name: str
    par: list[Atom]                  # parallel atoms (the written buffer's index atoms)
    red: list[Atom]                  # reduction atoms
    stmt: object

    def writes(self) -> Buffer:
        return self.stmt.out if isinstance(self.stmt, Rescaled) else self.stmt.buf


def walk(e: Expr):
    yield e
    for c in e.children():
        yield from walk(c)


def reads(e: Expr) -> list[Read]:
    return [x for x in walk(e) if isinstance(x, Read)]


def substitute(e: Expr, fn: Callable[[Expr], Optional[Expr]]) -> Expr:
    """Rebuild ``e`` bottom-up; ``fn(node)`` may return a replacement."""
    r = fn(e)
    if r is not None:
        return r
    if isinstance(e, Bin):
        return Bin(e.op, substitute(e.a, fn), substitute(e.b, fn))
    if isinstance(e, Un):
        return Un(e.op, substitute(e.a, fn))
    if isinstance(e, Select):
        return Select(e.clauses, substitute(e.a, fn), e.other)
    if type(e).__name__ == "Dot":
        return type(e)(substitute(e.a, fn), substitute(e.b, fn), e.over)
    return e


# ---------------------------------------------------------------- printing (DEBUG=1)
def _ix(atoms: Sequence[Atom]) -> str:
    ls = leaves(atoms)
    return "·".join(a.name for a in ls if not a.broadcast) or "0"


def show_expr(e: Expr) -> str:
    if isinstance(e, Const):
        return f"{e.value:g}"
    if isinstance(e, Scalar):
        return f"<{e.text}>"
    if isinstance(e, Read):
        parts = []
        for d, ix in enumerate(e.idx):
            if e.gather is not None and e.gather[0] == d:
                parts.append(f"{e.gather[1].name}[{', '.join(_ix(t) for t in e.gather[2])}]")
            else:
                parts.append(_ix(ix))
        return f"{e.buf.name}[{', '.join(parts)}]"
    if isinstance(e, Bin):
        sym = {"add": "+", "sub": "-", "mul": "*", "div": "/"}.get(e.op)
        return f"({show_expr(e.a)} {sym} {show_expr(e.b)})" if sym else f"{e.op}({show_expr(e.a)}, {show_expr(e.b)})"
    if isinstance(e, Un):
        return f"{e.op}({show_expr(e.a)})"
    if type(e).__name__ == "Dot":
        return f"dot[{_ix(e.over)}]({show_expr(e.a)}, {show_expr(e.b)})"
    if isinstance(e, Select):
        cl = " and ".join(f"{c.ci}*{_ix(c.row)} + {c.cj}*{_ix(c.col)} + {c.c0} <= 0" for c in e.clauses)
        return f"where({cl}, {show_expr(e.a)}, {e.other})"
    return repr(e)


def show(nests: Sequence[Nest]) -> str:
    out = []
    for n in nests:
        out.append(f"# {n.name}")
        pad = ""
        for a in leaves(n.par):
            out.append(f"{pad}for {a.name} in range({a.size}):")
            pad += "  "
        for a in leaves(n.red):
            out.append(f"{pad}for {a.name} in range({a.size}):   # reduction")
            pad += "  "
        s = n.stmt
        if isinstance(s, Assign):
            out.append(f"{pad}{s.buf.name}[...] = {show_expr(s.value)}")
        elif isinstance(s, Accum):
            out.append(f"{pad}{s.buf.name}[...] = {s.op}({s.buf.name}[...], {show_expr(s.value)})   # init {s.init}")
        else:
            t = f"  tiles {s.tile[0]}x{s.tile[1]}, kv tiles [{s.tile[2].text}]" if s.tile else ""
            out.append(f"{pad}m, l, acc = online_softmax({show_expr(s.score)}) @ {show_expr(s.weights)}{t}")
            den = "l" if not s.denom_add else "(l + " + " + ".join(show_expr(t) for t in s.denom_add) + ")"
            epi = f" + {show_expr(s.epilogue)}" if s.epilogue is not None else ""
            out.append(f"{pad[:-2 * max(len(leaves(n.red)), 0)]}{s.out.name}[...] = acc / {den}{epi}"
                       + ("   # exponentials to base 2" if s.base2 else ""))
    return "\n".join(out)


@dataclasses.dataclass(eq=False)
class Dot(Expr):
    """sum over the atoms ``over`` of a * b -- the tile-level ``dot`` of the reference
    (ops.py:344-413): a contraction that pointwise consumers can be fused onto."""

    a: Expr
    b: Expr
    over: list[Atom]

    def children(self):
        return (self.a, self.b)
