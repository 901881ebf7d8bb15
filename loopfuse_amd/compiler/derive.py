"""Read the fused nest off into what the HIP lowering takes (the step where the reference
prints Triton source, ``loopfuse/codegen.py:100-126``).

After the passes an attention graph is ONE nest,

    for rows r:  m, l, acc = online_softmax_j( where(clauses, mods(dot_d(Q, K)), -inf) ) @ V ;  out = acc / l

and everything the kernels are parametrised by is visible in it:
  * mask kind and window   from the clauses (j - i <= 0 ; i - j - (w - 1) <= 0),
  * scale and softcap      from the multiplications / divisions / tanh between dot and where,
  * GQA                    from head atoms Q iterates and K does not,
  * paging                 from reads whose first buffer dimension is gathered through a table,
  * operand layouts        from which buffer dimension carries the row / key / depth atoms.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Callable, Optional

from . import ir
from .passes import TileBounds


class NotDerivable(Exception):
    """The fused nest is not an attention the kernels implement."""


@dataclasses.dataclass
class OperandLayout:
    placeholder: int                 # graph input holding the tensor (the pool when paged); -1: see node
    perm: tuple = ()                 # dense: permutation of the input's dims giving [B, H, S, D]
    paged: bool = False
    table: int = -1                  # graph input holding the page table
    group: int = 1                   # query heads per kv head at the traced sizes
    node: object = None              # an operand the graph computes from its inputs (Q + q_bias): the node


@dataclasses.dataclass
class BiasLayout:
    """An added tensor as a view [B, Hq, rows, X]: per logical dim the source dim that walks it (None = broadcast)."""

    placeholder: int
    dims: tuple
    node: object = None


@dataclasses.dataclass
class DerivedAttention:
    mask: Optional[str]
    window: object                   # int, or a callable over the call's arguments (a run-time integer of the graph)
    pre: list                        # factors applied to the raw scores (before tanh if there is one)
    post: list                       # factors applied after tanh
    has_tanh: bool
    q: OperandLayout
    k: OperandLayout
    v: OperandLayout
    bounds: Optional[TileBounds]
    tile: tuple                      # (BM, BN) the bounds were derived for
    bias: Optional[BiasLayout] = None        # added to the scaled (capped) scores before the mask
    out_bias: Optional[BiasLayout] = None    # added to the normalised result
    q2: Optional[OperandLayout] = None       # second score product: scores = Q K^T + Q2 K2^T
    k2: Optional[OperandLayout] = None
    denom_add: tuple = ()                    # ("mul", value | callable) terms added to the softmax denominator
    base2: bool = False                      # exponentials to base 2
    late: list = dataclasses.field(default_factory=list)   # the factors of `pre` that the graph applies behind the mask

    def number(self, f, args) -> float:
        kind, x = f
        v = x(args) if callable(x) else float(x)
        return 1.0 / v if kind == "div" else v

    def scale_and_cap(self, args) -> tuple:
        pre = math.prod(self.number(f, args) for f in self.pre)
        if not self.has_tanh:
            return pre, None
        cap = math.prod(self.number(f, args) for f in self.post)
        return pre * cap, cap

    def describe(self) -> str:
        win = "<run-time>" if callable(self.window) else self.window
        return (f"mask={self.mask} window={win} tanh={self.has_tanh} pre={[f[0] for f in self.pre]} "
                f"post={[f[0] for f in self.post]} Q=in{self.q.placeholder}{self.q.perm} "
                f"K=in{self.k.placeholder}{'[paged by in%d]' % self.k.table if self.k.paged else self.k.perm} "
                f"V=in{self.v.placeholder}{'[paged by in%d]' % self.v.table if self.v.paged else self.v.perm} "
                f"group={self.k.group} kv tiles: {self.bounds.text if self.bounds else 'all'}"
                + (" +score_bias" if self.bias else "") + (" +out_bias" if self.out_bias else "")
                + (" +second product" if self.q2 else "") + (f" denom+{len(self.denom_add)}" if self.denom_add else "")
                + (" exp2" if self.base2 else ""))


def _ids(atoms) -> set:
    return {a.id for a in ir.leaves(atoms) if a.hint != 1}


def _has_dot(e: ir.Expr) -> bool:
    return any(isinstance(x, ir.Dot) for x in ir.walk(e))


def _peel(e: ir.Expr):
    """mods(core) -> (list of ("mul" | "div" | "tanh", value), core), outermost first; core is a Dot or the
    sum of two Dots (two-part scores)."""
    ops = []
    while not isinstance(e, ir.Dot):
        if isinstance(e, ir.Un) and e.op == "tanh":
            ops.append(("tanh", None))
            e = e.a
        elif isinstance(e, ir.Bin) and e.op in ("mul", "div") and isinstance(e.b, (ir.Const, ir.Scalar)):
            ops.append((e.op, e.b.value if isinstance(e.b, ir.Const) else e.b.fn))
            e = e.a
        elif isinstance(e, ir.Bin) and e.op == "mul" and isinstance(e.a, (ir.Const, ir.Scalar)):
            ops.append(("mul", e.a.value if isinstance(e.a, ir.Const) else e.a.fn))
            e = e.b
        elif isinstance(e, ir.Bin) and e.op == "add" and isinstance(e.a, ir.Dot) and isinstance(e.b, ir.Dot):
            break
        else:
            raise NotDerivable(f"score modification {type(e).__name__} is not a scale / softcap chain")
    return ops, e


def _dense_perm(read: ir.Read, roles: dict, what: str) -> tuple:
    """Permutation of the buffer's dims that gives [batch..., seq, depth] = [B, H, S, D]."""
    seq = [d for d, r in roles.items() if r == "seq"]
    if not seq:
        # a sequence of length 1 (decode) indexes nothing: it is the last size-1 dimension
        ones = [d for d, r in roles.items() if r == "one"]
        if ones:
            roles = {**roles, ones[-1]: "seq"}
            seq = [ones[-1]]
    batch = [d for d, r in roles.items() if r in ("batch", "one")]
    dep = [d for d, r in roles.items() if r == "depth"]
    if len(seq) != 1 or len(dep) != 1 or len(batch) != 2:
        raise NotDerivable(f"{what} is not a [B, H, S, D] tensor up to a permutation (roles {roles})")
    return tuple(sorted(batch)) + (seq[0], dep[0])


def attention(nests: list, inputs: list, out_view) -> DerivedAttention:
    from .passes import is_operand_prep

    main = [n for n in nests if isinstance(n.stmt, ir.Rescaled)]
    rest = [n for n in nests if not isinstance(n.stmt, ir.Rescaled)]
    if len(main) != 1 or not all(is_operand_prep(n) for n in rest):
        raise NotDerivable(f"{len(nests)} nests left after fusion: not a single attention")
    nest = main[0]
    st = nest.stmt
    # ---- factors the graph applies to the masked scores (x * c commutes with the mask for c > 0, which
    # the call checks: -inf must stay -inf)
    score = st.score
    late = []
    while isinstance(score, ir.Bin) and score.op in ("mul", "div") and isinstance(score.b, (ir.Const, ir.Scalar)) \
            and any(isinstance(x, ir.Select) for x in ir.walk(score.a)):
        late.append((score.op, score.b.value if isinstance(score.b, ir.Const) else score.b.fn))
        score = score.a
    # ---- mask
    clauses = []
    if isinstance(score, ir.Select):
        if score.other != float("-inf"):
            raise NotDerivable("masked scores are not -inf")
        clauses, score = score.clauses, score.a
    # ---- an added tensor (score bias): outermost, on top of the scale / softcap chain
    bias_read = None
    if isinstance(score, ir.Bin) and score.op == "add":
        for x, t in ((score.a, score.b), (score.b, score.a)):
            if isinstance(t, ir.Read) and _has_dot(x) and not isinstance(x, ir.Dot):
                score, bias_read = x, t
                break
            if isinstance(t, ir.Read) and isinstance(x, ir.Dot):
                score, bias_read = x, t
                break
    ops, core = _peel(score)
    if any(isinstance(x, ir.Select) for x in ir.walk(core)):
        raise NotDerivable("mask below the score product")
    dot, dot2 = core, None
    if not isinstance(core, ir.Dot):
        # two-part scores: the product with the deeper contraction is the main one
        d_a = math.prod(a.hint for a in ir.leaves(core.a.over))
        d_b = math.prod(a.hint for a in ir.leaves(core.b.over))
        dot, dot2 = (core.a, core.b) if d_a >= d_b else (core.b, core.a)
    for d in (dot, dot2):
        if d is not None and (not isinstance(d.a, ir.Read) or not isinstance(d.b, ir.Read)):
            raise NotDerivable("score product of something else than two tensors")
    qr, kr, vr = dot.a, dot.b, st.weights
    keys, depth = _ids(nest.red), _ids(dot.over)

    def all_ids(r: ir.Read) -> set:
        out = set().union(*[_ids(d) for d in r.idx]) if r.idx else set()
        if r.gather:
            out |= set().union(*[_ids(t) for t in r.gather[2]])
        return out

    if _ids([a for d in qr.idx for a in d]) & keys:
        qr, kr = kr, qr                               # bmm(K, Q^T) spelling
    k_all = all_ids(kr)

    def source(r: ir.Read, what: str):
        """(placeholder, node) of an operand: a graph input, or the node of an element-wise nest over inputs."""
        if r.buf.kind == "input":
            return r.buf.placeholder, None
        if r.buf.node is not None and any(n.writes() is r.buf for n in rest):
            return -1, r.buf.node
        raise NotDerivable(f"{what} {r.buf.name} is computed inside the graph")

    # the rows are what the result's second-to-last dim runs over (a key tensor shared by all heads leaves
    # the head atoms out of K as well, so "not in K" alone does not tell rows from heads)
    rows_out = _ids(out_view.dims[-2]) if len(out_view.dims) >= 2 else set()

    def q_layout(r: ir.Read, dep_ids: set, k_ids: set, what: str):
        roles, group, rows = {}, 1, set()
        for d, atoms in enumerate(r.idx):
            ids = _ids(atoms)
            if not ids:
                roles[d] = "one"                      # a size-1 dimension
            elif ids <= dep_ids:
                roles[d] = "depth"
            elif ids <= rows_out if rows_out else not (ids & k_ids):
                roles[d] = "seq"
                rows = ids
            else:
                roles[d] = "batch"
                group *= math.prod(a.hint for a in ir.leaves(atoms) if a.hint != 1 and a.id not in k_ids)
        if r.gather is not None:
            raise NotDerivable("paged queries")
        ph, node = source(r, what)
        return OperandLayout(ph, _dense_perm(r, roles, what), node=node), group, rows

    q, group, rows = q_layout(qr, depth, k_all, "Q")

    def kv_layout(r: ir.Read, dep_ids: set, what: str, grp: int) -> OperandLayout:
        roles = {}
        for d, atoms in enumerate(r.idx):
            ids = _ids(atoms)
            if r.gather is not None and r.gather[0] == d:
                roles[d] = "page"
            elif not ids:
                roles[d] = "one"
            elif ids and ids <= dep_ids:
                roles[d] = "depth"
            elif ids and ids <= keys:
                roles[d] = "seq"
            else:
                roles[d] = "batch"
        ph, node = source(r, what)
        if r.gather is None:
            return OperandLayout(ph, _dense_perm(r, roles, what), group=grp, node=node)
        # pool [N, (P,) Hkv, D] gathered through table [B, pages]
        order = [{"one": "batch"}.get(roles[d], roles[d]) for d in range(len(r.idx))]
        if order not in (["page", "seq", "batch", "depth"], ["page", "batch", "depth"]):
            raise NotDerivable(f"{what} pool is not [pages, page size, heads, depth] (roles {order})")
        tbuf, tidx = r.gather[1], r.gather[2]
        if len(tidx) != 2 or not (_ids(tidx[1]) <= keys) or (_ids(tidx[0]) & keys) or tbuf.kind != "input":
            raise NotDerivable(f"{what} page table is not [batch, pages]")
        return OperandLayout(ph, (), True, tbuf.placeholder, grp)

    k = kv_layout(kr, depth, "K", group)
    out_depth = _ids(out_view.dims[-1])
    v = kv_layout(vr, out_depth, "V", group)
    # ---- second score product
    q2 = k2 = None
    if dot2 is not None:
        q2r, k2r = dot2.a, dot2.b
        if _ids([a for d in q2r.idx for a in d]) & keys:
            q2r, k2r = k2r, q2r
        depth2 = _ids(dot2.over)
        q2, group2, rows2 = q_layout(q2r, depth2, all_ids(k2r), "Q2")
        if rows2 != rows or q2r.gather is not None or k2r.gather is not None:
            raise NotDerivable("the second score product runs over other rows, or is paged")
        k2 = kv_layout(k2r, depth2, "K2", group2)      # a positional key may be shared by more heads than K is
    # ---- output: [batch..., rows, depth] in the order the kernel writes
    if len(out_view.dims) != 4 or (rows and _ids(out_view.dims[2]) != rows) or (_ids(out_view.dims[0]) | _ids(out_view.dims[1])) & (rows | out_depth):
        raise NotDerivable("result is not laid out [B, H, rows, depth]")

    def added(r: Optional[ir.Read], last: set, what: str) -> Optional[BiasLayout]:
        """An added tensor as [B, Hq, rows, last]: which of its dims walks which of the four."""
        if r is None:
            return None
        if r.gather is not None:
            raise NotDerivable(f"{what} is gathered")
        ph, node = source(r, what)
        qb, qh = _ids(qr.idx[q.perm[0]]), _ids(qr.idx[q.perm[1]])
        dims = [None, None, None, None]
        for d, atoms in enumerate(r.idx):
            ids = {a.id for a in ir.leaves(atoms) if a.hint != 1 and not a.broadcast}
            if not ids:
                continue                              # size 1 or expanded: broadcast
            want = [(0, qb), (1, qh), (2, rows), (3, last)]
            slot = next((i for i, full in want if full and ids == full), None)
            if slot is None or dims[slot] is not None:
                raise NotDerivable(f"{what} does not broadcast over [batch, heads, rows, {'keys' if last is keys else 'depth'}]")
            dims[slot] = d
        return BiasLayout(ph, tuple(dims), node)

    bias = added(bias_read, keys, "score bias")
    out_bias = added(st.epilogue, out_depth, "output bias")
    # ---- clauses -> mask kind
    mask, window = None, 0
    for c in clauses:
        if _ids(c.row) != rows or _ids(c.col) != keys:
            raise NotDerivable("mask compares something else than query row and key position")
    by_shape = sorted(clauses, key=lambda c: (c.ci, c.cj, c.c0))
    shapes = [(c.ci, c.cj, c.c0) for c in by_shape]
    if shapes == [(-1, 1, 0)] and by_shape[0].c0_fn is None:
        mask = "causal"
    elif len(shapes) == 2 and shapes[0] == (-1, 1, 0) and shapes[1][:2] == (1, -1) and shapes[1][2] <= 0 \
            and by_shape[0].c0_fn is None:
        w = by_shape[1]
        mask, window = "sliding", (1 - w.c0 if w.c0_fn is None else (lambda args, f=w.c0_fn: 1 - f(args)))
    elif shapes:
        raise NotDerivable(f"mask clauses {shapes} are neither causal nor a causal window")
    # ---- score modifications: [post..., tanh, pre...] read from the outside in
    kinds = [o[0] for o in ops]
    if kinds.count("tanh") > 1:
        raise NotDerivable("more than one tanh")
    has_tanh = "tanh" in kinds
    cut = kinds.index("tanh") if has_tanh else 0
    post, pre = (ops[:cut], ops[cut + 1:]) if has_tanh else ([], ops)
    if late and has_tanh:
        raise NotDerivable("factors behind the mask of capped scores")
    pre = list(pre) + late
    if st.base2 and has_tanh:
        raise NotDerivable("softcap inside an exp2-based softmax")
    denom = tuple(("mul", t.value if isinstance(t, ir.Const) else t.fn) for t in st.denom_add)
    bounds, tile = (st.tile[2], st.tile[:2]) if st.tile else (None, ())
    return DerivedAttention(mask, window, list(pre), list(post), has_tanh, q, k, v, bounds, tile,
                            bias=bias, out_bias=out_bias, q2=q2, k2=k2, denom_add=denom, base2=st.base2, late=late)
