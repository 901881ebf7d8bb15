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
    placeholder: int                 # graph input holding the tensor (the pool when paged)
    perm: tuple = ()                 # dense: permutation of the input's dims giving [B, H, S, D]
    paged: bool = False
    table: int = -1                  # graph input holding the page table
    group: int = 1                   # query heads per kv head at the traced sizes


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
                f"group={self.k.group} kv tiles: {self.bounds.text if self.bounds else 'all'}")


def _ids(atoms) -> set:
    return {a.id for a in ir.leaves(atoms) if a.hint != 1}


def _peel(e: ir.Expr):
    """mods(dot) -> (list of ("mul" | "div" | "tanh", value), the Dot), outermost first."""
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
    if len(nests) != 1 or not isinstance(nests[0].stmt, ir.Rescaled):
        raise NotDerivable(f"{len(nests)} nests left after fusion: not a single attention")
    nest = nests[0]
    st = nest.stmt
    # ---- mask
    score = st.score
    clauses = []
    if isinstance(score, ir.Select):
        if score.other != float("-inf"):
            raise NotDerivable("masked scores are not -inf")
        clauses, score = score.clauses, score.a
    ops, dot = _peel(score)
    if any(isinstance(x, ir.Select) for x in ir.walk(dot)):
        raise NotDerivable("mask below the score product")
    if not isinstance(dot.a, ir.Read) or not isinstance(dot.b, ir.Read):
        raise NotDerivable("score product of something else than two tensors")
    qr, kr, vr = dot.a, dot.b, st.weights
    keys, depth = _ids(nest.red), _ids(dot.over)
    k_all = set().union(*[_ids(d) for d in kr.idx]) | (set().union(*[_ids(t) for t in kr.gather[2]]) if kr.gather else set())
    if _ids([a for d in qr.idx for a in d]) & keys:
        qr, kr = kr, qr                               # bmm(K, Q^T) spelling
        k_all = set().union(*[_ids(d) for d in kr.idx])
    # ---- Q
    q_roles, group, rows = {}, 1, set()
    for d, atoms in enumerate(qr.idx):
        ids = _ids(atoms)
        if not ids:
            q_roles[d] = "one"                        # a size-1 dimension
        elif ids <= depth:
            q_roles[d] = "depth"
        elif not (ids & k_all):
            q_roles[d] = "seq"
            rows = ids
        else:
            q_roles[d] = "batch"
            group *= math.prod(a.hint for a in ir.leaves(atoms) if a.hint != 1 and a.id not in k_all)
    if qr.gather is not None:
        raise NotDerivable("paged queries")
    q = OperandLayout(qr.buf.placeholder, _dense_perm(qr, q_roles, "Q"))

    def kv_layout(r: ir.Read, dep_ids: set, what: str) -> OperandLayout:
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
        if r.gather is None:
            return OperandLayout(r.buf.placeholder, _dense_perm(r, roles, what), group=group)
        # pool [N, (P,) Hkv, D] gathered through table [B, pages]
        order = [{"one": "batch"}.get(roles[d], roles[d]) for d in range(len(r.idx))]
        if order not in (["page", "seq", "batch", "depth"], ["page", "batch", "depth"]):
            raise NotDerivable(f"{what} pool is not [pages, page size, heads, depth] (roles {order})")
        tbuf, tidx = r.gather[1], r.gather[2]
        if len(tidx) != 2 or not (_ids(tidx[1]) <= keys) or (_ids(tidx[0]) & keys):
            raise NotDerivable(f"{what} page table is not [batch, pages]")
        return OperandLayout(r.buf.placeholder, (), True, tbuf.placeholder, group)

    k = kv_layout(kr, depth, "K")
    out_depth = _ids(out_view.dims[-1])
    v = kv_layout(vr, out_depth, "V")
    for r in (qr, kr, vr):
        if r.buf.kind != "input":
            raise NotDerivable(f"operand {r.buf.name} is computed inside the graph")
    # ---- output: [batch..., rows, depth] in the order the kernel writes
    if len(out_view.dims) != 4 or (rows and _ids(out_view.dims[2]) != rows) or (_ids(out_view.dims[0]) | _ids(out_view.dims[1])) & (rows | out_depth):
        raise NotDerivable("result is not laid out [B, H, rows, depth]")
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
    bounds, tile = (st.tile[2], st.tile[:2]) if st.tile else (None, ())
    return DerivedAttention(mask, window, list(pre), list(post), has_tanh, q, k, v, bounds, tile)
