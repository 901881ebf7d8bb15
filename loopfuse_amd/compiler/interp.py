"""Reference interpreter of the loop IR: evaluates nests with dense torch tensors at the traced
(hint) sizes.  For tests and debugging -- it shows that a pass left the meaning of the nests
unchanged; nothing on the launch path uses it."""
from __future__ import annotations

import math
from typing import Sequence

import torch

from . import ir
from .ir import Atom


def _axes(atoms: Sequence[Atom]) -> list[Atom]:
    return [a for a in ir.leaves(atoms) if a.hint != 1]


def _to_axes(t: torch.Tensor, have: list[Atom], want: list[Atom]) -> torch.Tensor:
    """``t`` has one axis per atom of ``have``; permute / broadcast it to the axes ``want``."""
    pos = {a.id: i for i, a in enumerate(have)}
    if len(pos) != len(have):
        raise ValueError("an atom indexes two dimensions of one read")
    t = t.permute([pos[a.id] for a in want if a.id in pos])
    shape, k = [], 0
    for a in want:
        if a.id in pos:
            shape.append(t.shape[k])
            k += 1
        else:
            shape.append(1)
    return t.reshape(shape)


class Interpreter:
    def __init__(self, inputs: dict):
        self.bufs: dict = dict(inputs)           # Buffer name -> tensor shaped like the buffer's dims

    def read(self, r: ir.Read, want: list[Atom]) -> torch.Tensor:
        t = self.bufs[r.buf.name].double() if self.bufs[r.buf.name].is_floating_point() else self.bufs[r.buf.name]
        idx = list(r.idx)
        if r.gather is not None:
            d, tbuf, tidx = r.gather
            assert d == 0
            table = self.bufs[tbuf.name].long()
            t = t[table]                          # [table dims..., rest of the pool dims]
            idx = list(tidx) + idx[1:]
        have: list[Atom] = []
        shape = []
        for atoms in idx:
            ax = [a for a in ir.leaves(atoms) if not a.broadcast]
            have.extend(a for a in ax if a.hint != 1)
            shape.extend(a.hint for a in ax if a.hint != 1)
        t = t.reshape(shape)
        return _to_axes(t, have, want)

    def value(self, e: ir.Expr, want: list[Atom]) -> torch.Tensor:
        if isinstance(e, ir.Const):
            return torch.tensor(e.value, dtype=torch.float64)
        if isinstance(e, ir.Scalar):
            return torch.tensor(float(e.fn(self.args)), dtype=torch.float64)
        if isinstance(e, ir.Read):
            return self.read(e, want)
        if isinstance(e, ir.Bin):
            a, b = self.value(e.a, want), self.value(e.b, want)
            return {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b, "max": torch.maximum(a, b)}[e.op]
        if isinstance(e, ir.Un):
            a = self.value(e.a, want)
            return {"exp": torch.exp, "exp2": torch.exp2, "tanh": torch.tanh, "neg": torch.neg,
                    "recip": torch.reciprocal, "relu": torch.relu, "sigmoid": torch.sigmoid,
                    "silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu,
                    "gelu_tanh": lambda x: torch.nn.functional.gelu(x, approximate="tanh"),
                    "sqrt": torch.sqrt, "rsqrt": torch.rsqrt, "abs": torch.abs}[e.op](a)
        if isinstance(e, ir.Dot):
            inner = want + [a for a in _axes(e.over) if a.id not in {w.id for w in want}]
            prod = self.value(e.a, inner) * self.value(e.b, inner)
            extra = list(range(len(want), len(inner)))
            return prod.sum(dim=extra) if extra else prod
        if isinstance(e, ir.Select):
            a = self.value(e.a, want)
            keep = torch.ones((), dtype=torch.bool)
            for c in e.clauses:
                keep = keep & (c.ci * self.index(c.row, want) + c.cj * self.index(c.col, want) + c.c0 <= 0)
            return torch.where(keep, a, torch.tensor(e.other, dtype=torch.float64))
        raise TypeError(type(e))

    def index(self, atoms: Sequence[Atom], want: list[Atom]) -> torch.Tensor:
        """Mixed-radix composition of ``atoms`` as an integer tensor over the axes ``want``."""
        total = torch.zeros((), dtype=torch.long)
        for a in ir.leaves(atoms):
            total = total * a.hint
            if a.hint != 1:
                total = total + _to_axes(torch.arange(a.hint), [a], want)
        return total

    def run(self, nests: Sequence[ir.Nest], args: Sequence) -> dict:
        self.args = args
        for n in nests:
            par, red = _axes(n.par), _axes(n.red)
            s = n.stmt
            if isinstance(s, ir.Assign):
                val = self.value(s.value, par)
            elif isinstance(s, ir.Accum):
                val = self.value(s.value, par + red)
                dims = list(range(len(par), len(par) + len(red)))
                val = val.amax(dim=dims) if s.op == "max" else val.sum(dim=dims)
            else:
                sc = self.value(s.score, par + red).expand([a.hint for a in par + red])
                flat = sc.reshape([a.hint for a in par] + [-1])
                if s.base2:
                    flat = flat * math.log(2.0)
                ex = torch.exp(flat - flat.amax(dim=-1, keepdim=True))
                den = ex.sum(dim=-1, keepdim=True)
                for t in s.denom_add:
                    den = den + self.value(t, [])
                p = (ex / den).reshape(sc.shape)
                w = self.read(s.weights, par + red)
                val = (p * w).sum(dim=list(range(len(par), len(par) + len(red))))
                if s.epilogue is not None:
                    val = val + self.read(s.epilogue, par)
            buf = n.writes()
            val = val.expand([a.hint for a in par])
            # store shaped like the buffer's dims (atoms of a dim merged, in the buffer's order)
            order = [a for d in buf.dims for a in _axes(d)]
            val = _to_axes(val, par, order).expand([a.hint for a in order])
            self.bufs[buf.name] = val.reshape([math.prod(a.hint for a in ir.leaves(d)) for d in buf.dims])
        return self.bufs
