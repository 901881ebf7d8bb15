"""ATen graph -> one loop nest per compute op (the counterpart of the reference's graph
parser and op builders, ``loopfuse/torch_backend/interface.py:357-527`` and
``loopfuse/torch_backend/ops.py:344-751``).

View ops (transpose, expand, unsqueeze, view/reshape, clone, ``loopfuse::paged_load``) build
nothing: they regroup the atoms of a ``View``.  Compute ops (bmm, scalar multiply / divide,
tanh, the two mask ops, softmax) instantiate their operands with fresh atoms, unify the index
ranges that must agree, and append one nest that writes a temporary buffer.
"""
from __future__ import annotations

import dataclasses
import math
import operator
from typing import Optional

import torch

from . import ir
from .ir import Atom, Buffer

aten = torch.ops.aten


class Unsupported(Exception):
    """The graph uses something these builders do not cover."""


@dataclasses.dataclass
class View:
    """A tensor value: ``dims[k]`` = atoms of view dimension k; ``idx[d]`` = atoms that index
    dimension d of ``buf``; ``gather`` = (d, table View): buffer dimension d is read at
    ``table[...]`` (page gather)."""

    buf: Buffer
    idx: list[list[Atom]]
    dims: list[list[Atom]]
    gather: Optional[tuple] = None

    def instantiate(self, memo: Optional[dict] = None) -> "View":
        """The same structure over fresh atoms (every use of a value gets its own)."""
        memo = {} if memo is None else memo

        def cp(a: Atom) -> Atom:
            a = a.rep()
            if a.id not in memo:
                n = Atom(a.size, a.hint, a.name.rstrip("'") + "'")
                n.broadcast = a.broadcast
                memo[a.id] = n
                if a.children is not None:
                    n.children = [cp(c) for c in a.children]
            return memo[a.id]

        g = None
        if self.gather is not None:
            g = (self.gather[0], self.gather[1].instantiate(memo))
        return View(self.buf, [[cp(a) for a in d] for d in self.idx], [[cp(a) for a in d] for d in self.dims], g)

    def read(self) -> ir.Read:
        g = None if self.gather is None else (self.gather[0], self.gather[1].buf, self.gather[1].idx)
        return ir.Read(self.buf, self.idx, g)


def _is_float(dtype_name: str) -> bool:
    return dtype_name.startswith(("float", "bfloat", "half", "double"))


def _hint(x) -> int:
    if isinstance(x, int):
        return x
    return int(x.node.hint)


def _sym(x) -> str:
    return str(x)


class Parser:
    """Walks the graph once; ``nests`` and ``out`` (the View of the graph's single output) result."""

    def __init__(self, gm: torch.fx.GraphModule):
        self.gm = gm
        self.env: dict = {}              # fx node -> View | ("scalar", fn, text) | ("size", fn, text, hint)
        self.nests: list[ir.Nest] = []
        self.inputs: list[Buffer] = []
        self.sizes: dict[str, int] = {}  # size symbol -> placeholder index (SymInt inputs), for evaluation per call
        self.ntemp = 0
        self.out: Optional[View] = None
        self.cur_node: Optional[torch.fx.Node] = None     # the node whose nests are being built

    # ------------------------------------------------------------ helpers
    def temp(self, name: str, dims: list[list[Atom]]) -> Buffer:
        self.ntemp += 1
        return Buffer(f"{name}{self.ntemp}", dims, "temp")

    def size_of(self, a):
        """(symbol text, hint) of a size argument: int, SymInt-valued node or python int."""
        if isinstance(a, torch.fx.Node):
            v = self.env[a]
            if v[0] != "size":
                raise Unsupported(f"{a} is not a size")
            return v[2], v[3]
        return str(int(a)), int(a)

    def emit(self, name: str, out_dims: list[list[Atom]], red: list[Atom], value: ir.Expr, accum=None) -> View:
        buf = self.temp(name, out_dims)
        buf.node = self.cur_node
        stmt = ir.Assign(buf, value) if accum is None else ir.Accum(buf, accum[0], value, accum[1])
        self.nests.append(ir.Nest(buf.name, [a for d in out_dims for a in d], red, stmt))
        return View(buf, [list(d) for d in out_dims], [list(d) for d in out_dims])

    # ------------------------------------------------------------ the walk
    def run(self) -> "Parser":
        ph = 0
        for n in self.gm.graph.nodes:
            if n.op == "placeholder":
                v = n.meta.get("val")
                if isinstance(v, torch.Tensor) and v.dim() == 0:
                    # a python float of the traced function that dynamo lifted into a 0-dim tensor input
                    # (a softcap held in a variable): a run-time scalar
                    self.env[n] = ("scalar", (lambda args, i=ph: float(args[i])), n.name)
                elif isinstance(v, torch.Tensor):
                    dims = [[Atom(_sym(s), _hint(s), f"{n.name}.{k}")] for k, s in enumerate(v.shape)]
                    buf = Buffer(n.name, dims, "input", str(v.dtype).replace("torch.", ""), ph)
                    self.inputs.append(buf)
                    self.env[n] = View(buf, [list(d) for d in dims], [list(d) for d in dims])
                elif isinstance(v, (torch.SymInt, int)):
                    idx = ph
                    self.sizes[_sym(v)] = idx
                    self.env[n] = ("size", (lambda args, i=idx: int(args[i])), _sym(v), _hint(v))
                elif isinstance(v, (torch.SymFloat, float)):
                    # a python float of the traced function that dynamo made a graph input (a softcap
                    # held in a variable): a run-time scalar
                    self.env[n] = ("scalar", (lambda args, i=ph: float(args[i])), n.name)
                else:
                    raise Unsupported(f"placeholder {n.name} of type {type(v).__name__}")
                ph += 1
            elif n.op == "call_function":
                self.cur_node = n
                self.env[n] = self.call(n)
            elif n.op == "output":
                outs = n.args[0]
                outs = outs if isinstance(outs, (tuple, list)) else (outs,)
                if len(outs) != 1 or not isinstance(self.env.get(outs[0]), View):
                    raise Unsupported("graphs with one tensor output only")
                self.out = self.env[outs[0]]
                if self.out.buf.kind == "input" and not _is_float(self.out.buf.dtype):
                    raise Unsupported("integer output")
            else:
                raise Unsupported(f"node kind {n.op}")
        return self

    # keyword arguments whose given value changes nothing (anything else is refused: the nests below are
    # built from the positional arguments alone)
    _NEUTRAL_KWARGS = {"alpha": 1, "beta": 1, "rounding_mode": None, "keepdim": None, "memory_format": None,
                       "pin_memory": None, "layout": None, "device": None, "non_blocking": False}
    _VIEW_OPS = None

    def _guard(self, n: torch.fx.Node) -> None:
        """Refuse what the builder would otherwise get silently wrong: scaled forms of add / sub / addmm
        (``alpha`` / ``beta``), rounding divisions, conversions to a non-floating type (the kernels compute
        in fp32 and treat a conversion as the identity), and integer tensors used as values (only gather
        tables may be integers)."""
        t, a = n.target, n.args
        for k, v in n.kwargs.items():
            if k == "keepdim" or (k == "dtype" and (v is None or (isinstance(v, torch.dtype) and v.is_floating_point))):
                continue
            if k in self._NEUTRAL_KWARGS and (v == self._NEUTRAL_KWARGS[k] or v is None):
                continue
            if k in ("memory_format", "layout", "device", "pin_memory"):
                continue                      # where a copy lives, not what it holds
            if k == "approximate" and t is torch.ops.aten.gelu.default and v in ("none", "tanh"):
                continue                      # read by the gelu handler
            raise Unsupported(f"{t}: keyword argument {k}={v!r}")
        aten = torch.ops.aten
        if t is torch.ops.prims.convert_element_type.default and len(a) > 1 and isinstance(a[1], torch.dtype) \
                and not a[1].is_floating_point:
            raise Unsupported(f"conversion to {a[1]}")
        if t is aten._softmax.default and len(a) > 2 and a[2]:
            raise Unsupported("_softmax with half_to_float")
        if Parser._VIEW_OPS is None:
            Parser._VIEW_OPS = {aten.transpose.int, aten.t.default, aten.permute.default, aten.unsqueeze.default, aten.clone.default,
                                aten.alias.default, aten.expand.default, aten.view.default, aten._unsafe_view.default,
                                aten.reshape.default, aten.sym_size.int}
        if t in Parser._VIEW_OPS:
            return
        for k, x in enumerate(a):
            v = self.env.get(x) if isinstance(x, torch.fx.Node) else None
            if isinstance(v, View) and v.buf.kind == "input" and not _is_float(v.buf.dtype):
                if t is torch.ops.loopfuse.paged_load.default and k == 1:
                    continue                  # the page table
                raise Unsupported(f"{t}: integer tensor {v.buf.name} used as a value")

    def call(self, n: torch.fx.Node):
        self._guard(n)
        t, a = n.target, n.args
        val = lambda x: self.env[x] if isinstance(x, torch.fx.Node) else x
        # ---- integer arithmetic on sizes
        if t in (operator.mul, operator.floordiv, operator.add, operator.sub):
            (sa, ha), (sb, hb) = self.size_of(a[0]), self.size_of(a[1])
            fa = val(a[0])[1] if isinstance(a[0], torch.fx.Node) else (lambda args, c=int(a[0]): c)
            fb = val(a[1])[1] if isinstance(a[1], torch.fx.Node) else (lambda args, c=int(a[1]): c)
            sym = {operator.mul: "*", operator.floordiv: "//", operator.add: "+", operator.sub: "-"}[t]
            fn = None if (fa is None or fb is None) else (lambda args, f=t, x=fa, y=fb: f(x(args), y(args)))
            return ("size", fn, f"({sa}{sym}{sb})", t(ha, hb))
        if t is aten.sym_size.int:
            # extent of a view dimension: only its traced value and text are needed (dims are atoms)
            v = val(a[0])
            d = v.dims[a[1] % len(v.dims)]
            return ("size", None, "*".join(x.size for x in ir.leaves(d)) or "1", math.prod(x.hint for x in ir.leaves(d)) if d else 1)
        # ---- 0-dim values computed from sizes (D ** -0.5 and the like)
        if t is aten.scalar_tensor.default:
            x = a[0]
            if isinstance(x, torch.fx.Node):
                s = self.env[x]
                return ("scalar", (lambda args, f=s[1]: float(f(args))), s[2])
            return ("scalar", (lambda args, c=float(x): c), f"{float(x):g}")
        if t is torch.ops.prims.convert_element_type.default and isinstance(val(a[0]), tuple):
            return val(a[0])
        if t in (aten.add.Tensor, aten.sub.Tensor, aten.mul.Tensor, aten.div.Tensor) and len(a) == 2 and \
                all(isinstance(val(x), tuple) and val(x)[0] == "scalar" or isinstance(x, (int, float)) for x in a) and \
                any(isinstance(val(x), tuple) for x in a):
            # arithmetic on 0-dim values ((D + D2) ** -0.5)
            def part(x):
                v = val(x)
                return (v[1], v[2]) if isinstance(v, tuple) else ((lambda args, c=float(x): c), f"{float(x):g}")
            (fa, ta), (fb, tb) = part(a[0]), part(a[1])
            op, sym = {aten.add.Tensor: (operator.add, "+"), aten.sub.Tensor: (operator.sub, "-"),
                       aten.mul.Tensor: (operator.mul, "*"), aten.div.Tensor: (operator.truediv, "/")}[t]
            return ("scalar", (lambda args, f=op, x=fa, y=fb: f(x(args), y(args))), f"({ta}{sym}{tb})")
        if t is aten.pow.Tensor_Tensor and isinstance(val(a[0]), tuple) and isinstance(val(a[1]), tuple):
            x, y = val(a[0]), val(a[1])
            return ("scalar", (lambda args, f=x[1], g=y[1]: f(args) ** g(args)), f"{x[2]}**{y[2]}")
        # ---- views
        if t is aten.transpose.int:
            v = val(a[0])
            d0, d1 = a[1] % len(v.dims), a[2] % len(v.dims)
            dims = list(v.dims)
            dims[d0], dims[d1] = dims[d1], dims[d0]
            return dataclasses.replace(v, dims=dims)
        if t is aten.t.default:
            v = val(a[0])
            if len(v.dims) > 2:
                raise Unsupported("t() of a tensor with more than two dims")
            return dataclasses.replace(v, dims=list(reversed(v.dims)))
        if t is aten.permute.default:
            v = val(a[0])
            return dataclasses.replace(v, dims=[v.dims[p % len(v.dims)] for p in a[1]])
        if t is aten.unsqueeze.default:
            v = val(a[0])
            dims = list(v.dims)
            dims.insert(a[1] % (len(dims) + 1), [])
            return dataclasses.replace(v, dims=dims)
        if t in (aten.clone.default, aten.alias.default, aten.contiguous.default if hasattr(aten, "contiguous") else None):
            return val(a[0])
        if t is torch.ops.prims.convert_element_type.default or t is aten._to_copy.default:
            return val(a[0])             # precision of intermediates is the kernels' business (fp32 throughout)
        if t is aten.expand.default:
            v = val(a[0])
            dims = [list(d) for d in v.dims]
            dims = [[] for _ in range(len(a[1]) - len(dims))] + dims
            for k, s in enumerate(a[1]):
                if not isinstance(s, torch.fx.Node) and int(s) == -1:
                    continue                  # -1: the dimension stays as it is
                sym, h = self.size_of(s)
                have = math.prod(x.hint for x in ir.leaves(dims[k])) if dims[k] else 1
                if have == 1 and h != 1:
                    b = Atom(sym, h, f"{n.name}.bc{k}")
                    b.broadcast = True
                    dims[k] = [b]
                elif have != h:
                    raise Unsupported(f"expand of dim {k}: {have} -> {h}")
            return dataclasses.replace(v, dims=dims)
        if t in (aten.view.default, aten._unsafe_view.default, aten.reshape.default):
            return self.reshape(val(a[0]), a[1])
        if t is torch.ops.loopfuse.paged_load.default:
            pool, table = val(a[0]), val(a[1])
            if pool.gather is not None or table.gather is not None or len(table.dims) != 2:
                raise Unsupported("paged_load of a view")
            # out[b, pg, *t] = pool[table[b, pg], *t]
            return View(pool.buf, pool.idx, [list(d) for d in table.dims] + [list(d) for d in pool.dims[1:]], (0, table))
        # ---- compute ops
        if t is aten.bmm.default:
            return self.bmm(val(a[0]).instantiate(), val(a[1]).instantiate())
        if t in (aten.add.Tensor, aten.sub.Tensor, aten.mul.Tensor, aten.div.Tensor) and \
                isinstance(val(a[0]), View) and isinstance(val(a[1]), View):
            return self.pointwise2({aten.add.Tensor: "add", aten.sub.Tensor: "sub", aten.mul.Tensor: "mul",
                                    aten.div.Tensor: "div"}[t], val(a[0]).instantiate(), val(a[1]).instantiate())
        if t in (aten.add.Tensor, aten.sub.Tensor) and isinstance(val(a[0]), View):
            y = val(a[1])
            const: ir.Expr = ir.Scalar(y[1], y[2]) if isinstance(y, tuple) else ir.Const(float(y))
            v = val(a[0]).instantiate()
            return self.emit("add", v.dims, [], ir.Bin("add" if t is aten.add.Tensor else "sub", v.read(), const))
        if t is aten.mm.default:
            x, y = val(a[0]).instantiate(), val(a[1]).instantiate()
            ir.unify(x.dims[1], y.dims[0])
            return self.emit("dot", [x.dims[0], y.dims[1]], [], ir.Dot(x.read(), y.read(), list(x.dims[1])))
        if t is aten.addmm.default:
            x, y = val(a[1]).instantiate(), val(a[2]).instantiate()
            ir.unify(x.dims[1], y.dims[0])
            prod = self.emit("dot", [x.dims[0], y.dims[1]], [], ir.Dot(x.read(), y.read(), list(x.dims[1])))
            return self.pointwise2("add", val(a[0]).instantiate(), prod.instantiate())
        if t is aten.exp.default or t is aten.exp2.default:
            v = val(a[0]).instantiate()
            op = "exp" if t is aten.exp.default else "exp2"
            return self.emit(op, v.dims, [], ir.Un(op, v.read()))
        if t is torch.ops.loopfuse.scan_max.default:
            # (running maximum along the last dim, its final value with the dim kept): the final value is a
            # max nest; the running one gets no nest -- the graphs that use it (the reference's online-softmax
            # hint exp2(x - run) * exp2(run - max), tests/test_attention.py:95-125) cancel it, which the
            # simplify pass carries out and insists on
            x = val(a[0]).instantiate()
            outer, red = x.dims[:-1], x.dims[-1]
            m = self.emit("max", list(outer) + [[]], list(red), x.read(), ("max", float("-inf")))
            run = Buffer(f"scan{self.ntemp}", [list(d) for d in x.dims], "scan")
            run.scan_of = m.buf
            return ("tuple", View(run, [list(d) for d in x.dims], [list(d) for d in x.dims]), m)
        if t in (aten.max.dim, aten.sum.dim_IntList, aten.amax.default):
            v = val(a[0]).instantiate()
            dims = a[1] if isinstance(a[1], (list, tuple)) else [a[1]]
            dims = [d % len(v.dims) for d in dims]
            keep = bool(a[2]) if len(a) > 2 else bool(n.kwargs.get("keepdim", False))
            red = [x for d in dims for x in v.dims[d]]
            outer = [([] if k in dims else v.dims[k]) for k in range(len(v.dims)) if keep or k not in dims]
            op = ("add", 0.0) if t is aten.sum.dim_IntList else ("max", float("-inf"))
            r = self.emit("sum" if op[0] == "add" else "max", outer, red, v.read(), op)
            return ("tuple", r) if t is aten.max.dim else r
        if t is operator.getitem and isinstance(val(a[0]), tuple) and val(a[0])[0] == "tuple":
            tup = val(a[0])
            if a[1] + 1 >= len(tup):
                raise Unsupported("indices of max are not lowered")
            return tup[a[1] + 1]
        if t in (aten.mul.Tensor, aten.div.Tensor):
            x, y = val(a[0]), val(a[1])
            if isinstance(x, View) and not isinstance(y, View):
                if isinstance(y, tuple):
                    factor: ir.Expr = ir.Scalar(y[1], y[2])
                else:
                    factor = ir.Const(float(y))
                v = x.instantiate()
                return self.emit("mul" if t is aten.mul.Tensor else "div", v.dims, [],
                                 ir.Bin("mul" if t is aten.mul.Tensor else "div", v.read(), factor))
            raise Unsupported("tensor-by-tensor products other than bmm")
        if t is aten.tanh.default:
            v = val(a[0]).instantiate()
            return self.emit("tanh", v.dims, [], ir.Un("tanh", v.read()))
        # ---- the activations of the layers around an attention (pointwise, one operand)
        unary = {aten.relu.default: "relu", aten.sigmoid.default: "sigmoid", aten.silu.default: "silu",
                 aten.neg.default: "neg", aten.reciprocal.default: "recip", aten.sqrt.default: "sqrt",
                 aten.rsqrt.default: "rsqrt", aten.abs.default: "abs"}
        if t in unary or t is aten.gelu.default:
            op = unary.get(t) or ("gelu_tanh" if n.kwargs.get("approximate", "none") == "tanh" else "gelu")
            v = val(a[0]).instantiate()
            return self.emit(op, v.dims, [], ir.Un(op, v.read()))
        if t is torch.ops.loopfuse.causal_mask.default:
            v = val(a[0]).instantiate()
            row, col = v.dims[-2], v.dims[-1]
            return self.emit("mask", v.dims, [], ir.Select([ir.Clause(-1, 1, 0, row, col)], v.read(), float("-inf")))
        if t is torch.ops.loopfuse.sliding_mask.default:
            v = val(a[0]).instantiate()
            row, col = v.dims[-2], v.dims[-1]
            # 0 <= i - j <= w - 1, top-left aligned (reference ops.py:733-741); the window may be a
            # run-time integer of the graph
            if isinstance(a[1], torch.fx.Node):
                wv = self.env[a[1]]
                w, wfn = wv[3], (lambda args, f=wv[1]: -(int(f(args)) - 1))
            else:
                w, wfn = int(a[1]), None
            cl = [ir.Clause(-1, 1, 0, row, col), ir.Clause(1, -1, -(w - 1), row, col, wfn)]
            return self.emit("mask", v.dims, [], ir.Select(cl, v.read(), float("-inf")))
        if t is aten._softmax.default:
            return self.softmax(val(a[0]), a[1])
        raise Unsupported(f"op {t}")

    def reshape(self, v: View, shape) -> View:
        """Regroup the atoms of all dims, outer to inner, into the requested sizes; an atom
        that straddles a boundary is split."""
        flat = [x for d in v.dims for x in ir.leaves(d)]
        out: list[list[Atom]] = []
        for s in shape:
            sym, want = self.size_of(s)
            cur: list[Atom] = []
            have = 1
            while have < want or (flat and flat[0].hint == 1 and have == want and len(out) == len(shape) - 1):
                if not flat:
                    raise Unsupported("reshape sizes do not multiply out")
                x = flat.pop(0)
                if have * x.hint <= want and want % (have * x.hint) == 0:
                    cur.append(x)
                    have *= x.hint
                else:
                    need = want // have
                    if x.hint % need:
                        raise Unsupported("reshape splits a dimension unevenly")
                    x.split(need, f"({sym})" if have == 1 else f"({sym})//{have}", f"({x.size})//({need})")
                    cur.append(x.children[0])
                    flat.insert(0, x.children[1])
                    have = want
            out.append(cur)
        if any(x.hint != 1 for x in flat):
            raise Unsupported("reshape sizes do not multiply out")
        return dataclasses.replace(v, dims=out)

    def pointwise2(self, op: str, x: View, y: View) -> View:
        """x op y with broadcasting: dims are aligned from the right; where both sides have an extent
        their index ranges are unified, where one side has none (size 1 / missing) the other's is taken."""
        n = max(len(x.dims), len(y.dims))
        xd = [[] for _ in range(n - len(x.dims))] + [list(d) for d in x.dims]
        yd = [[] for _ in range(n - len(y.dims))] + [list(d) for d in y.dims]
        out = []
        for a, b in zip(xd, yd):
            ha = math.prod(t.hint for t in ir.leaves(a)) if a else 1
            hb = math.prod(t.hint for t in ir.leaves(b)) if b else 1
            if ha != 1 and hb != 1:
                ir.unify(a, b)
                out.append(a)
            else:
                out.append(a if ha != 1 else b)
        return self.emit(op, out, [], ir.Bin(op, x.read(), y.read()))

    def bmm(self, x: View, y: View) -> View:
        # x [bh, m, k] @ y [bh, k, n]
        if len(x.dims) != 3 or len(y.dims) != 3:
            raise Unsupported("bmm of non-3-d operands")
        ir.unify(x.dims[0], y.dims[0])
        ir.unify(x.dims[2], y.dims[1])
        return self.emit("dot", [x.dims[0], x.dims[1], y.dims[2]], [], ir.Dot(x.read(), y.read(), list(x.dims[2])))

    def softmax(self, v: View, dim: int) -> View:
        """max, exp(x - max), sum, divide: four nests, as the reference decomposes it
        (ops.py:416-452)."""
        if dim % len(v.dims) != len(v.dims) - 1:
            raise Unsupported("softmax over a dim other than the last")
        x = v.instantiate()
        outer, red = x.dims[:-1], x.dims[-1]
        m = self.emit("max", outer, list(red), x.read(), ("max", float("-inf")))
        # the next nests read x and the row statistics over the same atoms
        e = self.emit("exp", x.dims, [], ir.Un("exp", ir.Bin("sub", x.read(), m.read())))
        e_in = e
        l = self.emit("sum", outer, list(red), e_in.read(), ("add", 0.0))
        return self.emit("prob", x.dims, [], ir.Bin("div", e_in.read(), l.read()))


def parse(gm: torch.fx.GraphModule) -> Parser:
    return Parser(gm).run()
