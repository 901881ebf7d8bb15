"""Generic lowering of fused loop nests to HIP source -- for graphs that are not an attention
(the reference's non-attention accuracy cases, tests/test_accuracy.py:29-82, 197-211, 235-250,
314-333: add, matmul + add, softmax @ matmul, paged add, the max + sum normalisation).

The reference prints every fused nest as a Triton kernel (``loopfuse/codegen.py:100-404``); this
is the same step for HIP, kept deliberately plain: one kernel per nest, one thread per element of
the nest's output, reduction atoms and ``Dot`` contractions as sequential loops of that thread,
fp32 arithmetic.  The attention path does not come through here -- it goes to the hand-written
MFMA kernels -- so nothing in this file is tuned.

A kernel takes one by-value block ``LfGenParams``: pointers of the buffers it touches, the run-time
extent of every leaf atom, the element strides of every buffer dimension, run-time scalars.
"""
from __future__ import annotations

import ctypes
import dataclasses
import math
from typing import Optional, Sequence

import torch

from . import ir
from .ir import Atom

MAX_PTR, MAX_N, MAX_F = 12, 96, 8

_DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2, torch.int32: 3, torch.int64: 4}
_CT = {0: "float", 1: "__bf16", 2: "_Float16", 3: "int", 4: "long long"}

PRELUDE = f"""
struct LfGenParams {{ void* ptr[{MAX_PTR}]; long long n[{MAX_N}]; float f[{MAX_F}]; }};
template <typename T> __device__ __forceinline__ float lfg_ld(const void* p, long long i) {{ return (float)reinterpret_cast<const T*>(p)[i]; }}
template <typename T> __device__ __forceinline__ long long lfg_ldi(const void* p, long long i) {{ return (long long)reinterpret_cast<const T*>(p)[i]; }}
template <typename T> __device__ __forceinline__ void lfg_st(void* p, long long i, float v) {{ reinterpret_cast<T*>(p)[i] = (T)v; }}
__device__ __forceinline__ float lfg_sigmoid(float x) {{ return 1.0f / (1.0f + __expf(-x)); }}
__device__ __forceinline__ float lfg_silu(float x) {{ return x / (1.0f + __expf(-x)); }}
__device__ __forceinline__ float lfg_gelu(float x) {{ return 0.5f * x * (1.0f + erff(x * 0.70710678f)); }}
__device__ __forceinline__ float lfg_gelu_tanh(float x) {{ return 0.5f * x * (1.0f + tanhf(0.79788456f * (x + 0.044715f * x * x * x))); }}
"""


class GenParams(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p * MAX_PTR), ("n", ctypes.c_longlong * MAX_N), ("f", ctypes.c_float * MAX_F)]


class NotLowerable(Exception):
    pass


@dataclasses.dataclass
class Kernel:
    name: str
    source: str
    bufs: list                      # Buffers in ptr[] order; the written one is last
    atoms: list                     # leaf atoms whose extents fill n[0 : len(atoms)]
    strides: list                   # (buffer, dim) pairs whose element strides follow in n[]
    scalars: list                   # ir.Scalar nodes filling f[]
    par: list                       # parallel leaf atoms (thread index, outer to inner)
    lanes_per_output: int = 1       # 64: one wave per output element (a reduction shared by its lanes)


class Emitter:
    """HIP source of one nest."""

    def __init__(self, nest: ir.Nest, dtypes: dict, name: str):
        self.nest, self.dtypes, self.name = nest, dtypes, name
        self.bufs: list = []
        self.atoms: list = []
        self.strides: list = []
        self.scalars: list = []
        self.lines: list = []
        self.tmp = 0

    def buf(self, b) -> int:
        for i, x in enumerate(self.bufs):
            if x is b:
                return i
        self.bufs.append(b)
        return len(self.bufs) - 1

    def atom(self, a: Atom) -> int:
        for i, x in enumerate(self.atoms):
            if x is a:
                return i
        self.atoms.append(a)
        return len(self.atoms) - 1

    def index(self, atoms: Sequence[Atom]) -> str:
        """C expression of the mixed-radix composition of ``atoms`` (loop variables i<k>)."""
        e = "0ll"
        for a in ir.leaves(atoms):
            if a.hint == 1 or a.broadcast:
                if a.hint != 1:
                    raise NotLowerable("a broadcast atom inside a buffer index")
                continue
            k = self.atom(a)
            e = f"({e} * N{k} + i{k})"
        return e

    def offset(self, b, idx, gather) -> str:
        parts = []
        for d, atoms in enumerate(idx):
            if gather is not None and gather[0] == d:
                tb, tidx = gather[1], gather[2]
                t = self.buf(tb)
                toff = " + ".join(f"{self.index(ta)} * S{self.stride(tb, k)}" for k, ta in enumerate(tidx)) or "0ll"
                ix = f"lfg_ldi<{_CT[self.dtypes[tb.name]]}>(p.ptr[{t}], {toff})"
            else:
                ix = self.index(atoms)
            parts.append(f"{ix} * S{self.stride(b, d)}")
        return " + ".join(parts) or "0ll"

    def stride(self, b, d: int) -> int:
        key = (b, d)
        for i, (x, y) in enumerate(self.strides):
            if x is b and y == d:
                return i
        self.strides.append(key)
        return len(self.strides) - 1

    def expr(self, e: ir.Expr) -> str:
        if isinstance(e, ir.Const):
            if math.isinf(e.value):
                return "(-__builtin_inff())" if e.value < 0 else "__builtin_inff()"
            return f"{float(e.value)!r}f"
        if isinstance(e, ir.Scalar):
            self.scalars.append(e)
            if len(self.scalars) > MAX_F:
                raise NotLowerable("too many run-time scalars")
            return f"p.f[{len(self.scalars) - 1}]"
        if isinstance(e, ir.Read):
            i = self.buf(e.buf)
            return f"lfg_ld<{_CT[self.dtypes[e.buf.name]]}>(p.ptr[{i}], {self.offset(e.buf, e.idx, e.gather)})"
        if isinstance(e, ir.Bin):
            a, b = self.expr(e.a), self.expr(e.b)
            return f"fmaxf({a}, {b})" if e.op == "max" else f"({a} {dict(add='+', sub='-', mul='*', div='/')[e.op]} {b})"
        if isinstance(e, ir.Un):
            a = self.expr(e.a)
            if e.op in ("sigmoid", "silu", "gelu", "gelu_tanh"):
                return f"lfg_{e.op}({a})"
            return {"exp": f"__expf({a})", "exp2": f"exp2f({a})", "tanh": f"tanhf({a})", "neg": f"(-{a})",
                    "recip": f"(1.0f / {a})", "relu": f"fmaxf({a}, 0.0f)", "sqrt": f"sqrtf({a})",
                    "rsqrt": f"(1.0f / sqrtf({a}))", "abs": f"fabsf({a})"}[e.op]
        if isinstance(e, ir.Select):
            conds = [f"({c.ci}ll * {self.index(c.row)} + {c.cj}ll * {self.index(c.col)} + {c.c0}ll <= 0)" for c in e.clauses]
            other = "(-__builtin_inff())" if e.other == float("-inf") else f"{float(e.other)!r}f"
            return f"(({' && '.join(conds)}) ? {self.expr(e.a)} : {other})"
        if isinstance(e, ir.Dot):
            # a sequential contraction: emitted as a statement block, its value a fresh variable
            self.tmp += 1
            v = f"acc{self.tmp}"
            self.lines.append(f"float {v} = 0.0f;")
            over = [a for a in ir.leaves(e.over) if a.hint != 1]
            for a in over:
                k = self.atom(a)
                self.lines.append(f"for (long long i{k} = 0; i{k} < N{k}; ++i{k}) {{")
            inner_a = self.expr(e.a)
            inner_b = self.expr(e.b)
            self.lines.append(f"{v} += {inner_a} * {inner_b};")
            self.lines.extend("}" for _ in over)
            return v
        raise NotLowerable(f"expression {type(e).__name__}")

    def emit(self, wave_reduce: bool = False) -> Kernel:
        """``wave_reduce``: a reduction nest as one wave per output element -- the 64 lanes stride over the reduced
        index space (innermost reduced atom fastest, so rows that are contiguous in memory are read coalesced) and
        combine through ``ds_bpermute`` -- instead of one thread walking it alone.  GPU only."""
        n = self.nest
        s = n.stmt
        if isinstance(s, ir.Rescaled):
            raise NotLowerable("attention nests go to the MFMA kernels")
        par = [a for a in ir.leaves(n.par) if a.hint != 1]
        red = [a for a in ir.leaves(n.red) if a.hint != 1]
        for a in par:
            self.atom(a)
        body: list = []
        if wave_reduce:
            if not isinstance(s, ir.Accum) or not red:
                raise NotLowerable("not a reduction")
            init = "(-__builtin_inff())" if s.init == float("-inf") else f"{float(s.init)!r}f"
            comb = (lambda a, b: f"fmaxf({a}, {b})") if s.op == "max" else (lambda a, b: f"{a} + {b}")
            ks = [self.atom(a) for a in red]
            self.lines.append(f"float result = {init};")
            self.lines.append(f"const long long R = {' * '.join(f'N{k}' for k in ks)};")
            self.lines.append("for (long long r = lane; r < R; r += 64) {")
            self.lines.append("long long rr = r;")
            for k in reversed(ks):
                self.lines.append(f"const long long i{k} = rr % N{k}; rr /= N{k};")
            val = self.expr(s.value)
            self.lines.append(f"result = {comb('result', val)};")
            self.lines.append("}")
            self.lines.append("#pragma unroll")
            self.lines.append("for (int off = 32; off > 0; off >>= 1) {")
            self.lines.append("const float other = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ off) << 2, __builtin_bit_cast(int, result)));")
            self.lines.append(f"result = {comb('result', 'other')};")
            self.lines.append("}")
            body = self.lines
        elif isinstance(s, ir.Assign):
            val = self.expr(s.value)
            body = self.lines + [f"const float result = {val};"]
        else:
            init = "(-__builtin_inff())" if s.init == float("-inf") else f"{float(s.init)!r}f"
            self.lines.append(f"float result = {init};")
            for a in red:
                k = self.atom(a)
                self.lines.append(f"for (long long i{k} = 0; i{k} < N{k}; ++i{k}) {{")
            val = self.expr(s.value)
            self.lines.append(f"result = {'fmaxf(result, ' + val + ')' if s.op == 'max' else 'result + ' + val};")
            self.lines.extend("}" for _ in red)
            body = self.lines
        out = n.writes()
        o = self.buf(out)
        ooff = self.offset(out, out.dims, None)
        # thread -> parallel atoms (inner atom fastest)
        if wave_reduce:
            dec = ["long long t = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);", "const int lane = threadIdx.x & 63;"]
        else:
            dec = ["long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;"]
        total = " * ".join(f"N{self.atom(a)}" for a in par) or "1"
        dec.append(f"if (t >= {total}) return;")
        for a in reversed(par):
            k = self.atom(a)
            dec.append(f"const long long i{k} = t % N{k}; t /= N{k};")
        na = len(self.atoms)
        if na + len(self.strides) > MAX_N or len(self.bufs) > MAX_PTR:
            raise NotLowerable("nest touches too many buffers / dimensions")
        defs = [f"const long long N{k} = p.n[{k}];" for k in range(na)] + \
               [f"const long long S{k} = p.n[{na + k}];" for k in range(len(self.strides))]
        src = (f'extern "C" __global__ void __launch_bounds__(256) {self.name}(const LfGenParams p) {{\n  ' +
               "\n  ".join(defs + dec + body) +
               f"\n  {'if (lane == 0) ' if wave_reduce else ''}lfg_st<{_CT[self.dtypes[out.name]]}>(p.ptr[{o}], {ooff}, result);\n}}\n")
        return Kernel(self.name, src, self.bufs, self.atoms, self.strides, self.scalars, par, 64 if wave_reduce else 1)
