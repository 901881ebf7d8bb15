"""MFMA lowering of a contraction nest with its pointwise epilogue fused -- the counterpart of the
``tl.dot`` the reference emits for every contraction (``loopfuse/codegen.py:658-668``; its accuracy
cases ``tests/test_accuracy.py:56-82``: ``a @ b + c`` in two and three dims).

A nest ``out[batch.., m, n] = f(sum_k A[batch.., m, k] * B[batch.., k, n], other reads)`` with bf16 /
fp16 operands becomes one kernel: a workgroup of four waves owns a 128 x 128 tile of the output and walks
k in steps of 64; both operand tiles go global -> registers -> LDS (16-byte pieces, XOR-swizzled,
double-buffered, one barrier per step) and come back as ``v_mfma_f32_32x32x16`` operands -- by plain
16-byte reads where k is the contiguous dimension of the operand in memory, by transposed reads
(``ds_read_b64_tr_b16``) where m / n is.  The product is formed transposed (C^T = B^T A^T), so a lane
ends up with four consecutive n of one m: the epilogue expression -- whatever the fused nest holds
around the contraction -- is evaluated per element on the fp32 accumulators and stored from there.

Which of the two layouts an operand has is decided per call from its strides (a flag in the
parameter block, uniform over the launch).  Calls the kernel cannot serve (strides that are not
multiples of 8 elements, k or the contiguous extent not a multiple of 8, unaligned bases) take the
plain one-thread-per-element kernel of the same nest.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

from . import ir
from .emit import _CT, MAX_N, MAX_PTR, Emitter, Kernel, NotLowerable

BM = BN = 128
BK = 64

GEMM_PRELUDE = r"""
typedef float lfg_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int lfg_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int lfg_u32x2 __attribute__((ext_vector_type(2)));
typedef short lfg_s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 lfg_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 lfg_f16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ lfg_f32x16 lfg_mfma(__bf16, lfg_u32x4 a, lfg_u32x4 b, lfg_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(lfg_bf16x8, a), __builtin_bit_cast(lfg_bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ lfg_f32x16 lfg_mfma(_Float16, lfg_u32x4 a, lfg_u32x4 b, lfg_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(lfg_f16x8, a), __builtin_bit_cast(lfg_f16x8, b), c, 0, 0, 0);
}
// Operand tiles in LDS, 8192 two-byte elements each.
//   k-contiguous operand ("rows"): [128 rows (m or n)][64 k]; the eight 16-byte pieces of a row are permuted by the
//   row pair, so that the 16-byte reads of 16 consecutive rows touch every bank once.
//   m/n-contiguous operand ("cols"): [64 k][128 m or n]; the 64-byte groups of a row are permuted by the row, for the
//   transposed reads (4 consecutive rows x 64 contiguous bytes per 32 lanes).
__device__ __forceinline__ int lfg_rows_at(int row, int piece) { return row * 64 + 8 * (piece ^ ((row >> 1) & 7)); }
__device__ __forceinline__ int lfg_cols_at(int row, int piece) { return row * 128 + 8 * (piece ^ (4 * (row & 3))); }
// global -> registers: the four 16-byte pieces of a 128 x 64 / 64 x 128 tile that thread `tid` stages; pieces outside
// [0, lim_outer) x [0, lim_k) arrive as zeros (extents are multiples of 8 along the contiguous dimension)
template <typename T>
__device__ __forceinline__ void lfg_fetch(lfg_u32x4 (&st)[4], const T* base, bool rows, long long s_outer, long long s_k,
                                          long long o0, long long lim_outer, long long k0, long long lim_k, int tid) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int idx = tid + 256 * j;
    long long o, k;
    if (rows) { o = o0 + (idx >> 3); k = k0 + 8 * (idx & 7); }
    else { k = k0 + (idx >> 4); o = o0 + 8 * (idx & 15); }
    const bool ok = o < lim_outer && k < lim_k;
    const T* src = base + (ok ? o * s_outer + k * s_k : 0ll);
    const lfg_u32x4 v = *reinterpret_cast<const lfg_u32x4*>(src);
    st[j] = ok ? v : lfg_u32x4{0u, 0u, 0u, 0u};
  }
}
__device__ __forceinline__ void lfg_stage(unsigned short* tile, const lfg_u32x4 (&st)[4], bool rows, int tid) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int idx = tid + 256 * j;
    const int at = rows ? lfg_rows_at(idx >> 3, idx & 7) : lfg_cols_at(idx >> 4, idx & 15);
    *reinterpret_cast<lfg_u32x4*>(&tile[at]) = st[j];
  }
}
// MFMA operand (either side: 32 rows or columns `blk`, lane % 32 picks one, lane / 32 the half of the 16-step `ks`):
// k = 16 * ks + 8 * (lane / 32) .. + 7 in both layouts
__device__ __forceinline__ lfg_u32x4 lfg_operand(const unsigned short* tile, bool rows, int blk, int ks, int lane) {
  const int l32 = lane & 31, g = lane >> 5;
  if (rows) return *reinterpret_cast<const lfg_u32x4*>(&tile[lfg_rows_at(32 * blk + l32, 2 * ks + g)]);
  const int j16 = lane & 15, dh = (lane >> 4) & 1;
  const int col = 32 * blk + 16 * dh + 4 * (j16 & 3);
  lfg_u32x2 h[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int row = 16 * ks + 8 * g + 4 * half + (j16 >> 2);
    const unsigned short* src = &tile[lfg_cols_at(row, col >> 3) + (col & 7)];
    const lfg_s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lfg_s16x4*)(src));
    h[half] = __builtin_bit_cast(lfg_u32x2, t);
  }
  return lfg_u32x4{h[0][0], h[0][1], h[1][0], h[1][1]};
}
"""


@dataclasses.dataclass
class GemmInfo:
    """What the launcher needs besides the usual parameter block."""
    m: ir.Atom
    n: ir.Atom
    k: ir.Atom
    batch: list                 # parallel atoms other than m, n (outer to inner)
    a_buf: ir.Buffer
    b_buf: ir.Buffer
    a_dims: tuple               # (dim of A indexed by m, dim indexed by k)
    b_dims: tuple               # (dim of B indexed by n, dim indexed by k)
    a_batch_dims: list          # dims of A indexed by a batch atom
    b_batch_dims: list
    flags_at: int = 0           # n[flags_at], n[flags_at + 1]: A / B are k-contiguous


def _single(atoms) -> Optional[ir.Atom]:
    """The one atom of extent > 1 that indexes a buffer dimension; None for a dimension of extent 1."""
    xs = [a for a in ir.leaves(atoms) if a.hint != 1]
    if len(xs) > 1 or any(a.broadcast for a in xs):
        raise NotLowerable("an operand dimension indexed by several atoms")
    return xs[0] if xs else None


def match(nest: ir.Nest, dtypes: dict) -> Optional[GemmInfo]:
    """The nest as batched matrix product + pointwise epilogue, or None."""
    s = nest.stmt
    if not isinstance(s, ir.Assign) or [a for a in ir.leaves(nest.red) if a.hint != 1]:
        return None
    dots = [e for e in ir.walk(s.value) if isinstance(e, ir.Dot)]
    if len(dots) != 1:
        return None
    d = dots[0]
    if not (isinstance(d.a, ir.Read) and isinstance(d.b, ir.Read)) or d.a.gather is not None or d.b.gather is not None:
        return None
    if dtypes.get(d.a.buf.name) not in (1, 2) or dtypes.get(d.a.buf.name) != dtypes.get(d.b.buf.name):
        return None
    over = [a for a in ir.leaves(d.over) if a.hint != 1]
    par = [a for a in ir.leaves(nest.par) if a.hint != 1]
    if len(over) != 1:
        return None
    k = over[0]
    try:
        ia = [_single(x) for x in d.a.idx]
        ib = [_single(x) for x in d.b.idx]
    except NotLowerable:
        return None

    def has(lst, a):
        return any(x is a for x in lst)

    ms = [a for a in par if has(ia, a) and not has(ib, a)]
    ns = [a for a in par if has(ib, a) and not has(ia, a)]
    if not ms or not ns or not has(ia, k) or not has(ib, k):
        return None
    m, n = ms[-1], ns[-1]          # the innermost one of each side; outer ones (a view of [.., M, K] rows) count as batch
    batch = [a for a in par if a is not m and a is not n]
    if any(x is not None and x is not m and x is not k and not has(batch, x) for x in ia) or \
            any(x is not None and x is not n and x is not k and not has(batch, x) for x in ib):
        return None
    # each of m, n, k indexes exactly one dimension of its operand
    if sum(x is m for x in ia) != 1 or sum(x is k for x in ia) != 1 or sum(x is n for x in ib) != 1 or sum(x is k for x in ib) != 1:
        return None
    pos = lambda lst, a: next(i for i, x in enumerate(lst) if x is a)      # noqa: E731
    return GemmInfo(m, n, k, batch, d.a.buf, d.b.buf, (pos(ia, m), pos(ia, k)), (pos(ib, n), pos(ib, k)),
                    [i for i, x in enumerate(ia) if x is not None and has(batch, x)],
                    [i for i, x in enumerate(ib) if x is not None and has(batch, x)])


class GemmEmitter(Emitter):
    """HIP source of a contraction nest on the MFMA path."""

    def __init__(self, nest: ir.Nest, dtypes: dict, name: str, info: GemmInfo):
        super().__init__(nest, dtypes, name)
        self.info = info

    def expr(self, e: ir.Expr) -> str:
        if isinstance(e, ir.Dot):
            return "accv"
        return super().expr(e)

    def emit(self) -> Kernel:
        g, n = self.info, self.nest
        par = [a for a in ir.leaves(n.par) if a.hint != 1]
        for a in par:
            self.atom(a)
        km, kn, kk = self.atom(g.m), self.atom(g.n), self.atom(g.k)
        ia, ib = self.buf(g.a_buf), self.buf(g.b_buf)
        elem = _CT[self.dtypes[g.a_buf.name]]

        def base(buf, ptr, read_idx, batch_dims):
            terms = []
            for d in batch_dims:
                a = _single(read_idx[d])
                terms.append(f"i{self.atom(a)} * S{self.stride(buf, d)}")
            return f"reinterpret_cast<const {elem}*>(p.ptr[{ptr}]) + ({' + '.join(terms) or '0ll'})"

        dot = next(e for e in ir.walk(n.stmt.value) if isinstance(e, ir.Dot))
        a_base = base(g.a_buf, ia, dot.a.idx, g.a_batch_dims)
        b_base = base(g.b_buf, ib, dot.b.idx, g.b_batch_dims)
        sam, sak = self.stride(g.a_buf, g.a_dims[0]), self.stride(g.a_buf, g.a_dims[1])
        sbn, sbk = self.stride(g.b_buf, g.b_dims[0]), self.stride(g.b_buf, g.b_dims[1])
        val = self.expr(n.stmt.value)              # epilogue on `accv`; registers its buffers, strides, scalars
        if self.lines:
            raise NotLowerable("a second contraction inside the epilogue")
        out = n.writes()
        o = self.buf(out)
        ooff = self.offset(out, out.dims, None)
        na, ns = len(self.atoms), len(self.strides)
        g.flags_at = na + ns
        if na + ns + 2 > MAX_N or len(self.bufs) > MAX_PTR:
            raise NotLowerable("nest touches too many buffers / dimensions")
        defs = [f"const long long N{k} = p.n[{k}];" for k in range(na)] + \
               [f"const long long S{k} = p.n[{na + k}];" for k in range(ns)]
        batch_decode = []
        for a in reversed(g.batch):
            k = self.atom(a)
            batch_decode.append(f"const long long i{k} = blk % N{k}; blk /= N{k};")
        src = f"""extern "C" __global__ void __launch_bounds__(256, 2) {self.name}(const LfGenParams p) {{
  {' '.join(defs)}
  const bool a_rows = p.n[{g.flags_at}] != 0, b_rows = p.n[{g.flags_at + 1}] != 0;
  __shared__ __attribute__((aligned(16))) unsigned short tile_a[2][8192];
  __shared__ __attribute__((aligned(16))) unsigned short tile_b[2][8192];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const long long M = N{km}, Nn = N{kn}, K = N{kk};
  const long long mt = (M + {BM - 1}) / {BM}, nt = (Nn + {BN - 1}) / {BN};
  long long total = mt * nt;
  {' '.join(f'total *= N{self.atom(a)};' for a in g.batch)}
  // workgroups go to the 8 XCDs round-robin: each XCD takes a contiguous run of tiles (n fastest), so the
  // workgroups resident on it share rows of A and columns of B in its L2
  const long long per_xcd = (total + 7) / 8;
  long long blk = (long long)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((long long)(blockIdx.x >> 3) >= per_xcd || blk >= total) return;
  const long long tn = blk % nt; blk /= nt;
  const long long tm = blk % mt; blk /= mt;
  {' '.join(batch_decode)}
  const long long m0 = tm * {BM}, n0 = tn * {BN};
  const {elem}* A = {a_base};
  const {elem}* B = {b_base};
  lfg_f32x16 acc[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[nb][i] = 0.0f;
  lfg_u32x4 sa[4], sb[4];
  lfg_fetch<{elem}>(sa, A, a_rows, S{sam}, S{sak}, m0, M, 0, K, tid);
  lfg_fetch<{elem}>(sb, B, b_rows, S{sbn}, S{sbk}, n0, Nn, 0, K, tid);
  lfg_stage(tile_a[0], sa, a_rows, tid);
  lfg_stage(tile_b[0], sb, b_rows, tid);
  __syncthreads();
  const long long steps = (K + {BK - 1}) / {BK};
  for (long long st = 0; st < steps; ++st) {{
    const int cur = (int)(st & 1);
    if (st + 1 < steps) {{
      lfg_fetch<{elem}>(sa, A, a_rows, S{sam}, S{sak}, m0, M, (st + 1) * {BK}, K, tid);
      lfg_fetch<{elem}>(sb, B, b_rows, S{sbn}, S{sbk}, n0, Nn, (st + 1) * {BK}, K, tid);
    }}
#pragma unroll
    for (int ks = 0; ks < {BK // 16}; ++ks) {{
      const lfg_u32x4 fm = lfg_operand(tile_a[cur], a_rows, wave, ks, lane);       // A rows of this wave: lane = m
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
        acc[nb] = lfg_mfma(({elem})0.0f, lfg_operand(tile_b[cur], b_rows, nb, ks, lane), fm, acc[nb]);
    }}
    if (st + 1 < steps) {{
      lfg_stage(tile_a[cur ^ 1], sa, a_rows, tid);
      lfg_stage(tile_b[cur ^ 1], sb, b_rows, tid);
    }}
    __syncthreads();
  }}
  // C^T[n][m]: lane holds m = m0 + 32 * wave + lane % 32; element i of block nb is n = n0 + 32 * nb + 8 * (i / 4) + 4 * (lane / 32) + i % 4
  const long long i{km} = m0 + 32 * wave + (lane & 31);
  if (i{km} >= M) return;
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int i = 0; i < 16; ++i) {{
      const long long i{kn} = n0 + 32 * nb + 8 * (i / 4) + 4 * (lane >> 5) + (i % 4);
      if (i{kn} < Nn) {{
        const float accv = acc[nb][i];
        const float result = {val};
        lfg_st<{_CT[self.dtypes[out.name]]}>(p.ptr[{o}], {ooff}, result);
      }}
    }}
}}
"""
        return Kernel(self.name, src, self.bufs, self.atoms, self.strides, self.scalars, par)
