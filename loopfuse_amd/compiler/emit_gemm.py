"""MFMA lowering of a contraction nest with its pointwise epilogue fused -- the counterpart of the
``tl.dot`` the reference emits for every contraction (``loopfuse/codegen.py:658-668``; its accuracy
cases ``tests/test_accuracy.py:56-82``: ``a @ b + c`` in two and three dims).

A nest ``out[batch.., m, n] = f(sum_k A[batch.., m, k] * B[batch.., k, n], other reads)`` with bf16 /
fp16 operands becomes one kernel.  A workgroup owns a tile of the output -- 128 x 128 on four waves (two
workgroups per CU) or 256 x 256 on eight (one per CU, half the L2 -> LDS bytes per flop; ``TILES``), a
compile-time choice -- and walks k in steps of 64.  Both operand tiles arrive by direct global -> LDS loads
(``buffer_load_dwordx4 ... lds``: 16-byte pieces, range-checked so that the edges arrive as zeros, the XOR
permutation applied on the global side), double-buffered, one barrier per step, and come back as
``v_mfma_f32_32x32x16`` operands -- by plain 16-byte reads where k is the contiguous dimension of the
operand in memory, by transposed reads (``ds_read_b64_tr_b16``) where m / n is.  The product is formed
transposed (C^T = B^T A^T); the fp32 accumulators then pass through LDS once so that a lane holds four
consecutive n of one m and neighbouring lanes neighbouring n: the epilogue expression -- whatever the
fused nest holds around the contraction -- is evaluated there per element, its reads coalesced, and the
results leave in 8- or 16-byte stores along the rows of the output.  Tiles are walked in bands of a few
tile rows, an XCD taking a contiguous run of them, so that its resident workgroups share operand rows and
columns in its L2.

Which of the two layouts an operand has is a compile-time flag of the kernel (``-DLFG_A_ROWS``,
``-DLFG_B_ROWS``); the launcher picks the code object per call from the strides.  Calls the kernel
cannot serve (strides that are not multiples of 8 elements, k or the contiguous extent not a multiple
of 8, unaligned bases, an operand beyond the 32-bit byte offsets of the loads) take the plain
one-thread-per-element kernel of the same nest.
"""
from __future__ import annotations

import dataclasses
from typing import Optional

from . import ir
from .emit import _CT, MAX_N, MAX_PTR, Emitter, Kernel, NotLowerable

BK = 64
# workgroup tiles (waves along m, waves along n, 32 x 32 blocks per wave along m, along n): 128 x 128 on four waves at
# two workgroups per CU; 256 x 256 on eight waves, one per CU, with half the L2 -> LDS bytes per flop
TILES = {"s": (2, 2, 2, 2), "l": (4, 2, 2, 4)}


def tile_extent(shape: str) -> tuple:
    wm, wn, mb, nb = TILES[shape]
    return 32 * wm * mb, 32 * wn * nb


def tile_options(shape: str) -> list:
    wm, wn, mb, nb = TILES[shape]
    return [f"-DLFG_WGM={wm}", f"-DLFG_WGN={wn}", f"-DLFG_MB={mb}", f"-DLFG_NB={nb}"]

GEMM_PRELUDE = r"""
typedef float lfg_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int lfg_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int lfg_u32x2 __attribute__((ext_vector_type(2)));
typedef float lfg_f32x4 __attribute__((ext_vector_type(4)));
typedef short lfg_s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 lfg_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 lfg_f16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ lfg_f32x16 lfg_mfma(__bf16, lfg_u32x4 a, lfg_u32x4 b, lfg_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(lfg_bf16x8, a), __builtin_bit_cast(lfg_bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ lfg_f32x16 lfg_mfma(_Float16, lfg_u32x4 a, lfg_u32x4 b, lfg_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(lfg_f16x8, a), __builtin_bit_cast(lfg_f16x8, b), c, 0, 0, 0);
}
// Operand tiles in LDS; `kExtent` = rows / columns of the workgroup's tile along m (A) or n (B), 64 k per step.
//   k-contiguous operand ("rows"): [kExtent rows][64 k]; the eight 16-byte pieces of a row are permuted by the
//   row pair, so that the 16-byte reads of 16 consecutive rows touch every bank once.
//   m/n-contiguous operand ("cols"): [64 k][kExtent]; the 64-byte groups of a row are permuted by the row, for the
//   transposed reads (4 consecutive rows x 64 contiguous bytes per 32 lanes).
__device__ __forceinline__ int lfg_rows_at(int row, int piece) { return row * 64 + 8 * (piece ^ ((row >> 1) & 7)); }
template <int kExtent>
__device__ __forceinline__ int lfg_cols_at(int row, int piece) { return row * kExtent + 8 * (piece ^ (4 * (row & 3))); }
// Tiles arrive by direct global -> LDS loads: a wave-level load writes 64 lanes x 16 bytes at M0 + 16 * lane, i.e. 64
// consecutive 16-byte positions `idx` of the tile, and the permutation is applied on the global side: the lane that
// fills position idx fetches the piece (outer = m or n, k) that lives there.
template <bool kRows, int kExtent> struct LfgPiece {
  static __device__ __forceinline__ int outer(int idx) {
    return kRows ? (idx >> 3) : 8 * ((idx % (kExtent / 8)) ^ (4 * ((idx / (kExtent / 8)) & 3)));
  }
  static __device__ __forceinline__ int k(int idx) {
    return kRows ? 8 * ((idx & 7) ^ ((idx >> 4) & 7)) : idx / (kExtent / 8);
  }
};
// Buffer resource over `bytes` bytes from `base` (raw buffer, 32-bit offsets, range checked: a load beyond the range
// delivers zeros)
__device__ __forceinline__ lfg_u32x4 lfg_make_buffer(const void* base, unsigned bytes) {
  const unsigned long long a = (unsigned long long)base;
  lfg_u32x4 rs;
  rs[0] = __builtin_amdgcn_readfirstlane((unsigned)a);
  rs[1] = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32) & 0xffffu);
  rs[2] = __builtin_amdgcn_readfirstlane(bytes);
  rs[3] = 0x00020000u;
  return rs;
}
// One wave-level direct-to-LDS load (not tracked by the compiler's wait counters: callers wait with s_waitcnt vmcnt)
__device__ __forceinline__ void lfg_dma(const lfg_u32x4& rs, unsigned voff, unsigned lds_addr) {
  unsigned m0_written;
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %3, 0 offen lds"
               : "={m0}"(m0_written) : "s"(lds_addr), "v"(voff), "s"(rs) : "memory");
}
// MFMA operand (either side: 32 rows or columns `blk`, lane % 32 picks one, lane / 32 the half of the 16-step `ks`):
// k = 16 * ks + 8 * (lane / 32) .. + 7 in both layouts
template <bool kRows, int kExtent>
__device__ __forceinline__ lfg_u32x4 lfg_operand(const unsigned short* tile, int blk, int ks, int lane) {
  const int l32 = lane & 31, g = lane >> 5;
  if (kRows) return *reinterpret_cast<const lfg_u32x4*>(&tile[lfg_rows_at(32 * blk + l32, 2 * ks + g)]);
  const int j16 = lane & 15, dh = (lane >> 4) & 1;
  const int col = 32 * blk + 16 * dh + 4 * (j16 & 3);
  lfg_u32x2 h[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int row = 16 * ks + 8 * g + 4 * half + (j16 >> 2);
    const unsigned short* src = &tile[lfg_cols_at<kExtent>(row, col >> 3) + (col & 7)];
    const lfg_s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lfg_s16x4*)(src));
    h[half] = __builtin_bit_cast(lfg_u32x2, t);
  }
  return lfg_u32x4{h[0][0], h[0][1], h[1][0], h[1][1]};
}
// four consecutive results of one output row: one store when the row is contiguous and aligned, else element-wise
template <typename T> struct LfgPack;
template <> struct LfgPack<float> { typedef lfg_u32x4 type; };
template <> struct LfgPack<__bf16> { typedef lfg_u32x2 type; };
template <> struct LfgPack<_Float16> { typedef lfg_u32x2 type; };
template <typename T>
__device__ __forceinline__ void lfg_st4(void* p, long long at, const float (&r)[4]) {
  T t[4] = {(T)r[0], (T)r[1], (T)r[2], (T)r[3]};
  typedef typename LfgPack<T>::type pack_t;
  *reinterpret_cast<pack_t*>(reinterpret_cast<T*>(p) + at) = __builtin_bit_cast(pack_t, t);
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
    flags_at: int = 0           # n[flags_at]: the output's rows are contiguous and aligned for 8- / 16-byte stores;
                                # n[flags_at + 1], n[flags_at + 2]: bytes of A / B reachable from a batch element's base
    out_buf: object = None
    out_n_dim: int = -1         # dimension of the output indexed by n alone (-1: none)


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
        g.out_buf = out
        for d, atoms in enumerate(out.dims):
            xs = [a for a in ir.leaves(atoms) if a.hint != 1]
            if len(xs) == 1 and xs[0] is g.n:
                g.out_n_dim = d
        na, ns = len(self.atoms), len(self.strides)
        g.flags_at = na + ns
        if na + ns + 3 > MAX_N or len(self.bufs) > MAX_PTR:
            raise NotLowerable("nest touches too many buffers / dimensions")
        defs = [f"const long long N{k} = p.n[{k}];" for k in range(na)] + \
               [f"const long long S{k} = p.n[{na + k}];" for k in range(ns)]
        batch_decode = []
        for a in reversed(g.batch):
            k = self.atom(a)
            batch_decode.append(f"const long long i{k} = blk % N{k}; blk /= N{k};")
        out_t = _CT[self.dtypes[out.name]]
        src = f"""extern "C" __global__ void __launch_bounds__(64 * LFG_WGM * LFG_WGN, 2)
{self.name}(const LfGenParams p) {{
  {' '.join(defs)}
  constexpr bool a_rows = LFG_A_ROWS != 0, b_rows = LFG_B_ROWS != 0;
  // the workgroup's tile: kWM x kWN waves, each kMB x kNB blocks of 32 x 32
  constexpr int kWM = LFG_WGM, kWN = LFG_WGN, kMB = LFG_MB, kNB = LFG_NB;
  constexpr int kBM = 32 * kWM * kMB, kBN = 32 * kWN * kNB, kWaves = kWM * kWN, kNT = 64 * kWaves;
  constexpr int kTileA = kBM * {BK}, kTileB = kBN * {BK};                    // elements of one operand tile
  constexpr int kPA = kBM * 8 / kNT, kPB = kBN * 8 / kNT;                   // 16-byte pieces per thread and tile
  static_assert(kNB % 2 == 0 && kBM * 8 % kNT == 0 && kBN * 8 % kNT == 0, "tile shape");
  static_assert(kWaves * kMB * 8192 <= 4 * (kTileA + kTileB), "the accumulators pass through the tiles' LDS");
  const bool row_stores = p.n[{g.flags_at}] != 0;
  __shared__ __attribute__((aligned(16))) unsigned short lds[2 * (kTileA + kTileB)];     // A tiles [2], then B tiles [2]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % kWM, wn = wave / kWM;
  const long long M = N{km}, Nn = N{kn}, K = N{kk};
  const long long mt = (M + kBM - 1) / kBM, nt = (Nn + kBN - 1) / kBN;
  long long total = mt * nt;
  {' '.join(f'total *= N{self.atom(a)};' for a in g.batch)}
  // workgroups go to the 8 XCDs round-robin: each XCD takes a contiguous run of tiles (n fastest), so the
  // workgroups resident on it share rows of A and columns of B in its L2
  const long long per_xcd = (total + 7) / 8;
  long long blk = (long long)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((long long)(blockIdx.x >> 3) >= per_xcd || blk >= total) return;
  // inside a batch element the tiles run in bands of kBand tile rows, column by column: the workgroups resident
  // on an XCD at a time (32 or 64 consecutive tiles) then cover a block of the output that is a few tiles tall and
  // wide, and read correspondingly few rows of A and columns of B past its L2
  constexpr long long kBand = kNT <= 256 ? 8 : 4;
  const long long t = blk % (mt * nt); blk /= mt * nt;
  const long long first = t / (kBand * nt) * kBand, tall = min(mt - first, kBand);
  const long long tm = first + (t % (kBand * nt)) % tall, tn = (t % (kBand * nt)) / tall;
  {' '.join(batch_decode)}
  const long long m0 = tm * kBM, n0 = tn * kBN;
  const {elem}* A = {a_base};
  const {elem}* B = {b_base};
  // this thread's pieces of a tile: byte offset at k = 0 and how many k are left from the piece's own k (0: the
  // piece lies outside the operand and is asked for beyond the buffer's range, i.e. arrives as zeros)
  const lfg_u32x4 rs_a = lfg_make_buffer(A, (unsigned)p.n[{g.flags_at + 1}]), rs_b = lfg_make_buffer(B, (unsigned)p.n[{g.flags_at + 2}]);
  unsigned offa[kPA], offb[kPB];
  int rooma[kPA], roomb[kPB];
#pragma unroll
  for (int j = 0; j < kPA; ++j) {{
    const int idx = tid + kNT * j;
    const long long oa = m0 + LfgPiece<a_rows, kBM>::outer(idx);
    const int ka = LfgPiece<a_rows, kBM>::k(idx);
    offa[j] = (unsigned)(2 * (oa * S{sam} + ka * S{sak}));
    rooma[j] = oa < M ? (int)min(K - ka, (long long)0x7fffffff) : 0;
  }}
#pragma unroll
  for (int j = 0; j < kPB; ++j) {{
    const int idx = tid + kNT * j;
    const long long ob = n0 + LfgPiece<b_rows, kBN>::outer(idx);
    const int kb = LfgPiece<b_rows, kBN>::k(idx);
    offb[j] = (unsigned)(2 * (ob * S{sbn} + kb * S{sbk}));
    roomb[j] = ob < Nn ? (int)min(K - kb, (long long)0x7fffffff) : 0;
  }}
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) const void*)lds;
  const unsigned stepa = (unsigned)(2 * {BK} * S{sak}), stepb = (unsigned)(2 * {BK} * S{sbk});
  // tile of k step `st` into buffer `buf`
  auto fetch = [&](int st, int buf) {{
    const int k0 = st * {BK};
#pragma unroll
    for (int j = 0; j < kPA; ++j)
      lfg_dma(rs_a, k0 < rooma[j] ? offa[j] + (unsigned)st * stepa : 0xffffffffu,
              lds0 + 2u * (unsigned)(kTileA * buf) + 1024u * (unsigned)(wave + kWaves * j));
#pragma unroll
    for (int j = 0; j < kPB; ++j)
      lfg_dma(rs_b, k0 < roomb[j] ? offb[j] + (unsigned)st * stepb : 0xffffffffu,
              lds0 + 2u * (unsigned)(2 * kTileA + kTileB * buf) + 1024u * (unsigned)(wave + kWaves * j));
  }};
  lfg_f32x16 acc[kMB][kNB];
#pragma unroll
  for (int x = 0; x < kMB; ++x)
#pragma unroll
    for (int y = 0; y < kNB; ++y)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[x][y][i] = 0.0f;
  fetch(0, 0);
  asm volatile("s_waitcnt vmcnt(0)\\n\\ts_barrier" ::: "memory");
  const int steps = (int)((K + {BK - 1}) / {BK});
  for (int st = 0; st < steps; ++st) {{
    const int cur = st & 1;
    if (st + 1 < steps) fetch(st + 1, cur ^ 1);
    const unsigned short* ta = &lds[kTileA * cur];
    const unsigned short* tb = &lds[2 * kTileA + kTileB * cur];
#pragma unroll
    for (int ks = 0; ks < {BK // 16}; ++ks) {{
      lfg_u32x4 fm[kMB], fn[kNB];
#pragma unroll
      for (int x = 0; x < kMB; ++x) fm[x] = lfg_operand<a_rows, kBM>(ta, kMB * wm + x, ks, lane);       // lane = m
#pragma unroll
      for (int y = 0; y < kNB; ++y) fn[y] = lfg_operand<b_rows, kBN>(tb, kNB * wn + y, ks, lane);       // lane = n: the A operand of C^T = B^T A^T
#pragma unroll
      for (int x = 0; x < kMB; ++x)
#pragma unroll
        for (int y = 0; y < kNB; ++y) acc[x][y] = lfg_mfma(({elem})0.0f, fn[y], fm[x], acc[x][y]);
    }}
    // this wave's loads of the next tile have landed, every wave is done reading this one
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\\n\\ts_barrier" ::: "memory");
  }}
  // acc[x][y][i] = C[m][n], m = 32 * (kMB * wm + x) + lane % 32, n = 32 * (kNB * wn + y) + 8 * (i / 4) + 4 * (lane / 32) + i % 4.
  // Two n blocks at a time through the wave's own part of LDS ([32 * kMB m][64 n] fp32, 16-byte pieces permuted by the
  // row): afterwards a lane holds four consecutive n of one m and 16 neighbouring lanes cover 64 consecutive n.
  float* mine = reinterpret_cast<float*>(lds) + wave * (kMB * 2048);
  auto epilogue = [&](float accv, long long i{km}, long long i{kn}) -> float {{ return {val}; }};
  auto out_at = [&](long long i{km}, long long i{kn}) -> long long {{ return {ooff}; }};
#pragma unroll
  for (int pass = 0; pass < kNB / 2; ++pass) {{
    if (pass) __syncthreads();
    {{
      const int l32 = lane & 31, gg = lane >> 5;
#pragma unroll
      for (int x = 0; x < kMB; ++x)
#pragma unroll
        for (int y = 0; y < 2; ++y)
#pragma unroll
          for (int q = 0; q < 4; ++q) {{
            const int row = 32 * x + l32, piece = 8 * y + 2 * q + gg;
            const lfg_f32x16& c = acc[x][2 * pass + y];
            *reinterpret_cast<lfg_u32x4*>(&mine[row * 64 + 4 * (piece ^ (row & 15))]) =
                __builtin_bit_cast(lfg_u32x4, lfg_f32x4{{c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]}});
          }}
    }}
    __syncthreads();
#pragma unroll 4
    for (int j = 0; j < 8 * kMB; ++j) {{
      const int row = 4 * j + (lane >> 4), piece = lane & 15;
      const lfg_f32x4 c = __builtin_bit_cast(lfg_f32x4, *reinterpret_cast<const lfg_u32x4*>(&mine[row * 64 + 4 * (piece ^ (row & 15))]));
      const long long m = m0 + 32 * kMB * wm + row, n = n0 + 32 * kNB * wn + 64 * pass + 4 * piece;
      if (m < M && n < Nn) {{
        float r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = epilogue(c[e], m, n + e < Nn ? n + e : n);
        if (row_stores && n + 3 < Nn) {{
          lfg_st4<{out_t}>(p.ptr[{o}], out_at(m, n), r);
        }} else {{
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < Nn) lfg_st<{out_t}>(p.ptr[{o}], out_at(m, n + e), r[e]);
        }}
      }}
    }}
  }}
}}
"""
        return Kernel(self.name, src, self.bufs, self.atoms, self.strides, self.scalars, par)
