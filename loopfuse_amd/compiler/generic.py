"""Run-time side of the generic lowering: compile the emitted kernels with hipRTC through the C
ABI, solve the run-time extents of the atoms from the argument shapes, allocate temporaries and
launch (the counterpart of the reference's generated ``launch_kernel_0``,
``loopfuse/codegen.py:215-298``)."""
from __future__ import annotations

import ctypes
import math
from typing import Sequence

import torch

from . import build, emit, emit_gemm, ir, passes
from .emit import NotLowerable


# One thread per output element with sequential inner loops is meant for the small graphs around
# an attention (epilogues, table look-ups, normalisations).  Element-wise nests move their bytes once,
# like the ATen ops they replace, at any size; a nest with a reduction or a contraction runs its inner
# loop per thread with strided reads, which rocBLAS beats by orders of magnitude on anything large:
# beyond this many inner-loop steps per call (all reducing nests together; 512 x 512 x 512 multiply-adds)
# the graph is left to the captured ATen ops.
MAX_SCALAR_WORK = 1 << 27

counters = {"mfma": 0, "plain": 0, "wave": 0}      # kernel launches by kind (tests read them; "wave" launches count as "plain" too)
WAVE_REDUCE_MIN = 128       # reduced elements per output from which a reduction takes the one-wave-per-output kernel


def _half_operand(nest: ir.Nest) -> bool:
    """A pointwise nest without a contraction of its own whose value the traced graph holds in bf16 / fp16."""
    val = getattr(getattr(nest.stmt.buf, "node", None), "meta", {}).get("val", None)
    return (isinstance(nest.stmt, ir.Assign) and not nest.red and getattr(val, "dtype", None) in (torch.bfloat16, torch.float16)
            and not any(isinstance(x, ir.Dot) for x in ir.walk(nest.stmt.value)))


class GenericProgram:
    def __init__(self, gm: torch.fx.GraphModule):
        try:
            p = build.parse(gm)
            # a half-precision tensor that only contractions read stays a tensor (stored as the graph stores it):
            # the contraction then has two plain operands and can run on MFMA
            nests = passes.fuse(p.nests, p.out.buf, keep_contractions=True, keep_operands=True, operand_pred=_half_operand)
        except (build.Unsupported, passes.PassError, ValueError) as e:
            raise NotLowerable(str(e)) from e
        if any(isinstance(n.stmt, ir.Rescaled) for n in nests):
            raise NotLowerable("attention nest")
        self.parsed, self.nests = p, nests
        out_val = next(n for n in gm.graph.nodes if n.op == "output").args[0]
        out_val = out_val[0] if isinstance(out_val, (tuple, list)) else out_val
        self.out_dtype = out_val.meta["val"].dtype
        # the graph's result must be the last nest's buffer, its dims regrouped in place
        flat_buf = [a for d in p.out.buf.dims for a in ir.leaves(d) if a.hint != 1]
        flat_view = [a for d in p.out.dims for a in ir.leaves(d) if a.hint != 1]
        if len(flat_buf) != len(flat_view) or any(x is not y for x, y in zip(flat_buf, flat_view)):
            raise NotLowerable("the result is a permuted or broadcast view of what the last nest writes")
        self.dtypes = {b.name: emit._DT.get(getattr(torch, b.dtype, None), None) for b in p.inputs}
        if any(v is None for v in self.dtypes.values()):
            raise NotLowerable("an input dtype the emitted kernels do not read")
        # temporaries are fp32, except one that another nest reads as a direct operand of a contraction and that
        # the traced graph holds in bf16 / fp16: it is stored as the graph stores it (the rounding eager does), so
        # that the contraction can take it on the MFMA path
        operand_of_dot = set()
        for n in nests:
            for e in ir.walk(n.stmt.value):
                if isinstance(e, ir.Dot):
                    operand_of_dot.update(x.buf.name for x in (e.a, e.b) if isinstance(x, ir.Read))
        self.torch_dtypes: dict = {}
        for n in nests:
            b = n.writes()
            traced = getattr(getattr(b, "node", None), "meta", {}).get("val", None)
            tdt = getattr(traced, "dtype", None)
            if b is not p.out.buf and b.name in operand_of_dot and tdt in (torch.bfloat16, torch.float16):
                self.dtypes.setdefault(b.name, emit._DT[tdt])
                self.torch_dtypes[b.name] = tdt
            self.dtypes.setdefault(b.name, 0)
        self.dtypes[p.out.buf.name] = emit._DT.get(self.out_dtype, 0)
        self.kernels = [emit.Emitter(n, self.dtypes, f"lf_gen_{i}").emit() for i, n in enumerate(nests)]
        self.source = emit.PRELUDE + "\n".join(k.source for k in self.kernels)
        # reductions also get a one-wave-per-output form (GPU only), taken when the reduced extent is long
        self.wave: dict = {}
        for i, n in enumerate(nests):
            if isinstance(n.stmt, ir.Accum) and [a for a in ir.leaves(n.red) if a.hint != 1]:
                try:
                    self.wave[i] = emit.Emitter(n, self.dtypes, f"lf_gen_{i}_wave").emit(wave_reduce=True)
                except NotLowerable:
                    pass
        self.gpu_source = self.source + "\n".join(k.source for k in self.wave.values())
        # contractions of bf16 / fp16 operands also get an MFMA kernel with the nest's epilogue fused; the plain
        # kernel of the same nest serves the calls whose strides or extents it cannot take
        self.gemm: dict = {}
        for i, n in enumerate(nests):
            info = emit_gemm.match(n, self.dtypes)
            if info is not None:
                try:
                    self.gemm[i] = (emit_gemm.GemmEmitter(n, self.dtypes, f"lf_gen_{i}_mfma", info).emit(), info)
                except NotLowerable:
                    pass
        # the MFMA kernels are specialised by operand layout at compile time: one code object per layout pair,
        # built when a call first needs it
        self.gemm_source = emit.PRELUDE + emit_gemm.GEMM_PRELUDE + "\n".join(k.source for k, _ in self.gemm.values())
        self._loaded: dict = {}
        self._gemm_loaded: dict = {}
        self._plans: dict = {}              # call signature -> recorded launches (see run)
        self.last_mfma_flop = 0.0           # flop the MFMA kernels of the last run() were launched for

    @property
    def code(self) -> str:
        return self.gpu_source + (self.gemm_source if self.gemm else "")

    def _module(self):
        from .. import lowering, runtime
        dev = torch.cuda.current_device()
        if dev not in self._loaded:
            code, _, _ = runtime.compile_source(self.gpu_source, "lf_generic", list(lowering.COMMON_OPTS))
            mod = runtime.Module(code)
            self._loaded[dev] = ([mod.kernel(k.name) for k in self.kernels], {i: mod.kernel(k.name) for i, k in self.wave.items()})
        return self._loaded[dev]

    def _gemm_kernel(self, ni: int, layouts, shape: str):
        from .. import lowering, runtime
        key = (torch.cuda.current_device(), tuple(layouts), shape)
        if key not in self._gemm_loaded:
            opts = list(lowering.COMMON_OPTS) + [f"-DLFG_A_ROWS={layouts[0]}", f"-DLFG_B_ROWS={layouts[1]}"] + \
                emit_gemm.tile_options(shape)
            code, _, _ = runtime.compile_source(self.gemm_source, "lf_generic_mfma", opts)
            mod = runtime.Module(code)
            self._gemm_loaded[key] = {i: mod.kernel(k.name) for i, (k, _) in self.gemm.items()}
        return self._gemm_loaded[key][ni]

    @staticmethod
    def _gemm_shape(info, ext: dict) -> str:
        """256 x 256 tiles when they fill most of the CUs, else 128 x 128."""
        import os
        forced = os.environ.get("LOOPFUSE_GEMM_TILE")
        if forced in emit_gemm.TILES:
            return forced
        bm, bn = emit_gemm.tile_extent("l")
        tiles = -(-ext[info.m.id] // bm) * -(-ext[info.n.id] // bn) * math.prod(ext[a.id] for a in info.batch)
        return "l" if tiles >= 192 and ext[info.m.id] >= bm and ext[info.n.id] >= bn else "s"

    @staticmethod
    def _gemm_layouts(info, bufs: dict, ext: dict):
        """(A is k-contiguous, B is k-contiguous) when the MFMA kernel can read both operands of this call with
        16-byte pieces, else None."""
        M, N, K = ext[info.m.id], ext[info.n.id], ext[info.k.id]
        flags = []
        for buf, (d_outer, d_k), batch_dims, outer in ((info.a_buf, info.a_dims, info.a_batch_dims, M),
                                                      (info.b_buf, info.b_dims, info.b_batch_dims, N)):
            t = bufs[buf.name]
            if t.data_ptr() % 16 or any(t.stride(d) % 8 for d in batch_dims if t.shape[d] > 1):
                return None
            s_outer, s_k = t.stride(d_outer), t.stride(d_k)
            if s_outer < 0 or s_k < 0 or 2 * ((outer + 256) * s_outer + (K + 64) * s_k) >= 1 << 32:
                return None                  # the direct loads address a batch element's operand with 32-bit byte offsets
            if (s_k == 1 or K == 1) and K % 8 == 0 and (s_outer % 8 == 0 or outer == 1):
                flags.append(1)
            elif (s_outer == 1 or outer == 1) and outer % 8 == 0 and (s_k % 8 == 0 or K == 1):
                flags.append(0)
            else:
                return None
        return flags

    def _solve(self, nest: ir.Nest, bufs: dict, known: dict, syms: dict) -> None:
        """Run-time extent of every leaf atom of ``nest`` into ``known``: each dimension of a
        buffer it reads (an argument, or a temporary an earlier nest wrote) is the product of the
        atoms that index it; atoms that index a dimension whole give values, the rest follows by
        division (fixed point).  Two atoms whose size is the same symbol of the traced graph
        (``s74``) have the same extent, whichever nest they belong to: ``syms`` carries those."""
        eqs = []
        every = [a for a in ir.leaves(nest.par) + ir.leaves(nest.red)]
        for e in ir.walk(nest.stmt.value):
            if isinstance(e, ir.Dot):
                every += ir.leaves(e.over)
        for a in every:
            if a.id not in known and a.hint != 1:
                if a.size.isdigit():
                    known[a.id] = int(a.size)
                elif a.size in syms:
                    known[a.id] = syms[a.size]
        for r in ir.reads(nest.stmt.value):
            t = bufs[r.buf.name]
            for d, atoms in enumerate(r.idx):
                if r.gather is not None and r.gather[0] == d:
                    continue
                eqs.append(([a for a in ir.leaves(atoms) if not a.broadcast], int(t.shape[d])))
            if r.gather is not None:
                tt = bufs[r.gather[1].name]
                for d, atoms in enumerate(r.gather[2]):
                    eqs.append((list(ir.leaves(atoms)), int(tt.shape[d])))
        progress = True
        while progress:
            progress = False
            for atoms, size in eqs:
                unknown = [a for a in atoms if a.id not in known and a.hint != 1]
                have = math.prod(known[a.id] for a in atoms if a.id in known)
                if len(unknown) == 1 and have and size % have == 0:
                    known[unknown[0].id] = size // have
                    syms.setdefault(unknown[0].size, size // have)
                    progress = True

    def run(self, args: Sequence, launchers=None):
        """One pass over the nests.  ``launchers`` (one callable(blocks, params) per kernel)
        replaces the HIP launch -- the CPU tests pass a host build of the same source."""
        tensors = [a for a in args if isinstance(a, torch.Tensor) and a.dim() > 0]
        if not tensors:
            raise NotLowerable("no tensor argument")
        dev = tensors[0].device
        if any(t.device != dev for t in tensors):
            raise NotLowerable("arguments on different devices")
        steps: list = []                   # what this call launches, for the next call of the same signature
        key = None
        if launchers is None:
            if dev.type != "cuda":
                raise NotLowerable("tensors are not on the GPU")
            # a call of a signature seen before repeats its launches: only pointers change
            key = tuple((tuple(a.shape), a.stride(), a.dtype, a.data_ptr() % 16, a.device.index) if isinstance(a, torch.Tensor) else a
                        for a in args)
            plan = self._plans.get(key)
            if plan is not None:
                return self._replay(plan, args, dev)
            kernels, wave_fns = self._module()
            launchers = [lambda blocks, prm, fn=fn: (fn.launch((blocks, 1, 1), (256, 1, 1), prm),
                                                     steps.append((fn, blocks, 256, prm)))[0] for fn in kernels]
            mfma = self.gemm
        else:
            mfma, wave_fns = {}, {}
        self.last_mfma_flop = 0.0
        n_mfma = n_plain = 0
        allocs: list = []                  # (steps before it, buffer name, shape, dtype)
        ext: dict = {}
        syms: dict = {name: int(args[i]) for name, i in self.parsed.sizes.items()}
        work = 0
        bufs: dict = {b.name: args[b.placeholder] for b in self.parsed.inputs}
        for ni, (nest, k, fn) in enumerate(zip(self.nests, self.kernels, launchers)):
            out = nest.writes()
            self._solve(nest, bufs, ext, syms)
            try:
                shape = [math.prod(1 if a.hint == 1 else ext[a.id] for a in ir.leaves(d)) for d in out.dims]
            except KeyError as e:
                raise NotLowerable("an extent could not be derived from the argument shapes") from e
            dt = self.out_dtype if out is self.parsed.out.buf else self.torch_dtypes.get(out.name, torch.float32)
            bufs[out.name] = torch.empty(shape, dtype=dt, device=dev)
            allocs.append((len(steps), out.name, tuple(shape), dt))
            if ni in mfma:
                try:
                    layouts = self._gemm_layouts(self.gemm[ni][1], bufs, ext)
                except KeyError:
                    layouts = None
                if layouts is not None and all(ext.get(a.id, 0) > 0 for a in self.gemm[ni][0].atoms):
                    shape = self._gemm_shape(self.gemm[ni][1], ext)
                    steps.append(self._launch_gemm(self._gemm_kernel(ni, layouts, shape), shape, *self.gemm[ni], bufs, ext, args)
                                 + ([b.name for b in self.gemm[ni][0].bufs],))
                    counters["mfma"] += 1
                    n_mfma += 1
                    info = self.gemm[ni][1]
                    self.last_mfma_flop += 2.0 * math.prod(ext[a.id] for a in [info.m, info.n, info.k] + list(info.batch))
                    continue
            if ni in wave_fns:
                # a long reduction: one wave per output element (the plain kernel's thread would walk it alone)
                wk = self.wave[ni]
                reduced = math.prod(ext[a.id] for a in ir.leaves(nest.red) if a.hint != 1)
                if reduced >= WAVE_REDUCE_MIN:
                    k, fn = wk, (lambda blocks, prm, f=wave_fns[ni]: (f.launch((blocks, 1, 1), (256, 1, 1), prm),
                                                                     steps.append((f, blocks, 256, prm)))[0])
            prm = emit.GenParams()
            for i, b in enumerate(k.bufs):
                prm.ptr[i] = bufs[b.name].data_ptr()
            for i, a in enumerate(k.atoms):
                prm.n[i] = ext[a.id]
            for i, (b, d) in enumerate(k.strides):
                prm.n[len(k.atoms) + i] = bufs[b.name].stride(d)
            for i, s in enumerate(k.scalars):
                prm.f[i] = float(s.fn(args))
            total = math.prod(ext[a.id] for a in k.par)
            inner = math.prod(ext[a.id] for a in k.atoms if not any(a is x for x in k.par))
            if inner > 1:
                work += total * inner // k.lanes_per_output
            if work > MAX_SCALAR_WORK:
                raise NotLowerable("more scalar work than the plain kernels are meant for")
            if total:
                per_block = 256 // k.lanes_per_output
                if (total + per_block - 1) // per_block >= 1 << 31:
                    raise NotLowerable("more output elements than one grid dimension holds")
                fn((total + per_block - 1) // per_block, prm)
                if key is not None:
                    steps[-1] = steps[-1] + ([b.name for b in k.bufs],)
                counters["plain"] += 1
                counters["wave"] += int(k.lanes_per_output == 64)
                n_plain += 1
        res = bufs[self.parsed.out.buf.name]
        view = [math.prod(1 if a.hint == 1 else ext[a.id] for a in ir.leaves(d)) for d in self.parsed.out.dims]
        if key is not None:
            if len(self._plans) >= 64:
                self._plans.clear()
            self._plans[key] = (steps, allocs, self.parsed.out.buf.name, view, n_mfma, n_plain, self.last_mfma_flop)
        return res.view(view)

    def _replay(self, plan, args, dev):
        steps, allocs, out_name, view, n_mfma, n_plain, flop = plan
        bufs: dict = {b.name: args[b.placeholder] for b in self.parsed.inputs}
        at = 0
        for i, (fn, blocks, threads, prm, names) in enumerate(steps):
            while at < len(allocs) and allocs[at][0] <= i:
                bufs[allocs[at][1]] = torch.empty(allocs[at][2], dtype=allocs[at][3], device=dev)
                at += 1
            for slot, name in enumerate(names):
                prm.ptr[slot] = bufs[name].data_ptr()
            fn.launch((blocks, 1, 1), (threads, 1, 1), prm)
        while at < len(allocs):
            bufs[allocs[at][1]] = torch.empty(allocs[at][2], dtype=allocs[at][3], device=dev)
            at += 1
        counters["mfma"] += n_mfma
        counters["plain"] += n_plain
        self.last_mfma_flop = flop
        return bufs[out_name].view(view)

    @staticmethod
    def _launch_gemm(fn, shape: str, k, info, bufs: dict, ext: dict, args) -> tuple:
        prm = emit.GenParams()
        for i, b in enumerate(k.bufs):
            prm.ptr[i] = bufs[b.name].data_ptr()
        for i, a in enumerate(k.atoms):
            prm.n[i] = ext[a.id]
        for i, (b, d) in enumerate(k.strides):
            prm.n[len(k.atoms) + i] = bufs[b.name].stride(d)
        # rows of the output contiguous along n, every row start and the extent a multiple of four elements:
        # results leave four at a time
        o = bufs[info.out_buf.name]
        prm.n[info.flags_at] = int(info.out_n_dim >= 0 and o.stride(info.out_n_dim) == 1 and ext[info.n.id] % 4 == 0
                                   and o.data_ptr() % 16 == 0
                                   and all(st % 4 == 0 for d, st in enumerate(o.stride()) if d != info.out_n_dim and o.shape[d] > 1))
        for j, (buf, (d_outer, d_k), outer) in enumerate(((info.a_buf, info.a_dims, ext[info.m.id]),
                                                          (info.b_buf, info.b_dims, ext[info.n.id]))):
            t = bufs[buf.name]
            prm.n[info.flags_at + 1 + j] = 2 * ((outer - 1) * t.stride(d_outer) + (ext[info.k.id] - 1) * t.stride(d_k) + 1)
        for i, s in enumerate(k.scalars):
            prm.f[i] = float(s.fn(args))
        bm, bn = emit_gemm.tile_extent(shape)
        tiles = -(-ext[info.m.id] // bm) * -(-ext[info.n.id] // bn) * math.prod(ext[a.id] for a in info.batch)
        blocks = 8 * -(-tiles // 8)
        if blocks >= 1 << 31:
            raise NotLowerable("more tiles than one grid dimension holds")
        wm, wn, _, _ = emit_gemm.TILES[shape]
        fn.launch((blocks, 1, 1), (64 * wm * wn, 1, 1), prm)
        return fn, blocks, 64 * wm * wn, prm
