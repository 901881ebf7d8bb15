"""``loopfuse_backend`` — the ``torch.compile`` backend — and its graph capture.

Same public surface as the reference (``loopfuse/torch_backend/interface.py:
77-86, 164-170, 640-644``):

    loopfuse_backend(gm, sample_inputs, mode="max-autotune", **kwargs)
        -> aot_module_simplified(gm, sample_inputs, fw_compiler=loopfuse_compiler)
    loopfuse_compiler(gm, sample_inputs, input_names=None, symint_names=None, mode=None)
        -> callable taking the flat placeholder list (tensors and SymInts as ints)

and the same environment switches ``DEBUG``, ``CODEGEN_ONLY`` and
``USE_HARDCODE_KERNEL`` (``interface.py:23-29``).

Where the reference parses the ATen graph into per-op loop nests, fuses them and
prints Triton (``interface.py:387-400``, ``optimize.py:34-60``,
``codegen.py:100-126``), this front end recognises the fused result directly: it
abstract-interprets the graph (``capture.py``), finds every sub-graph of the form
``softmax(mask(mods(Q K^T) [+ bias])) V [+ bias]`` and replaces it by one call that
``lowering.attention`` runs on the hand-written HIP kernels; the rest of the graph
keeps running as it is.

Graphs without such a sub-graph, and calls on CPU tensors, run the captured
graph unchanged (the reference raises ``ValueError``/``NotImplementedError``
there, ``interface.py:157-161``).  Set ``LOOPFUSE_STRICT=1`` to raise instead;
``stats`` counts which route each call took so tests can insist on the fused one.
"""
from __future__ import annotations

import logging
import os
from functools import partial
from typing import Callable

import torch
from torch._functorch.aot_autograd import aot_module_simplified, make_boxed_func

from .. import compiler, lowering
from . import capture

log = logging.getLogger("loopfuse_amd")

DEBUG = os.environ.get("DEBUG", "0") == "1"
CODEGEN_ONLY = os.environ.get("CODEGEN_ONLY", "0") == "1"
USE_HARDCODE_KERNEL = os.environ.get("USE_HARDCODE_KERNEL", "0") == "1"

# route taken by compiled callables since import: "fused" = HIP kernel launched,
# "eager_graph" = graph not recognised, "eager_runtime" = recognised but the call's
# tensors could not be served (CPU tensors, dtype, alignment ...)
# "eager_training" = graph traced with gradients enabled (forward or backward half)
# "refused_signatures" = argument layouts latched as not servable (see optimized_fn)
stats = {"fused": 0, "eager_graph": 0, "eager_runtime": 0, "eager_training": 0, "compiled_graphs": 0, "matched_graphs": 0,
         "refused_signatures": 0, "derived_graphs": 0, "generic_graphs": 0, "fused_generic": 0, "tuned_captured": 0,
         "training_graphs": 0, "fused_training": 0, "match_errors": 0}


def _frontend() -> str:
    """Which front end turns the graph into fused calls: "ir" (default) = the loop-nest front end
    (loopfuse_amd/compiler: per-op nests, fusion, online-softmax and block-skip passes, plan read
    off the fused nest), with the sub-graph matcher of capture.py as fallback for graphs it does not
    cover (an attention inside a larger graph, several attentions, torch's fused attention ops, mask
    tensors); "match" = the matcher alone; "check" = the matcher, cross-checked against the loop-nest
    front end wherever that derives a plan."""
    return os.environ.get("LOOPFUSE_FRONTEND", "ir")


def match_from_nests(gm: torch.fx.GraphModule, comp: "compiler.pipeline.Compiled") -> capture.AttentionMatch:
    """The attention the loop-nest front end derived, in the form the fused call takes."""
    att = comp.attention
    placeholders = [n for n in gm.graph.nodes if n.op == "placeholder"]
    out_node = next(n for n in gm.graph.nodes if n.op == "output").args[0]
    out_node = out_node[0] if isinstance(out_node, (tuple, list)) else out_node
    inputs = list(placeholders)

    def index_of(o) -> int:
        """Position of an operand among the fused call's inputs: a placeholder, or a node of the graph
        that keeps running (an operand computed from the inputs, such as Q + q_bias)."""
        if o.node is None:
            return o.placeholder
        if o.node not in inputs:
            inputs.append(o.node)
        return inputs.index(o.node)

    def operand(o):
        return None if o is None else capture.Operand(index_of(o), tuple(o.perm), o.paged, o.table, o.group)

    def added(bl):
        return None if bl is None else capture.BiasOperand(index_of(bl), tuple(bl.dims))

    def factor(f):
        kind, x = f
        x = ("fn", x) if callable(x) else float(x)
        return ("recip", x) if kind == "div" else x

    return capture.AttentionMatch(out_node=out_node, inputs=inputs, q=operand(att.q), k=operand(att.k),
                                  v=operand(att.v), factors=[factor(f) for f in att.pre],
                                  post_factors=[factor(f) for f in att.post], has_tanh=att.has_tanh,
                                  mask=att.mask, window=("fn", att.window) if callable(att.window) else att.window,
                                  out_rank=4, bias=added(att.bias), out_bias=added(att.out_bias),
                                  q2=operand(att.q2), k2=operand(att.k2),
                                  denom_add=tuple(factor(f) for f in att.denom_add), base2=att.base2,
                                  late_factors=tuple(factor(f) for f in att.late))


def _differences(m: capture.AttentionMatch, d: capture.AttentionMatch) -> str:
    """What two descriptions of one attention disagree on ("" = nothing): mask, window, cap, the number
    and the static values of the factors, operand sources / layouts / paging / head grouping, added
    tensors, second product, denominator terms and exponent base.  (LOOPFUSE_FRONTEND=check.)"""
    def static(fs):
        """(product of the factors known at trace time, number of the others)"""
        known = [float(f) for f in fs if isinstance(f, (int, float))]
        rec = [1.0 / float(f[1]) for f in fs if isinstance(f, tuple) and f[0] == "recip" and isinstance(f[1], (int, float))]
        r = 1.0
        for x in known + rec:
            r *= x
        return round(r, 9), len(fs) - len(known) - len(rec)

    def op(o):
        return None if o is None else (o.index, tuple(o.perm), o.paged, o.group)

    def table(match, o):
        return None if o is None or not o.paged else match.inputs[o.table_index].name

    def src(match, o):
        return None if o is None else match.inputs[o.index].name

    def added(b):
        return None if b is None else (tuple(b.dims), b.keep)

    checks = [
        ("mask", m.mask, d.mask), ("cap", m.has_tanh, d.has_tanh),
        ("factors before the cap", static(m.factors), static(d.factors)),
        ("factors behind the cap", static(m.post_factors), static(d.post_factors)),
        ("denominator terms", sorted(float(t) for t in m.denom_add if isinstance(t, (int, float))),
         sorted(float(t) for t in d.denom_add if isinstance(t, (int, float)))), ("exponent base", m.base2, d.base2),
        ("score bias", added(m.bias), added(d.bias)), ("output bias", added(m.out_bias), added(d.out_bias)),
    ]
    if m.mask == "sliding" and isinstance(m.window, int) and isinstance(d.window, int):
        checks.append(("window", m.window, d.window))
    for name in ("q", "k", "v", "q2", "k2"):
        om, od = getattr(m, name), getattr(d, name)
        checks.append((f"{name} source", src(m, om), src(d, od)))
        checks.append((f"{name} layout", op(om) and op(om)[1:], op(od) and op(od)[1:]))
        checks.append((f"{name} page table", table(m, om), table(d, od)))
    for name in ("bias", "out_bias"):
        bm_, bd = getattr(m, name), getattr(d, name)
        checks.append((f"{name} source", bm_ and m.inputs[bm_.index].name, bd and d.inputs[bd.index].name))
    return "; ".join(f"{what}: {x!r} vs {y!r}" for what, x, y in checks if x != y)


def _strict() -> bool:
    return os.environ.get("LOOPFUSE_STRICT", "0") == "1"


def get_input_names(gm: torch.fx.GraphModule) -> list[str]:
    """Placeholder names in order (reference ``interface.py:49-56``)."""
    return [n.name for n in gm.graph.nodes if n.op == "placeholder"]


def loopfuse_backend(gm: torch.fx.GraphModule, sample_inputs, mode="max-autotune", **kwargs):
    """``torch.compile`` backend entry point (reference ``interface.py:77-86``).

    ``mode="max-autotune"`` (the default, as in the reference) makes the first call of
    each shape class time the candidate kernel variants / work splits and keep the
    fastest (``lowering.tuned_attention``); ``mode=None`` uses the fixed heuristics.
    """
    if mode:
        kwargs["mode"] = mode
    if torch.is_grad_enabled() and (any(isinstance(t, torch.Tensor) and t.requires_grad for t in sample_inputs)
                                    or any(t.requires_grad for t in gm.parameters())):
        # AOTAutograd is about to trace a forward + backward pair: the forward graph must
        # hand the probabilities to the backward graph, which a fused forward never forms
        global _warned_training
        fused = _training_graph(gm, sample_inputs)
        if fused is not None:
            return fused
        if _strict():
            raise NotImplementedError("loopfuse_amd: this graph is traced with gradients enabled and the kernels are "
                                      "forward-only for it (its attention is not one the backward kernels serve, or "
                                      "its tensors are not on the GPU)")
        if not _warned_training:
            _warned_training = True
            log.warning("loopfuse_amd: graph traced with gradients enabled (an input requires grad) and its attention "
                        "is not one the backward kernels serve, so this graph runs unfused.  Wrap inference in "
                        "torch.no_grad().")
        return aot_module_simplified(gm, sample_inputs, fw_compiler=_unfused_compiler)
    compiler = partial(loopfuse_compiler, input_names=get_input_names(gm), **kwargs)
    return aot_module_simplified(gm, sample_inputs, fw_compiler=compiler)


_warned_training = False


def _training_graph(gm: torch.fx.GraphModule, sample_inputs):
    """A graph traced with gradients enabled: trace its forward to ATen once (for the matcher only),
    and when every attention found is one the backward kernels serve, hand AOTAutograd that graph
    with the attentions replaced by ``training.fused_call_train`` -- differentiable views around
    the custom op ``loopfuse_amd::attention_fwd``, whose registered formula is the HIP backward.
    None when the graph has to run unfused.  The forward trace bakes the traced sizes into the view
    ops it keeps, so under dynamic shapes only a graph that is nothing but its attentions is taken."""
    from torch.fx.experimental.proxy_tensor import make_fx

    from . import training

    if os.environ.get("LOOPFUSE_TRAINING", "1") != "1":
        return None
    if not all(t.is_cuda for t in sample_inputs if isinstance(t, torch.Tensor)):
        return None                                          # the kernels run on the GPU only: CPU graphs stay unfused
    try:
        with torch.no_grad():
            aten_gm = make_fx(gm, tracing_mode="real", _allow_non_fake_inputs=True)(*sample_inputs)
        matches = capture.match_attention(aten_gm)
    except capture.NoMatch as e:
        log.info("training graph: no attention found (%s)", e)
        return None
    except Exception as e:                                   # tracing a user graph a second way may fail in ways of its own
        log.info("training graph: forward trace for the matcher failed (%s: %s)", type(e).__name__, e)
        return None
    if not matches:
        return None
    for m in matches:
        vals = [n.meta.get("val") for n in m.inputs]
        why = training.trainable(m, lambda i: vals[i])
        if why:
            if _strict():
                raise NotImplementedError(f"loopfuse_amd: no backward kernel for this attention ({why})")
            log.info("training graph: attention runs unfused (%s)", why)
            return None
    rewritten = rewrite_graph(aten_gm, matches, call=training.fused_call_train)
    dynamic = any(isinstance(a, torch.SymInt) for a in sample_inputs)
    others = [n for n in rewritten.graph.nodes if n.op == "call_function" and n.target is not training.fused_call_train]
    if dynamic and others:
        log.info("training graph: other operations beside the attention under dynamic shapes; running unfused")
        return None
    stats["training_graphs"] += 1
    if DEBUG:
        print("---- loopfuse_amd: graph traced for training, attentions fused ----")
        for m in matches:
            print(m.describe())
        print(rewritten.code)
    return aot_module_simplified(rewritten, sample_inputs, fw_compiler=_training_compiler, bw_compiler=_training_compiler)


def _training_compiler(gm: torch.fx.GraphModule, sample_inputs) -> Callable:
    """fw_compiler / bw_compiler of a fused training graph: the graphs hold the custom ops
    (``loopfuse_amd::attention_fwd`` / ``attention_bwd``) and run as they are."""
    stats["compiled_graphs"] += 1

    def run(*args):
        stats["fused_training"] += 1
        return gm(*args)

    return make_boxed_func(run)


def _unfused_compiler(gm: torch.fx.GraphModule, sample_inputs) -> Callable:
    """fw_compiler / bw_compiler of graphs traced for training: they run as captured."""
    stats["compiled_graphs"] += 1

    def eager_fn(*args):
        stats["eager_training"] += 1
        return gm(*args)

    return make_boxed_func(eager_fn)


_codegen_sink: list | None = None     # CODEGEN_ONLY: compiled specialisations are collected here
last_matches: list = []               # attention sub-graphs of the most recently compiled graph (debugging, tests)


def _fused_call(match, *vals):
    """Stand-in for one attention sub-graph inside a rewritten graph; ``match`` is an attribute
    of the rewritten graph module, so it lives exactly as long as that compiled graph does."""
    if _codegen_sink is not None:
        _codegen_sink.extend(lowering.compile_spec(s) for s in match.kernel_specs_for(vals))
        q = vals[match.q.index]
        return match.empty_out(vals, q.dtype, q.device)
    return match.run(vals)


def rewrite_graph(gm: torch.fx.GraphModule, matches: list, call=None) -> torch.fx.GraphModule:
    """A copy of ``gm`` in which every matched attention output is produced by one
    ``_fused_call`` node (or ``call``); what only fed the unfused chain is dropped."""
    call = call or _fused_call
    new_graph = torch.fx.Graph()
    val_map: dict = {}
    out = new_graph.graph_copy(gm.graph, val_map)
    new_graph.output(out)
    last_matches[:] = matches
    names = []
    for i, m in enumerate(matches):
        name = f"_lf_match_{i}"
        setattr(gm, name, m)          # GraphModule() below copies the attributes its get_attr nodes name
        names.append(name)
        old = val_map[m.out_node]
        with new_graph.inserting_after(old):
            attr = new_graph.get_attr(name)
        with new_graph.inserting_after(attr):
            node = new_graph.call_function(call, (attr, *[val_map[n] for n in m.inputs]))
        old.replace_all_uses_with(node)
    new_graph.eliminate_dead_code()
    try:
        fused = torch.fx.GraphModule(gm, new_graph)
    finally:
        for name in names:
            delattr(gm, name)
    fused.graph.lint()
    return fused


# A graph whose contractions run on the generated MFMA kernels competes with the captured graph's library
# matmuls: under "max-autotune" a call shape with at least this many flop in such kernels is measured both ways
# once and keeps the faster route (smaller ones are bound by launches, where one fused kernel wins)
GENERIC_TUNE_MIN_FLOP = float(1 << 32)


def _time_call(fn, reps: int = 3) -> float:
    fn()
    torch.cuda.synchronize()
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record()
    for _ in range(reps):
        fn()
    t1.record()
    torch.cuda.synchronize()
    return t0.elapsed_time(t1) / reps


def _generic_program(gm: torch.fx.GraphModule, tune: bool = False):
    """A graph without an attention in it: its loop nests, fused, as one plain HIP kernel per
    nest (loopfuse_amd/compiler/generic.py) -- what the reference's code generator does for every
    graph (loopfuse/codegen.py:100-404).  None when the nest builder does not cover the graph or
    ``LOOPFUSE_GENERIC=0``; then the graph runs as captured."""
    if os.environ.get("LOOPFUSE_GENERIC", "1") != "1":
        return None
    from ..compiler import generic
    try:
        prog = generic.GenericProgram(gm)
    except generic.NotLowerable as e:
        log.info("generic lowering does not cover this graph: %s", e)
        return None
    except Exception as e:                                    # a front-end bug must not take the graph down
        log.warning("generic lowering failed on this graph (%s: %s); it runs as captured", type(e).__name__, e)
        return None
    stats["generic_graphs"] += 1
    if DEBUG:
        print("---- loopfuse_amd: no attention in the graph; fused nests ----")
        print(compiler.ir.show(prog.nests))
        print(prog.source)
    out_node = next(n for n in gm.graph.nodes if n.op == "output")
    as_tuple = isinstance(out_node.args[0], (tuple, list))
    if CODEGEN_ONLY:
        return lambda *args: [prog] if as_tuple else prog
    refused: list = []
    routes: dict = {}          # call signature -> "generated" | "captured" (measured choice)

    def generic_fn(*args):
        key = None
        if tune and prog.gemm and not refused:
            key = tuple((tuple(a.shape), tuple(a.stride())) if isinstance(a, torch.Tensor) else a for a in args)
            if routes.get(key) == "captured":
                stats["tuned_captured"] += 1
                return gm(*args)
        if not refused:
            try:
                out = prog.run(args)
                if key is not None and key not in routes:
                    if len(routes) >= 256:
                        routes.clear()
                    routes[key] = "generated"
                    if prog.last_mfma_flop >= GENERIC_TUNE_MIN_FLOP:
                        t_gen, t_cap = _time_call(lambda: prog.run(args)), _time_call(lambda: gm(*args))
                        log.info("generated kernels %.3f ms, captured graph %.3f ms", t_gen, t_cap)
                        if t_cap < 0.95 * t_gen:
                            routes[key] = "captured"
            except generic.NotLowerable as e:
                if _strict():
                    raise
                refused.append(str(e))
                log.warning("generic kernels not applicable to this call (%s); the graph runs as captured", e)
            else:
                stats["fused_generic"] += 1
                return (out,) if as_tuple else out
        stats["eager_runtime"] += 1
        return gm(*args)

    return generic_fn


def loopfuse_compiler(gm: torch.fx.GraphModule, sample_inputs, input_names: list[str] | None = None,
                      symint_names: dict[str, str] | None = None, mode: str | None = None) -> Callable:
    """fw_compiler: ATen graph -> callable over the flat placeholder list."""
    global _codegen_sink
    stats["compiled_graphs"] += 1
    if DEBUG:
        print("---- loopfuse_amd: ATen graph ----")
        print(gm.code)
    frontend = _frontend()
    derived = None
    if frontend in ("ir", "check") or DEBUG:
        try:
            derived = compiler.compile_graph(gm)
        except compiler.NotDerivable as e:
            log.info("loop-nest front end: %s", e)
            if DEBUG:
                print(f"---- loopfuse_amd: loop-nest front end does not cover this graph ({e})")
        except Exception as e:                     # a front-end bug must not take the graph down: the matcher gets it
            log.warning("loop-nest front end failed on this graph (%s: %s); the sub-graph matcher takes it",
                        type(e).__name__, e)
            stats["match_errors"] += 1
        else:
            stats["derived_graphs"] += 1
            if DEBUG:
                print("---- loopfuse_amd: loop nests ----")
                print(derived.before)
                print("---- loopfuse_amd: after fuse / online-softmax / block-skip ----")
                print(derived.after)
                print("---- loopfuse_amd: derived:", derived.attention.describe())
    if frontend == "ir" and derived is not None:
        matches, reason = [match_from_nests(gm, derived)], ""
    else:
        try:
            matches = capture.match_attention(gm)
        except capture.NoMatch as e:
            matches = []
            reason = str(e)
        except Exception as e:                     # a front-end bug must not take the graph down: it runs as captured
            log.warning("attention matching failed on this graph (%s: %s); it runs as captured", type(e).__name__, e)
            stats["match_errors"] += 1
            matches = []
            reason = f"{type(e).__name__}: {e}"
        else:
            reason = ""
        if frontend == "check" and derived is not None:
            d = match_from_nests(gm, derived)
            why = "the matcher finds %d attentions" % len(matches) if len(matches) != 1 else _differences(matches[0], d)
            if why:
                raise AssertionError(f"loopfuse_amd: the two front ends disagree ({why}): matcher "
                                     f"{[m.describe() for m in matches]} vs loop nests {d.describe()}")
    if not matches:
        if _strict():
            raise NotImplementedError(f"loopfuse_amd: no fused-attention pattern in the graph: {reason}")
        generic = _generic_program(gm, tune=(mode == "max-autotune") and os.environ.get("LOOPFUSE_AUTOTUNE", "1") == "1")
        if generic is not None:
            return generic
        log.info("graph not recognised (%s); running it unfused", reason)
        if DEBUG:
            print(f"---- loopfuse_amd: no match ({reason}); eager graph ----")

        def eager_fn(*args):
            stats["eager_graph"] += 1
            return gm(*args)

        return eager_fn

    stats["matched_graphs"] += 1
    for m in matches:
        # the reference's "max-autotune" searches Triton tile sizes (codegen.py:355-404);
        # here it measures which kernel variant / work split serves each shape class
        m.tune = (mode == "max-autotune") and os.environ.get("LOOPFUSE_AUTOTUNE", "1") == "1"
    fused_gm = rewrite_graph(gm, matches)
    if DEBUG:
        print("---- loopfuse_amd: matched ----")
        for m in matches:
            print(m.describe())
        print(fused_gm.code)

    if CODEGEN_ONLY:
        # no launch: hand back what would be compiled, as the reference hands back
        # KernelData under CODEGEN_ONLY (interface.py:615-622)
        out_node = next(n for n in gm.graph.nodes if n.op == "output")
        n_out = len(out_node.args[0]) if isinstance(out_node.args[0], (tuple, list)) else 1

        def codegen_fn(*args):
            global _codegen_sink
            _codegen_sink = []
            try:
                fused_gm(*args)
                # one object for the whole graph (its .code joins the kernels' sources), in
                # the place of the first graph output; AOTAutograd hands it to the caller
                return [lowering.CompiledKernels(_codegen_sink)] + [None] * (n_out - 1)
            finally:
                _codegen_sink = None

        return codegen_fn

    # Calls the kernels could not serve, by what the refusal depends on: dtype, shape, strides,
    # alignment and device of every tensor argument (and the integer arguments).  A call with a
    # signature refused before goes straight to the unfused graph -- each failed attempt runs the
    # graph up to the fused call for nothing -- while a call with another signature (another
    # shape under dynamic=True, an aligned tensor after an unaligned one) is tried again.
    refused: set = set()

    def signature(args):
        return tuple((a.dtype, tuple(a.shape), a.stride(), a.data_ptr() % 16, a.device) if isinstance(a, torch.Tensor) else a
                     for a in args)

    # where the attention kernels refuse a call (fp32 operands, a head dimension they are not
    # built for), the graph's plain generated kernels serve it if they can, else the captured ops
    unfused: list = []

    def run_unfused(args):
        if not unfused:
            unfused.append(_generic_program(gm) or None)
        if unfused[0] is not None:
            return unfused[0](*args)
        stats["eager_runtime"] += 1
        return gm(*args)

    def optimized_fn(*args):
        sig = signature(args) if refused else None
        if sig is not None and sig in refused:
            return run_unfused(args)
        try:
            out = fused_gm(*args)
        except lowering.UnsupportedPlan as e:
            if _strict():
                raise
            if len(refused) >= 64:      # bounded: forget old refusals rather than grow
                refused.clear()
            refused.add(signature(args))
            stats["refused_signatures"] += 1
            log.warning("fused path not applicable to this call (%s); calls with these argument layouts run "
                        "the graph unfused", e)
            return run_unfused(args)
        stats["fused"] += 1
        return out

    return optimized_fn
