"""Loop-nest front end: ATen graph -> per-op loop nests -> fusion, online-softmax and
block-skip passes -> attention plan.

The counterpart of the reference's compiler layers (``loopfuse/ir.py``, ``loopfuse/optimize.py``,
``loopfuse/compiler/passes/{fuse,factor_acc,skip_loop_iterations}.py``), written for what
the MI355X lowering consumes: instead of printing the fused nest as Triton source, the
nest is read off into the parameters of the hand-written HIP kernels (``derive.py``).

    build.parse(gm)        one loop nest per ATen op, tensors as mixed-radix "atom" dims
    passes.fuse            producer/consumer inlining of pointwise nests
    passes.online_softmax  the three KV reductions (max, sum, P V) become one rescaled pass
    passes.block_skip      interval analysis of the mask clauses over KV tiles -> loop bounds
    derive.attention       the fused nest -> mask / window / scale / softcap / paging / GQA group
"""
from . import build, derive, ir, passes  # noqa: F401
from .pipeline import compile_graph, NotDerivable  # noqa: F401
