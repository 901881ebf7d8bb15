"""Driver of the loop-nest front end (reference ``loopfuse/optimize.py:34-60`` plus the parse
and lowering steps around it, ``loopfuse/torch_backend/interface.py:387-400, 594-604``)."""
from __future__ import annotations

import dataclasses

import torch

from . import build, derive, ir, passes
from .derive import NotDerivable  # noqa: F401


@dataclasses.dataclass
class Compiled:
    parsed: build.Parser
    before: str                      # the per-op nests, printed
    after: str                       # the fused nest, printed
    attention: derive.DerivedAttention


def compile_graph(gm: torch.fx.GraphModule, bm: int = 128, bn: int = 64) -> Compiled:
    """ATen graph -> loop nests -> passes -> derived attention.  Raises ``NotDerivable`` when the
    graph is not (only) an attention these passes and the kernels cover."""
    try:
        p = build.parse(gm)
        before = ir.show(p.nests)
        nests = passes.fuse(p.nests, p.out.buf, keep_operands=True)
        nests = passes.simplify(nests)
        nests = passes.online_softmax(nests, p.out.buf)
        nests = passes.fuse(nests, p.out.buf, keep_operands=True)
        nests = passes.block_skip(nests, bm, bn)
        att = derive.attention(nests, p.inputs, p.out)
    except (build.Unsupported, passes.PassError, ValueError) as e:
        raise NotDerivable(str(e)) from e
    return Compiled(p, before, ir.show(nests), att)
