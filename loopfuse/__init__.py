"""Drop-in import path of the reference package: ``from loopfuse import loopfuse_backend``
(reference ``loopfuse/__init__.py:1-3``) resolves to the MI355X backend, and importing it
registers ``torch.ops.loopfuse.{causal_mask,sliding_mask,scan_max,paged_load}``."""
from loopfuse_amd import loopfuse_backend

__all__ = ["loopfuse_backend"]
