"""loopfuse_amd — MI355X (gfx950) backend for loopfuse-style fused attention.

    import torch
    from loopfuse_amd import loopfuse_backend

    @torch.compile(backend=loopfuse_backend, dynamic=True)
    def attn(q, k, v):
        s = q @ k.transpose(-2, -1) * q.shape[-1] ** -0.5
        return torch.softmax(torch.ops.loopfuse.causal_mask(s), dim=-1) @ v

Importing the package registers ``torch.ops.loopfuse.{causal_mask,sliding_mask,
scan_max,paged_load}`` (reference ``loopfuse/__init__.py:1-3``).
"""
from . import torch_backend  # noqa: F401  (registers the custom ops)
from .torch_backend.interface import loopfuse_backend

__all__ = ["loopfuse_backend"]
