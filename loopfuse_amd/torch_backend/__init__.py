"""The four ``torch.ops.loopfuse.*`` operators, registered on import.

Same qualified names and schemas as the reference
(``loopfuse/torch_backend/__init__.py:4-63``), so user graphs written for the
reference trace unchanged:

    loopfuse::causal_mask(Tensor a) -> Tensor
    loopfuse::sliding_mask(Tensor a, int window_size) -> Tensor
    loopfuse::scan_max(Tensor a) -> (Tensor, Tensor)
    loopfuse::paged_load(Tensor buffer, Tensor block_table) -> Tensor

The bodies below are the operators' eager semantics (any device).  Inside a
``torch.compile(backend=loopfuse_backend)`` region they are never executed: the
graph capture recognises them and the fused HIP kernel applies the mask / the
page-table gather itself.

One deliberate difference: the reference's eager ``sliding_mask`` keeps only the
window condition ``j > i - w`` (its causal conjunct is commented out,
``torch_backend/__init__.py:21-22``) while its compiled kernel and its
benchmark baseline use ``j <= i and i - j < w`` (``torch_backend/ops.py:733-741``,
``tests/benchmark.py:236``).  Here eager and compiled agree on the causal
window.

The operators also carry autograd formulas (the reference's have none, so a graph
traced with gradients enabled fails there with "no autograd formula was
registered"): a mask passes the gradient of the kept scores and blocks the rest,
``paged_load`` adds each gathered row's gradient into its page of the pool, and
``scan_max`` sends a gradient to the element that holds the running maximum.  The
fused kernels themselves are forward-only; ``loopfuse_backend`` runs graphs that
are traced for training unfused.
"""
from __future__ import annotations

import torch

_NEG_INF = float("-inf")


def _positions(a: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Row (query) and column (key) positions of the trailing [Sq, Sk] matrix, top-left aligned."""
    rows = torch.arange(a.shape[-2], device=a.device).unsqueeze(-1)
    cols = torch.arange(a.shape[-1], device=a.device).unsqueeze(0)
    return rows, cols


@torch.library.custom_op("loopfuse::causal_mask", mutates_args=())
def causal_mask(a: torch.Tensor) -> torch.Tensor:
    i, j = _positions(a)
    return torch.where(j <= i, a, _NEG_INF)


@causal_mask.register_fake
def _(a: torch.Tensor) -> torch.Tensor:
    return torch.empty_like(a)


@torch.library.custom_op("loopfuse::sliding_mask", mutates_args=())
def sliding_mask(a: torch.Tensor, window_size: int) -> torch.Tensor:
    i, j = _positions(a)
    keep = (j <= i) & (i - j < window_size)
    return torch.where(keep, a, _NEG_INF)


@sliding_mask.register_fake
def _(a: torch.Tensor, window_size: int) -> torch.Tensor:
    return torch.empty_like(a)


@torch.library.custom_op("loopfuse::scan_max", mutates_args=())
def scan_max(a: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    running = torch.cummax(a, dim=-1).values
    return running, running[..., -1:].clone()


@scan_max.register_fake
def _(a: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    return torch.empty_like(a), a.new_empty((*a.shape[:-1], 1))


@torch.library.custom_op("loopfuse::paged_load", mutates_args=())
def paged_load(buffer: torch.Tensor, block_table: torch.Tensor) -> torch.Tensor:
    # out[*s, *t] = buffer[block_table[*s], *t]
    flat = buffer.index_select(0, block_table.reshape(-1).to(torch.int64))
    return flat.reshape(*block_table.shape, *buffer.shape[1:])


@paged_load.register_fake
def _(buffer: torch.Tensor, block_table: torch.Tensor) -> torch.Tensor:
    return buffer.new_empty((*block_table.shape, *buffer.shape[1:]))


# ---- autograd formulas --------------------------------------------------------------

def _mask_setup(ctx, inputs, output):
    ctx.window = inputs[1] if len(inputs) > 1 else None


def _mask_backward(ctx, grad):
    i, j = _positions(grad)
    keep = j <= i
    if ctx.window is not None:
        keep = keep & (i - j < ctx.window)
        return torch.where(keep, grad, 0.0), None
    return torch.where(keep, grad, 0.0)


causal_mask.register_autograd(_mask_backward, setup_context=_mask_setup)
sliding_mask.register_autograd(_mask_backward, setup_context=_mask_setup)


def _scan_max_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[0])


def _scan_max_backward(ctx, grad_running, grad_last):
    (a,) = ctx.saved_tensors
    holder = torch.cummax(a, dim=-1).indices       # position whose value is the running maximum
    grad = torch.zeros_like(a).scatter_add_(-1, holder, grad_running)
    return grad.scatter_add_(-1, holder[..., -1:], grad_last)


scan_max.register_autograd(_scan_max_backward, setup_context=_scan_max_setup)


def _paged_load_setup(ctx, inputs, output):
    ctx.save_for_backward(inputs[1])
    ctx.pool_shape = inputs[0].shape


def _paged_load_backward(ctx, grad):
    (table,) = ctx.saved_tensors
    pool_grad = grad.new_zeros(ctx.pool_shape)
    pool_grad.index_add_(0, table.reshape(-1).to(torch.int64), grad.reshape(-1, *ctx.pool_shape[1:]))
    return pool_grad, None


paged_load.register_autograd(_paged_load_backward, setup_context=_paged_load_setup)
