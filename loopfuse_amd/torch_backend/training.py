"""Graphs traced for training: the fused forward with a registered backward.

The reference has no backward (README "future work"): under ``torch.compile`` its kernels serve
inference graphs only.  Here a graph traced with gradients enabled keeps its attention fused when
the attention is one the backward kernels serve (dense K/V, mask none / causal / sliding, scale
only): the forward sub-graph becomes one call of the custom op ``loopfuse_amd::attention_fwd``,
which AOTAutograd differentiates through its registered formula, ``loopfuse_amd::attention_bwd``
(``lowering.attention_backward``).  The forward hands the backward ``O`` and the rows'
log-sum-exp -- ``B*H*S`` floats instead of the ``B*H*S*S`` probabilities the unfused graph saves.
"""
from __future__ import annotations

import logging

import torch

from .. import lowering

log = logging.getLogger("loopfuse_amd")

_MASK_CODE = {None: 0, "none": 0, "causal": 1, "sliding": 2}
_MASK_NAME = {0: None, 1: "causal", 2: "sliding"}
counters = {"fwd": 0, "bwd": 0, "repacked": 0}


def _rows(t: torch.Tensor) -> torch.Tensor:
    """A tensor the kernels can read: rows of D contiguous elements, 16-byte aligned."""
    if t.stride(-1) != 1 or t.data_ptr() % 16 or any(n > 1 and s % 8 for n, s in zip(t.shape[:-1], t.stride()[:-1])):
        return t.contiguous()
    return t


@torch.library.custom_op("loopfuse_amd::attention_fwd", mutates_args=())
def attention_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: int, window: int,
                  scale: float, softcap: float) -> tuple[torch.Tensor, torch.Tensor]:
    """O [B, Hq, Sq, D] and the rows' log-sum-exp [B, Hq, Sq] (float32, log2 units)."""
    if not q.is_cuda:
        raise RuntimeError("loopfuse_amd: attention_fwd needs tensors on the GPU; the HIP path has no CPU fallback")
    plan = lowering.AttnPlan(mask=_MASK_NAME[mask], window=int(window), scale=float(scale),
                             softcap=float(softcap) if softcap else None)       # 0: no cap
    lse = torch.empty(q.shape[:-1], dtype=torch.float32, device=q.device)
    counters["fwd"] += 1
    # the log-sum-exp is written by the direct-to-LDS kernel only: ask for it whatever LOOPFUSE_PREFILL says
    try:
        return lowering.attention(_rows(q), _rows(k), _rows(v), plan, lse=lse, choice={"prefill": "swp"}), lse
    except lowering.UnsupportedPlan:
        # views whose rows lie beyond the direct loads' 32-bit reach: packed copies are always within it
        counters["repacked"] += 1
        return lowering.attention(q.contiguous(), k.contiguous(), v.contiguous(), plan, lse=lse,
                                  choice={"prefill": "swp"}), lse


@attention_fwd.register_fake
def _(q, k, v, mask, window, scale, softcap):
    return q.new_empty(q.shape), q.new_empty(q.shape[:-1], dtype=torch.float32)


@torch.library.custom_op("loopfuse_amd::attention_bwd", mutates_args=())
def attention_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, lse: torch.Tensor,
                  dout: torch.Tensor, mask: int, window: int, scale: float,
                  softcap: float) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    if not q.is_cuda:
        raise RuntimeError("loopfuse_amd: attention_bwd needs tensors on the GPU; the HIP path has no CPU fallback")
    plan = lowering.AttnPlan(mask=_MASK_NAME[mask], window=int(window), scale=float(scale),
                             softcap=float(softcap) if softcap else None)
    counters["bwd"] += 1
    try:
        return lowering.attention_backward(_rows(q), _rows(k), _rows(v), _rows(o), lse.contiguous(), _rows(dout), plan)
    except lowering.UnsupportedPlan:
        counters["repacked"] += 1
        return lowering.attention_backward(q.contiguous(), k.contiguous(), v.contiguous(), o.contiguous(),
                                           lse.contiguous(), dout.contiguous(), plan)


@attention_bwd.register_fake
def _(q, k, v, o, lse, dout, mask, window, scale, softcap):
    return q.new_empty(q.shape), k.new_empty(k.shape), v.new_empty(v.shape)


def _setup(ctx, inputs, output):
    q, k, v, mask, window, scale, softcap = inputs
    o, lse = output
    ctx.save_for_backward(q, k, v, o, lse)
    ctx.consts = (mask, window, scale, softcap)


def _backward(ctx, d_o, d_lse):
    q, k, v, o, lse = ctx.saved_tensors
    mask, window, scale, softcap = ctx.consts
    dq, dk, dv = attention_bwd(q, k, v, o, lse, d_o, mask, window, scale, softcap)
    return dq, dk, dv, None, None, None, None


attention_fwd.register_autograd(_backward, setup_context=_setup)


def trainable(match, dtype_of) -> str:
    """"" when the backward kernels serve the matched attention, else the reason they do not.
    ``dtype_of(i)`` / shapes come from the traced values of the match's inputs."""
    if match.k.paged or match.v.paged:
        return "paged K/V"
    if match.base2 or match.denom_add or match.q2 is not None:
        return "explicit softmax / two-part scores"
    if match.bias is not None or match.out_bias is not None:
        return "additive biases"
    # (an attention taken over from F.scaled_dot_product_attention asks for zeros in rows that see no key:
    # without a mask tensor -- refused above -- there is no such row, so the flag changes nothing here)
    if match.late_factors:
        return "factors applied after the mask"
    val = dtype_of(match.q.index)
    if val is None or val.dtype not in (torch.bfloat16, torch.float16):
        return "operands are not bf16 / fp16"
    if val.shape[-1] not in (64, 128):
        return "head dim other than 64 / 128"

    def tensor_arg(x) -> bool:
        if isinstance(x, tuple) and x[0] == "recip":
            return tensor_arg(x[1])
        return isinstance(x, tuple) and x[0] == "arg" and isinstance(dtype_of(x[1]), torch.Tensor)

    if any(tensor_arg(f) for f in list(match.factors) + list(match.post_factors)):
        return "a score factor held in a tensor"
    return ""


def fused_call_train(match, *vals):
    """The matched attention as differentiable views of its inputs around the custom op (what
    AOTAutograd traces in the place of the unfused sub-graph)."""
    def view(op):
        t = vals[op.index]
        if t.dim() == 3:
            t = t.unsqueeze(0)
        return t.permute(op.perm)

    plan = match.plan_for(vals)
    out, _ = torch.ops.loopfuse_amd.attention_fwd(view(match.q), view(match.k), view(match.v),
                                                  _MASK_CODE[plan.mask], plan.window, plan.scale,
                                                  float(plan.softcap) if plan.softcap is not None else 0.0)
    if match.out_order:
        # the traced graph goes on with the output's memory order (torch's fused attention ops return
        # [B, H, S, D] values stored as [B, S, H, D], and a view may rely on it): same values, that order
        inv = [0] * 4
        for pos, dim in enumerate(match.out_order):
            inv[dim] = pos
        out = out.permute(match.out_order).contiguous().permute(inv)
    if match.out_rank == 3:
        out = out.reshape(out.shape[0] * out.shape[1], out.shape[2], out.shape[3])
    return out
