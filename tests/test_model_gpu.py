"""A small GPT (embeddings, three blocks of layer norm / causal self-attention / MLP, head) through
``torch.compile(backend=loopfuse_backend)``: every attention of the model runs the HIP kernels, the
rest of the graph keeps running as ATen ops, in inference (dynamic shapes, two sequence lengths) and
in training (static shapes, fused forward and backward), against the uncompiled module.

Two spellings of the attention, as the common GPT module has them: the triangle kept in a buffer and
applied with ``masked_fill(bias[:, :, :T, :T] == 0, -inf)`` (a mask tensor: fused with the mask as a
score term in inference, left to autograd in training), and ``F.scaled_dot_product_attention(...,
is_causal=True)`` (the causal flag in both)."""
import math

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from loopfuse_amd import loopfuse_backend
from loopfuse_amd.torch_backend import interface, training

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class SelfAttention(nn.Module):
    def __init__(self, width, heads, context, sdpa):
        super().__init__()
        self.qkv, self.proj = nn.Linear(width, 3 * width), nn.Linear(width, width)
        self.heads, self.width, self.sdpa = heads, width, sdpa
        self.register_buffer("bias", torch.tril(torch.ones(context, context)).view(1, 1, context, context))

    def forward(self, x):
        B, T, C = x.size()
        q, k, v = (t.view(B, T, self.heads, C // self.heads).transpose(1, 2) for t in self.qkv(x).split(self.width, dim=2))
        if self.sdpa:
            y = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=True)
        else:
            att = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(k.size(-1)))
            att = att.masked_fill(self.bias[:, :, :T, :T] == 0, float("-inf"))
            y = F.softmax(att, dim=-1) @ v
        return self.proj(y.transpose(1, 2).contiguous().view(B, T, C))


class Block(nn.Module):
    def __init__(self, width, heads, context, sdpa):
        super().__init__()
        self.ln_1, self.ln_2 = nn.LayerNorm(width), nn.LayerNorm(width)
        self.attn = SelfAttention(width, heads, context, sdpa)
        self.mlp = nn.Sequential(nn.Linear(width, 4 * width), nn.GELU(), nn.Linear(4 * width, width))

    def forward(self, x):
        x = x + self.attn(self.ln_1(x))
        return x + self.mlp(self.ln_2(x))


class GPT(nn.Module):
    def __init__(self, sdpa, vocab=512, context=256, layers=3, heads=4, width=256):
        super().__init__()
        self.wte, self.wpe = nn.Embedding(vocab, width), nn.Embedding(context, width)
        self.h = nn.ModuleList([Block(width, heads, context, sdpa) for _ in range(layers)])
        self.ln_f, self.head = nn.LayerNorm(width), nn.Linear(width, vocab, bias=False)

    def forward(self, idx):
        pos = torch.arange(0, idx.size(1), dtype=torch.long, device=idx.device)
        x = self.wte(idx) + self.wpe(pos)
        for blk in self.h:
            x = blk(x)
        return self.head(self.ln_f(x))


def _model(sdpa):
    torch.manual_seed(0)
    return GPT(sdpa).to(DEV).to(torch.bfloat16)


@pytest.mark.parametrize("sdpa", [False, True])
def test_gpt_inference_runs_every_attention_fused(sdpa):
    m = _model(sdpa).eval()
    idx = torch.randint(0, 512, (2, 100), generator=torch.Generator().manual_seed(1)).to(DEV)
    torch._dynamo.reset()
    before = dict(interface.stats)
    cm = torch.compile(m, backend=loopfuse_backend, dynamic=True)
    with torch.no_grad():
        for tokens in (idx, idx[:, :77].contiguous()):
            got, want = cm(tokens), m(tokens)
            assert len(interface.last_matches) == 3                                  # one per block
            assert all((mm.mask == "causal") == sdpa and (mm.bias is not None) == (not sdpa) for mm in interface.last_matches)
            assert (got.float() - want.float()).abs().max().item() <= 4e-2 * max(1.0, want.float().abs().max().item())
    assert interface.stats["fused"] - before["fused"] == 2 and interface.stats["eager_runtime"] == before["eager_runtime"]


def test_gpt_training_keeps_the_attention_fused():
    m = _model(True)
    idx = torch.randint(0, 512, (2, 128), generator=torch.Generator().manual_seed(2)).to(DEV)
    torch._dynamo.reset()
    before, ops = dict(interface.stats), dict(training.counters)
    out = torch.compile(m, backend=loopfuse_backend)(idx)
    out.float().square().mean().backward()
    got = {n: p.grad.float().clone() for n, p in m.named_parameters()}
    m.zero_grad()
    ref = m(idx)
    ref.float().square().mean().backward()
    assert interface.stats["training_graphs"] == before["training_graphs"] + 1
    assert training.counters["fwd"] == ops["fwd"] + 3 and training.counters["bwd"] == ops["bwd"] + 3     # three blocks
    assert (out.float() - ref.float()).abs().max().item() <= 4e-2 * max(1.0, ref.float().abs().max().item())
    for n, p in m.named_parameters():
        r = p.grad.float()
        assert ((got[n] - r).norm() / r.norm().clamp_min(1e-20)).item() <= 5e-2, n
