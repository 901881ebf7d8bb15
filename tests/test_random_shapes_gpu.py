"""Seeded random run-time shapes through the HIP path against the oracle (forward) and float64
autograd (backward); seeded random graphs without an attention through the generated kernels.

The compile-time part of a case (dtype, head dim, mask kind, softcap yes / no, heads per kv head,
page size) comes from a short fixed list, so the sweep needs no code objects beyond those of the
other tests; everything a launch decides at run time -- batch, head counts, both lengths, the window,
the cap, the page table -- is drawn from a seeded generator: lengths around tile edges (31 .. 33,
63 .. 65, 127 .. 129, 257), one-row and one-key problems, Sq != Sk, windows of 1, of a tile, wider
than the sequence, (batch, kv head) counts that do not fill a group of workgroup slots.
"""
import random

import pytest
import torch

from loopfuse_amd import lowering

from test_backward_gpu import _ref
from test_parity_gpu import check, rand

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16

LENGTHS = [1, 2, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 256, 257, 300, 385, 512, 593, 700]
WINDOWS = [1, 2, 31, 32, 33, 64, 100, 128, 129, 256, 257, 1000]

# dtype, D, mask, softcap?, query heads per kv head, page size of K and V pools (0 = dense)
PREFILL = [
    (BF, 128, "causal", False, 1, 0),
    (BF, 128, "causal", True, 1, 0),
    (BF, 128, "sliding", True, 4, 0),
    (BF, 128, "sliding", False, 1, 0),
    (BF, 128, None, False, 1, 0),
    (BF, 64, "causal", False, 2, 0),
    (HF, 128, "causal", False, 1, 0),
    (HF, 64, None, False, 1, 0),
    (BF, 128, "causal", False, 4, 16),
]
DECODE = [
    (BF, 128, 1, 0),
    (BF, 128, 4, 16),
    (HF, 128, 8, 0),
    (BF, 64, 2, 0),
]
BACKWARD = [
    (BF, 128, "causal", False),
    (BF, 128, None, False),
    (BF, 128, "sliding", False),
    (HF, 64, "causal", False),
    (HF, 64, None, False),
    (HF, 128, "sliding", False),
    (BF, 128, "causal", True),
    (BF, 128, "sliding", True),
    (HF, 64, None, True),
    (HF, 64, "causal", True),
]


def _lengths(rng, mask):
    sq = rng.choice(LENGTHS)
    if mask is None:
        return sq, rng.choice(LENGTHS)
    if mask == "causal":       # top-left aligned: every row sees key 0 whatever Sk is
        return sq, rng.choice([sq, sq, sq + rng.randrange(0, 200), max(1, sq - rng.randrange(0, 100))])
    return sq, sq + rng.choice([0, 0, 5, 77])      # sliding: Sk >= Sq keeps a visible key in every row


def _pool(B, S, P, Hkv, D, dtype, seed):
    pages = B * (S // P)
    table = torch.randperm(pages, generator=torch.Generator().manual_seed(seed)).view(B, S // P).to(torch.int32)
    return rand((pages, P, Hkv, D), dtype, seed), table


@pytest.mark.parametrize("chunk", range(4))
def test_forward_random_shapes(chunk):
    rng = random.Random(1000 + chunk)
    for n in range(40):
        if rng.random() < 0.7:
            dtype, D, mask, capped, G, P = rng.choice(PREFILL)
            Sq, Sk = _lengths(rng, mask)
        else:
            dtype, D, G, P = rng.choice(DECODE)
            mask, capped, Sq, Sk = None, False, 1, rng.choice([1, 15, 16, 17, 100, 511, 777, 1024, 2049, 5000])
        B, Hkv = rng.choice([1, 2, 3]), rng.choice([1, 2, 3])
        window = rng.choice(WINDOWS) if mask == "sliding" else 0
        softcap = rng.choice([5.0, 30.0]) if capped else None
        if P:
            Sk = max(P, Sk // P * P)
            if mask == "sliding":
                Sq = min(Sq, Sk)
        seed = 100 * chunk + n
        print(f"case {chunk}.{n}: {dtype} D{D} mask={mask} window={window} softcap={softcap} B{B} Hq{Hkv * G} Hkv{Hkv} "
              f"Sq{Sq} Sk{Sk} page={P}", flush=True)
        q = rand((B, Hkv * G, Sq, D), dtype, seed)
        if P:
            (k, kt), (v, vt) = _pool(B, Sk, P, Hkv, D, dtype, seed + 1), _pool(B, Sk, P, Hkv, D, dtype, seed + 2)
        else:
            k, v, kt, vt = rand((B, Hkv, Sk, D), dtype, seed + 1), rand((B, Hkv, Sk, D), dtype, seed + 2), None, None
        check(q, k, v, mask=mask, window=window, softcap=softcap, k_table=kt, v_table=vt)


@pytest.mark.parametrize("chunk", range(4))
def test_backward_random_shapes(chunk):
    rng = random.Random(2000 + chunk)
    for n in range(25):
        dtype, D, mask, capped = rng.choice(BACKWARD)
        Sq, Sk = _lengths(rng, mask)
        B, Hkv, G = rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 5]), rng.choice([1, 1, 2, 3, 4, 8])
        window = rng.choice(WINDOWS) if mask == "sliding" else 0
        softcap = rng.choice([5.0, 30.0, -8.0]) if capped else None
        print(f"case {chunk}.{n}: {dtype} D{D} mask={mask} window={window} softcap={softcap} B{B} Hq{Hkv * G} Hkv{Hkv} "
              f"Sq{Sq} Sk{Sk}", flush=True)
        g = torch.Generator().manual_seed(100 * chunk + n)
        q, k, v, dout = (torch.randn(s, generator=g).to(dtype).to(DEV)
                         for s in ((B, Hkv * G, Sq, D), (B, Hkv, Sk, D), (B, Hkv, Sk, D), (B, Hkv * G, Sq, D)))
        scale = D ** -0.5
        plan = lowering.AttnPlan(mask=mask, window=window, scale=scale, softcap=softcap)
        lse = torch.empty((B, Hkv * G, Sq), dtype=torch.float32, device=DEV)
        o = lowering.attention(q, k, v, plan, lse=lse)
        o_ref, lse_ref, dq_ref, dk_ref, dv_ref = _ref(q, k, v, dout, mask, window, scale, abs(softcap) if softcap else None)
        assert (o.double() - o_ref).abs().max().item() <= (2e-2 if dtype == BF else 5e-3)
        torch.testing.assert_close(lse.double(), lse_ref, rtol=1e-3, atol=4e-3)
        dq, dk, dv = lowering.attention_backward(q, k, v, o, lse, dout, plan)
        for name, got, want in (("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
            assert torch.isfinite(got).all(), name
            if want.norm().item() > 1e-6:      # one visible key: dQ and dK are exactly zero, only the absolute bound applies
                rel = ((got.double() - want).norm() / want.norm()).item()
                assert rel <= (2e-2 if dtype == BF else 5e-3), f"{name}: relative error {rel}"
            err = (got.double() - want).abs().max().item()
            assert err <= (4e-2 if dtype == BF else 1e-2) * max(1.0, want.abs().max().item()), f"{name}: max abs err {err}"


def _generic_case(rng):
    """A random graph over the operations the loop-nest builder knows: elementwise chains with
    broadcast operands, matmul (+ scale, + bias), batched matmul, softmax @ y, reductions."""
    B, M = rng.choice([1, 2, 3]), rng.choice([1, 5, 16, 33, 64, 100])
    N, K = rng.choice([1, 7, 16, 48, 64, 130]), rng.choice([8, 16, 40, 64])
    dt = rng.choice([torch.float32, BF, HF])
    kind = rng.choice(["ew", "ew", "mm", "mm_add", "softmax_mm", "reduce", "bmm"])
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    r = lambda *shape: (torch.randn(*shape, generator=g) * 0.5).to(dt).to(DEV)
    c1, c2 = rng.choice([0.5, 2.0, -1.5, 3.0]), rng.choice([0.25, 1.0, -2.0])
    if kind == "ew":
        other = rng.choice([(B, M, N), (M, N), (1, N), (N,), (B, 1, N), (B, M, 1)])
        ops = rng.sample(["add", "sub", "mul", "scale", "tanh", "exp", "div"], k=rng.choice([1, 2, 3]))

        def fn(a, b):
            x = a
            for o in ops:
                x = {"add": lambda: x + b, "sub": lambda: x - b, "mul": lambda: x * b, "scale": lambda: x * c1 + c2,
                     "tanh": lambda: torch.tanh(x), "exp": lambda: torch.exp(x * 0.5), "div": lambda: x / (b * b + 1.0)}[o]()
            return x
        return f"{ops} with {other}", fn, (r(B, M, N), r(*other)), dt
    if kind == "mm":
        return "a @ b", (lambda a, b: a @ b), (r(M, K), r(K, N)), dt
    if kind == "mm_add":
        other = rng.choice([(M, N), (N,), (1, N)])
        return f"(a @ b) * c + bias{other}", (lambda a, b, c: (a @ b) * c1 + c), (r(M, K), r(K, N), r(*other)), dt
    if kind == "bmm":
        return "tanh(a @ b) + c", (lambda a, b, c: torch.tanh(a @ b) + c), (r(B, M, K), r(B, K, N), r(B, M, N)), dt
    if kind == "softmax_mm":
        return "softmax(x * c) @ y", (lambda x, y: torch.softmax(x * c1, dim=-1) @ y), (r(B, M, K), r(B, K, N)), dt
    which = rng.choice(["sum", "max", "scaled_by_sum", "softmax_by_hand"])
    fn = {"sum": lambda a, b: (a * b).sum(-1), "max": lambda a, b: (a + b).max(-1).values,
          "scaled_by_sum": lambda a, b: a / torch.exp(b).sum(-1, keepdim=True),
          "softmax_by_hand": lambda a, b: torch.exp(a - a.max(-1, keepdim=True).values)
          / torch.exp(a - a.max(-1, keepdim=True).values).sum(-1, keepdim=True) + b}[which]
    return which, fn, (r(B, M, N), r(B, M, N)), dt


@pytest.mark.parametrize("chunk", range(3))
def test_generated_kernels_random_graphs(chunk):
    """Every graph is lowered nest by nest to generated HIP kernels (counted: no eager route) and
    equals the same function evaluated in float64."""
    from loopfuse_amd import loopfuse_backend
    from loopfuse_amd.torch_backend import interface

    rng = random.Random(3000 + chunk)
    for n in range(20):
        desc, fn, ins, dt = _generic_case(rng)
        dynamic = rng.choice([True, None])
        print(f"case {chunk}.{n}: {desc} {dt} {[tuple(t.shape) for t in ins]} dynamic={dynamic}", flush=True)
        torch._dynamo.reset()
        before = dict(interface.stats)
        with torch.no_grad():
            got = torch.compile(fn, backend=loopfuse_backend, dynamic=dynamic)(*ins)
        want = fn(*[t.double() for t in ins])
        assert interface.stats["fused_generic"] == before["fused_generic"] + 1
        assert got.shape == want.shape and got.dtype == dt
        tol = {torch.float32: 2e-4, BF: 3e-2, HF: 6e-3}[dt] * (4 if "@" in desc else 1)
        assert (got.double() - want).abs().max().item() <= tol * max(1.0, want.abs().max().item())
