"""Contractions in graphs without an attention on the MFMA path (``compiler/emit_gemm.py``): the
reference emits ``tl.dot`` for every contraction (``loopfuse/codegen.py:658-668``) and checks
``a @ b + c`` in two and three dims (``tests/test_accuracy.py:56-82``).  Expected values are float64
einsums on the CPU; the tolerance is the output format's rounding (2^-8 relative for bf16, 2^-11 for
fp16) plus the fp32 accumulation of K products of rounded operands."""
import pytest
import torch

import loopfuse_amd  # noqa: F401
from loopfuse_amd import loopfuse_backend
from loopfuse_amd.compiler import generic
from loopfuse_amd.torch_backend import interface

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF, HF = torch.bfloat16, torch.float16


@pytest.fixture(autouse=True)
def _fixed_route(monkeypatch):
    """The route of a call is asserted below: the measured choice between generated and captured graph stays off
    except in the test of that choice."""
    monkeypatch.setenv("LOOPFUSE_AUTOTUNE", "0")


def rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _close(got, want, dtype):
    rel = 2.0 ** -8 if dtype == BF else 2.0 ** -11
    err = (got.double().cpu() - want).abs()
    budget = rel * want.abs() + 2e-3 * max(1.0, want.abs().max().item()) * (1.0 if dtype == BF else 0.25)
    assert torch.isfinite(got).all()
    assert (err <= budget).all(), f"max excess {(err - budget).max().item()}"


def _compiled(fn):
    torch._dynamo.reset()
    return torch.compile(fn, backend=loopfuse_backend, dynamic=True)


CASES = [
    # name, shapes of a, b (as stored), how the graph views them, epilogue operand shape
    ("ref_2dim", (1024, 64), (64, 128), "ab", (1024, 128)),            # reference tests/test_accuracy.py:56-64
    ("ref_3dim", (4, 1024, 64), (4, 64, 128), "ab", (4, 1024, 128)),   # reference tests/test_accuracy.py:69-82
    ("b_transposed", (300, 72), (136, 72), "abT", (300, 136)),         # B stored [N, K]: k-contiguous on both sides
    ("a_transposed", (200, 264), (200, 96), "aTb", (264, 96)),         # A stored [K, M]: transposed reads on both sides
    ("both_transposed", (64, 520), (40, 64), "aTbT", (520, 40)),
    ("ragged_rows", (777, 128), (128, 200), "ab", (777, 200)),         # M odd (A k-contiguous), N a multiple of 8 only
    ("odd_n_b_kcontig", (130, 64), (77, 64), "abT", (130, 77)),        # N odd with B k-contiguous
    ("long_k", (256, 4096), (4096, 256), "ab", (256, 256)),
    ("batch_broadcast_b", (3, 2, 160, 64), (64, 96), "ab", (96,)),     # B shared by every batch element; bias over n
    ("tiny", (8, 8), (8, 8), "ab", (8, 8)),
    # enough 256 x 256 tiles to fill the CUs: the eight-wave kernel, ragged at both edges, in every layout
    ("large_tiles", (3592, 192), (192, 3600), "ab", (3600,)),
    ("large_tiles_bT", (3592, 136), (3601, 136), "abT", (3592, 3601)),
    ("large_tiles_aT", (72, 3600), (72, 3592), "aTb", (3592,)),
    ("large_tiles_aTbT", (200, 3592), (3608, 200), "aTbT", (3592, 3608)),
]


@pytest.mark.parametrize("dtype", [BF, HF])
@pytest.mark.parametrize("name,sa,sb,form,sc", CASES, ids=[c[0] for c in CASES])
def test_matmul_with_epilogue_runs_on_mfma(name, sa, sb, form, sc, dtype):
    a, b, c = rand(sa, dtype, 1, 0.5), rand(sb, dtype, 2, 0.5), rand(sc, dtype, 3)
    va = (lambda t: t.transpose(-1, -2)) if form.startswith("aT") else (lambda t: t)
    vb = (lambda t: t.transpose(-1, -2)) if form.endswith("bT") else (lambda t: t)
    fn = lambda a, b, c: (va(a) @ vb(b)) * 0.25 + c           # noqa: E731
    ins = [t.to(DEV) for t in (a, b, c)]
    before, stats = dict(generic.counters), dict(interface.stats)
    got = _compiled(fn)(*ins)
    assert interface.stats["fused_generic"] == stats["fused_generic"] + 1
    assert generic.counters["mfma"] == before["mfma"] + 1 and generic.counters["plain"] == before["plain"]
    want = torch.matmul(va(a.double()), vb(b.double())) * 0.25 + c.double()
    assert got.dtype == dtype and tuple(got.shape) == tuple(want.shape)
    _close(got, want, dtype)


def test_calls_the_mfma_kernel_cannot_read_take_the_plain_kernel():
    """k not a multiple of 8, a misaligned base, an operand stride that is not a multiple of 8: same program, the
    one-thread-per-element kernel of the nest serves the call."""
    fn = lambda a, b, c: a @ b + c        # noqa: E731
    a, b, c = rand((64, 32), BF, 1).to(DEV), rand((32, 48), BF, 2).to(DEV), rand((64, 48), BF, 3).to(DEV)
    run = _compiled(fn)
    cases = [
        (rand((64, 20), BF, 4).to(DEV), rand((20, 48), BF, 5).to(DEV), c),                     # K = 20
        (rand((64, 33), BF, 6).to(DEV)[:, 1:], b, c),                                          # base 2 bytes off, row stride 33
        (a, rand((32, 52), BF, 7).to(DEV)[:, :48], c),                                         # row stride 52
    ]
    for x, y, z in cases:
        before = dict(generic.counters)
        got = run(x, y, z)
        assert generic.counters["mfma"] == before["mfma"] and generic.counters["plain"] == before["plain"] + 1
        _close(got, x.double().cpu() @ y.double().cpu() + z.double().cpu(), BF)
    before = dict(generic.counters)
    _close(run(a, b, c), a.double().cpu() @ b.double().cpu() + c.double().cpu(), BF)
    assert generic.counters["mfma"] == before["mfma"] + 1


def test_large_matmul_is_no_longer_left_to_the_captured_graph():
    """2048 x 2048 x 2048 is 2^33 multiply-adds, far beyond what the plain kernels are allowed: on the MFMA path the
    backend keeps the graph (counted as a generated-kernel run), a tanh epilogue and a bias over n fused."""
    fn = lambda a, b, bias: torch.tanh(a @ b.t() * 0.02 + bias)      # noqa: E731
    a, b, bias = rand((2048, 2048), BF, 1), rand((2048, 2048), BF, 2), rand((2048,), BF, 3)
    torch._dynamo.reset()
    before, kinds = dict(interface.stats), dict(generic.counters)
    got = torch.compile(fn, backend=loopfuse_backend)(a.to(DEV), b.to(DEV), bias.to(DEV))
    assert interface.stats["fused_generic"] == before["fused_generic"] + 1
    assert interface.stats["eager_runtime"] == before["eager_runtime"]
    assert generic.counters["mfma"] == kinds["mfma"] + 1 and generic.counters["plain"] == kinds["plain"]
    want = torch.tanh(a.double() @ b.double().t() * 0.02 + bias.double())
    _close(got, want, BF)


def test_two_products_in_a_row_keep_the_intermediate_and_both_run_on_mfma():
    """(a @ b) @ c (reference tests/test_accuracy.py:85-100, commented out there): the first product stays a
    temporary -- fp32, so the second contraction reads it through the plain kernel unless it is small; here only
    the first runs on MFMA and the result still matches."""
    fn = lambda a, b, c: (a @ b) @ c      # noqa: E731
    a, b, c = rand((256, 64), BF, 1, 0.3), rand((64, 128), BF, 2, 0.3), rand((128, 64), BF, 3, 0.3)
    ins = [t.to(DEV) for t in (a, b, c)]
    before = dict(generic.counters)
    got = _compiled(fn)(*ins)
    assert generic.counters["mfma"] + generic.counters["plain"] == before["mfma"] + before["plain"] + 2
    assert generic.counters["mfma"] >= before["mfma"] + 1
    _close(got, (a.double() @ b.double()) @ c.double(), BF)


def test_max_autotune_measures_large_products_against_the_captured_graph(monkeypatch):
    """Under mode="max-autotune" (the default) a call with 2^32 flop or more in generated MFMA kernels is timed
    against the captured graph once; later calls of that signature take the faster route.  Either way the values
    are right and every call is accounted for."""
    monkeypatch.setenv("LOOPFUSE_AUTOTUNE", "1")
    fn = lambda a, b, bias: a @ b.t() + bias      # noqa: E731
    a, b, bias = rand((4096, 2048), BF, 1, 0.5), rand((4096, 2048), BF, 2, 0.5), rand((4096,), BF, 3)
    ins = [t.to(DEV) for t in (a, b, bias)]
    want = a.double() @ b.double().t() + bias.double()
    torch._dynamo.reset()
    run = torch.compile(fn, backend=loopfuse_backend)
    before = dict(interface.stats)
    for _ in range(3):
        got = run(*ins)
        # the captured graph rounds the product to bf16 before the bias is added: one more half-ulp
        err = (got.double().cpu() - want).abs()
        assert (err <= 2.0 ** -7 * want.abs() + 0.02 * want.abs().max()).all()
    routed = {k: interface.stats[k] - before[k] for k in ("fused_generic", "tuned_captured", "eager_runtime", "eager_graph")}
    assert routed["fused_generic"] + routed["tuned_captured"] == 3 and routed["fused_generic"] >= 1, routed
    assert routed["eager_runtime"] == 0 and routed["eager_graph"] == 0, routed
    assert routed["tuned_captured"] in (0, 2), routed


@pytest.mark.parametrize("act", ["gelu_tanh", "relu", "silu"])
def test_mlp_block_runs_both_products_on_mfma(act):
    """linear -> activation -> linear (the layers around an attention): bias and activation are the first
    product's epilogue, its result is stored in the graph's own dtype -- the rounding eager does -- and read by
    the second product as an MFMA operand.  Expected: float64 with the hidden activations rounded the same way."""
    import torch.nn.functional as F
    fa = {"gelu_tanh": lambda h: F.gelu(h, approximate="tanh"), "relu": F.relu, "silu": F.silu}[act]

    def mlp(x, w1, b1, w2, b2):
        return F.linear(fa(F.linear(x, w1, b1)), w2, b2)

    x, w1, b1 = rand((4, 300, 256), BF, 1), rand((1024, 256), BF, 2, 0.06), rand((1024,), BF, 3, 0.1)
    w2, b2 = rand((256, 1024), BF, 4, 0.03), rand((256,), BF, 5, 0.1)
    ins = [t.to(DEV) for t in (x, w1, b1, w2, b2)]
    before, stats = dict(generic.counters), dict(interface.stats)
    got = _compiled(mlp)(*ins)
    assert interface.stats["fused_generic"] == stats["fused_generic"] + 1
    assert generic.counters["mfma"] == before["mfma"] + 2 and generic.counters["plain"] == before["plain"]
    h = fa(x.double() @ w1.double().t() + b1.double()).to(BF).double()
    want = h @ w2.double().t() + b2.double()
    assert got.dtype == BF and tuple(got.shape) == (4, 300, 256)
    # a hidden value that falls next to a rounding boundary may round the other way: one bf16 ulp of one of 1024 terms
    _close(got, want, BF)


@pytest.mark.parametrize("chunk", range(3))
def test_random_products_on_mfma(chunk, monkeypatch):
    """Seeded shapes, layouts, batch forms, epilogues and tile shapes: every call that satisfies the kernel's
    alignment rules runs on MFMA and equals float64; operands are slices of larger tensors half of the time, so
    that row strides differ from extents."""
    import random

    rng = random.Random(4000 + chunk)
    for n in range(12):
        dtype = rng.choice([BF, BF, HF])
        M = rng.choice([8, 64, 100, 129, 250, 256, 300, 511, 777])
        N = rng.choice([8, 40, 128, 136, 256, 264, 520])
        K = rng.choice([8, 16, 64, 72, 128, 200, 1024])
        batch = rng.choice([(), (), (2,), (3,), (2, 2)])
        a_t, b_t = rng.random() < 0.4, rng.random() < 0.5
        if a_t:
            M = -(-M // 8) * 8                       # m is the contiguous dimension of A: pieces of 8
        if not b_t:
            N = -(-N // 8) * 8
        pad_a, pad_b = rng.choice([0, 8, 24]), rng.choice([0, 8, 16])
        tile = rng.choice(["s", "l", None])
        monkeypatch.setenv("LOOPFUSE_GEMM_TILE", tile or "")
        sa = batch + ((K, M + pad_a) if a_t else (M, K + pad_a))
        b_batched = bool(batch) and rng.random() < 0.5
        sb = (batch if b_batched else ()) + ((N, K + pad_b) if b_t else (K, N + pad_b))
        a_full, b_full = rand(sa, dtype, 100 * chunk + n, 0.5).to(DEV), rand(sb, dtype, 100 * chunk + n + 50, 0.5).to(DEV)
        a = a_full[..., :M] if a_t else a_full[..., :K]
        b = b_full[..., :K] if b_t else b_full[..., :N]
        bias_shape = rng.choice([(N,), (M, N), (1, N), batch + (M, N), (M, 1)])
        bias = rand(bias_shape, dtype, 100 * chunk + n + 70).to(DEV)
        epi = rng.choice(["affine", "tanh", "relu", "gelu"])
        va = (lambda t: t.transpose(-1, -2)) if a_t else (lambda t: t)
        vb = (lambda t: t.transpose(-1, -2)) if b_t else (lambda t: t)
        act = {"affine": lambda x: x, "tanh": torch.tanh, "relu": torch.relu, "gelu": torch.nn.functional.gelu}[epi]
        fn = lambda a, b, c: act((va(a) @ vb(b)) * 0.125 + c)      # noqa: E731
        print(f"case {chunk}.{n}: {dtype} M{M} N{N} K{K} batch{batch} b_batched={b_batched} aT={a_t} bT={b_t} pads {pad_a},{pad_b} "
              f"bias{bias_shape} {epi} tile={tile}", flush=True)
        before = dict(generic.counters)
        got = _compiled(fn)(a, b, bias)
        assert generic.counters["mfma"] == before["mfma"] + 1 and generic.counters["plain"] == before["plain"]
        want = act((va(a.double().cpu()) @ vb(b.double().cpu())) * 0.125 + bias.double().cpu())
        assert tuple(got.shape) == tuple(want.shape)
        _close(got, want, dtype)


def test_softmax_times_matrix_at_the_reference_size():
    """``softmax(x) @ y`` with x [4, 8, 1024, 64], y [4, 8, 64, 1024] in bf16 (reference tests/test_accuracy.py:197-211,
    its own size): 2^31 multiply-adds, which the plain kernels are not allowed.  The row maxima and sums are plain
    reductions, the probabilities a bf16 tensor, the product an MFMA launch."""
    x, y = rand((4, 8, 1024, 64), BF, 1), rand((4, 8, 64, 1024), BF, 2)
    before, stats = dict(generic.counters), dict(interface.stats)
    got = _compiled(lambda x, y: torch.softmax(x, dim=-1) @ y)(x.to(DEV), y.to(DEV))
    assert interface.stats["fused_generic"] == stats["fused_generic"] + 1 and interface.stats["eager_runtime"] == stats["eager_runtime"]
    assert generic.counters["mfma"] == before["mfma"] + 1 and generic.counters["plain"] == before["plain"] + 3
    p = torch.softmax(x.double(), dim=-1).to(BF).double()
    _close(got, p @ y.double(), BF)


def test_long_reductions_take_one_wave_per_output():
    """A reduction over 128 or more elements per output runs one wave per output element (lanes stride over the
    reduced index space, combine through ds_bpermute); shorter ones keep one thread per output.  Sums, maxima, a
    reduction over two merged dims and one whose reduced dim is not the contiguous one."""
    x = rand((3, 5, 700), torch.float32, 1)
    y = rand((3, 5, 700), torch.float32, 2)
    cases = [
        ("sum", lambda a, b: (a * b).sum(-1), 1),
        ("max", lambda a, b: (a + b).max(-1).values, 1),
        ("two dims", lambda a, b: (a - b).sum(dim=(1, 2)), 1),
        ("strided", lambda a, b: (a * 2.0 + b).sum(dim=0), 0),                    # 3 elements per output: plain kernel
        ("through a transposed view", lambda a, b: torch.exp(a * 0.1).transpose(1, 2).sum(dim=1), 1),   # the 700-long dim again
        ("long and strided", lambda a, b: (a.permute(2, 0, 1) * 0.5 - b.permute(2, 0, 1)).sum(dim=0), 1),  # the long dim, reduced through permuted views
        ("short middle dim", lambda a, b: (a + b).sum(dim=1), 0),                    # 5 per output: plain
        ("softmax by hand", lambda a, b: torch.exp(a - a.max(-1, keepdim=True).values)
         / torch.exp(a - a.max(-1, keepdim=True).values).sum(-1, keepdim=True) + b, 3),      # the maximum is written twice
    ]
    for name, fn, n_wave in cases:
        before = dict(generic.counters)
        got = _compiled(fn)(x.to(DEV), y.to(DEV))
        want = fn(x.double(), y.double())
        assert generic.counters["wave"] == before["wave"] + n_wave, name
        torch.testing.assert_close(got.double().cpu(), want, rtol=1e-5, atol=1e-4)


def test_simplified_attention_at_the_reference_size():
    """(Q K^T / (max + sum + 1e-3)) V, no exponential (reference tests/test_accuracy.py:314-333, B4 H8 S1024 D64,
    bf16): both products on MFMA, the two row reductions over 1024 scores one wave per row, the quotient a bf16
    tensor.  The reference checks this case at rtol 1e-2."""
    def fn(Q, K, V):
        QK = Q @ K.transpose(-2, -1)
        m = torch.max(QK, dim=-1, keepdim=True)[0] + torch.sum(QK, dim=-1, keepdim=True)
        return (QK / (m + 1e-3)) @ V

    Q, K, V = (rand((4, 8, 1024, 64), BF, s, 0.2) for s in (1, 2, 3))
    before, stats = dict(generic.counters), dict(interface.stats)
    got = _compiled(fn)(Q.to(DEV), K.to(DEV), V.to(DEV))
    assert interface.stats["fused_generic"] == stats["fused_generic"] + 1 and interface.stats["eager_runtime"] == stats["eager_runtime"]
    assert generic.counters["mfma"] == before["mfma"] + 2 and generic.counters["wave"] == before["wave"] + 2
    s = torch.einsum("bhid,bhjd->bhij", Q.double(), K.double())
    den = s.amax(dim=-1) + s.sum(dim=-1) + 1e-3
    want = torch.einsum("bhij,bhjd->bhid", (s / den[..., None]).to(BF).double(), V.double())
    err = (got.double().cpu() - want).abs()
    assert (err <= 1e-2 * want.abs() + 1e-2 * want.abs().max()).all(), err.max().item()
