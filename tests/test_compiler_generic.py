"""Generic lowering of non-attention graphs (loop nests -> one HIP kernel per fused nest).

On the CPU the emitted source itself is exercised: the same text is built as host C++ (g++, with
the few HIP spellings defined away and a loop over blocks and threads in the place of the grid)
and run on the arguments, so the indexing, the strides and the extent solver are checked here
before any launch.  The graphs are the reference's non-attention accuracy cases
(reference tests/test_accuracy.py:29-82, 197-211, 235-250, 314-333); expected values come from
float64 computations spelled differently from the compiled function."""
import ctypes
import os
import subprocess

import pytest
import torch

import loopfuse_amd  # noqa: F401  (registers torch.ops.loopfuse.*)
from loopfuse_amd import lowering, runtime
from loopfuse_amd.compiler import emit, generic
from test_compiler_ir import _aten_graph, _r

HOST_PRELUDE = """
#include <cmath>
#define __global__
#define __device__
#define __forceinline__ inline
#define __launch_bounds__(x)
#define __expf expf
struct LfIdx { unsigned x, y, z; };
static thread_local LfIdx blockIdx, threadIdx, blockDim;
"""


def _host_build(prog: generic.GenericProgram, tmp_path):
    drivers = "".join(
        f'extern "C" void drive_{k.name}(const LfGenParams* p, long long blocks) {{ blockDim = {{256, 1, 1}};'
        f" for (long long b = 0; b < blocks; ++b) for (unsigned t = 0; t < 256; ++t) {{ blockIdx.x = (unsigned)b; threadIdx.x = t; {k.name}(*p); }} }}\n"
        for k in prog.kernels)
    src = tmp_path / "gen.cpp"
    src.write_text(HOST_PRELUDE + prog.source + drivers)
    so = tmp_path / "gen.so"
    subprocess.run(["g++", "-O1", "-shared", "-fPIC", "-std=c++17", str(src), "-o", str(so)], check=True)
    lib = ctypes.CDLL(str(so))
    out = []
    for k in prog.kernels:
        f = getattr(lib, "drive_" + k.name)
        f.argtypes = [ctypes.c_void_p, ctypes.c_longlong]
        f.restype = None
        out.append(lambda blocks, prm, f=f: f(ctypes.addressof(prm), blocks))
    return out


def _softmax64(x):
    e = torch.exp(x - x.amax(dim=-1, keepdim=True))
    return e / e.sum(dim=-1, keepdim=True)


def _simplified(Q, K, V):
    QK = Q @ K.transpose(-2, -1)
    m = torch.max(QK, dim=-1, keepdim=True)[0] + torch.sum(QK, dim=-1, keepdim=True)
    return (QK / (m + 1e-3)) @ V


def _simplified_ref(Q, K, V):
    s = torch.einsum("bhid,bhjd->bhij", Q, K)
    den = s.amax(dim=-1) + torch.einsum("bhij->bhi", s) + 1e-3
    return torch.einsum("bhij,bhjd->bhid", s, V) / den[..., None]


def _modified(Q, K, V, qb, sb, ob):
    QK = (Q + qb) @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
    QK = QK * 3.5 + sb
    return torch.softmax(torch.ops.loopfuse.causal_mask(QK), dim=-1) @ V + ob


def _modified_ref(Q, K, V, qb, sb, ob):
    s = torch.einsum("bhid,bhjd->bhij", Q + qb, K) * (3.5 / Q.shape[-1] ** 0.5) + sb
    i = torch.arange(s.shape[-2])[:, None]
    j = torch.arange(s.shape[-1])[None, :]
    s = torch.where(j <= i, s, torch.full_like(s, float("-inf")))
    return torch.einsum("bhij,bhjd->bhid", _softmax64(s), V) + ob


CASES = {
    "add": (lambda a, b: a + b, lambda: (_r(4, 10, 8), _r(4, 10, 8, seed=1)),
            lambda a, b: torch.stack([a, b]).sum(dim=0), 1),
    "add_2dim": (lambda a, b: a + b, lambda: (_r(12, 40), _r(12, 40, seed=1)),
                 lambda a, b: torch.stack([a, b]).sum(dim=0), 1),
    "add_broadcast": (lambda a, b: a + b, lambda: (_r(4, 10, 8), _r(10, 1, seed=1)),
                      lambda a, b: a + b.expand(10, 8)[None], 1),
    "matmul_add": (lambda a, b, c: a @ b + c, lambda: (_r(16, 8), _r(8, 12, seed=1), _r(16, 12, seed=2)),
                   lambda a, b, c: torch.einsum("ik,kj->ij", a, b) + c, 1),
    "matmul_add_3dim": (lambda a, b, c: a @ b + c, lambda: (_r(3, 16, 8), _r(3, 8, 12, seed=1), _r(3, 16, 12, seed=2)),
                        lambda a, b, c: torch.einsum("bik,bkj->bij", a, b) + c, 1),
    "softmax_matmul": (lambda x, y: torch.softmax(x, dim=-1) @ y, lambda: (_r(2, 4, 16, 8), _r(2, 4, 8, 12, seed=1)),
                       lambda x, y: torch.einsum("bhij,bhjd->bhid", _softmax64(x), y), 3),
    "paged_add": (lambda buf, tab: torch.ops.loopfuse.paged_load(buf, tab) + 1,
                  lambda: (_r(16, 4, 8), torch.randint(0, 16, (3, 5), generator=torch.Generator().manual_seed(3), dtype=torch.int32)),
                  lambda buf, tab: torch.stack([torch.stack([buf[int(tab[b, s])] for s in range(tab.shape[1])])
                                                for b in range(tab.shape[0])]) + 1, 1),
    "modified_attn": (_modified, lambda: tuple(_r(2, 2, 16, 8, seed=s) for s in (1, 2, 3, 4)) + (_r(2, 2, 16, 16, seed=5), _r(2, 2, 16, 8, seed=6)),
                      _modified_ref, 4),
    "simplified_attn": (_simplified, lambda: tuple(_r(2, 2, 16, 8, seed=s) * 0.2 for s in (1, 2, 3)), _simplified_ref, 4),
    # the layers around an attention: linear + activation + linear; every activation the builder knows, each written
    # out differently for the expected value
    "mlp_gelu": (lambda x, w1, b1, w2, b2: torch.nn.functional.linear(torch.nn.functional.gelu(torch.nn.functional.linear(x, w1, b1)), w2, b2),
                 lambda: (_r(3, 10, 8), _r(12, 8, seed=1), _r(12, seed=2), _r(6, 12, seed=3), _r(6, seed=4)),
                 lambda x, w1, b1, w2, b2: torch.einsum("bsh,oh->bso", (lambda h: 0.5 * h * (1 + torch.erf(h / 2 ** 0.5)))(
                     torch.einsum("bsk,hk->bsh", x, w1) + b1), w2) + b2, 2),
    "activations": (lambda x: torch.nn.functional.gelu(x, approximate="tanh") + torch.relu(x) * torch.sigmoid(x) -
                    torch.nn.functional.silu(x) + torch.rsqrt(torch.abs(x) + 1.0) * torch.sqrt(torch.abs(x)) + torch.reciprocal(-x - 3.0 * torch.abs(x) - 1.0),
                    lambda: (_r(5, 7),),
                    lambda x: 0.5 * x * (1 + torch.tanh((2 / torch.pi) ** 0.5 * (x + 0.044715 * x ** 3))) + x.clamp(min=0) / (1 + torch.exp(-x))
                    - x / (1 + torch.exp(-x)) + (x.abs() / (x.abs() + 1)) ** 0.5 + 1 / (-x - 3 * x.abs() - 1), 1),
}


@pytest.mark.parametrize("name", list(CASES))
def test_emitted_kernels_run_on_the_host(name, tmp_path):
    fn, make, ref, n_kernels = CASES[name]
    ins = make()
    gm, args, _ = _aten_graph(fn, ins)
    prog = generic.GenericProgram(gm)
    assert len(prog.kernels) == n_kernels          # element-wise producers are inlined into their consumers
    got = prog.run(args, launchers=_host_build(prog, tmp_path))
    want = ref(*[t.double() if t.is_floating_point() else t for t in ins])
    assert got.shape == want.shape
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)


def test_extents_follow_the_call_not_the_trace(tmp_path):
    """Traced with dynamic shapes at one size, run at another: every extent and stride is a
    run-time kernel argument solved from the argument shapes and the SymInt arguments."""
    from torch._functorch.aot_autograd import aot_module_simplified

    fn, _, ref, _ = CASES["matmul_add_3dim"]
    seen = {}

    def backend(gm, sample):
        def fw(g, flat):
            seen["gm"] = g

            def run(*args):
                seen["args"] = args
                return g(*args)
            return run
        return aot_module_simplified(gm, sample, fw_compiler=fw)

    torch._dynamo.reset()
    compiled = torch.compile(fn, backend=backend, dynamic=True)
    with torch.no_grad():
        compiled(_r(3, 16, 8), _r(3, 8, 12, seed=1), _r(3, 16, 12, seed=2))
        prog = generic.GenericProgram(seen["gm"])
        launchers = _host_build(prog, tmp_path)
        ins = (_r(5, 7, 9), _r(5, 9, 11, seed=1), _r(5, 7, 11, seed=2))
        compiled(*ins)                      # same graph, the flat arguments of the new shapes
    assert tuple(seen["args"][-1].shape) == (5, 7, 11)      # no recompilation replaced the graph
    got = prog.run(seen["args"], launchers=launchers)
    torch.testing.assert_close(got.double(), ref(*[t.double() for t in ins]), rtol=1e-5, atol=1e-5)


def test_strided_inputs_are_read_in_place(tmp_path):
    fn, _, ref, _ = CASES["matmul_add"]
    a, b, c = _r(8, 16).t(), _r(8, 24, seed=1)[:, ::2], _r(16, 12, seed=2)
    gm, args, _ = _aten_graph(fn, (a, b, c))
    prog = generic.GenericProgram(gm)
    got = prog.run(args, launchers=_host_build(prog, tmp_path))
    torch.testing.assert_close(got.double(), ref(a.double(), b.double(), c.double()), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("name", list(CASES))
def test_emitted_source_compiles_for_gfx950(name):
    fn, make, _, _ = CASES[name]
    gm, _, _ = _aten_graph(fn, make())
    prog = generic.GenericProgram(gm)
    code, _, _ = runtime.compile_source(prog.source, "lf_generic", list(lowering.COMMON_OPTS), "gfx950", None)
    assert code[:4] == b"\x7fELF"
    assert prog.source.count("__global__") == len(prog.kernels)


def test_graphs_outside_the_builder_are_refused():
    gm, _, _ = _aten_graph(lambda a: torch.cumsum(a, dim=-1), (_r(4, 8),))
    with pytest.raises(emit.NotLowerable):
        generic.GenericProgram(gm)


REFUSED = {
    "add_alpha": (lambda a, b: torch.add(a, b, alpha=3.0), lambda: (_r(6, 8), _r(6, 8, seed=1))),
    "sub_alpha": (lambda a, b: torch.sub(a, b, alpha=2.0), lambda: (_r(6, 8), _r(6, 8, seed=1))),
    "addmm_scaled": (lambda c, a, b: torch.addmm(c, a, b, beta=0.5, alpha=2.0),
                     lambda: (_r(6, 5, seed=2), _r(6, 8), _r(8, 5, seed=1))),
    "int64_add": (lambda a: a + 1, lambda: (torch.full((4, 4), 2 ** 30 + 1, dtype=torch.int64),)),
    "truncation": (lambda a: (a * 2.7).to(torch.int32).float() * 1.5, lambda: (_r(6, 8),)),
    "rounded_division": (lambda a, b: torch.div(a, b, rounding_mode="floor"), lambda: (_r(6, 8), _r(6, 8, seed=1) + 3.0)),
    "integer_values": (lambda a, t: a + t, lambda: (_r(3, 5), torch.arange(15, dtype=torch.int32).view(3, 5))),
}


@pytest.mark.parametrize("name", list(REFUSED))
def test_scaled_rounding_and_integer_forms_are_refused_and_run_as_captured(name):
    """What the nest builder cannot express -- ``alpha`` / ``beta`` of add / sub / addmm, rounding divisions,
    conversions to an integer type, integer tensors used as values -- gets no generic program (it would
    compute something else in fp32); through the backend such a graph runs as captured and agrees with eager."""
    from loopfuse_amd import loopfuse_backend
    from loopfuse_amd.torch_backend import interface

    fn, make = REFUSED[name]
    ins = make()
    gm, _, _ = _aten_graph(fn, ins)
    with pytest.raises(emit.NotLowerable):
        generic.GenericProgram(gm)
    before = dict(interface.stats)
    torch._dynamo.reset()
    got = torch.compile(fn, backend=loopfuse_backend)(*ins)
    want = fn(*ins)
    assert got.dtype == want.dtype
    torch.testing.assert_close(got, want)
    assert interface.stats["generic_graphs"] == before["generic_graphs"]
    assert interface.stats["eager_graph"] == before["eager_graph"] + 1


def test_backend_takes_the_generic_program_for_graphs_without_attention(monkeypatch):
    """Through ``torch.compile(backend=loopfuse_backend)``: the graph gets a generic program; on
    CPU tensors its kernels cannot run and the call goes to the captured graph (counted, not
    silent); ``LOOPFUSE_GENERIC=0`` leaves the graph to the captured ops altogether."""
    from loopfuse_amd import loopfuse_backend
    from loopfuse_amd.torch_backend import interface

    a, b, c = _r(16, 8), _r(8, 12, seed=1), _r(16, 12, seed=2)
    before = dict(interface.stats)
    torch._dynamo.reset()
    got = torch.compile(lambda a, b, c: a @ b + c, backend=loopfuse_backend, dynamic=True)(a, b, c)
    torch.testing.assert_close(got, a @ b + c)
    assert interface.stats["generic_graphs"] == before["generic_graphs"] + 1
    assert interface.stats["fused_generic"] == before["fused_generic"]
    assert interface.stats["eager_runtime"] == before["eager_runtime"] + 1

    monkeypatch.setenv("LOOPFUSE_GENERIC", "0")
    before = dict(interface.stats)
    torch._dynamo.reset()
    torch.compile(lambda a, b, c: a @ b + c, backend=loopfuse_backend, dynamic=True)(a, b, c)
    assert interface.stats["generic_graphs"] == before["generic_graphs"]
    assert interface.stats["eager_graph"] == before["eager_graph"] + 1


def test_work_bound_sends_large_graphs_to_the_captured_ops(tmp_path, monkeypatch):
    fn, make, _, _ = CASES["matmul_add"]
    gm, args, _ = _aten_graph(fn, make())
    prog = generic.GenericProgram(gm)
    monkeypatch.setattr(generic, "MAX_SCALAR_WORK", 100)
    with pytest.raises(emit.NotLowerable, match="scalar work"):
        prog.run(args, launchers=_host_build(prog, tmp_path))


def test_codegen_only_hands_back_the_generated_source(monkeypatch):
    """CODEGEN_ONLY (reference interface.py:615-622): a graph without an attention returns its
    generic program; ``.code`` is the HIP source that would be compiled."""
    from loopfuse_amd import loopfuse_backend
    from loopfuse_amd.torch_backend import interface

    monkeypatch.setattr(interface, "CODEGEN_ONLY", True)
    torch._dynamo.reset()
    prg = torch.compile(lambda a, b, c: a @ b + c, backend=loopfuse_backend, dynamic=True)(
        _r(16, 8), _r(8, 12, seed=1), _r(16, 12, seed=2))
    assert prg.code.count("__global__") == 1 and "lf_gen_0" in prg.code and "LfGenParams" in prg.code


# ---- contractions on the MFMA path (compiler/emit_gemm.py): recognition and code generation, no GPU needed
def _bf16_graph(fn, shapes):
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.fx.experimental.proxy_tensor import make_fx
    with FakeTensorMode():
        return make_fx(fn, tracing_mode="fake")(*[torch.empty(s, dtype=torch.bfloat16) for s in shapes])


def test_contractions_of_half_precision_operands_get_an_mfma_kernel():
    """``a @ b + c`` (reference tests/test_accuracy.py:56-82) on bf16 operands: the nest is recognised as a batched
    matrix product with a pointwise epilogue -- which atoms are rows, columns, the contraction and the batch, and
    which dimension of each operand they index -- and gets a second, MFMA kernel beside the plain one.  fp32
    operands and a gathered operand keep the plain kernel only."""
    from loopfuse_amd.compiler import emit_gemm

    prog = generic.GenericProgram(_bf16_graph(lambda a, b, c: (a @ b.transpose(-1, -2)) * 0.5 + c,
                                              [(4, 96, 64), (4, 40, 64), (40,)]))
    assert list(prog.gemm) == [0]
    k, info = prog.gemm[0]
    assert (info.m.hint, info.n.hint, info.k.hint, [a.hint for a in info.batch]) == (96, 40, 64, [4])
    assert info.a_dims == (1, 2) and info.b_dims == (1, 2) and info.a_batch_dims == [0] and info.b_batch_dims == [0]
    assert "v_mfma" not in k.source and "lfg_mfma" in k.source and "__launch_bounds__(64 * LFG_WGM * LFG_WGN, 2)" in k.source
    assert "accv * 0.5f" in k.source                     # the epilogue is evaluated on the accumulator
    assert prog.code.count("__global__") == 2            # plain + MFMA
    # rows of a [.., M, K] view that matmul flattened: the outer ones count as batch
    prog = generic.GenericProgram(_bf16_graph(lambda a, b: a @ b, [(3, 2, 160, 64), (64, 96)]))
    info = prog.gemm[0][1]
    assert (info.m.hint, info.n.hint, info.k.hint, sorted(a.hint for a in info.batch)) == (160, 96, 64, [2, 3])
    assert info.b_batch_dims == []
    # not served: fp32 operands; softmax(x) @ y (an operand computed in the nest)
    with_fp32 = generic.GenericProgram(_aten_graph(lambda a, b, c: a @ b + c, (_r(16, 8), _r(8, 12, seed=1), _r(16, 12, seed=2)))[0])
    assert not with_fp32.gemm
    # softmax(x) @ y (reference tests/test_accuracy.py:197-211) in bf16: the probabilities stay a bf16 tensor of their
    # own (the rounding eager does) instead of being recomputed inside the contraction, which then runs on MFMA;
    # in fp32 they are inlined as before and the plain kernels serve the graph
    sm = generic.GenericProgram(_bf16_graph(lambda x, y: torch.softmax(x, dim=-1) @ y, [(2, 64, 32), (2, 32, 48)]))
    assert [type(n.stmt).__name__ for n in sm.nests] == ["Accum", "Accum", "Assign", "Assign"] and list(sm.gemm) == [3]
    assert list(sm.torch_dtypes.values()) == [torch.bfloat16]
    sm32 = generic.GenericProgram(_aten_graph(lambda x, y: torch.softmax(x, dim=-1) @ y, (_r(2, 16, 8), _r(2, 8, 12, seed=1)))[0])
    assert len(sm32.nests) == 3 and not sm32.gemm


@pytest.mark.parametrize("shape", ["s", "l"])
@pytest.mark.parametrize("layouts", [(1, 1), (1, 0), (0, 1), (0, 0)])
def test_mfma_kernel_compiles_for_every_operand_layout(shim_built, layouts, shape):
    """The generated source builds for gfx950 with hipRTC in all four layout specialisations and both tile shapes,
    without scratch memory and within the registers of two waves per SIMD."""
    import re
    import subprocess

    from loopfuse_amd.compiler import emit_gemm

    prog = generic.GenericProgram(_bf16_graph(lambda a, b, c: torch.tanh(a @ b + c), [(256, 128), (128, 192), (192,)]))
    opts = list(lowering.COMMON_OPTS) + [f"-DLFG_A_ROWS={layouts[0]}", f"-DLFG_B_ROWS={layouts[1]}"] + emit_gemm.tile_options(shape)
    code, _, _ = runtime.compile_source(prog.gemm_source, "lf_generic_mfma", opts)
    readelf = "/opt/rocm/llvm/bin/llvm-readelf"
    if not os.path.exists(readelf):
        return
    path = os.path.join(os.environ.get("TMPDIR", "/tmp"), f"lf_gemm_{os.getpid()}.hsaco")
    with open(path, "wb") as fh:
        fh.write(code)
    try:
        notes = subprocess.run([readelf, "--notes", path], capture_output=True, text=True, check=True).stdout
    finally:
        os.unlink(path)
    assert int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", notes).group(1)) == 0
    assert int(re.search(r"\.vgpr_count:\s+(\d+)", notes).group(1)) <= 256
    assert int(re.search(r"\.group_segment_fixed_size:\s+(\d+)", notes).group(1)) == {"s": 65536, "l": 131072}[shape]
