"""The allocation-free entry point of the C ABI, ``lf_launch_decode_static``: a split decode
step whose split-K partials live in a static device array of the library.  Its output must be
bit-equal to the step through ``lf_launch`` with a caller-owned scratch buffer (same kernels,
same partials), on two calls in a row, the second with a smaller input; a step whose partials
exceed the array is refused before anything is launched."""
import pytest
import torch

from loopfuse_amd import lowering, runtime, workloads

pytestmark = pytest.mark.gpu


def _step(w, splits, **kw):
    plan = lowering.AttnPlan(scale=w.scale, k_paged=w.k_table is not None, v_paged=w.v_table is not None)
    return lowering.attention(w.q, w.k, w.v, plan, w.k_table, w.v_table, num_splits=splits, **kw)


def test_static_scratch_decode_matches_caller_owned_scratch():
    dev = torch.device("cuda:0")
    first = True
    for name, B, S, splits in (("c5", 16, 2048, 4), ("c5", 4, 512, 2), ("c4", 2, 1024, 4)):
        w = workloads.make(name, seed=7, B=B, S=S).to(dev)
        want = _step(w, splits).clone()
        assert lowering.attention.last_launch["kernels"] == ["lf_attn_decode", "lf_attn_decode_combine"]
        got = torch.full_like(want, float("nan"))
        torch.cuda.synchronize()
        allocs = torch.cuda.memory_stats()["allocation.all.allocated"]
        _step(w, splits, out=got, static_scratch=True)
        assert lowering.attention.last_launch.get("static_scratch") is True
        if not first:       # the first call may load the code object; later calls allocate nothing at all
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == allocs
        first = False
        torch.cuda.synchronize()
        assert torch.equal(got, want), (name, B, S, splits)


def test_static_scratch_refuses_oversized_steps():
    dev = torch.device("cuda:0")
    w = workloads.make("c5", seed=7, B=64, S=2048).to(dev)
    out = torch.empty_like(w.q)
    need = 64 * 8 * 4 * 16 * (128 + 2) * 4
    assert need > runtime.static_scratch_bytes()
    with pytest.raises(runtime.ShimError) as e:
        _step(w, 16, out=out, static_scratch=True)
    assert e.value.code == -4 and "static scratch" in str(e.value)
    # and an unsplit step is not what this entry point is for
    with pytest.raises(lowering.UnsupportedPlan):
        _step(w, 1, out=out, static_scratch=True)
