"""Known-answer fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU: the oracle reproduces every stored output (so the stored numbers and the oracle
cannot drift apart unnoticed).  GPU: the HIP kernels reproduce them within tolerance.
"""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import attention_oracle as O

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FILES = sorted(glob.glob(os.path.join(HERE, "*.npz")))
MASKS = {0: None, 1: "causal", 2: "sliding"}


def load(path):
    z = np.load(path, allow_pickle=False)
    dtype = torch.bfloat16 if int(z["dtype"]) == 0 else torch.float16
    t = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(dtype)
    case = dict(q=t(z["q"]), k=t(z["k"]), v=t(z["v"]), mask=MASKS[int(z["mask"])], window=int(z["window"]),
                softcap=float(z["softcap"]) or None, expected=torch.from_numpy(z["expected"]),
                table=torch.from_numpy(z["table"]) if "table" in z.files else None, dtype=dtype)
    # optional inputs of the widened graphs
    case["extra"] = {n: t(z[n]) for n in ("score_bias", "out_bias", "q2", "k2") if n in z.files}
    case["denom_add"] = float(z["denom_add"]) if "denom_add" in z.files else 0.0
    case["scale"] = float(z["scale"]) if "scale" in z.files else None
    return case


def test_fixtures_exist():
    assert len(FILES) >= 9


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[:-4] for f in FILES])
def test_oracle_reproduces_fixture(path):
    c = load(path)
    got = O.attention_reference(c["q"], c["k"], c["v"], mask=c["mask"], window=c["window"], softcap=c["softcap"],
                                k_table=c["table"], v_table=c["table"], denom_add=c["denom_add"], scale=c["scale"],
                                **c["extra"])
    assert torch.allclose(got, c["expected"], atol=1e-6, rtol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[:-4] for f in FILES])
def test_kernel_reproduces_fixture(path):
    from loopfuse_amd import lowering

    c = load(path)
    dev = torch.device("cuda:0")
    plan = lowering.AttnPlan(mask=c["mask"], window=c["window"], scale=c["scale"] or c["q"].shape[-1] ** -0.5,
                             softcap=c["softcap"], k_paged=c["table"] is not None, v_paged=c["table"] is not None,
                             denom_add=c["denom_add"])
    tab = None if c["table"] is None else c["table"].to(dev)
    got = lowering.attention(c["q"].to(dev), c["k"].to(dev), c["v"].to(dev), plan, tab, tab,
                             **{n: t.to(dev) for n, t in c["extra"].items()})
    torch.cuda.synchronize()
    tol = 2e-2 if c["dtype"] == torch.bfloat16 else 5e-3
    err = (got.float().cpu() - c["expected"]).abs()
    if "out_bias" in c["extra"]:     # the bias moves the result away from O(1): allow the storage format's half-ulp
        err = err - (2.0 ** -8 if c["dtype"] == torch.bfloat16 else 2.0 ** -11) * c["expected"].abs()
    assert err.max().item() <= tol
