"""A pure-C host (tests/abi_client/lf_client.c: no Python, no torch in the process) compiles,
loads and launches both prefill kernels and the paged decode kernel through include/lf_shim.h and
include/lf_attn_params.h and checks them against double-precision loops."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLIENT = os.path.join(ROOT, "tests", "abi_client", "lf_client")
KERNELS = os.path.join(ROOT, "loopfuse_amd", "csrc", "kernels")

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("which", ["prefill", "prefill_swp", "decode"])
def test_c_host_runs_the_kernels_through_the_c_abi(which):
    assert os.path.exists(CLIENT), "tests/abi_client/lf_client is not built (run __graft_entry__.build())"
    r = subprocess.run([CLIENT, KERNELS, which], capture_output=True, text=True, timeout=110)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, f"lf_client {which} failed ({r.returncode}): {r.stdout}\n{r.stderr}"
    assert "OK" in r.stdout and "max abs err" in r.stdout
