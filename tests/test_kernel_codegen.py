"""Static checks on the code objects of the kernels whose MFMAs are inline asm with explicit
register files (lf_attn_bwd_dkdv, the 4-wave lf_attn_bwd_dq).

The compiler does not know the latency of those MFMAs: a register copy or a spill it decides
to place right behind one reads the accumulator before the result is there, and nothing at run
time says so.  The sources are written so that it has no reason to (every accumulator is pinned
to one register file, the live ranges fit), and this test holds the generated code to it:
compiled as the library compiles them (hipRTC, no GPU needed), disassembled, and checked for
  * no scratch-memory access at all (no spills),
  * every read of an MFMA's AGPR result by a non-MFMA instruction at least MIN_GAP
    instructions behind the MFMA that wrote it, or behind an explicit drain (s_nop >= 9),
  * no instruction other than the chain's own MFMAs touching the VGPR destination of an MFMA
    between that MFMA and the drain behind its chain.
"""
import os
import re
import shutil
import subprocess

import pytest
import torch

from loopfuse_amd import lowering

OBJDUMP = "/opt/rocm/llvm/bin/llvm-objdump"
MIN_GAP = 24     # instructions; 12 wait states for the result plus one MFMA that may run ahead of it

pytestmark = pytest.mark.skipif(not os.path.exists(OBJDUMP) or shutil.which("hipcc") is None,
                                reason="needs the ROCm LLVM tools")


def _kernels(spec):
    code = lowering.compile_spec(spec).code_object
    path = os.path.join(os.environ.get("TMPDIR", "/tmp"), f"lf_codegen_{os.getpid()}.hsaco")
    with open(path, "wb") as fh:
        fh.write(code)
    try:
        text = subprocess.run([OBJDUMP, "-d", path], capture_output=True, text=True, check=True).stdout
    finally:
        os.unlink(path)
    parts = re.split(r"\n[0-9a-f]+ <(\w+)>:\n", text)
    out = {}
    for name, body in zip(parts[1::2], parts[2::2]):
        out[name] = [ln.split("//")[0].strip() for ln in body.splitlines() if ln.strip()]
    return out


def _check(name, lines):
    assert not [ln for ln in lines if ln.startswith("scratch_")], f"{name}: scratch memory accesses (spills)"
    mfma_dst = []           # (index, first, last) of MFMAs with an AGPR destination
    for i, ln in enumerate(lines):
        m = re.match(r"v_mfma_\S+ a\[(\d+):(\d+)\]", ln)
        if m:
            mfma_dst.append((i, int(m.group(1)), int(m.group(2))))
    for i, ln in enumerate(lines):
        m = re.match(r"v_accvgpr_read_b32 v\d+, a(\d+)", ln) or re.match(r"v_accvgpr_mov_b32 a\d+, a(\d+)", ln)
        if not m:
            continue
        reg = int(m.group(1))
        writers = [j for j, lo, hi in mfma_dst if j < i and lo <= reg <= hi]
        if not writers:
            continue
        j = writers[-1]
        between = lines[j + 1:i]
        drained = any(re.match(r"s_nop (\d+)", x) and int(re.match(r"s_nop (\d+)", x).group(1)) >= 9 for x in between)
        assert drained or len(between) >= MIN_GAP, \
            f"{name}: '{ln}' reads a{reg} {len(between)} instructions behind the MFMA that writes it ('{lines[j]}')"
    if not mfma_dst:
        return          # MFMAs issued through the builtin only: the compiler places their wait states itself
    # MFMAs with a VGPR destination (S^T / dP^T): until the drain behind the chain -- or MIN_GAP instructions --
    # nothing but the chain's own MFMAs may touch the destination registers (a copy or a live-range split the
    # compiler placed there would read or overwrite an accumulator that is not written yet)
    for j, ln in enumerate(lines):
        m = re.match(r"v_mfma_\S+ v\[(\d+):(\d+)\]", ln)
        if not m:
            continue
        lo, hi = int(m.group(1)), int(m.group(2))
        for gap, x in enumerate(lines[j + 1:j + 1 + MIN_GAP]):
            nop = re.match(r"s_nop (\d+)", x)
            if nop and int(nop.group(1)) >= 9:
                break
            if x.startswith("v_mfma"):
                continue
            regs = {int(r) for r in re.findall(r"\bv(\d+)\b", x)}
            for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", x):
                regs.update(range(int(a), int(b) + 1))
            hit = sorted(r for r in regs if lo <= r <= hi)
            assert not hit, f"{name}: '{x}' touches v{hit[0]} {gap} instructions behind '{ln}', before its drain"


SPECS = [
    lowering.bwd_spec(torch.bfloat16, 128, lowering.MASK_CAUSAL),
    lowering.bwd_spec(torch.float16, 64, lowering.MASK_NONE),
    lowering.bwd_spec(torch.bfloat16, 128, lowering.MASK_SLIDING),     # 4-wave dQ kernel
    lowering.bwd_spec(torch.float16, 64, lowering.MASK_SLIDING),
    lowering.bwd_spec(torch.bfloat16, 128, lowering.MASK_CAUSAL, True),     # with softcap
    lowering.bwd_spec(torch.float16, 128, lowering.MASK_SLIDING, True),
]


@pytest.mark.parametrize("spec", SPECS, ids=lambda s: s.name()[:48])
def test_no_spills_and_no_early_reads_of_mfma_results(shim_built, spec):
    kernels = _kernels(spec)
    assert kernels
    for name, lines in kernels.items():
        if "delta" in name:
            continue
        assert any(ln.startswith("v_mfma") for ln in lines), name
        _check(name, lines)


def test_the_check_sees_an_early_read():
    lines = ["v_mfma_f32_32x32x16_bf16 a[0:15], v[0:3], v[4:7], a[0:15]", "v_add_u32_e32 v1, v2, v3",
             "v_accvgpr_read_b32 v9, a3"]
    with pytest.raises(AssertionError):
        _check("probe", lines)
    _check("probe", lines[:1] + ["s_nop 9", "s_nop 9"] + lines[1:])
    _check("probe", lines[:1] + ["v_mov_b32_e32 v0, v0"] * MIN_GAP + lines[2:])
    with pytest.raises(AssertionError):
        _check("probe", lines[:2] + ["scratch_load_dword v1, off, s0"])
    # a VGPR-destination MFMA of such a kernel: a copy of its accumulator before the drain is seen, one behind it is not
    chain = ["v_mfma_f32_32x32x16_bf16 a[0:15], v[0:3], v[4:7], a[0:15]",
             "v_mfma_f32_32x32x16_bf16 v[16:31], v[0:3], a[16:19], 0",
             "v_mfma_f32_32x32x16_bf16 v[16:31], v[4:7], a[20:23], v[16:31]"]
    with pytest.raises(AssertionError):
        _check("probe", chain + ["v_mov_b32_e32 v40, v17", "s_nop 9", "s_nop 9"])
    with pytest.raises(AssertionError):
        _check("probe", chain + ["global_load_dwordx4 v[28:31], v[0:1], off", "s_nop 9", "s_nop 9"])
    _check("probe", chain + ["v_add_u32_e32 v1, v2, v3", "s_nop 9", "s_nop 9", "v_mov_b32_e32 v40, v17"])
