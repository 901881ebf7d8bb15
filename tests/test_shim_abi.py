"""The C-ABI library: loads, exports every symbol include/lf_shim.h declares, and its
host-side entry points (compile, cache, error reporting) behave.  No GPU, no launches."""
import ctypes
import os
import re

import pytest

from loopfuse_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "lf_shim.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lf_[a-z0-9_]+)\s*\(", text)))


def test_exports_every_declared_symbol(shim_built):
    syms = header_symbols()
    assert len(syms) >= 13
    for s in syms:
        assert hasattr(shim_built, s), f"{s} declared in lf_shim.h but not exported"
    assert sorted(runtime.ABI_SYMBOLS) == syms
    assert shim_built.lf_abi_version() == 2


def test_compile_without_gpu_and_cache(shim_built, tmp_path):
    src = 'extern "C" __global__ void k(float* x) { x[threadIdx.x] *= 2.0f; }'
    code, hit, log = runtime.compile_source(src, "unit_k", ["-O3"], "gfx950", str(tmp_path))
    assert code[:4] == b"\x7fELF" and not hit
    code2, hit2, _ = runtime.compile_source(src, "unit_k", ["-O3"], "gfx950", str(tmp_path))
    assert hit2 and code2 == code
    # a different option is a different cache entry
    _, hit3, _ = runtime.compile_source(src, "unit_k", ["-O2"], "gfx950", str(tmp_path))
    assert not hit3
    assert len(os.listdir(tmp_path)) == 2


def test_compile_error_is_reported(shim_built):
    with pytest.raises(runtime.ShimError) as e:
        runtime.compile_source("this is not HIP", "bad", [], "gfx950", None)
    assert e.value.code != 0
    assert "error" in str(e.value).lower()


def test_bad_arguments_are_rejected(shim_built):
    L = shim_built
    assert L.lf_launch(None, 1, 1, 1, 64, 1, 1, 0, None, None) == -1
    assert b"null function" in L.lf_last_error()
    fn = ctypes.c_void_p()
    assert L.lf_get_function(ctypes.c_void_p(1234), b"k", ctypes.byref(fn)) == -1
    assert L.lf_module_unload(ctypes.c_void_p(1234)) == -1
    mod = ctypes.c_void_p()
    assert L.lf_module_load(None, 0, ctypes.byref(mod)) == -1


def test_launch_geometry_checks(shim_built):
    L = shim_built
    dummy = ctypes.c_void_p(1)
    assert L.lf_launch(dummy, 0, 1, 1, 64, 1, 1, 0, None, None) == -1
    assert L.lf_launch(dummy, 1, 1, 1, 2048, 1, 1, 0, None, None) == -1
    assert L.lf_launch(dummy, 1, 1, 1, 64, 1, 1, 200 * 1024, None, None) == -1


def test_params_struct_layout():
    from loopfuse_amd.lowering import AttnParams

    # 13 pointers, 26 int64 strides / spans, 12 ints, 3 floats (+4 bytes tail padding to the 8-byte alignment)
    assert AttnParams.q.offset == 0 and AttnParams.q2.offset == 88 and AttnParams.q_sb.offset == 104
    assert AttnParams.q2_sb.offset == 104 + 144
    assert AttnParams.k_span.offset == 104 + 192
    assert AttnParams.B.offset == 104 + 208
    assert AttnParams.k2_group.offset == 104 + 208 + 44
    assert AttnParams.scale.offset == 104 + 208 + 48
    assert AttnParams.denom_add.offset == 104 + 208 + 48 + 8
    assert ctypes.sizeof(AttnParams) == 376


@pytest.mark.parametrize("host,mirror,device,source", [
    ("LfAttnParamsHost", "AttnParams", "LfAttnParams", "lf_common.hip.h"),
    ("LfAttnBwdParamsHost", "AttnBwdParams", "LfAttnBwdParams", "lf_attn_bwd.hip"),
])
def test_c_header_matches_the_ctypes_mirror_and_the_device_struct(tmp_path, host, mirror, device, source):
    """include/lf_attn_params.h (C hosts), the ctypes structure of lowering.py and the device
    struct list the same fields at the same offsets."""
    import subprocess

    from loopfuse_amd import lowering

    mirror = getattr(lowering, mirror)
    names = [n for n, _ in mirror._fields_]
    prog = "#include <stdio.h>\n#include <stddef.h>\n#include \"lf_attn_params.h\"\nint main(void) {\n"
    for n in names:
        prog += f'  printf("{n} %zu\\n", offsetof({host}, {n}));\n'
    prog += f'  printf("sizeof %zu\\n", sizeof({host}));\n  return 0;\n}}\n'
    src = tmp_path / "off.c"
    src.write_text(prog)
    exe = tmp_path / "off"
    subprocess.run(["gcc", "-std=c11", "-I" + os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = dict(line.split() for line in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.splitlines())
    for n in names:
        assert int(out[n]) == getattr(mirror, n).offset, n
    assert int(out["sizeof"]) == ctypes.sizeof(mirror)
    # the device struct declares the same field names in the same order
    dev = open(os.path.join(ROOT, "loopfuse_amd", "csrc", "kernels", source)).read()
    body = dev[dev.index("struct %s {" % device):]
    body = re.sub(r"//[^\n]*", "", body[:body.index("};")])
    fields = []
    for decl in body.split("{", 1)[1].split(";"):
        decl = decl.strip()
        if decl:
            fields += [re.sub(r"[^A-Za-z0-9_]", "", x.split()[-1]) for x in decl.split(",")]
    assert fields == names
