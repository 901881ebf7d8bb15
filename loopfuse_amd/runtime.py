"""ctypes binding of the C-ABI shim (``liblf_shim.so``, declared in ``include/lf_shim.h``).

This is the only place Python touches native code.  It replaces the reference's
"write the generated Triton module to a temp file and import it" step
(reference ``loopfuse/torch_backend/interface.py:624-638``): HIP source goes in,
a loaded gfx950 kernel handle comes out, and launches go to the HIP stream
PyTorch is currently using.

There is no fallback: if the shim is not built, or a launch is attempted
without a GPU, a ``RuntimeError`` is raised.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import Sequence

import torch  # noqa: F401  (loaded first so the shim binds to torch's HIP runtime)

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SHIM_PATH = os.path.join(_PKG_DIR, "liblf_shim.so")
KERNEL_DIR = os.path.join(_PKG_DIR, "csrc", "kernels")
CACHE_DIR = os.environ.get("LOOPFUSE_CACHE_DIR", os.path.join(_PKG_DIR, "_cache"))
DEFAULT_ARCH = "gfx950"

# symbols include/lf_shim.h declares; tests check that all of them are exported
ABI_SYMBOLS = (
    "lf_abi_version",
    "lf_last_error",
    "lf_compile",
    "lf_compile_cached",
    "lf_free_code",
    "lf_module_load",
    "lf_get_function",
    "lf_module_unload",
    "lf_launch",
    "lf_launch_decode_static",
    "lf_static_scratch_bytes",
    "lf_device_info",
    "lf_device_count",
)

_lib = None
_lib_lock = threading.Lock()


class ShimError(RuntimeError):
    """A C-ABI call returned non-zero; carries the code and ``lf_last_error()``."""

    def __init__(self, what: str, code: int, message: str):
        super().__init__(f"{what} failed with code {code}: {message}")
        self.code = code
        self.message = message


def lib() -> ctypes.CDLL:
    """Load the shim once and declare its prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(SHIM_PATH):
            raise RuntimeError(
                f"{SHIM_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(loopfuse_amd has no non-HIP fallback)"
            )
        L = ctypes.CDLL(SHIM_PATH)
        c_char_pp = ctypes.POINTER(ctypes.c_char_p)
        L.lf_abi_version.restype = ctypes.c_int
        L.lf_last_error.restype = ctypes.c_char_p
        L.lf_compile.restype = ctypes.c_int
        L.lf_compile.argtypes = [
            ctypes.c_char_p, ctypes.c_char_p, c_char_pp, ctypes.c_int, ctypes.c_char_p,
            ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_size_t),
            ctypes.c_char_p, ctypes.c_size_t,
        ]
        L.lf_compile_cached.restype = ctypes.c_int
        L.lf_compile_cached.argtypes = [
            ctypes.c_char_p, ctypes.c_char_p, c_char_pp, ctypes.c_int, ctypes.c_char_p,
            ctypes.c_char_p,
            ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_size_t),
            ctypes.POINTER(ctypes.c_int), ctypes.c_char_p, ctypes.c_size_t,
        ]
        L.lf_free_code.restype = None
        L.lf_free_code.argtypes = [ctypes.c_void_p]
        L.lf_module_load.restype = ctypes.c_int
        L.lf_module_load.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
        L.lf_get_function.restype = ctypes.c_int
        L.lf_get_function.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
        L.lf_module_unload.restype = ctypes.c_int
        L.lf_module_unload.argtypes = [ctypes.c_void_p]
        L.lf_launch.restype = ctypes.c_int
        L.lf_launch.argtypes = [ctypes.c_void_p] + [ctypes.c_uint] * 7 + [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
        L.lf_launch_decode_static.restype = ctypes.c_int
        L.lf_launch_decode_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                              ctypes.c_size_t, ctypes.c_size_t] + [ctypes.c_uint] * 5 + [ctypes.c_void_p]
        L.lf_static_scratch_bytes.restype = ctypes.c_size_t
        L.lf_device_info.restype = ctypes.c_int
        L.lf_device_info.argtypes = [
            ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t,
            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
        ]
        L.lf_device_count.restype = ctypes.c_int
        _lib = L
        return L


def _check(what: str, rc: int) -> None:
    if rc != 0:
        raise ShimError(what, rc, lib().lf_last_error().decode("utf-8", "replace"))


def compile_source(src: str, name: str, opts: Sequence[str], arch: str | None = DEFAULT_ARCH,
                   cache_dir: str | None = CACHE_DIR) -> tuple[bytes, bool, str]:
    """HIP source -> code object bytes via hipRTC.  Returns (code, cache_hit, log)."""
    L = lib()
    arr = (ctypes.c_char_p * max(len(opts), 1))(*[o.encode() for o in opts])
    code = ctypes.c_void_p()
    size = ctypes.c_size_t()
    hit = ctypes.c_int(0)
    log = ctypes.create_string_buffer(1 << 16)
    if cache_dir:
        os.makedirs(cache_dir, exist_ok=True)
    rc = L.lf_compile_cached(
        src.encode(), name.encode(), arr, len(opts), (arch or "").encode(),
        (cache_dir or "").encode(), ctypes.byref(code), ctypes.byref(size), ctypes.byref(hit),
        log, len(log),
    )
    _check(f"lf_compile[{name}]", rc)
    try:
        data = ctypes.string_at(code.value, size.value)
    finally:
        L.lf_free_code(code)
    return data, bool(hit.value), log.value.decode("utf-8", "replace")


def current_stream_handle() -> int:
    """hipStream_t of torch's current stream on the current device, as an integer
    (the raw accessor: the launch path is called once per kernel)."""
    try:
        return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())
    except AttributeError:            # older / newer torch without the raw accessor
        return torch.cuda.current_stream().cuda_stream


class Kernel:
    """A kernel of a loaded module; ``launch`` passes ONE by-value struct argument."""

    def __init__(self, module: "Module", symbol: str):
        self.module = module  # keeps the module alive
        self.symbol = symbol
        fn = ctypes.c_void_p()
        _check(f"lf_get_function[{symbol}]", lib().lf_get_function(module.handle, symbol.encode(), ctypes.byref(fn)))
        self.handle = fn
        self._launch = lib().lf_launch

    def launch(self, grid: tuple[int, int, int], block: tuple[int, int, int], params: ctypes.Structure,
               stream: int | None = None, lds_bytes: int = 0) -> None:
        if stream is None:
            stream = current_stream_handle()
        args = (ctypes.c_void_p * 1)(ctypes.addressof(params))
        rc = self._launch(self.handle, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                          lds_bytes, ctypes.c_void_p(stream), args)
        if rc:
            _check(f"lf_launch[{self.symbol}]", rc)


def launch_decode_static(decode: Kernel, combine: Kernel, params: ctypes.Structure, part_acc_bytes: int,
                         part_ml_bytes: int, grid: tuple[int, int], block: int, combine_grid: int,
                         combine_block: int, stream: int | None = None) -> None:
    """One split decode step through ``lf_launch_decode_static``: both kernels, with the
    split-K partials in the library's static device array (nothing is allocated)."""
    if stream is None:
        stream = current_stream_handle()
    rc = lib().lf_launch_decode_static(decode.handle, combine.handle, ctypes.addressof(params), ctypes.sizeof(params),
                                       part_acc_bytes, part_ml_bytes, grid[0], grid[1], block,
                                       combine_grid, combine_block, ctypes.c_void_p(stream))
    if rc:
        _check("lf_launch_decode_static", rc)


def static_scratch_bytes() -> int:
    return int(lib().lf_static_scratch_bytes())


class Module:
    """A code object loaded on the current device."""

    def __init__(self, code: bytes):
        self.code = code
        h = ctypes.c_void_p()
        _check("lf_module_load", lib().lf_module_load(code, len(code), ctypes.byref(h)))
        self.handle = h

    def kernel(self, symbol: str) -> Kernel:
        return Kernel(self, symbol)

    def unload(self) -> None:
        if self.handle:
            _check("lf_module_unload", lib().lf_module_unload(self.handle))
            self.handle = None


def device_info(dev: int = 0) -> dict:
    arch = ctypes.create_string_buffer(64)
    cus = ctypes.c_int()
    lds = ctypes.c_int()
    _check("lf_device_info", lib().lf_device_info(dev, arch, len(arch), ctypes.byref(cus), ctypes.byref(lds)))
    return {"arch": arch.value.decode(), "compute_units": cus.value, "lds_bytes": lds.value}


def device_count() -> int:
    return int(lib().lf_device_count())


def read_kernel_source(*files: str) -> str:
    """Concatenate building-block files from csrc/kernels into one hipRTC translation unit.

    With ``USE_HARDCODE_KERNEL=1`` a file ``hardcode_kernel.hip`` in the current
    directory replaces the last (kernel) file -- the debugging hook the reference
    offers with ``hardcode_kernel.py`` (``loopfuse/torch_backend/interface.py:606-613``).
    """
    parts = []
    hard = os.path.join(os.getcwd(), "hardcode_kernel.hip")
    use_hard = os.environ.get("USE_HARDCODE_KERNEL", "0") == "1" and os.path.exists(hard)
    for i, f in enumerate(files):
        path = hard if (use_hard and i == len(files) - 1) else os.path.join(KERNEL_DIR, f)
        with open(path, "r") as fh:
            parts.append(f"// ---- {os.path.basename(path)}\n" + fh.read())
    return "\n".join(parts)
