"""Lowering: attention plan -> specialised gfx950 HIP kernel -> launcher.

This module is the counterpart of the reference's Triton emitter
(``loopfuse/codegen.py:100-126`` ``codegen_program`` and the generated
``launch_kernel_0``, ``codegen.py:215-298``).  Instead of printing a kernel per
graph it selects hand-written building blocks from ``csrc/kernels`` and
specialises them with ``-D`` options (dtype, head dim, mask kind, softcap,
paging, rows per unit); hipRTC compiles the result once per specialisation and
the code object is cached on disk.

Everything dynamic (batch, heads, sequence lengths, strides, scale, window,
softcap value) is a run-time kernel parameter, so a new sequence length does not
recompile (the reference makes every dimension a ``tl.constexpr``,
``codegen.py:394-396``).
"""
from __future__ import annotations

import ctypes
import dataclasses
import functools
import json
import math
import os
import threading
from typing import Optional

import torch

from . import runtime
from .skip import TILE_SHAPES

MASK_NONE, MASK_CAUSAL, MASK_SLIDING = 0, 1, 2
DECODE_QROWS = 16    # query rows one decode unit holds (the MFMA N dimension)
_MASK_NAMES = {"none": MASK_NONE, None: MASK_NONE, "causal": MASK_CAUSAL, "sliding": MASK_SLIDING}
_DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1}

# hipcc/hipRTC flags common to every kernel.  Packed-FP32 instruction selection
# (v_pk_*_f32) is switched off on purpose: scalar fp32 VALU code only.
COMMON_OPTS = ("-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")


class AttnParams(ctypes.Structure):
    """Mirror of ``struct LfAttnParams`` in csrc/kernels/lf_common.hip.h."""

    _fields_ = (
        [(n, ctypes.c_void_p) for n in ("q", "k", "v", "o", "k_table", "v_table", "part_acc", "part_ml", "visits", "bias", "obias",
                                        "q2", "k2")]
        + [(n, ctypes.c_longlong) for n in (
            "q_sb", "q_sh", "q_ss", "k_sb", "k_sh", "k_ss", "v_sb", "v_sh", "v_ss", "o_sb", "o_sh", "o_ss",
            "bias_sb", "bias_sh", "bias_sq", "ob_sb", "ob_sh", "ob_sq",
            "q2_sb", "q2_sh", "q2_ss", "k2_sb", "k2_sh", "k2_ss", "k_span", "v_span")]
        + [(n, ctypes.c_int) for n in (
            "B", "Hq", "Hkv", "Sq", "Sk", "window", "kt_stride", "vt_stride", "nsplit", "rows", "split_len", "k2_group")]
        + [("scale", ctypes.c_float), ("softcap", ctypes.c_float), ("denom_add", ctypes.c_float)]
    )


@dataclasses.dataclass(frozen=True)
class KernelSpec:
    """Compile-time specialisation of one kernel family (= one code object)."""

    family: str            # "prefill" | "prefill_swp" | "decode" | "bwd"
    dtype: int             # 0 bf16, 1 fp16
    head_dim: int          # 64 | 128
    mask: int = MASK_NONE
    softcap: bool = False
    paged: int = 0         # bit 0: K paged, bit 1: V paged
    page_size: int = 1
    table_i64: bool = False
    rows: int = 1          # decode: query rows a unit can hold (fixed, the MFMA N dimension)
    waves: int = 4         # decode: waves per workgroup
    v_tr: bool = True      # prefill: transposed LDS reads for V
    headwave: bool = False  # decode: one kv head per wave (8 waves) instead of 4 waves sharing a head
    coop: bool = False     # decode, headwave: the workgroup loads whole 16-token blocks, rows reach the waves through LDS
    rowload: bool = False  # decode, register-staged path: whole-row non-temporal loads, K through a wave-private LDS tile
    denom: bool = False    # prefill: softmax denominator sum + c (c a run-time parameter)
    bias: int = 0          # prefill: bit 0 additive score bias tensor, bit 1 additive output bias tensor, bit 2 unaligned rows
    pack: int = 0          # prefill_swp, grouped-query attention: a workgroup's waves take 2 or 4 heads of one group
    page_size_v: int = 0   # tokens per page of the V pool when it differs from K's (0 = same)
    d2: int = 0            # prefill: depth of a second score product Q2 K2^T (0, 16, 32, 64)
    safe: bool = False     # rows that saw no key come out as zeros instead of NaN
    bn: int = 0            # prefill_swp: keys per LDS tile, 32 (three workgroups per CU) or 0 / 64 (two)
    extra: tuple = ()      # further -D options (tuning experiments)

    def options(self) -> list[str]:
        o = list(COMMON_OPTS) + [
            f"-DLF_DTYPE={self.dtype}",
            f"-DLF_HEAD_DIM={self.head_dim}",
            f"-DLF_MASK={self.mask}",
            f"-DLF_SOFTCAP={int(self.softcap)}",
            f"-DLF_PAGED={self.paged}",
            f"-DLF_PAGE_SIZE={self.page_size}",
            f"-DLF_TABLE_I64={int(self.table_i64)}",
        ]
        if self.page_size_v:
            o += [f"-DLF_PAGE_SIZE_V={self.page_size_v}"]
        if self.family == "decode":
            o += [f"-DLF_DW={self.waves}", f"-DLF_HEADWAVE={int(self.headwave)}"]
            if self.coop:
                o += ["-DLF_COOP=1"]
            if self.rowload:
                o += ["-DLF_ROWLOAD=1"]
            if self.bias:
                o += ["-DLF_BIAS=1"]
        elif self.family == "prefill":
            o += [f"-DLF_V_TR={int(self.v_tr)}", f"-DLF_BIAS={self.bias}", f"-DLF_DENOM={int(self.denom)}"]
            if self.d2:
                o += [f"-DLF_D2={self.d2}"]
        elif self.family == "prefill_swp":
            if self.bn == 32:
                # 32-key tiles: 40 KB of LDS and <= 168 registers, so three workgroups share a CU
                o += ["-DLF_BN=32", "-DLF_WPE=3", "-DLF_KPF=3", "-DLF_VPF=2"]
            if self.pack:
                o += [f"-DLF_GQAPACK={int(self.pack)}"]
            if self.bias:
                o += ["-DLF_BIAS=1"]
        if self.safe:
            o += ["-DLF_SAFE=1"]
        return o + list(self.extra)

    def files(self) -> tuple[str, ...]:
        kernel = {"prefill": "lf_attn_prefill.hip", "prefill_swp": "lf_attn_prefill_swp.hip",
                  "decode": "lf_attn_decode.hip", "bwd": "lf_attn_bwd.hip"}[self.family]
        if self.family == "decode":
            return ("lf_common.hip.h", kernel)
        # the two prefill kernels: their own tuning macros come first (the shared blocks use LF_BN)
        if self.family == "prefill_swp" and self.bias:
            # one code object holds the attention kernel and the kernel that classifies the bias tiles for it
            return ("lf_common.hip.h", "lf_prefill_blocks.hip.h", kernel, "lf_bias_classify.hip")
        return ("lf_common.hip.h", "lf_prefill_blocks.hip.h", kernel)

    def entry(self) -> str:
        return {"prefill": "lf_attn_prefill", "prefill_swp": "lf_attn_prefill_swp", "decode": "lf_attn_decode",
                "bwd": "lf_attn_bwd_dq"}[self.family]

    def name(self) -> str:
        return (f"lf_{self.family}_t{self.dtype}_d{self.head_dim}_m{self.mask}_c{int(self.softcap)}"
                f"_p{self.paged}x{self.page_size}i{int(self.table_i64)}_r{self.rows}w{self.waves}v{int(self.v_tr)}h{int(self.headwave)}b{self.bias}n{int(self.denom)}"
                + (f"_q{self.d2}" if self.d2 else "") + (f"_gp{int(self.pack)}" if self.pack else "") + (f"_pv{self.page_size_v}" if self.page_size_v else "")
                + ("_z" if self.safe else "") + (f"_bn{self.bn}" if self.bn else "") + ("_co" if self.coop else "") + ("_rl" if self.rowload else "")
                + "".join("_" + e.replace("-D", "").replace("=", "") for e in self.extra))

    def source(self) -> str:
        return runtime.read_kernel_source(*self.files())


@dataclasses.dataclass
class CompiledKernel:
    """What ``CODEGEN_ONLY`` returns in place of a runnable function (the
    reference returns ``KernelData(kernel_name, launch_name, code)``,
    ``loopfuse/codegen.py:66-71``)."""

    spec: KernelSpec
    code_object: bytes
    cache_hit: bool
    log: str

    @property
    def code(self) -> str:
        return "// options: " + " ".join(self.spec.options()) + "\n" + self.spec.source()


class CompiledKernels(list):
    """What a ``CODEGEN_ONLY`` call returns: the ``CompiledKernel`` of every fused call in
    the graph.  ``.code`` joins their sources, so the reference's usage
    ``print(compiled_fn(Q, K, V).code)`` (``tests/test_attention.py:28-29``) works as is."""

    @property
    def code(self) -> str:
        return "\n".join(k.code for k in self)


_compiled: dict[KernelSpec, CompiledKernel] = {}
_loaded: dict[tuple[KernelSpec, int], runtime.Module] = {}
_lock = threading.Lock()


def compile_spec(spec: KernelSpec, arch: str = runtime.DEFAULT_ARCH) -> CompiledKernel:
    """hipRTC-compile (or fetch from the on-disk cache) one specialisation.  Needs no GPU."""
    with _lock:
        ck = _compiled.get(spec)
    if ck is not None:
        return ck
    # outside the lock: different specialisations compile concurrently (the shim is re-entrant;
    # two threads asking for the same one both compile, the results are identical)
    code, hit, log = runtime.compile_source(spec.source(), spec.name(), spec.options(), arch)
    ck = CompiledKernel(spec, code, hit, log)
    record = os.environ.get("LOOPFUSE_RECORD_SPECS")
    with _lock:
        if record and spec not in _compiled:
            # one JSON line per specialisation a workload asked for: specs_from_file() reads
            # them back, so a deployment can fill the code-object cache ahead of time
            with open(record, "a") as fh:
                fh.write(json.dumps(dataclasses.asdict(spec), sort_keys=True) + "\n")
        return _compiled.setdefault(spec, ck)


def specs_from_file(path: str) -> list[KernelSpec]:
    """Specialisations recorded with ``LOOPFUSE_RECORD_SPECS=<path>`` (duplicates dropped)."""
    seen: dict[KernelSpec, None] = {}
    with open(path) as fh:
        for line in fh:
            if line.strip():
                d = json.loads(line)
                d["extra"] = tuple(d.get("extra", ()))
                seen.setdefault(KernelSpec(**d))
    return list(seen)


def load_spec(spec: KernelSpec) -> runtime.Module:
    dev = torch.cuda.current_device()
    key = (spec, dev)
    mod = _loaded.get(key)
    if mod is None:
        ck = compile_spec(spec)
        with _lock:
            mod = _loaded.get(key)
            if mod is None:
                mod = runtime.Module(ck.code_object)
                _loaded[key] = mod
    return mod


_kernels: dict[tuple[KernelSpec, int, str], runtime.Kernel] = {}


def get_kernel(spec: KernelSpec, symbol: str) -> runtime.Kernel:
    key = (spec, torch.cuda.current_device(), symbol)
    k = _kernels.get(key)
    if k is None:
        k = load_spec(spec).kernel(symbol)
        _kernels[key] = k
    return k


# ----------------------------------------------------------------------------
# plan
# ----------------------------------------------------------------------------

@dataclasses.dataclass
class AttnPlan:
    """What the front end extracts from a captured graph: the parameters of
    ``softmax(mask(mods(Q K^T))) V``.  ``scale`` multiplies the raw scores,
    ``softcap`` (if set) is applied as cap*tanh(s/cap) after scaling and before
    the mask, exactly the order of the reference graphs
    (``tests/benchmark.py:142-147``)."""

    mask: str | None = None            # None | "causal" | "sliding"
    window: int = 0
    scale: float = 1.0
    softcap: float | None = None
    k_paged: bool = False
    v_paged: bool = False
    denom_add: float = 0.0             # probabilities are e^(x-max) / (sum e^(x-max) + denom_add)
    zero_blind_rows: bool = False      # a row whose keys are all masked by the score bias gives zeros (as torch's
                                       # fused attention ops do) instead of the NaN of a softmax over -inf


class UnsupportedPlan(ValueError):
    """The shapes/dtypes cannot be served by the HIP kernels (caller falls back to eager)."""


def _check_tensor(name: str, t: torch.Tensor, dtype: torch.dtype) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"loopfuse_amd: {name} is not on the GPU; the HIP path has no CPU fallback")
    if t.dtype != dtype:
        raise UnsupportedPlan(f"{name} has dtype {t.dtype}, expected {dtype}")
    if t.data_ptr() % 16:
        raise UnsupportedPlan(f"{name} is not 16-byte aligned")
    if t.is_contiguous() and t.shape[-1] % 8 == 0:
        return
    if t.stride(-1) != 1:
        raise UnsupportedPlan(f"{name} must have unit stride in its last dimension")
    for n, s in zip(t.shape[:-1], t.stride()[:-1]):
        if n > 1 and s % 8:
            raise UnsupportedPlan(f"{name} strides must be multiples of 8 elements (16-byte loads)")


_scratch: dict[tuple[int, int], torch.Tensor] = {}


def _get_scratch(device: torch.device, nfloats: int) -> torch.Tensor:
    """Split-K scratch, one buffer per (device, stream): launches on one stream are
    ordered, so they can share it; launches on different streams must not."""
    key = (device.index or 0, runtime.current_stream_handle())
    t = _scratch.get(key)
    if t is None or t.numel() < nfloats:
        t = torch.empty(max(nfloats, 1 << 20), dtype=torch.float32, device=device)
        _scratch[key] = t
    return t


PREFILL_QGROUP = 8      # LF_QGROUP of lf_attn_prefill_swp.hip (its default)
BWD_GROUP = 4           # LF_BW_GROUP of lf_attn_bwd.hip (its default)


def decode_split(units: int, Sk: int, cus: int = 256, per_cu: int = 2) -> int:
    """Number of KV splits across workgroups.  One workgroup per unit is enough once
    there are ``per_cu`` workgroups per CU (8 resident waves, each with 32 KB of loads
    in flight: two workgroups of 4 waves, or one of 8); below that the KV range is
    split, down to 512 tokens per split and up to 64 splits, and a second kernel merges
    the partial results."""
    env = os.environ.get("LOOPFUSE_DECODE_SPLITS")
    if env:
        return max(1, int(env))
    want = max(1, (per_cu * cus + units - 1) // units)
    if want > 4:
        # few units (small batch, long context): one workgroup per CU measured best
        want = max(4, (cus + units - 1) // units)
    most = max(1, min(64, Sk // 512))      # measured: >= 512 tokens per split, at most 64 splits
    return max(1, min(want, most))


def _decode_headwave(paged: int, page_size: int, Hkv: int, D: int, P: "AttnParams", units_hw: int = 1 << 30,
                     Sk: int = 1 << 30, cus: int = 256) -> bool:
    """One kv head per wave pays when K and V are paged, token-major (head stride D,
    token stride Hkv*D), there are at least 8 heads to fill the 8 waves, and the
    (batch, head-chunk) units times at most 8 KV splits of >= 256 tokens still give one
    workgroup per CU (measured: below that, 4 waves per head with more splits win)."""
    env = os.environ.get("LOOPFUSE_DECODE_HEADWAVE")
    if env is not None:
        return env == "1"
    return (paged == 3 and Hkv % 8 == 0 and P.k_sh == D and P.v_sh == D
            and P.k_ss == Hkv * D and P.v_ss == Hkv * D
            and units_hw * max(1, min(8, Sk // 512)) >= cus)


def _decode_coop(headwave: bool, page_size: int, page_size_v: int, bias_bits: int, Hkv: int, waves: int,
                 P: "AttnParams", D: int) -> bool:
    """With one kv head per wave the workgroup reads every 16-token block of its 8 heads as one
    contiguous piece and hands the rows to the waves through LDS (``-DLF_COOP=1``) when a block
    lies inside a page (pages of a multiple of 16 tokens) and there is no score bias to carry
    along: a wave that fetches its own head reads 256-byte pieces 2 KB apart, which costs about a
    tenth of the HBM rate.  LOOPFUSE_DECODE_COOP=0 keeps the per-wave loads."""
    if os.environ.get("LOOPFUSE_DECODE_COOP", "1") != "1":
        return False
    # the block loads take a token's 8 heads as one run of 8 * D elements: the pool must hold the heads of a
    # token side by side (a permuted [pages, Hkv, page, D] pool view goes to the per-wave loads, which follow
    # the head stride)
    token_major = P.k_sh == D and P.v_sh == D and P.k_ss >= Hkv * D and P.v_ss >= Hkv * D
    return headwave and page_size % 16 == 0 and not page_size_v and not bias_bits and Hkv % waves == 0 and token_major


def _decode_rowload(paged: int, page_size: int, page_size_v: int, bias_bits: int) -> bool:
    """The register-staged decode path reads whole rows (every 128-byte line in one piece) with
    non-temporal loads and passes K through a wave-private LDS tile (``-DLF_ROWLOAD=1``) when a
    16-token step lies inside one page (or K/V are dense) and there is no score bias.
    LOOPFUSE_DECODE_ROWLOAD=0 keeps the loads in MFMA operand layout."""
    if os.environ.get("LOOPFUSE_DECODE_ROWLOAD", "1") != "1" or bias_bits:
        return False
    return not paged or (page_size % 16 == 0 and (page_size_v or page_size) % 16 == 0)


def prefill_kv_tile(D: int, bias_bits: int = 0, choice: Optional[dict] = None, workgroups: int = 1 << 30) -> int:
    """Keys per LDS tile of lf_attn_prefill_swp: 0 (the kernel's 64) or 32.  With 32-key tiles a
    workgroup needs 40 KB of LDS and at most 168 registers per lane, so three workgroups instead of
    two share a CU; at head dimension 128 that outweighs the second barrier per 64 keys (config 2
    -2.5 %, config 3 -10 %) once the launch has three workgroups for every CU -- a launch of 128
    workgroups is a quarter slower with them -- and at head dimension 64 it does not.  The bias tile
    classes are per 64 keys, so biased calls keep 64.  ``choice["bn"]`` (the tuner) or
    ``LOOPFUSE_BN`` override the default."""
    if bias_bits:
        return 0
    want = (choice or {}).get("bn", os.environ.get("LOOPFUSE_BN"))
    if want is not None:
        return 32 if int(want) == 32 else 0
    return 32 if D == 128 and workgroups >= 3 * 256 else 0


def prefill_variant(Sq: int, v_tr: bool = True) -> str:
    """Which prefill kernel serves a call.  Default: the software-pipelined kernel
    with direct-to-LDS staging (``prefill_swp``; dense K/V only, ``attention`` falls
    back to ``prefill`` for paged operands).  LOOPFUSE_PREFILL=w32 selects the
    register-staged kernel for comparison."""
    env = os.environ.get("LOOPFUSE_PREFILL", "swp")
    if not v_tr or env == "w32":
        return "prefill"
    return "prefill_swp"


# ---------------------------------------------------------------------------
# launch-heuristic tuning (the reference autotunes tile sizes with triton.autotune,
# loopfuse/codegen.py:355-404; the HIP kernels have fixed tiles, what varies here is
# which kernel variant and which work split serve a shape)
# ---------------------------------------------------------------------------
_tuned: dict = {}
_TUNE_FILE = os.path.join(runtime.CACHE_DIR, "autotune.json")


def _tune_key(q, k, plan: AttnPlan, k_table, bias_bits: int) -> str:
    B, Hq, Sq, D = q.shape
    if plan.k_paged:
        Hkv = k.shape[-2]
        Sk = k_table.shape[1] * (k.shape[1] if k.dim() == 4 else 1)
        ps = k.shape[1] if k.dim() == 4 else 1
    else:
        Hkv, Sk, ps = k.shape[1], k.shape[2], 0
    bucket = lambda n: 1 << max(0, (int(n) - 1)).bit_length()       # next power of two
    return (f"{q.dtype}|D{D}|m{plan.mask}|c{int(plan.softcap is not None)}|p{int(plan.k_paged)}{int(plan.v_paged)}x{ps}"
            f"|B{bucket(B * Hkv)}|g{Hq // Hkv}|q{bucket(Sq)}|k{bucket(Sk)}|b{bias_bits}")


def _load_tuned() -> None:
    if not _tuned and os.path.exists(_TUNE_FILE):
        try:
            import json
            with open(_TUNE_FILE) as fh:
                _tuned.update(json.load(fh))
        except (OSError, ValueError):
            pass


def tuned_attention(q, k, v, plan: AttnPlan, k_table=None, v_table=None, **kw):
    """``attention`` with the launch heuristics chosen by measurement: on the first call
    of a shape class each candidate is timed on the call's own tensors (HIP events, a few
    launches), the winner is remembered in the process and in ``autotune.json`` beside
    the code-object cache.  Used by the backend under ``mode="max-autotune"``."""
    if kw.get("score_bias") is not None or kw.get("out_bias") is not None or kw.get("record_visits") \
            or kw.get("force_family") or kw.get("num_splits") or kw.get("choice") or plan.denom_add != 0.0 or kw.get("q2") is not None:
        return attention(q, k, v, plan, k_table, v_table, **kw)
    _load_tuned()
    key = _tune_key(q, k, plan, k_table, 0)
    if key not in _tuned and q.is_cuda and torch.cuda.is_current_stream_capturing():
        # timing needs a host synchronisation, which a stream capture forbids: fixed heuristics
        return attention(q, k, v, plan, k_table, v_table, **kw)
    if key not in _tuned:
        B, Hq, Sq, D = q.shape
        Hkv = k.shape[-2] if plan.k_paged else k.shape[1]
        group = Hq // max(Hkv, 1)
        decode = plan.mask is None and ((Sq == 1 and group <= 64) or (group == 1 and Sq <= 16))
        if decode:
            cands = [{"head_per_wave": hw, "splits": sp} for hw in ((False, True) if plan.k_paged and plan.v_paged else (False,))
                     for sp in (None, 1, 2, 4, 8)]
        elif not (plan.k_paged or plan.v_paged):
            # kernel family, tile shape (keys per LDS tile, which also sets how many workgroups share a
            # CU; the reference's tuner searches tile sizes, codegen.py:360-393) and, for grouped query
            # heads, the packed / unpacked q tile
            cands = [{"prefill": "swp", "bn": 32}, {"prefill": "swp", "bn": 64}, {"prefill": "w32"}]
            if group % 2 == 0:
                cands[2:2] = [{"prefill": "swp", "bn": 32, "pack": False}, {"prefill": "swp", "bn": 64, "pack": False}]
        elif Sq > 1:
            cands = [{"bn": 32}, {"bn": 64}]
        else:
            cands = [{}]
        best, best_t = cands[0], float("inf")
        if len(cands) > 1:
            out = kw.get("out")
            for c in cands:
                c = {a: b for a, b in c.items() if b is not None}
                try:
                    for _ in range(2):
                        out = attention(q, k, v, plan, k_table, v_table, **{**kw, "out": out, "choice": c})
                    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    a.record()
                    for _ in range(5):
                        attention(q, k, v, plan, k_table, v_table, **{**kw, "out": out, "choice": c})
                    b.record()
                    b.synchronize()
                    t = a.elapsed_time(b)
                except UnsupportedPlan:
                    continue
                if t < best_t:
                    best, best_t = c, t
        _tuned[key] = best
        try:
            import json
            os.makedirs(os.path.dirname(_TUNE_FILE), exist_ok=True)
            with open(_TUNE_FILE, "w") as fh:
                json.dump(_tuned, fh, indent=0, sort_keys=True)
        except OSError:
            pass
    return attention(q, k, v, plan, k_table, v_table, **{**kw, "choice": _tuned[key]})


class _LastLaunch:
    """What the calling THREAD's last ``attention`` call launched (kernels, grid, block, tile
    shape): ``attention.last_launch["kernels"]``.  Each thread sees its own record."""

    def __init__(self):
        self._tls = threading.local()

    def set(self, record: dict) -> None:
        self._tls.record = record

    def _get(self) -> dict:
        return getattr(self._tls, "record", {})

    def __getitem__(self, key):
        return self._get()[key]

    def get(self, key, default=None):
        return self._get().get(key, default)

    def __repr__(self) -> str:
        return repr(self._get())


_last_launch = _LastLaunch()


def _on_device_of_first_argument(fn):
    """Kernel modules, the stream and the split-K scratch are looked up for the current
    device: make the device of Q current for the duration of the call when it is not."""
    @functools.wraps(fn)
    def guarded(q, *args, **kw):
        if isinstance(q, torch.Tensor) and q.is_cuda and q.device.index != torch.cuda.current_device():
            with torch.cuda.device(q.device):
                return fn(q, *args, **kw)
        return fn(q, *args, **kw)
    guarded.last_launch = _last_launch
    return guarded


@_on_device_of_first_argument
def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, plan: AttnPlan,
              k_table: Optional[torch.Tensor] = None, v_table: Optional[torch.Tensor] = None,
              *, out: Optional[torch.Tensor] = None, record_visits: bool = False,
              force_family: str | None = None, num_splits: int | None = None, v_tr: bool = True,
              score_bias: Optional[torch.Tensor] = None, out_bias: Optional[torch.Tensor] = None,
              choice: Optional[dict] = None, merge_splits: bool = True,
              q2: Optional[torch.Tensor] = None, k2: Optional[torch.Tensor] = None,
              static_scratch: bool = False, lse: Optional[torch.Tensor] = None):
    """Run fused attention on the GPU.

    q : [B, Hq, Sq, D];  k, v : [B, Hkv, Sk, D], or page pools [N, P, Hkv, D]
    ([N, Hkv, D] for one-token pages) with ``k_table``/``v_table`` [B, Sk/P].
    ``score_bias`` (broadcastable to [B, Hq, Sq, Sk], key stride 1) is added to the
    scaled / capped scores before the mask, ``out_bias`` (broadcastable to
    [B, Hq, Sq, D]) to the result -- the reference's "modified attention" graph
    (tests/test_accuracy.py:172-196).  Both are served by ``lf_attn_prefill`` only.
    ``q2`` [B, Hq, Sq, D2] and ``k2`` [B, H2, Sk, D2] (H2 divides Hq; D2 in 16, 32, 64) add a
    second product to the scores, ``Q K^T + Q2 K2^T`` before the scale -- the two-part scores
    of multi-head latent attention (reference tests/test_attention.py:126-151); served by
    ``lf_attn_prefill`` with dense K2.
    ``merge_splits=False`` leaves the partial results of a split decode unmerged (the
    output is then not written): for timing the streaming kernel alone.
    ``static_scratch=True`` (split decode only, ``out`` given): the step goes through the C ABI's
    ``lf_launch_decode_static``, whose split-K partials live in a static device array of the
    library -- no device memory is allocated anywhere in the call; a step whose partials exceed
    that array raises ``runtime.ShimError``.
    ``lse`` (float32 [B, Hq, Sq], contiguous): also write each row's log-sum-exp of the scaled,
    masked scores, in log2 units -- what ``attention_backward`` recomputes the probabilities
    from.  Served by ``lf_attn_prefill_swp`` (dense K/V); anything else raises ``UnsupportedPlan``.
    ``choice`` overrides the launch heuristics (what ``tuned_attention`` searches over):
    ``{"prefill": "swp" | "w32"}``, ``{"head_per_wave": bool, "splits": n}``.
    Returns O [B, Hq, Sq, D] and, with ``record_visits``, the uint8 record of the KV tiles
    each workgroup walked, ``[B * heads * q_tiles, kv_tiles]`` with ``heads = Hq`` and
    128-row q tiles, or ``heads = Hq / g`` and ``128 / g``-row q tiles when g = 2 or 4 query heads
    are packed (``last_launch["heads_per_workgroup"] == g``).
    """
    choice = choice or {}
    dtype = q.dtype
    if dtype not in _DTYPE_CODE:
        raise UnsupportedPlan(f"dtype {dtype} not supported by the MFMA kernels (bf16/fp16 only)")
    if q.dim() != 4:
        raise UnsupportedPlan("Q must be [B, Hq, Sq, D]")
    B, Hq, Sq, D = q.shape
    if D not in (64, 128):
        # Other head dimensions up to 128 (the reference takes any static D, ops.py:370-397): dense operands
        # are copied into zero-padded rows of 64 / 128 elements -- zeros add nothing to Q K^T, and the padded
        # columns of V give output columns that are cut off again -- at O(S D) beside the O(S^2 D) attention.
        Dp = 64 if D < 64 else 128
        if D > 128 or D < 1 or plan.k_paged or plan.v_paged or lse is not None or q2 is not None or static_scratch \
                or k.dim() != 4 or v.dim() != 4 or k.shape[-1] != D or v.shape[-1] != D:
            raise UnsupportedPlan(f"head dim {D} not supported (64 and 128; up to 128 by padding for dense operands)")
        grow = lambda t: None if t is None else torch.nn.functional.pad(t, (0, Dp - D))
        res = attention(grow(q), grow(k), grow(v), plan, None, None, record_visits=record_visits, score_bias=score_bias,
                        out_bias=grow(out_bias), force_family=force_family, num_splits=num_splits, v_tr=v_tr,
                        choice=choice, merge_splits=merge_splits)
        o_p, vis = res if record_visits else (res, None)
        if out is None:
            out = o_p[..., :D].contiguous()
        else:
            out.copy_(o_p[..., :D])
        return (out, vis) if record_visits else out
    if not (plan.scale > 0.0) or not math.isfinite(plan.scale):
        raise UnsupportedPlan("score scale must be positive and finite")
    softcap = None
    if plan.softcap is not None:
        # cap * tanh(s / cap) is even in cap: a negative cap (pre- and post-factor both negative
        # in the graph) is served as its magnitude; zero or a non-finite cap is not a softcap
        softcap = abs(float(plan.softcap))
        if not (softcap > 0.0) or not math.isfinite(softcap):
            raise UnsupportedPlan("softcap must be finite and non-zero")
    _check_tensor("Q", q, dtype)
    _check_tensor("K", k, dtype)
    _check_tensor("V", v, dtype)
    for name, t in (("K", k), ("V", v), ("K page table", k_table), ("V page table", v_table), ("score bias", score_bias),
                    ("output bias", out_bias), ("Q2", q2), ("K2", k2), ("O", out)):
        if t is not None and t.device != q.device:
            raise RuntimeError(f"loopfuse_amd: {name} is on {t.device}, Q on {q.device}")

    P = AttnParams()
    paged = 0
    page_size = 1          # K pool (both pools when they agree)
    page_size_v = 0        # V pool, when it differs from K's
    table_i64 = False

    def kv_layout(t: torch.Tensor, table: Optional[torch.Tensor], is_paged: bool, which: str):
        nonlocal paged, page_size, page_size_v, table_i64
        if not is_paged:
            if t.dim() != 4 or t.shape[0] != B or t.shape[3] != D:
                raise UnsupportedPlan(f"{which} must be [B, Hkv, Sk, D]")
            return t.shape[1], t.shape[2], t.stride(0), t.stride(1), t.stride(2), None, 0
        if table is None or table.dim() != 2 or table.shape[0] != B:
            raise UnsupportedPlan(f"{which} page table must be [B, pages]")
        if table.dtype not in (torch.int32, torch.int64):
            raise UnsupportedPlan("page table must be int32 or int64")
        if not table.is_cuda:
            raise RuntimeError(f"loopfuse_amd: {which} page table is not on the GPU")
        if table.stride(1) != 1:
            table = table.contiguous()
        if os.environ.get("LOOPFUSE_CHECK_TABLES", "0") == "1" and table.numel():
            # debugging aid (waits for the stream): the kernels trust page ids, an id outside
            # the pool is a read outside the allocation
            lo, hi = int(table.min()), int(table.max())
            if lo < 0 or hi >= t.shape[0]:
                raise ValueError(f"loopfuse_amd: {which} page table holds ids in [{lo}, {hi}] for a pool of {t.shape[0]} pages")
        if t.dim() == 3:       # [N, Hkv, D], one token per page (the reference's format)
            ps, hk, sp, st, sh = 1, t.shape[1], t.stride(0), 0, t.stride(1)
        elif t.dim() == 4:     # [N, P, Hkv, D]
            ps, hk, sp, st, sh = t.shape[1], t.shape[2], t.stride(0), t.stride(1), t.stride(2)
        else:
            raise UnsupportedPlan(f"{which} pool must be [N, Hkv, D] or [N, P, Hkv, D]")
        if t.shape[-1] != D:
            raise UnsupportedPlan(f"{which} pool has head dim {t.shape[-1]}, Q has {D}")
        if ps & (ps - 1):
            raise UnsupportedPlan("page size must be a power of two")
        i64 = table.dtype == torch.int64
        if paged and table_i64 != i64:
            raise UnsupportedPlan("K and V page tables must share their dtype")
        if which == "V" and paged and ps != page_size:
            page_size_v = ps               # pools with different page sizes
        else:
            page_size = ps
        table_i64 = i64
        paged |= 1 if which == "K" else 2
        return hk, table.shape[1] * ps, sp, sh, st, table, table.stride(0)

    Hkv, Sk, P.k_sb, P.k_sh, P.k_ss, kt, P.kt_stride = kv_layout(k, k_table, plan.k_paged, "K")
    Hkv2, Sk2, P.v_sb, P.v_sh, P.v_ss, vt, P.vt_stride = kv_layout(v, v_table, plan.v_paged, "V")
    if Hkv != Hkv2 or Sk != Sk2:
        raise UnsupportedPlan("K and V disagree on heads or length")
    if Hq % Hkv:
        raise UnsupportedPlan("Hq must be a multiple of Hkv")
    group = Hq // Hkv
    mask = _MASK_NAMES[plan.mask]
    if mask == MASK_SLIDING and plan.window < 1:
        raise UnsupportedPlan("sliding mask needs window >= 1")

    if Sk < 1:
        # softmax over no keys is 0/0 in the eager graph: nothing a kernel should invent
        raise UnsupportedPlan("attention over an empty key sequence")
    if out is None:
        out = torch.empty((B, Hq, Sq, D), dtype=dtype, device=q.device)
    else:
        _check_tensor("O", out, dtype)
        if tuple(out.shape) != (B, Hq, Sq, D):
            raise UnsupportedPlan(f"O must be [{B}, {Hq}, {Sq}, {D}]")
    if B == 0 or Hq == 0 or Sq == 0:
        # no query rows: the (empty) output is the whole result, nothing to launch
        _last_launch.set({"kernels": [], "grid": 0, "block": 0})
        return (out, torch.zeros((0, 0), dtype=torch.uint8, device=q.device)) if record_visits else out

    P.q, P.k, P.v, P.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    P.k_table = kt.data_ptr() if kt is not None else None
    P.v_table = vt.data_ptr() if vt is not None else None
    P.B, P.Hq, P.Hkv, P.Sq, P.Sk = B, Hq, Hkv, Sq, Sk
    P.window = int(plan.window)
    P.scale = float(plan.scale)
    P.softcap = softcap if softcap is not None else 0.0
    P.denom_add = float(plan.denom_add)
    if plan.denom_add < 0.0 or not math.isfinite(plan.denom_add):
        raise UnsupportedPlan("the denominator offset must be finite and >= 0")
    P.nsplit, P.rows, P.split_len = 1, 1, 0

    # ---- additive biases: [B, Hq, Sq, X] views with broadcast (stride 0) batch/head/row dims
    bias_bits = 0

    def bias_layout(t: torch.Tensor, what: str, last: int):
        nonlocal bias_bits
        if t.dtype != dtype or not t.is_cuda:
            raise UnsupportedPlan(f"{what} must be a {dtype} GPU tensor")
        if t.dim() > 4:
            raise UnsupportedPlan(f"{what} has more than 4 dims")
        if os.environ.get("LOOPFUSE_BIAS_COPY", "1") == "1" and \
                t.dim() >= 2 and t.shape[-1] == last and t.stride(-1) == 1 and t.numel() <= (1 << 25) and \
                (t.data_ptr() % 8 or any(st % 4 for n, st in zip(t.shape[:-1], t.stride()[:-1]) if n > 1)):
            # rows that do not start on 8-byte borders (a mask over an odd number of keys) would
            # be read element by element: a copy with padded rows is cheaper for tensors this small
            padded = torch.empty((*t.shape[:-1], (last + 3) // 4 * 4), dtype=t.dtype, device=t.device)
            t = padded[..., :last].copy_(t)
        try:
            t = t.expand(B, Hq, Sq, last)
        except RuntimeError:
            raise UnsupportedPlan(f"{what} does not broadcast to [{B}, {Hq}, {Sq}, {last}]")
        if t.stride(3) != 1 and t.shape[3] != 1:
            raise UnsupportedPlan(f"{what} needs last-dim stride 1")
        if t.data_ptr() % 8 or any(st % 4 for n, st in zip(t.shape[:3], t.stride()[:3]) if n > 1):
            bias_bits |= 4          # rows not 8-byte aligned: element loads
        return t

    if score_bias is not None:
        score_bias = bias_layout(score_bias, "score bias", Sk)
        P.bias = score_bias.data_ptr()
        P.bias_sb, P.bias_sh, P.bias_sq = score_bias.stride(0), score_bias.stride(1), score_bias.stride(2)
        bias_bits |= 1
    if out_bias is not None:
        out_bias = bias_layout(out_bias, "output bias", D)
        P.obias = out_bias.data_ptr()
        P.ob_sb, P.ob_sh, P.ob_sq = out_bias.stride(0), out_bias.stride(1), out_bias.stride(2)
        bias_bits |= 2
    d2 = 0
    if (q2 is None) != (k2 is None):
        raise UnsupportedPlan("q2 and k2 come together")
    if q2 is not None:
        if q2.dim() != 4 or k2.dim() != 4 or q2.shape[:3] != (B, Hq, Sq):
            raise UnsupportedPlan(f"Q2 must be [{B}, {Hq}, {Sq}, D2]")
        d2 = q2.shape[3]
        if d2 not in (16, 32, 64):
            raise UnsupportedPlan(f"depth {d2} of the second score product not supported (16, 32, 64)")
        if k2.shape[0] != B or k2.shape[2] != Sk or k2.shape[3] != d2 or k2.shape[1] < 1 or Hq % k2.shape[1]:
            raise UnsupportedPlan(f"K2 must be [{B}, H2 | {Hq}, {Sk}, {d2}]")
        _check_tensor("Q2", q2, dtype)
        _check_tensor("K2", k2, dtype)
        P.q2, P.k2 = q2.data_ptr(), k2.data_ptr()
        P.q2_sb, P.q2_sh, P.q2_ss = q2.stride(0), q2.stride(1), q2.stride(2)
        P.k2_sb, P.k2_sh, P.k2_ss = k2.stride(0), k2.stride(1), k2.stride(2)
        P.k2_group = Hq // k2.shape[1]
    if bias_bits not in (0, 1) or plan.denom_add != 0.0 or d2:
        force_family = "prefill"       # the decode kernel takes an aligned score bias and nothing else of these

    # ---- family: decode when there is no mask and few query rows share a KV head
    family = force_family
    if family is None:
        few = (Sq == 1 and group <= 64) or (group == 1 and Sq <= 16)
        # a caller that wants the row log-sum-exp (a forward that a backward will follow) gets the
        # prefill kernel, which writes it; the decode kernels do not
        family = "decode" if (mask == MASK_NONE and few and Sk >= 16 and lse is None) else "prefill"
    keep = (q, k, v, out, kt, vt, score_bias, out_bias, q2, k2)  # noqa: F841  (tensors stay alive until the launch is queued)

    if family == "prefill" and not bias_bits and plan.denom_add == 0.0 and not d2:
        family = {"swp": "prefill_swp", "w32": "prefill"}.get(choice.get("prefill"), None) or prefill_variant(Sq, v_tr)
    # a score bias with 8-byte aligned rows and nothing else special: the direct-to-LDS kernel with the bias
    # classified tile by tile first (lf_bias_classify) -- what a mask given as a tensor needs
    bias_tiles = (family == "prefill" and bias_bits == 1 and plan.denom_add == 0.0 and not d2
                  and lse is None and Sk >= 4 and (Sk + 63) // 64 <= 65535 * 4 and B * Hq <= 65535
                  and os.environ.get("LOOPFUSE_BIAS_TILES", "1") == "1" and choice.get("prefill") != "w32"
                  and prefill_variant(Sq, v_tr) == "prefill_swp")
    if bias_tiles:
        family = "prefill_swp"
    if family == "prefill_swp":
        # direct-to-LDS staging addresses memory with 32-bit byte offsets.  Dense operands:
        # offsets inside one (batch, kv head) span; the kernel also addresses up to three
        # tiles past Sk (those reads are range-checked to zeros, but their offsets must
        # not wrap).  Paged operands: offsets inside the whole pool (< 4 GiB), pages of a
        # multiple of 8 tokens (the rows of one wave-level load stay inside a page).
        def swp_ok(t, is_paged, ps_, ss):
            if is_paged:
                span_b = 2 * (sum((n - 1) * abs(st) for n, st in zip(t.shape, t.stride())) + 1)
                return ps_ % 8 == 0 and span_b < (1 << 32) - 64 and all(st >= 0 for st in t.stride())
            reach = abs(ss) * 2 * (Sk + 3 * 64) + 2 * D
            return ss >= 0 and reach < (1 << 32) and (Sk - 1) * abs(ss) * 2 + 2 * D < (1 << 31)
        if not (swp_ok(k, plan.k_paged, page_size, P.k_ss)
                and swp_ok(v, plan.v_paged, page_size_v or page_size, P.v_ss)) \
                or (paged and os.environ.get("LOOPFUSE_PAGED_SWP", "1") != "1"):
            family = "prefill"
        if plan.k_paged:
            P.k_span = sum((n - 1) * st for n, st in zip(k.shape, k.stride())) + 1
        if plan.v_paged:
            P.v_span = sum((n - 1) * st for n, st in zip(v.shape, v.stride())) + 1
    if family in ("prefill", "prefill_swp"):
        P.q_sb, P.q_sh, P.q_ss = q.stride(0), q.stride(1), q.stride(2)
        P.o_sb, P.o_sh, P.o_ss = out.stride(0), out.stride(1), out.stride(2)
        extra = tuple(os.environ.get("LOOPFUSE_KOPTS", "").split())
        # buffer loads address a (batch, kv head) span with 32-bit byte offsets
        span = max((Sk - 1) * abs(P.k_ss), (Sk - 1) * abs(P.v_ss)) * 2 + 2 * D
        if family == "prefill" and span >= (1 << 31):
            extra += ("-DLF_KVBUF=0",)
        elif family == "prefill" and (bias_bits or d2) and not paged:
            extra += ("-DLF_DMA=1",)     # frees the staging registers the bias values / Q2 fragments need
        # grouped-query attention: the 4 waves of a workgroup take 4 (or 2) query heads of one
        # group over the same query rows and share every K/V tile in LDS
        pack = 0
        if family == "prefill_swp" and group % 2 == 0 and not any(e.startswith("-DLF_NW=") for e in extra) and \
                choice.get("pack", os.environ.get("LOOPFUSE_GQAPACK", "1") == "1") and (not bias_bits or P.bias_sh == 0):
            # (with a score bias only when all heads share it: the tile classes are then the same for the
            # packed heads of a workgroup)
            pack = 4 if group % 4 == 0 else 2
        if family == "prefill_swp" and bias_bits and not bias_tiles:
            family = "prefill"                          # swp was refused above (spans): the register-staged kernel
        spec = KernelSpec(family, _DTYPE_CODE[dtype], D, mask, plan.softcap is not None, paged,
                          page_size, table_i64, v_tr=v_tr if family == "prefill" else True, bias=bias_bits,
                          denom=plan.denom_add != 0.0, d2=d2, page_size_v=page_size_v, pack=pack, extra=extra,
                          safe=plan.zero_blind_rows and bool(bias_bits & 1),
                          bn=prefill_kv_tile(D, bias_bits, choice, B * (Hq // (pack or 1)) * (-(-Sq // (128 // (pack or 1)))))
                          if family == "prefill_swp" else 0)
        bm, bn = TILE_SHAPES[family]
        nw = 4
        for e in spec.extra:                    # tuning: -DLF_NW=8 doubles the q tile
            if e.startswith("-DLF_NW="):
                nw = int(e.split("=")[1])
                bm = 32 * nw
        if spec.bn:
            bn = spec.bn
        heads = Hq
        if spec.pack:
            bm, heads = 128 // spec.pack, Hq // spec.pack      # q tiles of 32 rows x 4 heads, or 64 rows x 2 heads
        nqt = (Sq + bm - 1) // bm
        nkt = (Sk + bn - 1) // bn
        visits = None
        if record_visits:
            visits = torch.zeros((B * heads * nqt, nkt), dtype=torch.uint8, device=q.device)
            P.visits = visits.data_ptr()
        # 8 XCD classes x (batch*head pairs per class, padded to the kernel's groups) x q tiles
        per_xcd = (B * heads + 7) // 8
        if family == "prefill_swp":
            # one q tile per workgroup, groups of LF_QGROUP heads, longest q tiles first
            qgroup = PREFILL_QGROUP
            for e in spec.extra:
                if e.startswith("-DLF_QGROUP="):
                    qgroup = int(e.split("=")[1])
            grid = 8 * ((per_xcd + qgroup - 1) // qgroup * qgroup) * nqt
        else:
            # lf_attn_prefill takes two q tiles (heavy + light) per workgroup, groups of 4 heads
            grid = 8 * ((per_xcd + 3) // 4 * 4) * ((nqt + 1) // 2)
        if lse is not None:
            if family != "prefill_swp" or paged:
                raise UnsupportedPlan("the row log-sum-exp is written by lf_attn_prefill_swp for dense K/V only")
            if lse.dtype != torch.float32 or tuple(lse.shape) != (B, Hq, Sq) or not lse.is_contiguous() or lse.device != q.device:
                raise UnsupportedPlan(f"lse must be a contiguous float32 [{B}, {Hq}, {Sq}] tensor on the device of Q")
            P.part_ml = lse.data_ptr()
        names = [spec.entry()]
        if family == "prefill_swp" and bias_bits:
            # tile classes of the bias, once per distinct (batch, head) it holds: int32 [units][kv tiles]
            nb_, nh_ = (B if P.bias_sb else 1), (Hq if P.bias_sh else 1)
            table = torch.empty((nb_ * nh_ * nqt * nkt,), dtype=torch.int32, device=q.device)
            keep += (table,)
            P.part_acc = table.data_ptr()
            get_kernel(spec, "lf_bias_classify").launch((nqt, nb_ * nh_, (nkt + 3) // 4), (256, 1, 1), P)
            names.insert(0, "lf_bias_classify")
        get_kernel(spec, spec.entry()).launch((grid, 1, 1), (64 * nw, 1, 1), P)
        _last_launch.set({"kernels": names, "grid": grid, "block": 64 * nw, "q_tile_rows": bm, "kv_tile_rows": bn,
                                 "heads_per_workgroup": spec.pack or 1})
        return (out, visits) if record_visits else out

    if family != "decode":
        raise ValueError(f"unknown kernel family {family!r}")
    if lse is not None:
        raise UnsupportedPlan("the decode kernels do not write the row log-sum-exp")
    if mask != MASK_NONE:
        raise UnsupportedPlan("the decode kernel takes no mask")
    # query rows of one unit: the group's heads (Sq == 1) or the Sq rows (group == 1)
    if Sq == 1:
        rows = group
        P.q_sb, P.q_sh, P.q_ss = q.stride(0), group * q.stride(1), q.stride(1)
        P.o_sb, P.o_sh, P.o_ss = out.stride(0), group * out.stride(1), out.stride(1)
        if bias_bits:
            P.bias_sh, P.bias_sq = group * score_bias.stride(1), score_bias.stride(1)
    elif group == 1:
        rows = Sq
        P.q_sb, P.q_sh, P.q_ss = q.stride(0), q.stride(1), q.stride(2)
        P.o_sb, P.o_sh, P.o_ss = out.stride(0), out.stride(1), out.stride(2)
    else:
        raise UnsupportedPlan("decode needs Sq == 1 or group == 1")
    chunks = (rows + DECODE_QROWS - 1) // DECODE_QROWS
    units = B * Hkv * chunks
    waves = int(os.environ.get("LOOPFUSE_DECODE_WAVES", "4"))
    # Token-major page pools ([pages, page, Hkv, D]: the heads of a token side by side)
    # are read whole-page-wise when the 8 waves of a workgroup take 8 consecutive heads.
    headwave = _decode_headwave(paged, page_size, Hkv, D, P, B * ((Hkv + 7) // 8) * chunks, Sk) and not page_size_v
    if "head_per_wave" in choice:
        headwave = bool(choice["head_per_wave"]) and paged == 3 and Hkv % 8 == 0
    if headwave:
        waves = 8
        units = B * ((Hkv + waves - 1) // waves) * chunks
    num_splits = num_splits or choice.get("splits")
    nsplit = num_splits if num_splits else decode_split(units, Sk, per_cu=1 if headwave else 2)
    split_len = ((Sk + nsplit - 1) // nsplit + 31) // 32 * 32     # whole pairs of 16-token steps
    nsplit = (Sk + split_len - 1) // split_len
    P.rows, P.nsplit, P.split_len = rows, nsplit, split_len
    spec = KernelSpec("decode", _DTYPE_CODE[dtype], D, MASK_NONE, plan.softcap is not None, paged,
                      page_size, table_i64, rows=DECODE_QROWS, waves=waves, headwave=headwave, page_size_v=page_size_v,
                      coop=(coop := _decode_coop(headwave, page_size, page_size_v, bias_bits, Hkv, waves, P, D)),
                      rowload=not coop and _decode_rowload(paged, page_size, page_size_v, bias_bits),
                      bias=bias_bits, safe=plan.zero_blind_rows and bool(bias_bits),
                      extra=tuple(os.environ.get("LOOPFUSE_KOPTS", "").split()))
    rows_per_block = 1024 // D       # combine kernel: 256 threads, 4 consecutive d each
    combine_grid = (B * Hkv * rows + rows_per_block - 1) // rows_per_block
    if static_scratch:
        if nsplit <= 1 or not merge_splits:
            raise UnsupportedPlan("static_scratch serves split decode steps (this call does not split the keys)")
        nrow = B * Hkv * rows * nsplit
        runtime.launch_decode_static(get_kernel(spec, "lf_attn_decode"), get_kernel(spec, "lf_attn_decode_combine"), P,
                                     4 * nrow * D, 4 * nrow * 2, (units, nsplit), 64 * spec.waves, combine_grid, 256)
        _last_launch.set({"kernels": ["lf_attn_decode", "lf_attn_decode_combine"], "grid": (units, nsplit),
                                 "block": 64 * spec.waves, "head_per_wave": headwave, "cooperative_loads": spec.coop,
                                 "static_scratch": True})
        return out
    if nsplit > 1:
        nrow = B * Hkv * rows * nsplit
        scratch = _get_scratch(q.device, nrow * (D + 2))
        P.part_acc = scratch.data_ptr()
        P.part_ml = scratch.data_ptr() + 4 * nrow * D
    get_kernel(spec, "lf_attn_decode").launch((units, nsplit, 1), (64 * spec.waves, 1, 1), P)
    if nsplit > 1 and merge_splits:
        get_kernel(spec, "lf_attn_decode_combine").launch((combine_grid, 1, 1), (256, 1, 1), P)
    _last_launch.set({"kernels": ["lf_attn_decode"] + (["lf_attn_decode_combine"] if nsplit > 1 and merge_splits else []),
                             "grid": (units, nsplit), "block": 64 * spec.waves, "head_per_wave": headwave,
                             "cooperative_loads": spec.coop})
    return out


# ---------------------------------------------------------------------------
# backward (the reference has none: loopfuse README "future work")
# ---------------------------------------------------------------------------
class AttnBwdParams(ctypes.Structure):
    """Mirror of ``struct LfAttnBwdParams`` in csrc/kernels/lf_attn_bwd.hip."""

    _fields_ = (
        [(n, ctypes.c_void_p) for n in ("q", "k", "v", "o", "dout", "dq", "dk", "dv", "lse", "delta")]
        + [(f"{t}_{x}", ctypes.c_longlong) for t in ("q", "k", "v", "o", "do", "dq", "dk", "dv") for x in ("sb", "sh", "ss")]
        + [(n, ctypes.c_int) for n in ("B", "Hq", "Hkv", "Sq", "Sk", "window")]
        + [("scale", ctypes.c_float), ("softcap", ctypes.c_float)]
    )


def bwd_dq_threads(mask: int, softcap: bool = False) -> int:
    """Workgroup size of lf_attn_bwd_dq: 8 waves (256 query rows, two waves per SIMD on one K/V
    tile stream) except under a sliding window, where a 256-row tile walks too many kv tiles
    that only part of its rows can see, and with a softcap, whose extra values do not fit the
    256 registers a wave has at two per SIMD."""
    return 256 if mask == MASK_SLIDING or softcap else 512


def bwd_spec(dtype: torch.dtype, D: int, mask: int, softcap: bool = False) -> KernelSpec:
    return KernelSpec("bwd", _DTYPE_CODE[dtype], D, mask, softcap, extra=(f"-DLF_BW_DQ_NT={bwd_dq_threads(mask, softcap)}",))


def attention_backward(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, lse: torch.Tensor,
                       dout: torch.Tensor, plan: AttnPlan):
    """Gradients of ``attention(q, k, v, plan)`` for dense K/V (mask none / causal / sliding, scale,
    softcap; no bias or paging): returns ``(dq, dk, dv)`` in the operands' dtype.  ``o`` and ``lse``
    are the forward's output and row log-sum-exp (``attention(..., lse=...)``).  Three launches
    (csrc/kernels/lf_attn_bwd.hip): delta = rowsum(dO * O); dK and dV, one workgroup per 128 keys of
    a (batch, kv head); dQ, one workgroup per 128 query rows.  No atomics: results are
    reproducible bit for bit."""
    dtype = q.dtype
    if dtype not in _DTYPE_CODE:
        raise UnsupportedPlan(f"dtype {dtype} not supported by the MFMA kernels (bf16/fp16 only)")
    if plan.k_paged or plan.v_paged or plan.denom_add != 0.0:
        raise UnsupportedPlan("the backward kernels serve dense K/V and the plain softmax denominator")
    softcap = None
    if plan.softcap is not None:
        softcap = abs(float(plan.softcap))
        if not (softcap > 0.0) or not math.isfinite(softcap):
            raise UnsupportedPlan("softcap must be finite and non-zero")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise UnsupportedPlan("Q, K, V must be [B, H, S, D]")
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    if D not in (64, 128) or k.shape != v.shape or k.shape[0] != B or k.shape[3] != D or Hkv < 1 or Hq % Hkv:
        raise UnsupportedPlan(f"shapes not served: Q {tuple(q.shape)}, K {tuple(k.shape)}, V {tuple(v.shape)}")
    if Sq < 1 or Sk < 1:
        raise UnsupportedPlan("empty sequences")
    if o.shape != q.shape or dout.shape != q.shape or tuple(lse.shape) != (B, Hq, Sq):
        raise UnsupportedPlan("O, dO must have the shape of Q and lse must be [B, Hq, Sq]")
    if lse.dtype != torch.float32 or not lse.is_contiguous():
        raise UnsupportedPlan("lse must be contiguous float32")
    mask = {None: MASK_NONE, "none": MASK_NONE, "causal": MASK_CAUSAL, "sliding": MASK_SLIDING}.get(plan.mask)
    if mask is None:
        raise UnsupportedPlan(f"mask {plan.mask!r} not served")
    window = int(plan.window or 0)
    if mask == MASK_SLIDING and window < 1:
        raise UnsupportedPlan("sliding window must be >= 1")
    for name, t in (("Q", q), ("K", k), ("V", v), ("O", o), ("dO", dout)):
        _check_tensor(name, t, dtype)
    # the tiles travel global -> LDS with 32-bit byte offsets inside one (batch, head) span, rows
    # past the end addressed too (and range-checked to zeros)
    for name, t, S in (("Q", q, Sq), ("dO", dout, Sq), ("K", k, Sk), ("V", v, Sk)):
        if t.stride(2) < D or (S + 64) * t.stride(2) * 2 + 2 * D >= (1 << 32):
            raise UnsupportedPlan(f"{name}: row stride {t.stride(2)} not served by the backward kernels' direct loads")
    dq = torch.empty((B, Hq, Sq, D), dtype=dtype, device=q.device)
    dk = torch.empty((B, Hkv, Sk, D), dtype=dtype, device=q.device)
    dv = torch.empty((B, Hkv, Sk, D), dtype=dtype, device=q.device)
    delta = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    P = AttnBwdParams()
    for name, t in (("q", q), ("k", k), ("v", v), ("o", o), ("dout", dout), ("dq", dq), ("dk", dk), ("dv", dv),
                    ("lse", lse), ("delta", delta)):
        setattr(P, name, t.data_ptr())
    for pre, t in (("q", q), ("k", k), ("v", v), ("o", o), ("do", dout), ("dq", dq), ("dk", dk), ("dv", dv)):
        setattr(P, pre + "_sb", t.stride(0))
        setattr(P, pre + "_sh", t.stride(1))
        setattr(P, pre + "_ss", t.stride(2))
    P.B, P.Hq, P.Hkv, P.Sq, P.Sk, P.window = B, Hq, Hkv, Sq, Sk, window
    P.scale = float(plan.scale)
    P.softcap = softcap if softcap is not None else 0.0
    spec = bwd_spec(dtype, D, mask, softcap is not None)
    keep = (q, k, v, o, dout, lse, delta, dq, dk, dv)  # noqa: F841  (tensors stay alive until the launches are queued)
    rows = B * Hq * Sq
    get_kernel(spec, "lf_attn_bwd_delta").launch(((rows + 15) // 16, 1, 1), (256, 1, 1), P)
    # 8 XCD classes x (batch, kv head) pairs per class, padded to the kernels' groups, x the
    # workgroups of a pair (key blocks; query heads of the group x q tiles)
    grp = BWD_GROUP
    for e in spec.extra:
        if e.startswith("-DLF_BW_GROUP="):
            grp = int(e.split("=")[1])
    pairs = ((B * Hkv + 7) // 8 + grp - 1) // grp * grp
    get_kernel(spec, "lf_attn_bwd_dkdv").launch((8 * pairs * ((Sk + 127) // 128), 1, 1), (256, 1, 1), P)
    nt = bwd_dq_threads(mask, softcap is not None)
    get_kernel(spec, "lf_attn_bwd_dq").launch((8 * pairs * (Hq // Hkv) * ((Sq + nt // 2 - 1) // (nt // 2)), 1, 1),
                                              (nt, 1, 1), P)
    _last_launch.set({"kernels": ["lf_attn_bwd_delta", "lf_attn_bwd_dkdv", "lf_attn_bwd_dq"]})
    return dq, dk, dv
