#!/usr/bin/env python3
"""Benchmark of the fused-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one batch of synthetic input.  The
headline workload is config 2 (bf16 causal prefill, B8 H32 S2048 D128):
``value`` is its algorithmic TFLOP/s with the reference's flop convention
(2*B*H*S^2*D, reference tests/benchmark.py:110).  The same run also times the
memory-bound half of the metric, config 5 (paged GQA decode, B64 K_len 2048, page
16), reported under "decode" in GB/s with the reference's byte convention
(K and V only, tests/benchmark.py:452).  Inputs are resident in HBM before the
timed region.  One JSON line on stdout.

Order of the legs.  The GPU's power management makes the launches that follow an idle
period unrepresentative (the first few run at boost clocks, the next few dozen slower than
the steady state), so each kernel is first brought to its steady state the way the
reference's harness does it (``triton.testing.do_bench``, reference tests/benchmark.py:19-22:
about 25 ms of untimed launches, then about 100 ms of timed ones) -- that measurement is
reported as ``settled`` -- and the ``--warmup W`` untimed + ``--steps K`` timed launches that
``value`` is computed from follow immediately.
"""
from __future__ import annotations

import argparse
import dataclasses
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16/fp16, published
HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
# HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by a plain copy of known
# size: counters cannot be read from inside this process, so the figures are taken from the line
# "traffic_bytes_per_launch: <workload>=<bytes> ..." of the counter summary under profiles/
# (null when the summary or the workload's figure is missing)
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "lf_attn_prefill_swp_c2_and_lf_attn_decode_c5_hbm_traffic_mfma_and_stalls.md")


def _traffic_bytes() -> dict:
    import re

    try:
        with open(TRAFFIC_SUMMARY) as fh:
            for line in fh:
                if line.startswith("traffic_bytes_per_launch:"):
                    return {k: int(v) for k, v in re.findall(r"(\w+)=(\d+)", line)}
    except OSError:
        pass
    return {}


TRAFFIC_BYTES = _traffic_bytes()


def time_gpu(fn, steps: int, warmup: int):
    """Average seconds per call over `steps` calls, HIP events on the launch stream."""
    import torch

    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return start.elapsed_time(stop) * 1e-3 / steps, wall / steps


def time_settled(fn, warm_ms: float = 25.0, timed_ms: float = 100.0) -> dict:
    """Time-based conditioning like the reference's ``do_bench`` (tests/benchmark.py:19-22):
    an estimate from 5 launches sizes ~``warm_ms`` of untimed and ~``timed_ms`` of timed launches."""
    import torch

    fn(0)
    torch.cuda.synchronize()
    est, _ = time_gpu(fn, 5, 0)
    n_warm = max(1, int(warm_ms * 1e-3 / est))
    n_rep = max(1, int(timed_ms * 1e-3 / est))
    t, _ = time_gpu(fn, n_rep, n_warm)
    return {"us_per_launch": t * 1e6, "warmup_launches": n_warm + 6, "timed_launches": n_rep}


def mfma_ceiling(dev) -> dict:
    """What a loop of nothing but MFMAs sustains on this GPU for zeros and for N(0,1) bf16
    operands (csrc/kernels/lf_mfma_probe.hip): the chip lowers its clock with the switching
    activity of the operands, so the second figure, not the published peak, bounds any
    kernel on the benchmark's inputs."""
    import ctypes

    import torch

    from loopfuse_amd import lowering, runtime

    class Probe(ctypes.Structure):
        _fields_ = [("out", ctypes.c_void_p), ("data", ctypes.c_void_p), ("clk", ctypes.c_void_p), ("iters", ctypes.c_int)]

    nwg, iters = 512, 3000
    out = torch.zeros(nwg * 256, dtype=torch.float32, device=dev)
    clk = torch.zeros(2 * nwg, dtype=torch.int64, device=dev)
    res = {}
    for kind, shape in ((0, "32x32x16"), (1, "16x16x32")):
        code, _, _ = runtime.compile_source(runtime.read_kernel_source("lf_mfma_probe.hip"), f"lf_mfma_probe_k{kind}",
                                            list(lowering.COMMON_OPTS) + [f"-DLF_PROBE_KIND={kind}"])
        kern = runtime.Module(code).kernel("lf_mfma_probe")
        for name, data in (("zeros", torch.zeros(65536 * 8, dtype=torch.bfloat16, device=dev)),
                           ("normal", torch.randn(65536 * 8, device=dev).to(torch.bfloat16))):
            prm = Probe(out.data_ptr(), data.data_ptr(), clk.data_ptr(), iters)
            t, _ = time_gpu(lambda i: kern.launch((nwg, 1, 1), (256, 1, 1), prm), 6, 3)
            c = clk.cpu().view(-1, 2).double()
            res[f"{shape}_{name}"] = {"tflops": iters * 32 * 32768.0 * 4 * nwg / t / 1e12,
                                      "shader_mhz": float((c[:, 0] / c[:, 1]).median() * 100)}
    res["prefill_kernel"] = prefill_operand_and_shape_rates(dev)
    return res


def prefill_operand_and_shape_rates(dev) -> dict:
    """The product prefill kernel itself, same instruction stream, on other operands and
    shapes: config 2 with Q = K = V = 0 (what the operands' switching activity costs), without
    the mask (what the diagonal tiles and the short q tiles cost), and at S = 8192 with the
    same number of tokens (what is left of the per-q-tile costs when a q tile runs 130 kv tiles)."""
    import dataclasses

    import torch

    from loopfuse_amd import workloads

    res = {}
    for B, S in ((8, 2048), (2, 8192)):
        for mask in ("causal", None):
            for data in ("normal", "zeros"):
                w = dataclasses.replace(workloads.make("c2", seed=0, B=B, S=S), mask=mask)
                if data == "zeros":
                    w = dataclasses.replace(w, q=torch.zeros_like(w.q), k=torch.zeros_like(w.k), v=torch.zeros_like(w.v))
                w = w.to(dev)
                out = workloads.run(w)
                r = time_settled(lambda i: workloads.run(w, out=out))
                flops = 4.0 * B * 32 * S * S * 128 * (0.5 if mask else 1.0)
                res[f"B{B}_S{S}_{mask or 'nomask'}_{data}"] = {"us_per_launch": r["us_per_launch"],
                                                               "tflops": flops / r["us_per_launch"] / 1e6}
    return res


def backward_leg(dev) -> dict:
    """Forward (with the row log-sum-exp written) and backward of config 2, steady state.  The
    backward counts 2.5 times the forward's flop (five matrix products against two), the usual
    convention; it is not part of the headline metric -- the reference has no backward."""
    import torch

    from loopfuse_amd import lowering, workloads

    w = workloads.make("c2", seed=0).to(dev)
    plan = lowering.AttnPlan(mask=w.mask, window=w.window, scale=w.scale)
    lse = torch.empty(w.q.shape[:-1], dtype=torch.float32, device=dev)
    o = lowering.attention(w.q, w.k, w.v, plan, lse=lse)
    dout = torch.randn_like(o)
    fwd = time_settled(lambda i: lowering.attention(w.q, w.k, w.v, plan, lse=lse, out=o))
    bwd = time_settled(lambda i: lowering.attention_backward(w.q, w.k, w.v, o, lse, dout, plan), 25.0, 200.0)
    flop = w.flops()
    return {"workload": "config 2 (causal bf16 B8 H32 S2048 D128)",
            "forward_with_lse_us": fwd["us_per_launch"], "forward_tflops": flop / fwd["us_per_launch"] / 1e6,
            "backward_us": bwd["us_per_launch"], "backward_tflops": 2.5 * flop / bwd["us_per_launch"] / 1e6,
            "kernels": "lf_attn_bwd_delta+lf_attn_bwd_dkdv+lf_attn_bwd_dq"}


def via_backend(dev, steps: int, warmup: int) -> dict:
    """The two headline workloads through the drop-in path: the reference's own graph
    spellings (tests/benchmark.py:78-84 causal prefill, 400-406 paged GQA decode with the
    pool's pages folded into the sequence) under ``torch.compile(backend=loopfuse_backend,
    dynamic=True)``; device and host time per call."""
    import torch

    from loopfuse_amd import loopfuse_backend, workloads
    from loopfuse_amd.torch_backend import interface

    def prefill(q, k, v):
        qk = q @ k.transpose(-2, -1) * (q.shape[-1] ** -0.5)
        return torch.softmax(torch.ops.loopfuse.causal_mask(qk), dim=-1) @ v

    def decode(Q, Kc, kt, Vc, vt):
        B, pages = kt.shape
        P, H, D = Kc.shape[1:]
        K = torch.ops.loopfuse.paged_load(Kc, kt).reshape(B, pages * P, H, D).transpose(-3, -2)
        V = torch.ops.loopfuse.paged_load(Vc, vt).reshape(B, pages * P, H, D).transpose(-3, -2)
        QK = Q @ K.transpose(-2, -1) * (Q.shape[-1] ** -0.5)
        return torch.softmax(QK, dim=-1) @ V

    res = {}
    with torch.inference_mode():
        w = workloads.make("c2", seed=0).to(dev)
        fn = torch.compile(prefill, backend=loopfuse_backend, dynamic=True)
        before = interface.stats["fused"]
        fn(w.q, w.k, w.v)
        torch.cuda.synchronize()
        st = time_settled(lambda i: fn(w.q, w.k, w.v))
        t, wall = time_gpu(lambda i: fn(w.q, w.k, w.v), steps, warmup)
        res["prefill_c2"] = {"us_per_call": t * 1e6, "host_us_per_call": wall * 1e6, "settled_us_per_call": st["us_per_launch"],
                             "tflops": w.flops() / t / 1e12, "fused_calls": interface.stats["fused"] - before}
        del w
        base = workloads.make("c5", seed=0)
        nrot = max(2, int(1.5e9 // base.kv_bytes()) + 1)
        ws = [base.to(dev)]
        for _ in range(nrot - 1):
            ws.append(dataclasses.replace(ws[0], k=ws[0].k.clone(), v=ws[0].v.clone()))
        B, Hq, _, D = base.q.shape
        Hkv = base.k.shape[2]
        qv = [x.q.view(B, Hkv, Hq // Hkv, D) for x in ws]      # the reference's [B, Hkv, group, D] view of Q
        fn = torch.compile(decode, backend=loopfuse_backend, dynamic=True)
        before = interface.stats["fused"]
        call = lambda i: fn(qv[i % nrot], ws[i % nrot].k, ws[i % nrot].k_table, ws[i % nrot].v, ws[i % nrot].v_table)
        call(0)
        torch.cuda.synchronize()
        st = time_settled(call)
        t, wall = time_gpu(call, steps, warmup)
        res["decode_c5"] = {"us_per_call": t * 1e6, "host_us_per_call": wall * 1e6, "settled_us_per_call": st["us_per_launch"],
                            "gbs": base.kv_bytes() / t / 1e9, "fused_calls": interface.stats["fused"] - before}
    return res


def cpu_baseline(seconds: float = 12.0) -> dict:
    """The reference's eager CPU path (oracle port) on a bounded slice of the workload."""
    import torch

    from loopfuse_amd import workloads
    from oracle import attention_oracle as O

    cores = os.cpu_count() or 1
    if os.environ.get("OMP_NUM_THREADS"):
        cores = min(cores, int(os.environ["OMP_NUM_THREADS"]))
    torch.set_num_threads(cores)

    def run(q, k, v, budget):
        with torch.inference_mode():
            for _ in range(2):
                O.eager_reference_graph(q, k, v)
            ts = []
            t_end = time.perf_counter() + budget
            while time.perf_counter() < t_end and len(ts) < 2000:
                t0 = time.perf_counter()
                O.eager_reference_graph(q, k, v)
                ts.append(time.perf_counter() - t0)
        return statistics.median(ts), len(ts)

    # slice of config 2: one batch, four heads, full S and D; fp32 as the eager path computes
    w = workloads.make("c2", seed=0, B=1)
    q, k, v = (t[:, :4].float().contiguous() for t in (w.q, w.k, w.v))
    t2, n2 = run(q, k, v, seconds * 0.75)
    flops2 = 2 * 1 * 4 * 2048 * 2048 * 128
    # config 1 (the reference's own CPU-runnable case): fp32 B2 H8 S512 D64
    w1 = workloads.make("c1", seed=0)
    t1, n1 = run(w1.q, w1.k, w1.v, seconds * 0.25)
    flops1 = 2 * 2 * 8 * 512 * 512 * 64
    return {
        "value": flops2 / t2 / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"eager fp32 causal attention on config-2 slice B1 H4 S2048 D128, median of {n2} runs "
                  f"({t2 * 1e3:.1f} ms); config 1 (B2 H8 S512 D64 fp32): {flops1 / t1 / 1e12:.4f} TFLOP/s, "
                  f"{t1 * 1e3:.2f} ms median of {n1}",
        "c1_tflops": flops1 / t1 / 1e12,
        "c1_ms": t1 * 1e3,
    }


def generated_matmul(args, dev) -> dict:
    """Contractions of graphs without an attention on the generated MFMA kernels (loopfuse_amd/compiler/emit_gemm.py):
    ``a @ b.t() + bias`` on bf16 operands through the backend with its tuning off, against the same function run
    eagerly (library matmul + add) on the same GPU."""
    import torch

    from loopfuse_amd import loopfuse_backend
    from loopfuse_amd.compiler import generic

    res = {}
    old = os.environ.get("LOOPFUSE_AUTOTUNE")
    os.environ["LOOPFUSE_AUTOTUNE"] = "0"
    try:
        for m, n, k in ((4096, 4096, 4096), (8192, 8192, 8192), (16384, 4096, 1024)):
            g = torch.Generator().manual_seed(0)
            a, b, bias = (torch.randn(s, generator=g).to(torch.bfloat16).to(dev) for s in ((m, k), (n, k), (n,)))
            fn = lambda a, b, bias: a @ b.t() + bias      # noqa: E731
            torch._dynamo.reset()
            cf = torch.compile(fn, backend=loopfuse_backend)
            before = generic.counters["mfma"]
            cf(a, b, bias)
            assert generic.counters["mfma"] == before + 1, "the contraction did not run on the generated MFMA kernel"
            t, _ = time_gpu(lambda i: cf(a, b, bias), 30, 10)
            te, _ = time_gpu(lambda i: fn(a, b, bias), 30, 10)
            res[f"{m}x{n}x{k}"] = {"us_per_call": t * 1e6, "tflops": 2.0 * m * n * k / t / 1e12,
                                   "eager_us_per_call": te * 1e6, "eager_tflops": 2.0 * m * n * k / te / 1e12}
    finally:
        if old is None:
            os.environ.pop("LOOPFUSE_AUTOTUNE", None)
        else:
            os.environ["LOOPFUSE_AUTOTUNE"] = old
    return res


def torch_sdpa(args, dev) -> dict:
    """PyTorch's own fused attention on the same GPU and inputs: a same-hardware point of
    comparison (not the reference, which has no AMD path).  Softcap and the sliding window
    have no SDPA spelling, so only the causal config is timed for prefill; the decode config
    gets contiguous K/V (the page gather is done before the timed region)."""
    import torch
    import torch.nn.functional as F

    from loopfuse_amd import workloads

    res: dict = {}
    if args.workload == "c2" and args.only in (None, "prefill"):
        w = workloads.make("c2", seed=0).to(dev)
        t, _ = time_gpu(lambda i: F.scaled_dot_product_attention(w.q, w.k, w.v, is_causal=True), args.steps, args.warmup)
        res["prefill"] = {"workload": "c2", "us_per_launch": t * 1e6, "tflops": w.flops() / t / 1e12}
        del w
    if args.only in (None, "decode"):
        w = workloads.make(args.decode_workload, seed=0).to(dev)
        k, v = w.k, w.v
        if w.k_table is not None:
            B, hkv, d = w.q.shape[0], w.k.shape[-2], w.k.shape[-1]
            k = w.k[w.k_table.long()].reshape(B, -1, hkv, d).transpose(1, 2).contiguous()
            v = w.v[w.v_table.long()].reshape(B, -1, hkv, d).transpose(1, 2).contiguous()
        gqa = w.q.shape[1] != k.shape[1]
        t, _ = time_gpu(lambda i: F.scaled_dot_product_attention(w.q, k, v, enable_gqa=gqa), args.steps, min(args.warmup, 20))
        res["decode"] = {"workload": args.decode_workload + (" (contiguous K/V)" if w.k_table is not None else ""),
                         "us_per_launch": t * 1e6, "gbs": w.kv_bytes() / t / 1e9}
    return res


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", choices=["prefill", "decode"], default=None,
                    help="time only one of the two kernels (profiling aid)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 512 MiB device copy (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--torch-sdpa", action="store_true",
                    help="also time torch.nn.functional.scaled_dot_product_attention on the same GPU and inputs "
                         "(config 2 as is; the decode config with its pages gathered into contiguous K/V beforehand)")
    ap.add_argument("--no-settled", action="store_true",
                    help="skip the steady-state conditioning legs (for counter runs under rocprofv3, where every launch is slow)")
    ap.add_argument("--no-via-backend", action="store_true",
                    help="skip the legs that time the two headline workloads through torch.compile(backend=loopfuse_backend)")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="also run the MFMA-only probe on zeros and on N(0,1) operands (the data-dependent clock ceiling), and "
                         "the prefill kernel on zero operands, without the mask and at S = 8192")
    ap.add_argument("--generated-matmul", action="store_true",
                    help="also time a @ b.t() + bias on the generated MFMA kernels of the non-attention path")
    ap.add_argument("--backward", action="store_true",
                    help="also time the forward with its log-sum-exp output and the backward kernels on config 2")
    ap.add_argument("--workload", default="c2", help="prefill workload: c2 | c2_softcap | c3 | c2_mask (the causal mask given as a tensor)")
    ap.add_argument("--decode-workload", default="c5", help="decode workload: c5 | c4 | c5_padded | cache4096 (mask tensors: left padding / partly filled cache)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); "
              "the hot path shards over batch and heads with no exchange", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        return 3
    from loopfuse_amd import lowering, workloads

    dev = torch.device("cuda:0")
    out: dict = {}

    if args.copy_calibration:
        # a kernel whose HBM traffic is known exactly: 512 MiB read + 512 MiB written
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    pre = None
    if args.only in (None, "prefill"):
        w = workloads.make(args.workload, seed=0).to(dev)
        o = workloads.run(w)     # first call compiles / loads the code object
        torch.cuda.synchronize()
        settled = None if args.no_settled else time_settled(lambda i: workloads.run(w, out=o))
        t, wall = time_gpu(lambda i: workloads.run(w, out=o), args.steps, args.warmup)
        pre = {"workload": args.workload, "sec": t, "wall_sec": wall, "flops": w.flops(), "settled": settled,
               "kernels": lowering.attention.last_launch["kernels"]}
        del w, o

    dec = None
    if args.only in (None, "decode"):
        # rotate over copies of the KV pool so that no launch finds its input in the
        # 256 MB Infinity Cache
        base = workloads.make(args.decode_workload, seed=0)
        nrot = max(2, int(1.5e9 // base.kv_bytes()) + 1)
        ws = [base.to(dev)]
        for _ in range(nrot - 1):
            ws.append(dataclasses.replace(ws[0], k=ws[0].k.clone(), v=ws[0].v.clone()))
        o = workloads.run(ws[0])
        torch.cuda.synchronize()
        dsettled = None if args.no_settled else time_settled(lambda i: workloads.run(ws[i % nrot], out=o))
        t, wall = time_gpu(lambda i: workloads.run(ws[i % nrot], out=o), args.steps, args.warmup)
        dec = {"workload": args.decode_workload, "sec": t, "wall_sec": wall, "bytes": base.kv_bytes(), "rotation": nrot,
               "settled": dsettled, "kernels": lowering.attention.last_launch["kernels"]}
        # extra field: the streaming kernel alone (its partial results left unmerged, O not written)
        tk, _ = time_gpu(lambda i: workloads.run(ws[i % nrot], out=o, merge_splits=False), args.steps, 20)
        dec["kernel_sec"] = tk
        dec["stream_kernels"] = lowering.attention.last_launch["kernels"]
        del ws, o

    primary = pre if pre is not None else dec
    if pre is not None:
        tflops = pre["flops"] / pre["sec"] / 1e12
        out.update({
            "metric": "prefill TFLOP/s + decode HBM GB/s on 1 MI355X (% of roofline)",
            "value": tflops, "unit": "TFLOP/s",
        })
        out["roofline"] = {"bound": "mfma", "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                           "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": TRAFFIC_BYTES.get(args.workload),
                           "kernel": "+".join(pre["kernels"]), "us_per_launch": pre["sec"] * 1e6}
        st = pre["settled"]
        if st is not None:
            out["settled"] = {"value": pre["flops"] / st["us_per_launch"] / 1e6, "unit": "TFLOP/s",
                              "frac": pre["flops"] / st["us_per_launch"] / 1e6 / MFMA_BF16_PEAK_TFLOPS, **st,
                              "protocol": "about 25 ms of untimed launches, then about 100 ms of timed ones (the reference's do_bench)"}
    if dec is not None:
        gbs = dec["bytes"] / dec["sec"] / 1e9
        kgbs = dec["bytes"] / dec["kernel_sec"] / 1e9
        d = {"workload": dec["workload"], "value": gbs, "unit": "GB/s", "us_per_launch": dec["sec"] * 1e6,
             "frac_of_hbm_peak": gbs / HBM_PEAK_GBS, "kernels": "+".join(dec["kernels"]),
             "host_us_per_launch": dec["wall_sec"] * 1e6, "kv_pool_rotation": dec["rotation"],
             # the roofline is read on the whole step (every launch that it takes to write O)
             "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": gbs / HBM_PEAK_GBS, "traffic": TRAFFIC_BYTES.get(args.decode_workload),
                          "kernel": "+".join(dec["kernels"]), "us_per_launch": dec["sec"] * 1e6},
             "settled": None if dec["settled"] is None else
             {"value": dec["bytes"] / dec["settled"]["us_per_launch"] / 1e3, "unit": "GB/s",
              "frac": dec["bytes"] / dec["settled"]["us_per_launch"] / 1e3 / HBM_PEAK_GBS, **dec["settled"]},
             "stream_kernel_alone": {"kernel": "+".join(dec["stream_kernels"]), "us_per_launch": dec["kernel_sec"] * 1e6,
                                     "gbs": kgbs, "note": "partials left unmerged, O not written"}}
        if pre is None:
            out.update({"metric": "prefill TFLOP/s + decode HBM GB/s on 1 MI355X (% of roofline)",
                        "value": gbs, "unit": "GB/s", "roofline": d["roofline"]})
        out["decode"] = d
    out.update({
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": primary["sec"] * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": ("config 2: causal prefill bf16 B8 H32 S2048 D128" if pre is not None and args.workload == "c2"
                                else primary["workload"]),
                   "decode_workload": "config 5: paged GQA decode bf16 B64 Hq32/Hkv8 K_len2048 D128 page16"
                   if args.decode_workload == "c5" else args.decode_workload},
    })
    if not args.no_via_backend and not args.no_settled and args.only is None and args.workload == "c2" and args.decode_workload == "c5":
        out["via_backend"] = via_backend(dev, args.steps, args.warmup)
    if args.mfma_ceiling:
        out["mfma_ceiling"] = mfma_ceiling(dev)
    if args.backward:
        out["backward"] = backward_leg(dev)
    if args.torch_sdpa:
        out["torch_sdpa"] = torch_sdpa(args, dev)
    if args.generated_matmul:
        out["generated_matmul"] = generated_matmul(args, dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
