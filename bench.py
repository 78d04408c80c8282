#!/usr/bin/env python3
"""Benchmark of the MI355X W8A8 LoRA linear forward path.

One step = one pass of the hot path over one batch of synthetic input.  The
default workload is the Qwen3-8B gate/up projection at M = 4096 (RMSNorm ->
W8A8 [4096 x 4096] x [4096 x 24576] + 8 rank-32 adapters routed per row ->
SwiGLU).  Inputs are resident in HBM before the timed region.  Prints ONE JSON
line; ``value`` is int8 TOPS of the whole step (2*M*K*N per step, every kernel of
the step included); ``roofline`` prices the dominant kernel (the int8 MFMA GEMM)
from HIP events around that kernel alone, against the published peak and against
the rate the same MFMA instruction sustains on realistic operands in a
register-only loop; ``decode`` is the roofline block of the decode-shaped call
(M = 16 down projection, HBM-bound) against the published bandwidth and a measured
read-only stream; ``cpu_baseline`` times the NumPy oracle on a bounded row sample
of the same workload on the host cores.  ``--workload calibration`` prints the
ceilings alone, ``--workload qwen3-4b-attn-mixed-m`` a table over M of the
attention projections.
"""

from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

INT8_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA, published (5.0 POP/s)
BF16_PEAK_TFLOPS = 2500.0 # MI355X dense bf16 MFMA, published (2.5 PFLOP/s)
HBM_PEAK_GBS = 8000.0     # MI355X HBM3E, published

WORKLOADS = {
    # ceilings of the part: register-only int8 MFMA loops and a read-only stream
    "calibration": dict(calibration=True),
    # benchmark configuration 4: Qwen3-4B attention projections over M, 4 adapters rank 64 alpha 128, Student-t(3) rows
    "qwen3-4b-attn-mixed-m": dict(mixed_m=True, shapes=[("qkv", 2560, 6144), ("o_proj", 4096, 2560)],
                                  m_values=[1, 64, 512, 2048], n_adapters=4, rank=64, alpha=128, seed=4),
    # name: (m, k, n, adapters, rank, alpha, rms, swiglu, residual, idx_mode, seed)
    "qwen3-8b-gate_up-m4096": dict(m=4096, k=4096, n=24576, n_adapters=8, rank=32, rms=True, swiglu=True,
                                   idx_mode="uniform", seed=2),
    "qwen3-8b-down-m16-decode": dict(m=16, k=12288, n=4096, n_adapters=16, rank=32, residual=True,
                                     idx_mode="arange", seed=3),
    "single-linear-m128": dict(m=128, k=1024, n=3072, n_adapters=1, rank=16, idx_mode="zero", seed=1),
    # backward (dx pull-back + LoRA cotangents) of the plain linear at the gate/up and down shapes
    "qwen3-8b-gate_up-m4096-backward": dict(m=4096, k=4096, n=24576, n_adapters=8, rank=32, idx_mode="uniform",
                                            seed=2, backward=True),
    "qwen3-8b-down-m4096-backward": dict(m=4096, k=12288, n=4096, n_adapters=8, rank=32, idx_mode="uniform",
                                         seed=4, backward=True),
    # backward of the fused RMSNorm -> gate/up -> SwiGLU call: forward recomputation, SwiGLU pull-back,
    # linear backward, RMSNorm pull-back
    "qwen3-8b-gate_up-m4096-fused-backward": dict(m=4096, k=4096, n=24576, n_adapters=8, rank=32, rms=True,
                                                  swiglu=True, idx_mode="uniform", seed=2, backward=True),
    # token routing around the expert GEMMs at the Qwen3-30B-A3B geometry: softmax / top-8 of 128 experts,
    # stable sort of the 32768 (token, choice) pairs with the gather of their rows, weighted combine
    "qwen3-30b-a3b-moe-routing-t4096": dict(m=4096, n_experts=128, top_k=8, hidden=2048, seed=6, moe_routing=True),
    # the whole expert MLP of benchmark configuration 5 (T = 2048): route, dispatch, grouped gate/up + SwiGLU, grouped down,
    # combine; rank-16 LoRA on every expert
    "qwen3-30b-a3b-moe-mlp-t2048": dict(m=2048, n_experts=128, top_k=8, hidden=2048, intermediate=768, rank=16,
                                        seed=5, moe_mlp=True),
    # backward of the two grouped expert projections of that layer (16384 sorted pairs over 128 experts): dx and the
    # LoRA cotangents of gate/up [2048 -> 1536] and of down [768 -> 2048], one native call each
    "qwen3-30b-a3b-moe-experts-t2048-backward": dict(m=2048, n_experts=128, top_k=8, hidden=2048, intermediate=768,
                                                     rank=16, seed=5, moe_backward=True),
    # group-scaled W4A8 (int4 codes, one scale per 128 k and output, activations quantized per row and group)
    # at the Qwen3-8B down-projection shape, 8 adapters rank 32
    "qwen3-8b-down-m4096-w4a8-g128": dict(m=4096, k=12288, n=4096, n_adapters=8, rank=32, weight_bits=4,
                                          activation_bits=8, group_size=128, seed=8, gq=True),
    # Qwen3.5-4B attention input stage: RMSNorm -> W8A8 QKV [2560 -> 10240] + 4 adapters rank 64 ->
    # split, Q/K RMSNorm, partial RoPE (16 query heads, 4 kv heads, head_dim 256, 64 rotary dims)
    "qwen3.5-4b-qkv-m2048": dict(m=2048, k=2560, n=10240, n_adapters=4, rank=64, alpha=128, rms=True,
                                 idx_mode="uniform", seed=5,
                                 qkv=dict(num_query_heads=16, num_kv_heads=4, head_dim=256, rotary_dim=64)),
    # backward of that stage with frozen norm weights: split / norm / RoPE pull-back, linear backward with
    # the LoRA cotangents, decoder-norm pull-back (projection and normalized rows kept by the forward)
    "qwen3.5-4b-qkv-m2048-backward": dict(m=2048, k=2560, n=10240, n_adapters=4, rank=64, alpha=128, rms=True,
                                          idx_mode="uniform", seed=5, qkv_backward=True,
                                          qkv=dict(num_query_heads=16, num_kv_heads=4, head_dim=256, rotary_dim=64)),
}

# HBM bytes per launch of the dominant kernel(s): read from the counter lines of the committed rocprofv3
# --pmc summaries under profiles/ (FETCH_SIZE and WRITE_SIZE in KiB per dispatch), each scaled by what the same
# counter reads for the 256 MiB device copy of the same run (a kernel of known traffic, 16-byte loads).
# workload -> (summary file, regular expressions naming the kernels whose traffic is summed)
PROFILE_TRAFFIC = {
    "qwen3-8b-gate_up-m4096": ("w8a8_gemm16_kernel__qwen3-8b-gate_up-m4096.txt", [r"w8a8_gemm16_kernel<1, 2, 4>"]),
    "qwen3-8b-down-m16-decode": ("skinny_stream_kernel__qwen3-8b-down-m16-decode.txt",
                                 [r"skinny_quant_kernel<", r"skinny_stream_kernel<"]),
    "qwen3-8b-gate_up-m4096-backward": ("bwd_dx_kernel__qwen3-8b-gate_up-m4096-backward.txt", [r"bwd_dx_kernel<"]),
    "qwen3-30b-a3b-moe-mlp-t2048": ("w8a8_gemm_kernel_grouped__qwen3-30b-a3b-moe-mlp-t2048.txt",
                                    [r"w8a8_gemm_kernel<1, 1, "]),  # grouped gate/up with the SwiGLU epilogue
    "qwen3-30b-a3b-moe-experts-t2048-backward": ("bwd_dx_kernel_grouped__qwen3-30b-a3b-moe-experts-t2048-backward.txt",
                                                 [r"bwd_pack_dy_kernel<0>", r"bwd_dx_kernel<0, true>"]),
    "qwen3-8b-gate_up-m4096-fused-backward": ("swiglu_bwd_kernel__qwen3-8b-gate_up-m4096-fused-backward.txt",
                                              [r"bwd_dx_kernel<"]),
    "qwen3-8b-down-m4096-w4a8-g128": ("gq_gemm_kernel__qwen3-8b-down-m4096-w4a8-g128.txt", [r"gq_gemm_(lds_)?kernel<"]),
    "qwen3-30b-a3b-moe-routing-t4096": ("moe_spread_kernel__qwen3-30b-a3b-moe-routing-t4096.txt",
                                        [r"moe_hist_kernel", r"moe_scan_kernel", r"moe_scatter_kernel",
                                         r"moe_spread_kernel"]),
    "qwen3.5-4b-qkv-m2048": ("qkv_post_kernel__qwen3.5-4b-qkv-m2048.txt", [r"qkv_post_kernel\("]),
    "qwen3.5-4b-qkv-m2048-backward": ("qkv_post_bwd_kernel__qwen3.5-4b-qkv-m2048-backward.txt",
                                      [r"qkv_post_bwd_kernel<4, false>"]),
}
_COUNTER_LINE = re.compile(r"^(?P<name>.+?)\s+grid\s+(?P<grid>\d+)\s+(?P<ctr>FETCH_SIZE|WRITE_SIZE) avg\s+"
                           r"(?P<kib>[0-9.]+) KiB over (?P<n>\d+) dispatches")
COPY_KIB = 262144.0  # the calibration copy moves 256 MiB each way


def measured_traffic_bytes(workload, profiles_dir=None):
    """HBM bytes per launch of the workload's dominant kernel(s) from its committed counter summary, or None.

    Every kernel named for the workload must appear for each counter and the summary must hold the
    calibration copy; anything else (no summary yet, renamed kernel) gives None rather than a stale figure."""
    entry = PROFILE_TRAFFIC.get(workload)
    if entry is None:
        return None
    path = Path(profiles_dir or ROOT / "profiles") / entry[0]
    if not path.exists():
        return None
    copy = {}
    rows = []
    for line in path.read_text().splitlines():
        hit = _COUNTER_LINE.match(line)
        if not hit:
            continue
        # the copy of known size: the library's cal_copy_kernel, or in older summaries the runtime's 256 MiB
        # buffer copy (grid 131072, a single dispatch)
        if "cal_copy_kernel" in hit["name"] or (hit["name"].startswith("__amd_rocclr_copyBuffer")
                                               and int(hit["grid"]) == 131072 and int(hit["n"]) == 1):
            copy[hit["ctr"]] = float(hit["kib"])
        rows.append((hit["name"], hit["ctr"], float(hit["kib"]), int(hit["n"])))
    if set(copy) != {"FETCH_SIZE", "WRITE_SIZE"} or min(copy.values()) <= 0:
        return None
    total = 0.0
    for pattern in entry[1]:
        for ctr in ("FETCH_SIZE", "WRITE_SIZE"):
            # a kernel launched with several grids (a first call that also packs, then the steady calls)
            # has a line per grid: the one with the most dispatches is the steady call
            vals = sorted((n, kib) for name, c, kib, n in rows if c == ctr and re.search(pattern, name))
            if not vals or (len(vals) > 1 and vals[-1][0] == vals[-2][0]):
                return None
            total += vals[-1][1] * (COPY_KIB / copy[ctr])
    return int(total * 1024)


def algorithmic_bytes(c):
    m, k, n = c["m"], c["k"], c["n"]
    n_out = n // 2 if c.get("swiglu") else n
    total = 2 * m * k + k * n + 4 * n + 2 * m * n_out + 4 * m
    if c.get("n_adapters"):
        used = min(c["n_adapters"], m)
        total += 2 * used * c["rank"] * (k + n)
    if c.get("rms"):
        total += 4 * k
    if c.get("residual"):
        total += 2 * m * n_out
    return total


def gemm_kernel_bytes(c):
    """Algorithmic bytes of the GEMM kernel alone: int8 codes in, weights, LoRA B, output."""
    m, k, n = c["m"], c["k"], c["n"]
    n_out = n // 2 if c.get("swiglu") else n
    total = m * k + k * n + 4 * n + 4 * m + 2 * m * n_out
    if c.get("n_adapters"):
        used = min(c["n_adapters"], m)
        total += 2 * used * c["rank"] * n + 4 * m * c["rank"]
    if c.get("residual"):
        total += 2 * m * n_out
    return total


def _stream_ptr(dev):
    import torch

    return int(torch.cuda.current_stream(dev).cuda_stream)


def calibration_operands(kind, nbytes, seed=1234):
    """Operand bytes of the register-only MFMA loop.  Per wave 16 fragments of 1 KiB: 8 A then 8 B operands.
    "zeros"; "random": random bits; "codes": what the path multiplies - activation codes of normal rows
    quantized by their absolute maximum over 4096 samples (sigma about 127 / 3.9) against uniform weight codes."""
    rng = np.random.default_rng(seed)
    if kind == "zeros":
        return np.zeros(nbytes, np.uint8)
    if kind == "random":
        return rng.integers(0, 256, nbytes, dtype=np.uint8)
    frag = (np.arange(nbytes) >> 10) & 15
    act = np.clip(np.rint(rng.standard_normal(nbytes) * (127.0 / 3.9)), -127, 127).astype(np.int8)
    wgt = rng.integers(-127, 128, nbytes, dtype=np.int8)
    return np.where(frag < 8, act, wgt).astype(np.int8).view(np.uint8)


def measure_mfma_ceiling(native, dev, shape, kind, seconds=0.4, iters=2048):
    """Sustained int8 TOP/s of the register-only MFMA loop and the shader clock it ran at."""
    import torch

    lib = native.load()
    nbytes = int(lib.mi355_w8a8_calibrate_operand_bytes())
    ops = float(lib.mi355_w8a8_calibrate_mfma_ops(shape, iters))
    src = torch.from_numpy(calibration_operands(kind, nbytes)).to(dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = _stream_ptr(dev)

    def launch():
        native.check("mi355_w8a8_calibrate_mfma_v1",
                     lib.mi355_w8a8_calibrate_mfma_v1(shape, src.data_ptr(), iters, clocks.data_ptr(), sink.data_ptr(),
                                                      stream))

    launch()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record(); launch(); b.record()
    torch.cuda.synchronize()
    n = max(4, int(seconds * 1e3 / max(a.elapsed_time(b), 1e-3)))
    for _ in range(n):  # the power controller settles over some hundred milliseconds: untimed
        launch()
    a.record()
    for _ in range(n):
        launch()
    b.record()
    torch.cuda.synchronize()
    ms = a.elapsed_time(b) / n
    cyc, ticks = (int(v) for v in clocks.cpu())
    return {"shape": "16x16x64" if shape else "32x32x32", "operands": kind, "tops": ops / (ms * 1e-3) / 1e12,
            "kernel_avg_ms": ms, "launches": n, "shader_mhz": cyc / max(ticks, 1) * 100.0}


def measure_read_ceiling(native, dev, gib=2, launches=20):
    """Sustained GB/s of a read-only stream over a buffer far beyond the 256 MB last-level cache."""
    import torch

    lib = native.load()
    nbytes = gib << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(3)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = _stream_ptr(dev)

    def launch():
        native.check("mi355_w8a8_calibrate_read_v1",
                     lib.mi355_w8a8_calibrate_read_v1(src.data_ptr(), nbytes, sink.data_ptr(), stream))

    for _ in range(3):
        launch()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(launches):
        launch()
    b.record()
    torch.cuda.synchronize()
    ms = a.elapsed_time(b) / launches
    return {"bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9, "kernel_avg_ms": ms, "launches": launches}


def bench_calibration(args, pkg, dev):
    """What this part sustains: register-only int8 MFMA loops (both instruction shapes; zero, random and
    realistic operands) and a read-only stream.  The fractions of the other workloads can be read against
    these as well as against the published peaks."""
    native = pkg._native
    mfma = [measure_mfma_ceiling(native, dev, shape, kind, seconds=1.0)
            for kind in ("zeros", "random", "codes") for shape in (0, 1)]
    read = measure_read_ceiling(native, dev)
    best = max(r["tops"] for r in mfma if r["operands"] == "codes")
    print(json.dumps({
        "metric": "sustained int8 MFMA TOP/s on realistic operand codes (register-only loop); read stream GB/s",
        "value": best, "unit": "TOPS", "n_gpus": 1, "steps": sum(r["launches"] for r in mfma), "warmup": 0,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic", "config": {"workload": args.workload},
        "mfma": mfma, "read": read,
        "roofline": {"bound": "mfma", "achieved": best, "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                     "frac": best / INT8_PEAK_TOPS, "traffic": None, "kernel": "cal_mfma_kernel<1>"},
        "read_frac_of_hbm_peak": read["gbs"] / HBM_PEAK_GBS}))
    return 0


def cpu_baseline(case, cfg, sample_rows):
    """Time the NumPy oracle on the first ``sample_rows`` rows of the workload."""
    import w8a8_cases as wc

    def rows_of(count):
        sub = dict(case)
        sub["m"] = count
        sub["x"] = case["x"][:count]
        for key in ("idx", "residual"):
            if key in case:
                sub[key] = case[key][:count]
        return sub

    wc.oracle_forward(rows_of(min(sample_rows, 32)))  # warm-up: BLAS thread pool, page faults
    sub = rows_of(sample_rows)
    best = float("inf")
    out = None
    repeats = 0
    while repeats < 3 and (repeats == 0 or best < 5.0):
        t0 = time.perf_counter()
        out = wc.oracle_forward(sub)
        best = min(best, time.perf_counter() - t0)
        repeats += 1
    ops = 2.0 * sample_rows * cfg["k"] * cfg["n"]
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    threads = int(os.environ.get("OMP_NUM_THREADS", cores))
    return out, {"value": ops / best / 1e12, "unit": "TOPS", "cores": min(cores, threads), "kind": "port",
                 "sample": f"first {sample_rows} of {cfg['m']} rows, full K and N, NumPy oracle "
                           f"(float64 BLAS for the exact integer GEMM), best of {repeats} after a 32-row warm-up, {best:.3f} s",
                 "seconds": best}


def bench_backward(args, cfg, pkg, dev):
    """One step = one backward call (tables, dy packing + r, z, dx pull-back, dA / dB / dscaling).
    ``value`` counts the pull-back's 2*M*K*N only; the roofline prices bwd_dx_kernel alone
    (bf16 MFMA) from HIP events around launches of that kernel."""
    import torch

    import w8a8_cases as wc
    from oracle import w8a8_oracle as o

    native, w8 = pkg._native, pkg.w8a8_lora
    case = wc.make_case(cfg["m"], cfg["k"], cfg["n"], n_adapters=cfg["n_adapters"], rank=cfg["rank"],
                        seed=cfg["seed"], idx_mode=cfg.get("idx_mode", "uniform"))
    rng = np.random.default_rng(cfg["seed"] + 1000)
    dy = o.bf16_round(rng.standard_normal((cfg["m"], cfg["n"])).astype(np.float32))
    t = wc.to_torch(case, dev)
    dy_t = torch.from_numpy(dy).to(dev).to(torch.bfloat16)
    plan = w8.BackwardPlan(t["x"], dy_t, t["weight"], t.get("a"), t.get("b"), t.get("s"),
                           adapter_indices=t.get("idx"))
    dx_only = w8.BackwardPlan(None, dy_t, t["weight"], t.get("a"), t.get("b"), t.get("s"),
                              adapter_indices=t.get("idx"), need_lora_grads=False)
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        plan.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        plan.run()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    flops = 2.0 * cfg["m"] * cfg["k"] * cfg["n"]
    dx_only.run()  # fills its workspace; the kernel-only launches below reuse it
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in ev:
        a.record()
        dx_only.run(native.FLAG_SKIP_PROLOGUE)
        b.record()
    torch.cuda.synchronize()
    k_ms = np.asarray([a.elapsed_time(b) for a, b in ev])
    achieved = flops / (float(k_ms.mean()) * 1e-3) / 1e12
    got = [None if v is None else v.to(torch.float32).cpu().numpy() for v in plan.run()]
    torch.cuda.synchronize()
    m, k, n = cfg["m"], cfg["k"], cfg["n"]
    result = {
        "metric": "W8A8-LoRA linear backward (W8A16 pull-back + LoRA cotangents), TFLOP/s of 2*M*K*N per call",
        "value": flops / (ms_per_step * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, **{kk: v for kk, v in cfg.items() if kk != "seed"}},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / BF16_PEAK_TFLOPS, "traffic": measured_traffic_bytes(args.workload),
                     "kernel": "bwd_dx_kernel",
                     "kernel_avg_ms": float(k_ms.mean()), "kernel_min_ms": float(k_ms.min()),
                     "algorithmic_flops": flops,
                     # dy once, int8 weight once, dx once (the kernel reads dy re-laid-out by the packing pass)
                     "algorithmic_bytes": 2 * m * n + k * n + 2 * m * k},
    }
    if not args.no_cpu_baseline:
        rows = args.cpu_rows or 256
        sel = slice(0, rows)
        t1 = time.perf_counter()
        want = o.quantized_lora_linear_multi_bwd(case["x"][sel], case["weight"], case["a"], case["b"], case["s"],
                                                 case["idx"][sel], dy[sel], relaxed_weight=True)
        secs = time.perf_counter() - t1
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            cores = os.cpu_count() or 1
        threads = int(os.environ.get("OMP_NUM_THREADS", cores))
        result["cpu_baseline"] = {"value": 2.0 * rows * k * n / secs / 1e12, "unit": "TFLOP/s",
                                  "cores": min(cores, threads), "kind": "port",
                                  "sample": f"first {rows} of {m} rows, full K and N, NumPy oracle backward "
                                            f"(float64 BLAS), one run, {secs:.3f} s", "seconds": secs}
        rep = wc.compare(got[0][sel], want[0])  # dx rows are independent of the other rows
        result["parity_sample"] = {"rows": rows, "violations": rep["violations"], "size": rep["size"],
                                   "max_abs": rep["max_abs"], "bitwise_fraction": rep["bitwise_fraction"]}
    print(json.dumps(result))
    return 0


def bench_fused_backward(args, cfg, pkg, dev):
    """One step = one backward of the fused RMSNorm -> gate/up -> SwiGLU call: the forward
    recomputation (projection + normalized rows), the SwiGLU pull-back, the linear backward and the
    RMSNorm pull-back.  ``value`` counts the pull-back's 2*M*K*N only; the roofline prices
    bwd_dx_kernel (bf16 MFMA) as in the plain backward, and ``stages`` gives the two memory-bound
    pull-back kernels against HBM."""
    import torch

    import w8a8_cases as wc
    from oracle import w8a8_oracle as o

    native, w8 = pkg._native, pkg.w8a8_lora
    m, k, n = cfg["m"], cfg["k"], cfg["n"]
    case = wc.make_case(m, k, n, n_adapters=cfg["n_adapters"], rank=cfg["rank"], seed=cfg["seed"],
                        idx_mode=cfg.get("idx_mode", "uniform"), rms=True)
    rng = np.random.default_rng(cfg["seed"] + 2000)
    c = o.bf16_round(rng.standard_normal((m, n // 2)).astype(np.float32))
    t = wc.to_torch(case, dev)
    c_t = torch.from_numpy(c).to(dev).to(torch.bfloat16)
    plan = w8.FusedBackwardPlan(t["x"], t["gamma"], t["weight"], t["a"], t["b"], t["s"], c_t,
                                adapter_indices=t["idx"])
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        plan.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        plan.run()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    got = [v.to(torch.float32).cpu().numpy() for v in plan.run()]
    torch.cuda.synchronize()
    flops = 2.0 * m * k * n

    def timed(fn):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for a, b in ev:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return np.asarray([a.elapsed_time(b) for a, b in ev])

    # the stages on their own, on the buffers of a complete run; the two in-place stages write to
    # scratch outputs here so that every repetition sees the same operands
    lib = native.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    fwd_ms = timed(plan.fwd.run)
    scratch_n = torch.empty_like(plan.fwd.out)
    swiglu_ms = timed(lambda: native.check("swiglu_bwd", lib.mi355_w8a8_swiglu_bwd_v1(
        plan.fwd.out.data_ptr(), plan.d_product.data_ptr(), scratch_n.data_ptr(), m, n, stream)))
    plan.run_swiglu_stage()
    linear_ms = timed(plan.bwd.run)
    scratch_k = torch.empty_like(plan.bwd.dx)
    rms_ms = timed(lambda: native.check("rms_norm_bwd", lib.mi355_w8a8_rms_norm_bwd_v1(
        plan.x.data_ptr(), plan.gamma.data_ptr(), plan.bwd.dx.data_ptr(), scratch_k.data_ptr(), m, k, plan.eps,
        stream)))
    # the backward of a training forward that kept the projection and the normalized rows: no recomputation
    def saved_projection_backward():
        native.check("swiglu_bwd", lib.mi355_w8a8_swiglu_bwd_v1(
            plan.fwd.out.data_ptr(), plan.d_product.data_ptr(), scratch_n.data_ptr(), m, n, stream))
        plan.bwd.run()
        plan.run_rms_stage()
    saved_ms = timed(saved_projection_backward)
    dx_only = w8.BackwardPlan(None, plan.fwd.out, t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"],
                              need_lora_grads=False)
    dx_only.run()
    k_ms = timed(lambda: dx_only.run(native.FLAG_SKIP_PROLOGUE))
    achieved = flops / (float(k_ms.mean()) * 1e-3) / 1e12
    swiglu_bytes = 5 * m * n          # projection in and out (bf16 [M, N]) + cotangent in (bf16 [M, N/2])
    rms_bytes = 6 * m * k + 4 * k     # x, d_normalized in, d_x out (bf16 [M, K]) + gamma
    result = {
        "metric": "fused RMSNorm/gate-up/SwiGLU backward (recompute + pull-backs + LoRA cotangents), "
                  "TFLOP/s of 2*M*K*N per call",
        "value": flops / (ms_per_step * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, **{kk: v for kk, v in cfg.items() if kk != "seed"}},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / BF16_PEAK_TFLOPS, "traffic": measured_traffic_bytes(args.workload), "kernel": "bwd_dx_kernel",
                     "kernel_avg_ms": float(k_ms.mean()), "kernel_min_ms": float(k_ms.min()),
                     "algorithmic_flops": flops, "algorithmic_bytes": 2 * m * n + k * n + 2 * m * k},
        "stages": {
            "forward_recompute_ms": float(fwd_ms.mean()), "linear_backward_ms": float(linear_ms.mean()),
            "backward_with_saved_projection_ms": float(saved_ms.mean()),
            "swiglu_bwd_kernel": {"avg_ms": float(swiglu_ms.mean()), "algorithmic_bytes": swiglu_bytes,
                                  "achieved_gbs": swiglu_bytes / (float(swiglu_ms.mean()) * 1e-3) / 1e9,
                                  "frac_of_hbm": swiglu_bytes / (float(swiglu_ms.mean()) * 1e-3) / 1e9 / HBM_PEAK_GBS},
            "rms_norm_bwd_kernel": {"avg_ms": float(rms_ms.mean()), "algorithmic_bytes": rms_bytes,
                                    "achieved_gbs": rms_bytes / (float(rms_ms.mean()) * 1e-3) / 1e9,
                                    "frac_of_hbm": rms_bytes / (float(rms_ms.mean()) * 1e-3) / 1e9 / HBM_PEAK_GBS},
        },
    }
    if not args.no_cpu_baseline:
        rows = args.cpu_rows or 256
        sel = slice(0, rows)
        t1 = time.perf_counter()
        want = o.w8a8_rms_gate_up_lora_swiglu_bwd(case["x"][sel], case["gamma"], case["weight"], case["a"], case["b"],
                                                  case["s"], case["idx"][sel], c[sel])
        secs = time.perf_counter() - t1
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            cores = os.cpu_count() or 1
        threads = int(os.environ.get("OMP_NUM_THREADS", cores))
        result["cpu_baseline"] = {"value": 2.0 * rows * k * n / secs / 1e12, "unit": "TFLOP/s",
                                  "cores": min(cores, threads), "kind": "port",
                                  "sample": f"first {rows} of {m} rows, full K and N, NumPy oracle of the fused "
                                            f"backward (forward stages + pull-backs, float64 BLAS), one run, "
                                            f"{secs:.3f} s", "seconds": secs}
        gate = o.numerical_gate(got[0][sel], want[0])  # dx rows are independent of the other rows
        result["parity_sample"] = {"rows": rows, "relative_l2": gate["relative_l2"], "cosine": gate["cosine"]}
    print(json.dumps(result))
    return 0


def bench_moe_routing(args, cfg, pkg, dev):
    """One step = route + dispatch + combine (the expert GEMMs between dispatch and combine are the
    grouped workloads' business; here the sorted rows stand in for the expert output).  ``value`` and
    the roofline are HBM bytes per second: the roofline prices the dispatch call (histogram, scan,
    scatter and gather kernels), which moves the most bytes."""
    import torch

    from oracle import w8a8_oracle as o

    w8 = pkg.w8a8_lora
    t, e, k, h = cfg["m"], cfg["n_experts"], cfg["top_k"], cfg["hidden"]
    rng = np.random.default_rng(cfg["seed"])
    logits = (rng.standard_normal((t, e)) * 2.0).astype(np.float32)
    hidden = o.bf16_round(rng.standard_normal((t, h)).astype(np.float32))
    logits_t = torch.from_numpy(logits).to(dev)
    hidden_t = torch.from_numpy(hidden).to(dev).to(torch.bfloat16)

    def step():
        weights, selected = w8.moe_route(logits_t, k)
        xs, sizes, _, unsort, _ = w8.moe_dispatch(hidden_t, selected, e, repeat=k)
        return w8.moe_combine(xs, unsort, weights), weights, selected, xs, sizes, unsort

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = None
    for _ in range(args.steps):
        out = None  # (the last step's 128 MiB of sorted rows go back to torch's allocator before the next asks for them)
        out = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    combined, weights, selected, xs, sizes, unsort = out

    def timed(fn):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for a, b in ev:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return float(np.mean([a.elapsed_time(b) for a, b in ev]))

    route_ms = timed(lambda: w8.moe_route(logits_t, k))
    dispatch_ms = timed(lambda: w8.moe_dispatch(hidden_t, selected, e, repeat=k))
    combine_ms = timed(lambda: w8.moe_combine(xs, unsort, weights))
    p = t * k
    route_bytes = 4 * t * e + 8 * p
    dispatch_bytes = 2 * t * h + 2 * p * h + 4 * p * 3 + 4 * e   # rows in once, rows out, indices in, two index arrays out
    combine_bytes = 2 * p * h + 2 * t * h + 8 * p
    total_bytes = route_bytes + dispatch_bytes + combine_bytes
    achieved = dispatch_bytes / (dispatch_ms * 1e-3) / 1e9
    result = {
        "metric": "MoE token routing (route + dispatch + combine), GB/s of algorithmic HBM bytes per call",
        "value": total_bytes / (ms_per_step * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, **{kk: v for kk, v in cfg.items() if kk != "seed"}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic_bytes(args.workload),
                     "kernel": "moe_hist_kernel + moe_scan_kernel + moe_scatter_kernel + moe_spread_kernel (one dispatch call)",
                     "kernel_avg_ms": dispatch_ms, "algorithmic_bytes": dispatch_bytes},
        "stages": {"route_ms": route_ms, "route_bytes": route_bytes, "dispatch_ms": dispatch_ms,
                   "combine_ms": combine_ms, "combine_bytes": combine_bytes,
                   "combine_gbs": combine_bytes / (combine_ms * 1e-3) / 1e9},
    }
    if not args.no_cpu_baseline:
        t1 = time.perf_counter()
        want_w, want_sel = o.moe_route(logits, k)
        want_xs, want_sizes, want_unsort, _ = o.prepare_routing(np.repeat(hidden, k, axis=0), want_sel.ravel(), e)
        want_out = o.moe_combine(want_xs, want_unsort, want_w)
        secs = time.perf_counter() - t1
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            cores = os.cpu_count() or 1
        result["cpu_baseline"] = {"value": total_bytes / secs / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                  "sample": f"the whole workload ({t} tokens), NumPy oracle route + prepare_routing + "
                                            f"combine, one run, {secs:.3f} s", "seconds": secs}
        sel = selected.cpu().numpy()
        rows_same = (sel == want_sel).all(axis=1)
        got_out = combined.to(torch.float32).cpu().numpy()
        result["parity_sample"] = {
            "tokens": t, "tokens_with_equal_selection": int(rows_same.sum()),
            "group_sizes_equal": bool((sizes.cpu().numpy() == want_sizes).all()),
            "combine_violations": int(np.count_nonzero(~o.within_tolerance(got_out[rows_same], want_out[rows_same])))}
    print(json.dumps(result))
    return 0


def bench_moe_mlp(args, cfg, pkg, dev):
    """One step = the whole expert MLP: route, dispatch (indices only), grouped gate/up + SwiGLU
    (reading the hidden rows through the sort order), grouped down, combine.  ``value`` counts the
    integer GEMM work 2 * T * top_k * (H * 2I + I * H); the roofline prices the GEMM kernel
    of the grouped gate/up call (the dominant kernel) from HIP events around that kernel alone.  With 128
    rows per expert the kernel is bound by the int8 weights it streams (HBM), not by the matrix cores; the
    fraction of the int8 MFMA peak is reported next to it."""
    import torch

    from oracle import w8a8_oracle as o

    w8 = pkg.w8a8_lora
    t, e, k, h, inter, r = cfg["m"], cfg["n_experts"], cfg["top_k"], cfg["hidden"], cfg["intermediate"], cfg["rank"]
    rng = np.random.default_rng(cfg["seed"])
    hidden = o.bf16_round(rng.standard_normal((t, h)).astype(np.float32))
    logits = rng.standard_normal((t, e)).astype(np.float32)
    gu_codes = rng.integers(-127, 128, (e, h, 2 * inter), dtype=np.int8)
    gu_scales = rng.uniform(0.001, 0.01, (e, 2 * inter)).astype(np.float32)
    dn_codes = rng.integers(-127, 128, (e, inter, h), dtype=np.int8)
    dn_scales = rng.uniform(0.001, 0.01, (e, h)).astype(np.float32)
    mk = lambda shape: o.bf16_round((rng.standard_normal(shape) * 0.02).astype(np.float32))
    gua, gub, da, db = mk((e, h, r)), mk((e, r, 2 * inter)), mk((e, inter, r)), mk((e, r, h))
    bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(torch.bfloat16)
    guw = w8.prepare_grouped_weight(torch.from_numpy(gu_codes).to(dev), torch.from_numpy(gu_scales).to(dev))
    dnw = w8.prepare_grouped_weight(torch.from_numpy(dn_codes).to(dev), torch.from_numpy(dn_scales).to(dev))
    hidden_t, logits_t = bf(hidden), torch.from_numpy(logits).to(dev)
    gua_t, gub_t, da_t, db_t = bf(gua), bf(gub), bf(da), bf(db)

    def step():
        return w8.w8a8_moe_expert_mlp(hidden_t, logits_t, k, guw, dnw, gua_t, gub_t, da_t, db_t, 1.0, enabled=True)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        got = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    p = t * k
    ops = 2.0 * p * (h * 2 * inter + inter * h)

    def timed(fn):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for a, b in ev:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return float(np.mean([a.elapsed_time(b) for a, b in ev]))

    weights, selected = w8.moe_route(logits_t, k)
    _, sizes, sort_i, unsort, _ = w8.moe_dispatch(None, selected, e, repeat=k)
    act = w8.grouped_forward(hidden_t, sizes, guw, gua_t, gub_t, 1.0, swiglu=True, row_map=sort_i, row_repeat=k)
    down = w8.grouped_forward(act, sizes, dnw, da_t, db_t, 1.0)
    stages = {
        "route_ms": timed(lambda: w8.moe_route(logits_t, k)),
        "dispatch_ms": timed(lambda: w8.moe_dispatch(None, selected, e, repeat=k)),
        "gate_up_ms": timed(lambda: w8.grouped_forward(hidden_t, sizes, guw, gua_t, gub_t, 1.0, swiglu=True,
                                                       row_map=sort_i, row_repeat=k)),
        "down_ms": timed(lambda: w8.grouped_forward(act, sizes, dnw, da_t, db_t, 1.0)),
        "combine_ms": timed(lambda: w8.moe_combine(down, unsort, weights)),
    }
    gu_ops = 2.0 * p * h * 2 * inter
    # the gate/up GEMM kernel alone: the plan's workspace keeps the prologue's tables and codes
    gu_plan = w8.GroupedForwardPlan(hidden_t, sizes, guw, gua_t, gub_t, 1.0, swiglu=True, row_map=sort_i, row_repeat=k)
    gu_plan.run()
    gemm_ms = timed(lambda: gu_plan.run(pkg._native.FLAG_SKIP_PROLOGUE))
    stages["gate_up_gemm_kernel_ms"] = gemm_ms
    # every expert's int8 weight once, the codes and row scales, the channel scales, LoRA B and the three bf16
    # terms of x.A per row, the bf16 product out.  At 128 rows per expert the weights are 87 % of it: 3.4 int8
    # ops per byte at the two peaks' ratio of 625, so HBM is the roofline that bounds the kernel
    gemm_bytes = e * h * 2 * inter + p * h + 4 * p + 4 * e * 2 * inter + 2 * e * r * 2 * inter + 6 * p * r + 2 * p * inter
    achieved = gemm_bytes / (gemm_ms * 1e-3) / 1e9
    result = {
        "metric": "grouped W8A8-LoRA expert MLP (route, dispatch, gate/up + SwiGLU, down, combine), TOPS of the integer GEMM work",
        "value": ops / (ms_per_step * 1e-3) / 1e12, "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": args.workload, **{kk: v for kk, v in cfg.items() if kk != "seed"}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic_bytes(args.workload),
                     "kernel": "w8a8_gemm_kernel in grouped mode, gate/up projection with the SwiGLU epilogue",
                     "kernel_avg_ms": gemm_ms, "algorithmic_bytes": gemm_bytes, "algorithmic_ops": gu_ops,
                     "frac_of_int8_mfma_peak": gu_ops / (gemm_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS},
        "stages": stages,
    }
    if not args.no_cpu_baseline:
        rows = args.cpu_rows or 64
        gu = [o.GroupQuantizedWeight(gu_codes[i], gu_scales[i:i + 1], h, h, 8, h) for i in range(e)]
        dn = [o.GroupQuantizedWeight(dn_codes[i], dn_scales[i:i + 1], inter, inter, 8, inter) for i in range(e)]
        t1 = time.perf_counter()
        want = o.moe_expert_mlp(hidden[:rows], logits[:rows], k, gu, dn, gua, gub, da, db, np.float32(1.0))
        secs = time.perf_counter() - t1
        result["cpu_baseline"] = {"value": ops * rows / t / secs / 1e12, "unit": "TOPS", "cores": 1, "kind": "port",
                                  "sample": f"first {rows} of {t} tokens (tokens are independent), all experts, NumPy "
                                            f"oracle expert MLP, one run, {secs:.3f} s", "seconds": secs}
        gate = o.numerical_gate(got[:rows].to(torch.float32).cpu().numpy(), want)
        result["parity_sample"] = {"tokens": rows, "relative_l2": gate["relative_l2"], "cosine": gate["cosine"]}
    print(json.dumps(result))
    return 0


def bench_moe_backward(args, cfg, pkg, dev):
    """One step = the backward of the two grouped expert projections (gate/up without SwiGLU, down) over
    the sorted (token, choice) pairs: dx and dA, dB, dscaling for every expert, one native call per
    projection.  ``value`` counts the pull-backs' 2 * P * (H * 2I + I * H); the roofline prices
    the gate/up call without LoRA (tables, dy packing, bwd_dx_kernel) on the rows that exist.  With 128
    rows per expert the call is bound by the int8 weights it streams (HBM: 65 us of traffic against 41 us
    of bf16 MFMA work at the two peaks); the fraction of the bf16 MFMA peak is reported next to it."""
    import torch

    from oracle import w8a8_oracle as o

    native, w8 = pkg._native, pkg.w8a8_lora
    t, e, topk, h, inter, r = cfg["m"], cfg["n_experts"], cfg["top_k"], cfg["hidden"], cfg["intermediate"], cfg["rank"]
    p_rows = t * topk
    rng = np.random.default_rng(cfg["seed"])
    logits = torch.from_numpy(rng.standard_normal((t, e)).astype(np.float32)).to(dev)
    _, selected = w8.moe_route(logits, topk)
    _, sizes, _, _, _ = w8.moe_dispatch(None, selected, e, repeat=topk)
    gen = torch.Generator(device=dev).manual_seed(cfg["seed"])
    rnd = lambda *shape, scale=1.0: (torch.randn(*shape, device=dev, generator=gen) * scale).to(torch.bfloat16)

    def weight(k, n):
        codes = torch.randint(-127, 128, (e, k, n), dtype=torch.int8, device=dev, generator=gen)
        scales = torch.rand(e, n, device=dev, generator=gen) * 0.009 + 0.001
        return w8.prepare_grouped_weight(codes, scales), codes, scales

    guw, gu_codes, gu_scales = weight(h, 2 * inter)
    dnw, _, _ = weight(inter, h)
    x_gu, dy_gu = rnd(p_rows, h), rnd(p_rows, 2 * inter)
    x_dn, dy_dn = rnd(p_rows, inter), rnd(p_rows, h)
    gua, gub = rnd(e, h, r, scale=0.02), rnd(e, r, 2 * inter, scale=0.02)
    dna, dnb = rnd(e, inter, r, scale=0.02), rnd(e, r, h, scale=0.02)
    s = torch.ones(e, device=dev)
    plan_gu = w8.GroupedBackwardPlan(x_gu, dy_gu, sizes, guw, gua, gub, s)
    plan_dn = w8.GroupedBackwardPlan(x_dn, dy_dn, sizes, dnw, dna, dnb, s)

    def step():
        plan_gu.run()
        plan_dn.run()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3

    def timed(fn, reps=None):
        reps = reps or args.steps
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for a, b in ev:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return np.asarray([a.elapsed_time(b) for a, b in ev])

    gu_ms, dn_ms = timed(plan_gu.run), timed(plan_dn.run)
    dx_only = w8.GroupedBackwardPlan(None, dy_gu, sizes, guw, None, None, None)
    dx_ms = timed(dx_only.run)
    # the same cotangents from one dense call per expert (what the single call replaces)
    loop_ms = timed(lambda: w8.grouped_backward_per_weight(x_gu, dy_gu, sizes, guw, gua, gub, s), reps=3)
    # the whole layer through autograd: training forward (projection kept, separate SwiGLU) and its backward
    hid = rnd(t, h).requires_grad_(True)
    params = [v.clone().requires_grad_(True) for v in (gua, gub, dna, dnb)]
    d_hid = rnd(t, h)

    def train_step():
        out = w8.moe_expert_mlp(hid, logits, topk, guw, dnw, *params, 1.0)
        out.backward(d_hid)

    for _ in range(3):
        train_step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(10):
        train_step()
    torch.cuda.synchronize()
    layer_ms = (time.perf_counter() - t1) / 10 * 1e3
    flops = 2.0 * p_rows * (h * 2 * inter + inter * h)
    gu_flops = 2.0 * p_rows * h * 2 * inter
    # every expert's int8 weight once, dy in, dx out: at 128 rows per expert 5 ms of HBM time per ms of bf16
    # MFMA time at the two peaks, so HBM is the roofline that bounds the pull-back
    dx_bytes = e * h * 2 * inter + 2 * p_rows * 2 * inter + 2 * p_rows * h
    achieved = dx_bytes / (float(dx_ms.mean()) * 1e-3) / 1e9
    result = {
        "metric": "backward of the grouped W8A8-LoRA expert projections (dx + LoRA cotangents, gate/up and down), "
                  "TFLOP/s of 2*P*K*N per call",
        "value": flops / (ms_per_step * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, **{kk: v for kk, v in cfg.items() if kk != "seed"}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic_bytes(args.workload),
                     "kernel": "the gate/up call without LoRA (tables, bwd_pack_dy_kernel, bwd_dx_kernel)",
                     "kernel_avg_ms": float(dx_ms.mean()), "kernel_min_ms": float(dx_ms.min()),
                     "algorithmic_bytes": dx_bytes, "algorithmic_flops": gu_flops,
                     "frac_of_bf16_mfma_peak": gu_flops / (float(dx_ms.mean()) * 1e-3) / 1e12 / BF16_PEAK_TFLOPS},
        "stages": {"gate_up_call_ms": float(gu_ms.mean()), "down_call_ms": float(dn_ms.mean()),
                   "gate_up_one_dense_call_per_expert_ms": float(loop_ms.mean()),
                   "expert_mlp_forward_and_backward_through_autograd_ms": layer_ms},
    }
    if not args.no_cpu_baseline:
        n_exp = args.cpu_rows or 4     # experts of the sample
        counts = sizes.cpu().numpy()
        starts = np.concatenate(([0], np.cumsum(counts)))
        sel = slice(0, int(starts[n_exp]))
        xs, dys = (v[sel].to(torch.float32).cpu().numpy() for v in (x_gu, dy_gu))
        a_np, b_np = (v[:n_exp].to(torch.float32).cpu().numpy() for v in (gua, gub))
        codes_np, scales_np = gu_codes[:n_exp].cpu().numpy(), gu_scales[:n_exp].cpu().numpy()
        t1 = time.perf_counter()
        want = []
        for i in range(n_exp):
            w = o.GroupQuantizedWeight(codes_np[i], scales_np[i:i + 1], h, h, 8, h)
            rows = slice(int(starts[i]), int(starts[i + 1]))
            want.append(o.quantized_lora_linear_multi_bwd(xs[rows], w, a_np[i:i + 1], b_np[i:i + 1], np.ones(1, np.float32),
                                                          np.zeros(rows.stop - rows.start, np.int64), dys[rows], True))
        secs = time.perf_counter() - t1
        done = int(starts[n_exp])
        result["cpu_baseline"] = {"value": 2.0 * done * h * 2 * inter / secs / 1e12, "unit": "TFLOP/s", "cores": 1,
                                  "kind": "port",
                                  "sample": f"the first {n_exp} experts' {done} rows of the gate/up call, NumPy oracle "
                                            f"backward per expert (float64 BLAS), one run, {secs:.3f} s", "seconds": secs}
        got_dx = plan_gu.run()[0][sel].to(torch.float32).cpu().numpy()
        gate = o.numerical_gate(got_dx, np.concatenate([w_[0] for w_ in want]))
        result["parity_sample"] = {"rows": done, "relative_l2": gate["relative_l2"], "cosine": gate["cosine"]}
    print(json.dumps(result))
    return 0


def bench_gq(args, cfg, pkg, dev):
    """One step = one group-scaled quantized linear call (quantizer, LoRA z, GEMM with the group
    epilogue).  ``value`` counts 2*M*K*N; the roofline prices gq_gemm_kernel against int8 MFMA peak from
    HIP events around whole calls minus nothing -- the call is that kernel plus two short ones, so the
    figure is a lower bound for the kernel."""
    import torch

    import w8a8_cases as wc
    from oracle import w8a8_oracle as o

    gq, ql = pkg.gq_linear, pkg.quantized_lora
    m, k, n, r, n_ad = cfg["m"], cfg["k"], cfg["n"], cfg["rank"], cfg["n_adapters"]
    wb, ab, group = cfg["weight_bits"], cfg["activation_bits"], cfg["group_size"]
    rng = np.random.default_rng(cfg["seed"])
    x = o.bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    dense = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    w = o.quantize_frozen_weight(dense, bits=wb, group_size=group, scale_dtype="f32")
    a = o.bf16_round((rng.standard_normal((n_ad, k, r)) * 0.02).astype(np.float32))
    b = o.bf16_round((rng.standard_normal((n_ad, r, n)) * 0.02).astype(np.float32))
    s = np.ones(n_ad, np.float32)
    idx = rng.integers(0, n_ad, m).astype(np.int32)
    bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(dev).to(torch.bfloat16)
    wt = gq.prepare_group_weight(ql.GroupQuantizedWeight(torch.from_numpy(w.codes).to(dev),
                                                         torch.from_numpy(w.scales).to(dev), k, w.padded_in_features,
                                                         wb, group))
    x_t, a_t, b_t = bf(x), bf(a), bf(b)
    s_t, idx_t = torch.from_numpy(s).to(dev), torch.from_numpy(idx).to(dev)
    step = lambda: gq.forward(x_t, wt, a_t, b_t, s_t, activation_bits=ab, adapter_indices=idx_t)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        got = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for e0, e1 in ev:
        e0.record()
        step()
        e1.record()
    torch.cuda.synchronize()
    call_ms = float(np.mean([e0.elapsed_time(e1) for e0, e1 in ev]))
    ops = 2.0 * m * k * n
    achieved = ops / (call_ms * 1e-3) / 1e12
    result = {
        "metric": f"group-scaled W{wb}A{ab} LoRA linear forward (group {group}), TOPS of 2*M*K*N per call",
        "value": ops / (ms_per_step * 1e-3) / 1e12, "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": args.workload, **{kk: v for kk, v in cfg.items() if kk != "seed"}},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                     "frac": achieved / INT8_PEAK_TOPS, "traffic": measured_traffic_bytes(args.workload),
                     "kernel": "gq_gemm_lds_kernel (timed with gq_quant_kernel and the LoRA-A launches: whole calls)",
                     "kernel_avg_ms": call_ms, "algorithmic_ops": ops,
                     "algorithmic_bytes": 2 * m * k + k * n * wb // 8 + 4 * (k // group) * n + 2 * m * n},
    }
    if not args.no_cpu_baseline:
        rows = args.cpu_rows or 128
        t1 = time.perf_counter()
        want = o.bf16_round(o.quantized_frozen_linear_f32(x[:rows], w, activation_bits=ab)
                            + o.lora_delta_multi(x[:rows], a, b, s, idx[:rows]))
        secs = time.perf_counter() - t1
        result["cpu_baseline"] = {"value": 2.0 * rows * k * n / secs / 1e12, "unit": "TOPS", "cores": 1, "kind": "port",
                                  "sample": f"first {rows} of {m} rows, full K and N, NumPy oracle (group by group), "
                                            f"one run, {secs:.3f} s", "seconds": secs}
        rep = wc.compare(got[:rows].to(torch.float32).cpu().numpy(), want)
        result["parity_sample"] = {"rows": rows, "violations": rep["violations"], "size": rep["size"],
                                   "max_abs": rep["max_abs"], "bitwise_fraction": rep["bitwise_fraction"]}
    print(json.dumps(result))
    return 0


def bench_qkv(args, cfg, pkg, dev):
    """One step = the W8A8 QKV projection (RMSNorm prologue, GEMM, LoRA) + the split / Q-K norm /
    RoPE kernel.  ``value`` is int8 TOPS of the projection over the whole step; the roofline prices
    qkv_post_kernel (HBM-bound: it reads the fused projection once and writes q, k, v, gate once)."""
    import torch

    import w8a8_cases as wc
    from oracle import w8a8_oracle as o

    w8 = pkg.w8a8_lora
    geo = cfg["qkv"]
    qcfg = w8.Qwen35QKVStageConfig(geo["num_query_heads"], geo["num_kv_heads"], geo["head_dim"], geo["rotary_dim"],
                                   10_000_000.0, 1e-6)
    assert qcfg.fused_width == cfg["n"]
    case = wc.make_case(cfg["m"], cfg["k"], cfg["n"], n_adapters=cfg["n_adapters"], rank=cfg["rank"],
                        alpha=cfg.get("alpha"), seed=cfg["seed"], rms=True, idx_mode=cfg["idx_mode"])
    rng = np.random.default_rng(cfg["seed"] + 77)
    qw, kw = (rng.standard_normal(geo["head_dim"]).astype(np.float32) * 0.1 for _ in range(2))
    pos = rng.integers(0, 32768, cfg["m"]).astype(np.int32)
    t = wc.to_torch(case, dev)
    qw_t, kw_t, pos_t = (torch.from_numpy(v).to(dev) for v in (qw, kw, pos))
    plan = w8.ForwardPlan(t["x"], t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"],
                          rms_gamma=t["gamma"], eps=1e-6)

    post = w8.QkvPostPlan(plan.run(), qw_t, kw_t, pos_t, qcfg)  # reads the forward plan's (reused) output

    def step():
        plan.run()
        return post.run()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in ev:
        a.record()
        post.run()
        b.record()
    torch.cuda.synchronize()
    k_ms = np.asarray([a.elapsed_time(b) for a, b in ev])
    m, k, n = cfg["m"], cfg["k"], cfg["n"]
    bytes_alg = 4 * m * n + 4 * m + 8 * geo["head_dim"]
    achieved = bytes_alg / (float(k_ms.mean()) * 1e-3) / 1e9
    ops = 2.0 * m * k * n
    result = {
        "metric": "Qwen3.5 attention input stage on the W8A8 QKV projection, int8 TOPS of 2*M*K*N per step",
        "value": ops / (ms_per_step * 1e-3) / 1e12, "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": args.workload, **{kk: v for kk, v in cfg.items() if kk != "seed"}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic_bytes(args.workload),
                     "kernel": "qkv_post_kernel",
                     "kernel_avg_ms": float(k_ms.mean()), "kernel_min_ms": float(k_ms.min()),
                     "algorithmic_bytes": bytes_alg},
    }
    if not args.no_cpu_baseline:
        rows = args.cpu_rows or 256
        t1 = time.perf_counter()
        want = o.w8a8_qkv_lora_rope(case["x"][:rows], case["gamma"] - 1.0, qw, kw, case["weight"], case["a"], case["b"],
                                    case["s"], case["idx"][:rows], pos[:rows], num_query_heads=geo["num_query_heads"],
                                    num_kv_heads=geo["num_kv_heads"], head_dim=geo["head_dim"],
                                    rotary_dim=geo["rotary_dim"], rope_theta=10_000_000.0, eps=1e-6)
        secs = time.perf_counter() - t1
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            cores = os.cpu_count() or 1
        threads = int(os.environ.get("OMP_NUM_THREADS", cores))
        result["cpu_baseline"] = {"value": 2.0 * rows * k * n / secs / 1e12, "unit": "TOPS", "cores": min(cores, threads),
                                  "kind": "port", "sample": f"first {rows} of {m} rows, NumPy oracle of the whole stage, "
                                                            f"one run, {secs:.3f} s", "seconds": secs}
        viol = size = 0
        for u, w_ in zip(out, want):
            rep = wc.compare(u[:rows].to(torch.float32).cpu().numpy().reshape(w_.shape), w_)
            viol += rep["violations"]
            size += rep["size"]
        result["parity_sample"] = {"rows": rows, "violations": viol, "size": size}
    print(json.dumps(result))
    return 0


def bench_qkv_backward(args, cfg, pkg, dev):
    """One step = one backward of the attention input stage whose forward kept the projection and the
    normalized rows: split / Q-K norm / RoPE pull-back, linear backward (dx + LoRA cotangents), decoder
    RMSNorm pull-back.  ``value`` counts the pull-back's 2*M*K*N; the roofline prices
    qkv_post_bwd_kernel (HBM-bound: the projection and the four cotangents in, d_fused out)."""
    import torch

    import w8a8_cases as wc
    from oracle import w8a8_oracle as o

    native, w8 = pkg._native, pkg.w8a8_lora
    geo = cfg["qkv"]
    theta = 10_000_000.0
    qcfg = w8.Qwen35QKVStageConfig(geo["num_query_heads"], geo["num_kv_heads"], geo["head_dim"], geo["rotary_dim"],
                                   theta, 1e-6)
    m, k, n = cfg["m"], cfg["k"], cfg["n"]
    hq, hkv, d = geo["num_query_heads"], geo["num_kv_heads"], geo["head_dim"]
    assert qcfg.fused_width == n
    case = wc.make_case(m, k, n, n_adapters=cfg["n_adapters"], rank=cfg["rank"], alpha=cfg.get("alpha"),
                        seed=cfg["seed"], rms=True, idx_mode=cfg["idx_mode"])
    rng = np.random.default_rng(cfg["seed"] + 78)
    qw, kw = (rng.standard_normal(d).astype(np.float32) * 0.1 for _ in range(2))
    pos = rng.integers(0, 32768, m).astype(np.int32)
    cots = [o.bf16_round(rng.standard_normal(shape).astype(np.float32))
            for shape in ((m, hq, d), (m, hkv, d), (m, hkv, d), (m, hq * d))]
    t = wc.to_torch(case, dev)
    qw_t, kw_t, pos_t = (torch.from_numpy(v).to(dev) for v in (qw, kw, pos))
    cots_t = [torch.from_numpy(c).to(dev).to(torch.bfloat16) for c in cots]
    in_w = t["gamma"] - 1.0
    fwd = w8.ForwardPlan(t["x"], t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"], rms_gamma=t["gamma"],
                         eps=1e-6, want_normalized=True)
    fused = fwd.run()
    plan = w8.QkvStageBackwardPlan(t["x"], in_w, qw_t, kw_t, t["weight"], t["a"], t["b"], t["s"], pos_t, qcfg, *cots_t,
                                   adapter_indices=t["idx"], fused=fused, normalized=fwd.aux["normalized"])
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        plan.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        plan.run()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    got = [v.to(torch.float32).cpu().numpy() for v in plan.run()]
    torch.cuda.synchronize()

    def timed(fn):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for a, b in ev:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return np.asarray([a.elapsed_time(b) for a, b in ev])

    lib = native.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    k_ms = timed(plan.run_post_stage)
    linear_ms = timed(plan.bwd.run)
    scratch_k = torch.empty_like(plan.bwd.dx)
    rms_ms = timed(lambda: native.check("delta_rms_norm_bwd", lib.mi355_w8a8_delta_rms_norm_bwd_v1(
        plan.x.data_ptr(), plan.gamma.data_ptr(), plan.bwd.dx.data_ptr(), scratch_k.data_ptr(), None, None, 0, m, k,
        plan.eps, stream)))
    recompute_ms = timed(fwd.run)
    # with trainable norm weights: the two pull-backs also form the weight cotangents
    wgrad_post_ms = timed(lambda: w8.qkv_split_norm_rope_backward(fused, qw_t, kw_t, pos_t, qcfg, *cots_t,
                                                                  need_norm_weight_grads=True))
    dn_copy = plan.bwd.dx.clone()
    wgrad_rms_ms = timed(lambda: w8.delta_rms_norm_backward(plan.x, plan.gamma, dn_copy, eps=1e-6,
                                                            need_weight_grad=True))
    flops = 2.0 * m * k * n
    bytes_alg = 6 * m * n + 4 * m + 8 * d   # projection, cotangents (as wide together), d_fused: bf16 [M, N] each
    achieved = bytes_alg / (float(k_ms.mean()) * 1e-3) / 1e9
    rms_bytes = 6 * m * k + 4 * k
    result = {
        "metric": "Qwen3.5 attention input stage backward (pull-backs + LoRA cotangents, saved projection), "
                  "TFLOP/s of 2*M*K*N per call",
        "value": flops / (ms_per_step * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, **{kk: v for kk, v in cfg.items() if kk != "seed"}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic_bytes(args.workload),
                     "kernel": "qkv_post_bwd_kernel",
                     "kernel_avg_ms": float(k_ms.mean()), "kernel_min_ms": float(k_ms.min()),
                     "algorithmic_bytes": bytes_alg},
        "stages": {
            "linear_backward_ms": float(linear_ms.mean()), "forward_recompute_ms": float(recompute_ms.mean()),
            "delta_rms_norm_bwd_kernel": {"avg_ms": float(rms_ms.mean()), "algorithmic_bytes": rms_bytes,
                                          "achieved_gbs": rms_bytes / (float(rms_ms.mean()) * 1e-3) / 1e9,
                                          "frac_of_hbm": rms_bytes / (float(rms_ms.mean()) * 1e-3) / 1e9 / HBM_PEAK_GBS},
            "with_norm_weight_cotangents": {"post_call_ms": float(wgrad_post_ms.mean()),
                                            "decoder_norm_call_ms": float(wgrad_rms_ms.mean())},
        },
    }
    if not args.no_cpu_baseline:
        rows = args.cpu_rows or 256
        sel = slice(0, rows)
        t1 = time.perf_counter()
        want = o.w8a8_qkv_lora_rope_bwd(case["x"][sel], case["gamma"] - 1.0, qw, kw, case["weight"], case["a"],
                                        case["b"], case["s"], case["idx"][sel], pos[sel], *(c[sel] for c in cots),
                                        num_query_heads=hq, num_kv_heads=hkv, head_dim=d,
                                        rotary_dim=geo["rotary_dim"], rope_theta=theta, eps=1e-6)
        secs = time.perf_counter() - t1
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            cores = os.cpu_count() or 1
        threads = int(os.environ.get("OMP_NUM_THREADS", cores))
        result["cpu_baseline"] = {"value": 2.0 * rows * k * n / secs / 1e12, "unit": "TFLOP/s",
                                  "cores": min(cores, threads), "kind": "port",
                                  "sample": f"first {rows} of {m} rows, NumPy oracle of the stage's backward "
                                            f"(forward stages + pull-backs, float64 BLAS), one run, {secs:.3f} s",
                                  "seconds": secs}
        gate = o.numerical_gate(got[0][sel], want["dhidden"])  # rows of d_hidden are independent of each other
        result["parity_sample"] = {"rows": rows, "relative_l2": gate["relative_l2"], "cosine": gate["cosine"]}
    print(json.dumps(result))
    return 0


def measure_linear(args, cfg, pkg, dev, steps, warmup, rotate, workload=None, flags=None):
    """Time one dense forward workload: whole steps (host clock around `steps` back-to-back calls and one HIP
    event pair per step), the dominant kernel alone, the prologue alone."""
    import torch

    import w8a8_cases as wc

    native = pkg._native
    w8 = pkg.w8a8_lora
    workload = workload or args.workload
    flags = args.flags if flags is None else flags
    case = wc.make_case(cfg["m"], cfg["k"], cfg["n"], n_adapters=cfg.get("n_adapters", 0),
                        rank=cfg.get("rank", 16), seed=cfg["seed"], rms=cfg.get("rms", False),
                        residual=cfg.get("residual", False), swiglu=cfg.get("swiglu", False),
                        idx_mode=cfg.get("idx_mode", "uniform"), student_t=cfg.get("x_dist") == "student_t3",
                        alpha=cfg.get("alpha"))
    path_flags = flags | (native.FLAG_SWIGLU if cfg.get("swiglu") else 0)
    path = native.PATH_NAMES.get(native.load().mi355_w8a8_forward_path(cfg["m"], cfg["k"], cfg["n"], path_flags), "?")
    skinny = path.startswith("skinny")
    rotate = rotate or (max(1, -(-768_000_000 // algorithmic_bytes(cfg))) if skinny else 1)
    plans = []
    for _ in range(rotate):
        t = wc.to_torch(case, dev)  # a fresh copy of every operand (and its own packed weight)
        plans.append(w8.ForwardPlan(t["x"], t["weight"], t.get("a"), t.get("b"), t.get("s"),
                                    adapter_indices=t.get("idx"), rms_gamma=t.get("gamma"), eps=1e-6,
                                    residual=t.get("residual"), swiglu=bool(cfg.get("swiglu")),
                                    flags=flags))
    plan = plans[0]
    if getattr(args, "repack_lora", False):
        for pl in plans:
            pl.keep_lora_pack = False
    torch.cuda.synchronize()
    # Spin-up, untimed and before the warm-up steps: the first launches after idle run while clocks and the
    # power controller settle (up to 20 % slow); the figure quoted is the sustained one.
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < args.spin_up:
        for _ in range(8):
            plans[i % rotate].run()
            i += 1
        torch.cuda.synchronize()
    spin_up_s = time.perf_counter() - t0
    for i in range(warmup):
        plans[i % rotate].run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        plans[i % rotate].run()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / steps * 1e3
    ops = 2.0 * cfg["m"] * cfg["k"] * cfg["n"]

    def event_pairs(fn):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for i, (a, b) in enumerate(ev):
            a.record()
            fn(i)
            b.record()
        torch.cuda.synchronize()
        return np.asarray([a.elapsed_time(b) for a, b in ev])

    # whole steps again, one event pair each: where the step time sits when the host clock is not in it
    step_ms = event_pairs(lambda i: plans[i % rotate].run())
    step_event_ms = {"median": float(np.median(step_ms)), "p10": float(np.percentile(step_ms, 10)),
                     "p90": float(np.percentile(step_ms, 90))}

    # dominant kernel alone: HIP events (torch's current stream is the launch stream) around
    # GEMM-only launches; the workspace still holds the prologue's results.
    # (a call that runs as 32-row chunks of the streaming kernels keeps no stage to rerun: the library
    # says so, and the figures below are then taken around whole calls)
    try:
        plans[0].run(native.FLAG_SKIP_PROLOGUE)
        stage_flags = (native.FLAG_SKIP_PROLOGUE, native.FLAG_SKIP_GEMM)
    except native.NativeError as err:
        if err.status != -7:
            raise
        stage_flags = (0, 0)
    gemm_ms = event_pairs(lambda i: plans[i % rotate].run(stage_flags[0]))
    # average launch duration: one event pair around all the launches, back to back on the launch stream
    # (a pair around every single launch adds the launch latency the next launch would have hidden)
    ga, gb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ga.record()
    for i in range(steps):
        plans[i % rotate].run(stage_flags[0])
    gb.record()
    torch.cuda.synchronize()
    gemm_avg_ms = ga.elapsed_time(gb) / steps
    # prologue alone (routing + quantization + LoRA-A)
    pa, pb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    pa.record()
    for i in range(steps):
        plans[i % rotate].run(stage_flags[1])
    pb.record()
    torch.cuda.synchronize()
    prologue_ms = pa.elapsed_time(pb) / steps if stage_flags[1] else None
    # the training-style step: the adapters changed since the last call (every optimizer step does that),
    # so the launch that lays out the LoRA operands runs again -- timed over at least 20 steps
    repack = None
    if cfg.get("n_adapters", 0) and not getattr(args, "repack_lora", False) and not getattr(args, "no_repack", False):
        n_rep = max(steps, 20)
        for pl in plans:
            pl.keep_lora_pack = False
        for i in range(max(warmup, 3)):
            plans[i % rotate].run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_rep):
            plans[i % rotate].run()
        torch.cuda.synchronize()
        rep_ms = (time.perf_counter() - t0) / n_rep * 1e3
        for pl in plans:
            pl.keep_lora_pack = True
        repack = {"ms_per_step": rep_ms, "steps": n_rep, "value": ops / (rep_ms * 1e-3) / 1e12, "unit": "TOPS",
                  "frac_of_int8_peak_whole_step": ops / (rep_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS,
                  "lora_pack": "repacked every step (adapters updated between steps, as in LoRA training)"}
    out_gpu = plan.run()
    torch.cuda.synchronize()

    if skinny:
        # the decode path is two short kernels per 32 rows; the figure prices them together against the
        # algorithmic bytes of the whole call.  They last ~20 us together and an event pair around a single
        # call adds ~2.5 us of its own, so the average launch duration comes from one event pair around all
        # the steps (back-to-back calls on the launch stream), per call.
        ra, rb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ra.record()
        for i in range(steps):
            plans[i % rotate].run()
        rb.record()
        torch.cuda.synchronize()
        region_ms = ra.elapsed_time(rb) / steps
        bytes_alg = algorithmic_bytes(cfg)
        achieved = bytes_alg / (region_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic_bytes(workload),
                    "kernel": "skinny_quant_kernel + skinny_stream_kernel",
                    "kernel_avg_ms": region_ms, "single_call_event_avg_ms": float(step_ms.mean()),
                    "kernel_min_ms": float(step_ms.min()),
                    "stream_and_epilogue_avg_ms": gemm_avg_ms, "algorithmic_bytes": bytes_alg,
                    "operand_sets_rotated": rotate}
    else:
        achieved = ops / (gemm_avg_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "achieved": achieved, "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                    "frac": achieved / INT8_PEAK_TOPS, "traffic": measured_traffic_bytes(workload),
                    "kernel": "w8a8_gemm16_kernel" if path == "tiled-256x256" else "w8a8_gemm_kernel",
                    "kernel_avg_ms": gemm_avg_ms, "kernel_min_ms": float(gemm_ms.min()),
                    "kernel_event_pair_avg_ms": float(gemm_ms.mean()), "algorithmic_ops": ops,
                    "algorithmic_bytes": gemm_kernel_bytes(cfg)}
    return {"ms_per_step": ms_per_step, "ops": ops, "roofline": roofline, "prologue_ms": prologue_ms,
            "step_event_ms": step_event_ms, "spin_up_s": spin_up_s, "path": path, "case": case,
            "out_gpu": out_gpu, "repack": repack}


def bench_mixed_m(args, cfg, pkg, dev):
    """Benchmark configuration 4: the Qwen3-4B attention projections (QKV [2560 -> 6144] and o_proj
    [4096 -> 2560]) with 4 adapters of rank 64 on Student-t(3) activations, at M = 1, 64, 512, 2048.  One JSON
    line with a row per (shape, M); `value` is the int8 TOPS of the largest point."""
    rows = []
    for name, k, n in cfg["shapes"]:
        for m in cfg["m_values"]:
            c = dict(m=m, k=k, n=n, n_adapters=cfg["n_adapters"], rank=cfg["rank"], alpha=cfg["alpha"],
                     idx_mode="uniform", x_dist="student_t3", seed=cfg["seed"])
            r = measure_linear(args, c, pkg, dev, args.steps, args.warmup, 0, workload=f"{args.workload}/{name}/m{m}")
            roof = r["roofline"]
            bytes_alg = algorithmic_bytes(c)
            call_ms = roof["kernel_avg_ms"] if roof["bound"] == "hbm" else r["step_event_ms"]["median"]
            rows.append({"shape": name, "m": m, "k": k, "n": n, "path": r["path"], "ms_per_step": r["ms_per_step"],
                         "call_ms": call_ms, "tops": r["ops"] / (call_ms * 1e-3) / 1e12,
                         "gbs": bytes_alg / (call_ms * 1e-3) / 1e9,
                         # a point is priced against the bound it is nearer to at its published peak
                         "bound": "mfma" if r["ops"] / INT8_PEAK_TOPS / 1e12 > bytes_alg / HBM_PEAK_GBS / 1e9 else "hbm",
                         "frac_of_int8_peak": r["ops"] / (call_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS,
                         "frac_of_hbm_peak": bytes_alg / (call_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                         "dominant_kernel_ms": roof["kernel_avg_ms"], "prologue_ms": r["prologue_ms"]})
            del r
    for row in rows:
        row["frac"] = row["frac_of_int8_peak"] if row["bound"] == "mfma" else row["frac_of_hbm_peak"]
    top = max(rows, key=lambda row: row["tops"])
    print(json.dumps({
        "metric": "W8A8-LoRA linear TOPS / GB/s over M (Qwen3-4B attention projections, Student-t(3) activations)",
        "value": top["tops"], "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": top["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": args.workload, "n_adapters": cfg["n_adapters"], "rank": cfg["rank"],
                   "alpha": cfg["alpha"], "x_dist": "student_t3"},
        "points": rows,
        "roofline": {"bound": top["bound"], "achieved": top["tops"], "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                     "frac": top["frac_of_int8_peak"], "traffic": None,
                     "kernel": f"whole call, {top['shape']} M={top['m']} ({top['path']})"}}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="qwen3-8b-gate_up-m4096", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-rows", type=int, default=None, help="rows of the CPU-baseline sample")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--flags", type=int, default=0, help="extra mi355_w8a8_problem.flags")
    ap.add_argument("--override", default="", help="comma list key=int overriding workload fields (m,k,n,...)")
    ap.add_argument("--rotate", type=int, default=0,
                    help="independent operand sets cycled through by successive steps (0 = 1 for MFMA-bound "
                         "workloads; for the HBM-bound decode workloads enough sets to exceed 768 MB, so that "
                         "no step finds its weights in the 256 MB last-level cache)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device copy (a kernel of known traffic for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    ap.add_argument("--spin-up", type=float, default=0.5,
                    help="seconds of untimed calls before the warm-up steps (clocks and power controller settle)")
    ap.add_argument("--repack-lora", action="store_true",
                    help="transpose / pack the LoRA factors on every step (a training step's forward) instead of "
                         "keeping them in the plan's workspace while the adapters are unchanged")
    ap.add_argument("--no-repack", action="store_true",
                    help="skip the block that times the step with the LoRA operands packed again every step "
                         "(counter runs: the steady call then has the most dispatches of its kernel)")
    ap.add_argument("--no-decode", action="store_true", help="default workload: skip the decode block")
    ap.add_argument("--no-ceilings", action="store_true", help="default workload: skip the measured ceilings")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no collectives); use --gpus 1",
              file=sys.stderr)
        return 2

    import torch

    import w8a8_cases as wc
    from __graft_entry__ import load_package

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    pkg = load_package()
    native = pkg._native
    native.load()
    w8 = pkg.w8a8_lora
    dev = torch.device("cuda:0")
    cfg = dict(WORKLOADS[args.workload])
    for item in filter(None, args.override.split(",")):
        key, val = item.split("=")
        cfg[key] = int(val)
    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        native.check("mi355_w8a8_calibrate_copy_v1",
                     native.load().mi355_w8a8_calibrate_copy_v1(src.data_ptr(), dst.data_ptr(), 256 << 20,
                                                                _stream_ptr(dev)))
        torch.cuda.synchronize()
        del src, dst
    if cfg.pop("calibration", False):
        return bench_calibration(args, pkg, dev)
    if cfg.pop("backward", False):
        if cfg.get("swiglu"):
            return bench_fused_backward(args, cfg, pkg, dev)
        return bench_backward(args, cfg, pkg, dev)
    if cfg.pop("gq", False):
        return bench_gq(args, cfg, pkg, dev)
    if cfg.pop("moe_backward", False):
        return bench_moe_backward(args, cfg, pkg, dev)
    if cfg.pop("moe_mlp", False):
        return bench_moe_mlp(args, cfg, pkg, dev)
    if cfg.pop("moe_routing", False):
        return bench_moe_routing(args, cfg, pkg, dev)
    if cfg.pop("qkv_backward", False):
        return bench_qkv_backward(args, cfg, pkg, dev)
    if "qkv" in cfg:
        return bench_qkv(args, cfg, pkg, dev)
    if cfg.pop("mixed_m", False):
        return bench_mixed_m(args, cfg, pkg, dev)
    r = measure_linear(args, cfg, pkg, dev, args.steps, args.warmup, args.rotate)
    tops = r["ops"] / (r["ms_per_step"] * 1e-3) / 1e12
    result = {
        "metric": "W8A8-LoRA GEMM TOPS & % int8 MFMA peak (Qwen3-8B MLP, M=4096); decode GB/s",
        "value": tops, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": args.workload, **{k: v for k, v in cfg.items() if k != "seed"}},
        "frac_of_int8_peak_whole_step": tops / INT8_PEAK_TOPS,
        "whole_step_gbs": algorithmic_bytes(cfg) / (r["ms_per_step"] * 1e-3) / 1e9,
        "step_event_ms": r["step_event_ms"],
        "spin_up_s": r["spin_up_s"],
        "prologue_ms": r["prologue_ms"],
        "path": r["path"],
        # the steps reuse one plan with unchanged adapters: the transposed / packed LoRA factors stay in its
        # workspace (MI355_W8A8_FLAG_LORA_PACK_VALID) as they would between the calls of a serving loop;
        # --repack-lora makes every step pack them again, as a training step does after an adapter update
        "lora_pack": "repacked every step" if args.repack_lora else "kept in the workspace across steps",
        "roofline": r["roofline"],
    }
    if r.get("repack"):
        result["repack"] = r["repack"]
    if args.workload == "qwen3-8b-gate_up-m4096" and not args.no_decode:
        # the second half of the metric: the decode-shaped call (M = 16 down projection with residual),
        # enough independent operand sets that no call finds its weights in the last-level cache
        dcfg = dict(WORKLOADS["qwen3-8b-down-m16-decode"])
        d = measure_linear(args, dcfg, pkg, dev, max(args.steps, 48), max(args.warmup, 12), 0,
                           workload="qwen3-8b-down-m16-decode")
        result["decode"] = {"workload": "qwen3-8b-down-m16-decode",
                            "config": {k: v for k, v in dcfg.items() if k != "seed"},
                            "ms_per_step": d["ms_per_step"], "path": d["path"], **d["roofline"]}
        del d
    if args.workload == "qwen3-8b-gate_up-m4096" and not args.no_ceilings:
        # what the part sustains on the same instruction with realistic operand codes and nothing else to do,
        # and on a read-only stream: second denominators beside the published peaks
        ceil = measure_mfma_ceiling(native, dev, 1, "codes")
        result["roofline"]["measured_mfma_ceiling_tops"] = ceil["tops"]
        result["roofline"]["measured_mfma_ceiling_mhz"] = ceil["shader_mhz"]
        result["roofline"]["frac_of_measured_ceiling"] = result["roofline"]["achieved"] / ceil["tops"]
        if "decode" in result:
            rd = measure_read_ceiling(native, dev)
            result["decode"]["measured_read_ceiling_gbs"] = rd["gbs"]
            result["decode"]["frac_of_measured_ceiling"] = result["decode"]["achieved"] / rd["gbs"]
    if not args.no_cpu_baseline:
        rows = args.cpu_rows or cfg["m"]
        want, base = cpu_baseline(r["case"], cfg, rows)
        result["cpu_baseline"] = base
        got = r["out_gpu"][:rows].to(torch.float32).cpu().numpy()
        rep = wc.compare(got, want)
        result["parity_sample"] = {"rows": rows, "violations": rep["violations"], "size": rep["size"],
                                   "max_abs": rep["max_abs"], "bitwise_fraction": rep["bitwise_fraction"]}
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
