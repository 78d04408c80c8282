"""Seeded synthetic inputs of the benchmark configurations and torch <-> numpy plumbing
shared by the GPU parity tests, the smoke check and bench.py's CPU baseline."""

from __future__ import annotations

import numpy as np

from oracle import w8a8_oracle as o

F32 = np.float32
BASE_SEED = 20260714


def make_case(m, k, n, *, n_adapters=1, rank=16, alpha=None, seed=0, student_t=False, rms=False,
              residual=False, swiglu=False, idx_mode="uniform", scale_dtype="f32"):
    """Synthetic tensors in the distributions the benchmark configurations name."""
    rng = np.random.default_rng(BASE_SEED + seed)
    x = rng.standard_t(3, (m, k)) if student_t else rng.standard_normal((m, k))
    x = o.bf16_round(x.astype(F32))
    codes = rng.integers(-127, 128, (k, n), dtype=np.int8)
    scales = rng.uniform(0.001, 0.01, (1, n)).astype(F32)
    if scale_dtype == "bf16":
        scales = o.bf16_round(scales)
    case = {"m": m, "k": k, "n": n, "x": x, "codes": codes, "scales": scales, "swiglu": swiglu,
            "weight": o.GroupQuantizedWeight(codes, scales, k, k, 8, k)}
    if n_adapters:
        alpha = rank if alpha is None else alpha
        case["a"] = o.bf16_round((rng.standard_normal((n_adapters, k, rank)) * 0.02).astype(F32))
        case["b"] = o.bf16_round((rng.standard_normal((n_adapters, rank, n)) * 0.02).astype(F32))
        case["s"] = np.full((n_adapters,), alpha / rank, F32)
        if idx_mode == "uniform":
            case["idx"] = rng.integers(0, n_adapters, m).astype(np.int32)
        elif idx_mode == "arange":
            case["idx"] = (np.arange(m) % n_adapters).astype(np.int32)
        else:
            case["idx"] = np.zeros(m, np.int32)
    if rms:
        case["gamma"] = (1.0 + 0.1 * rng.standard_normal(k)).astype(F32)
    if residual:
        case["residual"] = o.bf16_round(rng.standard_normal((m, n)).astype(F32))
    return case


def oracle_forward(case, return_stages=False):
    """The oracle's answer for a case made by ``make_case`` (dict of stages)."""
    x = case["x"]
    st = {}
    if "gamma" in case:
        x = o.rms_norm(case["x"], case["gamma"], 1e-6)
        st["normalized"] = x
    base, xc, xs, acc = o.quantized_frozen_linear_f32(x, case["weight"], return_parts=True)
    st["x_codes"], st["x_scales"], st["acc"] = xc[:, 0, :], xs[:, 0], acc[:, 0, :]
    y = base
    if "a" in case:
        y = (y + o.lora_delta_multi(x, case["a"], case["b"], case["s"], case["idx"])).astype(F32)
    if "residual" in case:
        y = (y + case["residual"]).astype(F32)
    st["pre_cast"] = y
    fused = o.bf16_round(y)
    st["fused"] = fused
    out = o.swiglu_from_interleaved(fused) if case.get("swiglu") else fused
    st["out"] = out
    return st if return_stages else out


def to_torch(case, device):
    import torch

    from __graft_entry__ import load_package

    pkg = load_package()
    t = {}
    bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device).to(torch.bfloat16)
    t["x"] = bf(case["x"])
    t["weight"] = pkg.quantized_lora.GroupQuantizedWeight(
        torch.from_numpy(case["codes"]).to(device), torch.from_numpy(case["scales"]).to(device),
        case["k"], case["k"], 8, case["k"])
    if "a" in case:
        t["a"], t["b"] = bf(case["a"]), bf(case["b"])
        t["s"] = torch.from_numpy(case["s"]).to(device)
        t["idx"] = torch.from_numpy(case["idx"]).to(device)
    if "gamma" in case:
        t["gamma"] = torch.from_numpy(case["gamma"]).to(device)
    if "residual" in case:
        t["residual"] = bf(case["residual"])
    return t


def gpu_forward(case, device="cuda:0", flags=0, return_aux=True):
    """Run the HIP path through the C ABI on a case; returns numpy float32 out (+ aux dict)."""
    import torch

    from __graft_entry__ import load_package

    w8 = load_package().w8a8_lora
    t = to_torch(case, device)
    res = w8.forward(t["x"], t["weight"], t.get("a"), t.get("b"), t.get("s"),
                     adapter_indices=t.get("idx"), rms_gamma=t.get("gamma"), eps=1e-6,
                     residual=t.get("residual"), swiglu=bool(case.get("swiglu")), flags=flags,
                     return_aux=return_aux)
    torch.cuda.synchronize()
    if return_aux:
        out, aux = res
        aux_np = {k: (v.to(torch.float32) if v.dtype == torch.bfloat16 else v).cpu().numpy()
                  for k, v in aux.items()}
        return out.to(torch.float32).cpu().numpy(), aux_np
    return res.to(torch.float32).cpu().numpy()


def compare(got, want):
    ok = o.within_tolerance(got, want)
    gate = o.numerical_gate(got, want)
    return {"violations": int(np.count_nonzero(~ok)), "size": int(ok.size),
            "max_abs": float(np.max(np.abs(got.astype(np.float64) - want))) if ok.size else 0.0,
            "bitwise_fraction": float(np.mean(o.bf16_bits(got) == o.bf16_bits(want))), **gate}
