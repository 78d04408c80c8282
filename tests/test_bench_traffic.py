"""bench.py takes `roofline.traffic` from the committed rocprofv3 counter summaries, not from constants."""

import importlib.util
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def _bench():
    spec = importlib.util.spec_from_file_location("bench_module", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_headline_workloads_parse_to_more_than_their_algorithmic_bytes():
    bench = _bench()
    for workload in ("qwen3-8b-gate_up-m4096", "qwen3-8b-down-m16-decode"):
        got = bench.measured_traffic_bytes(workload)
        cfg = bench.WORKLOADS[workload]
        assert got is not None, workload
        floor = bench.gemm_kernel_bytes(cfg) if cfg.get("swiglu") else bench.algorithmic_bytes(cfg)
        assert floor <= got <= 8 * floor, (workload, got, floor)


def test_parser_scales_by_the_copy_of_known_size(tmp_path):
    bench = _bench()
    name = bench.PROFILE_TRAFFIC["qwen3-8b-gate_up-m4096"][0]
    lines = [
        "w8a8::cal_copy_kernel(int __vector(4) const*, int __vector(4)*, unsigned long)     grid   1048576  FETCH_SIZE avg     131072.0 KiB over 1 dispatches",
        "void w8a8::w8a8_gemm16_kernel<1, 2, 4>(w8a8::GemmArgs)                                grid    131072  FETCH_SIZE avg       1000.0 KiB over 15 dispatches",
        "w8a8::cal_copy_kernel(int __vector(4) const*, int __vector(4)*, unsigned long)     grid   1048576  WRITE_SIZE avg     262144.0 KiB over 1 dispatches",
        "void w8a8::w8a8_gemm16_kernel<1, 2, 4>(w8a8::GemmArgs)                                grid    131072  WRITE_SIZE avg        500.0 KiB over 15 dispatches",
    ]
    (tmp_path / name).write_text("\n".join(lines) + "\n")
    assert bench.measured_traffic_bytes("qwen3-8b-gate_up-m4096", tmp_path) == int((1000.0 * 2.0 + 500.0) * 1024)
    # a summary without the calibration copy, or without the kernel, gives no figure rather than a wrong one
    (tmp_path / name).write_text("\n".join(lines[1:]) + "\n")
    assert bench.measured_traffic_bytes("qwen3-8b-gate_up-m4096", tmp_path) is None
    (tmp_path / name).write_text("\n".join(lines[:1] + lines[2:3]) + "\n")
    assert bench.measured_traffic_bytes("qwen3-8b-gate_up-m4096", tmp_path) is None
    assert bench.measured_traffic_bytes("no-such-workload") is None
