"""Deterministic W8A8+LoRA host case of the reference (M3/K64/N17 padded to 32, rank 8).

The integer formulas restate rocm/probe_w8a8_lora_forward.py:1193-1261; the
expected digests in ``w8a8_host_case.json`` are the reference's own pins
(rocm/probe_w8a8_lora_forward.py:210-218).  Arrays that are bf16 in the reference
are returned as float32 holding bf16-exact values.
"""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np

from oracle import w8a8_oracle as o

SPEC = json.loads((Path(__file__).with_name("w8a8_host_case.json")).read_text())


def build():
    m, k, n, n_pad, r = (SPEC["rows"], SPEC["in_features"], SPEC["out_features"],
                         SPEC["padded_out_features"], SPEC["rank"])
    row = np.arange(m, dtype=np.int32)[:, None]
    kk = np.arange(k, dtype=np.int32)[None, :]
    x = o.bf16_round((((row * 11 + kk * 5) % 33) - 16).astype(np.float32) / np.float32(8.0))

    ki = np.arange(k, dtype=np.int32)[:, None]
    ni = np.arange(n, dtype=np.int32)[None, :]
    dense = (((ki * 7 + ni * 3) % 41) - 20).astype(np.float32) / np.float32(16.0)
    q = o.quantize_frozen_weight(dense, bits=8, group_size=SPEC["group_size"], scale_dtype="bf16")
    codes = np.zeros((k, n_pad), dtype=np.int8)
    codes[:, :n] = q.codes
    scales = np.zeros((1, n_pad), dtype=np.float32)
    scales[:, :n] = q.scales

    ri = np.arange(r, dtype=np.int32)
    a = o.bf16_round((((np.arange(k)[:, None] * 3 + ri[None, :]) % 17) - 8).astype(np.float32)
                     / np.float32(16.0))
    b_core = o.bf16_round((((ri[:, None] * 5 + np.arange(n)[None, :]) % 19) - 9).astype(np.float32)
                          / np.float32(16.0))
    b = np.zeros((r, n_pad), dtype=np.float32)
    b[:, :n] = b_core
    scaling = np.float32(SPEC["scaling"])
    weight = o.GroupQuantizedWeight(codes=codes, scales=scales, original_in_features=k,
                                    padded_in_features=k, bits=8, group_size=SPEC["group_size"])
    return {"x": x, "weight": weight, "weight_codes": codes, "weight_scales": scales,
            "lora_a": a, "lora_b": b, "lora_scaling": scaling, "dense_weight": dense,
            "out_features": n}
