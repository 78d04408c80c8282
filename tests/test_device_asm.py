"""A check on the compiled device code of the 16x16x64 GEMM kernel (no GPU: hipcc cross-compiles).

The kernel's integer MFMAs are inline assembly with the accumulator as one read-write operand, so the
compiler does not know that an MFMA has just written an accumulation register and inserts none of the
wait states a read of that register by another unit would need.  The kernel is written so that no such read
comes close; this test reads the assembly of every instantiation and measures it: between an int8 MFMA
and the next instruction of another kind that reads a register it wrote there must be at least MIN_GAP
instructions (the result of this MFMA is safe to read a dozen wait states behind its issue, and every
instruction takes at least one).  Text order stands in for execution order: the accumulators are read
in the epilogue, which follows the last stage in the text as it does in time.
"""

import re
import subprocess

import pytest

from __graft_entry__ import PKG_DIR, _load_build_module

MIN_GAP = 14
KERNEL = re.compile(r"^(_ZN4w8a818w8a8_gemm16_kernel\S+):")
INT8_MFMA = re.compile(r"v_mfma_i32_16x16x64_i8 a\[(\d+):(\d+)\]")
AGPR = re.compile(r"\ba(\d+)\b|a\[(\d+):(\d+)\]")
STORES = ("scratch_store", "global_store", "buffer_store", "ds_write", "flat_store")


def closest_reads(asm_text):
    """{kernel: smallest number of instructions between an int8 MFMA and a foreign read of its result}."""
    lines = asm_text.split("\n")
    out = {}
    i = 0
    while i < len(lines):
        m = KERNEL.match(lines[i])
        if not m:
            i += 1
            continue
        name = m.group(1)
        last_write, n, worst = {}, 0, None
        i += 1
        while i < len(lines) and not lines[i].startswith(".Lfunc_end"):
            raw = lines[i]
            t = raw.strip()
            i += 1
            if not raw.startswith("\t") or t.startswith((".", ";")):
                continue
            n += 1
            w = INT8_MFMA.match(t)
            if w:
                for r in range(int(w.group(1)), int(w.group(2)) + 1):
                    last_write[r] = n
                continue
            ops = t.split(None, 1)[1] if " " in t else ""
            srcs = ops if t.startswith(STORES) else ",".join(ops.split(",")[1:])
            for a in AGPR.finditer(srcs):
                regs = [int(a.group(1))] if a.group(1) else range(int(a.group(2)), int(a.group(3)) + 1)
                for r in regs:
                    if r in last_write:
                        gap = n - last_write[r]
                        worst = gap if worst is None else min(worst, gap)
        out[name] = worst
    return out


def test_checker_sees_a_close_read():
    asm = "\n".join([
        "_ZN4w8a818w8a8_gemm16_kernelILi1ELi2ELi4EEEvNS_8GemmArgsE:",
        "\tv_mfma_i32_16x16x64_i8 a[4:7], v[0:3], v[4:7], a[4:7]",
        "\ts_nop 1",
        "\tv_accvgpr_read_b32 v9, a5",
        "\tv_mfma_i32_16x16x64_i8 a[8:11], v[0:3], v[4:7], a[8:11]",
        "\tscratch_store_dwordx4 off, a[8:11], off",
        ".Lfunc_end0:",
    ])
    assert closest_reads(asm) == {"_ZN4w8a818w8a8_gemm16_kernelILi1ELi2ELi4EEEvNS_8GemmArgsE": 1}


def test_no_instantiation_reads_an_accumulator_right_behind_its_mfma(tmp_path):
    build = _load_build_module()
    try:
        hipcc = build.find_hipcc()
    except RuntimeError as e:  # pragma: no cover - the image ships hipcc
        pytest.skip(str(e))
    flags = [f for f in build.HIPCC_FLAGS if f not in ("-shared", "-fPIC") and not f.startswith("-Wl,")]
    out = tmp_path / "w8a8_api.s"
    cmd = [hipcc, *flags, "--cuda-device-only", "-S",
           str(PKG_DIR / "csrc" / "w8a8_api.hip"), "-o", str(out)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    gaps = closest_reads(out.read_text())
    assert len(gaps) >= 12, sorted(gaps)  # every (epilogue, rank chunks, geometry) instantiation
    close = {k: v for k, v in gaps.items() if v is not None and v < MIN_GAP}
    assert not close, close
