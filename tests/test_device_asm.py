"""A check on the compiled device code of the 16x16x64 GEMM kernel (no GPU: hipcc cross-compiles).

The kernel's MFMAs are inline assembly with the accumulator as one read-write operand (the integer ones
in accumulation registers, the bf16 ones of the LoRA term in vector registers), so the compiler does not
know that an MFMA has just written a register and inserts none of the wait states a read of that
register by another unit would need.  The kernel is written so that no such read
comes close; this test reads the assembly of every instantiation and measures it: between an int8 MFMA
and the next instruction of another kind that reads a register it wrote there must be at least MIN_GAP
wait states (the result of either MFMA is safe to read a dozen wait states behind its issue; every
instruction counts as one, an `s_nop n` as n + 1).  Text order stands in for execution order: the accumulators are read
in the epilogue, which follows the last stage in the text as it does in time.
"""

import re
import subprocess

import pytest

from __graft_entry__ import PKG_DIR, _load_build_module

MIN_GAP = 14
KERNEL = re.compile(r"^(_ZN4w8a818w8a8_gemm16_kernel\S+):")
INT8_MFMA = re.compile(r"v_mfma_i32_16x16x64_i8 a\[(\d+):(\d+)\]")
BF16_MFMA = re.compile(r"v_mfma_f32_16x16x32_bf16 v\[(\d+):(\d+)\]")
AGPR = re.compile(r"\ba(\d+)\b|a\[(\d+):(\d+)\]")
VGPR = re.compile(r"\bv(\d+)\b|v\[(\d+):(\d+)\]")
NOP = re.compile(r"s_nop (\d+)")
STORES = ("scratch_store", "global_store", "buffer_store", "ds_write", "flat_store")


def closest_reads(asm_text):
    """{kernel: fewest wait states between an assembly MFMA and a read of its result by anything else}."""
    lines = asm_text.split("\n")
    out = {}
    i = 0
    while i < len(lines):
        m = KERNEL.match(lines[i])
        if not m:
            i += 1
            continue
        name = m.group(1)
        last_a, last_v, n, worst = {}, {}, 0, None
        i += 1
        while i < len(lines) and not lines[i].startswith(".Lfunc_end"):
            raw = lines[i]
            t = raw.strip()
            i += 1
            if not raw.startswith("\t") or t.startswith((".", ";")):
                continue
            nop = NOP.match(t)
            n += int(nop.group(1)) + 1 if nop else 1
            w = INT8_MFMA.match(t)
            if w:
                for r in range(int(w.group(1)), int(w.group(2)) + 1):
                    last_a[r] = n
                continue
            w = BF16_MFMA.match(t)
            if w:  # the next MFMA on the same accumulator is interlocked by the hardware; operands are other registers
                for r in range(int(w.group(1)), int(w.group(2)) + 1):
                    last_v[r] = n
                continue
            ops = t.split(None, 1)[1] if " " in t else ""
            srcs = ops if t.startswith(STORES) else ",".join(ops.split(",")[1:])
            for rx, last in ((AGPR, last_a), (VGPR, last_v)):
                for a in rx.finditer(srcs):
                    regs = [int(a.group(1))] if a.group(1) else range(int(a.group(2)), int(a.group(3)) + 1)
                    for r in regs:
                        if r in last:
                            gap = n - last.pop(r)  # (a register is checked at its first read: later ones are farther)
                            worst = gap if worst is None else min(worst, gap)
            # a register written by something else is no longer an MFMA result
            if not t.startswith(STORES) and ops:
                d = VGPR.match(ops.split(",")[0].strip())
                if d:
                    for r in ([int(d.group(1))] if d.group(1) else range(int(d.group(2)), int(d.group(3)) + 1)):
                        last_v.pop(r, None)
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
    asm = "\n".join([
        "_ZN4w8a818w8a8_gemm16_kernelILi1ELi2ELi4EEEvNS_8GemmArgsE:",
        "\tv_mfma_f32_16x16x32_bf16 v[8:11], v[100:103], v[80:83], v[8:11]",
        "\tv_mfma_f32_16x16x32_bf16 v[12:15], v[100:103], v[84:87], v[12:15]",
        "\ts_nop 7",
        "\tv_add_f32_e32 v20, v9, v30",
        "\tv_add_f32_e32 v21, v13, v30",
        ".Lfunc_end0:",
    ])
    assert closest_reads(asm) == {"_ZN4w8a818w8a8_gemm16_kernelILi1ELi2ELi4EEEvNS_8GemmArgsE": 10}


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
