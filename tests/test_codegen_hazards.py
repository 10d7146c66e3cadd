"""The prefill kernel's row maximum uses v_max3_f32 through inline asm.  The compiler inserts the wait states an
MFMA result needs before a vector instruction reads it only for instructions it knows, so an asm statement that
reads a fresh MFMA result would see stale registers now and then.  This test compiles the kernel to assembly
(no GPU needed) and checks that every v_max3_f32 whose sources were written by an MFMA shortly before is
separated from that MFMA by an ordinary vector instruction that reads the MFMA's result (which the compiler does
space correctly)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "minivllm_amd", "csrc", "prefill_varlen.hip")
WINDOW = 40          # instructions looked back; an MFMA result is final after at most ~20 issue slots


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def unguarded_asm_reads(asm_text):
    lines = [l.strip() for l in asm_text.split("\n")
             if l.startswith("\t") and not l.strip().startswith((";", "."))]
    found, total = [], 0
    for i, line in enumerate(lines):
        if not line.startswith("v_max3_f32"):
            continue
        total += 1
        ops = [t.strip() for t in line.split(None, 1)[1].split(",")]
        sources = set().union(*[_regs(t) for t in ops[1:]])
        guarded = set()
        for j in range(i - 1, max(i - WINDOW, -1), -1):
            prev = lines[j]
            name = prev.split()[0]
            toks = [t.strip() for t in prev.split(None, 1)[1].split(",")] if " " in prev else []
            if name.startswith("v_mfma"):
                dst = _regs(toks[0])
                if dst & sources and not (dst & guarded):
                    found.append((line, prev))
            elif name.startswith("v_") and not name.startswith("v_max3"):
                for t in toks[1:]:
                    guarded |= _regs(t)
    return total, found


def test_checker_flags_a_bare_read_and_accepts_a_guarded_one():
    bad = "\tv_mfma_f32_32x32x16_bf16 v[84:99], v[4:7], v[8:11], v[84:99]\n\tv_max3_f32 v2, v84, v85, v86\n"
    good = ("\tv_mfma_f32_32x32x16_bf16 v[84:99], v[4:7], v[8:11], v[84:99]\n\ts_nop 9\n"
            "\tv_max_f32_e32 v2, v99, v99\n\tv_max3_f32 v2, v2, v84, v85\n")
    assert unguarded_asm_reads(bad) == (1, [("v_max3_f32 v2, v84, v85, v86",
                                             "v_mfma_f32_32x32x16_bf16 v[84:99], v[4:7], v[8:11], v[84:99]")])
    assert unguarded_asm_reads(good) == (1, [])


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not installed")
def test_prefill_kernel_has_no_asm_read_inside_mfma_latency(tmp_path):
    from minivllm_amd._build import HIPCC_FLAGS
    out = tmp_path / "prefill.s"
    cmd = ["hipcc"] + [f for f in HIPCC_FLAGS if f != "-c"] + ["-S", "--cuda-device-only", "-o", str(out), SRC]
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    total, found = unguarded_asm_reads(out.read_text())
    assert total > 500, total          # every instantiation of the tile body has its chain
    assert found == [], found[:3]
