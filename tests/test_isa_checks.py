"""The wide linear kernels issue their MFMAs from inline assembly, which the compiler cannot guard with wait states.
This test compiles their assembly listings (no GPU needed: hipcc cross-compiles) and runs the checker that looks for an
accumulator read right behind a matrix instruction — the defect that once made the half-height kernel return stale
values for k-tile counts of 2 mod 3."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "kernl_amd", "csrc")
sys.path.insert(0, CSRC)


def test_checker_reports_an_early_read_and_accepts_a_guarded_one():
    import check_mfma_reads as chk

    mfma = "\tv_mfma_f32_16x16x32_f16 a[0:3], v[2:5], v[6:9], a[0:3]"
    early = [mfma, "\ts_add_i32 s1, s2, s3", "\tv_accvgpr_read_b32 v2, a0"]
    guarded = [mfma, "\ts_nop 15", "\tv_accvgpr_read_b32 v2, a0"]
    distant = [mfma] + ["\ts_add_i32 s1, s2, s3"] * chk.MIN_DISTANCE + ["\tv_accvgpr_read_b32 v2, a0"]
    assert chk.early_reads(early) == (2, 1)
    assert chk.early_reads(guarded) is None
    assert chk.early_reads(distant) is None
    assert chk.early_reads(["\tv_accvgpr_read_b32 v2, a0", mfma]) is None   # a read BEFORE any MFMA is none of its business


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_no_accumulator_read_follows_an_inline_assembly_mfma():
    run = subprocess.run(["make", "-C", CSRC, "-j2", "isa-check"], capture_output=True, text=True, timeout=900)
    assert run.returncode == 0, run.stdout[-3000:] + run.stderr[-3000:]
    assert " 0 reported" in run.stdout
