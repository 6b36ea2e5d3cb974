"""The fp8 KV write divides every value of a block by the block's scale.  The kernel forms that quotient
from a refined reciprocal and one residual correction (nkipy_amd/csrc/pa_div.h) and claims the bits of a
correctly rounded division; this compiles that header for the CPU and checks the claim exhaustively over
mantissas (2^23 scales x 9 reciprocal estimates x 2^7 bf16 significands, a few seconds on 8 cores)."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "nkipy_amd", "csrc")


def _has_fma():
    try:
        with open("/proc/cpuinfo") as f:
            return " fma " in f.read().replace("\n", " ")
    except OSError:
        return False


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_reciprocal_quotient_equals_division_exhaustively(tmp_path):
    exe = str(tmp_path / "div_check")
    flags = ["-O2", "-fopenmp", "-ffp-contract=off"] + (["-mfma"] if _has_fma() else [])
    subprocess.run(["gcc", *flags, "-I", CSRC, os.path.join(HERE, "div_by_scale_check.c"), "-o", exe, "-lm"], check=True)
    step = "1" if _has_fma() else "257"        # without hardware FMA fmaf() is a slow library routine: sample
    env = dict(os.environ, OMP_NUM_THREADS=str(min(8, os.cpu_count() or 1)))
    r = subprocess.run([exe, step], capture_output=True, text=True, timeout=600, env=env)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "wrong quotients 0" in r.stdout
