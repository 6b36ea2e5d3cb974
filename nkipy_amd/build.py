"""Builds libpaged_attn.so (HIP kernels + C ABI) for gfx950 with hipcc, and libpa_bench.so, the
matrix-core ceiling probe that only the benchmark loads.

Neither library has a Python or torch dependency; they link only the HIP runtime.
Run `python -m nkipy_amd.build` or call `build()`.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libpaged_attn.so")

SOURCES = ["pa_capi.hip", "pa_decode_generic.hip", "pa_decode_mfma.hip", "pa_prefill.hip", "pa_prefill_async.hip", "pa_kv_write.hip", "pa_o_proj.hip"]
BENCH_SOURCES = ["pa_probe.hip"]
BENCH_LIB_PATH = os.path.join(LIB_DIR, "libpa_bench.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # hipcc must not form packed-fp32 instructions from float code on these machines
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
]


def _compile(src: str, extra) -> str:
    obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(extra_flags=(), jobs: int = 4) -> str:
    """Compile every HIP source and link the shared library; returns its path."""
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, list(extra_flags)), SOURCES + BENCH_SOURCES))
    for path, part in ((LIB_PATH, objs[:len(SOURCES)]), (BENCH_LIB_PATH, objs[len(SOURCES):])):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *part, "-o", path]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link of {os.path.basename(path)} failed:\n{r.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build(extra_flags=sys.argv[1:]))
