"""Builds ``equitorch_amd/lib/libcgtp.so`` (gfx950) from the HIP sources in this directory.

``python -m equitorch_amd.csrc.build`` regenerates the specialised tensor-product bodies, compiles every
``*.hip`` translation unit in parallel with hipcc and links them into one shared library with a plain C ABI
(``include/cgtp.h``).  Packed-fp32 instruction selection is disabled for all device code.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB_DIR = os.path.join(os.path.dirname(HERE), "lib")
OBJ_DIR = os.path.join(HERE, "_build")
LIB_PATH = os.path.join(LIB_DIR, "libcgtp.so")
BENCH_LIB_PATH = os.path.join(LIB_DIR, "libcgtp_bench.so")     # calibration kernels of bench.py, not the product ABI

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-ffp-contract=fast",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    f"-I{os.path.join(ROOT, 'include')}", f"-I{HERE}",
]


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src).replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    noise = "does not support 'packed-fp32-ops'"
    warn = "\n".join(l for l in res.stderr.splitlines() if l.strip() and noise not in l)
    if warn and os.environ.get("CGTP_BUILD_VERBOSE"):
        print(warn, file=sys.stderr)
    return obj


def build(jobs: int = 8) -> str:
    from . import gen_sh, gen_uv, gen_uvu, gen_uvu_big
    gen_sh.main()
    gen_uvu.main()
    gen_uvu_big.main()
    gen_uv.main()
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    sources = sorted(os.path.join(HERE, f) for f in os.listdir(HERE) if f.endswith(".hip"))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, sources))
    bench_dir = os.path.join(HERE, "bench")
    bench_sources = sorted(os.path.join(bench_dir, f) for f in os.listdir(bench_dir) if f.endswith(".hip"))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        bench_objs = list(pool.map(_compile, bench_sources))
    for path, parts in ((LIB_PATH, objs), (BENCH_LIB_PATH, bench_objs)):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", path, *parts]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link of {path} failed:\n{res.stdout}\n{res.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build())
