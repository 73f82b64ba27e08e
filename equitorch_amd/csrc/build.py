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
    build_torch_shim()
    return LIB_PATH


SHIM_PATH = os.path.join(LIB_DIR, "_cgtp_torch.so")


def build_torch_shim() -> str:
    """The PyTorch C++ extension over the C ABI (``torch_shim/cgtp_torch.cpp``: autograd node, argument block and
    allocation of the fused edge product), compiled with the host compiler against this interpreter's torch and
    linked to ``libcgtp.so`` next to it.  No device code."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension
    src = os.path.join(HERE, "torch_shim", "cgtp_torch.cpp")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-fPIC", "-shared", "-std=c++17", src, "-o", SHIM_PATH,
           "-DTORCH_EXTENSION_NAME=_cgtp_torch", "-DTORCH_API_INCLUDE_EXTENSION_H", "-DUSE_ROCM",
           "-D__HIP_PLATFORM_AMD__=1", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *[f"-I{d}" for d in cpp_extension.include_paths()], f"-I{sysconfig.get_paths()['include']}",
           "-I/opt/rocm/include", f"-I{os.path.join(ROOT, 'include')}",
           *[f"-L{d}" for d in cpp_extension.library_paths()], "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip",
           "-ltorch_hip", "-ltorch_python", f"-L{LIB_DIR}", "-lcgtp", "-Wl,-rpath,$ORIGIN"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"build of {SHIM_PATH} failed:\n{res.stdout}\n{res.stderr}")
    return SHIM_PATH


if __name__ == "__main__":
    print(build())
