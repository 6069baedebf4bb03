"""Compiles the HIP sources in this directory into ../libpbg_hip.so for gfx950.

Usage: python build.py   (needs hipcc on PATH or under /opt/rocm/bin)
"""
import os
import pathlib
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = pathlib.Path(__file__).resolve().parent
SOURCES = ["common.hip", "sort.hip", "row_adagrad.hip", "perm.hip", "gemm.hip", "seg_linear.hip", "step.hip", "fused.hip", "sliced.hip", "stream.hip", "plugins.hip"]
LIB = HERE.parent / "libpbg_hip.so"
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # keep packed fp32 instructions out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc() -> str:
    found = shutil.which("hipcc")
    if found:
        return found
    cand = "/opt/rocm/bin/hipcc"
    if os.path.exists(cand):
        return cand
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False) -> pathlib.Path:
    cc = hipcc()
    obj_dir = HERE / "build"
    obj_dir.mkdir(exist_ok=True)

    def compile_one(src: str) -> pathlib.Path:
        obj = obj_dir / (src + ".o")
        cmd = [cc, *FLAGS, "-c", str(HERE / src), "-o", str(obj)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{res.stderr}")
        if verbose:
            print("compiled", src)
        return obj

    with ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    tmp = LIB.with_suffix(".so.tmp")
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
