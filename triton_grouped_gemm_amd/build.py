"""Compile csrc/*.hip for gfx950 into libtgg_amd.so next to this file.

``python -m triton_grouped_gemm_amd.build`` (or ``build_library()``) runs hipcc once per
translation unit in parallel and links the objects.  hipcc cross-compiles, so no
GPU is needed to build.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libtgg_amd.so"
ARCH = "gfx950"
# packed fp32 VALU forms are switched off for every HIP translation unit
HIPCC_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; ROCm toolchain is required to build libtgg_amd.so")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(map(str, cmd)) + "\n" + err)
    return err


def build_library(verbose: bool = False, jobs: int | None = None) -> Path:
    hipcc = _hipcc()
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    objs = [obj_dir / (s.stem + ".o") for s in sources]
    jobs = jobs or min(len(sources), int(os.environ.get("MAX_JOBS", "8")))

    def compile_one(pair):
        src, obj = pair
        # -save-temps=obj leaves the intermediate files next to the object; only the device assembly is kept
        # (build/<stem>.gfx950.s): tests/test_isa_hazards.py reads it to check what the compiler cannot check
        # around the inline-assembly memory instructions.
        msg = _run([hipcc, *HIPCC_FLAGS, "-save-temps=obj", "-c", str(src), "-o", str(obj)])
        for tmp in obj_dir.glob(src.stem + "*"):
            if tmp == obj:
                continue
            if tmp.name == f"{src.stem}-hip-amdgcn-amd-amdhsa-{ARCH}.s":
                os.replace(tmp, obj_dir / f"{src.stem}.{ARCH}.s")
            elif tmp.suffix != ".s" or "-" in tmp.name:
                tmp.unlink()
        if verbose and msg.strip():
            print(msg, file=sys.stderr)

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(sources, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
