"""Ahead-of-time build of libmamba_hip.so for gfx950 (the build.rs equivalent).

The reference compiles its CUDA sources at run time with NVRTC
(src/mamba_ssm/gpu/kernels.rs:451-811); here every kernel is compiled by hipcc
into one shared library that sits next to this file, so a process only has to
dlopen it.  `python -m mamba_rs_amd.build` rebuilds it.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libmamba_hip.so"
ARCH = "gfx950"

# -packed-fp32-ops (a minus sign in front of the feature name): keep the compiler from forming v_pk_*_f32 out of scalar float code.
DEVICE_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators stay in ordinary VGPRs (no AccVGPR copies around each instruction).
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    # The first 16 dwords of a kernel's arguments arrive in scalar registers with the wave instead of being loaded by its
    # first instructions: 0.15 us per launch, which is 3 % of a batch-1 decode step (72 launches of 4.5 us).
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wno-unused-command-line-argument", "-Wno-unused-result", "-Wno-unused-value",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build_library(verbose: bool = True, jobs: int = 4) -> Path:
    """Compile every csrc/*.hip for gfx950 and link libmamba_hip.so. Always recompiles."""
    hipcc = _hipcc()
    objdir = PKG_DIR / "build"
    objdir.mkdir(exist_ok=True)
    srcs = sources()
    objs = [objdir / (s.stem + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        if verbose:
            print(f"[build] hipcc {src.name}", file=sys.stderr)
        _run([hipcc, *DEVICE_FLAGS, "-c", str(src), "-o", str(obj)])

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(compile_one, zip(srcs, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs),
          "-L/opt/rocm/lib", "-lrocblas", "-Wl,-rpath,/opt/rocm/lib"])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[build] wrote {LIB_PATH}", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
