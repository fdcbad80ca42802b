"""Ahead-of-time build of the native layer for gfx950.

    python -m autograd_amd.build            # build everything in-tree
    python -m autograd_amd.build --check    # exit 0 iff the built files exist

Produces, next to this file:
    libautograd_hip.so   the C-ABI library (include/autograd_hip.h)
    hip_ext*.so          the pybind11 module `autograd_amd.hip_ext` (HipContext)
and tests/c_abi/layer_check, a plain-C program (gcc, C99) that calls the library
without Python; the GPU tests run it.

The reference builds its Metal extension with setuptools (setup.py:13-31); here
the device code must be cross-compiled by hipcc for one architecture, so the
recipe is explicit.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = PKG / "csrc" / "build"
LIB = PKG / "libautograd_hip.so"
ARCH = "gfx950"

DEVICE_SOURCES = ["memops.hip", "norm.hip", "activation.hip", "rope.hip", "embedding.hip", "optimizer.hip", "loss.hip", "reduce.hip", "strided.hip", "pointwise.hip"]
HOST_SOURCES = ["context.cpp"]

COMMON_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Wall", "-Wno-unused-function", "-Wno-unused-but-set-variable", "-Wno-sometimes-uninitialized",
    "-Wno-unknown-pragmas", "-Wno-unused-result", "-Wno-conditional-uninitialized", "-Wno-pass-failed",
]
# packed-fp32 code generation is switched off for all device code
DEVICE_FLAGS = [f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def ext_path() -> Path:
    return PKG / ("hip_ext" + sysconfig.get_config_var("EXT_SUFFIX"))


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError(f"build step failed: {cmd[0]} ... {cmd[-1]}")
    noise = ("is not a recognized feature", "warning generated", "warnings generated")
    out = "\n".join(line for line in (proc.stdout + proc.stderr).splitlines()
                    if line.strip() and not any(n in line for n in noise))
    if out.strip():
        sys.stderr.write(out + "\n")


def _compile(src: str) -> Path:
    obj = OBJ / (src.rsplit(".", 1)[0] + ".o")
    cmd = [hipcc(), "-c", str(CSRC / src), "-o", str(obj)] + COMMON_FLAGS + DEVICE_FLAGS
    if src.endswith(".cpp"):
        cmd[1:1] = ["-x", "hip"]
    _run(cmd)
    return obj


def build_library(jobs: int = 6) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, DEVICE_SOURCES + HOST_SOURCES))
    _run([hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(LIB)] + [str(o) for o in objs])
    return LIB


def build_extension() -> Path:
    import pybind11

    out = ext_path()
    inc = [f"-I{pybind11.get_include()}", f"-I{sysconfig.get_paths()['include']}"]
    cmd = ([hipcc(), "-x", "hip", str(CSRC / "hip_ext.cpp"), "-shared", "-o", str(out)]
           + COMMON_FLAGS + DEVICE_FLAGS + inc
           + ["-fvisibility=hidden", f"-L{PKG}", "-lautograd_hip", "-Wl,-rpath,$ORIGIN"])
    _run(cmd)
    return out


C_CHECK_SRC = PKG.parent / "tests" / "c_abi" / "layer_check.c"
C_CHECK_BIN = C_CHECK_SRC.with_suffix("")


def build_c_check() -> Path:
    """the header and the library from plain C: gcc -std=c99 -pedantic, no hipcc"""
    _run(["gcc", "-std=c99", "-O1", "-Wall", "-Wextra", "-pedantic", "-Werror", f"-I{PKG.parent / 'include'}",
          str(C_CHECK_SRC), f"-L{PKG}", "-lautograd_hip", "-Wl,-rpath,$ORIGIN/../../autograd_amd", "-lm",
          "-o", str(C_CHECK_BIN)])
    return C_CHECK_BIN


def build_all(jobs: int = 6) -> None:
    build_library(jobs)
    build_extension()
    if C_CHECK_SRC.exists():
        build_c_check()


def is_built() -> bool:
    return LIB.exists() and ext_path().exists()


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--check", action="store_true")
    ap.add_argument("-j", type=int, default=6)
    args = ap.parse_args()
    if args.check:
        return 0 if is_built() else 1
    build_all(args.j)
    print(f"built {LIB.name} and {ext_path().name}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
