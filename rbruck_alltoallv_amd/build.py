"""Builds librbruck_vc.so (HIP kernels + C ABI) in-tree with hipcc for gfx950."""
from __future__ import annotations

import os
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "librbruck_vc.so")
SOURCES = ["vc_meta.hip", "vc_plan.hip", "vc_copy.hip", "vc_api.hip", "vc_tools.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed FP32 instructions stay off for every HIP translation unit of this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-shared", "-std=c++17", "-Wall",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build_library(verbose: bool = False) -> str:
    cmd = [HIPCC, *FLAGS, "-o", LIB_PATH, *[os.path.join(CSRC, s) for s in SOURCES]]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(" ".join(cmd))
        print(res.stdout)
        print("\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l))
    if res.returncode != 0:
        raise RuntimeError("hipcc failed building librbruck_vc.so")
    return LIB_PATH


EXAMPLES = ("vc_example", "vc_mlinputs_example")
EXAMPLE_BIN = os.path.join(PKG_DIR, "examples", "vc_example")
MLINPUTS_EXAMPLE_BIN = os.path.join(PKG_DIR, "examples", "vc_mlinputs_example")


def build_example(verbose: bool = False) -> list[str]:
    """The C++ drivers above the C ABI (host code only; they link the library next to them)."""
    built = []
    for name in EXAMPLES:
        src, out = os.path.join(PKG_DIR, "examples", name + ".cpp"), os.path.join(PKG_DIR, "examples", name)
        cmd = [HIPCC, "-O2", "-std=c++17", "-Wall", "-x", "hip", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", src, "-L" + PKG_DIR, "-lrbruck_vc", "-Wl,-rpath,$ORIGIN/..", "-o", out]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if verbose or res.returncode != 0:
            print(" ".join(cmd))
            print(res.stdout)
            print("\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l))
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed building examples/{name}")
        built.append(out)
    return built


VARIANTS_BIN = os.path.join(PKG_DIR, "examples", "vc_copy_variants")


def build_variants(verbose: bool = False) -> str:
    """The A/B program of the forwarded copy kernel (examples/vc_copy_variants.hip includes csrc/vc_copy.hip): the
    product kernel, the variants that were measured against it and the contiguous copies that bound them."""
    cmd = [HIPCC, "-O3", "-std=c++17", "-Wall", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           os.path.join(PKG_DIR, "examples", "vc_copy_variants.hip"), "-o", VARIANTS_BIN]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(" ".join(cmd))
        print(res.stdout)
        print("\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l))
    if res.returncode != 0:
        raise RuntimeError("hipcc failed building examples/vc_copy_variants")
    return VARIANTS_BIN


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_example(verbose=True))
    print(build_variants(verbose=True))
