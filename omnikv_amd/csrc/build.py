"""Compile the HIP sources in this directory into omnikv_amd/libomnikv_hip.so for gfx950.

Usage: python omnikv_amd/csrc/build.py [--force]
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OUT = os.path.join(PKG, "libomnikv_hip.so")
SOURCES = ["okv_api.hip", "okv_attn.hip", "okv_attn_mfma.hip", "okv_topk.hip", "okv_topk_mb.hip", "okv_gather.hip",
           "okv_window.hip", "okv_diag.hip", "okv_layer.hip"]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-pthread",
]


def build(force: bool = True, verbose: bool = True) -> str:
    srcs = [os.path.join(HERE, s) for s in SOURCES]
    if not force and os.path.exists(OUT):
        newest = max(os.path.getmtime(p) for p in srcs + [os.path.join(HERE, h) for h in ("okv_internal.h", "okv_device.h")])
        if os.path.getmtime(OUT) >= newest:
            return OUT
    cmd = ["hipcc"] + FLAGS + srcs + ["-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if verbose and out.strip():
        print(out)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    return OUT


ABI_SMOKE_SRC = os.path.join(os.path.dirname(PKG), "tests", "native", "abi_smoke.cpp")
ABI_SMOKE_BIN = os.path.join(os.path.dirname(PKG), "tests", "native", "abi_smoke")


def build_abi_smoke(verbose: bool = True) -> str:
    """The host-only C++ program that exercises the C ABI without Python (tests/native/)."""
    cmd = ["hipcc", "-O1", "-std=c++17", "-Wno-unused-command-line-argument", ABI_SMOKE_SRC, "-L", PKG,
           "-lomnikv_hip", "-Wl,-rpath,$ORIGIN/../../omnikv_amd", "-o", ABI_SMOKE_BIN]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout)
    return ABI_SMOKE_BIN


if __name__ == "__main__":
    build(force=True)
    print("built", OUT)
    print("built", build_abi_smoke())
