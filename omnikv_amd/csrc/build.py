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
           "okv_window.hip"]
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


if __name__ == "__main__":
    build(force=True)
    print("built", OUT)
