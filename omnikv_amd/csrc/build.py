"""Compile the HIP sources in this directory for gfx950 into

  omnikv_amd/libomnikv_hip.so       the product library: the entry points of include/omnikv_hip.h
  omnikv_amd/libomnikv_hip_diag.so  the measurement build: the same sources with -DOKV_DIAG plus
                                    okv_diag.hip (split-pass-only switch, load-only floor kernel, empty
                                    launch); loaded by bench.py and omnikv_amd.microbench only

  omnikv_amd/libomnikv_hip_stamps.so  only with --stamps: the measurement build plus device timestamps inside the
                                      gather-mode split pass and the merge (-DOKV_STAMPS), for
                                      `python -m omnikv_amd.microbench --op sparse_timeline`

Usage: python omnikv_amd/csrc/build.py [--no-diag] [--stamps]
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OUT = os.path.join(PKG, "libomnikv_hip.so")
OUT_DIAG = os.path.join(PKG, "libomnikv_hip_diag.so")
OUT_STAMPS = os.path.join(PKG, "libomnikv_hip_stamps.so")
SOURCES = ["okv_api.hip", "okv_attn.hip", "okv_attn_mfma.hip", "okv_topk.hip", "okv_topk_mb.hip", "okv_gather.hip",
           "okv_window.hip", "okv_layer.hip"]
DIAG_SOURCES = SOURCES + ["okv_diag.hip"]
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


def _compile(sources, out, extra, verbose):
    srcs = [os.path.join(HERE, s) for s in sources]
    cmd = ["hipcc"] + FLAGS + extra + srcs + ["-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    text = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if verbose and text.strip():
        print(text)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + text)
    return out


def build_stamps(verbose: bool = True) -> str:
    """The timeline build (not part of build(): nothing loads it but microbench --op sparse_timeline)."""
    return _compile(DIAG_SOURCES, OUT_STAMPS, ["-DOKV_DIAG", "-DOKV_STAMPS"], verbose)


def build(force: bool = True, verbose: bool = True, diag: bool = True) -> str:
    """Builds the product library and, unless diag=False, the measurement build next to it (the two
    compile side by side).  Returns the product library's path."""
    from concurrent.futures import ThreadPoolExecutor

    jobs = [(SOURCES, OUT, [])]
    if diag:
        jobs.append((DIAG_SOURCES, OUT_DIAG, ["-DOKV_DIAG"]))
    if not force:
        headers = [os.path.join(HERE, h) for h in ("okv_internal.h", "okv_device.h")]
        jobs = [j for j in jobs if not os.path.exists(j[1]) or os.path.getmtime(j[1]) < max(
            os.path.getmtime(p) for p in [os.path.join(HERE, s) for s in j[0]] + headers)]
    with ThreadPoolExecutor(max_workers=2) as pool:
        for f in [pool.submit(_compile, srcs, out, extra, verbose) for srcs, out, extra in jobs]:
            f.result()
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
    if "--stamps" in sys.argv:
        print("built", build_stamps())
        sys.exit(0)
    build(force=True, diag="--no-diag" not in sys.argv)
    print("built", OUT, "" if "--no-diag" in sys.argv else "and " + OUT_DIAG)
    print("built", build_abi_smoke())
