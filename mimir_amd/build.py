"""Builds libmimir_mi355x.so, the gfx950 code of this package, with hipcc.

The library is built in-tree (mimir_amd/lib/) ahead of time; nothing compiles
at run time. `python -m mimir_amd.build` rebuilds it.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmimir_mi355x.so")
OBJ_DIR = os.path.join(LIB_DIR, "obj")

ARCH = "gfx950"
# -packed-fp32-ops is switched off on purpose: hipcc must not form v_pk_*_f32.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
         "-Wno-unknown-warning-option", "-ffp-contract=on"] + DEVICE_FLAGS


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = ["hipcc", *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
    return obj


PROBE_SRC = os.path.join(HERE, "probe", "launch_cost.hip")
PROBE_BIN = os.path.join(LIB_DIR, "launch_cost")


def build_probe() -> list[str]:
    """The stand-alone launch-cost probe (no part of the library): once as it is, once with its kernels' arguments
    preloaded into scalar registers."""
    outs = []
    for suffix, extra in (("", []), ("_preload", ["-mllvm", "-amdgpu-kernarg-preload-count=16", '-DPRELOAD_NOTE="16 SGPRs"'])):
        out = PROBE_BIN + suffix
        cmd = ["hipcc", "-O3", "-std=c++17", f"--offload-arch={ARCH}", *DEVICE_FLAGS, *extra, PROBE_SRC, "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {PROBE_SRC}:\n{r.stderr[-4000:]}")
        outs.append(out)
    return outs


def build(verbose: bool = False) -> str:
    """Compiles every .hip source for gfx950 and links the shared library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = ["hipcc", "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, LIB_PATH)
    build_probe()
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
