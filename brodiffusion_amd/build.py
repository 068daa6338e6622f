"""Compiles the HIP sources in csrc/ into lib/libmi_attention.so for gfx950.

Run as `python -m brodiffusion_amd.build`. hipcc cross-compiles without a GPU; the built
library stays in-tree (git-ignored) and is what tests, smoke and bench load.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmi_attention.so")
SOURCES = ["capi.hip", "sdpa_fwd.hip", "sdpa_wide.hip", "rope.hip", "linear_attn.hip", "linear.hip", "linear_dma.hip", "attn_block.hip", "attn_map.hip", "elementwise.hip", "probe.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-fvisibility=hidden",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    # packed-FP32 VALU forms are switched off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no NaN is ever produced on these paths (masked scores are -inf, guarded before subtraction), so
    # max / compare need no signalling-NaN quieting moves; infinities keep their meaning
    "-fno-honor-nans",
    "-Wall", "-Wno-unused-value", "-Wno-unknown-pragmas",
]


def _compile(src: str, obj_dir: str, save_temps: bool) -> str:
    obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    if save_temps:
        cmd.append("-save-temps=obj")
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout + r.stderr)
        raise RuntimeError(f"hipcc failed on {src}")
    return obj


def build(save_temps: bool = False, verbose: bool = False) -> str:
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir, save_temps), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout + r.stderr)
        raise RuntimeError("link failed")
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


HOST_DIR = os.path.join(HERE, "host")
HOST_LIB = os.path.join(LIB_DIR, "libbrodiffusion_amd_host.so")
HOST_TEST = os.path.join(LIB_DIR, "test_host_ops")
SPLIT_TEST = os.path.join(LIB_DIR, "test_split_geo")
CXX = os.environ.get("CXX", "g++")


def build_host(with_test: bool = True, verbose: bool = False) -> str:
    """C++20 host operator layer (no HIP in it; g++) on top of the C ABI, plus its test executable,
    which also links the CPU checker (test-only)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    common = [CXX, "-std=c++20", "-O2", "-fPIC", "-Wall", "-Wextra", "-I" + os.path.join(ROOT, "include"), "-I" + HOST_DIR]
    rpath = ["-Wl,-rpath,$ORIGIN", "-L" + LIB_DIR]
    cmd = [*common, "-shared", os.path.join(HOST_DIR, "attention_ops.cpp"), "-o", HOST_LIB, *rpath, "-lmi_attention"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout + r.stderr)
        raise RuntimeError("host library build failed")
    if with_test:
        oracle_dir = os.path.join(ROOT, "oracle")
        cmd = [*common, os.path.join(ROOT, "tests", "cpp", "test_host_ops.cpp"), "-o", HOST_TEST, *rpath,
               "-Wl,-rpath,$ORIGIN/../../oracle", "-L" + oracle_dir, "-lbrodiffusion_amd_host", "-lmi_attention", "-loracle"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            sys.stderr.write(r.stdout + r.stderr)
            raise RuntimeError("host test build failed")
    if with_test:
        # host-only check of the launch-planning arithmetic shared by host and device code (needs the HIP headers: hipcc)
        cmd = [HIPCC, "-std=c++20", "-O1", "-Wall", "--offload-host-only", "-x", "hip", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
               os.path.join(ROOT, "tests", "cpp", "test_split_geo.cpp"), "-o", SPLIT_TEST]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            sys.stderr.write(r.stdout + r.stderr)
            raise RuntimeError("split-geometry test build failed")
    if verbose:
        print("built", HOST_LIB)
    return HOST_LIB


if __name__ == "__main__":
    build(save_temps="--save-temps" in sys.argv, verbose=True)
    build_host(verbose=True)
