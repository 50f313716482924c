"""Builds libnccl-net-fuselink.so (the HIP data path + the net plugin) for gfx950, in-tree.

Run as ``python -m fuselink_amd.build``.  hipcc cross-compiles without a GPU.  The artifact name
follows the reference's Makefile (``libnccl-net-fuselink.so``, Makefile:8 in the FuseLink tree) so
that ``NCCL_NET_PLUGIN=fuselink`` finds it.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "libnccl-net-fuselink.so"

SOURCES = ["fl_sched.hip", "fl_copy.hip", "fl_runtime.cc", "fl_vmm.cc", "fl_monitor.cc", "fl_plugin.cc"]

# -packed-fp32-ops: keep the compiler from forming packed FP32 instructions (none are wanted in a
# byte mover, and some forms are unreliable on this hardware).
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-pthread",
    "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build the gfx950 library")
    return exe


def lib_path() -> str:
    return os.path.join(LIBDIR, LIBNAME)


def build_library(verbose: bool = True) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    missing = [s for s in srcs if not os.path.exists(s)]
    if missing:
        raise RuntimeError("library sources missing: " + ", ".join(missing))
    cmd = [hipcc(), *FLAGS, "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, *srcs, "-o", lib_path(), "-ldl"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err)
    # RCCL looks a plugin named X up as librccl-net-X.so (NCCL as libnccl-net-X.so): offer both names
    alias = os.path.join(LIBDIR, "librccl-net-fuselink.so")
    if os.path.lexists(alias):
        os.remove(alias)
    shutil.copy2(lib_path(), alias)   # a copy, not a link: it must survive whatever carries the tree to another machine
    return lib_path()


def build_harness(verbose: bool = True) -> str | None:
    """The C++ plugin harness (dlopen()s the library exactly as a communication library would)."""
    src = os.path.join(ROOT, "tests", "harness", "plugin_harness.cc")
    if not os.path.exists(src):
        return None
    out = os.path.join(ROOT, "tests", "harness", "plugin_harness")
    # host code only: the HIP runtime is used for device buffers, no kernels are compiled here
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [shutil.which("g++") or "g++", "-O2", "-std=c++17", "-pthread", "-D__HIP_PLATFORM_AMD__",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(rocm, "include"), src, "-o", out,
           "-L" + os.path.join(rocm, "lib"), "-Wl,-rpath," + os.path.join(rocm, "lib"), "-lamdhip64", "-ldl"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("harness build failed:\n" + res.stderr)
    # the lane engine's own latency / rate harness
    esrc = os.path.join(ROOT, "tests", "harness", "engine_bench.cc")
    if os.path.exists(esrc):
        ecmd = cmd[:]
        ecmd[ecmd.index(src)] = esrc
        ecmd[ecmd.index(out)] = os.path.join(ROOT, "tests", "harness", "engine_bench")
        if verbose:
            print(" ".join(ecmd), flush=True)
        res = subprocess.run(ecmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("engine harness build failed:\n" + res.stderr)
    return out


def build_tsan(verbose: bool = True, sanitizer: str = "thread"):
    """Sanitizer build of the library's host code and of the harness (CPU-only check of the plugin's
    locking with "thread", of its memory handling with "address": device code is compiled as usual,
    only the host pass is instrumented)."""
    tag = {"thread": "tsan", "address": "asan"}[sanitizer]
    out_dir = os.path.join(ROOT, "tests", "harness", tag)
    os.makedirs(out_dir, exist_ok=True)
    lib = os.path.join(out_dir, f"libnccl-net-fuselink-{tag}.so")
    exe = os.path.join(out_dir, f"plugin_harness_{tag}")
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    flags = [f for f in FLAGS if f != "-O3"] + ["-O1", "-g", "-Xarch_host", "-fsanitize=" + sanitizer]
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    clang = os.path.join(rocm, "llvm", "bin", "clang++")
    cmds = [[hipcc(), *flags, "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, *srcs, "-o", lib, "-ldl"],
            [clang, "-O1", "-g", "-std=c++17", "-pthread", "-fsanitize=" + sanitizer, "-D__HIP_PLATFORM_AMD__",
             "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(rocm, "include"),
             os.path.join(ROOT, "tests", "harness", "plugin_harness.cc"), "-o", exe,
             "-L" + os.path.join(rocm, "lib"), "-Wl,-rpath," + os.path.join(rocm, "lib"), "-lamdhip64", "-ldl"]]
    for cmd in cmds:
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("sanitizer build failed:\n" + res.stderr)
    return lib, exe


def monitor_path() -> str:
    return os.path.join(LIBDIR, "fuselink-monitor")


def build_monitor(verbose: bool = True) -> str:
    """The lane-idleness daemon (host code only)."""
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = [shutil.which("g++") or "g++", "-O2", "-std=c++17", "-pthread", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
           os.path.join(CSRC, "fl_monitor.cc"), os.path.join(CSRC, "fl_monitor_main.cc"), "-o", monitor_path(), "-lrt"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("monitor build failed:\n" + res.stderr)
    return monitor_path()


def build_oracle(verbose: bool = True) -> None:
    """Compiles the CPU oracle (test infrastructure) and, where the reference tree is present,
    the reference's own monitor client under oracle/_ref."""
    cmd = ["make", "-B", "-C", os.path.join(ROOT, "oracle"), "all"]   # always recompiles, like the library
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + res.stdout + res.stderr)
    if verbose:
        print(res.stdout.strip())


def build_all(verbose: bool = True) -> None:
    build_library(verbose)
    build_monitor(verbose)
    build_harness(verbose)
    build_oracle(verbose)


if __name__ == "__main__":
    build_all()
    sys.exit(0)
