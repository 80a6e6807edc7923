"""Builds the two shared libraries of the package, in-tree, for gfx950.

``libkvmove.so``        hand-written HIP kernels + the C ABI (``include/kvmove.h``); no torch.
``libkvmove_torch.so``  torch op shim registering ``block_migration_ops`` / ``swapping_ops``.
``tests/lib_explore/libkvmove.so``  the HIP library again with ``-DKVM_EXPLORE``: every kernel flavour and the
                        knobs that select them, for sweeps and for the tests that show every flavour copies the
                        same bytes.  Never loaded by the package.
``libkvmove_torch_alt.so``  the same ops as ``kvmove_block_migration_ops`` / ``kvmove_swapping_ops``,
                        for a process that keeps another registration of DistServe's names.

Run as ``python distserve_amd/csrc/build.py`` (a plain script on purpose: it must work
when the libraries are missing or stale, so it does not import the package, which loads
them).  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

CSRC_DIR = os.path.dirname(os.path.abspath(__file__))
PKG_DIR = os.path.dirname(CSRC_DIR)
REPO_DIR = os.path.dirname(PKG_DIR)
LIB_DIR = os.path.join(PKG_DIR, "lib")
INCLUDE_DIR = os.path.join(REPO_DIR, "include")

KVMOVE_LIB = os.path.join(LIB_DIR, "libkvmove.so")
TORCH_LIB = os.path.join(LIB_DIR, "libkvmove_torch.so")
TORCH_ALT_LIB = os.path.join(LIB_DIR, "libkvmove_torch_alt.so")
EXPLORE_LIB = os.path.join(REPO_DIR, "tests", "lib_explore", "libkvmove.so")
ALT_NAMESPACES = ("kvmove_block_migration_ops", "kvmove_swapping_ops")

GPU_ARCH = "gfx950"
ROCM_HOME = os.environ.get("ROCM_PATH", "/opt/rocm")


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass of hipcc does not know the packed-fp32 target feature and says so
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip():
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"build step failed with exit code {res.returncode}: {' '.join(cmd)}")


def build_kvmove(explore: bool = False) -> str:
    hipcc = shutil.which("hipcc") or os.path.join(ROCM_HOME, "bin", "hipcc")
    out = EXPLORE_LIB if explore else KVMOVE_LIB
    os.makedirs(os.path.dirname(out), exist_ok=True)
    _run([
        hipcc, f"--offload-arch={GPU_ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wall", "-Wextra", f"-I{INCLUDE_DIR}", *(["-DKVM_EXPLORE"] if explore else []),
        os.path.join(CSRC_DIR, "kvmove.hip"), "-o", out,
    ])
    return out


def build_torch_shim(alt: bool = False) -> str:
    import torch
    from torch.utils import cpp_extension

    if not os.path.exists(KVMOVE_LIB):
        build_kvmove()
    torch_lib_dir = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-I{INCLUDE_DIR}", f"-I{os.path.join(ROCM_HOME, 'include')}"]
    cmd += [f"-I{p}" for p in cpp_extension.include_paths()]
    out = TORCH_LIB
    if alt:
        out = TORCH_ALT_LIB
        cmd += [f"-DKVM_MIGRATION_NS={ALT_NAMESPACES[0]}", f"-DKVM_SWAP_NS={ALT_NAMESPACES[1]}"]
    cmd += [os.path.join(CSRC_DIR, "kvmove_torch.cpp"), "-o", out,
            f"-L{LIB_DIR}", "-lkvmove", "-Wl,-rpath,$ORIGIN",
            f"-L{torch_lib_dir}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-Wl,--no-as-needed"]
    _run(cmd)
    return out


def build_all() -> None:
    build_kvmove()
    build_kvmove(explore=True)
    build_torch_shim()
    build_torch_shim(alt=True)


if __name__ == "__main__":
    build_all()
    print("built:", KVMOVE_LIB, TORCH_LIB, TORCH_ALT_LIB, EXPLORE_LIB)
    sys.exit(0)
