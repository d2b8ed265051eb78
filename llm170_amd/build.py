"""Builds the gfx950 code objects (assets/*.hsaco) and the host library libw4a16hip.so, in-tree.

Code objects are compiled offline with hipcc --genco for gfx950 only and loaded at run time with
hipModuleLoadData (the reference ships fatbins built by scripts/build_cuda_kernels.sh and loads them through the
driver API the same way).  Run:  python -m llm170_amd.build
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
KERNEL_DIR = os.path.join(PKG, "csrc", "kernels")
HOST_DIR = os.path.join(PKG, "csrc", "host")
ASSET_DIR = os.path.join(PKG, "assets")
LIB_PATH = os.path.join(PKG, "libw4a16hip.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

# packed FP32 instructions are disabled for all device code
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                "-packed-fp32-ops", "-ffp-contract=off", "--genco", "--no-gpu-bundle-output"]
# No code object is built with floating-point contraction: the lane twin must keep its un-fused multiply and add, and
# a library routine (expf) must expand identically in every code object so that fused epilogues give the bits of the
# separate kernels.  Kernels that want a fused multiply-add write __builtin_fmaf.
FUSED_OK = set()


def kernel_sources():
    return sorted(f[:-4] for f in os.listdir(KERNEL_DIR) if f.endswith(".hip"))


def build_asset(name):
    src = os.path.join(KERNEL_DIR, name + ".hip")
    out = os.path.join(ASSET_DIR, name + ".hsaco")
    flags = list(DEVICE_FLAGS)
    if name in FUSED_OK:
        flags[flags.index("-ffp-contract=off")] = "-ffp-contract=fast"
    cmd = ["hipcc"] + flags + ["-I", KERNEL_DIR, "-o", out, src]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (name, r.stdout))
    return out


def build_host():
    srcs = sorted(os.path.join(HOST_DIR, f) for f in os.listdir(HOST_DIR) if f.endswith(".cc"))
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(ROOT, "include"), "-I", HOST_DIR, "-I", os.path.join(ROCM, "include"),
           "-o", LIB_PATH] + srcs + ["-L", os.path.join(ROCM, "lib"), "-lamdhip64", "-ldl",
                                     "-Wl,-rpath," + os.path.join(ROCM, "lib")]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("host library build failed:\n%s" % r.stdout)
    return LIB_PATH


def build_all(verbose=True):
    os.makedirs(ASSET_DIR, exist_ok=True)
    names = kernel_sources()
    with ThreadPoolExecutor(max_workers=min(8, len(names))) as ex:
        outs = list(ex.map(build_asset, names))
    lib = build_host()
    if verbose:
        for o in outs + [lib]:
            print("built", os.path.relpath(o, ROOT), os.path.getsize(o), "bytes")
    return outs, lib


def ensure_built(verbose=False):
    """Build only when nothing is built yet (a fresh checkout): tests, the smoke run and the benchmark load what is
    there.  The library itself never builds or falls back: loading it without these files raises."""
    missing = not os.path.exists(LIB_PATH) or any(
        not os.path.exists(os.path.join(ASSET_DIR, n + ".hsaco")) for n in kernel_sources())
    if missing:
        build_all(verbose=verbose)
    return missing


if __name__ == "__main__":
    build_all()
    sys.exit(0)
