"""Builds the gfx950 code objects (assets/*.hsaco) and the host library libw4a16hip.so, in-tree.

Code objects are compiled offline with hipcc --genco for gfx950 only and loaded at run time with
hipModuleLoadData (the reference ships fatbins built by scripts/build_cuda_kernels.sh and loads them through the
driver API the same way).  Run:  python -m llm170_amd.build
"""
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
KERNEL_DIR = os.path.join(PKG, "csrc", "kernels")
HOST_DIR = os.path.join(PKG, "csrc", "host")
BENCH_DIR = os.path.join(PKG, "csrc", "bench")  # measurement probes: built beside the assets, not in the manifest
ASSET_DIR = os.path.join(PKG, "assets")
LIB_PATH = os.path.join(PKG, "libw4a16hip.so")
OBJ_DIR = os.path.join(PKG, "build")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

# packed FP32 instructions are disabled for all device code
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                "-packed-fp32-ops", "-ffp-contract=off", "--genco", "--no-gpu-bundle-output"]
# No code object is built with floating-point contraction: the lane twin must keep its un-fused multiply and add, and
# a library routine (expf) must expand identically in every code object so that fused epilogues give the bits of the
# separate kernels.  Kernels that want a fused multiply-add write __builtin_fmaf.
FUSED_OK = set()
# per-file backend options: the dense group-128 prefill kernels schedule for instruction-level parallelism
EXTRA_FLAGS = {"prefill_g128": ["-mllvm", "-amdgpu-sched-strategy=max-ilp"]}


HASH_PATH = os.path.join(PKG, "assets", "SOURCE_HASH")


def kernel_sources():
    return sorted(f[:-4] for f in os.listdir(KERNEL_DIR) if f.endswith(".hip"))


def source_hash():
    """sha256 over every file the artefacts are built from (kernel and host sources, headers, this script), in a fixed
    order.  Written next to the artefacts by a build; tests, smoke and the benchmark rebuild when it no longer matches
    and print it, so a record can be tied to the sources that produced it."""
    h = hashlib.sha256()
    files = [os.path.join(ROOT, "include", f) for f in sorted(os.listdir(os.path.join(ROOT, "include")))]
    for d in (KERNEL_DIR, HOST_DIR, BENCH_DIR):
        files += [os.path.join(d, f) for f in sorted(os.listdir(d)) if f.endswith((".hip", ".hpp", ".cc", ".h"))]
    files.append(os.path.abspath(__file__))
    for f in files:
        h.update(os.path.relpath(f, ROOT).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def built_hash():
    try:
        with open(HASH_PATH) as fh:
            return fh.read().strip()
    except OSError:
        return None


def build_asset(name):
    if name.startswith("bench/"):
        src = os.path.join(BENCH_DIR, name[6:] + ".hip")
        out = os.path.join(ASSET_DIR, "bench_" + name[6:] + ".hsaco")
    else:
        src = os.path.join(KERNEL_DIR, name + ".hip")
        out = os.path.join(ASSET_DIR, name + ".hsaco")
    flags = list(DEVICE_FLAGS)
    if name in FUSED_OK:
        flags[flags.index("-ffp-contract=off")] = "-ffp-contract=fast"
    cmd = ["hipcc"] + flags + EXTRA_FLAGS.get(name, []) + ["-I", KERNEL_DIR, "-o", out, src]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (name, r.stdout))
    return out


def build_host():
    """g++ for the host sources; hipcc for the one source that owns a device array (w4a16_noalloc.hip: its object
    carries a gfx950 device image); hipcc links."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    inc = ["-I", os.path.join(ROOT, "include"), "-I", HOST_DIR, "-I", os.path.join(ROCM, "include")]
    objs = []
    for f in sorted(os.listdir(HOST_DIR)):
        src, obj = os.path.join(HOST_DIR, f), os.path.join(OBJ_DIR, f + ".o")
        if f.endswith(".cc"):
            cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__"] + inc + ["-c", "-o", obj, src]
        elif f.endswith(".hip"):
            cmd = ["hipcc", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
                   "-packed-fp32-ops", "-Wno-unknown-warning-option"] + inc + ["-c", "-o", obj, src]
        else:
            continue
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("host library build failed (%s):\n%s" % (f, r.stdout))
        objs.append(obj)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs + [
        "-L", os.path.join(ROCM, "lib"), "-lamdhip64", "-ldl", "-Wl,-rpath," + os.path.join(ROCM, "lib")]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("host library link failed:\n%s" % r.stdout)
    return LIB_PATH


def build_all(verbose=True):
    os.makedirs(ASSET_DIR, exist_ok=True)
    names = kernel_sources() + ["bench/" + f[:-4] for f in sorted(os.listdir(BENCH_DIR)) if f.endswith(".hip")]
    with ThreadPoolExecutor(max_workers=min(8, len(names))) as ex:
        outs = list(ex.map(build_asset, names))
    lib = build_host()
    with open(HASH_PATH, "w") as fh:
        fh.write(source_hash() + "\n")
    if verbose:
        for o in outs + [lib]:
            print("built", os.path.relpath(o, ROOT), os.path.getsize(o), "bytes")
        print("source hash", source_hash())
    return outs, lib


def ensure_built(verbose=False):
    """Build when nothing is built yet (a fresh checkout) or when the artefacts were built from other sources than the
    tree holds now (the recorded source hash differs): tests, the smoke run and the benchmark otherwise load what is
    there.  The library itself never builds or falls back: loading it without these files raises."""
    missing = not os.path.exists(LIB_PATH) or any(
        not os.path.exists(os.path.join(ASSET_DIR, n + ".hsaco")) for n in kernel_sources())
    stale = not missing and built_hash() != source_hash()
    if missing or stale:
        build_all(verbose=verbose)
    return missing or stale


if __name__ == "__main__":
    build_all()
    sys.exit(0)
