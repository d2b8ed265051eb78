"""CPU-side checks of the host library: it loads, exports every declared entry point, its asset manifest matches the
kernel sources, and the shape contract behaves as the reference's (no GPU calls)."""
import os
import re

import pytest

from llm170_amd import ffi, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = ffi.load()
    header = open(os.path.join(ROOT, "include", "w4a16_hip.h")).read()
    declared = set(re.findall(r"\b(w4a16_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations parsed"
    for name in sorted(declared):
        assert hasattr(lib, name), name
    assert declared == set(ffi.declared_symbols())


def expand_kernel_macros(text):
    """Kernel names produced by function-like macros whose body contains `extern "C" __global__ ... void NAME...(`;
    macros may call other macros and paste suffixes with ##."""
    text = re.sub(r"\\\n", " ", text)
    macros = {}
    for m in re.finditer(r"^#define\s+(\w+)\(([^)]*)\)\s+(.*)$", text, flags=re.M):
        macros[m.group(1)] = ([a.strip() for a in m.group(2).split(",")], m.group(3))
    body_lines = [ln for ln in text.split("\n") if not ln.startswith("#define")]

    def expand(line, depth=0):
        out = line
        for name, (params, body) in macros.items():
            for call in list(re.finditer(r"\b%s\(([^()]*)\)" % name, out)):
                args = [a.strip() for a in call.group(1).split(",")]
                if len(args) != len(params):
                    continue
                rep = body
                for p_, a_ in zip(params, args):
                    rep = re.sub(r"\b%s\b" % p_, a_, rep)
                rep = re.sub(r"\s*##\s*", "", rep)
                out = out.replace(call.group(0), rep)
        return expand(out, depth + 1) if out != line and depth < 8 else out

    names = set()
    for ln in body_lines:
        if re.match(r"^[A-Z0-9_]+\(", ln):
            names.update(re.findall(r'__global__[^;{]*?\bvoid\s+(w4a16_\w+)\s*\(', expand(ln)))
    return names


def kernel_text(kdir, asset):
    """The text one code object is compiled from.  A source may be a few lines that define a selector and include
    another source (prefill_g128.hip builds the dense group-128 kernels of prefill.hip); `#ifdef SELECTOR ... #else ...
    #endif` blocks of the included text are resolved the way the preprocessor would for that code object."""
    text = open(os.path.join(kdir, asset + ".hip")).read()
    defined = set(re.findall(r"^#define\s+(\w+)\s*$", text, flags=re.M))
    inc = re.search(r'^#include "(\w+\.hip)"', text, flags=re.M)
    if inc:
        text = open(os.path.join(kdir, inc.group(1))).read()

    def pick(m):
        return m.group(2) if m.group(1) in defined else m.group(3)

    return re.sub(r"^#ifdef (PF_\w+)\n(.*?)^#else\n(.*?)^#endif\n", pick, text, flags=re.M | re.S)


def test_manifest_matches_kernel_sources():
    """Precedent: manifest symbols == extern "C" __global__ symbols of the .cu files (assets.rs:394-443)."""
    man = ffi.manifest()
    kdir = os.path.join(ROOT, "llm170_amd", "csrc", "kernels")
    for asset, syms in man.items():
        text = kernel_text(kdir, asset)
        names = set(re.findall(r'extern "C" __global__[^;{]*?\bvoid\s+(w4a16_\w+)\s*\(', text))
        # kernels stamped out by macros: expand `#define M(...) body` textually until only `void <name>(` remain
        names |= expand_kernel_macros(text)
        assert sorted(names) == sorted(syms), asset
        assert len(set(syms)) == len(syms)
    hips = sorted(f[:-4] for f in os.listdir(kdir) if f.endswith(".hip"))
    assert hips == sorted(man), "every kernel source is a manifest asset and vice versa"


def test_host_constants_mirror_kernel_defines():
    """Precedent: constants of the host must equal the #defines parsed out of the kernel text
    (w4a16_dec/tests.rs:87-202).  Host name = kW4 + CamelCase of the macro (W4_ prefix dropped)."""
    kdir = os.path.join(ROOT, "llm170_amd", "csrc", "kernels")
    defines = {}
    for f in os.listdir(kdir):
        for m in re.finditer(r"^#define\s+([A-Z0-9_]+)\s+(\d+)\b", open(os.path.join(kdir, f)).read(), flags=re.M):
            defines[m.group(1)] = int(m.group(2))
    host = open(os.path.join(ROOT, "llm170_amd", "csrc", "host", "w4a16_internal.h")).read()
    consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"constexpr int kW4(\w+) = (\d+);", host)}
    assert len(consts) >= 11
    for camel, value in consts.items():
        macro = re.sub(r"(?<!^)(?=[A-Z])", "_", camel).upper()
        hits = [v for k, v in defines.items() if k in (macro, "W4_" + macro)]
        assert hits == [value], (camel, macro, hits, value)
    # the sources use the names, not the numbers, where a launch depends on them
    moe = open(os.path.join(ROOT, "llm170_amd", "csrc", "host", "w4a16_moe.cc")).read()
    assert "kW4MoeAlignWaves" in moe and "kW4MoeLdx" in moe and "kW4MoeMaxKsplit" in moe


def test_shapes_accept_contract():
    # gptq4.rs:196-208
    ops.check_shapes(1, 8 * 640, 8 * 40, 5120, 8, 5120, 128)
    ops.check_shapes(8, 8 * 640, 8 * 40, 8 * 5120, 8, 5120, 128)
    ops.check_shapes(1, 512 * 256, 512 * 64, 2048, 512, 2048, 32)
    ops.check_shapes(8, 512 * 256, 512 * 64, 8 * 2048, 512, 2048, 32)
    ops.check_shapes(1, 8 * 1024, 8 * 256, 8192, 8, 8192, 32)


def test_shapes_reject_bad_rank_and_misalignment():
    # gptq4.rs:210-216
    for args in [(1, 8 * 640, 8 * 40, 5120, 8, 5121, 128), (0, 8 * 640, 8 * 40, 0, 8, 5120, 128),
                 (1, 7 * 640, 8 * 40, 5120, 8, 5120, 128), (1, 8 * 640, 8 * 40, 5120, 8, 5120, 64)]:
        with pytest.raises(ops.W4a16Error) as e:
            ops.check_shapes(*args)
        assert e.value.code == ffi.ERR_SHAPE and "shape contract" in str(e.value)


def test_gemv_k_limit_of_the_reference_is_not_carried_over():
    # gptq4.rs:218-223 rejects t == 1 with k > 256 * group (shared-memory scale cache); no such cache here
    ops.check_shapes(1, 8 * 4112, 8 * 257, 32896, 8, 32896, 128)
    ops.check_shapes(2, 8 * 4112, 8 * 257, 2 * 32896, 8, 32896, 128)


def test_kernel_sym_selects_variants():
    # gptq4.rs:225-233 (the two combinations the reference rejects are served here)
    assert ops.kernel_sym(128, False) == "w4a16_lane_g128_f16"
    assert ops.kernel_sym(32, True) == "w4a16_lane_g32_bf16"
    assert ops.kernel_sym(32, False) == "w4a16_lane_g32_f16"
    with pytest.raises(ops.W4a16Error) as e:
        ops.kernel_sym(64, False)
    assert e.value.code == ffi.ERR_UNSUPPORTED


def test_code_objects_are_gfx950():
    adir = os.path.join(ROOT, "llm170_amd", "assets")
    for asset in ffi.manifest():
        blob = open(os.path.join(adir, asset + ".hsaco"), "rb").read()
        assert blob[:4] == b"\x7fELF" and b"gfx950" in blob, asset


def test_bench_refuses_more_than_one_gpu():
    """The bench measures one GPU's share; asked for more it says so and exits non-zero without touching a device."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "--gpus 2" in r.stderr and r.stdout.strip() == ""


def test_product_path_fails_loudly_without_a_gpu():
    """No CPU fallback: creating a context where no HIP device exists raises the library's error."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from llm170_amd import ops
    with pytest.raises(ops.W4a16Error):
        ops.Ctx(0)
