"""Builds libssd_gfx950.so (the C-ABI library with the gfx950 HIP kernels) in-tree with hipcc.

Usage:  python build.py            (from anywhere)
hipcc cross-compiles for gfx950 without a GPU, so this runs on a CPU-only machine."""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libssd_gfx950.so")
OBJ_DIR = os.path.join(HERE, "build")
SOURCES = ["ssd_capi.hip", "ssd_mfma.hip", "ssd_quad.hip", "ssd_chain.hip", "ssd_generic.hip", "ssd_state_passing.hip", "ssd_chunk_cumsum.hip", "ssd_chunk_scan_states.hip", "ssd_mover.hip", "ssd_chain_scan.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep the compiler from forming packed-fp32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]
USAGE = os.path.join(OBJ_DIR, "resource_usage.json")
ISA_CHECK = os.path.join(OBJ_DIR, "async_operand_check.json")


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + out)
    return out


def _resource_usage(asm_text):
    """{kernel: {field: value}} from the gfx950 assembly the compiler leaves behind (--save-temps): the metadata entry of
    every kernel (registers, spills, scratch, dynamic stack) and the occupancy the compiler notes beside its code."""
    import re
    usage = {}
    occupancy = {}
    for m in re.finditer(r"^\s*\.amdhsa_kernel (\S+)$(.*?)^; Occupancy: (\d+)", asm_text, re.M | re.S):
        occupancy[m.group(1)] = int(m.group(3))
    for entry in re.split(r"^  - ", asm_text[asm_text.rfind("amdhsa.kernels:"):], flags=re.M)[1:]:
        f = dict(re.findall(r"^\s*\.(\w+):\s+(\S+)\s*$", entry, re.M))
        if "name" not in f:
            continue
        agpr, total = int(f.get("agpr_count", 0)), int(f.get("vgpr_count", 0))
        usage[f["name"]] = {"VGPRs": total - agpr, "AGPRs": agpr, "ScratchSize [bytes/lane]": int(f.get("private_segment_fixed_size", 0)),
                            "VGPRs Spill": int(f.get("vgpr_spill_count", 0)), "SGPRs Spill": int(f.get("sgpr_spill_count", 0)),
                            "Dynamic Stack": "True" if f.get("uses_dynamic_stack") == "true" else "False",
                            "Occupancy [waves/SIMD]": occupancy.get(f["name"], 0)}
    return usage


def build_library(verbose=False, extra_flags=(), jobs=None):
    """Compiles every source to an object (in parallel: the files are independent) and links the shared library."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(OBJ_DIR, exist_ok=True)
    compile_flags = [f for f in FLAGS if f != "-shared"]
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 8)

    def compile_one(src):
        # the compiler's intermediate files (the gfx950 assembly among them) go to a directory per source
        stem = os.path.splitext(src)[0]
        obj = os.path.join(OBJ_DIR, stem + ".o")
        tmp = os.path.join(OBJ_DIR, "temps_" + stem)
        shutil.rmtree(tmp, ignore_errors=True)
        os.makedirs(tmp)
        cmd = [hipcc(), *compile_flags, *extra_flags, "--save-temps", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=tmp)
        noise = "is not a recognized feature for this target"
        out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + out)
        return obj, out

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(compile_one, SOURCES))
    # the generated code, checked for copies of operands that inline assembly is still loading (isa_check.py)
    sys.path.insert(0, HERE)
    import isa_check
    findings, usage = {}, {}
    for src in SOURCES:
        tmp = os.path.join(OBJ_DIR, "temps_" + os.path.splitext(src)[0])
        usage[src] = {}
        for name in sorted(os.listdir(tmp)):
            if name.endswith("gfx950.s"):
                with open(os.path.join(tmp, name)) as f:
                    text = f.read()
                findings[src] = isa_check.check_text(text) + isa_check.check_operand_reads(text)
                usage[src] = _resource_usage(text)
        shutil.rmtree(tmp, ignore_errors=True)
    import json
    with open(USAGE, "w") as f:
        json.dump(usage, f, indent=1, sort_keys=True)
    with open(ISA_CHECK, "w") as f:
        json.dump(findings, f, indent=1, sort_keys=True)
    bad = {k: v for k, v in findings.items() if v}
    if bad:
        first = next(iter(bad.values()))[0]
        raise RuntimeError(f"the compiler moved operands that inline assembly is still loading in {sorted(bad)} "
                           f"({sum(len(v) for v in bad.values())} places, e.g. {first}); see {ISA_CHECK}")
    out = _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *[o for o, _ in results], "-o", LIB])
    for src, (_, text) in zip(SOURCES, results):
        if verbose and text.strip():
            print(text)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True, extra_flags=sys.argv[1:]))
