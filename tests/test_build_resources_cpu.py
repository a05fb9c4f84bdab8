"""What the compiler made of the kernels, checked after every build (mamba-fused-minimal_amd/build.py collects the
compiler's per-kernel resource report into build/resource_usage.json).

The matrix-core kernels load operands with inline assembly (LDS-direct buffer loads, transposing LDS reads) and wait
for them with hand-counted s_waitcnt instructions.  The compiler does not know that such a register is still being
written after the statement that names it, so a spill of one -- a copy to scratch memory right after the load was
issued -- would save a stale value and give wrong results with no error.  No kernel here may spill vector registers
or use scratch at all; the chain kernel in particular lives at the edge of the register file (4 x 64 parked state
registers + 64 accumulators + operands).  The reference has no counterpart (Triton allocates for it)."""
import importlib.util
import json
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "mamba-fused-minimal_amd")


@pytest.fixture(scope="module")
def usage():
    path = os.path.join(PKG, "build", "resource_usage.json")
    lib = os.path.join(PKG, "libssd_gfx950.so")
    if not os.path.exists(path) or not os.path.exists(lib) or os.path.getmtime(path) + 600 < os.path.getmtime(lib):
        spec = importlib.util.spec_from_file_location("ssd_build", os.path.join(PKG, "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_library()
    with open(path) as f:
        return json.load(f)


def test_every_source_reports_its_kernels(usage):
    counts = {src: len(kernels) for src, kernels in usage.items()}
    assert counts["ssd_capi.hip"] == 0                       # host code only
    for src in ("ssd_chain.hip", "ssd_quad.hip", "ssd_mfma.hip", "ssd_generic.hip", "ssd_state_passing.hip",
                "ssd_chunk_cumsum.hip", "ssd_chunk_scan_states.hip", "ssd_mover.hip"):
        assert counts[src] > 0, src
    # the chain kernel: dstate 64 / 128 x chunk 128 / 256 x 1 / 2 / 4 chunks per item (2 / 4 with bf16 out) x seq_idx or
    # not x LOCAL / GLOBAL, + the fill
    assert counts["ssd_chain.hip"] == 4 * (3 + 2) * 2 * 2 + 1


def test_no_kernel_spills_vector_registers_or_uses_scratch(usage):
    for src, kernels in usage.items():
        for name, r in kernels.items():
            assert r["ScratchSize [bytes/lane]"] == 0, (src, name, r)
            assert r["VGPRs Spill"] == 0, (src, name, r)
            assert r["Dynamic Stack"] == "False", (src, name, r)
            assert r["VGPRs"] + r["AGPRs"] <= 512 and r["Occupancy [waves/SIMD]"] >= 1, (src, name, r)


def test_register_budgets_of_the_two_four_tile_kernels(usage):
    # four-tile kernel: two workgroups per compute unit (<= 256 registers per lane); chain kernel with four chunks per
    # item: the whole file, one workgroup per compute unit
    for name, r in usage["ssd_quad.hip"].items():
        assert r["VGPRs"] + r["AGPRs"] <= 256 and r["Occupancy [waves/SIMD]"] >= 2, (name, r)
    big = [r for name, r in usage["ssd_chain.hip"].items() if "chain_kernelILi8ELi8ELi4E" in name]
    assert len(big) == 8 and all(448 < r["VGPRs"] + r["AGPRs"] <= 512 for r in big), big
