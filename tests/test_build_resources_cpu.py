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
                "ssd_chunk_cumsum.hip", "ssd_chunk_scan_states.hip", "ssd_mover.hip", "ssd_chain_scan.hip"):
        assert counts[src] > 0, src
    # the chain kernel: dstate 64 / 128 x chunk 128 / 256 x 1 / 2 / 4 chunks per item (2 / 4 with bf16 out) x seq_idx or
    # not x LOCAL / GLOBAL, + the fill
    assert counts["ssd_chain.hip"] == 4 * (3 + 2) * 2 * 2 + 1
    # ... and with the scan's state half in its chain step (items of two chunks): out fp32 or absent x seq_idx x
    # LOCAL / GLOBAL x chunk 128 / 256 x dstate 64 / 128
    assert counts["ssd_chain_scan.hip"] == 2 * 2 * 2 * 2 * 2


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


def test_generated_code_has_no_copies_of_operands_in_flight(usage):
    """The step loops read B operands with inline assembly whose results arrive later (an explicit wait in a later
    statement); a compiler copy of such a result, or a reuse of its registers, in between gives silently wrong states.
    The build scans the gfx950 assembly of every kernel for it (isa_check.py) and refuses to produce a library
    otherwise; the record of the last build must be clean, for every source file."""
    with open(os.path.join(PKG, "build", "async_operand_check.json")) as f:
        findings = json.load(f)
    assert set(findings) == set(usage)
    assert all(v == [] for v in findings.values()), {k: v[:2] for k, v in findings.items() if v}


def test_the_check_of_the_generated_code_finds_what_it_is_for():
    import sys
    sys.path.insert(0, PKG)
    import isa_check
    clean = """
_Z6kernelv:
	ds_read_b64_tr_b16 v[10:11], v5 offset:0
	ds_read_b64_tr_b16 v[12:13], v5 offset:0x100
	v_add_u32_e32 v1, v2, v3
	s_waitcnt lgkmcnt(0)
	v_mfma_f32_16x16x32_bf16 a[0:3], v[10:13], v[20:23], a[0:3]
	v_mov_b32_e32 v10, v1
	s_endpgm
"""
    assert isa_check.check_text(clean) == []
    copied = clean.replace("v_add_u32_e32 v1, v2, v3", "v_accvgpr_write_b32 a9, v11")
    found = isa_check.check_text(copied)
    assert len(found) == 1 and found[0]["registers"] == [11] and found[0]["kernel"] == "_Z6kernelv"
    reused = clean.replace("v_add_u32_e32 v1, v2, v3", "v_add_u32_e32 v12, v2, v3")
    assert [f["registers"] for f in isa_check.check_text(reused)] == [[12]]
    never_used = clean.replace("\tv_mfma_f32_16x16x32_bf16 a[0:3], v[10:13], v[20:23], a[0:3]\n", "")
    assert len(isa_check.check_text(never_used)) == 1          # overwritten by the v_mov without ever landing in a use


def test_the_check_covers_the_operand_reads_of_the_chain_kernel():
    """x and weight operands of a step are read in inline assembly too and waited for by the statement marked
    "; operands": nothing may touch their result registers in between, a read without such a wait is reported, and the
    compiler's own reads of the same kinds are left alone."""
    import sys
    sys.path.insert(0, PKG)
    import isa_check
    clean = """
_Z6kernelv:
	ds_read_b128 v[40:43], v7 offset:64
	;;#ASMSTART
	ds_read2st64_b32 v[10:11], v5 offset0:8 offset1:9
	ds_read_b128 v[12:15], v6 offset:0x80
	;;#ASMEND
	v_add_u32_e32 v40, v2, v3
	v_add_u32_e32 v1, v2, v3
	;;#ASMSTART
	s_waitcnt lgkmcnt(4) ; operands
	;;#ASMEND
	v_mul_f32_e32 v20, v10, v12
	s_endpgm
"""
    assert isa_check.check_operand_reads(clean) == []
    moved = clean.replace("v_add_u32_e32 v1, v2, v3", "v_accvgpr_write_b32 a9, v13")
    found = isa_check.check_operand_reads(moved)
    assert len(found) == 1 and found[0]["registers"] == [13] and found[0]["kernel"] == "_Z6kernelv"
    unwaited = clean.replace(" ; operands", "")
    assert len(isa_check.check_operand_reads(unwaited)) == 2          # both reads: used without their wait
