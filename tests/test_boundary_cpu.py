"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports what include/ssd_gfx950.h
declares, the wrappers mirror the reference's signatures and assertion behaviour, and nothing silently falls
back to a CPU computation."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from ssd_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import importlib.util
        spec = importlib.util.spec_from_file_location("ssd_build", os.path.join(ROOT, "mamba-fused-minimal_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_library()
    return _lib.load()


def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "ssd_gfx950.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ssd_[a-z_]+)\s*\(", header))
    assert {"ssd_version", "ssd_chunk_state_fwd", "ssd_state_passing_fwd", "ssd_fused_chunk_state_passing_fwd",
            "ssd_status_string", "ssd_query_path"} <= declared
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.ssd_version() == int(re.search(r"#define SSD_ABI_VERSION (\d+)", header).group(1))
    from ssd_amd import _lib
    assert set(_lib.EXPORTS) == declared


def test_struct_layouts_match_header():
    from ssd_amd import _lib
    assert ctypes.sizeof(_lib.SsdTensor) == 8 + 4 + 4 + 5 * 8
    assert ctypes.sizeof(_lib.SsdDims) == 8 * 4
    assert ctypes.sizeof(_lib.SsdFusedOpts) == 8 + 8 + 4 * 4 + 8           # workspace, bytes, four ints, used_workspace
    assert ctypes.sizeof(_lib.SsdFusedPlan) == 4 + 4 + 5 * 4


def test_status_strings_and_argument_rejection_without_gpu(lib):
    from ssd_amd import _lib
    assert lib.ssd_status_string(0) == b"ok"
    x = torch.zeros(1, 256, 2, 64, dtype=torch.bfloat16)
    B = torch.zeros(1, 256, 1, 128, dtype=torch.bfloat16)
    dims = _lib.dims_arg(1, 256, 2, 64, 128, 1, 256, 1)
    assert lib.ssd_query_path(_lib.tensor_arg(x), _lib.tensor_arg(B), dims) == 1          # MFMA path
    assert lib.ssd_query_path(_lib.tensor_arg(x.float()), _lib.tensor_arg(B.float()), dims) == 0   # generic path
    bad = _lib.dims_arg(1, 256, 3, 64, 128, 2, 256, 1)                                     # nheads % ngroups
    assert lib.ssd_query_path(_lib.tensor_arg(x), _lib.tensor_arg(B), bad) == -2
    bad = _lib.dims_arg(1, 256, 2, 64, 128, 1, 256, 2)                                     # wrong nchunks
    assert lib.ssd_query_path(_lib.tensor_arg(x), _lib.tensor_arg(B), bad) == -2
    assert lib.ssd_query_path(_lib.tensor_arg(x), _lib.tensor_arg(B.float()), dims) == -3  # mixed dtypes
    xs = x.transpose(2, 3)                                                                 # innermost stride != 1
    assert lib.ssd_query_path(_lib.tensor_arg(xs), _lib.tensor_arg(B), dims) == -4
    assert lib.ssd_query_path(_lib.tensor_arg(None), _lib.tensor_arg(B), dims) == -1
    odd = _lib.dims_arg(1, 256, 2, 40, 128, 1, 256, 1)                                     # headdim 40: generic
    assert lib.ssd_query_path(_lib.tensor_arg(x), _lib.tensor_arg(B), odd) == 0
    # chunk cumsum: argument rejection happens before any device work
    dt = torch.zeros(1, 256, 2)
    A = torch.zeros(2)
    o = torch.zeros(1, 2, 1, 256)
    T = _lib.tensor_arg
    assert lib.ssd_chunk_cumsum_fwd(T(None), T(A), T(None), T(o), T(o), 1, 256, 2, 256, 0, 0.0, 1.0, None) == -1
    assert lib.ssd_chunk_cumsum_fwd(T(dt), T(A), T(None), T(o), T(o), 1, 256, 2, 0, 0, 0.0, 1.0, None) == -2
    assert lib.ssd_chunk_cumsum_fwd(T(dt), T(A), T(None), T(o.bfloat16()), T(o), 1, 256, 2, 256, 0, 0.0, 1.0, None) == -3
    assert lib.ssd_chunk_cumsum_fwd(T(dt), T(A), T(None), T(o), T(o), 1, 4096, 2, 2048, 0, 0.0, 1.0, None) == -2   # chunk > 1024
    # scan consumer: same order of checks (null, shape, dtype, stride) before any device work
    Cm = torch.zeros(1, 256, 1, 128, dtype=torch.bfloat16)
    st = torch.zeros(1, 1, 2, 64, 128)
    dA = torch.zeros(1, 2, 1, 256)
    y = torch.zeros(1, 256, 2, 64)
    assert lib.ssd_chunk_scan_states_fwd(T(Cm), T(None), T(dA), T(None), T(y), dims, 0, None) == -1
    assert lib.ssd_chunk_scan_states_fwd(T(Cm), T(st), T(dA), T(None), T(y), bad, 0, None) == -2
    assert lib.ssd_chunk_scan_states_fwd(T(Cm), T(st), T(dA.bfloat16()), T(None), T(y), dims, 0, None) == -3
    assert lib.ssd_chunk_scan_states_fwd(T(Cm), T(st), T(dA), T(None), T(y.transpose(2, 3)), dims, 0, None) == -4
    assert lib.ssd_set_token_split(5) == -2 and lib.ssd_set_token_split(1) == 0 and lib.ssd_set_token_split(0) == 1
    assert lib.ssd_set_segment_chunks(-1) == -2 and lib.ssd_set_segment_chunks(3) == 0 and lib.ssd_set_segment_chunks(0) == 3


def test_workspace_size_by_element_type_of_the_passed_states(lib):
    # fp32 `out`: header + a flag per (state tile, chunk).  bf16 `out`: that, rounded up to 256 bytes, and 32 x dstate
    # fp32 per (state tile, work item) -- the running state crosses between work items in fp32, as the reference keeps
    # it in registers (kernels/ssd_state_passing.py:61-84).  fp16 `out`, or bf16 with items of one chunk: not offered.
    from ssd_amd import _lib
    big = _lib.dims_arg(4, 8192, 80, 64, 128, 1, 256, 32)
    tiles, flags = 4 * 80 * 2, 128 + 4 * 80 * 2 * 32
    assert lib.ssd_fused_workspace_bytes_for(big, _lib.SSD_F32, 0) == lib.ssd_fused_workspace_bytes(big) == 4 * flags
    for r in (2, 4):
        want = 4 * ((flags + 63) // 64 * 64) + tiles * (32 // r) * 32 * 128 * 4
        assert lib.ssd_fused_workspace_bytes_for(big, _lib.SSD_BF16, r) == want
    assert lib.ssd_fused_workspace_bytes_for(big, _lib.SSD_BF16, 0) == lib.ssd_fused_workspace_bytes_for(big, _lib.SSD_BF16, 4)
    assert lib.ssd_fused_workspace_bytes_for(big, _lib.SSD_BF16, 1) == 0
    assert lib.ssd_fused_workspace_bytes_for(big, _lib.SSD_F16, 0) == 0
    odd = _lib.dims_arg(1, 2304, 8, 64, 128, 1, 256, 9)                # 9 chunks: 5 items of two, 3 of four
    assert lib.ssd_fused_workspace_bytes_for(odd, _lib.SSD_BF16, 2) == 4 * ((128 + 16 * 9 + 63) // 64 * 64) + 16 * 5 * 32 * 128 * 4
    assert lib.ssd_fused_workspace_bytes_for(odd, _lib.SSD_BF16, 4) == 4 * ((128 + 16 * 9 + 63) // 64 * 64) + 16 * 3 * 32 * 128 * 4


def test_argument_validation_from_two_threads_with_different_hooks(lib):
    # The three ssd_set_* hooks are process-wide atomics and everything else is per call: two host threads that keep
    # setting different hook values while they call the argument-validation paths (which return before any device
    # work) must see the same status codes as a single thread, workspace sizes that depend on the dims alone, and
    # from every hook only values that one of the threads has stored (ctypes drops the GIL during the calls).
    import threading
    from ssd_amd import _lib
    T = _lib.tensor_arg
    x = torch.zeros(1, 256, 2, 64, dtype=torch.bfloat16)
    B = torch.zeros(1, 256, 1, 128, dtype=torch.bfloat16)
    dt = torch.zeros(1, 256, 2)
    A = torch.zeros(2)
    o = torch.zeros(1, 2, 1, 256)
    good = _lib.dims_arg(1, 256, 2, 64, 128, 1, 256, 1)
    bad = _lib.dims_arg(1, 256, 3, 64, 128, 2, 256, 1)
    big = _lib.dims_arg(4, 8192, 80, 64, 128, 1, 256, 32)
    want_ws = lib.ssd_fused_workspace_bytes(big)
    assert want_ws == 4 * (128 + 4 * 80 * 2 * 32)
    settings = {"a": (2, 3, 1), "b": (4, 5, 2)}
    seen = {"split": {0, 2, 4}, "segment": {0, 3, 5}, "scan": {0, 1, 2}}
    errors = []

    def worker(name):
        split, segment, scan = settings[name]
        try:
            for _ in range(300):
                for hook, value, key in ((lib.ssd_set_token_split, split, "split"),
                                         (lib.ssd_set_segment_chunks, segment, "segment"),
                                         (lib.ssd_set_scan_kernel, scan, "scan")):
                    old = hook(value)
                    assert old in seen[key], (key, old)
                assert lib.ssd_query_path(T(x), T(B), good) == 1
                assert lib.ssd_query_path(T(x), T(B), bad) == -2
                assert lib.ssd_query_path(T(None), T(B), good) == -1
                assert lib.ssd_chunk_cumsum_fwd(T(dt), T(A), T(None), T(o), T(o), 1, 256, 2, 0, 0, 0.0, 1.0, None) == -2
                assert lib.ssd_fused_workspace_bytes(big) == want_ws
                assert lib.ssd_fused_chunk_state_passing_fwd_ws(T(x), T(B), T(None), T(None), T(None), T(None), T(None),
                                                                T(None), T(None), good, 1, None, None) == -1
                assert lib.ssd_set_token_split(3) == -2
        except BaseException as e:      # report in the main thread
            errors.append((name, repr(e)))

    threads = [threading.Thread(target=worker, args=(n,)) for n in settings]
    try:
        for t in threads: t.start()
        for t in threads: t.join()
    finally:
        lib.ssd_set_token_split(0); lib.ssd_set_segment_chunks(0); lib.ssd_set_scan_kernel(0)
    assert not errors, errors


def test_signatures_match_reference_call_surface():
    import ssd_amd
    sig = lambda f: list(inspect.signature(f).parameters)
    # kernels/ssd_chunk_state.py:202
    assert sig(ssd_amd._chunk_state_fwd) == ["B", "x", "dt", "dA_cumsum", "seq_idx", "states", "states_in_fp32"]
    # kernels/ssd_state_passing.py:87
    assert sig(ssd_amd._state_passing_fwd) == ["states", "dA_chunk_cumsum", "initial_states", "seq_idx", "chunk_size", "out_dtype"]
    # kernels/fused_globalbar.py:201, kernels/fused_concurrent.py:255
    want = ["B", "x", "dt", "dA_cumsum", "out_dtype", "initial_states", "seq_idx", "states", "states_in_fp32"]
    assert sig(ssd_amd._fused_chunk_state_state_passing_fwd_globalbar) == want
    assert sig(ssd_amd._fused_chunk_state_state_passing_fwd_concurrent) == want
    d = inspect.signature(ssd_amd._chunk_state_fwd).parameters
    assert d["seq_idx"].default is None and d["states"].default is None and d["states_in_fp32"].default is True
    # kernels/ssd_chunk_state.py:176
    assert sig(ssd_amd._chunk_cumsum_fwd) == ["dt", "A", "chunk_size", "dt_bias", "dt_softplus", "dt_limit"]
    d = inspect.signature(ssd_amd._chunk_cumsum_fwd).parameters
    assert d["dt_bias"].default is None and d["dt_softplus"].default is False and d["dt_limit"].default == (0.0, float("inf"))
    import kernels.ssd_chunk_state as k
    assert k._chunk_cumsum_fwd is ssd_amd._chunk_cumsum_fwd and k._chunk_state_fwd is ssd_amd._chunk_state_fwd


def test_shape_asserts_mirror_the_reference():
    import ssd_amd
    x = torch.zeros(1, 256, 4, 64)
    B = torch.zeros(1, 256, 1, 128)
    dt = torch.zeros(1, 4, 1, 256)
    with pytest.raises(AssertionError):
        ssd_amd._chunk_state_fwd(torch.zeros(1, 256, 3, 128), x, dt, dt)                   # nheads % ngroups
    with pytest.raises(AssertionError):
        ssd_amd._chunk_state_fwd(B, x, torch.zeros(1, 4, 2, 256), dt)                      # dA_cumsum.shape != dt.shape
    with pytest.raises(AssertionError):
        ssd_amd._chunk_state_fwd(B, x, dt, dt, seq_idx=torch.zeros(1, 255, dtype=torch.int32))
    with pytest.raises(AssertionError):
        ssd_amd._chunk_state_fwd(B, x, dt, dt, states=torch.zeros(1, 1, 4, 64, 64))
    with pytest.raises(AssertionError):
        ssd_amd._chunk_cumsum_fwd(torch.zeros(1, 256, 4), torch.zeros(3), 256)              # A.shape != (nheads,)
    with pytest.raises(AssertionError):
        ssd_amd._chunk_cumsum_fwd(torch.zeros(1, 256, 4), torch.zeros(4), 256, dt_bias=torch.zeros(5))
    with pytest.raises(AssertionError):
        ssd_amd._state_passing_fwd(torch.zeros(1, 2, 4, 8), torch.zeros(1, 4, 3))
    with pytest.raises(AssertionError):
        ssd_amd._state_passing_fwd(torch.zeros(1, 2, 4, 8), torch.zeros(1, 4, 2), initial_states=torch.zeros(1, 4, 9))
    with pytest.raises(AssertionError):
        ssd_amd._state_passing_fwd(torch.zeros(1, 2, 4, 8), torch.zeros(1, 4, 2), seq_idx=torch.zeros(1, 16, dtype=torch.int32))
    with pytest.raises(AssertionError):
        ssd_amd._fused_chunk_state_state_passing_fwd_globalbar(B, x, dt, dt, torch.float32,
                                                               initial_states=torch.zeros(1, 4, 64 * 128))


def test_no_cpu_fallback():
    import ssd_amd
    x = torch.zeros(1, 256, 4, 64)
    B = torch.zeros(1, 256, 1, 128)
    dt = torch.zeros(1, 4, 1, 256)
    for call in (lambda: ssd_amd._chunk_state_fwd(B, x, dt, dt),
                 lambda: ssd_amd._state_passing_fwd(torch.zeros(1, 2, 4, 8), torch.zeros(1, 4, 2)),
                 lambda: ssd_amd._fused_chunk_state_state_passing_fwd_concurrent(B, x, dt, dt, torch.float32)):
        with pytest.raises(RuntimeError, match="no CPU path"):
            call()


def test_product_code_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "mamba-fused-minimal_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_header_is_plain_c(tmp_path):
    # the boundary is a C ABI: the header must compile as C99 (and as C++) on its own
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    src.write_text('#include "ssd_gfx950.h"\n'
                   "int main(void) { ssd_fused_opts o = {0}; ssd_fused_plan p; ssd_dims d = {0}; (void)o; (void)p; (void)d;\n"
                   "  return SSD_FAMILY_COUNT == 5 && SSD_KERNEL_CHAIN_GLOBAL == 3 ? 0 : 1; }\n")
    inc = os.path.join(ROOT, "include")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-I", inc, str(src)], check=True)
    subprocess.run(["g++", "-std=c++11", "-Wall", "-fsyntax-only", "-x", "c++", "-I", inc, str(src)], check=True)


def test_kept_workspaces_can_be_released():
    import ssd_amd
    from ssd_amd import ops
    with ops._WORKSPACES_LOCK:
        ops._WORKSPACES[("test", 0)] = ops._Kept(torch.zeros(4, dtype=torch.int32))
    ssd_amd.release_workspaces()
    assert not ops._WORKSPACES


def test_epochs_of_a_kept_workspace():
    # what the wrappers pass as ssd_fused_opts.epoch for the workspace they keep per device and stream
    from ssd_amd.ops import _Epochs
    e = _Epochs()
    assert e.next(100) == 0                                # contents unknown: the library clears, the call counts as 1
    e.done(0, 0, 1, 100)
    assert e.next(100) == 2
    e.done(2, 0, 1, 100)
    assert e.next(50) == 3                                 # fewer flags than the clearing covered: fine
    e.done(3, 0, 0, 50)                                    # another kernel family served the call: the epoch was not used
    assert e.next(100) == 3
    e.done(3, 0, 1, 100)
    assert e.next(100) == 4
    e.done(4, -6, 0, 100)                                  # a failed call: contents unknown again
    assert e.next(100) == 0
    e.done(0, 0, 0, 100)                                   # cleared by nobody (not the chain kernel): still unknown
    assert e.next(100) == 0
    e.done(0, 0, 1, 100)
    e.last = _Epochs.LIMIT                                 # before the count could overflow it starts over
    assert e.next(100) == 0
    e.done(0, 0, 1, 100)
    # a call that looks at more flags than the last clearing covered must not trust the ones beyond: clear again
    assert e.next(100) == 2
    e.done(2, 0, 1, 100)
    assert e.next(101) == 0
    e.done(0, 0, 1, 101)
    assert e.next(101) == 2 and e.cleared == 101


def _header(epoch, err=0, tickets=(), totals=(), tag=True):
    """The first 128 ints of a chain workspace after a launch with this epoch (layout: csrc/ssd_params.h)."""
    import ctypes
    h = (ctypes.c_int32 * 128)()
    bank = epoch & 1
    for s, t in enumerate(tickets):
        h[32 * bank + s] = t
    for s, t in enumerate(totals):
        h[32 * bank + 16 + s] = t
    h[64 + bank] = err
    h[66] = epoch
    h[67] = 0x53534443 if tag else 0
    return h


def test_workspace_status_decoding():
    """ssd_fused_workspace_status_of on host copies of a workspace header: every failure of the ticket / flag-chain
    kernel has its own code, and a ticket counter that owns work items but handed out fewer (an XCD that received no
    workgroup) is an error although no error bit is set."""
    from ssd_amd import _lib
    lib = _lib.load()
    st = lib.ssd_fused_workspace_status_of
    assert st(None) == -1
    assert st(_header(3, tag=False, err=7)) == 0                                  # never a chain workspace
    ok = dict(tickets=[40 + 32] * 8, totals=[40] * 8)                             # every workgroup draws one past the end
    assert st(_header(3, **ok)) == 0
    assert st(_header(4, **ok)) == 0                                              # the other parity
    assert st(_header(3, err=1, **ok)) == _lib.SSD_ERR_CHAIN_TIMEOUT == -7
    assert st(_header(3, err=2, **ok)) == _lib.SSD_ERR_CHAIN_XCD == -8
    assert st(_header(3, err=3, **ok)) == -8
    assert st(_header(3, err=4 | 1, **ok)) == _lib.SSD_ERR_CHAIN_WORKSPACE == -10
    # slot 5 owns 40 items and handed out none / some
    for drawn in (0, 39):
        t = [72] * 8
        t[5] = drawn
        assert st(_header(3, tickets=t, totals=[40] * 8)) == _lib.SSD_ERR_CHAIN_INCOMPLETE == -9
        assert st(_header(2, tickets=t, totals=[40] * 8)) == -9
    t = [72] * 8
    t[5] = 40
    assert st(_header(3, tickets=t, totals=[40] * 8)) == 0
    # slots without units need no workgroup (GLOBAL: one counter)
    assert st(_header(3, tickets=[1536], totals=[1280])) == 0
    # the error word of the other parity belongs to another launch
    h = _header(3, **ok)
    h[64] = 1
    assert st(h) == 0
    for code in (-7, -8, -9, -10):
        assert lib.ssd_status_string(code).decode() not in ("unknown status", "")
