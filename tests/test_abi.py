"""The C-ABI library on a machine without a GPU: it loads, exports every symbol the header
declares, and rejects bad arguments on the host before any launch."""
import ctypes
import os
import re

import pytest

from kernel_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "moe_a2a.h")

E_NULL, E_SHAPE, E_DTYPE, E_WORKSPACE, E_ALIGN, E_STATE = -1, -2, -3, -4, -5, -6
A = 0x1000  # any non-NULL, 16-byte aligned address; never dereferenced on the host


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_a2a_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def test_header_and_binding_agree():
    assert declared_functions() == sorted(_lib.PROTOTYPES)


def test_every_declared_symbol_is_exported():
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(raw, name), f"{name} is declared in include/moe_a2a.h but not exported"


def test_version_strings_and_queries(lib):
    assert lib.moe_a2a_abi_version() == _lib.ABI_VERSION
    assert lib.moe_a2a_strerror(0) == b"success"
    for code in (E_NULL, E_SHAPE, E_DTYPE, E_WORKSPACE, E_ALIGN, E_STATE):
        assert lib.moe_a2a_strerror(code).startswith(b"moe_a2a:")
    assert lib.moe_a2a_kernel_name(-1) == b"unknown"
    names = set()
    k = 0
    while lib.moe_a2a_kernel_name(k) != b"unknown":
        names.add(lib.moe_a2a_kernel_name(k))
        k += 1
    assert {b"route_tiles", b"route_dispatch", b"dispatch_rows", b"dispatch_fp8", b"combine_rows"} <= names
    # small tables route in one launch and need only the minimum scratch
    assert lib.moe_a2a_workspace_bytes(256, 8, 256) == 256
    assert lib.moe_a2a_workspace_bytes(4096, 8, 256) == 256
    assert lib.moe_a2a_workspace_bytes(16384, 4, 128) >= 64 * 128 * 4
    assert lib.moe_a2a_workspace_bytes(-1, 8, 256) == 0
    assert lib.moe_a2a_fused_max_rows() >= 2048
    assert lib.moe_a2a_fused_ok(256, 8, 7168) == 1  # the headline shape takes the one-launch path
    assert lib.moe_a2a_fused_ok(16384, 4, 4096) == 0
    assert lib.moe_a2a_fused_ok(1024, 6, 2048) == 1  # mid-size table: one launch with token tiles
    assert lib.moe_a2a_fused_ok(2048, 4, 2048) == 1
    assert lib.moe_a2a_fused_ok(4096, 8, 7168) == 0  # streaming sizes keep separate routing and dispatch
    assert lib.moe_a2a_fused_ok(33000, 8, 64) == 0  # short rows, long table: the table passes would outweigh the rows


def test_route_rejects_bad_arguments(lib):
    def route(T=4, K=2, E=8, W=2, indices=A, counts=A, offsets=A, soe=A, sos=A, meta=A, ws=A, wsb=1 << 20,
              max_recv=0):
        return lib.moe_a2a_route(indices, None, 0, T, K, E, W, max_recv, counts, offsets, soe, sos, meta, None, ws,
                                 wsb, None)

    assert route(K=0) == E_SHAPE
    assert route(K=33) == E_SHAPE
    assert route(E=0) == E_SHAPE
    assert route(E=1025) == E_SHAPE
    assert route(E=9, W=2) == E_SHAPE  # experts must split evenly over ranks
    assert route(W=0) == E_SHAPE
    assert route(T=-1) == E_SHAPE
    assert route(T=1 << 30, K=8) == E_SHAPE
    assert route(max_recv=-1) == E_SHAPE
    assert route(E=1024, W=8, max_recv=1 << 20) == E_SHAPE  # padded rows must stay addressable
    assert route(counts=None) == E_NULL
    assert route(indices=None) == E_NULL
    assert route(meta=None) == E_NULL
    # a table beyond the one-launch limit needs the workspace
    assert route(T=40000, K=8, E=8, W=2, ws=None) == E_WORKSPACE
    assert route(T=40000, K=8, E=8, W=2, wsb=16) == E_WORKSPACE


def test_row_functions_reject_bad_arguments(lib):
    assert lib.moe_a2a_dispatch(A, A, A, 4, 2, 12, None) == E_SHAPE  # H % 8
    assert lib.moe_a2a_dispatch(A, A, A, 4, 0, 64, None) == E_SHAPE
    assert lib.moe_a2a_dispatch(None, A, A, 4, 2, 64, None) == E_NULL
    assert lib.moe_a2a_dispatch(A + 4, A, A, 4, 2, 64, None) == E_ALIGN
    assert lib.moe_a2a_dispatch(A, None, A, 4, 2, 64, None) == E_NULL
    assert lib.moe_a2a_dispatch(A, A, A, 0, 2, 64, None) == 0  # nothing to do, nothing launched
    assert lib.moe_a2a_dispatch_fp8(A, 7, A, A, A, 4, 2, 128, 0, None) == E_DTYPE
    assert lib.moe_a2a_dispatch_fp8(A, _lib.BF16, A, A, A, 4, 2, 128, 2, None) == E_DTYPE  # scale mode
    assert lib.moe_a2a_dispatch_fp8(A, _lib.BF16, A, A, A, 4, 2, 64, 0, None) == E_SHAPE  # H % 128
    assert lib.moe_a2a_dispatch_fp8(A, _lib.BF16, A, A, None, 4, 2, 128, _lib.FP8_SCALE_POW2, None) == E_NULL
    assert lib.moe_a2a_stub(A, None, A, None, 5, _lib.BF16, 0, 8, 2, A, 8, 64, None) == E_DTYPE
    assert lib.moe_a2a_stub(A, None, A, None, _lib.BF16, _lib.BF16, 9, 8, 2, A, 8, 64, None) == E_DTYPE
    assert lib.moe_a2a_stub(A, None, A, None, _lib.BF16, _lib.BF16, 0, 9, 2, A, 8, 64, None) == E_SHAPE
    assert lib.moe_a2a_stub(A, None, None, None, _lib.BF16, _lib.BF16, 0, 8, 2, A, 8, 64, None) == E_NULL
    assert lib.moe_a2a_combine(A, A, A, 3, _lib.BF16, A, 4, 2, 64, None) == E_DTYPE
    assert lib.moe_a2a_combine(A, A, A, 0, 4, A, 4, 2, 64, None) == E_DTYPE
    assert lib.moe_a2a_combine(A, None, A, 0, _lib.BF16, A, 4, 2, 64, None) == E_NULL
    assert lib.moe_a2a_combine(A, A, A, 0, _lib.BF16, A + 8, 4, 2, 64, None) == E_ALIGN
    assert lib.moe_a2a_stub_combine(A, None, None, A, A, 0, _lib.BF16, _lib.BF16, 0, 8, 2, A, 4, 2, 64, None) == E_NULL
    assert lib.moe_a2a_stub_combine(A, None, A, A, A, 0, _lib.BF16, _lib.BF16, 0, 8, 3, A, 4, 2, 64, None) == E_SHAPE
    big = lib.moe_a2a_fused_max_rows() // 8 + 1
    assert lib.moe_a2a_route_dispatch(A, A, None, 0, big, 8, 8, 2, 64, 0, A, A, A, A, A, None, A, None) == E_SHAPE


def test_expert_gemm_rejects_bad_arguments(lib):
    def gemm(x=A, w=A, off=A, y=A, R=64, E=8, Kd=128, N=64, max_recv=0, elem=_lib.BF16):
        return lib.moe_a2a_expert_gemm(x, w, off, y, R, E, Kd, N, max_recv, elem, None)

    def gemm8(x=A, sc=A, w=A, off=A, y=A, R=64, E=8, Kd=128, N=64, max_recv=0, elem=_lib.BF16):
        return lib.moe_a2a_expert_gemm_fp8(x, sc, w, off, y, R, E, Kd, N, max_recv, elem, None)

    for f in (gemm, gemm8):
        assert f(elem=5) == E_DTYPE
        assert f(E=0) == E_SHAPE
        assert f(E=1025) == E_SHAPE
        assert f(N=12) == E_SHAPE
        assert f(max_recv=-1) == E_SHAPE
        assert f(R=-1) == E_SHAPE
        assert f(R=0) == 0  # nothing to do, nothing launched
        assert f(w=None) == E_NULL
        assert f(off=None) == E_NULL
        assert f(y=A + 8) == E_ALIGN
    def gemmq(x=A, xs=None, w=A, ws=A, off=A, y=A, R=64, E=8, Kd=128, N=128, max_recv=0, elem=_lib.BF16):
        return lib.moe_a2a_expert_gemm_q8(x, xs, w, ws, off, y, R, E, Kd, N, max_recv, elem, None)

    assert gemmq(elem=5) == E_DTYPE
    assert gemmq(N=64) == E_SHAPE   # one weight scale per 128 x 128 block
    assert gemmq(Kd=192) == E_SHAPE
    assert gemmq(ws=None) == E_NULL
    assert gemmq(R=0) == 0
    assert gemmq(y=A + 4) == E_ALIGN

    def gemmx(x=A, xs=A, w=A, ws=A, off=A, y=A, R=64, E=8, Kd=128, N=128, max_recv=0, elem=_lib.BF16):
        return lib.moe_a2a_expert_gemm_mx8(x, xs, w, ws, off, y, R, E, Kd, N, max_recv, elem, None)

    assert gemmx(elem=5) == E_DTYPE
    assert gemmx(N=192) == E_SHAPE
    assert gemmx(Kd=64) == E_SHAPE
    assert gemmx(xs=None) == E_NULL  # the rows are fp8: their scales are required
    assert gemmx(ws=None) == E_NULL
    assert gemmx(R=0) == 0
    assert gemmx(w=A + 8) == E_ALIGN
    assert gemm(Kd=72) == E_SHAPE    # hidden size in slabs of 64
    assert gemm8(Kd=192) == E_SHAPE  # fp8 rows carry one scale per 128 columns
    assert gemm8(sc=None) == E_NULL


def test_empty_world_never_reaches_a_kernel_that_reads_the_table(lib):
    """T == 0 goes to the kernel that only writes zero counts and offsets; the kernels that read
    `indices` are chosen for T >= 1 only.  (Host logic; the run on a GPU is in test_gpu_parity.py.)"""
    assert lib.moe_a2a_route_plan(0, 8) == b"route_empty"
    assert lib.moe_a2a_route_plan(0, 1) == b"route_empty"
    assert lib.moe_a2a_route_plan(1, 1) == b"route_tiles"
    assert lib.moe_a2a_route_plan(4096, 8) == b"route_tiles"
    assert lib.moe_a2a_route_plan(4097, 8) == b"route_hist"
    assert lib.moe_a2a_route_plan(-1, 8) == b"unknown"
    assert lib.moe_a2a_fused_ok(0, 8, 7168) == 0  # and the one-launch forms are never picked for it
    # T == 0 still needs somewhere to put the zeros, and takes NULL for everything else
    assert lib.moe_a2a_route(None, None, 0, 0, 8, 256, 8, 0, None, A, None, None, None, None, None, 0, None) == E_NULL
    assert lib.moe_a2a_route(None, None, 0, 0, 8, 256, 8, 0, A, None, None, None, None, None, None, 0, None) == E_NULL
    # the other row entry points return before any launch
    assert lib.moe_a2a_dispatch(None, None, None, 0, 8, 7168, None) == 0
    assert lib.moe_a2a_combine(None, None, None, 0, _lib.BF16, None, 0, 8, 7168, None) == 0
    assert lib.moe_a2a_stub_combine(None, None, None, None, None, 0, _lib.BF16, _lib.BF16, 0, 256, 8, None, 0, 8,
                                    7168, None) == 0
    assert lib.moe_a2a_stub(None, None, None, None, _lib.BF16, _lib.BF16, 0, 256, 8, None, 0, 7168, None) == 0


def test_option_switches(lib):
    n_options = _lib.OPT_FP8_TILE + 1  # the last one
    for opt in range(n_options):
        assert lib.moe_a2a_get_option(opt) == 0  # nothing is on unless a caller turns it on
    assert lib.moe_a2a_set_option(_lib.OPT_GEMM_TILE, 128) == 0
    assert lib.moe_a2a_get_option(_lib.OPT_GEMM_TILE) == 128
    assert lib.moe_a2a_set_option(_lib.OPT_GEMM_TILE, 0) == 128  # returns the previous value
    assert lib.moe_a2a_set_option(-1, 1) == E_DTYPE and lib.moe_a2a_set_option(n_options, 1) == E_DTYPE
    assert lib.moe_a2a_get_option(99) == E_DTYPE
    # no option takes a negative value, so a negative return always means an error
    assert lib.moe_a2a_set_option(_lib.OPT_GEMM_TILE, -3) == E_SHAPE
    assert lib.moe_a2a_get_option(_lib.OPT_GEMM_TILE) == 0


def test_library_reads_no_environment_variable():
    """The entry points take their switches from moe_a2a_set_option only."""
    src = os.path.join(ROOT, "kernel_amd", "csrc")
    for name in os.listdir(src):
        if name.endswith((".hip", ".inc", ".cpp")):
            assert "getenv" not in open(os.path.join(src, name)).read(), name


def test_gemm_rejects_padded_buffers_beyond_the_addressable_rows(lib):
    big = dict(E=1024, max_recv=1 << 20)
    assert lib.moe_a2a_expert_gemm(A, A, A, A, 64, big["E"], 128, 64, big["max_recv"], _lib.BF16, None) == E_SHAPE
    assert lib.moe_a2a_expert_gemm_fp8(A, A, A, A, A, 64, big["E"], 128, 64, big["max_recv"], _lib.BF16, None) == E_SHAPE
    assert lib.moe_a2a_expert_gemm_q8(A, None, A, A, A, A, 64, big["E"], 128, 128, big["max_recv"], _lib.BF16,
                                      None) == E_SHAPE
    assert lib.moe_a2a_expert_gemm_mx8(A, A, A, A, A, A, 64, big["E"], 128, 128, big["max_recv"], _lib.BF16,
                                       None) == E_SHAPE


def test_timer_needs_begin_first(lib):
    ids = (ctypes.c_int * 4)()
    us = (ctypes.c_float * 4)()
    assert lib.moe_a2a_timer_end(ids, us, 4) == E_STATE
    assert lib.moe_a2a_timer_skip(3) == E_STATE
    assert lib.moe_a2a_timer_begin(0) == E_STATE


def test_error_wrapper_raises_with_message(lib):
    with pytest.raises(_lib.MoeA2AError) as e:
        _lib.check(E_ALIGN, "moe_a2a_dispatch")
    assert "16-byte" in str(e.value) and e.value.code == E_ALIGN


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmoe_a2a.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_headers_are_plain_c_and_link_from_c(tmp_path):
    """The boundary is a C ABI: both headers compile as C99 with warnings on, and a C program links
    against the library and calls an entry point that touches no GPU."""
    import shutil
    import subprocess

    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "abi.c"
    src.write_text('#include "moe_a2a.h"\n#include "gemm_rs.h"\n'
                   "int main(void) { moe_a2a_forward_args a; (void)a;\n"
                   "  return (int)gemm_rs_workspace_bytes(0, 0, 0, 0) + moe_a2a_abi_version(); }\n")
    inc = os.path.join(ROOT, "include")
    lib_dir = os.path.dirname(_lib.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-I", inc, str(src)],
                   check=True)
    exe = tmp_path / "abi"
    subprocess.run(["gcc", "-std=c99", "-I", inc, str(src), "-o", str(exe), "-L", lib_dir, "-lmoe_a2a",
                    "-Wl,-rpath," + lib_dir], check=True)
    assert subprocess.run([str(exe)]).returncode == _lib.ABI_VERSION
