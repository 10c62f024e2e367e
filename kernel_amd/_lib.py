"""ctypes binding of ``libmoe_a2a.so`` (declared in include/moe_a2a.h).

There is no fallback: if the library is missing, ``load()`` raises.
"""
from __future__ import annotations

import ctypes as C
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmoe_a2a.so")

ABI_VERSION = 5
F16, BF16 = 0, 1
FP8_SCALE_F32, FP8_SCALE_POW2 = 0, 1
STATUS_BAD_EXPERT, STATUS_OVERFLOW = 1, 2  # bits of the routing status word
# option switches of moe_a2a_set_option (0 = the library decides)
(OPT_ROUTE_TILE, OPT_GEMM_TILE, OPT_GEMM_STAGED, OPT_COMBINE_LANES, OPT_COMBINE_VPL, OPT_TIMER_EVENT_FLAGS,
 OPT_COMBINE_PLAIN_MAP, OPT_TWO_LAUNCHES, OPT_FP8_TILE) = range(9)

_i32p = C.c_void_p  # device pointers travel as plain addresses
_vp = C.c_void_p
_int = C.c_int

# name -> (restype, argtypes); mirrors include/moe_a2a.h one to one
PROTOTYPES = {
    "moe_a2a_abi_version": (_int, []),
    "moe_a2a_strerror": (C.c_char_p, [_int]),
    "moe_a2a_workspace_bytes": (C.c_size_t, [_int, _int, _int]),
    "moe_a2a_route": (_int, [_i32p, _i32p, _int, _int, _int, _int, _int, _int, _i32p, _i32p, _i32p, _i32p, _i32p,
                             _i32p, _vp, C.c_size_t, _vp]),
    "moe_a2a_route_noalloc": (_int, [_i32p, _i32p, _int, _int, _int, _int, _int, _int, _i32p, _i32p, _i32p, _i32p,
                                     _i32p, _i32p, _vp]),
    "moe_a2a_route_noalloc_max_ints": (C.c_size_t, []),
    "moe_a2a_dispatch": (_int, [_vp, _i32p, _vp, _int, _int, _int, _vp]),
    "moe_a2a_fused_max_rows": (_int, []),
    "moe_a2a_fused_ok": (_int, [_int, _int, _int]),
    "moe_a2a_route_dispatch": (_int, [_vp, _i32p, _i32p, _int, _int, _int, _int, _int, _int, _int, _i32p, _i32p,
                                      _i32p, _i32p, _i32p, _i32p, _vp, _vp]),
    "moe_a2a_dispatch_fp8": (_int, [_vp, _int, _i32p, _vp, _vp, _int, _int, _int, _int, _vp]),
    "moe_a2a_stub": (_int, [_vp, _vp, _i32p, _i32p, _int, _int, _int, _int, _int, _vp, _int, _int, _vp]),
    "moe_a2a_combine": (_int, [_vp, _vp, _i32p, _int, _int, _vp, _int, _int, _int, _vp]),
    "moe_a2a_stub_combine": (_int, [_vp, _vp, _i32p, _vp, _i32p, _int, _int, _int, _int, _int, _int, _vp, _int, _int,
                                    _int, _vp]),
    "moe_a2a_forward": (_int, [_vp, _i32p, _vp, _i32p] + [_int] * 14 + [_i32p] * 6 + [_vp, _vp, _vp, _vp, _vp, C.c_size_t,
                                                                                      _vp]),
    "moe_a2a_forward_launches": (_int, [_int] * 9),
    "moe_a2a_expert_gemm": (_int, [_vp, _vp, _i32p, _vp, _int, _int, _int, _int, _int, _int, _vp]),
    "moe_a2a_expert_gemm_fp8": (_int, [_vp, _vp, _vp, _i32p, _vp, _int, _int, _int, _int, _int, _int, _vp]),
    "moe_a2a_expert_gemm_q8": (_int, [_vp, _vp, _vp, _vp, _i32p, _vp, _int, _int, _int, _int, _int, _int, _vp]),
    "moe_a2a_expert_gemm_mx8": (_int, [_vp, _vp, _vp, _vp, _i32p, _vp, _int, _int, _int, _int, _int, _int, _vp]),
    "moe_a2a_route_plan": (C.c_char_p, [_int, _int]),
    "moe_a2a_set_option": (_int, [_int, _int]),
    "moe_a2a_get_option": (_int, [_int]),
    "moe_a2a_timer_begin": (_int, [_int]),
    "moe_a2a_timer_skip": (_int, [_int]),
    "moe_a2a_timer_end": (_int, [C.POINTER(C.c_int), C.POINTER(C.c_float), _int]),
    "moe_a2a_kernel_name": (C.c_char_p, [_int]),
}



class ForwardArgs(C.Structure):
    """``moe_a2a_forward_args`` of include/moe_a2a.h."""
    _fields_ = ([(n, C.c_void_p) for n in ("x", "indices", "weights", "rank_start")] +
                [(n, C.c_int) for n in ("src_rank", "T", "K", "E", "W", "H", "max_recv", "in_type", "out_type",
                                        "fp8_dispatch", "stub_kind", "combine_mode", "fuse_route", "fuse_stub")] +
                [(n, C.c_void_p) for n in ("counts", "offsets", "slot_of_entry", "src_of_slot", "meta", "status", "disp",
                                           "disp_scale", "expert_y", "out", "workspace")] +
                [("workspace_bytes", C.c_size_t), ("stream", C.c_void_p), ("clear_status", C.c_void_p)])


PROTOTYPES["moe_a2a_forward_packed"] = (_int, [C.POINTER(ForwardArgs)])

# include/gemm_rs.h (same library)
GEMM_RS_PROTOTYPES = {
    "gemm_rs_workspace_bytes": (C.c_size_t, [_int, _int, _int, _int]),
    "gemm_rs_forward": (_int, [_vp, _vp, _vp, _vp, _int, _int, _int, _int, C.c_longlong, C.c_longlong, _int, _vp,
                               C.c_size_t, _vp]),
}

_lib = None


class MoeA2AError(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        msg = load().moe_a2a_strerror(code)
        super().__init__(f"{where}: {msg.decode() if msg else 'error'} (code {code})")


def load() -> C.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m kernel_amd.build` (there is no fallback path)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in list(PROTOTYPES.items()) + list(GEMM_RS_PROTOTYPES.items()):
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    got = lib.moe_a2a_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"libmoe_a2a.so has ABI {got}, binding expects {ABI_VERSION}")
    _lib = lib
    return lib


def check(code: int, where: str) -> None:
    if code != 0:
        raise MoeA2AError(code, where)
