"""ctypes binding of libhexa_moe_hip.so (the C ABI in include/hexa_moe_hip.h).

The library is built in-tree by `make -C hexa-moe_amd/csrc` (or __graft_entry__.build()).  There is
no fallback: if it is missing, or an entry point returns an error code, a RuntimeError is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.normpath(os.path.join(_HERE, "..", "lib", "libhexa_moe_hip.so"))

HEXA_F32, HEXA_F16, HEXA_BF16 = 0, 1, 2
HEXA_W_IN_OUT, HEXA_W_OUT_IN = 0, 1
HEXA_ACT_NONE, HEXA_ACT_GELU, HEXA_ACT_GELU_BWD = 0, 1, 2
HEXA_TILE_ROWS = 128
HEXA_TILE_ROWS_L = 256
HEXA_ROUTE_UNIT = 512


def estmm_plan_ints(num_experts):
    """HEXA_ESTMM_PLAN_INTS of the header: ints of an ESTMM work plan (with the work queue's counters)."""
    return 4 * int(num_experts) + 32

_vp, _i, _i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64


class RouteLayout(ctypes.Structure):
    _fields_ = [("counts", _i64), ("offsets", _i64), ("token_ids", _i64), ("expert_ids", _i64),
                ("tile_count", _i64), ("tile_info", _i64), ("tile_count_l", _i64), ("tile_info_l", _i64),
                ("scratch", _i64), ("total_ints", _i64),
                ("mt_ub", ctypes.c_int32), ("mt_ub_l", ctypes.c_int32), ("units", ctypes.c_int32),
                ("reserved", ctypes.c_int32)]


class DepthDesc(ctypes.Structure):
    """hexa_moe_depth_desc of include/hexa_moe_hip.h."""
    _fields_ = [(n, ctypes.c_int32) for n in ("num_tokens", "top_k", "num_experts", "d_in", "hidden", "d_out", "act_dt",
                                              "w_dt", "b1_dt", "b2_dt", "gw1_dt", "gw2_dt", "gb1_dt", "gb2_dt", "loss")] + \
               [("noise_scale", ctypes.c_float), ("sigma", ctypes.c_float), ("reserved", ctypes.c_int32)]


# name -> (restype, argtypes); kept in one table so the export test can walk it
SIGNATURES = {
    "hexa_route_layout_get": (_i, [_i, _i, _i, ctypes.POINTER(RouteLayout)]),
    "hexa_route_build": (_i, [_vp, _i, _i64, _i64, _i, _i, _i, _vp, _vp]),
    "hexa_token_count": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "hexa_token_assign": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "hexa_route_from_lists": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "hexa_route_from_padded_lists": (_i, [_vp, _vp, _vp, _i64, _i, _i, _i, _vp, _vp]),
    "hexa_esmm": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "hexa_estmm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp]),
    "hexa_estmm_plan": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "hexa_ess": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _i64, _vp]),
    "hexa_ess_noalloc": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "hexa_fused_grad": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp,
                             _vp, _i, _vp, _vp, _i64, _vp]),
    "hexa_gelu_bwd": (_i, [_vp, _vp, _vp, _i64, _i, _vp]),
    "hexa_esmm_ess_ws_floats": (_i, [_i, _i, _i, _i, ctypes.POINTER(_i64)]),
    "hexa_esmm_gelu_bwd_ess": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _i64, _vp]),
    "hexa_gate_logits": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "hexa_gate_ws_floats": (_i, [_i, _i, _i, ctypes.POINTER(_i64)]),
    "hexa_gate_backward": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "hexa_router_ws_floats": (_i, [_i, _i, ctypes.POINTER(_i64)]),
    "hexa_router_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_float, _i, _i, _i, _vp, _vp]),
    "hexa_router_backward": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp]),
    "hexa_router_forward_load_importance": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_float,
                                                 ctypes.c_float, _i, _i, _i, _vp, _vp]),
    "hexa_router_backward_load_importance": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_float, _i, _i, _i, _vp]),
    "hexa_moe_depth_ws_bytes": (_i, [ctypes.POINTER(DepthDesc), ctypes.POINTER(_i64), ctypes.POINTER(_i64)]),
    "hexa_moe_depth_forward": (_i, [ctypes.POINTER(DepthDesc)] + [_vp] * 17 + [_vp, _i64, _vp, _i, _vp]),
    "hexa_moe_depth_backward": (_i, [ctypes.POINTER(DepthDesc)] + [_vp] * 21 + [_vp, _i64, _vp, _i, _vp]),
    "hexa_last_error": (ctypes.c_char_p, []),
    "hexa_abi_version": (_i, []),
    "hexa_set_option": (_i, [ctypes.c_char_p, _i]),
}

_lib = None


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"hexa_moe: {LIB_PATH} is missing. Build it with `make -C hexa-moe_amd/csrc` "
            "(hipcc, gfx950). There is no fallback implementation.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.hexa_abi_version() != 9:
        raise RuntimeError("hexa_moe: libhexa_moe_hip.so has an unexpected ABI version")
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().hexa_last_error()
        raise RuntimeError(f"{what} failed (code {rc}): {msg.decode() if msg else ''}")


def route_layout(T, k, E):
    L = RouteLayout()
    check(load().hexa_route_layout_get(int(T), int(k), int(E), ctypes.byref(L)), "hexa_route_layout_get")
    return L
