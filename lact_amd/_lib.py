"""ctypes binding of liblact_hip.so (the C ABI declared in include/lact_hip.h).

There is no fallback: if the library has not been built, every operation raises."""
import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int32, c_int64, c_size_t, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "liblact_hip.so")

LACT_BF16, LACT_F32 = 0, 1
LACT_UPDATE, LACT_APPLY = 0, 1


class Step(Structure):
    _fields_ = [("kind", c_int32), ("start", c_int32), ("end", c_int32), ("out_start", c_int32)]


class Desc(Structure):
    _fields_ = [
        ("b", c_int32), ("d", c_int32), ("dh", c_int32),
        ("q_len", c_int32), ("kv_len", c_int32), ("out_len", c_int32),
        ("act_dtype", c_int32),
        ("n_steps", c_int32),
        ("steps", POINTER(Step)),
        ("ns_steps", c_int32),
        ("ns_coeffs", POINTER(c_float)),
        ("use_momentum", c_int32), ("prenorm", c_int32), ("weight_norm", c_int32),
        ("detach_norms", c_int32), ("muon_replaces_weight", c_int32), ("ns_mode", c_int32),
        ("q_bs", c_int64), ("k_bs", c_int64), ("v_bs", c_int64), ("o_bs", c_int64), ("do_bs", c_int64),
        ("q_ld", c_int32), ("k_ld", c_int32), ("v_ld", c_int32), ("o_ld", c_int32), ("do_ld", c_int32),
        ("muon_stacked", c_int32), ("renorm_eps_in_sqrt", c_int32), ("forward_only", c_int32),
        ("momentum_state_in", c_int32),
    ]


OPT_STREAM_OVERLAP, OPT_FUSED_NEWTON_SCHULZ, OPT_NS_BARRIER_SPIN_LIMIT, OPT_PERSISTENT_TILES, OPT_KEEP_PREACTIVATIONS = 0, 1, 2, 3, 4
EXPORTS = ("lact_last_error", "lact_version", "lact_query_sizes", "lact_forward", "lact_forward_from_state", "lact_backward",
           "lact_newton_schulz_workspace_bytes", "lact_newton_schulz", "lact_newton_schulz_static_capacity",
           "lact_newton_schulz_static", "lact_newton_schulz_backward_workspace_bytes", "lact_newton_schulz_backward",
           "lact_check_async_error", "lact_mfma_calibration", "lact_set_option", "lact_profile_enable",
           "lact_profile_report", "lact_layer_pre_forward", "lact_layer_pre_backward", "lact_layer_lr_forward",
           "lact_layer_lr_backward", "lact_layer_post_forward", "lact_layer_post_dw_rows", "lact_layer_post_backward")

_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m lact_amd.build` (hipcc, gfx950). "
            "lact_amd has no CPU or PyTorch fallback.")
    L = ctypes.CDLL(LIB_PATH)
    L.lact_last_error.restype = c_char_p
    L.lact_version.restype = c_int32
    L.lact_query_sizes.argtypes = [POINTER(Desc), POINTER(c_size_t), POINTER(c_size_t)]
    L.lact_query_sizes.restype = c_int32
    vp = c_void_p
    L.lact_forward.argtypes = [POINTER(Desc)] + [vp] * 10 + [vp, POINTER(vp), POINTER(vp), vp, vp, vp]
    L.lact_forward.restype = c_int32
    L.lact_forward_from_state.argtypes = [POINTER(Desc)] + [vp] * 10 + [POINTER(vp), vp, POINTER(vp), POINTER(vp), vp, vp, vp]
    L.lact_forward_from_state.restype = c_int32
    L.lact_backward.argtypes = [POINTER(Desc)] + [vp] * 8 + [POINTER(vp), vp, vp] + [vp] * 10 + [vp]
    L.lact_backward.restype = c_int32
    L.lact_newton_schulz_workspace_bytes.argtypes = [c_int32] * 4
    L.lact_newton_schulz_workspace_bytes.restype = c_size_t
    L.lact_newton_schulz.argtypes = [c_int32, c_int32, c_int32, vp, vp, c_int32, POINTER(c_float), c_int32, vp, vp]
    L.lact_newton_schulz.restype = c_int32
    L.lact_newton_schulz_static_capacity.argtypes = []
    L.lact_newton_schulz_static_capacity.restype = c_size_t
    L.lact_newton_schulz_static.argtypes = [c_int32, c_int32, c_int32, vp, vp, c_int32, POINTER(c_float), c_int32, vp]
    L.lact_newton_schulz_static.restype = c_int32
    L.lact_newton_schulz_backward_workspace_bytes.argtypes = [c_int32] * 4
    L.lact_newton_schulz_backward_workspace_bytes.restype = c_size_t
    L.lact_newton_schulz_backward.argtypes = [c_int32, c_int32, c_int32, vp, vp, vp, c_int32, POINTER(c_float), c_int32, vp, vp]
    L.lact_newton_schulz_backward.restype = c_int32
    L.lact_mfma_calibration.argtypes = [c_int32, c_int32, vp, vp]
    L.lact_mfma_calibration.restype = c_int32
    L.lact_check_async_error.argtypes = []
    L.lact_check_async_error.restype = c_int32
    L.lact_set_option.argtypes = [c_int32, c_int32]
    L.lact_set_option.restype = c_int32
    i32, f32 = c_int32, c_float
    L.lact_layer_pre_forward.argtypes = [i32] * 6 + [vp] * 5
    L.lact_layer_pre_backward.argtypes = [i32] * 6 + [vp] * 6
    L.lact_layer_lr_forward.argtypes = [i32] * 4 + [f32] + [vp] * 7
    L.lact_layer_lr_backward.argtypes = [i32] * 4 + [f32] + [vp] * 9
    L.lact_layer_post_forward.argtypes = [i32] * 6 + [f32] + [vp] * 5
    L.lact_layer_post_dw_rows.argtypes = [i32] * 3
    L.lact_layer_post_backward.argtypes = [i32] * 6 + [f32] + [vp] * 8
    for fn in ("lact_layer_pre_forward", "lact_layer_pre_backward", "lact_layer_lr_forward", "lact_layer_lr_backward",
               "lact_layer_post_forward", "lact_layer_post_dw_rows", "lact_layer_post_backward"):
        getattr(L, fn).restype = c_int32
    L.lact_profile_enable.argtypes = [c_int32]
    L.lact_profile_enable.restype = c_int32
    L.lact_profile_report.argtypes = [c_char_p, c_size_t]
    L.lact_profile_report.restype = c_int32
    _lib = L
    return L


def check(rc: int):
    if rc != 0:
        raise RuntimeError("liblact_hip: " + lib().lact_last_error().decode())
