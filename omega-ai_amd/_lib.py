"""Loads libomega_hip.so and declares the C ABI of include/omega_hip.h for ctypes.

There is no CPU fallback: if the shared library is missing, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libomega_hip.so")

OK, ERR_INVALID_ARG, ERR_OOM, ERR_HIP, ERR_UNSUPPORTED = range(5)
DTYPE_F32, DTYPE_BF16 = 0, 1
ROUTER_EXACT, ROUTER_FAST = 0, 1
W_GATE, W_GATE_BIAS, W_W1, W_W3, W_W2, W_NORM = range(6)
(STAGE_ROUTER, STAGE_DISPATCH, STAGE_UP, STAGE_DOWN, STAGE_COMBINE, STAGE_FORWARD, STAGE_INDEX, STAGE_GATHER,
 STAGE_FORWARD_BLOCK, STAGE_RMS) = range(10)


class MoEConfigStruct(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("T_max", "d", "E", "K", "H", "Es", "renorm", "has_gate_bias", "dtype", "router_mode")]


# name -> (restype, argtypes); every symbol include/omega_hip.h declares
SIGNATURES = {
    "omega_hip_version": (C.c_int, []),
    "omega_hip_ctx_create": (C.c_int, [C.c_int, C.POINTER(C.c_void_p)]),
    "omega_hip_ctx_destroy": (C.c_int, [C.c_void_p]),
    "omega_hip_last_error": (C.c_char_p, [C.c_void_p]),
    "omega_hip_malloc": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "omega_hip_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "omega_hip_memcpy_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "omega_hip_memcpy_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "omega_hip_memset": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t]),
    "omega_hip_sync": (C.c_int, [C.c_void_p]),
    "omega_hip_fill_normal": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_double,
                                        C.c_uint64, C.c_int]),
    "omega_hip_convert": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_uint64]),
    "omega_moe_create": (C.c_int, [C.c_void_p, C.POINTER(MoEConfigStruct), C.POINTER(C.c_void_p)]),
    "omega_moe_destroy": (C.c_int, [C.c_void_p]),
    "omega_moe_set_weights": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int]),
    "omega_moe_get_weights": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int]),
    "omega_moe_forward": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "omega_moe_forward_block": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "omega_moe_get_norm": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "omega_moe_backward": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "omega_moe_time_backward": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int,
                                          C.POINTER(C.c_float)]),
    "omega_moe_backward_block": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "omega_jrandom_seed": (None, [C.c_void_p, C.c_int64]),
    "omega_jrandom_next_int": (C.c_int32, [C.c_void_p]),
    "omega_jrandom_next_double": (C.c_double, [C.c_void_p]),
    "omega_jrandom_next_gaussian": (C.c_double, [C.c_void_p]),
    "omega_jrandom_normal": (None, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float, C.c_float]),
    "omega_moe_set_training": (C.c_int, [C.c_void_p, C.c_int]),
    "omega_moe_set_gather_mode": (C.c_int, [C.c_void_p, C.c_int]),
    "omega_moe_gather_on_load": (C.c_int, [C.c_void_p]),
    "omega_moe_get_grad": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int]),
    "omega_moe_acc_grad": (C.c_int, [C.c_void_p, C.c_float]),
    "omega_moe_update_adamw": (C.c_int, [C.c_void_p, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int]),
    "omega_moe_grad_sumsq": (C.c_int, [C.c_void_p, C.POINTER(C.c_float)]),
    "omega_moe_scale_grad": (C.c_int, [C.c_void_p, C.c_float]),
    "omega_moe_update": (C.c_int, [C.c_void_p, C.c_float]),
    "omega_moe_router": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "omega_moe_dispatch": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "omega_moe_experts": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "omega_moe_experts_up": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "omega_moe_experts_down": (C.c_int, [C.c_void_p, C.c_int]),
    "omega_moe_combine": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p]),
    "omega_moe_get_routing": (C.c_int, [C.c_void_p, C.c_int] + [C.c_void_p] * 6),
    "omega_moe_get_router_probs": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "omega_moe_get_router_probs_noalloc": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]),
    "omega_moe_get_workspace": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "omega_moe_fill_workspace": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "omega_moe_time_stage": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int,
                                       C.POINTER(C.c_float)]),
    "omega_moe_set_profiling": (C.c_int, [C.c_void_p, C.c_int]),
    "omega_moe_get_profile": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_int)]),
}

_lib = None


def load_library():
    """Returns the loaded library; raises if it has not been built (there is no other code path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(or __graft_entry__.build()); there is no CPU fallback")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
