"""ctypes binding of librbmoe.so — the declarations of include/rbmoe.h.

Loading fails loudly when the library has not been built; nothing here falls
back to a CPU implementation.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librbmoe.so")

# rbmoe_status
OK, INVALID_INPUT, INVALID_CONFIG, DEVICE_ERROR, BACKEND_UNAVAILABLE, MEMORY_BUDGET, OUT_OF_MEMORY, \
    UNSUPPORTED, NULL_POINTER = range(9)
# rbmoe_dtype
F32, BF16, I8 = 0, 1, 2
DTYPES = {"f32": F32, "bf16": BF16, "int8": I8}
# rbmoe_weight
W_ROUTER, W_GATE, W_UP, W_DOWN, W_SHARED_GATE, W_SHARED_UP, W_SHARED_DOWN, W_NORM = range(8)
# rbmoe_option
(OPT_FORCE_GENERIC, OPT_EXPLICIT_GATHER, OPT_GROUP_M, OPT_DECODE_PATH, OPT_DECODE_FRONT, OPT_FUSED_ROUTER,
 OPT_SIDE_STREAM, OPT_WGRAD_MODE, OPT_WGRAD_GENERIC, OPT_DECODE_COMBINE_FOLD, OPT_QUANT_RULE,
 OPT_QUANTIZE_ROUTER, OPT_DECODE_DOWN_BY_EXPERT) = range(13)
NUM_STAGES = 8
STATIC_SCRATCH_BYTES = 8 << 20
STAGE_NAMES = ("router", "empty", "dispatch", "gate_up", "down", "shared", "combine", "total")


class Config(C.Structure):
    _fields_ = [("d_model", C.c_int32), ("num_experts", C.c_int32), ("experts_per_token", C.c_int32),
                ("d_ff", C.c_int32), ("shared_expert", C.c_int32), ("shared_d_ff", C.c_int32),
                ("aux_loss_weight", C.c_float), ("router_z_loss_weight", C.c_float),
                ("weight_dtype", C.c_int32), ("act_dtype", C.c_int32), ("max_tokens", C.c_int32)]


class Routing(C.Structure):
    _fields_ = [("expert_of", C.POINTER(C.c_int32)), ("gate_of", C.POINTER(C.c_float)),
                ("counts", C.POINTER(C.c_int32)), ("offsets", C.POINTER(C.c_int32)),
                ("perm_slot", C.POINTER(C.c_int32)), ("perm_token", C.POINTER(C.c_int32)),
                ("probabilities", C.POINTER(C.c_float)), ("log_sum_exp", C.POINTER(C.c_float))]


# Every symbol include/rbmoe.h declares, with its signature.
SIGNATURES = {
    "rbmoe_config_init": (C.c_int, [C.POINTER(Config), C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "rbmoe_validate": (C.c_int, [C.POINTER(Config), C.c_char_p, C.c_size_t]),
    "rbmoe_parameter_counts": (C.c_int, [C.POINTER(Config), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "rbmoe_ctx_create": (C.c_int, [C.c_int32, C.c_size_t, C.POINTER(C.c_void_p)]),
    "rbmoe_ctx_destroy": (None, [C.c_void_p]),
    "rbmoe_ctx_set_stream": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rbmoe_synchronize": (C.c_int, [C.c_void_p]),
    "rbmoe_last_error": (C.c_char_p, [C.c_void_p]),
    "rbmoe_last_global_error": (C.c_char_p, []),
    "rbmoe_layer_create": (C.c_int, [C.c_void_p, C.POINTER(Config), C.POINTER(C.c_void_p)]),
    "rbmoe_layer_destroy": (None, [C.c_void_p]),
    "rbmoe_layer_set_option": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32]),
    "rbmoe_set_weight": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_int32,
                                   C.POINTER(C.c_float), C.c_int32, C.c_int32]),
    "rbmoe_forward": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                C.c_void_p, C.c_void_p]),
    "rbmoe_forward_static": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.c_void_p]),
    "rbmoe_forward_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                     C.c_void_p, C.c_void_p]),
    "rbmoe_forward_timed": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "rbmoe_get_losses": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "rbmoe_get_routing": (C.c_int, [C.c_void_p, C.POINTER(Routing)]),
    "rbmoe_get_expert_rows": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "rbmoe_expert_kernel_name": (C.c_char_p, [C.c_void_p]),
    "rbmoe_device_alloc": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "rbmoe_device_free": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rbmoe_copy_to_device": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "rbmoe_copy_to_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "rbmoe_copy_device": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "rbmoe_set_feed_forward_norm": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.c_int32, C.c_float]),
    "rbmoe_forward_block": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "rbmoe_forward_block_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                           C.c_void_p]),
    "rbmoe_layer_enable_training": (C.c_int, [C.c_void_p]),
    "rbmoe_backward": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "rbmoe_backward_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "rbmoe_backward_block": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "rbmoe_backward_block_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "rbmoe_zero_grads": (C.c_int, [C.c_void_p]),
    "rbmoe_get_weight_grad": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_float), C.c_int32, C.c_int32]),
    "rbmoe_forward_kernel_times": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                             C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "rbmoe_replay_stage": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_float)]),
    "rbmoe_version": (C.c_char_p, []),
}

_lib = None


def load() -> C.CDLL:
    """Load librbmoe.so; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m rustingbrain_amd.build` "
            "(hipcc, --offload-arch=gfx950). There is no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


# include/rbmoe_bench.h: the benchmark's measurement helpers, a library of their own
BENCH_LIB_PATH = os.path.join(_HERE, "librbmoe_bench.so")
BENCH_SIGNATURES = {
    "rbbench_stream_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "rbbench_stream_destroy": (C.c_int, [C.c_void_p]),
    "rbbench_timer_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "rbbench_timer_start": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rbbench_timer_stop": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "rbbench_timer_destroy": (None, [C.c_void_p]),
    "rbbench_flush_create": (C.c_int, [C.c_size_t, C.POINTER(C.c_void_p)]),
    "rbbench_flush": (C.c_int, [C.c_void_p, C.c_void_p]),
    "rbbench_flush_destroy": (None, [C.c_void_p]),
    "rbbench_mfma_only": (C.c_int, [C.c_void_p, C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "rbbench_read": (C.c_int, [C.c_void_p, C.c_size_t, C.c_int32, C.c_void_p, C.POINTER(C.c_double),
                               C.POINTER(C.c_double)]),
}
_bench_lib = None


def load_bench() -> C.CDLL:
    """Load librbmoe_bench.so (the benchmark's helpers); raises if it has not been built."""
    global _bench_lib
    if _bench_lib is not None:
        return _bench_lib
    if not os.path.exists(BENCH_LIB_PATH):
        raise ImportError(f"{BENCH_LIB_PATH} is missing: build it with `python -m rustingbrain_amd.build`")
    lib = C.CDLL(BENCH_LIB_PATH)
    for name, (restype, argtypes) in BENCH_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _bench_lib = lib
    return lib
