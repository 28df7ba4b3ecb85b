"""ctypes binding of the C ABI in include/kleos_amd.h. Loads the in-tree library; never falls back."""
from __future__ import annotations

import ctypes as C
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libkleos_amd.so")

KLEOS_OK, KLEOS_EINVAL, KLEOS_ESTATE, KLEOS_EUNSUPPORTED, KLEOS_EHIP, KLEOS_EIO, KLEOS_EPARSE = range(7)
DTYPE_FP32, DTYPE_TF32, DTYPE_BF16, DTYPE_FP16 = range(4)
ACT_RELU, ACT_GELU = 0, 1
MODE_FUSED, MODE_PHASED = 0, 1
SCHEDULE_AUTO, SCHEDULE_DYNAMIC, SCHEDULE_STATIC = 0, 1, 2


class KleosConfigStruct(C.Structure):
    """kleos_config_t"""
    _fields_ = [
        ("capacity_factor", C.c_double),
        ("drop_tokens", C.c_uint32), ("expert_top_k", C.c_uint32), ("global_batch", C.c_uint32),
        ("is_training", C.c_uint32), ("hidden_act", C.c_uint32), ("hidden_size", C.c_uint32),
        ("intermediate_size", C.c_uint32), ("mini_batch", C.c_uint32), ("moe_frequency", C.c_uint32),
        ("num_experts", C.c_uint32), ("num_layers", C.c_uint32), ("sequence_len", C.c_uint32),
        ("torch_dtype", C.c_uint32), ("vocab_size", C.c_uint32),
        ("S", C.c_uint32), ("H", C.c_uint32), ("I", C.c_uint32), ("E", C.c_uint32), ("k", C.c_uint32),
        ("PX", C.c_uint32), ("EC", C.c_uint32), ("pEC", C.c_uint32), ("cap_rows", C.c_uint32),
        ("elem_bytes", C.c_uint32),
        ("off_x", C.c_uint64), ("off_gate_w", C.c_uint64), ("off_w_up", C.c_uint64),
        ("off_w_down", C.c_uint64), ("off_b_up", C.c_uint64), ("off_b_down", C.c_uint64),
        ("in_elems", C.c_uint64),
        ("off_gate_out", C.c_uint64), ("off_moe_out", C.c_uint64), ("out_elems", C.c_uint64),
    ]


class DebugViewsStruct(C.Structure):
    """kleos_debug_views_t"""
    _fields_ = [(n, C.c_void_p) for n in
                ("logits", "topk_expert", "topk_prob", "combine_den", "topk_slot", "expert_count", "slot_token")]


# every symbol include/kleos_amd.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "kleos_config_parse_string": (C.c_int, [C.c_char_p, C.POINTER(KleosConfigStruct)]),
    "kleos_config_parse_file": (C.c_int, [C.c_char_p, C.POINTER(KleosConfigStruct)]),
    "kleos_config_defaults": (None, [C.POINTER(KleosConfigStruct)]),
    "kleos_config_derive": (C.c_int, [C.POINTER(KleosConfigStruct)]),
    "kleos_initialize": (C.c_int, [C.c_char_p]),
    "kleos_initialize_cfg": (C.c_int, [C.POINTER(KleosConfigStruct)]),
    "kleos_finalize": (C.c_int, []),
    "kleos_is_initialized": (C.c_int, []),
    "kleos_get_rank": (C.c_int, []),
    "kleos_set_device": (C.c_int, []),
    "kleos_get_config": (C.c_int, [C.POINTER(KleosConfigStruct)]),
    "kleos_moe_forward": (C.c_int, [C.c_void_p, C.c_void_p]),
    "kleos_moe_forward_dense": (C.c_int, [C.c_void_p, C.c_void_p]),
    "kleos_moe_forward_bench": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.POINTER(C.c_float)]),
    "kleos_moe_forward_static_scratch": (C.c_int, [C.POINTER(KleosConfigStruct), C.c_void_p, C.c_void_p, C.c_void_p]),
    "kleos_static_scratch_prepare": (C.c_int, [C.POINTER(KleosConfigStruct)]),
    "kleos_static_scratch_status": (C.c_int, [C.c_void_p]),
    "kleos_debug_static_scratch_expiry": (C.c_int, [C.c_ulonglong, C.c_uint32]),
    "kleos_debug_map_hip_error": (C.c_int, [C.c_int]),
    "kleos_debug_mfma_probe": (C.c_int, [C.c_int, C.c_uint32, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_double)]),
    "kleos_stream_synchronize": (C.c_int, []),
    "kleos_stream": (C.c_void_p, []),
    "kleos_set_mode": (C.c_int, [C.c_int]),
    "kleos_get_mode": (C.c_int, []),
    "kleos_set_schedule": (C.c_int, [C.c_int]),
    "kleos_get_schedule": (C.c_int, []),
    "kleos_set_cooperative_launch": (C.c_int, [C.c_int]),
    "kleos_schedule_taken": (C.c_int, [C.POINTER(C.c_int)]),
    "kleos_moe_debug_views": (C.c_int, [C.POINTER(DebugViewsStruct)]),
    "kleos_debug_copy_to_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "kleos_scheduler_stats": (C.c_int, [C.POINTER(C.c_double)]),
    "kleos_measure_throughput": (C.c_int, [C.c_uint32, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "kleos_measure_throughput_output": (C.c_int, [C.c_uint32, C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p,
                                                  C.c_size_t]),
    "kleos_debug_set_wait_ticks": (C.c_int, [C.c_ulonglong]),
    "kleos_debug_skip_launch_number": (C.c_int, []),
    "kleos_gate_loss": (C.c_int, [C.POINTER(C.c_float), C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "kleos_phase_stamps": (C.c_int, [C.POINTER(C.c_ulonglong), C.c_uint32, C.POINTER(C.c_uint32)]),
    "kleos_phase_times": (C.c_int, [C.POINTER(C.c_float)]),
    "kleos_last_error": (C.c_char_p, []),
}

_lib = None


class KleosError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"[kleos error {code}] {message}")
        self.code = code
        self.message = message


def lib() -> C.CDLL:
    """The loaded library. Raises if it has not been built: there is no other implementation."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m aristos_amd.build` (hipcc, gfx950). "
                "aristos_amd has no CPU or PyTorch fallback.")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code: int) -> None:
    if code != KLEOS_OK:
        raise KleosError(code, lib().kleos_last_error().decode("utf-8", "replace"))
