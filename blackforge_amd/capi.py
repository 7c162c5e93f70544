"""ctypes binding of the C ABI in include/bf_hip.h (blackforge_amd/lib/libbf_hip.so).

There is no fallback: if the library is missing or a call fails, an exception is raised.
``BF_ERR_INVALID_ARGUMENT`` maps to ``ValueError`` (the reference throws std::invalid_argument),
everything else to ``RuntimeError`` (std::runtime_error).
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libbf_hip.so")

OK, ERR_INVALID_ARGUMENT, ERR_RUNTIME, ERR_UNSUPPORTED = 0, 1, 2, 3
ACT_SILU, ACT_GELU, ACT_RELU = 0, 1, 2

c_size = ctypes.c_size_t
c_ptr = ctypes.c_void_p
c_int = ctypes.c_int
c_float = ctypes.c_float
c_ll = ctypes.c_longlong


class DeviceProps(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 32), ("compute_units", c_int),
                ("clock_khz", c_int), ("wavefront_size", c_int), ("lds_bytes_per_block", c_int),
                ("total_memory", c_size)]


class PoolStats(ctypes.Structure):
    _fields_ = [("bytes_from_driver", c_size), ("bytes_in_use", c_size), ("driver_allocations", c_size),
                ("acquires", c_size)]


class GemmF32Problem(ctypes.Structure):
    """bf_gemm_f32_problem: one member of a bf_hip_gemm_f32_group call."""
    _fields_ = [("A", c_ptr), ("B", c_ptr), ("C", c_ptr), ("bias", c_ptr), ("residual", c_ptr),
                ("M", c_size), ("N", c_size), ("K", c_size), ("transA", ctypes.c_int), ("transB", ctypes.c_int)]


P = c_ptr  # device pointer
S = c_ptr  # stream

# name -> argument types (every function returns int status unless listed in _SPECIAL)
SIGNATURES = {
    "bf_hip_device_count": [ctypes.POINTER(c_int)],
    "bf_hip_device_props": [c_int, ctypes.POINTER(DeviceProps)],
    "bf_hip_set_device": [c_int],
    "bf_hip_get_device": [ctypes.POINTER(c_int)],
    "bf_hip_synchronize": [],
    "bf_hip_stream_create": [ctypes.POINTER(c_ptr)],
    "bf_hip_stream_destroy": [S],
    "bf_hip_stream_synchronize": [S],
    "bf_hip_event_create": [ctypes.POINTER(c_ptr)],
    "bf_hip_event_destroy": [c_ptr],
    "bf_hip_event_record": [c_ptr, S],
    "bf_hip_event_synchronize": [c_ptr],
    "bf_hip_event_elapsed_ms": [c_ptr, c_ptr, ctypes.POINTER(c_float)],
    "bf_hip_pool_acquire": [c_size, ctypes.POINTER(c_ptr)],
    "bf_hip_pool_release": [P, c_size],
    "bf_hip_pool_stats": [ctypes.POINTER(PoolStats)],
    "bf_hip_pool_trim": [],
    "bf_hip_memcpy_h2d": [P, c_ptr, c_size],
    "bf_hip_memcpy_d2h": [c_ptr, P, c_size],
    "bf_hip_memcpy_d2d": [P, P, c_size, S],
    "bf_hip_capture_begin": [S],
    "bf_hip_capture_end": [ctypes.POINTER(c_ptr)],
    "bf_hip_graph_launch": [c_ptr, S],
    "bf_hip_graph_destroy": [c_ptr],
    "bf_hip_fill_zero": [P, c_size, S],
    "bf_hip_add": [P, P, P, c_size, S],
    "bf_hip_scale": [P, c_float, P, c_size, S],
    "bf_hip_add_bias": [P, P, P, c_size, c_size, S],
    "bf_hip_add_bias_act": [P, P, P, c_size, c_size, c_int, S],
    "bf_hip_add_bias_residual": [P, P, P, P, c_size, c_size, S],
    "bf_hip_act_forward": [P, P, c_size, c_int, S],
    "bf_hip_act_backward": [P, P, P, c_size, c_int, S],
    "bf_hip_add_bias_act_backward": [P, P, P, P, P, c_size, c_size, c_int, S],
    "bf_hip_accumulate": [P, P, c_size, S],
    "bf_hip_zero_multi": [ctypes.POINTER(c_ptr), ctypes.POINTER(c_size), c_size, S],
    "bf_hip_rmsnorm": [P, P, c_size, c_size, S],
    "bf_hip_rmsnorm_backward": [P, P, P, c_size, c_size, S],
    "bf_hip_rmsnorm_backward_add": [P, P, P, P, c_size, c_size, S],
    "bf_hip_rmsnorm_img": [P, P, P, c_size, c_size, S],
    "bf_hip_rmsnorm_backward_add_img": [P, P, P, P, P, c_size, c_size, S],
    "bf_hip_softmax": [P, P, c_size, c_size, S],
    "bf_hip_softmax_backward": [P, P, P, c_size, c_size, S],
    "bf_hip_bias_grad": [P, P, c_size, c_size, S],
    "bf_hip_bias_grad_static": [P, P, c_size, c_size, S],
    "bf_hip_count_out_of_range": [P, c_size, c_size, ctypes.POINTER(c_size), ctypes.POINTER(c_ll), S],
    "bf_hip_embedding_forward": [P, P, P, c_size, c_size, c_size, S],
    "bf_hip_embedding_backward": [P, P, P, c_size, c_size, c_size, S],
    "bf_hip_positional_forward": [P, P, P, c_size, c_size, c_size, c_size, c_size, S],
    "bf_hip_positional_backward": [P, P, c_size, c_size, c_size, c_size, S],
    "bf_hip_concat_seq": [P, P, P, c_size, c_size, c_size, c_size, S],
    "bf_hip_argmax_last_position": [P, c_size, c_size, ctypes.POINTER(c_ll), S],
    "bf_hip_gemm_f32": [c_int, c_int, P, P, P, c_size, c_size, c_size, S],
    "bf_hip_gemm_f32_adds": [c_int, c_int, P, P, P, P, P, c_size, c_size, c_size, S],
    "bf_hip_gemm_f32_group": [ctypes.POINTER(GemmF32Problem), c_size, S],
    "bf_hip_cvt_f32_bf16": [P, P, c_size, S],
    "bf_hip_cvt_f32_bf16_transpose": [P, P, c_size, c_size, S],
    "bf_hip_gemm_bf16_nt": [P, P, P, c_size, c_size, c_size, S],
    "bf_hip_gemm_bf16_tn": [P, P, P, c_size, c_size, c_size, S],
    "bf_hip_matmul_bf16": [P, P, P, c_size, c_size, c_size, c_int, S],
    "bf_hip_matmul_bf16_backward": [P, P, P, P, P, c_size, c_size, c_size, c_int, S],
    "bf_hip_linear_bf16": [P, P, P, P, P, c_size, c_size, c_size, c_int, S],
    "bf_hip_matmul_bf16_shared_input": [P, ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), c_size, c_size, c_size, c_size, c_int, S],
    "bf_hip_matmul_bf16_shared_input_backward": [P, ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), P, ctypes.POINTER(c_ptr), c_size,
                                                 c_size, c_size, c_size, c_int, S],
    "bf_hip_feedforward_bf16": [P, P, P, P, P, P, c_int, P, P, P, P, c_size, c_size, c_size, c_int, S],
    "bf_hip_feedforward_bf16_backward": [P, P, P, P, P, P, P, c_int, P, P, P, P, P, c_size, c_size, c_size, c_int, S],
    "bf_hip_linear_bf16_img": [P, P, P, P, P, P, c_size, c_size, c_size, c_int, S],
    "bf_hip_matmul_bf16_backward_img": [P, P, P, P, P, P, P, c_size, c_size, c_size, c_int, S],
    "bf_hip_matmul_bf16_shared_input_img": [P, P, ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), c_size, c_size, c_size, c_size, c_int, S],
    "bf_hip_matmul_bf16_shared_input_backward_img": [P, P, ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), P, P, ctypes.POINTER(c_ptr), c_size,
                                                     c_size, c_size, c_size, c_int, S],
    "bf_hip_feedforward_bf16_backward_img": [P, P, P, P, P, P, P, P, c_int, P, P, P, P, P, c_size, c_size, c_size, c_int, S],
    "bf_hip_invalidate_bf16_weight_cache": [],
    "bf_hip_bf16_weight_cache_refresh": [ctypes.POINTER(c_ptr), c_size, S],
    "bf_hip_gemm_bf16_set_route": [c_int],
    "bf_hip_mfma_only_loop": [P, P, c_int, c_int, c_int, S],
    "bf_hip_attention_forward": [P, P, P, P, P, P, c_size, c_size, c_size, c_size, c_size, c_float, c_size, S],
    "bf_hip_attention_forward_img": [P, P, P, P, P, c_size, P, P, c_size, c_size, c_size, c_size, c_size, c_float, c_size, S],
    "bf_hip_attention_forward_rows": [P, P, P, P, P, c_size, P, P, c_size, c_size, c_size, c_size, c_size, c_size, c_float, c_size, S],
    "bf_hip_copy_pitched": [P, c_size, P, c_size, c_size, c_size, S],
    "bf_hip_positional_forward_indirect": [P, P, P, c_size, c_size, c_size, c_size, P, S],
    "bf_hip_kv_append": [P, P, P, P, c_size, c_size, c_size, c_size, c_size, S],
    "bf_hip_kv_append_indirect": [P, P, P, P, c_size, c_size, c_size, c_size, P, S],
    "bf_hip_attention_forward_rows_indirect": [P, P, P, P, P, c_size, P, P, c_size, c_size, c_size, c_size, c_size, c_float, P, S],
    "bf_hip_argmax_last_position_device": [P, c_size, c_size, P, P, c_size, P, ctypes.c_int, ctypes.c_longlong, S],
    "bf_hip_counter_add": [P, ctypes.c_int, S],
    "bf_hip_rmsnorm_matmul_bf16_shared_input": [P, ctypes.POINTER(P), ctypes.POINTER(P), c_size, c_size, c_size, c_size, ctypes.c_int, S],
    "bf_hip_decode_projections_bf16": [P, P, P, P, P, P, P, c_size, c_size, c_size, c_size, P, ctypes.c_int, S],
    "bf_hip_decode_projections_f32": [P, P, P, P, P, P, P, c_size, c_size, c_size, c_size, P, S],
    "bf_hip_rmsnorm_matmul_f32_shared_input": [P, ctypes.POINTER(P), ctypes.POINTER(P), c_size, c_size, c_size, c_size, S],
    "bf_hip_rmsnorm_feedforward_f32": [P, P, P, P, P, ctypes.c_int, P, c_size, c_size, c_size, S],
    "bf_hip_rmsnorm_feedforward_bf16": [P, P, P, P, P, ctypes.c_int, P, c_size, c_size, c_size, ctypes.c_int, S],
    "bf_hip_attention_backward_img": [P, P, P, P, P, P, P, P, P, P, P, P, P, c_size, c_size, c_size, c_size, c_size, c_size, c_float,
                                      c_size, S],
    "bf_hip_attention_dot_o_do": [P, P, P, c_size, c_size, c_size, c_size, S],
    "bf_hip_attention_backward": [P, P, P, P, P, P, P, P, P, P, c_size, c_size, c_size, c_size, c_size, c_float,
                                  c_size, S],
    "bf_hip_attention_backward_prepare": [P, P, P, P, P, P, c_size, c_size, c_size, c_size, S],
    "bf_hip_attention_backward_dkv": [P, P, P, P, P, P, P, P, c_size, c_size, c_size, c_size, c_size, c_float, c_size, S],
    "bf_hip_attention_backward_dq": [P, P, P, P, P, P, P, c_size, c_size, c_size, c_size, c_size, c_float, c_size, S],
    "bf_hip_attention_ds_bytes": [c_size, c_size, c_size, c_size, ctypes.POINTER(c_size)],
    "bf_hip_attention_set_workspace_limit": [c_size],
    "bf_hip_attention_set_route": [c_int],
    "bf_hip_attention_backward_dkv_ds": [P, P, P, P, P, P, P, P, P, c_size, c_size, c_size, c_size, c_size, c_float, c_size, S],
    "bf_hip_attention_backward_dq_from_ds": [P, P, P, c_size, c_size, c_size, c_size, c_size, c_float, c_size, S],
    "bf_hip_mse": [P, P, P, P, c_size, c_int, S],
    "bf_hip_mse_img": [P, P, P, P, P, c_size, c_int, S],
    "bf_hip_cross_entropy": [P, P, P, P, c_size, c_size, c_int, S],
    "bf_hip_cross_entropy_sparse": [P, P, P, P, c_size, c_size, c_int, S],
    "bf_hip_cross_entropy_sparse_img": [P, P, P, P, P, c_size, c_size, c_int, S],
    "bf_hip_cross_entropy_sparse_head": [P, P, P, P, P, c_size, c_size, c_int, S],
    "bf_hip_cross_entropy_masked": [P, P, P, P, c_size, c_size, c_int, S],
    "bf_hip_sgd_publish": [P, c_float, S],
    "bf_hip_sgd_multi_indirect": [ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), ctypes.POINTER(c_size), c_size, P, S],
    "bf_hip_adamw_publish": [P, c_ll, c_float, c_float, c_float, c_float, c_float, S],
    "bf_hip_adamw_multi_indirect": [ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr),
                                    ctypes.POINTER(c_size), c_size, P, S],
    "bf_hip_sgd_multi": [ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), ctypes.POINTER(c_size), c_size, c_float, S],
    "bf_hip_adamw_multi": [ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr), ctypes.POINTER(c_ptr),
                           ctypes.POINTER(c_size), c_size, c_ll, c_float, c_float, c_float, c_float, c_float, S],
}
_SPECIAL = {"bf_hip_last_error": ctypes.c_char_p, "bf_hip_version": ctypes.c_char_p}

_lib = None


def load() -> ctypes.CDLL:
    """Loads the shipped library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                           "(there is no CPU fallback for the HIP operator library)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if a declared entry point is not exported
        fn.argtypes = argtypes
        fn.restype = c_int
    for name, restype in _SPECIAL.items():
        fn = getattr(lib, name)
        fn.argtypes = []
        fn.restype = restype
    _lib = lib
    return lib


def last_error() -> str:
    return load().bf_hip_last_error().decode(errors="replace")


def check(status: int, name: str = "") -> None:
    if status == OK:
        return
    message = last_error() or f"{name} failed with status {status}"
    if status == ERR_INVALID_ARGUMENT:
        raise ValueError(message)
    raise RuntimeError(message)


def call(name: str, *args) -> None:
    check(getattr(load(), name)(*args), name)


def device_count() -> int:
    n = c_int(0)
    call("bf_hip_device_count", ctypes.byref(n))
    return n.value


def device_props(index: int = 0) -> DeviceProps:
    props = DeviceProps()
    call("bf_hip_device_props", index, ctypes.byref(props))
    return props
