"""ctypes binding of libsthip.so — the only way Python reaches the HIP kernels.

There is no fallback: when the library has not been built, or no gfx950 device is usable, callers get
an exception, never a CPU result.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_size_t, c_uint16, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libsthip.so")

OK, ERR_NOT_ENABLED, ERR_INVALID, ERR_RUNTIME, ERR_NONFINITE, ERR_UNSUPPORTED = range(6)

c_float_p = POINTER(c_float)
c_u16_p = POINTER(c_uint16)


class DeviceProps(ctypes.Structure):
    _fields_ = [
        ("compute_units", c_int),
        ("clock_khz", c_int),
        ("memory_clock_khz", c_int),
        ("memory_bus_bits", c_int),
        ("wavefront_size", c_int),
        ("lds_bytes_per_block", c_int),
        ("l2_bytes", c_int),
        ("total_memory_bytes", c_uint64),
        ("arch", ctypes.c_char * 64),
    ]


class ProbeResult(ctypes.Structure):
    _fields_ = [("available", c_int), ("initialized", c_int), ("device_count", c_int), ("error", ctypes.c_char * 256)]


class AttentionPlan(ctypes.Structure):
    _fields_ = [("kernel", c_int), ("key_splits", c_int), ("keys_per_split", c_int), ("consistent", c_int),
                ("workgroups", c_uint64), ("items", c_uint64), ("items_expected", c_uint64), ("out_of_range", c_uint64),
                ("duplicates", c_uint64)]


class GemmTilePlan(ctypes.Structure):
    _fields_ = [("tile_cols", c_int), ("tiles_m", c_int), ("tiles_n", c_int), ("k_splits", c_int), ("k_tiles_per_split", c_int),
                ("consistent", c_int), ("workgroups", c_uint64), ("items", c_uint64), ("out_of_range", c_uint64),
                ("duplicates", c_uint64)]


class DecoderConfig(ctypes.Structure):
    _fields_ = [
        ("vocab", c_size_t),
        ("d_model", c_size_t),
        ("heads", c_size_t),
        ("layers", c_size_t),
        ("d_ff", c_size_t),
        ("batch", c_size_t),
        ("seq", c_size_t),
        ("ln_eps", c_float),
    ]


# name -> (restype, argtypes); this table is also what the symbol-export test walks.
SIGNATURES = {
    "st_hip_init": (c_int, []),
    "st_hip_real_backend_compiled": (c_int, []),
    "st_hip_device_count": (c_int, []),
    "st_hip_device_name": (c_int, [c_int, c_char_p, c_size_t]),
    "st_hip_device_properties": (c_int, [c_int, POINTER(DeviceProps)]),
    "st_hip_probe": (c_int, [POINTER(ProbeResult)]),
    "st_hip_last_error_message": (c_size_t, [c_char_p, c_size_t]),
    "st_hip_malloc": (c_int, [POINTER(c_void_p), c_size_t]),
    "st_hip_free": (c_int, [c_void_p]),
    "st_hip_memcpy_h2d": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "st_hip_memcpy_d2h": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "st_hip_memset_zero": (c_int, [c_void_p, c_size_t, c_void_p]),
    "st_hip_transfer_counters": (c_int, [POINTER(c_uint64), c_int]),
    "st_hip_stream_create": (c_int, [POINTER(c_void_p)]),
    "st_hip_stream_synchronize": (c_int, [c_void_p]),
    "st_hip_stream_destroy": (c_int, [c_void_p]),
    "st_hip_release_scratch": (c_int, [c_void_p]),
    "st_hip_scratch_buffer_count": (c_size_t, []),
    "st_hip_device_synchronize": (c_int, []),
    "st_hip_event_create": (c_int, [POINTER(c_void_p)]),
    "st_hip_event_record": (c_int, [c_void_p, c_void_p]),
    "st_hip_event_synchronize": (c_int, [c_void_p]),
    "st_hip_event_elapsed_ms": (c_int, [c_void_p, c_void_p, POINTER(c_float)]),
    "st_hip_event_destroy": (c_int, [c_void_p]),
    "st_hip_gemm_f32": (c_int, [c_size_t, c_size_t, c_size_t, c_float, c_int, c_void_p, c_size_t, c_void_p,
                                c_size_t, c_void_p, c_size_t]),
    "st_hip_gemm_f32_raw": (c_int, [c_size_t, c_size_t, c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_gemm_bias_act_f32": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_void_p, c_size_t, c_void_p,
                                         c_size_t, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_size_t]),
    "st_hip_gemm_bf16_f32acc": (c_int, [c_size_t, c_size_t, c_size_t, c_void_p, c_size_t, c_void_p, c_size_t,
                                        c_void_p, c_size_t]),
    "st_hip_conv2d_output_hw": (c_int, [c_size_t] * 10 + [POINTER(c_size_t), POINTER(c_size_t)]),
    "st_hip_conv2d_force_family": (c_int, [c_int]),
    "st_hip_conv2d_planned_kernel": (c_int, [c_size_t] * 13 + [c_int, POINTER(c_int)]),
    "st_hip_attention_f32_launch_plan": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_int, POINTER(AttentionPlan)]),
    "st_hip_gemm_row_block": (c_size_t, [c_size_t, c_size_t]),
    "st_hip_probe_mfma_bf16_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_probe_mfma_f32_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_probe_stream_lds_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_size_t, c_void_p]),
    "st_hip_gemm_bf16_tile_plan": (c_int, [c_size_t, c_size_t, c_size_t, POINTER(GemmTilePlan)]),
    "st_hip_conv2d_bias_act_f32": (c_int, [c_size_t] * 13 + [c_int, c_void_p, c_size_t, c_void_p, c_size_t,
                                                             c_void_p, c_size_t, c_void_p, c_size_t]),
    "st_hip_attention_f32": (c_int, [c_size_t, c_size_t, c_size_t, c_float, c_int, c_void_p, c_size_t, c_void_p,
                                     c_size_t, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_size_t,
                                     c_void_p, c_size_t]),
    "st_hip_gemm_f32_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_float, c_int, c_void_p, c_void_p, c_void_p,
                                    c_void_p]),
    "st_hip_gemm_bias_act_f32_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_void_p, c_void_p, c_void_p,
                                             c_void_p, c_void_p, c_void_p]),
    "st_hip_gemm_bf16_f32acc_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_gemm_bf16_bias_act_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_void_p, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_gemm_bf16_prepacked_bias_act_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_void_p, c_void_p,
                                                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_gemm_bf16_prepacked_residual_layer_norm_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_void_p, c_void_p, c_void_p,
                                                                    c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
                                                                    c_void_p]),
    "st_hip_pack_rhs_bf16_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_conv2d_bias_act_f32_dev": (c_int, [c_size_t] * 13 + [c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                                                 c_void_p]),
    "st_hip_conv2d_bias_act_bf16_dev": (c_int, [c_size_t] * 13 + [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                                  c_void_p]),
    "st_hip_attention_f32_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_float, c_int, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_attention_bf16_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_size_t, c_float, c_int, c_void_p, c_void_p,
                                          c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "st_hip_gemm_prepacked_bias_act_f32": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_void_p, c_size_t, c_void_p,
                                                   c_size_t, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p,
                                                   c_size_t]),
    "st_hip_gemm_prepacked_bias_act_f32_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_int, c_void_p, c_void_p,
                                                       c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_pack_rhs_f32_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_conv2d_backward_f32": (c_int, [c_size_t] * 13 + [c_void_p, c_size_t] * 6),
    "st_hip_conv2d_grad_input_f32_dev": (c_int, [c_size_t] * 13 + [c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_conv2d_grad_input_f32_noalloc_dev": (c_int, [c_size_t] * 13 + [c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_conv2d_grad_weight_f32_dev": (c_int, [c_size_t] * 13 + [c_void_p, c_void_p, c_float, c_void_p, c_void_p]),
    "st_hip_conv2d_grad_bias_f32_dev": (c_int, [c_size_t] * 13 + [c_void_p, c_float, c_void_p, c_void_p]),
    "st_hip_row_softmax_f32_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_gelu_f32_dev": (c_int, [c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_count_nonfinite_f32_dev": (c_int, [c_size_t, c_void_p, POINTER(c_uint64), POINTER(c_uint64),
                                               POINTER(c_float), c_void_p]),
    "st_hip_gelu_backward_f32_dev": (c_int, [c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_scale_f32_dev": (c_int, [c_size_t, c_void_p, c_float, c_void_p, c_void_p]),
    "st_hip_add_row_f32_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_sum_axis0_f32_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_float, c_void_p, c_void_p]),
    "st_hip_layer_norm_f32_dev": (c_int, [c_size_t, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                          c_void_p, c_void_p, c_void_p]),
    "st_hip_embedding_f32_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_f32_to_bf16_dev": (c_int, [c_size_t, c_void_p, c_void_p, c_void_p]),
    "st_hip_split_heads_f32_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_size_t, c_void_p, c_void_p, c_void_p,
                                           c_void_p, c_void_p]),
    "st_hip_merge_heads_f32_dev": (c_int, [c_size_t, c_size_t, c_size_t, c_size_t, c_void_p, c_void_p, c_void_p,
                                           c_void_p]),
    "st_hip_decoder_weight_count": (c_size_t, [POINTER(DecoderConfig)]),
    "st_hip_decoder_create": (c_int, [POINTER(DecoderConfig), c_void_p, c_size_t, POINTER(c_void_p)]),
    "st_hip_decoder_forward_dev": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "st_hip_decoder_destroy": (c_int, [c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Loads libsthip.so (once).  Raises OSError with a build hint when it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY_PATH):
        raise OSError(
            f"{LIBRARY_PATH} is missing: build it with `make -C spiraltorch_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no CPU fallback"
        )
    lib = ctypes.CDLL(LIBRARY_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error() -> str:
    lib = load()
    size = lib.st_hip_last_error_message(None, 0)
    buf = ctypes.create_string_buffer(size + 1)
    lib.st_hip_last_error_message(buf, size + 1)
    return buf.value.decode("utf-8", "replace")
