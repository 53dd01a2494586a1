"""ctypes binding of ``csrc/liba81w41.so`` (the C ABI in ``include/a81w41.h``).

The library is loaded from the source tree; if it has not been built the call
fails with instructions -- there is no fallback path.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "liba81w41.so")

OK = 0
_vp, _i, _i64, _sz = C.c_void_p, C.c_int, C.c_int64, C.c_size_t

# name -> (restype, argtypes): every symbol include/a81w41.h declares
SIGNATURES = {
    "a81w41_status_string": (C.c_char_p, [_i]),
    "a81w41_last_error": (C.c_char_p, []),
    "a81w41_weight_blob_bytes": (_sz, [_i, _i, _i]),
    "a81w41_act_blob_bytes": (_sz, [_i64, _i]),
    "a81w41_repack_w81_weight_fp16": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp]),
    "a81w41_repack_w81_weight_fp32": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp]),
    "a81w41_quantize_weight_q41": (_i, [_vp, _i, _i, _vp, _vp, _vp]),
    "a81w41_quantize_row_q8_1_repack_fp16": (_i, [_vp, _vp, _i64, _vp]),
    "a81w41_quantize_row_q8_1_repack_fp32": (_i, [_vp, _vp, _i64, _vp]),
    "a81w41_gemv_repack_A81W41_fp16": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "a81w41_gemm_repack_A81W41_fp32": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "a81w41_gemm_repack_A81W41_fp32_static": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "a81w41_gemm_schedule_selfcheck": (_i, [_i, _i, _i, _i, _i]),
    "a81w41_gemm_fp6_plan_selfcheck": (_i, [_i, _i, _i, _i]),
    "a81w41_block_idot": (_i, [_vp, _i, _vp, _i, _vp, _i, _i, _i, _vp]),
    "a81w41_repack_w80_weight": (_i, [_i, _i, _i, _vp, _vp, _vp]),
    "a81w41_quantize_weight_q40": (_i, [_vp, _i, _i, _vp, _vp]),
    "a81w41_quantize_row_q8_0_repack": (_i, [_vp, _vp, _i64, _vp]),
    "a81w41_gemv_repack_A80W40": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "a81w41_gemm_repack_A80W40_workspace_bytes": (_sz, [_i, _i, _i]),
    "a81w41_gemm_repack_A80W40": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _sz, _vp]),
    "a81w41_block_idot_A80W40": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "a81w41_context_create": (_i, [_i, _i, C.POINTER(_vp)]),
    "a81w41_context_destroy": (None, [_vp]),
    "a81w41_context_activation_scratch_dev": (_vp, [_vp]),
    "a81w41_linear_create": (_i, [_vp, _i, _i, _vp, _vp, _vp, C.POINTER(_vp)]),
    "a81w41_linear_create_from_blobs": (_i, [_vp, _i, _i, _vp, _vp, C.POINTER(_vp)]),
    "a81w41_linear_load": (_i, [_vp, C.c_char_p, _i, _i, _i, C.POINTER(_vp)]),
    "a81w41_linear_destroy": (None, [_vp]),
    "a81w41_linear_resident_bytes": (_sz, [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)]),
    "a81w41_linear_kernel_name": (C.c_char_p, [_vp, _i]),
    "a81w41_linear_in_features": (_i, [_vp]),
    "a81w41_linear_out_features": (_i, [_vp]),
    "a81w41_linear_weight_fp16_dev": (_vp, [_vp]),
    "a81w41_linear_weight_fp32_dev": (_vp, [_vp]),
    "a81w41_linear_forward": (_i, [_vp, _vp, _i, _vp, _vp]),
    "a81w41_linear_forward_quantized": (_i, [_vp, _vp, _i, _vp, _vp]),
    "a81w41_linear_set_kernel": (_i, [_vp, _i]),
    "a81w41_linear_forward_multi": (_i, [_i, C.POINTER(_vp), _vp, _i, C.POINTER(_vp), _vp]),
    "a81w41_linear_forward_host": (_i, [_vp, _vp, _i, _vp]),
    "a81w41_context_chain_begin": (_i, [_vp, _vp]),
    "a81w41_context_chain_end": (_i, [_vp]),
    "a81w41_context_chain_status": (_i, [_vp, C.POINTER(_i)]),
    "a81w41_context_chain_set_spin_limit": (_i, [_vp, C.c_uint]),
    "a81w41_context_chain_selfcheck_stuck_wait": (_i, [_vp, _vp, _vp, C.c_uint, _vp]),
    "a81w41_qwen3_create": (_i, [_vp, C.POINTER(_vp)]),
    "a81w41_qwen3_load": (_i, [C.c_char_p, _vp, C.POINTER(_vp)]),
    "a81w41_qwen3_destroy": (None, [_vp]),
    "a81w41_qwen3_set_linear": (_i, [_vp, _i, _i, _vp, _vp, _vp]),
    "a81w41_qwen3_set_linear_blobs": (_i, [_vp, _i, _i, _vp, _vp]),
    "a81w41_qwen3_set_norm": (_i, [_vp, _i, _i, _vp]),
    "a81w41_qwen3_set_embedding": (_i, [_vp, _vp]),
    "a81w41_qwen3_set_option": (_i, [_vp, _i, _i]),
    "a81w41_qwen3_chain_status": (_i, [_vp, C.POINTER(_i)]),
    "a81w41_qwen3_resident_bytes": (_sz, [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)]),
    "a81w41_qwen3_read_buffer": (_i, [_vp, _i, _vp, _sz]),
    "a81w41_qwen3_reset": (_i, [_vp]),
    "a81w41_qwen3_forward": (_i, [_vp, _vp, _i, _vp]),
    "a81w41_qwen3_attention": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, C.c_float, _i, _vp]),
    "a81w41_qwen3_attention_one_token": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, C.c_float, C.c_float,
                                              _i, _vp]),
    "a81w41_qwen3_generate_greedy": (_i, [_vp, _vp, _i, _i, _vp, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
}


class Qwen3Config(C.Structure):
    """a81w41_qwen3_config"""
    _fields_ = [("n_layers", _i), ("hidden", _i), ("n_q_heads", _i), ("n_kv_heads", _i), ("intermediate", _i),
                ("vocab", _i), ("max_seq", _i), ("rope_theta", C.c_float), ("rms_eps", C.c_float)]

_lib = None


class A81W41Error(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"a81w41 status {status}: {message}")
        self.status = status


def lib():
    """Load the HIP library (once) and bind every exported symbol."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.dirname(LIB_PATH)}` "
                "(or __graft_entry__.build()); this package has no CPU fallback")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status: int) -> None:
    if status != OK:
        raise A81W41Error(status, lib().a81w41_last_error().decode())
