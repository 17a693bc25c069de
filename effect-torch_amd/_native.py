"""ctypes binding of ``lib/libet_hip.so`` (the C ABI declared in ``include/et_hip.h`` and ``include/et_hip_calibrate.h``).

The library is loaded from inside the package directory only. There is no CPU
fallback: if the shared object is missing this module raises on import of
``lib()``, and every operator fails loudly without it.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libet_hip.so")
CALIBRATE_LIB_PATH = os.path.join(HERE, "lib", "libet_hip_calibrate.so")

# et_status
OK, ERR_UNSUPPORTED, ERR_EXECUTION, ERR_CANCELLED, ERR_UNAVAILABLE, ERR_INVALID = range(6)
# et_dtype
DTYPE_F32, DTYPE_F64, DTYPE_F16, DTYPE_BF16, DTYPE_U8, DTYPE_U32, DTYPE_I64 = range(7)
# et_activation_mode
ACT_F32, ACT_INT8 = 0, 1
STATUS_BYTES = 16


class EtTensor(ctypes.Structure):
    """``et_tensor`` of include/et_hip.h."""

    _fields_ = [
        ("data", ctypes.c_void_p),
        ("dtype", ctypes.c_int32),
        ("rank", ctypes.c_int32),
        ("shape", ctypes.POINTER(ctypes.c_uint64)),
        ("strides", ctypes.POINTER(ctypes.c_uint64)),
        ("offset", ctypes.c_uint64),
    ]


class EtPrepareSource(ctypes.Structure):
    """``et_prepare_source`` of include/et_hip.h."""

    _fields_ = [
        ("kind", ctypes.c_int32),
        ("x", ctypes.c_void_p),
        ("x_row_stride", ctypes.c_uint64),
        ("second", ctypes.c_void_p),
        ("eps", ctypes.c_double),
        ("second_dtype", ctypes.c_int32),
    ]


PREPARE_PLAIN, PREPARE_RMS_NORM, PREPARE_SILU_MUL = 0, 1, 2


class EtRotaryAfter(ctypes.Structure):
    """``et_rotary_after`` of include/et_hip.h."""

    _fields_ = [
        ("members", ctypes.c_uint32),
        ("offsets", ctypes.c_void_p),
        ("offsets_len", ctypes.c_uint64),
        ("theta", ctypes.c_double),
        ("sign", ctypes.c_double),
        ("layout", ctypes.c_int32),
        ("head_dim", ctypes.c_uint64),
    ]


class EtGroupShares(ctypes.Structure):
    """``et_group_shares`` of include/et_hip.h."""

    _fields_ = [
        ("shares", ctypes.c_void_p),
        ("count", ctypes.c_uint32),
        ("vectors", ctypes.c_uint64),
        ("launch_rows", ctypes.c_uint64),
        ("first_row", ctypes.c_uint64 * 4),
    ]


class EtKvProjected(ctypes.Structure):
    """``et_kv_projected`` of include/et_hip.h."""

    _fields_ = [
        ("shares", EtGroupShares),
        ("q_member", ctypes.c_uint32),
        ("k_member", ctypes.c_uint32),
        ("v_member", ctypes.c_uint32),
        ("q_bias", ctypes.c_void_p),
        ("k_bias", ctypes.c_void_p),
        ("v_bias", ctypes.c_void_p),
        ("offsets", ctypes.c_void_p),
        ("offsets_len", ctypes.c_uint64),
        ("theta", ctypes.c_double),
        ("sign", ctypes.c_double),
        ("layout", ctypes.c_int32),
    ]


class EtKvLayer(ctypes.Structure):
    """``et_kv_layer`` of include/et_hip.h."""

    _fields_ = [
        ("k_slab", ctypes.c_void_p),
        ("v_slab", ctypes.c_void_p),
        ("slab_dtype", ctypes.c_int32),
        ("max_tokens", ctypes.c_uint64),
        ("kv_heads", ctypes.c_uint64),
        ("head_dim", ctypes.c_uint64),
        ("block_size", ctypes.c_uint64),
        ("block_table", ctypes.c_void_p),
        ("table_stride", ctypes.c_uint64),
        ("cursors", ctypes.c_void_p),
        ("advances", ctypes.c_void_p),
        ("slots", ctypes.c_uint64),
        ("active_batch", ctypes.c_uint64),
        ("context_window", ctypes.c_uint64),
        ("max_context", ctypes.c_uint64),
        ("k_scales", ctypes.c_void_p),
        ("v_scales", ctypes.c_void_p),
    ]


class EtGgufTensor(ctypes.Structure):
    """``et_gguf_tensor`` of include/et_hip.h."""

    _fields_ = [
        ("name", ctypes.c_void_p),
        ("name_length", ctypes.c_uint64),
        ("format", ctypes.c_int32),
        ("logical_rank", ctypes.c_int32),
        ("logical_shape", ctypes.c_uint64 * 4),
        ("physical_rank", ctypes.c_int32),
        ("physical_shape", ctypes.c_uint64 * 4),
        ("data_offset", ctypes.c_uint64),
        ("byte_len", ctypes.c_uint64),
    ]


# Every symbol include/et_hip.h declares: name -> (restype, argtypes).
_vp, _u64, _i32 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int32
_T = ctypes.POINTER(EtTensor)
_PP = ctypes.POINTER(ctypes.c_void_p)
_KV = ctypes.POINTER(EtKvLayer)
SIGNATURES = {
    "et_hip_is_available": (ctypes.c_int, []),
    "et_hip_codec_name": (ctypes.c_char_p, [_i32]),
    "et_hip_block_values": (_u64, [_i32]),
    "et_hip_block_bytes": (_u64, [_i32]),
    "et_hip_encoded_row_bytes": (_u64, [_i32, _u64]),
    "et_hip_linear_requirements": (ctypes.c_int, [_T, _T, _T, _i32, _u64, _u64, _i32, _PP]),
    "et_hip_linear_plan_destroy": (None, [_vp]),
    "et_hip_linear_plan_output_rank": (_i32, [_vp]),
    "et_hip_linear_plan_output_shape": (None, [_vp, ctypes.POINTER(_u64)]),
    "et_hip_linear_plan_vectors": (_u64, [_vp]),
    "et_hip_linear_plan_output_bytes": (_u64, [_vp]),
    "et_hip_linear_plan_workspace_bytes": (_u64, [_vp]),
    "et_hip_linear_plan_kernel": (ctypes.c_char_p, [_vp]),
    "et_hip_linear_plan_algorithmic_bytes": (_u64, [_vp]),
    "et_hip_linear_into": (ctypes.c_int, [_vp, _T, _T, _T, _T, _vp, _u64, _vp, _vp]),
    "et_hip_linear_plan_create": (ctypes.c_int, [_i32, _u64, _u64, _u64, _i32, _i32, _PP]),
    "et_hip_linear_enqueue": (ctypes.c_int, [_vp, _vp, _u64, _vp, _vp, _vp, _vp, _u64, _vp, _vp]),
    "et_hip_linear_plan_prepared_input_bytes": (_u64, [_vp]),
    "et_hip_linear_prepare_input": (ctypes.c_int, [_vp, _vp, _u64, _vp, _u64, _vp]),
    "et_hip_linear_plan_fused_prepare": (ctypes.c_int, [_vp]),
    "et_hip_linear_group_workspace_bytes": (ctypes.c_int, [_vp, ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint64)]),
    "et_hip_linear_enqueue_prepared_group": (ctypes.c_int, [_vp, ctypes.c_uint32, _vp, _vp, _vp, _vp, _vp, _vp, _u64,
                                                            _vp, _vp]),
    "et_hip_linear_enqueue_static_workspace": (ctypes.c_int, [_vp, _vp, _u64, _vp, _vp, _vp, _vp, _vp]),
    "et_hip_linear_prepare_input_from": (ctypes.c_int, [_vp, ctypes.POINTER(EtPrepareSource), _vp, _u64, _vp]),
    "et_hip_linear_enqueue_prepared": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u64, _vp, _vp]),
    "et_hip_linear_enqueue_prepared_group_then_rotary": (ctypes.c_int, [_vp, ctypes.c_uint32, _vp, _vp, _vp, _vp, _vp, _vp,
                                                                        _u64, ctypes.POINTER(EtRotaryAfter), _vp, _vp]),
    "et_hip_linear_group_shares_layout": (ctypes.c_int, [_vp, ctypes.c_uint32, ctypes.POINTER(EtGroupShares)]),
    "et_hip_linear_enqueue_prepared_group_shares": (ctypes.c_int, [_vp, ctypes.c_uint32, _vp, _vp, _vp, _u64,
                                                                   ctypes.POINTER(EtGroupShares), _vp, _vp]),
    "et_hip_linear_enqueue_prepared_then_norm": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u64, _vp, _vp, _i32,
                                                                ctypes.c_double, _vp, _u64, _vp, _vp]),
    "et_hip_embedding_requirements": (ctypes.c_int, [_T, _T, _i32, _u64, _u64, _PP]),
    "et_hip_embedding_plan_destroy": (None, [_vp]),
    "et_hip_embedding_plan_output_rank": (_i32, [_vp]),
    "et_hip_embedding_plan_output_shape": (None, [_vp, ctypes.POINTER(_u64)]),
    "et_hip_embedding_plan_output_bytes": (_u64, [_vp]),
    "et_hip_embedding_into": (ctypes.c_int, [_vp, _T, _T, _T, _vp, _vp, _vp]),
    "et_hip_embedding_status_check": (ctypes.c_int, [_vp, _vp]),
    "et_hip_dequantize_rows": (ctypes.c_int, [_i32, _u64, _u64, _vp, _vp, _vp]),
    "et_hip_kv_attention_workspace_bytes": (_u64, [_KV, _u64, _u64]),
    "et_hip_kv_attention_into": (ctypes.c_int, [_KV, _T, _T, _T, ctypes.c_double, _u64, _T, _vp, _u64, _vp, _vp, _vp]),
    "et_hip_kv_attention_prepared_into": (ctypes.c_int, [_KV, _T, _T, _T, ctypes.c_double, _u64, _T, _vp, _u64, _vp, _vp,
                                                         _vp, _u64, _vp, _vp]),
    "et_hip_kv_attention_projected_into": (ctypes.c_int, [_KV, ctypes.POINTER(EtKvProjected), ctypes.c_double, _u64, _T, _vp,
                                                          _u64, _vp, _vp, _vp, _u64, _vp, _vp]),
    "et_hip_kv_attention_status_check": (ctypes.c_int, [_KV, _u64, _vp]),
    "et_hip_kv_attention_kernel": (ctypes.c_char_p, [_KV, _u64, _u64]),
    "et_hip_kv_commit": (ctypes.c_int, [_KV, _vp]),
    "et_hip_rms_norm_into": (ctypes.c_int, [_T, _T, ctypes.c_double, _T, _vp]),
    "et_hip_rotary_into": (ctypes.c_int, [_T, _vp, _u64, ctypes.c_double, ctypes.c_double, _i32, _T, _vp]),
    "et_hip_rotary_pair_into": (ctypes.c_int, [_T, _T, _vp, _u64, ctypes.c_double, ctypes.c_double, _i32, _T, _T, _vp]),
    "et_hip_add_into": (ctypes.c_int, [_T, _T, _T, _vp]),
    "et_hip_silu_mul_into": (ctypes.c_int, [_T, _T, _T, _vp]),
    "et_hip_greedy_workspace_bytes": (_u64, [_u64, _u64]),
    "et_hip_greedy_tokens_into": (ctypes.c_int, [_T, _vp, _vp, _u64, _vp, _vp]),
    "et_hip_greedy_status_check": (ctypes.c_int, [_u64, _vp]),
    "et_hip_gather_rows_into": (ctypes.c_int, [_T, _T, _T, _vp, _vp]),
    "et_hip_gather_rows_status_check": (ctypes.c_int, [_u64, _u64, _vp]),
    "et_hip_gguf_open": (ctypes.c_int, [ctypes.c_char_p, _vp, _PP]),
    "et_hip_gguf_close": (None, [_vp]),
    "et_hip_gguf_architecture": (ctypes.c_char_p, [_vp]),
    "et_hip_gguf_metadata_count": (_u64, [_vp]),
    "et_hip_gguf_metadata_find": (ctypes.c_int64, [_vp, ctypes.c_char_p]),
    "et_hip_gguf_metadata_key": (_vp, [_vp, _u64]),
    "et_hip_gguf_metadata_key_length": (_u64, [_vp, _u64]),
    "et_hip_gguf_metadata_type": (_i32, [_vp, _u64]),
    "et_hip_gguf_metadata_element_type": (_i32, [_vp, _u64]),
    "et_hip_gguf_metadata_length": (_u64, [_vp, _u64]),
    "et_hip_gguf_metadata_unsigned": (ctypes.c_int, [_vp, _u64, _u64, ctypes.POINTER(_u64)]),
    "et_hip_gguf_metadata_signed": (ctypes.c_int, [_vp, _u64, _u64, ctypes.POINTER(ctypes.c_int64)]),
    "et_hip_gguf_metadata_real": (ctypes.c_int, [_vp, _u64, _u64, ctypes.POINTER(ctypes.c_double)]),
    "et_hip_gguf_metadata_string": (_vp, [_vp, _u64, _u64, ctypes.POINTER(_u64)]),
    "et_hip_gguf_tensor_count": (_u64, [_vp]),
    "et_hip_gguf_tensor_find": (ctypes.c_int64, [_vp, ctypes.c_char_p]),
    "et_hip_gguf_tensor_at": (ctypes.c_int, [_vp, _u64, ctypes.POINTER(EtGgufTensor)]),
    "et_hip_gguf_read_tensor_into": (ctypes.c_int, [_vp, _u64, _vp, _u64, _vp]),
    "et_hip_gguf_upload_tensor": (ctypes.c_int, [_vp, _u64, _vp, _u64, _vp, _vp]),
    "et_hip_quantize_activations": (ctypes.c_int, [_vp, _u64, _u64, _u64, _vp, _vp, _vp, _vp]),
    "et_hip_handover_timeouts": (ctypes.c_int, [_vp]),
    "et_hip_test_set_handover_spin_limit": (None, [ctypes.c_uint32]),
    "et_hip_last_error": (ctypes.c_char_p, []),
}

# libet_hip_calibrate.so: the measurement aids (include/et_hip_calibrate.h)
CALIBRATE_SIGNATURES = {
    "et_hip_calibration_read": (ctypes.c_int, [_vp, _u64, _vp, ctypes.c_uint32, _vp]),
    "et_hip_calibration_read_variant": (ctypes.c_int, [_i32, _vp, _u64, _vp, ctypes.c_uint32, _vp]),
    "et_hip_calibration_copy": (ctypes.c_int, [_vp, _vp, _u64, _vp]),
    "et_hip_calibration_contraction": (ctypes.c_int, [_i32, _vp, _vp, _vp, _u64, _u64, _u64, _vp]),
    "et_hip_calibration_mfma": (ctypes.c_int, [_i32, ctypes.c_uint32, ctypes.c_uint32, _vp, _vp]),
    "et_hip_calibration_last_error": (ctypes.c_char_p, []),
}

_lib = None
_calibrate_lib = None


class NativeLibraryMissing(ImportError):
    pass


def lib() -> ctypes.CDLL:
    """Loads the built HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NativeLibraryMissing(
                f"{LIB_PATH} is missing: build it with `python effect-torch_amd/build.py` "
                "(there is no fallback implementation)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def calibrate_lib() -> ctypes.CDLL:
    """Loads the measurement library (after the operators' library, which it links against)."""
    global _calibrate_lib
    if _calibrate_lib is None:
        lib()
        if not os.path.exists(CALIBRATE_LIB_PATH):
            raise NativeLibraryMissing(f"{CALIBRATE_LIB_PATH} is missing: build it with `python effect-torch_amd/build.py`")
        handle = ctypes.CDLL(CALIBRATE_LIB_PATH)
        for name, (restype, argtypes) in CALIBRATE_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _calibrate_lib = handle
    return _calibrate_lib


def last_error() -> str:
    return lib().et_hip_last_error().decode()
