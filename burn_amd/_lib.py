"""Loads libburnq_mi355.so and declares every entry point of include/burnq.h for ctypes.

The library is the product; this module only binds it. If the shared object is missing the
import fails loudly -- there is no Python or CPU fallback for any operation.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libburnq_mi355.so")

MAX_RANK = 8

# bq_status
OK, ERR_NULL, ERR_UNSUPPORTED_SCHEME, ERR_SHAPE, ERR_DTYPE, ERR_HIP, ERR_SIZE, ERR_UNSUPPORTED_OP, ERR_NONFINITE = range(9)
STATUS_NAMES = ["OK", "ERR_NULL", "ERR_UNSUPPORTED_SCHEME", "ERR_SHAPE", "ERR_DTYPE", "ERR_HIP",
                "ERR_SIZE", "ERR_UNSUPPORTED_OP", "ERR_NONFINITE"]
# dtypes
F32, BF16, QFLOAT, I32, I64 = 0, 1, 2, 3, 4
# scheme enums
Q8S, Q4S, Q2S, Q8F, Q4F, Q2F = 0, 1, 2, 3, 4, 5
LEVEL_TENSOR, LEVEL_BLOCK = 0, 1
STORE_NATIVE, STORE_PACKED_U32 = 0, 1
SCALE_F32, SCALE_F16, SCALE_BF16, SCALE_UE4M3 = 0, 1, 2, 3


class CScheme(C.Structure):
    """bq_scheme"""

    _fields_ = [
        ("value", C.c_uint8),
        ("level", C.c_uint8),
        ("store", C.c_uint8),
        ("scale_dtype", C.c_uint8),
        ("block_rank", C.c_uint8),
        ("tensor_scale", C.c_uint8),
        ("reserved", C.c_uint8 * 2),
        ("block", C.c_uint8 * MAX_RANK),
    ]


class CPackEntry(C.Structure):
    """bq_pack_entry"""

    _fields_ = [
        ("name", C.c_char_p),
        ("dtype", C.c_int32),
        ("rank", C.c_int32),
        ("shape", C.c_size_t * MAX_RANK),
        ("data_begin", C.c_uint64),
        ("data_end", C.c_uint64),
        ("has_param_id", C.c_int32),
        ("param_id", C.c_uint64),
        ("has_scheme", C.c_int32),
        ("scheme", CScheme),
        ("data", C.c_void_p),
    ]


PACK_DTYPES = ["F64", "F32", "Flex32", "F16", "BF16", "I64", "I32", "I16", "I8", "U64", "U32", "U16", "U8", "Bool", "QFloat"]
PACK_F32, PACK_BF16, PACK_QFLOAT = 1, 4, 14

_vp, _sz, _i32 = C.c_void_p, C.c_size_t, C.c_int32
_psz = C.POINTER(C.c_size_t)
_pvp = C.POINTER(C.c_void_p)
_ps = C.POINTER(CScheme)

# name -> (restype, argtypes). Every symbol include/burnq.h declares is listed here; the CPU test
# suite checks that the built library exports all of them.
SIGNATURES = {
    "bq_last_error": (C.c_char_p, []),
    "bq_device_count": (_i32, [C.POINTER(_i32)]),
    "bq_device_open": (_i32, [_i32, _pvp]),
    "bq_device_close": (_i32, [_vp]),
    "bq_device_sync": (_i32, [_vp]),
    "bq_device_stream": (_vp, [_vp]),
    "bq_device_trim": (_i32, [_vp]),
    "bq_device_set_validate": (_i32, [_vp, _i32]),
    "bq_device_set_f32_matmul_exact": (_i32, [_vp, _i32]),
    "bq_timer_start": (_i32, [_vp]),
    "bq_timer_stop": (_i32, [_vp, C.POINTER(C.c_float)]),
    "bq_graph_begin_capture": (_i32, [_vp]),
    "bq_graph_end_capture": (_i32, [_vp, _pvp]),
    "bq_graph_launch": (_i32, [_vp]),
    "bq_graph_release": (_i32, [_vp]),
    "bq_tensor_retain": (_i32, [_vp]),
    "bq_tensor_release": (_i32, [_vp]),
    "bq_tensor_rank": (_i32, [_vp]),
    "bq_tensor_shape": (_i32, [_vp, _psz]),
    "bq_tensor_dtype": (_i32, [_vp]),
    "bq_tensor_scheme": (_i32, [_vp, _ps]),
    "bq_tensor_data_ptr": (_vp, [_vp]),
    "bq_tensor_scales_ptr": (_vp, [_vp]),
    "bq_tensor_num_scales": (_sz, [_vp]),
    "bq_float_from_data": (_i32, [_vp, _vp, _i32, _psz, _i32, _pvp]),
    "bq_float_into_data": (_i32, [_vp, _vp, _sz]),
    "bq_float_empty": (_i32, [_vp, _i32, _psz, _i32, _pvp]),
    "bq_float_from_device_ptr": (_i32, [_vp, _vp, _i32, _psz, _i32, _pvp]),
    "bq_float_matmul": (_i32, [_vp, _vp, _pvp]),
    "bq_scheme_supported": (_i32, [_ps]),
    "bq_quantized_data_len": (_i32, [_ps, _psz, _i32, _psz]),
    "bq_q_from_data": (_i32, [_vp, _vp, _sz, _psz, _i32, _ps, _pvp]),
    "bq_q_into_data": (_i32, [_vp, _vp, _sz, _psz]),
    "bq_quantize": (_i32, [_vp, _ps, _vp, _pvp]),
    "bq_quantize_two_level": (_i32, [_vp, C.POINTER(CScheme), _vp, _vp, _pvp]),
    "bq_quantize_dynamic": (_i32, [_vp, _ps, _pvp]),
    "bq_compute_range_abs_mean": (_i32, [_vp, _ps, _pvp]),
    "bq_quantize_abs_mean": (_i32, [_vp, _ps, _pvp]),
    "bq_dequantize": (_i32, [_vp, _i32, _pvp]),
    "bq_q_matmul": (_i32, [_vp, _vp, _pvp]),
    "bq_q_matmul_as": (_i32, [_vp, _vp, _i32, _pvp]),
    "bq_q_linear": (_i32, [_vp, _vp, _vp, _i32, _pvp]),
    "bq_q_matmul_propagate": (_i32, [_vp, _vp, _pvp]),
    "bq_q_to_device": (_i32, [_vp, _vp, _pvp]),
    "bq_q_reshape": (_i32, [_vp, _psz, _i32, _pvp]),
    "bq_q_swap_dims": (_i32, [_vp, _i32, _i32, _pvp]),
    "bq_q_permute": (_i32, [_vp, C.POINTER(_i32), _i32, _pvp]),
    "bq_q_flip": (_i32, [_vp, C.POINTER(_i32), _i32, _pvp]),
    "bq_int_from_data": (_i32, [_vp, _vp, _i32, _psz, _i32, _pvp]),
    "bq_int_into_data": (_i32, [_vp, _vp, _sz]),
    "bq_q_slice": (_i32, [_vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64), _i32, _pvp]),
    "bq_q_select": (_i32, [_vp, _i32, _vp, _pvp]),
    "bq_q_gather": (_i32, [_i32, _vp, _vp, _pvp]),
    "bq_q_expand": (_i32, [_vp, _psz, _i32, _pvp]),
    "bq_q_argmax": (_i32, [_vp, _i32, _i32, _pvp]),
    "bq_q_argmin": (_i32, [_vp, _i32, _i32, _pvp]),
    "bqk_selftest_division": (_i32, [_vp, _vp]),
    "bqk_copy": (_i32, [_vp, _vp, _sz, _vp]),
    "bqk_lds_request_status": (_i32, [_sz, _sz]),
    "bqk_absmax_f32": (_i32, [_vp, _sz, _vp, _vp]),
    "bqk_quantize_per_tensor_from_absmax": (_i32, [_vp, _sz, _vp, _vp, _i32, _i32, _vp, _vp]),
    "bqk_scales_from_absmax": (_i32, [_vp, _sz, _i32, _vp, _vp]),
    "bqk_quantize_per_tensor": (_i32, [_vp, _sz, _vp, _i32, _i32, _vp, _vp]),
    "bqk_quantize_dynamic_block": (_i32, [_vp, _sz, _i32, _i32, _i32, _vp, _vp, _vp]),
    "bqk_quantize_block": (_i32, [_vp, _sz, _i32, _vp, _i32, _i32, _vp, _vp]),
    "bqk_dequantize": (_i32, [_vp, _sz, _i32, _vp, _i32, _i32, _i32, _vp, _vp]),
    "bqk_q_matmul_workspace": (_sz, [_sz, _sz, _sz, _i32, _i32]),
    "bqk_q_matmul": (_i32, [_vp, _i32, _sz, _sz, _sz, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp,
                            _sz, _vp]),
    "bqk_q_linear": (_i32, [_vp, _i32, _sz, _sz, _sz, _vp, _vp, _i32, _i32, _i32, _vp, _i32, _vp, _vp,
                            _sz, _vp]),
    "bq_pack_data_section_start": (_sz, [_sz]),
    "bq_pack_open": (_i32, [C.c_char_p, _pvp]),
    "bq_pack_from_bytes": (_i32, [_vp, _sz, _i32, _pvp]),
    "bq_pack_close": (_i32, [_vp]),
    "bq_pack_num_tensors": (C.c_int64, [_vp]),
    "bq_pack_entry_at": (_i32, [_vp, C.c_int64, C.POINTER(CPackEntry)]),
    "bq_pack_find": (_i32, [_vp, C.c_char_p, C.POINTER(CPackEntry)]),
    "bq_pack_metadata": (C.c_char_p, [_vp, C.c_char_p]),
    "bq_pack_load": (_i32, [_vp, C.c_char_p, _ps, _vp, _pvp]),
    "bq_pack_writer_new": (_i32, [_pvp]),
    "bq_pack_writer_free": (_i32, [_vp]),
    "bq_pack_writer_set_metadata": (_i32, [_vp, C.c_char_p, C.c_char_p]),
    "bq_pack_writer_add_bytes": (_i32, [_vp, C.c_char_p, _i32, _ps, _psz, _i32, _vp, _sz, _i32, C.c_uint64]),
    "bq_pack_writer_add_tensor": (_i32, [_vp, C.c_char_p, _vp, _i32, C.c_uint64]),
    "bq_pack_writer_size": (_i32, [_vp, _psz]),
    "bq_pack_writer_write_into": (_i32, [_vp, _vp, _sz, _psz]),
    "bq_pack_writer_write_file": (_i32, [_vp, C.c_char_p]),
    "bqk_q_linear_static": (_i32, [_vp, _i32, _sz, _sz, _sz, _vp, _vp, _i32, _i32, _i32, _vp, _i32, _vp, _vp]),
}
STATIC_SCRATCH_BYTES = 16 << 20

_lib = None


def lib():
    """The loaded library. Raises if it has not been built (python -m burn_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build the HIP library with `python -m burn_amd.build` "
                "(there is no fallback implementation)")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


class BurnqError(RuntimeError):
    """A bq_status != BQ_OK. Where the reference panics, this is raised instead."""

    def __init__(self, status, message):
        self.status = status
        name = STATUS_NAMES[status] if 0 <= status < len(STATUS_NAMES) else str(status)
        super().__init__(f"{name}: {message}")


def check(status):
    if status != OK:
        raise BurnqError(status, lib().bq_last_error().decode())
