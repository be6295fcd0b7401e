"""ctypes wrapper over the C oracle (``libbq_oracle.so``). TEST INFRASTRUCTURE ONLY.

The library is built by ``oracle/Makefile`` (``__graft_entry__.build()`` runs it); this module
builds it on demand if it is missing, since gcc is all it needs.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libbq_oracle.so")

Q8S, Q4S, Q2S, Q8F, Q4F, Q2F = 0, 1, 2, 3, 4, 5
LEVEL_TENSOR, LEVEL_BLOCK = 0, 1
STORE_NATIVE, STORE_PACKED_U32 = 0, 1
MAX_RANK = 8


class Scheme(C.Structure):
    """Field-for-field image of ``bqo_scheme``."""

    _fields_ = [
        ("value", C.c_uint8),
        ("level", C.c_uint8),
        ("store", C.c_uint8),
        ("block_rank", C.c_uint8),
        ("block", C.c_uint8 * MAX_RANK),
    ]

    @classmethod
    def make(cls, value=Q8S, block=None, store=STORE_NATIVE):
        s = cls()
        s.value = value
        s.store = store
        if block is None:
            s.level = LEVEL_TENSOR
            s.block_rank = 0
        else:
            s.level = LEVEL_BLOCK
            s.block_rank = len(block)
            for i, b in enumerate(block):
                s.block[i] = b
        return s


def build(force: bool = False) -> str:
    # (make compares time stamps: a library older than its sources is rebuilt, a current one is not)
    subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        sz, i32, pf, pi8, pu8, pu32 = (C.c_size_t, C.c_int, C.POINTER(C.c_float),
                                       C.POINTER(C.c_int8), C.POINTER(C.c_uint8),
                                       C.POINTER(C.c_uint32))
        psz, ps = C.POINTER(C.c_size_t), C.POINTER(Scheme)
        L.bqo_value_range.argtypes = [i32, pf, pf]
        L.bqo_num_quants.argtypes = [i32]
        L.bqo_params_shape.argtypes = [psz, i32, ps, psz]
        L.bqo_params_shape.restype = sz
        L.bqo_block_of.argtypes = [psz, i32, ps, sz]
        L.bqo_block_of.restype = sz
        L.bqo_compute_range.argtypes = [pf, psz, i32, ps, pf, pf]
        L.bqo_compute_range_abs_mean.argtypes = [pf, psz, i32, ps, pf, pf]
        L.bqo_compute_q_params.argtypes = [pf, pf, sz, i32, pf]
        L.bqo_compute_q_params.restype = None
        L.bqo_quantize.argtypes = [pf, psz, i32, ps, pf, pi8]
        L.bqo_quantize_dynamic.argtypes = [pf, psz, i32, ps, pi8, pf]
        L.bqo_quantize_dynamic_mt.argtypes = [pf, psz, i32, ps, pi8, pf]
        L.bqo_dequantize.argtypes = [pi8, psz, i32, ps, pf, pf]
        L.bqo_dequantize_mt.argtypes = [pi8, psz, i32, ps, pf, pf]
        L.bqo_storage_elements.argtypes = [psz, i32, ps]
        L.bqo_storage_elements.restype = sz
        L.bqo_pack_u32.argtypes = [pi8, psz, i32, i32, pu32]
        L.bqo_pack_u32.restype = None
        L.bqo_unpack_u32.argtypes = [pu32, psz, i32, i32, pi8]
        L.bqo_unpack_u32.restype = None
        L.bqo_quantized_data_len.argtypes = [psz, i32, ps]
        L.bqo_quantized_data_len.restype = sz
        L.bqo_encode.argtypes = [pi8, psz, i32, ps, pf, pu8]
        L.bqo_encode.restype = sz
        L.bqo_decode.argtypes = [pu8, sz, psz, i32, ps, pi8, pf]
        L.bqo_matmul_f32.argtypes = [pf, pf, pf, sz, sz, sz]
        L.bqo_matmul_f32.restype = None
        L.bqo_q_matmul.argtypes = [pf, sz, pi8, psz, ps, pf, pf]
        L.bqo_max_threads.restype = i32
        L.bqo_ternary_matmul.argtypes = [pf, sz, sz, sz, pi8, C.c_float, pf]
        L.bqo_ternary_matmul.restype = None
        L.bqo_scale_to_dtype.argtypes = [C.c_float, i32]
        L.bqo_scale_to_dtype.restype = C.c_float
        L.bqo_scale_size.argtypes = [i32]
        L.bqo_scale_size.restype = sz
        L.bqo_encode_scales.argtypes = [pf, sz, i32, pu8]
        L.bqo_encode_scales.restype = None
        L.bqo_decode_scales.argtypes = [pu8, sz, i32, pf]
        L.bqo_decode_scales.restype = None
        L.bqo_normalize_scales.argtypes = [pf, sz, i32]
        L.bqo_normalize_scales.restype = C.c_float
        L.bqo_two_level_scales.argtypes = [pf, sz, i32, C.c_float, pf, pf]
        L.bqo_two_level_scales.restype = None
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(C.POINTER(ct))


def _shape(shape):
    shape = tuple(int(d) for d in shape)
    return (C.c_size_t * max(len(shape), 1))(*shape), len(shape)


def value_range(value):
    a, b = C.c_float(), C.c_float()
    if lib().bqo_value_range(value, C.byref(a), C.byref(b)):
        raise ValueError("unknown quant value")
    return a.value, b.value


def params_shape(shape, scheme):
    sh, rank = _shape(shape)
    out = (C.c_size_t * MAX_RANK)()
    n = lib().bqo_params_shape(sh, rank, C.byref(scheme), out)
    if scheme.level == LEVEL_TENSOR:
        return (1,), n
    return tuple(out[i] for i in range(rank)), n


def block_of(shape, scheme, index):
    sh, rank = _shape(shape)
    return lib().bqo_block_of(sh, rank, C.byref(scheme), index)


def compute_range(x, scheme):
    x = np.ascontiguousarray(x, dtype=np.float32)
    sh, rank = _shape(x.shape)
    pshape, n = params_shape(x.shape, scheme)
    lo = np.empty(n, np.float32)
    hi = np.empty(n, np.float32)
    if lib().bqo_compute_range(_p(x, C.c_float), sh, rank, C.byref(scheme),
                               _p(lo, C.c_float), _p(hi, C.c_float)):
        raise ValueError("shape not divisible by block")
    return lo.reshape(pshape), hi.reshape(pshape)


def compute_range_abs_mean(x, scheme):
    """compute_range under Calibration::AbsMean: (-gamma, +gamma), gamma = mean |x| per tensor or block."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    sh, rank = _shape(x.shape)
    pshape, n = params_shape(x.shape, scheme)
    lo = np.empty(n, np.float32)
    hi = np.empty(n, np.float32)
    if lib().bqo_compute_range_abs_mean(_p(x, C.c_float), sh, rank, C.byref(scheme),
                                        _p(lo, C.c_float), _p(hi, C.c_float)):
        raise ValueError("empty tensor or shape not divisible by block")
    return lo.reshape(pshape), hi.reshape(pshape)


def compute_q_params(lo, hi, value):
    lo = np.ascontiguousarray(lo, dtype=np.float32)
    hi = np.ascontiguousarray(hi, dtype=np.float32)
    out = np.empty(lo.shape, np.float32)
    lib().bqo_compute_q_params(_p(lo, C.c_float), _p(hi, C.c_float), lo.size, value,
                               _p(out, C.c_float))
    return out


def quantize(x, scheme, scales):
    x = np.ascontiguousarray(x, dtype=np.float32)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    sh, rank = _shape(x.shape)
    q = np.empty(x.shape, np.int8)
    if lib().bqo_quantize(_p(x, C.c_float), sh, rank, C.byref(scheme), _p(scales, C.c_float),
                          _p(q, C.c_int8)):
        raise ValueError("quantize failed")
    return q


def quantize_dynamic(x, scheme, mt=False):
    x = np.ascontiguousarray(x, dtype=np.float32)
    sh, rank = _shape(x.shape)
    pshape, n = params_shape(x.shape, scheme)
    q = np.empty(x.shape, np.int8)
    scales = np.empty(n, np.float32)
    fn = lib().bqo_quantize_dynamic_mt if mt else lib().bqo_quantize_dynamic
    if fn(_p(x, C.c_float), sh, rank, C.byref(scheme), _p(q, C.c_int8), _p(scales, C.c_float)):
        raise ValueError("quantize_dynamic failed")
    return q, scales.reshape(pshape)


def dequantize(q, scheme, scales, mt=False):
    q = np.ascontiguousarray(q, dtype=np.int8)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    sh, rank = _shape(q.shape)
    out = np.empty(q.shape, np.float32)
    fn = lib().bqo_dequantize_mt if mt else lib().bqo_dequantize
    if fn(_p(q, C.c_int8), sh, rank, C.byref(scheme), _p(scales, C.c_float), _p(out, C.c_float)):
        raise ValueError("dequantize failed")
    return out


def storage_elements(shape, scheme):
    sh, rank = _shape(shape)
    return lib().bqo_storage_elements(sh, rank, C.byref(scheme))


def pack_u32(q, value):
    q = np.ascontiguousarray(q, dtype=np.int8)
    sh, rank = _shape(q.shape)
    s = Scheme.make(value, store=STORE_PACKED_U32)
    words = np.empty(lib().bqo_storage_elements(sh, rank, C.byref(s)), np.uint32)
    lib().bqo_pack_u32(_p(q, C.c_int8), sh, rank, value, _p(words, C.c_uint32))
    return words


def unpack_u32(words, shape, value):
    words = np.ascontiguousarray(words, dtype=np.uint32)
    sh, rank = _shape(shape)
    q = np.empty(tuple(shape), np.int8)
    lib().bqo_unpack_u32(_p(words, C.c_uint32), sh, rank, value, _p(q, C.c_int8))
    return q


def quantized_data_len(shape, scheme):
    sh, rank = _shape(shape)
    return lib().bqo_quantized_data_len(sh, rank, C.byref(scheme))


def encode(q, scheme, scales):
    q = np.ascontiguousarray(q, dtype=np.int8)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    sh, rank = _shape(q.shape)
    out = np.empty(quantized_data_len(q.shape, scheme), np.uint8)
    n = lib().bqo_encode(_p(q, C.c_int8), sh, rank, C.byref(scheme), _p(scales, C.c_float),
                         _p(out, C.c_uint8))
    assert n == out.size
    return out


def decode(data, shape, scheme):
    data = np.ascontiguousarray(data, dtype=np.uint8)
    sh, rank = _shape(shape)
    pshape, n = params_shape(shape, scheme)
    q = np.empty(tuple(shape), np.int8)
    scales = np.empty(n, np.float32)
    if lib().bqo_decode(_p(data, C.c_uint8), data.size, sh, rank, C.byref(scheme),
                        _p(q, C.c_int8), _p(scales, C.c_float)):
        raise ValueError("blob shorter than its scheme requires")
    return q, scales.reshape(pshape)


def matmul_f32(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    c = np.empty((m, n), np.float32)
    lib().bqo_matmul_f32(_p(a, C.c_float), _p(b, C.c_float), _p(c, C.c_float), m, k, n)
    return c


def q_matmul(lhs, rhs_q, scheme, rhs_scales):
    lhs = np.ascontiguousarray(lhs, dtype=np.float32)
    rhs_q = np.ascontiguousarray(rhs_q, dtype=np.int8)
    rhs_scales = np.ascontiguousarray(rhs_scales, dtype=np.float32)
    m = lhs.shape[0]
    sh, _ = _shape(rhs_q.shape)
    out = np.empty((m, rhs_q.shape[1]), np.float32)
    if lib().bqo_q_matmul(_p(lhs, C.c_float), m, _p(rhs_q, C.c_int8), sh, C.byref(scheme),
                          _p(rhs_scales, C.c_float), _p(out, C.c_float)):
        raise ValueError("q_matmul failed")
    return out


def max_threads():
    return lib().bqo_max_threads()


SCALE_F32, SCALE_F16, SCALE_BF16, SCALE_UE4M3 = 0, 1, 2, 3


def scale_to_dtype(scales, dtype):
    """scale_to_dtype applied to every entry (burn-ndarray/src/ops/qtensor.rs:90-95)."""
    a = np.ascontiguousarray(scales, dtype=np.float32)
    f = lib().bqo_scale_to_dtype
    return np.array([f(float(v), dtype) for v in a.reshape(-1)], np.float32).reshape(a.shape)


def encode_scales(scales, dtype):
    a = np.ascontiguousarray(scales, dtype=np.float32).reshape(-1)
    out = np.empty(a.size * lib().bqo_scale_size(dtype), np.uint8)
    lib().bqo_encode_scales(_p(a, C.c_float), a.size, dtype, _p(out, C.c_uint8))
    return out


def decode_scales(data, dtype):
    d = np.ascontiguousarray(data, dtype=np.uint8)
    n = d.size // lib().bqo_scale_size(dtype)
    out = np.empty(n, np.float32)
    lib().bqo_decode_scales(_p(d, C.c_uint8), n, dtype, _p(out, C.c_float))
    return out


def encode_with_scale_dtype(q, scheme, scales, dtype):
    """The QuantizedBytes blob with the scales region written in `dtype`: values || encoded scales."""
    blob = encode(q, scheme, np.zeros_like(np.ascontiguousarray(scales, np.float32)))
    n = int(np.ascontiguousarray(scales).size)
    return np.concatenate([blob[: blob.size - 4 * n], encode_scales(scales, dtype)])


def ternary_matmul(lhs, rhs_q, gamma):
    lhs = np.ascontiguousarray(lhs, dtype=np.float32)
    rhs_q = np.ascontiguousarray(rhs_q, dtype=np.int8)
    m, k = lhs.shape
    n = rhs_q.shape[1]
    out = np.empty((m, n), np.float32)
    lib().bqo_ternary_matmul(_p(lhs, C.c_float), m, k, n, _p(rhs_q, C.c_int8), float(gamma), _p(out, C.c_float))
    return out


# ---- two-level schemes: block scales in a narrow dtype + one f32 per-tensor scale -------------------

def normalize_scales(scales, block_dtype):
    """normalize_scales (burn-backend/src/quantization/scheme.rs:106-134) -> (relative block scales, global)."""
    a = np.ascontiguousarray(scales, dtype=np.float32).copy()
    g = lib().bqo_normalize_scales(_p(a.reshape(-1), C.c_float), a.size, block_dtype)
    if g != g:
        raise ValueError("block scales of this dtype reach f32's range, which a per-tensor scale cannot absorb")
    return a, np.float32(g)


def two_level_scales(block_scales, block_dtype, global_scale):
    """(stored block scales, scale each block is quantized against = global * stored)."""
    a = np.ascontiguousarray(block_scales, dtype=np.float32)
    stored, eff = np.empty_like(a), np.empty_like(a)
    lib().bqo_two_level_scales(_p(a.reshape(-1), C.c_float), a.size, block_dtype, float(global_scale),
                               _p(stored.reshape(-1), C.c_float), _p(eff.reshape(-1), C.c_float))
    return stored, eff


def quantize_two_level(x, scheme, block_scales, global_scale, block_dtype):
    """NdArray::quantize with QuantizationParametersPrimitive { scales, global: Some(..) }:
    -> (values, stored block scales, effective scales)."""
    stored, eff = two_level_scales(block_scales, block_dtype, global_scale)
    return quantize(x, scheme, eff), stored, eff


def quantize_dynamic_two_level(x, scheme, block_dtype):
    """quantize_dynamic of a two-level scheme: range -> one-level f32 block scales -> normalize_scales
    -> quantize. -> (values, stored block scales, global, effective scales)."""
    _, scales = quantize_dynamic(x, scheme)
    rel, g = normalize_scales(scales, block_dtype)
    q, stored, eff = quantize_two_level(x, scheme, rel, g, block_dtype)
    return q, stored, g, eff


def encode_two_level(q, scheme, stored, global_scale, block_dtype):
    """QuantizedBytes::new for a two-level scheme: values || block scales in their dtype || f32 global."""
    blob = encode_with_scale_dtype(q, scheme, stored, block_dtype)
    return np.concatenate([blob, np.float32([global_scale]).view(np.uint8)])
