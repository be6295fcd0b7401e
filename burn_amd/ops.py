"""Host-side mirror of burn's `QTensorOps` for the MI355X backend.

Each method forwards to the C ABI function of the same name in libburnq_mi355.so; nothing is
computed here. Method names, argument order and error behaviour follow
crates/burn-backend/src/backend/ops/qtensor.rs:123-1324 (where the reference panics, a
`BurnqError` is raised). numpy only carries host bytes in and out.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import numpy as np

from . import _lib
from ._lib import BF16, F32, QFLOAT, check, lib
from .quantization import QuantScheme, params_shape


def _shape_arg(shape):
    shape = tuple(int(d) for d in shape)
    return (C.c_size_t * max(len(shape), 1))(*shape), len(shape)


class Device:
    """One MI355X: the counterpart of a backend `Device`. `Device(0)` opens GPU 0."""

    def __init__(self, ordinal: int = 0):
        h = C.c_void_p()
        check(lib().bq_device_open(ordinal, C.byref(h)))
        self.handle = h
        self.ordinal = ordinal

    @staticmethod
    def count() -> int:
        n = C.c_int32()
        check(lib().bq_device_count(C.byref(n)))
        return n.value

    def sync(self):
        """Backend::sync(device)."""
        check(lib().bq_device_sync(self.handle))

    def trim(self):
        check(lib().bq_device_trim(self.handle))

    def set_validate(self, on: bool):
        """Validate mode: quantize fails with ERR_NONFINITE where the reference panics on a NaN
        quotient (NaN input or scale, infinite input against an infinite scale)."""
        check(lib().bq_device_set_validate(self.handle, 1 if on else 0))

    def set_f32_matmul_exact(self, on: bool):
        """f32 activations with more than 32 rows: multiply the reference's way (dequantize to
        f32, f32 product) instead of the bf16 matrix-core kernel."""
        check(lib().bq_device_set_f32_matmul_exact(self.handle, 1 if on else 0))

    @property
    def stream(self) -> int:
        return lib().bq_device_stream(self.handle) or 0

    def capture(self, fn):
        """Records the kernels `fn()` enqueues into a HIP graph instead of running them.
        Returns (graph, whatever fn returned); keep the tensors fn created alive while the
        graph is replayed."""
        check(lib().bq_graph_begin_capture(self.handle))
        try:
            result = fn()
        finally:
            g = C.c_void_p()
            status = lib().bq_graph_end_capture(self.handle, C.byref(g))
        check(status)
        return Graph(g, self), result

    def timer_start(self):
        check(lib().bq_timer_start(self.handle))

    def timer_stop(self) -> float:
        ms = C.c_float()
        check(lib().bq_timer_stop(self.handle, C.byref(ms)))
        return ms.value


class Graph:
    """A captured HIP graph of library calls (see Device.capture)."""

    def __init__(self, handle, device: Device):
        self.handle = handle
        self.device = device

    def launch(self):
        check(lib().bq_graph_launch(self.handle))

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            try:
                lib().bq_graph_release(h)
            except Exception:
                pass


class Tensor:
    """Owns one reference of a bq_tensor handle (float or quantized primitive)."""

    def __init__(self, handle, device: Device):
        self.handle = handle
        self.device = device

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            try:
                lib().bq_tensor_release(h)
            except Exception:
                pass

    @property
    def shape(self):
        rank = lib().bq_tensor_rank(self.handle)
        out = (C.c_size_t * max(rank, 1))()
        check(lib().bq_tensor_shape(self.handle, out))
        return tuple(out[i] for i in range(rank))

    @property
    def dtype(self) -> int:
        return lib().bq_tensor_dtype(self.handle)

    @property
    def is_quantized(self) -> bool:
        return self.dtype == QFLOAT

    @property
    def scheme(self) -> QuantScheme:
        c = _lib.CScheme()
        check(lib().bq_tensor_scheme(self.handle, C.byref(c)))
        return QuantScheme.from_c(c)

    @property
    def data_ptr(self) -> int:
        return lib().bq_tensor_data_ptr(self.handle) or 0

    @property
    def scales_ptr(self) -> int:
        return lib().bq_tensor_scales_ptr(self.handle) or 0

    @property
    def num_scales(self) -> int:
        return lib().bq_tensor_num_scales(self.handle)


def _wrap(handle, device):
    return Tensor(handle, device)


def bf16_bits_from_f32(x: np.ndarray) -> np.ndarray:
    """Host helper: f32 -> bf16 bit patterns, round to nearest even (for building bf16 inputs)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def f32_from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


class FloatOps:
    """The slice of FloatTensorOps the quantized path needs."""

    @staticmethod
    def float_from_data(data: np.ndarray, device: Device, dtype: int = F32) -> Tensor:
        if dtype == F32:
            host = np.ascontiguousarray(data, np.float32)
        elif dtype == BF16:
            host = np.ascontiguousarray(data)
            if host.dtype != np.uint16:  # float input: round to bf16 on the host
                host = bf16_bits_from_f32(host.astype(np.float32)).reshape(host.shape)
        else:
            raise ValueError("dtype must be F32 or BF16")
        sh, rank = _shape_arg(host.shape)
        h = C.c_void_p()
        check(lib().bq_float_from_data(device.handle, host.ctypes.data, dtype, sh, rank, C.byref(h)))
        return _wrap(h, device)

    @staticmethod
    def float_into_data(t: Tensor) -> np.ndarray:
        """f32 tensors come back as float32, bf16 tensors as their uint16 bit patterns."""
        if t.dtype == F32:
            out = np.empty(t.shape, np.float32)
        elif t.dtype == BF16:
            out = np.empty(t.shape, np.uint16)
        else:
            raise _lib.BurnqError(_lib.ERR_DTYPE, "float_into_data on a quantized tensor")
        check(lib().bq_float_into_data(t.handle, out.ctypes.data, out.nbytes))
        return out

    @staticmethod
    def float_empty(shape, device: Device, dtype: int = F32) -> Tensor:
        sh, rank = _shape_arg(shape)
        h = C.c_void_p()
        check(lib().bq_float_empty(device.handle, dtype, sh, rank, C.byref(h)))
        return _wrap(h, device)

    @staticmethod
    def float_from_device_ptr(ptr: int, shape, device: Device, dtype: int = F32) -> Tensor:
        sh, rank = _shape_arg(shape)
        h = C.c_void_p()
        check(lib().bq_float_from_device_ptr(device.handle, C.c_void_p(ptr), dtype, sh, rank,
                                             C.byref(h)))
        return _wrap(h, device)

    @staticmethod
    def float_matmul(lhs: Tensor, rhs: Tensor) -> Tensor:
        h = C.c_void_p()
        check(lib().bq_float_matmul(lhs.handle, rhs.handle, C.byref(h)))
        return _wrap(h, lhs.device)


def f32_from_e4m3_bits(bits) -> np.ndarray:
    """OCP e4m3 bytes -> f32, exactly (e4m3::from_bits(b).to_f32(),
    crates/burn-std/src/tensor/quantization.rs:437): bias 7, 3 mantissa bits, subnormals m * 2^-9,
    0x7F / 0xFF NaN."""
    b = np.asarray(bits, np.uint8).astype(np.int64)
    e, m = (b >> 3) & 0xF, b & 7
    v = np.where(e == 0, m * 2.0 ** -9, (1 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7))
    v = np.where((e == 15) & (m == 7), np.nan, v)
    return np.where(b & 0x80, -v, v).astype(np.float32)


class TensorData:
    """bytes + shape + scheme: the QFloat TensorData blob (values || block scales, dense)."""

    def __init__(self, data: np.ndarray, shape, scheme: QuantScheme):
        self.bytes = np.ascontiguousarray(data, np.uint8)
        self.shape = tuple(int(d) for d in shape)
        self.scheme = scheme

    @staticmethod
    def data_len(shape, scheme: QuantScheme) -> int:
        sh, rank = _shape_arg(shape)
        n = C.c_size_t()
        c = scheme.to_c()
        check(lib().bq_quantized_data_len(C.byref(c), sh, rank, C.byref(n)))
        return n.value

    def global_scale(self):
        """The per-tensor scale of a two-level blob (its last four bytes), else None."""
        if self.scheme.tensor_scale is None:
            return None
        return self.bytes[self.bytes.size - 4:].copy().view(np.float32)[0]

    def split(self):
        """(values bytes, scales as f32) -- the two regions of the blob. 2-byte scales (f16 / bf16)
        are widened exactly (decode_scales, crates/burn-std/src/tensor/quantization.rs:418-441). A
        two-level blob ends with its per-tensor scale (`global_scale`), which is not part of them."""
        from .quantization import ScaleDtype
        pshape = params_shape(self.shape, self.scheme)
        n_scales = int(np.prod(pshape))
        end = self.bytes.size - (0 if self.scheme.tensor_scale is None else 4)
        cut = end - self.scheme.scale_dtype.size() * n_scales
        raw = self.bytes[cut:end]
        if self.scheme.scale_dtype == ScaleDtype.F32:
            scales = raw.copy().view(np.float32)
        elif self.scheme.scale_dtype == ScaleDtype.F16:
            scales = raw.copy().view(np.float16).astype(np.float32)
        elif self.scheme.scale_dtype == ScaleDtype.UE4M3:
            scales = f32_from_e4m3_bits(raw)
        else:
            scales = f32_from_bf16_bits(raw.copy().view(np.uint16))
        return self.bytes[:cut], scales.reshape(pshape)


class QTensorOps:
    """burn's QTensorOps for the MI355X backend (hot-path subset + layout ops)."""

    @staticmethod
    def q_from_data(data: TensorData, device: Device) -> Tensor:
        sh, rank = _shape_arg(data.shape)
        c = data.scheme.to_c()
        h = C.c_void_p()
        check(lib().bq_q_from_data(device.handle, data.bytes.ctypes.data, data.bytes.size, sh, rank,
                                   C.byref(c), C.byref(h)))
        return _wrap(h, device)

    @staticmethod
    def q_into_data(t: Tensor) -> TensorData:
        n = C.c_size_t()
        scheme = t.scheme
        out = np.empty(TensorData.data_len(t.shape, scheme), np.uint8)
        check(lib().bq_q_into_data(t.handle, out.ctypes.data, out.size, C.byref(n)))
        return TensorData(out[: n.value], t.shape, scheme)

    @staticmethod
    def quantize(tensor: Tensor, scheme: QuantScheme, scales: Tensor, global_scale: Optional[Tensor] = None) -> Tensor:
        """quantize(tensor, scheme, qparams): `global_scale` is qparams.global, the one-element f32
        tensor a two-level scheme takes besides its block scales."""
        c = scheme.to_c()
        h = C.c_void_p()
        if global_scale is None:
            check(lib().bq_quantize(tensor.handle, C.byref(c), scales.handle, C.byref(h)))
        else:
            check(lib().bq_quantize_two_level(tensor.handle, C.byref(c), scales.handle, global_scale.handle, C.byref(h)))
        return _wrap(h, tensor.device)

    @staticmethod
    def quantize_dynamic(tensor: Tensor, scheme: QuantScheme) -> Tensor:
        c = scheme.to_c()
        h = C.c_void_p()
        check(lib().bq_quantize_dynamic(tensor.handle, C.byref(c), C.byref(h)))
        return _wrap(h, tensor.device)

    @staticmethod
    def compute_range_abs_mean(tensor: Tensor, scheme: QuantScheme) -> Tensor:
        """compute_range(scheme, tensor, Calibration::AbsMean) (crates/burn-backend/src/quantization/scheme.rs:57-69):
        gamma = mean |x| per tensor or per block; the range is (-gamma, +gamma). Returns gamma."""
        c = scheme.to_c()
        h = C.c_void_p()
        check(lib().bq_compute_range_abs_mean(tensor.handle, C.byref(c), C.byref(h)))
        return _wrap(h, tensor.device)

    @staticmethod
    def quantize_abs_mean(tensor: Tensor, scheme: QuantScheme) -> Tensor:
        """The Quantizer's compute_range -> compute_q_params -> quantize under Calibration::AbsMean
        (crates/burn-core/src/module/quantize.rs:47-49)."""
        c = scheme.to_c()
        h = C.c_void_p()
        check(lib().bq_quantize_abs_mean(tensor.handle, C.byref(c), C.byref(h)))
        return _wrap(h, tensor.device)

    @staticmethod
    def dequantize(tensor: Tensor, dtype: int = F32) -> Tensor:
        h = C.c_void_p()
        check(lib().bq_dequantize(tensor.handle, dtype, C.byref(h)))
        return _wrap(h, tensor.device)

    @staticmethod
    def q_matmul(lhs: Tensor, rhs: Tensor, out_dtype: Optional[int] = None) -> Tensor:
        h = C.c_void_p()
        if out_dtype is None:
            check(lib().bq_q_matmul(lhs.handle, rhs.handle, C.byref(h)))
        else:
            check(lib().bq_q_matmul_as(lhs.handle, rhs.handle, out_dtype, C.byref(h)))
        return _wrap(h, lhs.device)

    @staticmethod
    def q_matmul_propagate(lhs: Tensor, rhs: Tensor) -> Tensor:
        """q_matmul with QuantPropagation::Propagate: the product comes back quantized with the
        quantized operand's scheme (crates/burn-ndarray/src/ops/qtensor.rs:262-265)."""
        h = C.c_void_p()
        check(lib().bq_q_matmul_propagate(lhs.handle, rhs.handle, C.byref(h)))
        return _wrap(h, lhs.device)

    @staticmethod
    def q_to_device(t: Tensor, device: Device) -> Tensor:
        h = C.c_void_p()
        check(lib().bq_q_to_device(t.handle, device.handle, C.byref(h)))
        return _wrap(h, device)

    @staticmethod
    def q_reshape(t: Tensor, shape) -> Tensor:
        sh, rank = _shape_arg(shape)
        h = C.c_void_p()
        check(lib().bq_q_reshape(t.handle, sh, rank, C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_swap_dims(t: Tensor, dim1: int, dim2: int) -> Tensor:
        h = C.c_void_p()
        check(lib().bq_q_swap_dims(t.handle, dim1, dim2, C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_permute(t: Tensor, axes: Sequence[int]) -> Tensor:
        arr = (C.c_int32 * max(len(axes), 1))(*axes)
        h = C.c_void_p()
        check(lib().bq_q_permute(t.handle, arr, len(axes), C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_slice(t: Tensor, slices) -> Tensor:
        """slices: one per leading dim, each a Python slice or an int (a single index keeps the dim, as
        burn's s![] does); burn's Slice semantics (negative indices, clamping, negative steps)."""
        n = len(slices)
        starts, ends, steps = (C.c_int64 * max(n, 1))(), (C.c_int64 * max(n, 1))(), (C.c_int64 * max(n, 1))()
        for i, s in enumerate(slices):
            if isinstance(s, int):                     # Slice::index: idx .. idx + 1 (None for -1)
                s = slice(s, None if s == -1 else s + 1, 1)
            step = 1 if s.step is None else s.step
            starts[i] = 0 if s.start is None else s.start
            ends[i] = (2 ** 63 - 1) if s.stop is None else s.stop
            steps[i] = step
        h = C.c_void_p()
        check(lib().bq_q_slice(t.handle, starts, ends, steps, n, C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_select(t: Tensor, dim: int, indices: Tensor) -> Tensor:
        h = C.c_void_p()
        check(lib().bq_q_select(t.handle, dim, indices.handle, C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_gather(dim: int, t: Tensor, indices: Tensor) -> Tensor:
        h = C.c_void_p()
        check(lib().bq_q_gather(dim, t.handle, indices.handle, C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_expand(t: Tensor, shape) -> Tensor:
        sh, rank = _shape_arg(shape)
        h = C.c_void_p()
        check(lib().bq_q_expand(t.handle, sh, rank, C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_argmax(t: Tensor, dim: int, out_dtype: int = _lib.I64) -> Tensor:
        h = C.c_void_p()
        check(lib().bq_q_argmax(t.handle, dim, out_dtype, C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_argmin(t: Tensor, dim: int, out_dtype: int = _lib.I64) -> Tensor:
        h = C.c_void_p()
        check(lib().bq_q_argmin(t.handle, dim, out_dtype, C.byref(h)))
        return _wrap(h, t.device)

    @staticmethod
    def q_flip(t: Tensor, axes: Sequence[int]) -> Tensor:
        arr = (C.c_int32 * max(len(axes), 1))(*axes)
        h = C.c_void_p()
        check(lib().bq_q_flip(t.handle, arr, len(axes), C.byref(h)))
        return _wrap(h, t.device)


class IntOps:
    """The slice of IntTensorOps the quantized index ops need (int_from_data / int_into_data)."""

    @staticmethod
    def int_from_data(data: np.ndarray, device: Device) -> Tensor:
        data = np.ascontiguousarray(data)
        if data.dtype not in (np.int32, np.int64):
            raise TypeError("index tensors are int32 or int64")
        shape, rank = _shape_arg(data.shape)
        h = C.c_void_p()
        check(lib().bq_int_from_data(device.handle, data.ctypes.data, _lib.I32 if data.dtype == np.int32 else _lib.I64,
                                     shape, rank, C.byref(h)))
        return _wrap(h, device)

    @staticmethod
    def int_into_data(t: Tensor) -> np.ndarray:
        out = np.empty(t.shape, np.int32 if t.dtype == _lib.I32 else np.int64)
        check(lib().bq_int_into_data(t.handle, out.ctypes.data, out.nbytes))
        return out


class ModuleOps:
    """`linear` of crates/burn-tensor/src/tensor/module.rs:527-567 for a quantized weight: what
    `nn::Linear::forward` (crates/burn-nn/src/modules/linear.rs:128-134) computes once
    `Module::quantize_weights` (crates/burn-core/src/module/quantize.rs:40-53) has replaced the
    weight by a QFloat tensor."""

    @staticmethod
    def linear(input: Tensor, weight: Tensor, bias: Optional[Tensor] = None,
               out_dtype: Optional[int] = None) -> Tensor:
        """y = x @ weight + [bias]; x is [.., d_input], weight [d_input, d_output] (not transposed,
        as in the reference), bias [d_output]. The bias is added by the kernel that writes y."""
        h = C.c_void_p()
        check(lib().bq_q_linear(input.handle, weight.handle, bias.handle if bias is not None else None,
                                -1 if out_dtype is None else out_dtype, C.byref(h)))
        return _wrap(h, input.device)


class PackReader:
    """burn-pack's `Reader` over a .bpk container (crates/burn-pack/src/reader.rs): header and
    metadata are parsed, the file stays memory-mapped, tensors load straight into device memory."""

    def __init__(self, source):
        h = C.c_void_p()
        if isinstance(source, (bytes, bytearray, np.ndarray)):
            self._keep = np.frombuffer(bytes(source), np.uint8) if not isinstance(source, np.ndarray) else np.ascontiguousarray(source, np.uint8)
            check(lib().bq_pack_from_bytes(self._keep.ctypes.data, self._keep.size, 0, C.byref(h)))
        else:
            check(lib().bq_pack_open(str(source).encode(), C.byref(h)))
        self.handle = h

    def close(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            lib().bq_pack_close(h)

    __del__ = close

    def __len__(self):
        return lib().bq_pack_num_tensors(self.handle)

    def _entry(self, e):
        scheme = QuantScheme.from_c(e.scheme) if e.has_scheme else None
        return {"name": e.name.decode(), "dtype": _lib.PACK_DTYPES[e.dtype], "shape": tuple(e.shape[i] for i in range(e.rank)),
                "data_offsets": (e.data_begin, e.data_end), "param_id": e.param_id if e.has_param_id else None,
                "scheme": scheme, "data_ptr": e.data}

    def entries(self):
        out = []
        for i in range(len(self)):
            e = _lib.CPackEntry()
            check(lib().bq_pack_entry_at(self.handle, i, C.byref(e)))
            out.append(self._entry(e))
        return out

    def find(self, name):
        e = _lib.CPackEntry()
        check(lib().bq_pack_find(self.handle, name.encode(), C.byref(e)))
        return self._entry(e)

    def metadata(self, key):
        v = lib().bq_pack_metadata(self.handle, key.encode())
        return v.decode() if v is not None else None

    def load(self, name, device: Device, scheme: Optional[QuantScheme] = None) -> Tensor:
        h = C.c_void_p()
        c = scheme.to_c() if scheme is not None else None
        check(lib().bq_pack_load(self.handle, name.encode(), C.byref(c) if c is not None else None, device.handle, C.byref(h)))
        return _wrap(h, device)


class PackWriter:
    """burn-pack's `Writer`: tensors in the order added, 256-byte aligned, descriptors by name."""

    def __init__(self):
        h = C.c_void_p()
        check(lib().bq_pack_writer_new(C.byref(h)))
        self.handle = h

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            lib().bq_pack_writer_free(h)

    def with_metadata(self, key, value):
        check(lib().bq_pack_writer_set_metadata(self.handle, key.encode(), value.encode()))
        return self

    def add_tensor(self, name, t: Tensor, param_id=None):
        check(lib().bq_pack_writer_add_tensor(self.handle, name.encode(), t.handle, 0 if param_id is None else 1, param_id or 0))
        return self

    def add_bytes(self, name, dtype: str, shape, data: np.ndarray, scheme: Optional[QuantScheme] = None, param_id=None):
        sh, rank = _shape_arg(shape)
        buf = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        c = scheme.to_c() if scheme is not None else None
        check(lib().bq_pack_writer_add_bytes(self.handle, name.encode(), _lib.PACK_DTYPES.index(dtype), C.byref(c) if c is not None else None,
                                             sh, rank, buf.ctypes.data if buf.size else None, buf.size,
                                             0 if param_id is None else 1, param_id or 0))
        return self

    def size(self) -> int:
        n = C.c_size_t()
        check(lib().bq_pack_writer_size(self.handle, C.byref(n)))
        return n.value

    def into_bytes(self) -> np.ndarray:
        out = np.empty(self.size(), np.uint8)
        n = C.c_size_t()
        check(lib().bq_pack_writer_write_into(self.handle, out.ctypes.data, out.size, C.byref(n)))
        return out[: n.value]

    def write_to_file(self, path):
        check(lib().bq_pack_writer_write_file(self.handle, str(path).encode()))
