"""Host-side mirror of burn's quantization descriptors (names follow the reference).

`QuantScheme` mirrors cubecl_common::quant::scheme::QuantScheme as burn re-exports it
(crates/burn-std/src/tensor/quantization.rs:4-6), restricted to what this backend implements:
symmetric Q8S / Q4S / Q2S and full-range Q8F / Q4F / Q2F values, per-tensor or per-block scales stored as f32, f16, bf16 or ue4m3, an
optional f32 per-tensor scale on top of block scales (two-level), Native or PackedU32(0) store.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from enum import IntEnum
from typing import Optional, Tuple

from . import _lib


class QuantValue(IntEnum):
    Q8S = _lib.Q8S
    Q4S = _lib.Q4S
    Q2S = _lib.Q2S   # ternary: -1, 0, +1
    Q8F = _lib.Q8F   # full range: -128..127 (the value of the reference's QuantScheme::default())
    Q4F = _lib.Q4F   # -8..7
    Q2F = _lib.Q2F   # -2..1

    def range(self) -> Tuple[float, float]:
        return {QuantValue.Q8S: (-127.0, 127.0), QuantValue.Q4S: (-7.0, 7.0), QuantValue.Q2S: (-1.0, 1.0),
                QuantValue.Q8F: (-128.0, 127.0), QuantValue.Q4F: (-8.0, 7.0), QuantValue.Q2F: (-2.0, 1.0)}[self]

    def size_bits(self) -> int:
        return {QuantValue.Q8S: 8, QuantValue.Q4S: 4, QuantValue.Q2S: 2,
                QuantValue.Q8F: 8, QuantValue.Q4F: 4, QuantValue.Q2F: 2}[self]


class QuantStore(IntEnum):
    Native = _lib.STORE_NATIVE
    PackedU32 = _lib.STORE_PACKED_U32  # packed along the innermost dim: PackedU32(0)


class ScaleDtype(IntEnum):
    F32 = _lib.SCALE_F32
    F16 = _lib.SCALE_F16
    BF16 = _lib.SCALE_BF16
    UE4M3 = _lib.SCALE_UE4M3   # one byte: the non-negative half of OCP e4m3

    def size(self) -> int:
        """scale_size -- crates/burn-std/src/tensor/quantization.rs:409-416."""
        return {ScaleDtype.F32: 4, ScaleDtype.UE4M3: 1}.get(self, 2)


@dataclass(frozen=True)
class QuantScheme:
    """value / level (block None = per tensor) / store / scale dtype / per-tensor scale on top of
    block scales. `QuantScheme()` is per-tensor, PackedU32(0), f32 scales like the reference's
    default, with Q8S values; the reference's own default value is defined in a crate outside its
    tree and is Q8F according to crates/burn-backend-tests/tests/cubecl/quantization/slice.rs:37-38:
    pass `value=QuantValue.Q8F` (or `.with_value`) for that."""

    value: QuantValue = QuantValue.Q8S
    block: Optional[Tuple[int, ...]] = None
    store: QuantStore = QuantStore.PackedU32
    scale_dtype: ScaleDtype = ScaleDtype.F32
    tensor_scale: Optional[ScaleDtype] = None   # block schemes only: two-level (global_scale_dtype)

    def with_value(self, value: QuantValue) -> "QuantScheme":
        return replace(self, value=value)

    def with_store(self, store: QuantStore) -> "QuantScheme":
        return replace(self, store=store)

    def per_block(self, block, scale_dtype: ScaleDtype = ScaleDtype.F32) -> "QuantScheme":
        """Block scales of `scale_dtype` (one level: a per-tensor scale on top is dropped)."""
        return replace(self, block=tuple(int(b) for b in block), scale_dtype=scale_dtype, tensor_scale=None)

    def per_tensor(self, scale_dtype: Optional[ScaleDtype] = None) -> "QuantScheme":
        """A per-tensor scale of `scale_dtype`. On a block scheme it comes on top of the block scales
        (two-level, as `.per_block(b, dt).per_tensor(ScaleDtype::F32)` in the reference) and has to
        be f32 ("a two-level scheme stores its per-tensor scale as f32",
        crates/burn-std/src/tensor/quantization.rs:250-255); otherwise it is the scheme's one scale."""
        dtype = ScaleDtype.F32 if scale_dtype is None and self.block is not None else scale_dtype
        if self.block is not None:
            if dtype != ScaleDtype.F32:
                raise ValueError("a two-level scheme stores its per-tensor scale as f32")
            return replace(self, tensor_scale=ScaleDtype.F32)
        return replace(self, scale_dtype=self.scale_dtype if dtype is None else dtype)

    def per_tensor_only(self, scale_dtype: Optional[ScaleDtype] = None) -> "QuantScheme":
        """Back to one scale for the whole tensor."""
        return replace(self, block=None, tensor_scale=None,
                       scale_dtype=self.scale_dtype if scale_dtype is None else scale_dtype)

    def with_scale_dtype(self, scale_dtype: ScaleDtype) -> "QuantScheme":
        return replace(self, scale_dtype=scale_dtype)

    def supported(self) -> bool:
        """What `Backend::dtype_usage(DType::QFloat(self))` answers: the library implements the
        scheme, and it is `quantizable` (crates/burn-std/src/tensor/quantization.rs:113-128)."""
        try:
            c = self.to_c()
        except ValueError:
            return False
        return _lib.lib().bq_scheme_supported(_lib.C.byref(c)) == _lib.OK

    def num_quants(self) -> int:
        return 32 // self.value.size_bits() if self.store == QuantStore.PackedU32 else 1

    def block_size(self):
        return self.block

    # ---- C ABI image
    def to_c(self) -> _lib.CScheme:
        c = _lib.CScheme()
        c.value = int(self.value)
        c.store = int(self.store)
        c.scale_dtype = int(self.scale_dtype)
        c.tensor_scale = 0 if self.tensor_scale is None else 1
        if self.tensor_scale is not None and self.block is None:
            raise ValueError("a per-tensor scale on top goes with block scales")
        if self.block is None:
            c.level = _lib.LEVEL_TENSOR
            c.block_rank = 0
        else:
            if len(self.block) > _lib.MAX_RANK:
                raise ValueError("block rank too large")
            c.level = _lib.LEVEL_BLOCK
            c.block_rank = len(self.block)
            for i, b in enumerate(self.block):
                if not 0 < b < 256:
                    raise ValueError("block extents are u8, as in the reference's BlockSize")
                c.block[i] = b
        return c

    @classmethod
    def from_c(cls, c: _lib.CScheme) -> "QuantScheme":
        block = None
        if c.level == _lib.LEVEL_BLOCK:
            block = tuple(c.block[i] for i in range(c.block_rank))
        return cls(QuantValue(c.value), block, QuantStore(c.store), ScaleDtype(c.scale_dtype),
                   ScaleDtype.F32 if c.tensor_scale else None)


def params_shape(shape, scheme: QuantScheme):
    """params_shape -- crates/burn-std/src/tensor/quantization.rs:141-146."""
    if scheme.block is None:
        return (1,)
    rank = len(shape)
    dims = [1] * rank
    for j in range(min(len(scheme.block), rank)):
        dims[rank - 1 - j] = scheme.block[len(scheme.block) - 1 - j]
    return tuple(d // b for d, b in zip(shape, dims))
