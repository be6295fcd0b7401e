"""Vectorised numpy restatement of the same reference semantics. TEST INFRASTRUCTURE ONLY.

Written independently of ``bq_oracle.c``: blocks are handled the way ``reduce_blocks`` does
(burn-backend/src/quantization/scheme.rs:14-41: view the tensor as ``[n0, b0, n1, b1, ...]``)
instead of through ``block_of``, so a wrong block index in one restatement shows up as a
disagreement with the other. All arithmetic is carried out in float32 with numpy's
correctly-rounded elementwise operations.
"""
from __future__ import annotations

import numpy as np

RANGES = {"Q8S": (-127.0, 127.0), "Q4S": (-7.0, 7.0), "Q2S": (-1.0, 1.0),
          "Q8F": (-128.0, 127.0), "Q4F": (-8.0, 7.0), "Q2F": (-2.0, 1.0)}
BITS = {"Q8S": 8, "Q4S": 4, "Q2S": 2, "Q8F": 8, "Q4F": 4, "Q2F": 2}


def _block_dims(shape, block):
    """BlockSize::to_dim_vec: trailing-aligned block extents, leading dims 1."""
    rank = len(shape)
    dims = [1] * rank
    for j in range(min(len(block), rank)):
        dims[rank - 1 - j] = block[len(block) - 1 - j]
    return dims


def _split_view(x, block):
    dims = _block_dims(x.shape, block)
    split = []
    for d, b in zip(x.shape, dims):
        if d % b:
            raise ValueError(f"tensor {x.shape} not divisible by block {dims}")
        split += [d // b, b]
    return x.reshape(split), tuple(range(1, len(split), 2))


def compute_range(x, block=None):
    """compute_range(MinMax) -- scheme.rs:44-56."""
    x = np.asarray(x, np.float32)
    if block is None:
        return x.min().reshape(1), x.max().reshape(1)
    v, axes = _split_view(x, block)
    return v.min(axis=axes), v.max(axis=axes)


def compute_range_abs_mean(x, block=None):
    """compute_range(AbsMean) -- scheme.rs:57-69: gamma = mean |x| per tensor or per block rectangle,
    range (-gamma, +gamma). The sum is taken in binary64 and rounded once."""
    x = np.asarray(x, np.float32)
    a = np.abs(x.astype(np.float64))
    if block is None:
        g = np.float32(a.mean()).reshape(1)
    else:
        v, axes = _split_view(a, block)
        g = v.mean(axis=axes).astype(np.float32)
    return -g, g


def compute_q_params(lo, hi, value="Q8S"):
    """compute_q_params -- scheme.rs:75-93."""
    a, b = RANGES[value]
    lo_abs = np.abs(np.asarray(lo, np.float32))
    hi_abs = np.abs(np.asarray(hi, np.float32))
    alpha = np.where(lo_abs < hi_abs, hi_abs, lo_abs).astype(np.float32)
    rng = alpha * np.float32(2.0)
    return (rng / np.float32(b - a)).astype(np.float32)


def _round_half_away(v32):
    v = v32.astype(np.float64)  # exact widening; v +/- 0.5 is exact in binary64
    return np.where(v >= 0, np.floor(v + 0.5), np.ceil(v - 0.5))


def _expand_scales(scales, shape, block):
    """One scale per element: repeat each block scale over its rectangle."""
    if block is None:
        return np.float32(np.asarray(scales, np.float32).reshape(-1)[0])
    dims = _block_dims(shape, block)
    s = np.asarray(scales, np.float32).reshape([d // b for d, b in zip(shape, dims)])
    for ax, b in enumerate(dims):
        if b > 1:
            s = np.repeat(s, b, axis=ax)
    return s


def quantize(x, scales, value="Q8S", block=None):
    """NdArray::quantize -- qtensor.rs:82-186, quantization.rs:128-133."""
    x = np.asarray(x, np.float32)
    a, b = RANGES[value]
    s = _expand_scales(scales, x.shape, block)
    s = np.where(s == 0, np.float32(0.1), s).astype(np.float32)
    with np.errstate(all="ignore"):
        quot = (x / s).astype(np.float32)
    return np.clip(_round_half_away(quot), a, b).astype(np.int8)


def quantize_dynamic(x, value="Q8S", block=None):
    lo, hi = compute_range(x, block)
    scales = compute_q_params(lo, hi, value)
    return quantize(x, scales, value, block), scales


def dequantize(q, scales, block=None):
    """NdArray::dequantize -- scale * (f32) q with valid_scale applied (tensor.rs:716-737)."""
    q = np.asarray(q, np.int8)
    s = _expand_scales(scales, q.shape, block)
    s = np.where(s == 0, np.float32(0.1), s).astype(np.float32)
    return (s * q.astype(np.float32)).astype(np.float32)


def pack_u32(q, value="Q8S"):
    """Words along the innermost dim, value j in bits [j*w, (j+1)*w) -- burn-std quantization.rs:514-542."""
    q = np.asarray(q, np.int8)
    bits = BITS[value]
    nq = 32 // bits
    last = q.shape[-1]
    pad = (-last) % nq
    if pad:
        q = np.concatenate([q, np.zeros(q.shape[:-1] + (pad,), np.int8)], axis=-1)
    u = (q.astype(np.int64) & ((1 << bits) - 1)).reshape(q.shape[:-1] + (-1, nq))
    shifts = (np.arange(nq, dtype=np.int64) * bits)
    return (u << shifts).sum(axis=-1).astype(np.uint32)


def unpack_u32(words, shape, value="Q8S"):
    bits = BITS[value]
    nq = 32 // bits
    w = np.asarray(words, np.uint32).astype(np.int64).reshape(tuple(shape[:-1]) + (-1, 1))
    shifts = np.arange(nq, dtype=np.int64) * bits
    raw = (w >> shifts) & ((1 << bits) - 1)
    raw = np.where(raw >= (1 << (bits - 1)), raw - (1 << bits), raw)
    return raw.reshape(tuple(shape[:-1]) + (-1,))[..., : shape[-1]].astype(np.int8)


def q_matmul_f64(lhs, q, scales, block=None):
    """x . dequantize(w) evaluated in float64 -- the yardstick for the 1e-2 q_matmul bound."""
    w = dequantize(q, scales, block).astype(np.float64)
    return np.asarray(lhs, np.float64) @ w


def q_linear_f64(x, q, scales, block=None, bias=None):
    """linear with a quantized weight (crates/burn-tensor/src/tensor/module.rs:527-567): the
    leading dims of x fold into rows, x @ dequantize(w), then + bias; float64 yardstick."""
    x = np.asarray(x, np.float64)
    out = q_matmul_f64(x.reshape(-1, x.shape[-1]), q, scales, block)
    if bias is not None:
        out = out + np.asarray(bias, np.float64)[None, :]
    return out.reshape(x.shape[:-1] + (out.shape[-1],))


def q_permute(q, scales, block, axes):
    """NdArray q_permute (crates/burn-ndarray/src/ops/qtensor.rs:310-336): the values are
    permuted; with a block scheme the scales, laid out in params_shape order, are permuted the same
    way and the block extents move with their dims (scheme.permute_block_dims). Returns
    (values, scales, block); block extents are returned padded to the rank."""
    q = np.asarray(q)
    axes = [a % q.ndim for a in axes]
    if sorted(axes) != list(range(q.ndim)):
        raise ValueError("axes must be a permutation")
    if block is None:
        return np.transpose(q, axes).copy(), np.asarray(scales, np.float32), None
    blk = [1] * (q.ndim - len(block)) + list(block)
    params = tuple(d // b for d, b in zip(q.shape, blk))
    s = np.transpose(np.asarray(scales, np.float32).reshape(params), axes).copy()
    return np.transpose(q, axes).copy(), s.reshape(-1), [blk[a] for a in axes]


def q_flip(q, scales, axes):
    """NdArray q_flip (qtensor.rs:338-347): the values are flipped, the parameters kept."""
    return np.flip(np.asarray(q), axis=tuple(axes)).copy(), np.asarray(scales, np.float32)


def scale_to_dtype(scales, dtype="F32"):
    """scale_to_dtype (crates/burn-std/src/tensor/quantization.rs:354-368): smallest value of the
    scale dtype that is no smaller. A second, independent restatement: numpy's own f16 conversion
    (round to nearest even) stepped up with nextafter where it fell below; bf16 through bit masks.
    A finite value past the largest finite one saturates to it."""
    s = np.asarray(scales, np.float32)
    if dtype == "F32":
        return s.copy()
    if dtype == "F16":
        with np.errstate(over="ignore"):
            h = s.astype(np.float16)
            below = h.astype(np.float32) < s
            h = np.where(below, np.nextafter(h, np.float16(np.inf)), h)
        out = h.astype(np.float32)
        big = np.float32(65504.0)
        out = np.where(np.isfinite(s) & (out == np.inf), big, out)
        return np.where(np.isfinite(s) & (out == -np.inf), -big, out).astype(np.float32)
    if dtype == "BF16":
        u = s.view(np.uint32).astype(np.uint64)
        low = u & 0xFFFF
        neg = (u >> 31) == 1
        up = np.where(neg, u & 0xFFFF0000, (u + 0xFFFF) & 0xFFFF0000)
        r = np.where(low == 0, u, up)
        r = np.where(np.isfinite(s) & ((r & 0x7FFFFFFF) >= 0x7F800000), (r & 0x80000000) | 0x7F7F0000, r)
        r = np.where(np.isfinite(s), r, u)
        return r.astype(np.uint32).view(np.float32)
    if dtype == "UE4M3":
        # the 127 non-negative e4m3 values in ascending order, then a search: an independent route
        # to "the smallest representable value that is no smaller"
        table = ue4m3_values()
        idx = np.searchsorted(table, s.astype(np.float64), side="left")
        out = table[np.minimum(idx, table.size - 1)].astype(np.float32)      # past 448: saturates
        out = np.where(s > 0, out, np.float32(0))
        return np.where(np.isfinite(s), out, s).astype(np.float32)
    raise ValueError(dtype)


def ue4m3_values():
    """Every value of the non-negative half of OCP e4m3 (bits 0x00 .. 0x7E), ascending, as float64:
    m * 2^-9 for exponent field 0, (1 + m/8) * 2^(e - 7) otherwise."""
    bits = np.arange(0x7F)
    e, m = bits >> 3, bits & 7
    return np.where(e == 0, m * 2.0 ** -9, (1 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7))


def quantize_dynamic_two_level(x, value="Q8S", block=None, block_dtype="F16"):
    """quantize_dynamic under a two-level scheme, a second restatement in numpy f32 arithmetic:
    compute_q_params + normalize_scales (crates/burn-backend/src/quantization/scheme.rs:75-134), then
    NdArray::quantize against global * scale_to_dtype(relative block scale)
    (crates/burn-ndarray/src/ops/qtensor.rs:90-101, 519-531).
    -> (values, stored block scales, global, effective scales)."""
    if block_dtype not in ("F16", "UE4M3"):
        raise ValueError("block scales of this dtype reach f32's range, which a per-tensor scale cannot absorb")
    top = np.float32(65504.0 if block_dtype == "F16" else 448.0)
    lo, hi = compute_range(x, block)
    scales = compute_q_params(lo, hi, value).astype(np.float32)
    g = np.maximum(np.float32(scales.max()) / top, np.float32(1.17549435e-38)).astype(np.float32)
    rel = (scales / g).astype(np.float32)
    stored = scale_to_dtype(rel, block_dtype)
    eff = (g * stored).astype(np.float32)
    return quantize(x, eff, value, block), stored, np.float32(g), eff


def ternary_matmul(lhs, q, gamma):
    """crates/burn-ndarray/src/ops/qtensor.rs:431-517: +1 adds, -1 subtracts, anything else is
    skipped, in ascending k; the per-tensor scale multiplies the finished sums."""
    lhs = np.asarray(lhs, np.float32)
    out = np.zeros((lhs.shape[0], q.shape[1]), np.float32)
    for k in range(lhs.shape[1]):
        x = lhs[:, k:k + 1]
        out = np.where(q[k] == 1, out + x, np.where(q[k] == -1, out - x, out)).astype(np.float32)
    return out * np.float32(gamma)
