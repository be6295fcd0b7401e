"""GPU parity: every result of the HIP path, reached through the C ABI, against the CPU oracle.

Bars: quantized integers, packed words, scales and dequantized f32 are compared bit for bit;
bf16 dequantize against the oracle's f32 rounded to nearest even; q_matmul within burn's
permissive tolerance (|y - y'| < max(1e-2 * max(|y|,|y'|), 1e-2)) and max|y - y'| / max|y'| <= 1e-2
against x . dequantize(W) evaluated in float64.
"""
import numpy as np
import pytest

from oracle import c_oracle as co
from oracle import np_oracle as no
from conftest import burn_approx_eq

pytestmark = pytest.mark.gpu

import burn_amd as ba  # noqa: E402
from burn_amd import FloatOps, IntOps, ModuleOps, QTensorOps, QuantScheme, QuantStore, QuantValue, TensorData  # noqa: E402
from burn_amd.quantization import ScaleDtype  # noqa: E402

VAL = {QuantValue.Q8S: (co.Q8S, "Q8S"), QuantValue.Q4S: (co.Q4S, "Q4S"), QuantValue.Q2S: (co.Q2S, "Q2S"),
       QuantValue.Q8F: (co.Q8F, "Q8F"), QuantValue.Q4F: (co.Q4F, "Q4F"), QuantValue.Q2F: (co.Q2F, "Q2F")}


@pytest.fixture(scope="module")
def dev():
    return ba.Device(0)


def oscheme(s: QuantScheme):
    store = co.STORE_NATIVE if s.store == QuantStore.Native else co.STORE_PACKED_U32
    return co.Scheme.make(VAL[s.value][0], list(s.block) if s.block else None, store)


def gpu_quantize_dynamic(dev, x, scheme):
    q = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
    return q, QTensorOps.q_into_data(q)


def unpack_blob(blob: TensorData):
    values, scales = blob.split()
    s = blob.scheme
    if s.store == QuantStore.Native:
        q = values.view(np.int8).reshape(blob.shape)
    else:
        q = no.unpack_u32(values.view(np.uint32), blob.shape, VAL[s.value][1])
    return q, scales


def check_quantize_dynamic(dev, x, scheme, mt=False):
    """GPU quantize_dynamic + dequantize of x against the oracle, all bit for bit."""
    tq, blob = gpu_quantize_dynamic(dev, x, scheme)
    q_ref, s_ref = co.quantize_dynamic(x, oscheme(scheme), mt=mt)
    q_gpu, s_gpu = unpack_blob(blob)
    assert s_gpu.shape == s_ref.shape
    assert s_gpu.tobytes() == s_ref.tobytes(), "scales differ"
    bad = np.argwhere(q_gpu != q_ref)
    assert bad.size == 0, f"{len(bad)} quantized values differ, first {bad[:3].tolist()}"
    # the blob is exactly what the oracle serialises
    assert blob.bytes.tobytes() == co.encode(q_ref, oscheme(scheme), s_ref).tobytes()
    d_gpu = FloatOps.float_into_data(QTensorOps.dequantize(tq))
    d_ref = co.dequantize(q_ref, oscheme(scheme), s_ref, mt=mt)
    assert d_gpu.tobytes() == d_ref.tobytes(), "dequantized floats differ"
    return tq, q_ref, s_ref, d_ref


def awkward(shape, seed, outliers=True):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(shape).astype(np.float32)
    if outliers:
        x[rng.random(shape) < 0.01] *= 50
    return x


# ------------------------------------------------------------------ reference KATs on the GPU

def test_kat_quantize_dynamic_int8(dev, kats):
    k = kats["quantize_dynamic_int8"]
    for store in (QuantStore.Native, QuantStore.PackedU32):
        _, blob = gpu_quantize_dynamic(dev, np.float32(k["x"]), QuantScheme(store=store))
        q, s = unpack_blob(blob)
        assert q.tolist() == k["expected_q"]
        assert s.tobytes() == np.float32([k["expected_scale"]]).tobytes()


def test_kat_explicit_scale_and_dequantize(dev, kats):
    k = kats["quantize_explicit_scale"]
    x = FloatOps.float_from_data(np.float32(k["x"]), dev)
    scales = FloatOps.float_from_data(np.float32([k["scale"]]), dev)
    for store in (QuantStore.Native, QuantStore.PackedU32):
        t = QTensorOps.quantize(x, QuantScheme(store=store), scales)
        q, s = unpack_blob(QTensorOps.q_into_data(t))
        assert q.tolist() == k["expected_q"] and s.tobytes() == np.float32([k["scale"]]).tobytes()
    k = kats["int8_symmetric_quantization"]
    blob = co.encode(np.int8(k["expected_q"]), oscheme(QuantScheme(store=QuantStore.Native)),
                     co.compute_q_params(np.float32([-1.8]), np.float32([0.5]), co.Q8S))
    t = QTensorOps.q_from_data(TensorData(blob, (4,), QuantScheme(store=QuantStore.Native)), dev)
    d = FloatOps.float_into_data(QTensorOps.dequantize(t))
    assert d.tobytes() == np.float32(k["expected_d"]).tobytes()


def test_kat_q4s_arange_words(dev, kats):
    k = kats["unpack_q4s_arange"]
    x = np.arange(128, dtype=np.float32)
    _, blob = gpu_quantize_dynamic(dev, x, QuantScheme(value=QuantValue.Q4S))
    values, _ = blob.split()
    assert values.view(np.uint32).tolist() == k["packed"]


def test_kat_blocks_not_spanning_trailing_dim(dev, kats, approx):
    k = kats["blocks_not_spanning_trailing_dim"]
    x = np.float32(k["x"])
    scheme = QuantScheme().per_block(k["block"])
    tq, q_ref, s_ref, d_ref = check_quantize_dynamic(dev, x, scheme)
    approx(s_ref.reshape(-1), np.float32(k["expected_scale_magnitudes"]) / np.float32(127), 1e-3, 0)


def test_kat_data_blobs_roundtrip(dev, kats):
    k = kats["data_per_block_blob"]
    for store in (QuantStore.Native, QuantStore.PackedU32):
        scheme = QuantScheme(store=store).per_block(k["block"])
        blob = co.encode(np.int8(k["values"]), oscheme(scheme), np.float32(k["scales"]))
        t = QTensorOps.q_from_data(TensorData(blob, k["shape"], scheme), dev)
        back = QTensorOps.q_into_data(t)
        assert back.bytes.tobytes() == blob.tobytes()
        t2 = QTensorOps.q_from_data(back, dev)
        assert QTensorOps.q_into_data(t2).bytes.tobytes() == blob.tobytes()
    for case in kats["packed_q4_data_len"]["cases"]:
        if case["shape"][-1] % 8 == 0:
            assert TensorData.data_len(case["shape"], QuantScheme(value=QuantValue.Q4S)) == case["len"]


def test_kat_matmuls(dev, kats, approx):
    k = kats["matmul_lhs_float_rhs_quantized"]
    lhs = FloatOps.float_from_data(np.float32(k["lhs"]), dev)
    rhs = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.float32(k["rhs"]), dev), QuantScheme())
    out = QTensorOps.q_matmul(lhs, rhs)
    assert out.dtype == ba.F32
    approx(FloatOps.float_into_data(out), k["expected"], k["tolerance"]["rel"], k["tolerance"]["abs"])

    k = kats["matmul_mixed_block_scale"]
    rhs = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.float32(k["rhs"]), dev),
                                      QuantScheme().per_block(k["block"]))
    out = QTensorOps.q_matmul(FloatOps.float_from_data(np.float32(k["lhs"]), dev), rhs)
    approx(FloatOps.float_into_data(out), k["expected"], k["tolerance"]["rel"], k["tolerance"]["abs"])

    k = kats["matmul_2d_aligned_qq"]
    ql = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.float32(k["lhs"]), dev), QuantScheme())
    qr = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.float32(k["rhs"]), dev), QuantScheme())
    approx(FloatOps.float_into_data(QTensorOps.q_matmul(ql, qr)), k["expected"], k["tolerance"]["rel"], 0)

    k = kats["matmul_lhs_quantized_rhs_float"]
    ql = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.float32(k["lhs"]), dev), QuantScheme())
    out = QTensorOps.q_matmul(ql, FloatOps.float_from_data(np.float32(k["rhs"]), dev))
    approx(FloatOps.float_into_data(out), k["expected"], k["tolerance"]["rel"], 0)


def test_reference_matmul_cases_both_operands_quantized(dev, approx):
    """crates/burn-backend-tests/tests/tensor/float/quantization/ops/matmul.rs:9-139: products of two
    quantized tensors (`QTensor::int8` = quantize_dynamic, default scheme) against the listed results,
    relative 2e-2 as there. The reference ignores most of them because their last dims do not fill
    packed words; with the Native store they run: vectors, 2-D, 3-D, broadcast batches."""
    native = QuantScheme(store=QuantStore.Native)

    def q(values):
        return QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.float32(values), dev), native)

    def check(a, b, expected):
        out = QTensorOps.q_matmul(q(a), q(b))
        assert out.dtype == ba.F32 and out.shape == np.float32(expected).shape
        approx(FloatOps.float_into_data(out), np.float32(expected), 2e-2, 0)

    check([[1.0, 2.0, 3.0, 6.35]], [[12.7], [4.0], [5.0], [1.0]], [[42.05]])
    check([[1.0, 6.35], [2.0, 3.0], [1.0, 3.0]], [[4.0, 8.0, 12.7], [2.0, 3.0, 6.0]],
          [[16.7, 27.05, 50.8], [14., 25., 43.4], [10., 17., 30.7]])
    check([[[1.0, 6.35], [2.0, 3.0]]], [[[12.7, 4.0], [2.0, 3.0]]], [[[25.4, 23.05], [31.4, 17.0]]])
    check([[[[1.0, 7.0], [2.0, 3.0]]], [[[2.0, 5.0], [6.0, 3.0]]]], [[[[9.0, 8.0], [1.0, 4.0]], [[2.0, 7.0], [3.0, 5.0]]]],
          [[[[16.0, 36.0], [21.0, 28.0]], [[23.0, 42.0], [13.0, 29.0]]],
           [[[23.0, 36.0], [57.0, 60.0]], [[19.0, 39.0], [21.0, 57.0]]]])
    check([[[1.0, 7.0], [2.0, 3.0]]], [[[4.0, 7.0], [2.0, 3.0]], [[2.0, 5.0], [6.0, 3.0]]],
          [[[18.0, 28.0], [14.0, 23.0]], [[44.0, 26.0], [22.0, 19.0]]])
    with pytest.raises(ba.BurnqError):   # should_panic_when_inner_dimensions_are_not_equal
        QTensorOps.q_matmul(q([[3., 3.], [4., 4.], [5., 5.], [6., 6.]]), q([[1., 2., 3., 4.]] * 3))


def test_reference_transposed_and_permuted_cases(dev, approx):
    """crates/burn-backend-tests/tests/tensor/float/quantization/ops/quantize.rs:119-169 and 292-488:
    quantize_dynamic -> dequantize of arange grids, per tensor and per block, directly, on transposed
    inputs, and with the quantized tensor transposed / permuted before it is dequantized (packed
    words then straddle blocks: blocks of [1, 2, 16] become [16, 1, 2] under permute([2, 0, 1])).
    Tolerance::absolute(1e-1).set_relative(1e-2), as there. (Float transposes are host-side: float
    tensor ops are outside this library.)"""
    def grid(n, shape):
        return (np.arange(n, dtype=np.float32) / np.float32(n)).reshape(shape)

    def roundtrip(x, scheme):
        return FloatOps.float_into_data(QTensorOps.dequantize(QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)))

    per_tensor = QuantScheme()
    approx(roundtrip(grid(256, (16, 16)), per_tensor), grid(256, (16, 16)), 1e-2, 1e-1)
    approx(roundtrip(grid(256, (16, 16)), per_tensor.per_block((2, 16))), grid(256, (16, 16)), 1e-2, 1e-1)
    # should_quantize_transposed: quantize the transposed input, transpose the result back
    for n, shape, scheme in ((256, (8, 32), per_tensor), (3072, (48, 64), per_tensor), (2048, (32, 64), per_tensor.per_block((32,)))):
        x = grid(n, shape)
        approx(roundtrip(np.ascontiguousarray(x.T), scheme).T, x, 1e-2, 1e-1)
    # should_dequantize_transposed: transpose the quantized tensor
    for n, shape, scheme in ((256, (8, 32), per_tensor), (2048, (32, 64), per_tensor.per_block((32,)))):
        x = grid(n, shape)
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
        d = FloatOps.float_into_data(QTensorOps.dequantize(QTensorOps.q_swap_dims(tq, 0, 1)))
        approx(d.T, x, 1e-2, 1e-1)
    # permutes of a [2, 8, 16] tensor in [1, 2, 16] blocks
    x = grid(256, (2, 8, 16))
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), per_tensor.per_block((1, 2, 16)))
    for axes in ((1, 2, 0), (2, 0, 1)):
        d = FloatOps.float_into_data(QTensorOps.dequantize(QTensorOps.q_permute(tq, axes)))
        approx(d, np.transpose(x, axes), 1e-2, 1e-1)
    # should_quantize_symmetric_int8_permuted_batch_dims
    x = grid(2048, (2, 4, 8, 32))
    approx(np.transpose(roundtrip(np.ascontiguousarray(np.transpose(x, (1, 2, 0, 3))), per_tensor), (2, 0, 1, 3)), x, 1e-2, 1e-1)


def test_reference_gpu_backend_quantize_dequantize_cases(dev):
    """crates/burn-backend-tests/tests/cubecl/quantization/quantize_dequantize.rs, case by case: the
    reference's GPU backend is checked there against its CPU backend with the Native store; here
    the same inputs go against the oracle, bit for bit (values, scales, blob, dequantized floats).
    :112-143 arange [8,16] per tensor, all six values, packed; :145-164 the literal [2,16] tensor
    in blocks of 8 (Q8S, Q4S, Q2S) and 16 (Q2S); :166-178 Native store; :180-223 arange [32,32] and [128,256] in blocks of 32,
    both stores; :225-235 a last dim that does not fill packed words is refused."""
    def arange(shape):
        return np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)

    packed, native = QuantStore.PackedU32, QuantStore.Native
    for value in (QuantValue.Q8S, QuantValue.Q8F, QuantValue.Q4S, QuantValue.Q4F, QuantValue.Q2S, QuantValue.Q2F):
        check_quantize_dynamic(dev, arange((8, 16)), QuantScheme(value=value, store=packed))
    literal = np.float32([[-1.8, -1.0, 0.0, 0.5, -1.8, -1.0, 0.0, 0.5, 0.01, 0.025, 0.03, 0.04, 0.01, 0.025, 0.03, 0.04],
                          [1.8, 1.0, 0.0, -0.5, 1.8, 1.0, 0.0, -0.5, -0.01, -0.025, -0.03, -0.04, -0.01, -0.025, -0.03, -0.04]])
    check_quantize_dynamic(dev, literal, QuantScheme(value=QuantValue.Q8S, store=packed).per_block((8,)))
    check_quantize_dynamic(dev, literal, QuantScheme(value=QuantValue.Q4S, store=packed).per_block((8,)))
    # should_panic_when_block_size_cannot_store_num_quants: the reference's GPU backend refuses blocks
    # of 8 two-bit values (half a packed word); its CPU backend takes them, and so does this library
    check_quantize_dynamic(dev, literal, QuantScheme(value=QuantValue.Q2S, store=packed).per_block((8,)))
    check_quantize_dynamic(dev, literal, QuantScheme(value=QuantValue.Q2S, store=packed).per_block((16,)))
    check_quantize_dynamic(dev, arange((32, 32)), QuantScheme(value=QuantValue.Q8S, store=native))
    check_quantize_dynamic(dev, literal, QuantScheme(value=QuantValue.Q8S, store=native).per_block((8,)))
    for shape in ((32, 32), (128, 256)):
        for store in (packed, native):
            check_quantize_dynamic(dev, arange(shape), QuantScheme(value=QuantValue.Q8S, store=store).per_block((32,)))
    with pytest.raises(ba.BurnqError):   # should_panic_when_shape_cannot_store_quants: "Can't store in u32"
        gpu_quantize_dynamic(dev, np.float32([[1.0, 6.35], [2.0, 3.0], [1.0, 3.0]]), QuantScheme(store=packed))


@pytest.mark.parametrize("value", [QuantValue.Q4S, QuantValue.Q2S, QuantValue.Q4F, QuantValue.Q2F])
@pytest.mark.parametrize("block", [None, (16,), (2, 8)])
def test_sub_byte_values_stored_natively(dev, value, block):
    """The reference's CPU backend keeps quantized values natively -- one i8 per value, 4- and 2-bit
    value types included (crates/burn-std/src/tensor/quantization.rs:219-272 writes them that way,
    :329-333 reads them back; burn-store/src/tensor_snapshot.rs:545-581 and
    burn-store/tests/direct_writer.rs:76-93 save and size them) -- so a checkpoint written from it
    holds such blobs. They quantize, serialise, load, dequantize, permute and multiply here like
    any other tensor, bit for bit against the oracle; element counts that are not multiples of 4."""
    scheme = QuantScheme(value=value, store=QuantStore.Native, block=block)
    shape = (6, 16) if block else (5, 5)
    x = awkward(shape, 77 + value.value)
    tq, q_ref, s_ref, d_ref = check_quantize_dynamic(dev, x, scheme)
    assert np.abs(q_ref).max() <= (8 if value.size_bits() == 4 else 2)
    blob = QTensorOps.q_into_data(tq)
    assert blob.bytes.size == x.size + 4 * s_ref.size == ba.TensorData.data_len(shape, scheme)
    back = QTensorOps.q_from_data(blob, dev)
    assert FloatOps.float_into_data(QTensorOps.dequantize(back)).tobytes() == d_ref.tobytes()
    # static quantize against the same scales gives the same tensor
    again = QTensorOps.quantize(FloatOps.float_from_data(x, dev), scheme, FloatOps.float_from_data(s_ref, dev))
    assert QTensorOps.q_into_data(again).bytes.tobytes() == blob.bytes.tobytes()
    if block is None:
        t = QTensorOps.q_swap_dims(tq, 0, 1)
        assert FloatOps.float_into_data(QTensorOps.dequantize(t)).tobytes() == np.ascontiguousarray(d_ref.T).tobytes()
    # a product with it: lhs [3, rows] x tensor [rows, cols]
    lhs = awkward((3, shape[0]), 5, outliers=False)
    out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(lhs, dev), tq))
    ref = lhs.astype(np.float64) @ d_ref.astype(np.float64)
    assert np.abs(out - ref).max() <= 1e-5 * max(np.abs(ref).max(), 1e-30)


# ------------------------------------------------------------------ seeded parity, all schemes

@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,), (16,), (8,), (64,), (128,), (4,), (2, 128)])
def test_quantize_dequantize_parity_small(dev, value, block):
    scheme = QuantScheme(value=value, block=block)
    if block and value == QuantValue.Q4S and block[-1] < 8:
        pytest.skip("a block smaller than one packed word")
    x = awkward((96, 512), 1234 + (block[0] if block else 0))
    x[3, :256] = 0.0           # all-zero blocks: stored scale 0, quantized against 0.1
    x[5, :64] = 1e-41          # subnormal inputs
    x[7, :] *= 1e30            # large magnitudes
    x[9, :] *= 1e-30
    check_quantize_dynamic(dev, x, scheme)


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
def test_scale_exponent_sweep(dev, value):
    """Blocks whose scale runs over the whole exponent range: exercises the reciprocal fast
    path, its guards at 2^-100 / 2^100, subnormal scales and scales near f32 max."""
    rng = np.random.default_rng(99)
    exps = np.arange(-148, 123)
    x = rng.standard_normal((len(exps), 64)).astype(np.float64)
    x = np.ldexp(x, exps[:, None]).astype(np.float32)
    x = np.nan_to_num(x, posinf=3e38, neginf=-3e38)
    check_quantize_dynamic(dev, x, QuantScheme(value=value).per_block((32,)))
    for row in (0, 20, 48, 150, 247, 269):
        check_quantize_dynamic(dev, x[row], QuantScheme(value=value))


def test_division_shortcuts_are_exact_on_this_gpu(dev):
    """The kernels replace IEEE divisions by reciprocal + fma sequences; the library compares the
    two exhaustively on the device: 1 / s and the two scale formulas over 2^23 mantissas x every
    admitted exponent, and the quotient x / s (bits, and the integer it rounds to) around every
    rounding tie (k + 1/2) * s for every scale mantissa."""
    from burn_amd import _lib
    buf = FloatOps.float_empty((16,), dev)
    _lib.check(_lib.lib().bqk_selftest_division(buf.data_ptr, dev.stream))
    counts = FloatOps.float_into_data(buf).view(np.uint64)[:5]
    assert counts.tolist() == [0, 0, 0, 0, 0], counts


def test_copy_kernel(dev):
    """bqk_copy (the calibration / ceiling kernel): bytes arrive intact, ragged tail included,
    and misaligned sizes are refused."""
    from burn_amd import _lib
    n = 1024 * 4 * 3 + 12  # not a multiple of the 1024-chunk workgroup pass
    src = np.random.default_rng(7).standard_normal(n).astype(np.float32)
    a = FloatOps.float_from_data(src, dev)
    b = FloatOps.float_from_data(np.zeros(n, np.float32), dev)
    _lib.check(_lib.lib().bqk_copy(a.data_ptr, b.data_ptr, 4 * n, dev.stream))
    np.testing.assert_array_equal(FloatOps.float_into_data(b), src)
    assert _lib.lib().bqk_copy(a.data_ptr, b.data_ptr, 4 * n - 4, dev.stream) == _lib.ERR_SHAPE


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
def test_random_magnitudes_large(dev, value):
    """4 M values, every block with its own random exponent and full-entropy mantissas."""
    rng = np.random.default_rng(2024)
    blocks = 1 << 17
    mant = rng.integers(0, 1 << 23, (blocks, 32), dtype=np.uint32)
    sign = rng.integers(0, 2, (blocks, 32), dtype=np.uint32) << 31
    ex = rng.integers(1, 250, (blocks, 1), dtype=np.uint32)
    spread = rng.integers(0, 12, (blocks, 32), dtype=np.uint32)
    e = np.maximum(ex.astype(np.int64) - spread, 0).astype(np.uint32)
    x = (sign | (e << 23) | mant).view(np.float32).reshape(4096, 1024)
    check_quantize_dynamic(dev, x, QuantScheme(value=value).per_block((32,)), mt=True)
    check_quantize_dynamic(dev, x[:512] * np.float32(1e-3), QuantScheme(value=value), mt=True)


def test_rounding_ties_on_gpu(dev):
    x = np.float32([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 127.5, -127.5, 300.0, -300.0,
                    0.49999997, -0.49999997, 0.0, -0.0])
    s = FloatOps.float_from_data(np.float32([1.0]), dev)
    t = QTensorOps.quantize(FloatOps.float_from_data(x, dev), QuantScheme(store=QuantStore.Native), s)
    q, _ = unpack_blob(QTensorOps.q_into_data(t))
    assert q.tolist() == co.quantize(x, co.Scheme.make(co.Q8S), np.float32([1.0])).tolist()
    assert q.tolist() == [1, -1, 2, -2, 3, -3, 127, -127, 127, -127, 127, -127, 0, 0, 0, 0]
    # products that land exactly on .5 after the division
    rng = np.random.default_rng(5)
    sc = rng.uniform(0.001, 3.0, 4096).astype(np.float32)
    k = rng.integers(-127, 127, 4096).astype(np.float32) + np.float32(0.5)
    xs = (k * sc).astype(np.float32).reshape(4096, 1).repeat(32, 1)
    xs[:, 1] = np.nextafter(xs[:, 0], np.float32(np.inf))
    xs[:, 2] = np.nextafter(xs[:, 0], np.float32(-np.inf))
    scales = FloatOps.float_from_data(sc, dev)
    scheme = QuantScheme().per_block((32,))
    t = QTensorOps.quantize(FloatOps.float_from_data(xs, dev), scheme, scales)
    q, s_out = unpack_blob(QTensorOps.q_into_data(t))
    assert s_out.reshape(-1).tobytes() == sc.tobytes()
    assert (q == co.quantize(xs, oscheme(scheme), sc)).all()


def test_static_quantize_with_zero_scales(dev):
    x = awkward((8, 64), 3)
    sc = np.float32([0.0, 0.5] * 8)
    scheme = QuantScheme().per_block((32,))
    t = QTensorOps.quantize(FloatOps.float_from_data(x, dev), scheme, FloatOps.float_from_data(sc, dev))
    q, s = unpack_blob(QTensorOps.q_into_data(t))
    assert s.reshape(-1).tobytes() == sc.tobytes()
    assert (q == co.quantize(x, oscheme(scheme), sc)).all()
    d = FloatOps.float_into_data(QTensorOps.dequantize(t))
    assert d.tobytes() == co.dequantize(q, oscheme(scheme), sc).tobytes()


@pytest.mark.parametrize("shape,block", [((4, 8), (2, 4)), ((16, 16), (2, 16)), ((2, 8, 16), (1, 2, 16)),
                                         ((6, 24), (3, 12)), ((4, 6, 8), (2, 3, 4)), ((5, 96), (96,))])
def test_rectangle_and_odd_blocks(dev, shape, block):
    x = awkward(shape, 17)
    for value in (QuantValue.Q8S, QuantValue.Q4S):
        if value == QuantValue.Q4S and shape[-1] % 8:
            continue
        check_quantize_dynamic(dev, x, QuantScheme(value=value).per_block(block))
    check_quantize_dynamic(dev, x, QuantScheme(store=QuantStore.Native).per_block(block))


@pytest.mark.parametrize("n", [1, 3, 5, 127, 1001, 4099])
def test_native_per_tensor_ragged_lengths(dev, n):
    x = awkward((n,), n)
    check_quantize_dynamic(dev, x, QuantScheme(store=QuantStore.Native))


@pytest.mark.parametrize("n", [8, 4096, 16376, 16384, 16392, 65536])
def test_small_per_tensor_quantize_one_launch_and_two(dev, n):
    """Per-tensor quantize_dynamic takes one launch up to 16 384 values and two passes above: the same
    bits either side of the limit, for every value type and scale dtype the per-tensor kernels take,
    extreme scales (the division path) and an all-zero tensor (scale 0, quantized against 0.1) included."""
    x = awkward((n,), n)
    for scheme in (QuantScheme(store=QuantStore.Native), QuantScheme(), QuantScheme(value=QuantValue.Q4S),
                   QuantScheme(value=QuantValue.Q8F), QuantScheme(value=QuantValue.Q4F)):
        check_quantize_dynamic(dev, x, scheme)
    for sdt in (ScaleDtype.F16, ScaleDtype.BF16, ScaleDtype.UE4M3):
        check_scale_dtype(dev, x, QuantScheme(scale_dtype=sdt))
        check_scale_dtype(dev, x, QuantScheme(value=QuantValue.Q4S, scale_dtype=sdt))
    check_quantize_dynamic(dev, np.zeros(n, np.float32), QuantScheme())
    check_quantize_dynamic(dev, (x * np.float32(1e-38)).astype(np.float32), QuantScheme(store=QuantStore.Native))
    check_quantize_dynamic(dev, (x * np.float32(1e36)).astype(np.float32), QuantScheme(value=QuantValue.Q4S))
    if n % 4 == 0:   # native i8 of a length that is no multiple of 4: the last values go one byte each
        check_quantize_dynamic(dev, x[: n - 3], QuantScheme(store=QuantStore.Native))


def test_empty_tensor(dev):
    x = np.zeros((0, 32), np.float32)
    for scheme in (QuantScheme(store=QuantStore.Native), QuantScheme().per_block((32,))):
        t = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
        assert t.shape == (0, 32)
        assert FloatOps.float_into_data(QTensorOps.dequantize(t)).shape == (0, 32)


def test_dequantize_bf16(dev):
    x = awkward((64, 256), 21)
    for scheme in (QuantScheme().per_block((32,)), QuantScheme(value=QuantValue.Q4S).per_block((32,)),
                   QuantScheme(store=QuantStore.Native)):
        tq, q_ref, s_ref, d_ref = check_quantize_dynamic(dev, x, scheme)
        bits = FloatOps.float_into_data(QTensorOps.dequantize(tq, ba.BF16))
        assert bits.dtype == np.uint16
        assert bits.tobytes() == ba.bf16_bits_from_f32(d_ref).reshape(x.shape).tobytes()


@pytest.mark.parametrize("shape,scheme", [
    ((3, 12), QuantScheme()),                                   # 9 words: an odd last word
    ((5, 20), QuantScheme().per_block((4,))),                   # one word per scale: a pair has two scales
    ((7, 36), QuantScheme().per_block((12,))),                  # three words per scale (no fused kernel: general path)
    ((1, 4), QuantScheme()),                                    # a single word
    ((11,), QuantScheme(store=QuantStore.Native)),              # native bytes with a tail of 3
    ((513, 8), QuantScheme().per_block((8,))),                  # several workgroups, 1026 words
    ((2, 1000), QuantScheme(store=QuantStore.Native).per_block((8,))),
])
def test_dequantize_bf16_q8s_word_pairs(dev, shape, scheme):
    """Q8S -> bf16 takes two words per lane: odd word counts, a scale per word, native tails."""
    x = awkward(shape, sum(shape) + 5)
    tq, q_ref, s_ref, d_ref = check_quantize_dynamic(dev, x, scheme)
    bits = FloatOps.float_into_data(QTensorOps.dequantize(tq, ba.BF16))
    assert bits.tobytes() == ba.bf16_bits_from_f32(d_ref).reshape(x.shape).tobytes()


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,), (64,)])
@pytest.mark.parametrize("m,k,n", [(8, 129, 256), (16, 130, 2112), (7, 131, 64), (12, 6, 32), (16, 1027, 320)])
def test_q_matmul_small_batch_k_not_multiple_of_4(dev, value, block, m, k, n):
    """f32 activations, 7 <= M <= 16, K % 4 != 0: the FP32-matrix kernel walks K in groups of four
    rows and its last group is partial (it once multiplied that group's activations by the
    weights of the four rows before)."""
    if block and n % block[0]:
        pytest.skip("block does not divide N")
    rng = np.random.default_rng(m + k + n)
    w = (rng.standard_normal((k, n)) * 0.1).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme(value=value, block=block))
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    ref = no.q_matmul_f64(x, q, s, list(block) if block else None)
    out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    assert np.abs(out - ref).max() <= 1e-5 * np.abs(ref).max()


@pytest.mark.parametrize("b,m,k,n", [(3, 1, 8, 4), (2, 3, 16, 12), (5, 1, 32, 20), (2, 2, 8, 8), (3, 2, 64, 32)])
@pytest.mark.parametrize("rhs_batched", [False, True])
def test_q_matmul_batched_small_operands(dev, b, m, k, n, rhs_batched):
    """Batches whose slices of the activations or of the output do not start on 16-byte
    boundaries (tiny M x N, bf16) are multiplied like the reference does it, by dequantizing;
    f32 and bf16 activations, a shared and a per-batch weight."""
    rng = np.random.default_rng(b * 100 + m * 10 + k + n)
    w = rng.standard_normal((b if rhs_batched else 1, k, n)).astype(np.float32)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme())
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    wd = no.dequantize(q.reshape(-1, n), s, None).reshape(w.shape).astype(np.float64)
    x = rng.standard_normal((b, m, k)).astype(np.float32)
    xb = ba.bf16_bits_from_f32(x)
    for data, dt, tol in ((x, ba.F32, 1e-5), (xb, ba.BF16, 1e-2)):
        y = QTensorOps.q_matmul(FloatOps.float_from_data(data, dev, dt), tq)
        assert y.shape == (b, m, n) and y.dtype == dt
        got = FloatOps.float_into_data(y)
        xf = x if dt == ba.F32 else ba.f32_from_bf16_bits(xb).reshape(b, m, k)
        if dt == ba.BF16:
            got = ba.f32_from_bf16_bits(got).reshape(b, m, n)
        ref = np.stack([xf[i].astype(np.float64) @ wd[i if rhs_batched else 0] for i in range(b)])
        assert np.abs(got - ref).max() <= tol * np.abs(ref).max()


@pytest.mark.parametrize("m,k,n", [(1, 1, 1), (5, 7, 3), (64, 64, 64), (65, 33, 130), (512, 512, 512),
                                   (200, 1000, 72), (1, 300, 640), (300, 24, 2112), (2100, 96, 2100)])
def test_q_matmul_other_operand_combinations(dev, m, k, n):
    """quantized x quantized, quantized x float, float x a weight in rectangle blocks: the
    quantized operands are dequantized (crates/burn-backend/src/backend/ops/qtensor.rs:498-544),
    then multiplied in f32 -- by the packed-weight kernels when the rhs is one they take, by the
    f32 matrix-core GEMM otherwise. Yardstick: the float64 product of the dequantized operands."""
    rng = np.random.default_rng(m * 131 + k * 17 + n)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)

    def quantized(x, scheme):
        t = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
        q, s = unpack_blob(QTensorOps.q_into_data(t))
        blk = list(scheme.block) if scheme.block else None
        return t, no.dequantize(q, s, blk).astype(np.float64)

    def check(out, ref, tol):
        assert out.shape == ref.shape and out.dtype == ba.F32
        assert np.abs(FloatOps.float_into_data(out) - ref).max() <= tol * max(np.abs(ref).max(), 1e-30)

    ql, al = quantized(a, QuantScheme() if k % 4 == 0 else QuantScheme(store=QuantStore.Native))
    packed = QuantScheme() if n % 4 == 0 else QuantScheme(store=QuantStore.Native)
    qr, br = quantized(b, packed)
    # (more than 32 rows against a packed weight: the prefill kernel, whose operands are bf16)
    check(QTensorOps.q_matmul(ql, qr), al @ br, 2e-5 if (m <= 32 or n % 4) else 1e-2)
    check(QTensorOps.q_matmul(ql, FloatOps.float_from_data(b, dev)), al @ b.astype(np.float64), 2e-5)
    if k % 2 == 0 and n % 8 == 0:
        qrect, brect = quantized(b, QuantScheme().per_block((2, 8)))
        check(QTensorOps.q_matmul(FloatOps.float_from_data(a, dev), qrect), a.astype(np.float64) @ brect, 2e-5)
        check(QTensorOps.q_matmul(ql, qrect), al @ brect, 2e-5)
    if n % 32 == 0:
        q4, b4 = quantized(b, QuantScheme(value=QuantValue.Q4S).per_block((32,)))
        check(QTensorOps.q_matmul(ql, q4), al @ b4, 2e-5 if m <= 32 else 1e-2)


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
def test_f32_matmul_exact_setting_removes_the_step_at_33_rows(dev, value):
    """f32 activations x a packed weight: up to 32 rows the products keep 16 significant bits;
    from 33 on the fast kernel rounds to bf16 (about 2e-3, inside the 1e-2 bound) unless the
    device is told to multiply in f32, as the reference's dequantize + sgemm does."""
    rng = np.random.default_rng(33)
    m, k, n = 96, 1024, 640
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme(value=value).per_block((32,)))
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    ref = no.q_matmul_f64(x, q, s, [32])
    xt = FloatOps.float_from_data(x, dev)

    def rel(y, r):
        return np.abs(FloatOps.float_into_data(y) - r).max() / np.abs(r).max()

    fast = rel(QTensorOps.q_matmul(xt, tq), ref)
    assert 1e-4 < fast <= 1e-2, fast                   # the bf16 kernel: the step is there
    dev.set_f32_matmul_exact(True)
    try:
        assert rel(QTensorOps.q_matmul(xt, tq), ref) <= 2e-6
        y = ModuleOps.linear(xt, tq, FloatOps.float_from_data(bias, dev))
        assert rel(y, ref + bias[None, :].astype(np.float64)) <= 2e-6
        # 32 rows and fewer are untouched by the setting
        small = rel(QTensorOps.q_matmul(FloatOps.float_from_data(x[:32], dev), tq), ref[:32])
    finally:
        dev.set_f32_matmul_exact(False)
    assert small <= 2e-5 and small == rel(QTensorOps.q_matmul(FloatOps.float_from_data(x[:32], dev), tq), ref[:32])


def test_matmul_exact_setting_with_bf16_activations(dev):
    """bf16 activations x Q4S block-32, K = 4096 (the prefill configuration's depth, a quarter of its
    width): the fast kernel rounds s * q to bf16, which on a product this deep puts a few outputs in a
    million outside burn's elementwise rule; with the setting on the weights are dequantized to f32 and
    multiplied in f32, and every output meets the rule -- f32 and bf16 output, with a bias."""
    rng = np.random.default_rng(55)
    m, k, n = 2048, 4096, 3584
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme(value=QuantValue.Q4S).per_block((32,)))
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    bits = ba.bf16_bits_from_f32(rng.standard_normal((m, k)).astype(np.float32))
    x = ba.f32_from_bf16_bits(bits)
    xt = FloatOps.float_from_data(bits, dev, ba.BF16)
    ref = no.q_matmul_f64(x, q, s, [32])
    fast = FloatOps.float_into_data(QTensorOps.q_matmul(xt, tq, out_dtype=ba.F32))
    outside_fast = int((~burn_approx_eq(fast, ref, 1e-2, 1e-2)).sum())
    assert np.abs(fast - ref).max() / np.abs(ref).max() <= 1e-2
    dev.set_f32_matmul_exact(True)
    try:
        exact = FloatOps.float_into_data(QTensorOps.q_matmul(xt, tq, out_dtype=ba.F32))
        bias = rng.standard_normal(n).astype(np.float32)
        lin = FloatOps.float_into_data(ModuleOps.linear(xt, tq, FloatOps.float_from_data(bias, dev), out_dtype=ba.F32))
    finally:
        dev.set_f32_matmul_exact(False)
    assert np.abs(exact - ref).max() / np.abs(ref).max() <= 1e-5      # f32 sums over 4096 terms
    assert burn_approx_eq(exact, ref, 1e-2, 1e-2).all()
    assert burn_approx_eq(lin, ref + bias[None, :].astype(np.float64), 1e-2, 1e-2).all()
    assert outside_fast <= 30, outside_fast       # (7.3 M outputs at 4.7 sigma: about 19 predicted)


def test_host_transfers_around_the_staging_size(dev):
    """Host buffers travel through two pinned halves of 2 MiB: sizes just under, at and over one and
    two halves, and far over, come back byte for byte, for float tensors and for quantized blobs
    (values and scales in one copy or in two), also when uploads follow each other without a
    synchronisation in between."""
    half = 2 << 20
    rng = np.random.default_rng(31)
    sizes = [1, 3, half // 4 - 1, half // 4, half // 4 + 1, half // 2 + 5, 2 * half // 4, 2 * half // 4 + 7, 5 * half // 4 + 3]
    held = []
    for n in sizes:                       # n floats = 4 n bytes: 4 B ... 10 MiB + 12 B
        x = rng.standard_normal(n).astype(np.float32)
        held.append((x, FloatOps.float_from_data(x, dev)))   # back to back: no sync between uploads
    for x, t in held:
        assert FloatOps.float_into_data(t).tobytes() == x.tobytes()
    for n in (half - 4, half, half + 4, 3 * half + 8):       # value bytes; scales behind them
        scheme = QuantScheme(store=QuantStore.Native).per_block((4,))
        blob = np.concatenate([rng.integers(-127, 128, n, dtype=np.int8).view(np.uint8),
                               rng.random(n // 4, dtype=np.float32).view(np.uint8)])
        t = QTensorOps.q_from_data(TensorData(blob, (n,), scheme), dev)
        assert QTensorOps.q_into_data(t).bytes.tobytes() == blob.tobytes()


def test_error_behaviour(dev):
    x = FloatOps.float_from_data(np.zeros((4, 6), np.float32), dev)
    with pytest.raises(ba.BurnqError, match="Can't store in u32"):
        QTensorOps.quantize_dynamic(x, QuantScheme())                    # 6 % 4 != 0
    # (4-bit values stored natively, one i8 each, are what the reference's CPU backend keeps: accepted)
    assert QTensorOps.quantize_dynamic(x, QuantScheme(value=QuantValue.Q4S, store=QuantStore.Native)).shape == (4, 6)
    x8 = FloatOps.float_from_data(np.zeros((4, 8), np.float32), dev)
    with pytest.raises(ba.BurnqError, match="evenly divisible"):
        QTensorOps.quantize_dynamic(x8, QuantScheme().per_block((3,)))
    q = QTensorOps.quantize_dynamic(x8, QuantScheme())
    with pytest.raises(ba.BurnqError, match="inner dimensions"):
        QTensorOps.q_matmul(FloatOps.float_from_data(np.zeros((2, 5), np.float32), dev), q)
    with pytest.raises(ba.BurnqError):
        QTensorOps.dequantize(x8)
    blob = QTensorOps.q_into_data(q)
    with pytest.raises(ba.BurnqError, match="bytes"):
        QTensorOps.q_from_data(TensorData(blob.bytes[:-1], blob.shape, blob.scheme), dev)


def test_q_reshape_is_metadata_only(dev):
    x = awkward((8, 128), 8)
    scheme = QuantScheme().per_block((32,))
    tq, q_ref, s_ref, d_ref = check_quantize_dynamic(dev, x, scheme)
    r = QTensorOps.q_reshape(tq, (4, 256))
    assert r.shape == (4, 256) and r.data_ptr == tq.data_ptr
    d = FloatOps.float_into_data(QTensorOps.dequantize(r))
    assert d.tobytes() == d_ref.reshape(4, 256).tobytes()
    # a last dim shorter than the block: the run of 32 becomes a [2, 16] block
    r = QTensorOps.q_reshape(tq, (64, 16))
    assert r.scheme.block == (2, 16) and r.data_ptr == tq.data_ptr
    assert FloatOps.float_into_data(QTensorOps.dequantize(r)).tobytes() == d_ref.reshape(64, 16).tobytes()
    t6, _, _, d6 = check_quantize_dynamic(dev, awkward((6, 64), 9), scheme)
    with pytest.raises(ba.BurnqError):
        QTensorOps.q_reshape(t6, (8, 48))    # runs of 32 do not tile rows of 48
    # runs of 256 values and more do not fit one block extent (a byte): spread over two dims
    big = QuantScheme().per_block((2, 128))
    tb, _, _, db = check_quantize_dynamic(dev, awkward((4, 2, 128), 10), big)
    r = QTensorOps.q_reshape(tb, (8, 128))
    assert r.scheme.block == (2, 128)
    assert FloatOps.float_into_data(QTensorOps.dequantize(r)).tobytes() == db.reshape(8, 128).tobytes()
    r = QTensorOps.q_reshape(tb, (2, 8, 64))
    assert r.scheme.block == (4, 64)
    assert FloatOps.float_into_data(QTensorOps.dequantize(r)).tobytes() == db.reshape(2, 8, 64).tobytes()
    with pytest.raises(ba.BurnqError):
        QTensorOps.q_reshape(tb, (2, 512))   # one extent of 256
    same = QTensorOps.q_to_device(tq, dev)
    assert QTensorOps.q_into_data(same).bytes.tobytes() == QTensorOps.q_into_data(tq).bytes.tobytes()


def test_reference_gpu_backend_reshape_cases(dev, approx):
    """crates/burn-backend-tests/tests/cubecl/quantization/reshape.rs, case by case: arange / n,
    quantize_dynamic, reshape, dequantize, against the reshaped input within the permissive
    tolerance as there, and -- sharper -- bit-equal to dequantize-then-reshape (:157-192). Where the
    reference's GPU backend refuses a reshape that its CPU backend performs (sub-byte values,
    :60-82; a block of 32 folded into rows of 16, :127-155) this library performs it like the CPU
    backend, since the memory order of values and scales does not change; a 2-D block that the new
    shape cuts is refused by both (:113-125)."""
    def case(block, value, store, shape, new_shape):
        n = int(np.prod(shape))
        x = (np.arange(n, dtype=np.float32) / np.float32(n)).reshape(shape)
        scheme = QuantScheme(value=value, store=store)
        if block is not None:
            scheme = scheme.per_block(block)
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
        d_flat = FloatOps.float_into_data(QTensorOps.dequantize(tq))
        r = QTensorOps.q_reshape(tq, new_shape)
        d = FloatOps.float_into_data(QTensorOps.dequantize(r))
        assert d.shape == tuple(new_shape) and d.tobytes() == d_flat.reshape(new_shape).tobytes()
        if value == QuantValue.Q8S:   # (the 4-bit cases never reach this comparison in the reference)
            approx(d, x.reshape(new_shape), 1e-2, 1e-2)

    packed, native = QuantStore.PackedU32, QuantStore.Native
    case((16,), QuantValue.Q8S, packed, (32,), (2, 16))
    case((16,), QuantValue.Q4S, packed, (32,), (2, 16))
    case(None, QuantValue.Q4S, packed, (32,), (2, 16))
    case((16,), QuantValue.Q8S, native, (32,), (2, 16))
    case((32,), QuantValue.Q8S, packed, (32,), (1, 1, 1, 32))
    with pytest.raises(ba.BurnqError):   # quantize_2d_block_reshape_should_panic
        case((2, 4), QuantValue.Q8S, packed, (4, 8), (32,))
    case((32,), QuantValue.Q8S, native, (2, 32), (4, 16))
    case((32,), QuantValue.Q8S, packed, (2, 32), (4, 16))
    case(None, QuantValue.Q8S, packed, (32,), (2, 16))


def test_layout_ops_known_answers(dev, approx):
    """q_permute / q_swap_dims / q_flip on the reference's own cases (crates/burn-backend-tests/
    tests/tensor/float/quantization/ops/extended/permute.rs:5-41, transpose.rs:6-40,
    flip.rs:6-21; edge cases permute.rs:43-66, flip.rs:23-40)."""
    def qt(x):
        return QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), QuantScheme(store=QuantStore.Native))
    def deq(t):
        return FloatOps.float_into_data(QTensorOps.dequantize(t))
    t = qt(np.arange(16, dtype=np.float32).reshape(2, 2, 4))
    want = np.float32([[[0, 8], [4, 12]], [[1, 9], [5, 13]], [[2, 10], [6, 14]], [[3, 11], [7, 15]]])
    p = QTensorOps.q_permute(t, [2, 1, 0])
    assert p.shape == (4, 2, 2)
    approx(deq(p), want, 1e-1, 1e-1)
    assert deq(QTensorOps.q_permute(t, [0, 1, 2])).tobytes() == deq(t).tobytes()
    for bad in ([0, 0, 1], [3, 0, 1]):
        with pytest.raises(ba.BurnqError):
            QTensorOps.q_permute(t, bad)
    t = qt(np.arange(12, dtype=np.float32).reshape(2, 2, 3))
    approx(deq(QTensorOps.q_swap_dims(t, 1, 2)), np.float32([[[0, 3], [1, 4], [2, 5]], [[6, 9], [7, 10], [8, 11]]]), 0, 1e-1)
    approx(deq(QTensorOps.q_swap_dims(t, 0, 2)), np.float32([[[0, 6], [3, 9]], [[1, 7], [4, 10]], [[2, 8], [5, 11]]]), 0, 1e-1)
    t = qt(np.float32([[[0, 1, 2]], [[3, 4, 5]]]))
    approx(deq(QTensorOps.q_flip(t, [0, 2])), np.float32([[[5, 4, 3]], [[2, 1, 0]]]), 0, 1e-1)
    assert QTensorOps.q_into_data(QTensorOps.q_flip(t, [])).bytes.tobytes() == QTensorOps.q_into_data(t).bytes.tobytes()
    for bad in ([0, 0, 1], [3, 0, 1]):
        with pytest.raises(ba.BurnqError):
            QTensorOps.q_flip(t, bad)


@pytest.mark.parametrize("value,store", [(QuantValue.Q8S, QuantStore.Native), (QuantValue.Q8S, QuantStore.PackedU32),
                                         (QuantValue.Q4S, QuantStore.PackedU32)])
@pytest.mark.parametrize("block", [None, (32,)])
@pytest.mark.parametrize("shape,axes", [((24, 64), (1, 0)), ((3, 8, 64), (2, 0, 1)), ((2, 16, 3, 32), (0, 3, 2, 1)),
                                        ((5, 32), (1, 0)),
                                        # the tiled transpose of 8-bit values: several tiles, ragged edges, batches
                                        ((132, 288), (1, 0)), ((256, 128), (1, 0)), ((3, 2, 36, 160), (0, 1, 3, 2)),
                                        ((4, 640), (1, 0)), ((2, 260, 32), (0, 2, 1))])
def test_q_permute_matches_oracle(dev, value, store, block, shape, axes):
    """Values and block scales after q_permute are the oracle's, byte for byte on the wire, and
    dequantize commutes with the permutation bit for bit."""
    vname = VAL[value][1]
    nq = 4 if value == QuantValue.Q8S else 8
    new_last = shape[axes[-1]]
    rng = np.random.default_rng(sum(shape) + len(axes))
    x = rng.standard_normal(shape).astype(np.float32)
    scheme = QuantScheme(value=value, block=block, store=store)
    if store == QuantStore.PackedU32 and shape[-1] % nq:
        pytest.skip("the source itself cannot be packed")
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    if store == QuantStore.PackedU32 and new_last % nq and value != QuantValue.Q8S:
        with pytest.raises(ba.BurnqError):   # "Can't store in u32" (sub-byte values have no native store)
            QTensorOps.q_permute(tq, axes)
        return
    tp = QTensorOps.q_permute(tq, axes)
    assert tp.shape == tuple(shape[a] for a in axes)
    # (a Q8S result whose last dim does not fill whole words comes back natively stored: same bytes)
    assert tp.scheme.store == (QuantStore.Native if new_last % nq else store)
    qp, sp, bp = no.q_permute(q, s, list(block) if block else None, axes)
    blob = QTensorOps.q_into_data(tp)
    got_q, got_s = unpack_blob(blob)
    assert (got_q == qp).all()
    assert np.asarray(got_s, np.float32).tobytes() == np.asarray(sp, np.float32).tobytes()
    d = FloatOps.float_into_data(QTensorOps.dequantize(tp))
    assert d.tobytes() == np.transpose(FloatOps.float_into_data(QTensorOps.dequantize(tq)), axes).copy().tobytes()
    assert d.tobytes() == no.dequantize(qp, sp, bp).tobytes()
    # q_flip: the values are flipped, the parameters stay where they are -- block scales too, as in
    # the reference (crates/burn-ndarray/src/ops/qtensor.rs:338-347)
    for flip_axes in ([0, len(shape) - 1], [len(shape) - 1], [0]):
        f = QTensorOps.q_flip(tq, flip_axes)
        qf, sf = no.q_flip(q, s, flip_axes)
        got_q, got_s = unpack_blob(QTensorOps.q_into_data(f))
        assert (got_q == qf).all()
        assert np.asarray(got_s, np.float32).tobytes() == np.asarray(sf, np.float32).tobytes()
        assert FloatOps.float_into_data(QTensorOps.dequantize(f)).tobytes() == \
            no.dequantize(qf, sf, list(block) if block else None).tobytes()


def test_hip_graph_replays_match_eager(dev):
    """Capture quantize_dynamic (per tensor: absmax + quantize, and block) + dequantize +
    q_matmul / linear through each kernel family into one graph; every replay, with eager work and syncs in between, must give
    the eager results bit for bit."""
    rng = np.random.default_rng(404)
    x = FloatOps.float_from_data(awkward((64, 512), 1), dev)
    a = FloatOps.float_from_data(rng.standard_normal((1, 512)).astype(np.float32), dev)
    a4 = FloatOps.float_from_data(rng.standard_normal((4, 512)).astype(np.float32), dev)
    w = QTensorOps.quantize_dynamic(FloatOps.float_from_data(awkward((512, 256), 2), dev),
                                    QuantScheme().per_block((32,)))

    from burn_amd import ModuleOps
    a16 = FloatOps.float_from_data(rng.standard_normal((16, 512)).astype(np.float32), dev)
    a64 = FloatOps.float_from_data(ba.bf16_bits_from_f32(rng.standard_normal((64, 512)).astype(np.float32)), dev, ba.BF16)
    bias = FloatOps.float_from_data(rng.standard_normal(256).astype(np.float32), dev)

    wt = QTensorOps.quantize_dynamic(FloatOps.float_from_data(awkward((512, 256), 4, outliers=False), dev),
                                     QuantScheme(value=QuantValue.Q2S))

    def step():
        qt = QTensorOps.quantize_dynamic(x, QuantScheme(store=QuantStore.Native))
        qb = QTensorOps.quantize_dynamic(x, QuantScheme(value=QuantValue.Q4S).per_block((32,)))
        # two-level scales (absmax, per-tensor scale, split block kernel), a full-range value,
        # the tiled transpose with its scale gather, the ternary product
        q2 = QTensorOps.quantize_dynamic(x, QuantScheme().per_block((32,), ScaleDtype.UE4M3).per_tensor(ScaleDtype.F32))
        qf = QTensorOps.quantize_dynamic(x, QuantScheme(value=QuantValue.Q8F).per_block((64,)))
        return (qt, qb, q2, qf, QTensorOps.dequantize(q2), QTensorOps.q_swap_dims(qf, 0, 1), QTensorOps.q_matmul(a4, wt),
                QTensorOps.dequantize(qt), QTensorOps.dequantize(qb),
                QTensorOps.q_matmul(a, w), QTensorOps.q_matmul(a4, w),
                # matrix cores over split activations; tiled kernel with split K; bias epilogues
                QTensorOps.q_matmul(a16, w), ModuleOps.linear(a16, w, bias),
                QTensorOps.q_matmul(a64, w, out_dtype=ba.F32), ModuleOps.linear(a64, w, bias))

    def snapshot(ts):
        return [QTensorOps.q_into_data(t).bytes.tobytes() if t.is_quantized
                else FloatOps.float_into_data(t).tobytes() for t in ts]

    eager = snapshot(step())          # also primes the allocation cache and the workspace
    graph, outs = dev.capture(step)
    for i in range(4):
        graph.launch()
        assert snapshot(outs) == eager, f"replay {i} differs from the eager result"
        # unrelated eager work between replays, scribbling over recycled buffers
        junk = QTensorOps.dequantize(QTensorOps.quantize_dynamic(
            FloatOps.float_from_data(awkward((64, 512), 50 + i), dev), QuantScheme()))
        FloatOps.float_into_data(junk)
        dev.sync()


def test_hip_graph_keeps_the_librarys_own_buffers(dev):
    """A captured call that allocates and frees inside itself (the f32 copy of a bf16 bias, the
    dequantized operands of the general q_matmul path, the float product of a propagating
    q_matmul) and a workspace that grows after the capture: neither may be recycled while the
    graph can be replayed. Bystander tensors allocated between replays keep their contents and
    every replay gives the eager result."""
    from burn_amd import ModuleOps
    rng = np.random.default_rng(77)
    w = QTensorOps.quantize_dynamic(FloatOps.float_from_data(awkward((512, 256), 2), dev), QuantScheme().per_block((32,)))
    wq_lhs = QTensorOps.quantize_dynamic(FloatOps.float_from_data(awkward((48, 512), 3), dev), QuantScheme().per_block((32,)))
    a16 = FloatOps.float_from_data(rng.standard_normal((16, 512)).astype(np.float32), dev)
    bias_bf16 = FloatOps.float_from_data(ba.bf16_bits_from_f32(rng.standard_normal(256).astype(np.float32)), dev, ba.BF16)

    def step():
        return (ModuleOps.linear(a16, w, bias_bf16),          # temporary: f32 copy of the bias
                QTensorOps.q_matmul(wq_lhs, w),                # temporaries: both operands dequantized
                QTensorOps.q_matmul_propagate(a16, w))         # temporary: the float product

    def snapshot(ts):
        return [QTensorOps.q_into_data(t).bytes.tobytes() if t.is_quantized
                else FloatOps.float_into_data(t).tobytes() for t in ts]

    eager = snapshot(step())
    graph, outs = dev.capture(step)
    bystanders = []
    for i in range(4):
        # eager allocations of the temporaries' sizes: they must not land on memory the graph writes
        fill = np.full(256, float(i + 1), np.float32)
        mine = [FloatOps.float_from_data(fill, dev) for _ in range(6)]
        mine += [FloatOps.float_from_data(np.full((48, 512), float(i + 1), np.float32), dev),
                 FloatOps.float_from_data(np.full((512, 256), float(i + 1), np.float32), dev),
                 FloatOps.float_from_data(np.full((16, 256), float(i + 1), np.float32), dev)]
        bystanders.append((i + 1, mine))
        if i == 1:  # a larger split-K workspace than the captured calls used
            big = QTensorOps.quantize_dynamic(FloatOps.float_from_data(awkward((2048, 4096), 9), dev),
                                              QuantScheme().per_block((32,)))
            a8 = FloatOps.float_from_data(rng.standard_normal((16, 2048)).astype(np.float32), dev)
            FloatOps.float_into_data(QTensorOps.q_matmul(a8, big))
        graph.launch()
        dev.sync()
        assert snapshot(outs) == eager, f"replay {i} differs from the eager result"
        for value, tensors in bystanders:
            for t in tensors:
                assert (FloatOps.float_into_data(t) == value).all(), "a replay wrote into a bystander tensor"
    del graph
    # once the graph is gone its parked blocks are reusable and still intact as allocations
    again = snapshot(step())
    assert again == eager


def test_validate_mode_fails_where_the_reference_panics(dev):
    """NaN quotients: the reference panics (Q::from(NaN).unwrap()); in validate mode the call
    fails with ERR_NONFINITE, out of it the call goes through."""
    from burn_amd import _lib
    x = awkward((8, 64), 5)
    bad_nan, bad_inf = x.copy(), x.copy()
    bad_nan[3, 7] = np.nan
    bad_inf[2, 9] = np.inf
    scheme = QuantScheme().per_block((32,))
    ok_scales = FloatOps.float_from_data(np.full(16, 0.05, np.float32), dev)
    inf_scales = FloatOps.float_from_data(np.float32([0.05] * 15 + [np.inf]), dev)
    nan_scales = FloatOps.float_from_data(np.float32([0.05] * 15 + [np.nan]), dev)
    dev.set_validate(True)
    try:
        QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)             # finite: fine
        QTensorOps.quantize(FloatOps.float_from_data(bad_inf, dev), scheme, ok_scales)    # inf / finite clamps
        QTensorOps.quantize(FloatOps.float_from_data(x, dev), scheme, inf_scales)         # finite / inf = 0
        for tensor, scales in ((bad_nan, None), (bad_inf, None), (bad_nan, ok_scales), (x, nan_scales),
                               (bad_inf, inf_scales)):
            with pytest.raises(ba.BurnqError) as e:
                t = FloatOps.float_from_data(tensor, dev)
                if scales is None:
                    QTensorOps.quantize_dynamic(t, scheme)
                    QTensorOps.quantize_dynamic(t, QuantScheme(store=QuantStore.Native))
                else:
                    QTensorOps.quantize(t, scheme, scales)
            assert e.value.status == _lib.ERR_NONFINITE
    finally:
        dev.set_validate(False)
    QTensorOps.quantize_dynamic(FloatOps.float_from_data(bad_nan, dev), scheme)  # unspecified integers, no error
    dev.sync()


# ------------------------------------------------------------------ f16 / bf16 scales

SDT = {ScaleDtype.F16: (co.SCALE_F16, "F16"), ScaleDtype.BF16: (co.SCALE_BF16, "BF16"), ScaleDtype.UE4M3: (co.SCALE_UE4M3, "UE4M3")}


def check_scale_dtype(dev, x, scheme, given_scales=None):
    """quantize / quantize_dynamic with 2-byte scales against the oracle composed the way
    burn-ndarray composes it (qtensor.rs:90-95): range -> q_params -> scale_to_dtype -> quantize
    against the rounded scale; the blob carries the scales encoded in the scale dtype."""
    code, _ = SDT[scheme.scale_dtype]
    osch = oscheme(scheme)
    if given_scales is None:
        lo, hi = co.compute_range(x, osch)
        raw = co.compute_q_params(lo, hi, osch.value)
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
    else:
        raw = np.ascontiguousarray(given_scales, np.float32)
        tq = QTensorOps.quantize(FloatOps.float_from_data(x, dev), scheme, FloatOps.float_from_data(raw, dev))
    s_ref = co.scale_to_dtype(raw, code)
    q_ref = co.quantize(x, osch, s_ref)
    blob = QTensorOps.q_into_data(tq)
    assert blob.bytes.size == TensorData.data_len(x.shape, scheme)
    assert blob.bytes.tobytes() == co.encode_with_scale_dtype(q_ref, osch, s_ref, code).tobytes(), "blob differs"
    q_gpu, s_gpu = unpack_blob(blob)
    assert s_gpu.reshape(-1).tobytes() == np.ascontiguousarray(s_ref, np.float32).reshape(-1).tobytes()
    assert (q_gpu == q_ref).all()
    d_ref = co.dequantize(q_ref, osch, s_ref)
    assert FloatOps.float_into_data(QTensorOps.dequantize(tq)).tobytes() == d_ref.tobytes()
    # save / load: the blob loads back to the same tensor (one H2D copy of values, scales widened)
    again = QTensorOps.q_from_data(blob, dev)
    assert QTensorOps.q_into_data(again).bytes.tobytes() == blob.bytes.tobytes()
    assert FloatOps.float_into_data(QTensorOps.dequantize(again)).tobytes() == d_ref.tobytes()
    return tq, q_ref, s_ref


@pytest.mark.parametrize("sdt", [ScaleDtype.F16, ScaleDtype.BF16, ScaleDtype.UE4M3])
@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,), (16,), (2, 32)])
def test_quantize_with_two_byte_scales(dev, sdt, value, block):
    x = awkward((48, 256), 21)
    scheme = QuantScheme(value=value, scale_dtype=sdt) if block is None else QuantScheme(value=value).per_block(block, sdt)
    check_scale_dtype(dev, x, scheme)
    if value == QuantValue.Q8S:
        native = QuantScheme(store=QuantStore.Native, scale_dtype=sdt) if block is None else \
            QuantScheme(store=QuantStore.Native).per_block(block, sdt)
        check_scale_dtype(dev, x, native)
    # given scales that the dtype does not represent: rounded up before anything is divided
    n = int(np.prod(ba.quantization.params_shape(x.shape, scheme)))
    given = np.random.default_rng(3).uniform(0.01, 0.2, n).astype(np.float32)
    given[:: 7] = 0.0           # zero scales stay zero (and quantize against 0.1)
    check_scale_dtype(dev, x, scheme, given_scales=given)


@pytest.mark.parametrize("sdt", [ScaleDtype.F16, ScaleDtype.BF16, ScaleDtype.UE4M3])
def test_two_byte_scales_over_the_exponent_range(dev, sdt):
    """Blocks whose scale runs from far below the format's subnormals to past its largest value."""
    rng = np.random.default_rng(12)
    exps = np.arange(-40, 30)
    x = np.ldexp(rng.standard_normal((len(exps), 64)), exps[:, None]).astype(np.float32)
    check_scale_dtype(dev, x, QuantScheme().per_block((32,), sdt))
    check_scale_dtype(dev, x[20], QuantScheme(store=QuantStore.Native, scale_dtype=sdt))


@pytest.mark.parametrize("sdt", [ScaleDtype.F16, ScaleDtype.BF16, ScaleDtype.UE4M3])
def test_q_matmul_with_two_byte_scales(dev, sdt):
    rng = np.random.default_rng(8)
    w = (rng.standard_normal((512, 384)) * 0.02).astype(np.float32)
    scheme = QuantScheme().per_block((32,), sdt)
    tw, q_ref, s_ref = check_scale_dtype(dev, w, scheme)
    for m in (1, 16, 80):
        x = rng.standard_normal((m, 512)).astype(np.float32)
        out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tw))
        ref = no.q_matmul_f64(x, q_ref, s_ref, [32])
        matmul_check(out, ref)


# ------------------------------------------------------------------ Q2S ternary weights

# ------------------------------------------------------------------ two-level schemes

def two_level_parts(blob: TensorData):
    values, stored = blob.split()
    q = values.view(np.int8).reshape(blob.shape) if blob.scheme.store == QuantStore.Native else \
        no.unpack_u32(values.view(np.uint32), blob.shape, VAL[blob.scheme.value][1])
    return q, stored, blob.global_scale()


@pytest.mark.parametrize("value,store", [(QuantValue.Q8S, QuantStore.Native), (QuantValue.Q8S, QuantStore.PackedU32),
                                         (QuantValue.Q4S, QuantStore.PackedU32)])
@pytest.mark.parametrize("shape,block,mag", [((16, 16), (2, 16), 1.0), ((64, 256), (32,), 0.02), ((4, 6, 32), (1, 2, 16), 300.0),
                                             ((128, 512), (64,), 1e-6), ((8, 64), (8,), 5.0)])
@pytest.mark.parametrize("sdt", [ScaleDtype.F16, ScaleDtype.UE4M3])
def test_two_level_quantize_dynamic(dev, sdt, value, store, shape, block, mag):
    """f16 block scales under an f32 per-tensor scale (`.per_block(b, F16).per_tensor(F32)`): values,
    stored block scales, the per-tensor scale, the blob and the dequantized floats, all bit for bit
    against the oracle; and the blob read back gives the same tensor (the reference's round trip,
    crates/burn-backend-tests/tests/tensor/float/quantization/ops/quantize.rs:489-516)."""
    x = (np.random.default_rng(len(shape) * 100 + shape[-1]).standard_normal(shape) * mag).astype(np.float32)
    scheme = QuantScheme(value=value, store=store).per_block(block, sdt).per_tensor(ScaleDtype.F32)
    assert scheme.tensor_scale == ScaleDtype.F32 and scheme.block == block
    check_two_level(dev, x, scheme)


def check_two_level(dev, x, scheme):
    osch, code = oscheme(scheme), SDT[scheme.scale_dtype][0]
    q_ref, stored_ref, g_ref, eff_ref = co.quantize_dynamic_two_level(x, osch, code)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
    assert tq.scheme == scheme
    blob = QTensorOps.q_into_data(tq)
    q, stored, g = two_level_parts(blob)
    assert g == g_ref and stored.tobytes() == stored_ref.tobytes() and (q == q_ref).all()
    assert blob.bytes.tobytes() == co.encode_two_level(q_ref, osch, stored_ref, g_ref, code).tobytes()
    assert blob.bytes.size == TensorData.data_len(x.shape, scheme)
    d_ref = co.dequantize(q_ref, osch, eff_ref)
    assert FloatOps.float_into_data(QTensorOps.dequantize(tq)).tobytes() == d_ref.tobytes()
    again = QTensorOps.q_from_data(blob, dev)
    assert FloatOps.float_into_data(QTensorOps.dequantize(again)).tobytes() == d_ref.tobytes()
    assert QTensorOps.q_into_data(again).bytes.tobytes() == blob.bytes.tobytes()
    return tq, q_ref, eff_ref


def test_two_level_reference_cases(dev, approx):
    """The reference's own two-level cases with f16 block scales, on their inputs:
    crates/burn-backend-tests/tests/tensor/float/quantization/ops/quantize.rs:489-516 (round trip
    through the blob exact, dequantized within rel 1e-2 / abs 1e-2 of the input) and
    ops/matmul.rs:253-281 (lhs x quantized within rel 1e-2 of lhs x dequantized)."""
    x = (np.arange(256, dtype=np.float32) / np.float32(256)).reshape(16, 16)
    scheme = QuantScheme(store=QuantStore.Native).per_block((2, 16), ScaleDtype.F16).per_tensor(ScaleDtype.F32)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
    direct = FloatOps.float_into_data(QTensorOps.dequantize(tq))
    reloaded = QTensorOps.q_from_data(QTensorOps.q_into_data(tq), dev)
    assert FloatOps.float_into_data(QTensorOps.dequantize(reloaded)).tobytes() == direct.tobytes()
    approx(direct, x, 1e-2, 1e-2)
    expected = x.astype(np.float64) @ direct.astype(np.float64)
    actual = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    approx(actual, expected, 1e-2, 0)
    # quantize.rs:213-236 and 238-290 as they stand, with ue4m3 block scales: exact round trip through
    # the blob; the error is the same at either magnitude; one-level 8-bit scales degrade on small weights
    ue = QuantScheme(store=QuantStore.Native).per_block((2, 16), ScaleDtype.UE4M3)
    two, one = ue.per_tensor(ScaleDtype.F32), ue
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), two)
    direct = FloatOps.float_into_data(QTensorOps.dequantize(tq))
    blob = QTensorOps.q_into_data(tq)
    assert blob.bytes.size == 256 + 8 + 4
    assert FloatOps.float_into_data(QTensorOps.dequantize(QTensorOps.q_from_data(blob, dev))).tobytes() == direct.tobytes()

    def error(t, scheme):
        d = FloatOps.float_into_data(QTensorOps.dequantize(QTensorOps.quantize_dynamic(FloatOps.float_from_data(t, dev), scheme)))
        return np.abs(t - d).sum() / np.abs(t).sum()

    big = (np.arange(-128, 128, dtype=np.float32) / np.float32(128)).reshape(16, 16)
    small = (big * np.float32(0.02)).astype(np.float32)
    big_error, small_error = error(big, two), error(small, two)
    assert abs(small_error - big_error) / big_error < 0.2
    assert error(small, one) > small_error * 2.0
    # (the input whose largest relative scale lands one f32 step above 65504 before it is stored)
    big = (np.arange(-128, 128, dtype=np.float32) / np.float32(128)).reshape(16, 16)
    tb = QTensorOps.quantize_dynamic(FloatOps.float_from_data(big, dev), scheme)
    q_ref, stored_ref, g_ref, eff_ref = co.quantize_dynamic_two_level(big, oscheme(scheme), co.SCALE_F16)
    q, stored, g = two_level_parts(QTensorOps.q_into_data(tb))
    assert stored.max() == np.float32(65504.0) and g == g_ref and stored.tobytes() == stored_ref.tobytes() and (q == q_ref).all()


def test_two_level_reference_scheme_cases(dev, approx):
    """crates/burn-backend-tests/tests/tensor/float/quantization/scheme.rs:51-90 and 92-123, through
    quantize_dynamic on inputs with those block ranges: the largest stored ue4m3 block scale is 448,
    stored x global gives back the one-level scales (default tolerance); an all-zero tensor gets a
    positive per-tensor scale and finite block scales."""
    x = np.float32([-1.8, 0.5, 0, 0, -0.5, 1.8, 0, 0, 0.01, 0.04, 0.02, 0.03, -0.04, -0.01, -0.02, -0.03])
    one = QuantScheme(store=QuantStore.Native).per_block((4,))
    two = QuantScheme(store=QuantStore.Native).per_block((4,), ScaleDtype.UE4M3).per_tensor(ScaleDtype.F32)
    expected = QTensorOps.q_into_data(QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), one)).split()[1]
    approx(expected, np.float32([0.01417323, 0.01417323, 0.00031496, 0.00031496]))   # (scheme.rs:30-49)
    blob = QTensorOps.q_into_data(QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), two))
    _, stored, g = two_level_parts(blob)
    approx(np.float32([stored.max()]), np.float32([448.0]))
    approx(stored * g, expected)
    z = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.zeros(4, np.float32), dev), two)
    _, stored, g = two_level_parts(QTensorOps.q_into_data(z))
    assert g > 0 and np.isfinite(stored).all()
    assert (FloatOps.float_into_data(QTensorOps.dequantize(z)) == 0).all()


def test_two_level_quantize_with_given_parameters_and_other_ops(dev, tmp_path):
    rng = np.random.default_rng(77)
    x = rng.standard_normal((32, 128)).astype(np.float32)
    block_scales = (np.abs(rng.standard_normal((32, 4))) * 50 + 1).astype(np.float32)   # relative block scales
    g = np.float32(3.0e-4)
    for sdt, odt in ((ScaleDtype.F16, co.SCALE_F16), (ScaleDtype.BF16, co.SCALE_BF16), (ScaleDtype.F32, co.SCALE_F32)):
        scheme = QuantScheme().per_block((32,), sdt).per_tensor(ScaleDtype.F32)
        q_ref, stored_ref, eff_ref = co.quantize_two_level(x, oscheme(scheme), block_scales, g, odt)
        tq = QTensorOps.quantize(FloatOps.float_from_data(x, dev), scheme, FloatOps.float_from_data(block_scales, dev),
                                 FloatOps.float_from_data(np.float32([g]), dev))
        blob = QTensorOps.q_into_data(tq)
        q, stored, g_out = two_level_parts(blob)
        assert g_out == g and stored.tobytes() == stored_ref.tobytes() and (q == q_ref).all()
        d_ref = co.dequantize(q_ref, oscheme(scheme), eff_ref)
        assert FloatOps.float_into_data(QTensorOps.dequantize(tq)).tobytes() == d_ref.tobytes()
    # the products read global * s_block like any other block scale
    scheme = QuantScheme().per_block((32,), ScaleDtype.F16).per_tensor(ScaleDtype.F32)
    w = (rng.standard_normal((256, 512)) * 0.03).astype(np.float32)
    tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q_ref, stored_ref, g_ref, eff_ref = co.quantize_dynamic_two_level(w, oscheme(scheme), co.SCALE_F16)
    wd = co.dequantize(q_ref, oscheme(scheme), eff_ref).astype(np.float64)
    for m in (1, 8, 64):
        a = rng.standard_normal((m, 256)).astype(np.float32)
        out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(a, dev), tw))
        assert np.abs(out - a.astype(np.float64) @ wd).max() <= (2e-5 if m <= 32 else 1e-2) * np.abs(a.astype(np.float64) @ wd).max()
    # layout ops carry both sets of parameters; a reshape shares them
    r = QTensorOps.q_reshape(tw, (128, 1024))
    assert FloatOps.float_into_data(QTensorOps.dequantize(r)).tobytes() == wd.astype(np.float32).reshape(128, 1024).tobytes()
    assert QTensorOps.q_into_data(r).bytes.tobytes() == QTensorOps.q_into_data(tw).bytes.tobytes()
    small = QuantScheme(store=QuantStore.Native).per_block((2, 16), ScaleDtype.F16).per_tensor()
    xs = rng.standard_normal((8, 32)).astype(np.float32)
    ts = QTensorOps.quantize_dynamic(FloatOps.float_from_data(xs, dev), small)
    qs, stored_s, gs, eff_s = co.quantize_dynamic_two_level(xs, oscheme(small), co.SCALE_F16)
    tt = QTensorOps.q_swap_dims(ts, 0, 1)
    assert tt.scheme.block == (16, 2) and tt.scheme.tensor_scale == ScaleDtype.F32
    assert FloatOps.float_into_data(QTensorOps.dequantize(tt)).tobytes() == \
        co.dequantize(qs, oscheme(small), eff_s).T.copy().tobytes()
    qt, stored_t, g_t = two_level_parts(QTensorOps.q_into_data(tt))
    assert g_t == gs and stored_t.tobytes() == stored_s.T.copy().tobytes() and (qt == qs.T).all()
    tf = QTensorOps.q_flip(ts, [1])
    qf, stored_f, g_f = two_level_parts(QTensorOps.q_into_data(tf))
    assert g_f == gs and stored_f.tobytes() == stored_s.tobytes() and (qf == qs[:, ::-1]).all()
    # burnpack: the scheme travels with the entry
    path = tmp_path / "two_level.bpk"
    ba.PackWriter().add_tensor("w", tw).write_to_file(path)
    reader = ba.PackReader(path)
    assert reader.find("w")["scheme"] == scheme
    back = reader.load("w", dev)
    reader.close()
    assert back.scheme == scheme
    assert QTensorOps.q_into_data(back).bytes.tobytes() == QTensorOps.q_into_data(tw).bytes.tobytes()
    # what the reference refuses
    bad = QuantScheme().per_block((32,), ScaleDtype.BF16).per_tensor()
    with pytest.raises(ba.BurnqError):      # normalize_scales: "reach f32's range"
        QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), bad)
    with pytest.raises(ba.BurnqError):      # "requires a per-tensor scale"
        QTensorOps.quantize(FloatOps.float_from_data(x, dev), scheme, FloatOps.float_from_data(block_scales, dev))
    with pytest.raises(ba.BurnqError):      # "does not take a per-tensor scale"
        QTensorOps.quantize(FloatOps.float_from_data(x, dev), QuantScheme().per_block((32,)),
                            FloatOps.float_from_data(block_scales, dev), FloatOps.float_from_data(np.float32([g]), dev))
    with pytest.raises(ValueError):         # "stores its per-tensor scale as f32"
        QuantScheme().per_block((32,), ScaleDtype.F16).per_tensor(ScaleDtype.F16)


@pytest.mark.parametrize("block", [None, (16,), (32,), (2, 32)])
def test_q2s_quantize_dequantize(dev, block):
    x = awkward((32, 96), 33)
    scheme = QuantScheme(value=QuantValue.Q2S) if block is None else QuantScheme(value=QuantValue.Q2S).per_block(block)
    tq, q_ref, s_ref, _ = check_quantize_dynamic(dev, x, scheme)
    assert set(np.unique(q_ref).tolist()) <= {-1, 0, 1}
    if block is None:   # layout ops carry 2-bit fields too
        got, gs = unpack_blob(QTensorOps.q_into_data(QTensorOps.q_swap_dims(tq, 0, 1)))
        assert (got == q_ref.T).all() and gs.reshape(-1).tobytes() == s_ref.reshape(-1).tobytes()


@pytest.fixture
def exact_matmul(dev):
    """bq_device_set_f32_matmul_exact for the duration of a test."""
    dev.set_f32_matmul_exact(True)
    yield dev
    dev.set_f32_matmul_exact(False)


def test_q2s_ternary_matmul_is_the_reference_sum(exact_matmul):
    """f32 activations x per-tensor Q2S weight under bq_device_set_f32_matmul_exact: the multiply-free
    path, bit for bit the reference's loop (same order of additions), the reference test's own inputs
    first. (Weights whose rows are not whole groups of 4 packed words take this path by default too.)"""
    dev = exact_matmul
    a = np.float32([[0.5, -1.2, 0.3, 2.0], [1.0, 0.0, -0.7, 0.4], [-2.0, 1.5, 0.1, -0.3]])
    w = np.zeros((4, 16), np.float32)
    w[:, :3] = [[0.9, -0.2, 0.5], [-0.8, 0.1, 0.7], [0.0, 0.6, -0.4], [0.3, -0.9, 0.2]]   # padded to one packed word
    scheme = QuantScheme(value=QuantValue.Q2S)
    tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tw))
    assert q[:, :3].tolist() == [[1, 0, 1], [-1, 0, 1], [0, 1, 0], [0, -1, 0]] and s.reshape(-1)[0] == np.float32(0.9)
    out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(a, dev), tw))
    assert out.tobytes() == co.ternary_matmul(a, q, s.reshape(-1)[0]).tobytes()
    ref = FloatOps.float_into_data(FloatOps.float_matmul(FloatOps.float_from_data(a, dev), QTensorOps.dequantize(tw)))
    assert np.allclose(out, ref, rtol=2e-2, atol=1e-6)
    # an all-zero weight: exactly 0
    tz = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.zeros((3, 16), np.float32), dev), scheme)
    z = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(np.float32([[1.0, -2.0, 3.0]]), dev), tz))
    assert (z == 0).all() and not np.isnan(z).any()
    # larger shapes, ragged row counts, leading dims folded by linear, bias
    from burn_amd import ModuleOps
    rng = np.random.default_rng(58)
    for m, k, n in ((1, 257, 64), (7, 512, 1040), (33, 96, 16)):
        wr = rng.standard_normal((k, n)).astype(np.float32)
        tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(wr, dev), scheme)
        q, s = unpack_blob(QTensorOps.q_into_data(tw))
        x = rng.standard_normal((m, k)).astype(np.float32)
        got = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tw))
        assert got.tobytes() == co.ternary_matmul(x, q, s.reshape(-1)[0]).tobytes()
        bias = rng.standard_normal(n).astype(np.float32)
        lin = FloatOps.float_into_data(ModuleOps.linear(FloatOps.float_from_data(x.reshape(1, m, k), dev), tw,
                                                        FloatOps.float_from_data(bias, dev)))
        assert lin.shape == (1, m, n) and lin.reshape(m, n).tobytes() == (got + bias).astype(np.float32).tobytes()
    # infinite and NaN activations: a skipped field leaves the sum alone, +-1 adds or subtracts them
    xs = rng.standard_normal((5, k)).astype(np.float32)
    xs[0, 3], xs[1, 10], xs[2, 40], xs[3, 7], xs[3, 8] = np.inf, -np.inf, np.nan, np.inf, np.inf
    got = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(xs, dev), tw))
    want = co.ternary_matmul(xs, q, s.reshape(-1)[0])
    assert (np.isnan(got) == np.isnan(want)).all() and (got[~np.isnan(want)] == want[~np.isnan(want)]).all()
    assert np.isinf(want).any() and np.isnan(want).any() and np.isfinite(want[4]).all()
    # per-block Q2S and bf16 activations take the dequantize route, like the reference
    twb = QTensorOps.quantize_dynamic(FloatOps.float_from_data(wr, dev), QuantScheme(value=QuantValue.Q2S).per_block((16,)))
    qb, sb = unpack_blob(QTensorOps.q_into_data(twb))
    gotb = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), twb))
    matmul_check(gotb, no.q_matmul_f64(x, qb, sb, [16]))


@pytest.mark.parametrize("m,k,n", [(1, 4096, 14336), (16, 4096, 14336), (1, 257, 64), (7, 512, 1088), (17, 96, 128),
                                   (33, 1000, 576), (4, 8192, 512), (16, 31, 192), (2, 2048, 4096), (3, 130, 32)])
def test_q2s_ternary_matmul_on_the_matrix_cores(dev, m, k, n):
    """The default ternary product: the reference's sums (crates/burn-ndarray/src/ops/qtensor.rs:442-517)
    in another order, on the bf16 matrix cores with two-term activations. Against the float64 product
    of the dequantized weight: max-normalised error <= 2e-5 (q_matmul's bound is 1e-2, the reference's
    ternary test allows 2e-2) and burn's permissive rule on every element; a linear layer's bias; the
    same bits on a second call; exactly 0 for an all-zero weight; and the reference's inf / NaN pattern
    (a zero weight skips its activation: no 0 * inf)."""
    rng = np.random.default_rng(m * 7 + k + n)
    scheme = QuantScheme(value=QuantValue.Q2S)
    w = rng.standard_normal((k, n)).astype(np.float32)
    # (weights as the Quantizer makes them under Calibration::AbsMean: about a third each of -1, 0, +1)
    tw = QTensorOps.quantize_abs_mean(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tw))
    assert set(np.unique(q).tolist()) == {-1, 0, 1} and (q != 0).mean() > 0.4
    gamma = s.reshape(-1)[0]
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[rng.random(x.shape) < 0.01] *= 40
    tx = FloatOps.float_from_data(x, dev)
    got = FloatOps.float_into_data(QTensorOps.q_matmul(tx, tw))
    ref = (x.astype(np.float64) @ q.astype(np.float64)) * float(gamma)
    rel = np.abs(got - ref).max() / np.abs(ref).max()
    assert rel <= 2e-5, rel
    matmul_check(got, ref)
    again = FloatOps.float_into_data(QTensorOps.q_matmul(tx, tw))
    assert again.tobytes() == got.tobytes()
    bias = rng.standard_normal(n).astype(np.float32)
    lin = FloatOps.float_into_data(ModuleOps.linear(tx, tw, FloatOps.float_from_data(bias, dev)))
    assert lin.tobytes() == (got + bias).astype(np.float32).tobytes()
    # the reference's order on request: bit for bit its loop, and close to the default
    dev.set_f32_matmul_exact(True)
    try:
        ordered = FloatOps.float_into_data(QTensorOps.q_matmul(tx, tw))
    finally:
        dev.set_f32_matmul_exact(False)
    if m * k * n <= 1 << 24:
        assert ordered.tobytes() == co.ternary_matmul(x, q, gamma).tobytes()
    assert np.abs(ordered - got).max() <= 2e-5 * np.abs(ref).max()
    # an all-zero weight: exactly 0, also under infinite activations
    tz = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.zeros((k, n), np.float32), dev), scheme)
    z = FloatOps.float_into_data(QTensorOps.q_matmul(tx, tz))
    assert (z == 0).all()
    # infinite and NaN activations: the pattern of the reference's loop, finite outputs as before
    xs = x.copy()
    xs[0, k // 3] = np.inf
    if m > 1:
        xs[1, k // 2] = -np.inf
    if m > 2:
        xs[2, 0] = np.nan
    if m > 3:
        xs[3, 1], xs[3, k - 1] = np.inf, np.inf
    g = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(xs, dev), tw))
    qf = q.astype(np.float32)
    hits = lambda mask, sign: (mask.astype(np.float32) @ (qf * sign > 0).astype(np.float32)) > 0   # noqa: E731
    pinf = hits(np.isposinf(xs), 1) | hits(np.isneginf(xs), -1)      # a +inf contribution reaches the output
    ninf = hits(np.isposinf(xs), -1) | hits(np.isneginf(xs), 1)
    nan = hits(np.isnan(xs), 1) | hits(np.isnan(xs), -1) | (pinf & ninf)
    fin = np.where(np.isfinite(xs), xs, 0.0).astype(np.float64) @ q.astype(np.float64) * float(gamma)
    assert nan.any() == (m > 2) and pinf.any()
    assert (np.isnan(g) == nan).all()
    assert (np.isposinf(g) == (pinf & ~nan)).all() and (np.isneginf(g) == (ninf & ~nan)).all()
    ok = np.isfinite(g)
    assert ok[4:].all() and np.abs(g[ok] - fin[ok]).max() <= 2e-5 * np.abs(ref).max()


# ------------------------------------------------------------------ full-range values

def test_q8f_reference_case(dev, kats):
    """crates/burn-flex/src/ops/qtensor.rs:665-692: Q8F spans [-128, 127], scale = 2 * 7.5 / 255,
    dequantized within 0.1 of the input."""
    k = kats["quantize_dynamic_q8f"]
    x = np.float32(k["x"])
    for store in (QuantStore.Native, QuantStore.PackedU32):
        xs = x if store == QuantStore.Native else np.concatenate([x, np.float32([0, 0])])   # (whole packed words)
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(xs, dev), QuantScheme(value=QuantValue.Q8F, store=store))
        q, s = unpack_blob(QTensorOps.q_into_data(tq))
        assert abs(float(s.reshape(-1)[0]) - k["expected_scale"]) < k["scale_abs_tol"]
        assert s.reshape(-1)[0] == np.float32(2 * 7.5) / np.float32(255)
        assert q[-1 if store == QuantStore.Native else 5] == 127 and q.min() >= -128
        d = FloatOps.float_into_data(QTensorOps.dequantize(tq))
        assert np.abs(d[:6] - x).max() < k["dequant_abs_tol"]
    # the negative end of the range is reached: -absmax / s = -127.5 rounds to -128
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(-x, dev), QuantScheme(value=QuantValue.Q8F, store=QuantStore.Native))
    q, _ = unpack_blob(QTensorOps.q_into_data(tq))
    assert q[5] == -128 and q[0] == 85


@pytest.mark.parametrize("value", [QuantValue.Q8F, QuantValue.Q4F, QuantValue.Q2F])
@pytest.mark.parametrize("block", [None, (32,), (16,), (2, 32), (128,)])
def test_full_range_values_against_the_oracle(dev, value, block):
    """quantize_dynamic / quantize / dequantize with full-range values on every kernel route (per
    tensor, fused run blocks, rectangles), f32 and narrow scales, two-level: bit for bit."""
    x = awkward((64, 256), 77)
    x[5, :64] = 0.0
    scheme = QuantScheme(value=value) if block is None else QuantScheme(value=value).per_block(block)
    tq, q_ref, s_ref, _ = check_quantize_dynamic(dev, x, scheme)
    lo, hi = value.range()
    assert q_ref.min() >= lo and q_ref.max() <= hi and (q_ref.min() == lo or q_ref.max() == hi)
    if block is not None:   # among many blocks both ends of the range are reached
        assert q_ref.min() == lo and q_ref.max() == hi
    if value == QuantValue.Q8F:
        native = QuantScheme(value=value, store=QuantStore.Native, block=block)
        check_quantize_dynamic(dev, x, native)
        check_quantize_dynamic(dev, x.reshape(-1)[: 64 * 256 - 3 if block is None else 64 * 256], native if block is None else
                               QuantScheme(value=value, store=QuantStore.Native).per_block((32,)))
    # given scales (every route quantizes against them, zero scales included)
    given = s_ref.copy().reshape(-1) * np.float32(0.75)
    given[::5] = 0.0
    t = QTensorOps.quantize(FloatOps.float_from_data(x, dev), scheme, FloatOps.float_from_data(given, dev))
    q, s = unpack_blob(QTensorOps.q_into_data(t))
    assert s.reshape(-1).tobytes() == given.tobytes() and (q == co.quantize(x, oscheme(scheme), given)).all()
    check_scale_dtype(dev, x, QuantScheme(value=value, block=block, scale_dtype=ScaleDtype.BF16))
    if block is not None:
        check_two_level(dev, x, scheme.with_scale_dtype(ScaleDtype.F16).per_tensor(ScaleDtype.F32))


@pytest.mark.parametrize("value", [QuantValue.Q8F, QuantValue.Q4F])
def test_q_matmul_with_full_range_weights(dev, value):
    """The products read two's complement fields: a weight that uses the extra negative code goes
    through every kernel family like its symmetric twin."""
    rng = np.random.default_rng(31)
    w = (rng.standard_normal((512, 384)) * 0.02).astype(np.float32)
    w[np.arange(512), rng.integers(0, 384, 512)] = -0.11          # the block minimum: quantized to the lowest code
    for block in (None, (32,), (128,)):
        scheme = QuantScheme(value=value) if block is None else QuantScheme(value=value).per_block(block)
        tw, q_ref, s_ref, wd = check_quantize_dynamic(dev, w, scheme)
        assert q_ref.min() == value.range()[0]
        for m, dt in ((1, ba.F32), (2, ba.BF16), (4, ba.F32), (16, ba.F32), (24, ba.BF16), (48, ba.F32), (130, ba.BF16)):
            xh = rng.standard_normal((m, 512)).astype(np.float32)
            if dt == ba.BF16:
                bits = ba.bf16_bits_from_f32(xh)
                lhs, xd = FloatOps.float_from_data(bits, dev, ba.BF16), ba.f32_from_bf16_bits(bits)
            else:
                lhs, xd = FloatOps.float_from_data(xh, dev), xh
            out = FloatOps.float_into_data(QTensorOps.q_matmul(lhs, tw, out_dtype=ba.F32))
            matmul_check(out, xd.astype(np.float64) @ wd.astype(np.float64))


# ------------------------------------------------------------------ random schemes

def random_scheme_case(rng, native_any=False):
    """A quantizable (shape, scheme, magnitude): value, store, rank 1-4, per tensor or a block of rank
    1-rank with power-of-two extents (whole packed words along the last dim), any scale dtype, the
    two-level form for f16 / ue4m3 block scales. `native_any`: the Native store (one i8 per value) for
    4- and 2-bit values too, as the reference's CPU backend keeps them."""
    value = [QuantValue.Q8S, QuantValue.Q4S, QuantValue.Q2S, QuantValue.Q8F, QuantValue.Q4F, QuantValue.Q2F][rng.integers(6)]
    nq = 32 // value.size_bits()
    store = QuantStore.Native if (nq == 4 or native_any) and rng.integers(2) else QuantStore.PackedU32
    rank = int(rng.integers(1, 5))
    sdt = [ScaleDtype.F32, ScaleDtype.F16, ScaleDtype.BF16, ScaleDtype.UE4M3][rng.integers(4)]
    block = None
    if rng.integers(4):
        br = int(rng.integers(1, rank + 1))
        block = [int(2 ** rng.integers(0, 4)) for _ in range(br)]
        block[-1] = int(nq * 2 ** rng.integers(0, 3)) if store == QuantStore.PackedU32 else int(2 ** rng.integers(0, 7))
        block = tuple(block)
    ext = [1] * rank
    if block:
        for j in range(len(block)):
            ext[rank - 1 - j] = block[len(block) - 1 - j]
    elif store == QuantStore.PackedU32:
        ext[-1] = nq
    shape = tuple(int(e * rng.integers(1, 4)) for e in ext)
    scheme = QuantScheme(value=value, store=store, scale_dtype=sdt) if block is None else \
        QuantScheme(value=value, store=store).per_block(block, sdt)
    if block is not None and sdt in (ScaleDtype.F16, ScaleDtype.UE4M3) and rng.integers(2):
        scheme = scheme.per_tensor(ScaleDtype.F32)
    return shape, scheme, float(10.0 ** rng.integers(-4, 4))


def test_random_schemes_against_the_oracle(dev):
    """300 seeded cases over the whole scheme space: quantize_dynamic's blob, the dequantized floats
    and the blob round trip bit for bit, then one layout op (swap / permute / flip) on the result,
    whose dequantized values must be the same permutation of the source's."""
    scheme_sweep(dev, np.random.default_rng(20240607), 300, False, 60)


def test_random_schemes_with_any_value_stored_natively(dev):
    """150 more cases of the same sweep in which 4- and 2-bit values are stored natively half of the
    time (one i8 per value: no word to fill, so any shape goes and every layout op applies)."""
    scheme_sweep(dev, np.random.default_rng(515), 150, True, 40)


def scheme_sweep(dev, rng, cases, native_any, distinct):
    seen = set()
    for case in range(cases):
        shape, scheme, mag = random_scheme_case(rng, native_any)
        x = (rng.standard_normal(shape) * mag).astype(np.float32)
        if rng.integers(5) == 0:
            x[rng.random(shape) < 0.3] = 0.0
        label = f"case {case}: {shape} {scheme}"
        try:
            if scheme.tensor_scale is not None:
                tq, _, _ = check_two_level(dev, x, scheme)
            elif scheme.scale_dtype != ScaleDtype.F32:
                tq, _, _ = check_scale_dtype(dev, x, scheme)
            else:
                tq, _, _, _ = check_quantize_dynamic(dev, x, scheme)
        except AssertionError as e:
            raise AssertionError(f"{label}: {e}") from e
        seen.add((scheme.value, scheme.store, scheme.block is None, scheme.scale_dtype, scheme.tensor_scale))
        d = FloatOps.float_into_data(QTensorOps.dequantize(tq))
        rank = len(shape)
        axes = [int(a) for a in rng.permutation(rank)]
        nq = tq.scheme.num_quants()
        if rank > 1 and (nq == 4 or scheme.store == QuantStore.Native or shape[axes[-1]] % nq == 0):
            tp = QTensorOps.q_permute(tq, axes)
            got = FloatOps.float_into_data(QTensorOps.dequantize(tp))
            assert got.tobytes() == np.ascontiguousarray(np.transpose(d, axes)).tobytes(), f"{label}: permute {axes}"
        fl = sorted({int(a) for a in rng.integers(0, rank, 2)})
        if scheme.block is None:   # (a flip keeps block scales in place: only per-tensor values commute with it)
            got = FloatOps.float_into_data(QTensorOps.dequantize(QTensorOps.q_flip(tq, fl)))
            assert got.tobytes() == np.ascontiguousarray(np.flip(d, fl)).tobytes(), f"{label}: flip {fl}"
    assert len(seen) >= distinct   # of the (value, store) x (level, scale dtype, two-level) combinations


def test_random_matmuls_against_float64(dev):
    """150 seeded products over the scheme space and the shapes that pick each kernel family: a float
    (f32 / bf16) or quantized lhs, a quantized rhs of any scheme (any block shape, scale dtype,
    two-level, ternary), batch dims that broadcast, M from 1 to 130. Against the float64 product of
    the dequantized operands (dequantize itself is checked bit for bit elsewhere)."""
    rng = np.random.default_rng(777)

    def family_case():
        """Weights shaped for the fused kernels: whole 128-column groups, K in 32-row steps (or not)."""
        value = [QuantValue.Q8S, QuantValue.Q4S, QuantValue.Q8F, QuantValue.Q4F][rng.integers(4)]
        store = QuantStore.Native if value.size_bits() == 8 and rng.integers(3) == 0 else QuantStore.PackedU32
        n = int([128, 256, 384, 640, 1024, 96, 48][rng.integers(7)])
        k = int([32, 64, 96, 256, 512, 1000, 40][rng.integers(7)])
        block = [None, (32,), (64,), (128,), (16,), (8,)][rng.integers(6)]
        if block is not None and n % block[0]:
            block = (16,)
        sdt = [ScaleDtype.F32, ScaleDtype.F16, ScaleDtype.BF16, ScaleDtype.UE4M3][rng.integers(4)]
        scheme = QuantScheme(value=value, store=store, scale_dtype=sdt) if block is None else \
            QuantScheme(value=value, store=store).per_block(block, sdt)
        if block is not None and sdt in (ScaleDtype.F16, ScaleDtype.UE4M3) and rng.integers(3) == 0:
            scheme = scheme.per_tensor(ScaleDtype.F32)
        batch = [(), (), (2,), (1, 3)][rng.integers(4)]
        return batch + (k, n), scheme

    for case in range(150):
        shape, scheme, _ = random_scheme_case(rng)
        if case % 2:
            shape, scheme = family_case()
        if len(shape) < 2:
            shape = (int(rng.integers(1, 5)) * 8,) + shape
            if scheme.block is not None and len(scheme.block) > 1:
                scheme = QuantScheme(value=scheme.value, store=scheme.store).per_block(scheme.block[-1:], scheme.scale_dtype)
        # a longer K now and then (the split-K and tiled kernels), keeping the block's divisibility
        if case % 2 == 0 and rng.integers(3) == 0:
            kb = 1
            if scheme.block is not None and len(scheme.block) >= 2:
                kb = scheme.block[-2]
            shape = shape[:-2] + (shape[-2] * int(rng.integers(2, 9)) * (32 // np.gcd(32, kb) if rng.integers(2) else 1),) + shape[-1:]
            # (K stays at 2048 and below: on the kernels that round to bf16 the error is 2.3e-3 of the
            # output's rms, and with these inputs the elementwise rule's absolute 1e-2 is 4.8 sigma
            # there; at K = 6144 it is 2.8 sigma and a few outputs in a thousand pass it)
            while shape[-2] > 2048 and shape[-2] % 2 == 0:
                shape = shape[:-2] + (shape[-2] // 2,) + shape[-1:]
        rank = len(shape)
        w = (rng.standard_normal(shape) * 0.02).astype(np.float32)
        tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
        wd = FloatOps.float_into_data(QTensorOps.dequantize(tw)).astype(np.float64)
        m = int([1, 2, 3, 4, 5, 8, 16, 17, 32, 33, 64, 130][rng.integers(12)])
        batch = tuple(1 if rng.integers(3) == 0 else b for b in shape[:-2])
        xs = batch + (m, shape[-2])
        xh = rng.standard_normal(xs).astype(np.float32)
        kind = int(rng.integers(4))
        label = f"case {case}: lhs {xs} kind {kind} x rhs {shape} {scheme}"
        if kind == 0:      # f32 activations
            lhs, xd = FloatOps.float_from_data(xh, dev), xh.astype(np.float64)
        elif kind == 1:    # bf16 activations
            bits = ba.bf16_bits_from_f32(xh)
            lhs, xd = FloatOps.float_from_data(bits, dev, ba.BF16), ba.f32_from_bf16_bits(bits).astype(np.float64)
        else:              # a quantized lhs (per tensor, or blocks along K)
            k = xs[-1]
            ls = QuantScheme(store=QuantStore.Native) if kind == 2 or k % 4 else QuantScheme().per_block((4,))
            lhs = QTensorOps.quantize_dynamic(FloatOps.float_from_data(xh, dev), ls)
            xd = FloatOps.float_into_data(QTensorOps.dequantize(lhs)).astype(np.float64)
        ref = xd @ wd
        try:
            out = FloatOps.float_into_data(QTensorOps.q_matmul(lhs, tw, out_dtype=ba.F32))
            assert out.shape == ref.shape
            if np.abs(ref).max() == 0:
                assert (out == 0).all()
            else:
                matmul_check(out, ref)
        except (AssertionError, ba.BurnqError) as e:
            raise AssertionError(f"{label}: {e}") from e


# ------------------------------------------------------------------ burnpack files

def test_burnpack_round_trip_of_device_tensors(dev, tmp_path):
    """Quantized and float tensors written to a .bpk file and loaded back into device memory:
    every blob comes back byte for byte, straight out of the mapped file."""
    from burn_amd import PackReader, PackWriter
    rng = np.random.default_rng(90)
    w = (rng.standard_normal((256, 512)) * 0.02).astype(np.float32)
    cases = {
        "layer.weight.q8_block": QuantScheme().per_block((32,)),
        "layer.weight.q4_block": QuantScheme(value=QuantValue.Q4S).per_block((32,)),
        "layer.weight.q8_tensor_native": QuantScheme(store=QuantStore.Native),
        "layer.weight.q8_bf16_scales": QuantScheme().per_block((32,), ScaleDtype.BF16),
        "layer.weight.ragged_native": QuantScheme(store=QuantStore.Native),      # value bytes not a multiple of 256
    }
    tensors, writer = {}, PackWriter().with_metadata("producer", "burn_amd tests")
    for i, (name, scheme) in enumerate(cases.items()):
        src = w[:3, :67] if "ragged" in name else w
        tensors[name] = QTensorOps.quantize_dynamic(FloatOps.float_from_data(np.ascontiguousarray(src), dev), scheme)
        writer.add_tensor(name, tensors[name], param_id=1000 + i)
    bias = rng.standard_normal(512).astype(np.float32)
    writer.add_tensor("layer.bias", FloatOps.float_from_data(bias, dev))
    path = tmp_path / "model.bpk"
    writer.write_to_file(path)
    raw = path.read_bytes()
    assert raw[:4] == b"NRUB" and len(raw) == writer.size()
    reader = PackReader(tmp_path / "model")                     # the canonical extension is appended
    assert len(reader) == len(cases) + 1 and reader.metadata("producer") == "burn_amd tests"
    for i, (name, scheme) in enumerate(cases.items()):
        e = reader.find(name)
        blob = QTensorOps.q_into_data(tensors[name])
        assert e["dtype"] == "QFloat" and e["scheme"] == scheme and e["param_id"] == 1000 + i
        assert e["data_offsets"][0] % 256 == 0 and e["data_offsets"][1] - e["data_offsets"][0] == blob.bytes.size
        for given in (None, scheme):                              # the file's own scheme, or the caller's
            back = reader.load(name, dev, scheme=given)
            assert back.shape == tensors[name].shape and back.scheme == scheme
            assert QTensorOps.q_into_data(back).bytes.tobytes() == blob.bytes.tobytes()
        d0 = FloatOps.float_into_data(QTensorOps.dequantize(tensors[name]))
        d1 = FloatOps.float_into_data(QTensorOps.dequantize(reader.load(name, dev)))
        assert d0.tobytes() == d1.tobytes()
    assert FloatOps.float_into_data(reader.load("layer.bias", dev)).tobytes() == bias.tobytes()
    # a scheme that does not describe the stored bytes is the reference's size mismatch
    with pytest.raises(ba.BurnqError):
        reader.load("layer.weight.q8_block", dev, scheme=QuantScheme(value=QuantValue.Q4S).per_block((32,)))


def test_burnpack_container_written_by_the_reference(dev):
    """tests/golden/mnist_model.bpk is examples/mnist-inference-web/model.bpk of the reference tree, a
    container its own BurnpackWriter wrote (18 f32 tensors). Every tensor goes from the mapped file to
    the device and comes back byte for byte; the two linear weights that fill whole blocks are then
    quantized, written by this library's writer next to the originals, and read back."""
    import os
    from burn_amd import PackReader, PackWriter
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mnist_model.bpk")
    raw = open(path, "rb").read()
    reader = PackReader(path)
    assert len(reader) == 18
    import struct
    msize = struct.unpack("<IHI", raw[:10])[2]
    start = (10 + msize + 255) // 256 * 256
    loaded = {}
    for e in reader.entries():
        assert e["dtype"] == "F32"
        begin, end = e["data_offsets"]
        t = reader.load(e["name"], dev)
        assert t.shape == tuple(e["shape"]) and t.dtype == ba.F32
        back = FloatOps.float_into_data(t)
        assert back.tobytes() == raw[start + begin:start + end], e["name"]
        loaded[e["name"]] = (t, back)
    # quantize what a Quantizer would (the linear weights), save, reload: blobs identical
    writer = PackWriter()
    for name, scheme in (("fc1.weight", QuantScheme().per_block((32,))), ("fc2.weight", QuantScheme(value=QuantValue.Q4S).per_block((32,)))):
        t, host = loaded[name]
        tq = QTensorOps.quantize_dynamic(t, scheme)
        q_ref, s_ref = co.quantize_dynamic(host, oscheme(scheme))
        blob = QTensorOps.q_into_data(tq).bytes
        assert blob.tobytes() == co.encode(q_ref, oscheme(scheme), s_ref).tobytes()
        writer.add_tensor(name, tq, param_id=reader.find(name)["param_id"])
    again = PackReader(writer.into_bytes())
    for name in ("fc1.weight", "fc2.weight"):
        e = again.find(name)
        assert e["dtype"] == "QFloat" and e["param_id"] == reader.find(name)["param_id"]
        d = FloatOps.float_into_data(QTensorOps.dequantize(again.load(name, dev)))
        assert np.abs(d - loaded[name][1]).max() <= np.abs(loaded[name][1]).max() / (127 if name == "fc1.weight" else 7)


def test_burnpack_quantized_entry_of_another_producer(dev):
    """A container assembled by hand whose dtype field is a `{"QFloat": <map>}` this library did not
    write (serde's image of DType::QFloat(scheme); the scheme's own image is decided outside the
    reference tree): the reader takes dtype, shape and bytes from the file, the scheme from the
    caller, and the tensor equals what the oracle serialises."""
    from test_pack import container
    from burn_amd import PackReader
    rng = np.random.default_rng(91)
    x = (rng.standard_normal((64, 96)) * 0.05).astype(np.float32)
    cases = {"q8": QuantScheme().per_block((32,)), "q4": QuantScheme(value=QuantValue.Q4S), "q8n": QuantScheme(store=QuantStore.Native).per_block((8, 16))}
    foreign = {"QFloat": {"value": "Q8S", "mode": "Symmetric", "store": {"PackedNative": 3}, "level": {"Blocks": [7]}, "param": "F64"}}
    blobs = {}
    for name, scheme in cases.items():
        q_ref, s_ref = co.quantize_dynamic(x, oscheme(scheme))
        blobs[name] = (co.encode(q_ref, oscheme(scheme), s_ref), co.dequantize(q_ref, oscheme(scheme), s_ref))
    raw = container([(name, foreign, x.shape, blobs[name][0].tobytes()) for name in cases])
    reader = PackReader(raw)
    for name, scheme in cases.items():
        e = reader.find(name)
        assert e["dtype"] == "QFloat" and e["scheme"] is None and tuple(e["shape"]) == x.shape
        with pytest.raises(ba.BurnqError, match="pass the scheme"):
            reader.load(name, dev)
        t = reader.load(name, dev, scheme=scheme)
        assert t.scheme == scheme and QTensorOps.q_into_data(t).bytes.tobytes() == blobs[name][0].tobytes()
        assert FloatOps.float_into_data(QTensorOps.dequantize(t)).tobytes() == blobs[name][1].tobytes()


# ------------------------------------------------------------------ integer-domain ops

REFERENCE_SLICE_CASES = [        # crates/burn-backend-tests/tests/cubecl/quantization/slice.rs:40-128
    ((8,), (slice(None),)), ((8,), (slice(2, 6),)), ((4, 8), (slice(1, 3), slice(None))), ((4, 8), (slice(None), slice(0, 4))),
    ((4, 8), (slice(1, 3), slice(4, 8))), ((2, 3, 8), (slice(0, 1), slice(1, 3), slice(None))), ((4, 8), (1, slice(None))),
    ((4, 8), (slice(1, 3), slice(None))),                    # s![1..=2, ..]
    ((4, 8), (slice(-2, None), slice(None))), ((4, 8), (slice(None), slice(-4, None))), ((8, 8), (slice(0, 8, 2), slice(None))),
    ((4, 8), (slice(None), slice(0, 8, 2))), ((4, 8), (slice(None, None, -1), slice(None))), ((4, 8), (slice(None), slice(None, None, -1))),
    ((4, 8), (slice(1, 3),)),
]


def burn_slice(a, slices):
    """numpy evaluation of burn's Slice (crates/burn-std/src/tensor/slice.rs:493-545): the range start..end is
    normalised first (negative indices from the end, clamped), then walked with the step -- backwards from its last
    element when the step is negative."""
    out = a
    for d, s in enumerate(slices):
        size = a.shape[d]
        if isinstance(s, int):
            s = slice(s, None if s == -1 else s + 1, 1)
        conv = lambda i: max(size + i, 0) if i < 0 else min(i, size)   # noqa: E731
        start = 0 if s.start is None else conv(s.start)
        end = size if s.stop is None else conv(s.stop)
        step = 1 if s.step is None else s.step
        idx = np.arange(start, max(end, start))
        idx = idx[::step] if step > 0 else idx[::-1][::-step]
        out = np.take(out, idx, axis=d)
    return out


@pytest.mark.parametrize("shape,slices", REFERENCE_SLICE_CASES)
def test_q_slice_reference_cases(dev, shape, slices):
    """The reference's q_slice cases (arange / numel, its default scheme: Q8F per tensor, packed): slicing
    the quantized tensor and dequantizing equals dequantizing and slicing -- bit for bit here, where the
    reference allows Tolerance::permissive() -- and the integers are the sliced integers."""
    numel = int(np.prod(shape))
    x = (np.arange(numel, dtype=np.float32) / np.float32(numel)).reshape(shape)
    scheme = QuantScheme(value=QuantValue.Q8F)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
    q_ref, s_ref = co.quantize_dynamic(x, oscheme(scheme))
    want = burn_slice(co.dequantize(q_ref, oscheme(scheme), s_ref), slices)
    got_t = QTensorOps.q_slice(tq, slices)
    assert got_t.shape == want.shape and got_t.scheme == scheme
    got = FloatOps.float_into_data(QTensorOps.dequantize(got_t))
    assert got.tobytes() == np.ascontiguousarray(want).tobytes()
    q, s = unpack_blob(QTensorOps.q_into_data(got_t))
    assert (q == burn_slice(q_ref, slices)).all() and s.tobytes() == s_ref.tobytes()


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S, QuantValue.Q2S])
@pytest.mark.parametrize("store", [QuantStore.PackedU32, QuantStore.Native])
def test_integer_domain_ops_against_numpy(dev, value, store):
    """q_slice / q_select / q_gather / q_expand / q_argmax / q_argmin (crates/burn-ndarray/src/ops/qtensor.rs:349-430)
    on seeded tensors, per tensor and per block: the result's integers are numpy's op on the oracle's
    integers, its scales the op on the scales (in block units), the scheme unchanged."""
    rng = np.random.default_rng(11 + 3 * int(value == QuantValue.Q4S) + int(store == QuantStore.Native))
    x = awkward((6, 8, 64), 77)
    for block in (None, (32,), (2, 1, 16)):
        scheme = QuantScheme(value=value, store=store) if block is None else QuantScheme(value=value, store=store).per_block(block)
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
        q_ref, s_ref = co.quantize_dynamic(x, oscheme(scheme))
        blk = (1, 1, 1) if block is None else tuple([1] * (3 - len(block)) + list(block))

        def check(t, q_want, s_want):
            q, s = unpack_blob(QTensorOps.q_into_data(t))
            assert t.shape == q_want.shape and (q == q_want).all()
            assert s.reshape(-1).tobytes() == np.ascontiguousarray(s_want, np.float32).reshape(-1).tobytes()
            d = FloatOps.float_into_data(QTensorOps.dequantize(t))
            return d

        pshape = [6 // blk[0], 8 // blk[1], 64 // blk[2]]
        s_elem = np.kron(s_ref.reshape(pshape), np.ones(blk, np.float32)) if block is not None else None   # one scale per element

        def scales_of(op):               # the op on the per-element scales, one value kept per block
            return s_ref if block is None else op(s_elem)[::blk[0], ::blk[1], ::blk[2]]

        # slices that keep whole blocks and whole packed words
        for slices in ((slice(2, 6), slice(None), slice(32, 64)), (slice(None, None, 1), slice(3, 8), slice(None)),
                       (slice(0, 2), 5, slice(0, 32)), (slice(-4, None), slice(None, None, -1), slice(None))):
            d = check(QTensorOps.q_slice(tq, slices), burn_slice(q_ref, slices), scales_of(lambda a: burn_slice(a, slices)))
            assert d.tobytes() == np.ascontiguousarray(burn_slice(co.dequantize(q_ref, oscheme(scheme), s_ref), slices)).tobytes()
        # a cut inside a block is declined (the trait's default takes over)
        if block is not None:
            with pytest.raises(ba.BurnqError) as e:
                QTensorOps.q_slice(tq, (slice(None), slice(None), slice(8, 40)))
            assert e.value.status == ba._lib.ERR_UNSUPPORTED_OP
        # select along a dim whose blocks are 1 wide
        idx = rng.integers(0, 8, 5)
        for np_idx in (idx.astype(np.int32), idx.astype(np.int64)):
            check(QTensorOps.q_select(tq, 1, IntOps.int_from_data(np_idx, dev)), np.take(q_ref, idx, axis=1),
                  scales_of(lambda a: np.take(a, idx, axis=1)))
        # expand: new leading dims
        check(QTensorOps.q_expand(tq, (3, 6, 8, 64)), np.broadcast_to(q_ref, (3, 6, 8, 64)),
              s_ref if block is None else np.broadcast_to(s_ref.reshape(pshape), [3] + pshape))
        if block is None:
            # gather along every dim, and a dim of 1 broadcast
            for dim in range(3):
                shape = list(x.shape)
                shape[dim] = 16 if dim == 2 else 4     # whole packed words along the last dim
                gi = rng.integers(0, x.shape[dim], shape)
                check(QTensorOps.q_gather(dim, tq, IntOps.int_from_data(gi.astype(np.int64), dev)), np.take_along_axis(q_ref, gi, axis=dim), s_ref)
            one = QTensorOps.q_slice(tq, (slice(None), slice(2, 3), slice(None)))
            check(QTensorOps.q_expand(one, (6, 5, 64)), np.broadcast_to(q_ref[:, 2:3, :], (6, 5, 64)), s_ref)
            for dim in range(3):
                for dtype, npd in ((ba.I32, np.int32), (ba.I64, np.int64)):
                    am = IntOps.int_into_data(QTensorOps.q_argmax(tq, dim, dtype))
                    an = IntOps.int_into_data(QTensorOps.q_argmin(tq, dim, dtype))
                    assert am.dtype == npd and (am == np.expand_dims(q_ref.argmax(axis=dim), dim)).all()
                    assert (an == np.expand_dims(q_ref.argmin(axis=dim), dim)).all()
            # the arg over the integers is the arg over the dequantized values
            deq = co.dequantize(q_ref, oscheme(scheme), s_ref)
            assert (IntOps.int_into_data(QTensorOps.q_argmax(tq, 2)) == np.expand_dims(deq.argmax(axis=2), 2)).all()
        else:
            with pytest.raises(ba.BurnqError) as e:
                QTensorOps.q_gather(0, tq, IntOps.int_from_data(np.zeros((2, 8, 64), np.int64), dev))
            assert e.value.status == ba._lib.ERR_UNSUPPORTED_OP
            with pytest.raises(ba.BurnqError) as e:
                QTensorOps.q_argmax(tq, 2)
            assert e.value.status == ba._lib.ERR_UNSUPPORTED_OP
    # results that do not fill packed words: Q8S goes native with the same bytes, sub-byte values are refused
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), QuantScheme(value=value, store=store))
    q_ref, s_ref = co.quantize_dynamic(x, oscheme(QuantScheme(value=value, store=store)))
    if value == QuantValue.Q8S or store == QuantStore.Native:
        t = QTensorOps.q_slice(tq, (slice(None), slice(None), slice(1, 4)))
        q, s = unpack_blob(QTensorOps.q_into_data(t))
        assert t.scheme.store == QuantStore.Native and (q == q_ref[:, :, 1:4]).all()
    else:
        with pytest.raises(ba.BurnqError) as e:
            QTensorOps.q_slice(tq, (slice(None), slice(None), slice(1, 4)))
        assert e.value.status == ba._lib.ERR_SHAPE
    # out-of-range indices are clamped, never a fault
    far = IntOps.int_from_data(np.int64([-5, 0, 7, 100]), dev)
    q, _ = unpack_blob(QTensorOps.q_into_data(QTensorOps.q_select(tq, 1, far)))
    assert (q == np.take(q_ref, [0, 0, 7, 7], axis=1)).all()


def test_integer_domain_ops_random_configurations(dev):
    """Seeded draws over ranks 1-4, Q8S / Q4S / Q2S, packed and native stores, per-tensor schemes and blocks
    along the last dim: random slices (negative indices, steps of either sign, single indices), selects,
    expands and arg reductions against numpy on the oracle's integers and scales. Both routes of the
    index map run: whole-row copies where the last dim is kept or cut at word boundaries, the element
    gather elsewhere."""
    rng = np.random.default_rng(20260)
    done = {"slice": 0, "select": 0, "expand": 0, "arg": 0, "declined": 0}
    for case in range(160):
        value = [QuantValue.Q8S, QuantValue.Q4S, QuantValue.Q2S][case % 3]
        store = QuantStore.PackedU32 if (case // 3) % 2 == 0 else QuantStore.Native
        nq = {QuantValue.Q8S: 4, QuantValue.Q4S: 8, QuantValue.Q2S: 16}[value]
        rank = int(rng.integers(1, 5))
        last = int(rng.choice([32, 64, 96, 128]))
        shape = tuple(int(rng.integers(1, 7)) for _ in range(rank - 1)) + (last,)
        blocked = case % 4 == 1
        scheme = QuantScheme(value=value, store=store)
        if blocked:
            scheme = scheme.per_block((32,))
        x = awkward(shape, 9000 + case)
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
        q_ref, s_ref = co.quantize_dynamic(x, oscheme(scheme))
        pshape = shape[:-1] + (last // 32,) if blocked else None
        s_nd = s_ref.reshape(pshape) if blocked else None

        def check(t, q_want, s_want):
            q, s = unpack_blob(QTensorOps.q_into_data(t))
            assert t.shape == q_want.shape, (case, t.shape, q_want.shape)
            assert (q == q_want).all(), case
            assert s.reshape(-1).tobytes() == np.ascontiguousarray(s_want, np.float32).reshape(-1).tobytes(), case

        kind = case % 5
        if kind in (0, 1):          # slice: any cut of the leading dims; the last dim in whole blocks / words, or freely
            slices = []
            for a, n in enumerate(shape[:-1]):
                pick = int(rng.integers(0, 4))
                if pick == 0:
                    slices.append(slice(None))
                elif pick == 1:
                    slices.append(int(rng.integers(-n, n)))
                else:
                    lo, hi = sorted(int(v) for v in rng.integers(-n, n + 1, 2))
                    step = int(rng.choice([1, 1, 2, -1, -2]))
                    slices.append(slice(lo, hi if hi != lo else None, step))
            free = kind == 1 and not blocked and (value == QuantValue.Q8S or store == QuantStore.Native)
            if free:                # any range and step: the result may not fill packed words (Q8S goes native)
                lo, hi = sorted(int(v) for v in rng.integers(0, last + 1, 2))
                slices.append(slice(lo, max(hi, lo + 1), int(rng.choice([1, 3, -1]))))
            else:
                lo = 32 * int(rng.integers(0, last // 32))
                hi = 32 * int(rng.integers(lo // 32 + 1, last // 32 + 1))
                slices.append(slice(lo, hi))
            want_q = burn_slice(q_ref, slices)
            if want_q.size == 0:
                continue
            if blocked:
                sb = list(slices[:-1]) + [slice(slices[-1].start // 32, slices[-1].stop // 32)]
                want_s = burn_slice(s_nd, sb)
            else:
                want_s = s_ref
            check(QTensorOps.q_slice(tq, tuple(slices)), want_q, want_s)
            done["slice"] += 1
        elif kind == 2:             # select along a leading dim (blocks of 1 there); the last dim only per tensor
            dim = int(rng.integers(0, rank)) if not blocked else int(rng.integers(0, max(rank - 1, 1)))
            if blocked and rank == 1:
                with pytest.raises(ba.BurnqError):
                    QTensorOps.q_select(tq, 0, IntOps.int_from_data(np.int64([0]), dev))
                done["declined"] += 1
                continue
            count = int(rng.integers(1, 9)) if dim < rank - 1 else nq * int(rng.integers(1, 4))
            idx = rng.integers(0, shape[dim], count)
            it = IntOps.int_from_data(idx.astype(np.int32 if case % 2 else np.int64), dev)
            if dim == rank - 1 and store == QuantStore.PackedU32 and value != QuantValue.Q8S and count % nq:
                continue
            want_s = np.take(s_nd, idx, axis=dim) if blocked else s_ref
            check(QTensorOps.q_select(tq, dim, it), np.take(q_ref, idx, axis=dim), want_s)
            done["select"] += 1
        elif kind == 3:             # expand: new leading dims and dims of 1
            if rank > 1 and shape[0] != 1:
                src_t, src_q, src_s = QTensorOps.q_slice(tq, (0,)), q_ref[0:1], (s_nd[0:1] if blocked else s_ref)
            else:
                src_t, src_q, src_s = tq, q_ref, (s_nd if blocked else s_ref)
            lead = tuple(int(v) for v in rng.integers(1, 4, int(rng.integers(0, 3))))
            target = lead + ((int(rng.integers(2, 5)),) + src_q.shape[1:] if rank > 1 else src_q.shape)
            if len(target) > 6:
                continue
            want_s = np.broadcast_to(src_s, lead + ((target[len(lead)],) + src_s.shape[1:] if rank > 1 else src_s.shape)) if blocked else s_ref
            check(QTensorOps.q_expand(src_t, target), np.broadcast_to(src_q, target), want_s)
            done["expand"] += 1
        else:                       # arg reductions: per tensor along any dim
            if blocked:             # blocks of 32 along a longer last dim: the order of the integers is not the values'
                if last > 32:
                    with pytest.raises(ba.BurnqError) as e:
                        QTensorOps.q_argmax(tq, rank - 1)
                    assert e.value.status == ba._lib.ERR_UNSUPPORTED_OP
                    done["declined"] += 1
                continue
            dim = int(rng.integers(0, rank))
            for fn, npf in ((QTensorOps.q_argmax, np.argmax), (QTensorOps.q_argmin, np.argmin)):
                got = IntOps.int_into_data(fn(tq, dim, ba.I32 if case % 2 else ba.I64))
                assert (got == np.expand_dims(npf(q_ref, axis=dim), dim)).all(), (case, dim)
            done["arg"] += 1
    assert done["slice"] >= 40 and done["select"] >= 15 and done["expand"] >= 15 and done["arg"] >= 15, done


@pytest.mark.parametrize("shape", [(37, 1000), (5, 8240), (3, 4, 16400), (64, 64), (9, 77)])
def test_q_arg_along_long_and_ragged_rows(dev, shape):
    """q_argmax / q_argmin along the last dim where the wave-per-row kernel walks several 16-byte pieces per
    lane, rows that do not start on 16-byte boundaries, tails shorter than a piece, and many ties (values
    quantized to a few levels): the first index of the extreme, as numpy's."""
    rng = np.random.default_rng(shape[-1])
    x = np.round(rng.standard_normal(shape) * 3).astype(np.float32)          # few distinct levels: ties everywhere
    x[..., -1] = x.max() if shape[-1] % 2 else x.min()                      # an extreme in the ragged tail
    scheme = QuantScheme(value=QuantValue.Q8S, store=QuantStore.Native)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
    q_ref, _ = co.quantize_dynamic(x, oscheme(scheme))
    last = len(shape) - 1
    for dtype in (ba.I32, ba.I64):
        assert (IntOps.int_into_data(QTensorOps.q_argmax(tq, last, dtype)) == np.expand_dims(q_ref.argmax(axis=last), last)).all()
        assert (IntOps.int_into_data(QTensorOps.q_argmin(tq, last, dtype)) == np.expand_dims(q_ref.argmin(axis=last), last)).all()
    assert (IntOps.int_into_data(QTensorOps.q_argmax(tq, 0)) == np.expand_dims(q_ref.argmax(axis=0), 0)).all()


def test_integer_domain_ops_on_two_level_and_narrow_scale_tensors(dev):
    """Slices, selects and expands of tensors whose block scales are stored narrow (f16 / ue4m3), alone or
    under an f32 per-tensor scale: the result dequantizes to the op on the dequantized source bit for bit,
    and its blob (stored block scales, per-tensor scale) survives q_into_data -> q_from_data."""
    x = awkward((12, 6, 128), 4242)
    for scheme in (QuantScheme(value=QuantValue.Q8S).per_block((32,), ScaleDtype.F16).per_tensor(ScaleDtype.F32),
                   QuantScheme(value=QuantValue.Q4S).per_block((32,), ScaleDtype.UE4M3).per_tensor(ScaleDtype.F32),
                   QuantScheme(value=QuantValue.Q8S).per_block((32,), ScaleDtype.BF16)):
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
        d = FloatOps.float_into_data(QTensorOps.dequantize(tq))
        idx = np.int64([11, 0, 3, 3, 7])
        for got_t, want in ((QTensorOps.q_slice(tq, (slice(2, 10, 3), slice(None, None, -1), slice(32, 128))), d[2:10:3, ::-1, 32:128]),
                            (QTensorOps.q_select(tq, 0, IntOps.int_from_data(idx, dev)), d[idx]),
                            (QTensorOps.q_expand(QTensorOps.q_slice(tq, (slice(4, 5),)), (3, 6, 128)), np.broadcast_to(d[4:5], (3, 6, 128)))):
            assert got_t.scheme == scheme
            got = FloatOps.float_into_data(QTensorOps.dequantize(got_t))
            assert got.tobytes() == np.ascontiguousarray(want).tobytes()
            blob = QTensorOps.q_into_data(got_t)
            assert blob.bytes.size == TensorData.data_len(got_t.shape, scheme)
            again = QTensorOps.q_from_data(blob, dev)
            assert FloatOps.float_into_data(QTensorOps.dequantize(again)).tobytes() == got.tobytes()
            assert QTensorOps.q_into_data(again).bytes.tobytes() == blob.bytes.tobytes()


def _int8(dev, floats):
    """The reference tests' QTensor::int8: quantize_dynamic, Q8S per tensor (native store, as the backends
    that run them; crates/burn-backend-tests/tests/tensor/float/quantization/mod.rs:23-50)."""
    x = np.asarray(floats, np.float32)
    return QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), QuantScheme(value=QuantValue.Q8S, store=QuantStore.Native))


def _deq(t):
    return FloatOps.float_into_data(QTensorOps.dequantize(t))


def test_q_arg_expand_select_gather_reference_cases(dev):
    """The reference's own cases for the integer-domain ops
    (crates/burn-backend-tests/tests/tensor/float/quantization/ops/extended/{arg,expand,select,gather_scatter}.rs),
    inputs and expected outputs as written there, with the tolerance each of them states."""
    # arg.rs:6-50
    a = [[10.0, 11.0, 2.0], [3.0, 4.0, 5.0]]
    b = [[10.0, 11.0, 2.0], [30.0, 4.0, 5.0]]
    assert IntOps.int_into_data(QTensorOps.q_argmax(_int8(dev, a), 0)).tolist() == [[0, 0, 1]]
    assert IntOps.int_into_data(QTensorOps.q_argmin(_int8(dev, b), 0)).tolist() == [[0, 1, 0]]
    assert IntOps.int_into_data(QTensorOps.q_argmax(_int8(dev, a), 1)).tolist() == [[1], [2]]
    assert IntOps.int_into_data(QTensorOps.q_argmin(_int8(dev, b), 1)).tolist() == [[2], [1]]
    # expand.rs:7-100 (Tolerance::absolute(1e-1); the single-value broadcast is exact)
    for src, shape in (([1.0, 2.0, 3.0], (3, 3)), ([4.0, 7.0, 2.0, 3.0], (2, 4)), ([[1.0, 2.0], [3.0, 4.0]], (3, 2, 2)),
                       ([[1.0, 2.0, 3.0, 4.0]], (2, 3, 4))):
        got = _deq(QTensorOps.q_expand(_int8(dev, src), shape))
        assert got.shape == shape and np.abs(got - np.broadcast_to(np.float32(src), shape)).max() <= 1e-1
    assert _deq(QTensorOps.q_expand(_int8(dev, [1.0]), (2, 3))).tolist() == [[1.0, 1.0, 1.0], [1.0, 1.0, 1.0]]
    with pytest.raises(ba.BurnqError) as e:                      # should_fail_expand_incompatible_shapes
        QTensorOps.q_expand(_int8(dev, [1.0, 2.0, 3.0]), (2, 2))
    assert e.value.status == ba._lib.ERR_SHAPE
    # select.rs:8-70 (Tolerance::rel_abs(2e-2, 1e-2))
    for src, dim, idx, want in (
            ([0.0, 1.0, 2.0, 3.0], 0, [1, 1, 0, 1, 2], [1.0, 1.0, 0.0, 1.0, 2.0]),
            ([[0.0, 1.0, 2.0], [3.0, 4.0, 5.0]], 0, [1, 0], [[3.0, 4.0, 5.0], [0.0, 1.0, 2.0]]),
            ([[0.0, 1.0, 2.0], [3.0, 4.0, 5.0]], 0, [1, 0, 1, 1], [[3.0, 4.0, 5.0], [0.0, 1.0, 2.0], [3.0, 4.0, 5.0], [3.0, 4.0, 5.0]]),
            ([[0.0, 1.0, 2.0], [3.0, 4.0, 5.0]], 1, [1, 1, 0, 1, 2], [[1.0, 1.0, 0.0, 1.0, 2.0], [4.0, 4.0, 3.0, 4.0, 5.0]])):
        got = _deq(QTensorOps.q_select(_int8(dev, src), dim, IntOps.int_from_data(np.int64(idx), dev)))
        want = np.float32(want)
        assert got.shape == want.shape and (np.abs(got - want) <= 1e-2 + 2e-2 * np.abs(want)).all()
    # gather_scatter.rs:8-100 (Tolerance::absolute(1e-1))
    m23 = [[0.0, 1.0, 2.0], [3.0, 4.0, 5.0]]
    for src, dim, idx, want in (
            ([0.0, 1.0, 2.0], 0, [1, 1, 0, 1, 2], [1.0, 1.0, 0.0, 1.0, 2.0]),
            (m23, 0, [[0, 1, 0], [1, 0, 1]], [[0.0, 4.0, 2.0], [3.0, 1.0, 5.0]]),
            (m23, 1, [[2, 1, 0, 0], [2, 0, 1, 2]], [[2.0, 1.0, 0.0, 0.0], [5.0, 3.0, 4.0, 5.0]]),
            ([[[0.0, 1.0, 2.0], [3.0, 4.0, 5.0]], [[6.0, 7.0, 8.0], [9.0, 10.0, 11.0]]], 1,
             [[[1, 0, 0], [0, 1, 0]], [[0, 0, 1], [0, 1, 1]]],
             [[[3.0, 1.0, 2.0], [0.0, 4.0, 2.0]], [[6.0, 7.0, 11.0], [6.0, 10.0, 11.0]]]),
            (m23, 1, [[1], [2]], [[1.0], [5.0]])):
        got = _deq(QTensorOps.q_gather(dim, _int8(dev, src), IntOps.int_from_data(np.int64(idx), dev)))
        want = np.float32(want)
        assert got.shape == want.shape and np.abs(got - want).max() <= 1e-1


# ------------------------------------------------------------------ Calibration::AbsMean

def test_abs_mean_calibration_reference_cases(dev, kats, approx):
    """crates/burn-backend-tests/tests/tensor/float/quantization/calibration.rs:62-125, with its
    tolerance (Tolerance::default(): relative 0.005, absolute 1e-5), and the ternary weights the
    Quantizer then makes of them."""
    k = kats["abs_mean_calibration_per_tensor"]
    scheme = QuantScheme(value=QuantValue.Q2S, store=QuantStore.Native)
    g = FloatOps.float_into_data(QTensorOps.compute_range_abs_mean(FloatOps.float_from_data(np.float32(k["x"]), dev), scheme))
    assert g.shape == (1,)
    approx(g, k["expected_max"])
    approx(-g, k["expected_min"])
    tq = QTensorOps.quantize_abs_mean(FloatOps.float_from_data(np.float32(k["x"]), dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    assert q.tolist() == [-1, -1, 0, 1]
    approx(s.reshape(-1), k["expected_max"])
    k = kats["abs_mean_calibration_per_block"]
    scheme = QuantScheme(value=QuantValue.Q2S, store=QuantStore.Native).per_block(k["block"])
    g = FloatOps.float_into_data(QTensorOps.compute_range_abs_mean(FloatOps.float_from_data(np.float32(k["x"]), dev), scheme))
    assert g.shape == (2, 1)
    approx(g, k["expected_max"])
    # a two-level scheme is refused, as the reference asserts
    two = QuantScheme().per_block((4,), ScaleDtype.F16).per_tensor()
    with pytest.raises(ba.BurnqError, match="two-level"):
        QTensorOps.compute_range_abs_mean(FloatOps.float_from_data(np.float32(k["x"]), dev), two)


@pytest.mark.parametrize("value", [QuantValue.Q2S, QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("shape,block", [((4096,), None), ((257, 96), None), ((64, 128), (32,)), ((48, 64), (16, 16)),
                                          ((6, 10, 32), (2, 5, 8)), ((1000, 1024), None), ((512, 512), (128,))])
def test_abs_mean_calibration_against_the_oracle(dev, value, shape, block):
    """gamma within 4 ulp-scale relative error (2e-6) of the oracle's binary64 mean -- the reference
    compares within 0.5 % --, and the quantized tensor bit for bit what the oracle's quantize makes of
    the scales the device derived (scale = 2 gamma / (b - a), one IEEE operation per step)."""
    x = awkward(shape, 17 + len(shape))
    store = QuantStore.Native if value == QuantValue.Q2S or shape[-1] % 8 else QuantStore.PackedU32
    scheme = QuantScheme(value=value, store=store) if block is None else QuantScheme(value=value, store=store).per_block(block)
    tx = FloatOps.float_from_data(x, dev)
    g = FloatOps.float_into_data(QTensorOps.compute_range_abs_mean(tx, scheme))
    lo_ref, g_ref = co.compute_range_abs_mean(x, oscheme(scheme))
    assert g.shape == g_ref.shape
    assert np.all(np.abs(g.astype(np.float64) - g_ref) <= 2e-6 * np.abs(g_ref)), float(np.abs(g - g_ref).max())
    tq = QTensorOps.quantize_abs_mean(tx, scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    assert s.reshape(-1).tobytes() == co.compute_q_params(-g, g, VAL[value][0]).reshape(-1).tobytes()
    q_ref = co.quantize(x, oscheme(scheme), s.reshape(g.shape))
    assert (q == q_ref).all()
    if value == QuantValue.Q2S:
        assert set(np.unique(q).tolist()) == {-1, 0, 1}
    # deterministic: the same bits on a second run
    g2 = FloatOps.float_into_data(QTensorOps.compute_range_abs_mean(tx, scheme))
    assert g2.tobytes() == g.tobytes()


# ------------------------------------------------------------------ host threads

def test_small_transfers_through_the_pinned_slots(dev):
    """Host buffers of at most 64 KiB travel through a few pinned slots that are refilled as soon as a copy
    kernel has reported: more uploads in a row than there are slots, sizes that are no multiple of 16 bytes,
    both sides of the 64 KiB limit, each read back, in the order made and in reverse."""
    rng = np.random.default_rng(77)
    sizes = [1, 3, 4, 5, 1023, 4096, 16383, 16384, 16385, 1, 16384, 7, 16384 + 4, 2, 16384, 16384, 9]
    hosts = [rng.standard_normal(n).astype(np.float32) for n in sizes]
    tensors = [FloatOps.float_from_data(h, dev) for h in hosts]      # 17 uploads, nothing waited for in between
    for h, t in zip(hosts, tensors):
        assert FloatOps.float_into_data(t).tobytes() == h.tobytes()
    for h, t in reversed(list(zip(hosts, tensors))):
        assert FloatOps.float_into_data(t).tobytes() == h.tobytes()
    # 2-byte elements: 6 and 65534 bytes
    for n in (3, 32767, 32768, 32769):
        bits = rng.integers(0, 1 << 16, n).astype(np.uint16)
        bits[(bits & 0x7F80) == 0x7F80] = 0x3F80                      # no NaN / Inf patterns
        t = FloatOps.float_from_data(bits, dev, dtype=ba.BF16)
        assert FloatOps.float_into_data(t).tobytes() == bits.tobytes()
    dev.sync()
    dev.sync()                                                        # a wait with nothing queued returns as well


def test_host_threads_share_one_device(dev):
    """crates/burn-backend-tests/tests/tensor/multi_threads.rs: tensors used from several host
    threads at once. Eight threads on one device, each running quantize_dynamic, dequantize and
    q_matmul on its own inputs, repeatedly and concurrently; every result must equal, bit for bit,
    what the same call gave on a single thread."""
    import threading
    rng = np.random.default_rng(404)
    jobs = []
    for t in range(8):
        x = rng.standard_normal((64 + 8 * t, 256)).astype(np.float32)
        w = (rng.standard_normal((256, 512)) * 0.02).astype(np.float32)
        a = rng.standard_normal((1 + 5 * t, 256)).astype(np.float32)   # decode, split and tiled kernels
        scheme = (QuantScheme().per_block((32,)), QuantScheme(value=QuantValue.Q4S).per_block((32,)), QuantScheme(store=QuantStore.Native))[t % 3]
        jobs.append((x, w, a, scheme))

    def run(job):
        x, w, a, scheme = job
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(x, dev), scheme)
        blob = QTensorOps.q_into_data(tq).bytes.tobytes()
        d = FloatOps.float_into_data(QTensorOps.dequantize(tq)).tobytes()
        tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
        y = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(a, dev), tw)).tobytes()
        return blob, d, y

    expected = [run(j) for j in jobs]
    for j, e in zip(jobs, expected):   # and the oracle agrees with the single-thread run
        q_ref, s_ref = co.quantize_dynamic(j[0], oscheme(j[3]))
        assert e[0] == co.encode(q_ref, oscheme(j[3]), s_ref).tobytes()
    failures, barrier = [], threading.Barrier(8)

    def worker(i):
        try:
            barrier.wait(timeout=60)
            for rep in range(12):
                got = run(jobs[i])
                if got != expected[i]:
                    failures.append((i, rep, [g == e for g, e in zip(got, expected[i])]))
        except Exception as exc:   # noqa: BLE001
            failures.append((i, repr(exc)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=110)
    assert not any(th.is_alive() for th in threads), "a worker thread did not finish"
    assert not failures, failures[:3]


# ------------------------------------------------------------------ the configs at full size

def test_config1_per_tensor_q8s_native_4096(dev):
    x = np.random.default_rng(0xC1).standard_normal((4096, 4096)).astype(np.float32)
    check_quantize_dynamic(dev, x, QuantScheme(store=QuantStore.Native), mt=True)


def test_config2_block32_q8s_packed_8192(dev):
    rng = np.random.default_rng(0xC2)
    x = rng.standard_normal((8192, 8192)).astype(np.float32)
    x[rng.random(x.shape) < 0.01] *= 50
    scheme = QuantScheme().per_block((32,))
    tq, q_ref, s_ref, d_ref = check_quantize_dynamic(dev, x, scheme, mt=True)
    # size-independent properties: error bound and idempotence of re-quantizing the round trip
    s_full = np.repeat(s_ref.reshape(8192, 256), 32, axis=1)
    assert (np.abs(d_ref.astype(np.float64) - x) <= 0.5 * s_full + 1e-6 * np.abs(x)).all()
    scales = FloatOps.float_from_data(s_ref, dev)
    again = QTensorOps.quantize(QTensorOps.dequantize(tq), scheme, scales)
    assert QTensorOps.q_into_data(again).bytes.tobytes() == QTensorOps.q_into_data(tq).bytes.tobytes()


def test_config3_q4s_block32_dequantize_14336x4096(dev):
    rng = np.random.default_rng(0xC3)
    w = (rng.standard_normal((14336, 4096)) * 0.02).astype(np.float32)
    scheme = QuantScheme(value=QuantValue.Q4S).per_block((32,))
    q_ref, s_ref = co.quantize_dynamic(w, oscheme(scheme), mt=True)   # pre-quantized on the host
    blob = co.encode(q_ref, oscheme(scheme), s_ref)
    t = QTensorOps.q_from_data(TensorData(blob, w.shape, scheme), dev)
    d = FloatOps.float_into_data(QTensorOps.dequantize(t))
    assert d.tobytes() == co.dequantize(q_ref, oscheme(scheme), s_ref, mt=True).tobytes()
    # and the GPU quantizes the same weights to the same words
    _, gblob = gpu_quantize_dynamic(dev, w, scheme)
    assert gblob.bytes.tobytes() == blob.tobytes()


def matmul_check(out, ref64, max_outside=0):
    """max |y - y'| / max |y'| <= 1e-2, and burn's permissive elementwise rule for every element
    (all but `max_outside`, a literal count the caller justifies)."""
    rel = np.abs(out - ref64).max() / np.abs(ref64).max()
    assert rel <= 1e-2, rel
    ok = burn_approx_eq(out, ref64, 1e-2, 1e-2)
    assert (~ok).sum() <= max_outside, f"{(~ok).sum()} of {ok.size} outside burn's permissive tolerance"
    return rel


@pytest.fixture(scope="module")
def weights_q8(dev):
    rng = np.random.default_rng(0xC4)
    w = (rng.standard_normal((4096, 14336)) * 0.02).astype(np.float32)
    scheme = QuantScheme().per_block((32,))
    q_ref, s_ref = co.quantize_dynamic(w, oscheme(scheme), mt=True)
    t = QTensorOps.q_from_data(TensorData(co.encode(q_ref, oscheme(scheme), s_ref), w.shape, scheme), dev)
    wd = co.dequantize(q_ref, oscheme(scheme), s_ref, mt=True).astype(np.float64)
    return t, wd


@pytest.mark.parametrize("m", [1, 4, 16])
def test_config4_decode_qgemv(dev, weights_q8, m):
    t, wd = weights_q8
    x = np.random.default_rng(100 + m).standard_normal((m, 4096)).astype(np.float32)
    out = QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), t)
    assert out.shape == (m, 14336) and out.dtype == ba.F32
    rel = matmul_check(FloatOps.float_into_data(out), x.astype(np.float64) @ wd)
    assert rel < 1e-4   # f32 accumulation of f32 operands: far inside the bound
    # reproducible: split-K partials are reduced in a fixed order
    out2 = QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), t)
    assert FloatOps.float_into_data(out2).tobytes() == FloatOps.float_into_data(out).tobytes()


# C5 against the f32 reference, burn's elementwise rule |y - y'| < max(1e-2 * max(|y|, |y'|), 1e-2):
# the weights reach the MFMA as bf16(s * q), a relative rounding error of at most 2^-8 (rms about
# 1.6e-3) per weight. An output sums 4096 products of N(0,1) activations and N(0, 0.02^2) weights
# (sum of squares 1.64), so its error is close to normal with sigma 1.28 * 1.6e-3 = 2.1e-3 (measured
# rms 2.126e-3, max 1.25e-2). The rule's 1e-2 floor is 4.70 sigma away: 29 360 128 outputs x
# P(|z| > 4.70) = 2.6e-6 predicts 76 outputs outside it; 52 are measured (the inputs are seeded and
# the kernel's summation order is fixed, so the count is reproducible). More than 100 would mean
# an error that the weight rounding does not explain; the sampled rows (688 128 outputs, 1
# measured) may hold 5.
C5_MAX_OUTSIDE = 100
C5_MAX_OUTSIDE_SAMPLE = 5


def test_config5_prefill_qgemm_bf16_q4s(dev):
    rng = np.random.default_rng(0xC5)
    w = (rng.standard_normal((4096, 14336)) * 0.02).astype(np.float32)
    scheme = QuantScheme(value=QuantValue.Q4S).per_block((32,))
    q_ref, s_ref = co.quantize_dynamic(w, oscheme(scheme), mt=True)
    t = QTensorOps.q_from_data(TensorData(co.encode(q_ref, oscheme(scheme), s_ref), w.shape, scheme), dev)
    a_bits = ba.bf16_bits_from_f32(rng.standard_normal((2048, 4096)).astype(np.float32))
    a = ba.f32_from_bf16_bits(a_bits)              # the bf16 activations, widened exactly
    out = QTensorOps.q_matmul(FloatOps.float_from_data(a_bits, dev, ba.BF16), t, out_dtype=ba.F32)
    assert out.shape == (2048, 14336) and out.dtype == ba.F32
    got = FloatOps.float_into_data(out)
    wd = co.dequantize(q_ref, oscheme(scheme), s_ref, mt=True)
    # float64 yardstick on a sample of rows, f32 sgemm on everything (see C5_MAX_OUTSIDE above)
    rows = rng.choice(2048, 48, replace=False)
    ref32 = (a @ wd).astype(np.float64)
    err = np.abs(got - ref32)
    outside = int((~burn_approx_eq(got, ref32, 1e-2, 1e-2)).sum())
    print(f"C5 elementwise: max |err| {err.max():.3e}, rms {np.sqrt((err ** 2).mean()):.3e}, "
          f"outside burn's permissive rule: {outside} of {got.size}")
    matmul_check(got[rows], a[rows].astype(np.float64) @ wd.astype(np.float64), max_outside=C5_MAX_OUTSIDE_SAMPLE)
    matmul_check(got, ref32, max_outside=C5_MAX_OUTSIDE)
    # against the product with the weights rounded the way the kernel rounds them, the kernel is
    # exact to f32 accumulation error
    wb = ba.f32_from_bf16_bits(ba.bf16_bits_from_f32(wd)).reshape(wd.shape).astype(np.float64)
    assert np.abs(got[rows] - a[rows].astype(np.float64) @ wb).max() <= 1e-4
    # linearity in the activations (exact scaling by a power of two). 128 rows are few tiles, so
    # K is split over several workgroups there: same products, another order of the f32 sums.
    out1 = FloatOps.float_into_data(
        QTensorOps.q_matmul(FloatOps.float_from_data(ba.bf16_bits_from_f32(a[:128]), dev, ba.BF16), t, out_dtype=ba.F32))
    out2 = FloatOps.float_into_data(
        QTensorOps.q_matmul(FloatOps.float_from_data(ba.bf16_bits_from_f32(a[:128] * 4), dev, ba.BF16), t, out_dtype=ba.F32))
    assert (out2 == out1 * 4).all()
    assert np.abs(out1 - got[:128]).max() <= 1e-5 * np.abs(got[:128]).max()


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,), (64,)])
@pytest.mark.parametrize("m,k,n", [(1, 96, 128), (3, 100, 192), (16, 64, 64), (17, 130, 320),
                                   (200, 72, 448), (130, 257, 136)])
def test_q_matmul_shapes(dev, value, block, m, k, n):
    if block and n % block[0]:
        pytest.skip("block does not divide N")
    rng = np.random.default_rng(m * 1000 + k + n)
    w = rng.standard_normal((k, n)).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    scheme = QuantScheme(value=value, block=block)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    ref = no.q_matmul_f64(x, q, s, list(block) if block else None)
    out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    assert np.abs(out - ref).max() <= 1e-2 * np.abs(ref).max()
    if m <= 16:   # f32 activations stay f32 on the decode path
        assert burn_approx_eq(out, ref, 1e-2, 1e-2).all()
    # bf16 activations through the MFMA path, f32 and bf16 out
    xb = ba.bf16_bits_from_f32(x)
    refb = no.q_matmul_f64(ba.f32_from_bf16_bits(xb), q, s, list(block) if block else None)
    outb = FloatOps.float_into_data(
        QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq, out_dtype=ba.F32))
    assert np.abs(outb - refb).max() <= 1e-2 * np.abs(refb).max() + 1e-2
    outh = QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq)
    assert outh.dtype == ba.BF16
    assert np.abs(ba.f32_from_bf16_bits(FloatOps.float_into_data(outh)) - refb).max() <= 2e-2 * np.abs(refb).max() + 1e-2


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,), (64,), (128,)])
@pytest.mark.parametrize("m,k,n", [(2, 64, 96), (7, 100, 160), (9, 2048, 1056), (12, 1000, 2080),
                                   (16, 4096, 512), (25, 264, 352), (32, 1536, 288),
                                   (3, 96, 128), (5, 1056, 640), (13, 544, 1152), (1, 256, 256),
                                   (24, 1056, 640), (32, 2048, 512), (17, 96, 128)])
def test_q_matmul_small_batches(dev, value, block, m, k, n):
    """The matrix-core kernels for 2 <= M <= 32: K slices with tails, N tiles with tails, both
    activation dtypes. f32 activations with M <= 16 keep at least 16 significant bits per product
    (FP32 MFMA, or bf16 MFMA over activations split into two bf16 terms)."""
    if block and n % block[0]:
        pytest.skip("block does not divide N")
    rng = np.random.default_rng(m * 7919 + k + n)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    scheme = QuantScheme(value=value, block=block)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    ref = no.q_matmul_f64(x, q, s, list(block) if block else None)
    out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    # whole 128-column groups and 32-row steps take the split-activation kernel up to M = 32
    split = n % 128 == 0 and k % 32 == 0
    rel = np.abs(out - ref).max() / np.abs(ref).max()
    assert rel <= (2e-5 if (m <= 16 or split) else 1e-2), rel
    xb = ba.bf16_bits_from_f32(x)
    refb = no.q_matmul_f64(ba.f32_from_bf16_bits(xb), q, s, list(block) if block else None)
    outb = FloatOps.float_into_data(
        QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq, out_dtype=ba.F32))
    # bf16 activations take the split-activation kernel as well: exact weights, 16 significant
    # bits of activation x scale
    assert np.abs(outb - refb).max() <= (2e-5 if split else 1e-2) * np.abs(refb).max()
    # reproducible run to run (fixed-order split-K reduction)
    again = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    assert again.tobytes() == out.tobytes()


def test_small_batch_kernels_random_shapes(dev):
    """200 seeded products with 1 <= M <= 32 over weights in whole 128-column groups and 32-row
    steps (any number of either, so the last tile and the last K slice are partly empty more often
    than not): the decode kernel and every form of the split-activation kernel -- row-packed,
    per-tensor, one scale per 32, 64 or 128 columns, one or two tiles of rows, both value widths,
    both activation dtypes, activations from 1e-3 to 1e3. Each within 2e-5 of the float64 product
    of the dequantized weights (the kernels keep 16 significant bits per product or better)."""
    rng = np.random.default_rng(4242)
    for case in range(200):
        value = [QuantValue.Q8S, QuantValue.Q4S, QuantValue.Q8F, QuantValue.Q4F][rng.integers(4)]
        block = [None, (32,), (64,), (128,)][rng.integers(4)]
        n, k, m = 128 * int(rng.integers(1, 30)), 32 * int(rng.integers(1, 70)), int(rng.integers(1, 33))
        w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
        if rng.integers(4) == 0:
            w[rng.random(w.shape) < 0.5] = 0.0
        tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme(value=value, block=block))
        wd = FloatOps.float_into_data(QTensorOps.dequantize(tw)).astype(np.float64)
        xh = (rng.standard_normal((m, k)) * 10.0 ** rng.integers(-3, 4)).astype(np.float32)
        bf16 = bool(rng.integers(2))
        if bf16:
            bits = ba.bf16_bits_from_f32(xh)
            xh = ba.f32_from_bf16_bits(bits).reshape(m, k)
            lhs = FloatOps.float_from_data(bits, dev, ba.BF16)
        else:
            lhs = FloatOps.float_from_data(xh, dev)
        ref = xh.astype(np.float64) @ wd
        out = FloatOps.float_into_data(QTensorOps.q_matmul(lhs, tw, out_dtype=ba.F32))
        rel = np.abs(out - ref).max() / max(np.abs(ref).max(), 1e-30)
        assert rel <= 2e-5, f"case {case}: m={m} k={k} n={n} {value.name} block={block} bf16={bf16}: {rel:.3e}"


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,), (64,)])
@pytest.mark.parametrize("m,k,n", [(1, 4096, 1024), (1, 100, 64), (2, 96, 256), (4, 1056, 640), (8, 96, 128),
                                   (8, 4096, 512), (16, 2080, 1152), (24, 96, 128), (64, 1024, 512),
                                   (130, 264, 256)])
def test_q_matmul_infinite_and_nan_activations(dev, value, block, m, k, n):
    """The reference multiplies by the dequantized weights: an infinite activation gives +-inf in
    its row (NaN where the weight is zero or where both signs meet), a NaN activation a NaN row,
    and every other row stays finite. The kernels' shortcuts (offset weight fields, activations
    split into two bf16 terms, zero-filled padding) must not turn that into something else."""
    if block and n % block[0]:
        pytest.skip("block does not divide N")
    rng = np.random.default_rng(m * 31 + k + n)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    w[rng.random((k, n)) < 0.05] = 0.0            # zero weights: inf * 0 = NaN
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[0, 5 % k] = np.inf                           # (row 0 of a slice: the row that padding re-reads)
    if m >= 2:
        x[m - 1, k - 1] = -np.inf
    if m >= 4:
        x[2, k // 2] = np.inf
        x[2, k // 3] = -np.inf                     # both signs in one row: NaN everywhere
        x[3, k // 5] = np.nan
    scheme = QuantScheme(value=value, block=block)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    with np.errstate(invalid="ignore", over="ignore"):
        ref = no.q_matmul_f64(x, q, s, list(block) if block else None)

    def same(out, ref):
        assert (np.isnan(out) == np.isnan(ref)).all(), (np.isnan(out).sum(), np.isnan(ref).sum())
        inf = np.isinf(ref)
        assert (np.isinf(out) == inf).all()
        assert (np.sign(out[inf]) == np.sign(ref[inf])).all()
        fin = np.isfinite(ref)
        assert fin.any() or m <= 2
        if fin.any():
            assert np.abs(out[fin] - ref[fin]).max() <= 1e-2 * np.abs(ref[fin]).max() + 1e-2

    same(FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq)), ref)
    xb = ba.bf16_bits_from_f32(x)
    with np.errstate(invalid="ignore", over="ignore"):
        refb = no.q_matmul_f64(ba.f32_from_bf16_bits(xb), q, s, list(block) if block else None)
    same(FloatOps.float_into_data(
        QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq, out_dtype=ba.F32)), refb)


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,)])
@pytest.mark.parametrize("m,k,n", [(64, 1024, 512), (200, 2112, 768), (40, 4096, 1024), (129, 520, 256)])
def test_q_matmul_split_k_tiles(dev, value, block, m, k, n):
    """Few output tiles: the tiled kernel splits K over several workgroups per tile and the
    partial products are added in a fixed order (K tails, odd stage counts, both tile heights)."""
    rng = np.random.default_rng(m * 31 + k + n)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    scheme = QuantScheme(value=value, block=block)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    xb = ba.bf16_bits_from_f32(x)
    refb = no.q_matmul_f64(ba.f32_from_bf16_bits(xb), q, s, list(block) if block else None)
    outb = FloatOps.float_into_data(
        QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq, out_dtype=ba.F32))
    assert np.abs(outb - refb).max() <= 1e-2 * np.abs(refb).max()
    outh = QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq)
    assert outh.dtype == ba.BF16
    assert np.abs(ba.f32_from_bf16_bits(FloatOps.float_into_data(outh)) - refb).max() <= 2e-2 * np.abs(refb).max()
    # f32 activations are rounded to bf16 on this path
    out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    ref = no.q_matmul_f64(x, q, s, list(block) if block else None)
    assert np.abs(out - ref).max() <= 1e-2 * np.abs(ref).max()
    again = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    assert again.tobytes() == out.tobytes()


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,), (64,)])
@pytest.mark.parametrize("m,k,n", [(1, 4096, 1024), (2, 1000, 448), (1, 130, 64), (2, 64, 4096)])
def test_bf16_decode_is_the_f32_decode_on_widened_activations(dev, value, block, m, k, n):
    """One or two rows of bf16 activations take the kernel f32 activations take and are widened
    exactly: the same bits as for the f32 activations of the same values. The decode kernel is
    within f32 rounding of the float64 product; two rows over 4-bit weights whose scales are per
    tensor or per 32 columns take the split-activation kernel where its layout applies (16
    significant bits per product)."""
    rng = np.random.default_rng(m * 17 + k + n)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    xb = ba.bf16_bits_from_f32(rng.standard_normal((m, k)).astype(np.float32))
    x = ba.f32_from_bf16_bits(xb).reshape(m, k)
    scheme = QuantScheme(value=value, block=block)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    ref = no.q_matmul_f64(x, q, s, list(block) if block else None)
    out_b = FloatOps.float_into_data(
        QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq, out_dtype=ba.F32))
    out_f = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    assert out_b.tobytes() == out_f.tobytes()
    split = m == 2 and value == QuantValue.Q4S and block in (None, (32,)) and n % 128 == 0 and k % 32 == 0
    assert np.abs(out_b - ref).max() <= (2e-5 if split else 2e-6) * np.abs(ref).max()
    # default output dtype follows the activations
    out_h = QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq)
    assert out_h.dtype == ba.BF16
    assert FloatOps.float_into_data(out_h).tobytes() == ba.bf16_bits_from_f32(out_b).tobytes()


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,)])
@pytest.mark.parametrize("m,k,n", [(300, 520, 800), (512, 1024, 1024), (130, 392, 2048)])
def test_q_gemm_exact_to_bf16_weights(dev, value, block, m, k, n):
    """The tiled kernel feeds the MFMA with bf16(s * q). Against the float64 product with the
    weights rounded exactly that way nothing but the order of the f32 sums is left, so a wrong
    field, scale or row anywhere in a tile shows at 1e-5 instead of hiding under the 1e-2 bar
    (both tile heights, K tails, per-tensor and block scales)."""
    rng = np.random.default_rng(m * 7 + k + n)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    xb = ba.bf16_bits_from_f32(rng.standard_normal((m, k)).astype(np.float32))
    x = ba.f32_from_bf16_bits(xb).reshape(m, k)
    scheme = QuantScheme(value=value, block=block)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    wd = no.dequantize(q, s, list(block) if block else None)
    wb = ba.f32_from_bf16_bits(ba.bf16_bits_from_f32(wd)).reshape(k, n).astype(np.float64)
    ref = x.astype(np.float64) @ wb
    out = FloatOps.float_into_data(
        QTensorOps.q_matmul(FloatOps.float_from_data(xb, dev, ba.BF16), tq, out_dtype=ba.F32))
    assert np.abs(out - ref).max() <= 1e-5 * np.abs(ref).max()
    # a bf16 output is the same f32 sum (plus the bias of a linear layer) rounded once; the tiled
    # kernel stores it as column pairs exchanged between neighbouring lanes
    from burn_amd import ModuleOps
    xt = FloatOps.float_from_data(xb, dev, ba.BF16)
    outh = QTensorOps.q_matmul(xt, tq)
    assert outh.dtype == ba.BF16
    assert FloatOps.float_into_data(outh).tobytes() == ba.bf16_bits_from_f32(out).tobytes()
    bias = FloatOps.float_from_data(rng.standard_normal(n).astype(np.float32), dev)
    lin32 = FloatOps.float_into_data(ModuleOps.linear(xt, tq, bias, out_dtype=ba.F32))
    lin16 = FloatOps.float_into_data(ModuleOps.linear(xt, tq, bias))
    assert lin16.tobytes() == ba.bf16_bits_from_f32(lin32).tobytes()


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,)])
@pytest.mark.parametrize("m,k,n", [(1, 256, 256), (3, 96, 160), (16, 1056, 640), (64, 1024, 512),
                                   (200, 264, 352), (300, 512, 256)])
def test_q_linear_bias_epilogue(dev, value, block, m, k, n):
    """linear with a quantized weight: every q_matmul kernel (decode, split activations, small
    batches, tiled with and without split K) adds the bias where it writes the output. For an f32
    output that is bit for bit the unfused result (the f32 sum, then one addition)."""
    from burn_amd import ModuleOps
    if block and n % block[0]:
        pytest.skip("block does not divide N")
    rng = np.random.default_rng(m * 131 + k + n)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    scheme = QuantScheme(value=value, block=block)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    tx, tb = FloatOps.float_from_data(x, dev), FloatOps.float_from_data(b, dev)
    plain = FloatOps.float_into_data(QTensorOps.q_matmul(tx, tq))
    y = ModuleOps.linear(tx, tq, tb)
    assert y.shape == (m, n) and y.dtype == ba.F32
    got = FloatOps.float_into_data(y)
    assert got.tobytes() == (plain + b[None, :]).astype(np.float32).tobytes()
    ref = no.q_linear_f64(x, q, s, list(block) if block else None, b)
    assert np.abs(got - ref).max() <= 1e-2 * np.abs(ref).max()
    # no bias: q_matmul itself
    assert FloatOps.float_into_data(ModuleOps.linear(tx, tq)).tobytes() == plain.tobytes()
    # bf16 activations, bf16 bias, bf16 output: one rounding of (f32 sum + bias)
    xb, bb = ba.bf16_bits_from_f32(x), ba.bf16_bits_from_f32(b)
    txb, tbb = FloatOps.float_from_data(xb, dev, ba.BF16), FloatOps.float_from_data(bb, dev, ba.BF16)
    plain_b = FloatOps.float_into_data(QTensorOps.q_matmul(txb, tq, out_dtype=ba.F32))
    yb = ModuleOps.linear(txb, tq, tbb)
    assert yb.dtype == ba.BF16
    want = ba.bf16_bits_from_f32((plain_b + ba.f32_from_bf16_bits(bb)[None, :]).astype(np.float32))
    assert FloatOps.float_into_data(yb).tobytes() == want.tobytes()


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("m,k,n,block", [(1, 4096, 14336, 32), (2, 1024, 2048, 32), (4, 4096, 512, 32), (1, 4096, 256, 32),
                                          (3, 2048, 1152, 0), (8, 512, 1024, 64), (16, 4096, 14336, 32), (16, 2048, 640, 128),
                                          (32, 1024, 1536, 32), (5, 8192, 128, 32), (1, 96, 4096, 32), (7, 4096, 2048, 0)])
def test_single_launch_split_k_is_the_two_launch_sum(dev, value, m, k, n, block):
    """The handle level runs the decode kernel of one or two rows as one launch (the last workgroup of a
    column strip adds up the K slices); the kernel level, given a plain workspace, runs the same
    kernel followed by the reduction kernel, as every larger batch does at both levels. Same partial
    sums, same summation order: the outputs are
    equal bit for bit, f32 and bf16, with and without a bias, for few and for many K slices, three
    times in a row (the ticket counters must come back to zero)."""
    import ctypes as C
    from burn_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(m * 131 + n)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    scheme = QuantScheme(value=value) if block == 0 else QuantScheme(value=value).per_block((block,))
    tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    cval = VAL[value][0]
    bias_h = rng.standard_normal(n).astype(np.float32)
    bias = FloatOps.float_from_data(bias_h, dev)
    need = L.bqk_q_matmul_workspace(m, k, n, ba.F32, cval)
    ws = FloatOps.float_empty((max(need, 4) // 4 + 64,), dev)
    for rep in range(3):
        x_h = rng.standard_normal((m, k)).astype(np.float32)
        x = FloatOps.float_from_data(x_h, dev)
        for out_dtype in (ba.F32, ba.BF16):
            for b in (None, bias):
                one = FloatOps.float_into_data(ModuleOps.linear(x, tw, b, out_dtype=out_dtype))
                out = FloatOps.float_empty((m, n), dev, out_dtype)
                _lib.check(L.bqk_q_linear(x.data_ptr, ba.F32, m, k, n, tw.data_ptr, tw.scales_ptr, block, cval,
                                          _lib.STORE_PACKED_U32, b.data_ptr if b is not None else None, out_dtype,
                                          out.data_ptr, ws.data_ptr, need, dev.stream))
                two = FloatOps.float_into_data(out)
                assert one.tobytes() == two.tobytes(), f"rep {rep}, out dtype {out_dtype}, bias {b is not None}"
    # and the product is right
    values, scales = QTensorOps.q_into_data(tw).split()
    q = no.unpack_u32(values.view(np.uint32), w.shape, VAL[value][1])
    got = FloatOps.float_into_data(QTensorOps.q_matmul(x, tw))
    matmul_check(got, no.q_matmul_f64(x_h, q, scales, [block] if block else None))


def test_q_linear_folds_leading_dims(dev):
    from burn_amd import ModuleOps
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((128, 256)) * 0.05).astype(np.float32)
    x = rng.standard_normal((2, 5, 128)).astype(np.float32)
    b = rng.standard_normal(256).astype(np.float32)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme().per_block((32,)))
    y = ModuleOps.linear(FloatOps.float_from_data(x, dev), tq, FloatOps.float_from_data(b, dev))
    assert y.shape == (2, 5, 256)
    flat = ModuleOps.linear(FloatOps.float_from_data(x.reshape(10, 128), dev), tq, FloatOps.float_from_data(b, dev))
    assert FloatOps.float_into_data(y).reshape(10, 256).tobytes() == FloatOps.float_into_data(flat).tobytes()
    y1 = ModuleOps.linear(FloatOps.float_from_data(x[0, 0], dev), tq, FloatOps.float_from_data(b, dev))
    assert y1.shape == (256,)
    # one row takes the decode kernel, ten rows the matrix-core kernel: same value, other rounding
    row = FloatOps.float_into_data(y)[0, 0]
    assert np.abs(FloatOps.float_into_data(y1) - row).max() <= 2e-5 * np.abs(row).max()
    with pytest.raises(ba.BurnqError):
        ModuleOps.linear(FloatOps.float_from_data(x[..., :64], dev), tq)
    with pytest.raises(ba.BurnqError):
        ModuleOps.linear(FloatOps.float_from_data(x, dev), tq, FloatOps.float_from_data(b[:128], dev))


@pytest.mark.parametrize("value", [QuantValue.Q8S, QuantValue.Q4S])
@pytest.mark.parametrize("block", [None, (32,)])
def test_q_matmul_propagate_requantizes(dev, value, block):
    """QuantPropagation::Propagate: the product, quantized dynamically with the weight's scheme
    (burn-ndarray/src/ops/qtensor.rs:262-265) -- exactly quantize_dynamic of q_matmul's result."""
    rng = np.random.default_rng(12)
    x = rng.standard_normal((6, 96)).astype(np.float32)
    w = (rng.standard_normal((96, 128)) * 0.1).astype(np.float32)
    scheme = QuantScheme(value=value, block=block)
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    tx = FloatOps.float_from_data(x, dev)
    out = QTensorOps.q_matmul_propagate(tx, tq)
    assert out.is_quantized and out.shape == (6, 128) and out.scheme.value == value
    two_steps = QTensorOps.quantize_dynamic(QTensorOps.q_matmul(tx, tq), scheme)
    assert QTensorOps.q_into_data(out).bytes.tobytes() == QTensorOps.q_into_data(two_steps).bytes.tobytes()
    # and it is the oracle's quantization of that product
    prod = FloatOps.float_into_data(QTensorOps.q_matmul(tx, tq))
    q_ref, s_ref = co.quantize_dynamic(prod, oscheme(scheme))
    q, s = unpack_blob(QTensorOps.q_into_data(out))
    assert (q == q_ref).all() and s.tobytes() == s_ref.tobytes()
    # a bf16 operand: the product is bf16 (the float operand's dtype), and its values are what is quantized
    tb = FloatOps.float_from_data(ba.bf16_bits_from_f32(x), dev, ba.BF16)
    out_b = QTensorOps.q_matmul_propagate(tb, tq)
    prod_b = ba.f32_from_bf16_bits(FloatOps.float_into_data(QTensorOps.q_matmul(tb, tq)))
    q_ref, s_ref = co.quantize_dynamic(prod_b, oscheme(scheme))
    q, s = unpack_blob(QTensorOps.q_into_data(out_b))
    assert out_b.is_quantized and (q == q_ref).all() and s.tobytes() == s_ref.tobytes()


@pytest.mark.parametrize("m", [1, 2, 4, 16, 32, 64, 300, 2048])
def test_q_matmul_propagate_quantized_in_the_reduction(dev, m):
    """Propagate with 32 or 64 columns per scale: where the product ends in the sum of its K slices (every batch
    up to 32 rows, larger ones while the tiled kernel splits K) that kernel writes the quantized tensor and no
    float product exists; elsewhere two steps. Either way: quantize_dynamic of q_matmul's result, byte for byte,
    and the CPU oracle's quantization of that product."""
    rng = np.random.default_rng(100 + m)
    k, n = 512, 1024
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[rng.random(x.shape) < 0.01] *= 30
    cases = [QuantScheme().per_block((32,)), QuantScheme().per_block((64,)), QuantScheme(value=QuantValue.Q4S).per_block((32,)),
             QuantScheme(value=QuantValue.Q4S).per_block((64,)), QuantScheme(store=QuantStore.Native).per_block((32,)),
             QuantScheme(value=QuantValue.Q8F).per_block((32,)), QuantScheme().per_block((32,), ScaleDtype.F16),
             QuantScheme().per_block((128,)), QuantScheme()]
    for scheme in cases:
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
        for tx in (FloatOps.float_from_data(x, dev), FloatOps.float_from_data(ba.bf16_bits_from_f32(x), dev, ba.BF16)):
            out = QTensorOps.q_matmul_propagate(tx, tq)
            assert out.is_quantized and out.shape == (m, n)
            prod_t = QTensorOps.q_matmul(tx, tq)
            prod = FloatOps.float_into_data(prod_t)
            if tx.dtype == ba.BF16:
                prod = ba.f32_from_bf16_bits(prod).reshape(m, n)
                prod_t = FloatOps.float_from_data(prod, dev)
            two_steps = QTensorOps.quantize_dynamic(prod_t, scheme)
            blob = QTensorOps.q_into_data(out)
            assert blob.bytes.tobytes() == QTensorOps.q_into_data(two_steps).bytes.tobytes(), (scheme, tx.dtype)
            if scheme.scale_dtype == ScaleDtype.F32:
                q_ref, s_ref = co.quantize_dynamic(prod, oscheme(scheme))
                assert blob.bytes.tobytes() == co.encode(q_ref, oscheme(scheme), s_ref).tobytes(), (scheme, tx.dtype)
    # with a bias the Linear layer adds: not part of Propagate, the plain product is unchanged by all this
    assert FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq)).shape == (m, n)


def test_q_matmul_empty_k_is_zero(dev):
    """[M,0] x [0,N]: an empty sum, written as zeros over whatever the output held."""
    from burn_amd import _lib
    out = FloatOps.float_from_data(np.full((3, 8), 7.0, np.float32), dev)
    dummy = FloatOps.float_from_data(np.zeros(8, np.float32), dev)
    _lib.check(_lib.lib().bqk_q_matmul(dummy.data_ptr, _lib.F32, 3, 0, 8, dummy.data_ptr, dummy.data_ptr, 0,
                                       _lib.Q8S, _lib.STORE_PACKED_U32, _lib.F32, out.data_ptr, None, 0,
                                       dev.stream))
    assert (FloatOps.float_into_data(out) == 0).all()


def test_q_matmul_batched_broadcast(dev):
    rng = np.random.default_rng(77)
    x = rng.standard_normal((2, 3, 5, 64)).astype(np.float32)
    w = rng.standard_normal((1, 3, 64, 32)).astype(np.float32)
    scheme = QuantScheme().per_block((32,))
    tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), scheme)
    q, s = unpack_blob(QTensorOps.q_into_data(tq))
    wd = no.dequantize(q, s, [32]).astype(np.float64)
    out = FloatOps.float_into_data(QTensorOps.q_matmul(FloatOps.float_from_data(x, dev), tq))
    assert out.shape == (2, 3, 5, 32)
    np.testing.assert_allclose(out, x.astype(np.float64) @ wd, rtol=1e-4, atol=1e-4)


TORCH_INTEROP = r"""
import sys
import numpy as np
import torch                      # first: this process must use the HIP runtime torch ships
xt_host = np.random.default_rng(31).standard_normal((256, 1024)).astype(np.float32)
xt = torch.from_numpy(xt_host).to("cuda:0")
words = torch.empty((256, 256), dtype=torch.int32, device="cuda:0")
scales = torch.empty((256, 32), dtype=torch.float32, device="cuda:0")
out = torch.empty_like(xt)
torch.cuda.synchronize()
sys.path.insert(0, sys.argv[1])
from burn_amd import _lib
from oracle import c_oracle as co
L = _lib.lib()
n = xt_host.size
_lib.check(L.bqk_quantize_dynamic_block(xt.data_ptr(), n, 32, _lib.Q8S, _lib.STORE_PACKED_U32,
                                        words.data_ptr(), scales.data_ptr(), None))
_lib.check(L.bqk_dequantize(words.data_ptr(), n, 32, scales.data_ptr(), _lib.Q8S,
                            _lib.STORE_PACKED_U32, _lib.F32, out.data_ptr(), None))
torch.cuda.synchronize()
q_ref, s_ref = co.quantize_dynamic(xt_host, co.Scheme.make(co.Q8S, [32], co.STORE_PACKED_U32))
assert words.cpu().numpy().view(np.uint32).tobytes() == co.pack_u32(q_ref, co.Q8S).tobytes()
assert scales.cpu().numpy().tobytes() == s_ref.tobytes()
assert out.cpu().numpy().tobytes() == co.dequantize(q_ref, co.Scheme.make(co.Q8S, [32]), s_ref).tobytes()
print("torch-interop-ok")
"""


def test_kernel_level_entry_points_on_torch_memory():
    """bqk_* take plain device pointers: drive them with memory torch owns. Runs in a child
    process that imports torch first, so both use the one HIP runtime torch loads."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", TORCH_INTEROP, root], capture_output=True, text=True,
                          timeout=600)
    assert proc.returncode == 0 and "torch-interop-ok" in proc.stdout, proc.stderr[-2000:]

@pytest.mark.parametrize("seed", [11, 12, 13])
def test_q_matmul_and_linear_random_configurations(dev, seed):
    """Eighty seeded draws of (value, block, M, K, N, activation dtype, output dtype, bias): sizes
    straddle every kernel boundary (decode, small batch, both tile heights, K and N tails), and
    each product is compared with the float64 product of the dequantized weight."""
    from burn_amd import ModuleOps
    rng = np.random.default_rng(seed)
    for it in range(80):
        value = [QuantValue.Q8S, QuantValue.Q4S][rng.integers(2)]
        vpl = 4 if value == QuantValue.Q8S else 8
        m = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 100, 128, 129, 200, 257, 300]))
        k = int(rng.choice([4, 8, 16, 24, 32, 40, 64, 72, 96, 128, 130, 136, 192, 256, 264, 320, 512, 520, 1024]))
        block = [None, 32, 64, 8, 16, 128][rng.integers(6)]
        if block is not None and block % vpl:
            block = None
        n = max(vpl, block or 1) * int(rng.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 40]))
        dt = [ba.F32, ba.BF16][rng.integers(2)]
        odt = [None, ba.F32, ba.BF16][rng.integers(3)]
        use_bias = bool(rng.integers(2))
        case = f"draw {it}: {VAL[value][1]} block={block} m={m} k={k} n={n} lhs={dt} out={odt} bias={use_bias}"
        w = (rng.standard_normal((k, n)) * 0.1).astype(np.float32)
        x = rng.standard_normal((m, k)).astype(np.float32)
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev),
                                         QuantScheme(value=value, block=(block,) if block else None))
        q, s = unpack_blob(QTensorOps.q_into_data(tq))
        if dt == ba.BF16:
            xb = ba.bf16_bits_from_f32(x)
            x = ba.f32_from_bf16_bits(xb).reshape(m, k)
            xt = FloatOps.float_from_data(xb, dev, ba.BF16)
        else:
            xt = FloatOps.float_from_data(x, dev)
        ref = no.q_matmul_f64(x, q, s, [block] if block else None)
        if use_bias:
            bias = rng.standard_normal(n).astype(np.float32)
            ref = ref + bias[None, :].astype(np.float64)
            y = ModuleOps.linear(xt, tq, FloatOps.float_from_data(bias, dev), out_dtype=odt)
        else:
            y = QTensorOps.q_matmul(xt, tq, out_dtype=odt)
        assert y.shape == (m, n), case
        assert y.dtype == (odt if odt is not None else dt), case
        got = FloatOps.float_into_data(y)
        if y.dtype == ba.BF16:
            got = ba.f32_from_bf16_bits(got).reshape(m, n)
        err = np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-6)
        assert err <= (2e-2 if y.dtype == ba.BF16 else 1e-2), f"{case}: {err}"
        # burn's elementwise rule where the path keeps f32 activations (M <= 16, f32 in and out);
        # with bf16-rounded weights or outputs an element near zero can miss the 1e-2 floor honestly
        if dt == ba.F32 and y.dtype == ba.F32 and m <= 16:
            assert burn_approx_eq(got, ref, 1e-2, 1e-2).all(), case

def test_more_than_2_pow_31_elements(dev):
    """[33792, 65536] f32 (2.2e9 elements, 8.9 GB): every index past 2^31 must land where the
    oracle puts it. The tensor is one [1024, 65536] block repeated, so the oracle's answer for the
    block is the answer for every repetition, bit for bit (block-32 and per-tensor scales)."""
    rng = np.random.default_rng(9)
    rows, cols, reps = 1024, 65536, 33
    base = rng.standard_normal((rows, cols)).astype(np.float32)
    base[rng.random((rows, cols)) < 0.01] *= 30
    x = np.tile(base, (reps, 1))
    assert x.size > 2 ** 31
    xt = FloatOps.float_from_data(x, dev)
    del x
    for scheme in (QuantScheme().per_block((32,)), QuantScheme(value=QuantValue.Q4S)):
        tq = QTensorOps.quantize_dynamic(xt, scheme)
        got = FloatOps.float_into_data(QTensorOps.dequantize(tq)).reshape(reps, rows, cols)
        q_ref, s_ref = co.quantize_dynamic(base, oscheme(scheme), mt=True)
        d_ref = co.dequantize(q_ref, oscheme(scheme), s_ref, mt=True)
        assert (got.view(np.uint32) == d_ref.view(np.uint32)[None]).all()
        del got, tq
        dev.trim()
