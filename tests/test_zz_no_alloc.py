"""The allocation-free entry point bqk_q_linear_static against bqk_q_linear (same kernels, the
split-K scratch in a static device array instead of a caller workspace): bit-identical outputs
through the C ABI, on two calls in a row, the second with a smaller input. Collected last
(the file name sorts behind the other test files)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import burn_amd as ba  # noqa: E402
from burn_amd import FloatOps, QTensorOps, QuantScheme, QuantValue, _lib  # noqa: E402


def _run_both(dev, rng, m, k, n, value, x_bf16, with_bias, out_dtype):
    L = _lib.lib()
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme(value=value).per_block((32,)))
    xh = rng.standard_normal((m, k)).astype(np.float32)
    if x_bf16:
        x = FloatOps.float_from_data(ba.bf16_bits_from_f32(xh), dev, ba.BF16)
    else:
        x = FloatOps.float_from_data(xh, dev)
    bias = FloatOps.float_from_data(rng.standard_normal(n).astype(np.float32), dev) if with_bias else None
    cval = _lib.Q8S if value == QuantValue.Q8S else _lib.Q4S
    xdt = ba.BF16 if x_bf16 else ba.F32
    need = L.bqk_q_matmul_workspace(m, k, n, xdt, cval)   # an upper bound over every kernel choice
    assert need > 0
    ws = FloatOps.float_empty((need // 4 + 64,), dev)
    outs = []
    for static in (False, True):
        out = FloatOps.float_from_data(np.full((m, n), 7.0, np.float32) if out_dtype == ba.F32
                                       else np.full((m, n), 0x40E0, np.uint16), dev, out_dtype)
        bias_ptr = bias.data_ptr if bias is not None else None
        if static:
            _lib.check(L.bqk_q_linear_static(x.data_ptr, xdt, m, k, n, tw.data_ptr, tw.scales_ptr, 32, cval,
                                             _lib.STORE_PACKED_U32, bias_ptr, out_dtype, out.data_ptr, dev.stream))
        else:
            _lib.check(L.bqk_q_linear(x.data_ptr, xdt, m, k, n, tw.data_ptr, tw.scales_ptr, 32, cval,
                                      _lib.STORE_PACKED_U32, bias_ptr, out_dtype, out.data_ptr, ws.data_ptr,
                                      need, dev.stream))
        outs.append(FloatOps.float_into_data(out).tobytes())
    assert outs[0] == outs[1], f"static scratch result differs (m={m}, k={k}, n={n})"
    return outs[1]


def test_static_scratch_matches_workspace_entry_point():
    dev = ba.Device(0)
    rng = np.random.default_rng(2025)
    # two calls in a row on the same static array, the second smaller: nothing of the first may leak
    big = _run_both(dev, rng, 16, 2048, 4096, QuantValue.Q8S, False, True, ba.F32)     # split activations, 8 K slices
    small = _run_both(dev, rng, 4, 512, 1024, QuantValue.Q8S, False, False, ba.F32)    # decode kernel
    assert len(big) == 16 * 4096 * 4 and len(small) == 4 * 1024 * 4
    # the tiled kernel with split K (bf16 copy of an f32 lhs + partials in the scratch), then smaller again
    _run_both(dev, rng, 64, 2048, 1024, QuantValue.Q4S, False, True, ba.F32)
    _run_both(dev, rng, 1, 256, 512, QuantValue.Q4S, True, False, ba.BF16)
    _run_both(dev, rng, 40, 1024, 512, QuantValue.Q4S, True, True, ba.BF16)
    dev.sync()


def test_static_scratch_refuses_products_beyond_its_size():
    dev = ba.Device(0)
    L = _lib.lib()
    x = FloatOps.float_empty((16,), dev)
    rc = L.bqk_q_linear_static(x.data_ptr, ba.F32, 128, 4096, 14336, x.data_ptr, x.data_ptr, 32, _lib.Q4S,
                               _lib.STORE_PACKED_U32, None, ba.F32, x.data_ptr, dev.stream)
    assert rc == _lib.ERR_SIZE
    dev.sync()
