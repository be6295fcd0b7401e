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


def _static_call(L, dev, x, tw, bias, out, m, k, n, cval):
    return L.bqk_q_linear_static(x.data_ptr, ba.F32, m, k, n, tw.data_ptr, tw.scales_ptr, 32, cval, _lib.STORE_PACKED_U32,
                                 bias.data_ptr, ba.F32, out.data_ptr, dev.stream)


def test_static_scratch_under_graph_capture_and_without_allocating():
    """The two properties the entry point is for. (1) It allocates nothing: the device's free memory, as
    hipMemGetInfo reports it, is the same before and after calls of every kernel family. (2) It can be
    recorded into a HIP graph: the captured call, replayed three times with eager work and
    synchronisations in between and fresh activations each time, gives the eager call's bytes."""
    dev = ba.Device(0)
    L = _lib.lib()
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    rng = np.random.default_rng(77)

    def free_bytes():
        free, total = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    for m, k, n, value in ((1, 1024, 2048, QuantValue.Q8S), (16, 2048, 4096, QuantValue.Q8S), (64, 2048, 1024, QuantValue.Q4S)):
        cval = _lib.Q8S if value == QuantValue.Q8S else _lib.Q4S
        w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
        tw = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme(value=value).per_block((32,)))
        bias = FloatOps.float_from_data(rng.standard_normal(n).astype(np.float32), dev)
        xs = [rng.standard_normal((m, k)).astype(np.float32) for _ in range(3)]
        x = FloatOps.float_from_data(xs[0], dev)
        out = FloatOps.float_empty((m, n), dev)
        eager = []
        for xh in xs:      # eager results for the three activations (also warms every code path)
            x = FloatOps.float_from_data(xh, dev)
            _lib.check(_static_call(L, dev, x, tw, bias, out, m, k, n, cval))
            eager.append(FloatOps.float_into_data(out).tobytes())
        dev.sync()
        before = free_bytes()
        for _ in range(4):
            _lib.check(_static_call(L, dev, x, tw, bias, out, m, k, n, cval))
        dev.sync()
        assert free_bytes() == before, "the allocation-free entry point changed the device's free memory"
        # captured: the graph reads `xin` and writes `gout`; both live outside the capture
        xin = FloatOps.float_from_data(xs[0], dev)
        gout = FloatOps.float_empty((m, n), dev)
        graph, rc = dev.capture(lambda: _static_call(L, dev, xin, tw, bias, gout, m, k, n, cval))
        assert rc == _lib.OK
        for rep, xh in enumerate(xs):
            # eager work between the replays: new activations copied into the graph's input, a sync
            tmp = FloatOps.float_from_data(xh, dev)
            _lib.check(L.bqk_copy(tmp.data_ptr, xin.data_ptr, m * k * 4, dev.stream))
            dev.sync()
            graph.launch()
            got = FloatOps.float_into_data(gout).tobytes()
            assert got == eager[rep], f"replay {rep} of the captured static call differs (m={m})"
    dev.sync()


def test_host_transfers_are_refused_while_capturing():
    """*_from_data / *_into_data go through pinned staging memory and wait on events; recorded into a
    graph they would replay stale bytes, so they fail loudly instead (and the capture still ends cleanly)."""
    dev = ba.Device(0)
    t = FloatOps.float_from_data(np.arange(64, dtype=np.float32), dev)
    seen = {}

    def body():
        for name, fn in (("from_data", lambda: FloatOps.float_from_data(np.ones(64, np.float32), dev)),
                         ("into_data", lambda: FloatOps.float_into_data(t))):
            try:
                fn()
                seen[name] = None
            except ba.BurnqError as e:
                seen[name] = e.status
    graph, _ = dev.capture(body)
    assert seen == {"from_data": _lib.ERR_UNSUPPORTED_OP, "into_data": _lib.ERR_UNSUPPORTED_OP}
    del graph
    assert FloatOps.float_into_data(t).tolist() == list(range(64))
    dev.sync()
