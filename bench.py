#!/usr/bin/env python3
"""Benchmark of the quantized-tensor hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-others] [--no-cpu] [--only c1,c3,c4,c5,next,reference_bench]

Prints ONE JSON line. The headline workload is block-32 Q8S PackedU32 quantize_dynamic +
dequantize of an 8192x8192 f32 tensor (1 % outliers); a "step" is one such round trip with the
input already resident in HBM. `value` is algorithmic GB/s over the timed steps (wall clock
between device syncs); `roofline` is the dominant kernel alone, timed with HIP events on the
library's stream; `cpu_baseline` is the CPU oracle (a port of burn-ndarray's algorithm) timed on
a bounded sample of the same workload. The other configurations (per-tensor Q8S, Q4S dequantize,
decode q-GEMV, prefill q-GEMM) are measured the same way and reported under "others", each with
its own `roofline` and `cpu_baseline`. No number is printed for a configuration whose results do
not pass its parity gate (bit-exact integers / scales / dequantized floats, q_matmul inside burn's
permissive tolerance) on a slice of the tensors that were timed.
"""
from __future__ import annotations

import argparse
import collections
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0    # MI355X dense bf16 MFMA, published
# HBM bytes per launch of the dominant kernels, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs
# of this script (profiles/*.hbm_traffic.md), each counter (KiB) scaled by what it reads for bqk_copy,
# a copy of known size (256 MiB in, 256 MiB out): FETCH_SIZE x 1.99985, WRITE_SIZE x 0.99934.
# (The counters sit between the L2s and the fabric: a read served by the Infinity Cache counts.)
MEASURED_TRAFFIC_BYTES = {
    "quantize_block_kernel<4,8,dynamic>": 344002253,                       # algorithmic 343932928
    "dequantize_kernel<4,f32>": 343877837,                                 # algorithmic 343932928
    "absmax_kernel + quantize_tensor_kernel<4,from_absmax>": 151143800,    # both passes; algorithmic 150994948
    "dequantize_kernel<4,f32> per tensor": 83885773,                       # algorithmic 83886084
    "dequantize_kernel<8,f32>": 271535104,                                 # algorithmic 271581184
    # weights + scales are 66060288. M = 1 is one launch (the last workgroup of a strip sums the K slices: the
    # partial sums written and read back are in the figure); M = 4 / 16: the main kernel of the pair (the
    # reduction launch adds about 2.1 / 8.3 MB)
    "qgemv1_kernel<4,block,1> (one launch: the last workgroup of a strip sums the K slices)": 68192000,            # 67.21 MB read + 0.98 MB written
    "qsplit_kernel<4,block,f32,row-packed> + qgemv_reduce_kernel": 68551000,   # 66.72 MB read + 1.83 MB written
    "qsplit_kernel<4,block,f32> + qgemv_reduce_kernel": 75667000,             # 68.33 MB read + 7.34 MB written
    "qgemm_kernel<8,256,f32>": 333632000,   # 216.3 MB read (activations + weights + scales are 53.5 MB) + 117.4 MB written
}
METRIC = "quant/dequant + q-GEMV GB/s (% HBM peak); prefill q-GEMM TFLOP/s (% MFMA)"


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def time_loop(dev, fn, steps, warmup):
    """(wall seconds per step, event milliseconds per step) of `fn` enqueued `steps` times."""
    # setup: the output rings hold up to 16 live tensors, and every buffer the allocator will hand
    # out must exist before the clock starts (no hipMalloc inside the timed loop)
    for _ in range(18):
        fn()
    dev.sync()
    for _ in range(warmup):
        fn()
    dev.sync()
    t0 = time.perf_counter()
    dev.timer_start()
    for _ in range(steps):
        fn()
    ev_ms = dev.timer_stop()          # records + waits for the stop event
    dev.sync()
    wall = time.perf_counter() - t0
    return wall / steps, ev_ms / steps


def graph_ms(dev, fn, count, steps, warmup):
    """Milliseconds per call of the `count` library calls `fn` makes, replayed as one HIP graph:
    back-to-back graph nodes leave out the host submission gaps of an eager loop."""
    fn()
    graph, keep = dev.capture(fn)
    _, ev = time_loop(dev, graph.launch, max(3, steps), max(2, warmup))
    del graph, keep
    return ev / count


_GAMMA = np.uint64(0x9E3779B97F4A7C15)


def _splitmix64_mix(z):
    """The output function of splitmix64 on an array of states (uint64, wrapping arithmetic)."""
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


_INPUT_CACHE = {}


def normal_f32(seed, shape, scale=1.0, outliers=False):
    """Cached (read-only) wrapper of generate_normal_f32: the same big tensor feeds several legs."""
    key = (seed, tuple(shape), scale, outliers)
    if key not in _INPUT_CACHE:
        x = generate_normal_f32(seed, shape, scale, outliers)
        x.setflags(write=False)
        if x.size < (1 << 20):
            return x
        _INPUT_CACHE[key] = x
    return _INPUT_CACHE[key]


def generate_normal_f32(seed, shape, scale=1.0, outliers=False):
    """Deterministic inputs of the measurement spec: the splitmix64 stream seeded with `seed`
    (state_i = seed + (i + 1) * 0x9E3779B97F4A7C15, output mix(state_i)) -> Box-Muller in float64
    (outputs 2j and 2j + 1 give elements 2j and 2j + 1) -> float32. outliers: element i is scaled by
    50 iff splitmix64(seed ^ i) % 100 == 0 (the first output of a generator seeded with seed ^ i).
    Generated in chunks; the same bytes on every machine up to libm's log / sin / cos."""
    n = int(np.prod(shape))
    out = np.empty(n, np.float32)
    chunk = 1 << 22
    with np.errstate(over="ignore"):
        for lo in range(0, n, chunk):
            hi = min(n, lo + chunk)
            first = lo - (lo & 1)                                  # whole Box-Muller pairs
            count = (hi - first + 1) // 2 * 2
            idx = np.arange(first, first + count, dtype=np.uint64)
            z = _splitmix64_mix(np.uint64(seed) + (idx + np.uint64(1)) * _GAMMA)
            u = (z >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)   # [0, 1)
            r = np.sqrt(-2.0 * np.log(1.0 - u[0::2]))             # 1 - u in (0, 1]
            theta = (2.0 * np.pi) * u[1::2]
            pair = np.empty(count, np.float64)
            pair[0::2] = r * np.cos(theta)
            pair[1::2] = r * np.sin(theta)
            vals = pair[lo - first:hi - first]
            if scale != 1.0:
                vals = vals * scale
            vals = vals.astype(np.float32)
            if outliers:
                i = np.arange(lo, hi, dtype=np.uint64)
                pick = _splitmix64_mix((np.uint64(seed) ^ i) + _GAMMA) % np.uint64(100) == 0
                vals[pick] *= np.float32(50)
            out[lo:hi] = vals
    return out.reshape(shape)


def roofline(bound, achieved, peak, unit, kernel, avg_launch_ms):
    return {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(kernel),
            "kernel": kernel, "avg_launch_ms": round(avg_launch_ms, 5)}


def blas_threads():
    try:
        from threadpoolctl import threadpool_info
        n = [p.get("num_threads", 1) for p in threadpool_info() if p.get("user_api") == "blas"]
        return max(n) if n else 1
    except Exception:
        return os.cpu_count() or 1


class ParityError(RuntimeError):
    pass


# ------------------------------------------------------------------------------ workloads

def run_c2(ba, dev, steps, warmup, rows=8192):
    """Block-32 Q8S PackedU32 quantize_dynamic + dequantize of [rows, 8192] f32."""
    from burn_amd import FloatOps, QTensorOps, QuantScheme
    scheme = QuantScheme().per_block((32,))
    n = rows * 8192
    host = normal_f32(0xC2, (rows, 8192), outliers=True)
    # Every timed launch must stream from HBM, not from the 256 MB Infinity Cache: inputs rotate
    # over 5 tensors (1.25 GB), the dequantize-only loop over 16 quantized tensors (1.1 GB), and
    # the last 4 outputs stay alive so the allocator cycles through 5 distinct output buffers.
    nx, nq = 5, 16
    xs = [FloatOps.float_from_data(np.roll(host, i * 977, axis=0), dev) for i in range(nx)]
    state = {"i": 0}
    ring_q, ring_d = collections.deque(maxlen=4), collections.deque(maxlen=4)

    def round_trip():
        x = xs[state["i"] % nx]
        state["i"] += 1
        q = QTensorOps.quantize_dynamic(x, scheme)
        ring_q.append(q)
        ring_d.append(QTensorOps.dequantize(q))

    def quant_only():
        x = xs[state["i"] % nx]
        state["i"] += 1
        ring_q.append(QTensorOps.quantize_dynamic(x, scheme))

    qs = [QTensorOps.quantize_dynamic(xs[i % nx], scheme) for i in range(nq)]

    def dequant_only():
        state["i"] += 1
        ring_d.append(QTensorOps.dequantize(qs[state["i"] % nq]))

    # Plain copy kernel over the same inputs (read 4N + write 4N): the practical streaming ceiling
    # of this GPU, and the known-traffic kernel that HBM byte counters are calibrated against.
    from burn_amd import _lib
    dsts = [FloatOps.float_empty((rows, 8192), dev) for _ in range(3)]

    def copy_only():
        state["i"] += 1
        _lib.check(_lib.lib().bqk_copy(xs[state["i"] % nx].data_ptr, dsts[state["i"] % 3].data_ptr,
                                       4 * n, dev.stream))

    _, ev_c = time_loop(dev, copy_only, steps, warmup)
    del dsts
    bytes_dir = 4 * n + n + 4 * n // 32          # 5.125 N each direction
    wall, ev = time_loop(dev, round_trip, steps, warmup)
    _, ev_q_eager = time_loop(dev, quant_only, steps, warmup)
    _, ev_d_eager = time_loop(dev, dequant_only, steps, warmup)
    # per-kernel figures: HIP-graph replays of the same launches (10 quantize / 16 dequantize calls)
    ev_q = graph_ms(dev, lambda: [QTensorOps.quantize_dynamic(xs[i % nx], scheme) for i in range(10)], 10,
                    steps // 4, 2)
    ev_d = graph_ms(dev, lambda: [QTensorOps.dequantize(q) for q in qs], nq, steps // 4, 2)
    dev.trim()
    gbs_q = bytes_dir / (ev_q * 1e-3) / 1e9
    gbs_d = bytes_dir / (ev_d * 1e-3) / 1e9
    dominant = ("quantize_block_kernel<4,8,dynamic>", gbs_q, ev_q) if ev_q >= ev_d else \
               ("dequantize_kernel<4,f32>", gbs_d, ev_d)
    return {
        "workload": f"C2: Q8S block-32 PackedU32 quantize_dynamic + dequantize, [{rows},8192] f32, 1% outliers x50",
        "bytes_per_step": 2 * bytes_dir,
        "sec_per_step": wall,
        "event_ms_per_step": ev,
        "value_gbs": 2 * bytes_dir / wall / 1e9,
        "kernels": {"quantize_dynamic": {"ms": ev_q, "GB/s": gbs_q, "ms_eager_submission": ev_q_eager},
                    "dequantize": {"ms": ev_d, "GB/s": gbs_d, "ms_eager_submission": ev_d_eager}},
        "dominant": dominant,
        "copy_ceiling": {"ms": ev_c, "GB/s": 8 * n / (ev_c * 1e-3) / 1e9,
                         "what": "bqk_copy of the same 256 MiB input, read + write bytes; the best of the copy "
                                 "shapes swept (16 B per lane, 256-thread workgroups, non-temporal)"},
        "host": host, "scheme": scheme, "q0": qs[0], "x0": xs[0],
    }


def parity_gate_c2(ba, res, rows=256):
    """Bit-exact check of a slice of what was just timed, against the CPU oracle."""
    from burn_amd import FloatOps, QTensorOps
    from oracle import c_oracle as co
    blob = QTensorOps.q_into_data(res["q0"])
    values, scales = blob.split()
    osch = co.Scheme.make(co.Q8S, [32], co.STORE_PACKED_U32)
    x = res["host"][:rows]
    q_ref, s_ref = co.quantize_dynamic(x, osch, mt=True)
    ok = values[: rows * 8192].tobytes() == q_ref.tobytes() and scales[:rows].tobytes() == s_ref.tobytes()
    d = FloatOps.float_into_data(QTensorOps.dequantize(res["q0"]))[:rows]
    ok = ok and d.tobytes() == co.dequantize(q_ref, osch, s_ref, mt=True).tobytes()
    return bool(ok)


def run_c1(ba, dev, steps, warmup, cpu):
    from burn_amd import FloatOps, QTensorOps, QuantScheme, QuantStore
    from oracle import c_oracle as co
    scheme = QuantScheme(store=QuantStore.Native)
    n = 4096 * 4096
    host = normal_f32(0xC1, (4096, 4096))
    # 20 inputs (1.25 GB) / 64 quantized tensors (1 GB): every launch streams from HBM (see run_c2)
    nx, nq = 20, 64
    xs = [FloatOps.float_from_data(np.roll(host, i * 131, axis=0), dev) for i in range(nx)]
    qs = [QTensorOps.quantize_dynamic(xs[i % nx], scheme) for i in range(nq)]
    # parity gate: the whole first tensor (a per-tensor scale needs the whole range), bit for bit
    osch = co.Scheme.make(co.Q8S, None, co.STORE_NATIVE)
    q_ref, s_ref = co.quantize_dynamic(host, osch, mt=True)
    values, scales = QTensorOps.q_into_data(qs[0]).split()
    d = FloatOps.float_into_data(QTensorOps.dequantize(qs[0]))
    if not (values.tobytes() == q_ref.tobytes() and scales.tobytes() == s_ref.tobytes() and
            d[:256].tobytes() == co.dequantize(q_ref[:256], osch, s_ref, mt=True).tobytes()):
        raise ParityError("C1 differs from the CPU oracle")
    ev_q = graph_ms(dev, lambda: [QTensorOps.quantize_dynamic(x, scheme) for x in xs], nx, steps, warmup)
    ev_d = graph_ms(dev, lambda: [QTensorOps.dequantize(q) for q in qs[:32]], 32, steps, warmup)
    bq, bd = 9 * n + 4, 5 * n + 4
    out = {"workload": "C1: Q8S per-tensor Native quantize_dynamic + dequantize, [4096,4096] f32",
           "parity": "bit-exact vs CPU oracle: integers and scale of a whole timed tensor, 256 dequantized rows",
           "quantize_dynamic": {"ms": ev_q, "GB/s": bq / ev_q / 1e6, "GB/s_single_read_bound": 5 * n / ev_q / 1e6,
                                "bytes": bq, "note": "two passes (absmax, then quantize): 4N + 4N + N bytes"},
           "dequantize": {"ms": ev_d, "GB/s": bd / ev_d / 1e6, "bytes": bd},
           "roofline": roofline("hbm", bq / ev_q / 1e6, HBM_PEAK_GBS, "GB/s",
                                "absmax_kernel + quantize_tensor_kernel<4,from_absmax>", ev_q),
           "roofline_dequantize": roofline("hbm", bd / ev_d / 1e6, HBM_PEAK_GBS, "GB/s", "dequantize_kernel<4,f32> per tensor", ev_d),
           "timing": "HIP graphs of 20 / 32 calls over distinct tensors; ms per call"}
    if cpu:
        t0 = time.perf_counter()
        for _ in range(4):
            q, s = co.quantize_dynamic(host, osch)
            co.dequantize(q, osch, s)
        t = (time.perf_counter() - t0) / 4
        out["cpu_baseline"] = {"value": round((9 + 5) * host.size / t / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"the whole tensor ({host.size} elements), quantize_dynamic + dequantize, 4 passes of {t:.3f} s"}
    return out


def quantized_weight(ba, dev, seed, shape, value):
    """N(0, 0.02^2) weights quantized to block-32 PackedU32 on the GPU (parity-tested path)."""
    from burn_amd import FloatOps, QTensorOps, QuantScheme
    w = normal_f32(seed, shape, scale=0.02)
    t = QTensorOps.quantize_dynamic(FloatOps.float_from_data(w, dev), QuantScheme(value=value).per_block((32,)))
    return t


def unpack_columns(values, scales, k, n, cols, q4):
    """float64 dequantized weights of the sampled columns, from the blob's bytes (host side of the gates)."""
    if q4:
        words = values.view(np.uint32).reshape(k, n // 8)
        nib = (words[:, cols // 8] >> (4 * (cols % 8)).astype(np.uint32)) & 0xF
        q = (nib.astype(np.int32) ^ 8) - 8
    else:
        q = values.view(np.int8).reshape(k, n)[:, cols].astype(np.int32)
    return q.astype(np.float64) * scales.reshape(k, n // 32)[:, cols // 32].astype(np.float64)


def matmul_gate(name, out, ref64, max_outside=0):
    """q_matmul's bar: max-normalised error <= 1e-2 and burn's permissive elementwise rule."""
    rel = float(np.abs(out - ref64).max() / np.abs(ref64).max())
    diff = np.abs(out - ref64)
    bound = np.maximum(1e-2, 1e-2 * np.maximum(np.abs(out), np.abs(ref64)))
    outside = int(((out != ref64) & ~(diff < bound)).sum())
    if not (rel <= 1e-2 and outside <= max_outside):
        raise ParityError(f"{name}: max-normalised error {rel:.3e}, {outside} outputs outside burn's tolerance")
    return rel


def run_c3(ba, dev, steps, warmup, cpu):
    from burn_amd import FloatOps, QTensorOps, QuantValue
    from oracle import c_oracle as co
    n = 14336 * 4096
    w0 = quantized_weight(ba, dev, 0xC3, (14336, 4096), QuantValue.Q4S)
    blob = QTensorOps.q_into_data(w0)
    ws = [w0] + [QTensorOps.q_from_data(blob, dev) for _ in range(27)]   # 28 x 36.7 MB = 1 GB
    # parity gate: 256 rows of the dequantized weight, bit for bit
    osch = co.Scheme.make(co.Q4S, [32], co.STORE_PACKED_U32)
    values, scales = blob.split()
    rows = 256
    q_rows = co.unpack_u32(values.view(np.uint32)[: rows * 4096 // 8], (rows, 4096), co.Q4S)
    d = FloatOps.float_into_data(QTensorOps.dequantize(ws[5]))[:rows]
    if d.tobytes() != co.dequantize(q_rows, osch, scales[:rows], mt=True).tobytes():
        raise ParityError("C3 differs from the CPU oracle")
    ev = graph_ms(dev, lambda: [QTensorOps.dequantize(q) for q in ws[:14]], 14, steps, warmup)
    b = n // 2 + n // 8 + 4 * n
    out = {"workload": "C3: Q4S block-32 PackedU32 dequantize, [14336,4096] -> f32",
           "parity": "bit-exact vs CPU oracle on 256 rows of a timed tensor",
           "dequantize": {"ms": ev, "GB/s": b / ev / 1e6, "bytes": b},
           "roofline": roofline("hbm", b / ev / 1e6, HBM_PEAK_GBS, "GB/s", "dequantize_kernel<8,f32>", ev),
           "timing": "HIP graph of 14 calls over distinct tensors; ms per call"}
    if cpu:
        rows, passes = 14336, 4
        q_s = co.unpack_u32(values.view(np.uint32)[: rows * 4096 // 8], (rows, 4096), co.Q4S)
        t0 = time.perf_counter()
        for _ in range(passes):
            co.dequantize(q_s, osch, scales[:rows])
        t = (time.perf_counter() - t0) / passes
        elems = rows * 4096
        out["cpu_baseline"] = {"value": round((elems // 2 + elems // 8 + 4 * elems) / t / 1e9, 4), "unit": "GB/s", "cores": 1,
                               "kind": "port", "sample": f"the whole tensor ({elems} elements), dequantize, {passes} passes of {t:.2f} s"}
    return out


def run_c4(ba, dev, steps, warmup, cpu):
    from burn_amd import FloatOps, QTensorOps, QuantValue
    from oracle import c_oracle as co
    k, n = 4096, 14336
    # 16 distinct weight copies (1 GB) so each launch streams its weights from HBM
    w0 = quantized_weight(ba, dev, 0xC4, (k, n), QuantValue.Q8S)
    blob = QTensorOps.q_into_data(w0)
    ws = [w0] + [QTensorOps.q_from_data(blob, dev) for _ in range(15)]
    values, scales = blob.split()
    cols = np.sort(np.random.default_rng(4).choice(n, 512, replace=False))
    wd_cols = unpack_columns(values, scales, k, n, cols, q4=False)
    weight_bytes = k * n + 4 * k * n // 32
    out = {"workload": "C4: f32 [M,4096] x Q8S block-32 PackedU32 [4096,14336] -> f32",
           "parity": "512 sampled columns of every timed product vs float64 x . dequantize(W): max-normalised "
                     "error <= 1e-2 and burn's permissive rule on every element",
           "weight_bytes": weight_bytes}
    kernels = {1: "qgemv1_kernel<4,block,1> (one launch: the last workgroup of a strip sums the K slices)", 4: "qsplit_kernel<4,block,f32,row-packed> + qgemv_reduce_kernel",
               16: "qsplit_kernel<4,block,f32> + qgemv_reduce_kernel"}
    for m in (1, 4, 16):
        xh = normal_f32(100 + m, (m, k))
        x = FloatOps.float_from_data(xh, dev)
        st = {"i": 0}

        def gemv():
            st["i"] += 1
            st["y"] = QTensorOps.q_matmul(x, ws[st["i"] % len(ws)])

        y = FloatOps.float_into_data(QTensorOps.q_matmul(x, ws[3]))
        rel = matmul_gate(f"C4 M={m}", y[:, cols].astype(np.float64), xh.astype(np.float64) @ wd_cols)
        # eager: one host submission per call (two ~10 us kernels, so this is launch-bound)
        _, ev_eager = time_loop(dev, gemv, steps * 4, warmup * 2)
        # HIP graph: the 16 calls (one per weight copy) recorded once, replayed with one submission
        ev = graph_ms(dev, lambda: [QTensorOps.q_matmul(x, w) for w in ws], len(ws), steps, warmup)
        out[f"M={m}"] = {"ms": ev, "weight_GB/s": weight_bytes / ev / 1e6,
                         "GFLOP/s": 2.0 * m * k * n / ev / 1e6, "ms_eager_submission": ev_eager,
                         "max_normalised_error": rel,
                         "roofline": roofline("hbm", weight_bytes / ev / 1e6, HBM_PEAK_GBS, "GB/s", kernels[m], ev),
                         "timing": "HIP graph of 16 calls over 16 weight copies; ms per call"}
    if cpu:
        # the reference's route: dequantize the whole weight to f32, then an sgemm (crates/burn-ndarray/src/ops/qtensor.rs:223-267)
        osch = co.Scheme.make(co.Q8S, [32], co.STORE_PACKED_U32)
        q = values.view(np.int8).reshape(k, n)
        t0 = time.perf_counter()
        wd = co.dequantize(q, osch, scales)
        t_deq = time.perf_counter() - t0
        for m in (1, 4, 16):
            xh = normal_f32(100 + m, (m, k))
            t0 = time.perf_counter()
            for _ in range(3):
                xh @ wd
            t_mm = (time.perf_counter() - t0) / 3
            out[f"M={m}"]["cpu_baseline"] = {
                "value": round(weight_bytes / (t_deq + t_mm) / 1e9, 4), "unit": "GB/s (weight bytes per call)", "cores": blas_threads(),
                "kind": "port", "sample": f"whole weight: oracle dequantize on 1 core {t_deq:.2f} s + numpy sgemm on "
                                          f"{blas_threads()} threads {t_mm * 1e3:.1f} ms"}
        del wd
    return out


NEXT_PART = "all"  # --next-part: "matmul" (Linear, Propagate, Q4S batches, ternary, burnpack) or "tensor" (the rest) alone
C5_N = 14336  # weight columns of C5; --c5-n runs the same product at another width (tile-count studies)


VENDOR_GEMM = r"""
import sys, torch
m, k, n = (int(v) for v in sys.argv[1:4])
a = [torch.randn(m, k, device="cuda:0", dtype=torch.bfloat16) for _ in range(4)]
b = [torch.randn(k, n, device="cuda:0", dtype=torch.bfloat16) * 0.02 for _ in range(4)]
for i in range(12): a[i % 4] @ b[i % 4]
torch.cuda.synchronize()
s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
best = 1e9
for rep in range(5):
    s.record()
    for i in range(20): a[i % 4] @ b[i % 4]
    e.record(); torch.cuda.synchronize()
    best = min(best, s.elapsed_time(e) / 20)
print(best)
"""


def vendor_gemm_yardstick(m, k, n):
    """A plain bf16 x bf16 -> bf16 GEMM of the same shape through torch.matmul (the vendor's GEMM
    library), weights already dequantized and row-major [K, N] as here: what the matrix pipe yields
    on this box with no dequantization to do. A yardstick beside the roofline, not part of the
    product; run in a process of its own, None if torch is not usable there."""
    import subprocess
    try:
        p = subprocess.run([sys.executable, "-c", VENDOR_GEMM, str(m), str(k), str(n)], capture_output=True, text=True,
                           timeout=180)
        ms = float(p.stdout.strip().splitlines()[-1])
    except Exception:
        return None
    return {"ms": round(ms, 4), "TFLOP/s": round(2.0 * m * k * n / ms / 1e9, 1),
            "what": "torch.matmul, bf16 [M,K] @ bf16 row-major [K,N] -> bf16, best of 5 runs of 20 calls over 4 operand pairs"}


def run_c5(ba, dev, steps, warmup, cpu):
    from burn_amd import FloatOps, QTensorOps, QuantValue
    from oracle import c_oracle as co
    m, k, n = 2048, 4096, C5_N
    w = quantized_weight(ba, dev, 0xC5, (k, n), QuantValue.Q4S)
    ah = ba.f32_from_bf16_bits(ba.bf16_bits_from_f32(normal_f32(0xA5, (m, k)))).reshape(m, k)
    a = FloatOps.float_from_data(ba.bf16_bits_from_f32(ah), dev, ba.BF16)
    st = {}

    def gemm():
        st["y"] = QTensorOps.q_matmul(a, w, out_dtype=ba.F32)

    for _ in range(30):  # untimed priming: the chip needs a few milliseconds of this load to settle its clock
        gemm()
    blob = QTensorOps.q_into_data(w)
    values, scales = blob.split()
    # parity gate: 256 sampled columns x all 2048 rows against float64. The weights enter the MFMA
    # as bf16(s * q): output error sigma 2.1e-3, burn's 1e-2 floor is 4.7 sigma away, which
    # predicts 1.4 of these 524 288 outputs outside it; more than 8 fails the gate.
    cols = np.sort(np.random.default_rng(5).choice(n, 256, replace=False))
    y = FloatOps.float_into_data(st["y"])
    rel = matmul_gate("C5", y[:, cols].astype(np.float64), ah.astype(np.float64) @ unpack_columns(values, scales, k, n, cols, q4=True),
                      max_outside=8)
    _, ev_eager = time_loop(dev, gemm, steps, warmup)
    # as for C4: the same calls recorded into a HIP graph (8 per replay, over 4 copies of the weight)
    ws = [w] + [QTensorOps.q_from_data(blob, dev) for _ in range(3)]
    ev = graph_ms(dev, lambda: [QTensorOps.q_matmul(a, ws[i % 4], out_dtype=ba.F32) for i in range(8)], 8,
                  max(steps // 2, 2), max(warmup // 2, 1))
    flops = 2.0 * m * k * n
    tf = flops / ev / 1e9
    # the same product as a quantized Linear forward: the bias is added by the kernel's epilogue
    from burn_amd import ModuleOps
    bias = FloatOps.float_from_data(normal_f32(0xB5, (n,)), dev)

    def linear():
        st["y"] = ModuleOps.linear(a, w, bias, out_dtype=ba.F32)

    _, ev_lin = time_loop(dev, linear, steps, warmup)

    def gemm_bf16_out():  # the output dtype follows the activations unless the caller asks for f32
        st["y"] = QTensorOps.q_matmul(a, w)

    _, ev_h = time_loop(dev, gemm_bf16_out, steps, warmup)
    out = {"workload": f"C5: bf16 [2048,4096] x Q4S block-32 PackedU32 [4096,{n}] -> f32",
           "parity": "256 sampled columns x 2048 rows vs float64 x . dequantize(W): max-normalised error <= 1e-2, "
                     "at most 8 of 524288 outputs outside burn's permissive rule (bf16 weight rounding predicts 1.4)",
           "max_normalised_error": rel,
           "ms": ev, "TFLOP/s": tf, "flop_per_call": flops,
           "roofline": roofline("mfma", tf, BF16_PEAK_TFLOPS, "TFLOP/s", "qgemm_kernel<8,256,f32>", ev),
           "ms_eager_submission": ev_eager, "timing": "HIP graph of 8 calls over 4 weight copies; ms per call",
           "linear_with_bias_ms_eager": ev_lin, "bf16_output_ms_eager": ev_h}
    out["vendor_bf16_gemm"] = vendor_gemm_yardstick(m, k, n)
    if cpu:
        osch = co.Scheme.make(co.Q4S, [32], co.STORE_PACKED_U32)
        q = co.unpack_u32(values.view(np.uint32), (k, n), co.Q4S)
        t0 = time.perf_counter()
        wd = co.dequantize(q, osch, scales)
        t_deq = time.perf_counter() - t0
        rows = 128
        t0 = time.perf_counter()
        ah[:rows] @ wd
        t_mm = (time.perf_counter() - t0) * (m / rows)
        out["cpu_baseline"] = {
            "value": round(flops / (t_deq + t_mm) / 1e12, 4), "unit": "TFLOP/s", "cores": blas_threads(), "kind": "port",
            "sample": f"oracle dequantize of the whole weight on 1 core {t_deq:.2f} s + numpy sgemm of the first {rows} of "
                      f"{m} activation rows on {blas_threads()} threads, scaled to all rows ({t_mm:.2f} s)"}
        del wd, q
    return out


def run_reference_bench(ba, dev, steps, warmup, cpu):
    """The reference's own quantization benchmark (crates/burn-backend-tests/benches/quantization_ops.rs:
    26-205): per-tensor Q8S, inputs (i % 1000) / 1000 - 0.5, 4K / 64K / 1M elements, every call
    followed by a device sync (`bench_synced`) -- call latencies, not throughput. As there,
    `quantize` builds the tensor from host data inside the timed call; `q_matmul` multiplies two
    quantized n x n matrices. Medians of 200 calls, in microseconds."""
    from burn_amd import FloatOps, QTensorOps, QuantScheme, QuantStore
    from oracle import c_oracle as co
    scheme = QuantScheme(store=QuantStore.Native)
    osch = co.Scheme.make(co.Q8S, None, co.STORE_NATIVE)

    def median_us(fn, reps=200):
        for _ in range(10):
            fn()
            dev.sync()
        t = []
        for _ in range(reps):
            t0 = time.perf_counter()
            r = fn()
            dev.sync()
            t.append(time.perf_counter() - t0)
            del r
        return float(np.median(t) * 1e6)

    def pattern(n):
        return ((np.arange(n) % 1000).astype(np.float32) / np.float32(1000.0) - np.float32(0.5))

    out = {"what": "call + device sync, median of 200, microseconds, timed from Python; `from_c` is the same benchmark timed by "
                   "the plain-C caller (tests/cpp/c_abi_driver --latency, medians of 400)",
           "scheme": "Q8S per tensor, Native store",
           "published_by_the_reference": {
               "what": "medians of its CPU backends on an Apple M3 Max (crates/burn-flex/BENCHMARKS.md:776-806), microseconds; "
                       "quantize includes building the tensor from host data, as quantize_with_upload_us does here",
               "ndarray": {"quantize": {"4K": 10.4, "64K": 145, "1M": 2310}, "dequantize": {"4K": 48.8, "64K": 801, "1M": 13000},
                           "q_matmul": {"64x64": 137, "256x256": 1930, "512x512": 8070}},
               "flex": {"quantize": {"4K": 6.93, "64K": 109, "1M": 1750}, "dequantize": {"4K": 0.399, "64K": 3.73, "1M": 54.6},
                        "q_matmul": {"64x64": 7.10, "256x256": 147, "512x512": 641}}}}
    driver = os.path.join(ROOT, "tests", "cpp", "c_abi_driver")
    if os.path.exists(driver):
        import subprocess
        r = subprocess.run([driver, "--latency"], capture_output=True, text=True, timeout=300)
        if r.returncode != 0:
            raise RuntimeError(f"c_abi_driver --latency failed: {r.stderr[-400:]}")
        out["from_c"] = json.loads(r.stdout.strip().splitlines()[-1])
    for name, n in (("4K", 64 * 64), ("64K", 256 * 256), ("1M", 1024 * 1024)):
        host = pattern(n)
        x = FloatOps.float_from_data(host, dev)
        q = QTensorOps.quantize_dynamic(x, scheme)
        q_ref, s_ref = co.quantize_dynamic(host, osch)
        values, scales = QTensorOps.q_into_data(q).split()
        if values.tobytes() != q_ref.tobytes() or scales.tobytes() != s_ref.tobytes() or \
                FloatOps.float_into_data(QTensorOps.dequantize(q)).tobytes() != co.dequantize(q_ref, osch, s_ref).tobytes():
            raise ParityError(f"reference bench {name}: differs from the CPU oracle")
        out[name] = {"quantize_with_upload_us": median_us(lambda: QTensorOps.quantize_dynamic(FloatOps.float_from_data(host, dev), scheme)),
                     "quantize_us": median_us(lambda: QTensorOps.quantize_dynamic(x, scheme)),
                     "dequantize_us": median_us(lambda: QTensorOps.dequantize(q))}
    for n in (64, 256, 512):
        host = pattern(n * n).reshape(n, n)
        a = QTensorOps.quantize_dynamic(FloatOps.float_from_data(host, dev), scheme)
        b = QTensorOps.quantize_dynamic(FloatOps.float_from_data(host, dev), scheme)
        ad = FloatOps.float_into_data(QTensorOps.dequantize(a)).astype(np.float64)
        matmul_gate(f"reference bench q_matmul {n}", FloatOps.float_into_data(QTensorOps.q_matmul(a, b)), ad @ ad)
        out[f"q_matmul_{n}x{n}_us"] = median_us(lambda: QTensorOps.q_matmul(a, b))
    return out


# ------------------------------------------------------------------------------ CPU baseline

def run_next(ba, dev, steps, warmup, cpu):
    """The callers and formats either side of the hot path, each gated against the oracle before
    its figure is kept: the quantized Linear with its bias, narrow and two-level scale dtypes,
    layout ops on packed tensors, ternary weights, and a burnpack file loaded to the device."""
    import tempfile
    from burn_amd import (FloatOps, QTensorOps, ModuleOps, QuantScheme, QuantValue, QuantStore, ScaleDtype,
                          PackWriter, PackReader, TensorData)
    from oracle import c_oracle as co
    from oracle import np_oracle as no
    out = {"timing": "HIP graphs over distinct tensors; ms per call"}
    rng = np.random.default_rng(0xF0)

    if NEXT_PART in ("all", "matmul"):
        # ---- quantized Linear: the bias rides in the product's epilogue ------------------------------
        k, n = 4096, 14336
        w0 = quantized_weight(ba, dev, 0xC4, (k, n), QuantValue.Q8S)
        blob = QTensorOps.q_into_data(w0)
        ws = [w0] + [QTensorOps.q_from_data(blob, dev) for _ in range(15)]
        values, scales = blob.split()
        bias_h = rng.standard_normal(n, dtype=np.float32)
        bias = FloatOps.float_from_data(bias_h, dev)
        cols = np.arange(0, n, 37)
        wd = unpack_columns(values, scales, k, n, cols, q4=False)
        lin = {}
        for m in (1, 16):
            xh = rng.standard_normal((m, k), dtype=np.float32)
            x = FloatOps.float_from_data(xh, dev)
            got = FloatOps.float_into_data(ModuleOps.linear(x, ws[3], bias))[:, cols]
            matmul_gate(f"linear M={m}", got, xh.astype(np.float64) @ wd + bias_h[cols].astype(np.float64))
            t_lin = graph_ms(dev, lambda: [ModuleOps.linear(x, wq, bias) for wq in ws], 16, steps, warmup)
            t_mm = graph_ms(dev, lambda: [QTensorOps.q_matmul(x, wq) for wq in ws], 16, steps, warmup)
            lin[f"M={m}"] = {"ms": t_lin, "ms_without_bias": t_mm, "GB/s": (k * n + 4 * k * n // 32) / t_lin / 1e6}
        out["linear"] = {"workload": "x[M,4096] f32 x Q8S block-32 [4096,14336] + bias[14336] -> f32 (C4's weight)",
                         "parity": "vs float64 on every 37th column, rel 1e-2 and burn's elementwise rule", **lin}
        # ---- QuantPropagation::Propagate: the product comes back quantized with the weight's scheme -----
        osch = co.Scheme.make(co.Q8S, [32], co.STORE_PACKED_U32)
        scheme = ws[0].scheme
        prop = {}
        for m in (4, 16):
            x = FloatOps.float_from_data(rng.standard_normal((m, k), dtype=np.float32), dev)
            prod = FloatOps.float_into_data(QTensorOps.q_matmul(x, ws[2]))
            q_ref, s_ref = co.quantize_dynamic(prod, osch)
            if QTensorOps.q_into_data(QTensorOps.q_matmul_propagate(x, ws[2])).bytes.tobytes() != co.encode(q_ref, osch, s_ref).tobytes():
                raise ParityError(f"Propagate M={m}: differs from the CPU oracle's quantization of the product")
            t_p = graph_ms(dev, lambda: [QTensorOps.q_matmul_propagate(x, wq) for wq in ws], 16, steps, warmup)
            t_2 = graph_ms(dev, lambda: [QTensorOps.quantize_dynamic(QTensorOps.q_matmul(x, wq), scheme) for wq in ws], 16, steps, warmup)
            prop[f"M={m}"] = {"ms": t_p, "ms_product_then_quantize_dynamic": t_2}
        out["propagate"] = {"workload": "x[M,4096] f32 x Q8S block-32 [4096,14336] -> Q8S block-32 [M,14336] (C4's weight; the K-slice "
                                        "reduction quantizes what it sums)",
                            "parity": "blob bit-exact vs the CPU oracle's quantize_dynamic of the device's float product", **prop}
        del ws, w0, blob, values, scales
        dev.trim()

        # ---- the same products over a 4-bit weight ------------------------------------------------------
        w0 = quantized_weight(ba, dev, 0xC4, (k, n), QuantValue.Q4S)
        blob = QTensorOps.q_into_data(w0)
        ws = [w0] + [QTensorOps.q_from_data(blob, dev) for _ in range(15)]
        values, scales = blob.split()
        wd = unpack_columns(values, scales, k, n, cols, q4=True)
        q4 = {}
        for m in (1, 4, 16):
            xh = rng.standard_normal((m, k), dtype=np.float32)
            x = FloatOps.float_from_data(xh, dev)
            got = FloatOps.float_into_data(QTensorOps.q_matmul(x, ws[5]))[:, cols]
            rel = matmul_gate(f"Q4S M={m}", got, xh.astype(np.float64) @ wd)
            t_mm = graph_ms(dev, lambda: [QTensorOps.q_matmul(x, wq) for wq in ws], 16, steps, warmup)
            wb = k * n // 2 + 4 * k * n // 32
            q4[f"M={m}"] = {"ms": t_mm, "weight_GB/s": wb / t_mm / 1e6, "frac_hbm": wb / t_mm / 1e6 / HBM_PEAK_GBS,
                            "max_normalised_error": rel}
        out["q4s_small_batch"] = {"workload": "x[M,4096] f32 x Q4S block-32 PackedU32 [4096,14336] -> f32 (C4's shape, half the weight bytes)",
                                  "parity": "vs float64 on every 37th column, rel 1e-2 and burn's elementwise rule", **q4}
        # batches between the decode kernels (M <= 32) and prefill: the tiled kernel on row tiles it does not fill
        mid = {}
        for m in (64, 128, 512):
            xh = ba.f32_from_bf16_bits(ba.bf16_bits_from_f32(rng.standard_normal((m, k), dtype=np.float32))).reshape(m, k)
            x = FloatOps.float_from_data(ba.bf16_bits_from_f32(xh), dev, ba.BF16)
            got = FloatOps.float_into_data(QTensorOps.q_matmul(x, ws[5], out_dtype=ba.F32))[:, cols]
            rel = matmul_gate(f"Q4S M={m}", got, xh.astype(np.float64) @ wd, max_outside=8)
            t_mm = graph_ms(dev, lambda: [QTensorOps.q_matmul(x, wq, out_dtype=ba.F32) for wq in ws], 16, steps, warmup)
            mid[f"M={m}"] = {"ms": t_mm, "TFLOP/s": 2.0 * m * k * n / t_mm / 1e9, "frac_mfma": 2.0 * m * k * n / t_mm / 1e9 / BF16_PEAK_TFLOPS,
                             "weight_GB/s": wb / t_mm / 1e6, "max_normalised_error": rel}
        out["q4s_mid_batch"] = {"workload": "x[M,4096] bf16 x Q4S block-32 PackedU32 [4096,14336] -> f32, 64 to 512 rows (C5's operand types)",
                                "parity": "vs float64 on every 37th column, rel 1e-2; at most 8 outputs outside burn's elementwise rule "
                                          "(the tiled kernel rounds s * q to bf16)", **mid}
        del ws, w0, blob, values, scales
        dev.trim()

    if NEXT_PART in ("all", "tensor"):
        # ---- scale dtypes: quantize_dynamic + dequantize of C2's tensor ------------------------------
        rows = 8192
        nel = rows * 8192
        host = normal_f32(0xC2, (rows, 8192), outliers=True)
        xs = [FloatOps.float_from_data(np.roll(host, i * 977, axis=0), dev) for i in range(5)]
        small = np.ascontiguousarray(host[:256])
        codes = {ScaleDtype.F16: co.SCALE_F16, ScaleDtype.BF16: co.SCALE_BF16, ScaleDtype.UE4M3: co.SCALE_UE4M3}
        osch = co.Scheme.make(co.Q8S, [32], co.STORE_PACKED_U32)
        sd = {}
        for name, sdt, two in (("f16", ScaleDtype.F16, False), ("bf16", ScaleDtype.BF16, False), ("ue4m3", ScaleDtype.UE4M3, False),
                               ("f16 under f32", ScaleDtype.F16, True), ("ue4m3 under f32", ScaleDtype.UE4M3, True)):
            scheme = QuantScheme().per_block((32,), sdt)
            if two:
                scheme = scheme.per_tensor(ScaleDtype.F32)
            tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(small, dev), scheme)
            if two:
                q_ref, stored, g, eff = co.quantize_dynamic_two_level(small, osch, codes[sdt])
                want = co.encode_two_level(q_ref, osch, stored, g, codes[sdt])
            else:
                lo, hi = co.compute_range(small, osch)
                eff = co.scale_to_dtype(co.compute_q_params(lo, hi, osch.value), codes[sdt])
                q_ref = co.quantize(small, osch, eff)
                want = co.encode_with_scale_dtype(q_ref, osch, eff, codes[sdt])
            if QTensorOps.q_into_data(tq).bytes.tobytes() != want.tobytes():
                raise ParityError(f"{name} scales: the blob differs from the CPU oracle's")
            if FloatOps.float_into_data(QTensorOps.dequantize(tq)).tobytes() != co.dequantize(q_ref, osch, eff).tobytes():
                raise ParityError(f"{name} scales: dequantize differs from the CPU oracle")
            t_q = graph_ms(dev, lambda: [QTensorOps.quantize_dynamic(xs[i % 5], scheme) for i in range(10)], 10, steps, warmup)
            qs = [QTensorOps.quantize_dynamic(xs[i % 5], scheme) for i in range(16)]
            t_d = graph_ms(dev, lambda: [QTensorOps.dequantize(q) for q in qs], 16, steps, warmup)
            del qs
            b = 4 * nel + nel + sdt.size() * nel // 32 + (4 if two else 0)
            sd[name] = {"quantize_dynamic": {"ms": t_q, "GB/s": b / t_q / 1e6, "frac_hbm": b / t_q / 1e6 / HBM_PEAK_GBS},
                        "dequantize": {"ms": t_d, "GB/s": b / t_d / 1e6, "frac_hbm": b / t_d / 1e6 / HBM_PEAK_GBS}, "bytes": b}
            dev.trim()
        out["scale_dtypes"] = {"workload": "C2's tensor, Q8S block-32 PackedU32, block scales stored as f16 / bf16 / ue4m3, alone or "
                                           "relative to an f32 per-tensor scale (two launches more: the largest scale, the split)",
                               "parity": "blob and dequantized floats bit-exact vs CPU oracle on a 256-row tensor of the same data", **sd}

        # ---- the full-range value of the reference's default scheme --------------------------------------
        osch_f = co.Scheme.make(co.Q8F, [32], co.STORE_PACKED_U32)
        scheme_f = QuantScheme(value=QuantValue.Q8F).per_block((32,))
        tq = QTensorOps.quantize_dynamic(FloatOps.float_from_data(small, dev), scheme_f)
        q_ref, s_ref = co.quantize_dynamic(small, osch_f)
        if QTensorOps.q_into_data(tq).bytes.tobytes() != co.encode(q_ref, osch_f, s_ref).tobytes() or \
                FloatOps.float_into_data(QTensorOps.dequantize(tq)).tobytes() != co.dequantize(q_ref, osch_f, s_ref).tobytes():
            raise ParityError("Q8F: blob or dequantized floats differ from the CPU oracle's")
        t_q = graph_ms(dev, lambda: [QTensorOps.quantize_dynamic(xs[i % 5], scheme_f) for i in range(10)], 10, steps, warmup)
        b = 4 * nel + nel + 4 * nel // 32
        out["full_range"] = {"workload": "C2's tensor, Q8F (-128..127, span 255) block-32 PackedU32, f32 scales: quantize_dynamic",
                             "parity": "blob and dequantized floats bit-exact vs CPU oracle on a 256-row tensor of the same data",
                             "quantize_dynamic": {"ms": t_q, "GB/s": b / t_q / 1e6, "frac_hbm": b / t_q / 1e6 / HBM_PEAK_GBS}, "bytes": b}
        dev.trim()

        # ---- layout ops on a packed tensor -------------------------------------------------------------
        scheme = QuantScheme().per_block((32,))
        tq_small = QTensorOps.quantize_dynamic(FloatOps.float_from_data(small, dev), scheme)
        q_ref, s_ref = co.quantize_dynamic(small, osch)
        tr = QTensorOps.q_into_data(QTensorOps.q_swap_dims(tq_small, 0, 1))
        tv, ts = tr.split()
        if no.unpack_u32(tv.view(np.uint32), tr.shape, "Q8S").tobytes() != np.ascontiguousarray(q_ref.T).tobytes() or \
                ts.reshape(-1).tobytes() != np.ascontiguousarray(s_ref.reshape(256, 256).T).tobytes():
            raise ParityError("swap_dims of a packed block-quantized tensor differs from the oracle's transpose")
        qs = [QTensorOps.quantize_dynamic(xs[i % 5], scheme) for i in range(8)]
        t_t = graph_ms(dev, lambda: [QTensorOps.q_swap_dims(q, 0, 1) for q in qs], 8, steps, warmup)
        b = 2 * (nel + 4 * nel // 32)
        out["layout"] = {"workload": "q_swap_dims(0, 1) of a Q8S block-32 PackedU32 [8192,8192] tensor: values repacked along "
                                     "the new last dim, scales moved with their blocks",
                         "parity": "values and scales bit-exact vs the transposed oracle tensor, 256 x 8192",
                         "swap_dims": {"ms": t_t, "GB/s": b / t_t / 1e6, "frac_hbm": b / t_t / 1e6 / HBM_PEAK_GBS, "bytes": b}}
        # ---- integer-domain ops on the same packed tensors ------------------------------------------------
        from burn_amd import IntOps
        import burn_amd as _ba
        idx_h = np.random.default_rng(0x5E1).integers(0, 256, 192)
        sl = (slice(32, 224), slice(2048, 6144))
        got = QTensorOps.q_into_data(QTensorOps.q_slice(tq_small, sl))
        gv, gs = got.split()
        if no.unpack_u32(gv.view(np.uint32), got.shape, "Q8S").tobytes() != np.ascontiguousarray(q_ref[sl]).tobytes() or \
                gs.reshape(-1).tobytes() != np.ascontiguousarray(s_ref.reshape(256, 256)[32:224, 64:192]).tobytes():
            raise ParityError("q_slice of a packed block-quantized tensor differs from the sliced oracle tensor")
        got = QTensorOps.q_into_data(QTensorOps.q_select(tq_small, 0, IntOps.int_from_data(idx_h.astype(np.int64), dev)))
        gv, gs = got.split()
        if no.unpack_u32(gv.view(np.uint32), got.shape, "Q8S").tobytes() != np.ascontiguousarray(q_ref[idx_h]).tobytes() or \
                gs.reshape(-1).tobytes() != np.ascontiguousarray(s_ref.reshape(256, 256)[idx_h]).tobytes():
            raise ParityError("q_select of a packed block-quantized tensor differs from the oracle's rows")
        t_sl = graph_ms(dev, lambda: [QTensorOps.q_slice(q, (slice(1024, 7168), slice(2048, 6144))) for q in qs], 8, steps, warmup)
        b_sl = 2 * (6144 * 4096 + 4 * 6144 * 4096 // 32)
        rows_idx = IntOps.int_from_data(np.random.default_rng(0x5E2).integers(0, rows, rows).astype(np.int64), dev)
        t_se = graph_ms(dev, lambda: [QTensorOps.q_select(q, 0, rows_idx) for q in qs], 8, steps, warmup)
        b_se = 2 * (nel + 4 * nel // 32) + 8 * rows
        pt = QuantScheme()                                                   # Q8S per tensor, packed
        osch_pt = co.Scheme.make(co.Q8S, None, co.STORE_PACKED_U32)
        q_pt, _ = co.quantize_dynamic(small, osch_pt)
        am = IntOps.int_into_data(QTensorOps.q_argmax(QTensorOps.quantize_dynamic(FloatOps.float_from_data(small, dev), pt), 1))
        if am.reshape(-1).tolist() != q_pt.argmax(axis=1).tolist():
            raise ParityError("q_argmax differs from the first maximum of the oracle's integers")
        qpt = [QTensorOps.quantize_dynamic(xs[i % 5], pt) for i in range(8)]
        t_am = graph_ms(dev, lambda: [QTensorOps.q_argmax(q, 1) for q in qpt], 8, steps, warmup)
        b_am = nel + 8 * rows
        out["integer_domain"] = {
            "workload": "q_slice [1024:7168, 2048:6144], q_select of 8192 random rows (dim 0) of a Q8S block-32 PackedU32 [8192,8192] "
                        "tensor, values and scales moved together; q_argmax along the last dim of the per-tensor one",
            "parity": "integers and scales bit-exact vs numpy on the oracle's tensor, 256 x 8192",
            "q_slice": {"ms": t_sl, "GB/s": b_sl / t_sl / 1e6, "frac_hbm": b_sl / t_sl / 1e6 / HBM_PEAK_GBS, "bytes": b_sl},
            "q_select": {"ms": t_se, "GB/s": b_se / t_se / 1e6, "frac_hbm": b_se / t_se / 1e6 / HBM_PEAK_GBS, "bytes": b_se},
            "q_argmax": {"ms": t_am, "GB/s": b_am / t_am / 1e6, "frac_hbm": b_am / t_am / 1e6 / HBM_PEAK_GBS, "bytes": b_am}}
        del qpt, rows_idx
        dev.trim()

        # ---- Calibration::AbsMean: the ranges of a ternary weight ------------------------------------------
        tsch_am = QuantScheme(value=QuantValue.Q2S)
        osch_t = co.Scheme.make(co.Q2S, None, co.STORE_PACKED_U32)
        g_ref = co.compute_range_abs_mean(small, osch_t)[1].reshape(-1)[0]
        tq_am = QTensorOps.quantize_abs_mean(FloatOps.float_from_data(small, dev), tsch_am)
        av, a_s = QTensorOps.q_into_data(tq_am).split()
        g_gpu = a_s.reshape(-1)
        # the mean is a sum the reference leaves to its backend (no order to match): Tolerance::default() between the
        # two, then everything computed from the device's own scale bit for bit
        if abs(float(g_gpu[0]) - float(g_ref)) > 1e-5 * abs(float(g_ref)):    # scale = 2 gamma / 2
            raise ParityError("AbsMean: gamma differs from the oracle's beyond a rounding of the sum")
        if no.unpack_u32(av.view(np.uint32), small.shape, "Q2S").tobytes() != co.quantize(small, osch_t, g_gpu.copy()).tobytes():
            raise ParityError("AbsMean: the integers differ from the oracle's quantize with the same scale")
        t_am2 = graph_ms(dev, lambda: [QTensorOps.quantize_abs_mean(xs[i % 5], tsch_am) for i in range(10)], 10, steps, warmup)
        b_am2 = 4 * nel + 4 * nel + nel // 4 + 4
        out["abs_mean"] = {"workload": "C2's tensor -> Q2S per tensor PackedU32 with Calibration::AbsMean: mean |x| (one pass), then quantize",
                           "parity": "gamma within 1e-5 of the oracle's f64 mean; integers bit-exact vs the oracle's quantize with the device's scale, 256 x 8192",
                           "quantize_abs_mean": {"ms": t_am2, "GB/s": b_am2 / t_am2 / 1e6, "frac_hbm": b_am2 / t_am2 / 1e6 / HBM_PEAK_GBS,
                                                 "bytes": b_am2, "note": "two passes over x: 4N + 4N + N/4 bytes"}}
        del qs, xs
        dev.trim()

    if NEXT_PART in ("all", "matmul"):  # (continued: ternary weights, burnpack)
        # ---- ternary weights ---------------------------------------------------------------------------
        wt = normal_f32(0xF4, (k, n), 0.02)
        tsch = QuantScheme(value=QuantValue.Q2S)
        tws = [QTensorOps.quantize_dynamic(FloatOps.float_from_data(wt, dev), tsch) for _ in range(8)]
        tblob = QTensorOps.q_into_data(tws[0])
        tvals, tscale = tblob.split()
        q_t = no.unpack_u32(tvals.view(np.uint32), (k, n), "Q2S")
        tern = {}
        for m in (1, 16):
            xh = rng.standard_normal((m, k), dtype=np.float32)
            x = FloatOps.float_from_data(xh, dev)
            got = FloatOps.float_into_data(QTensorOps.q_matmul(x, tws[1]))
            ref = (xh.astype(np.float64) @ q_t[:, cols].astype(np.float64)) * np.float64(tscale.reshape(-1)[0])
            matmul_gate(f"ternary M={m}", got[:, cols], ref)
            t = graph_ms(dev, lambda: [QTensorOps.q_matmul(x, wq) for wq in tws], 8, steps, warmup)
            tb = k * n // 4 + 4
            tern[f"M={m}"] = {"ms": t, "GB/s": tb / t / 1e6, "frac_hbm": tb / t / 1e6 / HBM_PEAK_GBS}
        out["ternary"] = {"workload": "x[M,4096] f32 x Q2S per-tensor PackedU32 [4096,14336] (16 values per word) -> f32",
                          "parity": "vs float64 on every 37th column, rel 1e-2 and burn's elementwise rule", **tern}
        del tws
        dev.trim()

        # ---- a burnpack file to the device -------------------------------------------------------------
        w3 = quantized_weight(ba, dev, 0xC3, (14336, 4096), QuantValue.Q4S)
        want = QTensorOps.q_into_data(w3).bytes.tobytes()
        wr = PackWriter()
        wr.add_tensor("mlp.up_proj.weight", w3)
        with tempfile.TemporaryDirectory() as tmp:
            path = os.path.join(tmp, "c3.bpk")
            wr.write_to_file(path)
            size = os.path.getsize(path)
            best = None
            for _ in range(3):
                t0 = time.perf_counter()
                rd = PackReader(path)
                t = rd.load("mlp.up_proj.weight", dev)
                dev.sync()
                dt = time.perf_counter() - t0
                rd.close()
                best = dt if best is None else min(best, dt)
            if QTensorOps.q_into_data(t).bytes.tobytes() != want:
                raise ParityError("the tensor loaded from the burnpack file differs from the one written")
        out["burnpack"] = {"workload": "C3's weight (Q4S block-32 [14336,4096]) written to a burnpack file and loaded back to the "
                                       "device: open, parse, one host-to-device copy of values || scales",
                           "parity": "blob of the loaded tensor byte-identical to the written one's",
                           "file_bytes": size, "load_ms": best * 1e3, "GB/s": size / best / 1e9,
                           "note": "host path (page cache + PCIe), not an HBM figure"}
    return out


def cpu_baseline_c2(passes=5):
    """The oracle (port of burn-ndarray's serial loops), one thread, on the whole C2 tensor,
    `passes` times over (about 10 s of CPU work)."""
    from oracle import c_oracle as co
    x = normal_f32(0xC2, (8192, 8192), outliers=True)
    osch = co.Scheme.make(co.Q8S, [32], co.STORE_NATIVE)
    n = x.size
    t0 = time.perf_counter()
    for _ in range(passes):
        q, s = co.quantize_dynamic(x, osch)
        d = co.dequantize(q, osch, s)
    t1 = time.perf_counter()
    qm, sm = co.quantize_dynamic(x, osch, mt=True)
    dm = co.dequantize(qm, osch, sm, mt=True)
    t2 = time.perf_counter()
    assert d.shape == x.shape and dm.shape == x.shape
    b = 2 * (4 * n + n + 4 * n // 32)
    return {"value": round(passes * b / (t1 - t0) / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"the whole [8192,8192] tensor ({n} elements), quantize_dynamic + dequantize, "
                      f"{passes} passes, {t1 - t0:.1f} s",
            "all_cores": {"value": round(b / (t2 - t1) / 1e9, 3), "cores": co.max_threads(),
                          "note": "same arithmetic, blocks spread over OpenMP threads, one pass"}}


def main():
    global C5_N, NEXT_PART
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-others", action="store_true", help="skip the C1/C3/C4/C5 side measurements")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--only", default="", help="comma list of side configs to run (c1,c3,c4,c5,next,reference_bench)")
    ap.add_argument("--next-part", default="all", choices=["all", "matmul", "tensor"],
                    help="run only one half of the `next` legs (a profiler may not survive all of their graphs in one process)")
    ap.add_argument("--c5-n", type=int, default=C5_N, help="weight columns of the C5 side measurement (default: C5's 14336)")
    args = ap.parse_args()
    C5_N = args.c5_n
    NEXT_PART = args.next_part
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU (the kernels shard by rows / columns with no "
              "exchange; no multi-GPU figure is produced). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import burn_amd as ba
    dev = ba.Device(0)

    log("C2 (headline) ...")
    res = run_c2(ba, dev, args.steps, args.warmup)
    parity = parity_gate_c2(ba, res)
    if not parity:
        print("bench.py: parity gate failed for C2; no number is reported", file=sys.stderr)
        sys.exit(1)
    name, gbs, ev_ms = res["dominant"]
    line = {
        "metric": METRIC,
        "value": round(res["value_gbs"], 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["sec_per_step"] * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": res["workload"], "bytes_per_step": res["bytes_per_step"],
                   "frac_hbm_peak": round(res["value_gbs"] / HBM_PEAK_GBS, 4),
                   "note": "value times the round trip: its dequantize half reads the 72 MB tensor the quantize half "
                           "just wrote, partly from the 256 MB Infinity Cache, so it can exceed what the two kernels "
                           "reach on cold inputs; roofline is the slower kernel alone on cold inputs"},
        "roofline": roofline("hbm", gbs, HBM_PEAK_GBS, "GB/s", name, ev_ms),
        "parity": "bit-exact vs CPU oracle on a 256-row slice of the timed tensors",
        "kernels": {k: {kk: round(vv, 4) for kk, vv in v.items()} for k, v in res["kernels"].items()},
        "copy_ceiling": {k: (round(v, 4) if isinstance(v, float) else v) for k, v in res["copy_ceiling"].items()},
    }
    for key in ("host", "q0", "x0"):
        res.pop(key, None)
    del res
    dev.trim()

    if not args.no_cpu:
        log("CPU baseline ...")
        line["cpu_baseline"] = cpu_baseline_c2()
    if not args.no_others:
        only = [s for s in args.only.split(",") if s]
        others = {}
        for key, fn in (("c1", run_c1), ("c3", run_c3), ("c4", run_c4), ("c5", run_c5), ("next", run_next),
                        ("reference_bench", run_reference_bench)):
            if only and key not in only:
                continue
            log(f"{key} ...")
            try:
                others[key] = fn(ba, dev, max(5, args.steps // 2), max(2, args.warmup // 2), not args.no_cpu)
            except ParityError as e:   # no number without parity
                others[key] = {"error": f"parity gate failed, nothing reported: {e}"}
            except Exception as e:     # a side measurement must not hide the headline
                others[key] = {"error": str(e)}
            dev.trim()

        def rnd(o):
            if isinstance(o, dict):
                return {k: rnd(v) for k, v in o.items()}
            if isinstance(o, float):
                return round(o, 4) if abs(o) >= 1 else float(f"{o:.4g}")
            return o
        line["others"] = rnd(others)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
