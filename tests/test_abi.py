"""CPU-side checks of the product library's boundary: it loads, exports every symbol that
include/burnq.h declares, validates arguments before touching a GPU, and refuses to run
without one (no CPU path)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import burn_amd as ba
from burn_amd import _lib
from burn_amd.quantization import QuantScheme, QuantStore, QuantValue, ScaleDtype, params_shape

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "burnq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bqk?_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _lib.lib()
    names = declared_symbols()
    assert len(names) >= 40
    for name in names:
        assert hasattr(L, name), f"{name} declared in burnq.h but not exported"
    # and the ctypes table covers the header exactly
    assert sorted(_lib.SIGNATURES) == names


def test_entry_points_named_in_the_guides_exist():
    """Every bq_* / bqk_* function the written guides name (binding guide, design notes, readme) is one
    the header declares: a maintainer who binds from the text gets names that link."""
    exported = set(declared_symbols())
    types = {"bq_status", "bq_tensor", "bq_device", "bq_scheme", "bq_graph", "bq_pack", "bq_pack_writer", "bq_pack_entry",
             "bq_backend", "bq_oracle"}          # C types, the oracle's file stem, and one name the text says was not built
    unknown = {}
    for doc in ("INTEGRATION.md", "DESIGN.md", "README.md"):
        path = os.path.join(ROOT, doc)
        if not os.path.exists(path):
            continue
        for name in set(re.findall(r"\b(bqk?_[a-z0-9_]*[a-z0-9])\b(?![_*])", open(path).read())):
            if name in exported or name in types:
                continue
            # families written with a wildcard or a brace list (bq_pack_*, bq_graph_{begin,end}_capture) leave a prefix
            if any(e.startswith(name + "_") for e in exported):
                continue
            unknown.setdefault(doc, []).append(name)
    assert not unknown, unknown


def test_scheme_struct_layout_matches_header():
    assert C.sizeof(_lib.CScheme) == 16
    c = QuantScheme(QuantValue.Q4S, (32,), QuantStore.PackedU32).to_c()
    raw = bytes(c)
    assert raw[0] == _lib.Q4S and raw[1] == _lib.LEVEL_BLOCK and raw[2] == _lib.STORE_PACKED_U32
    assert raw[4] == 1 and raw[8] == 32
    assert QuantScheme.from_c(c) == QuantScheme(QuantValue.Q4S, (32,), QuantStore.PackedU32)
    two = QuantScheme().per_block((2, 16), ScaleDtype.F16).per_tensor(ScaleDtype.F32)
    raw = bytes(two.to_c())
    assert raw[3] == _lib.SCALE_F16 and raw[4] == 2 and raw[5] == 1 and raw[8:10] == bytes([2, 16])
    assert QuantScheme.from_c(two.to_c()) == two and two.per_block((2, 16), ScaleDtype.F16).tensor_scale is None


def test_data_len_matches_reference_formula(kats):
    # quantized_data_len needs no device
    for case in kats["packed_q4_data_len"]["cases"]:
        assert ba.TensorData.data_len(case["shape"], QuantScheme(value=QuantValue.Q4S)) == case["len"]
    assert ba.TensorData.data_len((2, 3), QuantScheme(store=QuantStore.Native)) == 6 + 4
    assert ba.TensorData.data_len((16,), QuantScheme().per_block((8,))) == 16 + 8
    assert ba.TensorData.data_len((8192, 8192), QuantScheme().per_block((32,))) == 8192 * 8192 + 4 * 8192 * 256
    assert params_shape((8192, 8192), QuantScheme().per_block((32,))) == (8192, 256)
    # two-level: block scales in their dtype, then the f32 per-tensor scale
    # (crates/burn-std/src/tensor/quantization.rs:659-684: 8 values + 2 one-byte scales + 4 there)
    two = QuantScheme(store=QuantStore.Native).per_block((4,), ScaleDtype.F16).per_tensor()
    assert ba.TensorData.data_len((8,), two) == 8 + 2 * 2 + 4
    assert params_shape((4, 8), QuantScheme().per_block((2, 4))) == (2, 2)


def test_kernel_level_argument_validation_needs_no_gpu():
    L = _lib.lib()
    buf = np.zeros(64, np.float32)
    p = buf.ctypes.data
    assert L.bqk_quantize_dynamic_block(None, 64, 32, _lib.Q8S, _lib.STORE_PACKED_U32, p, p, None) == _lib.ERR_NULL
    assert L.bqk_quantize_dynamic_block(p, 64, 24, _lib.Q8S, _lib.STORE_PACKED_U32, p, p, None) == _lib.ERR_SHAPE
    assert L.bqk_quantize_dynamic_block(p, 64, 32, 7, _lib.STORE_PACKED_U32, p, p, None) == _lib.ERR_UNSUPPORTED_SCHEME
    assert L.bqk_quantize_per_tensor(p, 6, p, _lib.Q4S, _lib.STORE_NATIVE, p, None) == _lib.ERR_UNSUPPORTED_SCHEME
    assert b"sub-byte" in L.bq_last_error()
    assert L.bqk_quantize_per_tensor(p, 6, p, _lib.Q8S, _lib.STORE_PACKED_U32, p, None) == _lib.ERR_SHAPE
    assert b"Can't store in u32" in L.bq_last_error()
    assert L.bqk_dequantize(p, 64, 32, p, _lib.Q8S, _lib.STORE_PACKED_U32, 9, p, None) == _lib.ERR_DTYPE
    assert L.bqk_q_matmul_workspace(1, 4096, 14336, _lib.F32, _lib.Q8S) > 0
    assert L.bqk_q_matmul_workspace(2048, 4096, 14336, _lib.BF16, _lib.Q4S) == 0


def test_oversized_lds_request_is_refused_on_the_host():
    """Every kernel with a dynamic LDS request passes this guard before it is launched: a request
    beyond what the device grants per workgroup is an error on the host, never a launch."""
    L = _lib.lib()
    limit = 160 * 1024
    assert L.bqk_lds_request_status(limit, limit) == _lib.OK
    assert L.bqk_lds_request_status(64 * 1024, limit) == _lib.OK
    assert L.bqk_lds_request_status(limit + 512, limit) == _lib.ERR_HIP
    assert b"launch refused" in L.bq_last_error()
    assert L.bqk_lds_request_status(64 * 1024 + 1, 64 * 1024) == _lib.ERR_HIP


def test_data_len_of_natively_stored_values_of_any_width():
    """crates/burn-store/src/tensor_snapshot.rs:545-581 (data_len_matches_materialized_bytes_when_
    quantized): the reference's CPU backend stores quantized values natively, one i8 each, also for
    4- and 2-bit value types, and a tensor's bytes are that many values plus its f32 scale -- for
    element counts that are and are not multiples of 4."""
    for value in (QuantValue.Q8S, QuantValue.Q4S, QuantValue.Q2S):
        for shape in ((32, 32), (3, 3), (5, 5), (2, 3)):
            n = shape[0] * shape[1]
            assert ba.TensorData.data_len(shape, QuantScheme(value=value, store=QuantStore.Native)) == n + 4


def test_data_len_refuses_what_q_from_data_would_refuse():
    """quantized_data_len runs the full scheme check: no division by a zero block extent, no
    length for a shape the scheme cannot hold."""
    L = _lib.lib()
    out = C.c_size_t()

    def status(scheme, shape):
        arr = (C.c_size_t * len(shape))(*shape)
        c = scheme.to_c() if isinstance(scheme, QuantScheme) else scheme
        return L.bq_quantized_data_len(C.byref(c), arr, len(shape), C.byref(out))

    assert status(QuantScheme().per_block((32,)), (4, 64)) == _lib.OK and out.value == 256 + 4 * 8
    zero = QuantScheme().per_block((32,)).to_c()
    zero.block[0] = 0
    assert status(zero, (4, 64)) == _lib.ERR_SHAPE
    assert status(QuantScheme().per_block((32,)), (4, 48)) == _lib.ERR_SHAPE          # 48 % 32
    assert status(QuantScheme(value=QuantValue.Q4S), (3, 5)) == _lib.OK and out.value == 3 * 4 + 4  # padded words
    assert status(QuantScheme().per_block((2, 2, 32)), (4, 64)) == _lib.ERR_SHAPE      # block rank > rank
    bad = QuantScheme().to_c()
    bad.store = 9
    assert status(bad, (4, 64)) == _lib.ERR_UNSUPPORTED_SCHEME
    bad = QuantScheme().to_c()
    bad.level = 5
    assert status(bad, (4, 64)) == _lib.ERR_UNSUPPORTED_SCHEME
    bad = QuantScheme().to_c()
    bad.tensor_scale = 1                                   # a per-tensor scale on top of ... a per-tensor scale
    assert status(bad, (4, 64)) == _lib.ERR_UNSUPPORTED_SCHEME


def test_scheme_supported_follows_the_reference_quantizable_rule():
    """bq_scheme_supported on the cases of the reference's own test of `quantizable`
    (crates/burn-std/src/tensor/quantization.rs:713-744), and on what this library does not store."""
    from burn_amd.quantization import QuantStore, QuantValue
    base = QuantScheme()
    assert base.supported() and base.with_value(QuantValue.Q8F).supported()
    assert base.per_block((4,), ScaleDtype.F16).supported()
    assert base.per_block((4,), ScaleDtype.UE4M3).per_tensor(ScaleDtype.F32).supported()
    assert base.per_block((4,), ScaleDtype.F16).per_tensor(ScaleDtype.F32).supported()
    # block scales reaching f32's range leave the per-tensor scale subnormal
    assert not base.per_block((4,), ScaleDtype.F32).per_tensor(ScaleDtype.F32).supported()
    assert not base.per_block((4,), ScaleDtype.BF16).per_tensor(ScaleDtype.F32).supported()
    assert b"cannot absorb" in _lib.lib().bq_last_error()
    with pytest.raises(ValueError):          # a per-tensor scale narrower than f32 (refused where the scheme is built)
        base.per_block((4,), ScaleDtype.UE4M3).per_tensor(ScaleDtype.BF16)
    # every value, packed or native (one i8 per value); rectangle blocks; unknown codes
    for v in QuantValue:
        assert QuantScheme(value=v).supported() and QuantScheme(value=v).per_block((2, 32)).supported()
        assert QuantScheme(value=v, store=QuantStore.Native).supported()
    c = base.to_c()
    c.value = 9
    assert _lib.lib().bq_scheme_supported(C.byref(c)) == _lib.ERR_UNSUPPORTED_SCHEME
    c = base.to_c()
    c.scale_dtype = 7                        # (a dtype without a round-up rule, like ue8m0 there)
    assert _lib.lib().bq_scheme_supported(C.byref(c)) == _lib.ERR_UNSUPPORTED_SCHEME


def test_shapes_whose_sizes_would_overflow_are_refused():
    """Element and byte counts are products of caller-supplied dims: a shape past 2^44 elements is
    refused before anything is multiplied (no wrapped-around allocation size)."""
    L = _lib.lib()
    n = C.c_size_t(0)
    sch = QuantScheme().to_c()
    for dims in ((1 << 33, 1 << 33), (1 << 62, 4), (3, 1 << 45)):
        shape = (C.c_size_t * len(dims))(*dims)
        assert L.bq_quantized_data_len(C.byref(sch), shape, len(dims), C.byref(n)) == _lib.ERR_SIZE
        assert b"not addressable" in L.bq_last_error()
    shape = (C.c_size_t * 2)(1 << 20, 1 << 20)   # 2^40 values: a length, not an allocation
    assert L.bq_quantized_data_len(C.byref(sch), shape, 2, C.byref(n)) == _lib.OK and n.value == (1 << 40) + 4


def test_static_scratch_entry_point_refuses_large_products_without_a_gpu():
    """bqk_q_linear_static checks the scratch it would need against the static array before
    anything else happens."""
    L = _lib.lib()
    buf = np.zeros(64, np.float32)
    p = buf.ctypes.data
    buf16 = np.zeros(64 + 4, np.float32)
    p = (buf16.ctypes.data + 15) & ~15   # the entry points check 16-byte alignment first
    need = L.bqk_q_matmul_workspace(128, 4096, 14336, _lib.F32, _lib.Q4S)
    assert need > _lib.STATIC_SCRATCH_BYTES
    rc = L.bqk_q_linear_static(p, _lib.F32, 128, 4096, 14336, p, p, 32, _lib.Q4S, _lib.STORE_PACKED_U32, None,
                               _lib.F32, p, None)
    assert rc == _lib.ERR_SIZE and b"static array holds" in L.bq_last_error(), L.bq_last_error()


def test_block_cache_rules(tmp_path):
    """The allocation cache's graph-capture bookkeeping (which released block may be reused
    when) is plain C++ with no HIP call: compiled and run on the CPU."""
    import subprocess
    exe = tmp_path / "test_block_cache"
    src = os.path.join(ROOT, "tests", "cpp", "test_block_cache.cpp")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "burn_amd", "csrc"), src,
                    "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert "block cache: ok" in out


def c_driver():
    """The plain-C caller of the ABI (tests/cpp/c_abi_driver.c), built by __graft_entry__.build()."""
    exe = os.path.join(ROOT, "tests", "cpp", "c_abi_driver")
    if not os.path.exists(exe):
        import __graft_entry__
        __graft_entry__.build_c_driver()
    return exe


def test_header_is_plain_c_and_a_c_caller_links():
    """include/burnq.h compiles as C99 and as C++11, and a C program linked against the library
    gets the reference's packed-Q4 blob lengths and the ABI's refusals without a GPU."""
    import subprocess
    hdr = os.path.join(ROOT, "include", "burnq.h")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c", hdr], check=True)
    subprocess.run(["g++", "-std=c++11", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", hdr], check=True)
    out = subprocess.run([c_driver(), "--no-gpu"], check=True, capture_output=True, text=True).stdout
    assert "host-only cases ok" in out


@pytest.mark.gpu
def test_c_caller_runs_the_reference_cases_on_the_gpu():
    """The same C program on the GPU: the reference's quantize / dequantize / pack / q_matmul
    literals through the handle level of the ABI, no Python in between."""
    import subprocess
    r = subprocess.run([c_driver()], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "all cases ok" in r.stdout, r.stdout + r.stderr


def test_no_cpu_fallback():
    if ba.Device.count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(ba.BurnqError, match="no CPU path"):
        ba.Device(0)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "burn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"


def test_isa_check_flags_an_unwaited_load(tmp_path):
    """The build-time scan of the prefill GEMM (burn_amd/isa_check.py): a register that an
    outstanding load will write must not be read before an s_waitcnt vmcnt covers the load."""
    from burn_amd import isa_check
    head = "_ZN2bq12_GLOBAL__N_112qgemm_kernelILi8ELi256ELb0ELb0EEEvPKt:\n"
    loop = ".LBB0_1:  ; =>This Inner Loop Header: Depth=1\n"
    tail = "\ts_cbranch_scc1 .LBB0_1\n\ts_endpgm\n"
    good = head + "\tbuffer_load_dword v5, v1, s[0:3], 0 offen\n" + loop + \
        "\ts_waitcnt vmcnt(0)\n\tv_add_u32_e32 v6, v5, v5\n\tbuffer_load_dword v5, v1, s[0:3], 0 offen\n" + tail
    bad = head + "\tbuffer_load_dword v5, v1, s[0:3], 0 offen\n" + loop + \
        "\tv_add_u32_e32 v6, v5, v5\n\ts_waitcnt vmcnt(0)\n\tbuffer_load_dword v5, v1, s[0:3], 0 offen\n" + tail
    younger = head + "\tbuffer_load_dword v5, v1, s[0:3], 0 offen\n\tbuffer_load_dword v7, v1, s[0:3], 0 offen\n" + loop + \
        "\ts_waitcnt vmcnt(1)\n\tv_add_u32_e32 v6, v5, v5\n\tv_mov_b32_e32 v8, v7\n\ts_waitcnt vmcnt(0)\n" + tail
    # an accumulator read before its matrix instruction has drained (inline-asm MFMAs are invisible
    # to the compiler's own hazard recognizer)
    mfma = "\tv_mfma_f32_32x32x16_bf16 a[0:15], v[2:5], v[6:9], a[0:15]\n"
    drained = head + loop + mfma + "\ts_nop 15\n\ts_nop 15\n" + tail.replace("\ts_endpgm", "\tv_accvgpr_read_b32 v1, a3\n\ts_endpgm")
    early = head + loop + mfma + "\ts_nop 3\n" + tail.replace("\ts_endpgm", "\tv_accvgpr_read_b32 v1, a3\n\ts_endpgm")
    for name, text, findings in (("good", good, 0), ("bad", bad, 3), ("younger", younger, 1), ("drained", drained, 0),
                                 ("early", early, 1)):
        path = tmp_path / f"{name}.s"
        path.write_text(text)
        report = isa_check.check_listing(str(path))
        (hazards, _), = report.values()
        assert len(hazards) == findings, (name, hazards)
