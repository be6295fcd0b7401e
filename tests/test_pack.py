"""burnpack containers (crates/burn-pack): the format rules the reference's own tests hold --
header constants and round trip (tests/header.rs), data-section alignment (tests/alignment.rs),
reader rejections (tests/errors.rs) -- checked on the CPU against containers assembled by hand
here, and the packed-Q4 byte lengths of crates/burn-store/src/tensor_snapshot.rs:517-541. The
GPU round trip (device tensor -> file -> device tensor) is in test_gpu_parity.py."""
import os
import struct
import subprocess

import numpy as np
import pytest

import burn_amd as ba
from burn_amd import PackReader, PackWriter, QuantScheme, QuantStore, QuantValue, _lib


# ---- a minimal CBOR encoder, independent of the library's (RFC 8949: shortest-form heads) -------
def _head(major, v):
    if v < 24:
        return bytes([major << 5 | v])
    for info, fmt, lim in ((24, ">B", 1 << 8), (25, ">H", 1 << 16), (26, ">I", 1 << 32), (27, ">Q", 1 << 64)):
        if v < lim:
            return bytes([major << 5 | info]) + struct.pack(fmt, v)
    raise ValueError(v)


def cbor(o):
    if isinstance(o, bool):
        return bytes([0xF5 if o else 0xF4])
    if isinstance(o, int):
        return _head(0, o)
    if isinstance(o, str):
        b = o.encode()
        return _head(3, len(b)) + b
    if isinstance(o, (list, tuple)):
        return _head(4, len(o)) + b"".join(cbor(i) for i in o)
    if isinstance(o, dict):
        return _head(5, len(o)) + b"".join(cbor(k) + cbor(v) for k, v in o.items())
    raise TypeError(type(o))


def container(tensors, metadata=None, version=1, magic=0x4255524E):
    """tensors: list of (name, dtype, shape, bytes) laid out in the given order, 256-byte aligned."""
    desc, cur, chunks = {}, 0, []
    for name, dtype, shape, data in tensors:
        begin = (cur + 255) // 256 * 256
        desc[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [begin, begin + len(data)]}
        chunks.append((begin, data))
        cur = begin + len(data)
    meta = {"tensors": dict(sorted(desc.items()))}
    if metadata:
        meta["metadata"] = dict(sorted(metadata.items()))
    m = cbor(meta)
    start = (10 + len(m) + 255) // 256 * 256
    out = bytearray(start + cur)
    out[:10] = struct.pack("<IHI", magic, version, len(m))
    out[10:10 + len(m)] = m
    for begin, data in chunks:
        out[start + begin:start + begin + len(data)] = data
    return bytes(out)


def test_header_constants_and_alignment():
    """tests/header.rs `header_constants`, tests/alignment.rs `data_section_start_is_aligned`."""
    assert struct.pack("<I", 0x4255524E) == b"NRUB"
    L = _lib.lib()
    for metadata_size in (0, 1, 10, 245, 246, 247, 4096):
        start = L.bq_pack_data_section_start(metadata_size)
        assert start % 256 == 0 and 10 + metadata_size <= start < 10 + metadata_size + 256
    assert L.bq_pack_data_section_start(246) == 256 and L.bq_pack_data_section_start(247) == 512


def test_reader_parses_a_hand_assembled_container():
    a = np.float32([1, 2, 3]).tobytes()
    b = np.float32([4]).tobytes()
    raw = container([("b", "F32", (1,), b), ("a", "F32", (3,), a)], {"producer": "by hand"})
    r = PackReader(raw)
    assert len(r) == 2
    ea, eb = r.entries()                              # name order, whatever the layout order
    assert (ea["name"], ea["dtype"], ea["shape"]) == ("a", "F32", (3,))
    assert eb["data_offsets"] == (0, 4) and ea["data_offsets"] == (256, 268)   # each tensor on a 256-byte boundary
    assert r.metadata("producer") == "by hand" and r.metadata("missing") is None
    import ctypes as C
    assert C.string_at(ea["data_ptr"], 12) == a and C.string_at(eb["data_ptr"], 4) == b
    with pytest.raises(ba.BurnqError, match="TensorNotFound"):
        r.find("c")


def test_reader_rejections():
    """tests/header.rs / tests/errors.rs: bad magic, short input, unknown version, a container
    smaller than its descriptors claim."""
    good = container([("w", "F32", (2,), np.float32([1, 2]).tobytes())])
    PackReader(good)
    with pytest.raises(ba.BurnqError, match="InvalidMagicNumber"):
        PackReader(container([("w", "F32", (2,), bytes(8))], magic=0xDEADBEEF))
    with pytest.raises(ba.BurnqError, match="InvalidHeader"):
        PackReader(bytes(4))
    with pytest.raises(ba.BurnqError, match="InvalidVersion"):
        PackReader(container([("w", "F32", (2,), bytes(8))], version=2))
    with pytest.raises(ba.BurnqError, match="smaller than its tensors"):
        PackReader(good[:-1])
    with pytest.raises(ba.BurnqError, match="InvalidHeader"):
        PackReader(good[:12])
    with pytest.raises(ba.BurnqError, match="MetadataDeserializationError"):
        PackReader(struct.pack("<IHI", 0x4255524E, 1, 3) + b"\xff\xff\xff" + bytes(300))


def test_writer_emits_what_the_format_prescribes():
    """The writer's bytes equal a container assembled by hand from the format rules: tensors laid
    out in insertion order at 256-byte boundaries, descriptors and user metadata in key order,
    shortest-form CBOR integers."""
    a, b = np.float32([1, 2, 3]), np.float32([4])
    w = PackWriter().with_metadata("producer", "test").add_bytes("b", "F32", (1,), b).add_bytes("a", "F32", (3,), a, param_id=42)
    raw = w.into_bytes().tobytes()
    desc_a = {"dtype": "F32", "shape": [3], "data_offsets": [256, 268], "param_id": 42}
    desc_b = {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}
    m = cbor({"tensors": {"a": desc_a, "b": desc_b}, "metadata": {"producer": "test"}})
    assert raw[:10] == struct.pack("<IHI", 0x4255524E, 1, len(m)) and raw[10:10 + len(m)] == m
    start = (10 + len(m) + 255) // 256 * 256
    assert len(raw) == w.size() == start + 268
    assert raw[10 + len(m):start] == bytes(start - 10 - len(m))          # zero padding
    assert raw[start:start + 4] == b.tobytes() and raw[start + 256:start + 268] == a.tobytes()
    # size / write_into agree (tests/alignment.rs), a buffer one byte short is refused
    import ctypes as C
    n = C.c_size_t()
    small = np.empty(len(raw) - 1, np.uint8)
    assert _lib.lib().bq_pack_writer_write_into(w.handle, small.ctypes.data, small.size, C.byref(n)) == _lib.ERR_SIZE
    # duplicate names and impossible byte lengths are refused (writer.rs:264-330)
    with pytest.raises(ba.BurnqError, match="Duplicate tensor name"):
        w.add_bytes("a", "F32", (3,), a)
    with pytest.raises(ba.BurnqError, match="TensorBytesSizeMismatch"):
        PackWriter().add_bytes("x", "F32", (4,), a)


def test_quantized_entries_carry_the_blob_length(kats):
    """A QFloat tensor's bytes in the file are its QuantizedBytes blob; its length is
    quantized_data_len (tensor_snapshot.rs:253-262). The packed-Q4 cases of tensor_snapshot.rs:517-541."""
    scheme = QuantScheme(value=QuantValue.Q4S)
    w = PackWriter()
    for i, case in enumerate(kats["packed_q4_data_len"]["cases"]):
        w.add_bytes(f"t{i}", "QFloat", case["shape"], np.zeros(case["len"], np.uint8), scheme=scheme)
        with pytest.raises(ba.BurnqError, match="TensorBytesSizeMismatch"):
            PackWriter().add_bytes("bad", "QFloat", case["shape"], np.zeros(case["len"] + 4, np.uint8), scheme=scheme)
    r = PackReader(w.into_bytes())
    for i, case in enumerate(kats["packed_q4_data_len"]["cases"]):
        e = r.find(f"t{i}")
        assert e["dtype"] == "QFloat" and e["data_offsets"][1] - e["data_offsets"][0] == case["len"]
        assert e["data_offsets"][0] % 256 == 0 and e["scheme"] == scheme
    # crates/burn-store/tests/direct_writer.rs:76-93 (quantized_snapshot_writes_and_reads_back): a [5, 5]
    # Q4S tensor as the reference's CPU backend holds it -- natively, one i8 per value: a sub-byte
    # value type and a byte count (25 + 4) that is not a multiple of the scale alignment
    s4 = QuantScheme(value=QuantValue.Q4S, store=QuantStore.Native)
    blob = np.arange(29, dtype=np.uint8)
    e = PackReader(PackWriter().add_bytes("weight", "QFloat", (5, 5), blob, scheme=s4).into_bytes()).find("weight")
    assert tuple(e["shape"]) == (5, 5) and e["scheme"] == s4 and e["data_offsets"][1] - e["data_offsets"][0] == 29
    # a block scheme with 2-byte scales survives the scheme round trip too
    s2 = QuantScheme(store=QuantStore.Native).per_block((2, 16), ba.ScaleDtype.BF16)
    w2 = PackWriter().add_bytes("q", "QFloat", (4, 32), np.zeros(4 * 32 + 2 * 4, np.uint8), scheme=s2)
    assert PackReader(w2.into_bytes()).find("q")["scheme"] == s2


# ---- a container written by the reference -------------------------------------------------------
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MNIST = os.path.join(ROOT, "tests", "golden", "mnist_model.bpk")
# examples/mnist-inference-web/src/model.rs: two ConvBlocks (Conv2d [1, 64] and [64, 64], 3 x 3, with bias, + BatchNorm) and
# three Linear layers 1600 -> 128 -> 128 -> 10, whose weights burn stores [d_input, d_output]
MNIST_SHAPES = {
    "conv1.conv.weight": (64, 1, 3, 3), "conv1.conv.bias": (64,), "conv2.conv.weight": (64, 64, 3, 3), "conv2.conv.bias": (64,),
    **{f"conv{i}.norm.{p}": (64,) for i in (1, 2) for p in ("gamma", "beta", "running_mean", "running_var")},
    "fc1.weight": (1600, 128), "fc1.bias": (128,), "fc2.weight": (128, 128), "fc2.bias": (128,), "fc3.weight": (128, 10), "fc3.bias": (10,),
}


def test_reads_a_container_written_by_the_reference():
    """tests/golden/mnist_model.bpk is examples/mnist-inference-web/model.bpk of the reference tree,
    written by burn's own BurnpackWriter: header, the 18 descriptors of that model (names, shapes,
    dtypes, parameter ids), the layout rules (data section and every tensor on a 256-byte boundary,
    tensors in file order without overlap), and sane contents."""
    raw = open(MNIST, "rb").read()
    magic, version, msize = struct.unpack("<IHI", raw[:10])
    assert (magic, version) == (0x4255524E, 1) and raw[:4] == b"NRUB"
    start = _lib.lib().bq_pack_data_section_start(msize)
    assert start % 256 == 0 and start >= 10 + msize
    for r in (PackReader(raw), PackReader(MNIST), PackReader(MNIST[:-4])):     # bytes, path, path without its extension
        entries = r.entries()
        assert len(r) == 18 and [e["name"] for e in entries] == sorted(MNIST_SHAPES)
        spans = []
        for e in entries:
            assert e["dtype"] == "F32" and tuple(e["shape"]) == MNIST_SHAPES[e["name"]] and e["scheme"] is None
            begin, end = e["data_offsets"]
            assert begin % 256 == 0 and end - begin == 4 * int(np.prod(e["shape"])) and start + end <= len(raw)
            assert e["param_id"] is not None and 0 < e["param_id"] < 2 ** 64
            spans.append((begin, end))
        assert len({e["param_id"] for e in entries}) == 18
        spans.sort()
        assert all(a_end <= b_begin for (_, a_end), (b_begin, _) in zip(spans, spans[1:]))
        assert start + spans[-1][1] == len(raw)                                # the file ends with its last tensor
    import ctypes as C
    r = PackReader(raw)
    for e in r.entries():
        begin, end = e["data_offsets"]
        data = np.frombuffer(C.string_at(e["data_ptr"], end - begin), np.float32)
        assert data.tobytes() == raw[start + begin:start + end] and np.isfinite(data).all()
        if e["name"].endswith("running_var"):
            assert (data > 0).all()
    # cutting the file anywhere inside its data section is refused (tests/errors.rs rejects_truncated_data_section)
    for cut in (len(raw) - 1, len(raw) // 2, start + 1, start):
        with pytest.raises(ba.BurnqError, match="smaller than its tensors"):
            PackReader(raw[:cut])
    for cut in (9, 10, 10 + msize - 1):
        with pytest.raises(ba.BurnqError, match="InvalidHeader"):
            PackReader(raw[:cut])


def test_reader_limits_of_the_reference():
    """crates/burn-pack/tests/errors.rs:19-66: an oversized metadata claim is refused before anything is
    allocated for it, a metadata size past the end of the input is refused, and so is a version from
    the future."""
    header = lambda version, msize: struct.pack("<IHI", 0x4255524E, version, msize)   # noqa: E731
    with pytest.raises(ba.BurnqError, match="exceeds the maximum"):
        PackReader(header(1, 100 * 1024 * 1024 + 1))
    PackReader(container([]))                                                         # an empty pack is fine (round_trip.rs empty_pack)
    with pytest.raises(ba.BurnqError, match="InvalidHeader"):
        PackReader(header(1, 4096))
    with pytest.raises(ba.BurnqError, match="InvalidVersion"):
        PackReader(header(2, 0))
    # metadata made of a million one-byte items: refused by the node budget, not by the allocator
    bomb = header(1, 8 << 20) + b"\x9a\x00\x7f\xff\xf0" + b"\x80" * ((8 << 20) - 5)
    with pytest.raises(ba.BurnqError, match="MetadataDeserializationError"):
        PackReader(bomb)


def _sanitized(tmp_path, name, sources, lang):
    exe = tmp_path / name
    cc = ["g++", "-std=c++17"] if lang == "c++" else ["gcc", "-std=c11"]
    subprocess.run(cc + ["-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer",
                         "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "burn_amd", "csrc"), "-I", os.path.join(ROOT, "oracle")]
                   + sources + ["-lm", "-o", str(exe)], check=True)
    return str(exe)


def test_container_parser_under_sanitizers_and_a_mutation_fuzz(tmp_path):
    """The parser of untrusted containers (burn_amd/csrc/pack_format.hpp) built with the address and
    undefined-behaviour sanitizers, fed 100 000 seeded mutations (bit flips, truncations, blown-up
    lengths, nests) of valid containers, the reference-written one among them: every case is answered
    with a status, and whatever is accepted describes bytes the container holds."""
    exe = _sanitized(tmp_path, "fuzz_pack", [os.path.join(ROOT, "tests", "cpp", "fuzz_pack.cpp")], "c++")
    out = subprocess.run([exe, "100000", "20250", MNIST], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-4000:]
    assert "100000 cases" in out.stdout


def test_oracle_and_block_cache_under_sanitizers(tmp_path):
    """The C oracle and the allocator's block cache are host code too: both built with the address and
    undefined-behaviour sanitizers and run over ragged shapes with exactly sized buffers."""
    exe = _sanitized(tmp_path, "oracle_sanitize", [os.path.join(ROOT, "tests", "cpp", "oracle_sanitize.c"),
                                                   os.path.join(ROOT, "oracle", "bq_oracle.c")], "c")
    out = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-4000:]
    exe = _sanitized(tmp_path, "test_block_cache", [os.path.join(ROOT, "tests", "cpp", "test_block_cache.cpp")], "c++")
    out = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-4000:]
