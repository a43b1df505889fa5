"""GGUF container reader (CPU): files written by the numpy writer are parsed by the library's reader; names, shapes,
types, offsets, bytes and metadata must come back exactly, and malformed files must be refused with a message.
The layout checked is the published GGUF one the reference's parser reads (src/gguf.hpp:394-470): v2/v3 header with
u64 counts, typed key/values including arrays, tensor directory, data section at the next multiple of general.alignment."""
import os
import struct

import numpy as np
import pytest

from warpdecode_amd import capi, ggufio, synth

META = [("general.architecture", ggufio.STRING, "qwen38"), ("qwen38.block_count", ggufio.U32, 2),
        ("qwen38.expert_count", ggufio.U64, 16), ("t.i8", ggufio.I8, -5), ("t.u8", ggufio.U8, 200),
        ("t.i16", ggufio.I16, -300), ("t.u16", ggufio.U16, 60000), ("t.i32", ggufio.I32, -70000),
        ("t.f32", ggufio.F32, 1.5), ("t.f64", ggufio.F64, -2.25), ("t.i64", ggufio.I64, -(1 << 40)),
        ("t.bool", ggufio.BOOL, 1), ("qwen38.expert_weights_scale", ggufio.F32, 2.5),
        ("tok.list", ggufio.ARRAY, (ggufio.STRING, ["a", "bc", "", "def"])),
        ("tok.scores", ggufio.ARRAY, (ggufio.F32, [0.5, -1.0, 3.0])),
        ("tok.types", ggufio.ARRAY, (ggufio.I32, [1, 2, 3, 4, 5]))]


def small_layers():
    return [synth.make_layer(256, 64, 16, 4, synth.IQ3_S, synth.Q8_0, shared=True, layer=l) for l in range(2)]


@pytest.mark.parametrize("alignment,version", [(32, 3), (64, 2), (4096, 3)])
def test_round_trip(tmp_path, alignment, version):
    layers = small_layers()
    tensors = sum((ggufio.layer_tensors(L, l) for l, L in enumerate(layers)), [])
    tensors.append(("odd.f16", [7, 3], capi.F16, np.arange(21, dtype=np.float16)))
    path = tmp_path / "m.gguf"
    data_offset = ggufio.write_gguf(path, tensors, META, alignment=alignment, version=version)
    with ggufio.GgufFile(path) as g:
        assert g.version == version
        assert g.data_offset == data_offset and data_offset % alignment == 0
        assert list(g.tensors) == [t[0] for t in tensors]  # directory order kept
        at = 0
        for name, dims, ttype, data in tensors:
            t = g.tensors[name]
            assert t["dims"] == dims and t["type"] == ttype
            assert t["relative_offset"] == at and at % alignment == 0
            assert t["bytes"] == data.nbytes
            assert np.array_equal(g.bytes_of(name), np.ascontiguousarray(data).view(np.uint8).reshape(-1))
            at += data.nbytes + (-data.nbytes) % alignment
        assert g.string("general.architecture") == "qwen38"
        assert g.string("missing") is None and g.number("missing") is None
        assert g.number("general.architecture") is None  # a string is not a number
        for key, vtype, v in META:
            if vtype not in (ggufio.STRING, ggufio.ARRAY):
                assert g.number(key) == v, key
        assert g.array("tok.list") == 4
        assert np.array_equal(g.array("tok.scores"), np.float32([0.5, -1.0, 3.0]))
        assert np.array_equal(g.array("tok.types"), np.int32([1, 2, 3, 4, 5]))
        assert g.array("t.f32") is None
        lib = capi.load()
        assert lib.wd_gguf_find(g.h, b"blk.1.ffn_down_exps.weight") == 8 + 3
        assert lib.wd_gguf_find(g.h, b"nope") == -1
        assert lib.wd_gguf_tensor(g.h, 99, None) == -1


def test_empty_directory(tmp_path):
    path = tmp_path / "e.gguf"
    ggufio.write_gguf(path, [], [("k", ggufio.U32, 1)])
    with ggufio.GgufFile(path) as g:
        assert g.tensors == {} and g.number("k") == 1


def _open_fails(path, fragment):
    import ctypes as C
    h = C.c_void_p()
    lib = capi.load()
    assert lib.wd_gguf_open(C.byref(h), str(path).encode()) == -1
    assert not h.value
    assert fragment in lib.wd_last_error().decode(), lib.wd_last_error()


def test_malformed_files_are_refused(tmp_path):
    L = small_layers()[0]
    good = tmp_path / "g.gguf"
    ggufio.write_gguf(good, ggufio.layer_tensors(L, 0), META)
    raw = good.read_bytes()
    p = tmp_path / "bad.gguf"

    _open_fails(tmp_path / "absent.gguf", "cannot open")
    p.write_bytes(b"GGML" + raw[4:])
    _open_fails(p, "magic")
    p.write_bytes(raw[:4] + struct.pack("<I", 1) + raw[8:])
    _open_fails(p, "version")
    p.write_bytes(raw[:4] + struct.pack("<I", 4) + raw[8:])
    _open_fails(p, "version")
    p.write_bytes(raw[:10])
    _open_fails(p, "header size")
    p.write_bytes(raw[:200])
    _open_fails(p, "past the end")
    p.write_bytes(raw[:len(raw) - 4096])       # data section cut short: the last tensor no longer fits
    _open_fails(p, "outside the file")
    p.write_bytes(raw[:16] + struct.pack("<Q", 1 << 40) + raw[24:])   # absurd key/value count
    _open_fails(p, "implausible")
    # a key/value of type 13 (undefined)
    bad_kv = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 13) + b"\0" * 64
    p.write_bytes(bad_kv)
    _open_fails(p, "unknown type")
    # alignment that is not a power of two
    ggufio.write_gguf(p, [], [], alignment=48)
    _open_fails(p, "power of two")
    # a tensor with five dimensions
    five = struct.pack("<IIQQ", 0x46554747, 3, 1, 0) + struct.pack("<Q", 1) + b"t" + struct.pack("<I", 5) + b"\0" * 128
    p.write_bytes(five)
    _open_fails(p, "dimensions")


    # dimensions whose product wraps around 64 bits (2^32 x 2^32 x 2 F32 elements would read as 0 bytes)
    wrap = (struct.pack("<IIQQ", 0x46554747, 3, 1, 0) + struct.pack("<Q", 1) + b"t" + struct.pack("<I", 3) +
            struct.pack("<QQQ", 1 << 32, 1 << 32, 2) + struct.pack("<IQ", 0, 0))
    p.write_bytes(wrap + b"\0" * 64)
    _open_fails(p, "does not fit 64 bits")


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gguf")


def test_reference_fixtures_read_as_the_reference_tests_expect():
    """The two GGUF files the reference ships for its parser tests (copied as data), with the answers those tests check:
    tests/gguf_parser_test.cpp:6-8 prints version, tensor count and data offset of tests/min.gguf - 3, 1 and 160 (the
    header ends at byte 134, general.alignment is 32; the file's 16 data bytes are the floats 1..4);
    tests/gguf_array_test.cpp:11-27 asserts the arrays of the first shard of tests/qwen38-fixture (written by
    tests/make_qwen38_fixture.py: no tensors, 2400 bytes of header)."""
    with ggufio.GgufFile(os.path.join(GOLDEN, "min.gguf")) as g:
        assert (g.version, len(g.tensors), g.data_offset) == (3, 1, 160)
        assert g.string("general.architecture") == "llama" and g.number("general.alignment") == 32
        t = g.tensors["vec"]
        assert t["dims"] == [4] and t["type"] == 0 and t["relative_offset"] == 0 and t["bytes"] == 16
        assert g.bytes_of("vec").view(np.float32).tolist() == [1.0, 2.0, 3.0, 4.0]
    with ggufio.GgufFile(os.path.join(GOLDEN, "qwen38-fixture-00001-of-00002.gguf")) as g:
        assert (g.version, len(g.tensors), g.data_offset) == (3, 0, 2400)
        ratios = g.array("qwen4exp.attention.compress_ratios")
        assert ratios.dtype == np.int32 and len(ratios) == 49 and ratios[3] == 8 and ratios[48] == 0
        assert ratios.tolist() == [0, 0, 0, 8] * 12 + [0]
        assert g.array("qwen4exp.ple.layers").tolist() == [0]
        mult = g.array("qwen4exp.ple.layer_multipliers")
        assert mult.dtype == np.uint64 and mult.tolist() == [3, 5, 7]
        offsets, sizes = g.array("qwen4exp.ple.head_offsets"), g.array("qwen4exp.ple.head_vocab_sizes")
        assert len(offsets) == 16 and len(sizes) == 16 and offsets[-1] == 150 and sizes[-1] == 10
        assert g.array("qwen4exp.rope.dimension_sections").tolist() == [11, 11, 10, 0]
        assert g.number("qwen4exp.expert_weights_scale") == 1.25 and g.number("qwen4exp.hyper_connection.count") == 4
        assert g.number("qwen4exp.ple.eos_token_id") == 248044 and g.array("qwen4exp.absent") is None


def test_block_sizes_as_the_reference_test_lists_them():
    """tests/gguf_type_size_test.cpp:17-25 (the types this library computes with; F16 and BF16 are 2 bytes a value)."""
    lib = capi.load()
    for gtype, n, want in [(capi.Q4_0, 32, 18), (capi.Q8_0, 32, 34), (capi.Q6_K, 256, 210), (capi.IQ4_NL, 32, 18),
                           (capi.IQ3_S, 256, 110), (capi.IQ2_S, 256, 82)]:
        assert lib.wd_row_bytes(gtype, n) == want, gtype


def test_float_tensor_sizes(tmp_path):
    """F32 32 values = 128 bytes, F16 and BF16 32 values = 64 bytes (tests/gguf_type_size_test.cpp:17-19), as the
    reader sizes tensors of those types in a directory."""
    path = tmp_path / "f.gguf"
    ggufio.write_gguf(path, [("a", [32], 0, np.zeros(128, np.uint8)), ("b", [32], 1, np.zeros(64, np.uint8)),
                             ("c", [32], 30, np.zeros(64, np.uint8))])
    with ggufio.GgufFile(path) as g:
        assert [g.tensors[n]["bytes"] for n in "abc"] == [128, 64, 64]


def test_unknown_tensor_type_is_listed_without_size(tmp_path):
    path = tmp_path / "q6.gguf"
    ggufio.write_gguf(path, [("output.weight", [256, 4], 12, np.zeros(4 * 144, np.uint8)),   # Q4_K: not computed here
                             ("x", [32], capi.Q8_0, np.zeros(34, np.uint8))])
    with ggufio.GgufFile(path) as g:
        assert g.tensors["output.weight"]["bytes"] == 0 and g.tensors["output.weight"]["type"] == 12
        assert g.tensors["x"]["bytes"] == 34


def test_file_mapping_lookup(tmp_path):
    """wd_file_mapping_of finds a memory-mapped file (path, extent, file offset of the mapping's start) and refuses
    anonymous memory; a mapping that starts inside the file reports its offset."""
    import ctypes as C
    import mmap
    path = tmp_path / "blob.bin"
    payload = np.arange(3 * 65536, dtype=np.uint8).tobytes()
    path.write_bytes(payload)
    lib = capi.load()
    with open(path, "rb") as fh:
        for offset in (0, 65536):
            mm = mmap.mmap(fh.fileno(), len(payload) - offset, prot=mmap.PROT_READ, offset=offset)
            view = np.frombuffer(mm, dtype=np.uint8)
            addr = view.ctypes.data
            m = capi.FileMapping()
            assert lib.wd_file_mapping_of(C.c_void_p(addr + 1000), C.byref(m)) == 0
            assert os.path.realpath(m.path.decode()) == os.path.realpath(str(path))
            assert m.start <= addr and m.end >= addr + len(payload) - offset
            assert m.file_offset + (addr - m.start) == offset
            del view
            mm.close()
    anon = np.zeros(1 << 20, np.uint8)
    m = capi.FileMapping()
    assert lib.wd_file_mapping_of(C.c_void_p(anon.ctypes.data), C.byref(m)) == -1
    assert b"no readable file mapping" in lib.wd_last_error()
