"""CPU tests of the GGUF reader (oxh_gguf_*): the reference's own fixtures and
the expectations its tests hold for them (oxidize-c/tests/test_gguf.c:50-160,
fixtures oxidize-core/tests/fixtures/*.gguf, copied as data under
tests/golden/gguf/), every metadata value type, the weight-view rules of
oxidize-c/src/model/llama.c:108-127, and malformed input: truncated at every
byte, oversized counts and strings, bad alignment, tensors past the end."""
import os
import struct

import numpy as np
import pytest

import gguf_writer as gw
from oxidize_amd import _lib
from oxidize_amd import synth
from oxidize_amd.gguf import GgufFile

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gguf")


def write(tmp_path, data, name="m.gguf"):
    p = tmp_path / name
    p.write_bytes(data)
    return p


def status_of(path):
    try:
        GgufFile(path).close()
        return 0
    except _lib.OxhError as e:
        return e.status


def test_reference_fixture_valid_v3():
    with GgufFile(os.path.join(FIX, "valid-v3.gguf")) as g:
        assert (g.version, g.n_tensors, g.n_metadata) == (3, 1, 1)
        assert g.alignment == 64 and g.data_start == 128
        assert g.meta_u64("general.alignment") == 64
        t = g.tensor_at(0)
        assert t.name == b"tok_embeddings.weight"
        assert t.n_dims == 2 and list(t.dims[:2]) == [8, 4]
        assert t.ggml_type == 0 and t.qtype == 0 and t.offset == 0
        assert (t.rows, t.cols, t.row_bytes, t.nbytes) == (4, 8, 32, 128)
        # the data section starts with bytes 1, 2, 3, 4
        assert bytes((ctypes_bytes(t.data, 4))) == b"\x01\x02\x03\x04"
        assert g.find("tok_embeddings.weight").offset == 0 and g.find("nope") is None


def ctypes_bytes(addr, n):
    import ctypes
    return ctypes.string_at(addr, n)


@pytest.mark.parametrize("name", ["invalid-magic.gguf", "unsupported-version.gguf", "invalid-alignment.gguf"])
def test_reference_fixtures_rejected(name):
    assert status_of(os.path.join(FIX, name)) == _lib.ERR_FORMAT


def test_version_2_parses_like_version_3(tmp_path):
    raw = bytearray(open(os.path.join(FIX, "valid-v3.gguf"), "rb").read())
    raw[4] = 2
    with GgufFile(write(tmp_path, bytes(raw))) as g:
        assert g.version == 2 and g.alignment == 64 and g.data_start == 128
        assert g.tensor_at(0).name == b"tok_embeddings.weight"
    raw[4] = 1
    assert status_of(write(tmp_path, bytes(raw))) == _lib.ERR_FORMAT


def test_missing_file_is_an_io_error(tmp_path):
    assert status_of(tmp_path / "absent.gguf") == _lib.ERR_IO


def test_every_metadata_value_type(tmp_path):
    meta = [("k.u8", gw.U8, 200), ("k.i8", gw.I8, -50), ("k.u16", gw.U16, 50000), ("k.i16", gw.I16, -20000),
            ("k.u32", gw.U32, 4000000000), ("k.i32", gw.I32, -2000000000), ("k.f32", gw.F32, 1.5),
            ("k.bool", gw.BOOL, 1), ("k.str", gw.STRING, b"hello\0world"),
            ("k.arr", gw.ARRAY, (gw.U32, [1, 2, 3])), ("k.u64", gw.U64, 1 << 40), ("k.i64", gw.I64, -(1 << 40)),
            ("k.f64", gw.F64, 2.25), ("k.strs", gw.ARRAY, (gw.STRING, ["a", "bc", ""])),
            ("k.nest", gw.ARRAY, (gw.ARRAY, [(gw.U8, [1, 2]), (gw.U8, [])]))]
    with GgufFile(write(tmp_path, gw.build(meta, []))) as g:
        assert g.n_metadata == len(meta) and g.n_tensors == 0 and g.alignment == 32
        assert g.meta_u64("k.u8") == 200 and g.meta_u64("k.u16") == 50000 and g.meta_u64("k.u32") == 4000000000
        assert g.meta_u64("k.u64") == 1 << 40 and g.meta_u64("k.bool") == 1
        assert g.meta_u64("k.i8") is None and g.meta_u64("k.i64") is None      # negative: not a u64
        assert g.meta_f64("k.f32") == 1.5 and g.meta_f64("k.f64") == 2.25 and g.meta_f64("k.u8") is None
        assert g.meta_str("k.str") == b"hello\0world" and g.meta_str("k.u8") is None
        assert g.meta_u64("absent") is None


def model_file(alignment=None):
    """A small file shaped like a model: quantized matrices of every type the
    library runs, an f32 norm vector and a stacked expert tensor."""
    tensors = []
    for name, qt, ggml, rows, cols in (("blk.0.attn_q.weight", 13, 12, 48, 512), ("blk.0.ffn_down.weight", 16, 14, 24, 768),
                                       ("output.weight", 7, 8, 40, 96), ("blk.0.attn_v.weight", 15, 13, 9, 256)):
        tensors.append((name, [cols, rows], ggml, gw.as_bytes(synth.weights(qt, rows, cols, seed=3, stream=ggml))))
    tensors.append(("blk.0.attn_norm.weight", [512], 0, gw.as_bytes(synth.normal(512, seed=3))))
    tensors.append(("blk.0.ffn_gate_exps.weight", [256, 16, 4], 12,
                    gw.as_bytes(synth.weights(13, 64, 256, seed=4))))
    meta = [("general.architecture", gw.STRING, "llama"), ("llama.embedding_length", gw.U32, 512),
            ("llama.attention.layer_norm_rms_epsilon", gw.F32, 1e-5)]
    return gw.build(meta, tensors, alignment=alignment), tensors


@pytest.mark.parametrize("alignment", [None, 64, 4096])
def test_tensor_views_follow_the_reference_rules(tmp_path, alignment):
    data, tensors = model_file(alignment)
    with GgufFile(write(tmp_path, data)) as g:
        assert g.alignment == (alignment or 32) and g.data_start % g.alignment == 0
        assert g.meta_str("general.architecture") == b"llama" and g.meta_u64("llama.embedding_length") == 512
        assert abs(g.meta_f64("llama.attention.layer_norm_rms_epsilon") - 1e-5) < 1e-12
        want = {"blk.0.attn_q.weight": (13, 48, 512, 288), "blk.0.ffn_down.weight": (16, 24, 768, 630),
                "output.weight": (7, 40, 96, 102), "blk.0.attn_v.weight": (15, 9, 256, 176),
                "blk.0.attn_norm.weight": (0, 1, 512, 2048), "blk.0.ffn_gate_exps.weight": (13, 64, 256, 144)}
        for (name, dims, ggml, payload), t in zip(tensors, g.tensors()):
            assert t.name.decode() == name and t.ggml_type == ggml and t.offset % g.alignment == 0
            assert (t.qtype, t.rows, t.cols, t.row_bytes) == want[name]
            assert t.nbytes == len(payload) == t.rows * t.row_bytes
            assert ctypes_bytes(t.data, t.nbytes) == payload
            assert t.resident == 0


def test_on_disk_type_ids_map_like_the_reference():
    # oxidize-c/src/compute/quantization.c:2925-2988
    lib = _lib.lib()
    table = {0: 0, 1: 1, 30: 2, 2: 3, 3: 4, 6: 5, 7: 6, 8: 7, 10: 8, 11: 9, 12: 13, 13: 15, 14: 16,
             24: 31, 25: 32, 26: 33, 27: 34, 28: 35,
             21: 25, 66: 36, 20: 26, 23: 27,               # IQ3_S, IQ1_XXXS, IQ4_NL, IQ4_XS (:2949-2958)
             240: 17, 241: 20, 242: 19, 243: 18}           # AL family (quantization.c:2943-2947)
    for ggml, q in table.items():
        assert lib.oxh_qtype_from_ggml_id(ggml) == q
    for ggml in (4, 5, 9, 15, 99, 1000):
        assert lib.oxh_qtype_from_ggml_id(ggml) == 0xFFFFFFFF


def test_truncated_at_every_byte_never_crashes(tmp_path):
    data, _ = model_file()
    # every prefix of the header, and a sample of prefixes of the data section
    with GgufFile(write(tmp_path, data)) as g:
        start = g.data_start
    cuts = list(range(0, start + 1)) + list(range(start + 1, len(data), 977))
    for n in cuts:
        st = status_of(write(tmp_path, data[:n], "cut.gguf")) if n else None
        if n == 0:
            (tmp_path / "cut.gguf").write_bytes(b"")
            st = status_of(tmp_path / "cut.gguf")
        assert st == _lib.ERR_FORMAT, "prefix of %d bytes gave %r" % (n, st)
    assert status_of(write(tmp_path, data)) == 0


def test_malformed_tables_are_format_errors(tmp_path):
    hdr = struct.pack("<II", 0x46554747, 3)

    def bad(body):
        return status_of(write(tmp_path, hdr + body + b"\0" * 64, "bad.gguf"))

    assert bad(struct.pack("<QQ", 1 << 40, 0)) == _lib.ERR_FORMAT                      # absurd tensor count
    assert bad(struct.pack("<QQ", 0, 1 << 40)) == _lib.ERR_FORMAT                      # absurd metadata count
    assert bad(struct.pack("<QQ", 0, 1) + struct.pack("<Q", 1 << 30) + b"k") == _lib.ERR_FORMAT   # key longer than the file
    assert bad(struct.pack("<QQ", 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 13)) == _lib.ERR_FORMAT
    assert bad(struct.pack("<QQ", 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 4, 1 << 50)) \
        == _lib.ERR_FORMAT                                                               # array longer than the file
    # nine dimensions
    t9 = struct.pack("<QQ", 1, 0) + struct.pack("<Q", 1) + b"t" + struct.pack("<I", 9) + b"\0" * 72
    assert bad(t9) == _lib.ERR_FORMAT
    for align_type, align in ((gw.U32, 3), (gw.U32, 0), (gw.I32, -32), (gw.F32, 32.0), (gw.STRING, "32")):
        data = gw.build([("general.alignment", align_type, align)], [])
        assert status_of(write(tmp_path, data, "al.gguf")) == _lib.ERR_FORMAT
    ok = gw.build([("general.alignment", gw.I64, 128)], [], pad_to=128)
    assert status_of(write(tmp_path, ok, "al.gguf")) == 0
    assert status_of(write(tmp_path, ok[:127], "al.gguf")) == _lib.ERR_FORMAT   # data section would start past the end
    # a tensor whose declared extent runs past the end, and one that starts past it
    w = gw.as_bytes(synth.weights(13, 4, 256, seed=1))
    ok = gw.build([], [("w", [256, 4], 12, w)])
    assert status_of(write(tmp_path, ok, "t.gguf")) == 0
    assert status_of(write(tmp_path, ok[:-1], "t.gguf")) == _lib.ERR_FORMAT
    grown = gw.build([], [("w", [256, 5], 12, w)])
    assert status_of(write(tmp_path, grown, "t.gguf")) == _lib.ERR_FORMAT
    far = bytearray(ok)
    pos = ok.index(struct.pack("<I", 12), 24) + 4          # the tensor's offset field
    far[pos:pos + 8] = struct.pack("<Q", 1 << 40)
    assert status_of(write(tmp_path, bytes(far), "t.gguf")) == _lib.ERR_FORMAT
    huge = gw.build([], [("w", [1 << 40, 1 << 40], 12, b"")])
    assert status_of(write(tmp_path, huge, "t.gguf")) == _lib.ERR_FORMAT
    # a width that is not whole blocks has no fixed extent: the table is accepted, the view says so
    with GgufFile(write(tmp_path, gw.build([], [("odd", [100, 2], 12, b"\0" * 144)]), "t.gguf")) as g:
        t = g.tensor_at(0)
        assert (t.nbytes, t.row_bytes, t.rows, t.cols) == (0, 0, 2, 100)


def test_register_all_needs_a_device(tmp_path):
    data, _ = model_file()
    if _lib.lib().oxh_init(0) == 0:
        pytest.skip("a GPU is present: covered by the GPU test")
    with GgufFile(write(tmp_path, data)) as g:
        with pytest.raises(_lib.OxhError) as e:
            g.register_all()
        assert e.value.status == _lib.ERR_NO_DEVICE
