"""The GGUF reader (no GPU): files written by tests/gguf_writer.py are parsed back -- version, metadata of every scalar
type, strings, skipped arrays, the tensor directory, aligned tensor bytes -- and damaged files are refused with a
message instead of being read past their end (the checks of the reference's GgufFile::parse, src/gguf.h:306-360)."""
import numpy as np
import pytest

import arcinferzero_amd as az
import gguf_writer as gw
from common import make_weights


def sample(tmp_path, alignment=32, version=3, nested=True):
    rng = np.random.default_rng(5)
    W8 = make_weights(az.Q8_0, 8, 256, seed=1)
    W4 = make_weights(az.Q4_K, 4, 512, seed=2)
    W6 = make_weights(az.Q6_K, 6, 256, seed=3)
    f32 = rng.standard_normal(7).astype(np.float32)
    kv = [("general.architecture", gw.T_STR, "qwen3"), ("a.u8", gw.T_U8, 200), ("a.i8", gw.T_I8, -5),
          ("a.u16", gw.T_U16, 60000), ("a.i16", gw.T_I16, -30000), ("a.u32", gw.T_U32, 4000000000),
          ("a.i32", gw.T_I32, -2000000000), ("a.f32", gw.T_F32, 1.5), ("a.bool", gw.T_BOOL, 1),
          ("a.u64", gw.T_U64, 1 << 40), ("a.i64", gw.T_I64, -(1 << 40)), ("a.f64", gw.T_F64, 2.25),
          ("tok.list", gw.T_ARR, (gw.T_STR, ["<s>", "</s>", "hello"])), ("tok.scores", gw.T_ARR, (gw.T_F32, [0.0, 1.0, 2.0])),
          ("nested", gw.T_ARR, (gw.T_ARR, [(gw.T_I32, [1, 2]), (gw.T_I32, [3])])), ("after.arrays", gw.T_I32, 77)]
    if not nested:  # (arrays of arrays: this reader skips them, the reference's refuses the file)
        kv = [e for e in kv if e[0] != "nested"]
    tensors = [("blk.0.ffn_up.weight", az.Q4_K, [512, 4], W4), ("output.weight", az.Q6_K, [256, 6], W6),
               ("blk.0.attn_q.weight", az.Q8_0, [256, 8], W8), ("blk.0.norm.weight", 0, [7], f32.view(np.uint8))]
    p = tmp_path / "m.gguf"
    gw.write_gguf(p, kv, tensors, alignment=alignment, version=version)
    return p, tensors


@pytest.mark.parametrize("alignment,version", [(32, 3), (64, 3), (4096, 2)])
def test_reads_back(tmp_path, alignment, version):
    p, tensors = sample(tmp_path, alignment, version)
    with az.GgufFile(p) as g:
        assert g.version == version and g.n_tensors == 4 and g.alignment == alignment
        assert g.n_kv == (16 if alignment == 32 else 17)
        assert g.get_str("general.architecture") == "qwen3" and g.get_str("a.u8") is None and g.get_str("nope") is None
        assert g.get_int("a.u8") == 200 and g.get_int("a.i8") == -5 and g.get_int("a.u16") == 60000
        assert g.get_int("a.i16") == -30000 and g.get_int("a.u32") == 4000000000 and g.get_int("a.i32") == -2000000000
        assert g.get_int("a.bool") == 1 and g.get_int("a.u64") == 1 << 40 and g.get_int("a.i64") == -(1 << 40)
        assert g.get_float("a.f32") == 1.5 and g.get_float("a.f64") == 2.25 and g.get_float("a.i8") == -5.0
        assert g.get_int("a.f32") is None and g.get_int("tok.list") is None and g.get_int("after.arrays") == 77
        for i, (name, typ, dims, data) in enumerate(tensors):
            t = g.tensor(i)
            assert t["name"] == name and t["type"] == typ and t["dims"] == dims and g.find(name) == i
            assert t["nbytes"] == np.asarray(data).view(np.uint8).size
            assert np.array_equal(t["data"], np.asarray(data).view(np.uint8).ravel())
            assert t["data"].ctypes.data % alignment == 0 or alignment > 4096
        assert g.find("missing") == -1
        with pytest.raises(IndexError):
            g.tensor(4)


def test_block_info():
    import ctypes as C
    for typ, blk, nb in ((0, 1, 4), (1, 1, 2), (8, 32, 34), (12, 256, 144), (14, 256, 210), (2, 32, 18), (13, 256, 176)):
        b, n = C.c_int(), C.c_int()
        assert az.lib.arcz_ggml_block_info(typ, C.byref(b), C.byref(n)) == 1 and (b.value, n.value) == (blk, nb)
    assert az.lib.arcz_ggml_block_info(9999, None, None) == 0


def test_damaged_files_are_refused(tmp_path):
    p, _ = sample(tmp_path)
    raw = p.read_bytes()

    def refused(data, what):
        q = tmp_path / "bad.gguf"
        q.write_bytes(data)
        with pytest.raises(az.ArczError) as e:
            az.GgufFile(q)
        assert what in str(e.value), str(e.value)

    refused(b"GGML" + raw[4:], "not a GGUF file")
    refused(raw[:4] + (1).to_bytes(4, "little") + raw[8:], "version")
    refused(raw[:8] + (1 << 60).to_bytes(8, "little") + raw[16:], "count")           # a tensor count the file cannot hold
    refused(raw[:40], "count")                                                       # too short for its own counts
    refused(raw[:300], "truncated")                                                  # ends inside the metadata
    refused(raw[:len(raw) - 100], "out of range")                                    # the last tensor's bytes are cut
    with pytest.raises(az.ArczError):
        az.GgufFile(tmp_path / "does_not_exist.gguf")
    # a string length past the end of the file
    i = raw.index(b"general.architecture") + len(b"general.architecture") + 4
    refused(raw[:i] + (1 << 50).to_bytes(8, "little") + raw[i + 8:], "truncated")
    # an alignment that is no power of two
    q = tmp_path / "al.gguf"
    gw.write_gguf(q, [("general.alignment", gw.T_U32, 48)], [("t", 0, [4], np.zeros(16, np.uint8))])
    with pytest.raises(az.ArczError) as e:
        az.GgufFile(q)
    assert "alignment" in str(e.value)
    # an unknown tensor type, and a row that is no whole number of blocks
    gw.write_gguf(q, [], [("t", 777, [4], np.zeros(16, np.uint8))])
    with pytest.raises(az.ArczError) as e:
        az.GgufFile(q)
    assert "unsupported ggml type" in str(e.value)
    gw.write_gguf(q, [], [("t", az.Q4_K, [100, 2], np.zeros(144, np.uint8))])
    with pytest.raises(az.ArczError) as e:
        az.GgufFile(q)
    assert "block" in str(e.value)
