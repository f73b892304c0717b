"""The library's GGUF reader against the reference's own (GgufFile, src/gguf.h:93-361, compiled from where it lies
into oracle/_ref by oracle/Makefile): the same files -- written by tests/gguf_writer.py -- opened by both, and
everything the matmul path takes from a file compared: counts, metadata scalars and strings, every directory entry's
name, type, dimensions and byte count, where each tensor's bytes start relative to the first's, and the bytes
themselves.  Also the block sizes of every ggml type id.  Skipped where oracle/_ref is not built (no reference tree)."""
import ctypes as C

import numpy as np
import pytest

import arcinferzero_amd as az
import gguf_writer as gw
import oracle_lib as orc
from test_gguf import sample

pytestmark = pytest.mark.skipif(orc.ref is None or not hasattr(orc.ref, "ref_gguf_open"),
                                reason="oracle/_ref (the compiled reference) is not built here")


def _ref():
    r = orc.ref
    r.ref_gguf_open.restype = C.c_void_p
    r.ref_gguf_open.argtypes = [C.c_char_p]
    r.ref_gguf_close.argtypes = [C.c_void_p]
    r.ref_gguf_n_tensors.restype = C.c_int64
    r.ref_gguf_n_tensors.argtypes = [C.c_void_p]
    r.ref_gguf_n_kv.restype = C.c_int64
    r.ref_gguf_n_kv.argtypes = [C.c_void_p]
    r.ref_gguf_tensor.argtypes = [C.c_void_p, C.c_int64, C.c_char_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                  C.c_void_p, C.c_void_p]
    r.ref_gguf_find.restype = C.c_int64
    r.ref_gguf_find.argtypes = [C.c_void_p, C.c_char_p]
    r.ref_gguf_has.argtypes = [C.c_void_p, C.c_char_p]
    r.ref_gguf_get_int.restype = C.c_int64
    r.ref_gguf_get_int.argtypes = [C.c_void_p, C.c_char_p, C.c_int64]
    r.ref_gguf_get_float.restype = C.c_double
    r.ref_gguf_get_float.argtypes = [C.c_void_p, C.c_char_p, C.c_double]
    r.ref_gguf_get_str.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_int]
    r.ref_ggml_block_info.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p]
    return r


def ref_tensor(r, h, i):
    name = C.create_string_buffer(256)
    typ, nd, dims, data, nb = C.c_uint32(), C.c_uint32(), (C.c_uint64 * 8)(), C.c_void_p(), C.c_uint64()
    assert r.ref_gguf_tensor(h, i, name, 256, C.byref(typ), C.byref(nd), dims, C.byref(data), C.byref(nb)) == 0
    buf = np.frombuffer((C.c_uint8 * nb.value).from_address(data.value), np.uint8) if nb.value else np.zeros(0, np.uint8)
    return {"name": name.value.decode(), "type": typ.value, "dims": [int(dims[k]) for k in range(nd.value)],
            "nbytes": nb.value, "addr": data.value, "data": buf}


KEYS = ["general.architecture", "a.u8", "a.i8", "a.u16", "a.i16", "a.u32", "a.i32", "a.f32", "a.bool", "a.u64", "a.i64",
        "a.f64", "tok.list", "tok.scores", "nested", "after.arrays", "general.alignment", "not.there"]


@pytest.mark.parametrize("alignment,version", [(32, 3), (64, 3), (4096, 2), (8, 3)])
def test_same_directory_and_metadata_as_the_reference(tmp_path, alignment, version):
    r = _ref()
    p, _ = sample(tmp_path, alignment, version, nested=False)
    h = r.ref_gguf_open(str(p).encode())
    assert h
    try:
        with az.GgufFile(p) as g:
            assert g.n_tensors == r.ref_gguf_n_tensors(h) and g.n_kv == r.ref_gguf_n_kv(h)
            assert g.alignment == r.ref_gguf_get_int(h, b"general.alignment", 32)
            first_mine = first_ref = None
            for i in range(g.n_tensors):
                a, b = g.tensor(i), ref_tensor(r, h, i)
                assert (a["name"], a["type"], a["dims"], a["nbytes"]) == (b["name"], b["type"], b["dims"], b["nbytes"])
                assert np.array_equal(a["data"], b["data"])
                if first_mine is None:
                    first_mine, first_ref = a["data"].ctypes.data, b["addr"]
                # the same place in the file (both map it from offset 0: equal distances from the first tensor)
                assert a["data"].ctypes.data - first_mine == b["addr"] - first_ref
                assert g.find(a["name"]) == r.ref_gguf_find(h, a["name"].encode()) == i
            assert g.find("missing") == r.ref_gguf_find(h, b"missing") == -1
            for key in KEYS:
                k = key.encode()
                # integers and floats: the reference returns its default for a key of another kind, the library None
                assert g.get_int(key, -12345) == r.ref_gguf_get_int(h, k, -12345), key
                assert g.get_float(key, -0.125) == r.ref_gguf_get_float(h, k, -0.125), key
                out = C.create_string_buffer(256)
                has = r.ref_gguf_get_str(h, k, out, 256)
                assert g.get_str(key) == (out.value.decode() if has else None), key
    finally:
        r.ref_gguf_close(h)


def test_header_without_padding_and_no_tensors(tmp_path):
    """A part that holds metadata only may end right after its header (src/gguf.h:347-349): both readers take it."""
    r = _ref()
    p = tmp_path / "meta.gguf"
    gw.write_gguf(p, [("general.architecture", gw.T_STR, "x"), ("n", gw.T_I32, 3)], [], pad_header=False)
    h = r.ref_gguf_open(str(p).encode())
    assert h
    try:
        with az.GgufFile(p) as g:
            assert g.n_tensors == r.ref_gguf_n_tensors(h) == 0 and g.get_int("n") == r.ref_gguf_get_int(h, b"n", -1) == 3
    finally:
        r.ref_gguf_close(h)


def test_both_refuse_the_same_damaged_files(tmp_path):
    r = _ref()
    p, _ = sample(tmp_path, nested=False)
    raw = p.read_bytes()
    i = raw.index(b"general.architecture") + len(b"general.architecture") + 4
    for n, data in enumerate([b"GGML" + raw[4:], raw[:4] + (1).to_bytes(4, "little") + raw[8:],
                              raw[:8] + (1 << 60).to_bytes(8, "little") + raw[16:], raw[:40], raw[:300],
                              raw[:len(raw) - 100], raw[:i] + (1 << 50).to_bytes(8, "little") + raw[i + 8:]]):
        q = tmp_path / f"bad{n}.gguf"
        q.write_bytes(data)
        assert not r.ref_gguf_open(str(q).encode())
        with pytest.raises(az.ArczError):
            az.GgufFile(q)


def test_block_sizes_of_every_type_id():
    r = _ref()
    for typ in list(range(0, 64)) + [0x41523447, 777]:
        b0, n0, b1, n1 = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        ok_ref = r.ref_ggml_block_info(typ, C.byref(b0), C.byref(n0))
        ok = az.lib.arcz_ggml_block_info(typ, C.byref(b1), C.byref(n1))
        assert ok == ok_ref, typ
        if ok:
            assert (b1.value, n1.value) == (b0.value, n0.value), typ
