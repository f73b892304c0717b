"""What can be checked without a GPU: the C-ABI library loads and exports every symbol its headers declare, fails
loudly (not silently) when there is no device, and its host-side helpers -- the GGUF -> device planes regrouping,
the Q8_0 row quantizer, the synthetic generators -- do what they say."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import ALL_TYPES, TYPES, make_weights

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = []
    for hdr in sorted(os.listdir(os.path.join(ROOT, "include"))):
        src = open(os.path.join(ROOT, "include", hdr)).read()
        src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
        names += re.findall(r"\b(arcz_[a-z0-9_]+)\s*\(", src)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) > 50
    missing = [n for n in names if not hasattr(az.lib, n)]
    assert not missing, missing


def test_no_device_fails_loudly():
    """Without a GPU nothing computes: init reports an error, allocation and engine creation return NULL."""
    import subprocess, sys
    code = ("import arcinferzero_amd as az, sys\n"
            "r = az.lib.arcz_init(0)\n"
            "if r == 0: sys.exit(77)\n"
            "assert r < 0 and az.lib.arcz_last_error()\n"
            "assert not az.lib.arcz_alloc(1024)\n"
            "try:\n    az.Engine(16, 256)\nexcept az.ArczError as e:\n    print('engine refused:', e)\nelse:\n    sys.exit(1)\n")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=ROOT, timeout=120)
    if r.returncode == 77:
        pytest.skip("a GPU is present")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "engine refused" in r.stdout


@pytest.mark.parametrize("qtype", ALL_TYPES)
def test_repack_planes_layout(qtype):
    rows, K = 6, 768
    nsb = K // 256
    W = make_weights(qtype, rows, K, seed=21)
    P = az.repack_planes(qtype, rows, K, W)
    assert P.size == az.planes_bytes(qtype, rows, K)
    u = rows * nsb
    if qtype in (az.Q4_K, az.Q5_K):
        q5 = qtype == az.Q5_K
        sbb = 176 if q5 else 144
        sb = W.reshape(u, sbb)
        assert P.size == W.size
        assert np.array_equal(P[:u * 128].reshape(u, 128), sb[:, sbb - 128:])
        hdr = P[u * 128:u * 144].reshape(u, 16)
        if q5:
            # the fifth bits, one word per 16-byte unit of nibbles: byte c, bit 4 + k = the low-nibble value of the
            # unit's byte 4 k + c, bit k = its high-nibble value; put back on the nibbles they must give the oracle's q
            H = P[u * 144:].view(np.uint32).reshape(u, 8)
            qs = P[:u * 128].reshape(u, 8, 16)
            q = np.zeros((u, 256), np.int64)
            for un in range(8):
                j, half = divmod(un, 2)
                for m in range(16):
                    k, c = divmod(m, 4)
                    lo = (qs[:, un, m] & 15) | (((H[:, un] >> (8 * c + 4 + k)) & 1) << 4)
                    hi = (qs[:, un, m] >> 4) | (((H[:, un] >> (8 * c + k)) & 1) << 4)
                    q[:, 64 * j + 16 * half + m] = lo
                    q[:, 64 * j + 32 + 16 * half + m] = hi
            want = np.stack([orc.decode_row_fields(qtype, W[r * nsb * sbb:(r + 1) * nsb * sbb], K)[0] for r in range(rows)])
            assert np.array_equal(q.reshape(rows, K), want)
        assert np.array_equal(hdr[:, :4], sb[:, :4])                       # d, dmin
        bits = np.zeros(u, dtype=object)
        for k in range(12):
            bits = bits + (hdr[:, 4 + k].astype(object) << (8 * k))
        for r in range(rows):                                               # entries sc | mn << 6 at bit 12 b
            _, isc, imn, _, _ = orc.decode_row_fields(qtype, W[r * nsb * sbb:(r + 1) * nsb * sbb], K)
            for s in range(nsb):
                for b in range(8):
                    e = (int(bits[r * nsb + s]) >> (12 * b)) & 0xFFF
                    assert e == int(isc[s * 16 + 2 * b]) | (int(imn[s * 16 + 2 * b]) << 6)
    elif qtype == az.Q6_K:
        sb = W.reshape(u, 210)
        o = 0
        for lo, n in ((0, 128), (128, 64), (192, 16), (208, 2)):
            assert np.array_equal(P[o:o + u * n].reshape(u, n), sb[:, lo:lo + n])
            o += u * n
        assert not P[o:].any() and P.size % 16 == 0
    elif qtype == az.IQ4_XS:
        sb = W.reshape(u, 136)
        assert np.array_equal(P[:u * 128].reshape(u, 128), sb[:, 8:]) and np.array_equal(P[u * 128:u * 136].reshape(u, 8), sb[:, :8])
        assert not P[u * 136:].any() and P.size % 16 == 0
    elif qtype == az.IQ3_XXS:
        sb = W.reshape(u, 98)                                                # d, 64 index bytes, 8 words of sign codes and scales
        assert P.size == (W.size + 15) // 16 * 16
        assert np.array_equal(P[:u * 64].reshape(u, 64), sb[:, 2:66]) and np.array_equal(P[u * 64:u * 96].reshape(u, 32), sb[:, 66:98])
        assert np.array_equal(P[u * 96:u * 98].reshape(u, 2), sb[:, :2]) and not P[u * 98:].any()
    elif qtype == az.Q3_K:
        # a block's bits together: words D0, D1 of bit pairs (value j of a half in byte j % 4, bits 2 (j / 4)), a word of
        # third bits (value j at bit 8 (j % 4) + j / 4), eight 12-bit header entries of two 6-bit scales, d; put back
        # together they must give the oracle's fields
        sb = W.reshape(u, 110)
        assert P.size == (W.size + 15) // 16 * 16
        D = P[:u * 64].view(np.uint32).reshape(u, 8, 2).astype(np.int64)
        H = P[u * 64:u * 96].view(np.uint32).reshape(u, 8).astype(np.int64)
        j = np.arange(32)
        q = (((D[:, :, j >> 4] >> (8 * (j & 3) + 2 * ((j & 15) >> 2))) & 3) | (((H[:, :, None] >> (8 * (j & 3) + (j >> 2))) & 1) << 2)) - 4
        hd = P[u * 96:u * 108].reshape(u, 12)
        bits = np.zeros(u, dtype=object)
        for k in range(12):
            bits = bits + (hd[:, k].astype(object) << (8 * k))
        sc = np.array([[((int(bits[i]) >> (6 * k)) & 63) - 32 for k in range(16)] for i in range(u)])
        for r in range(rows):
            wq, isc, imn, d, dmin = orc.decode_row_fields(qtype, W[r * nsb * 110:(r + 1) * nsb * 110], K)
            assert np.array_equal(q[r * nsb:(r + 1) * nsb].reshape(K), wq)
            assert np.array_equal(sc[r * nsb:(r + 1) * nsb].reshape(K // 16), isc)
        assert np.array_equal(P[u * 108:u * 110].reshape(u, 2), sb[:, 108:110]) and not P[u * 110:].any()
    elif qtype == az.MXFP4:
        blk = W.reshape(u, 8, 17)                                            # eight 17-byte blocks: E8M0 byte, 16 nibble bytes
        assert P.size == (W.size + 15) // 16 * 16
        assert np.array_equal(P[:u * 128].reshape(u, 8, 16), blk[:, :, 1:]) and np.array_equal(P[u * 128:u * 136].reshape(u, 8), blk[:, :, 0])
        assert not P[u * 136:].any()
    elif qtype in (az.Q4_0, az.IQ4_NL):
        blk = W.reshape(u, 8, 18)                                            # eight 18-byte blocks: f16 d, 16 nibble bytes
        assert P.size == W.size == u * 144
        assert np.array_equal(P[:u * 128].reshape(u, 8, 16), blk[:, :, 2:]) and np.array_equal(P[u * 128:].reshape(u, 8, 2), blk[:, :, :2])
    elif qtype == az.IQ3_S:
        sb = W.reshape(u, 110)                                               # d, 64 index bytes, 8 ninth-bit bytes, 32 sign bytes, 4 scale bytes
        assert P.size == (W.size + 15) // 16 * 16
        assert np.array_equal(P[:u * 64].reshape(u, 64), sb[:, 2:66]) and np.array_equal(P[u * 64:u * 96].reshape(u, 32), sb[:, 74:106])
        hd = P[u * 96:u * 108].reshape(u, 12)
        assert np.array_equal(hd[:, :8], sb[:, 66:74]) and np.array_equal(hd[:, 8:], sb[:, 106:110])
        assert np.array_equal(P[u * 108:u * 110].reshape(u, 2), sb[:, :2]) and not P[u * 110:].any()
    else:
        blk = W.reshape(u, 8, 34)
        assert np.array_equal(P[:u * 256].reshape(u, 8, 32), blk[:, :, 2:]) and np.array_equal(P[u * 256:].reshape(u, 8, 2), blk[:, :, :2])


def test_q8_0_quantizer_is_the_reference_one():
    w = az.gen_normal(5, (32, 512), std=0.02)
    w[3, 64:96] = 0
    assert np.array_equal(az.quantize_rows(az.Q8_0, w), orc.quantize_rows_q8_0(w))


@pytest.mark.parametrize("qtype,rel", [(az.Q4_K, 0.08), (az.Q5_K, 0.04), (az.Q6_K, 0.02), (az.Q8_0, 0.006), (az.IQ4_XS, 0.09),
                                       (az.IQ4_NL, 0.10), (az.MXFP4, 0.15), (az.Q3_K, 0.25), (az.IQ3_XXS, 0.25)])
def test_block_makers_make_valid_close_blocks(qtype, rel):
    """The Q4_K / Q5_K / Q6_K block makers are input generators (the reference has none): valid fields and a round-trip
    error of the size the bit width allows."""
    N, K = 64, 1024
    w = az.gen_normal(6, (N, K), std=0.02)
    B = az.quantize_rows(qtype, w)
    back = orc.dequant_rows(qtype, B, N, K)
    assert np.isfinite(back).all()
    err = np.sqrt(((back - w) ** 2).mean()) / np.sqrt((w ** 2).mean())
    assert err < rel, err
    q, isc, imn, d, dmin = orc.decode_row_fields(qtype, B[:az.gguf_bytes(qtype, 1, K)], K)
    if qtype == az.Q4_K:
        assert q.min() >= 0 and q.max() <= 15 and isc.max() <= 63 and imn.max() <= 63 and len(np.unique(q)) == 16
    elif qtype == az.Q5_K:
        assert q.min() >= 0 and q.max() <= 31 and isc.max() <= 63 and imn.max() <= 63 and len(np.unique(q)) == 32
    elif qtype == az.Q6_K:
        assert q.min() >= -32 and q.max() <= 31 and isc.max() <= 127 and isc.min() >= 1
    elif qtype == az.IQ4_XS:
        assert isc.min() >= 1 and isc.max() <= 31 and len(np.unique(q)) == 16


def test_generators_are_seeded_and_normal():
    a, b = az.gen_normal(42, (1000, 256)), az.gen_normal(42, (1000, 256))
    assert np.array_equal(a, b) and not np.array_equal(a, az.gen_normal(43, (1000, 256)))
    assert abs(a.mean()) < 0.01 and abs(a.std() - 1.0) < 0.01 and abs((a ** 4).mean() - 3.0) < 0.1
    w1, w2 = az.gen_weights(az.Q4_K, 1, 5000, 256), az.gen_weights(az.Q4_K, 1, 5000, 256)
    assert np.array_equal(w1, w2)


def test_byte_counts_match_the_formats():
    assert az.gguf_bytes(az.Q4_K, 17408, 5120) == 50135040       # the figures the roofline uses
    assert az.gguf_bytes(az.Q6_K, 151936, 5120) == 638131200
    assert az.gguf_bytes(az.Q8_0, 4096, 4096) == 17825792
    assert az.gguf_bytes(az.Q4_K, 128 * 768, 2048) * 2 + az.gguf_bytes(az.Q4_K, 128 * 2048, 768) == 339738624
    assert az.gguf_bytes(5, 1, 256) == 0
