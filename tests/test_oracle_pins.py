"""Pins the CPU oracle (oracle/arcz_oracle.c) before anything is compared with it: golden vectors taken from the
reference's own header, the compiled reference itself where it is built (oracle/_ref), and what the mathematics
fixes -- closed forms, brute force in numpy, exhaustive fp16 -- chosen so that a dropped term, a wrong index or a
transposed operand fails."""
import ctypes as C
import os

import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import TYPES, make_acts, make_weights, rel_err_rows, unit_scale_acts, unit_scale_weights

G = dict(np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors.npz")))
G.update(np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors_types2.npz")))
G.update(np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors_types3.npz")))
G.update(np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_vectors_types4.npz")))
Q8_0, Q4_K, Q5_K, Q6_K, IQ4_XS = 8, 12, 13, 14, 23
NAMES = {Q4_K: "q4k", Q5_K: "q5k", Q6_K: "q6k", Q8_0: "q80", IQ4_XS: "iq4xs"}


# ---------------------------------------------------------------- fp16
def test_fp16_to_f32_exhaustive():
    h = np.arange(65536, dtype=np.uint16)
    got = np.array([np.float32(orc.orc.orc_fp16_to_f32(int(v))).view(np.uint32) for v in h], np.uint32)
    want = h.view(np.float16).astype(np.float32).view(np.uint32)
    nan = np.isnan(h.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(got[nan].view(np.float32)).all()
    assert np.array_equal(got, G["fp16_all_to_f32_bits"])          # the reference, bit for bit (NaN payloads too)


def test_f32_to_fp16_golden_and_numpy():
    f = G["f32_in"]
    got = np.array([orc.orc.orc_f32_to_fp16(C.c_float(float(v))) for v in f], np.uint16)
    assert np.array_equal(got, G["f32_to_fp16"])
    ok = ~np.isnan(f)
    with np.errstate(over="ignore"):
        assert np.array_equal(got[ok], f[ok].astype(np.float16).view(np.uint16))   # IEEE round to nearest even


def test_fp16_round_trip_all_finite():
    h = np.arange(65536, dtype=np.uint16)
    fin = np.isfinite(h.view(np.float16))
    back = np.array([orc.orc.orc_f32_to_fp16(C.c_float(orc.orc.orc_fp16_to_f32(int(v)))) for v in h[fin]], np.uint16)
    assert np.array_equal(back, h[fin])


# ---------------------------------------------------------------- decoders
@pytest.mark.parametrize("qtype", TYPES)
def test_dequant_golden(qtype):
    nm = NAMES[qtype]
    got = orc.dequant_rows(qtype, G[f"{nm}_raw"], 4, 512)
    assert np.array_equal(got.view(np.uint32), G[f"{nm}_dequant"].view(np.uint32))
    if qtype == IQ4_XS:
        return                              # (rows only: its decoded fields are pinned by the closed form below)
    q, isc, imn, d, dmin = orc.decode_row_fields(qtype, G[f"{nm}_raw"][:512 // 256 * orc.SB_BYTES[qtype]], 512)
    gq = G[f"{nm}_sb0_q"].astype(np.int32) - (32 if qtype == Q6_K else 0)
    assert np.array_equal(q[:256], gq)
    if qtype in (Q4_K, Q5_K):
        assert np.array_equal(isc[:16:2], G[f"{nm}_sb0_sc"]) and np.array_equal(imn[:16:2], G[f"{nm}_sb0_mn"])
        assert d[0] == G[f"{nm}_sb0_d"][0] and dmin[0] == G[f"{nm}_sb0_d"][1]
    elif qtype == Q6_K:
        assert np.array_equal(isc[:16], G[f"{nm}_sb0_sc6"]) and d[0] == G[f"{nm}_sb0_d"][0]
    else:
        assert np.array_equal(d[:8], G[f"{nm}_sb0_d8"])


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref is not built (no reference tree here)")
@pytest.mark.parametrize("qtype", TYPES)
def test_dequant_vs_compiled_reference(qtype):
    W = make_weights(qtype, 16, 1024, seed=3)
    assert np.array_equal(orc.dequant_rows(qtype, W, 16, 1024).view(np.uint32),
                          orc.dequant_rows(qtype, W, 16, 1024, lib=orc.ref).view(np.uint32))


def test_q4k_closed_form():
    """Exact binary fractions, expected values without the decoder (the pattern of tests/test_quant_rows.cpp:17-29)."""
    K = 512
    blk = np.zeros((2, 144), np.uint8)
    exp = np.zeros(K, np.float32)
    for s in range(2):
        d, dmin = (0.25, 0.5) if s == 0 else (2.0, 0.125)
        blk[s, 0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
        blk[s, 2:4] = np.frombuffer(np.float16(dmin).tobytes(), np.uint8)
        sc = [(7 * b + 3 + 11 * s) % 64 for b in range(8)]
        mn = [(13 * b + 5 + 17 * s) % 64 for b in range(8)]
        sb = blk[s, 4:16]
        for j in range(8):                       # the packing of get_scale_min_k4, written out from its definition
            if j < 4:
                sb[j] |= sc[j]; sb[j + 4] |= mn[j]
            else:
                sb[j + 4] |= (sc[j] & 15) | ((mn[j] & 15) << 4)
                sb[j - 4] |= (sc[j] >> 4) << 6
                sb[j] |= (mn[j] >> 4) << 6
        for e in range(256):
            q = (e * 5 + 3 * s) % 16
            j, r = divmod(e, 64)
            if r < 32: blk[s, 16 + 32 * j + r] |= q
            else: blk[s, 16 + 32 * j + r - 32] |= q << 4
            exp[256 * s + e] = d * sc[e // 32] * q - dmin * mn[e // 32]
    got = orc.dequant_rows(Q4_K, blk.reshape(-1), 1, K)[0]
    assert np.array_equal(got, exp)


def test_q5k_closed_form():
    """As the Q4_K case with five-bit values: bit b of byte l of the 32 bytes after the scales is the fifth bit of element
    32 b + l (src/quants.h:101-108); expected values without the decoder."""
    K = 256
    blk = np.zeros(176, np.uint8)
    d, dmin = 0.5, 0.25
    blk[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.float16(dmin).tobytes(), np.uint8)
    sc = [(5 * b + 9) % 64 for b in range(8)]
    mn = [(11 * b + 2) % 64 for b in range(8)]
    sb = blk[4:16]
    for j in range(8):
        if j < 4:
            sb[j] |= sc[j]; sb[j + 4] |= mn[j]
        else:
            sb[j + 4] |= (sc[j] & 15) | ((mn[j] & 15) << 4)
            sb[j - 4] |= (sc[j] >> 4) << 6
            sb[j] |= (mn[j] >> 4) << 6
    exp = np.zeros(K, np.float32)
    for e in range(256):
        q = (e * 7 + 3) % 32
        b, l = divmod(e, 32)
        blk[48 + 32 * (b // 2) + l] |= (q & 15) << (4 * (b % 2))
        blk[16 + l] |= (q >> 4) << b
        exp[e] = d * sc[b] * q - dmin * mn[b]
    assert np.array_equal(orc.dequant_rows(Q5_K, blk, 1, K)[0], exp)
    q, isc, imn, dd, dm = orc.decode_row_fields(Q5_K, blk, K)
    assert np.array_equal(q, [(e * 7 + 3) % 32 for e in range(256)])


def test_iq4xs_closed_form():
    """Every code in every position, scales across their range (the 6-bit scale's low nibble and its two high bits come
    from different places), expected values from the table written out here (src/quants.h:297-311)."""
    tab = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]
    K = 256
    blk = np.zeros(136, np.uint8)
    d = 0.0625
    blk[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    ls = [0, 63, 31, 32, 17, 46, 5, 58]
    sh = 0
    for b in range(8):
        blk[4 + b // 2] |= (ls[b] & 15) << (4 * (b % 2))
        sh |= (ls[b] >> 4) << (2 * b)
    blk[2:4] = [sh & 0xFF, sh >> 8]
    exp = np.zeros(K, np.float32)
    for e in range(256):
        c = (e * 5 + e // 32) % 16
        b, j = divmod(e, 32)
        blk[8 + 16 * b + j % 16] |= c << (4 * (j // 16))
        exp[e] = d * (ls[b] - 32) * tab[c]
    assert np.array_equal(orc.dequant_rows(IQ4_XS, blk, 1, K)[0], exp)
    q, isc, imn, dd, dm = orc.decode_row_fields(IQ4_XS, blk, K)
    assert np.array_equal(isc, np.repeat(np.array(ls) - 32, 2)) and not imn.any() and (dd == d).all()


def test_iq3s_closed_form():
    """IQ3_S (src/quants.h:240-262): groups of four magnitudes by 9-bit codebook index (the ninth bit of group g of a
    block is bit g of the block's qh byte), one sign bit per value, sub-scale 1 + 2 s from a nibble.  Expected values
    from codebook entries written out here (entry i as a little-endian word: its low byte is the first magnitude)."""
    known = {0: (1, 1, 1, 1), 1: (3, 1, 1, 1), 4: (15, 1, 1, 1), 100: (1, 1, 15, 1), 255: (1, 5, 9, 5),
             256: (7, 5, 9, 5), 300: (3, 5, 3, 7), 511: (1, 1, 15, 15)}
    idxs = list(known)
    K = 256
    blk = np.zeros(110, np.uint8)
    d = 0.125
    blk[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    sn = [0, 15, 7, 8, 1, 14, 3, 12]
    exp = np.zeros(K, np.float32)
    for b in range(8):
        blk[106 + b // 2] |= sn[b] << (4 * (b % 2))
        for g in range(8):
            idx = idxs[(3 * b + 5 * g) % len(idxs)]
            blk[2 + 8 * b + g] = idx & 255
            blk[66 + b] |= (idx >> 8) << g
            for j in range(4):
                e = 4 * g + j
                neg = (e * 7 + b) % 3 == 0
                if neg:
                    blk[74 + 4 * b + e // 8] |= 1 << (e % 8)
                exp[32 * b + e] = d * (1 + 2 * sn[b]) * (-known[idx][j] if neg else known[idx][j])
    assert np.array_equal(orc.dequant_rows(orc.IQ3_S, blk, 1, K)[0], exp)
    q, isc, imn, dd, dm = orc.decode_row_fields(orc.IQ3_S, blk, K)
    assert np.array_equal(isc, np.repeat(1 + 2 * np.array(sn), 2)) and not imn.any() and (dd == d).all()


def test_iq3s_golden_with_whole_codebook():
    """The reference's decode of random IQ3_S blocks, and of blocks that name codebook entries 0..511 in order with
    d = 1, sub-scale 1 and no signs: the second pins every entry of the codebook (odd magnitudes 1..15, 2048 values)."""
    got = orc.dequant_rows(orc.IQ3_S, G["iq3s_raw"], 4, 512)
    assert np.array_equal(got.view(np.uint32), G["iq3s_dequant"].view(np.uint32))
    got = orc.dequant_rows(orc.IQ3_S, G["iq3s_grid_raw"], 1, 2048)
    assert np.array_equal(got, G["iq3s_grid_dequant"])
    v = got.reshape(512, 4)
    assert set(np.unique(v)) == {1.0, 3.0, 5.0, 7.0, 9.0, 11.0, 13.0, 15.0}
    assert len({tuple(r) for r in v}) == 512          # (all entries differ)
    # the product's own copy of the codebook, as its kernels take it (512 words, magnitude j of an entry in byte j)
    grid = np.zeros(512, np.uint32)
    az.lib.arcz_iq3s_grid(grid.ctypes.data_as(C.c_void_p))
    assert np.array_equal(grid.view(np.uint8).reshape(512, 4), v.astype(np.uint8))


def _iq3s_as_q6k(W3, N, K):
    """The same values as GGUF Q6_K superblocks: d kept, sub-scale 1 + 2 s for both halves of a block, q = value + 32."""
    nsb = N * K // 256
    out = np.zeros((nsb, 210), np.uint8)
    src = W3.reshape(nsb, 110)
    for s in range(nsb):
        qq, sc, _, _, _ = orc.decode_row_fields(orc.IQ3_S, src[s], 256)
        b = (qq + 32).astype(np.int64)
        for n in range(2):
            q0, q1, q2, q3 = (b[128 * n + 32 * i:128 * n + 32 * i + 32] for i in range(4))
            out[s, 64 * n:64 * n + 32] = (q0 & 15) | ((q2 & 15) << 4)
            out[s, 64 * n + 32:64 * n + 64] = (q1 & 15) | ((q3 & 15) << 4)
            out[s, 128 + 32 * n:128 + 32 * n + 32] = (q0 >> 4) | ((q1 >> 4) << 2) | ((q2 >> 4) << 4) | ((q3 >> 4) << 6)
        out[s, 192:208] = sc.astype(np.int8).view(np.uint8)
        out[s, 208:210] = src[s, 0:2]
    return out.reshape(-1)


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref is not built (no reference tree here)")
def test_iq3s_vs_compiled_reference():
    W = az.quantize_rows(az.IQ3_S, (make_acts(16, 1024, seed=9) * 0.02).astype(np.float32))
    a = orc.dequant_rows(orc.IQ3_S, W, 16, 1024)
    assert np.array_equal(a.view(np.uint32), orc.dequant_rows(orc.IQ3_S, W, 16, 1024, lib=orc.ref).view(np.uint32))
    rng = np.random.default_rng(12)
    R = rng.integers(0, 256, size=(64, 110), dtype=np.uint8)          # every field random: all indices, signs, scales
    R[:, 0:2] = np.frombuffer(np.float16(rng.normal(0, 0.01, size=64)).tobytes(), np.uint8).reshape(64, 2)
    R = R.reshape(-1)
    assert np.array_equal(orc.dequant_rows(orc.IQ3_S, R, 16, 1024).view(np.uint32),
                          orc.dequant_rows(orc.IQ3_S, R, 16, 1024, lib=orc.ref).view(np.uint32))
    # the Q6_K superblocks the GEMM forms expand the matrix to decode to the same f32 values, bit for bit
    assert np.array_equal(orc.dequant_rows(Q6_K, _iq3s_as_q6k(R, 16, 1024), 16, 1024).view(np.uint32),
                          orc.dequant_rows(orc.IQ3_S, R, 16, 1024).view(np.uint32))


def test_q6k_closed_form():
    K = 256
    blk = np.zeros(210, np.uint8)
    d = 0.125
    blk[208:210] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    sc = np.array([(9 * i) % 31 - 15 for i in range(16)], np.int8)
    blk[192:208] = sc.view(np.uint8)
    exp = np.zeros(K, np.float32)
    for e in range(256):
        q = (e * 7 + 1) % 64
        n, r = divmod(e, 128)
        quarter, l = divmod(r, 32)
        lb = 64 * n + l + (32 if quarter & 1 else 0)
        blk[lb] |= (q & 15) << (4 if quarter >= 2 else 0)
        blk[128 + 32 * n + l] |= (q >> 4) << (2 * quarter)
        exp[e] = d * sc[e // 16] * (q - 32)
    assert np.array_equal(orc.dequant_rows(Q6_K, blk, 1, K)[0], exp)


def test_q80_closed_form():
    K = 256
    blk = np.zeros((8, 34), np.uint8)
    exp = np.zeros(K, np.float32)
    for b in range(8):
        d = [0.0, 0.25, 0.5, 2.0][b % 4]
        blk[b, 0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
        for i in range(32):
            q = (i * 13 + b * 7) % 256 - 128
            blk[b, 2 + i] = np.int8(q).view(np.uint8)
            exp[32 * b + i] = d * q
    assert np.array_equal(orc.dequant_rows(Q8_0, blk.reshape(-1), 1, K)[0], exp)


def test_q40_closed_form_and_quantizer():
    """Q4_0 (src/quants.h:136-148, 444-463): blocks made by hand decode to d * (q - 8); the quantizer on values that
    are exact multiples of a power-of-two step, with the extreme at -8 steps, returns exactly those nibbles; a zero
    block gives d = 0 and the nibble 8 everywhere; element i sits in the low nibble of byte i, i + 16 in the high."""
    K = 256
    blk = np.zeros((8, 18), np.uint8)
    exp = np.zeros(K, np.float32)
    for b in range(8):
        d = [0.0, 0.25, -0.5, 2.0][b % 4]
        blk[b, 0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
        for i in range(16):
            q0, q1 = (i * 5 + b) % 16, (i * 11 + 3 * b + 1) % 16
            blk[b, 2 + i] = q0 | (q1 << 4)
            exp[32 * b + i] = d * (q0 - 8)
            exp[32 * b + 16 + i] = d * (q1 - 8)
    assert np.array_equal(orc.dequant_rows(az.Q4_0, blk.reshape(-1), 1, K)[0], exp)
    rng = np.random.default_rng(4)
    q = rng.integers(1, 16, size=(4, K)).astype(np.int32)
    q.reshape(4, 8, 32)[:, :, 7] = 0            # the extreme of every block: -8 steps
    step = 0.125
    w = ((q - 8) * step).astype(np.float32)
    w[3, 32:64] = 0.0                           # a zero block
    out = orc.quantize_rows_q4_0(w).reshape(4, 8, 18)
    d = out[:, :, 0:2].copy().view(np.float16).astype(np.float32)[..., 0]
    lo, hi = (out[:, :, 2:] & 0xF).astype(np.int32), (out[:, :, 2:] >> 4).astype(np.int32)
    got = np.concatenate([lo, hi], axis=2)
    want = q.reshape(4, 8, 32).copy()
    want[3, 1] = 8
    assert np.array_equal(got, want)
    want_d = np.full((4, 8), step, np.float32)
    want_d[3, 1] = 0.0
    assert np.array_equal(d, want_d)
    assert np.array_equal(orc.dequant_rows(az.Q4_0, out.reshape(-1), 4, K), w)


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref is not built (no reference tree here)")
def test_q40_vs_compiled_reference():
    w = (make_acts(16, 512, seed=8) * 0.02).astype(np.float32)
    a, b = orc.quantize_rows_q4_0(w), orc.quantize_rows_q4_0(w, lib=orc.ref)
    assert np.array_equal(a, b)
    assert np.array_equal(orc.dequant_rows(az.Q4_0, a, 16, 512).view(np.uint32),
                          orc.dequant_rows(az.Q4_0, a, 16, 512, lib=orc.ref).view(np.uint32))
    # the product's own generator makes the same blocks as the reference's quantizer, and its device planes hold
    # exactly the values the reference decodes
    assert np.array_equal(az.quantize_rows(az.Q4_0, w), b)
    planes = az.repack_planes(az.Q4_0, 16, 512, a)
    nsb = 2
    nib = planes[:16 * nsb * 128].reshape(16, nsb * 8, 16)                      # a block's 16 nibble bytes
    qs = np.concatenate([nib & 0xF, nib >> 4], axis=2).astype(np.float32) - 8.0   # low nibbles: values 0..15, high: 16..31
    dd = planes[16 * nsb * 128:].view(np.float16).reshape(16, nsb * 8, 1).astype(np.float32)
    assert np.array_equal((qs * dd).reshape(16, 512), orc.dequant_rows(az.Q4_0, a, 16, 512))


def _e8m0_half(e):
    """2^(e - 128) in f32, e = 0 and 1 being subnormals (src/quants.h:498-503)."""
    return np.float32(np.ldexp(1.0, int(e) - 128))


def test_iq4_nl_and_mxfp4_closed_form():
    """IQ4_NL (src/quants.h:594-606): f16 d times the nibble's entry of the IQ4 table; MXFP4 (src/quants.h:495-503,
    520-530): 2^(e - 128) times the doubled E2M1 magnitude of the nibble.  Blocks made by hand with every code in both
    nibble positions, power-of-two and zero scales, and every E8M0 exponent (0 and 1: f32 subnormals; 255: 2^127)."""
    from common import IQ4_VALUES, MXFP4_VALUES
    K = 256
    blk = np.zeros((8, 18), np.uint8)
    exp = np.zeros(K, np.float32)
    for b in range(8):
        d = [0.0, 0.25, -0.5, 2.0, 1.0, -1.0, 0.0078125, 4.0][b]
        blk[b, 0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
        for i in range(16):
            c0, c1 = (i + b) % 16, (5 * i + 3 * b + 1) % 16
            blk[b, 2 + i] = c0 | (c1 << 4)
            exp[32 * b + i] = np.float32(d) * np.float32(IQ4_VALUES[c0])
            exp[32 * b + 16 + i] = np.float32(d) * np.float32(IQ4_VALUES[c1])
    assert np.array_equal(orc.dequant_rows(az.IQ4_NL, blk.reshape(-1), 1, K)[0], exp)
    # MXFP4: all 256 exponents over 32 superblocks, every code in both positions
    K = 256 * 32
    blk = np.zeros((256, 17), np.uint8)
    exp = np.zeros(K, np.float32)
    for b in range(256):
        blk[b, 0] = b
        for i in range(16):
            c0, c1 = (i + b) % 16, (7 * i + b + 3) % 16
            blk[b, 1 + i] = c0 | (c1 << 4)
            with np.errstate(over="ignore"):             # (e = 255: 2^127 times 4 and more is inf, in the oracle too)
                exp[32 * b + i] = _e8m0_half(b) * np.float32(MXFP4_VALUES[c0])
                exp[32 * b + 16 + i] = _e8m0_half(b) * np.float32(MXFP4_VALUES[c1])
    got = orc.dequant_rows(az.MXFP4, blk.reshape(-1), 1, K)[0]
    assert np.array_equal(got.view(np.uint32) & 0x7FFFFFFF, exp.view(np.uint32) & 0x7FFFFFFF)   # (-0.0 from the codes 8)
    assert np.array_equal(got, exp)
    # the integer fields the dot products see, and one scale per 32-block
    q, isc, imn, d, dmin = orc.decode_row_fields(az.MXFP4, blk[:8].reshape(-1), 256)
    assert np.array_equal(isc, np.ones(16)) and not imn.any() and not dmin.any()
    assert np.array_equal(d, [_e8m0_half(b) for b in range(8)])
    assert np.array_equal(q.reshape(8, 32)[:, :16], MXFP4_VALUES[blk[:8, 1:] & 15])


@pytest.mark.parametrize("name,qtype", [("q3k", az.Q3_K), ("iq3xxs", az.IQ3_XXS), ("iq4nl", az.IQ4_NL), ("mxfp4", az.MXFP4)])
def test_further_types_golden(name, qtype):
    """The compiled reference's decode of blocks of random bytes (tests/golden/ref_vectors_types3.npz), bit for bit."""
    got = orc.dequant_rows(qtype, G[name + "_raw"], 4, 512)
    assert np.array_equal(got.view(np.uint32), G[name + "_dequant"].view(np.uint32))


def test_iq3xxs_closed_form_and_whole_codebook():
    """IQ3_XXS (src/quants.h:220-239): groups of four magnitudes by 8-bit codebook index, the signs of 8 values as a
    7-bit code whose parity is the eighth, the scale in the top nibble of the block's word; value = d / 4 * (1 + 2 s) *
    the signed magnitude.  A block made by hand from codebook entries written out here; then blocks that name entries
    0..255 in order with d / 4 = 1, scale 1 and no signs (golden): every entry of the codebook, and the product's own
    copy of it as its kernels take it."""
    known = {0: (4, 4, 4, 4), 1: (20, 4, 4, 4), 2: (36, 4, 4, 4), 3: (12, 12, 4, 4), 255: (4, 28, 52, 62)}
    idxs = list(known)
    K = 256
    blk = np.zeros(98, np.uint8)
    d = 0.5
    blk[0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
    sn = [0, 15, 7, 8, 1, 14, 3, 12]
    exp = np.zeros(K, np.float32)
    for b in range(8):
        a = sn[b] << 28
        for l in range(4):
            code = (37 * b + 11 * l + 5) % 128
            a |= code << (7 * l)
            sg = code | ((bin(code).count("1") & 1) << 7)
            for h in range(2):
                idx = idxs[(3 * b + 2 * l + h) % len(idxs)]
                blk[2 + 8 * b + 2 * l + h] = idx
                for j in range(4):
                    neg = (sg >> (4 * h + j)) & 1
                    exp[32 * b + 8 * l + 4 * h + j] = np.float32(d / 4) * np.float32(1 + 2 * sn[b]) * np.float32(-known[idx][j] if neg else known[idx][j])
        blk[66 + 4 * b:70 + 4 * b] = np.frombuffer(np.uint32(a).tobytes(), np.uint8)
    assert np.array_equal(orc.dequant_rows(az.IQ3_XXS, blk, 1, K)[0], exp)
    got = orc.dequant_rows(az.IQ3_XXS, G["iq3xxs_grid_raw"], 1, 1024)
    assert np.array_equal(got, G["iq3xxs_grid_dequant"])
    v = got.reshape(256, 4)
    assert set(np.unique(v)) == {4.0, 12.0, 20.0, 28.0, 36.0, 44.0, 52.0, 62.0} and len({tuple(r) for r in v}) == 256
    grid = np.zeros(256, np.uint32)
    az.lib.arcz_iq3xxs_grid(grid.ctypes.data_as(C.c_void_p))
    assert np.array_equal(grid.view(np.uint8).reshape(256, 4), v.astype(np.uint8))


def test_q3_k_closed_form():
    """Q3_K (src/quants.h:465-494): a superblock made by hand -- every 3-bit value in every block, sixteen different
    6-bit scales on both sides of 32, d a power of two -- decodes to d * (scale - 32) * (q - 4)."""
    K = 256
    blk = np.zeros(110, np.uint8)
    blk[108:110] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    sc = [(7 * i + 3) % 64 for i in range(16)]
    for i, s6 in enumerate(sc):
        blk[96 + (i & 7)] |= (s6 & 0xF) << (4 * (i >> 3))
        blk[104 + (i & 3)] |= (s6 >> 4) << (2 * (i >> 2))
    exp = np.zeros(K, np.float32)
    for b in range(8):
        for e in range(32):
            q = (3 * e + 5 * b + 1) % 8
            blk[32 + 32 * (b // 4) + e] |= (q & 3) << (2 * (b % 4))
            blk[e] |= (q >> 2) << b
            exp[32 * b + e] = np.float32(0.5) * np.float32(sc[2 * b + e // 16] - 32) * np.float32(q - 4)
    assert np.array_equal(orc.dequant_rows(az.Q3_K, blk, 1, K)[0], exp)
    q, isc, imn, d, dmin = orc.decode_row_fields(az.Q3_K, blk, K)
    assert np.array_equal(isc, np.array(sc) - 32) and not imn.any() and q.min() == -4 and q.max() == 3


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref is not built (no reference tree here)")
def test_q3_k_vs_compiled_reference():
    N, K = 16, 512
    W = az.gen_weights(az.Q3_K, 7, N, K, 0.02)
    R = np.random.default_rng(9).integers(0, 256, size=W.size, dtype=np.uint8)
    R.reshape(-1, 110)[:, 109] &= 0x7B                      # finite f16 d
    for blocks in (W, R):
        a, b = orc.dequant_rows(az.Q3_K, blocks, N, K), orc.dequant_rows(az.Q3_K, blocks, N, K, lib=orc.ref)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref is not built (no reference tree here)")
@pytest.mark.parametrize("qtype", [az.IQ4_NL, az.MXFP4])
def test_iq4_nl_and_mxfp4_vs_compiled_reference(qtype):
    """The oracle's decode of generated blocks and of blocks of random bytes (IQ4_NL: finite f16 scales) against the
    compiled reference header's dequant_row, bit for bit; and the device planes against the reference's own GPU form
    of a superblock (src/quants.h gpu_raw_sb: the eight scales, then the eight blocks' nibble bytes)."""
    N, K = 16, 512
    nsb, hb = K // 256, 1 if qtype == az.MXFP4 else 2
    W = az.gen_weights(qtype, 7, N, K, 0.02)
    R = np.random.default_rng(9).integers(0, 256, size=W.size, dtype=np.uint8)
    if qtype == az.IQ4_NL:
        R.reshape(-1, 18)[:, 1] &= 0x7B
    for blocks in (W, R):
        a, b = orc.dequant_rows(qtype, blocks, N, K), orc.dequant_rows(qtype, blocks, N, K, lib=orc.ref)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    planes = az.repack_planes(qtype, N, K, W)
    u = N * nsb
    rsb = int(orc.ref.ref_raw_padded_sb_bytes(qtype))
    assert rsb == 128 + 8 * hb
    raw = np.zeros(rsb, np.uint8)
    for i in range(u):
        orc.ref.ref_gpu_raw_sb(qtype, orc.ptr(W[i * (16 + hb) * 8:]), orc.ptr(raw))
        assert np.array_equal(raw[:8 * hb], planes[u * 128 + i * 8 * hb:u * 128 + (i + 1) * 8 * hb])
        assert np.array_equal(raw[8 * hb:], planes[i * 128:(i + 1) * 128])


def _ar4_q20_by_hand():
    """One superblock of each type written field by field, with the values it must decode to: every code in every
    position class (AR4_128: low and high nibble of every byte of a run; Q2_0: each of the four 2-bit slots of a byte),
    scales of both signs, zero and a subnormal."""
    ar = np.zeros((2, 66), np.uint8)
    ar_exp = np.zeros(256, np.float32)
    for b, d in enumerate([-0.75, 6.103515625e-05 / 4]):                  # (the second: an f16 subnormal)
        ar[b, 0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
        for c in range(4):
            for j in range(16):
                lo, hi = (j + 3 * c + b) % 16, (7 * j + c + 5 * b + 2) % 16
                ar[b, 2 + 16 * c + j] = lo | (hi << 4)
                ar_exp[128 * b + 32 * c + j] = np.float32(np.float16(d)) * np.float32(lo - 8)
                ar_exp[128 * b + 32 * c + 16 + j] = np.float32(np.float16(d)) * np.float32(hi - 8)
    q2 = np.zeros((4, 18), np.uint8)
    q2_exp = np.zeros(256, np.float32)
    for b, d in enumerate([0.5, -3.0, 0.0, 1024.0]):
        q2[b, 0:2] = np.frombuffer(np.float16(d).tobytes(), np.uint8)
        for j in range(64):
            q = (j + j // 4 + b) % 4
            q2[b, 2 + j // 4] |= q << (2 * (j % 4))
            q2_exp[64 * b + j] = np.float32(d) * np.float32(q - 1)
    return ar.reshape(-1), ar_exp, q2.reshape(-1), q2_exp


def test_ar4_128_and_q2_0_closed_form_and_golden():
    """AR4_128 (src/quants.h:531-542): the 128-block's f16 d times (nibble - 8), four runs of 16 bytes laid out as
    Q4_0's; Q2_0 (src/quants.h:607-616): the 64-block's f16 d times (code - 1), element j in bits 2 (j % 4) of byte
    j / 4.  By hand, then the compiled reference's decode of blocks of random bytes, bit for bit."""
    ar, ar_exp, q2, q2_exp = _ar4_q20_by_hand()
    assert np.array_equal(orc.dequant_rows(orc.AR4_128, ar, 1, 256)[0], ar_exp)
    assert np.array_equal(orc.dequant_rows(orc.Q2_0, q2, 1, 256)[0], q2_exp)
    q, isc, imn, d, dmin = orc.decode_row_fields(orc.Q2_0, q2, 256)
    assert np.array_equal(isc, np.ones(16)) and not imn.any() and not dmin.any()
    assert np.array_equal(d, np.repeat(np.float32([0.5, -3.0, 0.0, 1024.0]), 2)) and q.min() == -1 and q.max() == 2
    for name, qtype in (("ar4128", orc.AR4_128), ("q20", orc.Q2_0)):
        got = orc.dequant_rows(qtype, G[name + "_raw"], 4, 512)
        assert np.array_equal(got.view(np.uint32), G[name + "_dequant"].view(np.uint32))


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref is not built (no reference tree here)")
@pytest.mark.parametrize("qtype", [orc.AR4_128, orc.Q2_0])
def test_ar4_128_and_q2_0_vs_compiled_reference(qtype):
    """Blocks of random bytes (finite f16 scales) through the oracle and the compiled reference header, bit for bit."""
    N, K = 8, 1024
    nb = orc.SB_BYTES[qtype] // (2 if qtype == orc.AR4_128 else 4)
    R = np.random.default_rng(11).integers(0, 256, size=(N * K // 256 * orc.SB_BYTES[qtype] // nb, nb), dtype=np.uint8)
    R[:, 1] &= 0x7B
    a, b = orc.dequant_rows(qtype, R.reshape(-1), N, K), orc.dequant_rows(qtype, R.reshape(-1), N, K, lib=orc.ref)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_relayout_q4_0_keeps_every_value():
    """The library writes AR4_128 and Q2_0 rows out as Q4_0 blocks before it uploads them: the Q4_0 decode of what it
    writes is the decode of the source, bit for bit (by hand, golden blocks, random bytes), and K that is not whole
    source blocks, another type or a wrong byte count are refused."""
    ar, ar_exp, q2, q2_exp = _ar4_q20_by_hand()
    assert np.array_equal(orc.dequant_rows(az.Q4_0, az.relayout_q4_0(az.AR4_128, 1, 256, ar), 1, 256)[0], ar_exp)
    assert np.array_equal(orc.dequant_rows(az.Q4_0, az.relayout_q4_0(az.Q2_0, 1, 256, q2), 1, 256)[0], q2_exp)
    for name, qtype in (("ar4128", az.AR4_128), ("q20", az.Q2_0)):
        out = az.relayout_q4_0(qtype, 4, 512, G[name + "_raw"])
        assert out.size == 4 * 16 * 18
        assert np.array_equal(orc.dequant_rows(az.Q4_0, out, 4, 512).view(np.uint32), G[name + "_dequant"].view(np.uint32))
    # rows that end inside a superblock: 3 rows of 384 (AR4_128) and of 320 (Q2_0) values
    rng = np.random.default_rng(5)
    for qtype, K, blk, nbytes in ((az.AR4_128, 384, 128, 66), (az.Q2_0, 320, 64, 18)):
        raw = rng.integers(0, 256, size=(3 * K // blk, nbytes), dtype=np.uint8)
        raw[:, 1] &= 0x7B
        out = az.relayout_q4_0(qtype, 3, K, raw.reshape(-1)).reshape(3, K // 32 * 18)
        for r in range(3):     # (each row alone, padded with zero blocks to 512 for the oracle's whole superblocks)
            src = np.zeros(512 // blk * nbytes, np.uint8)
            src[:K // blk * nbytes] = raw.reshape(3, -1)[r]
            dst = np.zeros(16 * 18, np.uint8)
            dst[:K // 32 * 18] = out[r]
            assert np.array_equal(orc.dequant_rows(az.Q4_0, dst, 1, 512), orc.dequant_rows(qtype, src, 1, 512))
    for bad in (lambda: az.relayout_q4_0(az.AR4_128, 1, 192, np.zeros(99, np.uint8)),
                lambda: az.relayout_q4_0(az.Q2_0, 1, 96, np.zeros(27, np.uint8)),
                lambda: az.relayout_q4_0(az.Q4_0, 1, 256, np.zeros(144, np.uint8)),
                lambda: az.relayout_q4_0(az.Q2_0, 2, 128, np.zeros(71, np.uint8))):
        with pytest.raises(ValueError):
            bad()


# ---------------------------------------------------------------- quantizers
def test_quantize_act_golden():
    for a32 in (1, 0):
        aq, asc, absum = orc.quantize_act(G["act_x"], act32=bool(a32))
        assert np.array_equal(aq, G[f"act{a32}_aq"])
        assert np.array_equal(asc.view(np.uint32), G[f"act{a32}_asc"].view(np.uint32))
        assert np.array_equal(absum, G[f"act{a32}_absum"].view(np.int16))


def test_quantize_act_closed_forms():
    x = np.zeros((3, 64), np.float32)
    x[0, :32] = np.linspace(-2.0, 2.0, 32)
    x[1, :32] = np.array([127.0] + [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5] * 4 + [0.0] * 3)
    x[2, 32:] = -5.0
    aq, asc, absum = orc.quantize_act(x)
    assert aq[0, 0] == -127 and aq[0, 31] == 127 and np.array_equal(aq[0, :32], -aq[0, :32][::-1])   # sign symmetry
    assert asc[0, 0] == np.float32(2.0) / np.float32(127.0)
    assert asc[1, 0] == 0.0 and not aq[0, 32:].any()                                               # zero block
    assert aq[1, 1:8].tolist() == [0, 2, 2, 0, -2, -2, 4]                                           # ties to even
    assert (aq[2, 32:] == -127).all() and absum[2, 2] == -127 * 16
    assert np.array_equal(aq.reshape(3, 4, 16).astype(np.int32).sum(axis=2).T, absum.astype(np.int32))


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref is not built (no reference tree here)")
def test_quantizers_vs_compiled_reference():
    x = make_acts(32, 1024, seed=5, outliers=True)
    for a32 in (True, False):
        a, b = orc.quantize_act(x, act32=a32), orc.quantize_act(x, act32=a32, lib=orc.ref)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))
        assert np.array_equal(a[2], b[2])
    w = (make_acts(16, 512, seed=6) * 0.02).astype(np.float32)
    assert np.array_equal(orc.quantize_rows_q8_0(w), orc.quantize_rows_q8_0(w, lib=orc.ref))


def test_quantize_rows_q8_0_golden_and_roundtrip():
    w = G["q80_rows_in"]
    out = orc.quantize_rows_q8_0(w)
    assert np.array_equal(out, G["q80_rows_out"])
    back = orc.dequant_rows(Q8_0, out, 8, 256)
    amax = np.abs(w.reshape(8, 8, 32)).max(axis=2, keepdims=True)
    # half a step of the block's scale, plus the fp16 rounding of the scale itself
    assert (np.abs(back.reshape(8, 8, 32) - w.reshape(8, 8, 32)) <= amax / 127.0 * 0.5 + amax * 2.0 ** -11 + 1e-12).all()


def test_act_residual_identities():
    """The two-pass residual v - q * scale: the subtraction is exact (q * scale is within a factor of two of v wherever
    q != 0, and 0 where q == 0), so q * scale + res gives v back exactly; it is at most half a step; and quantizing it
    leaves an error 254 times smaller than the first pass's step.  A wrong factor (127 / amax for amax / 127), a dropped
    term or a wrong block index fails the bound."""
    x = make_acts(6, 1024, seed=31, outliers=True)
    x[1, 64:96] = 0.0
    x[2, 128:160] *= 1e-30
    (aq, asc, _), (rq, rsc, _), res = orc.quantize_act_two_pass(x)
    sc = np.repeat(asc.T, 32, axis=1)
    p = (aq.astype(np.float32) * sc).astype(np.float32)
    assert np.array_equal(p.astype(np.float64) + res.astype(np.float64), x.astype(np.float64))
    assert (np.abs(res) <= sc * 0.5 * (1 + 2.0 ** -21) + 1e-45).all()
    assert not res[1, 64:96].any() and not rq[1, 64:96].any() and not rsc[2:3, 1].any()
    rs = np.repeat(rsc.T, 32, axis=1)
    left = x.astype(np.float64) - p.astype(np.float64) - rq.astype(np.float64) * rs.astype(np.float64)
    assert (np.abs(left) <= rs * 0.5 * (1 + 2.0 ** -21) + 1e-45).all() and (rs <= sc / 253.9).all()


# ---------------------------------------------------------------- integer sums and the f32 references
@pytest.mark.parametrize("qtype", TYPES)
def test_block_sums_brute_force(qtype):
    N, K, M = 5, 512, 3
    W = make_weights(qtype, N, K, seed=7)
    aq, asc, absum = orc.quantize_act(make_acts(M, K, seed=8))
    I = orc.block_sums(qtype, W, N, K, aq)
    q = np.stack([orc.decode_row_fields(qtype, W[n * (K // 256) * orc.SB_BYTES[qtype]:(n + 1) * (K // 256) * orc.SB_BYTES[qtype]], K)[0]
                  for n in range(N)]).astype(np.int64)
    want = np.einsum("nhk,mhk->mnh", q.reshape(N, K // 16, 16), aq.astype(np.int64).reshape(M, K // 16, 16))
    assert np.array_equal(I, want)


@pytest.mark.parametrize("qtype", TYPES)
def test_matmul_ref_is_a_float64_dot(qtype):
    N, K, M = 24, 768, 5
    W = make_weights(qtype, N, K, seed=9)
    aq, asc, absum = orc.quantize_act(make_acts(M, K, seed=10, outliers=True))
    Y = orc.matmul_ref(qtype, W, N, K, aq, asc)
    w = orc.dequant_rows(qtype, W, N, K).astype(np.float64)
    x = (aq.astype(np.float32) * np.repeat(asc.T, 32, axis=1)).astype(np.float64)
    want = x @ w.T
    assert np.abs(Y - want).max() <= 2e-7 * np.abs(want).max()       # one rounding to f32 (summation order aside)
    for form in (0, 1):
        F = orc.matmul_formula(qtype, form, W, N, K, aq, asc, absum)
        assert rel_err_rows(F, want).max() <= 5e-6                      # the engine's f32 formulas: rounding only


@pytest.mark.parametrize("qtype", TYPES)
def test_unit_scale_known_answer(qtype):
    """All scales 1: both f32 evaluations must give the exact integer sum (catches a dropped min term, a wrong
    sub-scale index, a swapped nibble)."""
    N, K, M = 12, 512, 4
    W, wi = unit_scale_weights(qtype, N, K, seed=11)
    x = unit_scale_acts(M, K, seed=12)
    aq, asc, absum = orc.quantize_act(x)
    assert np.array_equal(aq.astype(np.float32), x) and (asc == 1.0).all()
    exact = (x.astype(np.int64) @ wi.T).astype(np.float32)
    assert np.array_equal(orc.matmul_ref(qtype, W, N, K, aq, asc), exact)
    for form in (0, 1):
        assert np.array_equal(orc.matmul_formula(qtype, form, W, N, K, aq, asc, absum), exact)


def test_q4k_min_term_matters():
    """A Q4_K matrix with zero quants and non-zero mins: the output is -dmin * mn * sum(a), nothing else."""
    K, N = 256, 1
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    blk[4:8] = 1
    blk[8:12] = [2, 3, 4, 5]               # mn[0..3]
    blk[12:16] = 1 | (6 << 4)              # sc[4..7] = 1, mn[4..7] = 6
    x = unit_scale_acts(2, K, seed=13)
    aq, asc, absum = orc.quantize_act(x)
    mn = np.array([2, 3, 4, 5, 6, 6, 6, 6], np.float64)
    want = -(0.5 * mn * x.reshape(2, 8, 32).sum(axis=2)).sum(axis=1)
    for Y in (orc.matmul_ref(Q4_K, blk, N, K, aq, asc), orc.matmul_formula(Q4_K, 0, blk, N, K, aq, asc, absum),
              orc.matmul_formula(Q4_K, 1, blk, N, K, aq, asc, absum)):
        assert np.array_equal(Y[:, 0].astype(np.float64), want)


# ---------------------------------------------------------------- mixture of experts
def test_route_vs_stable_sort():
    rng = np.random.default_rng(11)
    NE, NU, T = 256, 6, 7                  # the reference's own case (tests/test_route.cpp:20)
    lg = (rng.standard_normal((T, NE + 1)) * 2.0).astype(np.float32)
    lg[2, 10] = lg[2, 200] = lg[2].max() + 1
    ids, wts, sgate, counts = orc.moe_route(lg, NE, NU)
    cnt = np.zeros(NE, np.int64)
    for t in range(T):
        idx = np.argsort(-lg[t, :NE], kind="stable")[:NU]
        assert np.array_equal(ids[t], idx)
        p = np.exp(lg[t, idx].astype(np.float64) - float(lg[t, idx[0]]))
        assert np.abs(wts[t] - p / p.sum()).max() < 1e-6
        assert abs(sgate[t] - 1.0 / (1.0 + np.exp(-float(lg[t, NE])))) < 1e-6
        cnt[idx] += 1
    assert np.array_equal(counts, cnt)


def test_scan_scatter_invariants():
    rng = np.random.default_rng(12)
    NE, NU, T, TM = 16, 4, 100, 16
    lg = rng.standard_normal((T, NE)).astype(np.float32)
    lg[:, 3] -= 100
    ids, wts, _, counts = orc.moe_route(lg, NE, NU)
    offs, tiles, tstart = orc.moe_scan(counts, TM)
    assert counts[3] == 0 and counts.sum() == T * NU
    assert np.array_equal(offs, np.concatenate([[0], np.cumsum(counts)[:-1]]))
    nt = tiles[0]
    assert nt == ((counts + TM - 1) // TM).sum() == tstart[NE]
    t3 = tiles[1:1 + 3 * nt].reshape(nt, 3)
    for e in range(NE):
        mine = t3[tstart[e]:tstart[e + 1]]
        assert (mine[:, 0] == e).all() and mine[:, 2].sum() == counts[e] and (mine[:, 2] <= TM).all()
        assert np.array_equal(mine[:, 1], offs[e] + TM * np.arange(len(mine)))
    stok, swt, inv = orc.moe_scatter(ids, wts, offs)
    n = T * NU
    assert sorted(inv.tolist()) == list(range(n))
    assert np.array_equal(stok[inv], np.arange(n) // NU) and np.array_equal(swt[inv], wts.reshape(-1))
    assert np.array_equal(np.repeat(np.arange(NE), counts)[inv], ids.reshape(-1))


def test_moe_quant_matches_act_quant():
    h = make_acts(5, 256, seed=14)
    hq, hsc = orc.moe_quant(h)
    aq, asc, _ = orc.quantize_act(h)
    assert np.array_equal(hq, aq) and np.array_equal(hsc, asc)


def test_moe_layer_composition():
    """orc_moe_layer against a float64 numpy composition of its parts."""
    qtype, NE, NU, E, F, T = Q4_K, 4, 2, 256, 256, 6
    Wg, Wu, Wd = (make_weights(qtype, NE * F, E, seed=1), make_weights(qtype, NE * F, E, seed=2),
                  make_weights(qtype, NE * E, F, seed=3))
    aq, asc, _ = orc.quantize_act(make_acts(T, E, seed=4))
    lg = np.random.default_rng(5).standard_normal((T, NE)).astype(np.float32)
    out, h = orc.moe_layer(qtype, Wg, Wu, Wd, NE, NU, E, F, aq, asc, lg)
    wg = orc.dequant_rows(qtype, Wg, NE * F, E).astype(np.float64).reshape(NE, F, E)
    wu = orc.dequant_rows(qtype, Wu, NE * F, E).astype(np.float64).reshape(NE, F, E)
    wd = orc.dequant_rows(qtype, Wd, NE * E, F).astype(np.float64).reshape(NE, E, F)
    x = (aq.astype(np.float32) * np.repeat(asc.T, 32, axis=1)).astype(np.float64)
    ids, wts, _, _ = orc.moe_route(lg, NE, NU)
    want = np.zeros((T, E))
    for t in range(T):
        for k in range(NU):
            e = ids[t, k]
            g = (wg[e] @ x[t]).astype(np.float32).astype(np.float64)
            u = (wu[e] @ x[t]).astype(np.float32)
            hh = (g / (1 + np.exp(-g))).astype(np.float32) * u
            assert np.abs(hh - h[t * NU + k]).max() <= 1e-5 * np.abs(hh).max()
            hq, hsc = orc.moe_quant(h[t * NU + k][None, :])
            hx = (hq[0].astype(np.float32) * np.repeat(hsc[:, 0], 32)).astype(np.float64)
            want[t] += float(wts[t, k]) * (wd[e] @ hx)
    assert rel_err_rows(out, want).max() <= 1e-5
