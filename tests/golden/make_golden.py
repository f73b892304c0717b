#!/usr/bin/env python3
"""Writes tests/golden/ref_vectors.npz: inputs and outputs of the reference's own CPU functions (src/quants.h), taken
from oracle/_ref/libarcz_ref.so, which oracle/Makefile compiles from the reference header where it lies.  Run it in a
container that has the reference tree (make -C oracle ref); the fixture it writes is data only and is what travels.

Functions covered: fp16_to_f32 / f32_to_fp16 (:17-52), decode_sb / dequant_row for Q8_0, Q4_K, Q6_K (:89-158,
:519-622), quantize_act_cpu (:626-643, both scale widths), quantize_rows_q8_0 (:429-442).  A second file,
ref_vectors_types2.npz, holds the same decode vectors for Q5_K (:91-113), IQ4_XS (:297-311) and IQ3_S (:240-262, with
the whole codebook), drawn from a generator of its own so that the first file's bytes stay what they were.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as orc  # noqa: E402

if orc.ref is None:
    sys.exit("oracle/_ref/libarcz_ref.so is not built (needs the reference tree): make -C oracle ref")
ref = orc.ref
rng = np.random.default_rng(20261125)
out = {}

# ---- fp16
h_all = np.arange(65536, dtype=np.uint16)
out["fp16_all_to_f32_bits"] = np.array([np.float32(ref.ref_fp16_to_f32(int(h))).view(np.uint32) for h in h_all], np.uint32)
f = np.concatenate([
    rng.standard_normal(1500).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 6, 1500).astype(np.float32),
    np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65520.0, 65519.99, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, 6.0975552e-5,
              np.inf, -np.inf, np.nan, 1.0009765625, 1.00048828125, 1.00146484375, 0.333333, 1e30, -1e30], np.float32)])
# exact ties between neighbouring halves, normal and subnormal range
hh = rng.integers(0, 0x7BFF, 400).astype(np.uint16)
lo = np.array([ref.ref_fp16_to_f32(int(h)) for h in hh], np.float64)
hi = np.array([ref.ref_fp16_to_f32(int(h) + 1) for h in hh], np.float64)
f = np.concatenate([f, ((lo + hi) / 2).astype(np.float32)])
out["f32_in"] = f
out["f32_to_fp16"] = np.array([ref.ref_f32_to_fp16(C.c_float(float(v))) for v in f], np.uint16)


def finite_f16(n, lo_exp=-12, hi_exp=2):
    v = (rng.standard_normal(n) * np.exp2(rng.integers(lo_exp, hi_exp, n))).astype(np.float16)
    return v.view(np.uint16)


# ---- blocks: random bytes with finite scales
K, N = 512, 4
for qtype, name, bb in ((12, "q4k", 144), (14, "q6k", 210), (8, "q80", 34)):
    nblk = N * K // (256 if qtype != 8 else 32)
    raw = rng.integers(0, 256, size=(nblk, bb), dtype=np.uint8)
    if qtype == 12:
        raw[:, 0:2] = finite_f16(nblk).reshape(-1, 1).view(np.uint8)
        raw[:, 2:4] = finite_f16(nblk).reshape(-1, 1).view(np.uint8)
    elif qtype == 14:
        raw[:, 208:210] = finite_f16(nblk).reshape(-1, 1).view(np.uint8)
    else:
        raw[:, 0:2] = finite_f16(nblk).reshape(-1, 1).view(np.uint8)
    raw = raw.reshape(-1)
    out[f"{name}_raw"] = raw
    out[f"{name}_dequant"] = orc.dequant_rows(qtype, raw, N, K, lib=ref)
    sbb = 144 if qtype == 12 else 210 if qtype == 14 else 272
    q = np.zeros(256, np.int16); sc = np.zeros(8, np.int32); mn = np.zeros(8, np.int32); sc6 = np.zeros(16, np.int32)
    d8 = np.zeros(8, np.float32); d = C.c_float(); dm = C.c_float()
    first = np.ascontiguousarray(raw[:sbb])
    assert ref.ref_decode_sb(C.c_uint32(qtype), orc.ptr(first), orc.ptr(q), orc.ptr(sc), orc.ptr(mn), orc.ptr(sc6), orc.ptr(d8),
                             C.byref(d), C.byref(dm)) == 0
    out[f"{name}_sb0_q"] = q.copy(); out[f"{name}_sb0_sc"] = sc.copy(); out[f"{name}_sb0_mn"] = mn.copy()
    out[f"{name}_sb0_sc6"] = sc6.copy(); out[f"{name}_sb0_d8"] = d8.copy()
    out[f"{name}_sb0_d"] = np.array([d.value, dm.value], np.float32)

# ---- activation quantizer: outliers, a zero block, exact ties
x = rng.standard_normal((8, 512)).astype(np.float32)
x *= (1.0 + 3.0 * (rng.integers(0, 97, x.shape) == 0)).astype(np.float32)
x[1, 64:96] = 0.0
x[2, :32] = np.array([127.0] + [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5] * 4 + [0.0] * 3, np.float32)
x[3, 256:] *= 1e-20
out["act_x"] = x
for a32 in (1, 0):
    aq, asc, absum = orc.quantize_act(x, act32=bool(a32), lib=ref)
    out[f"act{a32}_aq"] = aq; out[f"act{a32}_asc"] = asc; out[f"act{a32}_absum"] = absum

# ---- Q8_0 row quantizer
w = (rng.standard_normal((8, 256)) * 0.02).astype(np.float32)
w[0, :32] = 0.0
out["q80_rows_in"] = w
out["q80_rows_out"] = orc.quantize_rows_q8_0(w, lib=ref)

np.savez_compressed(os.path.join(HERE, "ref_vectors.npz"), **out)
print("wrote", os.path.join(HERE, "ref_vectors.npz"), {k: v.shape for k, v in out.items()})

# ---- Q5_K blocks (176 bytes: d, dmin, 12 bytes of scales, 32 bytes of fifth bits, 128 bytes of nibbles)
rng = np.random.default_rng(20261126)
out5 = {}
nblk = N * K // 256
raw = rng.integers(0, 256, size=(nblk, 176), dtype=np.uint8)
raw[:, 0:2] = finite_f16(nblk).reshape(-1, 1).view(np.uint8)
raw[:, 2:4] = finite_f16(nblk).reshape(-1, 1).view(np.uint8)
raw = raw.reshape(-1)
out5["q5k_raw"] = raw
out5["q5k_dequant"] = orc.dequant_rows(13, raw, N, K, lib=ref)
q = np.zeros(256, np.int16); sc = np.zeros(8, np.int32); mn = np.zeros(8, np.int32); sc6 = np.zeros(16, np.int32)
d8 = np.zeros(8, np.float32); d = C.c_float(); dm = C.c_float()
first = np.ascontiguousarray(raw[:176])
assert ref.ref_decode_sb(C.c_uint32(13), orc.ptr(first), orc.ptr(q), orc.ptr(sc), orc.ptr(mn), orc.ptr(sc6), orc.ptr(d8),
                         C.byref(d), C.byref(dm)) == 0
out5["q5k_sb0_q"] = q.copy(); out5["q5k_sb0_sc"] = sc.copy(); out5["q5k_sb0_mn"] = mn.copy()
out5["q5k_sb0_d"] = np.array([d.value, dm.value], np.float32)
# ---- IQ4_XS blocks (136 bytes: d, 16 bits + 4 bytes of scales, 128 bytes of 4-bit codes)
raw = rng.integers(0, 256, size=(nblk, 136), dtype=np.uint8)
raw[:, 0:2] = finite_f16(nblk).reshape(-1, 1).view(np.uint8)
raw = raw.reshape(-1)
out5["iq4xs_raw"] = raw
out5["iq4xs_dequant"] = orc.dequant_rows(23, raw, N, K, lib=ref)
# ---- IQ3_S blocks (110 bytes: d, 64 index bytes, 8 bytes of ninth index bits, 32 sign bytes, 4 bytes of scale nibbles;
# src/quants.h:240-262): random ones, and 8 superblocks whose 512 groups of four name the codebook's entries 0..511 in
# order with d = 1, sub-scale 1 and no signs: their decoded row is the codebook itself as the reference holds it
raw = rng.integers(0, 256, size=(nblk, 110), dtype=np.uint8)
raw[:, 0:2] = finite_f16(nblk).reshape(-1, 1).view(np.uint8)
raw = raw.reshape(-1)
out5["iq3s_raw"] = raw
out5["iq3s_dequant"] = orc.dequant_rows(21, raw, N, K, lib=ref)
grid = np.zeros((8, 110), np.uint8)
grid[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
for sb in range(8):
    for b in range(8):
        for g in range(8):
            idx = 64 * sb + 8 * b + g
            grid[sb, 2 + 8 * b + g] = idx & 255
            grid[sb, 66 + b] |= (idx >> 8) << g
out5["iq3s_grid_raw"] = grid.reshape(-1)
out5["iq3s_grid_dequant"] = orc.dequant_rows(21, grid.reshape(-1), 1, 2048, lib=ref)
np.savez_compressed(os.path.join(HERE, "ref_vectors_types2.npz"), **out5)
print("wrote", os.path.join(HERE, "ref_vectors_types2.npz"), {k: v.shape for k, v in out5.items()})
