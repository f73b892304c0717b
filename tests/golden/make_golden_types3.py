#!/usr/bin/env python3
"""Writes tests/golden/ref_vectors_types3.npz: decode vectors of the reference's own CPU code (src/quants.h dequant_row,
taken from oracle/_ref/libarcz_ref.so as make_golden.py takes them) for the weight types added after the first two
files: Q3_K (:465-494), IQ3_XXS (:220-239, with the whole codebook: four superblocks whose 256 groups of four name its
entries 0..255 in order with d / 4 = 1, scale 1 and no signs -- their decoded row is the codebook as the reference
holds it), IQ4_NL (:594-606) and MXFP4 (:495-503, 520-530).  Blocks of random bytes with finite f16 scales (MXFP4:
scale bytes 88..167, 2^-40 .. 2^39, so that sums of products stay finite in f32), 4 rows x 512.
Run it in a container that has the reference tree (make -C oracle ref); the fixture is data only."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as orc  # noqa: E402

if orc.ref is None:
    sys.exit("oracle/_ref/libarcz_ref.so is not built (needs the reference tree): make -C oracle ref")
ref = orc.ref
rng = np.random.default_rng(20261127)
N, K = 4, 512
out = {}


def finite_f16(n):
    h = rng.integers(0, 65536, n).astype(np.uint16)
    h[(h & 0x7C00) == 0x7C00] &= 0xBFFF          # no inf / NaN
    return h


def blocks(name, qtype, sb_bytes, f16_at, e8m0_at=()):
    raw = rng.integers(0, 256, size=(N * K // 256, sb_bytes), dtype=np.uint8)
    for o in e8m0_at:
        raw[:, o] = rng.integers(88, 168, raw.shape[0])
    for o, stride, cnt in f16_at:                 # (offset of the first f16 scale, stride, how many per superblock)
        for i in range(cnt):
            raw[:, o + i * stride:o + i * stride + 2] = finite_f16(raw.shape[0]).reshape(-1, 1).view(np.uint8)
    raw = raw.reshape(-1)
    out[name + "_raw"] = raw
    out[name + "_dequant"] = orc.dequant_rows(qtype, raw, N, K, lib=ref)


blocks("q3k", 11, 110, [(108, 0, 1)])
blocks("iq3xxs", 18, 98, [(0, 0, 1)])
blocks("iq4nl", 20, 144, [(0, 18, 8)])
blocks("mxfp4", 39, 136, [], e8m0_at=range(0, 136, 17))
grid = np.zeros((4, 98), np.uint8)
grid[:, 0:2] = np.frombuffer(np.float16(4.0).tobytes(), np.uint8)
grid[:, 2:66] = np.arange(256, dtype=np.uint8).reshape(4, 64)
out["iq3xxs_grid_raw"] = grid.reshape(-1)
out["iq3xxs_grid_dequant"] = orc.dequant_rows(18, grid.reshape(-1), 1, 1024, lib=ref)
np.savez_compressed(os.path.join(HERE, "ref_vectors_types3.npz"), **out)
print("wrote", os.path.join(HERE, "ref_vectors_types3.npz"), {k: v.shape for k, v in out.items()})
