#!/usr/bin/env python3
"""Writes tests/golden/ref_vectors_types4.npz: decode vectors of the reference's own CPU code (src/quants.h dequant_row,
taken from oracle/_ref/libarcz_ref.so as make_golden.py takes them) for AR4_128 (:531-542) and Q2_0 (:607-616):
blocks of random bytes with finite f16 scales, 4 rows x 512 values.
Run it in a container that has the reference tree (make -C oracle ref); the fixture is data only."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as orc  # noqa: E402

if orc.ref is None:
    sys.exit("oracle/_ref/libarcz_ref.so is not built (needs the reference tree): make -C oracle ref")
rng = np.random.default_rng(20261128)
N, K = 4, 512
out = {}
for name, qtype, blk, nbytes in (("ar4128", orc.AR4_128, 128, 66), ("q20", orc.Q2_0, 64, 18)):
    raw = rng.integers(0, 256, size=(N * K // blk, nbytes), dtype=np.uint8)
    h = rng.integers(0, 65536, raw.shape[0]).astype(np.uint16)
    h[(h & 0x7C00) == 0x7C00] &= 0xBFFF          # no inf / NaN
    raw[:, 0:2] = h.reshape(-1, 1).view(np.uint8)
    out[name + "_raw"] = raw.reshape(-1)
    out[name + "_dequant"] = orc.dequant_rows(qtype, raw.reshape(-1), N, K, lib=orc.ref)
np.savez_compressed(os.path.join(HERE, "ref_vectors_types4.npz"), **out)
print("wrote", os.path.join(HERE, "ref_vectors_types4.npz"), {k: v.shape for k, v in out.items()})
