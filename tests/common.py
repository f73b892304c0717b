"""Shared builders of test inputs: seeded synthetic tensors (the library's generators), hand-made blocks with unit
scales, and the error measures the reference's own harness uses."""
import numpy as np

import arcinferzero_amd as az
import oracle_lib as orc

import os

Q8_0, Q4_K, Q5_K, Q6_K, IQ4_XS, Q4_0, IQ3_S = az.Q8_0, az.Q4_K, az.Q5_K, az.Q6_K, az.IQ4_XS, az.Q4_0, az.IQ3_S
IQ4_NL, MXFP4, Q3_K, IQ3_XXS = az.IQ4_NL, az.MXFP4, az.Q3_K, az.IQ3_XXS
TYPES = (Q8_0, Q4_K, Q6_K, Q5_K, IQ4_XS)
ALL_TYPES = TYPES + (Q4_0, IQ3_S, IQ4_NL, MXFP4, Q3_K, IQ3_XXS)     # with the types the golden files of the first five do not cover
# the IQ3_S codebook as the compiled reference decodes it (a golden vector): 512 entries of four magnitudes
IQ3S_GRID = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors_types2.npz"))[
    "iq3s_grid_dequant"].reshape(512, 4).astype(np.int64)
TYPE_NAMES = {Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", IQ4_XS: "IQ4_XS", az.IQ3_S: "IQ3_S", az.Q4_0: "Q4_0",
              az.IQ4_NL: "IQ4_NL", az.MXFP4: "MXFP4", az.Q3_K: "Q3_K", az.IQ3_XXS: "IQ3_XXS"}
# ... and the IQ3_XXS codebook likewise: 256 entries of four magnitudes
IQ3XXS_GRID = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors_types3.npz"))[
    "iq3xxs_grid_dequant"].reshape(256, 4).astype(np.int64)
IQ4_VALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.int64)
MXFP4_VALUES = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.int64)   # (src/quants.h:497)


def make_weights(qtype, N, K, seed):
    return az.gen_weights(qtype, seed, N, K, 0.02)


def make_acts(M, K, seed, outliers=False):
    x = az.gen_normal(seed, (M, K))
    if outliers:  # the reference's bench multiplies one value in 97 by 4 (bench/gemv_bench.cpp:112)
        rng = np.random.default_rng(seed)
        x = x * (1.0 + 3.0 * (rng.integers(0, 97, size=x.shape) == 0)).astype(np.float32)
    return x


def pad_rows(a, Mp):
    """[M][K] -> [Mp][K] with zero rows."""
    out = np.zeros((Mp,) + a.shape[1:], a.dtype)
    out[:a.shape[0]] = a
    return out


def quantize_padded(x, Mp):
    """Oracle quantization of x [T][K] laid out for Mp rows (rows >= T zero, scale 0)."""
    return orc.quantize_act(pad_rows(x, Mp))


def rel_err_rows(y, ref):
    """Per token row: max_n |y - ref| / max_n |ref| (bench/gemv_bench.cpp:199-214)."""
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    return np.abs(y - ref).max(axis=1) / np.maximum(np.abs(ref).max(axis=1), 1e-30)


def mixed_err(y, ref):
    """Per element |y - ref| / (|ref| + rms(ref)): shows that the row normalization is not doing the work."""
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    return (np.abs(y - ref) / (np.abs(ref) + np.sqrt((ref ** 2).mean()))).max()


def unit_scale_weights(qtype, N, K, seed):
    """GGUF blocks whose scales are exactly 1 (d = 1.0, sub-scales 1, mins 0) over random quants, and the integer
    matrix [N][K] they decode to: with activations whose scales are exactly 1 the f32 output is the integer sum."""
    rng = np.random.default_rng(seed)
    nsb = K // 256
    one = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    if qtype == Q4_K:
        q = rng.integers(0, 16, size=(N, nsb, 256), dtype=np.int64)
        blk = np.zeros((N, nsb, 144), np.uint8)
        blk[..., 0:2] = one
        blk[..., 4:8] = 1      # sc[0..3] = 1, mn = 0
        blk[..., 12:16] = 1    # sc[4..7] low nibble = 1
        for j in range(4):
            blk[..., 16 + 32 * j:16 + 32 * j + 32] = (q[..., 64 * j:64 * j + 32] | (q[..., 64 * j + 32:64 * j + 64] << 4)).astype(np.uint8)
        return blk.reshape(-1), q.reshape(N, K)
    if qtype == Q5_K:
        q = rng.integers(0, 32, size=(N, nsb, 256), dtype=np.int64)
        blk = np.zeros((N, nsb, 176), np.uint8)
        blk[..., 0:2] = one
        blk[..., 4:8] = 1
        blk[..., 12:16] = 1
        for j in range(4):
            lo, hi = q[..., 64 * j:64 * j + 32], q[..., 64 * j + 32:64 * j + 64]
            blk[..., 48 + 32 * j:48 + 32 * j + 32] = ((lo & 15) | ((hi & 15) << 4)).astype(np.uint8)
            blk[..., 16:48] |= (((lo >> 4) << (2 * j)) | ((hi >> 4) << (2 * j + 1))).astype(np.uint8)
        return blk.reshape(-1), q.reshape(N, K)
    if qtype == IQ4_XS:
        c = rng.integers(0, 16, size=(N, nsb, 8, 32), dtype=np.int64)     # codes per block
        blk = np.zeros((N, nsb, 136), np.uint8)
        blk[..., 0:2] = one
        blk[..., 2:4] = [0xAA, 0xAA]    # high two bits of every 6-bit scale = 2, low nibble 1: 33 - 32 = 1
        blk[..., 4:8] = 0x11
        blk[..., 8:] = (c[..., :16] | (c[..., 16:] << 4)).astype(np.uint8).reshape(N, nsb, 128)
        return blk.reshape(-1), IQ4_VALUES[c].reshape(N, K)
    if qtype == Q4_0:
        q = rng.integers(0, 16, size=(N, nsb * 8, 32), dtype=np.int64)
        blk = np.zeros((N, nsb * 8, 18), np.uint8)
        blk[..., 0:2] = one
        blk[..., 2:] = (q[..., :16] | (q[..., 16:] << 4)).astype(np.uint8)
        return blk.reshape(-1), (q - 8).reshape(N, K)
    if qtype == IQ3_XXS:
        # d = 4 (d / 4 = 1), every scale nibble 0 (1 + 2 s = 1): values = the codebook's magnitudes with the signs of
        # random 7-bit codes, the eighth sign their parity
        idx = rng.integers(0, 256, size=(N, nsb, 8, 8), dtype=np.int64)            # [block][group of 4]
        code = rng.integers(0, 128, size=(N, nsb, 8, 4), dtype=np.int64)           # [block][group of 8]
        par = np.zeros_like(code)
        for k in range(7):
            par ^= (code >> k) & 1
        sg8 = code | (par << 7)
        sg = ((sg8[..., None] >> np.arange(8)) & 1).reshape(N, nsb, 8, 32)         # sign bit per value
        blk = np.zeros((N, nsb, 98), np.uint8)
        blk[..., 0:2] = np.frombuffer(np.float16(4.0).tobytes(), np.uint8)
        blk[..., 2:66] = idx.astype(np.uint8).reshape(N, nsb, 64)
        words = (code << (7 * np.arange(4))).sum(axis=-1).astype(np.uint32)        # [N][nsb][8]
        blk[..., 66:98] = words.view(np.uint8).reshape(N, nsb, 32)
        vals = IQ3XXS_GRID[idx].reshape(N, nsb, 8, 32) * (1 - 2 * sg)
        return blk.reshape(-1), vals.reshape(N, K)
    if qtype == Q3_K:
        # d = 1, every 6-bit scale 33 (- 32 = 1): low nibbles 1, high two bits 2; values = the three bits - 4
        q = rng.integers(0, 8, size=(N, nsb, 8, 32), dtype=np.int64)               # [block][element]
        blk = np.zeros((N, nsb, 110), np.uint8)
        blk[..., 96:104] = 0x11
        blk[..., 104:108] = 0xAA
        blk[..., 108:110] = one
        for b in range(8):
            blk[..., 32 + 32 * (b // 4):64 + 32 * (b // 4)] |= ((q[..., b, :] & 3) << (2 * (b % 4))).astype(np.uint8)
            blk[..., 0:32] |= ((q[..., b, :] >> 2) << b).astype(np.uint8)
        return blk.reshape(-1), (q - 4).reshape(N, K)
    if qtype == IQ4_NL:
        c = rng.integers(0, 16, size=(N, nsb * 8, 32), dtype=np.int64)
        blk = np.zeros((N, nsb * 8, 18), np.uint8)
        blk[..., 0:2] = one
        blk[..., 2:] = (c[..., :16] | (c[..., 16:] << 4)).astype(np.uint8)
        return blk.reshape(-1), IQ4_VALUES[c].reshape(N, K)
    if qtype == MXFP4:
        c = rng.integers(0, 16, size=(N, nsb * 8, 32), dtype=np.int64)
        blk = np.zeros((N, nsb * 8, 17), np.uint8)
        blk[..., 0] = 128                     # E8M0 128: 2^(128 - 128) = 1
        blk[..., 1:] = (c[..., :16] | (c[..., 16:] << 4)).astype(np.uint8)
        return blk.reshape(-1), MXFP4_VALUES[c].reshape(N, K)
    if qtype == IQ3_S:
        # d = 1, every 4-bit scale 0 (sub-scale 1): values = the codebook's magnitudes with random signs
        idx = rng.integers(0, 512, size=(N, nsb, 8, 8), dtype=np.int64)            # [block][group of 4]
        sg = rng.integers(0, 2, size=(N, nsb, 8, 32), dtype=np.int64)              # sign bit per value
        blk = np.zeros((N, nsb, 110), np.uint8)
        blk[..., 0:2] = one
        blk[..., 2:66] = (idx & 255).astype(np.uint8).reshape(N, nsb, 64)
        blk[..., 66:74] = ((idx >> 8) << np.arange(8)).sum(axis=-1).astype(np.uint8)
        blk[..., 74:106] = (sg.reshape(N, nsb, 8, 4, 8) << np.arange(8)).sum(axis=-1).astype(np.uint8).reshape(N, nsb, 32)
        vals = IQ3S_GRID[idx].reshape(N, nsb, 8, 32) * (1 - 2 * sg)
        return blk.reshape(-1), vals.reshape(N, K)
    if qtype == Q6_K:
        q = rng.integers(0, 64, size=(N, nsb, 256), dtype=np.int64)
        blk = np.zeros((N, nsb, 210), np.uint8)
        blk[..., 192:208] = 1
        blk[..., 208:210] = one
        for n in range(2):
            b = q[..., 128 * n:128 * n + 128]
            q0, q1, q2, q3 = b[..., 0:32], b[..., 32:64], b[..., 64:96], b[..., 96:128]
            blk[..., 64 * n:64 * n + 32] = ((q0 & 15) | ((q2 & 15) << 4)).astype(np.uint8)
            blk[..., 64 * n + 32:64 * n + 64] = ((q1 & 15) | ((q3 & 15) << 4)).astype(np.uint8)
            blk[..., 128 + 32 * n:128 + 32 * n + 32] = ((q0 >> 4) | ((q1 >> 4) << 2) | ((q2 >> 4) << 4) | ((q3 >> 4) << 6)).astype(np.uint8)
        return blk.reshape(-1), (q - 32).reshape(N, K)
    q = rng.integers(-128, 128, size=(N, K // 32, 32), dtype=np.int64)
    blk = np.zeros((N, K // 32, 34), np.uint8)
    blk[..., 0:2] = one
    blk[..., 2:] = q.astype(np.int8).view(np.uint8)
    return blk.reshape(-1), q.reshape(N, K)


def unit_scale_acts(M, K, seed):
    """Integer-valued activations whose every 32-block has |max| = 127: they quantize to themselves with scale 1."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-127, 128, size=(M, K // 32, 32)).astype(np.float32)
    x[..., 0] = np.where(rng.integers(0, 2, size=(M, K // 32)) == 0, 127.0, -127.0)
    return x.reshape(M, K)
