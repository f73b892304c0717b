"""IQ3_XXS weights (reference src/quants.h:220-239: d / 4 * (1 + 2 s) * a signed codebook magnitude, one s per 32
values, the signs of 8 values as a 7-bit code).  The device holds them in their own form (98 bytes per 256 values, the
GGUF byte count).  The GEMVs (1-8 tokens) decode them in registers through the codebook in LDS; the GEMM forms first
write the matrix out as Q6_K planes of half the values (the magnitudes are even: q = value / 2 + 32, sub-scale 1 + 2 s,
d unchanged) and run the Q6_K kernels on that with half their factor of d -- so every chunk equals, to float rounding,
what the same values uploaded as Q6_K superblocks give where d / 2 is an f16 (it is not always: the reason for that
form).  All against the double-accumulated reference on the IQ3_XXS rows
themselves.  (MoE layers of IQ3_XXS experts: test_gpu_moe.py; every other matmul form: the type-parametrized tests.)"""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import make_acts, make_weights, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu


def _iq3xxs_as_q6k(W, N, K):
    """The Q6_K superblocks that hold the same values: q = value / 2 + 32, int8 sub-scales 1 + 2 s, d / 2 for d / 4."""
    nsb = K // 256
    out = np.zeros((N * nsb, 210), np.uint8)
    for r in range(N):
        q, isc, _, _, _ = orc.decode_row_fields(az.IQ3_XXS, W[r * nsb * 98:(r + 1) * nsb * 98], K)
        assert not (q & 1).any()
        q6 = (q // 2 + 32).reshape(nsb, 2, 4, 32)              # [superblock][half n][quarter][l]
        for s in range(nsb):
            o = out[r * nsb + s]
            for n in range(2):
                q0, q1, q2, q3 = q6[s, n]
                o[64 * n:64 * n + 32] = (q0 & 15) | ((q2 & 15) << 4)
                o[64 * n + 32:64 * n + 64] = (q1 & 15) | ((q3 & 15) << 4)
                o[128 + 32 * n:160 + 32 * n] = (q0 >> 4) | ((q1 >> 4) << 2) | ((q2 >> 4) << 4) | ((q3 >> 4) << 6)
            o[192:208] = isc[16 * s:16 * s + 16].astype(np.int8).view(np.uint8)
            d = W[(r * nsb + s) * 98:(r * nsb + s) * 98 + 2].copy().view(np.float16)
            o[208:210] = (d * np.float16(0.5)).view(np.uint8)
    return out.reshape(-1)


@pytest.mark.parametrize("T,Mp,N,K", [(1, 16, 300, 1024), (2, 16, 129, 2048), (5, 16, 64, 512), (8, 16, 40, 17408),
                                      (12, 16, 200, 768), (100, 112, 272, 768), (300, 384, 200, 512)])
def test_iq3_xxs_matmul(rt, T, Mp, N, K):
    print(f"IQ3_XXS T={T} Mp={Mp} N={N} K={K}", flush=True)
    eng = az.Engine(384, 17408)
    try:
        W = make_weights(az.IQ3_XXS, N, K, seed=720 + T)
        x = make_acts(T, K, seed=730 + T, outliers=True)
        W = W.reshape(-1, 98)
        W[:, 0:2] = np.frombuffer(np.float16(0.00390625).tobytes(), np.uint8)   # d = 2^-8: d / 2 and d / 4 are f16 values
        W = W.reshape(-1)
        W6 = _iq3xxs_as_q6k(W, N, K)
        assert np.array_equal(orc.dequant_rows(az.Q6_K, W6, N, K).view(np.uint32), orc.dequant_rows(az.IQ3_XXS, W, N, K).view(np.uint32))
        w3 = eng.make_weight(az.IQ3_XXS, N, K, W)
        w6 = eng.make_weight(az.Q6_K, N, K, W6)
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, K, K, Mp, T)
        rows = T if T <= 8 else Mp
        ys = []
        for w in (w3, w6):
            cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
            eng.matmul("iq3_xxs", w, Mp, cb, N, 0, 0)
            ys.append(cb.read(np.float32, rows * N).reshape(rows, N)[:T])
            cb.free()
        aq, asc, _ = quantize_padded(x, Mp)
        ref = orc.matmul_ref(az.IQ3_XXS, W, N, K, aq[:T], asc)
        assert np.isfinite(ys[0]).all()
        assert rel_err_rows(ys[0], ref).max() <= 1e-3
        assert rel_err_rows(ys[0], ys[1]).max() <= 2e-5
        assert az.lib.arcz_mem_size(az.lib.arcz_weight_raw(w3.h)) == (az.gguf_bytes(az.IQ3_XXS, N, K) + 15) // 16 * 16
        xb.free(); w3.free(); w6.free()
    finally:
        eng.close()
