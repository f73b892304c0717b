"""Q3_K weights (reference src/quants.h:465-494: d * (scale - 32) * (three bits - 4), a 6-bit scale per 16 values).  The
device holds them at the GGUF byte count (110 bytes per 256 values), a block's bits regrouped so that four values leave
a word with a shift and a mask.  The GEMVs (chunks of 16 rows) decode them in registers; the GEMM forms first write the matrix
out as Q6_K planes, value for value (same d, the scales - 32 as the int8 sub-scales, q = value + 32), and run the Q6_K
kernels on that -- so a chunk of more than 16 rows is bit for bit what the same matrix uploaded as Q6_K superblocks
gives, and the shorter ones equal it to float rounding.  All against the double-accumulated reference on the Q3_K rows
themselves.  (MoE layers of Q3_K experts: test_gpu_moe.py; every other matmul form: the type-parametrized tests.)"""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import make_acts, make_weights, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu


def _q3k_as_q6k(W, N, K):
    """The Q6_K superblocks that hold the same values: q = value + 32, int8 sub-scales = the scales - 32, the same d."""
    nsb = K // 256
    out = np.zeros((N * nsb, 210), np.uint8)
    for r in range(N):
        q, isc, _, _, _ = orc.decode_row_fields(az.Q3_K, W[r * nsb * 110:(r + 1) * nsb * 110], K)
        q6 = (q + 32).reshape(nsb, 2, 4, 32)                    # [superblock][half n][quarter][l]
        for s in range(nsb):
            o = out[r * nsb + s]
            for n in range(2):
                q0, q1, q2, q3 = q6[s, n]
                o[64 * n:64 * n + 32] = (q0 & 15) | ((q2 & 15) << 4)
                o[64 * n + 32:64 * n + 64] = (q1 & 15) | ((q3 & 15) << 4)
                o[128 + 32 * n:160 + 32 * n] = (q0 >> 4) | ((q1 >> 4) << 2) | ((q2 >> 4) << 4) | ((q3 >> 4) << 6)
            o[192:208] = isc[16 * s:16 * s + 16].astype(np.int8).view(np.uint8)
            o[208:210] = W[(r * nsb + s) * 110 + 108:(r * nsb + s) * 110 + 110]
    return out.reshape(-1)


@pytest.mark.parametrize("T,Mp,N,K", [(1, 16, 300, 1024), (2, 16, 129, 2048), (5, 16, 64, 512), (8, 16, 40, 17408),
                                      (12, 16, 200, 768), (100, 112, 272, 768), (300, 384, 200, 512)])
def test_q3_k_matmul(rt, T, Mp, N, K):
    print(f"Q3_K T={T} Mp={Mp} N={N} K={K}", flush=True)
    eng = az.Engine(384, 17408)
    try:
        W = make_weights(az.Q3_K, N, K, seed=700 + T)
        x = make_acts(T, K, seed=710 + T, outliers=True)
        W6 = _q3k_as_q6k(W, N, K)
        assert np.array_equal(orc.dequant_rows(az.Q6_K, W6, N, K).view(np.uint32), orc.dequant_rows(az.Q3_K, W, N, K).view(np.uint32))
        w3 = eng.make_weight(az.Q3_K, N, K, W)
        w6 = eng.make_weight(az.Q6_K, N, K, W6)
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, K, K, Mp, T)
        rows = T if T <= 8 else Mp
        ys = []
        for w in (w3, w6):
            cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
            eng.matmul("q3_k", w, Mp, cb, N, 0, 0)
            ys.append(cb.read(np.float32, rows * N).reshape(rows, N)[:T])
            cb.free()
        aq, asc, _ = quantize_padded(x, Mp)
        ref = orc.matmul_ref(az.Q3_K, W, N, K, aq[:T], asc)
        assert np.isfinite(ys[0]).all()
        assert rel_err_rows(ys[0], ref).max() <= 1e-3
        if Mp > 16:
            assert np.array_equal(ys[0].view(np.uint32), ys[1].view(np.uint32))
        else:
            assert rel_err_rows(ys[0], ys[1]).max() <= 2e-5
        assert az.planes_bytes(az.Q3_K, N, K) == (az.gguf_bytes(az.Q3_K, N, K) + 15) // 16 * 16 == (N * K // 256 * 110 + 15) // 16 * 16
        assert az.lib.arcz_mem_size(az.lib.arcz_weight_raw(w3.h)) == az.planes_bytes(az.Q3_K, N, K)   # 3.44 bits a weight on the device
        xb.free(); w3.free(); w6.free()
    finally:
        eng.close()
