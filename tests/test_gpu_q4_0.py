"""Q4_0 weights (reference src/quants.h:136-148: Q8_0 with q - 8 in four bits).  The device holds them in their own
4-bit form (128 bytes of nibbles and 8 f16 scales per 256 values: the GGUF byte count) and every matmul form decodes
them in registers: GEMV, multi-token GEMV and GEMM against the double-accumulated reference on the Q4_0 rows themselves,
and against the same values uploaded as Q8_0 blocks (the same integer sums and scales: equal to float rounding)."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import make_acts, make_weights, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu


def _as_q8_0(W4, N, K):
    """The same values as GGUF Q8_0 blocks (f16 d kept, q - 8 as int8)."""
    b = W4.reshape(N * K // 32, 18)
    out = np.empty((N * K // 32, 34), np.uint8)
    out[:, 0:2] = b[:, 0:2]
    out[:, 2:18] = ((b[:, 2:] & 0xF).astype(np.int16) - 8).astype(np.int8).view(np.uint8)
    out[:, 18:34] = ((b[:, 2:] >> 4).astype(np.int16) - 8).astype(np.int8).view(np.uint8)
    return out.reshape(-1)


@pytest.mark.parametrize("T,Mp,N,K", [(1, 16, 300, 1024), (2, 16, 129, 4096), (5, 16, 64, 512), (100, 112, 272, 768),
                                      (300, 384, 200, 512)])
def test_q4_0_matmul(rt, T, Mp, N, K):
    print(f"Q4_0 T={T} Mp={Mp} N={N} K={K}", flush=True)
    eng = az.Engine(384, 4096)
    try:
        W = make_weights(az.Q4_0, N, K, seed=500 + T)
        x = make_acts(T, K, seed=510 + T, outliers=True)
        w4 = eng.make_weight(az.Q4_0, N, K, W)
        w8 = eng.make_weight(az.Q8_0, N, K, _as_q8_0(W, N, K))
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, K, K, Mp, T)
        rows = T if T <= 8 else Mp
        ys = []
        for w in (w4, w8):
            cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
            eng.matmul("q4_0", w, Mp, cb, N, 0, 0)
            ys.append(cb.read(np.float32, rows * N).reshape(rows, N)[:T])
            cb.free()
        aq, asc, _ = quantize_padded(x, Mp)
        ref = orc.matmul_ref(az.Q4_0, W, N, K, aq[:T], asc)
        assert np.isfinite(ys[0]).all()
        assert rel_err_rows(ys[0], ref).max() <= 1e-3
        assert rel_err_rows(ys[0], ys[1]).max() <= 2e-5
        assert az.planes_bytes(az.Q4_0, N, K) == az.gguf_bytes(az.Q4_0, N, K) == N * K // 32 * 18
        assert az.lib.arcz_mem_size(az.lib.arcz_weight_raw(w4.h)) == az.gguf_bytes(az.Q4_0, N, K)   # 4.5 bits a weight on the device
        xb.free(); w4.free(); w8.free()
    finally:
        eng.close()
