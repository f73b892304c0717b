"""IQ3_S weights (reference src/quants.h:240-262: d * (1 + 2 s) * a signed codebook magnitude, one s per 32 values).  The
device holds them in their own form (110 bytes per 256 values, the GGUF byte count).  The GEMVs (1-8 tokens) decode
them in registers through the codebook in LDS; the GEMM forms first write the matrix out as Q6_K planes, value for value
(same d, sub-scale 1 + 2 s for both halves of a block, q = value + 32: the place of the reference's decode pass), and run
the Q6_K tile kernels on that in the form for equal sub-scales (one product per block, the scale in the scale tile) --
so every chunk equals, to float rounding, what the same matrix uploaded as Q6_K superblocks gives.  All against the double-accumulated reference on the IQ3_S
rows themselves.  (MoE layers of IQ3_S experts: test_gpu_moe.py; a tensor from a GGUF file: test_gpu_gguf.py.)"""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import make_acts, make_weights, quantize_padded, rel_err_rows
from test_oracle_pins import _iq3s_as_q6k

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("T,Mp,N,K", [(1, 16, 300, 1024), (2, 16, 129, 2048), (5, 16, 64, 512), (100, 112, 272, 768),
                                      (300, 384, 200, 512)])
def test_iq3_s_matmul(rt, T, Mp, N, K):
    print(f"IQ3_S T={T} Mp={Mp} N={N} K={K}", flush=True)
    eng = az.Engine(384, 2048)
    try:
        W = make_weights(az.IQ3_S, N, K, seed=600 + T)
        x = make_acts(T, K, seed=610 + T, outliers=True)
        w3 = eng.make_weight(az.IQ3_S, N, K, W)
        w6 = eng.make_weight(az.Q6_K, N, K, _iq3s_as_q6k(W, N, K))
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, K, K, Mp, T)
        rows = T if T <= 8 else Mp
        ys = []
        for w in (w3, w6):
            cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
            eng.matmul("iq3_s", w, Mp, cb, N, 0, 0)
            ys.append(cb.read(np.float32, rows * N).reshape(rows, N)[:T])
            cb.free()
        aq, asc, _ = quantize_padded(x, Mp)
        ref = orc.matmul_ref(az.IQ3_S, W, N, K, aq[:T], asc)
        assert np.isfinite(ys[0]).all()
        assert rel_err_rows(ys[0], ref).max() <= 1e-3
        assert rel_err_rows(ys[0], ys[1]).max() <= 2e-5
        assert az.lib.arcz_mem_size(az.lib.arcz_weight_raw(w3.h)) == (az.gguf_bytes(az.IQ3_S, N, K) + 15) // 16 * 16
        xb.free(); w3.free(); w6.free()
    finally:
        eng.close()
