"""A seeded sweep over ragged shapes, so that every launch form the engine can pick is exercised somewhere: lanes per
row 32 / 64 / 128 / 256 and 1-6 units per lane for the GEMVs, every token count 1-8, rows that do not fill a pass,
GEMM chunks that do not fill a tile in either direction, the short-chunk tile form, all four weight types.  Each case
against the double-accumulated dequantized reference (tolerance 1e-3 as max|err| / max|ref| per token row)."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import TYPES, TYPE_NAMES, make_acts, make_weights, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _cases(seed, n, kind):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        qt = TYPES[i % len(TYPES)]
        if kind == "gemv":
            K = 256 * int(rng.choice([1, 2, 3, 5, 8, 12, 16, 20, 24, 31, 40, 48, 68]))
            N = int(rng.integers(1, 700))
            T = 1 + i % 8
        else:
            K = 256 * int(rng.choice([1, 2, 3, 4, 6, 11]))
            N = int(rng.integers(1, 520))
            T = int(rng.integers(9, 400))
        out.append((qt, N, K, T, 1000 * seed + i))
    return out


@pytest.fixture(scope="module")
def eng(rt):
    e = az.Engine(512, 17408)
    yield e
    e.close()


def _run(eng, qt, N, K, T, Mp, seed):
    W = make_weights(qt, N, K, seed=seed)
    x = make_acts(T, K, seed=seed + 1, outliers=True)
    w = eng.make_weight(qt, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T)
    rows = T if T <= 8 else Mp
    cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
    eng.matmul("sweep", w, Mp, cb, N, 0, 0)
    y = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
    aq, asc, _ = quantize_padded(x, Mp)
    ref = orc.matmul_ref(qt, W, N, K, aq[:T], asc)
    for b in (cb, xb):
        b.free()
    w.free()
    return y, ref


@pytest.mark.parametrize("qt,N,K,T,seed", _cases(7, 48, "gemv"))
def test_gemv_shapes(eng, qt, N, K, T, seed):
    print(f"sweep gemv {TYPE_NAMES[qt]} N={N} K={K} T={T}", flush=True)
    y, ref = _run(eng, qt, N, K, T, 16, seed)
    assert np.isfinite(y).all()
    assert rel_err_rows(y, ref).max() <= TOL


@pytest.mark.parametrize("qt,N,K,T,seed", _cases(9, 30, "gemm"))
def test_gemm_shapes(eng, qt, N, K, T, seed):
    Mp = min(512, (T + 15) // 16 * 16)
    print(f"sweep gemm {TYPE_NAMES[qt]} N={N} K={K} T={T} Mp={Mp}", flush=True)
    y, ref = _run(eng, qt, N, K, T, Mp, seed)
    assert np.isfinite(y).all()
    assert rel_err_rows(y, ref).max() <= TOL
