"""gemv_mm: the matrix-vector form for a few tokens on the matrix pipe (Q4_K, Q5_K, Q6_K, Q8_0, Q4_0,
IQ4_XS, IQ3_S, IQ4_NL, MXFP4, Q3_K, IQ3_XXS).  The engine takes it for 9-16 tokens in a
16-row chunk, for 5-8 tokens, and for 3-4 tokens whose activations do not fit the LDS of the dot-product kernels; every
case here lands on it.  Against the double-accumulated dequantized reference (1e-3 as max|err| / max|ref| per token
row), with unit scales against the exact integer sums, with K in one slice and in several (later slices accumulate),
storing and accumulating, rows that do not fill a group of 16."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import make_acts, make_weights, pad_rows, quantize_padded, rel_err_rows, unit_scale_acts, unit_scale_weights

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng(rt):
    e = az.Engine(16, 17408)
    yield e
    e.close()


CASES = [(7, 100, 256), (8, 1000, 5120), (9, 333, 2048), (13, 4097, 1024), (16, 64, 6144), (16, 250, 6400),
         (3, 77, 17408), (6, 300, 17408), (12, 129, 17408), (5, 200, 5120), (4, 5120, 17408),
         # rounds of one, two and four waves a group, then the rest spread wider
         (7, 33000, 256), (16, 20000, 1024), (8, 17408, 512), (11, 17408, 5120),
         # several slices of K inside the kernel (more than 12 groups a compute unit: K is not shared out over
         # work-groups): the sums wait in LDS, or (13 groups to a work-group) are added to C slice by slice
         (8, 53000, 6400)]


def _parity(eng, qt, T, N, K):
    print(f"gemv_mm type={qt} T={T} N={N} K={K}", flush=True)
    W = make_weights(qt, N, K, seed=800 + T)
    x = make_acts(T, K, seed=801 + T, outliers=True)
    w = eng.make_weight(qt, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, 16, T)
    rows = T if T <= 8 else 16
    cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
    eng.matmul("mm", w, 16, cb, N, 0, 0)
    y = cb.read(np.float32, rows * N).reshape(rows, N)
    aq, asc, _ = quantize_padded(x, 16)
    ref = orc.matmul_ref(qt, W, N, K, aq[:T], asc)
    assert np.isfinite(y).all()
    assert rel_err_rows(y[:T], ref).max() <= 1e-3
    if rows > T:
        assert not y[T:].any()                       # the chunk's padding rows: zeros, as the GEMM writes them
    eng.matmul("mm", w, 16, cb, N, 0, 1)             # accumulate: C + the same product
    y2 = cb.read(np.float32, rows * N).reshape(rows, N)
    assert rel_err_rows(y2[:T], 2.0 * ref).max() <= 1e-3
    # the same bits on every run
    eng.matmul("mm", w, 16, cb, N, 0, 0)
    assert np.array_equal(cb.read(np.float32, rows * N).reshape(rows, N), y)
    for b in (cb, xb):
        b.free()
    w.free()


@pytest.mark.parametrize("T,N,K", CASES)
def test_gemv_mm_parity(eng, T, N, K):
    _parity(eng, az.Q4_K, T, N, K)


# the other types of the matrix-pipe form: a slice of K, several slices (22 / 20 / 24 superblocks at most for Q5_K / Q6_K /
# Q8_0; shared out over work-groups with a reduce behind them, or -- the last case -- walked inside the kernel), rows
# that do not fill a group, work-groups with several groups, more groups than wait in LDS
CASES_TYPES = [(8, 100, 256), (16, 333, 2048), (13, 1000, 5120), (7, 129, 17408), (16, 5120, 6400), (9, 17408, 1024),
               (8, 53000, 6400)]


@pytest.mark.parametrize("T,N,K", CASES_TYPES)
@pytest.mark.parametrize("qt", [az.Q5_K, az.Q6_K, az.Q8_0, az.Q4_0, az.IQ4_XS, az.IQ3_S, az.IQ4_NL, az.MXFP4, az.Q3_K, az.IQ3_XXS])
def test_gemv_mm_parity_types(eng, qt, T, N, K):
    _parity(eng, qt, T, N, K)


@pytest.mark.parametrize("qt,T,N,K", [(az.Q4_K, 7, 200, 1024), (az.Q4_K, 12, 130, 17408), (az.Q6_K, 16, 96, 6400),
                                      (az.Q8_0, 5, 333, 8192)])
def test_gemv_mm_into_a_wider_output(eng, qt, T, N, K):
    """The output as columns [c_off, c_off + N) of rows of ldc values, stored and accumulated: nothing outside them is
    touched (K within a slice, and shared out over work-groups with the reduce behind them)."""
    print(f"gemv_mm wide output type={qt} T={T} N={N} K={K}", flush=True)
    ldc, c_off = N + 24, 8
    W = make_weights(qt, N, K, seed=840 + T)
    x = make_acts(T, K, seed=841 + T, outliers=True)
    w = eng.make_weight(qt, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, 16, T)
    rows = T if T <= 8 else 16
    c0 = np.random.default_rng(842).standard_normal((rows, ldc)).astype(np.float32)
    cb = az.Runtime.alloc(rows * ldc * 4)
    aq, asc, _ = quantize_padded(x, 16)
    ref = orc.matmul_ref(qt, W, N, K, aq[:T], asc)
    for acc in (0, 1):
        cb.write(c0)
        eng.matmul("mm", w, 16, cb, ldc, c_off, acc)
        y = cb.read(np.float32, rows * ldc).reshape(rows, ldc)
        assert np.array_equal(y[:, :c_off], c0[:, :c_off]) and np.array_equal(y[:, c_off + N:], c0[:, c_off + N:])
        want = ref + (c0[:T, c_off:c_off + N] if acc else 0.0)
        assert rel_err_rows(y[:T, c_off:c_off + N], want).max() <= 1e-3
        if rows > T:
            pad = y[T:, c_off:c_off + N]
            assert np.array_equal(pad, c0[T:, c_off:c_off + N]) if acc else not pad.any()
    for b in (cb, xb):
        b.free()
    w.free()


@pytest.mark.parametrize("T,N,K", [(8, 48, 512), (16, 37, 7168)])
@pytest.mark.parametrize("qt", [az.Q4_K, az.Q5_K, az.Q6_K, az.Q4_0, az.IQ4_XS, az.IQ3_S, az.IQ4_NL, az.MXFP4, az.Q3_K, az.IQ3_XXS])
def test_gemv_mm_unit_scales_exact(eng, qt, T, N, K):
    """All scales 1: the f32 output is the exact integer sum (partial sums stay below 2^24)."""
    W, wi = unit_scale_weights(qt, N, K, seed=820)
    x = unit_scale_acts(T, K, seed=821)
    w = eng.make_weight(qt, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, 16, T)
    rows = T if T <= 8 else 16
    cb = az.Runtime.alloc(rows * N * 4)
    eng.matmul("mm", w, 16, cb, N, 0, 0)
    y = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
    assert np.array_equal(y, (x.astype(np.int64) @ wi.T).astype(np.float32))
    for b in (cb, xb):
        b.free()
    w.free()
