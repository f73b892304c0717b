"""Seeded random cases over everything a matmul call can vary at once: the eleven weight types, 1 to 2047 tokens in
chunks with and without an empty group of 16 rows, 1 to 40000 weight rows, K of 1 to 68 superblocks, an output wider
than the matrix (ldc > N) at a column offset, the three epilogues (store, add to C, SwiGLU on the gate in C), per-32
and per-256 activation scales.  Each case against the double-accumulated dequantized reference (1e-3), the columns of
C outside the output bit for bit untouched, padding rows of a stored chunk zero.  The matrix-vector kernels (at most 8
tokens) store or add; the SwiGLU epilogue with them is refused with an error, which the cases check as well."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import ALL_TYPES, TYPE_NAMES, make_acts, make_weights, mixed_err, rel_err_rows

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _draw(rng):
    qt = ALL_TYPES[int(rng.integers(0, len(ALL_TYPES)))]
    kind = int(rng.integers(0, 4))
    if kind == 0:      # a few tokens: the matrix-vector forms
        T, K, N = int(rng.integers(1, 17)), 256 * int(rng.choice([1, 2, 3, 5, 8, 13, 20, 24, 25, 40, 48, 68])), int(rng.integers(1, 3000))
    elif kind == 1:    # short chunks
        T, K, N = int(rng.integers(17, 300)), 256 * int(rng.choice([1, 2, 3, 4, 7, 20])), int(rng.integers(1, 1500))
    elif kind == 2:    # long chunks
        T, K, N = int(rng.integers(300, 2048)), 256 * int(rng.choice([1, 2, 3, 5])), int(rng.integers(1, 800))
    else:              # many rows, few tokens
        T, K, N = int(rng.integers(1, 33)), 256 * int(rng.choice([1, 4, 6])), int(rng.integers(3000, 40000))
    while N * K * T > 3e9:
        N = max(1, N // 2)
    Mp = min(2048, (T + 15) // 16 * 16 + 16 * int(rng.integers(0, 2)))
    pad = int(rng.choice([0, 0, 1, 3, 4, 16, 100]))
    c_off = int(rng.choice([0, 0, 1, 2, 4, 64])) if pad else 0
    return qt, T, Mp, N, K, N + pad + c_off, c_off, int(rng.choice([0, 0, 1, 2])), int(rng.choice([1, 1, 0]))


@pytest.mark.parametrize("seed,count", [(11, 150), (12, 150)])
def test_random_matmul_cases(rt, seed, count):
    rng = np.random.default_rng(seed)
    eng = az.Engine(2048, 17408)
    refused = 0
    for i in range(count):
        qt, T, Mp, N, K, ldc, c_off, acc, a32 = _draw(rng)
        desc = f"random case {seed}/{i} {TYPE_NAMES[qt]} T={T} Mp={Mp} N={N} K={K} ldc={ldc} c_off={c_off} acc={acc} act32={a32}"
        print(desc, flush=True)
        W = make_weights(qt, N, K, seed=seed * 1000 + i)
        x = make_acts(T, K, seed=seed * 1000 + i + 500, outliers=True)
        w = eng.make_weight(qt, N, K, W)
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, K, K, Mp, T, act32=a32)
        rows = T if T <= 8 else Mp
        c0 = rng.standard_normal((rows, ldc)).astype(np.float32)
        cb = az.Runtime.from_numpy(c0)
        if T <= 8 and acc == 2:
            with pytest.raises(az.ArczError):
                eng.matmul("random", w, Mp, cb, ldc, c_off, acc, act32=bool(a32))
            refused += 1
        else:
            eng.matmul("random", w, Mp, cb, ldc, c_off, acc, act32=bool(a32))
            y = cb.read(np.float32, rows * ldc).reshape(rows, ldc)
            xp = np.zeros((Mp, K), np.float32)
            xp[:T] = x
            raq, rasc, _ = orc.quantize_act(xp, act32=bool(a32))
            asc = rasc if a32 else np.ascontiguousarray(np.repeat(rasc, 8, axis=0))
            ref = orc.matmul_ref(qt, W, N, K, raq[:T], asc)
            g = c0[:T, c_off:c_off + N].astype(np.float64)
            if acc == 1:
                ref = ref + g
            elif acc == 2:
                ref = ref * (g / (1.0 + np.exp(-g)))
            out = y[:T, c_off:c_off + N]
            assert np.isfinite(out).all(), desc
            assert (mixed_err(out, ref) if acc else rel_err_rows(out, ref).max()) <= TOL, desc
            outside = np.ones(ldc, bool)
            outside[c_off:c_off + N] = False
            assert np.array_equal(y[:, outside].view(np.uint32), c0[:, outside].view(np.uint32)), desc
            if rows > T and acc == 0:
                assert not y[T:, c_off:c_off + N].any(), desc
        for b in (cb, xb):
            b.free()
        w.free()
    eng.close()
    assert refused < count // 4
