"""Activation quantizer on the GPU against the oracle: int8 values, scales (as bit patterns) and per-16 sums must be
equal bit for bit (reference src/quants.h:626-643 == zero/kernels/ops.cl:38-72)."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import make_acts, pad_rows

pytestmark = pytest.mark.gpu


def run_quant(eng, x, Mp):
    T, K = x.shape
    xb = az.Runtime.from_numpy(x)
    # poison the outputs first: a missing store shows up
    eng.aq.fill(0x7B7B7B7B)
    eng.asc.fill(0xFFFFFFFF)
    eng.absum.fill(0x7B7B7B7B)
    eng.quantize(xb, K, K, Mp, T)
    out = eng.read_activations(K, Mp)
    xb.free()
    return out


def check(eng, x, Mp):
    aq, asc, absum = run_quant(eng, x, Mp)
    raq, rasc, rabsum = orc.quantize_act(pad_rows(x, Mp))
    assert np.array_equal(aq, raq)
    assert np.array_equal(asc.view(np.uint32), rasc.view(np.uint32))
    assert np.array_equal(absum, rabsum)


@pytest.fixture(scope="module")
def eng(rt):
    e = az.Engine(1024, 5120)
    yield e
    e.close()


@pytest.mark.parametrize("T,Mp,K", [(1, 1, 5120), (1, 16, 256), (5, 16, 512), (64, 64, 4096), (200, 256, 5120),
                                    (512, 512, 4096), (1000, 1024, 1024)])
def test_quant_matches_oracle(eng, T, Mp, K):
    print(f"quant T={T} Mp={Mp} K={K}", flush=True)
    check(eng, make_acts(T, K, seed=100 + T, outliers=True), Mp)


def test_quant_special_blocks(eng):
    K = 256
    x = np.zeros((4, K), np.float32)
    x[0, 32:64] = -3.0                     # a block whose maximum is negative, all equal
    x[1, :32] = np.linspace(-1, 1, 32)     # plain
    x[1, 64:96] = 0.0                      # a zero block inside a row: scale 0, q 0
    # ties: v * inv = k + 0.5 exactly (amax 127 -> inv 1): round to even
    x[2, :32] = np.array([127.0] + [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5] * 4 + [0.0] * 3, np.float32)
    x[3, :] = 1e-30                        # tiny values: 127 / amax is huge but finite
    check(eng, x, 16)
    aq, asc, absum = run_quant(eng, x, 16)
    assert aq[0, 32:64].tolist() == [-127] * 32 and asc[1, 0] == np.float32(3.0) / np.float32(127.0)
    assert asc[2, 1] == 0.0 and not aq[1, 64:96].any()
    assert aq[2, 1:8].tolist() == [0, 2, 2, 0, -2, -2, 4]
    assert absum[2, 0] == aq[0, 32:48].astype(np.int32).sum()


def test_quant_full_config_sizes(eng, rt):
    """The headline configuration's activation shape (8192 x 5120) through size-independent properties: the row of maximum magnitude of
    every block maps to +-127, sums are the sums of the int8 values, padding rows are zero; and equality with the
    oracle on a sample of rows."""
    big = az.Engine(8192, 5120)
    try:
        T = K = None
        T, Mp, K = 8000, 8192, 5120
        x = make_acts(T, K, seed=7)
        aq, asc, absum = run_quant(big, x, Mp)
        assert not aq[T:].any() and not asc[:, T:].any() and not absum[:, T:].any()
        assert np.array_equal(np.abs(aq[:T].reshape(T, K // 32, 32)).max(axis=2), np.full((T, K // 32), 127))
        assert np.array_equal(aq.reshape(Mp, K // 16, 16).astype(np.int32).sum(axis=2).T, absum.astype(np.int32))
        rows = np.arange(0, T, 97)
        raq, rasc, rabsum = orc.quantize_act(x[rows])
        assert np.array_equal(aq[rows], raq)
        assert np.array_equal(asc[:, rows].view(np.uint32), rasc.view(np.uint32))
        assert np.array_equal(absum[:, rows], rabsum)
    finally:
        big.close()
