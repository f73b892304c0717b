"""The matmul entry point that allocates nothing (arcz_engine_matmul_noalloc) against the ordinary one
(arcz_engine_matmul), through the C ABI: the same kernels on the library's static device scratch instead of the
engine's workspace, so the outputs must be equal bit for bit.  Two calls in a row, the second with a smaller input (the
array keeps the first call's partial tiles), every matmul form (only the short-chunk GEMM uses the scratch), the
device-memory count unchanged by the calls, and the refusal of a launch whose partial tiles would not fit the array."""
import ctypes as C

import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import make_acts, make_weights, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu


def both(eng, qtype, N, K, T, Mp, seed, acc=0):
    """(ordinary, no-alloc) outputs of one matmul on the same inputs, and the device bytes around the no-alloc call."""
    W = make_weights(qtype, N, K, seed=seed)
    w = eng.make_weight(qtype, N, K, W)
    x = make_acts(T, K, seed=seed + 1, outliers=True)
    xb = az.Runtime.from_numpy(x)
    rows = Mp if T > 8 else T
    c0 = az.gen_normal(seed + 2, (rows, N))
    ca, cb = az.Runtime.from_numpy(c0), az.Runtime.from_numpy(c0)
    eng.quantize(xb, K, K, Mp, T)
    eng.matmul("plain", w, Mp, ca, N, 0, acc)
    before = az.lib.arcz_device_bytes()
    eng.matmul_noalloc("noalloc", w, Mp, cb, N, 0, acc)
    after = az.lib.arcz_device_bytes()
    ya = ca.read(np.uint32, rows * N)
    yb = cb.read(np.uint32, rows * N)
    for b in (ca, cb, xb):
        b.free()
    w.free()
    return ya, yb, before, after


def test_noalloc_equals_matmul_two_calls_in_a_row(rt):
    az.lib.arcz_device_bytes.restype = C.c_size_t
    eng = az.Engine(512, 5120)
    try:
        # short chunks over a long K: K shared out over work-groups, partial tiles in the scratch.  The larger first.
        for qtype, N, K, T, Mp in [(az.Q4_K, 2176, 5120, 128, 128), (az.Q4_K, 200, 4096, 20, 32),
                                   (az.Q6_K, 1024, 5120, 64, 64), (az.Q8_0, 130, 4096, 40, 48), (az.Q5_K, 300, 2560, 17, 32)]:
            for acc in (0, 1):
                print(f"noalloc split-K type {qtype} N={N} K={K} T={T} acc={acc}", flush=True)
                ya, yb, b0, b1 = both(eng, qtype, N, K, T, Mp, seed=3 + T, acc=acc)
                assert np.array_equal(ya, yb) and b0 == b1
                assert np.isfinite(ya.view(np.float32)).all()
        # the forms that use no scratch go through the same entry point: GEMV, multi-token GEMV, matrix-pipe GEMV, GEMM
        for qtype, N, K, T, Mp in [(az.Q4_K, 264, 512, 1, 16), (az.Q6_K, 264, 512, 3, 16), (az.Q4_K, 264, 1024, 12, 16),
                                   (az.Q4_K, 4352, 1024, 512, 512), (az.Q8_0, 520, 512, 300, 384)]:
            print(f"noalloc type {qtype} N={N} K={K} T={T}", flush=True)
            ya, yb, b0, b1 = both(eng, qtype, N, K, T, Mp, seed=50 + T)
            assert np.array_equal(ya, yb) and b0 == b1
    finally:
        eng.close()


def _free_device_bytes():
    """hipMemGetInfo's free bytes, asked of the HIP runtime the library itself runs on."""
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


@pytest.mark.parametrize("qtype,N,K,T,Mp", [(az.Q6_K, 1040, 6144, 12, 16),    # gemv_mm, K shared out: partial sums in the scratch
                                            (az.Q4_K, 1040, 7168, 7, 16),
                                            (az.Q4_K, 2176, 5120, 128, 128),  # the short-chunk GEMM's partial tiles
                                            (az.Q4_K, 264, 1024, 1, 16)])
def test_noalloc_as_the_first_call_of_a_fresh_engine(rt, qtype, N, K, T, Mp):
    """No ordinary matmul has run before it on this engine (no kernel object of the form exists yet, no workspace has
    been touched): the result is held to the oracle, and the device's free memory is what it was before the call."""
    print(f"noalloc first call type {qtype} N={N} K={K} T={T}", flush=True)
    eng = az.Engine(Mp, 8192)
    try:
        W = make_weights(qtype, N, K, seed=77)
        w = eng.make_weight(qtype, N, K, W)
        x = make_acts(T, K, seed=78, outliers=True)
        xb = az.Runtime.from_numpy(x)
        rows = Mp if T > 8 else T
        cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
        eng.quantize(xb, K, K, Mp, T)
        az.Runtime.sync()
        free0, bytes0 = _free_device_bytes(), az.lib.arcz_device_bytes()
        eng.matmul_noalloc("first", w, Mp, cb, N, 0, 0)
        az.Runtime.sync()
        assert _free_device_bytes() == free0 and az.lib.arcz_device_bytes() == bytes0
        y = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
        aq, asc, _ = quantize_padded(x, Mp)
        ref = orc.matmul_ref(qtype, W, N, K, aq[:T], asc)
        assert np.isfinite(y).all() and rel_err_rows(y, ref).max() <= 1e-3
        ca = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
        eng.matmul("plain", w, Mp, ca, N, 0, 0)                 # and the ordinary entry point gives the same bits
        assert np.array_equal(ca.read(np.uint32, rows * N).reshape(rows, N)[:T], y.view(np.uint32))
        for b in (ca, cb, xb):
            b.free()
        w.free()
    finally:
        eng.close()


def test_noalloc_refuses_what_does_not_fit(rt, monkeypatch):
    """Eight pieces forced on a chunk whose partial tiles take 8 x 512 x 4352 x 4 = 71 MB: past the 32 MiB array."""
    monkeypatch.setenv("ARCZ_Q4_SPLITK", "8")   # (read when an engine is made)
    eng = az.Engine(512, 5120)
    try:
        N, K, T = 4352, 5120, 512
        w = eng.make_weight(az.Q4_K, N, K, make_weights(az.Q4_K, N, K, seed=9))
        xb = az.Runtime.from_numpy(make_acts(T, K, seed=10))
        eng.quantize(xb, K, K, T, T)
        cb = az.Runtime.alloc(T * N * 4).fill(0)
        with pytest.raises(az.ArczError) as e:
            eng.matmul_noalloc("big", w, T, cb, N, 0, 0)
        assert "static scratch holds 33554432" in str(e.value) and "71303168" in str(e.value)
        assert not cb.read(np.uint32, T * N).any()          # nothing was launched
        eng.matmul("big", w, T, cb, N, 0, 0)                # the ordinary entry point grows its own workspace
        assert np.isfinite(cb.read(np.float32, T * N)).all()
        for b in (cb, xb):
            b.free()
        w.free()
    finally:
        eng.close()
