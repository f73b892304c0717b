"""Decode GEMV (1 token) and multi-token GEMV (2..8 tokens) on the GPU against the oracle.

f32 outputs: per token row max|y - ref| / max|ref| <= 1e-3 against the double-accumulated dequantized reference
(tools/ref_forward.cpp:268-303 semantics; the measure of bench/gemv_bench.cpp:199-214) -- the stated tolerance; the
observed error is float rounding only, so a much tighter bound against the engine-formula restatement is checked too.
int32 block sums: exact, through unit scales (every scale 1: the f32 output is the integer sum itself).
"""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import (ALL_TYPES, TYPES, TYPE_NAMES, make_acts, make_weights, mixed_err, quantize_padded, rel_err_rows,
                    unit_scale_acts, unit_scale_weights)

pytestmark = pytest.mark.gpu
TOL = 1e-3        # the tolerance the path is specified to
TIGHT = 2e-5      # what float rounding alone allows against the same-formula restatement


@pytest.fixture(scope="module")
def eng(rt):
    e = az.Engine(16, 17408)
    yield e
    e.close()


def run_gemv(eng, qtype, W, N, K, x, Mp, acc=0, c_init=None, ldc=None, c_off=0):
    T = x.shape[0]
    ldc = N + c_off if ldc is None else ldc
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T)
    cb = az.Runtime.alloc(T * ldc * 4)
    if c_init is None:
        cb.fill(0xFFFFFFFF)  # NaN poison (bench/gemv_bench.cpp:154-157)
    else:
        cb.write(c_init)
    eng.matmul("test", w, Mp, cb, ldc, c_off, acc)
    y = cb.read(np.float32, T * ldc).reshape(T, ldc)
    for b in (cb, xb):
        b.free()
    w.free()
    return y


@pytest.mark.parametrize("qtype", ALL_TYPES)
@pytest.mark.parametrize("T", [1, 2, 3, 5, 8])
def test_gemv_small_vs_oracle(eng, qtype, T):
    N, K, Mp = 264, 512, 16   # N not a multiple of the rows per work-group
    print(f"gemv {TYPE_NAMES[qtype]} T={T} N={N} K={K}", flush=True)
    W = make_weights(qtype, N, K, seed=11 + qtype)
    x = make_acts(T, K, seed=21 + T, outliers=True)
    y = run_gemv(eng, qtype, W, N, K, x, Mp)
    aq, asc, absum = quantize_padded(x, Mp)
    ref = orc.matmul_ref(qtype, W, N, K, aq[:T], asc)
    assert np.isfinite(y).all()
    assert rel_err_rows(y, ref).max() <= TOL
    form = orc.matmul_formula(qtype, 0, W, N, K, aq[:T], asc, absum)
    assert rel_err_rows(y, form).max() <= TIGHT
    print(f"  rel {rel_err_rows(y, ref).max():.2e} mixed {mixed_err(y, ref):.2e} vs formula {rel_err_rows(y, form).max():.2e}")


@pytest.mark.parametrize("qtype", ALL_TYPES)
@pytest.mark.parametrize("T", [1, 2, 7])
def test_gemv_block_sums_exact(eng, qtype, T):
    """Unit scales: the f32 output must be the exact integer dot product (all partial sums stay below 2^24)."""
    N, K = 96, 768
    W, wi = unit_scale_weights(qtype, N, K, seed=5)
    x = unit_scale_acts(T, K, seed=6)
    y = run_gemv(eng, qtype, W, N, K, x, 16)
    exact = x.astype(np.int64) @ wi.T
    assert np.abs(exact).max() < 2 ** 24
    assert np.array_equal(y.astype(np.int64), exact) and np.array_equal(y, exact.astype(np.float32))


@pytest.mark.parametrize("qtype,N,K,T", [(az.Q4_K, 17408, 5120, 1), (az.Q4_K, 5120, 17408, 2), (az.Q6_K, 4096, 5120, 1),
                                         (az.Q8_0, 4096, 4096, 4)])
def test_gemv_config_shapes_sampled(eng, qtype, N, K, T):
    """The decode shapes of the configs, checked on ~512 sampled rows (the reference samples ~4096, gemv_bench.cpp:202)
    plus determinism: two runs give the same bits."""
    print(f"gemv config {TYPE_NAMES[qtype]} N={N} K={K} T={T}", flush=True)
    W = make_weights(qtype, N, K, seed=3)
    x = make_acts(T, K, seed=4)
    y = run_gemv(eng, qtype, W, N, K, x, 16)
    y2 = run_gemv(eng, qtype, W, N, K, x, 16)
    assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))
    rows = np.arange(0, N, max(1, N // 512))
    rb = az.gguf_bytes(qtype, 1, K)
    Wr = np.concatenate([W[r * rb:(r + 1) * rb] for r in rows])
    aq, asc, _ = quantize_padded(x, 16)
    ref = orc.matmul_ref(qtype, Wr, len(rows), K, aq[:T], asc)
    err = rel_err_rows(y[:, rows], ref)
    print(f"  rel {err.max():.2e}")
    assert err.max() <= TOL


def test_gemv_accumulate_and_offset(eng):
    N, K, T, Mp = 128, 512, 3, 16
    W = make_weights(az.Q4_K, N, K, seed=8)
    x = make_acts(T, K, seed=9)
    ldc, c_off = 200, 40
    c0 = az.gen_normal(77, (T, ldc))
    y0 = run_gemv(eng, az.Q4_K, W, N, K, x, Mp)
    y = run_gemv(eng, az.Q4_K, W, N, K, x, Mp, acc=1, c_init=c0, ldc=ldc, c_off=c_off)
    assert np.array_equal(y[:, :c_off], c0[:, :c_off]) and np.array_equal(y[:, c_off + N:], c0[:, c_off + N:])
    assert np.array_equal(y[:, c_off:c_off + N], c0[:, c_off:c_off + N] + y0)


@pytest.mark.parametrize("qtype,F,K", [(az.Q4_K, 17408, 5120), (az.Q4_K, 264, 512), (az.Q6_K, 1024, 2048), (az.Q8_0, 512, 1024),
                                       (az.Q5_K, 776, 2560), (az.IQ4_XS, 128, 17408), (az.Q4_0, 520, 1024), (az.IQ3_S, 264, 2048),
                                       (az.IQ4_NL, 1032, 1536), (az.MXFP4, 136, 5120), (az.Q3_K, 264, 1024)])
def test_gemv_gu_equals_two_launches(eng, qtype, F, K):
    """Gate and up of one token in one launch (zero/engine.h:1124-1146): rows [0, F) of gate, then of up at C + F, bit
    for bit what the two launches give; and the cases that are not taken."""
    print(f"gemv_gu {TYPE_NAMES[qtype]} F={F} K={K}", flush=True)
    Wg, Wu = make_weights(qtype, F, K, seed=61), make_weights(qtype, F, K, seed=62)
    g, u = eng.make_weight(qtype, F, K, Wg), eng.make_weight(qtype, F, K, Wu)
    x = make_acts(1, K, seed=63, outliers=True)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, 16, 1)
    c2 = az.Runtime.alloc(2 * F * 4).fill(0xFFFFFFFF)
    eng.matmul("gate", g, 16, c2, 2 * F, 0, 0)
    eng.matmul("up", u, 16, c2, 2 * F, F, 0)
    want = c2.read(np.uint32, 2 * F)
    c1 = az.Runtime.alloc(2 * F * 4).fill(0xFFFFFFFF)
    assert eng.gemv_gu(g, u, 16, c1)
    got = c1.read(np.uint32, 2 * F)
    assert np.array_equal(got, want) and np.isfinite(got.view(np.float32)).all()
    aq, asc, _ = quantize_padded(x, 16)
    rows = np.arange(0, F, max(1, F // 256))
    rb = az.gguf_bytes(qtype, 1, K)
    for W, y in ((Wg, got[:F]), (Wu, got[F:])):
        ref = orc.matmul_ref(qtype, np.concatenate([W[r * rb:(r + 1) * rb] for r in rows]), len(rows), K, aq[:1], asc)
        assert rel_err_rows(y.view(np.float32)[rows][None], ref).max() <= TOL
    # not taken: two tokens in the chunk; matrices of different shapes
    eng.quantize(az.Runtime.from_numpy(make_acts(2, K, seed=64)), K, K, 16, 2)
    assert not eng.gemv_gu(g, u, 16, c1)
    eng.quantize(xb, K, K, 16, 1)
    if F > 8:
        w3 = eng.make_weight(qtype, F - 8, K, make_weights(qtype, F - 8, K, seed=65))
        assert not eng.gemv_gu(g, w3, 16, c1)
        w3.free()
    for b in (c1, c2, xb):
        b.free()
    g.free(); u.free()


@pytest.mark.parametrize("qtype,N,K,T", [(az.Q6_K, 1000, 512, 1), (az.Q4_K, 264, 512, 3), (az.Q8_0, 300, 17408, 2),
                                         (az.Q6_K, 520, 17408, 5), (az.Q4_K, 264, 1024, 8), (az.IQ4_NL, 300, 768, 2),
                                         (az.MXFP4, 264, 17408, 4), (az.Q4_0, 100, 512, 1), (az.IQ3_S, 200, 1024, 6)])
def test_gemv_softcap_output_head(eng, qtype, N, K, T):
    """The output head's soft cap (the reference's -DSOFTCAP=c, zero/kernels/decode.cl:882-886, 1029-1031): the GEMVs
    write c * tanh(v / c), then add C when accumulating.  LDS-staged and global-memory kernels, 1-8 tokens."""
    cap = 30.0
    print(f"softcap {TYPE_NAMES[qtype]} N={N} K={K} T={T}", flush=True)
    W = make_weights(qtype, N, K, seed=81)
    # (values large enough for the cap to bend them)
    x = make_acts(T, K, seed=82) * np.float32(40.0)
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, 16, T)
    plain = az.Runtime.alloc(T * N * 4)
    eng.matmul("head", w, 16, plain, N, 0, 0)
    y = plain.read(np.float32, T * N).reshape(T, N)
    w.set_softcap(cap)
    c0 = az.gen_normal(83, (T, N))
    capped, capped_acc = az.Runtime.alloc(T * N * 4).fill(0xFFFFFFFF), az.Runtime.from_numpy(c0)
    eng.matmul("head", w, 16, capped, N, 0, 0)
    eng.matmul("head", w, 16, capped_acc, N, 0, 1)
    yc = capped.read(np.float32, T * N).reshape(T, N)
    ya = capped_acc.read(np.float32, T * N).reshape(T, N)
    want = cap * np.tanh(y.astype(np.float64) / cap)
    assert np.abs(y).max() > cap / 2                               # the cap matters here
    assert np.abs(yc - want).max() <= 2e-6 * cap
    assert np.abs(ya - (c0 + yc)).max() <= 1e-6 * cap
    w.set_softcap(0.0)
    eng.matmul("head", w, 16, capped, N, 0, 0)
    assert np.array_equal(capped.read(np.uint32, T * N), y.view(np.uint32).ravel())
    for b in (plain, capped, capped_acc, xb):
        b.free()
    w.free()


@pytest.mark.parametrize("T,Mp", [(9, 16), (12, 16), (16, 16)])
def test_softcap_head_over_more_than_eight_rows_is_refused(eng, T, Mp):
    """Only the GEMVs of 1-8 tokens apply a matrix's logit soft cap: a capped matrix over more token rows is an error,
    not a matmul with uncapped results (one-pass engines too)."""
    N, K = 264, 512
    w = eng.make_weight(az.Q4_K, N, K, make_weights(az.Q4_K, N, K, seed=84))
    w.set_softcap(30.0)
    xb = az.Runtime.from_numpy(make_acts(T, K, seed=85))
    eng.quantize(xb, K, K, Mp, T)
    cb = az.Runtime.alloc(Mp * N * 4).fill(0)
    with pytest.raises(az.ArczError) as e:
        eng.matmul("head", w, Mp, cb, N, 0, 0)
    assert "soft cap" in str(e.value) and not cb.read(np.uint32, Mp * N).any()
    w.set_softcap(0.0)
    eng.matmul("head", w, Mp, cb, N, 0, 0)          # without the cap the same call goes through
    assert np.isfinite(cb.read(np.float32, Mp * N)).all()
    for b in (xb, cb):
        b.free()
    w.free()


def _sched(rows, g, wgs):
    """Engine::gemv_sched for one matrix: whole rounds << 10 | rows of the last, shorter pass."""
    full = rows // (g * wgs)
    tail = (rows - full * g * wgs + wgs - 1) // wgs or g   # (Q4_K, one or two tokens: a short last pass whatever its size)
    return (full << 10) | tail


@pytest.mark.parametrize("N,K,T", [(1000, 1024, 1), (1001, 1024, 2), (2176, 2048, 1), (333, 5120, 1), (96, 17408, 2)])
def test_gemv_row_schedule(eng, N, K, T):
    """The LDS-staged GEMV deals its rows out by the grid it is launched with; the schedule comes from the launcher
    (-DSCHED) or, left out, from the kernel's own arithmetic.  Whatever the grid and whoever works the schedule out, every
    row is computed once, by the same lanes in the same order: the output equals the engine's launch bit for bit."""
    qtype, Mp = az.Q4_K, 16
    print(f"gemv schedule N={N} K={K} T={T}", flush=True)
    W = make_weights(qtype, N, K, seed=5)
    x = make_acts(T, K, seed=6)
    ref = run_gemv(eng, qtype, W, N, K, x, Mp)
    units = K // 256 * 8
    lpr = next(l for l in (32, 64, 128, 256) if (units + l - 1) // l <= 6)
    pf, g, wpr = (units + lpr - 1) // lpr, 256 // lpr, max(1, lpr // 64)
    lds = T * 2 * units * 24 + (16 * g * wpr * T * 4 if wpr > 1 else 0)
    raw = az.Runtime.from_numpy(az.repack_planes(qtype, N, K, W))
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T)
    cb = az.Runtime.alloc(T * N * 4)
    npass = (N + g - 1) // g
    for wgs in sorted({1, 3, min(37, npass), max(1, npass // 2), npass}):
        for given in (0, 1, 2):   # the kernel's own schedule; the launcher's; the launcher's with non-temporal weight loads
            defs = f"-DQT={qtype} -DLPR={lpr} -DPF={pf}" + (f" -DTB={T}" if T > 1 else "") + f" -DLDS={lds}"
            if given:
                defs += f" -DSCHED={_sched(N, g, wgs) | ((1 << 30) if given == 2 else 0)}"
            k = az.Runtime.kernel("decode", defs, "gemv" if T == 1 else "gemv_mt")
            cb.fill(0xFFFFFFFF)
            args = [raw, N, K, None, eng.aq, eng.asc, eng.absum, Mp]
            args += [cb, 0, 0] if T == 1 else [T, cb, N, 0, 0]
            az.Runtime.launch(k, (wgs * 256,), (256,), args)
            y = cb.read(np.float32, T * N).reshape(T, N)
            assert np.array_equal(y.view(np.uint32), ref.view(np.uint32)), (wgs, given)
    for b in (raw, xb, cb):
        b.free()
