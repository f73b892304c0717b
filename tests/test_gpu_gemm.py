"""Prefill GEMM (int8 MFMA) on the GPU against the oracle: tolerance 1e-3 of the f32 reference per token row, exact
integer block sums through unit scales, the three epilogues, agreement with the GEMV on the same inputs, determinism."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import (ALL_TYPES, TYPES, TYPE_NAMES, make_acts, make_weights, mixed_err, quantize_padded, rel_err_rows,
                    unit_scale_acts, unit_scale_weights)

pytestmark = pytest.mark.gpu
TOL = 1e-3
TIGHT = 2e-5


@pytest.fixture(scope="module")
def eng(rt):
    e = az.Engine(512, 5120)
    yield e
    e.close()


def run_gemm(eng, qtype, W, N, K, x, Mp, acc=0, c_init=None, ldc=None, c_off=0):
    T = x.shape[0]
    ldc = N + c_off if ldc is None else ldc
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T)
    cb = az.Runtime.alloc(Mp * ldc * 4)
    if c_init is None:
        cb.fill(0xFFFFFFFF)
    else:
        cb.write(c_init)
    eng.matmul("test", w, Mp, cb, ldc, c_off, acc)
    y = cb.read(np.float32, Mp * ldc).reshape(Mp, ldc)
    for b in (cb, xb):
        b.free()
    w.free()
    return y


@pytest.mark.parametrize("qtype", ALL_TYPES)
@pytest.mark.parametrize("T,Mp,N,K", [(16, 16, 64, 256), (100, 112, 272, 512), (128, 128, 128, 1024), (300, 384, 384, 768),
                                      (180, 192, 520, 512)])
def test_gemm_vs_oracle(eng, qtype, T, Mp, N, K):
    print(f"gemm {TYPE_NAMES[qtype]} T={T} Mp={Mp} N={N} K={K}", flush=True)
    W = make_weights(qtype, N, K, seed=31 + qtype)
    x = make_acts(T, K, seed=41 + T, outliers=True)
    y = run_gemm(eng, qtype, W, N, K, x, Mp)
    aq, asc, absum = quantize_padded(x, Mp)
    ref = orc.matmul_ref(qtype, W, N, K, aq[:T], asc)
    assert np.isfinite(y).all()
    assert not y[T:].any()                      # padding rows: zero activations give exact zeros
    err = rel_err_rows(y[:T], ref)
    form = orc.matmul_formula(qtype, 1, W, N, K, aq[:T], asc, absum)
    print(f"  rel {err.max():.2e} mixed {mixed_err(y[:T], ref):.2e} vs formula {rel_err_rows(y[:T], form).max():.2e}")
    assert err.max() <= TOL
    assert rel_err_rows(y[:T], form).max() <= TIGHT
    y2 = run_gemm(eng, qtype, W, N, K, x, Mp)
    assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))   # bit-identical run to run


@pytest.mark.parametrize("qtype", ALL_TYPES)
def test_gemm_block_sums_exact(eng, qtype):
    T, N, K = 160, 160, 512
    W, wi = unit_scale_weights(qtype, N, K, seed=15)
    x = unit_scale_acts(T, K, seed=16)
    y = run_gemm(eng, qtype, W, N, K, x, 160)
    exact = x.astype(np.int64) @ wi.T
    assert np.abs(exact).max() < 2 ** 24
    assert np.array_equal(y, exact.astype(np.float32))


@pytest.mark.parametrize("qtype", ALL_TYPES)
def test_gemm_matches_gemv(eng, qtype):
    """Rows 0..7 of a 16-row GEMM against the 8-token GEMV on the same inputs: both within tolerance of the same
    reference and of each other."""
    N, K, T = 192, 1024, 16
    W = make_weights(qtype, N, K, seed=51)
    x = make_acts(T, K, seed=52)
    yg = run_gemm(eng, qtype, W, N, K, x, 16)
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(x[:8])
    eng.quantize(xb, K, K, 16, 8)
    cb = az.Runtime.alloc(8 * N * 4)
    eng.matmul("test", w, 16, cb, N, 0, 0)
    yv = cb.read(np.float32, 8 * N).reshape(8, N)
    cb.free(); xb.free(); w.free()
    assert rel_err_rows(yg[:8], yv).max() <= TIGHT


def test_gemm_epilogues(eng):
    qtype, T, Mp, N, K = az.Q4_K, 64, 64, 128, 512
    W = make_weights(qtype, N, K, seed=61)
    x = make_acts(T, K, seed=62)
    ldc, c_off = 300, 100
    c0 = az.gen_normal(63, (Mp, ldc))
    y0 = run_gemm(eng, qtype, W, N, K, x, Mp)
    ya = run_gemm(eng, qtype, W, N, K, x, Mp, acc=1, c_init=c0, ldc=ldc, c_off=c_off)
    assert np.array_equal(ya[:, :c_off], c0[:, :c_off]) and np.array_equal(ya[:, c_off + N:], c0[:, c_off + N:])
    assert np.array_equal(ya[:, c_off:c_off + N], y0 + c0[:, c_off:c_off + N])
    ys = run_gemm(eng, qtype, W, N, K, x, Mp, acc=2, c_init=c0, ldc=ldc, c_off=c_off)
    g = c0[:, c_off:c_off + N].astype(np.float64)
    want = y0.astype(np.float64) * (g / (1.0 + np.exp(-g)))   # C = silu(C) * result (gemm.cl:562-565)
    assert np.abs(ys[:, c_off:c_off + N] - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(ys[:, :c_off], c0[:, :c_off])


@pytest.mark.parametrize("qtype", [az.Q4_K, az.Q5_K])
@pytest.mark.parametrize("T,Mp,N,K", [(64, 64, 130, 4096), (40, 48, 300, 5120), (100, 112, 260, 2560), (128, 128, 128, 4096),
                                      (20, 32, 200, 4096), (17, 32, 129, 2560)])
def test_gemm_split_k(eng, qtype, T, Mp, N, K):
    """Short Q4_K / Q5_K chunks whose tiles are few: K shared out over several work-groups per tile, partial tiles added
    in a fixed order by a second kernel that also applies c_off and the accumulate mode (tiles of 32 tokens up to 32
    tokens, of 64 up to 64, of 128 above).  Parity with the oracle, the three epilogues, the same bits on every run."""
    print(f"gemm split-K {TYPE_NAMES[qtype]} T={T} Mp={Mp} N={N} K={K}", flush=True)
    W = make_weights(qtype, N, K, seed=71)
    x = make_acts(T, K, seed=72 + T, outliers=True)
    y0 = run_gemm(eng, qtype, W, N, K, x, Mp)
    aq, asc, absum = quantize_padded(x, Mp)
    ref = orc.matmul_ref(qtype, W, N, K, aq[:T], asc)
    assert rel_err_rows(y0[:T], ref).max() <= TOL and not y0[T:].any()
    assert np.array_equal(run_gemm(eng, qtype, W, N, K, x, Mp).view(np.uint32), y0.view(np.uint32))
    ldc, c_off = N + 70, 33
    c0 = az.gen_normal(73, (Mp, ldc))
    ya = run_gemm(eng, qtype, W, N, K, x, Mp, acc=1, c_init=c0, ldc=ldc, c_off=c_off)
    assert np.array_equal(ya[:, :c_off], c0[:, :c_off]) and np.array_equal(ya[:, c_off + N:], c0[:, c_off + N:])
    assert np.array_equal(ya[:, c_off:c_off + N], y0 + c0[:, c_off:c_off + N])
    ys = run_gemm(eng, qtype, W, N, K, x, Mp, acc=2, c_init=c0, ldc=ldc, c_off=c_off)
    g = c0[:, c_off:c_off + N].astype(np.float64)
    want = y0.astype(np.float64) * (g / (1.0 + np.exp(-g)))
    assert np.abs(ys[:, c_off:c_off + N] - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(ys[:, :c_off], c0[:, :c_off])


@pytest.mark.parametrize("qtype", [az.Q4_K, az.Q5_K])
@pytest.mark.parametrize("T", [64, 32])
def test_gemm_split_k_unit_scales_exact(eng, qtype, T):
    """Unit scales: the sum of the partial tiles is the exact integer sum (every partial sum below 2^24)."""
    N, K = 96, 4096
    W, wi = unit_scale_weights(qtype, N, K, seed=75)
    x = unit_scale_acts(T, K, seed=76)
    y = run_gemm(eng, qtype, W, N, K, x, T)
    assert np.array_equal(y, (x.astype(np.int64) @ wi.T).astype(np.float32))


def test_startup_self_check(rt):
    """Tuned GEMM == simple GEMM == host integer sums, bit for bit, on the reference's LCG data with unit scales
    (the start-up check in the pattern of xmx_check, zero/engine_setup.h:424-520)."""
    az.self_check()


@pytest.mark.parametrize("qtype", [az.Q4_K, az.Q6_K, az.Q8_0, az.Q4_0, az.IQ4_NL, az.MXFP4])
@pytest.mark.parametrize("T,Mp,N,K", [(1, 16, 264, 1024), (5, 16, 136, 512), (100, 112, 272, 768), (64, 64, 130, 4096)])
def test_per_256_activation_scales(eng, qtype, T, Mp, N, K):
    """act32 = 0: one activation scale per superblock (the reference's quant_store16 with act32 = 0, zero/kernels/ops.cl:
    38-72, and its non-ACT32 GEMM, gemm.cl:489-520).  The quantizer's output bit for bit against the oracle's, the
    matmul against the double-accumulated reference with that one scale on each of a superblock's eight blocks."""
    print(f"act32=0 {TYPE_NAMES[qtype]} T={T} Mp={Mp} N={N} K={K}", flush=True)
    W = make_weights(qtype, N, K, seed=91)
    x = make_acts(T, K, seed=92 + T, outliers=True)
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T, act32=0)
    xp = np.zeros((Mp, K), np.float32)
    xp[:T] = x
    raq, rasc, rabsum = orc.quantize_act(xp, act32=False)
    assert np.array_equal(eng.aq.read(np.int8, Mp * K).reshape(Mp, K), raq)
    assert np.array_equal(eng.asc.read(np.uint32, Mp * K // 256).reshape(K // 256, Mp), rasc.view(np.uint32))
    rows = Mp if T > 8 else T
    cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
    with pytest.raises(az.ArczError):
        eng.matmul("m", w, Mp, cb, N, 0, 0, act32=True)          # the chunk has per-256 scales
    eng.matmul("m", w, Mp, cb, N, 0, 0, act32=False)
    y = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
    ref = orc.matmul_ref(qtype, W, N, K, raq[:T], np.ascontiguousarray(np.repeat(rasc, 8, axis=0)))
    assert np.isfinite(y).all() and rel_err_rows(y, ref).max() <= TOL
    for b in (cb, xb):
        b.free()
    w.free()


@pytest.mark.parametrize("T,Mp,N,K,acc", [(1100, 1104, 392, 512, 0), (1030, 1040, 640, 768, 1), (760, 768, 520, 1024, 2),
                                          (2050, 2064, 136, 256, 1), (300, 384, 388, 5120, 0)])
def test_gemm_per_256_scales_integer_sums(rt, T, Mp, N, K, acc):
    """act32 = 0 on chunks of at least 256 token rows of Q4_K: the form of the 128 x 128 kernel that adds a superblock's
    block sums up as integers (sc * I) and applies sa * d once per four blocks.  Against the double-accumulated
    reference with the one scale on each of a superblock's eight blocks, the three epilogues, partly empty last tiles,
    run to run."""
    print(f"per-256 integer sums T={T} Mp={Mp} N={N} K={K} acc={acc}", flush=True)
    eng = az.Engine(Mp, K)
    W = make_weights(az.Q4_K, N, K, seed=75)
    x = make_acts(T, K, seed=76, outliers=True)
    c0 = np.random.default_rng(77).standard_normal((Mp, N)).astype(np.float32)
    w = eng.make_weight(az.Q4_K, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T, act32=0)
    ys = []
    for _ in range(2):
        cb = az.Runtime.alloc(Mp * N * 4)
        cb.write(c0) if acc else cb.fill(0xFFFFFFFF)
        eng.matmul("test", w, Mp, cb, N, 0, acc, act32=False)
        ys.append(cb.read(np.float32, Mp * N).reshape(Mp, N))
        cb.free()
    xb.free(); w.free(); eng.close()
    assert np.array_equal(ys[0].view(np.uint32), ys[1].view(np.uint32))
    xp = np.zeros((Mp, K), np.float32)
    xp[:T] = x
    raq, rasc, _ = orc.quantize_act(xp, act32=False)
    ref = orc.matmul_ref(az.Q4_K, W, N, K, raq[:T], np.ascontiguousarray(np.repeat(rasc, 8, axis=0)[:, :T]))
    if acc == 1:
        ref = ref + c0[:T]
    elif acc == 2:
        g = c0[:T].astype(np.float64)
        ref = ref * (g / (1.0 + np.exp(-g)))
    y = ys[0][:T]
    assert np.isfinite(y).all() and mixed_err(y, ref) <= TOL
    if acc == 0:
        assert not ys[0][T:].any()


@pytest.mark.parametrize("qtype", [az.Q4_K, az.Q5_K])
@pytest.mark.parametrize("T,Mp,N,K,acc", [(1100, 1104, 392, 512, 0), (1100, 1104, 390, 512, 0), (1030, 1040, 640, 768, 1),
                                          (760, 768, 520, 1024, 2), (1200, 1216, 132, 256, 0),
                                          (2100, 2112, 392, 512, 0), (2050, 2064, 136, 256, 1), (2048, 2048, 256, 768, 2)])
def test_gemm_ready_made_scale_vectors(rt, monkeypatch, qtype, T, Mp, N, K, acc):
    """The 128 x 128 Q4_K / Q5_K kernel whose scale vectors are written by small kernels in front of it (token side: sa and
    sa * S; row side, from 256 token rows on when N is a multiple of 4: d * sc and -(dmin * mn), for Q4_K with the min
    term's factors as bf16 pieces for the matrix instruction) and go into LDS by DMA:
    chunks whose last token tile and last row tile are partly empty, so that the whole-row reads run into the next
    block's entries and past the arrays' ends; the three epilogues.  Against the oracle, and run to run."""
    print(f"ready-made scales {TYPE_NAMES[qtype]} T={T} Mp={Mp} N={N} K={K} acc={acc}", flush=True)
    monkeypatch.setenv("ARCZ_Q4_WM", "2")   # (the 128 x 128 tiles also where the launch rule would take 64 x 128)
    eng = az.Engine(Mp, K)            # (an engine of exactly this chunk: the arrays end where the chunk ends)
    W = make_weights(qtype, N, K, seed=71)
    x = make_acts(T, K, seed=72, outliers=True)
    c0 = np.random.default_rng(73).standard_normal((Mp, N)).astype(np.float32)
    y = run_gemm(eng, qtype, W, N, K, x, Mp, acc=acc, c_init=c0 if acc else None)[:T]
    y2 = run_gemm(eng, qtype, W, N, K, x, Mp, acc=acc, c_init=c0 if acc else None)[:T]
    eng.close()
    assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))
    aq, asc, _ = quantize_padded(x, Mp)
    ref = orc.matmul_ref(qtype, W, N, K, aq[:T], np.ascontiguousarray(asc[:, :T]))
    if acc == 1:
        ref = ref + c0[:T]
    elif acc == 2:
        g = c0[:T].astype(np.float64)
        ref = ref * (g / (1.0 + np.exp(-g)))
    assert np.isfinite(y).all() and mixed_err(y, ref) <= TOL


@pytest.mark.parametrize("T,Mp,N,K,acc", [(1100, 1104, 392, 512, 0), (1030, 1040, 640, 768, 1), (760, 768, 520, 1024, 2),
                                          (300, 304, 132, 256, 0), (2050, 2064, 136, 256, 1)])
def test_gemm_tiles_of_256_tokens(rt, monkeypatch, T, Mp, N, K, acc):
    """The Q4_K kernel in tiles of 256 tokens x 128 rows, work-groups of 8 waves (ARCZ_Q4_WM=4, which an engine reads
    when it is made; not the default launch): the same arithmetic in the same order as the 128 x 128 kernel, so the same
    bits, on chunks whose last tiles are partly empty, with the three epilogues."""
    print(f"256-token tiles T={T} Mp={Mp} N={N} K={K} acc={acc}", flush=True)
    W = make_weights(az.Q4_K, N, K, seed=91)
    x = make_acts(T, K, seed=92, outliers=True)
    c0 = np.random.default_rng(93).standard_normal((Mp, N)).astype(np.float32)
    monkeypatch.setenv("ARCZ_Q4_WM", "2")
    eng = az.Engine(Mp, K)
    want = run_gemm(eng, az.Q4_K, W, N, K, x, Mp, acc=acc, c_init=c0 if acc else None)[:T]
    eng.close()
    monkeypatch.setenv("ARCZ_Q4_WM", "4")
    monkeypatch.setenv("ARCZ_Q4_WM_MIN", "256")
    eng = az.Engine(Mp, K)
    y = run_gemm(eng, az.Q4_K, W, N, K, x, Mp, acc=acc, c_init=c0 if acc else None)[:T]
    eng.close()
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("wm", ["1", "0"])
@pytest.mark.parametrize("T,Mp,N,K,acc", [(1100, 1104, 392, 512, 0), (1100, 1104, 390, 512, 0), (1030, 1040, 640, 768, 1),
                                          (760, 768, 520, 1024, 2), (300, 304, 132, 256, 0), (257, 260, 1000, 2048, 0),
                                          (2050, 2064, 136, 256, 1)])
def test_gemm_tiles_of_64_tokens_on_ready_made_scales(rt, monkeypatch, wm, T, Mp, N, K, acc):
    """The Q4_K kernel in tiles of 64 tokens x 128 rows that takes all four scale vectors ready-made -- the launch
    rule's choice for chunks of a few rounds of work-groups (ARCZ_Q4_WM=0, the default; =1 always, =2 never; read when
    an engine is made) -- on chunks whose last tiles are partly empty, so that the whole-row reads run into the next
    block's entries and past the arrays' ends, with the three epilogues.  Against the oracle, and run to run."""
    print(f"64-token tiles T={T} Mp={Mp} N={N} K={K} acc={acc} ARCZ_Q4_WM={wm}", flush=True)
    W = make_weights(az.Q4_K, N, K, seed=91)
    x = make_acts(T, K, seed=92, outliers=True)
    c0 = np.random.default_rng(93).standard_normal((Mp, N)).astype(np.float32)
    monkeypatch.setenv("ARCZ_Q4_WM", wm)
    eng = az.Engine(Mp, K)            # (an engine of exactly this chunk: the arrays end where the chunk ends)
    y = run_gemm(eng, az.Q4_K, W, N, K, x, Mp, acc=acc, c_init=c0 if acc else None)[:T]
    y2 = run_gemm(eng, az.Q4_K, W, N, K, x, Mp, acc=acc, c_init=c0 if acc else None)[:T]
    eng.close()
    assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))
    aq, asc, _ = quantize_padded(x, Mp)
    ref = orc.matmul_ref(az.Q4_K, W, N, K, aq[:T], np.ascontiguousarray(asc[:, :T]))
    if acc == 1:
        ref = ref + c0[:T]
    elif acc == 2:
        g = c0[:T].astype(np.float64)
        ref = ref * (g / (1.0 + np.exp(-g)))
    assert np.isfinite(y).all() and mixed_err(y, ref) <= TOL
