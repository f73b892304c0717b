"""Two-pass matmul inputs on the GPU (reference zero/engine.h:1034-1101, zero/kernels/ops.cl:49-59, 73-101): every
producer also quantizes what its int8 values miss, and every matmul adds a second pass over that half.  The residual's
quants, scales and sums are checked bit for bit against the oracle on exactly the f32 rows the GPU quantized; the
matmul against the double-accumulated sum of both passes (1e-3, as for one pass) and, which is the point of the mode,
against the product with the unquantized activations, where two passes must come an order of magnitude closer than
one."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import ALL_TYPES, TYPES, TYPE_NAMES, make_acts, make_weights, pad_rows, rel_err_rows

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng(rt):
    e = az.Engine(256, 2048)
    e.two_pass(True)
    yield e
    e.close()


def check_halves(eng, v, K, Mp, rows):
    """Both halves of the engine's buffers against the oracle's two-pass quantization of the rows v [rows][K]."""
    (aq, asc, absum), (rq, rsc, rsum), _ = orc.quantize_act_two_pass(np.ascontiguousarray(v))
    g1, g2 = eng.read_activations(K, Mp), eng.read_residual(K, Mp)
    for (gq, gs, gb), (wq, ws, wb) in ((g1, (aq, asc, absum)), (g2, (rq, rsc, rsum))):
        assert np.array_equal(gq[:rows], wq)
        assert np.array_equal(gs[:, :rows].view(np.uint32), ws.view(np.uint32))
        assert np.array_equal(gb[:, :rows], wb)


@pytest.mark.parametrize("T,Mp,K", [(1, 16, 2048), (7, 16, 512), (100, 112, 1024), (256, 256, 2048)])
def test_quant_rows_residual(eng, T, Mp, K):
    print(f"two-pass quant_rows T={T} Mp={Mp} K={K}", flush=True)
    x = make_acts(T, K, seed=700 + T, outliers=True)
    x[0, 32:64] = 0.0                       # a zero block: scale 0, residual 0
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T)
    check_halves(eng, pad_rows(x, Mp), K, Mp, Mp)
    xb.free()


@pytest.mark.parametrize("T,Mp,K", [(1, 16, 2048), (5, 16, 1024), (60, 64, 2048)])
def test_fused_producers_residual(eng, T, Mp, K):
    print(f"two-pass producers T={T} Mp={Mp} K={K}", flush=True)
    rows = T if T <= 8 else Mp
    x = make_acts(T, K, seed=720 + T, outliers=True)
    w = (1.0 + 0.1 * az.gen_normal(721, (K,))).astype(np.float32)
    xb, wb = az.Runtime.from_numpy(x), az.Runtime.from_numpy(w)
    hb = az.Runtime.alloc(Mp * K * 4).fill(0)
    eng.rmsnorm_quant(xb, 0, wb, K, Mp, T, 1e-6, hout=hb)
    check_halves(eng, hb.read(np.float32, Mp * K).reshape(Mp, K)[:rows], K, Mp, rows)
    # swiglu_quant on rows the matmul before has already multiplied (fused): the rows themselves are quantized
    eng.swiglu_quant(xb, K, Mp, T, fused=1)
    check_halves(eng, pad_rows(x, Mp)[:rows], K, Mp, rows)
    # add_norm_quant without the second norm: the new residual-stream rows are quantized as they are
    t = make_acts(T, K, seed=730 + T)
    tb = az.Runtime.from_numpy(t)
    eng.add_norm_quant(xb, tb, wb, K, T, Mp, 0.5, None, False, 1e-6)
    xn = xb.read(np.float32, T * K).reshape(T, K)
    check_halves(eng, pad_rows(xn, Mp)[:rows], K, Mp, rows)
    for b in (xb, wb, hb, tb):
        b.free()


@pytest.mark.parametrize("T,Mp", [(1, 16), (2, 16), (5, 16), (100, 112)])
@pytest.mark.parametrize("qtype", ALL_TYPES)
def test_matmul_two_pass(eng, qtype, T, Mp):
    N, K = 320, 2048
    print(f"two-pass matmul {TYPE_NAMES[qtype]} T={T} Mp={Mp} N={N} K={K}", flush=True)
    W = make_weights(qtype, N, K, seed=740)
    x = make_acts(T, K, seed=741 + T, outliers=True)
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T)
    rows = T if T <= 8 else Mp
    cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
    eng.matmul("two", w, Mp, cb, N, 0, 0)
    y = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
    (aq, asc, _), (rq, rsc, _), _ = orc.quantize_act_two_pass(pad_rows(x, Mp))
    y1 = orc.matmul_ref(qtype, W, N, K, aq[:T], asc).astype(np.float64)
    y2 = orc.matmul_ref(qtype, W, N, K, rq[:T], rsc).astype(np.float64)
    assert rel_err_rows(y, y1 + y2).max() <= 1e-3
    # against the unquantized activations: one pass is limited by the int8 rounding, two passes are not
    exact = x.astype(np.float64) @ orc.dequant_rows(qtype, W, N, K).astype(np.float64).T
    e1, e2 = rel_err_rows(y1, exact).max(), rel_err_rows(y, exact).max()
    print(f"  error against f32 activations: one pass {e1:.2e}, two passes {e2:.2e}", flush=True)
    assert e2 < e1 / 10
    if T > 8:
        with pytest.raises(az.ArczError):
            eng.matmul("two", w, Mp, cb, N, 0, 2)      # no fused epilogue with two passes (zero/engine.h:1091)
    # accumulating, and as two launches: the one-launch form of 1-4 tokens gives the same bits (one token of Q4_K /
    # Q5_K aside: its two launches run the one-token kernel, which groups a term's factors differently)
    eng.matmul("two", w, Mp, cb, N, 0, 1)
    ya = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
    eng.two_pass(True, fuse=False)
    eng.quantize(xb, K, K, Mp, T)
    cb.fill(0xFFFFFFFF)
    eng.matmul("two", w, Mp, cb, N, 0, 0)
    y2l = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
    eng.matmul("two", w, Mp, cb, N, 0, 1)
    y2a = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
    eng.two_pass(True, fuse=True)
    if T == 1 and qtype in (az.Q4_K, az.Q5_K):
        assert rel_err_rows(y, y2l).max() <= 1e-5 and rel_err_rows(ya, y2a).max() <= 1e-5
    else:
        assert np.array_equal(y, y2l) and np.array_equal(ya, y2a)
    for b in (cb, xb):
        b.free()
    w.free()


def test_mode_switch(rt):
    """Off -> on -> off: the one-pass results are the same before and after, and caller-quantized inputs are refused
    while the mode is on."""
    e = az.Engine(16, 1024)
    N, K = 64, 1024
    W = make_weights(az.Q4_K, N, K, seed=760)
    x = make_acts(1, K, seed=761)
    w = e.make_weight(az.Q4_K, N, K, W)
    xb = az.Runtime.from_numpy(x)
    cb = az.Runtime.alloc(N * 4)
    outs = []
    for on in (False, True, False):
        e.two_pass(on)
        e.quantize(xb, K, K, 16, 1)
        e.matmul("m", w, 16, cb, N, 0, 0)
        outs.append(cb.read(np.float32, N))
        if on:
            aq, asc, absum = orc.quantize_act(pad_rows(x, 16))
            with pytest.raises(az.ArczError):
                e.set_activations(aq, asc, absum, K, 16, 1)
    assert np.array_equal(outs[0], outs[2]) and not np.array_equal(outs[0], outs[1])
    e.close()


@pytest.mark.parametrize("qtype,T", [(az.Q6_K, 1), (az.Q4_K, 3), (az.Q8_0, 7)])
def test_two_pass_output_head_softcap(eng, qtype, T):
    """An output head with a soft cap under two-pass inputs (zero/engine.h:1081-1110): both passes run without the cap and
    the cap is applied to their sum -- c * tanh((v1 + v2) / c), not the sum of two capped values."""
    N, K, cap = 264, 1024, 30.0
    W = make_weights(qtype, N, K, seed=91)
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(make_acts(T, K, seed=92) * np.float32(40.0))
    eng.quantize(xb, K, K, 16, T)
    plain = az.Runtime.alloc(T * N * 4)
    eng.matmul("head", w, 16, plain, N, 0, 0)
    y = plain.read(np.float32, T * N).reshape(T, N)
    w.set_softcap(cap)
    capped = az.Runtime.alloc(T * N * 4).fill(0xFFFFFFFF)
    eng.matmul("head", w, 16, capped, N, 0, 0)
    yc = capped.read(np.float32, T * N).reshape(T, N)
    assert np.abs(y).max() > cap / 2
    assert np.abs(yc - cap * np.tanh(y.astype(np.float64) / cap)).max() <= 2e-6 * cap
    for b in (plain, capped, xb):
        b.free()
    w.free()
