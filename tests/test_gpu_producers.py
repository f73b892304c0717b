"""The fused producers of the matmul input on the GPU (reference zero/kernels/ops.cl:107-141 rmsnorm_quant, :271-315
swiglu_quant).  The f32 values before quantization follow the reference's formulas; their last bits depend on the order
of the row's sum of squares and on the library's exp / tanh / rsqrt, which the reference leaves to the OpenCL
implementation.  So: the f32 rows are compared with a float64 restatement (1e-6), and the quantization is checked bit
for bit on exactly the rows the GPU normalized (rmsnorm_quant can store them) -- the same split as the reference's own
kernels, where quant_store16 is the shared, exactly specified part.  For swiglu_quant, whose f32 product is not stored,
the scales must agree to 1e-6 and the int8 values may differ by one level in at most 0.1 % of places (a product
within an ulp of a rounding tie)."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import make_acts, pad_rows

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng(rt):
    e = az.Engine(512, 5120)
    yield e
    e.close()


def poison(eng):
    eng.aq.fill(0x7B7B7B7B)
    eng.asc.fill(0xFFFFFFFF)
    eng.absum.fill(0x7B7B7B7B)


@pytest.mark.parametrize("T,Mp,K,row_off", [(1, 16, 5120, 0), (3, 16, 1024, 2), (8, 16, 4096, 0), (9, 16, 512, 0),
                                            (200, 256, 5120, 7), (512, 512, 2048, 0)])
def test_rmsnorm_quant(eng, T, Mp, K, row_off):
    print(f"rmsnorm_quant T={T} Mp={Mp} K={K} row_off={row_off}", flush=True)
    eps = 1e-6
    x = make_acts(T + row_off, K, seed=300 + T, outliers=True)
    w = (1.0 + 0.1 * az.gen_normal(301, (K,))).astype(np.float32)
    xb, wb = az.Runtime.from_numpy(x), az.Runtime.from_numpy(w)
    hb = az.Runtime.alloc(Mp * K * 4).fill(0xFFFFFFFF)
    poison(eng)
    eng.rmsnorm_quant(xb, row_off, wb, K, Mp, T, eps, hout=hb)
    rows = T if T <= 8 else Mp          # a pass of 1-8 tokens writes the valid rows only
    h = hb.read(np.float32, Mp * K).reshape(Mp, K)[:rows]
    aq, asc, absum = eng.read_activations(K, Mp)
    x64 = x[row_off:row_off + T].astype(np.float64)
    ref = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps) * w.astype(np.float64)
    assert np.abs(h[:T] - ref).max() <= 1e-6 * np.abs(ref).max()
    if rows > T:
        assert not h[T:].any()
    raq, rasc, rabsum = orc.quantize_act(np.ascontiguousarray(h))
    assert np.array_equal(aq[:rows], raq)
    assert np.array_equal(asc[:, :rows].view(np.uint32), rasc.view(np.uint32))
    assert np.array_equal(absum[:, :rows], rabsum)
    # the same call without the f32 copy gives the same quantized rows
    poison(eng)
    eng.rmsnorm_quant(xb, row_off, wb, K, Mp, T, eps)
    aq2, asc2, absum2 = eng.read_activations(K, Mp)
    assert np.array_equal(aq2[:rows], aq[:rows]) and np.array_equal(asc2[:, :rows].view(np.uint32), asc[:, :rows].view(np.uint32))
    assert np.array_equal(absum2[:, :rows], absum[:, :rows])
    for b in (xb, wb, hb):
        b.free()


@pytest.mark.parametrize("T,Mp,F,gelu", [(1, 16, 768, 0), (5, 16, 4096, 0), (100, 112, 1024, 0), (64, 64, 5120, 1),
                                         (300, 512, 768, 0)])
def test_swiglu_quant(eng, T, Mp, F, gelu):
    print(f"swiglu_quant T={T} Mp={Mp} F={F} gelu={gelu}", flush=True)
    gu = (2.0 * az.gen_normal(310 + T, (T, 2 * F))).astype(np.float32)
    gb = az.Runtime.from_numpy(gu)
    poison(eng)
    eng.swiglu_quant(gb, F, Mp, T, fused=0, gelu=gelu)
    rows = T if T <= 8 else Mp
    aq, asc, absum = eng.read_activations(F, Mp)
    g, u = gu[:, :F].astype(np.float64), gu[:, F:].astype(np.float64)
    act = 0.5 * g * (1.0 + np.tanh(0.7978845608 * (g + 0.044715 * g ** 3))) if gelu else g / (1.0 + np.exp(-g))
    v = pad_rows((act * u).astype(np.float32), rows)
    raq, rasc, rabsum = orc.quantize_act(v)
    assert np.abs(asc[:, :rows] - rasc).max() <= 1e-6 * np.abs(rasc).max()
    d = np.abs(aq[:rows].astype(np.int32) - raq.astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() <= 1e-3
    assert np.array_equal(absum[:, :rows].T.reshape(rows, F // 16), aq[:rows].astype(np.int32).reshape(rows, F // 16, 16).sum(axis=2))
    # fused form: the rows are taken as they are -> the plain quantizer, bit for bit
    vb = az.Runtime.from_numpy(np.ascontiguousarray(v[:T]))
    poison(eng)
    eng.swiglu_quant(vb, F, Mp, T, fused=1)
    aq2, asc2, absum2 = eng.read_activations(F, Mp)
    assert np.array_equal(aq2[:rows], raq) and np.array_equal(asc2[:, :rows].view(np.uint32), rasc.view(np.uint32))
    assert np.array_equal(absum2[:, :rows], rabsum)
    gb.free(); vb.free()


@pytest.mark.parametrize("T,Mp,K,act32", [(256, 256, 16384, 1), (300, 320, 5120, 1), (250, 256, 4096, 0), (1000, 1024, 256, 0)])
def test_producers_16_rows_a_work_group(rt, T, Mp, K, act32):
    """Chunks of at least 256 rows go through the forms that take 16 rows a work-group and write scales and sums in
    pieces of 16 rows: the same bits as the plain quantizer on the f32 rows (RMS norm: on the rows the kernel itself
    wrote out), per-32 and per-256 scales, rows past T as zeros, the longest rows each form takes."""
    print(f"producers r16 T={T} Mp={Mp} K={K} act32={act32}", flush=True)
    eng = az.Engine(Mp, max(K, 256))
    try:
        B = 32 if act32 else 256
        def read(K):
            return (eng.aq.read(np.int8, Mp * K).reshape(Mp, K), eng.asc.read(np.float32, Mp * K // B).reshape(K // B, Mp),
                    eng.absum.read(np.int16, Mp * K // 16).reshape(K // 16, Mp))
        x = make_acts(T, K, seed=330 + T, outliers=True)
        w = (1.0 + 0.1 * az.gen_normal(331, (K,))).astype(np.float32)
        xb, wb = az.Runtime.from_numpy(x), az.Runtime.from_numpy(w)
        hb = az.Runtime.alloc(Mp * K * 4).fill(0xFFFFFFFF)
        poison(eng)
        eng.rmsnorm_quant(xb, 0, wb, K, Mp, T, 1e-6, hout=hb, act32=act32)
        h = hb.read(np.float32, Mp * K).reshape(Mp, K)
        x64 = x.astype(np.float64)
        ref = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + 1e-6) * w.astype(np.float64)
        assert np.abs(h[:T] - ref).max() <= 1e-6 * np.abs(ref).max() and not h[T:].any()
        aq, asc, absum = read(K)
        raq, rasc, rabsum = orc.quantize_act(np.ascontiguousarray(h), act32=bool(act32))
        assert np.array_equal(aq, raq) and np.array_equal(asc.view(np.uint32), rasc.view(np.uint32)) and np.array_equal(absum, rabsum)
        # SwiGLU on rows taken as they are (the fused form) and on gate | up
        vb = az.Runtime.from_numpy(np.ascontiguousarray(h[:T]))
        poison(eng)
        eng.swiglu_quant(vb, K, Mp, T, fused=1, act32=act32)
        aq2, asc2, absum2 = read(K)
        assert np.array_equal(aq2, raq) and np.array_equal(asc2.view(np.uint32), rasc.view(np.uint32)) and np.array_equal(absum2, rabsum)
        F = K // 2
        if F % 256 == 0:
            gb = az.Runtime.from_numpy(x)          # rows [gate(F) | up(F)]
            poison(eng)
            eng.swiglu_quant(gb, F, Mp, T, fused=0, act32=act32)
            g, u = x[:, :F].astype(np.float64), x[:, F:].astype(np.float64)
            v = pad_rows((g / (1.0 + np.exp(-g)) * u).astype(np.float32), Mp)
            vaq, vasc, vabsum = orc.quantize_act(v, act32=bool(act32))
            gaq = eng.aq.read(np.int8, Mp * F).reshape(Mp, F)
            gasc = eng.asc.read(np.float32, Mp * F // B).reshape(F // B, Mp)
            gabsum = eng.absum.read(np.int16, Mp * F // 16).reshape(F // 16, Mp)
            assert np.abs(gasc - vasc).max() <= 1e-6 * np.abs(vasc).max()
            d = np.abs(gaq.astype(np.int32) - vaq.astype(np.int32))
            assert d.max() <= 1 and (d != 0).mean() <= 1e-3
            assert np.array_equal(gabsum.T.reshape(Mp, F // 16), gaq.astype(np.int32).reshape(Mp, F // 16, 16).sum(axis=2))
            gb.free()
        for b in (xb, wb, hb, vb):
            b.free()
    finally:
        eng.close()


def test_producer_feeds_matmul(eng):
    """rmsnorm_quant -> GEMV and GEMM: the matmul of the normalized rows, against the oracle on the GPU's own int8 rows."""
    from common import make_weights, rel_err_rows
    K, N = 1024, 512
    W = make_weights(az.Q4_K, N, K, seed=320)
    w = eng.make_weight(az.Q4_K, N, K, W)
    nw = np.ones(K, np.float32)
    nwb = az.Runtime.from_numpy(nw)
    for T, Mp in ((1, 16), (40, 48)):
        x = make_acts(T, K, seed=321 + T)
        xb = az.Runtime.from_numpy(x)
        eng.rmsnorm_quant(xb, 0, nwb, K, Mp, T, 1e-6)
        aq, asc, _ = eng.read_activations(K, Mp)
        rows = T if T <= 8 else Mp
        cb = az.Runtime.alloc(rows * N * 4)
        eng.matmul("t", w, Mp, cb, N, 0, 0)
        y = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
        ref = orc.matmul_ref(az.Q4_K, W, N, K, aq[:T], asc)
        assert rel_err_rows(y, ref).max() <= 1e-3
        cb.free(); xb.free()
    w.free(); nwb.free()


@pytest.mark.parametrize("T,Mp,K,norm2,s", [(1, 16, 5120, True, 1.0), (4, 16, 2048, False, 0.5), (8, 16, 17408 // 4, True, 0.75),
                                            (100, 128, 1024, True, 1.0), (300, 512, 768, False, 1.0)])
def test_add_norm_quant(rt, T, Mp, K, norm2, s):
    """x = (x + rmsnorm(t) * w) * s in place, then the next input from the new x (reference zero/kernels/ops_attn_g.cl:
    616-667).  The new x against float64 (1e-6); with norm2 off the quantized rows are the quantizer's, bit for bit, of
    the x the GPU stored; with norm2 on the scales agree to 1e-6 and the int8 values differ by at most one level in at
    most 0.1 % of places (the row's second sum of squares is taken in the kernel's own order)."""
    print(f"add_norm_quant T={T} Mp={Mp} K={K} norm2={norm2} s={s}", flush=True)
    e = az.Engine(512, 5120)
    try:
        eps = 1e-6
        x = make_acts(T, K, seed=400 + T)
        t = (3.0 * az.gen_normal(401 + T, (T, K))).astype(np.float32)
        w = (1.0 + 0.1 * az.gen_normal(402, (K,))).astype(np.float32)
        w2 = (1.0 + 0.1 * az.gen_normal(403, (K,))).astype(np.float32)
        xb, tb, wb, w2b = (az.Runtime.from_numpy(a) for a in (x, t, w, w2))
        poison(e)
        e.add_norm_quant(xb, tb, wb, K, T, Mp, s, w2b if norm2 else None, norm2, eps)
        rows = T if T <= 8 else Mp
        xn = xb.read(np.float32, T * K).reshape(T, K)
        t64 = t.astype(np.float64)
        ref = (x.astype(np.float64) + t64 / np.sqrt((t64 * t64).mean(axis=1, keepdims=True) + eps) * w) * s
        assert np.abs(xn - ref).max() <= 1e-6 * np.abs(ref).max()
        aq, asc, absum = e.read_activations(K, Mp)
        if norm2:
            x64 = xn.astype(np.float64)
            v = (x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps) * w2).astype(np.float32)
        else:
            v = xn
        raq, rasc, rabsum = orc.quantize_act(pad_rows(np.ascontiguousarray(v), rows))
        if norm2:
            assert np.abs(asc[:, :rows] - rasc).max() <= 1e-6 * np.abs(rasc).max()
            d = np.abs(aq[:rows].astype(np.int32) - raq.astype(np.int32))
            assert d.max() <= 1 and (d != 0).mean() <= 1e-3
            assert np.array_equal(absum[:, :rows].T.reshape(rows, K // 16),
                                  aq[:rows].astype(np.int32).reshape(rows, K // 16, 16).sum(axis=2))
        else:
            assert np.array_equal(aq[:rows], raq)
            assert np.array_equal(asc[:, :rows].view(np.uint32), rasc.view(np.uint32))
            assert np.array_equal(absum[:, :rows], rabsum)
        if rows > T:
            assert not aq[T:rows].any()
        # the quantized rows feed the next matmul: a second call on the same inputs gives the same bits
        xb2 = az.Runtime.from_numpy(x)
        e.add_norm_quant(xb2, tb, wb, K, T, Mp, s, w2b if norm2 else None, norm2, eps)
        aq2, asc2, _ = e.read_activations(K, Mp)
        assert np.array_equal(aq2[:rows], aq[:rows]) and np.array_equal(asc2[:, :rows].view(np.uint32), asc[:, :rows].view(np.uint32))
        for b in (xb, xb2, tb, wb, w2b):
            b.free()
    finally:
        e.close()
