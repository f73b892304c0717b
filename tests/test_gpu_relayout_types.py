"""AR4_128 and Q2_0 (the reference's src/quants.h:531-542, 607-616; zero/kernels/decode.cl PER32 on its GPU side).

Both are one f16 scale times a small integer, like Q4_0; the library writes their rows out as Q4_0 blocks of the same
values when it uploads them.  Here: every matmul form on such a weight against the oracle's own decode of the source
bytes (1e-3 per token row, bench/gemv_bench.cpp:199-214) and, bit for bit, against the upload of the same rows as Q4_0;
rows that end inside a superblock; an expert layer; tensors of a GGUF file.
"""
import numpy as np
import pytest

import arcinferzero_amd as az
import gguf_writer as gw
import oracle_lib as orc
from common import make_acts, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu
GEOM = {az.AR4_128: (128, 66), az.Q2_0: (64, 18)}      # values and bytes of a block
NAME = {az.AR4_128: "AR4_128", az.Q2_0: "Q2_0"}


def random_rows(qtype, rows, K, seed, scale=0.02):
    """rows x K values as blocks of random codes with f16 scales of both signs around `scale`."""
    blk, nbytes = GEOM[qtype]
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 256, size=(rows * K // blk, nbytes), dtype=np.uint8)
    d = (rng.uniform(0.5, 1.5, raw.shape[0]) * scale * rng.choice([-1.0, 1.0], raw.shape[0])).astype(np.float16)
    raw[:, 0:2] = d.reshape(-1, 1).view(np.uint8)
    return raw.reshape(-1)


def run(eng, qtype, W, N, K, x, Mp):
    T = x.shape[0]
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, x.shape[1], x.shape[1], Mp, T)
    rows = Mp if T > 8 else T
    cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
    eng.matmul("relayout", w, Mp, cb, N, 0, 0)
    y = cb.read(np.float32, rows * N).reshape(rows, N)
    k = w.K
    for b in (cb, xb):
        b.free()
    w.free()
    return y, k


# T = 1, 3: the dot-product GEMVs; 12: the matrix-pipe GEMV; 100, 300: the GEMM; K = 5120 at 20 tokens: K in pieces
@pytest.mark.parametrize("T,Mp,N,K", [(1, 16, 136, 1024), (3, 16, 136, 1024), (12, 16, 200, 768), (100, 112, 136, 1024),
                                      (300, 384, 264, 512), (20, 32, 200, 5120)])
@pytest.mark.parametrize("qtype", [az.AR4_128, az.Q2_0])
def test_matmul_forms(rt, qtype, T, Mp, N, K):
    print(f"relayout {NAME[qtype]} T={T} Mp={Mp} N={N} K={K}", flush=True)
    W = random_rows(qtype, N, K, seed=500 + T)
    x = make_acts(T, K, seed=501 + T, outliers=True)
    eng = az.Engine(Mp, K)
    try:
        y, k = run(eng, qtype, W, N, K, x, Mp)
        assert k == K and not y[T:].any()
        y40, _ = run(eng, az.Q4_0, az.relayout_q4_0(qtype, N, K, W), N, K, x, Mp)
        assert np.array_equal(y.view(np.uint32), y40.view(np.uint32))
        aq, asc, _ = quantize_padded(x, Mp)
        ref = orc.matmul_ref(qtype, W, N, K, aq[:T], asc)
        e = rel_err_rows(y[:T], ref).max()
        print(f"  vs oracle {e:.2e}")
        assert np.isfinite(y).all() and e <= 1e-3
    finally:
        eng.close()


@pytest.mark.parametrize("qtype,N,K,T,Mp", [(az.AR4_128, 136, 384, 2, 16), (az.Q2_0, 200, 320, 12, 16), (az.Q2_0, 264, 2880, 100, 112),
                                            (az.AR4_128, 130, 2944, 40, 48)])
def test_rows_that_end_inside_a_superblock(rt, qtype, N, K, T, Mp):
    """K in whole source blocks but not whole superblocks: the rows become Q4_0 blocks and are then padded with zero
    blocks like any Q4_0 rows (the reference's loader: zero/engine_load.h:371-387); the activations are rows of the
    rounded-up length whose tail is zero."""
    print(f"relayout padded {NAME[qtype]} N={N} K={K} T={T}", flush=True)
    Kp = (K + 255) // 256 * 256
    blk, nbytes = GEOM[qtype]
    W = random_rows(qtype, N, K, seed=520)
    full = np.zeros((N, Kp // blk * nbytes), np.uint8)              # the same rows with zero blocks behind them
    full[:, :K // blk * nbytes] = W.reshape(N, -1)
    x = np.zeros((T, Kp), np.float32)
    x[:, :K] = make_acts(T, K, seed=521, outliers=True)
    eng = az.Engine(Mp, Kp)
    try:
        y, k = run(eng, qtype, W, N, K, x, Mp)
        assert k == Kp
        aq, asc, _ = quantize_padded(x, Mp)
        ref = orc.matmul_ref(qtype, full.reshape(-1), N, Kp, aq[:T], asc)
        assert np.isfinite(y).all() and rel_err_rows(y[:T], ref).max() <= 1e-3
        with pytest.raises(az.ArczError):
            eng.make_weight(qtype, N, K + 32, W)                    # not whole blocks of the type
        with pytest.raises(az.ArczError):
            eng.make_weight(qtype, N, K, W[:-1])                    # a byte short
    finally:
        eng.close()


@pytest.mark.parametrize("T,Mp", [(1, 16), (4, 16), (150, 160)])
@pytest.mark.parametrize("qtype", [az.AR4_128, az.Q2_0])
def test_expert_layer(rt, qtype, T, Mp):
    NE, NU, E, F = 8, 2, 512, 256
    print(f"relayout expert layer {NAME[qtype]} T={T}", flush=True)
    Wg, Wu = random_rows(qtype, NE * F, E, seed=531, scale=0.01), random_rows(qtype, NE * F, E, seed=532, scale=0.01)
    Wd = random_rows(qtype, NE * E, F, seed=533, scale=0.01)
    x = make_acts(T, E, seed=534)
    logits = az.gen_normal(535, (T, NE))
    aq, asc, absum = quantize_padded(x, Mp)
    eng = az.Engine(Mp, max(E, F))
    outs = []
    try:
        for t, (g, u, d) in ((qtype, (Wg, Wu, Wd)),
                             (az.Q4_0, (az.relayout_q4_0(qtype, NE * F, E, Wg), az.relayout_q4_0(qtype, NE * F, E, Wu),
                                        az.relayout_q4_0(qtype, NE * E, F, Wd)))):
            L = eng.make_moe_layer(t, g, u, d, NE, NU, E, F)
            eng.set_activations(aq, asc, absum, E, Mp, T)
            lb = az.Runtime.from_numpy(logits)
            ob = az.Runtime.alloc(T * E * 4).fill(0)
            eng.layer_moe(L, lb, NE, ob, T, Mp)
            outs.append(ob.read(np.float32, T * E).reshape(T, E))
            lb.free(); ob.free()
            L.free()
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
        # against the oracle on the source bytes: h, then the layer for every token whose int8 h is the oracle's (a
        # value of h on a rounding boundary may land one int8 step away: the sums run in another order)
        n, S = T * NU, eng.moe_slots
        inv = eng.moe_buffer("inv").read(np.int32, n)
        h = eng.moe_buffer("h").read(np.float32, S * F).reshape(S, F)[inv]
        hq = eng.moe_buffer("hq").read(np.int8, S * F).reshape(S, F)[inv]
        ref, href = orc.moe_layer(qtype, Wg, Wu, Wd, NE, NU, E, F, aq[:T], asc, logits)
        dq = hq.astype(np.int32) - orc.moe_quant(href)[0].astype(np.int32)
        same = ~np.isin(np.arange(T), np.nonzero(dq.any(axis=1))[0] // NU)
        eh, e = rel_err_rows(h, href).max(), rel_err_rows(outs[0], ref)[same].max(initial=0.0)
        print(f"  vs oracle: h {eh:.2e}, layer {e:.2e} over {int(same.sum())} of {T} tokens")
        assert np.isfinite(outs[0]).all() and eh <= 1e-3 and e <= 1e-3
        assert np.abs(dq).max() <= 1 and (dq != 0).sum() <= 4 + dq.size // 10000
    finally:
        eng.close()


def test_tensors_of_a_gguf_file(rt, tmp_path):
    """A matrix and the three expert tensors of a layer as a file holds them (type ids 0x41523447 and 42), the layer's
    gate / up and down of different types, F = 384 not whole superblocks."""
    N, K, NE, NU, E, F, T, Mp = 136, 640, 4, 2, 512, 384, 5, 16
    W = random_rows(az.Q2_0, N, K, seed=541)
    Wg, Wu = random_rows(az.AR4_128, NE * F, E, seed=542, scale=0.01), random_rows(az.AR4_128, NE * F, E, seed=543, scale=0.01)
    Wd = random_rows(az.Q2_0, NE * E, F, seed=544, scale=0.01)
    p = tmp_path / "relayout.gguf"
    gw.write_gguf(p, [], [("m.weight", az.Q2_0, [K, N], W), ("g.weight", az.AR4_128, [E, F, NE], Wg),
                          ("u.weight", az.AR4_128, [E, F, NE], Wu), ("d.weight", az.Q2_0, [F, E, NE], Wd)])
    eng = az.Engine(Mp, 768)
    try:
        with az.GgufFile(p) as g:
            w = eng.make_weight_gguf(g, "m.weight")
            L = eng.make_moe_layer_gguf(g, "g.weight", "u.weight", "d.weight", NU)
        assert w.K == 768 and (L.E, L.F) == (512, 512)
        # the matrix
        x = np.zeros((T, 768), np.float32)
        x[:, :K] = make_acts(T, K, seed=545)
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, 768, 768, Mp, T)
        cb = az.Runtime.alloc(T * N * 4).fill(0xFFFFFFFF)
        eng.matmul("gguf", w, Mp, cb, N, 0, 0)
        y = cb.read(np.float32, T * N).reshape(T, N)
        full = np.zeros((N, 768 // 64 * 18), np.uint8)
        full[:, :K // 64 * 18] = W.reshape(N, -1)
        aq, asc, _ = quantize_padded(x, Mp)
        assert rel_err_rows(y, orc.matmul_ref(az.Q2_0, full.reshape(-1), N, 768, aq[:T], asc)).max() <= 1e-3
        # the layer: against the same layer made from Q4_0 blocks of the same values, F padded by the upload
        xe = make_acts(T, E, seed=546)
        logits = az.gen_normal(547, (T, NE))
        aq, asc, absum = quantize_padded(xe, Mp)
        L40 = eng.make_moe_layer(az.Q4_0, az.relayout_q4_0(az.AR4_128, NE * F, E, Wg), az.relayout_q4_0(az.AR4_128, NE * F, E, Wu),
                                 az.relayout_q4_0(az.Q2_0, NE * E, F, Wd), NE, NU, E, F)
        outs = []
        for layer in (L, L40):
            eng.set_activations(aq, asc, absum, E, Mp, T)
            lb = az.Runtime.from_numpy(logits)
            ob = az.Runtime.alloc(T * E * 4).fill(0)
            eng.layer_moe(layer, lb, NE, ob, T, Mp)
            outs.append(ob.read(np.float32, T * E).reshape(T, E))
            lb.free(); ob.free()
        assert np.isfinite(outs[0]).all() and np.abs(outs[0]).max() > 0
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
        for b in (cb, xb):
            b.free()
        w.free()
    finally:
        eng.close()
