"""The reference's own decode vectors through the HIP kernels.

tests/golden/ref_vectors*.npz hold superblocks whose every field is random (6-bit scales and mins over their whole
range, negative d and dmin, Q6_K int8 sub-scales of both signs, every IQ codebook index) together with what the
compiled reference (src/quants.h dequant_row) decodes them to.  Here those blocks are dealt out over the rows of a
matrix and go through every matmul form -- one-token and multi-token GEMV, the matrix-pipe GEMV, the dense GEMM, the
GEMM with K shared out over work-groups, expert tiles -- and the f32 output is held to 1e-3 (per token row,
max|y - ref| / max|ref|, bench/gemv_bench.cpp:199-214) of two references: the oracle's matmul_ref on the raw blocks and
the plain float64 product of the int8-rounded activations with the golden decoded values.
"""
import os

import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import TYPE_NAMES, make_acts, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu
TOL = 1e-3
HERE = os.path.dirname(os.path.abspath(__file__))
G1 = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))
G2 = np.load(os.path.join(HERE, "golden", "ref_vectors_types2.npz"))
G3 = np.load(os.path.join(HERE, "golden", "ref_vectors_types3.npz"))
# type -> (raw bytes of the 8 golden superblocks, their decoded values [8][256], bytes per superblock)
GOLD = {
    az.Q4_K: (G1["q4k_raw"], G1["q4k_dequant"], 144),
    az.Q6_K: (G1["q6k_raw"], G1["q6k_dequant"], 210),
    az.Q8_0: (G1["q80_raw"], G1["q80_dequant"], 272),
    az.Q5_K: (G2["q5k_raw"], G2["q5k_dequant"], 176),
    az.IQ4_XS: (G2["iq4xs_raw"], G2["iq4xs_dequant"], 136),
    az.IQ3_S: (G2["iq3s_raw"], G2["iq3s_dequant"], 110),
    az.Q3_K: (G3["q3k_raw"], G3["q3k_dequant"], 110),
    az.IQ3_XXS: (G3["iq3xxs_raw"], G3["iq3xxs_dequant"], 98),
    az.IQ4_NL: (G3["iq4nl_raw"], G3["iq4nl_dequant"], 144),
    az.MXFP4: (G3["mxfp4_raw"], G3["mxfp4_dequant"], 136),
}
GTYPES = tuple(GOLD)


def golden_matrix(qtype, N, K, seed):
    """N rows of K values dealt from the 8 golden superblocks (every one used, in a seeded order): the GGUF bytes and
    the reference's decoded values [N][K]."""
    raw, deq, sbb = GOLD[qtype]
    sb_raw = raw.reshape(8, sbb)
    sb_val = deq.reshape(8, 256)
    nsb = K // 256
    rng = np.random.default_rng(seed)
    pick = rng.integers(0, 8, size=(N, nsb))
    pick.reshape(-1)[:8] = np.arange(8)
    W = np.ascontiguousarray(sb_raw[pick].reshape(-1))
    vals = sb_val[pick].reshape(N, K).astype(np.float64)
    return W, vals


def references(qtype, W, vals, N, K, x, Mp):
    T = x.shape[0]
    aq, asc, _ = quantize_padded(x, Mp)
    ref = orc.matmul_ref(qtype, W, N, K, aq[:T], asc)
    xa = aq[:T].astype(np.float64).reshape(T, K // 32, 32) * asc[:, :T].T.astype(np.float64)[:, :, None]
    gold = xa.reshape(T, K) @ vals.T
    return ref, gold


def run_matmul(eng, qtype, W, N, K, x, Mp):
    T = x.shape[0]
    w = eng.make_weight(qtype, N, K, W)
    xb = az.Runtime.from_numpy(x)
    eng.quantize(xb, K, K, Mp, T)
    rows = Mp if T > 8 else T
    cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
    eng.matmul("golden", w, Mp, cb, N, 0, 0)
    y = cb.read(np.float32, rows * N).reshape(rows, N)
    for b in (cb, xb):
        b.free()
    w.free()
    return y


@pytest.fixture(scope="module")
def eng(rt):
    e = az.Engine(384, 5120)
    yield e
    e.close()


def test_oracle_decodes_the_dealt_rows(rt):
    """The dealing itself: the oracle's decode of the dealt rows is the golden values, bit for bit."""
    for qtype in GTYPES:
        W, vals = golden_matrix(qtype, 12, 768, seed=1)
        assert np.array_equal(orc.dequant_rows(qtype, W, 12, 768), vals.astype(np.float32))


# T = 1, 2, 5: the dot-product GEMVs; 7, 12 (Mp = 16): the matrix-pipe GEMV for Q4_K, gemv_mt / the GEMM for the rest
@pytest.mark.parametrize("T", [1, 2, 5, 7, 12])
@pytest.mark.parametrize("qtype", GTYPES)
def test_golden_blocks_gemv(eng, qtype, T):
    N, K, Mp = 136, 1024, 16
    print(f"golden gemv {TYPE_NAMES[qtype]} T={T}", flush=True)
    W, vals = golden_matrix(qtype, N, K, seed=100 + T)
    x = make_acts(T, K, seed=7 + T, outliers=True)
    y = run_matmul(eng, qtype, W, N, K, x, Mp)[:T]
    ref, gold = references(qtype, W, vals, N, K, x, Mp)
    assert np.isfinite(y).all()
    e1, e2 = rel_err_rows(y, ref).max(), rel_err_rows(y, gold).max()
    print(f"  vs oracle {e1:.2e}  vs golden values {e2:.2e}")
    assert e1 <= TOL and e2 <= TOL


# the dense GEMM (full and ragged tiles), and short chunks over a long K: K in pieces over several work-groups
@pytest.mark.parametrize("T,Mp,N,K", [(100, 112, 136, 1024), (300, 384, 264, 512), (64, 64, 130, 4096), (20, 32, 200, 5120)])
@pytest.mark.parametrize("qtype", GTYPES)
def test_golden_blocks_gemm(eng, qtype, T, Mp, N, K):
    print(f"golden gemm {TYPE_NAMES[qtype]} T={T} Mp={Mp} N={N} K={K}", flush=True)
    W, vals = golden_matrix(qtype, N, K, seed=200 + T)
    x = make_acts(T, K, seed=17 + T, outliers=True)
    y = run_matmul(eng, qtype, W, N, K, x, Mp)
    assert not y[T:].any()
    y = y[:T]
    ref, gold = references(qtype, W, vals, N, K, x, Mp)
    assert np.isfinite(y).all()
    e1, e2 = rel_err_rows(y, ref).max(), rel_err_rows(y, gold).max()
    print(f"  vs oracle {e1:.2e}  vs golden values {e2:.2e}")
    assert e1 <= TOL and e2 <= TOL


def test_golden_q6k_has_negative_subscales():
    """What the library's own generator never emits and the golden blocks do."""
    raw, _, _ = GOLD[az.Q6_K]
    sc = raw.reshape(8, 210)[:, 192:208].view(np.int8)
    assert (sc < 0).any() and (sc > 0).any()
    d4 = GOLD[az.Q4_K][0].reshape(8, 144)[:, 0:4].view(np.float16)
    assert (d4 < 0).any()


# expert tiles: gate/up (gathered rows, fused SwiGLU) and down (routing weights) of a layer whose experts are golden
# blocks, T = 150 through the tile GEMMs and T = 3 through the matrix-vector expert kernels
@pytest.mark.parametrize("T,Mp", [(150, 160), (3, 16)])
@pytest.mark.parametrize("qtype", GTYPES)
def test_golden_blocks_expert_tiles(rt, qtype, T, Mp):
    NE, NU, E, F = 4, 2, 512, 256
    print(f"golden expert tiles {TYPE_NAMES[qtype]} T={T}", flush=True)
    e = az.Engine(Mp, max(E, F))
    try:
        Wg, vg = golden_matrix(qtype, NE * F, E, seed=31)
        Wu, vu = golden_matrix(qtype, NE * F, E, seed=32)
        Wd, vd = golden_matrix(qtype, NE * E, F, seed=33)
        # (golden blocks decode to values up to a few thousand: keep the gate's argument in silu's working range)
        x = make_acts(T, E, seed=34) * np.float32(1e-4)
        L = e.make_moe_layer(qtype, Wg, Wu, Wd, NE, NU, E, F)
        logits = np.random.default_rng(35).standard_normal((T, NE)).astype(np.float32)
        xb = az.Runtime.from_numpy(x)
        e.quantize(xb, E, E, Mp, T)
        lb = az.Runtime.from_numpy(logits)
        x0 = np.zeros((T, E), np.float32)
        ob = az.Runtime.from_numpy(x0)
        e.layer_moe(L, lb, NE, ob, T, Mp)
        out = ob.read(np.float32, T * E).reshape(T, E)
        n, S = T * NU, e.moe_slots
        inv = e.moe_buffer("inv").read(np.int32, n)
        ids = e.moe_buffer("ids").read(np.int32, n)
        swt = e.moe_buffer("swt").read(np.float32, n)
        h = e.moe_buffer("h").read(np.float32, S * F).reshape(S, F)[inv]          # pair order
        hq = e.moe_buffer("hq").read(np.int8, S * F).reshape(S, F)[inv]
        hsc = e.moe_buffer("hsc").read(np.float32, (F // 32) * S).reshape(F // 32, S)[:, inv]
        # gate/up against the golden values
        aq, asc, _ = quantize_padded(x, Mp)
        xa = (aq[:T].astype(np.float64).reshape(T, E // 32, 32) * asc[:, :T].T.astype(np.float64)[:, :, None]).reshape(T, E)
        href = np.zeros((n, F))
        for p in range(n):
            ex, t = int(ids[p]), p // NU
            g = vg[ex * F:(ex + 1) * F] @ xa[t]
            u = vu[ex * F:(ex + 1) * F] @ xa[t]
            with np.errstate(over="ignore"):      # (random f16 scales: exp(-g) may be inf, the quotient then 0)
                href[p] = g / (1.0 + np.exp(-g)) * u
        eh = rel_err_rows(h, href).max()
        # down + combine on the GPU's own int8 h against the golden values
        ha = (hq.astype(np.float64).reshape(n, F // 32, 32) * hsc.T.astype(np.float64)[:, :, None]).reshape(n, F)
        want = np.zeros((T, E))
        for p in range(n):
            ex = int(ids[p])
            want[p // NU] += float(swt[inv[p]]) * (vd[ex * E:(ex + 1) * E] @ ha[p])
        eo = rel_err_rows(out, want).max()
        print(f"  h {eh:.2e}  out {eo:.2e}")
        assert np.isfinite(out).all() and eh <= TOL and eo <= TOL
        for b in (xb, lb, ob):
            b.free()
    finally:
        e.close()
