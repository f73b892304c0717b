"""The configurations of the headline measurements at their full sizes.  The oracle cannot redo a trillion products in a
test, so each case checks (a) sampled outputs (rows x tokens spread over the whole matrix, first and last included)
against the oracle's double-accumulated reference to the stated 1e-3, (b) properties that hold at any size: the GEMM's
row for a token equals the GEMV of that token to rounding, two runs are bit-identical, padding rows come out zero,
and for the MoE layer the invariants of the sort plus sampled tokens through the oracle's whole layer."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import rel_err_rows

pytestmark = pytest.mark.gpu


def sampled_check(qtype, W, N, K, y, aq, asc, toks, rows):
    rb = az.gguf_bytes(qtype, 1, K)
    Wr = np.concatenate([W[r * rb:(r + 1) * rb] for r in rows])
    ref = orc.matmul_ref(qtype, Wr, len(rows), K, aq[toks], np.ascontiguousarray(asc[:, toks]))
    got = y[np.ix_(toks, rows)]
    err = rel_err_rows(got, ref)
    assert np.isfinite(got).all() and err.max() <= 1e-3, err.max()
    return err.max()


def spread(n, k):
    idx = np.unique(np.concatenate([np.linspace(0, n - 1, k).astype(np.int64), [0, n - 1]]))
    return idx


@pytest.mark.parametrize("qtype,N,K,M,T", [(az.Q4_K, 17408, 5120, 8192, 8192), (az.Q4_K, 17408, 5120, 8192, 8000),
                                           (az.Q6_K, 151936, 5120, 64, 64), (az.Q8_0, 4096, 4096, 512, 512),
                                           # the output head as a prefill GEMM: 2048 tokens, 1.24 GB of output
                                           (az.Q6_K, 151936, 5120, 2048, 2048),
                                           # the other weight types and launch forms at the headline matrix's size:
                                           # Q5_K and IQ4_XS, a 64- and a 128-token chunk (K shared out over several
                                           # work-groups per tile), 16 and 7 tokens (the matrix-pipe GEMV)
                                           (az.Q5_K, 17408, 5120, 2048, 2048), (az.IQ4_XS, 17408, 5120, 1024, 1000),
                                           (az.Q4_K, 17408, 5120, 64, 64), (az.Q4_K, 17408, 5120, 128, 100),
                                           (az.Q4_K, 17408, 5120, 16, 16), (az.Q4_K, 5120, 17408, 16, 7)])
def test_prefill_configs_full_size(rt, qtype, N, K, M, T):
    print(f"full size type {qtype} N={N} K={K} M={M} T={T}", flush=True)
    eng = az.Engine(M, K)
    try:
        W = az.gen_weights(qtype, 1, N, K, 0.02)
        w = eng.make_weight(qtype, N, K, W)
        x = az.gen_normal(2, (T, K))
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, K, K, M, T)
        aq, asc, _ = eng.read_activations(K, M)
        cb = az.Runtime.alloc(M * N * 4).fill(0x7FC00000)          # NaN: a tile that is not written shows
        eng.matmul("full", w, M, cb, N, 0, 0)
        y = cb.read(np.float32, M * N).reshape(M, N)
        if T <= 8:                                                  # a pass of 1-8 tokens writes its T rows only
            y[T:] = 0.0
        assert np.isfinite(y).all()
        if T < M:
            assert not y[T:].any()                                  # padding rows: zero activations, zero output
        toks, rows = spread(T, 24), spread(N, 96)
        e = sampled_check(qtype, W, N, K, y, aq, asc, toks, rows)
        print(f"  sampled rel err {e:.2e}", flush=True)
        # bit-identical run to run
        cb2 = az.Runtime.alloc(M * N * 4).fill(0)
        eng.matmul("full", w, M, cb2, N, 0, 0)
        y2 = cb2.read(np.float32, M * N).reshape(M, N)
        assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))
        # the GEMM's row of a token against the GEMV of that token alone (same int8 row, same scales)
        for t in (0, T // 2, T - 1):
            a1 = np.zeros((16, K), np.int8); a1[0] = aq[t]
            s1 = np.zeros((K // 32, 16), np.float32); s1[:, 0] = asc[:, t]
            b1 = a1.astype(np.int32).reshape(16, K // 16, 16).sum(axis=2).T.astype(np.int16)
            eng1 = az.Engine(16, K)
            eng1.set_activations(a1, s1, np.ascontiguousarray(b1), K, 16, 1)
            c1 = az.Runtime.alloc(N * 4)
            eng1.matmul("row", w, 16, c1, N, 0, 0)
            yv = c1.read(np.float32, N)
            assert np.abs(yv - y[t]).max() <= 2e-5 * np.abs(y[t]).max()
            c1.free(); eng1.close()
        for b in (cb, cb2, xb):
            b.free()
        w.free()
    finally:
        eng.close()


def test_decode_output_head_full_size(rt):
    """Q6_K 151936 x 5120, one and two tokens: every output against sampled oracle rows; the two-token launch's rows
    against the one-token launches."""
    qtype, N, K = az.Q6_K, 151936, 5120
    eng = az.Engine(16, K)
    try:
        W = az.gen_weights(qtype, 3, N, K, 0.02)
        w = eng.make_weight(qtype, N, K, W)
        x = az.gen_normal(4, (2, K))
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, K, K, 16, 2)
        aq, asc, _ = eng.read_activations(K, 16)
        cb = az.Runtime.alloc(2 * N * 4).fill(0x7FC00000)
        eng.matmul("head", w, 16, cb, N, 0, 0)
        y = cb.read(np.float32, 2 * N).reshape(2, N)
        sampled_check(qtype, W, N, K, y, aq, asc, np.arange(2), spread(N, 256))
        eng.quantize(xb, K, K, 16, 1)
        c1 = az.Runtime.alloc(N * 4).fill(0x7FC00000)
        eng.matmul("head", w, 16, c1, N, 0, 0)
        y1 = c1.read(np.float32, N)
        assert np.isfinite(y1).all() and np.abs(y1 - y[0]).max() <= 2e-5 * np.abs(y1).max()
        for b in (cb, c1, xb):
            b.free()
    finally:
        eng.close()


def test_moe_layer_full_size(rt):
    """128 experts, top 8, 4096 tokens, hidden 2048, expert FFN 768, Q4_K: sort invariants on all 32768 pairs, sampled
    tokens through the oracle's layer (routing is per token, so a subset of tokens is a valid sub-problem)."""
    NE, NU, T, E, F, qt = 128, 8, 4096, 2048, 768, az.Q4_K
    eng = az.Engine(T, E)
    try:
        Wg = az.gen_weights(qt, 21, NE * F, E, 0.02)
        Wu = az.gen_weights(qt, 22, NE * F, E, 0.02)
        Wd = az.gen_weights(qt, 23, NE * E, F, 0.02)
        L = eng.make_moe_layer(qt, Wg, Wu, Wd, NE, NU, E, F)
        x = az.gen_normal(24, (T, E))
        logits = az.gen_normal(25, (T, NE))
        xb, lb = az.Runtime.from_numpy(x), az.Runtime.from_numpy(logits)
        ob = az.Runtime.alloc(T * E * 4).fill(0)
        eng.quantize(xb, E, E, T, T)
        aq, asc, _ = eng.read_activations(E, T)
        eng.layer_moe(L, lb, NE, ob, T, T)
        out = ob.read(np.float32, T * E).reshape(T, E)
        n = T * NU
        inv = eng.moe_buffer("inv").read(np.int32, n)
        stok = eng.moe_buffer("stok").read(np.int32, n)
        ids = eng.moe_buffer("ids").read(np.int32, n)
        offs = eng.moe_buffer("offs").read(np.int32, NE)
        assert sorted(inv.tolist()) == list(range(n)) and np.array_equal(stok[inv], np.arange(n) // NU)
        counts = np.bincount(ids, minlength=NE)
        assert counts.sum() == n and np.array_equal(offs, np.concatenate([[0], np.cumsum(counts)[:-1]]))
        slot_expert = np.repeat(np.arange(NE), counts)
        assert np.array_equal(slot_expert[inv], ids)                # every pair sits in its expert's run of slots
        toks = spread(T, 12)
        ref, _ = orc.moe_layer(qt, Wg, Wu, Wd, NE, NU, E, F, aq[toks], np.ascontiguousarray(asc[:, toks]), logits[toks])
        err = rel_err_rows(out[toks], ref)
        print(f"  MoE sampled rel err {err.max():.2e}", flush=True)
        assert np.isfinite(out).all() and err.max() <= 1e-3
        ob2 = az.Runtime.alloc(T * E * 4).fill(0)
        eng.layer_moe(L, lb, NE, ob2, T, T)                         # bit-identical run to run (the sort is deterministic)
        assert np.array_equal(ob2.read(np.uint32, T * E), out.view(np.uint32).ravel())
        for b in (xb, lb, ob, ob2):
            b.free()
    finally:
        eng.close()
