"""Weights taken from a GGUF file (the upload of the reference's zero/engine_load.h:84-196 on tensors of its GgufFile):
a matrix of each type through GEMV and GEMM, and a MoE layer from three expert tensors, against the oracle."""
import numpy as np
import pytest

import arcinferzero_amd as az
import gguf_writer as gw
import oracle_lib as orc
from common import TYPE_NAMES, make_acts, make_weights, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu


def test_matrices_from_gguf(rt, tmp_path):
    K, N = 1024, 384
    Ws = {az.Q8_0: make_weights(az.Q8_0, N, K, seed=401), az.Q4_K: make_weights(az.Q4_K, N, K, seed=402),
          az.Q6_K: make_weights(az.Q6_K, N, K, seed=403), az.Q4_0: make_weights(az.Q4_0, N, K, seed=404),
          az.Q5_K: make_weights(az.Q5_K, N, K, seed=405), az.IQ4_XS: make_weights(az.IQ4_XS, N, K, seed=406),
          az.IQ3_S: make_weights(az.IQ3_S, N, K, seed=407)}
    tensors = [(f"blk.{t}.weight", t, [K, N], W) for t, W in Ws.items()]
    tensors.insert(1, ("pad.me", 0, [3], np.zeros(12, np.uint8)))      # makes the next tensor's offset matter
    p = tmp_path / "w.gguf"
    gw.write_gguf(p, [("general.architecture", gw.T_STR, "test")], tensors)
    eng = az.Engine(128, K)
    try:
        with az.GgufFile(p) as g:
            ws = {t: eng.make_weight_gguf(g, f"blk.{t}.weight") for t in Ws}
            with pytest.raises(az.ArczError):
                eng.make_weight_gguf(g, "nope")
            with pytest.raises(az.ArczError):
                eng.make_weight_gguf(g, "pad.me")                       # F32 vector: no matrix of a supported type
        # (the file is closed: the weights live on the device)
        for T, Mp in ((1, 16), (100, 112)):
            x = make_acts(T, K, seed=410 + T)
            aq, asc, absum = quantize_padded(x, Mp)
            eng.set_activations(aq, asc, absum, K, Mp, T)
            rows = T if T <= 8 else Mp
            for t, w in ws.items():
                assert (w.N, w.K, w.type) == (N, K, t)
                cb = az.Runtime.alloc(rows * N * 4)
                eng.matmul("t", w, Mp, cb, N, 0, 0)
                y = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
                ref = orc.matmul_ref(t, Ws[t], N, K, aq[:T], asc)
                assert rel_err_rows(y, ref).max() <= 1e-3
                cb.free()
    finally:
        eng.close()


def test_moe_layer_from_gguf(rt, tmp_path):
    NE, NU, E, F, T, Mp = 8, 2, 512, 256, 40, 48
    qt = az.Q4_K
    Wg, Wu = make_weights(qt, NE * F, E, seed=421), make_weights(qt, NE * F, E, seed=422)
    Wd = make_weights(qt, NE * E, F, seed=423)
    p = tmp_path / "moe.gguf"
    gw.write_gguf(p, [], [("blk.0.ffn_gate_exps.weight", qt, [E, F, NE], Wg), ("blk.0.ffn_up_exps.weight", qt, [E, F, NE], Wu),
                          ("blk.0.ffn_down_exps.weight", qt, [F, E, NE], Wd)])
    eng = az.Engine(Mp, E)
    try:
        with az.GgufFile(p) as g:
            L = eng.make_moe_layer_gguf(g, "blk.0.ffn_gate_exps.weight", "blk.0.ffn_up_exps.weight",
                                        "blk.0.ffn_down_exps.weight", NU)
            with pytest.raises(az.ArczError):
                eng.make_moe_layer_gguf(g, "blk.0.ffn_gate_exps.weight", "blk.0.ffn_down_exps.weight",
                                        "blk.0.ffn_down_exps.weight", NU)   # shapes of different projections
        assert (L.NE, L.NU, L.E, L.F) == (NE, NU, E, F)
        x = make_acts(T, E, seed=424)
        logits = az.gen_normal(425, (T, NE))
        aq, asc, absum = quantize_padded(x, Mp)
        eng.set_activations(aq, asc, absum, E, Mp, T)
        lb = az.Runtime.from_numpy(logits)
        ob = az.Runtime.alloc(T * E * 4).fill(0)
        eng.layer_moe(L, lb, NE, ob, T, Mp)
        out = ob.read(np.float32, T * E).reshape(T, E)
        ref, _ = orc.moe_layer(qt, Wg, Wu, Wd, NE, NU, E, F, aq[:T], asc, logits)
        assert rel_err_rows(out, ref).max() <= 1e-3
        lb.free(); ob.free()
    finally:
        eng.close()


@pytest.mark.parametrize("qtype,N,K,T,Mp", [(az.Q8_0, 200, 640, 1, 16), (az.MXFP4, 136, 2880, 3, 16), (az.IQ4_NL, 64, 96, 12, 16),
                                            (az.Q4_0, 300, 2880, 100, 112), (az.MXFP4, 520, 2880, 300, 304)])
def test_rows_that_end_inside_a_superblock(rt, qtype, N, K, T, Mp):
    """Rows of a 32-value-block type whose K is a multiple of 32 but not of 256 (the reference's 640-wide shared expert;
    MXFP4 matrices of 2880 columns): the upload pads them with zero blocks to whole superblocks, as the reference's
    loader does (zero/engine_load.h:371-387, src/quants.h:661-671), the weight reports the rounded-up K, and the
    product with activation rows of that length whose tail is zero equals the double-accumulated reference on the
    unpadded rows."""
    print(f"padded rows {TYPE_NAMES[qtype]} N={N} K={K} T={T}", flush=True)
    Kp = (K + 255) // 256 * 256
    bb = az.gguf_bytes(qtype, 1, 256) // 8                          # bytes of a 32-value block
    full = make_weights(qtype, N, Kp, seed=470).reshape(N, Kp // 32, bb)
    W = np.ascontiguousarray(full[:, :K // 32]).reshape(-1)         # rows of K values as a file would hold them
    eng = az.Engine(Mp, Kp)
    try:
        w = eng.make_weight(qtype, N, K, W)
        assert w.K == Kp and az.lib.arcz_mem_size(az.lib.arcz_weight_raw(w.h)) == az.planes_bytes(qtype, N, Kp)
        x = np.zeros((T, Kp), np.float32)
        x[:, :K] = make_acts(T, K, seed=471, outliers=True)
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, Kp, Kp, Mp, T)
        rows = T if T <= 8 else Mp
        cb = az.Runtime.alloc(rows * N * 4).fill(0xFFFFFFFF)
        eng.matmul("padded", w, Mp, cb, N, 0, 0)
        y = cb.read(np.float32, rows * N).reshape(rows, N)[:T]
        zero_tail = full.copy()
        zero_tail[:, K // 32:] = 0                                   # what the device holds: zero blocks behind the rows
        aq, asc, _ = quantize_padded(x, Mp)
        ref = orc.matmul_ref(qtype, zero_tail.reshape(-1), N, Kp, aq[:T], asc)
        assert np.isfinite(y).all() and rel_err_rows(y, ref).max() <= 1e-3
        # ... which is the product over the first K columns alone
        assert np.abs(orc.dequant_rows(qtype, zero_tail.reshape(-1), N, Kp)[:, K:]).max() == 0.0
        with pytest.raises(az.ArczError):
            eng.make_weight(az.Q4_K, N, K, W)                       # superblock types: whole superblocks only
        for b in (cb, xb):
            b.free()
        w.free()
    finally:
        eng.close()
