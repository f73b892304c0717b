"""Mixture-of-experts path on the GPU against the oracle: routing (ids and counts equal, weights < 1e-6, the bar of
the reference's own tests/test_route.cpp:28-96), the counting sort (invariants, and equality with the oracle's serial
order: the GPU scatter is deterministic), the expert-input quantizer (bit-exact on the GPU's own h), the grouped GEMM
and the whole layer (1e-3 of the f32 reference)."""
import numpy as np
import pytest

import arcinferzero_amd as az
import oracle_lib as orc
from common import TYPE_NAMES, make_acts, make_weights, quantize_padded, rel_err_rows

pytestmark = pytest.mark.gpu


def route_on_gpu(eng, L, logits, tm):
    T = logits.shape[0]
    lb = az.Runtime.from_numpy(logits)
    eng.moe_route(L, lb, logits.shape[1], T, tm)
    n = T * L.NU
    out = {
        "ids": eng.moe_buffer("ids").read(np.int32, n).reshape(T, L.NU),
        "wts": eng.moe_buffer("wts").read(np.float32, n).reshape(T, L.NU),
        "offs": eng.moe_buffer("offs").read(np.int32, L.NE),
        "tstart": eng.moe_buffer("tstart").read(np.int32, L.NE + 1),
        "stok": eng.moe_buffer("stok").read(np.int32, n),
        "swt": eng.moe_buffer("swt").read(np.float32, n),
        "inv": eng.moe_buffer("inv").read(np.int32, n),
    }
    nt = int(out["tstart"][-1])
    out["tiles"] = eng.moe_buffer("tiles").read(np.int32, 1 + 3 * nt)
    lb.free()
    return out


@pytest.mark.parametrize("NE,NU,T,tm", [(8, 2, 40, 16), (128, 8, 300, 128), (256, 6, 7, 16), (64, 8, 1, 128)])
def test_routing_and_sort(rt, NE, NU, T, tm):
    print(f"route NE={NE} NU={NU} T={T}", flush=True)
    eng = az.Engine(512, 256)
    try:
        dummy = np.zeros(az.gguf_bytes(az.Q8_0, NE * 256, 256), np.uint8)
        L = eng.make_moe_layer(az.Q8_0, dummy, dummy, dummy, NE, NU, 256, 256)
        rng = np.random.default_rng(11)
        logits = (rng.standard_normal((T, NE + 1)) * 2.0).astype(np.float32)
        logits[0, 3] = logits[0, 5] = logits[0].max() + 1.0       # a tie: the lower expert first
        g = route_on_gpu(eng, L, logits, tm)
        # the reference's CPU check: stable sort by descending logit
        for t in range(T):
            idx = np.argsort(-logits[t, :NE], kind="stable")[:NU]
            assert np.array_equal(g["ids"][t], idx)
            p = np.exp(logits[t, idx].astype(np.float64) - float(logits[t, idx[0]]))
            assert np.abs(g["wts"][t] - p / p.sum()).max() < 1e-6
        ids, wts, _, counts = orc.moe_route(logits, NE, NU)
        assert np.array_equal(g["ids"], ids) and np.abs(g["wts"] - wts).max() < 1e-6
        offs, tiles, tstart = orc.moe_scan(counts, tm)
        assert np.array_equal(g["offs"], offs) and np.array_equal(g["tstart"], tstart)
        assert np.array_equal(g["tiles"], tiles[:g["tiles"].size])
        # invariants of the sort
        n = T * NU
        assert counts.sum() == n and sorted(g["inv"].tolist()) == list(range(n))
        assert np.array_equal(g["stok"][g["inv"]], np.arange(n) // NU)
        assert np.array_equal(g["swt"][g["inv"]], g["wts"].reshape(-1))
        e_of_slot = np.repeat(np.arange(NE), counts)
        assert np.array_equal(e_of_slot[g["inv"]], g["ids"].reshape(-1))
        # and the deterministic order: equal to the oracle's serial scatter
        stok, swt, inv = orc.moe_scatter(g["ids"], g["wts"], offs)
        assert np.array_equal(g["inv"], inv) and np.array_equal(g["stok"], stok)
        # a second layer call must start from zeroed counts
        g2 = route_on_gpu(eng, L, logits, tm)
        assert np.array_equal(g2["offs"], offs) and np.array_equal(g2["inv"], inv)
    finally:
        eng.close()


@pytest.mark.parametrize("qtype,NE,NU,E,F,T,Mp", [(az.Q4_K, 8, 2, 256, 256, 40, 48), (az.Q8_0, 4, 2, 256, 512, 20, 32),
                                                   (az.Q6_K, 6, 3, 512, 256, 33, 48), (az.Q4_K, 16, 4, 512, 768, 300, 384),
                                                   (az.Q5_K, 8, 2, 512, 256, 70, 80),
                                                   # Q5_K experts with several tiles each, full ones among them
                                                   (az.Q5_K, 4, 2, 256, 512, 300, 320),
                                                   (az.IQ4_XS, 4, 2, 256, 512, 150, 160),
                                                   # passes of 1-16 tokens: the matrix-vector expert kernels on one-slot
                                                   # tiles (one or two tokens: routed inside the gate/up kernel)
                                                   (az.Q4_K, 128, 8, 512, 768, 1, 16), (az.Q4_K, 16, 4, 512, 256, 2, 16),
                                                   (az.Q4_K, 8, 2, 256, 768, 3, 16), (az.Q4_K, 128, 8, 2048, 768, 8, 16),
                                                   (az.Q8_0, 4, 2, 256, 512, 1, 16), (az.Q6_K, 6, 3, 512, 256, 5, 16),
                                                   (az.Q5_K, 8, 2, 512, 256, 7, 16), (az.IQ4_XS, 4, 2, 256, 512, 4, 16),
                                                   # IQ4_NL and MXFP4 experts: small passes and tile passes
                                                   (az.IQ4_NL, 4, 2, 256, 512, 1, 16), (az.IQ4_NL, 4, 2, 256, 512, 150, 160),
                                                   (az.MXFP4, 4, 2, 256, 512, 4, 16), (az.MXFP4, 6, 2, 512, 256, 40, 48),
                                                   # IQ3_XXS experts
                                                   (az.IQ3_XXS, 4, 2, 256, 512, 2, 16), (az.IQ3_XXS, 6, 2, 512, 256, 40, 48),
                                                   # Q3_K experts
                                                   (az.Q3_K, 4, 2, 256, 512, 3, 16), (az.Q3_K, 6, 2, 512, 256, 70, 80),
                                                   # IQ3_S experts (uploaded as Q6_K planes): one token and a tile pass
                                                   (az.IQ3_S, 4, 2, 256, 512, 1, 16), (az.IQ3_S, 6, 2, 512, 256, 40, 48),
                                                   # 9-16 tokens: still the matrix-vector form, the routing kernel's waves
                                                   # take two tokens each; 17: the tile GEMMs
                                                   (az.Q4_K, 128, 8, 512, 256, 16, 16), (az.Q6_K, 8, 3, 256, 256, 11, 16),
                                                   (az.Q4_K, 16, 4, 512, 256, 17, 32)])
def test_moe_layer_vs_oracle(rt, qtype, NE, NU, E, F, T, Mp):
    _moe_layer_vs_oracle(qtype, NE, NU, E, F, T, Mp)


@pytest.mark.parametrize("env", [{"ARCZ_MOE_TMD": "2"}, {"ARCZ_MOE_TMD": "4"}, {"ARCZ_MOE_TMD": "8"},
                                 {"ARCZ_MOE_FUSE": "0"}, {"ARCZ_MOE_FUSE": "0", "ARCZ_MOE_TMD": "4"},
                                 {"ARCZ_MOE_DECODE": "0"}, {"ARCZ_MOE_DECODE_MAX": "4"}])
@pytest.mark.parametrize("qtype,NE,NU,E,F,T", [(az.Q4_K, 16, 4, 512, 256, 7), (az.Q6_K, 8, 3, 256, 256, 2),
                                               (az.Q5_K, 128, 8, 512, 256, 1)])
def test_moe_small_pass_other_forms(rt, monkeypatch, env, qtype, NE, NU, E, F, T):
    """The earlier forms of a small pass, which the launch-rule switches bring back (an engine reads them when it is
    made): larger tiles, the five-launch form, the tile GEMMs.  Same checks as the default form."""
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    _moe_layer_vs_oracle(qtype, NE, NU, E, F, T, 16)


@pytest.mark.parametrize("env", [{}, {"ARCZ_MOE_QFUSE": "0"}, {"ARCZ_MOE_PRE": "0"}, {"ARCZ_MOE_PRE": "0", "ARCZ_MOE_QFUSE": "0"}])
@pytest.mark.parametrize("NE,NU,E,F,T,Mp", [(16, 4, 512, 256, 300, 304), (8, 2, 256, 512, 70, 80), (8, 3, 256, 768, 90, 96)])
def test_moe_tile_pass_quantization_forms(rt, monkeypatch, env, NE, NU, E, F, T, Mp):
    """Q4_K experts, a tile pass: the expert inputs quantized in the gate/up kernel's epilogue (F a multiple of 128, the
    default) and by the separate launch (ARCZ_MOE_QFUSE=0); the tile kernels on ready-made scale vectors (the default;
    with ARCZ_MOE_QFUSE=0 only the down kernel, its token side from a launch of its own) and forming them per tile and
    step (ARCZ_MOE_PRE=0): the layer checks hold for all, among them hq / hsc / hbs bit for bit what the quantizer
    makes of the GPU's own h."""
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    _moe_layer_vs_oracle(az.Q4_K, NE, NU, E, F, T, Mp)


@pytest.mark.parametrize("variant", [None, "escale"])
@pytest.mark.parametrize("NE,NU,E,F,T,Mp", [(16, 4, 512, 256, 300, 304), (128, 8, 2048, 768, 520, 528), (8, 2, 256, 512, 17, 32)])
def test_moe_ready_made_scale_vectors_change_no_bit(rt, monkeypatch, variant, NE, NU, E, F, T, Mp):
    """Unless ARCZ_MOE_PRE=0 (read when the engine is made) the Q4_K tile kernels take d * sc, -(dmin * mn) and sa * S from
    buffers made beforehand -- the rows' at upload, the tokens' by the routing launch (by a launch of its own with a
    routing variant) and by the gate / up kernel's epilogue -- instead of forming them per tile and step, the gate / up
    kernel in steps of 64 values instead of 128.  The same expressions in the same order: the layer's output, h, its
    int8 form and y are the plain engine's, bit for bit."""
    print(f"moe PRE NE={NE} NU={NU} E={E} F={F} T={T} {variant}", flush=True)
    Wg, Wu, Wd = (make_weights(az.Q4_K, NE * n, k, seed=s) for n, k, s in ((F, E, 1), (F, E, 2), (E, F, 3)))
    x = make_acts(T, E, seed=4)
    logits = np.random.default_rng(5).standard_normal((T, NE)).astype(np.float32)
    x0 = az.gen_normal(9, (T, E))
    escale = (0.5 + np.random.default_rng(6).random(NE)).astype(np.float32)
    got = []
    for pre in ("0", "1"):
        monkeypatch.setenv("ARCZ_MOE_PRE", pre)
        eng = az.Engine(Mp, max(E, F))
        try:
            L = eng.make_moe_layer(az.Q4_K, Wg, Wu, Wd, NE, NU, E, F)
            if variant:
                eng.set_moe_routing(L, escale=escale)
            xb, lb = az.Runtime.from_numpy(x), az.Runtime.from_numpy(logits)
            outs = []
            for rep in range(2):          # (the second call: on buffers the first has used)
                ob = az.Runtime.from_numpy(x0)
                eng.quantize(xb, E, E, Mp, T)
                eng.layer_moe(L, lb, NE, ob, T, Mp)
                outs.append(ob.read(np.float32, T * E).copy())
                ob.free()
            assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
            S, n = eng.moe_slots, T * NU
            used = np.sort(eng.moe_buffer("inv").read(np.int32, n))
            got.append((outs[0], eng.moe_buffer("h").read(np.float32, S * F).reshape(S, F)[used].copy(),
                        eng.moe_buffer("hq").read(np.int8, S * F).reshape(S, F)[used].copy(),
                        eng.moe_buffer("y").read(np.float32, S * E).reshape(S, E)[used].copy()))
            L.free(); xb.free(); lb.free()
        finally:
            eng.close()
    assert np.isfinite(got[0][0]).all() and np.abs(got[0][0] - x0.reshape(-1)).max() > 0
    for other in got[1:]:
        for a, b in zip(got[0], other):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


def _moe_layer_vs_oracle(qtype, NE, NU, E, F, T, Mp):
    print(f"moe layer {TYPE_NAMES[qtype]} NE={NE} NU={NU} E={E} F={F} T={T}", flush=True)
    eng = az.Engine(Mp, max(E, F))
    try:
        Wg = make_weights(qtype, NE * F, E, seed=1)
        Wu = make_weights(qtype, NE * F, E, seed=2)
        Wd = make_weights(qtype, NE * E, F, seed=3)
        L = eng.make_moe_layer(qtype, Wg, Wu, Wd, NE, NU, E, F)
        x = make_acts(T, E, seed=4)
        rng = np.random.default_rng(5)
        logits = rng.standard_normal((T, NE)).astype(np.float32)
        logits[:, 1] -= 50.0                                  # an expert that gets no token
        xb = az.Runtime.from_numpy(x)
        eng.quantize(xb, E, E, Mp, T)
        lb = az.Runtime.from_numpy(logits)
        x0 = az.gen_normal(9, (T, E))
        ob = az.Runtime.from_numpy(x0)
        eng.layer_moe(L, lb, NE, ob, T, Mp)
        out = ob.read(np.float32, T * E).reshape(T, E)
        aq, asc, _ = quantize_padded(x, Mp)
        ref, href = orc.moe_layer(qtype, Wg, Wu, Wd, NE, NU, E, F, aq[:T], asc, logits)
        err = rel_err_rows(out - x0, ref)
        print(f"  layer rel err {err.max():.2e}")
        assert np.isfinite(out).all()
        # h on the GPU (slot order) against the oracle's (pair order), then the second quantization bit for bit
        n = T * NU
        S = eng.moe_slots
        inv = eng.moe_buffer("inv").read(np.int32, n)
        h = eng.moe_buffer("h").read(np.float32, S * F).reshape(S, F)
        assert rel_err_rows(h[inv], href).max() <= 1e-3
        hq = eng.moe_buffer("hq").read(np.int8, S * F).reshape(S, F)
        hsc = eng.moe_buffer("hsc").read(np.float32, (F // 32) * S).reshape(F // 32, S)
        # Down projection and combine, every token count and launch form, on the GPU's own int8 h: out - x0 against
        # sum_k swt * (Wd_e . hq) in k order, 1e-3 for every token.  (The oracle's own h differs from the GPU's in its
        # last bits -- summation order -- so a value on a rounding boundary can quantize one int8 step apart; the
        # second quantization is defined on the GPU's h and checked bit for bit below, and this check carries the
        # layer's second half from exactly those int8 values.)
        ids = eng.moe_buffer("ids").read(np.int32, n)
        swt = eng.moe_buffer("swt").read(np.float32, n)
        rb = az.gguf_bytes(qtype, E, F)
        want = np.zeros((T, E), np.float64)
        for k in range(NU):
            for e in np.unique(ids[k::NU]):
                toks = np.nonzero(ids[k::NU] == e)[0]
                sl = inv[toks * NU + k]
                yr = orc.matmul_ref(qtype, Wd[e * rb:(e + 1) * rb], E, F, np.ascontiguousarray(hq[sl]),
                                    np.ascontiguousarray(hsc[:, sl]))
                want[toks] += yr.astype(np.float64) * swt[sl, None].astype(np.float64)
        err2 = rel_err_rows(out - x0, want)
        print(f"  down + combine on the GPU's int8 h: rel err {err2.max():.2e}")
        assert err2.max() <= 1e-3
        # The whole layer against the oracle's own two stages: every token whose int8 h equals the oracle's
        dq = hq[inv].astype(np.int32) - orc.moe_quant(href)[0].astype(np.int32)
        same = ~np.isin(np.arange(T), np.nonzero(dq.any(axis=1))[0] // NU)
        print(f"  int8 h values one step from the oracle's: {int((dq != 0).sum())} of {dq.size}, in {int((~same).sum())} tokens")
        # (a value of h within an ulp or two of a rounding boundary, or a block whose largest value is: a few in a million,
        #  never more than one step)
        assert np.abs(dq).max() <= 1 and (dq != 0).sum() <= 4 + dq.size // 10000
        assert err[same].max(initial=0.0) <= 1e-3
        if T >= 17:
            # the tile passes keep the down projection's weighted rows in y [S][E]: each expert's slots against the
            # oracle's matmul on the GPU's own int8 h
            y = eng.moe_buffer("y").read(np.float32, S * E).reshape(S, E)
            e_of_slot = np.full(S, -1)
            e_of_slot[inv] = ids
            for e in range(NE):
                sl = np.nonzero(e_of_slot == e)[0]
                if sl.size:
                    yr = orc.matmul_ref(qtype, Wd[e * rb:(e + 1) * rb], E, F, hq[sl], np.ascontiguousarray(hsc[:, sl]))
                    assert rel_err_rows(y[sl], yr * swt[sl, None]).max() <= 1e-3
        used = np.sort(inv)
        rq, rsc = orc.moe_quant(h[used])
        assert np.array_equal(hq[used], rq)
        assert np.array_equal(hsc[:, used].view(np.uint32), rsc.view(np.uint32))
        hbs = eng.moe_buffer("hbs").read(np.int16, (F // 16) * S).reshape(F // 16, S)
        assert np.array_equal(hbs[:, used].T, rq.astype(np.int32).reshape(len(used), F // 16, 16).sum(axis=2))
        for b in (xb, lb, ob):
            b.free()
    finally:
        eng.close()


@pytest.mark.parametrize("T", [1, 7, 40, 300])
@pytest.mark.parametrize("variant", ["escale", "route_ds"])
def test_routing_variants(rt, variant, T):
    """The reference's routing variants (zero/kernels/moe.cl:17-46): expert scales applied after the normalization; the
    sqrt(softplus) scores chosen with a bias.  Against the oracle and against the same formulas in float64."""
    NE, NU = 64, 6
    print(f"routing variant {variant} T={T}", flush=True)
    eng = az.Engine(512, 256)
    try:
        dummy = np.zeros(az.gguf_bytes(az.Q8_0, NE * 256, 256), np.uint8)
        L = eng.make_moe_layer(az.Q8_0, dummy, dummy, dummy, NE, NU, 256, 256)
        rng = np.random.default_rng(31 + T)
        logits = (rng.standard_normal((T, NE + 1)) * 2.0).astype(np.float32)
        escale = (0.5 + rng.random(NE)).astype(np.float32)
        ebias = (rng.standard_normal(NE) * 0.3).astype(np.float32)
        rscale = 2.5
        if variant == "escale":
            eng.set_moe_routing(L, escale=escale)
            ids, wts, sgate, counts = orc.moe_route_v(logits, NE, NU, escale=escale)
        else:
            eng.set_moe_routing(L, ebias=ebias, rscale=rscale)
            ids, wts, sgate, counts = orc.moe_route_v(logits, NE, NU, ebias=ebias, rscale=rscale)
        lb = az.Runtime.from_numpy(logits)
        x = az.Runtime.from_numpy(az.gen_normal(1, (T, 256)))
        eng.quantize(x, 256, 256, 512 if T > 16 else 16, T)
        out = az.Runtime.alloc(T * 256 * 4).fill(0)
        eng.layer_moe(L, lb, NE + 1, out, T, 512 if T > 16 else 16)       # (zero weights: only the routing matters)
        n = T * NU
        gi = eng.moe_buffer("ids").read(np.int32, n).reshape(T, NU) if T > 1 else None
        inv = eng.moe_buffer("inv").read(np.int32, n)
        gw = eng.moe_buffer("swt").read(np.float32, n)[inv].reshape(T, NU)
        gs = eng.moe_sgate.read(np.float32, T)
        if gi is not None:
            assert np.array_equal(gi, ids)
        else:   # one token: the chosen experts are the tiles' experts
            tiles = eng.moe_buffer("tiles").read(np.int32, 1 + 3 * NU)
            assert tiles[0] == NU and np.array_equal(tiles[1::3], ids[0])
        assert np.abs(gw - wts).max() < 1e-6 * max(1.0, np.abs(wts).max())
        assert np.abs(gs - sgate).max() < 1e-6
        # the formulas in float64
        l64 = logits[:, :NE].astype(np.float64)
        if variant == "escale":
            for t in range(T):
                idx = np.argsort(-l64[t], kind="stable")[:NU]
                p = np.exp(l64[t, idx] - l64[t, idx[0]])
                assert np.array_equal(ids[t], idx) and np.abs(wts[t] - p / p.sum() * escale[idx]).max() < 1e-5
            assert np.abs(sgate - 1.0 / (1.0 + np.exp(-logits[:, NE].astype(np.float64)))).max() < 1e-6
        else:
            sp = np.sqrt(np.where(l64 > 20, l64 + np.log1p(np.exp(-l64)), np.log1p(np.exp(l64))))
            for t in range(T):
                idx = np.argsort(-(sp[t].astype(np.float32) + ebias), kind="stable")[:NU]
                assert np.array_equal(ids[t], idx)
                assert np.abs(wts[t] - sp[t, idx] / (sp[t, idx].sum() + 1e-20) * rscale).max() < 1e-5
            assert (sgate == 1.0).all()
        eng.set_moe_routing(L)                                           # back to the softmax routing
        eng.layer_moe(L, lb, NE + 1, out, T, 512 if T > 16 else 16)
        inv = eng.moe_buffer("inv").read(np.int32, n)
        gw = eng.moe_buffer("swt").read(np.float32, n)[inv].reshape(T, NU)
        assert np.abs(gw - orc.moe_route(logits, NE, NU)[1]).max() < 1e-6
        for b in (lb, x, out):
            b.free()
    finally:
        eng.close()


@pytest.mark.parametrize("qtype,T,Mp", [(az.Q4_K, 1, 16), (az.Q4_K, 2, 16), (az.Q6_K, 6, 16), (az.Q4_K, 70, 80), (az.Q8_0, 33, 48)])
def test_moe_layer_with_shared_expert_term(rt, qtype, T, Mp):
    """moe_combine's shared-expert term (zero/kernels/moe.cl:344-352): router rows of NE + 1 logits, the last the shared
    expert's gate; x += sigmoid(gate) * sh + the experts' sum.  Against the same layer without the term."""
    NE, NU, E, F = 8, 2, 256, 256
    print(f"moe layer with sh, type {qtype} T={T}", flush=True)
    eng = az.Engine(Mp, 256)
    try:
        L = eng.make_moe_layer(qtype, make_weights(qtype, NE * F, E, seed=1), make_weights(qtype, NE * F, E, seed=2),
                               make_weights(qtype, NE * E, F, seed=3), NE, NU, E, F)
        rng = np.random.default_rng(7)
        logits = rng.standard_normal((T, NE + 1)).astype(np.float32)
        x0 = az.gen_normal(9, (T, E))
        sh = az.gen_normal(10, (T, E))
        xb = az.Runtime.from_numpy(make_acts(T, E, seed=4))
        eng.quantize(xb, E, E, Mp, T)
        lb, shb = az.Runtime.from_numpy(logits), az.Runtime.from_numpy(sh)
        o0, o1 = az.Runtime.from_numpy(x0), az.Runtime.from_numpy(x0)
        eng.layer_moe(L, lb, NE + 1, o0, T, Mp)
        eng.layer_moe(L, lb, NE + 1, o1, T, Mp, sh=shb)
        plain = o0.read(np.float32, T * E).reshape(T, E)
        with_sh = o1.read(np.float32, T * E).reshape(T, E)
        gate = 1.0 / (1.0 + np.exp(-logits[:, NE].astype(np.float64)))
        assert np.abs(eng.moe_sgate.read(np.float32, T) - gate).max() < 1e-6
        want = plain.astype(np.float64) + gate[:, None] * sh
        assert np.abs(with_sh - want).max() <= 2e-6 * np.abs(want).max()
        # and the routing ignored the extra column
        ids, _, _, _ = orc.moe_route(logits, NE, NU)
        if T > 1:
            assert np.array_equal(eng.moe_buffer("ids").read(np.int32, T * NU).reshape(T, NU), ids)
        for b in (xb, lb, shb, o0, o1):
            b.free()
    finally:
        eng.close()


@pytest.mark.parametrize("qtype,NE,NU,E,F,T,Mp", [(az.MXFP4, 4, 2, 352, 160, 3, 16), (az.MXFP4, 4, 2, 352, 160, 70, 80),
                                                   (az.Q8_0, 6, 3, 512, 96, 40, 48), (az.IQ4_NL, 4, 2, 2880, 2880, 5, 16)])
def test_moe_layer_of_widths_that_are_not_whole_superblocks(rt, qtype, NE, NU, E, F, T, Mp):
    """Expert tensors whose hidden or FFN width is not a multiple of 256 (the reference's Gemma 4 layers with F = 704;
    MXFP4 layers of 2880 x 2880): the upload pads rows and columns with zeros to whole superblocks, as the reference's
    loader pads (zero/engine_load.h:371-387), the layer reports the rounded-up widths, and on activations and residual
    rows of those widths whose tails are zero it gives, bit for bit, what the same tensors padded by hand give -- a
    layer of whole superblocks, which the other tests hold to the oracle."""
    print(f"moe layer padded {TYPE_NAMES[qtype]} NE={NE} NU={NU} E={E} F={F} T={T}", flush=True)
    Ep, Fp = (E + 255) // 256 * 256, (F + 255) // 256 * 256
    bb = az.gguf_bytes(qtype, 1, 256) // 8
    def cut(seed, N, K, Np, Kp):
        """[NE][Np][Kp] generated, then the rows and blocks past N and K zeroed: the padded tensor and the one a file holds."""
        full = make_weights(qtype, NE * Np, Kp, seed=seed).reshape(NE, Np, Kp // 32, bb).copy()
        full[:, N:] = 0
        full[:, :, K // 32:] = 0
        return full.reshape(-1), np.ascontiguousarray(full[:, :N, :K // 32]).reshape(-1)
    Gp, G = cut(1, F, E, Fp, Ep)
    Up, U = cut(2, F, E, Fp, Ep)
    Dp, D = cut(3, E, F, Ep, Fp)
    eng = az.Engine(Mp, max(Ep, Fp))
    try:
        x = np.zeros((T, Ep), np.float32)
        x[:, :E] = make_acts(T, E, seed=4)
        x0 = np.zeros((T, Ep), np.float32)
        x0[:, :E] = az.gen_normal(9, (T, E))
        logits = np.random.default_rng(5).standard_normal((T, NE)).astype(np.float32)
        xb, lb = az.Runtime.from_numpy(x), az.Runtime.from_numpy(logits)
        eng.quantize(xb, Ep, Ep, Mp, T)
        outs = []
        for tensors, dims in (((G, U, D), (E, F)), ((Gp, Up, Dp), (Ep, Fp))):
            L = eng.make_moe_layer(qtype, *tensors, NE, NU, *dims)
            assert (L.E, L.F) == (Ep, Fp)
            ob = az.Runtime.from_numpy(x0)
            eng.layer_moe(L, lb, NE, ob, T, Mp)
            outs.append(ob.read(np.float32, T * Ep).reshape(T, Ep))
            ob.free()
        assert np.isfinite(outs[0]).all() and np.abs(outs[0] - x0).max() > 0
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
        assert np.array_equal(outs[0][:, E:], x0[:, E:])            # the padding columns of x: nothing added
        with pytest.raises(az.ArczError):
            eng.make_moe_layer(az.Q4_K, G, U, D, NE, NU, E, F)       # superblock types: whole superblocks only
        xb.free(); lb.free()
    finally:
        eng.close()


def test_moe_layer_upload_checks_the_tensors_byte_counts(rt):
    """An expert tensor with fewer (or more) bytes than its type and shape come to is refused before anything is read,
    for whole-superblock widths and for the padded ones alike."""
    for qtype, NE, E, F in [(az.Q4_K, 4, 512, 256), (az.Q8_0, 4, 640, 352)]:
        eng = az.Engine(16, 1024)   # (an engine takes one expert geometry)
        try:
            Wg = make_weights(qtype, NE * F, E, seed=1) if E % 256 == 0 else np.zeros(NE * F * (E // 32) * 34, np.uint8)
            Wd = make_weights(qtype, NE * E, F, seed=3) if F % 256 == 0 else np.zeros(NE * E * (F // 32) * 34, np.uint8)
            for bad in ("gate", "up", "down"):
                g, u, d = Wg, Wg.copy(), Wd
                if bad == "gate":
                    g = g[:-34]
                elif bad == "up":
                    u = np.concatenate([u, u[:34]])
                else:
                    d = d[: d.size // 2]
                with pytest.raises(az.ArczError) as e:
                    eng.make_moe_layer(qtype, g, u, d, NE, 2, E, F)
                assert "bytes" in str(e.value)
            L = eng.make_moe_layer(qtype, Wg, Wg.copy(), Wd, NE, 2, E, F)
            L.free()
        finally:
            eng.close()
