"""numpy front end of the CPU oracle (oracle/libarcz_oracle.so) and, where it was built, of the reference's own
header compiled as oracle/_ref/libarcz_ref.so.  Test infrastructure: only tests, the smoke check and the bench's
cpu_baseline leg import this."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
Q4_0, Q8_0, Q3_K, Q4_K, Q5_K, Q6_K, IQ3_XXS, IQ4_NL, IQ3_S, IQ4_XS, MXFP4 = 2, 8, 11, 12, 13, 14, 18, 20, 21, 23, 39
Q2_0, AR4_128 = 42, 0x41523447
SB_BYTES = {Q2_0: 72, AR4_128: 132, Q4_0: 144, Q8_0: 272, Q4_K: 144, Q5_K: 176, Q6_K: 210, IQ3_S: 110, IQ4_XS: 136, IQ4_NL: 144, MXFP4: 136, Q3_K: 110, IQ3_XXS: 98}

_p, _i = C.c_void_p, C.c_int


def _load(path, build_target=None):
    if not os.path.exists(path) and build_target is not None:
        subprocess.run(["make", "-C", ORACLE_DIR, build_target], check=True, capture_output=True)
    return C.CDLL(path)


orc = _load(os.path.join(ORACLE_DIR, "libarcz_oracle.so"), "libarcz_oracle.so")
orc.orc_fp16_to_f32.restype = C.c_float
orc.orc_fp16_to_f32.argtypes = [C.c_uint16]
orc.orc_f32_to_fp16.restype = C.c_uint16
orc.orc_f32_to_fp16.argtypes = [C.c_float]
orc.orc_silu.restype = C.c_float
orc.orc_silu.argtypes = [C.c_float]

_ref_path = os.path.join(ORACLE_DIR, "_ref", "libarcz_ref.so")
ref = C.CDLL(_ref_path) if os.path.exists(_ref_path) else None
if ref is not None:
    ref.ref_fp16_to_f32.restype = C.c_float
    ref.ref_fp16_to_f32.argtypes = [C.c_uint16]
    ref.ref_f32_to_fp16.restype = C.c_uint16
    ref.ref_f32_to_fp16.argtypes = [C.c_float]


def ptr(a):
    return a.ctypes.data_as(_p)


def c8(a):
    return np.ascontiguousarray(a, dtype=np.uint8)


def dequant_rows(qtype, W, N, K, lib=None):
    """GGUF rows -> f32 [N][K] (oracle, or the compiled reference with lib=ref)."""
    W = c8(W)
    rb = K // 256 * SB_BYTES[qtype]
    out = np.empty((N, K), dtype=np.float32)
    f = orc.orc_dequant_row if lib is None else lib.ref_dequant_row
    for n in range(N):
        row = W[n * rb:(n + 1) * rb]
        assert f(C.c_uint32(qtype), ptr(row), _i(K), ptr(out[n])) == 0
    return out


def decode_row_fields(qtype, row, K):
    row = c8(row)
    q = np.empty(K, np.int8)
    isc = np.empty(K // 16, np.int32)
    imn = np.empty(K // 16, np.int32)
    d = np.empty(K // 32, np.float32)
    dmin = np.empty(K // 32, np.float32)
    assert orc.orc_decode_row_fields(C.c_uint32(qtype), ptr(row), _i(K), ptr(q), ptr(isc), ptr(imn), ptr(d), ptr(dmin)) == 0
    return q, isc, imn, d, dmin


def quantize_act(x, act32=True, lib=None):
    """f32 [M][K] -> aq int8 [M][K], asc f32 [K/B][M], absum int16 [K/16][M]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    B = 32 if act32 else 256
    aq = np.empty((M, K), np.int8)
    asc = np.empty((K // B, M), np.float32)
    absum = np.empty((K // 16, M), np.int16)
    if lib is None:
        orc.orc_quantize_act(ptr(x), _i(M), _i(K), ptr(aq), ptr(asc), ptr(absum), _i(1 if act32 else 0))
    else:
        lib.ref_quantize_act_cpu(ptr(x), _i(M), _i(K), ptr(aq), ptr(asc), ptr(absum), _i(1 if act32 else 0))
    return aq, asc, absum


def quantize_act_two_pass(x):
    """The two-pass inputs: (aq, asc, absum) of x and of what they miss (per-32 scales)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    aq, asc, absum = quantize_act(x)
    res = np.empty((M, K), np.float32)
    orc.orc_act_residual(ptr(x), _i(M), _i(K), ptr(aq), ptr(asc), _i(1), ptr(res))
    return (aq, asc, absum), quantize_act(res), res


def moe_quant(h, S=None):
    h = np.ascontiguousarray(h, dtype=np.float32)
    n, F = h.shape
    S = n if S is None else S
    hq = np.zeros((n, F), np.int8)
    hsc = np.zeros((F // 32, S), np.float32)
    orc.orc_moe_quant(ptr(h), _i(n), _i(F), _i(S), ptr(hq), ptr(hsc))
    return hq, hsc


def quantize_rows_q8_0(w, lib=None):
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    out = np.empty(N * (K // 32) * 34, np.uint8)
    (orc.orc_quantize_rows_q8_0 if lib is None else lib.ref_quantize_rows_q8_0)(ptr(w), _i(N), _i(K), ptr(out))
    return out


def quantize_rows_q4_0(w, lib=None):
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    out = np.empty(N * (K // 32) * 18, np.uint8)
    (orc.orc_quantize_rows_q4_0 if lib is None else lib.ref_quantize_rows_q4_0)(ptr(w), _i(N), _i(K), ptr(out))
    return out


def block_sums(qtype, W, N, K, aq):
    W = c8(W)
    aq = np.ascontiguousarray(aq, dtype=np.int8)
    M = aq.shape[0]
    out = np.empty((M, N, K // 16), np.int32)
    assert orc.orc_block_sums(C.c_uint32(qtype), ptr(W), _i(N), _i(K), ptr(aq), _i(M), ptr(out)) == 0
    return out


def matmul_ref(qtype, W, N, K, aq, asc):
    """Y [M][N] f32: double-accumulated dot of dequantized rows with q * scale activations."""
    W = c8(W)
    aq = np.ascontiguousarray(aq, dtype=np.int8)
    asc = np.ascontiguousarray(asc, dtype=np.float32)
    M, Ms = aq.shape[0], asc.shape[1]
    Y = np.empty((M, N), np.float32)
    assert orc.orc_matmul_ref(C.c_uint32(qtype), ptr(W), _i(N), _i(K), ptr(aq), ptr(asc), _i(Ms), _i(M), ptr(Y), _i(N)) == 0
    return Y


def matmul_formula(qtype, form, W, N, K, aq, asc, absum):
    W = c8(W)
    aq = np.ascontiguousarray(aq, dtype=np.int8)
    asc = np.ascontiguousarray(asc, dtype=np.float32)
    absum = np.ascontiguousarray(absum, dtype=np.int16)
    M, Ms = aq.shape[0], asc.shape[1]
    Y = np.empty((M, N), np.float32)
    assert orc.orc_matmul_formula(C.c_uint32(qtype), _i(form), ptr(W), _i(N), _i(K), ptr(aq), ptr(asc), ptr(absum), _i(Ms),
                                  _i(M), ptr(Y), _i(N)) == 0
    return Y


def moe_route(logits, NE, NU):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    T, ldl = logits.shape
    ids = np.empty((T, NU), np.int32)
    wts = np.empty((T, NU), np.float32)
    sgate = np.empty(T, np.float32)
    counts = np.empty(NE, np.int32)
    orc.orc_moe_route(ptr(logits), _i(ldl), _i(T), _i(NE), _i(NU), ptr(ids), ptr(wts), ptr(sgate), ptr(counts))
    return ids, wts, sgate, counts


def moe_route_v(logits, NE, NU, escale=None, ebias=None, rscale=1.0):
    """The routing with the reference's variants (moe.cl:17-46): expert scales, or the biased sqrt(softplus) scores."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    T, ldl = logits.shape
    ids = np.empty((T, NU), np.int32)
    wts = np.empty((T, NU), np.float32)
    sgate = np.empty(T, np.float32)
    counts = np.empty(NE, np.int32)
    es = None if escale is None else np.ascontiguousarray(escale, dtype=np.float32)
    eb = None if ebias is None else np.ascontiguousarray(ebias, dtype=np.float32)
    orc.orc_moe_route_v(ptr(logits), _i(ldl), _i(T), _i(NE), _i(NU), ptr(ids), ptr(wts), ptr(sgate), ptr(counts),
                        ptr(es) if es is not None else None, ptr(eb) if eb is not None else None, C.c_float(rscale))
    return ids, wts, sgate, counts


def moe_scan(counts, TM):
    counts = np.ascontiguousarray(counts, dtype=np.int32)
    NE = counts.size
    ntmax = int(((counts + TM - 1) // TM).sum())
    offs = np.empty(NE, np.int32)
    tiles = np.zeros(1 + 3 * max(ntmax, 1), np.int32)
    tstart = np.empty(NE + 1, np.int32)
    orc.orc_moe_scan(ptr(counts), _i(NE), _i(TM), ptr(offs), ptr(tiles), ptr(tstart))
    return offs, tiles, tstart


def moe_scatter(ids, wts, offs):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    wts = np.ascontiguousarray(wts, dtype=np.float32)
    T, NU = ids.shape
    n = T * NU
    stok = np.empty(n, np.int32)
    swt = np.empty(n, np.float32)
    inv = np.empty(n, np.int32)
    offs = np.ascontiguousarray(offs, dtype=np.int32)
    orc.orc_moe_scatter(ptr(ids), ptr(wts), _i(n), _i(NU), ptr(offs), _i(offs.size), ptr(stok), ptr(swt), ptr(inv))
    return stok, swt, inv


def moe_layer(qtype, Wg, Wu, Wd, NE, NU, E, F, aq, asc, logits):
    Wg, Wu, Wd = c8(Wg), c8(Wu), c8(Wd)
    aq = np.ascontiguousarray(aq, dtype=np.int8)
    asc = np.ascontiguousarray(asc, dtype=np.float32)
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    T, Ms = logits.shape[0], asc.shape[1]
    out = np.zeros((T, E), np.float32)
    h = np.zeros((T * NU, F), np.float32)
    assert orc.orc_moe_layer(C.c_uint32(qtype), ptr(Wg), ptr(Wu), ptr(Wd), _i(NE), _i(NU), _i(E), _i(F), ptr(aq), ptr(asc),
                             _i(Ms), _i(T), ptr(logits), _i(logits.shape[1]), ptr(out), ptr(h)) == 0
    return out, h


def num_threads():
    return orc.orc_num_threads()
