"""ctypes binding of libarcz_hip.so (include/arcz_hip.h, include/arcz_engine.h).

Names follow the reference engine: Engine.matmul(name, w, Mp, C, ldc, c_off, acc, act32) is zero/engine.h:1080,
Runtime.kernel(which, defs, name) is zero/engine_setup.h:317, Buffer is a cl_mem.  Every call goes through the C ABI;
errors come back as status codes and are raised as ArczError with the library's message.
"""
import ctypes as C
import os

import numpy as np

Q4_0, Q8_0, Q3_K, Q4_K, Q5_K, Q6_K, IQ3_XXS, IQ4_NL, IQ3_S, IQ4_XS, MXFP4 = 2, 8, 11, 12, 13, 14, 18, 20, 21, 23, 39  # GGUF type ids
Q2_0, AR4_128 = 42, 0x41523447   # (uploaded as Q4_0 blocks of the same values)

lib_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libarcz_hip.so")
if not os.path.exists(lib_path):
    raise ImportError(
        f"{lib_path} is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
        "(or make -C arcinferzero_amd/csrc); there is no fallback path")
lib = C.CDLL(lib_path)


class ArczError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"[{code}] {msg}")
        self.code = code


def _sig(name, restype, *argtypes):
    f = getattr(lib, name)
    f.restype = restype
    f.argtypes = list(argtypes)
    return f


_p, _i, _z, _u32, _u64 = C.c_void_p, C.c_int, C.c_size_t, C.c_uint32, C.c_uint64
_sig("arcz_init", _i, _i)
_sig("arcz_shutdown", None)
_sig("arcz_last_error", C.c_char_p)
_sig("arcz_device_name", C.c_char_p)
_sig("arcz_device_cus", _i)
_sig("arcz_device_mem", _z)
_sig("arcz_device_bytes", _z)
_sig("arcz_alloc", _p, _z)
_sig("arcz_view", _p, _p, _z, _z)
_sig("arcz_free", _i, _p)
_sig("arcz_mem_size", _z, _p)
_sig("arcz_mem_ptr", _p, _p)
_sig("arcz_h2d", _i, _p, _z, _p, _z)
_sig("arcz_d2h", _i, _p, _p, _z, _z)
_sig("arcz_d2d", _i, _p, _z, _p, _z, _z)
_sig("arcz_fill", _i, _p, _p, _z, _z, _z)
_sig("arcz_kernel_get", _p, C.c_char_p, C.c_char_p, C.c_char_p)
_sig("arcz_kernel_symbol", C.c_char_p, _p)
_sig("arcz_launch", _i, _p, C.c_uint, C.POINTER(_z), C.POINTER(_z), C.POINTER(_p), C.POINTER(_z), C.c_uint, C.POINTER(_p))
_sig("arcz_sync", _i)
_sig("arcz_event_ms", C.c_double, _p)
_sig("arcz_event_release", None, _p)
_sig("arcz_event_record", _p)
_sig("arcz_event_elapsed_ms", C.c_double, _p, _p)
_sig("arcz_set_fake_oom", None, C.c_long)
_sig("arcz_set_oom_hook", None, _p)
_sig("arcz_launch_count", _u64)
_sig("arcz_record_begin", _i)
_sig("arcz_record_end", _i, _p)
_sig("arcz_recording", _i)
_sig("arcz_list_run", _i, _p)
_sig("arcz_list_launches", _u64, _p)
_sig("arcz_list_free", _i, _p)
_sig("arcz_engine_error", C.c_char_p)
_sig("arcz_engine_create", _p, _i, _i)
_sig("arcz_engine_destroy", None, _p)
_sig("arcz_weight_upload", _p, _p, _u32, _i, _i, _p, _z)
_sig("arcz_weight_upload_gguf", _p, _p, _p, C.c_char_p)
_sig("arcz_moe_layer_upload_gguf", _p, _p, _p, C.c_char_p, C.c_char_p, C.c_char_p, _i)
_sig("arcz_gguf_open", _p, C.c_char_p)
_sig("arcz_gguf_close", None, _p)
_sig("arcz_gguf_error", C.c_char_p)
_sig("arcz_gguf_version", _u32, _p)
_sig("arcz_gguf_n_kv", _z, _p)
_sig("arcz_gguf_n_tensors", _z, _p)
_sig("arcz_gguf_alignment", _u64, _p)
_sig("arcz_gguf_kv_i64", _i, _p, C.c_char_p, C.POINTER(C.c_int64))
_sig("arcz_gguf_kv_f64", _i, _p, C.c_char_p, C.POINTER(C.c_double))
_sig("arcz_gguf_kv_str", C.c_char_p, _p, C.c_char_p)
_sig("arcz_gguf_tensor", _i, _p, _z, C.POINTER(C.c_char_p), C.POINTER(_u32), C.POINTER(_u32), C.POINTER(_u64 * 8),
     C.POINTER(_p), C.POINTER(_u64))
_sig("arcz_gguf_find", C.c_long, _p, C.c_char_p)
_sig("arcz_ggml_block_info", _i, _u32, C.POINTER(_i), C.POINTER(_i))
_sig("arcz_weight_free", _i, _p, _p)
_sig("arcz_weight_raw", _p, _p)
_sig("arcz_mem_listed", C.c_int, _p)
_sig("arcz_weight_k", C.c_int, _p)
_sig("arcz_moe_layer_dims", C.c_int, _p, C.POINTER(C.c_int), C.POINTER(C.c_int))
_sig("arcz_engine_quantize", _i, _p, _p, _i, _i, _i, _i, _i)
_sig("arcz_engine_rmsnorm_quant", _i, _p, _p, _i, _p, _i, _i, _i, _i, C.c_float, _p)
_sig("arcz_engine_add_norm_quant", _i, _p, _p, _p, _p, _i, _i, _i, C.c_float, _p, _i, _i, C.c_float)
_sig("arcz_engine_swiglu_quant", _i, _p, _p, _i, _i, _i, _i, _i, _i)
_sig("arcz_engine_set_activations", _i, _p, _p, _p, _p, _i, _i, _i)
_sig("arcz_engine_aq", _p, _p)
_sig("arcz_engine_two_pass", _i, _p, _i)
_sig("arcz_engine_residual", _p, _p, _i)
_sig("arcz_engine_asc", _p, _p)
_sig("arcz_engine_absum", _p, _p)
_sig("arcz_engine_matmul", _i, _p, C.c_char_p, _p, _i, _p, _i, _i, _i, _i)
_sig("arcz_iq3s_grid", None, _p)
_sig("arcz_iq3xxs_grid", None, _p)
_sig("arcz_weight_set_softcap", _i, _p, C.c_float)
_sig("arcz_engine_gemv_gu", _i, _p, _p, _p, _i, _p)
_sig("arcz_engine_matmul_noalloc", _i, _p, C.c_char_p, _p, _i, _p, _i, _i, _i, _i)
_sig("arcz_moe_layer_upload", _p, _p, _u32, _p, _z, _p, _z, _p, _z, _i, _i, _i, _i)
_sig("arcz_engine_layer_moe", _i, _p, _p, _p, _i, _p, _i, _i)
_sig("arcz_engine_moe_route", _i, _p, _p, _p, _i, _i, _i)
_sig("arcz_engine_layer_moe_sh", _i, _p, _p, _p, _i, _p, _i, _i, _p)
_sig("arcz_moe_layer_set_routing", _i, _p, _p, _p, _p, C.c_float)
_sig("arcz_moe_layer_free", _i, _p, _p)
_sig("arcz_engine_moe_sgate", _p, _p)
_sig("arcz_engine_moe_buffer", _p, _p, _i)
_sig("arcz_engine_moe_slots", _i, _p)
_sig("arcz_engine_self_check", _i)
_sig("arcz_engine_profile", None, _p, _i)
_sig("arcz_engine_profile_collect", _i, _p)
_sig("arcz_engine_profile_get", _i, _p, C.c_char_p, C.POINTER(C.c_double), C.POINTER(_i))
_sig("arcz_engine_profile_stats", _i, _p, C.c_char_p, C.POINTER(C.c_double), C.POINTER(C.c_double))
_sig("arcz_engine_profile_reset", None, _p)
_sig("arcz_engine_rd_bytes", _u64, _p)
_sig("arcz_gguf_bytes", _z, _u32, _z, _i)
_sig("arcz_planes_bytes", _z, _u32, _z, _i)
_sig("arcz_repack_planes", _i, _u32, _z, _i, _p, _p)
_sig("arcz_relayout_q4_0", _z, _u32, _z, _i, _p, _p)
_sig("arcz_quantize_rows", _i, _u32, _p, _z, _i, _p)
_sig("arcz_gen_normal", None, _u64, _z, C.c_float, C.c_float, _p)
_sig("arcz_gen_weights", _i, _u32, _u64, _z, _i, C.c_float, _p)


def _check(code, engine=False):
    if code != 0:
        msg = (lib.arcz_engine_error() if engine and code == -100 else lib.arcz_last_error()) or b""
        raise ArczError(code, msg.decode(errors="replace"))


def _np_ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def self_check():
    """Tuned GEMM against the simple GEMM and integer sums on LCG data (zero/engine_setup.h:424-520); raises on a
    difference."""
    _check(lib.arcz_engine_self_check(), engine=True)


# ---------------------------------------------------------------- GGUF files (no GPU)
class GgufFile:
    """A memory-mapped GGUF file: metadata scalars and strings, the tensor directory, tensor bytes as numpy views."""

    def __init__(self, path):
        self.h = lib.arcz_gguf_open(str(path).encode())
        if not self.h:
            raise ArczError(-100, lib.arcz_gguf_error().decode())

    def close(self):
        if self.h:
            lib.arcz_gguf_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    @property
    def version(self):
        return lib.arcz_gguf_version(self.h)

    @property
    def n_kv(self):
        return lib.arcz_gguf_n_kv(self.h)

    @property
    def n_tensors(self):
        return lib.arcz_gguf_n_tensors(self.h)

    @property
    def alignment(self):
        return lib.arcz_gguf_alignment(self.h)

    def get_int(self, key, default=None):
        v = C.c_int64()
        return v.value if lib.arcz_gguf_kv_i64(self.h, key.encode(), C.byref(v)) else default

    def get_float(self, key, default=None):
        v = C.c_double()
        return v.value if lib.arcz_gguf_kv_f64(self.h, key.encode(), C.byref(v)) else default

    def get_str(self, key, default=None):
        s = lib.arcz_gguf_kv_str(self.h, key.encode())
        return s.decode() if s is not None else default

    def find(self, name):
        return lib.arcz_gguf_find(self.h, name.encode())

    def tensor(self, i):
        name, typ, nd, dims, data, nb = C.c_char_p(), _u32(), _u32(), (_u64 * 8)(), _p(), _u64()
        if lib.arcz_gguf_tensor(self.h, i, C.byref(name), C.byref(typ), C.byref(nd), C.byref(dims), C.byref(data),
                                C.byref(nb)) != 0:
            raise IndexError(i)
        buf = (C.c_uint8 * nb.value).from_address(data.value) if nb.value else None
        return {"name": name.value.decode(), "type": typ.value, "dims": [int(dims[k]) for k in range(nd.value)],
                "nbytes": nb.value, "data": np.frombuffer(buf, np.uint8) if buf is not None else np.zeros(0, np.uint8)}


# ---------------------------------------------------------------- host helpers (no GPU)
def gguf_bytes(qtype, rows, K):
    return lib.arcz_gguf_bytes(qtype, rows, K)


def relayout_q4_0(qtype, rows, K, src):
    """AR4_128 / Q2_0 rows as Q4_0 blocks of the same values (what make_weight does with them first)."""
    src = np.ascontiguousarray(src, dtype=np.uint8)
    if src.size != lib.arcz_relayout_q4_0(qtype, rows, K, None, None) or src.size == 0:
        raise ValueError("relayout_q4_0: type, K or byte count do not fit")
    out = np.empty(rows * (K // 32) * 18, np.uint8)
    lib.arcz_relayout_q4_0(qtype, rows, K, _np_ptr(src), _np_ptr(out))
    return out


def planes_bytes(qtype, rows, K):
    return lib.arcz_planes_bytes(qtype, rows, K)


def repack_planes(qtype, rows, K, gguf):
    gguf = np.ascontiguousarray(gguf, dtype=np.uint8)
    out = np.empty(planes_bytes(qtype, rows, K), dtype=np.uint8)
    if gguf.size != gguf_bytes(qtype, rows, K) or lib.arcz_repack_planes(qtype, rows, K, _np_ptr(gguf), _np_ptr(out)) != 0:
        raise ValueError("repack_planes: unsupported type or size")
    return out


def quantize_rows(qtype, w):
    """f32 rows [N][K] -> GGUF blocks (uint8).  Q8_0 as the reference's quantize_rows_q8_0; Q4_K / Q6_K: this
    library's own block makers (input generators)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    out = np.empty(gguf_bytes(qtype, N, K), dtype=np.uint8)
    if out.size == 0 or lib.arcz_quantize_rows(qtype, _np_ptr(w), N, K, _np_ptr(out)) != 0:
        raise ValueError("quantize_rows: unsupported type or K")
    return out


def gen_normal(seed, shape, mean=0.0, std=1.0):
    out = np.empty(shape, dtype=np.float32)
    lib.arcz_gen_normal(seed, out.size, mean, std, _np_ptr(out))
    return out


def gen_weights(qtype, seed, N, K, std=0.02):
    out = np.empty(gguf_bytes(qtype, N, K), dtype=np.uint8)
    if out.size == 0 or lib.arcz_gen_weights(qtype, seed, N, K, std, _np_ptr(out)) != 0:
        raise ValueError("gen_weights: unsupported type or K")
    return out


# ---------------------------------------------------------------- runtime (include/arcz_hip.h)
class Buffer:
    """A device buffer (the reference's cl_mem)."""

    def __init__(self, handle, owner=True):
        self.h = handle
        self.owner = owner

    @property
    def size(self):
        return lib.arcz_mem_size(self.h)

    def write(self, a, offset=0):
        a = np.ascontiguousarray(a)
        _check(lib.arcz_h2d(self.h, offset, _np_ptr(a), a.nbytes))
        return self

    def read(self, dtype, count=None, offset=0):
        dt = np.dtype(dtype)
        n = (self.size - offset) // dt.itemsize if count is None else int(count)
        out = np.empty(n, dtype=dt)
        _check(lib.arcz_d2h(_np_ptr(out), self.h, offset, out.nbytes))
        return out

    def fill(self, value, dtype=np.uint32, offset=0, nbytes=None):
        pat = np.array([value], dtype=dtype)
        _check(lib.arcz_fill(self.h, _np_ptr(pat), pat.nbytes, offset, self.size - offset if nbytes is None else nbytes))
        return self

    def view(self, offset, nbytes):
        h = lib.arcz_view(self.h, offset, nbytes)
        if not h:
            raise ArczError(-13, lib.arcz_last_error().decode())
        return Buffer(h, owner=False)

    def free(self):
        if self.h:
            _check(lib.arcz_free(self.h))
            self.h = None


class Runtime:
    """Process-wide runtime: one device, one stream."""

    @staticmethod
    def init(device=0):
        _check(lib.arcz_init(device))

    @staticmethod
    def shutdown():
        lib.arcz_shutdown()

    @staticmethod
    def device_name():
        return lib.arcz_device_name().decode()

    @staticmethod
    def cus():
        return lib.arcz_device_cus()

    @staticmethod
    def alloc(nbytes):
        h = lib.arcz_alloc(nbytes)
        if not h:
            raise ArczError(-4, lib.arcz_last_error().decode())
        return Buffer(h)

    @staticmethod
    def from_numpy(a):
        a = np.ascontiguousarray(a)
        return Runtime.alloc(max(a.nbytes, 1)).write(a)

    @staticmethod
    def sync():
        _check(lib.arcz_sync())

    @staticmethod
    def kernel(which, defs, name):
        h = lib.arcz_kernel_get(which.encode(), defs.encode(), name.encode())
        if not h:
            raise ArczError(-11, lib.arcz_last_error().decode())
        return h

    @staticmethod
    def launch(kernel, global_size, local_size, args, timed=False):
        """args: Buffer, None (null pointer), int (32-bit), float (32-bit), np.uint64 / ('z', n) size_t by value."""
        dim = len(global_size)
        g = (_z * dim)(*global_size)
        l = (_z * dim)(*local_size) if local_size is not None else None
        n = len(args)
        store, ptrs, sizes = [], (_p * n)(), (_z * n)()
        for i, a in enumerate(args):
            if isinstance(a, Buffer):
                v = C.c_void_p(a.h)
            elif a is None:
                v = C.c_void_p(0)
            elif isinstance(a, tuple) and a[0] == "z":
                v = C.c_size_t(a[1])
            elif isinstance(a, (float, np.floating)):
                v = C.c_float(a)
            else:
                v = C.c_int(int(a))
            store.append(v)
            ptrs[i] = C.cast(C.pointer(v), _p)
            sizes[i] = C.sizeof(v)
        ev = _p()
        _check(lib.arcz_launch(kernel, dim, g, l, ptrs, sizes, n, C.byref(ev) if timed else None))
        if timed:
            ms = lib.arcz_event_ms(ev)
            lib.arcz_event_release(ev)
            return ms
        return None

    @staticmethod
    def event():
        return lib.arcz_event_record()

    @staticmethod
    def elapsed_ms(a, b):
        return lib.arcz_event_elapsed_ms(a, b)

    @staticmethod
    def event_release(e):
        lib.arcz_event_release(e)

    @staticmethod
    def record(fn):
        """Records the kernel launches that fn() makes into a LaunchList (nothing runs meanwhile).  fn must have run
        once before, so that every buffer it needs exists: allocation, copies and waits are refused while recording.
        If fn raises, the recording is dropped and the exception goes on."""
        _check(lib.arcz_record_begin())
        try:
            fn()
        except BaseException:
            lib.arcz_record_end(None)
            raise
        h = C.c_void_p()
        _check(lib.arcz_record_end(C.byref(h)))
        return LaunchList(h)


class LaunchList:
    """A recorded sequence of kernel launches (arcz_record_begin / arcz_record_end), submitted as one."""

    def __init__(self, h):
        self.h = h
        self.launches = lib.arcz_list_launches(h)

    def run(self):
        _check(lib.arcz_list_run(self.h))

    def free(self):
        if self.h:
            _check(lib.arcz_list_free(self.h))
            self.h = None


# ---------------------------------------------------------------- engine (include/arcz_engine.h)
class Weight:
    def set_softcap(self, cap):
        """This matrix is an output head with final-logit soft-capping c: GEMVs over 1-8 tokens write c * tanh(v / c)."""
        _check(lib.arcz_weight_set_softcap(self.h, float(cap)), engine=True)

    def __init__(self, eng, h, qtype, N, K):
        self.eng, self.h, self.type, self.N, self.K = eng, h, qtype, N, K

    def free(self):
        if self.h:
            _check(lib.arcz_weight_free(self.eng.h, self.h), engine=True)
            self.h = None


class MoeLayer:
    def __init__(self, eng, h, NE, NU, E, F):
        self.eng, self.h, self.NE, self.NU, self.E, self.F = eng, h, NE, NU, E, F

    def free(self):
        if self.h:
            lib.arcz_moe_layer_free(self.eng.h, self.h)
            self.h = None


class Engine:
    """The matmul dispatch of the reference's Engine for one GPU (zero/engine.h:936-1251, zero/engine_moe.h)."""

    MOE_BUFFERS = ("ids", "wts", "offs", "tiles", "tstart", "stok", "swt", "inv", "h", "hq", "hsc", "y", "hbs")

    def __init__(self, max_chunk, max_k):
        self.h = lib.arcz_engine_create(max_chunk, max_k)
        if not self.h:
            raise ArczError(-100, lib.arcz_engine_error().decode())
        self.max_chunk, self.max_k = max_chunk, max_k

    def close(self):
        if self.h:
            lib.arcz_engine_destroy(self.h)
            self.h = None

    def make_weight(self, qtype, N, K, gguf):
        gguf = np.ascontiguousarray(gguf, dtype=np.uint8)
        h = lib.arcz_weight_upload(self.h, qtype, N, K, _np_ptr(gguf), gguf.nbytes)
        if not h:
            raise ArczError(-100, lib.arcz_engine_error().decode())
        return Weight(self, h, qtype, N, lib.arcz_weight_k(h))     # (K rounded up when the rows were padded)

    def make_weight_gguf(self, gguf, name):
        """A matrix of an open GgufFile, by name, as it lies in the file."""
        h = lib.arcz_weight_upload_gguf(self.h, gguf.h, name.encode())
        if not h:
            raise ArczError(-100, lib.arcz_engine_error().decode())
        t = gguf.tensor(gguf.find(name))
        return Weight(self, h, t["type"], t["dims"][1], lib.arcz_weight_k(h))

    def make_moe_layer_gguf(self, gguf, gate, up, down, NU):
        h = lib.arcz_moe_layer_upload_gguf(self.h, gguf.h, gate.encode(), up.encode(), down.encode(), NU)
        if not h:
            raise ArczError(-100, lib.arcz_engine_error().decode())
        t = gguf.tensor(gguf.find(gate))
        Ep, Fp = C.c_int(), C.c_int()
        lib.arcz_moe_layer_dims(h, C.byref(Ep), C.byref(Fp))
        return MoeLayer(self, h, t["dims"][2], NU, Ep.value, Fp.value)

    def quantize(self, x, ldx, K, Mp, T, act32=1):
        _check(lib.arcz_engine_quantize(self.h, x.h, ldx, K, Mp, T, act32), engine=True)

    def add_norm_quant(self, x, t, w, K, T, Mp, s, w2, norm2, eps, act32=1):
        _check(lib.arcz_engine_add_norm_quant(self.h, x.h, t.h, w.h, K, T, Mp, s, w2.h if w2 else None, 1 if norm2 else 0,
                                              act32, eps), "add_norm_quant")

    def rmsnorm_quant(self, x, row_off, w, K, Mp, T, eps, hout=None, act32=1):
        _check(lib.arcz_engine_rmsnorm_quant(self.h, x.h, row_off, w.h, K, Mp, T, act32, eps, hout.h if hout else None),
               engine=True)

    def swiglu_quant(self, gu, F, Mp, T, fused=0, gelu=0, act32=1):
        _check(lib.arcz_engine_swiglu_quant(self.h, gu.h, F, Mp, T, act32, fused, gelu), engine=True)

    def set_activations(self, aq, asc, absum, K, Mp, T):
        aq = np.ascontiguousarray(aq, dtype=np.int8)
        asc = np.ascontiguousarray(asc, dtype=np.float32)
        absum = np.ascontiguousarray(absum, dtype=np.int16)
        assert aq.size == Mp * K and asc.size == Mp * K // 32 and absum.size == Mp * K // 16
        _check(lib.arcz_engine_set_activations(self.h, _np_ptr(aq), _np_ptr(asc), _np_ptr(absum), K, Mp, T), engine=True)

    @property
    def aq(self):
        return Buffer(lib.arcz_engine_aq(self.h), owner=False)

    @property
    def asc(self):
        return Buffer(lib.arcz_engine_asc(self.h), owner=False)

    @property
    def absum(self):
        return Buffer(lib.arcz_engine_absum(self.h), owner=False)

    def two_pass(self, on=True, fuse=True):
        """Two-pass matmul inputs (the reference's q2mm_ mode): producers also quantize the residual, matmuls add its pass
        (fuse: the GEMV of 1-4 tokens takes both in one launch)."""
        _check(lib.arcz_engine_two_pass(self.h, (1 if fuse else 2) if on else 0), engine=True)

    def read_residual(self, K, Mp):
        b = [Buffer(lib.arcz_engine_residual(self.h, i), owner=False) for i in range(3)]
        return (b[0].read(np.int8, Mp * K).reshape(Mp, K), b[1].read(np.float32, Mp * K // 32).reshape(K // 32, Mp),
                b[2].read(np.int16, Mp * K // 16).reshape(K // 16, Mp))

    def read_activations(self, K, Mp):
        return (self.aq.read(np.int8, Mp * K).reshape(Mp, K), self.asc.read(np.float32, Mp * K // 32).reshape(K // 32, Mp),
                self.absum.read(np.int16, Mp * K // 16).reshape(K // 16, Mp))

    def matmul(self, name, w, Mp, Cbuf, ldc, c_off=0, acc=0, act32=True):
        _check(lib.arcz_engine_matmul(self.h, name.encode(), w.h, Mp, Cbuf.h, ldc, c_off, acc, 1 if act32 else 0), engine=True)

    def gemv_gu(self, g, u, Mp, Cbuf):
        """Gate and up of one token in one launch: True if taken, False if the caller must run the two matmuls."""
        r = lib.arcz_engine_gemv_gu(self.h, g.h, u.h, Mp, Cbuf.h)
        if r < 0:
            _check(r, engine=True)
        return r == 1

    def matmul_noalloc(self, name, w, Mp, Cbuf, ldc, c_off=0, acc=0, act32=True):
        """The same matmul on the library's static device scratch: no device allocation, event or free in the call."""
        _check(lib.arcz_engine_matmul_noalloc(self.h, name.encode(), w.h, Mp, Cbuf.h, ldc, c_off, acc, 1 if act32 else 0),
               engine=True)

    def make_moe_layer(self, qtype, gate, up, down, NE, NU, E, F):
        g, u, d = (np.ascontiguousarray(a, dtype=np.uint8) for a in (gate, up, down))
        # (the library checks the byte counts against the type and the shape, padded shapes included)
        h = lib.arcz_moe_layer_upload(self.h, qtype, _np_ptr(g), g.size, _np_ptr(u), u.size, _np_ptr(d), d.size, NE, NU, E, F)
        if not h:
            raise ArczError(-100, lib.arcz_engine_error().decode())
        Ep, Fp = C.c_int(), C.c_int()
        lib.arcz_moe_layer_dims(h, C.byref(Ep), C.byref(Fp))       # (E and F rounded up where the tensors were padded)
        return MoeLayer(self, h, NE, NU, Ep.value, Fp.value)

    def layer_moe(self, L, logits, ldl, x, T, Mp, sh=None):
        if sh is None:
            _check(lib.arcz_engine_layer_moe(self.h, L.h, logits.h, ldl, x.h, T, Mp), engine=True)
        else:
            _check(lib.arcz_engine_layer_moe_sh(self.h, L.h, logits.h, ldl, x.h, T, Mp, sh.h), engine=True)

    def set_moe_routing(self, L, escale=None, ebias=None, rscale=1.0):
        es = None if escale is None else np.ascontiguousarray(escale, dtype=np.float32)
        eb = None if ebias is None else np.ascontiguousarray(ebias, dtype=np.float32)
        _check(lib.arcz_moe_layer_set_routing(self.h, L.h, _np_ptr(es) if es is not None else None,
                                              _np_ptr(eb) if eb is not None else None, float(rscale)), engine=True)

    @property
    def moe_sgate(self):
        return Buffer(lib.arcz_engine_moe_sgate(self.h), owner=False)

    def moe_route(self, L, logits, ldl, T, tm):
        _check(lib.arcz_engine_moe_route(self.h, L.h, logits.h, ldl, T, tm), engine=True)

    def moe_buffer(self, name):
        return Buffer(lib.arcz_engine_moe_buffer(self.h, self.MOE_BUFFERS.index(name)), owner=False)

    @property
    def moe_slots(self):
        return lib.arcz_engine_moe_slots(self.h)

    def profile(self, on=True):
        lib.arcz_engine_profile(self.h, 1 if on else 0)

    def profile_collect(self):
        _check(lib.arcz_engine_profile_collect(self.h), engine=True)

    def profile_get(self, name):
        ms, n = C.c_double(), C.c_int()
        if lib.arcz_engine_profile_get(self.h, name.encode(), C.byref(ms), C.byref(n)) != 0:
            return 0.0, 0
        return ms.value, n.value

    def profile_stats(self, name):
        """(minimum, median) of the per-launch times of `name`, ms."""
        lo, med = C.c_double(), C.c_double()
        if lib.arcz_engine_profile_stats(self.h, name.encode(), C.byref(lo), C.byref(med)) != 0:
            return 0.0, 0.0
        return lo.value, med.value

    def profile_reset(self):
        lib.arcz_engine_profile_reset(self.h)
