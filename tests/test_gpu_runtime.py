"""The drop-in boundary on the GPU: buffers, views, bounds-checked transfers, kernel lookup by the reference's
(which, defs, name) key, launch checks -- the behaviours of the reference's zero/clrt.h that the engine relies on."""
import numpy as np
import pytest

import arcinferzero_amd as az

pytestmark = pytest.mark.gpu


def test_buffers_views_transfers(rt):
    b = rt.alloc(4096)
    assert b.size == 4096
    data = np.arange(1024, dtype=np.uint32)
    b.write(data)
    assert np.array_equal(b.read(np.uint32), data)
    v = b.view(1024, 512)
    assert np.array_equal(v.read(np.uint32), data[256:384])
    v.fill(7)
    assert (b.read(np.uint32)[256:384] == 7).all() and b.read(np.uint32)[255] == 255 and b.read(np.uint32)[384] == 384
    b.fill(0x55, dtype=np.uint8, offset=1, nbytes=6)       # the unaligned byte path
    assert b.read(np.uint8, 8).tolist() == [0, 0x55, 0x55, 0x55, 0x55, 0x55, 0x55, 0]
    with pytest.raises(az.ArczError) as e:                 # a write past the end is refused, nothing is touched
        b.write(np.zeros(2048, np.uint32))
    assert e.value.code == -30
    with pytest.raises(az.ArczError):
        b.read(np.uint32, 10, offset=4090)
    with pytest.raises(az.ArczError) as e:
        b.view(4000, 200)
    assert e.value.code == -13
    with pytest.raises(az.ArczError) as e:                 # a parent with a live view is not freed
        b.free()
    assert e.value.code == -50 and np.array_equal(v.read(np.uint32, 4), np.full(4, 7, np.uint32))
    small = rt.alloc(1)                                    # at least 64 bytes are there
    small.write(np.zeros(1, np.uint8))
    for x in (v, small, b):
        x.free()


def test_kernel_lookup_and_launch_checks(rt):
    k = rt.kernel("decode", "-cl-intel-256-GRF-per-thread -DQT=12 -DGROWS=2", "gemv_v")   # non -D options are ignored
    assert az.lib.arcz_kernel_symbol(k) == b"gemv_v__QT12_GROWS2"
    assert rt.kernel("decode", "-cl-intel-256-GRF-per-thread -DQT=12 -DGROWS=2", "gemv_v") == k   # cached by key
    for bad in (("decode", "-DQT=12", "gemv_v"), ("decode", "-DQT=99 -DGROWS=1", "gemv_v"), ("nope", "", "gemv_v"),
                ("moe", "-DNU=8", "moe_route")):
        with pytest.raises(az.ArczError) as e:
            rt.kernel(*bad)
        assert e.value.code == -11
    f = rt.kernel("ops", "", "fill32")
    buf = rt.alloc(4096)
    rt.launch(f, (1024,), (256,), [buf, 0x01020304, ("z", 1024)])
    assert (buf.read(np.uint32) == 0x01020304).all()
    rt.launch(f, (0,), (256,), [buf, 9, ("z", 1024)])                  # a zero global size: success, no launch
    assert (buf.read(np.uint32) == 0x01020304).all()
    with pytest.raises(az.ArczError) as e:
        rt.launch(f, (1000,), (256,), [buf, 9, ("z", 1000)])           # not a multiple of the work-group
    assert e.value.code == -54
    with pytest.raises(az.ArczError) as e:
        rt.launch(f, (1 << 33,), (256,), [buf, 9, ("z", 4)])
    assert e.value.code == -63
    with pytest.raises(az.ArczError) as e:
        rt.launch(f, (256,), (256,), [buf, 9])                         # wrong argument count
    assert e.value.code == -49
    with pytest.raises(az.ArczError) as e:
        rt.launch(f, (256,), (256,), [buf, ("z", 9), ("z", 4)])        # wrong argument size
    assert e.value.code == -51
    ms = rt.launch(f, (1024,), (256,), [buf, 5, ("z", 1024)], timed=True)
    assert ms >= 0 and (buf.read(np.uint32) == 5).all()
    buf.free()


def test_engine_refuses_bad_shapes(rt):
    eng = az.Engine(64, 1024)
    try:
        W = az.gen_weights(az.Q4_K, 1, 64, 512)
        w = eng.make_weight(az.Q4_K, 64, 512, W)
        with pytest.raises(az.ArczError):
            eng.make_weight(az.Q4_K, 64, 512, W[:-1])
        with pytest.raises(az.ArczError):
            eng.make_weight(5, 64, 512, W)
        x = rt.from_numpy(az.gen_normal(1, (4, 512)))
        c = rt.alloc(4 * 64 * 4)
        with pytest.raises(az.ArczError):
            eng.matmul("m", w, 16, c, 64)                               # no activations yet
        with pytest.raises(az.ArczError):
            eng.quantize(x, 512, 2048, 16, 4)                           # K beyond the engine's buffers
        eng.quantize(x, 512, 512, 16, 4)
        with pytest.raises(az.ArczError):
            eng.matmul("m", w, 32, c, 64)                               # another chunk's Mp
        with pytest.raises(az.ArczError):
            eng.matmul("m", w, 16, c, 64, c_off=8)                      # the output does not fit C
        with pytest.raises(az.ArczError):
            eng.matmul("m", w, 16, c, 64, acc=2)                        # fused epilogue on the GEMV form
        eng.matmul("m", w, 16, c, 64)
        assert np.isfinite(c.read(np.float32)).all()
        for b in (x, c):
            b.free()
    finally:
        eng.close()


def test_fake_oom_and_hook(rt):
    az.lib.arcz_set_fake_oom(2)
    try:
        a = rt.alloc(1024)
        with pytest.raises(az.ArczError) as e:                          # every second allocation "fails", no hook
            rt.alloc(1024)
        assert e.value.code == -4
        a.free()
    finally:
        az.lib.arcz_set_fake_oom(0)


def test_reference_style_snippet_against_the_shim(rt):
    """tests/clrt_snippet.cpp -- clCreateBuffer, cl.build, cl.kernel, set_args, clEnqueueNDRangeKernel, CL_CHECK,
    clEnqueueMapBuffer / clEnqueueUnmapMemObject written as the reference's engine code writes them (zero/clrt.h:711-743,
    1189-1307) -- compiled against clrt_hip.h by the library's Makefile, run here as a process of its own."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "clrt_snippet")
    assert os.path.exists(exe), "tests/clrt_snippet is not built (make -C arcinferzero_amd/csrc)"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0 and "clrt_snippet ok" in r.stdout
