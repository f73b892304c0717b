"""Recorded launch lists (arcz_record_begin / arcz_record_end / arcz_list_run; the reference's ARC_BATCH lists,
zero/clrt.h:170-265): a decode step's kernels recorded once and submitted as one list.

A list is replayed several times, each time on new input written into the same buffers, with the program's own eager
launches and waits between the replays, and every replay is held bit for bit to the eager run of the same sequence on
the same input.  What a list cannot hold (allocation, copies, waits, timed launches) is refused while recording and
leaves the runtime usable.
"""
import numpy as np
import pytest

import arcinferzero_amd as az
from common import make_acts, make_weights

pytestmark = pytest.mark.gpu
E_RECORDING = -59


def chain(eng, T, Mp, dims, types, seed):
    """x [T][dims[0]] -> quantize -> W1 -> quantize -> W2 -> ...: the buffers, the weights and the step function."""
    ws = [eng.make_weight(t, dims[i + 1], dims[i], make_weights(t, dims[i + 1], dims[i], seed=seed + i))
          for i, t in enumerate(types)]
    rows = Mp if T > 8 else T
    bufs = [az.Runtime.alloc(T * dims[0] * 4)] + [az.Runtime.alloc(rows * d * 4).fill(0) for d in dims[1:]]

    def step():
        for i, w in enumerate(ws):
            eng.quantize(bufs[i], dims[i], dims[i], Mp, T)
            eng.matmul("chain", w, Mp, bufs[i + 1], dims[i + 1], 0, 0)

    return ws, bufs, step


@pytest.mark.parametrize("T,Mp", [(1, 16), (2, 16), (6, 16), (40, 48)])
def test_replays_equal_the_eager_sequence(rt, T, Mp):
    dims = [1024, 2048, 768, 512]
    types = [az.Q4_K, az.Q8_0, az.Q6_K]
    print(f"launch list chain T={T}", flush=True)
    eng = az.Engine(Mp, 2048)
    lst = None
    try:
        ws, bufs, step = chain(eng, T, Mp, dims, types, seed=700)
        rows = Mp if T > 8 else T

        def eager(x):
            bufs[0].write(x)
            step()
            return bufs[-1].read(np.float32, rows * dims[-1]).copy()

        x0 = make_acts(T, dims[0], seed=701) * np.float32(0.05)
        y0 = eager(x0)                                              # (also sizes every workspace the sequence needs)
        assert np.isfinite(y0).all() and np.abs(y0).max() > 0
        before = az.lib.arcz_launch_count()
        lst = az.Runtime.record(step)
        assert az.lib.arcz_launch_count() == before and not az.lib.arcz_recording()   # nothing ran
        assert lst.launches >= 2 * len(types)
        for i in range(5):
            x = make_acts(T, dims[0], seed=710 + i) * np.float32(0.05)
            bufs[0].write(x)
            bufs[-1].fill(0xFFFFFFFF)
            n0 = az.lib.arcz_launch_count()
            lst.run()
            assert az.lib.arcz_launch_count() - n0 == lst.launches
            y = bufs[-1].read(np.float32, rows * dims[-1]).copy()
            want = eager(x)                                         # eager launches and waits between the replays
            assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), f"replay {i}"
            assert not np.array_equal(y, y0)
        # two runs back to back without a wait between them: stream order holds
        bufs[0].write(x0)
        lst.run()
        lst.run()
        assert np.array_equal(bufs[-1].read(np.float32, rows * dims[-1]).view(np.uint32), y0.view(np.uint32))
    finally:
        if lst:
            lst.free()
        eng.close()


def test_an_expert_layer_step_as_a_list(rt):
    """One token through a MoE layer (routing, gate / up, down, combine: all on the device) recorded and replayed."""
    NE, NU, E, F, T, Mp = 16, 4, 512, 256, 1, 16
    eng = az.Engine(Mp, E)
    lst = None
    try:
        L = eng.make_moe_layer(az.Q4_K, make_weights(az.Q4_K, NE * F, E, seed=720), make_weights(az.Q4_K, NE * F, E, seed=721),
                               make_weights(az.Q4_K, NE * E, F, seed=722), NE, NU, E, F)
        xb, lb, ob = az.Runtime.alloc(T * E * 4), az.Runtime.alloc(T * NE * 4), az.Runtime.alloc(T * E * 4)

        def step():
            eng.quantize(xb, E, E, Mp, T)
            eng.layer_moe(L, lb, NE, ob, T, Mp)

        def load(i):
            xb.write(make_acts(T, E, seed=730 + i))
            lb.write(az.gen_normal(740 + i, (T, NE)))
            ob.fill(0)

        load(0)
        step()
        lst = az.Runtime.record(step)
        for i in range(1, 5):
            load(i)
            lst.run()
            y = ob.read(np.float32, T * E).copy()
            load(i)
            step()
            want = ob.read(np.float32, T * E)
            assert np.abs(want).max() > 0 and np.array_equal(y.view(np.uint32), want.view(np.uint32)), f"replay {i}"
        lst.free()   # (a list before the buffers it names)
        lst = None
        L.free()
        for b in (xb, lb, ob):
            b.free()
    finally:
        if lst:
            lst.free()
        eng.close()


def test_what_a_list_cannot_hold_is_refused(rt):
    eng = az.Engine(32, 5120)
    try:
        b = az.Runtime.alloc(4096).fill(0)
        for bad in (lambda: az.Runtime.alloc(64), lambda: az.Runtime.sync(), lambda: b.read(np.uint8, 16),
                    lambda: b.write(np.zeros(16, np.uint8)), lambda: b.free(), lambda: az.Runtime.record(lambda: None)):
            with pytest.raises(az.ArczError) as ei:
                az.Runtime.record(bad)
            # (the code of the call that was refused, ARCZ_E_RECORDING, or -- a call that returns a handle -- the
            #  wrapper's own for a null handle)
            assert "being recorded" in str(ei.value) and not az.lib.arcz_recording()
        assert az.Runtime.event() is not None                       # (events work again once the recording is dropped)
        with pytest.raises(az.ArczError):                           # nothing recorded
            az.Runtime.record(lambda: None)
        assert az.lib.arcz_record_end(None) == E_RECORDING          # no recording open
        assert az.lib.arcz_list_run(None) != 0 and az.lib.arcz_list_free(None) == 0
        # a sequence that has not run before asks for its workspace while it is recorded: refused, loudly, and the
        # same sequence records after one eager run
        T, Mp, N, K = 20, 32, 200, 5120
        w = eng.make_weight(az.Q4_K, N, K, make_weights(az.Q4_K, N, K, seed=750))
        xb = az.Runtime.from_numpy(make_acts(T, K, seed=751))
        cb = az.Runtime.alloc(Mp * N * 4).fill(0)

        def step():
            eng.quantize(xb, K, K, Mp, T)
            eng.matmul("splitk", w, Mp, cb, N, 0, 0)

        try:
            lst = az.Runtime.record(step)
        except az.ArczError as e:
            assert not az.lib.arcz_recording() and "record" in str(e).lower()
            lst = None
        step()
        want = cb.read(np.float32, Mp * N).copy()
        if lst is None:
            lst = az.Runtime.record(step)
        cb.fill(0)
        lst.run()
        assert np.array_equal(cb.read(np.float32, Mp * N).view(np.uint32), want.view(np.uint32))
        lst.free()
        assert az.lib.arcz_list_run(lst.h) != 0                     # (a freed handle: h is None)
        for m in (xb, cb, b):
            m.free()
        w.free()
    finally:
        eng.close()


def test_a_list_keeps_the_buffers_it_names(rt):
    """A list holds the device addresses of the buffers its kernels were given -- the caller's and the engine's own
    workspaces (a chunk of 256 token rows over a Q4_K matrix reads the ready-made scale vectors).  While the list lives
    none of them is freed or replaced: the call that would have to is refused and leaves everything as it was, the list
    still replays on valid memory, and once the list is freed the same calls go through."""
    T = Mp = 256
    N, K = 512, 1024
    eng = az.Engine(Mp, 2048)
    lst = None
    try:
        w = eng.make_weight(az.Q4_K, N, K, make_weights(az.Q4_K, N, K, seed=41))
        xb = az.Runtime.from_numpy(make_acts(T, K, seed=42))
        cb = az.Runtime.alloc(Mp * N * 4).fill(0)

        def step():
            eng.quantize(xb, K, K, Mp, T)
            eng.matmul("listed", w, Mp, cb, N, 0, 0)

        step()
        ref = cb.read(np.float32, Mp * N).copy()
        lst = az.Runtime.record(step)
        assert az.lib.arcz_mem_listed(cb.h) == 1 and az.lib.arcz_mem_listed(xb.h) == 1
        with pytest.raises(az.ArczError):        # the caller's output buffer
            cb.free()
        with pytest.raises(az.ArczError):        # a larger Q4_K matrix would replace the workspace of scale vectors
            eng.make_weight(az.Q4_K, 4 * N, 2 * K, make_weights(az.Q4_K, 4 * N, 2 * K, seed=43))
        with pytest.raises(az.ArczError):        # the activation buffers are made anew when the mode changes
            eng.two_pass(True)
        cb.fill(0xFFFFFFFF)
        lst.run()
        assert np.array_equal(cb.read(np.float32, Mp * N).view(np.uint32), ref.view(np.uint32))
        lst.free()
        lst = None
        assert az.lib.arcz_mem_listed(cb.h) == 0
        w2 = eng.make_weight(az.Q4_K, 4 * N, 2 * K, make_weights(az.Q4_K, 4 * N, 2 * K, seed=43))
        w2.free()
        for b in (xb, cb):
            b.free()
        w.free()
    finally:
        if lst is not None:
            lst.free()
        eng.close()
