"""Two host threads, two optimizers, two streams: the ABI is re-entrant on distinct handles
(the reference requires `Send + Sync` of an optimizer, crates/training/src/optimizer.rs:11)."""
import ctypes as C
import threading

import numpy as np
import pytest

import harness as hs

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01


def _worker(idx, bf16, steps, out, barrier):
    import torch
    from eridiffusion_amd import _lib as L
    try:
        torch.cuda.set_device(0)
        sizes = [2048 * (9 + idx) + 13 * (idx + 1), 640 * 16, 2048, 77 + idx]
        ps, gs = hs.make_inputs(sizes, bf16, 400 + idx)
        states = hs.oracle_states(sizes)
        gt = hs.GpuTensors(ps, gs, states, bf16)
        stream = C.c_void_p()
        L.check(L.lib().eri_hip_stream_create(C.byref(stream)), "stream_create")
        torch.cuda.synchronize()  # the uploads above ran on torch's stream
        rows = gt.rows()
        table = C.c_void_p()
        # the table is uploaded on the NULL stream and stepped on the thread's own stream
        L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
        barrier.wait()
        all_g = [gs] + [hs.fresh_grads(sizes, bf16, 9000 + 100 * idx + k) for k in range(1, steps)]
        for k in range(steps):
            if k:
                L.check(L.lib().eri_hip_stream_sync(stream), "sync")
                gt.set_grads(all_g[k])
                torch.cuda.synchronize()
            h = L.hyper_pack(LR, B1, B2, EPS, WD, k + 1, L.MODE_ERI, L.FLAG_EXACT_PARAM)
            L.check(L.lib().eri_adam8_grad_norm(table, 1e9, 0.0, stream), "grad_norm")
            L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")
            # a bad call on this thread leaves its message on this thread only
            assert L.lib().eri_adam8_step_table(None, C.byref(h), stream) == -1
            assert b"NULL" in L.lib().eri_last_error()
        L.check(L.lib().eri_hip_stream_sync(stream), "sync")
        for k in range(steps):
            hs.oracle_step(ps, all_g[k], states, (LR, B1, B2, EPS, WD, k + 1), bf16, threads=2)
        got_p, got_st = gt.fetch()
        stats = hs.compare(got_p, got_st, ps, states, bf16, True, "thread %d" % idx)
        assert stats["code_mismatch"] == 0
        L.lib().eri_adam8_table_destroy(table)
        L.lib().eri_hip_stream_destroy(stream)
        out[idx] = "ok"
    except BaseException as e:  # reported by the main thread
        out[idx] = repr(e)
        try:
            barrier.abort()
        except Exception:
            pass


@pytest.mark.parametrize("bf16", [True, False])
def test_two_threads_two_streams_each_bit_exact(bf16):
    out = {}
    barrier = threading.Barrier(2)
    threads = [threading.Thread(target=_worker, args=(i, bf16, 4, out, barrier)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert out == {0: "ok", 1: "ok"}, out
