"""The storage functions of the C ABI (what replaces cuda_malloc_zeroed and the pinned-copy helpers,
crates/core/src/cuda/mod.rs:47-66, cuda/utils_pinned.cu:4-20) and eri_adam8_table_update, on the device."""
import ctypes as C

import numpy as np
import pytest

import harness as hs

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-3, 0.9, 0.999, 1e-8, 0.01


def _L():
    from eridiffusion_amd import _lib
    return _lib


def test_allocation_copies_fill_and_streams():
    L = _L()
    lib = L.lib()
    count, dev = C.c_int(), C.c_int(-1)
    L.check(lib.eri_hip_device_count(C.byref(count)), "device_count")
    L.check(lib.eri_hip_get_device(C.byref(dev)), "get_device")
    assert count.value >= 1 and 0 <= dev.value < count.value
    L.check(lib.eri_hip_set_device(dev.value), "set_device")
    assert lib.eri_hip_set_device(count.value + 3) > 0  # a HIP error code comes back as it is
    free0, total = C.c_size_t(), C.c_size_t()
    L.check(lib.eri_hip_mem_info(C.byref(free0), C.byref(total)), "mem_info")
    assert 0 < free0.value <= total.value and total.value > 100 << 30

    n = (96 << 20) + 40  # large enough for the allocate / release / allocate path, and not a round size
    buf = C.c_void_p()
    L.check(lib.eri_hip_malloc_zeroed(dev.value, n, C.byref(buf)), "malloc_zeroed")
    assert buf.value % 256 == 0
    assert lib.eri_hip_malloc_zeroed(dev.value, 0, C.byref(C.c_void_p())) == -6
    free1 = C.c_size_t()
    L.check(lib.eri_hip_mem_info(C.byref(free1), None), "mem_info")
    assert free0.value - free1.value >= n

    stream = C.c_void_p()
    L.check(lib.eri_hip_stream_create(C.byref(stream)), "stream_create")
    lib.eri_hip_host_alloc.restype = C.c_void_p
    pinned = lib.eri_hip_host_alloc(1 << 20)
    assert pinned
    host = (C.c_ubyte * (1 << 20)).from_address(pinned)
    view = np.frombuffer(host, np.uint8)
    # the fresh allocation reads zero at both ends (device -> pinned host, kind 2)
    for off in (0, n - (1 << 20)):
        view[:] = 0xAB
        L.check(lib.eri_hip_memcpy_async(pinned, buf.value + off, 1 << 20, 2, stream), "d2h")
        L.check(lib.eri_hip_stream_sync(stream), "sync")
        assert not view.any()
    # host -> device (1), device -> device (3), fill, and back
    pattern = (np.arange(1 << 20, dtype=np.uint32) * 2654435761 >> 13).astype(np.uint8)
    view[:] = pattern
    L.check(lib.eri_hip_memcpy_async(buf.value + 4096, pinned, 1 << 20, 1, stream), "h2d")
    L.check(lib.eri_hip_memcpy_async(buf.value + (8 << 20), buf.value + 4096, 1 << 20, 3, stream), "d2d")
    L.check(lib.eri_hip_memset_async(buf.value + (8 << 20) + 100, 0x5A, 1000, stream), "memset")
    view[:] = 0
    L.check(lib.eri_hip_memcpy_async(pinned, buf.value + (8 << 20), 1 << 20, 2, stream), "d2h")
    L.check(lib.eri_hip_stream_sync(stream), "sync")
    want = pattern.copy()
    want[100:1100] = 0x5A
    assert np.array_equal(view, want)
    assert lib.eri_hip_memcpy_async(None, pinned, 16, 1, stream) == -1
    assert lib.eri_hip_memcpy_async(None, None, 0, 1, stream) == 0  # nothing to copy is not an error
    del view, host
    L.check(lib.eri_hip_host_free(pinned), "host_free")
    L.check(lib.eri_hip_stream_destroy(stream), "stream_destroy")
    L.check(lib.eri_hip_free(buf), "free")
    L.check(lib.eri_hip_free(None), "free(NULL)")


def test_table_update_points_the_same_table_at_new_buffers():
    import torch
    L = _L()
    sizes = [2048 * 4 + 33, 500, 2048]
    ps, gs = hs.make_inputs(sizes, True, 901)
    states = hs.oracle_states(sizes)
    gt = hs.GpuTensors(ps, gs, states, True)
    stream = torch.cuda.current_stream().cuda_stream
    rows = gt.rows()
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), stream, C.byref(table)), "table_create")
    h = L.hyper_pack(LR, B1, B2, EPS, WD, 1, L.MODE_ERI, L.FLAG_EXACT_PARAM)
    L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step")
    hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, 1), True)
    # second step: gradients live in other buffers, the last tensor carries a multiplier
    gs2 = hs.fresh_grads(sizes, True, 902)
    other = hs.GpuTensors(ps, gs2, states, True)  # only its gradient buffers are used
    for i in range(len(sizes)):
        rows[i].g = other.ptr(other.g[i])
    rows[2].grad_scale = 0.5
    L.check(L.lib().eri_adam8_table_update(table, rows, len(rows), stream), "table_update")
    h = L.hyper_pack(LR, B1, B2, EPS, WD, 2, L.MODE_ERI, L.FLAG_EXACT_PARAM | L.FLAG_GRAD_SCALE)
    L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step")
    torch.cuda.synchronize()
    for i, s in enumerate((1.0, 1.0, 0.5)):
        hs.oracle_step([ps[i]], [gs2[i]], [states[i]], (LR, B1, B2, EPS, WD, 2), True, grad_scale=s)
    got_p, got_st = gt.fetch()
    stats = hs.compare(got_p, got_st, ps, states, True, True, "table_update")
    assert stats["code_mismatch"] == 0
    # a different shape is refused and leaves the table usable
    rows[1].numel = 501
    assert L.lib().eri_adam8_table_update(table, rows, len(rows), stream) != 0
    assert L.lib().eri_adam8_table_update(table, rows, len(rows) - 1, stream) != 0
    rows[1].numel = 500
    L.check(L.lib().eri_adam8_table_update(table, rows, len(rows), stream), "table_update")
    L.lib().eri_adam8_table_destroy(table)


def test_checkpoint_conversions_refuse_memory_a_kernel_cannot_reach():
    """eri_hip_pointer_kind tells ordinary host memory from pinned host and device memory, and the calls that
    convert optimizer state to and from fp32 refuse the first kind before any kernel is launched (the refusals
    are only attempted after the runtime has shown that it tells the kinds apart)."""
    import torch
    L = _L()
    lib = L.lib()
    n = 2048 * 3 + 17
    nb = (n + 2047) // 2048
    dev_x = torch.randn(n, device="cuda:0")
    dev_codes = torch.empty(n, dtype=torch.uint8, device="cuda:0")
    dev_absmax = torch.empty(nb, dtype=torch.float32, device="cuda:0")
    dev_out = torch.empty(n, device="cuda:0")
    host = np.zeros(n, np.float32)
    lib.eri_hip_host_alloc.restype = C.c_void_p
    pinned = lib.eri_hip_host_alloc(4 * n)
    assert pinned

    def kind(p):
        k = C.c_int(-1)
        L.check(lib.eri_hip_pointer_kind(C.c_void_p(p), C.byref(k)), "pointer_kind")
        return k.value

    assert kind(host.ctypes.data) == 0
    assert kind(pinned) == 1
    assert kind(dev_x.data_ptr()) == 2 and kind(dev_x.data_ptr() + 4 * 1000) == 2
    assert kind(None) == 0

    stream = torch.cuda.current_stream().cuda_stream
    x, codes, absmax, out = dev_x.data_ptr(), dev_codes.data_ptr(), dev_absmax.data_ptr(), dev_out.data_ptr()
    L.check(lib.eri_adam8_quantize(x, 1, n, codes, absmax, stream), "quantize")
    assert lib.eri_adam8_quantize(host.ctypes.data, 1, n, codes, absmax, stream) == -6
    assert b"not device, pinned or managed memory" in lib.eri_last_error()
    assert lib.eri_adam8_dequantize(codes, absmax, 1, n, host.ctypes.data, stream) == -6
    # pinned host memory is reachable: the dequantised values land in it and equal the device copy
    L.check(lib.eri_adam8_dequantize(codes, absmax, 1, n, out, stream), "dequantize")
    L.check(lib.eri_adam8_dequantize(codes, absmax, 1, n, pinned, stream), "dequantize to pinned")
    torch.cuda.synchronize()
    got = np.frombuffer((C.c_float * n).from_address(pinned), np.float32)
    assert np.array_equal(got.view(np.uint32), dev_out.cpu().numpy().view(np.uint32))
    lib.eri_hip_host_free(C.c_void_p(pinned))
