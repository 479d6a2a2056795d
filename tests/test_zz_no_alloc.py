"""The allocation-free gradient-norm entry point, eri_adam8_grad_norm_static, against eri_adam8_grad_norm.

Same kernels, same launch geometry, same reduction order: norm, clip factor and the count of non-finite
elements must be bit-identical, and so must a following step that takes the clip factor from the table.
Two calls in a row, the second on a smaller table: the static scratch keeps the first call's partial sums,
and none of them may leak into the second result.
"""
import ctypes as C

import numpy as np
import pytest

import harness as hs

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01


def _norm_both_ways(L, torch, sizes, bf16, seed, result, poison_grad=None):
    """Returns ((norm, scale, count) of the allocating call, the same of the static call, parameters and
    states after a clipped step of each)."""
    stream = torch.cuda.current_stream().cuda_stream
    ps, gs = hs.make_inputs(sizes, bf16, seed, g_std=1e-2)
    if poison_grad is not None:
        t, i, bits = poison_grad
        gs[t][i] = bits
    outs = []
    for static in (False, True):
        gt = hs.GpuTensors([p.copy() for p in ps], [g.copy() for g in gs], hs.oracle_states(sizes), bf16)
        rows = gt.rows()
        table = C.c_void_p()
        L.check(L.lib().eri_adam8_table_create(rows, len(rows), stream, C.byref(table)), "table_create")
        if static:
            result.fill_(-1)  # stale bytes must be overwritten
            L.check(L.lib().eri_adam8_grad_norm_static(table, 0.05, 1e-6, result.data_ptr(), stream), "grad_norm_static")
        else:
            L.check(L.lib().eri_adam8_grad_norm(table, 0.05, 1e-6, stream), "grad_norm")
        norm, scale, bad = C.c_float(), C.c_float(), C.c_uint64(12345)
        L.check(L.lib().eri_adam8_grad_norm_read(table, C.byref(norm), C.byref(scale), stream), "grad_norm_read")
        L.check(L.lib().eri_adam8_grad_nonfinite_read(table, C.byref(bad), stream), "grad_nonfinite_read")
        if static:  # the caller's buffer holds what the read calls report
            raw = result.cpu().numpy()
            assert raw[:2].view(np.float32)[0] == np.float32(norm.value) or np.isnan(norm.value)
            assert raw[:2].view(np.float32)[1] == np.float32(scale.value)
            assert int(raw.view(np.uint64)[1]) == bad.value
        h = L.hyper_pack(LR, B1, B2, EPS, WD, 1, L.MODE_ERI, L.FLAG_EXACT_PARAM | L.FLAG_CLIP_FROM_TABLE)
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")
        torch.cuda.synchronize()
        outs.append(((norm.value, scale.value, bad.value), gt.fetch()))
        L.lib().eri_adam8_table_destroy(table)
    return outs


def _same(a, b):
    (na, sa, ca), (pa, sta) = a
    (nb, sb, cb), (pb, stb) = b
    assert np.float32(na).view(np.uint32) == np.float32(nb).view(np.uint32), (na, nb)
    assert np.float32(sa).view(np.uint32) == np.float32(sb).view(np.uint32), (sa, sb)
    assert ca == cb
    for x, y in zip(pa, pb):
        assert np.array_equal(x.view(np.uint8), y.view(np.uint8))
    for x, y in zip(sta, stb):
        for u, v in zip(x, y):
            assert np.array_equal(u.view(np.uint8), v.view(np.uint8))


@pytest.mark.parametrize("bf16", [True, False])
def test_static_norm_equals_the_allocating_one_twice_in_a_row(bf16):
    import torch
    from eridiffusion_amd import _lib as L
    result = torch.empty(4, dtype=torch.int32, device="cuda:0")  # 16 bytes the caller owns
    big = [2048 * 300 + 77, 2048 * 40, 5, 640 * 16, 2048 * 1200 + 8]
    small = [2048 * 3 + 19, 320]
    first = _norm_both_ways(L, torch, big, bf16, 31 + bf16, result)
    _same(*first)
    assert first[0][0][1] < 1.0  # the clip factor is in play
    second = _norm_both_ways(L, torch, small, bf16, 57 + bf16, result)
    _same(*second)
    assert second[0][0][0] < first[0][0][0]  # fewer gradients, smaller norm: nothing of the first call is left
    # a NaN gradient: counted, and the clip factor stays 1 in both entry points
    nan_bits = np.uint16(0x7FC0) if bf16 else np.float32(np.nan)
    third = _norm_both_ways(L, torch, small, bf16, 91 + bf16, result, poison_grad=(0, 100, nan_bits))
    assert third[0][0][2] == 1 and third[1][0][2] == 1 and third[1][0][1] == 1.0
    assert np.isnan(third[0][0][0]) and np.isnan(third[1][0][0])


def test_static_norm_refuses_bad_arguments():
    import torch
    from eridiffusion_amd import _lib as L
    sizes = [4096]
    ps, gs = hs.make_inputs(sizes, True, 3)
    gt = hs.GpuTensors(ps, gs, hs.oracle_states(sizes), True)
    rows = gt.rows()
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    result = torch.empty(8, dtype=torch.int32, device="cuda:0")
    assert L.lib().eri_adam8_grad_norm_static(table, 1.0, 0.0, None, None) == -1
    assert L.lib().eri_adam8_grad_norm_static(None, 1.0, 0.0, result.data_ptr(), None) == -1
    assert L.lib().eri_adam8_grad_norm_static(table, 1.0, 0.0, result.data_ptr() + 4, None) == -2
    torch.cuda.synchronize()
    L.lib().eri_adam8_table_destroy(table)
