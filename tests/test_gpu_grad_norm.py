"""Global gradient norm on the device and the clip factor folded into the step."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01


def _L():
    from eridiffusion_amd import _lib
    return _lib


def _f32(gs, bf16):
    return [onp.bf16_to_f32(g) if bf16 else g for g in gs]


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("max_norm,denom", [(0.05, 0.0), (0.05, 1e-6), (1e9, 0.0)])
def test_norm_and_clip_factor_then_step(bf16, max_norm, denom):
    import torch
    L = _L()
    sizes = [2048 * 5 + 333, 7, 2048, 4096 + 1, 320, 100000]
    ps, gs = hs.make_inputs(sizes, bf16, 77 + bf16, g_std=1e-3)
    states = hs.oracle_states(sizes)
    gt = hs.GpuTensors(ps, gs, states, bf16)
    rows = gt.rows()
    stream = torch.cuda.current_stream().cuda_stream
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), stream, C.byref(table)), "table_create")
    L.check(L.lib().eri_adam8_grad_norm(table, max_norm, denom, stream), "grad_norm")
    norm, scale = C.c_float(), C.c_float()
    L.check(L.lib().eri_adam8_grad_norm_read(table, C.byref(norm), C.byref(scale), stream), "grad_norm_read")
    # tolerance: squares are exact products rounded to fp32 and each lane adds 32 of them in fp32
    # before the f64 total; 2e-6 relative on the norm covers that with margin
    want = np.sqrt(sum(float(np.sum(g.astype(np.float32).astype(np.float64) ** 2)) for g in _f32(gs, bf16)))
    assert abs(norm.value - want) <= 2e-6 * want
    if norm.value > max_norm:
        assert scale.value == np.float32(max_norm) / (np.float32(norm.value) + np.float32(denom))
        assert scale.value < 1
    else:
        assert scale.value == 1.0
    h = L.hyper_pack(LR, B1, B2, EPS, WD, 1, L.MODE_ERI, L.FLAG_EXACT_PARAM | L.FLAG_CLIP_FROM_TABLE)
    L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")
    torch.cuda.synchronize()
    hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, 1), bf16, grad_scale=float(scale.value))
    got_p, got_st = gt.fetch()
    stats = hs.compare(got_p, got_st, ps, states, bf16, True, "clip")
    assert stats["code_mismatch"] == 0
    L.lib().eri_adam8_table_destroy(table)


def test_non_finite_gradients_do_not_clip():
    import torch
    L = _L()
    sizes = [4096, 100]
    ps, gs = hs.make_inputs(sizes, False, 5)
    gs[0][17] = np.inf
    gt = hs.GpuTensors(ps, gs, hs.oracle_states(sizes), False)
    rows = gt.rows()
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    L.check(L.lib().eri_adam8_grad_norm(table, 1.0, 0.0, None), "grad_norm")
    norm, scale = C.c_float(), C.c_float()
    L.check(L.lib().eri_adam8_grad_norm_read(table, C.byref(norm), C.byref(scale), None), "read")
    assert np.isinf(norm.value) and scale.value == 1.0
    bad = C.c_uint64(99)
    L.check(L.lib().eri_adam8_grad_nonfinite_read(table, C.byref(bad), None), "nonfinite_read")
    assert bad.value == 1
    h = L.hyper_pack(LR, B1, B2, EPS, WD, 1, L.MODE_ERI, L.FLAG_CLIP_FROM_TABLE)
    fresh = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(fresh)), "table_create")
    assert L.lib().eri_adam8_step_table(fresh, C.byref(h), None) == -6  # no norm was computed for that table
    L.lib().eri_adam8_table_destroy(table)
    L.lib().eri_adam8_table_destroy(fresh)


def test_optimizer_object_clips_inside_step():
    import torch
    L = _L()
    sizes = [2048 * 3 + 5, 640]
    ps, gs = hs.make_inputs(sizes, True, 91, g_std=1e-2)
    states = hs.oracle_states(sizes)
    gt = hs.GpuTensors(ps, gs, states, True)
    handles = (C.c_void_p * 2)()
    for i in range(2):
        hnd = C.c_void_p()
        L.check(L.lib().eri_param_create(gt.ptr(gt.p[i]), sizes[i], 2, C.byref(hnd)), "param_create")
        L.check(L.lib().eri_param_set_grad(hnd, gt.ptr(gt.g[i])), "set_grad")
        handles[i] = hnd
    opt = C.c_void_p()
    L.check(L.lib().eri_adam8bit_new(handles, 2, None, None, C.byref(opt)), "new")
    L.check(L.lib().eri_adam8bit_set_flags(opt, L.FLAG_EXACT_PARAM), "flags")
    L.check(L.lib().eri_adam8bit_set_max_grad_norm(opt, 0.5, 0.0), "max_norm")
    L.check(L.lib().eri_adam8bit_set_param_grad_scale(opt, 1, 0.5), "param_scale")
    L.check(L.lib().eri_adam8bit_step(opt, None), "step")
    norm, scale = C.c_float(), C.c_float()
    L.check(L.lib().eri_adam8bit_last_grad_norm(opt, C.byref(norm), C.byref(scale)), "last_norm")
    assert norm.value > 0.5 and scale.value == np.float32(0.5) / np.float32(norm.value)
    torch.cuda.synchronize()
    for i, ts in enumerate((1.0, 0.5)):
        s = (np.float32(1.0) * np.float32(ts)) * np.float32(scale.value)
        hs.oracle_step([ps[i]], [gs[i]], [states[i]], (1e-3, B1, B2, EPS, WD, 1), True, grad_scale=float(s))
    got_p = [gt.down(b) for b in gt.p]
    for g, w in zip(got_p, ps):
        assert np.array_equal(g, w)
    L.lib().eri_adam8bit_destroy(opt)


@pytest.mark.parametrize("bf16", [True, False])
def test_non_finite_gradient_count(bf16):
    """NaN and +-inf elements are counted exactly, in full blocks and in partial last blocks; huge
    finite values whose squares overflow make the norm infinite but are not counted."""
    L = _L()
    sizes = [2048 * 4 + 100, 50, 2048 * 2, 2048 * 3 + 1]
    ps, gs = hs.make_inputs(sizes, bf16, 13)

    def put(i, j, value):
        gs[i][j] = onp.f32_to_bf16(np.array([value], np.float32))[0] if bf16 else value

    put(0, 5, np.nan); put(0, 2048 * 2 + 77, -np.inf); put(0, 2048 * 4 + 99, np.inf)   # full blocks and the tail
    put(1, 49, np.nan)                                                               # a tensor that is only a tail
    put(2, 2048 + 3, np.nan); put(2, 2048 + 4, np.nan); put(2, 4095, np.inf)          # three in one block
    put(3, 10, 3.0e38)                                                               # finite, square overflows
    want = sum(int(np.count_nonzero(~np.isfinite(g))) for g in _f32(gs, bf16))
    assert want == 7
    gt = hs.GpuTensors(ps, gs, hs.oracle_states(sizes), bf16)
    rows = gt.rows()
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    for _ in range(2):  # the count does not accumulate over calls
        L.check(L.lib().eri_adam8_grad_norm(table, 1.0, 0.0, None), "grad_norm")
        bad = C.c_uint64()
        L.check(L.lib().eri_adam8_grad_nonfinite_read(table, C.byref(bad), None), "nonfinite_read")
        assert bad.value == want
    L.lib().eri_adam8_table_destroy(table)
    # clean gradients: zero
    ps, gs = hs.make_inputs(sizes, bf16, 14)
    gt = hs.GpuTensors(ps, gs, hs.oracle_states(sizes), bf16)
    rows = gt.rows()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    L.check(L.lib().eri_adam8_grad_norm(table, 1.0, 0.0, None), "grad_norm")
    L.check(L.lib().eri_adam8_grad_nonfinite_read(table, C.byref(bad), None), "nonfinite_read")
    assert bad.value == 0
    L.lib().eri_adam8_table_destroy(table)


def test_joint_norm_over_a_step_table_and_a_gradient_only_table():
    """Tensors that take another step than the 8-bit one (fp32 moments) still count in the global norm: their
    gradients sit in a gradient-only table, eri_adam8_grad_norm_joint norms both tables as one, the 8-bit step
    and the scaled 32-bit step then apply the one clip factor.  The gradient-only table refuses to step."""
    import torch
    L = _L()
    sizes8, sizes32 = [2048 * 3 + 40, 4096, 777], [300, 2048 + 16, 64]
    ps, gs = hs.make_inputs(sizes8, True, 4242, g_std=1e-3)
    states = hs.oracle_states(sizes8)
    gt = hs.GpuTensors(ps, gs, states, True)
    rows = gt.rows()
    table, gtable = C.c_void_p(), C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    # the other tensors: fp32 parameters with fp32 moments
    rng = np.random.default_rng(99)
    p32 = [(rng.standard_normal(n) * 0.02).astype(np.float32) for n in sizes32]
    g32 = [(rng.standard_normal(n) * 3e-3).astype(np.float32) for n in sizes32]
    m32 = [np.zeros(n, np.float32) for n in sizes32]
    v32 = [np.zeros(n, np.float32) for n in sizes32]
    up = lambda a: torch.from_numpy(a.copy()).to("cuda:0")
    d_p, d_g, d_m, d_v = ([up(a) for a in xs] for xs in (p32, g32, m32, v32))
    grows = (L.TensorRow * len(sizes32))()
    start = 0
    for i, n in enumerate(sizes32):
        grows[i].p, grows[i].g, grows[i].numel = d_p[i].data_ptr(), d_g[i].data_ptr(), n
        grows[i].block_start, grows[i].dtype_tag, grows[i].grad_scale = start, L.DTYPE_F32, 1.0
        start += (n + 2047) // 2048
    L.check(L.lib().eri_adam8_grad_table_create(grows, len(grows), None, C.byref(gtable)), "grad_table_create")
    h = L.hyper_pack(LR, B1, B2, EPS, WD, 1, L.MODE_ERI, L.FLAG_EXACT_PARAM | L.FLAG_CLIP_FROM_TABLE)
    assert L.lib().eri_adam8_step_table(gtable, C.byref(h), None) == -6
    assert b"gradient-only" in L.lib().eri_last_error()
    assert L.lib().eri_adam8_grad_norm_joint(table, None, 0.01, 0.0, None) == -1
    assert L.lib().eri_adam8_grad_norm_joint(table, table, 0.01, 0.0, None) == -6
    L.check(L.lib().eri_adam8_grad_norm_joint(table, gtable, 0.01, 0.0, None), "grad_norm_joint")
    norm, scale, norm2, scale2 = C.c_float(), C.c_float(), C.c_float(), C.c_float()
    L.check(L.lib().eri_adam8_grad_norm_read(table, C.byref(norm), C.byref(scale), None), "read")
    L.check(L.lib().eri_adam8_grad_norm_read(gtable, C.byref(norm2), C.byref(scale2), None), "read")
    assert (norm.value, scale.value) == (norm2.value, scale2.value)
    want = np.sqrt(sum(float(np.sum(g.astype(np.float64) ** 2)) for g in _f32(gs, True) + g32))
    alone = np.sqrt(sum(float(np.sum(g.astype(np.float64) ** 2)) for g in _f32(gs, True)))
    assert abs(norm.value - want) <= 2e-6 * want and abs(norm.value - alone) > 1e-3 * want
    assert scale.value == np.float32(0.01) / np.float32(norm.value) and scale.value < 1
    dev_scale = C.c_void_p()
    L.check(L.lib().eri_adam8_grad_norm_scale_ptr(gtable, C.byref(dev_scale)), "scale_ptr")
    # both steps under the one factor
    L.check(L.lib().eri_adam8_step_table(table, C.byref(h), None), "step_table")
    rows32 = (L.AdamW32Row * len(sizes32))()
    for i, n in enumerate(sizes32):
        rows32[i].p, rows32[i].g, rows32[i].m, rows32[i].v = (t[i].data_ptr() for t in (d_p, d_g, d_m, d_v))
        rows32[i].numel, rows32[i].dtype_tag = n, L.DTYPE_F32
    rows32[1].grad_scale = 0.5  # a per-layer multiplier on one row; the zeroed rows read as 1
    h32 = L.AdamW32Hyper(1e-3, B1, B2, EPS, WD)
    L.check(L.lib().eri_adamw32_step_multi_scaled(rows32, len(sizes32), C.byref(h32), 2.0, dev_scale, None), "adamw32_scaled")
    torch.cuda.synchronize()
    hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, 1), True, grad_scale=float(scale.value))
    got_p, got_st = gt.fetch()
    assert hs.compare(got_p, got_st, ps, states, True, True, "joint clip")["code_mismatch"] == 0
    for i, n in enumerate(sizes32):
        factor = float((np.float32(2.0) * np.float32(0.5 if i == 1 else 1.0)) * np.float32(scale.value))
        oc.lib().eri_oracle_adamw32_step_scaled(oc.ptr(p32[i]), oc.ptr(g32[i]), oc.ptr(m32[i]), oc.ptr(v32[i]), n, oc.DT_F32,
                                                1e-3, B1, B2, EPS, WD, None, factor)
        for got, want_a in ((d_p[i], p32[i]), (d_m[i], m32[i]), (d_v[i], v32[i])):
            assert np.array_equal(got.cpu().numpy().view(np.uint32), want_a.view(np.uint32)), i
    # a gradient-only table normed alone
    L.check(L.lib().eri_adam8_grad_norm(gtable, 0.0, 0.0, None), "grad_norm")
    L.check(L.lib().eri_adam8_grad_norm_read(gtable, C.byref(norm2), C.byref(scale2), None), "read")
    only = np.sqrt(sum(float(np.sum(g.astype(np.float64) ** 2)) for g in g32))
    assert abs(norm2.value - only) <= 2e-6 * only and scale2.value == 1.0
    L.lib().eri_adam8_table_destroy(gtable)
    L.lib().eri_adam8_table_destroy(table)
