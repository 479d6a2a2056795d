"""One call over rows of both dtypes: the library keeps one device table per dtype and launches once per
group, so the norm's partial sums, the error statistics and the row order all cross a group boundary."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-3, 0.9, 0.999, 1e-8, 0.01
SIZES_B = [2048 * 3 + 5, 700, 4096, 2048 * 9]
SIZES_F = [2048 * 2 + 100, 9, 2048 * 4]
ORDER = [(1, 0), (0, 0), (0, 1), (1, 1), (1, 2), (0, 2), (1, 3)]  # (is bf16, index in its list), interleaved


def _L():
    from eridiffusion_amd import _lib
    return _lib


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _merged_rows(L, gt_f, gt_b):
    parts = {0: gt_f.rows(), 1: gt_b.rows()}
    rows = (L.TensorRow * len(ORDER))()
    start = 0
    for k, (b, i) in enumerate(ORDER):
        src = parts[b][i]
        for name, _ in L.TensorRow._fields_:
            setattr(rows[k], name, getattr(src, name))
        rows[k].block_start = start
        start += (rows[k].numel + 2047) // 2048
    return rows


@pytest.mark.parametrize("mode", [0, 2])
def test_table_with_rows_of_both_dtypes_norm_clip_statistics_and_step(mode):
    import torch
    L = _L()
    omode = oc.MODE_ERI if mode == 0 else oc.MODE_BNB
    ps_f, gs_f = hs.make_inputs(SIZES_F, False, 501, g_std=1e-3)
    ps_b, gs_b = hs.make_inputs(SIZES_B, True, 502, g_std=1e-3)
    st_f, st_b = hs.oracle_states(SIZES_F), hs.oracle_states(SIZES_B)
    gt_f, gt_b = hs.GpuTensors(ps_f, gs_f, st_f, False), hs.GpuTensors(ps_b, gs_b, st_b, True)
    rows = _merged_rows(L, gt_f, gt_b)
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), _stream(), C.byref(table)), "table_create")
    numel, blocks = C.c_uint64(), C.c_uint64()
    L.check(L.lib().eri_adam8_table_info(table, C.byref(numel), C.byref(blocks)), "table_info")
    assert numel.value == sum(SIZES_F) + sum(SIZES_B)
    max_norm = 0.01
    for t in (1, 2, 3):
        if t > 1:
            gs_f = hs.fresh_grads(SIZES_F, False, 510 + t, 1e-3)
            gs_b = hs.fresh_grads(SIZES_B, True, 520 + t, 1e-3)
            gt_f.set_grads(gs_f)
            gt_b.set_grads(gs_b)
        L.check(L.lib().eri_adam8_grad_norm(table, max_norm, 1e-6, _stream()), "grad_norm")
        norm, scale = C.c_float(), C.c_float()
        L.check(L.lib().eri_adam8_grad_norm_read(table, C.byref(norm), C.byref(scale), _stream()), "norm_read")
        all_sq = [float(np.sum(g.astype(np.float64) ** 2)) for g in gs_f]
        all_sq += [float(np.sum(onp.bf16_to_f32(g).astype(np.float64) ** 2)) for g in gs_b]
        want = np.sqrt(sum(all_sq))
        assert abs(norm.value - want) <= 2e-6 * want  # the norm covers both groups
        assert scale.value == np.float32(max_norm) / (np.float32(norm.value) + np.float32(1e-6))
        bad = C.c_uint64(7)
        L.check(L.lib().eri_adam8_grad_nonfinite_read(table, C.byref(bad), _stream()), "nonfinite")
        assert bad.value == 0
        flags = L.FLAG_EXACT_PARAM | L.FLAG_CLIP_FROM_TABLE
        h = L.hyper_pack(LR, B1, B2, EPS, WD, t, mode, flags)
        if mode == 0:
            L.check(L.lib().eri_adam8_quant_error(table, C.byref(h), _stream()), "quant_error")
            m_err, v_err = C.c_float(), C.c_float()
            L.check(L.lib().eri_adam8_quant_error_read(table, C.byref(m_err), C.byref(v_err), _stream()), "qerr_read")
            assert 0 < m_err.value < 1e-4 and 0 < v_err.value < 1e-6
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), _stream()), "step_table")
        torch.cuda.synchronize()
        hs.oracle_step(ps_f, gs_f, st_f, (LR, B1, B2, EPS, WD, t), False, omode, grad_scale=float(scale.value))
        hs.oracle_step(ps_b, gs_b, st_b, (LR, B1, B2, EPS, WD, t), True, omode, grad_scale=float(scale.value))
    for gt, ps, st, bf16 in ((gt_f, ps_f, st_f, False), (gt_b, ps_b, st_b, True)):
        got_p, got_st = gt.fetch()
        stats = hs.compare(got_p, got_st, ps, st, bf16, True, "mixed-bf16%d" % bf16)
        assert stats["code_mismatch"] == 0
    # a non-finite gradient in the second group is counted
    poisoned = [g.copy() for g in gs_b]
    poisoned[2][5] = 0x7FC0  # NaN
    poisoned[3][2048 * 8 + 7] = 0x7F80  # +inf
    gt_b.set_grads(poisoned)
    L.check(L.lib().eri_adam8_grad_norm(table, max_norm, 1e-6, _stream()), "grad_norm")
    bad = C.c_uint64()
    L.check(L.lib().eri_adam8_grad_nonfinite_read(table, C.byref(bad), _stream()), "nonfinite")
    assert bad.value == 2
    L.lib().eri_adam8_table_destroy(table)


def _up(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).cuda()


def test_adamw32_and_ema_over_rows_of_both_dtypes():
    import torch
    L = _L()
    rng = np.random.default_rng(77)
    sizes = [(2048 * 2 + 9, True), (100, False), (2048 * 3, False), (4100, True), (7, True), (2048 * 5 + 1, False)]
    ps, gs, ms, vs, sh = [], [], [], [], []
    for n, bf16 in sizes:
        p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        s = rng.standard_normal(n).astype(np.float32)
        ps.append(onp.f32_to_bf16(p) if bf16 else p)
        gs.append(onp.f32_to_bf16(g) if bf16 else g)
        sh.append(onp.f32_to_bf16(s) if bf16 else s)
        ms.append(np.zeros(n, np.float32))
        vs.append(np.zeros(n, np.float32))
    dp, dg, dm, dv, ds = ([_up(a) for a in xs] for xs in (ps, gs, ms, vs, sh))
    rows = (L.AdamW32Row * len(sizes))()
    erows = (L.EmaRow * len(sizes))()
    for i, (n, bf16) in enumerate(sizes):
        tag = 2 if bf16 else 0
        rows[i].p, rows[i].g, rows[i].m, rows[i].v = dp[i].data_ptr(), dg[i].data_ptr(), dm[i].data_ptr(), dv[i].data_ptr()
        rows[i].numel, rows[i].dtype_tag = n, tag
        erows[i].shadow, erows[i].p, erows[i].numel, erows[i].dtype_tag = ds[i].data_ptr(), dp[i].data_ptr(), n, tag
    h = L.AdamW32Hyper(1e-3, 0.9, 0.999, 1e-8, 0.01)
    stream = torch.cuda.current_stream().cuda_stream
    for step in range(2):
        L.check(L.lib().eri_adamw32_step_multi(rows, len(sizes), C.byref(h), stream), "adamw32")
        L.check(L.lib().eri_ema_update_multi(erows, len(sizes), 0.99, stream), "ema")
        for i, (n, bf16) in enumerate(sizes):
            tag = 2 if bf16 else 0
            oc.lib().eri_oracle_adamw32_step(oc.ptr(ps[i]), oc.ptr(gs[i]), oc.ptr(ms[i]), oc.ptr(vs[i]), n, tag,
                                             1e-3, 0.9, 0.999, 1e-8, 0.01, None)
            oc.lib().eri_oracle_ema_update(oc.ptr(sh[i]), oc.ptr(ps[i]), n, tag, 0.99)
    torch.cuda.synchronize()
    for i, (n, bf16) in enumerate(sizes):
        bits = np.uint16 if bf16 else np.uint32
        assert np.array_equal(dp[i].cpu().numpy().view(bits), ps[i].view(bits)), i
        assert np.array_equal(ds[i].cpu().numpy().view(bits), sh[i].view(bits)), i
        assert np.array_equal(dm[i].cpu().numpy().view(np.uint32), ms[i].view(np.uint32)), i
        assert np.array_equal(dv[i].cpu().numpy().view(np.uint32), vs[i].view(np.uint32)), i
