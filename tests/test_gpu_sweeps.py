"""GPU parity of the 32-bit AdamW sibling and the EMA sweep against the oracle (bit-exact: every
operation is an individually rounded fp32 operation on both sides)."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
SIZES = [2048 * 3 + 17, 5, 2048, 4100, 640 * 16]


def _up(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).cuda()


def _down(t, dtype):
    return t.cpu().numpy().view(dtype)


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("wd", [0.01, 0.0])
def test_adamw32_multi_tensor(bf16, wd):
    import torch
    from eridiffusion_amd import _lib as L
    rng = np.random.default_rng(3 + bf16)
    dt = np.uint16 if bf16 else np.float32
    tag = 2 if bf16 else 0
    ps, ms, vs = [], [], []
    for n in SIZES:
        p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        ps.append(onp.f32_to_bf16(p) if bf16 else p)
        ms.append(np.zeros(n, np.float32))
        vs.append(np.zeros(n, np.float32))
    dp, dm, dv = [_up(a) for a in ps], [_up(a) for a in ms], [_up(a) for a in vs]
    rows = (L.AdamW32Row * len(SIZES))()
    h = L.AdamW32Hyper(1e-3, 0.9, 0.999, 1e-8, wd)
    for step in range(3):
        gs = []
        for n in SIZES:
            g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
            gs.append(onp.f32_to_bf16(g) if bf16 else g)
        dg = [_up(a) for a in gs]
        for i, n in enumerate(SIZES):
            rows[i].p, rows[i].g, rows[i].m, rows[i].v = dp[i].data_ptr(), dg[i].data_ptr(), dm[i].data_ptr(), dv[i].data_ptr()
            rows[i].numel, rows[i].dtype_tag = n, tag
            oc.lib().eri_oracle_adamw32_step(oc.ptr(ps[i]), oc.ptr(gs[i]), oc.ptr(ms[i]), oc.ptr(vs[i]), n, tag,
                                             1e-3, 0.9, 0.999, 1e-8, wd, None)
        L.check(L.lib().eri_adamw32_step_multi(rows, len(SIZES), C.byref(h), torch.cuda.current_stream().cuda_stream), "adamw32")
        torch.cuda.synchronize()
    for i in range(len(SIZES)):
        assert np.array_equal(_down(dp[i], dt).view(np.uint16 if bf16 else np.uint32), ps[i].view(np.uint16 if bf16 else np.uint32))
        assert np.array_equal(_down(dm[i], np.uint32), ms[i].view(np.uint32))
        assert np.array_equal(_down(dv[i], np.uint32), vs[i].view(np.uint32))


def test_adamw32_with_fp32_master_copies():
    """Rows with and without a master copy in one launch; bf16 parameters, bit-exact against the oracle."""
    import torch
    from eridiffusion_amd import _lib as L
    rng = np.random.default_rng(21)
    ps, ws, ms, vs = [], [], [], []
    for i, n in enumerate(SIZES):
        p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        ps.append(onp.f32_to_bf16(p))
        ws.append(p.copy() if i % 2 == 0 else None)  # every other tensor keeps a master
        ms.append(np.zeros(n, np.float32))
        vs.append(np.zeros(n, np.float32))
    dp, dm, dv = [_up(a) for a in ps], [_up(a) for a in ms], [_up(a) for a in vs]
    dw = [_up(a) if a is not None else None for a in ws]
    rows = (L.AdamW32Row * len(SIZES))()
    h = L.AdamW32Hyper(1e-3, 0.9, 0.999, 1e-8, 0.01)
    for step in range(3):
        gs = [onp.f32_to_bf16((rng.standard_normal(n) * 1e-3).astype(np.float32)) for n in SIZES]
        dg = [_up(a) for a in gs]
        for i, n in enumerate(SIZES):
            rows[i].p, rows[i].g, rows[i].m, rows[i].v = dp[i].data_ptr(), dg[i].data_ptr(), dm[i].data_ptr(), dv[i].data_ptr()
            rows[i].master = dw[i].data_ptr() if dw[i] is not None else None
            rows[i].numel, rows[i].dtype_tag = n, 2
            oc.lib().eri_oracle_adamw32_step(oc.ptr(ps[i]), oc.ptr(gs[i]), oc.ptr(ms[i]), oc.ptr(vs[i]), n, 2,
                                             1e-3, 0.9, 0.999, 1e-8, 0.01, oc.ptr(ws[i]) if ws[i] is not None else None)
        L.check(L.lib().eri_adamw32_step_multi(rows, len(SIZES), C.byref(h), torch.cuda.current_stream().cuda_stream), "adamw32")
        torch.cuda.synchronize()
    for i in range(len(SIZES)):
        assert np.array_equal(_down(dp[i], np.uint16), ps[i])
        assert np.array_equal(_down(dm[i], np.uint32), ms[i].view(np.uint32))
        assert np.array_equal(_down(dv[i], np.uint32), vs[i].view(np.uint32))
        if ws[i] is not None:
            assert np.array_equal(_down(dw[i], np.uint32), ws[i].view(np.uint32))
            assert np.array_equal(ps[i], onp.f32_to_bf16(ws[i]))


@pytest.mark.parametrize("bf16", [True, False])
def test_ema_multi_tensor(bf16):
    import torch
    from eridiffusion_amd import _lib as L
    rng = np.random.default_rng(9)
    dt = np.uint16 if bf16 else np.float32
    tag = 2 if bf16 else 0
    sh, ps = [], []
    for n in SIZES:
        a = rng.standard_normal(n).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32)
        sh.append(onp.f32_to_bf16(a) if bf16 else a)
        ps.append(onp.f32_to_bf16(b) if bf16 else b)
    ds, dp = [_up(a) for a in sh], [_up(a) for a in ps]
    rows = (L.EmaRow * len(SIZES))()
    for i, n in enumerate(SIZES):
        rows[i].shadow, rows[i].p, rows[i].numel, rows[i].dtype_tag = ds[i].data_ptr(), dp[i].data_ptr(), n, tag
    for decay in (0.999, 0.9):
        L.check(L.lib().eri_ema_update_multi(rows, len(SIZES), decay, torch.cuda.current_stream().cuda_stream), "ema")
        for i, n in enumerate(SIZES):
            oc.lib().eri_oracle_ema_update(oc.ptr(sh[i]), oc.ptr(ps[i]), n, tag, decay)
    torch.cuda.synchronize()
    for i in range(len(SIZES)):
        assert np.array_equal(_down(ds[i], dt).view(np.uint16 if bf16 else np.uint32), sh[i].view(np.uint16 if bf16 else np.uint32))
        assert np.array_equal(_down(dp[i], dt), ps[i])


def test_sweep_argument_errors():
    from eridiffusion_amd import _lib as L
    rows = (L.EmaRow * 1)()
    rows[0].shadow, rows[0].p, rows[0].numel, rows[0].dtype_tag = 0x1000, 0x2000, 0, 2
    assert L.lib().eri_ema_update_multi(rows, 1, 0.9, None) == -3
    rows[0].numel, rows[0].dtype_tag = 8, 1
    assert L.lib().eri_ema_update_multi(rows, 1, 0.9, None) == -4
    rows[0].dtype_tag, rows[0].p = 2, 0x2004
    assert L.lib().eri_ema_update_multi(rows, 1, 0.9, None) == -2
    assert L.lib().eri_ema_update_multi(None, 1, 0.9, None) == -1


def _same_bits_nan_aware(got, want, bf16):
    g32 = onp.bf16_to_f32(got) if bf16 else got
    w32 = onp.bf16_to_f32(want) if bf16 else want
    both_nan = np.isnan(g32) & np.isnan(w32)
    raw = np.uint16 if bf16 else np.uint32
    return np.array_equal(got.view(raw)[~both_nan], want.view(raw)[~both_nan])


@pytest.mark.parametrize("bf16", [True, False])
def test_sweeps_with_extreme_and_non_finite_values(bf16):
    """Magnitudes from the denormal range to overflow, zeros, NaN and infinities through the 32-bit step
    (with and without a master copy) and the EMA sweep: same bits as the oracle, NaN in the same places."""
    import torch
    from eridiffusion_amd import _lib as L
    rng = np.random.default_rng(77 + bf16)
    tag = 2 if bf16 else 0
    n = 2048 * 2 + 333

    def wild():
        with np.errstate(over="ignore"):
            x = (rng.standard_normal(n) * 10.0 ** rng.uniform(-44, 38, n)).astype(np.float32)
        x[::53] = 0.0
        x[7], x[2048 + 3], x[4096 + 100] = np.nan, np.inf, -np.inf
        return x

    for use_master in (False, True):
        p32, g32 = wild(), wild()
        p = onp.f32_to_bf16(p32) if bf16 else p32.copy()
        g = onp.f32_to_bf16(g32) if bf16 else g32.copy()
        w = (onp.bf16_to_f32(p) if bf16 else p).astype(np.float32).copy() if use_master else None
        m, v = np.abs(wild()), np.abs(wild())
        m[7] = 0.0
        dp, dg, dm, dv = _up(p), _up(g), _up(m), _up(v)
        dw = _up(w) if use_master else None
        rows = (L.AdamW32Row * 1)()
        rows[0].p, rows[0].g, rows[0].m, rows[0].v = dp.data_ptr(), dg.data_ptr(), dm.data_ptr(), dv.data_ptr()
        rows[0].master = dw.data_ptr() if use_master else None
        rows[0].numel, rows[0].dtype_tag = n, tag
        h = L.AdamW32Hyper(1e-3, 0.9, 0.999, 1e-8, 0.01)
        for _ in range(2):
            L.check(L.lib().eri_adamw32_step_multi(rows, 1, C.byref(h), torch.cuda.current_stream().cuda_stream), "adamw32")
            with np.errstate(all="ignore"):
                oc.lib().eri_oracle_adamw32_step(oc.ptr(p), oc.ptr(g), oc.ptr(m), oc.ptr(v), n, tag, 1e-3, 0.9, 0.999, 1e-8, 0.01,
                                                 oc.ptr(w) if use_master else None)
        torch.cuda.synchronize()
        assert _same_bits_nan_aware(_down(dp, np.uint16 if bf16 else np.float32), p, bf16)
        assert _same_bits_nan_aware(_down(dm, np.float32), m, False)
        assert _same_bits_nan_aware(_down(dv, np.float32), v, False)
        if use_master:
            assert _same_bits_nan_aware(_down(dw, np.float32), w, False)
    sh32, p32 = wild(), wild()
    sh = onp.f32_to_bf16(sh32) if bf16 else sh32
    pp = onp.f32_to_bf16(p32) if bf16 else p32
    ds, dp = _up(sh), _up(pp)
    rows = (L.EmaRow * 1)()
    rows[0].shadow, rows[0].p, rows[0].numel, rows[0].dtype_tag = ds.data_ptr(), dp.data_ptr(), n, tag
    L.check(L.lib().eri_ema_update_multi(rows, 1, 0.999, torch.cuda.current_stream().cuda_stream), "ema")
    with np.errstate(all="ignore"):
        oc.lib().eri_oracle_ema_update(oc.ptr(sh), oc.ptr(pp), n, tag, 0.999)
    torch.cuda.synchronize()
    assert _same_bits_nan_aware(_down(ds, np.uint16 if bf16 else np.float32), sh, bf16)


def test_quantize_dequantize_with_extreme_values():
    """Checkpoint traffic: blocks whose maximum is denormal, huge or infinite, all-zero blocks, NaN."""
    import torch
    from eridiffusion_amd import _lib as L
    import harness as hs
    rng = np.random.default_rng(5150)
    n = 2048 * 6 + 77
    scale = np.repeat(10.0 ** np.array([-43.0, -30.0, 0.0, 30.0, 38.0, -5.0, 3.0]), 2048)[:n]
    with np.errstate(over="ignore"):
        x = (rng.standard_normal(n) * scale).astype(np.float32)
    x[2048 * 2:2048 * 3] = 0.0
    x[2048 * 5 + 9] = np.inf
    x[2048 * 6 + 5] = np.nan
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    for signed, table in ((1, hs.MAPS[0]), (0, hs.MAPS[1])):
        xs = x if signed else np.abs(x)
        xd = torch.from_numpy(xs).to(dev)
        codes = torch.empty(n, dtype=torch.uint8, device=dev)
        absmax = torch.empty(7, dtype=torch.float32, device=dev)
        back = torch.empty(n, dtype=torch.float32, device=dev)
        L.check(L.lib().eri_adam8_quantize(xd.data_ptr(), signed, n, codes.data_ptr(), absmax.data_ptr(), stream), "q")
        L.check(L.lib().eri_adam8_dequantize(codes.data_ptr(), absmax.data_ptr(), signed, n, back.data_ptr(), stream), "dq")
        torch.cuda.synchronize()
        wc, wa, wb = np.empty(n, np.uint8), np.empty(7, np.float32), np.empty(n, np.float32)
        with np.errstate(all="ignore"):
            oc.lib().eri_oracle_quantize(oc.ptr(xs), oc.ptr(table), n, oc.ptr(wc), oc.ptr(wa))
            oc.lib().eri_oracle_dequantize(oc.ptr(wc), oc.ptr(wa), oc.ptr(table), n, oc.ptr(wb))
        assert np.array_equal(codes.cpu().numpy(), wc), signed
        assert np.array_equal(absmax.cpu().numpy().view(np.uint32), wa.view(np.uint32)), signed
        assert _same_bits_nan_aware(back.cpu().numpy(), wb, False), signed


def test_traffic_probe_moves_the_bytes_and_changes_none():
    """eri_adam8_traffic_probe reads and rewrites every full block of the BF16 rows as the step does, with the
    bits they had: parameters, gradients, codes and absmax are unchanged afterwards (guard bands included), a
    table without such rows and a gradient-only table are refused."""
    import ctypes as C
    import torch
    from eridiffusion_amd import _lib as L
    sizes = [2048 * 7 + 99, 2048 * 2, 100, 2048 * 33]
    ps, gs = hs.make_inputs(sizes, True, 606)
    states = hs.oracle_states(sizes)
    hs.oracle_step(ps, gs, states, (1e-4, 0.9, 0.999, 1e-8, 0.01, 1), True)  # states with real contents
    want_p = [p.copy() for p in ps]
    gt = hs.GpuTensors(ps, gs, states, True)
    rows = gt.rows()
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    for _ in range(3):
        L.check(L.lib().eri_adam8_traffic_probe(table, None), "traffic_probe")
    torch.cuda.synchronize()
    got_p, got_st = gt.fetch()
    for i in range(len(sizes)):
        assert np.array_equal(got_p[i], want_p[i]), i
        for k in range(4):
            assert np.array_equal(got_st[i][k].view(np.uint8), states[i][k].view(np.uint8)), (i, k)
        assert np.array_equal(gt.down(gt.g[i]), gs[i]), i
    L.lib().eri_adam8_table_destroy(table)
    # fp32 rows only: nothing for the probe
    ps32, gs32 = hs.make_inputs([4096], False, 607)
    gt32 = hs.GpuTensors(ps32, gs32, hs.oracle_states([4096]), False)
    rows32 = gt32.rows()
    t32 = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows32, 1, None, C.byref(t32)), "table_create")
    assert L.lib().eri_adam8_traffic_probe(t32, None) == -6
    L.lib().eri_adam8_table_destroy(t32)
    assert L.lib().eri_adam8_traffic_probe(None, None) == -1
