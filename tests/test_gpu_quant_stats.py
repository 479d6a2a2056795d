"""quantization_stats(): mean absolute quantisation error of the moments at the last step."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-3, 0.9, 0.999, 1e-8, 0.01


def test_stats_equal_the_error_of_the_oracles_quantisation():
    import torch
    from eridiffusion_amd import _lib as L
    sizes = [2048 * 3 + 100, 300, 4096]
    ps, gs = hs.make_inputs(sizes, True, 11)
    states = hs.oracle_states(sizes)
    gt = hs.GpuTensors(ps, gs, states, True)
    handles = (C.c_void_p * 3)()
    for i in range(3):
        h = C.c_void_p()
        L.check(L.lib().eri_param_create(gt.ptr(gt.p[i]), sizes[i], 2, C.byref(h)), "param_create")
        L.check(L.lib().eri_param_set_grad(h, gt.ptr(gt.g[i])), "set_grad")
        handles[i] = h
    opt = C.c_void_p()
    L.check(L.lib().eri_adam8bit_new(handles, 3, None, None, C.byref(opt)), "new")
    m_err, v_err = C.c_float(-1), C.c_float(-1)
    L.check(L.lib().eri_adam8bit_quantization_stats(opt, C.byref(m_err), C.byref(v_err)), "stats")
    assert (m_err.value, v_err.value) == (0.0, 0.0)  # nothing tracked yet
    L.check(L.lib().eri_adam8bit_track_quantization_error(opt, 1), "track")
    s_map, u_map = hs.MAPS
    omb1, omb2 = np.float32(1) - np.float32(B1), np.float32(1) - np.float32(B2)
    for t in (1, 2):
        want_m, want_v = [], []
        for i, n in enumerate(sizes):
            blk = np.arange(n) // 2048
            g = onp.bf16_to_f32(gs[i])
            m = (s_map[states[i][0]] * states[i][2][blk]) * np.float32(B1) + g * omb1   # the moments the step forms
            v = (u_map[states[i][1]] * states[i][3][blk]) * np.float32(B2) + (g * g) * omb2
            hs.oracle_step([ps[i]], [gs[i]], [states[i]], (LR, B1, B2, EPS, WD, t), True)
            want_m.append(np.abs(m.astype(np.float64) - (s_map[states[i][0]] * states[i][2][blk]).astype(np.float64)).mean())
            want_v.append(np.abs(v.astype(np.float64) - (u_map[states[i][1]] * states[i][3][blk]).astype(np.float64)).mean())
        L.check(L.lib().eri_adam8bit_step(opt, None), "step")
        L.check(L.lib().eri_adam8bit_quantization_stats(opt, C.byref(m_err), C.byref(v_err)), "stats")
        assert np.isclose(m_err.value, np.mean(want_m), rtol=1e-5)
        assert np.isclose(v_err.value, np.mean(want_v), rtol=1e-5)
        assert m_err.value > 0 and v_err.value > 0
    torch.cuda.synchronize()
    for i in range(3):
        assert hs.bf16_ulp_distance(gt.down(gt.p[i]), ps[i]).max() <= 1
    L.lib().eri_adam8bit_destroy(opt)
