"""A seeded random sequence of calls on the list-of-parameters optimizer, mirrored call by call on the
oracle: changing subsets of parameters with gradients (the launch table is rebuilt when the subset
changes), learning-rate and scale changes, clipping switched on and off, and a save / load into a
fresh optimizer in the middle.  Parameters of both dtypes; exact flag, so everything is bit for bit."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
B1, B2, EPS, WD = 0.9, 0.999, 1e-8, 0.01
SIZES = [(2048 * 3 + 77, True), (640, False), (2048 * 2, True), (5000, False), (9, True), (2048 * 6 + 1, False)]


def _L():
    from eridiffusion_amd import _lib
    return _lib


def _new_optimizer(L, handles, lr):
    cfg = L.Adam8bitConfigC()
    L.lib().eri_adam8bit_config_default(C.byref(cfg))
    cfg.lr = lr
    opt = C.c_void_p()
    L.check(L.lib().eri_adam8bit_new(handles, len(SIZES), C.byref(cfg), None, C.byref(opt)), "adam8bit_new")
    L.check(L.lib().eri_adam8bit_set_flags(opt, L.FLAG_EXACT_PARAM), "set_flags")
    return opt


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_call_sequence_matches_the_oracle(seed, tmp_path):
    import torch
    L = _L()
    rng = np.random.default_rng(1000 + seed)
    n_par = len(SIZES)
    ps = []
    for k, (n, bf16) in enumerate(SIZES):
        p, _ = hs.make_inputs([n], bf16, 2000 + 10 * seed + k)
        ps.append(p[0])
    gts = [hs.GpuTensors([ps[k]], [ps[k]], [list(oc.state_init(SIZES[k][0]))], SIZES[k][1]) for k in range(n_par)]
    handles = (C.c_void_p * n_par)()
    for k, (n, bf16) in enumerate(SIZES):
        h = C.c_void_p()
        L.check(L.lib().eri_param_create(gts[k].ptr(gts[k].p[0]), n, 2 if bf16 else 0, C.byref(h)), "param_create")
        handles[k] = h
    lr = 1e-3
    opt = _new_optimizer(L, handles, lr)
    states = [None] * n_par  # oracle states, created at a parameter's first gradient
    step = 0
    global_scale = np.float32(1.0)
    par_scale = [np.float32(1.0)] * n_par
    max_norm = 0.0

    def check_all(tag):
        torch.cuda.synchronize()
        for k, (n, bf16) in enumerate(SIZES):
            got = gts[k].down(gts[k].p[0])
            bits = np.uint16 if bf16 else np.uint32
            assert np.array_equal(got.view(bits), ps[k].view(bits)), (tag, "parameter", k)
            ptrs = [C.c_void_p() for _ in range(4)]
            L.check(L.lib().eri_adam8bit_state_ptrs(opt, k, *[C.byref(q) for q in ptrs]), "state_ptrs")
            if states[k] is None:
                assert not ptrs[0].value, (tag, "state without a gradient", k)
                continue
            nb = (n + 2047) // 2048
            for q, want in zip(ptrs, states[k]):
                host = np.empty_like(want)
                L.check(L.lib().eri_hip_memcpy_async(host.ctypes.data, q.value, host.nbytes, 2, None), "d2h")
                L.check(L.lib().eri_hip_stream_sync(None), "sync")
                assert np.array_equal(host.view(np.uint8), want.view(np.uint8)), (tag, "state", k)
            assert len(states[k][2]) == nb

    for it in range(14):
        # settings
        if rng.random() < 0.3:
            lr = float(rng.choice([1e-3, 3e-4, 5e-5]))
            L.check(L.lib().eri_adam8bit_set_learning_rate(opt, lr), "set_lr")
        if rng.random() < 0.3:
            global_scale = np.float32(rng.choice([1.0, 0.5, 0.125]))
            L.check(L.lib().eri_adam8bit_set_grad_scale(opt, float(global_scale)), "set_grad_scale")
        if rng.random() < 0.3:
            k = int(rng.integers(0, n_par))
            par_scale[k] = np.float32(rng.choice([1.0, 0.25, 2.0]))
            L.check(L.lib().eri_adam8bit_set_param_grad_scale(opt, k, float(par_scale[k])), "set_param_scale")
        if rng.random() < 0.4:
            max_norm = float(rng.choice([0.0, 0.02, 1e6]))
            L.check(L.lib().eri_adam8bit_set_max_grad_norm(opt, max_norm, 1e-6), "set_max_grad_norm")
        # gradients for a random subset
        live = [k for k in range(n_par) if rng.random() < 0.7]
        grads = {}
        for k in range(n_par):
            if k in live:
                g = hs.fresh_grads([SIZES[k][0]], SIZES[k][1], 3000 + 100 * seed + 10 * it + k)[0]
                gts[k].set_grads([g])
                grads[k] = g
                L.check(L.lib().eri_param_set_grad(handles[k], gts[k].ptr(gts[k].g[0])), "set_grad")
            else:
                L.check(L.lib().eri_param_set_grad(handles[k], None), "set_grad")
        skipped = C.c_uint32(99)
        L.check(L.lib().eri_adam8bit_step(opt, C.byref(skipped)), "step")
        assert skipped.value == n_par - len(live)
        step += 1
        assert L.lib().eri_adam8bit_get_step(opt) == step
        clip = np.float32(1.0)
        if live and max_norm > 0.0:
            norm, scale = C.c_float(), C.c_float()
            L.check(L.lib().eri_adam8bit_last_grad_norm(opt, C.byref(norm), C.byref(scale)), "last_grad_norm")
            sq = 0.0
            for k in live:
                g32 = onp.bf16_to_f32(grads[k]) if SIZES[k][1] else grads[k]
                sq += float(np.sum(g32.astype(np.float64) ** 2))
            assert abs(norm.value - np.sqrt(sq)) <= 2e-6 * np.sqrt(sq)
            clip = np.float32(scale.value)
            if norm.value > max_norm:
                assert clip == np.float32(max_norm) / (np.float32(norm.value) + np.float32(1e-6))
            else:
                assert clip == 1.0
        scaled = max_norm > 0.0 or global_scale != 1.0 or any(par_scale[k] != 1.0 for k in live)
        for k in live:
            if states[k] is None:
                states[k] = list(oc.state_init(SIZES[k][0]))
            gs = float(np.float32(global_scale * par_scale[k]) * clip) if scaled else None
            hs.oracle_step([ps[k]], [grads[k]], [states[k]], (lr, B1, B2, EPS, WD, step), SIZES[k][1], oc.MODE_ERI, gs)
        check_all("iteration %d" % it)
        if it == 6:  # checkpoint, then carry on in a fresh optimizer over the same parameters
            path = str(tmp_path / "sequence.safetensors")
            L.check(L.lib().eri_adam8bit_save_state(opt, path.encode()), "save_state")
            L.lib().eri_adam8bit_destroy(opt)
            opt = _new_optimizer(L, handles, 123.0)
            L.check(L.lib().eri_adam8bit_load_state(opt, path.encode()), "load_state")
            assert L.lib().eri_adam8bit_get_step(opt) == step and L.lib().eri_adam8bit_current_lr(opt) == lr
            L.check(L.lib().eri_adam8bit_set_grad_scale(opt, float(global_scale)), "set_grad_scale")
            for k in range(n_par):
                L.check(L.lib().eri_adam8bit_set_param_grad_scale(opt, k, float(par_scale[k])), "set_param_scale")
            L.check(L.lib().eri_adam8bit_set_max_grad_norm(opt, max_norm, 1e-6), "set_max_grad_norm")
            check_all("after reload")
    L.lib().eri_adam8bit_destroy(opt)
    for h in handles:
        L.lib().eri_param_release(h)
