"""ERI_ADAM8_FLAG_EMA: the EMA of the parameters (src/trainers/ema_enhanced.rs:91-100) taken in the same call
as the step -- inside the prefetching kernel for large bf16 tables in mode ERI, as a sweep right behind the
step everywhere else.  Either way the shadows must equal the oracle's EMA of the oracle's new parameters,
bit for bit (exact flag), rows without a shadow must be left alone, and partial blocks must be covered."""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).to("cuda:0")


@pytest.mark.parametrize("case", ["bf16-in-the-step-kernel", "bf16-f32-grads-in-the-step-kernel", "bf16-small-table",
                                  "bf16-plain-kernel", "f32", "bf16-mode-bnb"])
def test_shadows_follow_the_updated_parameters(case):
    import torch
    from eridiffusion_amd import _lib as L
    bf16 = case != "f32"
    mode = L.MODE_BNB if case.endswith("bnb") else L.MODE_ERI
    extra = {"bf16-in-the-step-kernel": L.FLAG_ONE_WAVE, "bf16-f32-grads-in-the-step-kernel": L.FLAG_ONE_WAVE,
             "bf16-plain-kernel": L.FLAG_NO_PIPELINE}.get(case, 0)
    grad_f32 = "f32-grads" in case  # bf16 parameters whose gradients are fp32 and enter the arithmetic unrounded
    sizes = [2048 * 5 + 24, 2048 * 3, 77, 2048 * 2 + 1001, 640]
    has_shadow = [True, False, True, True, True]
    ps, gs = hs.make_inputs(sizes, bf16, 21)
    if grad_f32:
        gs = hs.fresh_grads(sizes, False, 299)
    states = hs.oracle_states(sizes)
    gt = hs.GpuTensors(ps, gs, states, bf16)
    rng = np.random.default_rng(4)
    shadows = []
    for n in sizes:
        x = (rng.standard_normal(n) * 0.02).astype(np.float32)
        shadows.append(onp.f32_to_bf16(x) if bf16 else x)
    sh_dev = [_dev(s) for s in shadows]
    rows = gt.rows()
    for r, d, yes in zip(rows, sh_dev, has_shadow):
        r.ema_shadow = d.data_ptr() if yes else None
        r.grad_f32 = 1 if grad_f32 else 0
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    decays = [0.5, 0.999, 0.9]
    all_g = [gs] + [hs.fresh_grads(sizes, bf16 and not grad_f32, 300 + k) for k in (1, 2)]
    for k, d in enumerate(decays):
        if k:
            gt.set_grads(all_g[k])
        h = L.hyper_pack(LR, B1, B2, EPS, WD, k + 1, mode, L.FLAG_EXACT_PARAM | L.FLAG_EMA | extra)
        h.ema_decay = d
        L.check(L.lib().eri_adam8_step_table(table, C.byref(h), None), "step_table")
        if grad_f32:
            ho = oc.hyper_pack(LR, B1, B2, EPS, WD, k + 1)
            for pa, ga, st in zip(ps, all_g[k], states):
                assert oc.step_tensor(pa, ga, *st, ho, hs.MAPS, oc.DT_BF16, 4, g_dtype=oc.DT_F32) == 0
        else:
            hs.oracle_step(ps, all_g[k], states, (LR, B1, B2, EPS, WD, k + 1), bf16, oc.MODE_BNB if mode == L.MODE_BNB else oc.MODE_ERI)
        for i, n in enumerate(sizes):
            if has_shadow[i]:
                oc.lib().eri_oracle_ema_update(oc.ptr(shadows[i]), oc.ptr(ps[i]), n, oc.DT_BF16 if bf16 else oc.DT_F32, d)
    torch.cuda.synchronize()
    got_p, got_st = gt.fetch()
    stats = hs.compare(got_p, got_st, ps, states, bf16, True, case)
    assert stats["code_mismatch"] == 0
    bits = np.uint16 if bf16 else np.uint32
    for i in range(len(sizes)):
        assert np.array_equal(sh_dev[i].cpu().numpy().view(bits), shadows[i].view(bits)), (case, i)
    # a decay outside [0, 1] is refused before anything runs
    h.ema_decay = 1.5
    assert L.lib().eri_adam8_step_table(table, C.byref(h), None) == -6
    L.lib().eri_adam8_table_destroy(table)


def test_attached_ema_model_equals_step_then_update():
    """Two identical trainers: one calls optimizer.step() and then ema.update(all parameters), as the reference's
    trainers do, the other attaches the EMA model to the optimizer and only calls step().  Parameters, states
    and shadows must agree bit for bit after every step.  The parameter set has bf16 and fp32 tensors, one
    tensor below min_8bit_size, and a tensor that has no gradient in some steps."""
    import torch
    from eridiffusion_amd import _lib as L
    sizes = [2048 * 4 + 40, 300, 2048 * 2, 5000, 2048 * 6 + 8]
    bf = [True, True, False, True, True]
    names = [b"a.w", b"a.b", b"b.w", b"c.w", b"d.w"]
    trainers = []
    for which in range(2):
        handles = (C.c_void_p * len(sizes))()
        datas = []
        for i, (n, bf16) in enumerate(zip(sizes, bf)):
            ps, _ = hs.make_inputs([n], bf16, 50 + i)
            datas.append(_dev(ps[0]))
            h = C.c_void_p()
            L.check(L.lib().eri_param_create(datas[i].data_ptr(), n, 2 if bf16 else 0, C.byref(h)), "param_create")
            handles[i] = h
        cfg = L.Adam8bitConfigC(1e-4, B1, B2, EPS, WD, 0, 1, 100)
        opt, ema = C.c_void_p(), C.c_void_p()
        L.check(L.lib().eri_adam8bit_new(handles, len(sizes), C.byref(cfg), None, C.byref(opt)), "new")
        L.check(L.lib().eri_adam8bit_set_min_8bit_size(opt, 1024), "min_8bit")
        L.check(L.lib().eri_ema_new(0.99, 1, 1.0, None, C.byref(ema)), "ema_new")
        trainers.append((opt, ema, handles, datas))
    c_names = (C.c_char_p * len(sizes))(*names)
    L.check(L.lib().eri_adam8bit_attach_ema(trainers[1][0], trainers[1][1], c_names, len(sizes)), "attach_ema")
    assert L.lib().eri_adam8bit_attach_ema(trainers[1][0], trainers[1][1], c_names, 2) == -6
    keep = []
    for step in range(4):
        grads = [_dev(hs.fresh_grads([n], bf16, 1000 * step + i)[0]) for i, (n, bf16) in enumerate(zip(sizes, bf))]
        keep.append(grads)
        for which, (opt, ema, handles, datas) in enumerate(trainers):
            for i in range(len(sizes)):
                no_grad = i == 3 and step in (1, 2)
                L.check(L.lib().eri_param_set_grad(handles[i], None if no_grad else grads[i].data_ptr()), "set_grad")
            L.check(L.lib().eri_adam8bit_step(opt, None), "step")
            if which == 0:
                L.check(L.lib().eri_ema_update(ema, c_names, handles, len(sizes)), "ema_update")
        torch.cuda.synchronize()
        assert L.lib().eri_ema_step(trainers[0][1]) == L.lib().eri_ema_step(trainers[1][1]) == step + 1
        for i, n in enumerate(sizes):
            assert torch.equal(trainers[0][3][i], trainers[1][3][i]), (step, i)
            got = []
            for _, ema, _, _ in trainers:
                ptr, numel, tag = C.c_void_p(), C.c_uint64(), C.c_int()
                L.check(L.lib().eri_ema_shadow(ema, names[i], C.byref(ptr), C.byref(numel), C.byref(tag)), "ema_shadow")
                out = torch.empty(n * (2 if bf[i] else 4), dtype=torch.uint8, device="cuda:0")
                L.check(L.lib().eri_hip_memcpy_async(out.data_ptr(), ptr.value, out.numel(), 3, None), "memcpy")
                got.append(out)
            torch.cuda.synchronize()
            assert torch.equal(got[0], got[1]), (step, i)
    for opt, ema, handles, _ in trainers:
        L.lib().eri_adam8bit_destroy(opt)
        L.lib().eri_ema_destroy(ema)
        for h in handles:
            L.lib().eri_param_release(h)
