"""Pins the oracle's 32-bit AdamW and EMA restatements."""
import numpy as np
import torch

import oracle_c as oc
from oracle import adam8_numpy as onp


def adamw(p, g, m, v, dtype, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, wd=0.01, master=None):
    oc.lib().eri_oracle_adamw32_step(oc.ptr(p), oc.ptr(g), oc.ptr(m), oc.ptr(v), m.size, dtype, lr, b1, b2, eps, wd,
                                     oc.ptr(master) if master is not None else None)


def test_reference_test_case_two_by_two_bf16_ones():
    # crates/common/optim/src/tests/adamw_step.rs:6-30: param = 1.0 (bf16, 2x2), grad = 1.0, one step
    # with lr 1e-3, betas (0.9, 0.999), eps 1e-8, wd 0.01; the reference asserts sum |delta| > 0
    one = onp.f32_to_bf16(np.ones(4, np.float32))
    p, g = one.copy(), one.copy()
    m, v = np.zeros(4, np.float32), np.zeros(4, np.float32)
    adamw(p, g, m, v, oc.DT_BF16)
    delta = np.abs(onp.bf16_to_f32(p) - 1.0).sum()
    assert delta > 0
    # closed form: m = 0.1, v = 0.001, update = 0.1/sqrt(0.001) = 3.1623, p = 1 - 1e-3*(3.1623 + 0.01) = 0.99683
    want = torch.tensor(1 - 1e-3 * (0.1 / np.sqrt(0.001) + 0.01)).to(torch.bfloat16).float().item()
    assert np.all(onp.bf16_to_f32(p) == np.float32(want))
    assert np.allclose(m, 0.1, rtol=1e-6) and np.allclose(v, 0.001, rtol=2e-5)


def test_adamw32_tracks_a_float64_recurrence_without_bias_correction():
    rng = np.random.default_rng(0)
    n = 5000
    p0 = rng.standard_normal(n).astype(np.float32)
    p = p0.copy()
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    P, M, V = p0.astype(np.float64), np.zeros(n), np.zeros(n)
    b1, b2 = float(np.float32(0.9)), float(np.float32(0.999))
    for t in range(30):
        g = (rng.standard_normal(n) * 1e-2).astype(np.float32)
        adamw(p, g, m, v, oc.DT_F32, lr=1e-3, wd=0.01)
        G = g.astype(np.float64)
        M = b1 * M + (1 - b1) * G
        V = b2 * V + (1 - b2) * G * G
        P = P - 1e-3 * (M / (np.sqrt(V) + 1e-8) + float(np.float32(0.01)) * P)
    assert np.allclose(p, P, rtol=0, atol=5e-6) and np.abs(P - p0).mean() > 1e-2
    assert np.allclose(m, M, rtol=1e-5, atol=1e-9) and np.allclose(v, V, rtol=1e-4, atol=1e-12)


def test_adamw32_zero_decay_leaves_no_decay_term():
    rng = np.random.default_rng(1)
    p0 = rng.standard_normal(64).astype(np.float32)
    g = np.zeros(64, np.float32)
    p = p0.copy()
    adamw(p, g, np.zeros(64, np.float32), np.zeros(64, np.float32), oc.DT_F32, wd=0.0)
    assert np.array_equal(p, p0)  # zero grad, zero state, no decay: 0/(0+eps) = 0
    p = p0.copy()
    adamw(p, g, np.zeros(64, np.float32), np.zeros(64, np.float32), oc.DT_F32, wd=0.5, lr=0.1)
    assert np.allclose(p, p0 * (1 - 0.05), rtol=1e-6)


def test_adamw32_master_copy_is_the_fp32_run_and_the_parameter_its_rounding():
    # mixed precision: bf16 parameter and gradient, fp32 master.  The master must follow, bit for bit, an
    # fp32 run fed the same (bf16-valued) gradients, and the bf16 parameter is the rounded master each step;
    # without the master the bf16 parameter drifts away from that run (updates below half an ulp are lost).
    rng = np.random.default_rng(5)
    n = 3000
    p32 = rng.standard_normal(n).astype(np.float32)
    master = p32.copy()
    p_mixed = onp.f32_to_bf16(p32)
    p_plain = p_mixed.copy()
    st = [[np.zeros(n, np.float32), np.zeros(n, np.float32)] for _ in range(3)]
    for t in range(40):
        g16 = onp.f32_to_bf16((rng.standard_normal(n) * 1e-2).astype(np.float32))
        adamw(p32, onp.bf16_to_f32(g16), *st[0], oc.DT_F32, lr=1e-4)
        adamw(p_mixed, g16, *st[1], oc.DT_BF16, lr=1e-4, master=master)
        adamw(p_plain, g16, *st[2], oc.DT_BF16, lr=1e-4)
        assert np.array_equal(master.view(np.uint32), p32.view(np.uint32))
        assert np.array_equal(p_mixed, onp.f32_to_bf16(master))
    assert np.array_equal(st[0][0], st[1][0]) and np.array_equal(st[0][1], st[1][1])
    drift_plain = np.abs(onp.bf16_to_f32(p_plain) - p32).mean()
    drift_mixed = np.abs(onp.bf16_to_f32(p_mixed) - p32).mean()
    assert drift_plain > 1.5 * drift_mixed


def test_ema_is_a_convex_combination():
    rng = np.random.default_rng(2)
    s0 = rng.standard_normal(1000).astype(np.float32)
    p = rng.standard_normal(1000).astype(np.float32)
    s = s0.copy()
    oc.lib().eri_oracle_ema_update(oc.ptr(s), oc.ptr(p), 1000, oc.DT_F32, 0.999)
    d = float(np.float32(0.999))
    assert np.allclose(s, d * s0.astype(np.float64) + (1 - d) * p, rtol=0, atol=3e-7)
    same = p.copy()
    oc.lib().eri_oracle_ema_update(oc.ptr(same), oc.ptr(p), 1000, oc.DT_F32, 0.5)
    assert np.array_equal(same, p)  # shadow == p is a fixed point when decay = 0.5 (exact halves)
    sb, pb = onp.f32_to_bf16(s0), onp.f32_to_bf16(p)
    oc.lib().eri_oracle_ema_update(oc.ptr(sb), oc.ptr(pb), 1000, oc.DT_BF16, 0.9)
    want = 0.9 * onp.bf16_to_f32(onp.f32_to_bf16(s0)).astype(np.float64) + 0.1 * onp.bf16_to_f32(pb)
    assert np.all(np.abs(onp.bf16_to_f32(sb) - want) <= np.abs(want) * 2 ** -8 + 1e-30)


def test_adamw32_with_the_bias_corrected_step_size_is_the_8bit_update_without_a_quantiser():
    """min_8bit_size sends short tensors to the 32-bit step with lr = the step size of Adam8bit::step.  That is
    the same update with fp32 moments: restated here in NumPy from adam8bit_enhanced.rs:252-275, one rounded
    operation per line, it must agree with the 32-bit oracle bit for bit over several steps, bf16 and fp32."""
    F = np.float32
    rng = np.random.default_rng(5)
    n = 3000
    for bf16 in (False, True):
        p32 = (rng.standard_normal(n) * 0.02).astype(F)
        p = onp.f32_to_bf16(p32) if bf16 else p32.copy()
        q = p.copy()
        m, v = np.zeros(n, F), np.zeros(n, F)
        mm, vv = np.zeros(n, F), np.zeros(n, F)
        for t in range(1, 6):
            g32 = (rng.standard_normal(n) * 1e-3).astype(F)
            g = onp.f32_to_bf16(g32) if bf16 else g32
            h = oc.hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, t)
            adamw(p, g, m, v, oc.DT_BF16 if bf16 else oc.DT_F32, lr=float(h.step_size), b1=0.9, b2=0.999, eps=1e-8, wd=0.01)
            gf = onp.bf16_to_f32(g) if bf16 else g
            qf = onp.bf16_to_f32(q) if bf16 else q
            mm = mm * F(h.beta1) + gf * F(h.omb1)            # :256
            vv = vv * F(h.beta2) + (gf * gf) * F(h.omb2)     # :259-260
            r = mm / (np.sqrt(vv) + F(h.eps))                # :263-264
            u = r + qf * F(h.weight_decay)                   # :267-271
            qn = (qf - u * F(h.step_size)).astype(F)         # :274-275
            q = onp.f32_to_bf16(qn) if bf16 else qn
            assert np.array_equal(m.view(np.uint32), mm.view(np.uint32)) and np.array_equal(v.view(np.uint32), vv.view(np.uint32))
            assert np.array_equal(p.view(np.uint16 if bf16 else np.uint32), q.view(np.uint16 if bf16 else np.uint32)), (bf16, t)


def test_adamw32_scaled_equals_the_unscaled_step_on_gradients_multiplied_beforehand():
    """The scale enters as one rounded fp32 product with the gradient and nowhere else: on fp32 tensors the
    scaled step equals the plain step on g * scale (formed in fp32), moments and parameters bit for bit, over
    several steps; on bf16 tensors the product is not rounded to bf16 in between, so it equals the fp32-gradient
    arithmetic and differs from the step on the bf16-rounded product; and a wrong place for the scale (after
    the square, or on the update) would fail the first comparison."""
    rng = np.random.default_rng(5)
    n, lr, b1, b2, eps, wd = 4099, 3e-4, 0.9, 0.999, 1e-8, 0.01
    scale = np.float32(0.37)
    p0 = (rng.standard_normal(n) * 0.05).astype(np.float32)
    pa, pb = p0.copy(), p0.copy()
    ma, va, mb, vb = (np.zeros(n, np.float32) for _ in range(4))
    for t in range(4):
        g = (rng.standard_normal(n) * 1e-2).astype(np.float32)
        oc.lib().eri_oracle_adamw32_step_scaled(oc.ptr(pa), oc.ptr(g), oc.ptr(ma), oc.ptr(va), n, oc.DT_F32, lr, b1, b2, eps, wd,
                                                None, float(scale))
        gs = (g * scale).astype(np.float32)
        adamw(pb, gs, mb, vb, oc.DT_F32, lr, b1, b2, eps, wd)
        assert np.array_equal(pa.view(np.uint32), pb.view(np.uint32))
        assert np.array_equal(ma.view(np.uint32), mb.view(np.uint32)) and np.array_equal(va.view(np.uint32), vb.view(np.uint32))
    # scale 1 is the plain step
    pc, mc, vc = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    pd, md, vd = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    g = (rng.standard_normal(n) * 1e-2).astype(np.float32)
    oc.lib().eri_oracle_adamw32_step_scaled(oc.ptr(pc), oc.ptr(g), oc.ptr(mc), oc.ptr(vc), n, oc.DT_F32, lr, b1, b2, eps, wd, None, 1.0)
    adamw(pd, g, md, vd, oc.DT_F32, lr, b1, b2, eps, wd)
    assert np.array_equal(pc.view(np.uint32), pd.view(np.uint32)) and np.array_equal(mc, md) and np.array_equal(vc, vd)
    # bf16: the product stays fp32 (first moment = (1 - b1) * (g * scale) exactly as fp32 arithmetic gives it)
    gb = onp.f32_to_bf16(g)
    pe = onp.f32_to_bf16(p0)
    me, ve = np.zeros(n, np.float32), np.zeros(n, np.float32)
    oc.lib().eri_oracle_adamw32_step_scaled(oc.ptr(pe), oc.ptr(gb), oc.ptr(me), oc.ptr(ve), n, oc.DT_BF16, lr, b1, b2, eps, wd,
                                            None, float(scale))
    want_m = (onp.bf16_to_f32(gb) * scale).astype(np.float32) * (np.float32(1.0) - np.float32(b1))
    assert np.array_equal(me.view(np.uint32), want_m.astype(np.float32).view(np.uint32))
    rounded = onp.bf16_to_f32(onp.f32_to_bf16((onp.bf16_to_f32(gb) * scale).astype(np.float32)))
    assert not np.array_equal(me, rounded * (np.float32(1.0) - np.float32(b1)))
