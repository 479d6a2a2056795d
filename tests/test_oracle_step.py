"""Pins the oracle's step: closed forms, torch.optim.Adam, brute-force block maxima, and bit-for-bit
agreement of the two independent restatements (scalar C and vectorised NumPy)."""
import math

import numpy as np
import pytest
import torch

import oracle_c as oc
from oracle import adam8_numpy as onp

MAPS = oc.load_maps()
LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01


def run_c(p, g, state, t, dtype=oc.DT_F32, mode=oc.MODE_ERI, lr=LR, wd=WD, eps=EPS, threads=1, gs=None):
    h = oc.hyper_pack(lr, B1, B2, eps, wd, t, mode, gs)
    rc = oc.step_tensor(p, g, *state, h, MAPS, dtype, threads)
    assert rc == 0
    return h


def test_hyper_pack_cast_points():
    h = oc.hyper_pack(LR, B1, B2, EPS, WD, 1)
    # `1.0 - beta as f32` is an fp32 subtraction: not the fp32 nearest of 0.1 / 0.001
    assert h.omb1 == np.float32(1) - np.float32(0.9) and h.omb1 != np.float32(0.1)
    assert h.omb2 == np.float32(1) - np.float32(0.999) and h.omb2 != np.float32(0.001)
    # t = 1: lr * sqrt(1 - b2) / (1 - b1)
    assert h.step_size == np.float32(LR * math.sqrt(1 - B2) / (1 - B1))
    h7 = oc.hyper_pack(LR, B1, B2, EPS, WD, 7)
    assert h7.step_size == np.float32(LR * math.sqrt(1 - B2 ** 7) / (1 - B1 ** 7))
    n = onp.hyper_pack(LR, B1, B2, EPS, WD, 7)
    assert (h7.step_size, h7.omb1, h7.omb2, h7.beta1, h7.beta2, h7.eps, h7.weight_decay) == \
        (n["step_size"], n["omb1"], n["omb2"], n["beta1"], n["beta2"], n["eps"], n["wd"])
    # functional flavour: f64 subtraction then cast, s = max(step, 1)
    l0 = oc.hyper_pack(LR, B1, B2, EPS, WD, 0, oc.MODE_L2)
    l1 = oc.hyper_pack(LR, B1, B2, EPS, WD, 1, oc.MODE_L2)
    assert l0.omb1 == np.float32(0.1) and l0.omb2 == np.float32(1.0 - 0.999)
    assert (l0.bc1, l0.bc2) == (l1.bc1, l1.bc2) == (np.float32(1 - B1), np.float32(1 - B2))
    assert l0.step_size == np.float32(LR)


def test_zero_grad_zero_state_is_pure_decay():
    n = 2048 + 100
    rng = np.random.default_rng(0)
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    p = p0.copy()
    g = np.zeros(n, np.float32)
    st = oc.state_init(n)
    h = run_c(p, g, st, 1)
    want = p0 - (p0 * np.float32(WD)) * np.float32(h.step_size)
    assert np.array_equal(p, want)
    assert np.all(st[0] == 127) and np.all(st[1] == 0) and np.all(st[2] == 0) and np.all(st[3] == 0)


def test_first_step_is_sign_descent():
    # from a zero state, m = (1-b1) g and v = (1-b2) g^2, so with wd = 0 the step is
    # lr * g / (|g| + eps / sqrt(1 - b2)): the textbook first Adam step
    n = 4096
    rng = np.random.default_rng(1)
    p0 = rng.standard_normal(n).astype(np.float32)
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    p = p0.copy()
    st = oc.state_init(n)
    run_c(p, g, st, 1, wd=0.0)
    g64 = g.astype(np.float64)
    want = p0 - LR * g64 / (np.abs(g64) + EPS / math.sqrt(1 - B2))
    assert np.allclose(p, want, rtol=0, atol=2e-7 * LR + 1e-7 * np.abs(p0).max())
    # block maxima of the fresh moments, by brute force
    m64 = (1 - B1) * g64
    v64 = (1 - B2) * g64 ** 2
    for b in range(2):
        seg = slice(b * 2048, (b + 1) * 2048)
        assert np.isclose(st[2][b], np.abs(m64[seg]).max(), rtol=1e-6)
        assert np.isclose(st[3][b], v64[seg].max(), rtol=1e-6)
        # the element holding the block maximum quantises to +-full scale
        i = np.argmax(np.abs(m64[seg]))
        assert st[0][seg][i] in (0, 255)
        assert st[1][seg][np.argmax(v64[seg])] == 255


def test_matches_torch_adam_when_quantisation_is_exact():
    # one positive gradient value per block and step keeps m/absmax = v/absmax = 1.0, an exact map
    # entry, so the 8-bit state carries the moments without loss and 60 steps must track
    # torch.optim.Adam.  Adam puts eps outside the bias correction: eps_here = eps_adam*sqrt(bc2).
    n = 3 * 2048
    rng = np.random.default_rng(2)
    p0 = rng.standard_normal(n).astype(np.float32)
    p = p0.copy()
    st = oc.state_init(n)
    tp = torch.tensor(p0.astype(np.float64), requires_grad=True)
    opt = torch.optim.Adam([tp], lr=1e-2, betas=(B1, B2), eps=1e-8)
    for t in range(1, 61):
        per_block = 10.0 ** rng.uniform(-4, -2, 3)
        g = np.repeat(per_block, 2048).astype(np.float32)
        run_c(p, g, st, t, lr=1e-2, wd=0.0, eps=1e-8 * math.sqrt(1 - B2 ** t))
        tp.grad = torch.tensor(g.astype(np.float64))
        opt.step()
        assert np.all(st[0] == 255) and np.all(st[1] == 255)
    # The reference feeds fp32-rounded betas to the moment updates (1 - (float)0.999 = 0.0009999871)
    # but f64 betas to the bias correction, a 1.3e-5 relative mismatch in v, 6.5e-6 in the step.
    # Over a total movement of 60 * 1e-2 that allows ~4e-6; a dropped term or sign shows as >1e-2.
    moved = np.abs(tp.detach().numpy() - p0)
    assert moved.min() > 0.3
    assert np.allclose(p, tp.detach().numpy(), rtol=0, atol=8e-6)


def test_decoupled_decay_is_scaled_by_the_bias_corrected_step():
    n = 2048
    rng = np.random.default_rng(3)
    p0 = rng.standard_normal(n).astype(np.float32)
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    pa, pb = p0.copy(), p0.copy()
    ha = run_c(pa, g, oc.state_init(n), 5, wd=0.0)
    run_c(pb, g, oc.state_init(n), 5, wd=0.1)
    # p_b - p_a = -(wd * p) * step_size up to the rounding of the sum
    want = -(0.1 * p0.astype(np.float64)) * float(ha.step_size)
    assert np.allclose(pb.astype(np.float64) - pa, want, rtol=0, atol=6e-7)  # two fp32 roundings near |p| ~ 3


@pytest.mark.parametrize("n", [1, 7, 320, 2047, 2048, 2049, 5 * 2048 + 321])
def test_partial_blocks_absmax_and_untouched_tail(n):
    rng = np.random.default_rng(n)
    pad = 64
    p = (rng.standard_normal(n + pad) * 0.02).astype(np.float32)
    g = (rng.standard_normal(n + pad) * 1e-3).astype(np.float32)
    m = np.full(n + pad, 77, np.uint8)
    v = np.full(n + pad, 99, np.uint8)
    m[:n], v[:n] = 127, 0
    nb = (n + 2047) // 2048
    am = np.zeros(nb + 1, np.float32)
    av = np.zeros(nb + 1, np.float32)
    am[nb] = av[nb] = -5.0
    p_before = p.copy()
    h = oc.hyper_pack(LR, B1, B2, EPS, WD, 1)
    rc = oc.lib().eri_oracle_step_tensor(oc.ptr(p), oc.ptr(g), oc.ptr(m), oc.ptr(v), oc.ptr(am), oc.ptr(av), n,
                                         oc.DT_F32, oc.C.byref(h), oc.ptr(MAPS[0]), oc.ptr(MAPS[1]), 1)
    assert rc == 0
    assert np.array_equal(p[n:], p_before[n:]) and np.all(m[n:] == 77) and np.all(v[n:] == 99)
    assert am[nb] == -5.0 and av[nb] == -5.0
    omb1 = np.float32(1) - np.float32(B1)
    omb2 = np.float32(1) - np.float32(B2)
    mm = np.abs(g[:n] * omb1)
    vv = (g[:n] * g[:n]) * omb2
    for b in range(nb):
        seg = slice(b * 2048, min((b + 1) * 2048, n))
        assert am[b] == mm[seg].max() and av[b] == vv[seg].max()
    # block maxima do not depend on the order of the elements
    perm = rng.permutation(min(n, 2048))
    p2 = p_before.copy()
    g2 = g.copy()
    g2[:perm.size] = g[:perm.size][perm]
    st2 = oc.state_init(n)
    run_c(p2[:n].copy(), g2[:n].copy(), st2, 1)
    assert st2[2][0] == am[0] and st2[3][0] == av[0]


def test_empty_tensor_is_refused():
    z = np.zeros(1, np.float32)
    zb = np.zeros(1, np.uint8)
    h = oc.hyper_pack(LR, B1, B2, EPS, WD, 1)
    rc = oc.lib().eri_oracle_step_tensor(oc.ptr(z), oc.ptr(z), oc.ptr(zb), oc.ptr(zb), oc.ptr(z), oc.ptr(z), 0,
                                         oc.DT_F32, oc.C.byref(h), oc.ptr(MAPS[0]), oc.ptr(MAPS[1]), 1)
    assert rc == -1
    with pytest.raises(ValueError):
        onp.step_tensor(z[:0], z[:0], zb[:0], zb[:0], z[:0], z[:0], onp.hyper_pack(LR, B1, B2, EPS, WD, 1), *MAPS)


def _agree(n, bf16, mode, steps, seed, p_std, g_std, wd=WD, threads=1):
    rng = np.random.default_rng(seed)
    p32 = (rng.standard_normal(n) * p_std).astype(np.float32)
    if bf16:
        p_c = onp.f32_to_bf16(p32)
    else:
        p_c = p32.copy()
    p_n = p_c.copy()
    st_c = oc.state_init(n)
    st_n = onp.state_init(n)
    for t in range(1, steps + 1):
        g32 = (rng.standard_normal(n) * g_std).astype(np.float32)
        g = onp.f32_to_bf16(g32) if bf16 else g32
        step = t - 1 if mode == oc.MODE_L2 else t
        run_c(p_c, g, st_c, step, oc.DT_BF16 if bf16 else oc.DT_F32, mode, wd=wd, threads=threads)
        hn = onp.hyper_pack(LR, B1, B2, EPS, wd, step, {oc.MODE_ERI: "eri", oc.MODE_L2: "l2", oc.MODE_BNB: "bnb"}[mode])
        p_n, *st_n = onp.step_tensor(p_n, g, *st_n, hn, *MAPS, bf16=bf16)
        assert np.array_equal(p_c.view(np.uint16 if bf16 else np.uint32), p_n.view(np.uint16 if bf16 else np.uint32)), t
        for a, b in zip(st_c, st_n):
            assert np.array_equal(a.view(np.uint8), np.asarray(b).view(np.uint8)), t
    return p_c, st_c


def test_two_restatements_agree_config1_fp32_eleven_steps():
    # configuration 1: 2**20 fp32 params ~N(0, 0.02), grads ~N(0, 1e-3), ten prior steps + one
    p, st = _agree(1 << 20, False, oc.MODE_ERI, 11, 0xE21D + 1, 0.02, 1e-3, threads=4)
    assert st[2].min() > 0 and len(np.unique(st[0])) > 100 and len(np.unique(st[1])) > 100


@pytest.mark.parametrize("mode", [oc.MODE_ERI, oc.MODE_L2, oc.MODE_BNB])
@pytest.mark.parametrize("bf16", [False, True])
def test_two_restatements_agree_ragged(mode, bf16):
    _agree(7 * 2048 + 1234, bf16, mode, 6, 17 + mode + 2 * bf16, 0.02, 1e-3)


def test_two_restatements_agree_lora_scales_bf16():
    # LoRA-B-like tensor: params ~1e-4, grads ~1e-4, updates of the same size as the params
    _agree(16 * 5120 + 77, True, oc.MODE_ERI, 8, 23, 1e-4, 1e-4)
    _agree(4, True, oc.MODE_ERI, 3, 24, 0.02, 1e-3)


def test_threads_do_not_change_results():
    n = 40 * 2048 + 5
    rng = np.random.default_rng(31)
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    outs = []
    for th in (1, 3, 8):
        p = p0.copy()
        st = oc.state_init(n)
        run_c(p, g, st, 1, threads=th)
        run_c(p, g, st, 2, threads=th)
        outs.append((p, *st))
    for o in outs[1:]:
        for a, b in zip(outs[0], o):
            assert np.array_equal(a, b)


def test_grad_scale_equals_prescaled_gradient():
    n = 2048 + 9
    rng = np.random.default_rng(41)
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    pa, pb = p0.copy(), p0.copy()
    sa, sb = oc.state_init(n), oc.state_init(n)
    run_c(pa, g, sa, 1, gs=0.25)
    run_c(pb, (g * np.float32(0.25)).astype(np.float32), sb, 1)
    assert np.array_equal(pa, pb)
    for a, b in zip(sa, sb):
        assert np.array_equal(a, b)


def test_l2_mode_first_call_follows_the_functional_update():
    # adam8bit.rs:101-208 with step = 0: g' = g + wd p, m = 0.1 g', v = 0.001 g'^2, both divided by
    # (1 - beta), so the update is lr * g' / (|g'| + eps)
    n = 2048
    rng = np.random.default_rng(51)
    p0 = rng.standard_normal(n).astype(np.float32)
    g = (rng.standard_normal(n) * 1e-2).astype(np.float32)
    p = p0.copy()
    run_c(p, g, oc.state_init(n), 0, mode=oc.MODE_L2)
    g2 = g.astype(np.float64) + WD * p0.astype(np.float64)
    want = p0 - LR * g2 / (np.abs(g2) + EPS)
    assert np.allclose(p, want, rtol=0, atol=6e-7)  # two fp32 roundings near |p| ~ 3


@pytest.mark.parametrize("step", [2, 7, 40])
def test_l2_mode_bias_correction_at_later_steps(step):
    """adam8bit.rs:164-187 beyond the first call: s = max(step, 1), m_hat = m / (1 - b1^s), v_hat = v / (1 - b2^s).
    From a zero state one call gives m = (1-b1) g', v = (1-b2) g'^2, so the update has the closed form
    lr * g' * [(1-b1)/(1-b1^s)] / (|g'| * sqrt((1-b2)/(1-b2^s)) + eps); a bias correction that took the wrong
    exponent (s-1, s+1, or the other beta) is off by percents, far outside the tolerance."""
    n = 2048
    rng = np.random.default_rng(60 + step)
    p0 = rng.standard_normal(n).astype(np.float32)
    g = (rng.standard_normal(n) * 1e-2).astype(np.float32)
    h = oc.hyper_pack(LR, 0.9, 0.999, EPS, WD, step, oc.MODE_L2)
    assert h.bc1 == np.float32(1.0 - 0.9 ** step) and h.bc2 == np.float32(1.0 - 0.999 ** step)
    assert h.omb1 == np.float32(1.0 - 0.9) and h.step_size == np.float32(LR)
    p = p0.copy()
    run_c(p, g, oc.state_init(n), step, mode=oc.MODE_L2)
    g2 = g.astype(np.float64) + WD * p0.astype(np.float64)
    c1 = (1 - 0.9) / (1 - 0.9 ** step)
    c2 = np.sqrt((1 - 0.999) / (1 - 0.999 ** step))
    want = p0 - LR * g2 * c1 / (np.abs(g2) * c2 + EPS)
    assert np.allclose(p, want, rtol=0, atol=6e-7)
    for wrong in (step - 1, step + 1):
        w1 = (1 - 0.9) / (1 - 0.9 ** wrong)
        w2 = np.sqrt((1 - 0.999) / (1 - 0.999 ** wrong))
        assert not np.allclose(p, p0 - LR * g2 * w1 / (np.abs(g2) * w2 + EPS), rtol=0, atol=6e-7)
    # the NumPy restatement agrees bit for bit
    hn = onp.hyper_pack(LR, 0.9, 0.999, EPS, WD, step, "l2")
    q = onp.step_tensor(p0, g, *onp.state_init(n), hn, *oc.load_maps())[0]
    assert np.array_equal(q.view(np.uint32), p.view(np.uint32))


# ---- mode BNB: eps under the bias correction, decay as a factor, sign of the first moment kept ----

def test_bnb_scalars():
    t = 7
    h = oc.hyper_pack(LR, B1, B2, EPS, WD, t, oc.MODE_BNB)
    e = oc.hyper_pack(LR, B1, B2, EPS, WD, t, oc.MODE_ERI)
    assert h.step_size == e.step_size and h.omb1 == e.omb1 and h.omb2 == e.omb2
    assert h.eps == np.float32(EPS * math.sqrt(1 - B2 ** t))
    assert h.weight_decay == np.float32(1.0 - LR * WD) and h.weight_decay < 1
    assert oc.hyper_pack(LR, B1, B2, EPS, 0.0, t, oc.MODE_BNB).weight_decay == 1.0


def test_bnb_is_torch_adam_without_decay():
    # with eps riding on sqrt(bc2) the update is lr/bc1 * m / (sqrt(v/bc2) + eps): Adam itself.  Same
    # exactly-quantisable gradients as the ERI test above, and no eps adjustment this time.
    n = 3 * 2048
    rng = np.random.default_rng(2)
    p0 = rng.standard_normal(n).astype(np.float32)
    p = p0.copy()
    st = oc.state_init(n)
    tp = torch.tensor(p0.astype(np.float64), requires_grad=True)
    opt = torch.optim.Adam([tp], lr=1e-2, betas=(B1, B2), eps=1e-8)
    for t in range(1, 61):
        per_block = 10.0 ** rng.uniform(-4, -2, 3)
        g = np.repeat(per_block, 2048).astype(np.float32)
        run_c(p, g, st, t, mode=oc.MODE_BNB, lr=1e-2, wd=0.0, eps=1e-8)
        tp.grad = torch.tensor(g.astype(np.float64))
        opt.step()
    assert np.abs(tp.detach().numpy() - p0).min() > 0.3
    assert np.allclose(p, tp.detach().numpy(), rtol=0, atol=8e-6)  # fp32-rounded betas, as in the ERI test


def test_bnb_decay_is_a_factor_applied_after_the_adam_term():
    n = 2048
    rng = np.random.default_rng(61)
    p0 = rng.standard_normal(n).astype(np.float32)
    # zero gradient, zero state: the Adam term is 0 / (0 + eps) = 0 and only the factor remains
    p = p0.copy()
    run_c(p, np.zeros(n, np.float32), oc.state_init(n), 1, mode=oc.MODE_BNB, lr=1e-2, wd=0.5)
    assert np.array_equal(p, p0 * np.float32(1.0 - 1e-2 * 0.5))
    # with a gradient: (p - adam) * factor, where "p - adam" is what wd = 0 gives
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    pa, pb = p0.copy(), p0.copy()
    run_c(pa, g, oc.state_init(n), 3, mode=oc.MODE_BNB, lr=1e-2, wd=0.0)
    run_c(pb, g, oc.state_init(n), 3, mode=oc.MODE_BNB, lr=1e-2, wd=0.5)
    assert np.array_equal(pb, pa * np.float32(1.0 - 1e-2 * 0.5))
    assert not np.array_equal(pa, pb)


def test_bnb_first_moment_keeps_its_sign():
    # one element sets the block's scale; moments 1e-9 of it round to the zero entry (the smallest
    # non-zero map value is 5.5e-7).  ERI stores 127 for both signs; BNB stores 126 for the negative one.
    n = 2048
    g = np.zeros(n, np.float32)
    g[0] = 1.0
    g[1], g[2] = 1e-9, -1e-9
    g[3], g[4] = 1e-3, -1e-3
    codes = {}
    for mode in (oc.MODE_ERI, oc.MODE_BNB):
        st = oc.state_init(n)
        run_c(np.zeros(n, np.float32), g, st, 1, mode=mode, wd=0.0)
        codes[mode] = st[0].copy()
        assert st[0][0] == 255 and st[1][0] == 255
    assert codes[oc.MODE_ERI][1] == 127 and codes[oc.MODE_ERI][2] == 127
    assert codes[oc.MODE_BNB][1] == 127 and codes[oc.MODE_BNB][2] == 126
    # everything else is untouched by the rule, zeros included
    rest = np.ones(n, bool)
    rest[2] = False
    assert np.array_equal(codes[oc.MODE_ERI][rest], codes[oc.MODE_BNB][rest])
    assert MAPS[0][126] < 0 and MAPS[0][127] == 0 and MAPS[0][codes[oc.MODE_BNB][4]] < 0 < MAPS[0][codes[oc.MODE_BNB][3]]
    # a block of zeros keeps the codes of zero
    st = oc.state_init(n)
    run_c(np.ones(n, np.float32), np.zeros(n, np.float32), st, 1, mode=oc.MODE_BNB)
    assert np.all(st[0] == 127) and np.all(st[1] == 0) and st[2][0] == 0


def test_two_restatements_agree_on_randomized_cases_with_extreme_values():
    """Thirty seeded random cases: sizes, dtype, mode, decay, gradient scale, magnitudes from 1e-30 to
    1e30, exact zeros, and (in some cases) NaN and infinite gradients.  The scalar C and the vectorised
    NumPy restatements must produce the same bits; NaN parameters are compared as NaN."""
    rng = np.random.default_rng(424242)
    modes = [(oc.MODE_ERI, "eri"), (oc.MODE_L2, "l2"), (oc.MODE_BNB, "bnb")]
    for case in range(30):
        n = int(rng.choice([1, 5, 2047, 2048, 2049, 5000, 3 * 2048 + 17]))
        bf16 = bool(rng.integers(0, 2))
        cmode, nmode = modes[int(rng.integers(0, 3))]
        wd = float(rng.choice([0.0, 0.01, 0.3]))
        gs = None if rng.random() < 0.5 else float(rng.uniform(0.05, 3.0))
        mag_p = 10.0 ** rng.uniform(-6, 3)
        mag_g = 10.0 ** rng.uniform(-30, 30) if rng.random() < 0.3 else 10.0 ** rng.uniform(-6, 0)
        p32 = (rng.standard_normal(n) * mag_p).astype(np.float32)
        p_c = onp.f32_to_bf16(p32) if bf16 else p32.copy()
        p_n = p_c.copy()
        st_c, st_n = oc.state_init(n), onp.state_init(n)
        for t in range(1, 4):
            with np.errstate(over="ignore"):
                g32 = (rng.standard_normal(n) * mag_g).astype(np.float32)
            g32[rng.random(n) < 0.05] = 0.0
            if case % 5 == 4 and n > 4:
                g32[int(rng.integers(0, n))] = np.nan
                g32[int(rng.integers(0, n))] = np.inf
                g32[int(rng.integers(0, n))] = -np.inf
            g = onp.f32_to_bf16(g32) if bf16 else g32
            step = t - 1 if cmode == oc.MODE_L2 else t
            run_c(p_c, g, st_c, step, oc.DT_BF16 if bf16 else oc.DT_F32, cmode, wd=wd, gs=gs)
            hn = onp.hyper_pack(LR, B1, B2, EPS, wd, step, nmode)
            if gs is not None:
                hn["grad_scale"] = gs
            p_n, *st_n = onp.step_tensor(p_n, g, *st_n, hn, *MAPS, bf16=bf16)
            fc = onp.bf16_to_f32(p_c) if bf16 else p_c
            fn = onp.bf16_to_f32(p_n) if bf16 else p_n
            both_nan = np.isnan(fc) & np.isnan(fn)
            raw_c = p_c.view(np.uint16 if bf16 else np.uint32)
            raw_n = p_n.view(np.uint16 if bf16 else np.uint32)
            assert np.array_equal(raw_c[~both_nan], raw_n[~both_nan]), (case, t)
            for k, (a, b) in enumerate(zip(st_c, st_n)):
                a, b = np.asarray(a), np.asarray(b)
                if k >= 2:  # absmax: NaN never enters (fmaxf ignores it), inf may
                    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (case, t, k)
                else:
                    assert np.array_equal(a, b), (case, t, k)


@pytest.mark.parametrize("mode", [oc.MODE_ERI, oc.MODE_L2, oc.MODE_BNB])
def test_f32_gradient_for_bf16_parameters_is_used_unrounded(mode):
    """The storage type of the gradient (adam8bit_enhanced.rs:231-235: cast to F32, never rounded).
    Pinned three ways: (1) a float32 gradient whose values are bf16 values gives exactly what the same
    values stored as bf16 give -- the storage type alone changes nothing; (2) a float32 gradient with low
    mantissa bits set gives what float32 *parameters* holding the same bf16 values give for the moments
    (the moments of the modes ERI and BNB depend on the gradient only), i.e. no rounding happened on the
    way in; (3) the C and NumPy restatements agree bit for bit."""
    n = 3 * 2048 + 321
    rng = np.random.default_rng(77 + mode)
    p16 = onp.f32_to_bf16((rng.standard_normal(n) * 0.02).astype(np.float32))
    g32 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    assert (g32.view(np.uint32) & 0xFFFF).any()
    step = 0 if mode == oc.MODE_L2 else 1
    h = oc.hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, step, mode)
    maps = oc.load_maps()

    def run(p, g, dtype, g_dtype):
        p = p.copy()
        st = list(oc.state_init(n))
        assert oc.step_tensor(p, g, *st, h, maps, dtype, 2, g_dtype=g_dtype) == 0
        return p, st

    # (1)
    g16 = onp.f32_to_bf16(g32)
    a_p, a_st = run(p16, g16, oc.DT_BF16, oc.DT_BF16)
    b_p, b_st = run(p16, onp.bf16_to_f32(g16), oc.DT_BF16, oc.DT_F32)
    assert np.array_equal(a_p, b_p) and all(np.array_equal(x.view(np.uint8), y.view(np.uint8)) for x, y in zip(a_st, b_st))
    # (2)
    c_p, c_st = run(p16, g32, oc.DT_BF16, oc.DT_F32)
    assert not all(np.array_equal(x.view(np.uint8), y.view(np.uint8)) for x, y in zip(a_st, c_st))  # rounding first differs
    if mode != oc.MODE_L2:  # (in mode L2 the decay enters the gradient, and with it the parameter's dtype does not matter either)
        d_p, d_st = run(onp.bf16_to_f32(p16), g32, oc.DT_F32, oc.DT_F32)
        assert all(np.array_equal(x.view(np.uint8), y.view(np.uint8)) for x, y in zip(c_st, d_st))
        assert np.array_equal(c_p, onp.f32_to_bf16(d_p))  # one parameter update from the same fp32 values, rounded once
    # (3)
    modes = {oc.MODE_ERI: "eri", oc.MODE_L2: "l2", oc.MODE_BNB: "bnb"}
    hn = onp.hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, step, modes[mode])
    st0 = onp.state_init(n)
    n_p, n_m, n_v, n_am, n_av = onp.step_tensor(p16, g32, *st0, hn, *maps, bf16=True, grad_bf16=False)
    assert np.array_equal(n_p, c_p) and np.array_equal(n_m, c_st[0]) and np.array_equal(n_v, c_st[1])
    assert np.array_equal(n_am.view(np.uint32), c_st[2].view(np.uint32)) and np.array_equal(n_av.view(np.uint32), c_st[3].view(np.uint32))
