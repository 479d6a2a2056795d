"""GPU parity: the HIP step, called through the C ABI, against the CPU oracle on the same inputs.

The bar, written out: absmax bit-exact; state codes bit-exact (any +-1 neighbour is counted, and
the counts are asserted to be zero here because the kernel and the oracle share the tie rule);
fp32 parameters bit-exact; bf16 parameters bit-exact with ERI_ADAM8_FLAG_EXACT_PARAM and within
one bf16 ulp (counted) on the default approximate square root / reciprocal path.
"""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu

LR, B1, B2, EPS, WD = 1e-4, 0.9, 0.999, 1e-8, 0.01


@pytest.fixture(autouse=True, params=["split-kernel-for-small-tables", "prefetching-kernels", "plain-kernels"])
def which_kernels(request):
    """The tables of these tests are small, so by default they all run on the four-waves-per-block kernel.
    Every test therefore runs three times: as shipped, on the one-wave-per-block kernels that prefetch the
    next block (what the largest tables take), and on the one-wave kernels without the prefetch (mid-size
    tables)."""
    global KERNEL_FLAGS
    L = _lib()
    KERNEL_FLAGS = {"split": 0, "prefe": L.FLAG_ONE_WAVE, "plain": L.FLAG_NO_PIPELINE}[request.param[:5]]
    yield request.param
    KERNEL_FLAGS = 0


KERNEL_FLAGS = 0


def _lib():
    from eridiffusion_amd import _lib
    return _lib


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _sync():
    import torch
    torch.cuda.synchronize()


def gpu_steps(gt, steps_grads, first_step, mode=0, flags=0, wd=WD, lr=LR, grad_scale=None, tensor_scales=None,
              use_multi=False):
    """Runs len(steps_grads) steps on the device; the first uses the gradients already uploaded."""
    L = _lib()
    rows = gt.rows(tensor_scales)
    table = C.c_void_p()
    if not use_multi:
        L.check(L.lib().eri_adam8_table_create(rows, len(rows), _stream(), C.byref(table)), "table_create")
    for k, gs in enumerate(steps_grads):
        if gs is not None:
            gt.set_grads(gs)
        step = first_step + k
        h = L.hyper_pack(lr, B1, B2, EPS, wd, step - 1 if mode == 1 else step, mode, flags | KERNEL_FLAGS, grad_scale)
        if use_multi:
            L.check(L.lib().eri_adam8_step_multi(rows, len(rows), C.byref(h), _stream()), "step_multi")
        else:
            L.check(L.lib().eri_adam8_step_table(table, C.byref(h), _stream()), "step_table")
    _sync()
    if not use_multi:
        L.lib().eri_adam8_table_destroy(table)


def check_steps(gt, ps, states, all_g, first_step, mode, flags, wd, bf16, grad_scale=None, use_multi=False, label=""):
    """Runs len(all_g) steps on the device and on the oracle (in place on ps / states) and compares."""
    omode = {0: oc.MODE_ERI, 1: oc.MODE_L2, 2: oc.MODE_BNB}[mode]
    exact = (not bf16) or bool(flags & 2) or mode == 1  # the functional update always takes the IEEE chain
    hyper = lambda t: (LR, B1, B2, EPS, wd, t - 1 if mode == 1 else t)
    if exact or len(all_g) == 1:
        for k, g_k in enumerate(all_g):
            hs.oracle_step(ps, g_k, states, hyper(first_step + k), bf16, omode, grad_scale)
        gpu_steps(gt, [None] + all_g[1:], first_step, mode, flags, wd, grad_scale=grad_scale, use_multi=use_multi)
        got_p, got_st = gt.fetch()
        return hs.compare(got_p, got_st, ps, states, bf16, exact, label)
    # The approximate bf16 update promises one bf16 step per step, from the same inputs: a parameter
    # that came out one step off is a different input to the next step, so the oracle continues from
    # the device's parameters after every step (the states never differ and are not touched).
    stats = None
    for k, g_k in enumerate(all_g):
        hs.oracle_step(ps, g_k, states, hyper(first_step + k), bf16, omode, grad_scale)
        gpu_steps(gt, [None if k == 0 else g_k], first_step + k, mode, flags, wd, grad_scale=grad_scale, use_multi=use_multi)
        got_p, got_st = gt.fetch()
        one = hs.compare(got_p, got_st, ps, states, bf16, False, "%s step %d" % (label, k))
        stats = one if stats is None else {key: stats[key] + one[key] for key in stats}
        for a, b in zip(ps, got_p):
            a[:] = b
    stats["params"] //= len(all_g)
    return stats


def run_case(sizes, bf16, seed, steps=3, mode=0, flags=0, wd=WD, p_std=0.02, g_std=1e-3, prior=0,
             grad_scale=None, use_multi=False, label=""):
    ps, gs = hs.make_inputs(sizes, bf16, seed, p_std, g_std)
    states = hs.oracle_states(sizes)
    omode = {0: oc.MODE_ERI, 1: oc.MODE_L2, 2: oc.MODE_BNB}[mode]
    for t in range(1, prior + 1):  # seed the states with a few oracle steps
        g_t = hs.fresh_grads(sizes, bf16, seed * 1000 + t, g_std)
        hs.oracle_step(ps, g_t, states, (LR, B1, B2, EPS, wd, t - 1 if mode == 1 else t), bf16, omode, grad_scale)
    gt = hs.GpuTensors(ps, gs, states, bf16)
    all_g = [gs] + [hs.fresh_grads(sizes, bf16, seed * 7777 + k, g_std) for k in range(1, steps)]
    stats = check_steps(gt, ps, states, all_g, prior + 1, mode, flags, wd, bf16, grad_scale, use_multi, label)
    print("%s: params=%d code_mismatch=%d param_1ulp=%d" % (label, stats["params"], stats["code_mismatch"],
                                                              stats["param_1ulp"]), flush=True)
    assert stats["code_mismatch"] == 0
    return stats


@pytest.mark.parametrize("name", ["eri_f32", "eri_bf16", "l2_f32", "l2_bf16", "bnb_f32", "bnb_bf16", "eri_bf16_gs"])
def test_committed_step_vectors(name):
    """tests/golden/step_vectors.npz: three steps from a zero state, bit for bit (bf16 with the exact flag)."""
    import os
    vec = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "step_vectors.npz"))
    mode = {"eri": 0, "l2": 1, "bnb": 2}[name.split("_")[0]]
    bf16 = "bf16" in name
    gs = 0.37 if name.endswith("_gs") else None
    p0 = vec[name + ".p0"].copy()
    gt = hs.GpuTensors([p0], [vec[name + ".g0"].copy()], hs.oracle_states([p0.size]), bf16)
    gpu_steps(gt, [None, [vec[name + ".g1"]], [vec[name + ".g2"]]], 1, mode, flags=2, grad_scale=gs)
    got_p, got_st = gt.fetch()
    raw = np.uint16 if bf16 else np.uint32
    assert np.array_equal(got_p[0].view(raw), vec[name + ".p"].view(raw))
    assert np.array_equal(got_st[0][0], vec[name + ".m"]) and np.array_equal(got_st[0][1], vec[name + ".v"])
    assert np.array_equal(got_st[0][2].view(np.uint32), vec[name + ".absmax_m"].view(np.uint32))
    assert np.array_equal(got_st[0][3].view(np.uint32), vec[name + ".absmax_v"].view(np.uint32))


def test_config1_flat_fp32_after_ten_prior_steps():
    # benchmark configuration 1: 2**20 fp32 params ~N(0, 0.02), grads ~N(0, 1e-3), states from ten
    # prior steps, block 2048, lr 1e-4, betas (0.9, 0.999), eps 1e-8, wd 0.01; one step
    run_case([1 << 20], False, 0xE21D + 1, steps=1, prior=10, label="c1")


def test_config1_all_eleven_steps_on_the_device():
    run_case([1 << 20], False, 0xE21D + 1, steps=11, prior=0, label="c1-11")


@pytest.mark.parametrize("flags", [0, 2, 4, 6])
def test_bf16_ragged_multi_tensor(flags):
    sizes = [2048 * 3 + 5, 1, 7, 320, 2047, 2048, 2049, 16 * 640, 1280 * 16, 4, 100000]
    run_case(sizes, True, 100 + flags, steps=4, flags=flags, label="bf16-ragged-flags%d" % flags)


@pytest.mark.parametrize("flags", [0, 4])
def test_fp32_ragged_multi_tensor(flags):
    sizes = [2048 * 2 + 1234, 1, 7, 320, 2047, 2049, 65536 + 3]
    run_case(sizes, False, 200 + flags, steps=4, flags=flags, label="fp32-ragged-flags%d" % flags)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_l2_mode_follows_the_functional_update(bf16, wd):
    sizes = [2048 * 5 + 77, 320, 2048, 9]
    run_case(sizes, bf16, 300 + bf16, steps=3, mode=1, flags=2, wd=wd, label="l2-bf16%d-wd%g" % (bf16, wd))


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("wd,gscale", [(0.0, None), (0.01, None), (0.01, 0.37)])
@pytest.mark.parametrize("flags", [0, 2])
def test_bnb_mode(bf16, wd, gscale, flags):
    # flags 0: bf16 parameters through the hardware square root and reciprocal, within one bf16 step of
    # the oracle; flags 2 (ERI_ADAM8_FLAG_EXACT_PARAM): bit for bit.  fp32 parameters are always exact.
    sizes = [2048 * 5 + 77, 320, 2048, 9, 2047, 40000]
    run_case(sizes, bf16, 350 + bf16, steps=3, mode=2, flags=flags, wd=wd, grad_scale=gscale, prior=2,
             label="bnb-bf16%d-wd%g-gs%s-flags%d" % (bf16, wd, gscale, flags))


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("wd", [0.0, 0.01])
@pytest.mark.parametrize("flags", [0, 8])
def test_update_that_cancels_the_parameter_stays_within_one_bf16_step(mode, wd, flags):
    """Parameters chosen equal (to bf16 precision) to the update they are about to receive, as weights
    that start at zero are after their first steps: p - update cancels 9 to 25 leading bits.  The
    approximate bf16 chain's few ulp of error in the update would then show as several bf16 steps of the
    tiny result; such elements must be recomputed with the exact chain."""
    sizes = [2048 * 30 + 1000, 2047]
    omode = oc.MODE_ERI if mode == 0 else oc.MODE_BNB
    _, gs = hs.make_inputs(sizes, True, 4242, 0.02, 1e-3)
    states = hs.oracle_states(sizes)
    for t in (1, 2):  # two earlier steps, so that m / sqrt(v) differs from element to element
        scrap = [np.zeros(n, np.uint16) for n in sizes]
        hs.oracle_step(scrap, hs.fresh_grads(sizes, True, 4300 + t, 1e-3), states, (LR, B1, B2, EPS, wd, t), True, omode)
    hyper = (LR, B1, B2, EPS, wd, 3)
    probe = [np.zeros(n, np.uint16) for n in sizes]
    hs.oracle_step(probe, gs, [[a.copy() for a in st] for st in states], hyper, True, omode)  # from p = 0: minus the update
    ps = [a ^ np.uint16(0x8000) for a in probe]                                              # p = +update, rounded to bf16
    gt = hs.GpuTensors(ps, gs, states, True)
    want = [a.copy() for a in ps]
    hs.oracle_step(want, gs, states, hyper, True, omode)
    gpu_steps(gt, [None], 3, mode, flags, wd)
    got_p, got_st = gt.fetch()
    f32 = lambda a: (a.astype(np.uint32) << 16).view(np.float32)
    deep = sum(int((np.abs(f32(w)) * 32768.0 < np.abs(f32(p))).sum()) for w, p in zip(want, ps))
    assert deep > 200  # enough elements that lose 15 bits or more for the test to bite
    stats = hs.compare(got_p, got_st, want, states, True, False, "cancel-mode%d-wd%g-flags%d" % (mode, wd, flags))
    assert stats["code_mismatch"] == 0


@pytest.mark.parametrize("bf16", [False, True])
def test_bnb_mode_keeps_the_sign_of_tiny_first_moments(bf16):
    # moments 1e-9 of the block's largest round to the zero entry: BNB stores 126 for the negative
    # ones (full blocks and a partial last block), ERI 127; the oracle must agree element for element
    sizes = [2048 * 2 + 300]
    ps, gs = hs.make_inputs(sizes, bf16, 360)
    g = np.zeros(sizes[0], np.float32)
    for base in (0, 2048, 4096):
        g[base] = 1.0
        g[base + 1:base + 40:2] = 1e-9
        g[base + 2:base + 40:2] = -1e-9
        g[base + 100:base + 200] = np.linspace(-1e-3, 1e-3, 100, dtype=np.float32)
    gs = [onp.f32_to_bf16(g) if bf16 else g]
    for mode, zero_code in ((0, 127), (2, 126)):
        p_m = [ps[0].copy()]
        states = hs.oracle_states(sizes)
        gt = hs.GpuTensors(p_m, gs, states, bf16)
        omode = oc.MODE_ERI if mode == 0 else oc.MODE_BNB
        hs.oracle_step(p_m, gs, states, (LR, B1, B2, EPS, WD, 1), bf16, omode)
        gpu_steps(gt, [None], 1, mode, flags=2)
        got_p, got_st = gt.fetch()
        stats = hs.compare(got_p, got_st, p_m, states, bf16, True, "sign-%d" % mode)
        assert stats["code_mismatch"] == 0
        for base in (0, 2048, 4096):
            assert np.all(got_st[0][0][base + 2:base + 40:2] == zero_code)
            assert np.all(got_st[0][0][base + 1:base + 40:2] == 127)


@pytest.mark.parametrize("bf16", [False, True])
def test_l2_mode_bias_correction_with_tiny_huge_and_infinite_moments(bf16):
    """The functional update divides the moments by 1 - beta^s.  Gradients from the denormal range up to
    values whose squares overflow, and infinities, must give the oracle's bits: the kernel's exactly
    rounded fast division has to hand every out-of-range case to the IEEE division."""
    n = 2048 * 2 + 700
    rng = np.random.default_rng(31 + bf16)
    mags = 10.0 ** rng.uniform(-45, 38, n)
    with np.errstate(over="ignore"):
        g = (rng.standard_normal(n) * mags).astype(np.float32)
    g[::97] = 0.0
    g[5], g[2048 + 9], g[4096 + 11] = np.inf, -np.inf, np.inf
    ps, _ = hs.make_inputs([n], bf16, 33)
    gs = [onp.f32_to_bf16(g) if bf16 else g]
    g2 = [onp.f32_to_bf16((g * np.float32(0.5)).astype(np.float32)) if bf16 else (g * np.float32(0.5)).astype(np.float32)]
    states = hs.oracle_states([n])
    gt = hs.GpuTensors(ps, gs, states, bf16)
    with np.errstate(all="ignore"):
        hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, 0), bf16, oc.MODE_L2)
        hs.oracle_step(ps, g2, states, (LR, B1, B2, EPS, WD, 1), bf16, oc.MODE_L2)
    gpu_steps(gt, [None, g2], 1, mode=1, flags=2)
    got_p, got_st = gt.fetch()
    stats = hs.compare(got_p, got_st, ps, states, bf16, True, "l2-range")
    assert stats["code_mismatch"] == 0


@pytest.mark.parametrize("eps", [1e-8, 0.0])
def test_l2_mode_with_every_moment_of_a_block_near_the_denormal_range(eps):
    """Whole blocks of gradients between 1e-44 and 1e-28: the block maxima are tiny too, so the dequantised
    moments stay non-zero down to the denormal range instead of rounding to the zero entry.  The fast chain of
    the functional update multiplies by reciprocals of the bias corrections, which is not the division's
    rounding there (the kernel sends such elements to the division); with eps = 0 nothing swallows the second
    moment's square root either.  The oracle's bits, bf16 parameters, three steps."""
    L = _lib()
    n = 2048 * 3 + 300
    rng = np.random.default_rng(4242)
    ps, _ = hs.make_inputs([n], True, 77, p_std=0.0)  # parameters at zero: the first result is the rounded update itself
    states = hs.oracle_states([n])

    def grads(lo, hi):
        g = (rng.standard_normal(n) * 10.0 ** rng.uniform(lo, hi, n)).astype(np.float32)
        g[::53] = 0.0
        return [onp.f32_to_bf16(g)]

    all_g = [grads(-40, -28), grads(-44, -30), grads(-38, -28)]
    gt = hs.GpuTensors(ps, all_g[0], states, True)
    rows = gt.rows(None)
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), _stream(), C.byref(table)), "table_create")
    with np.errstate(all="ignore"):
        for k, g_k in enumerate(all_g):
            hs.oracle_step(ps, g_k, states, (LR, B1, B2, eps, 0.0, k), True, oc.MODE_L2)
            if k:
                gt.set_grads(g_k)
            h = L.hyper_pack(LR, B1, B2, eps, 0.0, k, 1, 2 | KERNEL_FLAGS)
            L.check(L.lib().eri_adam8_step_table(table, C.byref(h), _stream()), "step_table")
    _sync()
    L.lib().eri_adam8_table_destroy(table)
    got_p, got_st = gt.fetch()
    assert any((a.view(np.uint32) != 0).any() for a in (states[0][2], states[0][3]))  # the block maxima are not all zero
    stats = hs.compare(got_p, got_st, ps, states, True, True, "l2-denormal-range eps=%g" % eps)
    assert stats["code_mismatch"] == 0


def test_l2_mode_with_first_moments_of_a_few_denormal_steps():
    """States built by hand: first moments of 10 to 100,000 denormal steps (absmax 1e-44 to 1e-40), ordinary
    second moments, zero gradients, and a learning rate large enough to lift the update out of the denormal
    range.  m / (1 - beta1^s) then has few significant bits, where a product with the rounded reciprocal can
    land a whole step of that coarse grid away from the quotient (a host search finds a few such first moments
    per 10^5 and none among 2 * 10^7 that also changes the rounded update, so this is coverage of the regime,
    not a case that fails without the kernel's fallback to the division)."""
    L = _lib()
    n = 2048 * 96
    rng = np.random.default_rng(99)
    ps, _ = hs.make_inputs([n], True, 78, p_std=0.0)
    states = hs.oracle_states([n])
    m, v, am, av = states[0]
    m[:] = rng.integers(0, 256, n, dtype=np.uint8)
    v[:] = rng.integers(1, 256, n, dtype=np.uint8)
    m[::2048] = 255
    v[::2048] = 255
    am[:] = (10.0 ** rng.uniform(-44, -40, am.size)).astype(np.float32)
    av[:] = np.float32(1e-6)
    gs = [onp.f32_to_bf16(np.zeros(n, np.float32))]
    gt = hs.GpuTensors(ps, gs, states, True)
    lr = 1e12
    for step in (3, 4):
        with np.errstate(all="ignore"):
            hs.oracle_step(ps, gs, states, (lr, B1, B2, EPS, 0.0, step), True, oc.MODE_L2)
        gpu_steps(gt, [None], step + 1, mode=1, flags=2, wd=0.0, lr=lr)
    got_p, got_st = gt.fetch()
    assert np.count_nonzero(ps[0] & 0x7FFF) > n // 2  # the updates are visible in the parameters
    stats = hs.compare(got_p, got_st, ps, states, True, True, "l2-few-denormal-steps")
    assert stats["code_mismatch"] == 0


def test_no_weight_decay_variant():
    run_case([2048 * 9 + 3, 640], True, 400, steps=3, wd=0.0, flags=2, label="wd0")
    run_case([2048 * 9 + 3, 640], False, 401, steps=3, wd=0.0, label="wd0-fp32")


def test_grad_scale_folded_into_the_step():
    run_case([2048 * 4 + 3, 640], True, 500, steps=3, flags=2, grad_scale=0.37, label="gscale")
    run_case([2048 * 4 + 3, 640], False, 501, steps=2, grad_scale=0.37, label="gscale-fp32")


def test_step_multi_convenience_entry_point():
    run_case([2048 * 4 + 3, 640, 5000], True, 600, steps=3, flags=2, use_multi=True, label="step_multi")


def test_lora_scale_values_bf16():
    # LoRA-B-like: params and updates of the same magnitude (heavy cancellation in p - update)
    run_case([16 * 5120, 1280 * 16, 16 * 320], True, 700, steps=5, p_std=1e-4, g_std=1e-4, flags=2, label="lora-exact")
    run_case([16 * 5120, 1280 * 16, 16 * 320], True, 700, steps=5, p_std=1e-4, g_std=1e-4, flags=0, label="lora-fast")


def test_scaled_model_shapes_bf16():
    from eridiffusion_amd import workloads as w
    for name, tensors in (("c2", w.c2_sdxl_lora(pairs=60, scale=4)), ("c3", w.c3_flux_lora(scale=16)),
                          ("c4", w.c4_sdxl_full(scale=8)), ("c5", w.c5_flux_full(scale=32))):
        sizes = [w.numel(s) for _, s in tensors]
        if name in ("c3", "c5"):
            sizes = sizes[::6]
        run_case(sizes, True, 800 + len(sizes), steps=2, label=name + "-scaled")


def test_hundred_steps_of_a_lora_set_stay_on_the_oracle():
    """The rank-32 FLUX LoRA list (every sixth tensor, widths / 16) for a hundred steps with fresh
    gradients each step, as the LoRA configurations of the benchmark prescribe: states start at zero,
    LoRA-B weights start at zero and grow to the size of their updates.  Exact flag: states and bf16
    parameters bit for bit after step 100 -- one wrong code early on would have spread by then."""
    from eridiffusion_amd import workloads as w
    sizes = [w.numel(s) for _, s in w.c3_flux_lora(scale=16)][::6]
    ps, _ = hs.make_inputs(sizes, True, 1234, 0.02, 1e-4)
    for i in range(1, len(ps), 2):
        ps[i][:] = 0  # every other tensor starts at zero, as LoRA-B matrices do
    states = hs.oracle_states(sizes)
    all_g = [hs.fresh_grads(sizes, True, 50000 + t, 1e-4) for t in range(100)]
    gt = hs.GpuTensors(ps, all_g[0], states, True)
    for t, g_t in enumerate(all_g):
        hs.oracle_step(ps, g_t, states, (LR, B1, B2, EPS, WD, t + 1), True, oc.MODE_ERI)
    gpu_steps(gt, [None] + all_g[1:], 1, 0, 2, WD)
    got_p, got_st = gt.fetch()
    stats = hs.compare(got_p, got_st, ps, states, True, True, "lora-100-steps")
    assert stats["code_mismatch"] == 0


def test_zero_gradients_and_zero_state():
    sizes = [2048 * 2 + 9]
    ps, gs = hs.make_inputs(sizes, False, 900)
    gs = [np.zeros_like(g) for g in gs]
    states = hs.oracle_states(sizes)
    gt = hs.GpuTensors(ps, gs, states, False)
    hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, 1), False)
    gpu_steps(gt, [None], 1)
    got_p, got_st = gt.fetch()
    hs.compare(got_p, got_st, ps, states, False, True, "zero")
    assert np.all(got_st[0][0] == 127) and np.all(got_st[0][1] == 0) and np.all(got_st[0][2] == 0)


def test_extreme_and_non_finite_gradients():
    sizes = [2048 * 4]
    ps, gs = hs.make_inputs(sizes, False, 901)
    g = gs[0]
    g[0:2048] *= 1e-30           # absmax of v far below 2^-60: the IEEE-division branch
    g[2048:4096] *= 1e18         # huge moments
    g[4096 + 5] = np.nan         # one NaN inside a block
    g[6144 + 9] = np.inf         # one Inf inside a block
    states = hs.oracle_states(sizes)
    gt = hs.GpuTensors(ps, gs, states, False)
    g2 = hs.fresh_grads(sizes, False, 902)
    with np.errstate(all="ignore"):
        hs.oracle_step(ps, gs, states, (LR, B1, B2, EPS, WD, 1), False)
        hs.oracle_step(ps, g2, states, (LR, B1, B2, EPS, WD, 2), False)
    gpu_steps(gt, [None, g2], 1)
    got_p, got_st = gt.fetch()
    # absmax may be NaN/Inf here; compare bit patterns of finite entries and the NaN pattern
    for k in (2, 3):
        a, b = got_st[0][k], states[0][k]
        assert np.array_equal(np.isnan(a), np.isnan(b))
        assert np.array_equal(a[~np.isnan(a)].view(np.uint32), b[~np.isnan(b)].view(np.uint32))
    for k in (0, 1):
        assert np.array_equal(got_st[0][k], states[0][k])
    nan = np.isnan(ps[0])
    assert np.array_equal(nan, np.isnan(got_p[0]))
    assert np.array_equal(got_p[0][~nan].view(np.uint32), ps[0][~nan].view(np.uint32))


def test_state_init_and_quantize_round_trip():
    import torch
    L = _lib()
    n = 2048 * 3 + 17
    dev = torch.device("cuda:0")
    m = torch.full((n,), 9, dtype=torch.uint8, device=dev)
    v = torch.full((n,), 9, dtype=torch.uint8, device=dev)
    am = torch.full((4,), 3.0, device=dev)
    av = torch.full((4,), 3.0, device=dev)
    L.check(L.lib().eri_adam8_state_init(m.data_ptr(), v.data_ptr(), am.data_ptr(), av.data_ptr(), n, _stream()), "init")
    _sync()
    assert bool((m == 127).all()) and bool((v == 0).all()) and bool((am == 0).all()) and bool((av == 0).all())
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    x[2048:4096] = 0
    for signed, table in ((1, hs.MAPS[0]), (0, hs.MAPS[1])):
        xs = x if signed else np.abs(x)
        xd = torch.from_numpy(xs).to(dev)
        codes = torch.empty(n, dtype=torch.uint8, device=dev)
        absmax = torch.empty(4, dtype=torch.float32, device=dev)
        back = torch.empty(n, dtype=torch.float32, device=dev)
        L.check(L.lib().eri_adam8_quantize(xd.data_ptr(), signed, n, codes.data_ptr(), absmax.data_ptr(), _stream()), "q")
        L.check(L.lib().eri_adam8_dequantize(codes.data_ptr(), absmax.data_ptr(), signed, n, back.data_ptr(), _stream()), "dq")
        _sync()
        wc = np.empty(n, np.uint8)
        wa = np.empty(4, np.float32)
        wb = np.empty(n, np.float32)
        oc.lib().eri_oracle_quantize(oc.ptr(xs), oc.ptr(table), n, oc.ptr(wc), oc.ptr(wa))
        oc.lib().eri_oracle_dequantize(oc.ptr(wc), oc.ptr(wa), oc.ptr(table), n, oc.ptr(wb))
        assert np.array_equal(codes.cpu().numpy(), wc)
        assert np.array_equal(absmax.cpu().numpy().view(np.uint32), wa.view(np.uint32))
        assert np.array_equal(back.cpu().numpy().view(np.uint32), wb.view(np.uint32))


def test_quantization_as_in_the_reference():
    # adam8bit_enhanced.rs:486-498 on the device: 10x10 ~N(0, 1), quantise, dequantise, mean |error| < 0.1
    import torch
    L = _lib()
    x = torch.randn(100, device="cuda", generator=torch.Generator(device="cuda").manual_seed(486))
    codes = torch.empty(100, dtype=torch.uint8, device="cuda")
    absmax = torch.empty(1, device="cuda")
    back = torch.empty(100, device="cuda")
    L.check(L.lib().eri_adam8_quantize(x.data_ptr(), 1, 100, codes.data_ptr(), absmax.data_ptr(), _stream()), "q")
    L.check(L.lib().eri_adam8_dequantize(codes.data_ptr(), absmax.data_ptr(), 1, 100, back.data_ptr(), _stream()), "dq")
    _sync()
    assert back.shape == x.shape and float(absmax[0]) == float(x.abs().max())
    assert float((back - x).abs().mean()) < 0.02


def test_randomized_cases_against_the_oracle():
    """Forty seeded random combinations of tensor lists (ragged, tiny, multi-block), dtype, mode, flags,
    decay, gradient scale and prior history; every one must match the oracle to the bar above."""
    rng = np.random.default_rng(20240607)
    pool = [1, 3, 8, 63, 64, 65, 320, 511, 512, 1000, 2047, 2048, 2049, 4095, 4096, 5120, 10240, 12289, 20480, 65536 + 17]
    flips = 0
    for case in range(40):
        k = int(rng.integers(1, 9))
        sizes = [int(rng.choice(pool)) for _ in range(k)]
        if rng.random() < 0.3:
            sizes.append(int(rng.integers(1, 40000)))
        bf16 = bool(rng.integers(0, 2))
        mode = int(rng.choice([0, 0, 1, 2]))
        flags = int(rng.choice([0, 2, 4, 8, 2 | 4, 2 | 8])) if mode != 2 else 0
        if mode == 1:
            flags |= 2  # the functional update is compared bit for bit
        wd = float(rng.choice([0.0, 0.01, 0.1]))
        gscale = None if rng.random() < 0.6 else float(rng.uniform(0.1, 2.0))
        g_std = float(10.0 ** rng.uniform(-5, -1))
        p_std = float(10.0 ** rng.uniform(-4, 0))
        st = run_case(sizes, bf16, 9000 + case, steps=int(rng.integers(1, 4)), mode=mode, flags=flags, wd=wd,
                      p_std=p_std, g_std=g_std, prior=int(rng.integers(0, 3)), grad_scale=gscale,
                      use_multi=bool(rng.random() < 0.25), label="rand%d" % case)
        flips += st["param_1ulp"]
    print("randomized cases: bf16 parameters one ulp off on the approximate path: %d" % flips, flush=True)


def test_randomized_extreme_values_against_the_oracle():
    """Gradient magnitudes from 1e-30 to 1e30, exact zeros, NaN and infinities, both dtypes, all modes,
    default (approximate bf16 update) and exact flags: states bit-exact, parameters to the bar, NaN in the
    same places."""
    rng = np.random.default_rng(777)
    for case in range(24):
        sizes = [int(rng.choice([5, 2047, 2048, 2049, 6 * 2048 + 100])) for _ in range(int(rng.integers(1, 4)))]
        bf16 = bool(rng.integers(0, 2))
        mode = int(rng.choice([0, 0, 1, 2]))
        flags = 2 if mode == 1 else int(rng.choice([0, 2]) if mode == 2 else rng.choice([0, 2, 4, 8]))
        wd = float(rng.choice([0.0, 0.01]))
        mag_g = 10.0 ** rng.uniform(-30, 30) if case % 2 else 10.0 ** rng.uniform(-8, 2)
        ps, _ = hs.make_inputs(sizes, bf16, 3000 + case, p_std=float(10.0 ** rng.uniform(-4, 2)))
        states = hs.oracle_states(sizes)

        def grads():
            out = []
            for n in sizes:
                with np.errstate(over="ignore"):
                    g = (rng.standard_normal(n) * mag_g).astype(np.float32)
                g[rng.random(n) < 0.05] = 0.0
                if case % 3 == 2 and n > 8:
                    g[int(rng.integers(0, n))] = np.nan
                    g[int(rng.integers(0, n))] = np.inf
                    g[int(rng.integers(0, n))] = -np.inf
                out.append(onp.f32_to_bf16(g) if bf16 else g)
            return out

        all_g = [grads() for _ in range(3)]
        gt = hs.GpuTensors(ps, all_g[0], states, bf16)
        with np.errstate(all="ignore"):
            stats = check_steps(gt, ps, states, all_g, 1, mode, flags, wd, bf16, label="extreme%d" % case)
        assert stats["code_mismatch"] == 0, case


@pytest.mark.parametrize("blocks", [255, 257, 513, 768, 769, 1300])
def test_tables_around_the_team_counts_of_the_small_table_kernel(blocks):
    """The four-waves-per-block kernel runs a table of up to one, two, three blocks per compute unit with that many
    teams per workgroup and anything larger with four; the block counts here sit on both sides of each change (256
    units).  Three ragged tensors, bf16 and fp32."""
    a = blocks // 3
    sizes = [2048 * a + 5, 2048 * (blocks - 2 * a), 2048 * a + 2047]
    for bf16 in (True, False):
        run_case(sizes, bf16, 600 + blocks, steps=2, flags=2, label="teams-%d-%s" % (blocks, "bf16" if bf16 else "f32"))


def test_five_thousand_small_tensors_in_one_launch():
    """A long launch table: 5,000 tensors of 1 to 6,000 elements (most of them nothing but a partial
    block), both through the table handle and through step_multi."""
    rng = np.random.default_rng(5000)
    sizes = [int(x) for x in rng.integers(1, 6000, 5000)]
    run_case(sizes, True, 5001, steps=2, flags=2, label="5000-tensors")
    run_case(sizes[:1500], False, 5002, steps=2, use_multi=True, label="1500-tensors-multi")
