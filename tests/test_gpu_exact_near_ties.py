"""ERI_ADAM8_FLAG_EXACT_PARAM on bf16 parameters where it is hardest: results on the edge of a bf16 rounding.

With the flag the kernel computes the fast chain (hardware square root and reciprocal, fused multiply-adds)
and recomputes, with the IEEE chain, every element whose fast result lies so close to a tie point of the
bf16 grid that the exact chain could round the other way.  Random inputs put about four elements in a
million there, so this test builds tensors that consist of nothing else: pairs (p, g) are searched on the
host, with the update restated in NumPy float32, for exact fp32 results within a few fp32 ulp of a tie
(with every block's absmax fixed, an element's moments depend on its own codes and gradient alone, so
elements can be chosen one by one).
The device must reproduce the oracle's parameters bit for bit on all of them, for each step kernel.
"""
import ctypes as C

import numpy as np
import pytest

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu
F32 = np.float32


A_M, A_V = F32(2.5e-4), F32(1.5e-6)  # absmax of every block's first and second moment in the constructed state


def _step_fp32(p16, g16, mc, vc, h, mode):
    """fp32 result of one step before its rounding to bf16 (one rounded operation per line), from the state
    {codes mc, vc; every block's absmax A_M, A_V}."""
    p = onp.bf16_to_f32(p16)
    g = onp.bf16_to_f32(g16)
    with np.errstate(all="ignore"):
        m = (hs.MAPS[0][mc] * A_M) * h.beta1 + g * h.omb1
        v = (hs.MAPS[1][vc] * A_V) * h.beta2 + (g * g) * h.omb2
        den = np.sqrt(v) + h.eps
        r = m / den
        if mode == oc.MODE_BNB:
            pn = p - r * h.step_size
            if h.weight_decay != F32(1.0):
                pn = pn * h.weight_decay
        else:
            u = r + p * h.weight_decay if h.weight_decay > 0 else r
            pn = p - u * h.step_size
    return pn.astype(F32)


_found = {}


DEFAULT_HYP = (0.9, 0.999, 1e-8, 7)  # beta1, beta2, eps, step


def _near_tie_elements(mode, wd, lr, want, seed, p_std, hyp=DEFAULT_HYP):
    key = (mode, wd, lr, want, seed, p_std, hyp)
    if key in _found:
        return _found[key]
    h = oc.hyper_pack(lr, hyp[0], hyp[1], hyp[2], wd, hyp[3], mode)
    hh = type("H", (), {k: F32(getattr(h, k)) for k in ("beta1", "beta2", "omb1", "omb2", "eps", "weight_decay", "step_size")})
    rng = np.random.default_rng(seed)
    keep = [[], [], [], []]
    have = 0
    for _ in range(400):
        n = 1 << 21
        p16 = onp.f32_to_bf16((rng.standard_normal(n) * p_std).astype(F32))
        g16 = onp.f32_to_bf16((rng.standard_normal(n) * 1e-3).astype(F32))
        mc = rng.integers(0, 256, n, dtype=np.uint8)
        vc = rng.integers(0, 256, n, dtype=np.uint8)
        pn = _step_fp32(p16, g16, mc, vc, hh, mode)
        low = (pn.view(np.uint32) & 0xFFFF).astype(np.int32)
        near = np.abs(low - 0x8000) <= 3  # within three fp32 ulp of a bf16 tie point
        for dst, src in zip(keep, (p16, g16, mc, vc)):
            dst.append(src[near])
        have += int(near.sum())
        if have >= want:
            break
    _found[key] = tuple(np.concatenate(k)[:want] for k in keep)
    return _found[key]


@pytest.mark.parametrize("kernels", ["default-kernels", "one-wave", "plain"])
@pytest.mark.parametrize("mode,wd,lr,p_std", [(oc.MODE_ERI, 0.01, 1e-4, 0.02), (oc.MODE_ERI, 0.0, 1e-3, 0.02),
                                             (oc.MODE_BNB, 0.01, 1e-4, 0.02), (oc.MODE_ERI, 0.01, 1e-4, 2e-4)])
def test_results_on_the_edge_of_a_bf16_rounding_are_bit_exact(mode, wd, lr, p_std, kernels):
    _run_near_ties(mode, wd, lr, p_std, kernels, DEFAULT_HYP)


@pytest.mark.parametrize("kernels", ["default-kernels", "one-wave", "plain"])
@pytest.mark.parametrize("mode,wd,lr,p_std,hyp", [
    (oc.MODE_ERI, 0.1, 3e-2, 0.5, (0.5, 0.9, 1e-3, 1)),        # first step, large eps, strong decay
    (oc.MODE_ERI, 1.0, 0.1, 0.05, (0.0, 0.99, 1e-6, 3)),       # no momentum; a decay of a tenth per step
    (oc.MODE_ERI, 0.0, 2e-3, 1.0, (0.99, 0.99999, 0.0, 100000)),  # late in a run, eps 0, steps of half a bf16 unit
    (oc.MODE_BNB, 0.1, 1e-2, 0.1, (0.95, 0.95, 1e-6, 2)),
])
def test_near_ties_under_other_hyper_parameters_are_bit_exact(mode, wd, lr, p_std, hyp, kernels):
    """The margins of the recomputation are functions of the step size and the decay; the same construction
    away from the default hyper-parameters."""
    _run_near_ties(mode, wd, lr, p_std, kernels, hyp)


def _run_near_ties(mode, wd, lr, p_std, kernels, hyp):
    import torch
    from eridiffusion_amd import _lib as L
    extra = {"default-kernels": 0, "one-wave": L.FLAG_ONE_WAVE, "plain": L.FLAG_NO_PIPELINE}[kernels]
    n = 2048 * 3 + 40
    p16, g16, mc, vc = _near_tie_elements(mode, wd, lr, n, 11 + mode, p_std, hyp)
    assert p16.size == n, "the search found too few near-tie elements"
    b1, b2, eps, t = hyp
    sizes = [2048 * 2, 2048 + 40]
    cut = sizes[0]

    def fresh():
        ps = [p16[:cut].copy(), p16[cut:].copy()]
        states = [[mc[:cut].copy(), vc[:cut].copy(), np.full(2, A_M, F32), np.full(2, A_V, F32)],
                  [mc[cut:].copy(), vc[cut:].copy(), np.full(2, A_M, F32), np.full(2, A_V, F32)]]
        return ps, states

    ps, states = fresh()
    gs = [g16[:cut].copy(), g16[cut:].copy()]
    gt = hs.GpuTensors(ps, gs, states, True)
    rows = gt.rows()
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    gmode = {oc.MODE_ERI: L.MODE_ERI, oc.MODE_BNB: L.MODE_BNB}[mode]
    h = L.hyper_pack(lr, b1, b2, eps, wd, t, gmode, L.FLAG_EXACT_PARAM | extra)
    L.check(L.lib().eri_adam8_step_table(table, C.byref(h), None), "step_table")
    torch.cuda.synchronize()
    hs.oracle_step(ps, gs, states, (lr, b1, b2, eps, wd, t), True, mode)
    got_p, got_st = gt.fetch()
    stats = hs.compare(got_p, got_st, ps, states, True, True, "near ties")
    assert stats["code_mismatch"] == 0
    # the default arithmetic on the same inputs: within one bf16 step, and off by one somewhere (which is
    # what makes these inputs a test of the flag)
    gt2 = hs.GpuTensors(*(lambda f: (f[0], gs, f[1]))(fresh()), True)
    rows2 = gt2.rows()
    L.check(L.lib().eri_adam8_table_update(table, rows2, len(rows2), None), "table_update")
    h0 = L.hyper_pack(lr, b1, b2, eps, wd, t, gmode, extra)
    L.check(L.lib().eri_adam8_step_table(table, C.byref(h0), None), "step_table")
    torch.cuda.synchronize()
    got_p2, got_st2 = gt2.fetch()
    stats2 = hs.compare(got_p2, got_st2, ps, states, True, False, "near ties, default arithmetic")
    print("near-tie inputs: default arithmetic one bf16 step off on %d of %d" % (stats2["param_1ulp"], n), flush=True)
    L.lib().eri_adam8_table_destroy(table)


def _update_fp32_l2(p16, g16, mc, vc, h):
    """The functional update's fp32 update term before its rounding to bf16 (adam8bit.rs:113-196, one rounded
    operation per line), from the state {codes mc, vc; every block's absmax A_M, A_V}."""
    p = onp.bf16_to_f32(p16)
    g = onp.bf16_to_f32(g16)
    with np.errstate(all="ignore"):
        if h.weight_decay > 0:
            g = g + p * h.weight_decay
        m = (hs.MAPS[0][mc] * A_M) * h.beta1 + g * h.omb1
        v = (hs.MAPS[1][vc] * A_V) * h.beta2 + (g * g) * h.omb2
        mh = m / h.bc1
        vh = np.maximum(v / h.bc2, F32(0.0))
        den = np.sqrt(vh) + h.eps
        us = (mh / den) * h.step_size
    return us.astype(F32)


@pytest.mark.parametrize("kernels", ["default-kernels", "one-wave", "plain"])
@pytest.mark.parametrize("wd,lr,step,spread", [(0.01, 1e-4, 7, 3), (0.0, 1e-3, 1, 3), (0.01, 1e-4, 40, 30)])
def test_functional_updates_on_the_edge_of_a_bf16_rounding_are_bit_exact(wd, lr, step, spread, kernels):
    """Mode L2 rounds the update itself to bf16 and decides by the low half of its fast chain's update whether the
    exact chain has to be asked.  Tensors that consist of nothing but updates within `spread` fp32 patterns of a
    bf16 tie point -- 3: where the two chains' roundings part; 30: on both sides of the edge of the window in
    which the fast chain is not trusted -- must come out with the oracle's bits on every step kernel."""
    import torch
    from eridiffusion_amd import _lib as L
    extra = {"default-kernels": 0, "one-wave": L.FLAG_ONE_WAVE, "plain": L.FLAG_NO_PIPELINE}[kernels]
    n = 2048 * 3 + 40
    key = ("l2", wd, lr, step, spread)
    if key not in _found:
        h = oc.hyper_pack(lr, 0.9, 0.999, 1e-8, wd, step, oc.MODE_L2)
        hh = type("H", (), {k: F32(getattr(h, k)) for k in ("beta1", "beta2", "omb1", "omb2", "eps", "weight_decay", "step_size", "bc1", "bc2")})
        rng = np.random.default_rng(500 + step)
        keep, have = [[], [], [], []], 0
        for _ in range(400):
            k = 1 << 21
            p16 = onp.f32_to_bf16((rng.standard_normal(k) * 0.02).astype(F32))
            g16 = onp.f32_to_bf16((rng.standard_normal(k) * 1e-3).astype(F32))
            mc = rng.integers(0, 256, k, dtype=np.uint8)
            vc = rng.integers(0, 256, k, dtype=np.uint8)
            us = _update_fp32_l2(p16, g16, mc, vc, hh)
            low = (us.view(np.uint32) & 0xFFFF).astype(np.int32)
            near = (np.abs(low - 0x8000) <= spread) & np.isfinite(us) & (np.abs(us) > F32(1e-30))
            for dst, src in zip(keep, (p16, g16, mc, vc)):
                dst.append(src[near])
            have += int(near.sum())
            if have >= n:
                break
        _found[key] = tuple(np.concatenate(x)[:n] for x in keep)
    p16, g16, mc, vc = _found[key]
    assert p16.size == n, "the search found too few near-tie updates"
    sizes = [2048 * 2, 2048 + 40]
    cut = sizes[0]
    ps = [p16[:cut].copy(), p16[cut:].copy()]
    gs = [g16[:cut].copy(), g16[cut:].copy()]
    states = [[mc[:cut].copy(), vc[:cut].copy(), np.full(2, A_M, F32), np.full(2, A_V, F32)],
              [mc[cut:].copy(), vc[cut:].copy(), np.full(2, A_M, F32), np.full(2, A_V, F32)]]
    gt = hs.GpuTensors(ps, gs, states, True)
    rows = gt.rows()
    table = C.c_void_p()
    L.check(L.lib().eri_adam8_table_create(rows, len(rows), None, C.byref(table)), "table_create")
    h = L.hyper_pack(lr, 0.9, 0.999, 1e-8, wd, step, L.MODE_L2, L.FLAG_EXACT_PARAM | extra)
    L.check(L.lib().eri_adam8_step_table(table, C.byref(h), None), "step_table")
    torch.cuda.synchronize()
    hs.oracle_step(ps, gs, states, (lr, 0.9, 0.999, 1e-8, wd, step), True, oc.MODE_L2)
    got_p, got_st = gt.fetch()
    stats = hs.compare(got_p, got_st, ps, states, True, True, "near ties, functional update")
    assert stats["code_mismatch"] == 0
    L.lib().eri_adam8_table_destroy(table)
