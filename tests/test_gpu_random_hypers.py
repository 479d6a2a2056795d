"""GPU parity under hyper-parameters away from the defaults.

The other parity files vary sizes, values, modes and flags at lr 1e-4, betas (0.9, 0.999), eps 1e-8.  The
margins that decide which elements the exact instantiations recompute, and the folded constants of the
functional update's chain, are functions of the hyper-parameters, so this file draws them: learning rates
from 1e-7 to 0.3, beta1 from 0 to 0.999, beta2 from 0.5 to 0.99999, eps from 0 to 1e-2, decay from 0 to 1,
step counters from 1 to 10^7 (the bias corrections run from 1e-5 to 1).  The bar is the one of
test_gpu_parity.py: 8-bit states and fp32 parameters bit-exact, bf16 parameters bit-exact with
ERI_ADAM8_FLAG_EXACT_PARAM and in the functional mode, within one bf16 step otherwise.
"""
import ctypes as C
import os

import numpy as np
import pytest

import harness as hs
import oracle_c as oc

pytestmark = pytest.mark.gpu

SIZES = [2048 * 9 + 13, 2048 * 4, 777, 2048 * 2 + 2047, 2048 * 23 + 1]
CASES = int(os.environ.get("ERI_HYPER_CASES", "48"))  # per combination of dtype, mode and kernel; more for a soak


def _lib():
    from eridiffusion_amd import _lib
    return _lib


def _draw(rng):
    return dict(
        lr=float(10.0 ** rng.uniform(-7, -0.5)),
        b1=float(rng.choice([0.0, 0.5, 0.9, 0.95, 0.99, 0.999])),
        b2=float(rng.choice([0.5, 0.9, 0.95, 0.99, 0.999, 0.9999, 0.99999])),
        eps=float(rng.choice([0.0, 1e-15, 1e-12, 1e-8, 1e-6, 1e-3, 1e-2])),
        wd=float(rng.choice([0.0, 0.0, 1e-4, 0.01, 0.1, 1.0])),
        t=int(rng.choice([1, 2, 3, 10, 100, 1000, 30000, 10 ** 7])),
        g_std=float(10.0 ** rng.uniform(-6, 0)),
        p_std=float(10.0 ** rng.uniform(-3, 0.5)),
    )


@pytest.mark.parametrize("kernels", ["default-kernels", "one-wave", "plain"])
@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("bf16", [True, False])
def test_drawn_hyper_parameters_against_the_oracle(bf16, mode, kernels):
    import torch
    L = _lib()
    kflags = {"default-kernels": 0, "one-wave": L.FLAG_ONE_WAVE, "plain": L.FLAG_NO_PIPELINE}[kernels]
    omode = {0: oc.MODE_ERI, 1: oc.MODE_L2, 2: oc.MODE_BNB}[mode]
    rng = np.random.default_rng(5150 + 10 * mode + bf16)  # the same draws for the three kernels
    stream = torch.cuda.current_stream().cuda_stream
    flips = 0
    for case in range(CASES):
        d = _draw(rng)
        flags = 2 if mode == 1 else int(rng.choice([0, 2, 2]))
        exact = (not bf16) or bool(flags & 2)
        label = "hypers bf16=%d mode=%d %s case %d %r flags=%d" % (bf16, mode, kernels, case, d, flags)
        print(label, flush=True)
        ps, gs = hs.make_inputs(SIZES, bf16, 100 * case + mode, d["p_std"], d["g_std"])
        states = hs.oracle_states(SIZES)
        count = lambda t: t - 1 if mode == 1 else t  # the functional update bumps its counter afterwards
        hyper = lambda t: (d["lr"], d["b1"], d["b2"], d["eps"], d["wd"], count(t))
        # two oracle steps give the states a history; the device then runs steps t and t+1
        for k, t in enumerate((max(d["t"] - 2, 1), max(d["t"] - 1, 1))):
            with np.errstate(all="ignore"):
                hs.oracle_step(ps, hs.fresh_grads(SIZES, bf16, 31 * case + k, d["g_std"]), states, hyper(t), bf16, omode)
        gt = hs.GpuTensors(ps, gs, states, bf16)
        rows = gt.rows()
        table = C.c_void_p()
        L.check(L.lib().eri_adam8_table_create(rows, len(rows), stream, C.byref(table)), "table_create")
        for k in range(2):
            g_k = gs if k == 0 else hs.fresh_grads(SIZES, bf16, 57 * case + 5, d["g_std"])
            if k:
                gt.set_grads(g_k)
            h = L.hyper_pack(*hyper(d["t"] + k)[:5], count(d["t"] + k), mode, flags | kflags)
            L.check(L.lib().eri_adam8_step_table(table, C.byref(h), stream), "step_table")
            torch.cuda.synchronize()
            with np.errstate(all="ignore"):
                hs.oracle_step(ps, g_k, states, hyper(d["t"] + k), bf16, omode)
            got_p, got_st = gt.fetch()
            st = hs.compare(got_p, got_st, ps, states, bf16, exact, label)
            assert st["code_mismatch"] == 0, label
            flips += st["param_1ulp"]
            if not exact:  # one bf16 step per step from the same inputs: continue from the device's parameters
                for a, b in zip(ps, got_p):
                    a[:] = b
        L.lib().eri_adam8_table_destroy(table)
    print("drawn hyper-parameters: bf16 parameters one step off on the faster chain: %d" % flips, flush=True)
