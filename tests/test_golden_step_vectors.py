"""The committed step vectors (tests/golden/step_vectors.npz, written once by make_step_vectors.py) against
both CPU restatements: any later change of the oracle's arithmetic shows up here."""
import os

import numpy as np
import pytest

import oracle_c as oc
from oracle import adam8_numpy as onp

HERE = os.path.dirname(os.path.abspath(__file__))
VEC = np.load(os.path.join(HERE, "golden", "step_vectors.npz"))
HYPER = (1e-4, 0.9, 0.999, 1e-8, 0.01)
CASES = {"eri_f32": (oc.MODE_ERI, "eri", False, None), "eri_bf16": (oc.MODE_ERI, "eri", True, None),
         "l2_f32": (oc.MODE_L2, "l2", False, None), "l2_bf16": (oc.MODE_L2, "l2", True, None),
         "bnb_f32": (oc.MODE_BNB, "bnb", False, None), "bnb_bf16": (oc.MODE_BNB, "bnb", True, None),
         "eri_bf16_gs": (oc.MODE_ERI, "eri", True, 0.37)}


def expect(name, p, st):
    raw = np.uint16 if p.dtype == np.uint16 else np.uint32
    assert np.array_equal(p.view(raw), VEC[name + ".p"].view(raw))
    assert np.array_equal(np.asarray(st[0]), VEC[name + ".m"]) and np.array_equal(np.asarray(st[1]), VEC[name + ".v"])
    assert np.array_equal(np.asarray(st[2]).view(np.uint32), VEC[name + ".absmax_m"].view(np.uint32))
    assert np.array_equal(np.asarray(st[3]).view(np.uint32), VEC[name + ".absmax_v"].view(np.uint32))


@pytest.mark.parametrize("name", sorted(CASES))
def test_c_oracle_reproduces_the_vectors(name):
    cmode, _, bf16, gs = CASES[name]
    maps = oc.load_maps()
    p = VEC[name + ".p0"].copy()
    st = oc.state_init(p.size)
    for t in range(3):
        h = oc.hyper_pack(*HYPER, t if cmode == oc.MODE_L2 else t + 1, cmode, gs)
        assert oc.step_tensor(p, VEC["%s.g%d" % (name, t)].copy(), *st, h, maps, oc.DT_BF16 if bf16 else oc.DT_F32, 1) == 0
    expect(name, p, st)


@pytest.mark.parametrize("name", sorted(CASES))
def test_numpy_oracle_reproduces_the_vectors(name):
    cmode, nmode, bf16, gs = CASES[name]
    maps = oc.load_maps()
    p = VEC[name + ".p0"].copy()
    st = list(onp.state_init(p.size))
    for t in range(3):
        h = onp.hyper_pack(*HYPER, t if nmode == "l2" else t + 1, nmode)
        if gs is not None:
            h["grad_scale"] = gs
        p, *st = onp.step_tensor(p, VEC["%s.g%d" % (name, t)], *st, h, *maps, bf16=bf16)
    expect(name, p, st)
