#!/usr/bin/env python3
"""Write tests/golden/step_vectors.npz: inputs and expected outputs of a few optimizer steps.

The reference holds no vectors for any optimizer, so these are produced by this repository's own CPU
oracle (oracle/adam8_oracle.c, pinned by tests/test_oracle_*.py) and frozen: once committed they guard
the oracle, the NumPy restatement and the HIP kernels against silent drift.  Per case: a ragged tensor of
5,000 elements, parameters and three steps of gradients (stored, not regenerated), and the parameters,
codes and absmax after the third step.  Cases: modes ERI / L2 / BNB x fp32 / bf16, decay 0.01, and one
ERI case with a gradient scale of 0.37.
Run from the repository root: python tests/golden/make_step_vectors.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle_c as oc  # noqa: E402
from oracle import adam8_numpy as onp  # noqa: E402

N = 5000
HYPER = (1e-4, 0.9, 0.999, 1e-8, 0.01)
CASES = [("eri_f32", oc.MODE_ERI, False, None), ("eri_bf16", oc.MODE_ERI, True, None), ("l2_f32", oc.MODE_L2, False, None),
         ("l2_bf16", oc.MODE_L2, True, None), ("bnb_f32", oc.MODE_BNB, False, None), ("bnb_bf16", oc.MODE_BNB, True, None),
         ("eri_bf16_gs", oc.MODE_ERI, True, 0.37)]


def main():
    maps = oc.load_maps()
    out = {}
    rng = np.random.default_rng(20240611)
    for name, mode, bf16, gs in CASES:
        p32 = (rng.standard_normal(N) * 0.02).astype(np.float32)
        p = onp.f32_to_bf16(p32) if bf16 else p32.copy()
        out[name + ".p0"] = p.copy()
        st = oc.state_init(N)
        for t in range(3):
            g32 = (rng.standard_normal(N) * 1e-3).astype(np.float32)
            g32[::41] = 0.0
            g = onp.f32_to_bf16(g32) if bf16 else g32
            out["%s.g%d" % (name, t)] = g.copy()
            step = t if mode == oc.MODE_L2 else t + 1
            h = oc.hyper_pack(*HYPER, step, mode, gs)
            assert oc.step_tensor(p, g, *st, h, maps, oc.DT_BF16 if bf16 else oc.DT_F32, 1) == 0
        out[name + ".p"] = p
        out[name + ".m"], out[name + ".v"], out[name + ".absmax_m"], out[name + ".absmax_v"] = st
    np.savez_compressed(os.path.join(HERE, "step_vectors.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
