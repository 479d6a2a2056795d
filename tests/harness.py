"""Shared plumbing of the parity tests: seeded inputs, the oracle run, the library run, the compare."""
import ctypes as C

import numpy as np

import oracle_c as oc
from oracle import adam8_numpy as onp

MAPS = oc.load_maps()
BLOCK = 2048


def make_inputs(sizes, bf16, seed, p_std=0.02, g_std=1e-3):
    """Per tensor: parameter and gradient arrays (float32, or uint16 bf16 patterns)."""
    rng = np.random.default_rng(seed)
    ps, gs = [], []
    for n in sizes:
        p = (rng.standard_normal(n) * p_std).astype(np.float32)
        g = (rng.standard_normal(n) * g_std).astype(np.float32)
        ps.append(onp.f32_to_bf16(p) if bf16 else p)
        gs.append(onp.f32_to_bf16(g) if bf16 else g)
    return ps, gs


def fresh_grads(sizes, bf16, seed, g_std=1e-3):
    rng = np.random.default_rng(seed)
    out = []
    for n in sizes:
        g = (rng.standard_normal(n) * g_std).astype(np.float32)
        out.append(onp.f32_to_bf16(g) if bf16 else g)
    return out


def oracle_states(sizes):
    return [list(oc.state_init(n)) for n in sizes]


def oracle_step(ps, gs, states, hyper_args, bf16, mode=oc.MODE_ERI, grad_scale=None, threads=8):
    """In place on ps/states.  hyper_args = (lr, b1, b2, eps, wd, step)."""
    h = oc.hyper_pack(*hyper_args, mode, grad_scale)
    for p, g, st in zip(ps, gs, states):
        rc = oc.step_tensor(p, g, *st, h, MAPS, oc.DT_BF16 if bf16 else oc.DT_F32, threads)
        assert rc == 0


class GpuTensors:
    """Device copies of a list of tensors with guard bands of poison around every buffer."""

    GUARD = 64  # elements of the buffer's dtype on each side

    def __init__(self, ps, gs, states, bf16):
        import torch
        self.torch = torch
        self.bf16 = bf16
        self.dev = torch.device("cuda:0")
        self.p = [self._up(a, 0xFF if not bf16 else 0xFF) for a in ps]
        self.g = [self._up(a, 0xFF) for a in gs]
        self.m = [self._up(st[0], 0xEE) for st in states]
        self.v = [self._up(st[1], 0xDD) for st in states]
        self.am = [self._up(st[2], 0xFF) for st in states]
        self.av = [self._up(st[3], 0xFF) for st in states]

    def _up(self, a, poison):
        torch = self.torch
        a = np.ascontiguousarray(a)
        item = a.dtype.itemsize
        # 16-byte alignment of the payload: guard of 64 elements of 1, 2 or 4 bytes keeps it
        raw = np.full((a.size + 2 * self.GUARD) * item, poison, np.uint8)
        raw[self.GUARD * item:(self.GUARD + a.size) * item] = a.view(np.uint8).reshape(-1)
        t = torch.from_numpy(raw).to(self.dev)
        assert (t.data_ptr() + self.GUARD * item) % 16 == 0
        return (t, a.dtype, a.size, poison)

    def ptr(self, buf):
        t, dt, n, _ = buf
        return t.data_ptr() + self.GUARD * dt.itemsize

    def down(self, buf):
        t, dt, n, poison = buf
        raw = t.cpu().numpy()
        item = dt.itemsize
        lo = raw[:self.GUARD * item]
        hi = raw[(self.GUARD + n) * item:]
        assert np.all(lo == poison) and np.all(hi == poison), "guard band overwritten"
        return raw[self.GUARD * item:(self.GUARD + n) * item].view(dt).copy()

    def set_grads(self, gs):
        torch = self.torch
        for buf, a in zip(self.g, gs):
            t, dt, n, _ = buf
            item = dt.itemsize
            t[self.GUARD * item:(self.GUARD + n) * item] = torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)).to(self.dev)

    def rows(self, grad_scales=None):
        from eridiffusion_amd._lib import TensorRow
        n = len(self.p)
        rows = (TensorRow * n)()
        start = 0
        for i in range(n):
            r = rows[i]
            r.p, r.g, r.m, r.v = self.ptr(self.p[i]), self.ptr(self.g[i]), self.ptr(self.m[i]), self.ptr(self.v[i])
            r.absmax_m, r.absmax_v = self.ptr(self.am[i]), self.ptr(self.av[i])
            r.numel = self.p[i][2]
            r.block_start = start
            r.dtype_tag = 2 if self.bf16 else 0
            r.grad_scale = 1.0 if grad_scales is None else grad_scales[i]
            start += (r.numel + BLOCK - 1) // BLOCK
        return rows

    def fetch(self):
        ps = [self.down(b) for b in self.p]
        states = [[self.down(self.m[i]), self.down(self.v[i]), self.down(self.am[i]), self.down(self.av[i])]
                  for i in range(len(self.p))]
        return ps, states


def bf16_ulp_distance(a, b):
    """Distance in bf16 steps between two uint16 bf16 patterns (sign-magnitude aware)."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a) - key(b))


def compare(got_ps, got_states, want_ps, want_states, bf16, exact_params, label=""):
    """Asserts the correctness bar and returns the counts it is stated in."""
    stats = {"code_mismatch": 0, "code_off_by_more": 0, "param_1ulp": 0, "params": 0}
    for i, (gp, gst, wp, wst) in enumerate(zip(got_ps, got_states, want_ps, want_states)):
        tag = "%s tensor %d" % (label, i)
        assert np.array_equal(gst[2].view(np.uint32), wst[2].view(np.uint32)), tag + ": absmax_m differs"
        assert np.array_equal(gst[3].view(np.uint32), wst[3].view(np.uint32)), tag + ": absmax_v differs"
        for k in (0, 1):
            d = np.abs(gst[k].astype(np.int32) - wst[k].astype(np.int32))
            stats["code_mismatch"] += int((d != 0).sum())
            stats["code_off_by_more"] += int((d > 1).sum())
        stats["params"] += gp.size
        if bf16:
            nan = (wp & 0x7FFF) > 0x7F80
            assert np.array_equal(nan, (gp & 0x7FFF) > 0x7F80), tag + ": NaN pattern differs"
            d = bf16_ulp_distance(gp[~nan], wp[~nan])
            assert d.max(initial=0) <= 1, tag + ": bf16 parameter off by more than one ulp"
            stats["param_1ulp"] += int((d != 0).sum())
            if exact_params:
                assert d.max(initial=0) == 0, tag + ": exact mode must reproduce bf16 parameters bit for bit"
        else:
            nan = np.isnan(wp)
            assert np.array_equal(nan, np.isnan(gp)), tag + ": NaN pattern differs"
            assert np.array_equal(gp[~nan].view(np.uint32), wp[~nan].view(np.uint32)), tag + ": fp32 parameters differ"
    assert stats["code_off_by_more"] == 0, label + ": a state code is more than one index away"
    return stats
